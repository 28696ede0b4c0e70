from __future__ import annotations

import numpy as np
import torch

from ..config.specs import NoPositionSpec, RotaryHalfSplitSpec
from ..errors import ConfigError
from .base import PositionEncoding, register_part


def rotary_tables(head_dim: int, theta: float, max_positions: int):
    """cos and sin as float32 [max_positions, head_dim/2].  The angle is formed in 32-bit as
    the reference forms it (`src/kernel/attention/rope.zig:25-34`): exponent = 2i/hd,
    inv_freq = 1/pow(theta, exponent), angle = position * inv_freq; its cosine and sine are
    then taken in 64-bit and rounded once."""
    if head_dim == 0 or head_dim % 2 != 0:
        raise ConfigError(f"InvalidHeadDim: head_dim={head_dim} must be even")
    half = head_dim // 2
    exponent = (np.arange(half, dtype=np.float32) * np.float32(2.0)) / np.float32(head_dim)
    inv_freq = np.float32(1.0) / np.power(np.float32(theta), exponent, dtype=np.float32)
    pos = np.arange(max_positions, dtype=np.float32)[:, None]
    angle = (pos * inv_freq[None, :]).astype(np.float32).astype(np.float64)
    return (torch.from_numpy(np.cos(angle).astype(np.float32)),
            torch.from_numpy(np.sin(angle).astype(np.float32)))


_device_tables = {}     # (specification, device) -> (cos, sin): layers with equal specs share


def device_rotary_tables(spec, device):
    """The tables of ``spec`` on ``device``, built and uploaded once however many layers ask."""
    key = (spec, str(device))
    held = _device_tables.get(key)
    if held is None:
        cos, sin = rotary_tables(spec.head_dim, spec.theta, spec.max_positions)
        held = (cos.to(device), sin.to(device))
        _device_tables[key] = held
        for k in [k for k in _device_tables if k != key and k[1] == key[1]
                  and len(_device_tables) > 8]:
            del _device_tables[k]      # a process that builds many models keeps the newest
    return held


class RotaryHalfSplit(PositionEncoding):
    """Half-split rotation over the full head (`src/kernel/attention/rope.zig:92-109`); the
    attention kernel applies it from the tables."""
    graph_safe = True


    def __init__(self, spec, ctx, prefix):
        super().__init__(spec, ctx, prefix)
        self.cos, self.sin = device_rotary_tables(spec, ctx.device)

    def rotation_tables(self):
        return self.cos, self.sin


class NoPosition(PositionEncoding):
    """q and k go into the attention as they are."""
    graph_safe = True



register_part("position", RotaryHalfSplitSpec, RotaryHalfSplit)
register_part("position", NoPositionSpec, NoPosition)
