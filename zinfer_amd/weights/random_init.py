"""Random-weights mode: draws every declared tensor from a seed and writes a model folder
(config.json and model.safetensors) that the ordinary loader then reads.

Distributions: matrices and the embedding N(0, 0.02); every norm gain (the per-head q and k
norms included) 1 + U(-0.1, 0.1).  One counter-based generator (`counter_rng`) serves every
caller: an element's value depends on the seed, the tensor's name and the element's index
alone, so it does not depend on which other tensors exist, on the pieces a tensor is drawn in,
or on whether the GPU's kernel or numpy draws it.
"""
from __future__ import annotations

import json
import os
from collections.abc import Mapping
from typing import Dict, Iterator, Optional

import numpy as np
import torch

from ..parts.base import TensorDecl
from . import counter_rng
from .safetensors_io import write_safetensors

_CHUNK = 1 << 22
STD = 0.02


def _on_gpu(device) -> bool:
    return device is not None and torch.device(device).type == "cuda"


def draw_tensor(name: str, decl: TensorDecl, seed: int, dtype: torch.dtype,
                device=None) -> torch.Tensor:
    """The tensor ``name`` of ``seed``: every element is a function of (seed, name, its index)
    alone (`counter_rng`), the same bits whether the device's kernel or numpy draws it."""
    if dtype not in (torch.float32, torch.bfloat16):
        raise ValueError(f"random weights are stored as float32 or bfloat16, not {dtype}")
    if decl.init not in counter_rng.KIND:
        raise ValueError(f"tensor {name!r}: unknown init {decl.init!r}")
    n = 1
    for d in decl.shape:
        n *= d
    key = counter_rng.tensor_key(seed, name)
    if _on_gpu(device):
        from .. import ops
        out = torch.empty((n,), dtype=dtype, device=device)
        ops.randinit(out, key, 0, decl.init, STD)
        return out.view(*decl.shape)
    out = torch.empty((n,), dtype=dtype)
    for lo in range(0, n, _CHUNK):            # in pieces: a big matrix never exists in 64-bit
        m = min(_CHUNK, n - lo)
        piece = counter_rng.draw(key, lo, m, decl.init, STD)
        if dtype == torch.bfloat16:
            bits = counter_rng.to_bfloat16_bits(piece).view(np.int16)
            out[lo:lo + m] = torch.from_numpy(bits).view(torch.bfloat16)
        else:
            out[lo:lo + m] = torch.from_numpy(piece)
    return out.view(*decl.shape)


class DrawnTensors(Mapping):
    """The tensors of a seed, each drawn when it is asked for and not kept: binding a large
    model never holds more than one tensor beside the model's own copy."""

    def __init__(self, decls: Dict[str, TensorDecl], seed: int, dtype: torch.dtype, device=None,
                 tied: bool = False, head_name: str = "lm_head.weight"):
        # tied: the head is the embedding, nothing is drawn for it
        self._decls = {n: d for n, d in decls.items()
                       if not (tied and n == head_name and d.optional)}
        self._seed, self._dtype, self._device = seed, dtype, device

    def __getitem__(self, name: str) -> torch.Tensor:
        return draw_tensor(name, self._decls[name], self._seed, self._dtype, self._device)

    def __iter__(self) -> Iterator[str]:
        return iter(self._decls)

    def __len__(self) -> int:
        return len(self._decls)


def draw_tensors(decls: Dict[str, TensorDecl], seed: int, dtype: torch.dtype = torch.bfloat16,
                 tied: bool = False, head_name: str = "lm_head.weight",
                 device=None) -> Dict[str, torch.Tensor]:
    return dict(DrawnTensors(decls, seed, dtype, device, tied, head_name))


def write_model_dir(path: str, config, seed: int, dtype: torch.dtype = torch.bfloat16,
                    device=None) -> str:
    """Writes ``config.json`` and ``model.safetensors`` for ``config`` (a typed configuration
    with ``to_dict()`` and ``model_spec()``) with weights drawn from ``seed``; on ``device`` if
    it is a GPU (faster, the same values)."""
    from ..models.build import declare_tensors
    os.makedirs(path, exist_ok=True)
    raw = config.to_dict()
    raw["torch_dtype"] = {torch.bfloat16: "bfloat16", torch.float32: "float32"}[dtype]
    with open(os.path.join(path, "config.json"), "w") as f:
        json.dump(raw, f, indent=1)
    spec = config.model_spec()
    decls = declare_tensors(spec)
    tensors = {name: t.cpu() for name, t in
               DrawnTensors(decls, seed, dtype, device, spec.tie_word_embeddings,
                            spec.head_name).items()}
    write_safetensors(os.path.join(path, "model.safetensors"), tensors,
                      metadata={"format": "pt", "seed": str(seed)})
    return path
