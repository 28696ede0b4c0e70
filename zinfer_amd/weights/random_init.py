"""Random-weights mode: draws every declared tensor from a seed and writes a model folder
(config.json and model.safetensors) that the ordinary loader then reads.

Distributions: matrices and the embedding N(0, 0.02); every norm gain (the per-head q and k
norms included) 1 + U(-0.1, 0.1).  Each tensor has its own generator, seeded from the seed
and the tensor's name, so a tensor's values do not depend on which others exist.
"""
from __future__ import annotations

import hashlib
import json
import os
from typing import Dict

import torch

from ..parts.base import TensorDecl
from .safetensors_io import write_safetensors

_CHUNK = 1 << 24


def _generator(seed: int, name: str) -> torch.Generator:
    digest = hashlib.sha256(f"{seed}:{name}".encode()).digest()
    g = torch.Generator(device="cpu")
    g.manual_seed(int.from_bytes(digest[:8], "little") & ((1 << 63) - 1))
    return g


def draw_tensor(name: str, decl: TensorDecl, seed: int, dtype: torch.dtype) -> torch.Tensor:
    g = _generator(seed, name)
    n = 1
    for d in decl.shape:
        n *= d
    out = torch.empty((n,), dtype=dtype)
    for lo in range(0, n, _CHUNK):            # in pieces: a big matrix never exists in float32
        m = min(_CHUNK, n - lo)
        if decl.init == "gain":
            piece = 1.0 + (torch.rand((m,), generator=g, dtype=torch.float32) * 0.2 - 0.1)
        elif decl.init == "zeros":
            piece = torch.zeros((m,), dtype=torch.float32)
        else:
            piece = torch.randn((m,), generator=g, dtype=torch.float32) * 0.02
        out[lo:lo + m] = piece.to(dtype)
    return out.view(*decl.shape)


def draw_tensors(decls: Dict[str, TensorDecl], seed: int, dtype: torch.dtype = torch.bfloat16,
                 tied: bool = False, head_name: str = "lm_head.weight") -> Dict[str, torch.Tensor]:
    out = {}
    for name, decl in decls.items():
        if tied and name == head_name and decl.optional:
            continue          # tied: the head is the embedding, nothing is stored for it
        out[name] = draw_tensor(name, decl, seed, dtype)
    return out


def write_model_dir(path: str, config, seed: int, dtype: torch.dtype = torch.bfloat16) -> str:
    """Writes ``config.json`` and ``model.safetensors`` for ``config`` (a typed configuration
    with ``to_dict()`` and ``model_spec()``) with weights drawn from ``seed``."""
    from ..models.build import declare_tensors
    os.makedirs(path, exist_ok=True)
    raw = config.to_dict()
    raw["torch_dtype"] = {torch.bfloat16: "bfloat16", torch.float32: "float32"}[dtype]
    with open(os.path.join(path, "config.json"), "w") as f:
        json.dump(raw, f, indent=1)
    spec = config.model_spec()
    decls = declare_tensors(spec)
    tensors = draw_tensors(decls, seed, dtype, tied=spec.tie_word_embeddings,
                           head_name=spec.head_name)
    write_safetensors(os.path.join(path, "model.safetensors"), tensors,
                      metadata={"format": "pt", "seed": str(seed)})
    return path
