"""Binding a model's declared tensors to the tensors of a model folder, by name.

Names are the HF names the reference binds (`src/model/families/qwen3/weights.zig:4-35`).
Everything is checked at load, before anything runs: one error lists every missing tensor,
every unexpected one and every wrong shape.  (The reference finds a missing name at
`src/tensor/backends/backend.zig:98` and a wrong shape only at first use,
`src/tensor/storage/store.zig:177-182`.)  Tensors keep the dtype they are stored in
(bfloat16 or 32-bit float; float16 and float64 become 32-bit floats, integer tables int32);
what a compute dtype does with them is the parts' business.

Tensors the model does not declare are an error, not ignored: a folder that brings a bias, a
second head or another architecture's layers would otherwise load and run with formulas that
are not its own.
"""
from __future__ import annotations

import json
import os
from typing import Dict, List

import torch

from ..errors import WeightError
from ..parts.base import TensorDecl
from .safetensors_io import SafetensorsFile

_FLOAT = ("F32", "BF16", "F16", "F64")
_INT = ("I8", "U8", "I16", "U16", "I32", "U32", "I64", "U64")


def _files_of(model_dir: str) -> List[str]:
    single = os.path.join(model_dir, "model.safetensors")
    if os.path.exists(single):
        return [single]
    index = os.path.join(model_dir, "model.safetensors.index.json")
    if os.path.exists(index):
        with open(index) as f:
            weight_map = json.load(f).get("weight_map", {})
        return [os.path.join(model_dir, n) for n in sorted(set(weight_map.values()))]
    raise WeightError(f"no model.safetensors (or model.safetensors.index.json) in {model_dir!r}")


def load_tensors(model_dir: str, decls: Dict[str, TensorDecl]) -> Dict[str, torch.Tensor]:
    """Host tensors for every declared name; raises one WeightError naming all that is wrong."""
    files = [SafetensorsFile(p) for p in _files_of(model_dir)]
    try:
        where = {}
        for f in files:
            for name in f.names():
                where[name] = f
        missing = [n for n, d in decls.items() if n not in where and not d.optional]
        unexpected = [n for n in where if n not in decls]
        wrong = []
        for n, d in decls.items():
            if n not in where:
                continue
            info = where[n].infos[n]
            if tuple(info.shape) != tuple(d.shape):
                wrong.append(f"{n}: expected shape {list(d.shape)}, file has {list(info.shape)}")
            elif info.dtype not in _FLOAT + _INT:
                wrong.append(f"{n}: dtype {info.dtype} is not readable")
        if missing or unexpected or wrong:
            lines = [f"the tensors of {model_dir!r} do not match the model:"]
            if missing:
                lines.append(f"  missing ({len(missing)}): " + ", ".join(sorted(missing)))
            if unexpected:
                lines.append(f"  unexpected ({len(unexpected)}): " + ", ".join(sorted(unexpected)))
            if wrong:
                lines.append(f"  wrong shape or dtype ({len(wrong)}):")
                lines += ["    " + w for w in wrong]
            raise WeightError("\n".join(lines))
        out = {}
        for n in decls:
            if n not in where:
                continue
            t = where[n].tensor(n)
            info = where[n].infos[n]
            if info.dtype in _INT:
                t = t.to(torch.int32)
            # float16 and float64 are handed on as they are stored: a 32-bit build widens
            # float16 exactly (rounding it to bfloat16 here would take 3 bits of mantissa from
            # its weights), a bfloat16 build rounds both to bfloat16 (``place_matrix``)
            out[n] = t
        return out
    finally:
        for f in files:
            f.close()
