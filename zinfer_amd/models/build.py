"""From a model folder (or a typed configuration and tensors) to a bound model."""
from __future__ import annotations

from typing import Dict, Optional

import torch

from ..config import load_config
from ..config.specs import ModelSpec
from ..parts import BuildContext, TensorDecl
from ..weights.loader import load_tensors
from .decoder import DecoderModel

_DTYPES = {"bfloat16": torch.bfloat16, "bf16": torch.bfloat16, "float32": torch.float32,
           "fp32": torch.float32, "f32": torch.float32}


def parse_dtype(name) -> torch.dtype:
    if isinstance(name, torch.dtype):
        if name not in (torch.bfloat16, torch.float32):
            raise ValueError(f"compute dtype must be bfloat16 or float32, not {name}")
        return name
    try:
        return _DTYPES[str(name).lower()]
    except KeyError:
        raise ValueError(f"dtype {name!r}: choose bfloat16 or float32") from None


def declare_tensors(spec: ModelSpec) -> Dict[str, TensorDecl]:
    """The tensors a model of ``spec`` binds; no device is touched."""
    ctx = BuildContext(torch.float32, torch.device("meta"))
    return DecoderModel(spec, ctx).declare()


def build_model(spec: ModelSpec, tensors: Dict[str, torch.Tensor], dtype, device) -> DecoderModel:
    ctx = BuildContext(parse_dtype(dtype), torch.device(device))
    model = DecoderModel(spec, ctx)
    model.bind(tensors)
    return model


def load_model(model_dir: str, dtype="bfloat16", device="cuda:0"):
    """(typed configuration, bound model) of a folder with config.json and model.safetensors;
    the architecture is chosen by config.json."""
    import os
    config = load_config(model_dir)
    spec = config.model_spec()
    ctx = BuildContext(parse_dtype(dtype), torch.device(device))
    # kernel plans measured at this model's own widths (``bench-ops --tune`` writes them)
    from .. import ops
    plans = os.path.join(model_dir, ops.PLAN_FILE)
    if os.path.exists(plans):
        ops.load_plans(plans)
    model = DecoderModel(spec, ctx)
    tensors = load_tensors(model_dir, model.declare())
    model.bind(tensors)
    return config, model


def random_model(config, seed: int, dtype="bfloat16", device="cuda:0", store_dtype=None):
    """(typed configuration, bound model) with weights drawn from ``seed``: the values that
    ``write_model_dir(config, seed, store_dtype)`` stores, without the file, drawn on the
    device one tensor at a time.  ``config``: a typed configuration, a dict of config.json
    keys, or the path of a config.json.  ``store_dtype``: what the drawn values are rounded to
    before the model takes them (default: the compute dtype)."""
    import json
    from ..config import entry_for
    from ..weights.random_init import DrawnTensors
    if isinstance(config, str):
        with open(config, "r", encoding="utf-8") as f:
            config = json.load(f)
    if isinstance(config, dict):
        config = entry_for(config).config_type.from_dict(config)
    spec = config.model_spec()
    ctx = BuildContext(parse_dtype(dtype), torch.device(device))
    model = DecoderModel(spec, ctx)
    store = parse_dtype(store_dtype) if store_dtype is not None else ctx.compute_dtype
    model.bind(DrawnTensors(model.declare(), seed, store, ctx.device,
                            tied=spec.tie_word_embeddings, head_name=spec.head_name))
    return config, model
