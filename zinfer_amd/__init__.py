"""zinfer_amd: a small, whole inference engine for the Qwen3 dense decoder on one MI355X."""
from . import config, errors
from .config import Qwen3Config, load_config, register_architecture
from .errors import (CacheFull, ConfigError, FormatError, KernelUnavailable, PositionOutOfBounds,
                     StepError, TokenIdOutOfBounds, UnsupportedModelType, WeightError, ZinferError)

__version__ = "0.1.0"

_LAZY = {"LLM": ("entrypoints", "LLM"), "Engine": ("engine", "Engine"),
         "StepEntry": ("engine", "StepEntry"), "Scheduler": ("engine.scheduler", "Scheduler"),
         "SamplingParams": ("sampling", "SamplingParams"), "Tokenizer": ("text", "Tokenizer"),
         "run_trace": ("engine.replay", "run_trace"), "load_model": ("models.build", "load_model"),
         "write_model_dir": ("weights", "write_model_dir")}


def __getattr__(name):
    """The entry points by name (``zinfer_amd.LLM``, ``.Engine``, ``.SamplingParams``, ...),
    imported when first asked for so that ``import zinfer_amd`` stays light."""
    if name in _LAZY:
        import importlib
        module, attr = _LAZY[name]
        return getattr(importlib.import_module("." + module, __name__), attr)
    raise AttributeError(f"module {__name__!r} has no attribute {name!r}")
