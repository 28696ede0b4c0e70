"""zinfer_amd: a small, whole inference engine for the Qwen3 dense decoder on one MI355X."""
from . import config, errors
from .config import Qwen3Config, load_config, register_architecture
from .errors import (CacheFull, ConfigError, FormatError, KernelUnavailable, PositionOutOfBounds,
                     StepError, TokenIdOutOfBounds, UnsupportedModelType, WeightError, ZinferError)

__version__ = "0.1.0"
