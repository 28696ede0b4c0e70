from .registry import (ArchitectureEntry, TextHooks, entry_for, load_config, read_config_json,
                       register_architecture, registered_architectures,
                       unregister_architecture)
from .specs import (GqaAttentionSpec, ModelSpec, NoPositionSpec, PreNormBlockSpec, RmsNormSpec,
                    RotaryHalfSplitSpec, ScheduleEntry, SwiGluSpec)
from .qwen3 import Qwen3Config
