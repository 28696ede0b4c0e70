"""One registry from an architecture's name to its configuration type and model.

The reference detects the architecture from ``model_type`` in config.json and looks the
family's entry up (`src/model/runtime/decoder_family.zig:58-63,249-281`,
`src/model/runtime/decoder_registry.zig:7-21`).  Here an entry is keyed by the names of
``architectures`` and by ``model_type``; its ``config_type`` turns the JSON object into a
typed configuration whose ``model_spec()`` describes the model's parts.
"""
from __future__ import annotations

import json
import os
from dataclasses import dataclass
from typing import Callable, Dict, Optional

from ..errors import ConfigError, UnsupportedModelType


@dataclass
class TextHooks:
    """What an architecture brings for text in and out, as the reference's entry does
    (`decoder_registry.zig:16-19`): the engine itself takes and returns token ids."""
    load_tokenizer: Callable[[str], object]                  # model folder -> encode/decode
    render_messages: Callable[..., str]                      # (messages, thinking) -> prompt
    render_single_user: Callable[..., str]                   # (text, thinking, system) -> prompt
    assistant_history_content: Callable[[str], str]          # an earlier answer as history


@dataclass
class ArchitectureEntry:
    name: str                      # e.g. "Qwen3ForCausalLM"
    model_type: Optional[str]      # e.g. "qwen3"
    config_type: type              # has from_dict(dict), to_dict(), model_spec()
    text: Optional[TextHooks] = None


_BY_NAME: Dict[str, ArchitectureEntry] = {}
_BY_MODEL_TYPE: Dict[str, ArchitectureEntry] = {}


def register_architecture(name: str, config_type: type, model_type: Optional[str] = None,
                          text: Optional[TextHooks] = None) -> None:
    entry = ArchitectureEntry(name, model_type, config_type, text)
    _BY_NAME[name] = entry
    if model_type is not None:
        _BY_MODEL_TYPE[model_type] = entry


def unregister_architecture(name: str) -> None:
    entry = _BY_NAME.pop(name, None)
    if entry is not None and entry.model_type is not None:
        _BY_MODEL_TYPE.pop(entry.model_type, None)


def registered_architectures():
    return sorted(_BY_NAME)


def entry_for(config: dict) -> ArchitectureEntry:
    """`decoder_family.zig:267-281`: a missing ``model_type`` and a non-string one are errors
    of their own; an unknown one is UnsupportedModelType."""
    archs = config.get("architectures", [])
    if isinstance(archs, list):
        for a in archs:
            if isinstance(a, str) and a in _BY_NAME:
                return _BY_NAME[a]
    if "model_type" not in config:
        raise ConfigError("MissingModelType: config.json has no 'model_type' and no registered "
                          f"name in 'architectures' ({archs!r})")
    mt = config["model_type"]
    if not isinstance(mt, str):
        raise ConfigError(f"InvalidModelType: 'model_type' must be a string, got {mt!r}")
    if mt in _BY_MODEL_TYPE:
        return _BY_MODEL_TYPE[mt]
    raise UnsupportedModelType(
        f"UnsupportedModelType: {mt!r} (architectures {archs!r}); registered: "
        f"{registered_architectures()}")


def read_config_json(model_dir: str) -> dict:
    path = os.path.join(model_dir, "config.json")
    try:
        with open(path, "r", encoding="utf-8") as f:
            data = json.load(f)
    except FileNotFoundError:
        raise ConfigError(f"no config.json in {model_dir!r}") from None
    except json.JSONDecodeError as e:
        raise ConfigError(f"{path}: not valid JSON ({e})") from None
    if not isinstance(data, dict):
        raise ConfigError(f"{path}: the root must be a JSON object")
    return data


def load_config(model_dir: str):
    """Typed configuration of the model in ``model_dir``, chosen by its config.json."""
    raw = read_config_json(model_dir)
    return entry_for(raw).config_type.from_dict(raw)
