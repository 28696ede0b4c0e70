"""Typed configuration of the Qwen3 dense decoder, read from its config.json keys.

The reference's struct (`src/model/families/qwen3/config.zig:3-23`) lists the keys; all are
required there except ``architectures`` and unknown keys are ignored (`:41-43`).  Keys the
reference does not parse but that would change the computation are read here only to refuse
values the formulas do not cover.
"""
from __future__ import annotations

from dataclasses import dataclass, asdict, field
from typing import List, Tuple

from ..errors import ConfigError
from .registry import TextHooks, register_architecture
from .specs import (GqaAttentionSpec, ModelSpec, PreNormBlockSpec, RmsNormSpec,
                    RotaryHalfSplitSpec, ScheduleEntry, SwiGluSpec)

# `src/model/families/qwen3/generation_policy.zig:3-6`
QWEN3_EOS_TOKEN_IDS = (151645, 151643)
QWEN3_DEFAULT_STOPS = ("<|im_end|>",)

_INT_KEYS = ("head_dim", "hidden_size", "intermediate_size", "max_position_embeddings",
             "num_attention_heads", "num_hidden_layers", "num_key_value_heads", "vocab_size")
_FLOAT_KEYS = ("rms_norm_eps", "rope_theta")


@dataclass(frozen=True)
class Qwen3Config:
    head_dim: int
    hidden_size: int
    intermediate_size: int
    max_position_embeddings: int
    model_type: str
    num_attention_heads: int
    num_hidden_layers: int
    num_key_value_heads: int
    rms_norm_eps: float
    rope_theta: float
    tie_word_embeddings: bool
    torch_dtype: str
    vocab_size: int
    architectures: Tuple[str, ...] = ()

    # ------------------------------------------------------------------ parsing
    @classmethod
    def from_dict(cls, raw: dict) -> "Qwen3Config":
        missing = [k for k in (*_INT_KEYS, *_FLOAT_KEYS, "model_type", "tie_word_embeddings",
                               "torch_dtype") if k not in raw]
        if missing:
            raise ConfigError(f"config.json: missing keys {missing}")
        vals = {}
        for k in _INT_KEYS:
            v = raw[k]
            if isinstance(v, bool) or not isinstance(v, int):
                raise ConfigError(f"config.json: {k!r} must be an integer, got {v!r}")
            if v < 0:
                raise ConfigError(f"config.json: {k!r} must not be negative, got {v}")
            vals[k] = v
        for k in _FLOAT_KEYS:
            v = raw[k]
            if isinstance(v, bool) or not isinstance(v, (int, float)):
                raise ConfigError(f"config.json: {k!r} must be a number, got {v!r}")
            vals[k] = float(v)
        if not isinstance(raw["model_type"], str):
            raise ConfigError("config.json: 'model_type' must be a string")
        if not isinstance(raw["tie_word_embeddings"], bool):
            raise ConfigError("config.json: 'tie_word_embeddings' must be true or false")
        if not isinstance(raw["torch_dtype"], str):
            raise ConfigError("config.json: 'torch_dtype' must be a string")
        archs = raw.get("architectures", [])
        if not isinstance(archs, list) or any(not isinstance(a, str) for a in archs):
            raise ConfigError("config.json: 'architectures' must be a list of strings")
        # keys the reference ignores; a value that changes the formulas is refused
        if raw.get("use_sliding_window", False):
            raise ConfigError("config.json: use_sliding_window=true is not covered "
                              "(the architecture is full causal attention in every layer)")
        if raw.get("attention_bias", False):
            raise ConfigError("config.json: attention_bias=true is not covered (no biases)")
        if raw.get("hidden_act", "silu") != "silu":
            raise ConfigError(f"config.json: hidden_act={raw['hidden_act']!r}; only 'silu'")
        if raw.get("rope_scaling", None) is not None:
            raise ConfigError("config.json: rope_scaling is not covered")
        cfg = cls(model_type=raw["model_type"], tie_word_embeddings=raw["tie_word_embeddings"],
                  torch_dtype=raw["torch_dtype"], architectures=tuple(archs), **vals)
        cfg.validate()
        return cfg

    def validate(self) -> None:
        """`src/model/layers/rmsnorm_gqa_swiglu_block.zig:34-40`,
        `src/model/layers/gqa_attention/spec.zig:10-17`, `src/kernel/attention/rope.zig:16`."""
        for k in ("hidden_size", "intermediate_size", "num_attention_heads",
                  "num_key_value_heads", "head_dim", "vocab_size", "max_position_embeddings"):
            if getattr(self, k) == 0:
                raise ConfigError(f"InvalidDimensions: {k} is 0")
        if self.num_attention_heads % self.num_key_value_heads != 0:
            raise ConfigError(
                f"InvalidGrouping: num_attention_heads={self.num_attention_heads} is not a "
                f"multiple of num_key_value_heads={self.num_key_value_heads}")
        if self.head_dim % 2 != 0:
            raise ConfigError(f"InvalidHeadDim: head_dim={self.head_dim} must be even")
        if not (self.rms_norm_eps >= 0.0):
            raise ConfigError(f"rms_norm_eps={self.rms_norm_eps} must not be negative")
        if not (self.rope_theta > 0.0):
            raise ConfigError(f"rope_theta={self.rope_theta} must be positive")

    def to_dict(self) -> dict:
        d = asdict(self)
        d["architectures"] = list(self.architectures) or ["Qwen3ForCausalLM"]
        return d

    # ------------------------------------------------------------------ the model's parts
    def model_spec(self) -> ModelSpec:
        """Every layer: pre-norm block of grouped-query attention with per-head norm of q
        and k (`src/model/families/qwen3/layout.zig:3-6`) and rotation, and a SwiGLU
        feed-forward; layers run once each, in order, each with its own cache."""
        rope = RotaryHalfSplitSpec(self.head_dim, self.rope_theta, self.max_position_embeddings)
        attn = GqaAttentionSpec(self.hidden_size, self.num_attention_heads,
                                self.num_key_value_heads, self.head_dim,
                                qk_norm_eps=self.rms_norm_eps, position=rope, window=None)
        ff = SwiGluSpec(self.hidden_size, self.intermediate_size)
        norm = RmsNormSpec(self.hidden_size, self.rms_norm_eps)
        block = PreNormBlockSpec(mixer=attn, feed_forward=ff, mixer_norm=norm, ff_norm=norm)
        n = self.num_hidden_layers
        return ModelSpec(
            vocab_size=self.vocab_size, hidden_size=self.hidden_size,
            max_positions=self.max_position_embeddings,
            layers=tuple(block for _ in range(n)),
            schedule=tuple(ScheduleEntry(i) for i in range(n)),
            final_norm=norm, tie_word_embeddings=self.tie_word_embeddings,
            eos_token_ids=QWEN3_EOS_TOKEN_IDS, default_stop_sequences=QWEN3_DEFAULT_STOPS)


# `src/model/runtime/decoder_family.zig:249-265`: the family's tokenizer and templates; the
# text front end is only imported when one of them is called
def _load_tokenizer(model_dir: str):
    from ..text import Tokenizer
    return Tokenizer.from_dir(model_dir)


def _render_messages(messages, thinking: bool) -> str:
    from ..text.chat import render_messages
    return render_messages(messages, thinking)


def _render_single_user(user_text: str, thinking: bool, system=None) -> str:
    from ..text.chat import render_single_user
    return render_single_user(user_text, thinking, system)


def _assistant_history_content(content: str) -> str:
    from ..text.chat import strip_historical_thinking
    return strip_historical_thinking(content)


register_architecture(
    "Qwen3ForCausalLM", Qwen3Config, model_type="qwen3",
    text=TextHooks(_load_tokenizer, _render_messages, _render_single_user,
                   _assistant_history_content))
