"""Error types of the engine.  The names follow the reference's error names where it has one
(`src/model/runtime/optimized_kv_cache/cache.zig:96` CacheFull,
`src/model/runtime/optimized_decoder/runtime.zig:109` TokenIdOutOfBounds,
`src/kernel/attention/rope.zig:135` PositionOutOfBounds,
`src/model/runtime/decoder_family.zig:267-281` Missing/Invalid/UnsupportedModelType)."""


class ZinferError(Exception):
    """Base class of every error the engine raises on purpose."""


class ConfigError(ZinferError):
    """config.json is missing a key, has a wrong type or an inconsistent value."""


class UnsupportedModelType(ConfigError):
    """config.json names an architecture that is not registered."""


class WeightError(ZinferError):
    """The tensors of a model folder do not match what the model declares."""


class FormatError(WeightError):
    """A safetensors container is malformed; ``code`` is the reference's error name
    (`src/format/safetensors.zig:38,139-336`)."""

    def __init__(self, code: str, detail: str = ""):
        super().__init__(f"{code}: {detail}" if detail else code)
        self.code = code


class CacheFull(ZinferError):
    """No free page (or state slot) is left for what a step needs."""


class TokenIdOutOfBounds(ZinferError):
    pass


class PositionOutOfBounds(ZinferError):
    pass


class StepError(ZinferError):
    """A step was given something it cannot run (unknown request, empty portion, ...)."""


class KernelUnavailable(ZinferError):
    """The HIP extension is missing, cannot be built, or refuses the given sizes."""
