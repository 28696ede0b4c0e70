from .base import (Block, BuildContext, FeedForward, KVNeed, Mixer, Norm, Part,
                   PositionEncoding, StateNeed, StepHints, StepShape, TensorDecl, build_part,
                   register_part, unregister_part)
from .linear import Linear, place_gain, place_matrix
from . import norm, position, attention, mlp, block  # registers the built-in parts
