from .build import build_model, declare_tensors, load_model, parse_dtype
from .decoder import DecoderModel
