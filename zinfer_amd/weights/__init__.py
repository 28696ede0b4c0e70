from .loader import load_tensors
from .random_init import draw_tensor, draw_tensors, write_model_dir
from .safetensors_io import SafetensorsFile, TensorInfo, parse_header, write_safetensors
