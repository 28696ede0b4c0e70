"""The tiny configurations the tests run: two Qwen3 shapes that differ in every size and
option, plus helpers that make weights and model folders for them."""
from __future__ import annotations

import os
import tempfile
from typing import Dict

import torch

from zinfer_amd.config import Qwen3Config
from zinfer_amd.models.build import declare_tensors
from zinfer_amd.weights import draw_tensors, write_model_dir

TINY_A = dict(architectures=["Qwen3ForCausalLM"], model_type="qwen3", num_hidden_layers=2,
              hidden_size=64, num_attention_heads=4, num_key_value_heads=2, head_dim=16,
              intermediate_size=192, vocab_size=512, rope_theta=10000.0, rms_norm_eps=1e-6,
              tie_word_embeddings=True, max_position_embeddings=256, torch_dtype="float32")

TINY_B = dict(architectures=["Qwen3ForCausalLM"], model_type="qwen3", num_hidden_layers=3,
              hidden_size=96, num_attention_heads=8, num_key_value_heads=2, head_dim=32,
              intermediate_size=320, vocab_size=1000, rope_theta=1000000.0, rms_norm_eps=1e-5,
              tie_word_embeddings=False, max_position_embeddings=512, torch_dtype="float32")

# a third shape with sizes that are no power of two anywhere: 3 query heads on 1 kv head,
# head_dim 48, hidden 80, vocabulary 777
TINY_C = dict(architectures=["Qwen3ForCausalLM"], model_type="qwen3", num_hidden_layers=2,
              hidden_size=80, num_attention_heads=3, num_key_value_heads=1, head_dim=48,
              intermediate_size=112, vocab_size=777, rope_theta=50000.0, rms_norm_eps=3e-6,
              tie_word_embeddings=False, max_position_embeddings=384, torch_dtype="float32")

# a fourth shape whose sizes the bfloat16 MFMA kernels cover (head_dim 64, pages of 16, widths
# that are multiples of 8), so that those kernels run inside the engine tests as well
TINY_D = dict(architectures=["Qwen3ForCausalLM"], model_type="qwen3", num_hidden_layers=2,
              hidden_size=192, num_attention_heads=6, num_key_value_heads=2, head_dim=64,
              intermediate_size=456, vocab_size=1210, rope_theta=100000.0, rms_norm_eps=2e-6,
              tie_word_embeddings=True, max_position_embeddings=640, torch_dtype="bfloat16")

# a fifth shape with the serving model's head size and widths that are multiples of 128 (and a
# feed-forward width of 2048), so that the kernels chosen by size run inside the engine tests:
# the product for 17 to 128 tokens, the products split along K whose partials one kernel adds,
# sums into the residual and norms, the 128 x 256 tiles, the head-size-128 attention
TINY_E = dict(architectures=["Qwen3ForCausalLM"], model_type="qwen3", num_hidden_layers=2,
              hidden_size=256, num_attention_heads=4, num_key_value_heads=2, head_dim=128,
              intermediate_size=2048, vocab_size=2304, rope_theta=500000.0, rms_norm_eps=1e-6,
              tie_word_embeddings=False, max_position_embeddings=768, torch_dtype="bfloat16")

# two layers of the widths that are served (hidden 4096, 32 / 8 heads of 128, feed-forward
# 12288) under a small vocabulary that is no multiple of 64: the kernels at the sizes and
# with the splits along K that the benchmark runs them with, against the plain implementation
WIDE = dict(architectures=["Qwen3ForCausalLM"], model_type="qwen3", num_hidden_layers=2,
            hidden_size=4096, num_attention_heads=32, num_key_value_heads=8, head_dim=128,
            intermediate_size=12288, vocab_size=8200, rope_theta=1000000.0, rms_norm_eps=1e-6,
            tie_word_embeddings=False, max_position_embeddings=1024, torch_dtype="bfloat16")

# the served model's heads (4 query heads to a kv head, head size 128) under narrow widths and
# a position table of 4096: contexts of thousands of keys, where the decode attention runs
# more than 8 splits and the merge of their partials takes more than one load a lane
LONG = dict(architectures=["Qwen3ForCausalLM"], model_type="qwen3", num_hidden_layers=2,
            hidden_size=256, num_attention_heads=8, num_key_value_heads=2, head_dim=128,
            intermediate_size=768, vocab_size=1536, rope_theta=1000000.0, rms_norm_eps=1e-6,
            tie_word_embeddings=False, max_position_embeddings=4096, torch_dtype="bfloat16")

# the served model's depth and heads (36 layers, 32 query heads on 8 kv heads of 128) under
# narrow widths: how far bfloat16 drifts from the exact result over a real number of layers
DEEP = dict(architectures=["Qwen3ForCausalLM"], model_type="qwen3", num_hidden_layers=36,
            hidden_size=256, num_attention_heads=32, num_key_value_heads=8, head_dim=128,
            intermediate_size=512, vocab_size=1024, rope_theta=1000000.0, rms_norm_eps=1e-6,
            tie_word_embeddings=False, max_position_embeddings=512, torch_dtype="bfloat16")

CONFIGS = {"A": TINY_A, "B": TINY_B, "C": TINY_C, "D": TINY_D, "E": TINY_E, "W": WIDE,
           "L": LONG, "P": DEEP}
PAGE_SIZE = {"A": 16, "B": 8, "C": 16, "D": 16, "E": 16, "W": 16, "L": 16, "P": 16}
SEEDS = {"A": 11, "B": 22, "C": 33, "D": 44, "E": 55, "W": 66, "L": 77, "P": 88}


def config_of(name: str) -> Qwen3Config:
    return Qwen3Config.from_dict(CONFIGS[name])


def _draw_device():
    """Where the tests' weights are drawn: the GPU's kernel when there is one (the same values
    as numpy's, much sooner for the widest configuration)."""
    return "cuda:0" if torch.cuda.is_available() else None


def weights_of(name: str, dtype=torch.float32) -> Dict[str, torch.Tensor]:
    cfg = config_of(name)
    spec = cfg.model_spec()
    drawn = draw_tensors(declare_tensors(spec), SEEDS[name], dtype,
                         tied=spec.tie_word_embeddings, device=_draw_device())
    return {k: t.cpu() for k, t in drawn.items()}


def model_dir_of(name: str, root: str, dtype=torch.float32) -> str:
    path = os.path.join(root, f"tiny_{name}_{str(dtype).split('.')[-1]}")
    if not os.path.exists(os.path.join(path, "model.safetensors")):
        write_model_dir(path, config_of(name), SEEDS[name], dtype, device=_draw_device())
    return path


def random_tokens(n: int, vocab: int, seed: int):
    g = torch.Generator().manual_seed(seed)
    return torch.randint(0, vocab, (n,), generator=g).tolist()
