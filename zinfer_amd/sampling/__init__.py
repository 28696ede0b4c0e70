from .sampler import (SamplingParams, Xoshiro256pp, adjust_logits, count_history, sample_token,
                      thinking_defaults, top_k_candidates)
