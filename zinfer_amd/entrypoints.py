"""The Python entry point: a model folder in, token ids out.

The reference's generation loop (`src/app/cli/runtime/generator.zig:53-123`) encodes a
prompt, prefills, then samples, checks end-of-sequence (the id is neither appended nor
forwarded, `:103-105`) and forwards the sampled token; here the scheduler does the same for
many requests at once and without the reference's discarded last forward (`:115`).
"""
from __future__ import annotations

from typing import Dict, List, Optional, Sequence

import torch

from .engine import Engine
from .engine.scheduler import Request, Scheduler
from .models.build import load_model, random_model
from .sampling import SamplingParams


class LLM:
    def __init__(self, model_dir: Optional[str] = None, dtype: str = "bfloat16",
                 device: str = "cuda:0",
                 page_size: int = 16, max_tokens: Optional[int] = None,
                 num_pages: Optional[int] = None, max_step_tokens: int = 2048,
                 chunk_size: Optional[int] = None, max_seqs: int = 64,
                 kv_dtype: Optional[str] = None, multi_step: int = 8,
                 config=None, random_seed: Optional[int] = None, debug_tables: bool = False):
        """A model folder, or ``config`` (a typed configuration, a dict of config.json keys or
        the path of a config.json) with ``random_seed``: weights drawn from the seed, the same
        values that ``write_model_dir`` stores for it.  ``max_tokens`` (or ``num_pages``) sizes the cache pool; by default the pool holds
        ``max_seqs`` requests of ``max_position_embeddings`` tokens, capped at 1/2 of the free
        device memory.  ``multi_step``: the most decode steps that run in a row on the device
        without the host between them (1: the host sees every step).  ``debug_tables``: every
        step's block tables and slots are checked on the device before its kernels run."""
        if (config is None) != (random_seed is None):
            raise ValueError("config and random_seed go together")
        if config is not None:
            self.config, self.model = random_model(config, random_seed, dtype, device)
        elif model_dir is not None:
            self.config, self.model = load_model(model_dir, dtype, device)
        else:
            raise ValueError("a model folder, or config and random_seed, is needed")
        spec = self.model.spec
        if num_pages is None:
            if max_tokens is None:
                max_tokens = self._default_max_tokens(spec, page_size, max_seqs)
            num_pages = (max_tokens + page_size - 1) // page_size
        from .models.build import parse_dtype
        self.engine = Engine(self.model, page_size=page_size, num_pages=num_pages,
                             max_requests=max_seqs,
                             kv_dtype=parse_dtype(kv_dtype) if kv_dtype else None,
                             debug_tables=debug_tables)
        self.scheduler_options = dict(max_step_tokens=max_step_tokens, chunk_size=chunk_size,
                                      max_seqs=max_seqs, eos_token_ids=spec.eos_token_ids,
                                      multi_step=multi_step)

    @classmethod
    def from_config(cls, config, seed: int = 0, **options) -> "LLM":
        """An engine over random weights of ``config``, without a model folder."""
        return cls(None, config=config, random_seed=seed, **options)

    def _default_max_tokens(self, spec, page_size: int, max_seqs: int) -> int:
        from .parts.base import KVNeed, StateNeed
        want = max_seqs * spec.max_positions
        elem = 2 if self.model.ctx.compute_dtype == torch.bfloat16 else 4   # the cache's dtype
        per_token, state_bytes = 0, 0
        for need in self.model.cache_needs():
            if isinstance(need, KVNeed):
                size = elem if need.dtype is None else torch.empty((), dtype=need.dtype).element_size()
                per_token += need.n_kv_heads * (need.key_width + need.value_width) * size
            elif isinstance(need, StateNeed):
                n = max_seqs
                for d in need.shape:
                    n *= d
                state_bytes += n * torch.empty((), dtype=need.dtype).element_size()
        if self.model.ctx.device.type == "cuda" and per_token:
            free, _ = torch.cuda.mem_get_info(self.model.ctx.device)
            want = min(want, int(max(free - state_bytes, 0) * 0.5) // per_token)
        return max(page_size, want)

    def new_scheduler(self) -> Scheduler:
        return Scheduler(self.engine, **self.scheduler_options)

    def generate(self, prompts: Sequence[Sequence[int]],
                 params: Optional[SamplingParams] = None) -> List[List[int]]:
        """Generated token ids for every prompt (token ids), in the prompts' order."""
        sched = self.new_scheduler()
        plist = params if isinstance(params, (list, tuple)) else [params] * len(prompts)
        ids = [sched.add_request(p, sp) for p, sp in zip(prompts, plist)]
        finished = sched.run()
        return [finished[i].generated for i in ids]
