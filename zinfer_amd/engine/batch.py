"""What one step runs: for each request its next tokens, and where logits are wanted."""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Dict, List, Optional, Sequence

import numpy as np
import torch


@dataclass
class StepEntry:
    """``tokens`` are the request's next tokens (a portion of its prompt, or one decoded
    token); ``want`` the places among them whose logits are asked for."""
    request_id: object
    tokens: Sequence[int]
    want: Sequence[int] = ()


@dataclass
class KVStepTables:
    block_table: torch.Tensor     # int32 [n_seqs, max_pages]; -1 where no page is held
    slot_mapping: torch.Tensor    # int32 [T]: page * page_size + row, for the write
    max_pages: int


class Scratch:
    """Named work buffers that live across steps and grow when a step needs more, so that a
    step allocates nothing once sizes have settled."""

    def __init__(self, device):
        self.device = device
        self._bufs: Dict[str, torch.Tensor] = {}
        self._views: Dict[str, Dict[tuple, torch.Tensor]] = {}   # per buffer: (shape, dtype) -> view
        self.generation = 0            # goes up whenever a buffer moves (captured graphs die)

    def get(self, name: str, shape, dtype: torch.dtype) -> torch.Tensor:
        key = (tuple(shape), dtype)
        views = self._views.get(name)
        if views is not None:
            view = views.get(key)
            if view is not None:
                return view
        n = 1
        for d in shape:
            n *= int(d)
        size = _ELEMENT_SIZE.get(dtype) or torch.empty((), dtype=dtype).element_size()
        nbytes = max(n, 1) * size
        buf = self._bufs.get(name)
        if buf is None or buf.numel() < nbytes:
            buf = torch.empty(((nbytes + 255) // 256 * 256,), dtype=torch.uint8, device=self.device)
            self._bufs[name] = buf
            self._views[name] = {}
            self.generation += 1
        view = buf[:n * size].view(dtype).view(*shape)
        self._views[name][key] = view
        return view


_ELEMENT_SIZE = {torch.float32: 4, torch.bfloat16: 2, torch.int32: 4, torch.int64: 8,
                 torch.float16: 2, torch.uint8: 1, torch.float64: 8}


@dataclass
class StepContext:
    """Everything the parts may read about the step.  Device tensors are int32."""
    n_tokens: int
    n_seqs: int
    n_want: int
    token_ids: torch.Tensor       # [T]
    positions: torch.Tensor       # [T] absolute position of each token in its request
    seq_index: torch.Tensor       # [T] which sequence of this step a token belongs to
    q_start: torch.Tensor         # [n_seqs + 1] first token of each sequence in the batch
    ctx_len: torch.Tensor         # [n_seqs] tokens the request holds after this step
    state_slots: torch.Tensor     # [n_seqs] slot of each request's fixed-size state
    want_rows: torch.Tensor       # [n_want] token rows whose logits are wanted
    kv: List[KVStepTables]
    max_q_len: int
    max_ctx_len: int
    q_lens: List[int]             # host copies, for parts that loop on the host
    ctx_lens: List[int]
    slots: List[int]
    # what parts asked to know about the step's shape (``Part.step_hints``), by their
    # ``hint_key``: ``StepHints`` whose arrays are int32 views on the device
    hints: Dict[object, object] = field(default_factory=dict)
    meta_offset: int = 0          # address of the packed metadata (part of a graph's key)
    wants_all_rows: bool = False  # want_rows is 0, 1, ..., n_tokens - 1
    # A part that adds into the residual stream may, in the same kernel, leave what the norm
    # reading the stream next needs (``Linear.forward(..., step=step)``): ``norm_after`` is
    # that norm (set by whoever calls the part), ``norm_ready`` what was left for it.
    norm_after: object = None
    norm_after_block: object = None   # the norm that reads the stream first after this block
    norm_ready: object = None
    _scratch: Scratch = None

    def scratch(self, name: str, shape, dtype) -> torch.Tensor:
        return self._scratch.get(name, shape, dtype)

    def kv_tables(self, group: int) -> KVStepTables:
        return self.kv[group]
