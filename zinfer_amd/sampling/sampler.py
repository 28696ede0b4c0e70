"""Sampling with the reference's options and order of operations
(`src/sampling/sampler.zig:8-16` options, `:18-91` sampleToken, `:186-201` penalties).

This host sampler is the definition; the device kernels (``zinfer_amd.ops.argmax`` and the
top-k sampler) are checked against it.  The random stream is xoshiro256++ seeded through
SplitMix64 with ``float64 = (next() >> 11) * 2^-53`` (the construction behind the
reference's ``std.Random.DefaultPrng``, `src/app/cli/runtime/generator.zig:100`); the stream
is documented here and need not be bit-compatible with Zig's.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Dict, Optional, Sequence, Tuple

import numpy as np

_M = (1 << 64) - 1


@dataclass
class SamplingParams:
    """Defaults are the reference's struct defaults (`sampler.zig:8-16`); ``top_k`` 0 keeps
    every token.  ``max_new_tokens`` 64 is the reference's default for ``generate``
    (`src/app/cli/args.zig:100`)."""
    temperature: float = 1.0
    top_k: int = 0
    top_p: float = 1.0
    min_p: float = 0.0
    presence_penalty: float = 0.0
    frequency_penalty: float = 0.0
    repetition_penalty: float = 1.0
    seed: int = 0
    max_new_tokens: int = 64
    ignore_eos: bool = False
    stop_token_ids: Tuple[int, ...] = ()

    @property
    def greedy(self) -> bool:
        """`sampler.zig:30`: temperature <= 0 or top_k == 1 takes the arg-max."""
        return self.temperature <= 0.0 or self.top_k == 1

    @property
    def has_penalties(self) -> bool:
        return (self.repetition_penalty > 0.0 and self.repetition_penalty != 1.0) or \
            self.presence_penalty != 0.0 or self.frequency_penalty != 0.0


def thinking_defaults(think: bool) -> SamplingParams:
    """The command line's presets (`src/app/cli/args.zig:352-373`)."""
    if think:
        return SamplingParams(temperature=0.6, top_k=20, top_p=0.95, repetition_penalty=1.1)
    return SamplingParams(temperature=0.7, top_k=20, top_p=0.8, repetition_penalty=1.1)


class Xoshiro256pp:
    def __init__(self, seed: int):
        x = seed & _M
        self.s = []
        for _ in range(4):
            x = (x + 0x9E3779B97F4A7C15) & _M
            z = x
            z = ((z ^ (z >> 30)) * 0xBF58476D1CE4E5B9) & _M
            z = ((z ^ (z >> 27)) * 0x94D049BB133111EB) & _M
            self.s.append(z ^ (z >> 31))

    def next_u64(self) -> int:
        s0, s1, s2, s3 = self.s
        t = (s0 + s3) & _M
        result = ((((t << 23) | (t >> 41)) & _M) + s0) & _M
        t = (s1 << 17) & _M
        s2 ^= s0
        s3 ^= s1
        s1 ^= s2
        s0 ^= s3
        s2 ^= t
        s3 = ((s3 << 45) | (s3 >> 19)) & _M
        self.s = [s0, s1, s2, s3]
        return result

    def float64(self) -> float:
        return (self.next_u64() >> 11) * (2.0 ** -53)


def count_history(history: Sequence[int], vocab: int) -> Dict[int, int]:
    """`sampler.zig:107-122`: ids beyond the vocabulary are ignored."""
    counts: Dict[int, int] = {}
    for t in history:
        if 0 <= t < vocab:
            counts[t] = counts.get(t, 0) + 1
    return counts


def adjust_logits(logits: np.ndarray, counts: Dict[int, int], p: SamplingParams) -> np.ndarray:
    """Repetition (negative logits multiplied, others divided), presence, frequency, in this
    order, for seen tokens only (`sampler.zig:186-201`)."""
    if not counts or not p.has_penalties:
        return logits
    out = logits.astype(np.float32, copy=True)
    ids = np.fromiter(counts.keys(), dtype=np.int64, count=len(counts))
    cnt = np.fromiter(counts.values(), dtype=np.float32, count=len(counts))
    v = out[ids]
    rp = np.float32(p.repetition_penalty)
    if rp > 0.0 and rp != 1.0:
        v = np.where(v < 0.0, v * rp, v / rp).astype(np.float32)
    v = (v - np.float32(p.presence_penalty)).astype(np.float32)
    v = (v - cnt * np.float32(p.frequency_penalty)).astype(np.float32)
    out[ids] = v
    return out


def top_k_candidates(adj: np.ndarray, k: int) -> Tuple[np.ndarray, np.ndarray]:
    """Ids and values of the k largest, descending.  Among equal values the lower id comes
    first (the reference's order among exact ties follows its replace-the-minimum scan,
    `sampler.zig:143-184`, and only matters for exactly equal logits)."""
    V = adj.shape[0]
    if k >= V:
        order = np.argsort(-adj, kind="stable")
    else:
        part = np.argpartition(-adj, k - 1)[:k]
        # everything equal to the k-th value competes by id
        kth = adj[part].min()
        above = np.nonzero(adj > kth)[0]
        equal = np.nonzero(adj == kth)[0][:k - above.shape[0]]
        ids = np.concatenate([above, equal])
        order = ids[np.argsort(-adj[ids], kind="stable")]
    return order, adj[order]


def sample_token(logits: np.ndarray, history: Sequence[int], p: SamplingParams,
                 rng: Xoshiro256pp) -> int:
    """One token id from a row of float32 logits (`sampler.zig:18-91`)."""
    logits = np.asarray(logits, dtype=np.float32)
    V = logits.shape[0]
    if V == 0:
        raise ValueError("EmptyLogits")
    adj = adjust_logits(logits, count_history(history, V), p)
    if p.greedy:
        return int(np.argmax(adj))            # first maximum wins (`:124-141`)
    k = V if p.top_k == 0 else min(p.top_k, V)
    ids, vals = top_k_candidates(adj, k)
    scaled = (vals / np.float32(p.temperature)).astype(np.float32)
    probs = np.exp((scaled - scaled.max()).astype(np.float32)).astype(np.float32)
    total = float(probs.astype(np.float64).sum())
    if total <= 0.0:
        return int(ids[0])
    keep = ids.shape[0]
    min_p = float(min(max(np.float32(p.min_p), np.float32(0.0)), np.float32(1.0)))
    if min_p > 0.0:
        thr = np.float32(probs[0] * np.float32(min_p))
        below = np.nonzero(probs < thr)[0]
        keep = max(int(below[0]) if below.shape[0] else keep, 1)
        total = float(probs[:keep].astype(np.float64).sum())
    top_p = float(min(max(np.float32(p.top_p), np.float32(0.0)), np.float32(1.0)))
    if top_p < 1.0:
        cum = np.cumsum(probs[:keep].astype(np.float64) / total)
        hit = np.nonzero(cum >= top_p)[0]
        n = int(hit[0]) + 1 if hit.shape[0] else keep
        keep = min(max(n, 1), keep)
    kept = probs[:keep].astype(np.float64)
    kept_sum = float(kept.sum())
    if kept_sum <= 0.0:
        return int(ids[0])
    threshold = rng.float64() * kept_sum
    rest = threshold - np.cumsum(kept)
    hit = np.nonzero(rest <= 0.0)[0]
    return int(ids[int(hit[0])]) if hit.shape[0] else int(ids[keep - 1])
