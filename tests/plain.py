"""Plain, slow implementation of the Qwen3 dense decoder, written from the formulas of
NeoZedAtlas/Zinfer's CPU engine (file:line citations are relative to that repository).

Whole sequences, no cache, one function for each part, float64 arithmetic on the CPU.
It shares no code with the engine under ``zinfer_amd/``: it is the oracle the engine is
compared with.  Weights come in as a ``dict`` of HF tensor names to ``torch.Tensor`` and are
widened to float64; only the rotation angles follow the reference's 32-bit arithmetic
(`src/kernel/attention/rope.zig:25-34`), because there the precision of the angle is part of
what the model computes.
"""
from __future__ import annotations

import math
from typing import Dict, List, Optional, Sequence

import numpy as np
import torch

F64 = torch.float64


# ----------------------------------------------------------------------------- parts
def linear(x: torch.Tensor, weight: torch.Tensor) -> torch.Tensor:
    """y[r] = sum_c W[r, c] * x[c]; the weight is [out, in] and there is no bias.
    `src/kernel/core/cpu.zig:21-36`, `src/tensor/storage/store.zig:286-319`."""
    w = weight.to(F64)
    out = torch.zeros(x.shape[:-1] + (w.shape[0],), dtype=F64)
    for r in range(w.shape[0]):
        out[..., r] = (x.to(F64) * w[r]).sum(dim=-1)
    return out


def rms_norm(x: torch.Tensor, weight: torch.Tensor, eps: float) -> torch.Tensor:
    """n_i = x_i * w_i / sqrt(mean(x^2) + eps): plain weight (not 1+w), eps added to the mean
    inside the root.  `src/kernel/core/cpu.zig:38-48` (rmsNorm), `:73-96` (computeInvRms),
    `:98-110` (applyRmsNormScaled)."""
    x = x.to(F64)
    mean_square = (x * x).sum(dim=-1, keepdim=True) / x.shape[-1]
    inv_rms = 1.0 / torch.sqrt(mean_square + eps)
    return x * inv_rms * weight.to(F64)


def per_head_rms_norm(x: torch.Tensor, n_heads: int, head_dim: int, weight: torch.Tensor,
                      eps: float) -> torch.Tensor:
    """RMSNorm of every head's contiguous slice [h*hd, (h+1)*hd) with one [hd] weight shared
    by all heads.  `src/kernel/core/cpu.zig:50-71` (rmsNormRepeated), called at
    `src/model/layers/rmsnorm_gqa_swiglu_block.zig:105-131`."""
    assert x.shape[-1] == n_heads * head_dim
    out = torch.empty(x.shape, dtype=F64)
    for h in range(n_heads):
        sl = slice(h * head_dim, (h + 1) * head_dim)
        out[..., sl] = rms_norm(x[..., sl], weight, eps)
    return out


def rope_cos_sin(position: int, head_dim: int, theta: float):
    """cos and sin of the head_dim/2 rotation angles at one position.  The reference forms
    the angle in 32-bit: exponent = f32(2i)/f32(hd), inv_freq = 1/pow(f32 theta, exponent),
    angle = f32(position) * inv_freq  (`src/kernel/attention/rope.zig:25-34`, `:76-83`).
    The cosine and sine of that 32-bit angle are taken exactly (float64)."""
    if head_dim == 0 or head_dim % 2 != 0:
        raise ValueError("InvalidHeadDim")  # rope.zig:16
    half = head_dim // 2
    i2 = (np.arange(half, dtype=np.float32) * np.float32(2.0))
    exponent = i2 / np.float32(head_dim)
    inv_freq = np.float32(1.0) / np.power(np.float32(theta), exponent, dtype=np.float32)
    angle = (np.float32(position) * inv_freq).astype(np.float32)
    a64 = angle.astype(np.float64)
    return torch.from_numpy(np.cos(a64)), torch.from_numpy(np.sin(a64))


def rope_head(head: torch.Tensor, position: int, theta: float) -> torch.Tensor:
    """Half-split rotation of one head: (x_i, x_{i+hd/2}) <- (x_i c - x_{i+hd/2} s,
    x_{i+hd/2} c + x_i s).  `src/kernel/attention/rope.zig:67-90`."""
    hd = head.shape[-1]
    half = hd // 2
    cos, sin = rope_cos_sin(position, hd, theta)
    x0 = head[..., :half].to(F64)
    x1 = head[..., half:].to(F64)
    return torch.cat([x0 * cos - x1 * sin, x1 * cos + x0 * sin], dim=-1)


def rope_heads(x: torch.Tensor, n_heads: int, head_dim: int, position: int,
               theta: float) -> torch.Tensor:
    """Every head of a projected vector rotated at the same position.
    `src/kernel/attention/rope.zig:111-124`, `src/model/layers/gqa_attention/forward.zig:4-28`."""
    out = torch.empty(x.shape, dtype=F64)
    for h in range(n_heads):
        sl = slice(h * head_dim, (h + 1) * head_dim)
        out[..., sl] = rope_head(x[..., sl], position, theta)
    return out


def softmax(values: torch.Tensor) -> torch.Tensor:
    """max / exp / sum / scale over a 1-D score row.  `src/kernel/attention/basic.zig:5-25`."""
    m = values.max()
    e = torch.exp(values - m)
    s = e.sum()
    if s == 0.0:
        raise ValueError("InvalidSoftmaxSum")
    return e / s


def attention_single_query(query: torch.Tensor, keys: torch.Tensor, values: torch.Tensor,
                           n_heads: int, n_kv_heads: int, head_dim: int,
                           window: Optional[int] = None) -> torch.Tensor:
    """One query token against ``seq_len`` cached positions (its own included, last).
    keys/values are token-major [seq_len, n_kv, hd].  Query head h reads kv head h // G;
    scores are scaled by 1/sqrt(hd) after the dot product; causality is the loop bound.
    `src/kernel/attention/basic.zig:27-76`, `src/model/layers/gqa_attention/spec.zig:19-25`.
    ``window`` (not in the reference, which has full attention only) restricts the query to
    the last ``window`` positions; None is the reference's behaviour."""
    if n_heads % n_kv_heads != 0:
        raise ValueError("InvalidGrouping")
    seq_len = keys.shape[0]
    group = n_heads // n_kv_heads
    scale = 1.0 / math.sqrt(float(head_dim))
    first = 0 if window is None else max(0, seq_len - window)
    out = torch.zeros(n_heads * head_dim, dtype=F64)
    for h in range(n_heads):
        q = query[h * head_dim:(h + 1) * head_dim].to(F64)
        kvh = h // group
        scores = torch.empty(seq_len - first, dtype=F64)
        for t in range(first, seq_len):
            scores[t - first] = (q * keys[t, kvh].to(F64)).sum() * scale
        a = softmax(scores)
        acc = torch.zeros(head_dim, dtype=F64)
        for t in range(first, seq_len):
            acc += a[t - first] * values[t, kvh].to(F64)
        out[h * head_dim:(h + 1) * head_dim] = acc
    return out


def silu(x: torch.Tensor) -> torch.Tensor:
    """x / (1 + exp(-x)).  `src/kernel/core/cpu.zig:130-132`."""
    return x / (1.0 + torch.exp(-x))


def swiglu(gate: torch.Tensor, up: torch.Tensor) -> torch.Tensor:
    """silu(gate) * up.  `src/kernel/core/cpu.zig:134-147`."""
    return silu(gate.to(F64)) * up.to(F64)


def bf16_round(x: torch.Tensor) -> torch.Tensor:
    """Round-to-nearest-even to bfloat16 and back to float32: (bits + 0x7fff + lsb) >> 16,
    then bits << 16.  `src/tensor/formats/bfloat16.zig:3-13`."""
    bits = x.to(torch.float32).contiguous().numpy().view(np.uint32).astype(np.uint64)
    lsb = (bits >> np.uint64(16)) & np.uint64(1)
    rounded = ((bits + np.uint64(0x7FFF) + lsb) >> np.uint64(16)) & np.uint64(0xFFFF)
    back = (rounded << np.uint64(16)).astype(np.uint32)
    return torch.from_numpy(back.view(np.float32).copy()).reshape(x.shape)


# ----------------------------------------------------------------------------- block, model
def layer_name(layer: int, suffix: str) -> str:
    """`src/model/families/qwen3/weights.zig:10-35`."""
    return f"model.layers.{layer}.{suffix}"


def block_token(cfg: dict, weights: Dict[str, torch.Tensor], layer: int, x: torch.Tensor,
                position: int, k_cache: List[torch.Tensor], v_cache: List[torch.Tensor],
                window: Optional[int] = None) -> torch.Tensor:
    """One token through one pre-norm block, in the reference's order
    (`src/model/layers/rmsnorm_gqa_swiglu_block.zig:53-184`): input norm, q/k/v projections,
    per-head norm of q and k, rotation of q and k at the token's position, append (k, v),
    attention over positions 0..p, output projection, residual, post-attention norm, SwiGLU
    MLP, residual.  ``k_cache``/``v_cache`` are this layer's lists of earlier [n_kv, hd] rows."""
    H = cfg["hidden_size"]; nH = cfg["num_attention_heads"]; nKV = cfg["num_key_value_heads"]
    hd = cfg["head_dim"]; eps = cfg["rms_norm_eps"]; theta = cfg["rope_theta"]
    w = lambda s: weights[layer_name(layer, s)]
    assert x.shape == (H,)
    n = rms_norm(x, w("input_layernorm.weight"), eps)
    q = linear(n, w("self_attn.q_proj.weight"))
    k = linear(n, w("self_attn.k_proj.weight"))
    v = linear(n, w("self_attn.v_proj.weight"))
    q = per_head_rms_norm(q, nH, hd, w("self_attn.q_norm.weight"), eps)
    k = per_head_rms_norm(k, nKV, hd, w("self_attn.k_norm.weight"), eps)
    assert position == len(k_cache)  # position = cache.len, block.zig:133
    q = rope_heads(q, nH, hd, position, theta)
    k = rope_heads(k, nKV, hd, position, theta)
    k_cache.append(k.reshape(nKV, hd))
    v_cache.append(v.reshape(nKV, hd))
    attn = attention_single_query(q, torch.stack(k_cache), torch.stack(v_cache), nH, nKV, hd,
                                  window)
    r = x.to(F64) + linear(attn, w("self_attn.o_proj.weight"))
    m = rms_norm(r, w("post_attention_layernorm.weight"), eps)
    a = swiglu(linear(m, w("mlp.gate_proj.weight")), linear(m, w("mlp.up_proj.weight")))
    return r + linear(a, w("mlp.down_proj.weight"))


def lm_head_weight(cfg: dict, weights: Dict[str, torch.Tensor]) -> torch.Tensor:
    """The reference always reads `lm_head.weight` (`src/model/runtime/optimized_decoder/
    runtime.zig:50`); with tied embeddings and no stored head the embedding stands in."""
    if "lm_head.weight" in weights:
        return weights["lm_head.weight"]
    if cfg.get("tie_word_embeddings", False):
        return weights["model.embed_tokens.weight"]
    raise KeyError("TensorNotFound: lm_head.weight")


def model_forward(cfg: dict, weights: Dict[str, torch.Tensor], token_ids: Sequence[int],
                  window: Optional[int] = None) -> torch.Tensor:
    """Logits [T, V] (float64) of a whole sequence, token after token as the reference runs
    it (`src/model/layers/decoder_only_stack.zig:48-93`): embedding row (no scale), L blocks,
    final norm, head."""
    L = cfg["num_hidden_layers"]; V = cfg["vocab_size"]
    k_caches = [[] for _ in range(L)]
    v_caches = [[] for _ in range(L)]
    head = lm_head_weight(cfg, weights)
    rows = []
    for p, tok in enumerate(token_ids):
        if tok < 0 or tok >= V:
            raise IndexError("TokenIdOutOfBounds")  # runtime.zig:109
        x = weights["model.embed_tokens.weight"][tok].to(F64)
        for l in range(L):
            x = block_token(cfg, weights, l, x, p, k_caches[l], v_caches[l], window)
        n = rms_norm(x, weights["model.norm.weight"], cfg["rms_norm_eps"])
        rows.append(linear(n, head))
    return torch.stack(rows)


# A faster whole-sequence form of the same formulas (matrix products instead of loops); the
# tests check it against ``model_forward`` and then use it for the longer sequences.
def model_forward_batched(cfg: dict, weights: Dict[str, torch.Tensor],
                          token_ids: Sequence[int], window: Optional[int] = None,
                          return_hidden: bool = False, act_round=None) -> torch.Tensor:
    """``act_round``: a rounding (such as ``bf16_round``) applied wherever an engine that
    keeps its activations in bfloat16 between kernels stores one: the normed rows, q/k/v,
    q and k after norm and rotation, the soft-max terms before they meet the values, the
    attention's output, the feed-forward's activation, the final normed rows.  The residual
    stream and every sum stay exact.  It models what such an engine's distance from the exact
    result should be; it is no reference for values."""
    rnd = (lambda t: act_round(t).to(F64)) if act_round is not None else (lambda t: t)
    H = cfg["hidden_size"]; nH = cfg["num_attention_heads"]; nKV = cfg["num_key_value_heads"]
    hd = cfg["head_dim"]; eps = cfg["rms_norm_eps"]; theta = cfg["rope_theta"]
    L = cfg["num_hidden_layers"]; G = nH // nKV
    T = len(token_ids)
    ids = torch.tensor(list(token_ids), dtype=torch.long)
    if int(ids.min()) < 0 or int(ids.max()) >= cfg["vocab_size"]:
        raise IndexError("TokenIdOutOfBounds")
    x = weights["model.embed_tokens.weight"].to(F64)[ids]
    cos = torch.stack([rope_cos_sin(p, hd, theta)[0] for p in range(T)])  # [T, hd/2]
    sin = torch.stack([rope_cos_sin(p, hd, theta)[1] for p in range(T)])

    def rot(t, n):  # t: [T, n*hd]
        t = t.reshape(T, n, hd)
        x0, x1 = t[..., :hd // 2], t[..., hd // 2:]
        c, s = cos[:, None, :], sin[:, None, :]
        return torch.cat([x0 * c - x1 * s, x1 * c + x0 * s], dim=-1)

    def headnorm(t, n, wgt):
        t = t.reshape(T, n, hd)
        ms = (t * t).sum(-1, keepdim=True) / hd
        return (t / torch.sqrt(ms + eps) * wgt.to(F64)).reshape(T, n * hd)

    pos = torch.arange(T)
    allowed = pos[None, :] <= pos[:, None]
    if window is not None:
        allowed &= pos[None, :] > pos[:, None] - window
    for l in range(L):
        w = lambda s: weights[layer_name(l, s)].to(F64)
        n = rnd(rms_norm(x, w("input_layernorm.weight"), eps))
        q = rnd(n @ w("self_attn.q_proj.weight").T)
        k = rnd(n @ w("self_attn.k_proj.weight").T)
        v = rnd(n @ w("self_attn.v_proj.weight").T)
        q = rnd(rot(headnorm(q, nH, w("self_attn.q_norm.weight")), nH))      # [T, nH, hd]
        k = rnd(rot(headnorm(k, nKV, w("self_attn.k_norm.weight")), nKV))    # [T, nKV, hd]
        v = v.reshape(T, nKV, hd)
        kx = k.repeat_interleave(G, dim=1)  # query head h reads kv head h // G
        vx = v.repeat_interleave(G, dim=1)
        s = torch.einsum("thd,shd->hts", q, kx) * (1.0 / math.sqrt(float(hd)))
        s = s.masked_fill(~allowed[None], float("-inf"))
        if act_round is None:
            a = torch.softmax(s, dim=-1)
            o = torch.einsum("hts,shd->thd", a, vx).reshape(T, nH * hd)
        else:       # the terms are rounded, their sum is not
            e = torch.exp(s - s.max(dim=-1, keepdim=True).values)
            o = torch.einsum("hts,shd->thd", rnd(e), vx) / e.sum(-1).T[:, :, None]
            o = rnd(o.reshape(T, nH * hd))
        r = x + o @ w("self_attn.o_proj.weight").T
        m = rnd(rms_norm(r, w("post_attention_layernorm.weight"), eps))
        act = rnd(swiglu(m @ w("mlp.gate_proj.weight").T, m @ w("mlp.up_proj.weight").T))
        x = r + act @ w("mlp.down_proj.weight").T
    if return_hidden:
        return x
    n = rnd(rms_norm(x, weights["model.norm.weight"], eps))
    return n @ lm_head_weight(cfg, weights).to(F64).T


# ----------------------------------------------------------------------------- sampling
class PlainRng:
    """xoshiro256++ seeded through SplitMix64, the construction of the reference's
    `std.Random.DefaultPrng.init(seed)` (`src/app/cli/runtime/generator.zig:100`);
    ``float64()`` is (next() >> 11) * 2^-53."""
    M = (1 << 64) - 1

    def __init__(self, seed: int):
        s = seed & self.M
        st = []
        for _ in range(4):
            s = (s + 0x9E3779B97F4A7C15) & self.M
            z = s
            z = ((z ^ (z >> 30)) * 0xBF58476D1CE4E5B9) & self.M
            z = ((z ^ (z >> 27)) * 0x94D049BB133111EB) & self.M
            st.append(z ^ (z >> 31))
        self.s = st

    @staticmethod
    def _rotl(x, k):
        return ((x << k) | (x >> (64 - k))) & PlainRng.M

    def next(self) -> int:
        s = self.s
        r = (self._rotl((s[0] + s[3]) & self.M, 23) + s[0]) & self.M
        t = (s[1] << 17) & self.M
        s[2] ^= s[0]; s[3] ^= s[1]; s[1] ^= s[2]; s[0] ^= s[3]
        s[2] ^= t
        s[3] = self._rotl(s[3], 45)
        return r

    def float64(self) -> float:
        return (self.next() >> 11) * (1.0 / (1 << 53))


def adjusted_logit(logit: np.float32, seen: int, cfg: dict) -> np.float32:
    """Repetition, presence and frequency penalties, in that order, only for seen tokens.
    `src/sampling/sampler.zig:186-201`."""
    a = np.float32(logit)
    if seen == 0:
        return a
    rp = np.float32(cfg.get("repetition_penalty", 1.0))
    if rp > 0.0 and rp != 1.0:
        a = a * rp if a < 0.0 else a / rp
    a = np.float32(a - np.float32(cfg.get("presence_penalty", 0.0)))
    a = np.float32(a - np.float32(seen) * np.float32(cfg.get("frequency_penalty", 0.0)))
    return np.float32(a)


def sample_token(logits: np.ndarray, history: Sequence[int], cfg: dict, rng: PlainRng) -> int:
    """`src/sampling/sampler.zig:18-91`: counts of the history, greedy when temperature <= 0
    or top_k == 1 (first maximum wins, `:124-141`), else top-k by replace-the-minimum and a
    stable descending sort (`:143-184`), exp((l/T) - max) in 32-bit with 64-bit sums, min-p
    prefix, top-p prefix on the renormalised kept set, draw u * kept_sum and walk."""
    logits = np.asarray(logits, dtype=np.float32)
    V = logits.shape[0]
    if V == 0:
        raise ValueError("EmptyLogits")
    counts: Dict[int, int] = {}
    for t in history:
        if t >= V:
            continue
        counts[t] = counts.get(t, 0) + 1
    adj = logits.copy()
    for t, c in counts.items():
        adj[t] = adjusted_logit(logits[t], c, cfg)
    temperature = float(cfg.get("temperature", 1.0))
    top_k = int(cfg.get("top_k", 0))
    if temperature <= 0.0 or top_k == 1:
        best, best_v = 0, adj[0]
        for i in range(1, V):
            if adj[i] > best_v:
                best, best_v = i, adj[i]
        return best
    k = V if top_k == 0 else min(top_k, V)
    top_ids = list(range(k))
    top_val = [adj[i] for i in range(k)]
    for cur in range(k, V):
        mi = 0
        for j in range(1, k):
            if top_val[j] < top_val[mi]:
                mi = j
        if adj[cur] > top_val[mi]:
            top_ids[mi] = cur
            top_val[mi] = adj[cur]
    order = sorted(range(k), key=lambda j: -float(top_val[j]))  # stable
    cand = [top_ids[j] for j in order]
    scaled = np.array([np.float32(top_val[j]) / np.float32(temperature) for j in order],
                      dtype=np.float32)
    probs = np.exp((scaled - scaled.max()).astype(np.float32)).astype(np.float32)
    total = float(np.sum(probs.astype(np.float64)))
    if total <= 0.0:
        return cand[0]
    keep = len(cand)
    min_p = min(max(float(np.float32(cfg.get("min_p", 0.0))), 0.0), 1.0)
    if min_p > 0.0:
        thr = np.float32(probs[0] * np.float32(min_p))
        keep = 0
        while keep < len(probs) and probs[keep] >= thr:
            keep += 1
        keep = max(keep, 1)
        total = float(np.sum(probs[:keep].astype(np.float64)))
    top_p = min(max(float(np.float32(cfg.get("top_p", 1.0))), 0.0), 1.0)
    if top_p < 1.0:
        cum = 0.0
        n = 0
        while n < keep:
            cum += float(probs[n]) / total
            if cum >= top_p:
                n += 1
                break
            n += 1
        keep = min(max(n, 1), keep)
    kept_sum = float(np.sum(probs[:keep].astype(np.float64)))
    if kept_sum <= 0.0:
        return cand[0]
    thr = rng.float64() * kept_sum
    for j in range(keep):
        thr -= float(probs[j])
        if thr <= 0.0:
            return cand[j]
    return cand[keep - 1]


def greedy_generate(cfg: dict, weights: Dict[str, torch.Tensor], prompt: Sequence[int],
                    steps: int) -> List[int]:
    """`src/app/cli/inspect.zig:246-312` (generate-token-ids): argmax of the last logits,
    first maximum wins (`src/model/layers/logits.zig:47-59`), no EOS check."""
    toks = list(prompt)
    for _ in range(steps):
        logits = model_forward_batched(cfg, weights, toks)[-1]
        toks.append(int(torch.argmax(logits)))  # torch.argmax returns the first maximum
    return toks[len(prompt):]
