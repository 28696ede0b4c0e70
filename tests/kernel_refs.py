"""Plain torch references of the engine's kernels, one function per operation of
``zinfer_amd.ops`` with the same arguments.  They compute in float64 and round once to the
output's dtype.  The GPU tests compare each HIP kernel with its function here; the CPU tests
put them in the kernels' place (``install``) to drive the engine's host logic (batching,
paging, scheduling) where no GPU is present.  Nothing under ``zinfer_amd/`` imports this.
"""
from __future__ import annotations

import torch

F64 = torch.float64


def embed(table, ids, out, scale=1.0):
    out.copy_((table[ids.long()].to(F64) * float(torch.tensor(scale, dtype=torch.float32)))
              .to(out.dtype))


def scale_cap(x, scale=1.0, cap=0.0):
    v = x.to(F64) * float(torch.tensor(scale, dtype=torch.float32))
    if cap > 0:
        c = float(torch.tensor(cap, dtype=torch.float32))
        v = c * torch.tanh(v / c)
    x.copy_(v.to(x.dtype))


def rmsnorm(x, gain, eps, out):
    x64 = x.to(F64)
    inv = 1.0 / torch.sqrt((x64 * x64).sum(-1, keepdim=True) / x.shape[-1] + eps)
    out.copy_((x64 * inv * gain.to(F64)).to(out.dtype))


def can_pretile(w):
    return False


def can_fuse_swiglu(w):
    return False


def gemm_swiglu(a, w, out, w_tiled=False):
    """``w`` rows alternate in groups of 16 between gate and up."""
    N, K = w.shape
    wv = w.to(F64).view(N // 32, 2, 16, K)
    g = a.to(F64) @ wv[:, 0].reshape(N // 2, K).T
    u = a.to(F64) @ wv[:, 1].reshape(N // 2, K).T
    out.copy_((g / (1.0 + torch.exp(-g)) * u).to(out.dtype))


def gemm(a, w, out, accumulate=False, w_tiled=False):
    r = a.to(F64) @ w.to(F64).T
    if accumulate:
        r = r + out.to(F64)
    out.copy_(r.to(out.dtype))


def qk_norm_rope_kv_write(qkv, q_gain, k_gain, eps, cos, sin, positions, slot_mapping, k_pool,
                          v_pool, q_out, n_heads, n_kv_heads, head_dim, page_size):
    T = qkv.shape[0]
    hd, half = head_dim, head_dim // 2
    qw, kw = n_heads * hd, n_kv_heads * hd
    x = qkv.to(F64)
    q = x[:, :qw].reshape(T, n_heads, hd)
    k = x[:, qw:qw + kw].reshape(T, n_kv_heads, hd)
    v = x[:, qw + kw:].reshape(T, n_kv_heads, hd)

    def norm(t, g):
        if g is None:
            return t
        return t / torch.sqrt((t * t).sum(-1, keepdim=True) / hd + eps) * g.to(F64)

    def rot(t):
        if cos is None:
            return t
        c = cos.to(F64)[positions.long()][:, None, :]
        s = sin.to(F64)[positions.long()][:, None, :]
        x0, x1 = t[..., :half], t[..., half:]
        return torch.cat([x0 * c - x1 * s, x1 * c + x0 * s], dim=-1)

    q = rot(norm(q, q_gain))
    k = rot(norm(k, k_gain))
    if q_out is not None:
        q_out.copy_(q.reshape(T, qw).to(q_out.dtype))
    else:
        qkv[:, :qw] = q.reshape(T, qw).to(qkv.dtype)
    if slot_mapping is not None:
        kp = k_pool.view(-1, n_kv_heads, page_size, hd)
        vp = v_pool.view(-1, n_kv_heads, hd, page_size)     # values: rows of a page contiguous
        page = (slot_mapping // page_size).long()
        row = (slot_mapping % page_size).long()
        kp[page, :, row] = k.to(kp.dtype)
        vp[page, :, :, row] = v.to(vp.dtype)
    else:
        qkv[:, qw:qw + kw] = k.reshape(T, kw).to(qkv.dtype)


def paged_attention(q, k_pool, v_pool, block_table, q_start, ctx_len, seq_index, out, scale,
                    window, n_heads, n_kv_heads, head_dim, page_size, max_q_len, max_ctx_len,
                    n_single=None, n_query_tiles=None, q_tile_map=None, prefill_max_ctx=None,
                    prefill_variant=0):
    T = q.shape[0]
    hd = head_dim
    G = n_heads // n_kv_heads
    kp = k_pool.view(-1, n_kv_heads, page_size, hd)
    vp = v_pool.view(-1, n_kv_heads, hd, page_size)
    for t in range(T):
        s = int(seq_index[t])
        q_len = int(q_start[s + 1] - q_start[s])
        pos = int(ctx_len[s]) - q_len + (t - int(q_start[s]))
        lo = max(0, pos - window + 1) if window > 0 else 0
        keys = torch.arange(lo, pos + 1)
        pages = block_table[s].long()[keys // page_size]
        assert (pages >= 0).all(), "attention would read a page that is not held"
        rows = keys % page_size
        K = kp[pages, :, rows].to(F64)      # [n, nKV, hd]
        V = vp[pages, :, :, rows].to(F64)
        qt = q[t].to(F64).reshape(n_heads, hd)
        Kx = K.repeat_interleave(G, dim=1)  # [n, nH, hd]
        Vx = V.repeat_interleave(G, dim=1)
        sc = torch.einsum("hd,nhd->hn", qt, Kx) * scale
        a = torch.softmax(sc, dim=-1)
        out[t] = torch.einsum("hn,nhd->hd", a, Vx).reshape(-1).to(out.dtype)


def swiglu(gate_up, out):
    I = out.shape[1]
    g = gate_up[:, :I].to(F64)
    u = gate_up[:, I:].to(F64)
    out.copy_((g / (1.0 + torch.exp(-g)) * u).to(out.dtype))


def gather_rows(x, idx, out):
    out.copy_(x[idx.long()])


def argmax(logits, out):
    out.copy_(torch.argmax(logits, dim=-1).to(torch.int32))


ALL = ("embed", "rmsnorm", "gemm", "can_pretile", "can_fuse_swiglu", "gemm_swiglu", "qk_norm_rope_kv_write", "paged_attention", "swiglu",
       "gather_rows", "argmax", "scale_cap")


def install(monkeypatch):
    """Puts these functions in the place of the HIP wrappers (CPU tests of host logic only)."""
    import zinfer_amd.ops as ops
    for name in ALL:
        monkeypatch.setattr(ops, name, globals()[name])


# ------------------------------------------------------------------- pool layouts
def tile_k_pool(k_pool, n_kv_heads, page_size, hd):
    """[page, kv head, row, hd] -> the MFMA attention kernels' order: every group of 16 rows
    as [hd / 32][16 * ((d % 32) / 8) + row][d % 8]."""
    p = k_pool.view(-1, n_kv_heads, page_size // 16, 16, hd // 32, 4, 8)
    return p.permute(0, 1, 2, 4, 5, 3, 6).contiguous().view(k_pool.shape)


def tile_v_pool(v_pool, n_kv_heads, page_size, hd):
    """[page, kv head, hd, row] -> every group of 16 rows as
    [hd / 16][16 * (row / 4) + d % 16][row % 4]."""
    p = v_pool.view(-1, n_kv_heads, hd // 16, 16, page_size // 16, 4, 4)
    return p.permute(0, 1, 4, 2, 5, 3, 6).contiguous().view(v_pool.shape)
