"""Pins the plain implementation by what fixes it beside the reference's text: vectors the
reference's own tests hold, special cases that reduce to a library routine, and invariants,
each chosen so that a plausible mistake (a wrong sign or pairing, a norm in the wrong place,
a wrong head mapping) fails it."""
import math

import numpy as np
import pytest
import torch

import plain
import tiny

F64 = torch.float64


# ------------------------------------------------------------------ vectors of the reference
def test_rms_norm_vector():
    """src/kernel/core/cpu.zig:193-204"""
    out = plain.rms_norm(torch.tensor([3.0, 4.0]), torch.tensor([1.0, 2.0]), 0.0)
    assert torch.allclose(out, torch.tensor([0.84852814, 2.2627418], dtype=F64), atol=1e-6)


def test_rms_norm_repeated_vector():
    """src/kernel/core/cpu.zig:274-287: the same pair twice."""
    out = plain.per_head_rms_norm(torch.tensor([3.0, 4.0, 6.0, 8.0]), 2, 2,
                                  torch.tensor([1.0, 2.0]), 0.0)
    assert torch.allclose(out, torch.tensor([0.84852814, 2.2627418] * 2, dtype=F64), atol=1e-6)


def test_swiglu_vector():
    """src/kernel/core/cpu.zig:233-245"""
    out = plain.swiglu(torch.tensor([0.0, 1.0, -1.0]), torch.tensor([1.0, 2.0, 3.0]))
    assert torch.allclose(out, torch.tensor([0.0, 1.4621172, -0.8068243], dtype=F64), atol=1e-6)


def test_linear_vector():
    """src/kernel/core/cpu.zig:177-191, src/tensor/storage/store.zig:562-603"""
    out = plain.linear(torch.tensor([1.0, 0.5, -1.0]),
                       torch.tensor([[1.0, 2.0, 3.0], [4.0, 5.0, 6.0]]))
    assert torch.allclose(out, torch.tensor([-1.0, 0.5], dtype=F64))


def test_rope_vectors():
    """src/kernel/attention/rope.zig:145-155 (position 0 is the identity) and :174-190 (the
    pairing (i, i + hd/2) and the frequency theta^(-2i/hd))."""
    x = torch.tensor([1.0, 2.0, 3.0, 4.0])
    assert torch.equal(plain.rope_head(x, 0, 10000.0), x.to(F64))
    out = plain.rope_head(x, 1, 10000.0)
    a = 1.0 / math.sqrt(10000.0)
    want = torch.tensor([math.cos(1) - 3 * math.sin(1), 2 * math.cos(a) - 4 * math.sin(a),
                         3 * math.cos(1) + math.sin(1), 4 * math.cos(a) + 2 * math.sin(a)])
    assert torch.allclose(out, want.to(F64), atol=1e-6)


def test_bf16_vectors():
    """src/tensor/formats/bfloat16.zig:15-29: 0x3f80 = 1, 0xbf80 = -1, 0x4000 = 2; 0, 1 and
    -2.5 survive the round trip; rounding is to nearest even."""
    x = torch.tensor([0.0, 1.0, -1.0, 2.0, -2.5])
    assert torch.equal(plain.bf16_round(x), x)
    bits = lambda v: np.float32(v).view(np.uint32) >> 16
    assert bits(1.0) == 0x3F80 and bits(-1.0) == 0xBF80 and bits(2.0) == 0x4000
    r = torch.randn(1000)
    assert torch.equal(plain.bf16_round(r), r.to(torch.bfloat16).float())
    # 1 + 2^-8 lies halfway between 1 and 1 + 2^-7: the even neighbour (1) wins
    assert plain.bf16_round(torch.tensor([1.0 + 2.0 ** -8]))[0] == 1.0
    assert plain.bf16_round(torch.tensor([1.0 + 3 * 2.0 ** -8]))[0] == 1.0 + 2.0 ** -6


def test_attention_gqa_vectors():
    """src/kernel/attention/basic.zig:178-252: one cached token -> every head returns its kv
    head's value row; 4 query heads on 2 kv heads -> heads 0, 1 read kv 0 and heads 2, 3 read
    kv 1 (h // G, not h % nKV).  src/model/layers/gqa_attention/spec.zig:41-44."""
    hd = 4
    q = torch.randn(4 * hd)
    K = torch.randn(1, 2, hd)
    V = torch.tensor([[[1.0, 2.0, 3.0, 4.0], [5.0, 6.0, 7.0, 8.0]]])
    out = plain.attention_single_query(q, K, V, 4, 2, hd).reshape(4, hd)
    assert torch.allclose(out[0], V[0, 0].to(F64)) and torch.allclose(out[1], V[0, 0].to(F64))
    assert torch.allclose(out[2], V[0, 1].to(F64)) and torch.allclose(out[3], V[0, 1].to(F64))


def test_softmax_vector():
    """src/kernel/attention/basic.zig:133-143: sums to one, monotone."""
    a = plain.softmax(torch.tensor([1.0, 2.0, 3.0], dtype=F64))
    assert abs(float(a.sum()) - 1.0) < 1e-12 and a[0] < a[1] < a[2]


# ------------------------------------------------------------------ library special cases
def test_rms_norm_is_library_rms_norm():
    x = torch.randn(5, 48, dtype=F64)
    w = torch.rand(48, dtype=F64) + 0.5
    want = torch.nn.functional.rms_norm(x, (48,), w, 1e-5)
    assert torch.allclose(plain.rms_norm(x, w, 1e-5), want, atol=1e-12)


def test_attention_without_rotation_is_library_sdpa():
    """The attention of whole sequences equals torch's scaled_dot_product_attention with a
    causal mask and grouped heads laid out [nKV, S, hd]."""
    S, nH, nKV, hd = 9, 6, 2, 8
    q = torch.randn(S, nH * hd, dtype=F64)
    K = torch.randn(S, nKV, hd, dtype=F64)
    V = torch.randn(S, nKV, hd, dtype=F64)
    got = torch.stack([plain.attention_single_query(q[t], K[:t + 1], V[:t + 1], nH, nKV, hd)
                       for t in range(S)])
    want = torch.nn.functional.scaled_dot_product_attention(
        q.reshape(S, nH, hd).transpose(0, 1)[None], K.transpose(0, 1)[None],
        V.transpose(0, 1)[None], is_causal=True, enable_gqa=True)[0]
    assert torch.allclose(got, want.transpose(0, 1).reshape(S, nH * hd), atol=1e-12)


def test_one_head_is_plain_attention():
    S, hd = 7, 16
    q = torch.randn(hd, dtype=F64)
    K = torch.randn(S, 1, hd, dtype=F64)
    V = torch.randn(S, 1, hd, dtype=F64)
    a = torch.softmax(K[:, 0] @ q / math.sqrt(hd), dim=0)
    assert torch.allclose(plain.attention_single_query(q, K, V, 1, 1, hd), a @ V[:, 0], atol=1e-12)


def test_swiglu_and_linear_are_library_routines():
    g, u = torch.randn(33, dtype=F64), torch.randn(33, dtype=F64)
    assert torch.allclose(plain.swiglu(g, u), torch.nn.functional.silu(g) * u, atol=1e-12)
    x, w = torch.randn(4, 10, dtype=F64), torch.randn(6, 10, dtype=F64)
    assert torch.allclose(plain.linear(x, w), torch.nn.functional.linear(x, w), atol=1e-12)
    # a one-hot input picks a column of the weight (the reference's probe-linear)
    e = torch.zeros(10, dtype=F64); e[3] = 1.0
    assert torch.allclose(plain.linear(e, w), w[:, 3])


# ------------------------------------------------------------------ invariants
def test_rope_depends_on_distance_only_and_keeps_norms():
    hd, theta = 16, 10000.0
    q, k = torch.randn(hd, dtype=F64), torch.randn(hd, dtype=F64)
    base = (plain.rope_head(q, 7, theta) * plain.rope_head(k, 3, theta)).sum()
    for shift in (1, 20, 100):
        moved = (plain.rope_head(q, 7 + shift, theta) * plain.rope_head(k, 3 + shift, theta)).sum()
        assert abs(float(moved - base)) < 1e-4      # the angle is formed in 32-bit
    r = plain.rope_head(q, 11, theta)
    half = hd // 2
    assert torch.allclose(r[:half] ** 2 + r[half:] ** 2, q[:half] ** 2 + q[half:] ** 2, atol=1e-12)
    # a swapped sign would turn the rotation around: q rotated by +p then -p must not be q
    assert not torch.allclose(r, q)


def test_heads_are_normed_independently():
    x = torch.randn(3 * 8, dtype=F64)
    w = torch.rand(8, dtype=F64) + 0.5
    a = plain.per_head_rms_norm(x, 3, 8, w, 1e-6)
    y = x.clone(); y[8:16] *= 5.0
    b = plain.per_head_rms_norm(y, 3, 8, w, 1e-6)
    assert torch.allclose(a[:8], b[:8]) and torch.allclose(a[16:], b[16:])
    assert torch.allclose(a[8:16], b[8:16], atol=1e-6)    # scale-invariant up to eps


def test_future_tokens_have_no_influence():
    cfg, w = tiny.CONFIGS["A"], tiny.weights_of("A")
    toks = tiny.random_tokens(12, cfg["vocab_size"], 1)
    a = plain.model_forward_batched(cfg, w, toks)
    toks2 = list(toks); toks2[8] = (toks2[8] + 1) % cfg["vocab_size"]
    b = plain.model_forward_batched(cfg, w, toks2)
    assert torch.equal(a[:8], b[:8]) and not torch.allclose(a[8:], b[8:])


def test_zero_output_projections_make_layers_the_identity():
    """With W_o = W_down = 0 every block is the identity: logits = W_lm RMS(E[id])."""
    cfg, w = tiny.CONFIGS["B"], dict(tiny.weights_of("B"))
    for l in range(cfg["num_hidden_layers"]):
        for s in ("self_attn.o_proj.weight", "mlp.down_proj.weight"):
            w[plain.layer_name(l, s)] = torch.zeros_like(w[plain.layer_name(l, s)])
    toks = [5, 900, 17]
    got = plain.model_forward_batched(cfg, w, toks)
    x = w["model.embed_tokens.weight"][torch.tensor(toks)]
    want = plain.linear(plain.rms_norm(x, w["model.norm.weight"], cfg["rms_norm_eps"]),
                        w["lm_head.weight"])
    assert torch.allclose(got, want, atol=1e-12)


def test_norm_sits_before_the_mixer_and_residual_is_unnormed():
    """One token through one block with W_down = 0: out = x + W_o W_v norm(x).  The branch sees
    the normed input, so it is the same for x and 3x (up to eps) and the outputs differ by
    exactly 2x; a norm after the mixer, or a residual taken from the normed input, would not
    give that."""
    cfg, w = tiny.CONFIGS["A"], dict(tiny.weights_of("A"))
    name = plain.layer_name(0, "mlp.down_proj.weight")
    w[name] = torch.zeros_like(w[name])
    x = torch.randn(cfg["hidden_size"], dtype=F64)
    out1 = plain.block_token(cfg, w, 0, x, 0, [], [])
    out3 = plain.block_token(cfg, w, 0, 3.0 * x, 0, [], [])
    assert (out3 - out1 - 2.0 * x).abs().max() < 1e-5
    assert (out1 - x).abs().max() > 1e-3          # the branch does add something


@pytest.mark.parametrize("name", ["A", "B", "C"])
def test_token_by_token_equals_batched(name):
    cfg, w = tiny.CONFIGS[name], tiny.weights_of(name)
    toks = tiny.random_tokens(7, cfg["vocab_size"], 3)
    a = plain.model_forward(cfg, w, toks)
    b = plain.model_forward_batched(cfg, w, toks)
    assert torch.allclose(a, b, atol=1e-12)


def test_window_restricts_to_last_positions():
    cfg, w = tiny.CONFIGS["A"], tiny.weights_of("A")
    toks = tiny.random_tokens(10, cfg["vocab_size"], 4)
    full = plain.model_forward_batched(cfg, w, toks)
    win = plain.model_forward_batched(cfg, w, toks, window=4)
    assert torch.allclose(full[:4], win[:4], atol=1e-12)     # the window has not filled yet
    assert not torch.allclose(full[4:], win[4:])
    assert torch.allclose(win[:7], plain.model_forward(cfg, w, toks[:7], window=4), atol=1e-12)


# ------------------------------------------------------------------ sampler
def test_sampler_vectors():
    """src/sampling/sampler.zig:203-268."""
    rng = plain.PlainRng(1)
    assert plain.sample_token(np.array([0.2, 1.2, 0.9], np.float32), [],
                              dict(temperature=0.0, top_k=20), rng) == 1
    for _ in range(16):
        assert plain.sample_token(np.array([5.0, 4.0, 1.0, 0.5], np.float32), [],
                                  dict(temperature=1.0, top_k=2), rng) in (0, 1)
    assert plain.sample_token(np.array([5.0, 4.0], np.float32), [0],
                              dict(temperature=0.0, presence_penalty=2.0), rng) == 1
    assert plain.sample_token(np.array([6.0, 5.0], np.float32), [0],
                              dict(temperature=0.0, repetition_penalty=2.0), rng) == 1
    for _ in range(16):
        assert plain.sample_token(np.array([10.0, 9.0, 0.0], np.float32), [],
                                  dict(temperature=1.0, min_p=0.5, top_k=0), rng) in (0, 1)
    assert plain.sample_token(np.array([1.0, 3.0, 3.0], np.float32), [], dict(temperature=0.0),
                              rng) == 1        # the first maximum wins


def test_rng_is_xoshiro256pp():
    """Known first outputs of xoshiro256++ for the state {1, 2, 3, 4}."""
    r = plain.PlainRng(0)
    r.s = [1, 2, 3, 4]
    assert [r.next() for _ in range(3)] == [41943041, 58720359, 3588806011781223]


def test_sampler_order_vectors():
    """Where the order of the sampler's operations decides the token."""
    import sampler_vectors as sv
    for logits, history, params, us, want, why in sv.ORDER_CASES:
        for u in us:
            got = plain.sample_token(np.array(logits, np.float32), history, params, sv.FixedU(u))
            assert got == want, f"{why}: u = {u}: token {got}, not {want}"


def test_qk_norm_sits_before_the_rotation():
    """Scores may depend on the distance between query and key only, so a block's output does
    not change when all positions move by the same amount.  With per-head gains that differ
    inside a rotated pair (i, i + hd/2), that holds only if the norm comes before the rotation
    (`layer.zig:114-128`): a gain applied after it does not commute with the rotation."""
    cfg, w = tiny.CONFIGS["B"], dict(tiny.weights_of("B"))
    hd, nH, nKV, theta = cfg["head_dim"], cfg["num_attention_heads"], cfg["num_key_value_heads"], \
        cfg["rope_theta"]
    g = torch.Generator().manual_seed(9)
    for l in range(cfg["num_hidden_layers"]):
        for n in ("q_norm", "k_norm"):        # gains far from 1 and unequal inside every pair
            w[plain.layer_name(l, f"self_attn.{n}.weight")] = 0.5 + 2.0 * torch.rand(hd, generator=g)
    xs = torch.randn(6, cfg["hidden_size"], generator=g, dtype=torch.float32).to(F64)

    def run(shift):
        keys, values, out = [], [], []
        # the cache is pre-filled with `shift` unreadable entries through a window, so the
        # token at list index `shift + t` has position `shift + t` and sees only tokens >= shift
        for _ in range(shift):
            keys.append(torch.zeros(nKV, hd, dtype=F64)); values.append(torch.zeros(nKV, hd, dtype=F64))
        for t in range(xs.shape[0]):
            out.append(plain.block_token(cfg, w, 0, xs[t], shift + t, keys, values, window=t + 1))
        return torch.stack(out)
    base = run(0)
    for shift in (1, 13, 200):
        assert (run(shift) - base).abs().max() < 2e-4 * base.abs().max()
    # the invariant notices the other order: gains applied after the rotation
    q = torch.randn(hd, generator=g).to(F64); k = torch.randn(hd, generator=g).to(F64)
    gq = w[plain.layer_name(0, "self_attn.q_norm.weight")].to(F64)
    gk = w[plain.layer_name(0, "self_attn.k_norm.weight")].to(F64)
    one = torch.ones(hd, dtype=F64)

    def wrong(pq, pk):
        a = plain.rope_head(plain.rms_norm(q, one, 1e-6), pq, theta) * gq
        b = plain.rope_head(plain.rms_norm(k, one, 1e-6), pk, theta) * gk
        return float((a * b).sum())

    def right(pq, pk):
        a = plain.rope_head(plain.rms_norm(q, gq, 1e-6), pq, theta)
        b = plain.rope_head(plain.rms_norm(k, gk, 1e-6), pk, theta)
        return float((a * b).sum())
    assert abs(right(5, 2) - right(18, 15)) < 1e-4
    assert abs(wrong(5, 2) - wrong(18, 15)) > 1e-2
