"""The product's host sampler against the plain one and the reference's own vectors
(src/sampling/sampler.zig:203-268)."""
import numpy as np
import pytest

import plain
from zinfer_amd.sampling import (SamplingParams, Xoshiro256pp, sample_token, thinking_defaults)


def test_reference_vectors():
    rng = Xoshiro256pp(1)
    assert sample_token(np.array([0.2, 1.2, 0.9], np.float32), [], SamplingParams(temperature=0.0, top_k=20), rng) == 1
    for _ in range(16):
        assert sample_token(np.array([5.0, 4.0, 1.0, 0.5], np.float32), [],
                            SamplingParams(temperature=1.0, top_k=2), rng) in (0, 1)
    assert sample_token(np.array([5.0, 4.0], np.float32), [0],
                        SamplingParams(temperature=0.0, presence_penalty=2.0), rng) == 1
    assert sample_token(np.array([6.0, 5.0], np.float32), [0],
                        SamplingParams(temperature=0.0, repetition_penalty=2.0), rng) == 1
    for _ in range(16):
        assert sample_token(np.array([10.0, 9.0, 0.0], np.float32), [],
                            SamplingParams(temperature=1.0, min_p=0.5), rng) in (0, 1)


def test_random_stream_matches_plain():
    a, b = Xoshiro256pp(12345), plain.PlainRng(12345)
    assert [a.next_u64() for _ in range(20)] == [b.next() for _ in range(20)]
    assert 0.0 <= a.float64() < 1.0


@pytest.mark.parametrize("params", [
    dict(temperature=0.8, top_k=50), dict(temperature=0.7, top_k=20, top_p=0.8, repetition_penalty=1.1),
    dict(temperature=0.6, top_k=20, top_p=0.95, repetition_penalty=1.1),
    dict(temperature=1.0, top_k=0, min_p=0.05), dict(temperature=1.3, top_k=0, top_p=0.9),
    dict(temperature=1.0, top_k=5, presence_penalty=0.5, frequency_penalty=0.3),
    dict(temperature=0.0, repetition_penalty=1.3), dict(temperature=1.0, top_k=1),
    dict(temperature=0.9, top_k=2000, top_p=0.5, min_p=0.01)])
def test_same_token_as_plain_sampler(params):
    rs = np.random.RandomState(3)
    for trial in range(25):
        V = int(rs.choice([7, 100, 1000]))
        logits = (rs.randn(V) * 3).astype(np.float32)
        history = rs.randint(0, V + 3, size=rs.randint(0, 30)).tolist()
        seed = int(rs.randint(0, 1 << 30))
        want = plain.sample_token(logits, history, params, plain.PlainRng(seed))
        got = sample_token(logits, history, SamplingParams(**params), Xoshiro256pp(seed))
        assert got == want, (trial, V, params)


def test_distribution_is_softmax_when_nothing_is_cut():
    logits = np.array([1.0, 2.0, 0.0, -1.0], np.float32)
    p = np.exp(logits / 0.7) / np.exp(logits / 0.7).sum()
    rng = Xoshiro256pp(7)
    n = 20000
    counts = np.bincount([sample_token(logits, [], SamplingParams(temperature=0.7), rng)
                          for _ in range(n)], minlength=4)
    chi2 = ((counts - n * p) ** 2 / (n * p)).sum()
    assert chi2 < 16.3          # 3 degrees of freedom, p = 0.001


def test_command_line_presets():
    """src/app/cli/args.zig:352-373"""
    a, b = thinking_defaults(False), thinking_defaults(True)
    assert (a.temperature, a.top_k, a.top_p, a.repetition_penalty) == (0.7, 20, 0.8, 1.1)
    assert (b.temperature, b.top_k, b.top_p, b.repetition_penalty) == (0.6, 20, 0.95, 1.1)


def test_order_vectors():
    """Where the order of the sampler's operations decides the token: the same cases that pin
    the plain sampler."""
    import sampler_vectors as sv
    for logits, history, params, us, want, why in sv.ORDER_CASES:
        for u in us:
            got = sample_token(np.array(logits, np.float32), history, SamplingParams(**params),
                               sv.FixedU(u))
            assert got == want, f"{why}: u = {u}: token {got}, not {want}"
