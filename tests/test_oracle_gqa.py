"""Pins the CPU oracle for Qwen grouped-query attention (prepare, cached step,
whole sequence) with the reference tests' known answers and an independent
float64 formulation written from the published model equations."""
import math

import numpy as np
import pytest


def values(count, phase, scale=1.0):
    # input generator of cached_attention_ops_test.cc:33-38
    i = np.arange(count, dtype=np.float32)
    return (np.float32(scale) * np.sin(np.float32(phase) + i * np.float32(0.29))).astype(np.float32)


def sigmoid(x):
    return 1.0 / (1.0 + np.exp(-np.asarray(x, np.float64)))


def test_known_answers_zero_query_uniform_rows(oracle):
    # cached_attention_test.cc:108-156
    p = oracle.attention_params(2, 1, 4, 2, capacity=2)
    ref = oracle.CachedAttention(p)
    norm = np.zeros(4, np.float32)
    q = np.zeros(16, np.float32)
    k = np.ones(4, np.float32)
    out, probs = ref.step(q, k, [2, 4, -2, -4], norm, norm, True)
    np.testing.assert_array_equal(out.ravel(), [1, 2, -1, -2, 1, 2, -1, -2])
    np.testing.assert_array_equal(probs, np.ones((2, 1), np.float32))
    out, probs = ref.step(q, k, [4, 8, 2, 4], norm, norm, True)
    np.testing.assert_array_equal(out.ravel(), [1.5, 3, 0, 0, 1.5, 3, 0, 0])
    np.testing.assert_array_equal(probs, np.full((2, 2), 0.5, np.float32))
    with pytest.raises(OverflowError):
        ref.step(q, k, [2, 4, -2, -4], norm, norm)
    assert ref.position == 2
    ref.reset()
    out = ref.step(q, k, [2, 4, -2, -4], norm, norm)
    np.testing.assert_array_equal(out.ravel(), [1, 2, -1, -2, 1, 2, -1, -2])


def test_gate_expectation_is_exact(oracle):
    # cached_attention_ops_test.cc:364-398
    p = oracle.attention_params(2, 1, 4, 2)
    ref = oracle.CachedAttention(p)
    q = np.array([1, 2, 3, 4, -2, 0, 1, 3, 4, 3, 2, 1, 2, -1, 0, -3], np.float32)
    value = np.array([0.31, -0.9, 1.2, 2.7], np.float32)
    zero = np.zeros(4, np.float32)
    out = ref.step(q, np.ones(4, np.float32), value, zero, zero)
    expected = np.zeros(8, np.float32)
    for h in range(2):
        for d in range(4):
            gate = np.float32(1) / (np.float32(1) + np.exp(-q[(h * 2 + 1) * 4 + d], dtype=np.float32))
            expected[h * 4 + d] = oracle.bf16_round(
                oracle.bf16_round(value[d]) * oracle.bf16_round(gate))
    np.testing.assert_array_equal(out.ravel(), expected)


def test_uniform_probabilities_across_cache_tiles(oracle):
    # cached_attention_ops_test.cc:472-503: 35 steps, every row 1/length to 1e-7
    p = oracle.attention_params(2, 1, 4, 2, capacity=35)
    ref = oracle.CachedAttention(p)
    zero = np.zeros(4, np.float32)
    for length in range(1, 36):
        _, probs = ref.step(np.zeros(16, np.float32), np.ones(4, np.float32),
                            [1, 2, 3, 4], zero, zero, True)
        assert probs.shape == (2, length)
        assert np.max(np.abs(probs - 1.0 / length)) <= 1e-7


def independent_prepare(x, w, position, rotary, theta, eps):
    """RMSNorm with (1 + w) and rotate-half RoPE on the leading `rotary`
    channels, as published for Qwen3-style attention; float64, no rounding."""
    x = np.asarray(x, np.float64)
    n = x / np.sqrt(np.mean(x * x) + eps) * (1 + np.asarray(w, np.float64))
    half = rotary // 2
    inv_freq = theta ** (-np.arange(half, dtype=np.float64) * 2 / rotary)
    ang = position * inv_freq
    cos = np.concatenate([np.cos(ang), np.cos(ang)])
    sin = np.concatenate([np.sin(ang), np.sin(ang)])
    r = n[:rotary]
    rotate_half = np.concatenate([-r[half:], r[:half]])
    out = n.copy()
    out[:rotary] = r * cos + rotate_half * sin
    return out


def independent_sequence(p, qg, k, v, qw, kw):
    T = qg.shape[0]
    d, qh, kh = p.head_dim, p.query_heads, p.key_value_heads
    Q = np.zeros((T, qh, d)); K = np.zeros((T, kh, d))
    for t in range(T):
        for h in range(qh):
            Q[t, h] = independent_prepare(qg[t, h, 0], qw, t, p.rotary_dim, p.rope_theta, p.rms_norm_epsilon)
        for h in range(kh):
            K[t, h] = independent_prepare(k[t, h], kw, t, p.rotary_dim, p.rope_theta, p.rms_norm_epsilon)
    out = np.zeros((T, qh, d))
    for h in range(qh):
        kv = h // (qh // kh)
        s = Q[:, h] @ K[:, kv].T / math.sqrt(d)
        s[np.triu_indices(T, 1)] = -np.inf
        pr = np.exp(s - s.max(-1, keepdims=True))
        pr /= pr.sum(-1, keepdims=True)
        out[:, h] = (pr @ np.asarray(v[:, kv], np.float64)) * sigmoid(qg[:, h, 1])
    return out, K


@pytest.mark.parametrize("dim,qh,kh,rotary,theta", [(6, 4, 2, 4, 73.0), (64, 6, 2, 16, 1e7), (256, 4, 4, 64, 1e7)])
def test_unrounded_sequence_matches_independent_float64(oracle, dim, qh, kh, rotary, theta):
    T = 19
    p = oracle.attention_params(qh, kh, dim, rotary, capacity=T, rope_theta=theta,
                                round_to_bfloat16=False)
    rng = np.random.default_rng(dim)
    qg = rng.standard_normal((T, qh, 2, dim)).astype(np.float32)
    k = rng.standard_normal((T, kh, dim)).astype(np.float32)
    v = rng.standard_normal((T, kh, dim)).astype(np.float32)
    qw = values(dim, 0.2, 0.3); kw = values(dim, 0.8, 0.4)
    got = oracle.gqa_sequence(p, qg, k, v, qw, kw)
    want, want_keys = independent_sequence(p, qg, k, v, qw, kw)
    np.testing.assert_allclose(got["keys"], want_keys, rtol=2e-6, atol=2e-6)
    np.testing.assert_allclose(got["out"], want, rtol=1e-5, atol=1e-5)
    np.testing.assert_array_equal(got["values"], v)


def test_rounded_sequence_close_to_float64_and_bf16_representable(oracle):
    T, dim, qh, kh = 40, 128, 6, 2
    p = oracle.attention_params(qh, kh, dim, 32, capacity=T)
    rng = np.random.default_rng(2)
    qg = oracle.bf16_round(0.5 * rng.standard_normal((T, qh, 2, dim)).astype(np.float32))
    k = oracle.bf16_round(0.5 * rng.standard_normal((T, kh, dim)).astype(np.float32))
    v = oracle.bf16_round(0.5 * rng.standard_normal((T, kh, dim)).astype(np.float32))
    qw = values(dim, 0.2, 0.3); kw = values(dim, 0.8, 0.4)
    got = oracle.gqa_sequence(p, qg, k, v, qw, kw)
    want, _ = independent_sequence(p, qg, k, v, qw, kw)
    for name in ("out", "keys", "values"):
        np.testing.assert_array_equal(got[name], oracle.bf16_round(got[name]))
    # every rounding point moves a value by at most 2^-9 relative; the rounded
    # path must stay within a few such steps of the unrounded mathematics
    err = np.abs(got["out"] - want)
    assert np.all(err <= 2e-3 + 2e-2 * np.abs(want)), err.max()


@pytest.mark.parametrize("round_flag", [False, True])
def test_sequence_equals_cached_steps_bit_exact(oracle, round_flag):
    # qwen_attention_test.cc:209-226
    T, dim, qh, kh = 35, 6, 4, 2
    p = oracle.attention_params(qh, kh, dim, 4, capacity=T, rope_theta=73.0,
                                round_to_bfloat16=round_flag)
    qw = values(dim, 0.2, 0.3); kw = values(dim, 0.8, 0.4)
    qg = np.stack([values(qh * 2 * dim, 0.15 + t * 0.21) for t in range(T)]).reshape(T, qh, 2, dim)
    k = np.stack([values(kh * dim, 0.78 + t * 0.13) for t in range(T)]).reshape(T, kh, dim)
    v = np.stack([values(kh * dim, -0.31 + t * 0.37) for t in range(T)]).reshape(T, kh, dim)
    seq = oracle.gqa_sequence(p, qg, k, v, qw, kw)
    ref = oracle.CachedAttention(p)
    first = None
    for t in range(T):
        out, probs = ref.step(qg[t], k[t], v[t], qw, kw, True)
        np.testing.assert_array_equal(out, seq["out"][t])
        np.testing.assert_allclose(probs.sum(-1), 1.0, atol=3e-6)
        if t == 0:
            first = out.copy()
    np.testing.assert_array_equal(ref.keys, seq["keys"])
    np.testing.assert_array_equal(ref.values, seq["values"])
    # replay after Reset is bit-equal (cached_attention_ops_test.cc:346-359)
    ref.reset()
    np.testing.assert_array_equal(ref.step(qg[0], k[0], v[0], qw, kw), first)


def test_rows_beyond_position_are_never_read(oracle):
    # the mirror's cache starts NaN filled; Reset() never clears
    # (key_value_cache_test.cc:78-110)
    p = oracle.attention_params(4, 2, 8, 4, capacity=8)
    ref = oracle.CachedAttention(p)
    rng = np.random.default_rng(1)
    w = np.zeros(8, np.float32)
    for t in range(5):
        out = ref.step(rng.standard_normal(64), rng.standard_normal(16),
                       rng.standard_normal(16), w, w)
        assert np.all(np.isfinite(out))
    assert np.all(np.isnan(ref.keys[5:]))


def test_attend_on_head_major_cache_matches_step(oracle):
    p = oracle.attention_params(6, 2, 16, 8, capacity=12)
    ref = oracle.CachedAttention(p)
    rng = np.random.default_rng(4)
    w = values(16, 0.2, 0.3)
    for t in range(12):
        qg = oracle.bf16_round(rng.standard_normal((6, 2, 16)).astype(np.float32))
        out = ref.step(qg, oracle.bf16_round(rng.standard_normal(32).astype(np.float32)),
                       rng.standard_normal(32), w, w)
    q = np.stack([oracle.gqa_normalize_rotate(p, 11, qg[h, 0], w) for h in range(6)])
    keys = np.ascontiguousarray(ref.keys.transpose(1, 0, 2))
    vals = np.ascontiguousarray(ref.values.transpose(1, 0, 2))
    np.testing.assert_array_equal(oracle.gqa_attend(p, q, qg[:, 1], keys, vals), out)


def test_rejects_invalid_parameters(oracle):
    # cached_attention_ops_test.cc:505-560
    good = dict(query_heads=2, key_value_heads=1, head_dim=4, rotary_dim=2, capacity=2)
    bad = [dict(query_heads=0), dict(key_value_heads=-1), dict(query_heads=3, key_value_heads=2),
           dict(head_dim=257), dict(head_dim=0), dict(rotary_dim=3), dict(rotary_dim=6),
           dict(rope_theta=0.0), dict(rope_theta=float("inf")), dict(rms_norm_epsilon=float("nan")),
           dict(capacity=0)]
    z = np.zeros(16, np.float32)
    for change in bad:
        p = oracle.attention_params(**{**good, **change})
        ref = oracle.CachedAttention(oracle.attention_params(**good))
        ref.p = p
        with pytest.raises(ValueError):
            ref.step(z, z, z, z, z)
        assert ref.position == 0
