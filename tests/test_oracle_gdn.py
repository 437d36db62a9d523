"""Pins the CPU oracle for the gated delta-net: textbook special cases of the
delta rule, the matrix form of the published recurrence in float64, softplus
extremes, and the reference's sequence-vs-step consistency checks."""
import math

import numpy as np
import pytest


def values(count, phase, scale=1.0):
    i = np.arange(count, dtype=np.float32)
    return (np.float32(scale) * np.sin(np.float32(phase) + i * np.float32(0.29))).astype(np.float32)


def matrix_form(q, k, v, log_decay, beta, normalize, q_scale, S0=None):
    """Gated delta rule as published (Yang et al., Gated Delta Networks), in
    matrix form on S in R^{dk x dv}:
        S_t = alpha_t (I - beta_t k_t k_t^T) S_{t-1} + beta_t k_t v_t^T
        o_t = S_t^T q_t
    float64, written independently of the oracle's scalar loops."""
    T, kh, kd = q.shape
    vh, vd = v.shape[1:]
    S = np.zeros((vh, kd, vd)) if S0 is None else np.array(S0, np.float64)
    out = np.zeros((T, vh, vd))
    for t in range(T):
        for h in range(vh):
            g = h // (vh // kh)
            qt = q[t, g].astype(np.float64); kt = k[t, g].astype(np.float64)
            if normalize:
                qt = qt / math.sqrt(qt @ qt + 1e-6)
                kt = kt / math.sqrt(kt @ kt + 1e-6)
            qt = qt * q_scale
            alpha = math.exp(float(log_decay[t, h])); b = float(beta[t, h])
            S[h] = alpha * (np.eye(kd) - b * np.outer(kt, kt)) @ S[h] + b * np.outer(kt, v[t, h].astype(np.float64))
            out[t, h] = S[h].T @ qt
    return out, S


@pytest.mark.parametrize("kh,vh,kd,vd", [(1, 2, 3, 5), (2, 4, 5, 35), (2, 2, 16, 16)])
@pytest.mark.parametrize("normalize", [False, True])
def test_scan_matches_published_matrix_form(oracle, kh, vh, kd, vd, normalize):
    T = 23
    p = oracle.delta_params(kh, vh, kd, vd, round_to_bfloat16=False)
    rng = np.random.default_rng(kd * 10 + vd)
    q = rng.standard_normal((T, kh, kd)).astype(np.float32)
    k = rng.standard_normal((T, kh, kd)).astype(np.float32)
    if not normalize:
        k /= np.linalg.norm(k, axis=-1, keepdims=True)
    v = rng.standard_normal((T, vh, vd)).astype(np.float32)
    g = -np.log1p(np.exp(rng.standard_normal((T, vh)))).astype(np.float32)
    beta = (1 / (1 + np.exp(-rng.standard_normal((T, vh))))).astype(np.float32)
    S0 = rng.standard_normal((vh, kd, vd))
    scale = 1 / math.sqrt(kd)
    core, state = oracle.gdn_scan(p, q, k, v, g, beta, normalize, scale, S0)
    want, want_state = matrix_form(q, k, v, g, beta, normalize, scale, S0)
    np.testing.assert_allclose(core, want, rtol=1e-5, atol=1e-6)
    np.testing.assert_allclose(state, want_state, rtol=1e-9, atol=1e-12)


def test_beta_zero_is_pure_decay(oracle):
    T, kd, vd = 9, 4, 6
    p = oracle.delta_params(1, 1, kd, vd, round_to_bfloat16=False)
    rng = np.random.default_rng(0)
    q = rng.standard_normal((T, 1, kd)).astype(np.float32)
    k = rng.standard_normal((T, 1, kd)).astype(np.float32)
    v = rng.standard_normal((T, 1, vd)).astype(np.float32)
    g = -rng.random((T, 1)).astype(np.float32)
    S0 = rng.standard_normal((1, kd, vd))
    core, state = oracle.gdn_scan(p, q, k, v, g, np.zeros((T, 1), np.float32), False, 1.0, S0)
    cumulative = np.exp(np.cumsum(g.astype(np.float64), 0))
    np.testing.assert_allclose(state[0], cumulative[-1, 0] * S0[0], rtol=1e-12)
    for t in range(T):
        np.testing.assert_allclose(core[t, 0], cumulative[t, 0] * (S0[0].T @ q[t, 0]), rtol=1e-5, atol=1e-6)


def test_orthonormal_keys_no_decay_builds_outer_product_memory(oracle):
    # textbook delta rule: g = 0, beta = 1, orthonormal keys => S = sum k v^T
    kd = vd = 8
    T = kd
    p = oracle.delta_params(1, 1, kd, vd, round_to_bfloat16=False)
    rng = np.random.default_rng(1)
    basis, _ = np.linalg.qr(rng.standard_normal((kd, kd)))
    k = basis.T.reshape(T, 1, kd).astype(np.float32)
    v = rng.standard_normal((T, 1, vd)).astype(np.float32)
    zeros = np.zeros((T, 1), np.float32)
    core, state = oracle.gdn_scan(p, k, k, v, zeros, zeros + 1, False, 1.0)
    np.testing.assert_allclose(state[0], k[:, 0].astype(np.float64).T @ v[:, 0], atol=1e-6)
    # querying with the key just written returns its value
    np.testing.assert_allclose(core[:, 0], v[:, 0], atol=1e-5)
    # writing the same key again with a new value overwrites the old one
    v2 = rng.standard_normal((1, 1, vd)).astype(np.float32)
    core2, state2 = oracle.gdn_scan(p, k[:1], k[:1], v2, zeros[:1], zeros[:1] + 1, False, 1.0, state)
    np.testing.assert_allclose(core2[0, 0], v2[0, 0], atol=1e-5)


def make_layer_inputs(p, T, rng, oracle):
    channels = 2 * p.key_heads * p.key_head_dim + p.value_heads * p.value_head_dim
    width = p.value_heads * p.value_head_dim
    qkv = oracle.bf16_round(rng.standard_normal((T, channels)).astype(np.float32))
    z = oracle.bf16_round(rng.standard_normal((T, width)).astype(np.float32))
    a = oracle.bf16_round(rng.standard_normal((T, p.value_heads)).astype(np.float32))
    b = oracle.bf16_round(rng.standard_normal((T, p.value_heads)).astype(np.float32))
    w = values(channels * p.conv_kernel_dim, 0.73, 0.6)
    a_log = values(p.value_heads, 0.18, 0.5)
    dt = values(p.value_heads, -0.7, 0.3)
    norm = values(p.value_head_dim, 0.5, 0.6)
    return qkv, z, a, b, w, a_log, dt, norm


@pytest.mark.parametrize("round_flag", [False, True])
@pytest.mark.parametrize("dims", [(2, 6, 5, 7), (2, 4, 32, 16)])
def test_sequence_agrees_with_repeated_steps(oracle, round_flag, dims):
    # sequence_delta_net_test.cc:257-291 (tolerance 1.5e-4 + 1.5e-2 |x|, :253-255)
    kh, vh, kd, vd = dims
    T = 7
    p = oracle.delta_params(kh, vh, kd, vd, round_to_bfloat16=round_flag)
    rng = np.random.default_rng(kd)
    qkv, z, a, b, w, a_log, dt, norm = make_layer_inputs(p, T, rng, oracle)
    a[:, 0] = 100.0; a[:, 1] = -100.0     # softplus extremes, cached_attention_ops_test.cc:442-444
    seq = oracle.gdn_sequence(p, qkv, z, a, b, w, a_log, dt, norm)
    assert np.all(np.isfinite(seq["out"]))
    stepper = oracle.DeltaNetStep(p)
    first = None
    for t in range(T):
        out = stepper.step(qkv[t], z[t], a[t], b[t], w, a_log, dt, norm)
        assert np.all(np.abs(out - seq["out"][t]) <= 1.5e-4 + 1.5e-2 * np.abs(seq["out"][t]))
        if t == 0:
            first = out.copy()
    np.testing.assert_allclose(stepper.state, seq["state"], rtol=1e-2, atol=1e-4)
    # Reset() replays bit-equal (cached_attention_ops_test.cc:463-466)
    stepper.reset()
    np.testing.assert_array_equal(stepper.step(qkv[0], z[0], a[0], b[0], w, a_log, dt, norm), first)


def test_sequence_core_is_scan_of_convolved_inputs(oracle):
    # With a one-tap identity convolution the layer's recurrence input is
    # bf16(silu(x)); the layer core must equal the bare scan on that input
    # with g = -exp(A_log) softplus(a + dt_bias) and beta = sigmoid(b).
    kh, vh, kd, vd, T = 2, 4, 8, 16, 11
    p = oracle.delta_params(kh, vh, kd, vd, conv_kernel_dim=1, round_to_bfloat16=False)
    rng = np.random.default_rng(9)
    channels = 2 * kh * kd + vh * vd
    qkv = rng.standard_normal((T, channels)).astype(np.float32)
    z = rng.standard_normal((T, vh * vd)).astype(np.float32)
    a = rng.standard_normal((T, vh)).astype(np.float32)
    b = rng.standard_normal((T, vh)).astype(np.float32)
    a_log = values(vh, 0.18, 0.5); dt = values(vh, -0.7, 0.3)
    seq = oracle.gdn_sequence(p, qkv, z, a, b, np.ones((channels, 1), np.float32), a_log, dt,
                              np.ones(vd, np.float32))
    x = qkv.astype(np.float64)
    silu = (x / (1 + np.exp(-x))).astype(np.float32)
    q = silu[:, :kh * kd].reshape(T, kh, kd)
    k = silu[:, kh * kd:2 * kh * kd].reshape(T, kh, kd)
    v = silu[:, 2 * kh * kd:].reshape(T, vh, vd)
    alpha = a.astype(np.float64) + dt
    g = -np.exp(a_log.astype(np.float64)) * (np.maximum(alpha, 0) + np.log1p(np.exp(-np.abs(alpha))))
    beta = 1 / (1 + np.exp(-b.astype(np.float64)))
    want, want_state = matrix_form(q, k, v, g, beta, True, 1 / math.sqrt(kd))
    np.testing.assert_allclose(seq["core"], want, rtol=2e-5, atol=2e-6)
    np.testing.assert_allclose(seq["state"], want_state, rtol=1e-5, atol=1e-7)
    # output norm: RMSNorm (plain weight) times SiLU(z), stored as bf16
    core = want.reshape(T * vh, vd)
    normed = core / np.sqrt((core ** 2).mean(-1, keepdims=True) + 1e-6)
    zz = z.reshape(T * vh, vd).astype(np.float64)
    want_out = normed * zz / (1 + np.exp(-zz))
    np.testing.assert_allclose(seq["out"].reshape(T * vh, vd), want_out, rtol=1e-2, atol=1e-4)
    np.testing.assert_array_equal(seq["out"], oracle.bf16_round(seq["out"]))


def test_rejects_bad_parameters(oracle):
    # cached_attention_ops.cc:376-383
    with pytest.raises(ValueError):
        p = oracle.delta_params(2, 3, 4, 4)
        oracle.gdn_scan(p, np.zeros((1, 2, 4)), np.zeros((1, 2, 4)), np.zeros((1, 3, 4)),
                        np.zeros((1, 3)), np.zeros((1, 3)), False, 1.0)
