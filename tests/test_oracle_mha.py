"""Pins the CPU oracle for GPT-2 causal attention against evidence that does
not come from the oracle itself: the reference's closed form, a float64
library routine with autograd, brute force, and causality invariants."""
import math

import numpy as np
import pytest
import torch


def packed(rng, rows, E, scale=1.0):
    return (scale * rng.standard_normal((rows, 3 * E))).astype(np.float32)


def torch_attention(qkv64, T, H):
    """Independent oracle: float64 SDPA (is_causal) on [B, H, T, D]."""
    rows, packed_width = qkv64.shape
    E = packed_width // 3
    D = E // H
    B = rows // T
    x = qkv64.reshape(B, T, 3, H, D).permute(2, 0, 3, 1, 4)
    out = torch.nn.functional.scaled_dot_product_attention(
        x[0], x[1], x[2], is_causal=True)
    return out.permute(0, 2, 1, 3).reshape(rows, E)


def test_closed_form_two_tokens(oracle):
    # reference: src/llm/layers/attention_test.cc:282-360 (T=4, H=2, E=32).
    T, H, E, rows = 4, 2, 32, 32
    x = np.zeros((rows, 3 * E), np.float32)
    x[0, 0] = 1; x[0, E] = 1; x[0, 2 * E] = 1
    x[1, 0] = 2; x[1, E] = 2; x[1, 2 * E] = 2
    x[2, 2 * E] = 4
    out, maxima, normalizers = oracle.mha_fwd(x, T, H)
    scale = 1 / math.sqrt(E // H)
    w1, w2 = math.exp(2 * scale), math.exp(4 * scale)
    assert out[0, 0] == pytest.approx(1.0, abs=1e-6)
    assert out[1, 0] == pytest.approx((w1 + 2 * w2) / (w1 + w2), abs=1e-5)
    # the same closed form evaluated for a head width of 16: sigmoid(0.5) + 1
    assert out[1, 0] == pytest.approx(1.622459, abs=1e-5)
    d_out = np.zeros((rows, E), np.float32)
    d_out[0, 0] = 1
    g = oracle.mha_bwd(x, out, d_out, T, H)
    assert g[0, 0] == pytest.approx(0, abs=1e-6)
    assert g[0, E] == pytest.approx(0, abs=1e-6)
    assert g[0, 2 * E] == pytest.approx(1, abs=1e-6)
    assert g[1, 0] == pytest.approx(0, abs=1e-6)
    # softmax statistics: row 1 of head 0 has max 4*scale, sum 1+exp(-2 scale)
    assert maxima[0, 1] == pytest.approx(4 * scale, rel=1e-6)
    assert normalizers[0, 1] == pytest.approx(1 + math.exp(-2 * scale), rel=1e-6)


# (context, heads, width, sequences): attention_reference_test.cc:148-160,186-189
SHAPES = [(1, 1, 16, 3), (4, 2, 32, 2), (33, 2, 64, 2), (65, 2, 128, 2),
          (65, 3, 21, 2), (33, 1, 7, 2), (65, 2, 256, 2)]


@pytest.mark.parametrize("T,H,E,B", SHAPES)
def test_forward_backward_match_float64_library(oracle, T, H, E, B):
    rng = np.random.default_rng(T * 1000 + E)
    x = packed(rng, B * T, E)
    d_out = rng.standard_normal((B * T, E)).astype(np.float32)
    out, maxima, normalizers = oracle.mha_fwd(x, T, H)
    g = oracle.mha_bwd(x, out, d_out, T, H)
    x64 = torch.tensor(x, dtype=torch.float64, requires_grad=True)
    ref = torch_attention(x64, T, H)
    ref.backward(torch.tensor(d_out, dtype=torch.float64))
    np.testing.assert_allclose(out, ref.detach().numpy(), rtol=2e-5, atol=2e-6)
    np.testing.assert_allclose(g, x64.grad.numpy(), rtol=1e-4, atol=2e-5)
    # LSE from the saved statistics equals the textbook log-sum-exp
    D = E // H
    q = x64.detach().reshape(B, T, 3, H, D)
    s = torch.einsum("bthd,bshd->bhts", q[:, :, 0], q[:, :, 1]) / math.sqrt(D)
    s = s.masked_fill(torch.triu(torch.ones(T, T, dtype=torch.bool), 1), -math.inf)
    lse = torch.logsumexp(s, -1).reshape(B * H, T).numpy()
    np.testing.assert_allclose(maxima + np.log(normalizers), lse, rtol=1e-5,
                               atol=1e-5)


def test_peaked_scores(oracle):
    # attention_reference_test.cc:163-169 (Q/K scaled by 20)
    T, H, E, B = 65, 1, 64, 2
    rng = np.random.default_rng(7)
    x = packed(rng, B * T, E)
    x[:, :2 * E] *= 20
    out, _, _ = oracle.mha_fwd(x, T, H)
    ref = torch_attention(torch.tensor(x, dtype=torch.float64), T, H).numpy()
    # scores of magnitude ~1e3 carry fp32 rounding of ~1e-4 into the exponent;
    # the reference's own tolerance for this case is 2e-3 abs + 2e-3 rel.
    np.testing.assert_allclose(out, ref, rtol=2e-3, atol=2e-3)


def test_bf16_storage_loads_and_rounds(oracle):
    T, H, E, B = 33, 2, 64, 2
    rng = np.random.default_rng(3)
    x = packed(rng, B * T, E)
    bits = oracle.f32_to_bf16_bits(x).reshape(x.shape)
    xr = oracle.bf16_bits_to_f32(bits).reshape(x.shape)
    out_bits, m_b, n_b = oracle.mha_fwd(bits, T, H, dtype=oracle.BF16)
    out_f32, m_f, n_f = oracle.mha_fwd(xr, T, H)
    # bf16 storage = same arithmetic on the rounded inputs, output rounded RNE
    np.testing.assert_array_equal(out_bits, oracle.f32_to_bf16_bits(out_f32).reshape(out_f32.shape))
    np.testing.assert_array_equal(m_b, m_f)
    np.testing.assert_array_equal(n_b, n_f)
    # backward reads the STORED (rounded) output for delta
    d_out = rng.standard_normal((B * T, E)).astype(np.float32)
    g_bits = oracle.mha_bwd(bits, out_bits, d_out, T, H, dtype=oracle.BF16)
    g_f32 = oracle.mha_bwd(xr, oracle.bf16_bits_to_f32(out_bits).reshape(out_f32.shape), d_out, T, H)
    np.testing.assert_array_equal(g_bits, g_f32)


def test_bf16_rounding_rule(oracle):
    # ties to even, reference_internal.h:109-115
    vals = np.array([1.0, 1.00390625, 1.01171875, -1.00390625, 3.140625, 65280.0],
                    np.float32)
    got = oracle.bf16_round(vals)
    want = torch.tensor(vals).to(torch.bfloat16).to(torch.float32).numpy()
    np.testing.assert_array_equal(got, want)
    rng = np.random.default_rng(0)
    x = rng.standard_normal(100000).astype(np.float32) * 100
    np.testing.assert_array_equal(
        oracle.bf16_round(x),
        torch.tensor(x).to(torch.bfloat16).to(torch.float32).numpy())


def test_future_tokens_and_other_sequences_cannot_matter(oracle):
    # attention_reference_test.cc:207-308: exact equality
    T, H, E, B = 65, 2, 128, 2
    rng = np.random.default_rng(11)
    x = packed(rng, B * T, E)
    d_out = rng.standard_normal((B * T, E)).astype(np.float32)
    out, _, _ = oracle.mha_fwd(x, T, H)
    g = oracle.mha_bwd(x, out, d_out, T, H)
    cut = 40
    y = x.copy()
    y[cut:T] = rng.standard_normal((T - cut, 3 * E))   # future of sequence 0
    y[T:] = rng.standard_normal((T, 3 * E))            # all of sequence 1
    out2, _, _ = oracle.mha_fwd(y, T, H)
    np.testing.assert_array_equal(out[:cut], out2[:cut])
    d2 = d_out.copy()
    d2[cut:] = 0
    d1 = d_out.copy()
    d1[cut:] = 0
    g1 = oracle.mha_bwd(x, out, d1, T, H)
    g2 = oracle.mha_bwd(y, out2, d2, T, H)
    np.testing.assert_array_equal(g1[:cut], g2[:cut])
    assert np.all(g2[T:] == 0)


def test_brute_force_tiny(oracle):
    T, H, E = 5, 1, 3
    rng = np.random.default_rng(5)
    x = packed(rng, T, E)
    out, _, _ = oracle.mha_fwd(x, T, H)
    for i in range(T):
        s = np.array([np.dot(x[i, :E].astype(np.float64), x[j, E:2 * E]) for j in range(i + 1)]) / math.sqrt(E)
        p = np.exp(s - s.max()); p /= p.sum()
        want = sum(p[j] * x[j, 2 * E:].astype(np.float64) for j in range(i + 1))
        np.testing.assert_allclose(out[i], want, rtol=1e-5, atol=1e-6)


def test_rejects_bad_shapes(oracle):
    x = np.zeros((6, 12), np.float32)
    with pytest.raises(ValueError):
        oracle.mha_fwd(x, 4, 2)      # rows not divisible by context_length
    with pytest.raises(ValueError):
        oracle.mha_fwd(x, 3, 3)      # E=4 not divisible by heads=3
