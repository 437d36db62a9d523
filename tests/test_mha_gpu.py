"""GPU parity of GPT-2 style causal attention (forward, backward, statistics)
against the CPU oracle, through the C ABI.  Shapes and invariants follow the
reference's attention_reference_test.cc / attention_test.cc."""
import math
import os

import numpy as np
import pytest

from tests.util import (assert_close, assert_close_bf16, assert_close_bf16_gradient,
                        beyond_reference_tolerance, from_bf16_bits, to_bf16_bits)

pytestmark = pytest.mark.gpu

torch = pytest.importorskip("torch")

FP32_REL = 1e-4   # stated tolerance for FP32 storage
BF16_REL = 2e-2   # stated tolerance for bf16 storage (see tests/util.py:assert_close_bf16)


@pytest.fixture(scope="module")
def capi():
    from pluto_amd import capi
    assert torch.cuda.is_available(), "these tests need the GPU"
    capi.lib()
    return capi


def device_inputs(x, d_out, bf16):
    xt = torch.from_numpy(x).cuda()
    if bf16:
        xt = xt.to(torch.bfloat16)
    return xt, torch.from_numpy(d_out).cuda()


def run_device(capi, x, d_out, T, H, bf16):
    xt, gt = device_inputs(x, d_out, bf16)
    out, maxima, normalizers = capi.mha_forward(xt, T, H)
    d_qkv = capi.mha_backward(xt, out, gt, maxima, normalizers, T, H)
    torch.cuda.synchronize()
    return (out.float().cpu().numpy(), maxima.cpu().numpy(), normalizers.cpu().numpy(),
            d_qkv.cpu().numpy())


def run_oracle(oracle, x, d_out, T, H, bf16, seqs=None, heads=None):
    if bf16:
        bits = to_bf16_bits(oracle, x)
        out_bits, maxima, normalizers = oracle.mha_fwd(bits, T, H, oracle.BF16, seqs, heads)
        d_qkv = oracle.mha_bwd(bits, out_bits, d_out, T, H, oracle.BF16, seqs, heads)
        return from_bf16_bits(oracle, out_bits), maxima, normalizers, d_qkv
    out, maxima, normalizers = oracle.mha_fwd(x, T, H, oracle.F32, seqs, heads)
    d_qkv = oracle.mha_bwd(x, out, d_out, T, H, oracle.F32, seqs, heads)
    return out, maxima, normalizers, d_qkv


def check(capi, oracle, T, H, E, B, bf16, seed, qk_scale=1.0):
    rng = np.random.default_rng(seed)
    x = rng.standard_normal((B * T, 3 * E)).astype(np.float32)
    x[:, :2 * E] *= qk_scale
    d_out = rng.standard_normal((B * T, E)).astype(np.float32)
    got = run_device(capi, x, d_out, T, H, bf16)
    want = run_oracle(oracle, x, d_out, T, H, bf16)
    tag = "T%d H%d E%d B%d %s" % (T, H, E, B, "bf16" if bf16 else "fp32")
    # peaked scores leave most gradients tiny next to the few large ones
    gradient_outliers = 2e-2 if qk_scale > 1 else 2e-3
    lse_got = got[1] + np.log(got[2])
    lse_want = want[1] + np.log(want[2])
    # the saved maximum itself is part of the layer state (attention.cc:161-168), not only
    # its combination with the normalizer
    assert_close(got[1], want[1], 1e-3 if bf16 else 1e-4, tag + " maxima")
    if bf16:
        assert_close_bf16(got[0], want[0], tag + " out")
        assert_close(lse_got, lse_want, 1e-3, tag + " lse")
        assert_close_bf16_gradient(got[3], want[3], tag + " d_qkv", outliers=gradient_outliers)
        return
    # peaked scores: the reference's own tolerance (attention_reference_test.cc:56-73)
    rel = 2e-3 if qk_scale > 1 else FP32_REL
    assert_close(got[0], want[0], rel, tag + " out")
    assert_close(lse_got, lse_want, 1e-4, tag + " lse")
    assert_close(got[3], want[3], rel, tag + " d_qkv")


# attention_reference_test.cc:148-160
SHAPES = [(1, 1, 16, 3), (4, 1, 16, 2), (4, 2, 32, 2), (8, 2, 32, 1), (33, 2, 64, 2),
          (33, 2, 128, 2), (65, 2, 64, 2), (65, 2, 128, 2), (65, 2, 160, 2),
          (65, 2, 192, 2), (65, 2, 256, 2)]


@pytest.mark.parametrize("bf16", [False, True])
@pytest.mark.parametrize("T,H,E,B", SHAPES)
def test_matches_oracle_across_configurations(capi, oracle, T, H, E, B, bf16):
    check(capi, oracle, T, H, E, B, bf16, seed=T * 7 + E)


@pytest.mark.parametrize("bf16", [False, True])
def test_peaked_scores(capi, oracle, bf16):
    check(capi, oracle, 65, 1, 64, 2, bf16, seed=5, qk_scale=20.0 if not bf16 else 4.0)


@pytest.mark.parametrize("bf16", [False, True])
@pytest.mark.parametrize("width", [1, 3, 7, 8, 15, 24, 33])
def test_sub_tile_head_widths(capi, oracle, width, bf16):
    check(capi, oracle, 33, 1, width, 2, bf16, seed=width)


def test_three_odd_heads(capi, oracle):
    check(capi, oracle, 65, 3, 21, 2, False, seed=1)
    check(capi, oracle, 65, 3, 96, 2, True, seed=2, qk_scale=2.0)


@pytest.mark.parametrize("bf16", [False, True])
def test_production_context_one_head(capi, oracle, bf16):
    # attention_reference_test.cc:171-176: T=1024, one 64-wide head
    check(capi, oracle, 1024, 1, 64, 1, bf16, seed=9)


REFERENCE_BF16_CASES = [(33, 2, 64, 2), (33, 2, 128, 2), (65, 2, 64, 2), (65, 2, 128, 2),
                        (65, 2, 256, 2), (1024, 1, 64, 1)]


@pytest.mark.parametrize("T,H,E,B", REFERENCE_BF16_CASES)
def test_reference_device_tolerance_on_its_bf16_cases(capi, oracle, T, H, E, B):
    """The reference's own device-vs-CPU test (attention_reference_test.cc:19-73) with
    its inputs (0.35 sin + 0.05 cos; upstream gradient 0.2 cos) and its bounds,
    2e-3 + 2e-3|x| forward and 3e-3 + 3e-3|x| backward, on the bf16 cases whose heads
    the matrix-core kernels serve.  The reference keeps P in FP32; these kernels
    round P, dS and dO to bf16 for the matrix cores, so a fraction of the elements
    could lie beyond the reference's bound; on the reference's inputs none does."""
    index = np.arange(B * T * 3 * E, dtype=np.float32)
    x = (np.float32(0.35) * np.sin(index * np.float32(0.071)) +
         np.float32(0.05) * np.cos(index * np.float32(0.19))).astype(np.float32).reshape(B * T, 3 * E)
    index = np.arange(B * T * E, dtype=np.float32)
    d_out = (np.float32(0.2) * np.cos(index * np.float32(0.13))).astype(np.float32).reshape(B * T, E)
    got = run_device(capi, x, d_out, T, H, True)
    want = run_oracle(oracle, x, d_out, T, H, True)
    forward = beyond_reference_tolerance(got[0], want[0], 2e-3, 2e-3)
    backward = beyond_reference_tolerance(got[3], want[3], 3e-3, 3e-3)
    print("T%d H%d E%d B%d: %.3f %% of the outputs beyond 2e-3 + 2e-3|x| (max-abs %.2e), "
          "%.3f %% of the gradients beyond 3e-3 + 3e-3|x| (max-abs %.2e)" % (
              T, H, E, B, 100 * forward, np.abs(got[0] - want[0]).max(), 100 * backward,
              np.abs(got[3] - want[3]).max()))
    assert forward == 0.0 and backward == 0.0
    assert_close_bf16(got[0], want[0], "reference case out")
    assert_close_bf16_gradient(got[3], want[3], "reference case d_qkv")


def test_mfma_heads_of_128(capi, oracle):
    check(capi, oracle, 300, 2, 256, 2, True, seed=12)


@pytest.mark.parametrize("T, H, E, B", [(2100, 3, 384, 2), (2048, 5, 320, 3), (2301, 2, 128, 9),
                                        (2048, 12, 768, 6), (4096, 4, 512, 3),
                                        (256, 2, 512, 3), (301, 3, 768, 2), (2100, 2, 512, 2)])
def test_long_sequences_take_the_eight_wave_kernel(capi, oracle, T, H, E, B):
    # From 2048 rows on the forward at head widths 64 and 128 runs the kernel
    # with the hand-scheduled loop (256-row tiles, 128 at width 64; here with the
    # packed [rows, 3E] layout, several sequences and heads, lengths that are
    # not a multiple of its tile, more and fewer tiles than compute units); at
    # head width 256 from 256 rows (128-row tiles, one wave a SIMD).  It must
    # leave exactly what the four-wave kernel leaves, which the oracle pins.
    rng = np.random.default_rng(31)
    host = rng.standard_normal((B * T, 3 * E)).astype(np.float32)
    x = torch.from_numpy(host).cuda().to(torch.bfloat16)
    new = capi.mha_forward(x, T, H)
    with capi.only_kernels(0xffffffff & ~capi.EIGHT_WAVE):
        old = capi.mha_forward(x, T, H)
    torch.cuda.synchronize()
    for a, b in zip(new, old):
        assert torch.equal(a, b)
    # one (sequence, head) against the oracle
    bits = to_bf16_bits(oracle, host)
    out_bits, maxima, normalizers = oracle.mha_fwd(bits, T, H, oracle.BF16, (1, 2), (1, 2))
    want = from_bf16_bits(oracle, out_bits)
    D = E // H
    got = new[0].float().cpu().numpy()
    assert_close_bf16(got[T:2 * T, D:2 * D], want[T:2 * T, D:2 * D], "sequence 1, head 1")


def test_closed_form_two_tokens(capi):
    # attention_test.cc:282-360
    T, H, E, rows = 4, 2, 32, 32
    x = np.zeros((rows, 3 * E), np.float32)
    x[0, 0] = 1; x[0, E] = 1; x[0, 2 * E] = 1
    x[1, 0] = 2; x[1, E] = 2; x[1, 2 * E] = 2
    x[2, 2 * E] = 4
    d_out = np.zeros((rows, E), np.float32)
    d_out[0, 0] = 1
    out, _, _, g = run_device(capi, x, d_out, T, H, False)
    scale = 1 / math.sqrt(E // H)
    w1, w2 = math.exp(2 * scale), math.exp(4 * scale)
    assert abs(out[0, 0] - 1.0) <= 1e-6
    assert abs(out[1, 0] - (w1 + 2 * w2) / (w1 + w2)) <= 1e-5
    assert abs(g[0, 0]) <= 1e-6 and abs(g[0, E]) <= 1e-6
    assert abs(g[0, 2 * E] - 1.0) <= 1e-6
    assert abs(g[1, 0]) <= 1e-6


@pytest.mark.parametrize("bf16,T,E,H", [(False, 65, 128, 2), (True, 65, 128, 2), (True, 300, 128, 2)])
def test_future_tokens_and_other_sequences_cannot_matter(capi, bf16, T, E, H):
    # attention_reference_test.cc:207-308: exact equality
    B = 2
    rng = np.random.default_rng(11)
    x = rng.standard_normal((B * T, 3 * E)).astype(np.float32)
    d_out = rng.standard_normal((B * T, E)).astype(np.float32)
    cut = T * 2 // 3
    d_out[cut:] = 0
    y = x.copy()
    y[cut:T] = rng.standard_normal((T - cut, 3 * E))
    y[T:] = rng.standard_normal((T, 3 * E))
    a = run_device(capi, x, d_out, T, H, bf16)
    b = run_device(capi, y, d_out, T, H, bf16)
    np.testing.assert_array_equal(a[0][:cut], b[0][:cut])
    np.testing.assert_array_equal(a[3][:cut], b[3][:cut])
    assert np.all(b[3][T:] == 0)


@pytest.mark.parametrize("bf16", [False, True])
def test_bitwise_repeatable(capi, bf16):
    # attention_test.cc:362-475
    T, H, E, B = 200, 3, 192, 2
    rng = np.random.default_rng(21)
    x = rng.standard_normal((B * T, 3 * E)).astype(np.float32)
    d_out = rng.standard_normal((B * T, E)).astype(np.float32)
    first = run_device(capi, x, d_out, T, H, bf16)
    for _ in range(4):
        again = run_device(capi, x, d_out, T, H, bf16)
        for a, b in zip(first, again):
            np.testing.assert_array_equal(a, b)


@pytest.mark.parametrize("T,H,B", [(32, 1, 1), (64, 1, 2), (65, 2, 2), (129, 1, 1), (257, 3, 2),
                                   (1000, 2, 3), (1024, 4, 2), (4096, 2, 1), (4100, 1, 1)])
def test_hand_scheduled_key_owned_backward_gives_the_same_bits(capi, oracle, T, H, B):
    """The key-owned backward kernel with the hand-scheduled loop (heads of 64,
    taken from 4096 rows) against the compiler-scheduled one it replaces there:
    same products, same reduction order over query blocks, hence the same bits,
    at every length (the switch below lifts the length threshold) including
    those that end inside a block of 32 or a tile of 128.  One case of moderate
    size also goes against the oracle."""
    E = 64 * H
    rng = np.random.default_rng(T + H)
    x = torch.from_numpy(rng.standard_normal((B * T, 3 * E)).astype(np.float32)).cuda().to(torch.bfloat16)
    d_out = torch.from_numpy(rng.standard_normal((B * T, E)).astype(np.float32)).cuda()
    out, maxima, normalizers = capi.mha_forward(x, T, H)
    with capi.only_kernels(0xffffffff & ~capi.FROM_LENGTH):
        wide = capi.mha_backward(x, out, d_out, maxima, normalizers, T, H)
    with capi.only_kernels(0xffffffff & ~capi.EIGHT_WAVE):
        plain = capi.mha_backward(x, out, d_out, maxima, normalizers, T, H)
    torch.cuda.synchronize()
    assert torch.isfinite(wide).all()
    assert torch.equal(wide, plain)
    if T == 257:
        want = oracle.mha_bwd(to_bf16_bits(oracle, x.float().cpu().numpy()),
                              to_bf16_bits(oracle, out.float().cpu().numpy()),
                              d_out.cpu().numpy(), T, H, oracle.BF16, None, None)
        assert_close_bf16_gradient(wide.cpu().numpy(), want, "wide dK/dV T%d" % T)


@pytest.mark.parametrize("bf16", [False, True])
def test_probabilities_pass(capi, bf16):
    # attention_test.cc:41-146: rows sum to one, zeros above the diagonal, P.V = out
    T, H, E, B = 70, 2, 64, 2
    rng = np.random.default_rng(3)
    x = rng.standard_normal((B * T, 3 * E)).astype(np.float32)
    xt, _ = device_inputs(x, np.zeros((B * T, E), np.float32), bf16)
    out, maxima, normalizers = capi.mha_forward(xt, T, H)
    probs = capi.mha_probabilities(xt, maxima, normalizers, T, H).cpu().numpy()
    assert np.all(np.triu(probs, 1) == 0)
    np.testing.assert_allclose(probs.sum(-1), 1.0, atol=3e-5 if not bf16 else 2e-3)
    xv = xt.float().cpu().numpy().reshape(B, T, 3, H, E // H)
    pv = np.einsum("bhts,bshd->bthd", probs, xv[:, :, 2]).reshape(B * T, E)
    np.testing.assert_allclose(out.float().cpu().numpy(), pv, atol=5e-3 if bf16 else 3e-5)


def test_config1_gpt2_small_forward_fp32(capi, oracle):
    # B=4, T=256, H=12, D=64, fp32 storage, N(0,1), seed 0
    T, H, E, B = 256, 12, 768, 4
    rng = np.random.default_rng(0)
    x = rng.standard_normal((B * T, 3 * E)).astype(np.float32)
    xt = torch.from_numpy(x).cuda()
    out, maxima, normalizers = capi.mha_forward(xt, T, H)
    assert capi.last_path() == capi.PATH_MATRIX_F32   # not the any-shape kernel
    want, wm, wn = oracle.mha_fwd(x, T, H)
    assert_close(out.cpu().numpy(), want, FP32_REL, "config 1 out")
    assert_close((maxima + normalizers.log()).cpu().numpy(), wm + np.log(wn), 1e-4, "config 1 lse")


def test_config2_gpt2_small_forward_backward_bf16(capi, oracle):
    # B=16, T=1024, H=12, D=64, bf16 storage, N(0,1), seed 1.  The oracle is run
    # on whole (sequence, head) units (they are independent); the rest of the
    # tensor is checked against the any-shape FP32-arithmetic kernels.
    T, H, E, B = 1024, 12, 768, 16
    rng = np.random.default_rng(1)
    x = rng.standard_normal((B * T, 3 * E)).astype(np.float32)
    d_out = rng.standard_normal((B * T, E)).astype(np.float32)
    xt, gt = device_inputs(x, d_out, True)
    out, maxima, normalizers = capi.mha_forward(xt, T, H)
    assert capi.last_path() == capi.PATH_FLASH
    d_qkv = capi.mha_backward(xt, out, gt, maxima, normalizers, T, H)
    assert capi.last_path() == capi.PATH_FLASH
    D = E // H
    # Every one of the 192 (sequence, head) units against the oracle, sixteen at
    # a time (its C code runs outside the interpreter lock): a unit is handed
    # over as a one-head problem, which is the same arithmetic.
    import concurrent.futures
    bits = to_bf16_bits(oracle, x)

    def unit(index):
        seq, head = divmod(index, H)
        rows = slice(seq * T, (seq + 1) * T)
        cols = [slice(part * E + head * D, part * E + (head + 1) * D) for part in range(3)]
        one = np.ascontiguousarray(np.concatenate([bits[rows, c] for c in cols], axis=1))
        upstream = np.ascontiguousarray(d_out[rows, head * D:(head + 1) * D])
        o_bits, wm, wn = oracle.mha_fwd(one, T, 1, oracle.BF16)
        grads = oracle.mha_bwd(one, o_bits, upstream, T, 1, oracle.BF16)
        return from_bf16_bits(oracle, o_bits), wm[0] + np.log(wn[0]), grads

    with concurrent.futures.ThreadPoolExecutor(max_workers=16) as pool:
        results = list(pool.map(unit, range(B * H)))
    want_out = np.empty((B * T, E), np.float32)
    want_lse = np.empty((B * H, T), np.float32)
    want_g = np.empty((B * T, 3 * E), np.float32)
    for index, (o, lse, grads) in enumerate(results):
        seq, head = divmod(index, H)
        rows = slice(seq * T, (seq + 1) * T)
        want_out[rows, head * D:(head + 1) * D] = o
        want_lse[index] = lse
        for part in range(3):
            want_g[rows, part * E + head * D:part * E + (head + 1) * D] = grads[:, part * D:(part + 1) * D]
    assert_close_bf16(out.float().cpu().numpy(), want_out, "config 2 out, all 192 units")
    assert_close((maxima + normalizers.log()).cpu().numpy(), want_lse, 1e-3, "config 2 lse, all 192 units")
    g = d_qkv.cpu().numpy()
    for part, name in ((0, "dQ"), (1, "dK"), (2, "dV")):
        c = slice(part * E, (part + 1) * E)
        assert_close_bf16_gradient(g[:, c], want_g[:, c], "config 2 %s, all 192 units" % name)
    with capi.force_generic():
        out2, m2, n2 = capi.mha_forward(xt, T, H)
        d2 = capi.mha_backward(xt, out2, gt, m2, n2, T, H)
        assert capi.last_path() == capi.PATH_GENERIC
        torch.cuda.synchronize()
    assert_close_bf16(out.float().cpu().numpy(), out2.float().cpu().numpy(), "config 2 out vs fp32-arithmetic kernel")
    g1, g2 = d_qkv.cpu().numpy(), d2.cpu().numpy()
    for part, name in ((0, "dQ"), (1, "dK"), (2, "dV")):
        c = slice(part * E, (part + 1) * E)
        assert_close_bf16_gradient(g1[:, c], g2[:, c], "config 2 %s vs fp32-arithmetic kernel" % name)


def test_rejects_bad_arguments_before_any_work(capi):
    # attention_test.cc:549-626
    x = torch.zeros((6, 12), device="cuda")
    for T, H in ((4, 2), (3, 3), (0, 2), (3, 0)):
        with pytest.raises(capi.PlutoHipError) as info:
            capi.mha_forward(x, T, H)
        assert info.value.code == capi.EINVAL
