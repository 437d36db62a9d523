"""GPU parity of the whole-sequence Qwen GQA backward
(QwenAttentionLayer::SequenceBackward, qwen_attention.cc:450-499) with the CPU
oracle, through the C ABI.  Shapes follow qwen_attention_test.cc:230-345 (tiny,
FP32 kernels, both rounding modes) and add head widths that take the
matrix-core kernels."""
import numpy as np
import pytest

from tests.util import assert_close, assert_close_bf16_gradient

pytestmark = pytest.mark.gpu

torch = pytest.importorskip("torch")


@pytest.fixture(scope="module")
def capi():
    from pluto_amd import capi
    assert torch.cuda.is_available(), "these tests need the GPU"
    capi.lib()
    return capi


def values(count, phase, scale=0.8):
    i = np.arange(count, dtype=np.float32)
    return (np.float32(scale) * np.sin(np.float32(phase) + i * np.float32(0.29))).astype(np.float32)


def dev(x, dtype=None):
    t = torch.from_numpy(np.ascontiguousarray(x)).cuda()
    return t.to(dtype) if dtype is not None else t


def run_case(capi, T, qh, kh, d, rot, rounding, seed=None, weight_grads=True):
    from oracle import pyoracle as po
    kw = dict(query_heads=qh, key_value_heads=kh, head_dim=d, rotary_dim=rot, capacity=max(T, 1),
              round_to_bfloat16=rounding)
    p, op = capi.attention_params(**kw), po.attention_params(**kw)
    if seed is None:
        qg = po.bf16_round(values(T * qh * 2 * d, .1)).reshape(T, qh, 2, d)
        k = po.bf16_round(values(T * kh * d, 1.2)).reshape(T, kh, d)
        v = po.bf16_round(values(T * kh * d, 2.3)).reshape(T, kh, d)
        qw, kw_ = values(d, .2), values(d, .4)
        dy = values(T * qh * d, .7).reshape(T, qh, d)
    else:
        rng = np.random.default_rng(seed)
        qg = po.bf16_round(rng.standard_normal((T, qh, 2, d)).astype(np.float32))
        k = po.bf16_round(rng.standard_normal((T, kh, d)).astype(np.float32))
        v = po.bf16_round(rng.standard_normal((T, kh, d)).astype(np.float32))
        qw = (0.1 * rng.standard_normal(d)).astype(np.float32)
        kw_ = (0.1 * rng.standard_normal(d)).astype(np.float32)
        dy = rng.standard_normal((T, qh, d)).astype(np.float32)
    want = po.gqa_sequence_backward(op, qg, k, v, qw, kw_, dy, weight_grads=weight_grads)
    dq_norm = torch.zeros(d, device="cuda") if weight_grads else None
    dk_norm = torch.zeros(d, device="cuda") if weight_grads else None
    args = (p, dev(qg, torch.bfloat16), dev(k, torch.bfloat16), dev(v, torch.bfloat16), dev(qw),
            dev(kw_), dev(dy))
    dqg, dk, dv = capi.gqa_prefill_backward(*args, dq_norm=dq_norm, dk_norm=dk_norm)
    torch.cuda.synchronize()
    got = dict(dqg=dqg.cpu().numpy(), dk=dk.cpu().numpy(), dv=dv.cpu().numpy())
    if weight_grads:
        got["dq_norm"], got["dk_norm"] = dq_norm.cpu().numpy(), dk_norm.cpu().numpy()
    return got, want, args, (dq_norm, dk_norm)


@pytest.mark.parametrize("rounding", [False, True])
@pytest.mark.parametrize("shape", [(3, 2, 1, 3, 2), (3, 2, 1, 4, 2), (33, 4, 2, 24, 8),
                                   (128, 6, 2, 32, 8)])
def test_fp32_kernels_match_oracle(capi, shape, rounding):
    T, qh, kh, d, rot = shape
    got, want, _, _ = run_case(capi, T, qh, kh, d, rot, rounding)
    for name in ("dqg", "dk", "dv", "dq_norm", "dk_norm"):
        what = "%s T%d d%d" % (name, T, d)
        if not rounding:
            # 3e-5 is the reference's own bound against finite differences
            # (qwen_attention_test.cc:287); sums over many rows carry FP32 rounding
            assert_close(got[name], want[name], 1e-4, what)
            continue
        # The gate gradient multiplies by bf16(core): where the FP32 and the
        # double-precision core straddle a rounding tie that factor differs by
        # one bf16 ulp.  At most 0.1% of the elements may use the one-ulp bound.
        expected = want[name].astype(np.float64)
        diff = np.abs(got[name] - expected)
        scale = np.abs(expected) + np.sqrt(np.mean(expected ** 2))
        print("%s: max-abs error %.3e" % (what, diff.max()))
        assert np.all(diff <= 8e-3 * scale), what
        assert np.mean(diff > 1e-4 * scale) <= 1e-3, what


@pytest.mark.parametrize("shape", [(33, 4, 2, 64, 16), (128, 6, 2, 128, 32), (200, 8, 1, 64, 64),
                                   (65, 4, 4, 128, 32)])
def test_matrix_core_kernels_match_oracle(capi, shape):
    T, qh, kh, d, rot = shape
    got, want, _, _ = run_case(capi, T, qh, kh, d, rot, True, seed=T + d)
    for name in ("dqg", "dk", "dv", "dq_norm", "dk_norm"):
        assert_close_bf16_gradient(got[name], want[name], "%s T%d d%d" % (name, T, d))


@pytest.mark.parametrize("shape", [(200, 8, 2, 64, 32), (333, 6, 2, 128, 64)])
def test_state_saved_by_forward_gives_the_recomputed_gradients(capi, shape):
    """pluto_hip_gqa_prefill can leave the attention output before the gate and
    the row statistics for the backward pass (the role of the state
    SequenceForward hands to SequenceBackward, qwen_attention.cc:445-447); the
    gradients must be those of the self-contained call."""
    T, qh, kh, d, rot = shape
    got, want, args, _ = run_case(capi, T, qh, kh, d, rot, True, seed=T)
    p, qg, k, v, qw, kw_, dy = args
    cache = capi.KvCache(T, kh, d)
    saved = capi.gqa_prefill_saved(p, T, cache)
    assert saved is not None and saved.numel() >= T * qh * (2 * d + 8)
    capi.gqa_prefill(p, qg, k, v, qw, kw_, cache, saved=saved)
    dq_norm, dk_norm = torch.zeros(d, device="cuda"), torch.zeros(d, device="cuda")
    dqg, dk, dv = capi.gqa_prefill_backward(p, qg, k, v, qw, kw_, dy, dq_norm=dq_norm,
                                            dk_norm=dk_norm, saved=saved)
    torch.cuda.synchronize()
    with_saved = dict(dqg=dqg, dk=dk, dv=dv, dq_norm=dq_norm, dk_norm=dk_norm)
    for name, value in with_saved.items():
        # same kernels, same operands: the forward pass of the two calls differs
        # only in where K and V are read from
        np.testing.assert_allclose(value.cpu().numpy(), got[name], rtol=1e-5, atol=1e-6,
                                   err_msg=name)
        assert_close_bf16_gradient(value.cpu().numpy(), want[name], "%s T%d d%d" % (name, T, d))


def test_long_sequence_with_saved_state_matches_oracle(capi):
    """T=1024, one kv group of six 128-wide heads (the grouping of the benchmarked
    shape): eight query tiles, so the unpaired heaviest-first grid, with the block
    the forward pass saves.  Every gradient against the oracle."""
    T, qh, kh, d, rot = 1024, 6, 1, 128, 32
    got, want, args, _ = run_case(capi, T, qh, kh, d, rot, True, seed=77)
    assert capi.last_path() == capi.PATH_FLASH
    p, qg, k, v, qw, kw_, dy = args
    cache = capi.KvCache(T, kh, d)
    saved = capi.gqa_prefill_saved(p, T, cache)
    capi.gqa_prefill(p, qg, k, v, qw, kw_, cache, saved=saved)
    dq_norm, dk_norm = torch.zeros(d, device="cuda"), torch.zeros(d, device="cuda")
    dqg, dk, dv = capi.gqa_prefill_backward(p, qg, k, v, qw, kw_, dy, dq_norm=dq_norm,
                                            dk_norm=dk_norm, saved=saved)
    torch.cuda.synchronize()
    assert capi.last_path() == capi.PATH_FLASH
    with_saved = dict(dqg=dqg, dk=dk, dv=dv, dq_norm=dq_norm, dk_norm=dk_norm)
    for name, value in with_saved.items():
        assert_close_bf16_gradient(got[name], want[name], "%s T%d self-contained" % (name, T))
        assert_close_bf16_gradient(value.cpu().numpy(), want[name], "%s T%d saved" % (name, T))


def test_benchmarked_shape_against_fp32_kernels(capi):
    """The shape bench.py times (T=8192, 24 query / 4 kv heads of 128, saved block):
    the matrix-core kernels against the any-shape FP32-arithmetic kernels of the same
    library.  The CPU oracle would need an hour for this length; it covers the same
    kernels at T=1024 above."""
    T, qh, kh, d, rot = 8192, 24, 4, 128, 32
    p = capi.attention_params(query_heads=qh, key_value_heads=kh, head_dim=d, rotary_dim=rot,
                              capacity=T, round_to_bfloat16=True)
    gen = torch.Generator(device="cuda").manual_seed(2)
    bf = torch.bfloat16
    qg = (0.5 * torch.randn((T, qh, 2, d), generator=gen, device="cuda")).to(bf)
    k = (0.5 * torch.randn((T, kh, d), generator=gen, device="cuda")).to(bf)
    v = (0.5 * torch.randn((T, kh, d), generator=gen, device="cuda")).to(bf)
    dy = torch.randn((T, qh, d), generator=gen, device="cuda")
    qw, kw_ = dev(values(d, 0.2, 0.3)), dev(values(d, 0.8, 0.4))

    def once(saved):
        dq_norm, dk_norm = torch.zeros(d, device="cuda"), torch.zeros(d, device="cuda")
        dqg, dk, dv = capi.gqa_prefill_backward(p, qg, k, v, qw, kw_, dy, dq_norm=dq_norm,
                                                dk_norm=dk_norm, saved=saved)
        torch.cuda.synchronize()
        return dict(dqg=dqg, dk=dk, dv=dv, dq_norm=dq_norm, dk_norm=dk_norm)

    cache = capi.KvCache(T, kh, d)
    saved = capi.gqa_prefill_saved(p, T, cache)
    capi.gqa_prefill(p, qg, k, v, qw, kw_, cache, saved=saved)
    fast = once(saved)
    assert capi.last_path() == capi.PATH_FLASH
    with capi.force_generic():
        slow = once(None)
        assert capi.last_path() == capi.PATH_GENERIC
    for name in fast:
        # (fifty million elements: the tail of the per-element error reaches further
        # than in the small cases: the farthest observed sits at 19.1 times the
        # per-element bound; the max-norm bound still holds for every element)
        assert_close_bf16_gradient(fast[name].cpu().numpy(), slow[name].cpu().numpy(),
                                   "%s T%d vs fp32-arithmetic kernels" % (name, T), far=20.0)


def test_saved_state_is_refused_where_none_is_kept(capi):
    T, qh, kh, d, rot = 16, 2, 1, 32, 8
    kw = dict(query_heads=qh, key_value_heads=kh, head_dim=d, rotary_dim=rot, capacity=T,
              round_to_bfloat16=True)
    p = capi.attention_params(**kw)
    cache = capi.KvCache(T, kh, d)
    assert capi.gqa_prefill_saved(p, T, cache) is None  # head width without matrix-core backward
    lib = capi.lib()
    import ctypes
    fp32 = capi.attention_params(**dict(kw, head_dim=64, rotary_dim=16, round_to_bfloat16=False))
    assert lib.pluto_hip_gqa_prefill_saved_bytes(ctypes.byref(fp32), T, capi.BF16) == 0
    wide = capi.attention_params(**dict(kw, head_dim=64, rotary_dim=16))
    assert lib.pluto_hip_gqa_prefill_saved_bytes(ctypes.byref(wide), T, capi.F32) == 0
    assert lib.pluto_hip_gqa_prefill_saved_bytes(ctypes.byref(wide), T, capi.BF16) > 0
    # a block offered where none can be filled is an error, not silently ignored
    qg = torch.zeros((T, qh, 2, d), dtype=torch.bfloat16, device="cuda")
    k = torch.zeros((T, kh, d), dtype=torch.bfloat16, device="cuda")
    w = torch.zeros(d, device="cuda")
    bogus = torch.empty(1 << 16, dtype=torch.uint8, device="cuda")
    with pytest.raises(capi.PlutoHipError):
        capi.gqa_prefill(p, qg, k, k, w, w, cache, saved=bogus)
    dy = torch.zeros((T, qh, d), device="cuda")
    with pytest.raises(capi.PlutoHipError):
        capi.gqa_prefill_backward(p, qg, k, k, w, w, dy, saved=bogus)


def test_weight_gradients_accumulate_and_are_optional(capi):
    T, qh, kh, d, rot = 5, 2, 1, 8, 4
    got, want, args, (dq_norm, dk_norm) = run_case(capi, T, qh, kh, d, rot, True)
    again = capi.gqa_prefill_backward(*args, dq_norm=dq_norm, dk_norm=dk_norm)
    torch.cuda.synchronize()
    # shared norm gradients accumulate across calls (qwen_attention_test.cc:291-300)
    np.testing.assert_allclose(dq_norm.cpu().numpy(), 2 * got["dq_norm"], rtol=1e-6, atol=1e-7)
    np.testing.assert_allclose(dk_norm.cpu().numpy(), 2 * got["dk_norm"], rtol=1e-6, atol=1e-7)
    for a, name in zip(again, ("dqg", "dk", "dv")):
        np.testing.assert_array_equal(a.cpu().numpy(), got[name])  # repeatable, bit for bit
    frozen, _, _, _ = run_case(capi, T, qh, kh, d, rot, True, weight_grads=False)
    for name in ("dqg", "dk", "dv"):
        np.testing.assert_array_equal(frozen[name], got[name])


def test_later_rows_reach_earlier_keys_and_values(capi):
    # qwen_attention_test.cc:303-345: a gradient on the last row only still
    # reaches the first token's key and value
    from oracle import pyoracle as po
    T, qh, kh, d, rot = 3, 2, 1, 4, 2
    p = capi.attention_params(query_heads=qh, key_value_heads=kh, head_dim=d, rotary_dim=rot,
                              capacity=T, round_to_bfloat16=True)
    qg = po.bf16_round(values(T * qh * 2 * d, .1)).reshape(T, qh, 2, d)
    k = po.bf16_round(values(T * kh * d, 1.2)).reshape(T, kh, d)
    v = po.bf16_round(values(T * kh * d, 2.3)).reshape(T, kh, d)
    dy = np.zeros((T, qh, d), np.float32)
    dy[2] = 0.5
    _, dk, dv = capi.gqa_prefill_backward(p, dev(qg, torch.bfloat16), dev(k, torch.bfloat16),
                                          dev(v, torch.bfloat16), dev(values(d, .2)),
                                          dev(values(d, .4)), dev(dy))
    assert dk[0].abs().sum().item() > 1e-5 and dv[0].abs().sum().item() > 1e-5


def test_rejects_bad_arguments_before_touching_outputs(capi):
    p = capi.attention_params(query_heads=2, key_value_heads=1, head_dim=4, rotary_dim=2,
                              capacity=4, round_to_bfloat16=True)
    import ctypes
    lib = capi.lib()
    assert lib.pluto_hip_gqa_prefill_backward_workspace_bytes(ctypes.byref(p), 0, 0, 0) == 0
    size = lib.pluto_hip_gqa_prefill_backward_workspace_bytes(ctypes.byref(p), 3, 1, 1)
    assert size > 0
    x = torch.zeros(1024, device="cuda")
    rc = lib.pluto_hip_gqa_prefill_backward(capi.current_stream(), ctypes.byref(p), 3, capi.ptr(x),
                                            capi.ptr(x), capi.ptr(x), capi.ptr(x), capi.ptr(x),
                                            capi.ptr(x), None, capi.ptr(x), capi.ptr(x), capi.ptr(x),
                                            None, None, capi.ptr(x), 16)
    assert rc == capi.EWORKSPACE if hasattr(capi, "EWORKSPACE") else rc != 0
    rc = lib.pluto_hip_gqa_prefill_backward(capi.current_stream(), ctypes.byref(p), 3, None,
                                            capi.ptr(x), capi.ptr(x), capi.ptr(x), capi.ptr(x),
                                            capi.ptr(x), None, capi.ptr(x), capi.ptr(x), capi.ptr(x),
                                            None, None, capi.ptr(x), size)
    assert rc != 0
