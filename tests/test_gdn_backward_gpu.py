"""GPU parity of the gated delta-net layer backward
(SequenceDeltaNetLayer::bwd_impl, sequence_delta_net.cc:482-561) with the CPU
oracle, through the C ABI.  Shapes follow sequence_delta_net_test.cc (small odd
widths, grouped heads) and add the 128 x 128 head of the headline config."""
import numpy as np
import pytest

from tests.util import assert_close

pytestmark = pytest.mark.gpu

torch = pytest.importorskip("torch")


@pytest.fixture(scope="module")
def capi():
    from pluto_amd import capi
    assert torch.cuda.is_available(), "these tests need the GPU"
    capi.lib()
    return capi


def dev(x, dtype=None):
    t = torch.from_numpy(np.ascontiguousarray(x)).cuda()
    return t.to(dtype) if dtype is not None else t


def make_case(T, kh, vh, kd, vd, K, seed, batch=1):
    from oracle import pyoracle as po
    rng = np.random.default_rng(seed)
    channels = 2 * kh * kd + vh * vd
    r = lambda *shape: po.bf16_round(rng.standard_normal(shape).astype(np.float32))
    return dict(qkv=r(batch, T, channels), z=r(batch, T, vh * vd), a=r(batch, T, vh),
                b=r(batch, T, vh),
                conv=(0.5 * rng.standard_normal((channels, K))).astype(np.float32),
                a_log=(0.3 * rng.standard_normal(vh)).astype(np.float32),
                dt_bias=(0.3 * rng.standard_normal(vh)).astype(np.float32),
                norm=(1 + 0.2 * rng.standard_normal(vd)).astype(np.float32),
                dy=rng.standard_normal((batch, T, vh * vd)).astype(np.float32))


def run(capi, shape, rounding, seed=0, batch=1, with_parameters=True):
    from oracle import pyoracle as po
    T, kh, vh, kd, vd, K = shape
    kw = dict(key_heads=kh, value_heads=vh, key_head_dim=kd, value_head_dim=vd, conv_kernel_dim=K,
              round_to_bfloat16=rounding)
    p, op = capi.delta_params(**kw), po.delta_params(**kw)
    c = make_case(T, kh, vh, kd, vd, K, seed, batch)
    want = None
    for s in range(batch):
        one = po.gdn_sequence_backward(op, c["qkv"][s], c["z"][s], c["a"][s], c["b"][s], c["conv"],
                                       c["a_log"], c["dt_bias"], c["norm"], c["dy"][s])
        if want is None:
            want = {k: ([v] if k in ("dqkv", "dz", "da", "db") else v.copy()) for k, v in one.items()}
        else:
            for k, v in one.items():
                if k in ("dqkv", "dz", "da", "db"):
                    want[k].append(v)
                else:
                    want[k] += v
    for k in ("dqkv", "dz", "da", "db"):
        want[k] = np.stack(want[k])
    channels = 2 * kh * kd + vh * vd
    grads = None
    if with_parameters:
        grads = dict(conv_weight=torch.zeros(channels, K, device="cuda"),
                     a_log=torch.zeros(vh, device="cuda"), dt_bias=torch.zeros(vh, device="cuda"),
                     norm=torch.zeros(vd, device="cuda"))
    bf = torch.bfloat16
    args = (p, dev(c["qkv"], bf), dev(c["z"], bf), dev(c["a"], bf), dev(c["b"], bf), dev(c["conv"]),
            dev(c["a_log"]), dev(c["dt_bias"]), dev(c["norm"]), dev(c["dy"]))
    dqkv, dz, da, db = capi.gdn_layer_backward(*args, parameter_grads=grads)
    torch.cuda.synchronize()
    got = dict(dqkv=dqkv.cpu().numpy(), dz=dz.cpu().numpy(), da=da.cpu().numpy(),
               db=db.cpu().numpy())
    if grads:
        got.update(d_conv_weight=grads["conv_weight"].cpu().numpy(),
                   d_a_log=grads["a_log"].cpu().numpy(), d_dt_bias=grads["dt_bias"].cpu().numpy(),
                   d_norm=grads["norm"].cpu().numpy())
    return got, want, args, grads


# (T, key heads, value heads, key width, value width, conv taps).  128 x 128
# heads take the chunked kernels (64-token chunks: one full chunk, a ragged
# tail, grouped heads over several chunks, and 1, 2, 3, 4 and 5 chunks for the
# three operand sets the sequential kernels rotate); the other widths go token
# by token.
SHAPES = [(4, 1, 2, 3, 5, 3), (9, 2, 4, 5, 35, 4), (33, 2, 2, 16, 40, 4), (64, 1, 2, 128, 128, 4),
          (37, 1, 1, 128, 128, 4), (200, 1, 2, 128, 128, 4), (130, 2, 4, 128, 128, 3),
          (100, 1, 1, 128, 128, 2), (300, 1, 1, 128, 128, 4)]


@pytest.mark.parametrize("rounding", [False, True])
@pytest.mark.parametrize("shape", SHAPES)
def test_backward_matches_oracle(capi, shape, rounding):
    got, want, _, _ = run(capi, shape, rounding, seed=sum(shape))
    for name in want:
        what = "%s %s" % (name, shape)
        if not rounding:
            assert_close(got[name], want[name], 2e-4, what)
            continue
        # Rounded forward values enter as operands: where the FP32 and the
        # double-precision forward straddle a bf16 rounding tie an operand differs
        # by one ulp.  The bulk must agree to FP32 accuracy.
        expected = want[name].astype(np.float64)
        diff = np.abs(got[name] - expected)
        scale = np.abs(expected) + np.sqrt(np.mean(expected ** 2))
        print("%s: max-abs error %.3e" % (what, diff.max()))
        assert np.all(diff <= 2e-2 * scale), what
        assert np.mean(diff > 2e-4 * scale) <= 2e-2, what


def test_batch_and_parameter_gradient_accumulation(capi):
    shape = (7, 1, 2, 4, 6, 3)
    got, want, args, grads = run(capi, shape, False, seed=3, batch=3)
    for name in want:
        assert_close(got[name], want[name], 2e-4, name)
    first = {k: v.clone() for k, v in grads.items()}
    again = capi.gdn_layer_backward(*args, parameter_grads=grads)
    torch.cuda.synchronize()
    for k in grads:  # parameter gradients accumulate across calls
        np.testing.assert_allclose(grads[k].cpu().numpy(), 2 * first[k].cpu().numpy(), rtol=1e-5,
                                   atol=1e-6)
    for a, name in zip(again, ("dqkv", "dz", "da", "db")):
        np.testing.assert_array_equal(a.cpu().numpy(), got[name])  # repeatable
    frozen, _, _, _ = run(capi, shape, False, seed=3, batch=3, with_parameters=False)
    for name in ("dqkv", "dz", "da", "db"):
        np.testing.assert_array_equal(frozen[name], got[name])


def test_chunked_and_token_by_token_kernels_agree(capi):
    """128 x 128 heads over 9 chunks: the chunked kernels against the
    token-by-token kernels of the same library (FP32 both, different order of
    summation), at a length the CPU oracle would take minutes for."""
    import os
    shape = (520, 2, 4, 128, 128, 4)
    T, kh, vh, kd, vd, K = shape
    kw = dict(key_heads=kh, value_heads=vh, key_head_dim=kd, value_head_dim=vd, conv_kernel_dim=K,
              round_to_bfloat16=False)
    p = capi.delta_params(**kw)
    c = make_case(T, kh, vh, kd, vd, K, seed=11)
    bf = torch.bfloat16
    args = (p, dev(c["qkv"], bf), dev(c["z"], bf), dev(c["a"], bf), dev(c["b"], bf), dev(c["conv"]),
            dev(c["a_log"]), dev(c["dt_bias"]), dev(c["norm"]), dev(c["dy"]))
    channels = 2 * kh * kd + vh * vd

    def once():
        grads = dict(conv_weight=torch.zeros(channels, K, device="cuda"),
                     a_log=torch.zeros(vh, device="cuda"), dt_bias=torch.zeros(vh, device="cuda"),
                     norm=torch.zeros(vd, device="cuda"))
        out = capi.gdn_layer_backward(*args, parameter_grads=grads)
        torch.cuda.synchronize()
        named = dict(zip(("dqkv", "dz", "da", "db"), out))
        named.update(grads)
        return {k: v.cpu().numpy() for k, v in named.items()}

    chunked = once()
    with capi.force_generic():
        sequential = once()
    for name in sequential:
        assert_close(chunked[name], sequential[name], 2e-4, name)


def test_long_sequence_two_heads_matches_oracle(capi):
    """T=2048 (32 chunks), two 128 x 128 heads: the length bench.py times, at a head
    count the scalar oracle finishes in seconds.  The chunked kernels treat heads
    independently (one workgroup row per head)."""
    shape = (2048, 2, 2, 128, 128, 4)
    got, want, _, _ = run(capi, shape, False, seed=5)
    assert capi.last_path() == capi.PATH_CHUNKED
    for name in want:
        assert_close(got[name], want[name], 2e-4, "%s %s" % (name, shape))


def test_benchmarked_shape_against_token_by_token_kernels(capi):
    """The shape bench.py times (T=2048, sixteen 128 x 128 heads, every parameter
    trains): the chunked kernels against the token-by-token kernels of the same
    library, FP32 both."""
    shape = (2048, 16, 16, 128, 128, 4)
    T, kh, vh, kd, vd, K = shape
    p = capi.delta_params(key_heads=kh, value_heads=vh, key_head_dim=kd, value_head_dim=vd,
                          conv_kernel_dim=K, round_to_bfloat16=False)
    c = make_case(T, kh, vh, kd, vd, K, seed=4)
    bf = torch.bfloat16
    args = (p, dev(c["qkv"], bf), dev(c["z"], bf), dev(c["a"], bf), dev(c["b"], bf), dev(c["conv"]),
            dev(c["a_log"]), dev(c["dt_bias"]), dev(c["norm"]), dev(c["dy"]))
    channels = 2 * kh * kd + vh * vd

    def once():
        grads = dict(conv_weight=torch.zeros(channels, K, device="cuda"),
                     a_log=torch.zeros(vh, device="cuda"), dt_bias=torch.zeros(vh, device="cuda"),
                     norm=torch.zeros(vd, device="cuda"))
        out = capi.gdn_layer_backward(*args, parameter_grads=grads)
        torch.cuda.synchronize()
        named = dict(zip(("dqkv", "dz", "da", "db"), out))
        named.update(grads)
        return {k: v.cpu().numpy() for k, v in named.items()}

    chunked = once()
    assert capi.last_path() == capi.PATH_CHUNKED
    with capi.force_generic():
        sequential = once()
        assert capi.last_path() == capi.PATH_RECURRENCE
    for name in sequential:
        assert_close(chunked[name], sequential[name], 2e-4, name)


def test_rejects_bad_arguments(capi):
    import ctypes
    p = capi.delta_params(key_heads=1, value_heads=2, key_head_dim=4, value_head_dim=6,
                          conv_kernel_dim=3)
    lib = capi.lib()
    assert lib.pluto_hip_gdn_layer_backward_workspace_bytes(ctypes.byref(p), 0, 0) == 0
    assert lib.pluto_hip_gdn_layer_backward_workspace_bytes(ctypes.byref(p), 70000, 0) == 0
    size = lib.pluto_hip_gdn_layer_backward_workspace_bytes(ctypes.byref(p), 5, 1)
    assert size > 0
    x = torch.zeros(4096, device="cuda")
    ptrs = [capi.ptr(x)] * 13
    rc = lib.pluto_hip_gdn_layer_backward(capi.current_stream(), ctypes.byref(p), 1, 5, *ptrs, None,
                                          None, None, None, capi.ptr(x), 16)
    assert rc != 0  # workspace too small
    rc = lib.pluto_hip_gdn_layer_backward(capi.current_stream(), ctypes.byref(p), 1, 5, None,
                                          *ptrs[1:], None, None, None, None, capi.ptr(x), size)
    assert rc != 0  # null input
