"""GPU parity of the FullyConnectedLayer kernels (fully_connected.cc:97-247)
with the CPU oracle, through the C ABI: widths on the matrix cores (multiples
of 64, ragged row counts) and arbitrary positive widths."""
import ctypes

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


def case(oracle, dtype, rows, n_in, n_out, seed):
    rng = np.random.default_rng(seed)
    x = rng.standard_normal((rows, n_in)).astype(np.float32)
    if dtype == "bf16":
        x = oracle.bf16_round(x)
    w = (rng.standard_normal((n_in, n_out)) / np.sqrt(n_in)).astype(np.float32)
    b = rng.standard_normal(n_out).astype(np.float32)
    dy = rng.standard_normal((rows, n_out)).astype(np.float32)
    return x, w, b, dy


# (rows, input_dim, output_dim): matrix-core widths with whole and ragged
# tiles, a width of 64 mod 128 on either side, and widths the matrix-core
# kernels do not take (fully_connected.h:18: any positive width)
SHAPES = [(128, 64, 64), (200, 128, 192), (77, 192, 64), (300, 64, 320), (1, 128, 128),
          (5, 7, 3), (70, 65, 129), (33, 128, 66),
          # contractions of 1536 and more take the 256 x 256 tiles (forward:
          # input_dim, input gradient: output_dim), here with ragged tiles
          (300, 1536, 64), (260, 64, 1536)]


@pytest.mark.parametrize("dtype", ["bf16", "f32"])
@pytest.mark.parametrize("shape", SHAPES)
def test_forward_and_backward_match_oracle(capi, oracle, dtype, shape):
    rows, n_in, n_out = shape
    x, w, b, dy = case(oracle, dtype, rows, n_in, n_out, seed=sum(shape))
    code = oracle.BF16 if dtype == "bf16" else oracle.F32
    want_y = oracle.dense_forward(code, x, w, b)
    want_dx, want_dw, want_db = oracle.dense_backward(code, x, w, dy)
    tx = torch.from_numpy(x).cuda()
    if dtype == "bf16":
        tx = tx.to(torch.bfloat16)
    tw, tb, tdy = (torch.from_numpy(v).cuda() for v in (w, b, dy))
    y = capi.dense_forward(tx, tw, tb)
    dx, dw, db = capi.dense_backward(tx, tw, tdy)
    torch.cuda.synchronize()
    got_y = y.float().cpu().numpy()
    if dtype == "bf16":
        # the FP32 sum differs from the double one in its last bits: an output
        # next to a bf16 rounding tie may land on the neighbouring value
        diff = np.abs(got_y - want_y)
        assert np.all(diff <= 2.0 ** -7 * np.abs(want_y) + 1e-6), diff.max()
        assert np.mean(diff > 0) <= 2e-2
    else:
        assert_close(got_y, want_y, 1e-5, "y %s" % (shape,))
    # operands are rounded identically on both sides; only the FP32 summation
    # order differs from the oracle's double sums
    assert_close(dx.cpu().numpy(), want_dx, 1e-5, "dx %s" % (shape,))
    assert_close(dw.cpu().numpy(), want_dw, 2e-5, "dw %s" % (shape,))
    assert_close(db.cpu().numpy(), want_db, 1e-5, "db %s" % (shape,))


def test_bench_shape_matches_float64_products(capi, oracle):
    """The GPT-2-small QKV projection at its full size (16384 rows, 768 ->
    2304, bf16): every output against float64 matrix products of the same
    rounded operands, computed by the library on the GPU; the weight gradient
    there runs in four row slices and the bias gradient in 64 partitions."""
    rows, n_in, n_out = 16384, 768, 2304
    g = torch.Generator(device="cuda").manual_seed(7)
    x = torch.randn(rows, n_in, device="cuda", generator=g).to(torch.bfloat16)
    w = torch.randn(n_in, n_out, device="cuda", generator=g) / n_in ** 0.5
    b = torch.randn(n_out, device="cuda", generator=g)
    dy = torch.randn(rows, n_out, device="cuda", generator=g)
    y = capi.dense_forward(x, w, b)
    dx, dw, db = capi.dense_backward(x, w, dy)
    x64 = x.double()
    w64 = w.to(torch.bfloat16).double()
    dy64 = dy.to(torch.bfloat16).double()
    want_y = x64 @ w64 + b.double()
    diff = (y.double() - want_y).abs()
    assert bool((diff <= 2.0 ** -7 * want_y.abs() + 1e-6).all()), float(diff.max())

    def close(got, want, tolerance, what):
        error = float((got.double() - want).abs().max())
        scale = float(want.abs().max())
        assert error <= tolerance * scale, (what, error, scale)

    close(dx, dy64 @ w64.t(), 1e-5, "dx")
    close(dw, x64.t() @ dy64, 2e-5, "dw")
    close(db, dy.double().sum(0), 1e-5, "db")


def test_gradients_are_overwritten_and_repeatable(capi, oracle):
    rows, n_in, n_out = 700, 128, 192
    x, w, b, dy = case(oracle, "bf16", rows, n_in, n_out, seed=1)
    tx = torch.from_numpy(x).cuda().to(torch.bfloat16)
    tw, tdy = torch.from_numpy(w).cuda(), torch.from_numpy(dy).cuda()
    first = capi.dense_backward(tx, tw, tdy)
    second = capi.dense_backward(tx, tw, tdy)
    torch.cuda.synchronize()
    for a, c in zip(first, second):
        np.testing.assert_array_equal(a.cpu().numpy(), c.cpu().numpy())


def test_packed_qkv_projection_feeds_attention(capi, oracle):
    """gpt2.cc:55-71: the QKV projection's output is the attention layer's packed
    operand; no repacking or cast sits between the two calls."""
    T, H, E, B = 64, 2, 128, 2
    rng = np.random.default_rng(9)
    x = oracle.bf16_round(rng.standard_normal((B * T, E)).astype(np.float32))
    w = (rng.standard_normal((E, 3 * E)) / np.sqrt(E)).astype(np.float32)
    b = np.zeros(3 * E, np.float32)
    tx = torch.from_numpy(x).cuda().to(torch.bfloat16)
    qkv = capi.dense_forward(tx, torch.from_numpy(w).cuda(), torch.from_numpy(b).cuda())
    out, _, _ = capi.mha_forward(qkv, T, H)
    torch.cuda.synchronize()
    want_qkv = oracle.dense_forward(oracle.BF16, x, w, b)
    got_qkv = qkv.float().cpu().numpy()
    assert np.mean(np.abs(got_qkv - want_qkv) > 0) <= 2e-2
    # attention of the oracle on the values the projection produced
    want, _, _ = oracle.mha_fwd(got_qkv, T, H)
    from tests.util import assert_close_bf16
    assert_close_bf16(out.float().cpu().numpy(), want, "attention on the projected QKV")


def test_rejects_bad_arguments(capi):
    lib = capi.lib()
    assert lib.pluto_hip_dense_workspace_bytes(capi.BF16, 0, 64, 64) == 0
    assert lib.pluto_hip_dense_workspace_bytes(7, 8, 64, 64) == 0
    size = lib.pluto_hip_dense_workspace_bytes(capi.BF16, 8, 64, 64)
    assert size > 0
    x = torch.zeros(8192, device="cuda")
    px = capi.ptr(x)
    stream = capi.current_stream()
    assert lib.pluto_hip_dense_forward(stream, 7, px, px, px, 8, 64, 64, px, px, size) != 0
    assert lib.pluto_hip_dense_forward(stream, capi.BF16, px, px, px, 8, 64, 64, px, px, 16) != 0
    assert lib.pluto_hip_dense_forward(stream, capi.BF16, None, px, px, 8, 64, 64, px, px, size) != 0
    assert lib.pluto_hip_dense_backward(stream, capi.BF16, px, px, px, 8, 0, 64, px, px, px, px,
                                        size) != 0
