"""Pins the CPU oracle of the imported (frozen, output-major) projection of
FullyConnectedLayer (fully_connected.cc:40-94,295-341): the FP8 E4M3
conversions against torch's float8_e4m3fn (a library routine) over all codes
and over ties, the group quantization against the known answers of
fully_connected_imported_test.cc:213-253, and the projection against float64
products for the three storages (the scalar projection of :190-205)."""
import numpy as np
import pytest

torch = pytest.importorskip("torch")


def test_every_fp8_code_decodes_like_the_library(oracle):
    codes = np.arange(256, dtype=np.uint8)
    got = oracle.fp8_e4m3_to_f32(codes)
    want = torch.from_numpy(codes).view(torch.float8_e4m3fn).float().numpy()
    assert np.array_equal(np.isnan(got), np.isnan(want))
    keep = ~np.isnan(want)
    assert np.array_equal(got[keep], want[keep])
    assert got[0x7e] == 448.0 and got[0x01] == 2.0 ** -9 and got[0x08] == 2.0 ** -6


def test_fp8_encoding_rounds_to_even_and_saturates(oracle):
    rng = np.random.default_rng(3)
    values = np.concatenate([
        rng.standard_normal(4000) * 3, rng.standard_normal(2000) * 200,
        rng.standard_normal(2000) * 1e-2, rng.standard_normal(1000) * 2e-3,
        # ties between neighbours, zero, the subnormal edge, the largest value
        [1.0625, 1.1875, -1.0625, 0.0, -0.0, 2.0 ** -10, 3 * 2.0 ** -10, 2.0 ** -9, 447.0, 448.0,
         464.0, 480.0, 1e9, -1e9, 2.0 ** -6, 0.0175]]).astype(np.float32)
    got = oracle.f32_to_fp8_e4m3(values)
    inside = np.abs(values) <= 464.0   # the library does not saturate beyond that
    want = torch.from_numpy(values).to(torch.float8_e4m3fn).view(torch.uint8).numpy()
    assert np.array_equal(got[inside], want[inside])
    outside = oracle.fp8_e4m3_to_f32(got[~inside])
    assert np.array_equal(np.abs(outside), np.full(outside.shape, 448.0, np.float32))
    decoded = oracle.fp8_e4m3_to_f32(oracle.f32_to_fp8_e4m3(np.float32([1.0625, 1.1875])))
    assert list(decoded) == [1.0, 1.25]


def test_group_quantization_known_answers(oracle):
    # fully_connected_imported_test.cc:213-253
    width = 389
    x = np.zeros(width, np.float32)
    for i in range(128, 256):
        x[i] = ((i % 31) - 15) * 0.0625
    x[128], x[129], x[130], x[131] = 448, -448, 1.0625, 1.1875
    for i in range(256, 384):
        x[i] = oracle.bf16_round(np.float32((i % 5 - 2) * 1e-14))
    for i in range(384, width):
        x[i] = oracle.bf16_round(np.float32((i - 386) * 25.3))
    q = oracle.imported_quantize(x)
    assert np.all(q[:128] == 0)                       # zero group stays zero
    assert q[128] == 448 and q[129] == -448
    assert q[130] == 1.0 and q[131] == 1.25            # unit scale, ties to even
    # every element within half a step of its group's grid
    for g0 in (128, 384):
        group = slice(g0, min(g0 + 128, width))
        scale = np.abs(x[group]).max() / 448
        assert np.all(np.abs(q[group] - x[group]) <= 0.0625 * np.abs(x[group]) + scale * 2.0 ** -10)
    # the tiny group: its scale (max / 448 = 4.5e-17) is below the divisor's
    # floor, so x / 1e-12 = +-0.01, +-0.02 lands on the grid values 5 * 2^-9
    # and 10 * 2^-9, and the result carries the group's own scale
    tiny = slice(256, 384)
    scale = np.float32(np.abs(x[tiny]).max() / np.float32(448))
    ratio = np.abs(q[tiny]) / scale
    assert set(np.round(ratio * 512).astype(int)) == {0, 5, 10}
    assert np.array_equal(np.sign(q[tiny]), np.sign(x[tiny]))


@pytest.mark.parametrize("cols,rows", [(263, 259), (5120, 131), (3, 2)])
def test_projection_matches_float64_products(oracle, cols, rows):
    # fully_connected_imported_test.cc:143-211
    i = np.arange(cols * rows)
    source = (1.9 * np.sin((i % 1009).astype(np.float32) * np.float32(0.037))).astype(np.float32)
    source = source.reshape(rows, cols)
    x = oracle.bf16_round((np.cos(np.arange(cols) * 0.123) * 0.25).astype(np.float32))
    scale_cols, scale_rows = (cols + 127) // 128, (rows + 127) // 128
    scales = np.float32([[(r + 1) * (c + 1) * 0.03125 for c in range(scale_cols)]
                         for r in range(scale_rows)])
    w_bf16 = oracle.bf16_round(source)
    bits = (w_bf16.view(np.uint32) >> 16).astype(np.uint16)
    codes = oracle.f32_to_fp8_e4m3(source)
    w_fp8 = oracle.fp8_e4m3_to_f32(codes) * np.repeat(np.repeat(scales, 128, 0), 128, 1)[:rows, :cols]
    cases = [(oracle.MATRIX_F32, source, None, source, x),
             (oracle.MATRIX_BF16, bits, None, w_bf16, x),
             (oracle.MATRIX_FP8_E4M3, codes, scales, w_fp8, oracle.imported_quantize(x))]
    for storage, weights, s, values, token in cases:
        got = oracle.imported_matvec(storage, weights, s, x)
        want = values.astype(np.float64) @ token.astype(np.float64)
        assert np.all(np.abs(got - want) <= 2.0 ** -8 * np.abs(want) + 1e-30), storage
        assert np.array_equal(got, oracle.bf16_round(got))   # bf16 values


def test_smallest_case_known_answer(oracle):
    # fully_connected_imported_test.cc:93-136: [[1,2,3],[4,5,6]] . (1,0,-1) = (-2,-2)
    w = np.float32([[1, 2, 3], [4, 5, 6]])
    x = np.float32([1, 0, -1])
    bits = (w.view(np.uint32) >> 16).astype(np.uint16)
    assert list(oracle.imported_matvec(oracle.MATRIX_F32, w, None, x)) == [-2, -2]
    assert list(oracle.imported_matvec(oracle.MATRIX_BF16, bits, None, x)) == [-2, -2]
    assert list(oracle.imported_matvec(oracle.MATRIX_FP8_E4M3, oracle.f32_to_fp8_e4m3(w),
                                       np.float32([1]), x)) == [-2, -2]
    with pytest.raises(ValueError):
        oracle.imported_matvec(oracle.MATRIX_F32, w, np.float32([1]), x)
