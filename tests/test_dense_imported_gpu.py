"""GPU parity of the imported FullyConnectedLayer projection
(fully_connected.cc:40-94,295-341) with the CPU oracle, through the C ABI; the
cases are those of fully_connected_imported_test.cc."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu

torch = pytest.importorskip("torch")


@pytest.fixture(scope="module")
def capi():
    from pluto_amd import capi
    assert torch.cuda.is_available(), "these tests need the GPU"
    capi.lib()
    return capi


def bf16_tensor(oracle, values):
    return torch.from_numpy(oracle.bf16_round(np.float32(values))).cuda().to(torch.bfloat16)


def run(capi, oracle, storage, source, scales, x):
    """(library result, oracle result) for weights given as float values."""
    if storage == oracle.MATRIX_F32:
        host = np.float32(source)
        device = torch.from_numpy(host).cuda()
    elif storage == oracle.MATRIX_BF16:
        rounded = oracle.bf16_round(np.float32(source))
        host = (rounded.view(np.uint32) >> 16).astype(np.uint16)
        device = torch.from_numpy(rounded).cuda().to(torch.bfloat16)
    else:
        host = oracle.f32_to_fp8_e4m3(np.float32(source))
        device = torch.from_numpy(host).cuda()
    s_host = None if scales is None else np.float32(scales)
    s_device = None if scales is None else torch.from_numpy(s_host).cuda()
    token = oracle.bf16_round(np.float32(x))
    got = capi.dense_imported_forward(storage, device, s_device, bf16_tensor(oracle, token))
    torch.cuda.synchronize()
    want = oracle.imported_matvec(storage, host, s_host, token)
    return got.float().cpu().numpy(), want


def test_smallest_case_for_every_storage(capi, oracle):
    # fully_connected_imported_test.cc:93-136
    w = [[1, 2, 3], [4, 5, 6]]
    for storage, scales in ((oracle.MATRIX_F32, None), (oracle.MATRIX_BF16, None),
                            (oracle.MATRIX_FP8_E4M3, [1.0])):
        got, want = run(capi, oracle, storage, w, scales, [1, 0, -1])
        assert list(got) == [-2, -2] and list(want) == [-2, -2]


@pytest.mark.parametrize("cols,rows", [(263, 259), (5120, 131), (1024, 1000), (130, 9)])
def test_block_scales_tails_and_real_width(capi, oracle, cols, rows):
    # fully_connected_imported_test.cc:143-211: straddles the row tiles and the
    # 128 x 128 scale blocks, includes the checkpoint's 5120-wide input; rows
    # that start 16-byte aligned (vector loads) and rows that do not
    i = np.arange(cols * rows)
    source = (1.9 * np.sin((i % 1009).astype(np.float32) * np.float32(0.037))).reshape(rows, cols)
    x = (np.cos(np.arange(cols) * 0.123) * 0.25).astype(np.float32)
    scale_cols, scale_rows = (cols + 127) // 128, (rows + 127) // 128
    scales = [[(r + 1) * (c + 1) * 0.03125 for c in range(scale_cols)] for r in range(scale_rows)]
    for storage, s in ((oracle.MATRIX_F32, None), (oracle.MATRIX_BF16, None),
                       (oracle.MATRIX_FP8_E4M3, scales)):
        got, want = run(capi, oracle, storage, source, s, x)
        # the reference's own bound for this test (:206), FP32 against double sums
        assert np.all(np.abs(got - want) <= 5e-5 + 0.008 * np.abs(want)), storage
        # and nearly every output is the same bf16 value
        assert np.mean(got != want) <= 0.05, storage


def test_dynamic_quantization_zero_tiny_ties_and_tail(capi, oracle):
    # fully_connected_imported_test.cc:213-253: an identity matrix exposes every
    # quantized input
    width = 389
    x = np.zeros(width, np.float32)
    for i in range(128, 256):
        x[i] = ((i % 31) - 15) * 0.0625
    x[128], x[129], x[130], x[131] = 448, -448, 1.0625, 1.1875
    for i in range(256, 384):
        x[i] = (i % 5 - 2) * 1e-14
    for i in range(384, width):
        x[i] = (i - 386) * 25.3
    x = oracle.bf16_round(x)
    got, want = run(capi, oracle, oracle.MATRIX_FP8_E4M3, np.eye(width, dtype=np.float32),
                    np.ones((4, 4), np.float32), x)
    expected = oracle.bf16_round(oracle.imported_quantize(x))
    assert np.array_equal(want, expected)
    assert np.array_equal(got, expected)   # one product per row: no summation-order slack
    assert got[130] == 1.0 and got[131] == 1.25
    assert np.all(got[:128] == 0) and got[128] == 448 and got[129] == -448
    assert np.abs(got[256:384]).max() > 0


def test_every_fp8_code_as_a_weight(capi, oracle):
    """Row r holds code r once, in a column that the 16-byte path reads (rows
    of 128 codes) or in one that the element path reads (rows of 130)."""
    codes = np.arange(256)
    keep = (codes & 0x7f) != 0x7f   # the two NaN codes
    for cols, column in ((128, 37), (130, 129)):
        weights = np.zeros((256, cols), np.uint8)
        weights[codes, column] = codes
        x = np.zeros(cols, np.float32)
        x[column] = 1.0     # a group maximum of 1: quantized exactly
        scales = np.ones((2, (cols + 127) // 128), np.float32)
        got = capi.dense_imported_forward(capi.MATRIX_FP8_E4M3, torch.from_numpy(weights).cuda(),
                                          torch.from_numpy(scales).cuda(), bf16_tensor(oracle, x))
        torch.cuda.synchronize()
        got = got.float().cpu().numpy()
        want = oracle.bf16_round(oracle.fp8_e4m3_to_f32(codes.astype(np.uint8)))
        assert np.array_equal(got[keep], want[keep]), cols
        assert np.all(np.isnan(got[~keep]))


@pytest.mark.parametrize("cols,tokens", [(263, 11), (512, 7), (512, 40), (1024, 33)])
def test_batch_rows_match_the_one_token_calls(capi, oracle, cols, tokens):
    """Up to eight tokens, and rows that are not whole 128-element blocks, run
    as vector passes of 8, 4, 2 and 1 tokens whose rows are bit for bit the
    one-token results; larger batches of whole blocks run on the matrix cores
    (passes of 32 tokens, here with a partial pass and partial row tiles) and
    agree to FP32 summation order."""
    rows = 70
    exact = tokens <= 8 or cols % 128 != 0
    rng = np.random.default_rng(cols + tokens)
    source = rng.standard_normal((rows, cols)).astype(np.float32)
    x = bf16_tensor(oracle, rng.standard_normal((tokens, cols)))
    scales = torch.from_numpy(rng.uniform(0.5, 2.0, ((rows + 127) // 128, (cols + 127) // 128))
                              .astype(np.float32)).cuda()
    cases = [(capi.MATRIX_F32, torch.from_numpy(source).cuda(), None),
             (capi.MATRIX_BF16, torch.from_numpy(source).cuda().to(torch.bfloat16), None),
             (capi.MATRIX_FP8_E4M3, torch.from_numpy(oracle.f32_to_fp8_e4m3(source)).cuda(), scales)]
    for storage, weights, s in cases:
        batch = capi.dense_imported_forward_batch(storage, weights, s, x)
        singles = torch.stack([capi.dense_imported_forward(storage, weights, s, x[t].contiguous())
                               for t in range(tokens)])
        torch.cuda.synchronize()
        if exact or storage == capi.MATRIX_F32:
            assert torch.equal(batch.view(torch.int16), singles.view(torch.int16)), storage
        else:
            got, want = batch.float().cpu().numpy(), singles.float().cpu().numpy()
            # the reference's bound for this layer (fully_connected_imported_test.cc:206)
            assert np.all(np.abs(got - want) <= 5e-5 + 0.008 * np.abs(want)), storage
            assert np.mean(got != want) <= 0.05, storage
    lib = capi.lib()
    assert lib.pluto_hip_dense_imported_batch_workspace_bytes(0, cols) == 0
    assert lib.pluto_hip_dense_imported_batch_workspace_bytes(4097, cols) == 0
    assert lib.pluto_hip_dense_imported_batch_workspace_bytes(tokens, cols) >= tokens * cols * 4


def test_matrix_core_batch_matches_the_oracle(capi, oracle):
    """32 tokens against the CPU oracle for bf16 and FP8 weights with block
    scales that differ per block, 300 rows (partial row tile and three scale
    row blocks), 384 columns."""
    rows, cols, tokens = 300, 384, 32
    rng = np.random.default_rng(5)
    source = (rng.standard_normal((rows, cols)) * 1.5).astype(np.float32)
    x_host = oracle.bf16_round(rng.standard_normal((tokens, cols)).astype(np.float32))
    x = torch.from_numpy(x_host).cuda().to(torch.bfloat16)
    scales = rng.uniform(0.25, 4.0, ((rows + 127) // 128, cols // 128)).astype(np.float32)
    rounded = oracle.bf16_round(source)
    bits = (rounded.view(np.uint32) >> 16).astype(np.uint16)
    codes = oracle.f32_to_fp8_e4m3(source)
    for storage, device, host, s in (
            (capi.MATRIX_BF16, torch.from_numpy(rounded).cuda().to(torch.bfloat16), bits, None),
            (capi.MATRIX_FP8_E4M3, torch.from_numpy(codes).cuda(), codes, scales)):
        got = capi.dense_imported_forward_batch(
            storage, device, None if s is None else torch.from_numpy(s).cuda(), x)
        torch.cuda.synchronize()
        got = got.float().cpu().numpy()
        for t in range(tokens):
            want = oracle.imported_matvec(storage, host, s, x_host[t])
            assert np.all(np.abs(got[t] - want) <= 5e-5 + 0.008 * np.abs(want)), (storage, t)
            assert np.mean(got[t] != want) <= 0.05, (storage, t)


@pytest.mark.parametrize("cols,tokens", [(512, 32), (512, 40), (1024, 33), (512, 5), (263, 11)])
def test_several_matrices_of_one_input_match_the_single_calls(capi, oracle, cols, tokens):
    """The query | gate, key and value projections of a block (qwen/model.cc:174-274)
    see the same rows: pluto_hip_dense_imported_forward_many prepares the tokens
    once and walks the tiles of all matrices in one launch a pass.  Bit for
    bit the batch call's results for every matrix, on the matrix-core path
    (partial passes, partial row tiles, a matrix smaller than a tile) and on the
    vector path it falls back to (few tokens, ragged widths, FP32 weights)."""
    heights = [70, 1000, 32, 7, 129]
    rng = np.random.default_rng(cols * 3 + tokens)
    x = bf16_tensor(oracle, rng.standard_normal((tokens, cols)))
    sources = [rng.standard_normal((rows, cols)).astype(np.float32) for rows in heights]
    scales = [torch.from_numpy(rng.uniform(0.5, 2.0, ((rows + 127) // 128, (cols + 127) // 128))
                               .astype(np.float32)).cuda() for rows in heights]
    cases = [(capi.MATRIX_F32, [torch.from_numpy(w).cuda() for w in sources], None),
             (capi.MATRIX_BF16, [torch.from_numpy(w).cuda().to(torch.bfloat16) for w in sources], None),
             (capi.MATRIX_FP8_E4M3,
              [torch.from_numpy(oracle.f32_to_fp8_e4m3(w)).cuda() for w in sources], scales)]
    for storage, weights, s in cases:
        many = capi.dense_imported_forward_many(storage, weights, s, x)
        for i, w in enumerate(weights):
            single = capi.dense_imported_forward_batch(storage, w, None if s is None else s[i], x)
            torch.cuda.synchronize()
            assert torch.isfinite(single.float()).all()
            assert torch.equal(many[i].view(torch.int16), single.view(torch.int16)), (storage, i)
    # one matrix is the batch call
    storage, weights, s = cases[2]
    alone = capi.dense_imported_forward_many(storage, weights[1:2], s[1:2], x)[0]
    assert torch.equal(alone, capi.dense_imported_forward_batch(storage, weights[1], s[1], x))


def test_several_matrices_rejections(capi):
    import ctypes
    lib = capi.lib()
    w = torch.zeros((32, 128), dtype=torch.bfloat16, device="cuda")
    x = torch.zeros((16, 128), dtype=torch.bfloat16, device="cuda")
    y = torch.full((16, 32), -3.0, dtype=torch.bfloat16, device="cuda")
    ws = torch.zeros(1 << 16, dtype=torch.uint8, device="cuda")
    s = torch.ones(1, dtype=torch.float32, device="cuda")
    stream = capi.current_stream()
    pointers = ctypes.c_void_p * 9

    def call(storage=capi.MATRIX_BF16, count=2, weights=(w, w), scales=None, dims=(32, 32),
             outs=(y, y), tokens=16, cols=128, workspace_bytes=1 << 16, null_arrays=False):
        w_list = pointers(*[t.data_ptr() for t in weights])
        o_list = pointers(*[t.data_ptr() for t in outs])
        s_list = None if scales is None else pointers(*[None if t is None else t.data_ptr()
                                                        for t in scales])
        return lib.pluto_hip_dense_imported_forward_many(
            stream, storage, count, None if null_arrays else w_list, s_list,
            (ctypes.c_int * 9)(*dims), capi.ptr(x), tokens, cols, o_list, capi.ptr(ws),
            workspace_bytes)

    assert call() == 0
    assert call(count=0) == capi.EINVAL and call(count=9, weights=(w,) * 9, dims=(32,) * 9,
                                                 outs=(y,) * 9) == capi.EINVAL
    assert call(null_arrays=True) == capi.EINVAL
    assert call(dims=(32, 0)) == capi.EINVAL and call(cols=0) == capi.EINVAL
    assert call(tokens=0) == capi.EINVAL and call(tokens=4097) == capi.EINVAL
    assert call(storage=capi.MATRIX_FP8_E4M3) == capi.EINVAL            # FP8 without scales
    assert call(storage=capi.MATRIX_FP8_E4M3, scales=(s, None)) == capi.EINVAL
    assert call(scales=(s, s)) == capi.EINVAL                             # scales without FP8
    assert call(workspace_bytes=4) == capi.EWORKSPACE
    torch.cuda.synchronize()


def test_rejects_bad_arguments(capi):
    lib = capi.lib()
    w = torch.zeros(6, dtype=torch.float32, device="cuda")
    x = torch.zeros(3, dtype=torch.bfloat16, device="cuda")
    y = torch.zeros(2, dtype=torch.bfloat16, device="cuda")
    ws = torch.zeros(4096, dtype=torch.uint8, device="cuda")
    s = torch.ones(1, dtype=torch.float32, device="cuda")
    stream = capi.current_stream()

    def call(storage=capi.MATRIX_F32, scales=None, cols=3, rows=2, workspace_bytes=4096):
        return lib.pluto_hip_dense_imported_forward(
            stream, storage, capi.ptr(w), None if scales is None else capi.ptr(scales),
            capi.ptr(x), cols, rows, capi.ptr(y), capi.ptr(ws), workspace_bytes)

    assert call() == 0
    assert call(storage=7) == capi.EINVAL
    assert call(scales=s) == capi.EINVAL                       # scales without FP8 weights
    assert call(storage=capi.MATRIX_FP8_E4M3) == capi.EINVAL   # FP8 weights without scales
    assert call(cols=0) == capi.EINVAL and call(rows=-1) == capi.EINVAL
    assert call(cols=1048577) == capi.EINVAL
    assert call(workspace_bytes=4) == capi.EWORKSPACE
    assert lib.pluto_hip_dense_imported_workspace_bytes(0) == 0
    assert lib.pluto_hip_dense_imported_workspace_bytes(3) >= 12
    torch.cuda.synchronize()
