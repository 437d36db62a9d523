"""pluto_hip_gqa_decode_static, the decode step for callers that cannot allocate
(fixed scratch inside the library), against pluto_hip_gqa_decode on the same
inputs, through the C ABI: bit for bit, on two calls in a row, the second one
smaller than the first.  Collected last: a failure here must not hide the
parity tests."""
import ctypes

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


def values(count, phase, scale=1.0):
    i = np.arange(count, dtype=np.float32)
    return (np.float32(scale) * np.sin(np.float32(phase) + i * np.float32(0.29))).astype(np.float32)


def make_case(capi, seed, batch, qh, kh, d, capacity, lengths):
    gen = torch.Generator(device="cuda").manual_seed(seed)
    bf = torch.bfloat16

    def caches():
        made = []
        g = torch.Generator(device="cuda").manual_seed(seed + 1)
        for L in lengths:
            c = capi.KvCache(capacity, kh, d, fill=float("nan"))
            c.keys[:, :L - 1] = torch.randn((kh, L - 1, d), generator=g, device="cuda").to(bf)
            c.values[:, :L - 1] = torch.randn((kh, L - 1, d), generator=g, device="cuda").to(bf)
            c.position = int(L - 1)
            made.append(c)
        return made

    q_gate = torch.randn((batch, qh, 2, d), generator=gen, device="cuda").to(bf)
    k = torch.randn((batch, kh, d), generator=gen, device="cuda").to(bf)
    v = torch.randn((batch, kh, d), generator=gen, device="cuda").to(bf)
    qw = torch.from_numpy(values(d, 0.2, 0.3)).cuda()
    kw = torch.from_numpy(values(d, 0.8, 0.4)).cuda()
    return caches, q_gate, k, v, qw, kw


def run_both(capi, p, case, lengths, split):
    caches, q_gate, k, v, qw, kw = case
    positions = [int(L - 1) for L in lengths]
    with_workspace, fixed = caches(), caches()
    want = capi.gqa_decode(p, q_gate, k, v, qw, kw, with_workspace, positions=positions,
                           split_tokens=split, advance=False)
    got = torch.full_like(want, float("nan"))
    capi.gqa_decode_static(p, q_gate, k, v, qw, kw, fixed, positions, got, split_tokens=split)
    torch.cuda.synchronize()
    assert torch.isfinite(want.float()).all()
    assert torch.equal(got, want)
    # both calls appended the same row to their caches
    for a, b, L in zip(with_workspace, fixed, lengths):
        assert torch.equal(a.keys[:, :L], b.keys[:, :L])
        assert torch.equal(a.values[:, :L], b.values[:, :L])


def test_two_calls_in_a_row_second_one_smaller(capi):
    handle = capi.lib()
    assert handle.pluto_hip_gqa_decode_static_bytes() == 16 * 2 ** 20
    assert handle.pluto_hip_gqa_decode_static_prepare() == 0
    batch, qh, kh, d, capacity = 32, 24, 4, 128, 32768
    p = capi.attention_params(qh, kh, d, 32, capacity=capacity)
    rng = np.random.default_rng(3)
    lengths = 1024 + np.floor(rng.random(batch) * 31745).astype(int)
    lengths[0], lengths[1] = 1024, 32768
    run_both(capi, p, make_case(capi, 11, batch, qh, kh, d, capacity, lengths), lengths, 512)
    # smaller: fewer sequences, shorter contexts, another block size; the scratch
    # still holds the first call's partial results
    batch, lengths = 5, np.array([1, 64, 65, 700, 2049])
    run_both(capi, p, make_case(capi, 12, batch, qh, kh, d, capacity, lengths), lengths, 128)
    # and the first shape once more, after the smaller call
    batch = 32
    lengths = 1024 + np.floor(np.random.default_rng(5).random(batch) * 31745).astype(int)
    run_both(capi, p, make_case(capi, 13, batch, qh, kh, d, capacity, lengths), lengths, 512)


def test_the_models_head_width_on_both_block_size_paths(capi):
    """Heads of 256 (cached_attention_ops.h:13-22): the default block of 1024
    rows takes the kernel's compile-time request order, 512 its run-time loops;
    the same scratch serves both, one call after the other."""
    batch, qh, kh, d, capacity = 6, 12, 2, 256, 4096
    p = capi.attention_params(qh, kh, d, 64, capacity=capacity)
    lengths = np.array([4096, 1, 1024, 1025, 2500, 300])
    run_both(capi, p, make_case(capi, 31, batch, qh, kh, d, capacity, lengths), lengths, 0)
    lengths = np.array([700, 3000, 513, 4096, 64, 1024])
    run_both(capi, p, make_case(capi, 32, batch, qh, kh, d, capacity, lengths), lengths, 512)
    run_both(capi, p, make_case(capi, 33, batch, qh, kh, d, capacity, lengths), lengths, 1024)


def test_reset_then_another_call(capi):
    """pluto_hip_gqa_decode_static_reset between two calls: the second call starts
    from cleared arrival counters and still matches the workspace entry point."""
    handle = capi.lib()
    batch, qh, kh, d, capacity = 7, 24, 4, 128, 8192
    p = capi.attention_params(qh, kh, d, 32, capacity=capacity)
    lengths = np.array([1, 513, 4097, 8192, 700, 1024, 2048])
    run_both(capi, p, make_case(capi, 21, batch, qh, kh, d, capacity, lengths), lengths, 512)
    assert handle.pluto_hip_gqa_decode_static_reset(capi.current_stream()) == 0
    lengths = np.array([8192, 5, 1025, 64, 3000, 512, 6000])
    run_both(capi, p, make_case(capi, 22, batch, qh, kh, d, capacity, lengths), lengths, 256)
    # a reset with nothing before it on the stream changes nothing either
    assert handle.pluto_hip_gqa_decode_static_reset(capi.current_stream()) == 0
    assert handle.pluto_hip_gqa_decode_static_reset(capi.current_stream()) == 0
    run_both(capi, p, make_case(capi, 23, batch, qh, kh, d, capacity, lengths), lengths, 512)


def test_recorded_into_a_graph(capi):
    """The stated use of the entry point: {reset, decode on the fixed scratch}
    recorded into a HIP graph; every replay, with eager calls of the same entry
    point and synchronizations in between, leaves what the workspace entry
    point leaves."""
    handle = capi.lib()
    batch, qh, kh, d, capacity = 5, 12, 2, 128, 4096
    p = capi.attention_params(qh, kh, d, 32, capacity=capacity)
    lengths = [700, 4096, 33, 1500, 2049]
    positions = [L - 1 for L in lengths]
    caches, q_gate, k, v, qw, kw = make_case(capi, 31, batch, qh, kh, d, capacity, lengths)
    want = capi.gqa_decode(p, q_gate, k, v, qw, kw, caches(), positions=positions, advance=False)
    fixed = caches()
    out = torch.empty_like(want)

    def step():
        assert handle.pluto_hip_gqa_decode_static_reset(capi.current_stream()) == 0
        capi.gqa_decode_static(p, q_gate, k, v, qw, kw, fixed, positions, out)

    step()
    torch.cuda.synchronize()
    assert torch.equal(out, want)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        step()
    for replay in range(4):
        out.zero_()
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out, want), "replay %d" % replay
        step()   # eager work on the same scratch between the replays
        torch.cuda.synchronize()
        assert torch.equal(out, want)


def test_rejects_what_does_not_fit(capi):
    handle = capi.lib()
    batch, qh, kh, d, capacity = 64, 24, 4, 128, 32768
    p = capi.attention_params(qh, kh, d, 32, capacity=capacity)
    positions = [capacity - 1] * batch
    pos = (ctypes.c_int * batch)(*positions)
    needed = handle.pluto_hip_gqa_decode_workspace_bytes(ctypes.byref(p), batch, pos, 512)
    assert needed > handle.pluto_hip_gqa_decode_static_bytes()
    # one small cache stands in for all of them: the call must fail on its size
    # before it looks at any row
    cache = capi.KvCache(64, kh, d)
    q_gate = torch.zeros((batch, qh, 2, d), dtype=torch.bfloat16, device="cuda")
    k = torch.zeros((batch, kh, d), dtype=torch.bfloat16, device="cuda")
    out = torch.full((batch, qh, d), 7.0, dtype=torch.bfloat16, device="cuda")
    w = torch.ones(d, device="cuda")
    with pytest.raises(capi.PlutoHipError) as info:
        capi.gqa_decode_static(p, q_gate, k, k, w, w, [cache] * batch, positions, out)
    assert info.value.code == capi.ELIMIT
    assert b"fixed scratch" in handle.pluto_hip_error_string(capi.ELIMIT)
    torch.cuda.synchronize()
    assert (out == 7.0).all()
