"""The training step and the decode step replayed from a HIP graph: every
replay, with eager work of the same library and synchronizations in between,
must leave bit for bit what the eager call leaves (the kernels are bitwise
repeatable and the entry points launch nothing but kernels)."""
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


def replay_and_compare(graph, outputs, expected, eager):
    for replay in range(4):
        for t in outputs:
            t.zero_()
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        for got, want in zip(outputs, expected):
            assert torch.equal(got, want), "replay %d" % replay
        eager()   # the program's own eager work between replays
        torch.cuda.synchronize()


def test_training_step_replays_bit_equal(capi):
    B, T, H, D = 2, 512, 4, 64
    E = H * D
    gen = torch.Generator(device="cuda").manual_seed(7)
    qkv = torch.randn((B * T, 3 * E), generator=gen, device="cuda").to(torch.bfloat16)
    d_out = torch.randn((B * T, E), generator=gen, device="cuda")
    workspace = capi.mha_backward_workspace(qkv, T, H)
    d_qkv = torch.empty((B * T, 3 * E), dtype=torch.float32, device="cuda")
    fwd = capi.mha_forward(qkv, T, H)

    def step():
        capi.mha_forward(qkv, T, H, into=fwd)
        capi.mha_backward(qkv, fwd[0], d_out, fwd[1], fwd[2], T, H, workspace, d_qkv)

    step()
    torch.cuda.synchronize()
    assert capi.last_path() == capi.PATH_FLASH
    outputs = list(fwd) + [d_qkv]
    expected = [t.clone() for t in outputs]
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        step()
    replay_and_compare(graph, outputs, expected, step)


def test_decode_step_replays_bit_equal(capi):
    batch, qh, kh, d, capacity = 5, 12, 2, 128, 4096
    p = capi.attention_params(qh, kh, d, 32, capacity=capacity)
    gen = torch.Generator(device="cuda").manual_seed(8)
    bf = torch.bfloat16
    lengths = [700, 4096, 33, 1500, 2049]
    caches = []
    for L in lengths:
        c = capi.KvCache(capacity, kh, d)
        c.keys[:, :L] = torch.randn((kh, L, d), generator=gen, device="cuda").to(bf)
        c.values[:, :L] = torch.randn((kh, L, d), generator=gen, device="cuda").to(bf)
        caches.append(c)
    positions = [L - 1 for L in lengths]
    q_gate = torch.randn((batch, qh, 2, d), generator=gen, device="cuda").to(bf)
    k = torch.randn((batch, kh, d), generator=gen, device="cuda").to(bf)
    v = torch.randn((batch, kh, d), generator=gen, device="cuda").to(bf)
    qw = torch.rand(d, generator=gen, device="cuda")
    kw = torch.rand(d, generator=gen, device="cuda")
    workspace = capi.gqa_decode_workspace(p, positions, 0)
    out = torch.empty((batch, qh, d), dtype=bf, device="cuda")

    def step():
        capi.gqa_decode(p, q_gate, k, v, qw, kw, caches, positions=positions, workspace=workspace,
                        out=out, advance=False)

    step()
    torch.cuda.synchronize()
    assert capi.last_path() == capi.PATH_SPLIT_K
    expected = [out.clone()]
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        step()
    replay_and_compare(graph, [out], expected, step)
