"""GPU parity of the gated delta-net scan (chunked matrix-core path and the
token-by-token recurrence) with the CPU oracle, through the C ABI.  Cases follow
sequence_delta_net_test.cc and cached_attention_ops_test.cc of the reference."""
import math
import os

import numpy as np
import pytest

from tests.util import assert_close, assert_close_bf16

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


def make_inputs(oracle, rng, B, T, kh, vh, kd, vd, normalized):
    q = rng.standard_normal((B, T, kh, kd)).astype(np.float32)
    k = rng.standard_normal((B, T, kh, kd)).astype(np.float32)
    if normalized:  # L2-normalised per head, as the scan configuration states
        q /= np.linalg.norm(q, axis=-1, keepdims=True)
        k /= np.linalg.norm(k, axis=-1, keepdims=True)
    q, k = oracle.bf16_round(q), oracle.bf16_round(k)
    v = oracle.bf16_round(rng.standard_normal((B, T, vh, vd)).astype(np.float32))
    beta = (1 / (1 + np.exp(-rng.standard_normal((B, T, vh))))).astype(np.float32)
    g = (-np.log1p(np.exp(rng.standard_normal((B, T, vh))))).astype(np.float32)
    return q, k, v, g, beta


def run_device(capi, fn, p, q, k, v, g, beta, state0, normalize, scale):
    bf = torch.bfloat16
    state = dev(state0.astype(np.float32))
    out = fn(p, dev(q, bf), dev(k, bf), dev(v, bf), dev(g), dev(beta), state,
             normalize_qk=normalize, q_scale=scale)
    torch.cuda.synchronize()
    return out.float().cpu().numpy(), state.cpu().numpy()


def run_oracle(oracle, po, q, k, v, g, beta, state0, normalize, scale, heads=None):
    outs, states = [], []
    for b in range(q.shape[0]):
        core, state = oracle.gdn_scan(po, q[b], k[b], v[b], g[b], beta[b], normalize, scale,
                                      state0[b], heads)
        outs.append(core)
        states.append(state)
    return np.stack(outs), np.stack(states)


@pytest.mark.parametrize("kh,vh,kd,vd", [(1, 2, 3, 5), (2, 4, 5, 35), (2, 6, 128, 128), (1, 1, 64, 256)])
@pytest.mark.parametrize("normalize", [False, True])
def test_recurrence_matches_oracle(capi, oracle, kh, vh, kd, vd, normalize):
    B, T = 2, 37
    p = capi.delta_params(kh, vh, kd, vd)
    po = oracle.delta_params(kh, vh, kd, vd)
    rng = np.random.default_rng(kd + vd)
    q, k, v, g, beta = make_inputs(oracle, rng, B, T, kh, vh, kd, vd, not normalize)
    state0 = 0.1 * rng.standard_normal((B, vh, kd, vd))
    scale = 1 / math.sqrt(kd)
    got, got_state = run_device(capi, capi.gdn_recurrence, p, q, k, v, g, beta, state0, normalize, scale)
    want, want_state = run_oracle(oracle, po, q, k, v, g, beta, state0, normalize, scale)
    # fp32 state and sums, output rounded to bf16: sequence_delta_net_test.cc:253-255
    assert np.all(np.abs(got - want) <= 1.5e-4 + 1.5e-2 * np.abs(want))
    assert_close(got_state, want_state, 1e-4, "recurrence state")


@pytest.mark.parametrize("T", [64, 65, 200, 1024])
@pytest.mark.parametrize("normalize", [False, True])
def test_chunked_scan_matches_oracle(capi, oracle, T, normalize):
    B, kh, vh, kd, vd = 2, 2, 4, 128, 128
    p = capi.delta_params(kh, vh, kd, vd)
    po = oracle.delta_params(kh, vh, kd, vd)
    rng = np.random.default_rng(T)
    q, k, v, g, beta = make_inputs(oracle, rng, B, T, kh, vh, kd, vd, not normalize)
    state0 = 0.1 * rng.standard_normal((B, vh, kd, vd))
    scale = 1 / math.sqrt(kd)
    got, got_state = run_device(capi, capi.gdn_scan, p, q, k, v, g, beta, state0, normalize, scale)
    want, want_state = run_oracle(oracle, po, q, k, v, g, beta, state0, normalize, scale)
    assert_close_bf16(got, want, "chunked scan T%d out" % T)
    assert_close_bf16(got_state, want_state, "chunked scan T%d state" % T)


def test_textbook_special_cases(capi, oracle):
    # beta = 0: pure decay of the initial state; g = 0, beta = 1 with orthonormal
    # keys: the state becomes sum k v^T and reading with a key returns its value.
    kd = vd = 128
    T = 128
    p = capi.delta_params(1, 1, kd, vd)
    rng = np.random.default_rng(0)
    basis, _ = np.linalg.qr(rng.standard_normal((kd, kd)))
    k = oracle.bf16_round(basis.T.reshape(1, T, 1, kd).astype(np.float32))
    v = oracle.bf16_round(rng.standard_normal((1, T, 1, vd)).astype(np.float32))
    zeros = np.zeros((1, T, 1), np.float32)
    state0 = np.zeros((1, 1, kd, vd))
    got, state = run_device(capi, capi.gdn_scan, p, k, k, v, zeros, zeros + 1, state0, False, 1.0)
    # bf16 keys are orthonormal only to 2^-9: compare with that slack
    np.testing.assert_allclose(got[0, :, 0], v[0, :, 0], atol=0.05)
    np.testing.assert_allclose(state[0, 0], k[0, :, 0].astype(np.float64).T @ v[0, :, 0], atol=0.05)
    s0 = rng.standard_normal((1, 1, kd, vd))
    g = -rng.random((1, T, 1)).astype(np.float32)
    got, state = run_device(capi, capi.gdn_scan, p, k, k, v, g, zeros, s0, False, 1.0)
    total = math.exp(float(g.astype(np.float64).sum()))
    np.testing.assert_allclose(state[0, 0], total * s0[0, 0], rtol=2e-2, atol=1e-30)


def test_state_carries_across_calls(capi, oracle):
    B, kh, vh, kd, vd = 1, 1, 2, 128, 128
    p = capi.delta_params(kh, vh, kd, vd)
    rng = np.random.default_rng(6)
    q, k, v, g, beta = make_inputs(oracle, rng, B, 320, kh, vh, kd, vd, True)
    state0 = np.zeros((B, vh, kd, vd))
    whole, whole_state = run_device(capi, capi.gdn_scan, p, q, k, v, g, beta, state0, False, 0.1)
    first, mid = run_device(capi, capi.gdn_scan, p, q[:, :128], k[:, :128], v[:, :128], g[:, :128],
                            beta[:, :128], state0, False, 0.1)
    second, end = run_device(capi, capi.gdn_scan, p, q[:, 128:], k[:, 128:], v[:, 128:], g[:, 128:],
                             beta[:, 128:], mid, False, 0.1)
    # the split falls on a chunk boundary: identical arithmetic, identical bits
    np.testing.assert_array_equal(np.concatenate([first, second], 1), whole)
    np.testing.assert_array_equal(end, whole_state)


def test_config5_chunked_scan(capi, oracle):
    # B=2, T=16384, 16 heads, d_k=d_v=128, chunk 64, bf16 inputs, fp32 state;
    # q,k ~ N(0,1) L2-normalised, beta = sigmoid(N(0,1)), g = -softplus(N(0,1)), seed 4.
    B, T, H, kd, vd = 2, 16384, 16, 128, 128
    p = capi.delta_params(H, H, kd, vd)
    po = oracle.delta_params(H, H, kd, vd)
    rng = np.random.default_rng(4)
    q, k, v, g, beta = make_inputs(oracle, rng, B, T, H, H, kd, vd, True)
    state0 = np.zeros((B, H, kd, vd))
    scale = 1 / math.sqrt(kd)
    bf = torch.bfloat16
    dq, dk, dv, dg, db = dev(q, bf), dev(k, bf), dev(v, bf), dev(g), dev(beta)
    state = dev(state0.astype(np.float32))
    out = capi.gdn_scan(p, dq, dk, dv, dg, db, state, q_scale=scale, chunk=64)
    assert capi.last_path() == capi.PATH_CHUNKED
    torch.cuda.synchronize()
    got, got_state = out.float().cpu().numpy(), state.cpu().numpy()
    # CPU recurrence on every one of the 32 (sequence, head) chains (they are
    # independent; the oracle's C code runs outside the interpreter lock)
    import concurrent.futures

    def chain(index):
        b, h = divmod(index, H)
        core, want_state = oracle.gdn_scan(po, q[b], k[b], v[b], g[b], beta[b], False, scale,
                                           state0[b], (h, h + 1))
        return core[:, h], want_state[h]

    with concurrent.futures.ThreadPoolExecutor(max_workers=16) as pool:
        chains = list(pool.map(chain, range(B * H)))
    want = np.stack([c[0] for c in chains]).reshape(B, H, T, vd).transpose(0, 2, 1, 3)
    want_state = np.stack([c[1] for c in chains]).reshape(B, H, kd, vd)
    assert_close_bf16(got, want, "config 5 out, all 32 chains")
    assert_close_bf16(got_state, want_state, "config 5 state, all 32 chains")
    # every chain: against the token-by-token kernel
    state2 = dev(state0.astype(np.float32))
    out2 = capi.gdn_recurrence(p, dq, dk, dv, dg, db, state2, q_scale=scale)
    torch.cuda.synchronize()
    assert_close_bf16(got, out2.float().cpu().numpy(), "config 5 vs recurrence kernel out")
    assert_close_bf16(got_state, state2.cpu().numpy(), "config 5 vs recurrence kernel state")
    # bitwise repeatable
    state3 = dev(state0.astype(np.float32))
    out3 = capi.gdn_scan(p, dq, dk, dv, dg, db, state3, q_scale=scale, chunk=64)
    assert torch.equal(out, out3) and torch.equal(state, state3)


def test_rejects_bad_arguments(capi):
    # cached_attention_ops_test.cc:622-636
    t = torch.zeros(64, device="cuda")
    for kw in (dict(key_head_dim=129), dict(key_heads=0), dict(key_heads=2, value_heads=3),
               dict(value_head_dim=257), dict(conv_kernel_dim=33), dict(rms_norm_epsilon=0.0)):
        p = capi.delta_params(**{**dict(key_heads=1, value_heads=1, key_head_dim=4, value_head_dim=4), **kw})
        code = capi.lib().pluto_hip_gdn_recurrence(capi.current_stream(), p, 1, 1, capi.ptr(t),
                                                   capi.ptr(t), capi.ptr(t), capi.ptr(t), capi.ptr(t),
                                                   0, 1.0, capi.ptr(t), capi.ptr(t), capi.F32)
        assert code == capi.EINVAL
    p = capi.delta_params(1, 1, 4, 4)
    code = capi.lib().pluto_hip_gdn_recurrence(capi.current_stream(), p, 1, 1, None, None, None,
                                               None, None, 0, 1.0, None, None, capi.F32)
    assert code == capi.EINVAL


def values(count, phase, scale=1.0):
    i = np.arange(count, dtype=np.float32)
    return (np.float32(scale) * np.sin(np.float32(phase) + i * np.float32(0.29))).astype(np.float32)


def layer_weights(kh, vh, kd, vd, kernel):
    channels = 2 * kh * kd + vh * vd
    return (values(channels * kernel, 0.73, 0.6).reshape(channels, kernel), values(vh, 0.18, 0.5),
            values(vh, -0.7, 0.3), values(vd, 0.5, 0.6))


@pytest.mark.parametrize("round_flag", [False, True])
@pytest.mark.parametrize("dim", [5, 128])
def test_single_token_step_matches_scalar_specification(capi, oracle, dim, round_flag):
    # cached_attention_ops_test.cc:400-470
    kh, vh, kd, vd = 2, 6, dim, (7 if dim == 5 else 128)
    p = capi.delta_params(kh, vh, kd, vd, round_to_bfloat16=round_flag)
    po = oracle.delta_params(kh, vh, kd, vd, round_to_bfloat16=round_flag)
    channels = 2 * kh * kd + vh * vd
    w, a_log, dt, norm = layer_weights(kh, vh, kd, vd, 4)
    dw, dal, ddt, dn = dev(w), dev(a_log), dev(dt), dev(norm)
    state = capi.DeltaNetStep(p)
    reference = oracle.DeltaNetStep(po)
    first = None
    for step in range(7):
        t = 0 if step == 6 else step
        if step == 6:
            state.reset()
        qkv = values(channels, 0.3 + t * 0.71)
        z = values(vh * vd, -0.6 + t * 0.27)
        a = values(vh, 0.1 + t * 0.1)
        b = values(vh, -0.7 + t * 0.3)
        a[0], a[1] = 100.0, -100.0   # softplus at both extremes
        got = state.step(dev(qkv), dev(z), dev(a), dev(b), dw, dal, ddt, dn).cpu().numpy()
        assert np.all(np.isfinite(got))
        if step < 6:
            want = reference.step(qkv, z, a, b, w, a_log, dt, norm)
            bound = (2e-4 + 8e-3 * np.abs(want)) if round_flag else (3e-5 + 1e-4 * np.abs(want))
            loose = 2e-4 + 1.6e-2 * np.abs(want)
            diff = np.abs(got - want)
            assert np.all(diff <= (loose if round_flag else bound)), diff.max()
            assert np.mean(diff > bound) <= 5e-3
        if step == 0:
            first = got.copy()
        if step == 6:
            np.testing.assert_array_equal(got, first)   # Reset replays bit-equal


@pytest.mark.parametrize("round_flag", [False, True])
@pytest.mark.parametrize("dim", [5, 128])
def test_batched_step_is_the_single_step_of_every_sequence(capi, oracle, dim, round_flag):
    """pluto_hip_gdn_step_batch: the decoder step of Model::Step
    (qwen/model.cc:405-428) lifted to several sequences with their own
    DeltaNetState.  Each row must be bit for bit what the single-sequence entry
    point gives, over several tokens (so states carry over), and match the
    scalar specification."""
    kh, vh, kd, vd = 2, 6, dim, (7 if dim == 5 else 128)
    batch, steps = 5, 4
    p = capi.delta_params(kh, vh, kd, vd, round_to_bfloat16=round_flag)
    po = oracle.delta_params(kh, vh, kd, vd, round_to_bfloat16=round_flag)
    channels = 2 * kh * kd + vh * vd
    w, a_log, dt, norm = layer_weights(kh, vh, kd, vd, 4)
    dw, dal, ddt, dn = dev(w), dev(a_log), dev(dt), dev(norm)
    together = capi.DeltaNetStep(p, batch=batch)
    alone = [capi.DeltaNetStep(p) for _ in range(batch)]
    reference = oracle.DeltaNetStep(po)   # sequence 3
    rng = np.random.default_rng(dim + round_flag)
    for step in range(steps):
        qkv = rng.standard_normal((batch, channels)).astype(np.float32)
        z = rng.standard_normal((batch, vh * vd)).astype(np.float32)
        a = rng.standard_normal((batch, vh)).astype(np.float32)
        b = rng.standard_normal((batch, vh)).astype(np.float32)
        got = together.step(dev(qkv), dev(z), dev(a), dev(b), dw, dal, ddt, dn).cpu().numpy()
        for s in range(batch):
            one = alone[s].step(dev(qkv[s]), dev(z[s]), dev(a[s]), dev(b[s]), dw, dal, ddt, dn)
            np.testing.assert_array_equal(got[s], one.cpu().numpy())
        want = reference.step(qkv[3], z[3], a[3], b[3], w, a_log, dt, norm)
        loose = 2e-4 + 1.6e-2 * np.abs(want) if round_flag else 3e-5 + 1e-4 * np.abs(want)
        assert np.all(np.abs(got[3] - want) <= loose)
    for s in range(batch):
        np.testing.assert_array_equal(together.state[s].cpu().numpy(),
                                      alone[s].state.cpu().numpy())
        np.testing.assert_array_equal(together.conv[s].cpu().numpy(), alone[s].conv.cpu().numpy())


def test_batched_step_rejects_bad_arguments(capi):
    import ctypes
    p = capi.delta_params(2, 4, 16, 16)
    lib = capi.lib()
    assert lib.pluto_hip_gdn_step_batch_workspace_bytes(ctypes.byref(p), 0) == 0
    size = lib.pluto_hip_gdn_step_batch_workspace_bytes(ctypes.byref(p), 3)
    assert size >= 3 * lib.pluto_hip_gdn_step_workspace_bytes(ctypes.byref(p)) // 2
    x = torch.zeros(4096, device="cuda")
    px = capi.ptr(x)
    args = [px] * 11
    stream, f32 = capi.current_stream(), capi.F32
    assert lib.pluto_hip_gdn_step_batch(stream, ctypes.byref(p), 0, f32, *args, px, size) != 0
    assert lib.pluto_hip_gdn_step_batch(stream, ctypes.byref(p), 3, f32, *args, px, 16) != 0
    assert lib.pluto_hip_gdn_step_batch(stream, ctypes.byref(p), 3, f32, None, *args[1:], px,
                                        size) != 0
    assert lib.pluto_hip_gdn_step_batch(stream, ctypes.byref(p), 3, 77, *args, px, size) != 0


@pytest.mark.parametrize("round_flag", [False, True])
@pytest.mark.parametrize("dim", [5, 128])
def test_bf16_step_is_the_fp32_step_between_casts(capi, dim, round_flag):
    """io_dtype = bf16: what DeltaNetLayer::fwd_impl (delta_net.cc:70-102) computes
    with four ToFloat launches before the FP32 step and one ToBFloat16 after it,
    bit for bit, over several tokens (both states carry over) and five sequences."""
    kh, vh, kd, vd = 2, 6, dim, (7 if dim == 5 else 128)
    batch, steps = 5, 4
    p = capi.delta_params(kh, vh, kd, vd, round_to_bfloat16=round_flag)
    channels = 2 * kh * kd + vh * vd
    w, a_log, dt, norm = layer_weights(kh, vh, kd, vd, 4)
    dw, dal, ddt, dn = dev(w), dev(a_log), dev(dt), dev(norm)
    direct = capi.DeltaNetStep(p, batch=batch)
    through_casts = capi.DeltaNetStep(p, batch=batch)
    rng = np.random.default_rng(10 * dim + round_flag)
    bf = torch.bfloat16
    for step in range(steps):
        qkv, z, a, b = (dev(rng.standard_normal((batch, n)).astype(np.float32)).to(bf)
                        for n in (channels, vh * vd, vh, vh))
        got = direct.step(qkv, z, a, b, dw, dal, ddt, dn)
        assert got.dtype == bf
        want = through_casts.step(qkv.float(), z.float(), a.float(), b.float(), dw, dal, ddt, dn)
        assert torch.equal(got, want.to(bf)), step
    assert torch.equal(direct.state, through_casts.state)
    assert torch.equal(direct.conv, through_casts.conv)


@pytest.mark.parametrize("kh,vh,kd,vd,T,round_flag", [(2, 6, 5, 7, 9, False), (2, 6, 5, 7, 9, True),
                                                     (2, 4, 128, 128, 7, True), (2, 4, 128, 128, 200, True),
                                                     (1, 2, 128, 128, 70, False)])
def test_layer_forward_matches_scalar_specification(capi, oracle, kh, vh, kd, vd, T, round_flag):
    # sequence_delta_net_test.cc:213-255
    B = 2
    p = capi.delta_params(kh, vh, kd, vd, round_to_bfloat16=round_flag)
    po = oracle.delta_params(kh, vh, kd, vd, round_to_bfloat16=round_flag)
    channels = 2 * kh * kd + vh * vd
    w, a_log, dt, norm = layer_weights(kh, vh, kd, vd, 4)
    rng = np.random.default_rng(T + kd)
    qkv = oracle.bf16_round(rng.standard_normal((B, T, channels)).astype(np.float32))
    z = oracle.bf16_round(rng.standard_normal((B, T, vh * vd)).astype(np.float32))
    a = oracle.bf16_round(rng.standard_normal((B, T, vh)).astype(np.float32))
    b = oracle.bf16_round(rng.standard_normal((B, T, vh)).astype(np.float32))
    bf = torch.bfloat16
    state = torch.zeros((B, vh, kd, vd), device="cuda")
    out = capi.gdn_layer_forward(p, dev(qkv, bf), dev(z, bf), dev(a, bf), dev(b, bf), dev(w),
                                 dev(a_log), dev(dt), dev(norm), state)
    torch.cuda.synchronize()
    got = out.float().cpu().numpy()
    for i in range(B):
        want = oracle.gdn_sequence(po, qkv[i], z[i], a[i], b[i], w, a_log, dt, norm)
        if kd == 128 and round_flag:
            assert_close_bf16(got[i], want["out"], "delta-net layer T%d" % T)
            assert_close_bf16(state[i].cpu().numpy(), want["state"], "delta-net layer state")
        else:
            # sequence_delta_net_test.cc:253-255
            assert np.all(np.abs(got[i] - want["out"]) <= 1.5e-4 + 1.5e-2 * np.abs(want["out"]))
            assert_close(state[i].cpu().numpy(), want["state"], 2e-3, "delta-net layer state")
