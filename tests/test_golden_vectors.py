"""The reference tests' known-answer vectors (tests/golden/) against the CPU
oracle (CPU suite) and against the HIP library through the C ABI (GPU suite)."""
import json
import os

import numpy as np
import pytest

GOLDEN = os.path.join(os.path.dirname(__file__), "golden", "reference_known_answers.json")


@pytest.fixture(scope="module")
def golden():
    with open(GOLDEN) as handle:
        return json.load(handle)


def mha_inputs(case):
    E = case["embedding_dim"]
    x = np.zeros((case["rows"], 3 * E), np.float32)
    for row, column, value in case["nonzero_qkv"]:
        x[row, column] = value
    d_out = np.zeros((case["rows"], E), np.float32)
    for row, column, value in case["d_out_nonzero"]:
        d_out[row, column] = value
    return x, d_out


def test_oracle_cached_attention_known_answers(oracle, golden):
    case = golden["cached_attention_two_steps"]
    ref = oracle.CachedAttention(oracle.attention_params(**case["params"]))
    f = lambda name: np.asarray(case[name], np.float32)
    for step in case["steps"]:
        out, probs = ref.step(f("q_gate"), f("k"), np.asarray(step["v"], np.float32), f("q_norm"),
                              f("k_norm"), True)
        np.testing.assert_array_equal(out.ravel(), step["output"])
        np.testing.assert_array_equal(probs, np.asarray(step["probabilities"], np.float32))
    with pytest.raises(OverflowError):
        ref.step(f("q_gate"), f("k"), f("k"), f("q_norm"), f("k_norm"))
    assert ref.position == 2


def test_oracle_uniform_rows(oracle, golden):
    case = golden["uniform_rows"]
    ref = oracle.CachedAttention(oracle.attention_params(**case["params"]))
    zero = np.zeros(4, np.float32)
    for t in range(case["steps"]):
        _, probs = ref.step(np.zeros(16, np.float32), np.ones(4, np.float32),
                            np.full(4, t, np.float32), zero, zero, True)
        np.testing.assert_allclose(probs, 1.0 / (t + 1), atol=1e-7)


def test_oracle_mha_closed_form(oracle, golden):
    case = golden["mha_closed_form"]
    x, d_out = mha_inputs(case)
    out, _, _ = oracle.mha_fwd(x, case["context_length"], case["num_heads"])
    for row, column, value in case["expected_out"]:
        assert out[row, column] == pytest.approx(value, abs=1e-5)
    grad = oracle.mha_bwd(x, out, d_out, case["context_length"], case["num_heads"])
    for row, column, value in case["expected_d_qkv"]:
        assert grad[row, column] == pytest.approx(value, abs=1e-6)


@pytest.mark.gpu
def test_library_cached_attention_known_answers(golden):
    torch = pytest.importorskip("torch")
    from pluto_amd import capi
    capi.lib()
    case = golden["cached_attention_two_steps"]
    p = capi.attention_params(**case["params"])
    dev = lambda values, shape: torch.tensor(values, dtype=torch.float32, device="cuda").reshape(shape)
    kv = case["params"]["key_value_heads"]
    cache = capi.KvCache(case["params"]["capacity"], kv, case["params"]["head_dim"])
    q_gate = dev(case["q_gate"], (1, 2, 2, 4))
    k = dev(case["k"], (1, 1, 4))
    norm = dev(case["q_norm"], (4,))
    for step in case["steps"]:
        out = capi.gqa_decode(p, q_gate, k, dev(step["v"], (1, 1, 4)), norm, norm, [cache])
        torch.cuda.synchronize()
        np.testing.assert_array_equal(out.cpu().numpy().ravel(), step["output"])


@pytest.mark.gpu
def test_library_mha_closed_form(golden):
    torch = pytest.importorskip("torch")
    from pluto_amd import capi
    capi.lib()
    case = golden["mha_closed_form"]
    x, d_out = mha_inputs(case)
    T, H = case["context_length"], case["num_heads"]
    qkv = torch.from_numpy(x).cuda()
    out, maxima, normalizers = capi.mha_forward(qkv, T, H)
    grad = capi.mha_backward(qkv, out, torch.from_numpy(d_out).cuda(), maxima, normalizers, T, H)
    torch.cuda.synchronize()
    out, grad = out.cpu().numpy(), grad.cpu().numpy()
    for row, column, value in case["expected_out"]:
        assert out[row, column] == pytest.approx(value, abs=1e-5)
    for row, column, value in case["expected_d_qkv"]:
        assert grad[row, column] == pytest.approx(value, abs=1e-6)
