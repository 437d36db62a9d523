"""Pins the CPU oracle of the FullyConnectedLayer dense path
(fully_connected.cc:97-247): operand rounding against numpy's own float16 and
against the bf16 rule, the three products against float64 matrix products of
the rounded operands (a library routine), closed forms, and torch float64
autograd for the gradients' structure."""
import numpy as np
import pytest


def test_half_rounding_is_ieee_binary16(oracle):
    rng = np.random.default_rng(0)
    x = np.concatenate([rng.standard_normal(2000).astype(np.float32) * s
                        for s in (1e-7, 1e-5, 1e-3, 1.0, 300.0, 7e4)] +
                       [np.array([0.0, -0.0, 65504.0, 65519.9, 65520.0, 1e9, 2.0 ** -24,
                                  2.0 ** -25, 1.5 * 2.0 ** -24, 6.1e-5, np.inf, -np.inf],
                                 np.float32)])
    want = x.astype(np.float16).astype(np.float32)
    np.testing.assert_array_equal(oracle.half_round(x), want)


@pytest.mark.parametrize("dtype_name", ["bf16", "f32"])
@pytest.mark.parametrize("rows,n_in,n_out", [(1, 1, 1), (5, 7, 3), (70, 65, 129), (33, 128, 64)])
def test_products_match_float64_library(oracle, dtype_name, rows, n_in, n_out):
    rng = np.random.default_rng(rows * 1000 + n_in)
    dtype = oracle.BF16 if dtype_name == "bf16" else oracle.F32
    R = oracle.bf16_round if dtype_name == "bf16" else (
        lambda v: np.asarray(v, np.float32).astype(np.float16).astype(np.float32))
    x = rng.standard_normal((rows, n_in)).astype(np.float32)
    if dtype_name == "bf16":
        x = oracle.bf16_round(x)
    w = (0.3 * rng.standard_normal((n_in, n_out))).astype(np.float32)
    b = rng.standard_normal(n_out).astype(np.float32)
    dy = rng.standard_normal((rows, n_out)).astype(np.float32)
    y = oracle.dense_forward(dtype, x, w, b)
    want = R(x).astype(np.float64) @ R(w).astype(np.float64) + b
    want = oracle.bf16_round(want.astype(np.float32)) if dtype_name == "bf16" else want
    np.testing.assert_allclose(y, want, rtol=1e-6, atol=1e-6)
    dx, dw, db = oracle.dense_backward(dtype, x, w, dy)
    np.testing.assert_allclose(dx, R(dy).astype(np.float64) @ R(w).astype(np.float64).T,
                               rtol=1e-6, atol=1e-6)
    np.testing.assert_allclose(dw, R(x).astype(np.float64).T @ R(dy).astype(np.float64),
                               rtol=1e-6, atol=1e-6)
    np.testing.assert_allclose(db, dy.astype(np.float64).sum(0), rtol=1e-6, atol=1e-6)


def test_identity_matrix_and_bias_closed_form(oracle):
    # InitializeIdentity (fully_connected.h:53-55): scaled identity on the
    # available diagonal, zero bias -> y = scale * x on the diagonal part
    x = np.arange(12, dtype=np.float32).reshape(3, 4) - 5
    w = np.zeros((4, 6), np.float32)
    w[np.arange(4), np.arange(4)] = 2.0
    y = oracle.dense_forward(oracle.F32, x, w, np.full(6, 0.5, np.float32))
    np.testing.assert_array_equal(y[:, :4], 2 * x + 0.5)
    np.testing.assert_array_equal(y[:, 4:], 0.5)


def test_gradients_are_those_of_the_forward(oracle):
    torch = pytest.importorskip("torch")
    rng = np.random.default_rng(3)
    # values exactly representable in half and bf16: rounding is the identity
    x = rng.integers(-8, 9, (9, 5)).astype(np.float32) / 4
    w = rng.integers(-8, 9, (5, 7)).astype(np.float32) / 8
    dy = rng.integers(-8, 9, (9, 7)).astype(np.float32) / 2
    tx = torch.tensor(x, dtype=torch.float64, requires_grad=True)
    tw = torch.tensor(w, dtype=torch.float64, requires_grad=True)
    tb = torch.zeros(7, dtype=torch.float64, requires_grad=True)
    ((tx @ tw + tb) * torch.tensor(dy, dtype=torch.float64)).sum().backward()
    for dtype in (oracle.F32, oracle.BF16):
        dx, dw, db = oracle.dense_backward(dtype, x, w, dy)
        np.testing.assert_allclose(dx, tx.grad.numpy(), rtol=0, atol=1e-6)
        np.testing.assert_allclose(dw, tw.grad.numpy(), rtol=0, atol=1e-6)
        np.testing.assert_allclose(db, tb.grad.numpy(), rtol=0, atol=1e-6)


def test_rejects_bad_arguments(oracle):
    with pytest.raises(ValueError):
        oracle.dense_forward(7, np.zeros((1, 1)), np.zeros((1, 1)), np.zeros(1))
