"""Pins the oracle's whole-sequence GQA backward (no GPU).

The reference checks its backward against central finite differences of a
double-precision forward in which every bf16 rounding is replaced by the
rounding error recorded at the unperturbed point (qwen_attention_test.cc:
22-99, 230-300): casts then have derivative one, and every other operand is the
rounded forward value.  The same check is applied to the oracle here, with a
forward written independently in numpy; in addition the unrounded case is
compared with torch autograd of a float64 formulation."""
import math

import numpy as np
import pytest
import torch

from oracle import pyoracle as po


def values(n, phase):
    return po.bf16_round(0.8 * np.sin(phase + 0.29 * np.arange(n))).astype(np.float64)


class FrozenRounding:
    """round(x) = x + (bf16(x0) - x0) with x0 the value seen at recording time."""

    def __init__(self, enabled):
        self.enabled, self.errors, self.recording, self.at = enabled, [], True, 0

    def replay(self):
        self.recording, self.at = False, 0

    def __call__(self, x):
        if not self.enabled:
            return x
        if self.recording:
            self.errors.append(float(po.bf16_round(np.float32(x))) - x)
            return x + self.errors[-1]
        error = self.errors[self.at]
        self.at += 1
        return x + error


def forward(p, T, qg, k, v, qw, kw, rnd):
    d, qh, kh, rot = p.head_dim, p.query_heads, p.key_value_heads, p.rotary_dim

    def prepare(x, w, heads, stride):
        out = np.zeros((T, heads, d))
        for row in range(T):
            for h in range(heads):
                vec = x[(row * heads + h) * stride:(row * heads + h) * stride + d]
                inverse = 1.0 / math.sqrt(float(np.dot(vec, vec)) / d + p.rms_norm_epsilon)
                r = [rnd(vec[c] * inverse * (1 + w[c])) for c in range(d)]
                for c in range(rot // 2):
                    partner = c + rot // 2
                    angle = row * p.rope_theta ** (-2.0 * c / rot)
                    first, second = r[c], r[partner]
                    cosine, sine = rnd(math.cos(angle)), rnd(math.sin(angle))
                    fc, ss = rnd(first * cosine), rnd(second * sine)
                    sc, fs = rnd(second * cosine), rnd(first * sine)
                    r[c], r[partner] = rnd(fc - ss), rnd(sc + fs)
                out[row, h] = r
        return out

    query, key = prepare(qg, qw, qh, 2 * d), prepare(k, kw, kh, d)
    value = v.reshape(T, kh, d)
    out = np.zeros((T, qh, d))
    for row in range(T):
        for h in range(qh):
            kv = h // (qh // kh)
            scores = np.array([np.dot(query[row, h], key[t, kv]) / math.sqrt(d)
                               for t in range(row + 1)])
            prob = np.exp(scores - scores.max())
            prob /= prob.sum()
            for c in range(d):
                core = rnd(float(np.dot(prob, value[:row + 1, kv, c])))
                gate = rnd(1.0 / (1.0 + math.exp(-qg[((row * qh + h) * 2 + 1) * d + c])))
                out[row, h, c] = rnd(core * gate)
    return out


@pytest.mark.parametrize("use_rounding", [False, True])
@pytest.mark.parametrize("shape", [(3, 2, 1, 3, 2), (4, 4, 2, 6, 4)])
def test_backward_matches_finite_differences_of_frozen_rounding_forward(use_rounding, shape):
    T, qh, kh, d, rot = shape
    p = po.attention_params(query_heads=qh, key_value_heads=kh, head_dim=d, rotary_dim=rot,
                            capacity=T, round_to_bfloat16=use_rounding)
    inputs = [values(T * qh * 2 * d, .1), values(T * kh * d, 1.2), values(T * kh * d, 2.3),
              values(d, .2), values(d, .4)]
    upstream = values(T * qh * d, .7)
    got = po.gqa_sequence_backward(p, inputs[0].reshape(T, qh, 2, d), inputs[1].reshape(T, kh, d),
                                   inputs[2].reshape(T, kh, d), inputs[3], inputs[4],
                                   upstream.reshape(T, qh, d))
    actual = [got["dqg"].ravel(), got["dk"].ravel(), got["dv"].ravel(), got["dq_norm"],
              got["dk_norm"]]
    rnd = FrozenRounding(use_rounding)
    forward(p, T, *inputs, rnd)

    def loss():
        rnd.replay()
        return float(np.sum(forward(p, T, *inputs, rnd).ravel() * upstream))

    epsilon = 1e-5
    for which, array in enumerate(inputs):
        for i in range(array.size):
            original = array[i]
            array[i] = original + epsilon
            plus = loss()
            array[i] = original - epsilon
            minus = loss()
            array[i] = original
            assert abs(actual[which][i] - (plus - minus) / (2 * epsilon)) < 3e-5, (which, i)


def test_weight_gradients_accumulate_and_can_be_skipped():
    T, qh, kh, d, rot = 3, 2, 1, 4, 2
    p = po.attention_params(query_heads=qh, key_value_heads=kh, head_dim=d, rotary_dim=rot,
                            capacity=T, round_to_bfloat16=True)
    qg, k, v = values(T * qh * 2 * d, .1), values(T * kh * d, 1.2), values(T * kh * d, 2.3)
    args = (qg.reshape(T, qh, 2, d), k.reshape(T, kh, d), v.reshape(T, kh, d), values(d, .2),
            values(d, .4), values(T * qh * d, .7).reshape(T, qh, d))
    once = po.gqa_sequence_backward(p, *args)
    skipped = po.gqa_sequence_backward(p, *args, weight_grads=False)
    for name in ("dqg", "dk", "dv"):
        np.testing.assert_array_equal(once[name], skipped[name])
    assert np.abs(once["dq_norm"]).sum() > 0 and np.abs(once["dk_norm"]).sum() > 0
    assert not skipped["dq_norm"].any() and not skipped["dk_norm"].any()


def test_unrounded_backward_matches_float64_autograd():
    torch.manual_seed(5)
    T, qh, kh, d, rot = 9, 4, 2, 8, 4
    p = po.attention_params(query_heads=qh, key_value_heads=kh, head_dim=d, rotary_dim=rot,
                            capacity=T, round_to_bfloat16=False, rope_theta=1e4)
    qg = torch.randn(T, qh, 2, d).bfloat16().double().requires_grad_()
    k = torch.randn(T, kh, d).bfloat16().double().requires_grad_()
    v = torch.randn(T, kh, d).bfloat16().double().requires_grad_()
    qw = (0.1 * torch.randn(d)).float().double().requires_grad_()
    kw = (0.1 * torch.randn(d)).float().double().requires_grad_()
    dy = torch.randn(T, qh, d).float().double()

    def prepare(x, w):
        x = x * torch.rsqrt((x * x).mean(-1, keepdim=True) + p.rms_norm_epsilon) * (1 + w)
        position = torch.arange(T, dtype=torch.float64)[:, None]
        frequency = p.rope_theta ** (-2.0 * torch.arange(rot // 2, dtype=torch.float64) / rot)
        angle = (position * frequency)[:, None, :]
        first, second = x[..., :rot // 2], x[..., rot // 2:rot]
        return torch.cat([first * angle.cos() - second * angle.sin(),
                          second * angle.cos() + first * angle.sin(), x[..., rot:]], -1)

    q = prepare(qg[:, :, 0], qw)
    keys = prepare(k, kw).repeat_interleave(qh // kh, 1)
    vals = v.repeat_interleave(qh // kh, 1)
    scores = torch.einsum("rhc,thc->hrt", q, keys) / math.sqrt(d)
    scores = scores.masked_fill(torch.ones(T, T).triu(1).bool(), -math.inf)
    core = torch.einsum("hrt,thc->rhc", scores.softmax(-1), vals)
    out = core * torch.sigmoid(qg[:, :, 1])
    (out * dy).sum().backward()
    got = po.gqa_sequence_backward(p, qg.detach().numpy(), k.detach().numpy(), v.detach().numpy(),
                                   qw.detach().numpy(), kw.detach().numpy(), dy.numpy())
    for name, want in (("dqg", qg.grad), ("dk", k.grad), ("dv", v.grad), ("dq_norm", qw.grad),
                       ("dk_norm", kw.grad)):
        np.testing.assert_allclose(got[name], want.numpy(), rtol=1e-4, atol=2e-5, err_msg=name)
