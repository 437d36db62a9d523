"""Pins the oracle's gated delta-net layer backward (no GPU): central finite
differences of an independently written double-precision forward whose bf16
roundings are frozen at the unperturbed point (the construction the reference
uses for its own check, sequence_delta_net_test.cc:66-159,293-380), and torch
float64 autograd of the unrounded layer."""
import math

import numpy as np
import pytest
import torch

from oracle import pyoracle as po
from tests.test_oracle_qwen_backward import FrozenRounding


def values(n, phase, scale=0.8):
    return po.bf16_round(scale * np.sin(phase + 0.37 * np.arange(n))).astype(np.float64)


def forward(p, T, qkv, z, a, b, conv, a_log, dt_bias, norm, rnd):
    kh, vh, kd, vd, K = (p.key_heads, p.value_heads, p.key_head_dim, p.value_head_dim,
                         p.conv_kernel_dim)
    channels = 2 * kh * kd + vh * vd
    x = qkv.reshape(T, channels)
    post = np.zeros((T, channels))
    for t in range(T):
        for c in range(channels):
            total = 0.0
            for tap in range(K):
                source = t + tap - K + 1
                if source >= 0:
                    total += x[source, c] * conv[c * K + tap]
            total = rnd(total)
            post[t, c] = rnd(total / (1 + math.exp(-total)))
    out = np.zeros((T, vh, vd))
    for head in range(vh):
        key_head = head // (vh // kh)
        state = np.zeros((kd, vd))
        for t in range(T):
            q = post[t, key_head * kd:(key_head + 1) * kd]
            k = post[t, (kh + key_head) * kd:(kh + key_head + 1) * kd]
            v = post[t, 2 * kh * kd + head * vd:2 * kh * kd + (head + 1) * vd]
            q = q / math.sqrt(1e-6 + float(q @ q)) / math.sqrt(kd)
            k = k / math.sqrt(1e-6 + float(k @ k))
            alpha = a[t * vh + head] + dt_bias[head]
            softplus = max(alpha, 0.0) + math.log1p(math.exp(-abs(alpha)))
            decay = math.exp(-math.exp(a_log[head]) * softplus)
            beta = rnd(1 / (1 + math.exp(-b[t * vh + head])))
            state = state * decay
            delta = (v - k @ state) * beta
            state = state + np.outer(k, delta)
            core = np.array([rnd(value) for value in q @ state])
            inverse = 1 / math.sqrt(float(core @ core) / vd + p.rms_norm_epsilon)
            for c in range(vd):
                normalized = rnd(core[c] * inverse)
                affine = rnd(normalized * norm[c])
                gate = z[(t * vh + head) * vd + c]
                # the final store to bf16 is a rounding point like the others
                out[t, head, c] = rnd(affine * gate / (1 + math.exp(-gate)))
    return out


SHAPES = [dict(key_heads=1, value_heads=2, key_head_dim=3, value_head_dim=5, conv_kernel_dim=3),
          dict(key_heads=2, value_heads=2, key_head_dim=4, value_head_dim=3, conv_kernel_dim=4)]


@pytest.mark.parametrize("use_rounding", [False, True])
@pytest.mark.parametrize("shape", SHAPES)
def test_backward_matches_finite_differences_of_frozen_rounding_forward(use_rounding, shape):
    T = 4
    p = po.delta_params(round_to_bfloat16=use_rounding, **shape)
    kh, vh, kd, vd, K = (p.key_heads, p.value_heads, p.key_head_dim, p.value_head_dim,
                         p.conv_kernel_dim)
    channels = 2 * kh * kd + vh * vd
    inputs = [values(T * channels, .1), values(T * vh * vd, 1.1), values(T * vh, 2.1, 1.5),
              values(T * vh, 3.1, 1.5), values(channels * K, .5, 0.6), values(vh, .7, 0.5),
              values(vh, .9, 0.5), 1.0 + values(vd, 1.3, 0.3)]
    upstream = values(T * vh * vd, .7)
    got = po.gdn_sequence_backward(p, inputs[0].reshape(T, channels), inputs[1].reshape(T, vh * vd),
                                   inputs[2].reshape(T, vh), inputs[3].reshape(T, vh),
                                   inputs[4].reshape(channels, K), inputs[5], inputs[6], inputs[7],
                                   upstream.reshape(T, vh * vd))
    actual = [got[n].ravel() for n in ("dqkv", "dz", "da", "db", "d_conv_weight", "d_a_log",
                                       "d_dt_bias", "d_norm")]
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


def test_parameter_gradients_accumulate_and_can_be_skipped():
    T = 3
    p = po.delta_params(round_to_bfloat16=True, **SHAPES[0])
    kh, vh, kd, vd, K = 1, 2, 3, 5, 3
    channels = 2 * kh * kd + vh * vd
    args = (values(T * channels, .1).reshape(T, channels), values(T * vh * vd, 1.1).reshape(T, -1),
            values(T * vh, 2.1).reshape(T, vh), values(T * vh, 3.1).reshape(T, vh),
            values(channels * K, .5).reshape(channels, K), values(vh, .7), values(vh, .9),
            1.0 + values(vd, 1.3, 0.3), values(T * vh * vd, .7).reshape(T, -1))
    once = po.gdn_sequence_backward(p, *args)
    skipped = po.gdn_sequence_backward(p, *args, parameter_grads=False)
    for name in ("dqkv", "dz", "da", "db"):
        np.testing.assert_array_equal(once[name], skipped[name])
    for name in ("d_conv_weight", "d_a_log", "d_dt_bias", "d_norm"):
        assert np.abs(once[name]).sum() > 0 and not skipped[name].any()


def test_unrounded_backward_matches_float64_autograd():
    torch.manual_seed(11)
    T, kh, vh, kd, vd, K = 7, 2, 4, 6, 5, 4
    p = po.delta_params(key_heads=kh, value_heads=vh, key_head_dim=kd, value_head_dim=vd,
                        conv_kernel_dim=K, round_to_bfloat16=False)
    channels = 2 * kh * kd + vh * vd
    bf = lambda t: t.bfloat16().double()
    qkv, z = bf(torch.randn(T, channels)).requires_grad_(), bf(torch.randn(T, vh * vd)).requires_grad_()
    a, b = bf(torch.randn(T, vh)).requires_grad_(), bf(torch.randn(T, vh)).requires_grad_()
    conv = (0.5 * torch.randn(channels, K)).float().double().requires_grad_()
    a_log = (0.3 * torch.randn(vh)).float().double().requires_grad_()
    dt_bias = (0.3 * torch.randn(vh)).float().double().requires_grad_()
    norm = (1 + 0.2 * torch.randn(vd)).float().double().requires_grad_()
    dy = torch.randn(T, vh * vd).float().double()
    padded = torch.cat([torch.zeros(K - 1, channels, dtype=torch.float64), qkv])
    pre = sum(padded[tap:tap + T] * conv[:, tap] for tap in range(K))
    post = pre * torch.sigmoid(pre)
    outs = []
    for head in range(vh):
        key_head = head // (vh // kh)
        state = torch.zeros(kd, vd, dtype=torch.float64)
        for t in range(T):
            q = post[t, key_head * kd:(key_head + 1) * kd]
            k = post[t, (kh + key_head) * kd:(kh + key_head + 1) * kd]
            v = post[t, 2 * kh * kd + head * vd:2 * kh * kd + (head + 1) * vd]
            q = q * torch.rsqrt((q * q).sum() + 1e-6) / math.sqrt(kd)
            k = k * torch.rsqrt((k * k).sum() + 1e-6)
            decay = torch.exp(-torch.exp(a_log[head]) *
                              torch.nn.functional.softplus(a[t, head] + dt_bias[head]))
            beta = torch.sigmoid(b[t, head])
            state = state * decay
            state = state + torch.outer(k, (v - k @ state) * beta)
            core = q @ state
            normalized = core * torch.rsqrt((core * core).mean() + p.rms_norm_epsilon)
            gate = z[t, head * vd:(head + 1) * vd]
            outs.append((t, head, normalized * norm * gate * torch.sigmoid(gate)))
    loss = sum((o * dy[t, head * vd:(head + 1) * vd]).sum() for t, head, o in outs)
    loss.backward()
    got = po.gdn_sequence_backward(p, *[x.detach().numpy() for x in
                                        (qkv, z, a, b, conv, a_log, dt_bias, norm)], dy.numpy())
    for name, want in (("dqkv", qkv.grad), ("dz", z.grad), ("da", a.grad), ("db", b.grad),
                       ("d_conv_weight", conv.grad), ("d_a_log", a_log.grad),
                       ("d_dt_bias", dt_bias.grad), ("d_norm", norm.grad)):
        np.testing.assert_allclose(got[name], want.numpy(), rtol=1e-4, atol=2e-5, err_msg=name)
