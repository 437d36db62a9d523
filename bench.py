#!/usr/bin/env python3
"""Benchmark of the attention hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload NAME]

A step is one pass of the hot path over one batch of synthetic input that is
already resident in HBM when the timed region starts.  The headline workload
is the configuration the metric is quoted on: GPT-2-small causal attention
forward+backward, bf16 storage with fp32 accumulation, B=16, T=1024, H=12,
D=64.  The default run (--workload all) appends the other four configurations
of the path under "workloads", each with its own `roofline` and
`cpu_baseline`; --workload NAME runs one workload alone.

Each workload runs its W warm-up steps and times K steps straight after them
(`first_steps_ms`: the clocks of a part that was idle a moment ago), then runs
untimed for --settle-seconds (0.3 s) of continuous work and times K steps
again: `ms_per_step` and `value`.  The part reaches the clocks it sustains only
after some 30 ms of work, and a training or serving loop lives in that state
(the first 20 steps after an idle period run 10-15 % slower in the matrix-core
kernels).  `config.settle_s` records the setting; both figures are in the line.

`ms_per_step` (and `value`) come from HIP events recorded on the launch
stream just inside the two synchronizations that bracket the K steps;
`host_ms_per_step` is the host clock over the same bracket, which also
contains the host's wake-up after the last kernel.

Exactly one JSON line is printed.  `roofline` describes the kernel of the
step that takes longest.  Kernel durations come from one source: K further
steps in which every kernel group of the step is queued by a call of its own
(the library's measurement hook switches the other kernels of that call off;
a complete step has filled every buffer before), in the step's order, with a
HIP event on the launch stream between the groups.  The groups thus run in the
thermal state of the step, their durations add up to that split step's
(`split_step_ms`, a few microseconds of event gaps above `ms_per_step`), and
none can exceed it.  `achieved` is the kernel's algorithmic work divided by
its duration; where the step moves more bytes than the algorithm needs
(`roofline.moved_bytes`, from the counters), `frac_moved` prices those.  `cpu_baseline` is the scalar CPU
oracle timed on this host on a bounded sample of the same workload, on one
thread as the reference runs it (`value`, `cores` 1) and on `threads.cores`
threads over independent units (a reported baseline only).
"""
import argparse
import json
import math
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

PEAK_BF16_TFLOPS = 2500.0   # MI355X dense bf16 MFMA (published)
PEAK_FP32_TFLOPS = 157.3    # MI355X fp32 matrix (published)
PEAK_HBM_GBS = 8000.0       # MI355X HBM3E (published)

# HBM bytes per step of a kernel group, from rocprofv3 --pmc FETCH_SIZE and
# WRITE_SIZE runs of this file (FETCH_SIZE x 2.0 KiB and WRITE_SIZE x 1.0 KiB,
# the factors a 1 GiB device copy gives: `--workload copy`).  The summaries are
# kept as profiles/*_hbm_traffic.md.  None = not measured.
MEASURED_TRAFFIC_BYTES = {
    # (workload, kernel group): (bytes read + written, commit the counters were read at)
    ("mha_train_bf16", "flash_forward_kernel<64>"): (99.1e6 + 26.7e6, "4f26c5a"),
    ("mha_train_bf16", "flash_dq_kernel<64>"): (179.5e6 + 77.1e6, "4f26c5a"),
    ("mha_train_bf16", "flash_dkv_kernel<64>"): (154.5e6 + 100.7e6, "4f26c5a"),
    ("gqa_prefill", "flash_forward_pipelined_kernel<128>"): (184.6e6 + 88.1e6, "4f26c5a"),
    ("gqa_prefill_d256", "flash_forward_pipelined_kernel<256>"): (444.8e6 + 100.9e6, "4f26c5a"),
    ("gqa_decode", "decode_fused_kernel<128,6>"): (1044.2e6 + 13.0e6, "4f26c5a"),
    ("gdn_scan", "gdn_chunk_scan"): (524.5e6 + 138.8e6, "4f26c5a"),
}

NAMES = ["mha_train_bf16", "mha_fwd_fp32", "gqa_prefill", "gqa_decode", "gdn_scan"]
# "copy" is a plain device copy of known size: the calibration case for the
# FETCH_SIZE / WRITE_SIZE counters that `roofline.traffic` is derived from.
# "gqa_prefill_d256" is the prefill shape at head width 256; "gqa_prefill_bwd"
# and "gdn_layer_bwd" time the two sequence backward passes.
EXTRA = ["copy", "gqa_prefill_d256", "gqa_prefill_bwd", "gdn_layer_bwd", "gdn_decode", "dense_qkv", "dense_imported",
         "decode_block"]


def parse_args():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--workload", default="all", choices=NAMES + EXTRA + ["all"])
    ap.add_argument("--cpu-seconds", type=float, default=5.0,
                    help="CPU time budget of each cpu_baseline leg")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--settle-seconds", type=float, default=0.3,
                    help="untimed continuous running of each workload before its warm-up steps, "
                         "so that the timed steps see the clocks the part sustains (0 = none)")
    ap.add_argument("--launch", default="eager", choices=["graph", "eager"],
                    help="graph: replay the timed steps from a HIP graph where the workload supports "
                         "it (measured: 0.232 instead of 0.235 ms for the training step, 0.203 "
                         "instead of 0.198 ms for the decode step)")
    return ap.parse_args()


def causal_pairs(T):
    return T * (T + 1) // 2


def values(np, count, phase, scale):
    i = np.arange(count, dtype=np.float32)
    return (np.float32(scale) * np.sin(np.float32(phase) + i * np.float32(0.29))).astype(np.float32)


# --------------------------------------------------------------------------
# Workloads.  Each returns a dict:
#   step        callable running the whole hot path once
#   parts       [(name, callable, algorithmic work of that part)]
#   work        algorithmic FLOPs (bound mfma) or bytes (bound hbm) per step
# --------------------------------------------------------------------------

def mha_train_bf16(torch, capi):
    B, T, H, D = 16, 1024, 12, 64
    E = H * D
    gen = torch.Generator(device="cuda").manual_seed(1)
    qkv = torch.randn((B * T, 3 * E), generator=gen, device="cuda").to(torch.bfloat16)
    d_out = torch.randn((B * T, E), generator=gen, device="cuda")
    workspace = capi.mha_backward_workspace(qkv, T, H)
    d_qkv = torch.empty((B * T, 3 * E), dtype=torch.float32, device="cuda")
    state = {}

    def forward():
        state["fwd"] = capi.mha_forward(qkv, T, H, into=state.get("fwd"))

    def backward():
        out, maxima, normalizers = state["fwd"]
        capi.mha_backward(qkv, out, d_out, maxima, normalizers, T, H, workspace, d_qkv)

    def step():
        forward()
        backward()

    fwd = 4.0 * B * H * D * causal_pairs(T)
    bwd = 10.0 * B * H * D * causal_pairs(T)
    # The backward is two kernels that both recompute the scores and dP: the
    # query-owned one executes 3 products (S, dP, dQ), the key-owned one 4 (S,
    # dP, dK, dV).  The 5 counted products are shared out in that proportion.
    return dict(step=step, graph_outputs=lambda: list(state["fwd"]) + [d_qkv],
                kernels=[("flash_forward_kernel<64>", forward, None, fwd),
                         ("flash_dq_kernel<64>", backward, capi.QUERY_KERNEL, bwd * 3 / 7),
                         ("flash_dkv_kernel<64>", backward, capi.MAIN_KERNEL, bwd * 4 / 7)],
                work=fwd + bwd, metric="attention_fwd_bwd_tflops", unit="TFLOP/s", dtype="bf16",
                bound="mfma", peak=PEAK_BF16_TFLOPS,
                config={"workload": "gpt2_small_causal_mha_fwd_bwd", "batch": B, "seq_len": T,
                        "heads": H, "head_dim": D, "storage": "bf16", "accumulate": "fp32"},
                cpu=("mha", dict(B=B, T=T, H=H, D=D, bf16=True, backward=True)))


def mha_fwd_fp32(torch, capi):
    B, T, H, D = 4, 256, 12, 64
    E = H * D
    gen = torch.Generator(device="cuda").manual_seed(0)
    qkv = torch.randn((B * T, 3 * E), generator=gen, device="cuda")

    state = {}

    def forward():
        state["fwd"] = capi.mha_forward(qkv, T, H, into=state.get("fwd"))

    work = 4.0 * B * H * D * causal_pairs(T)
    return dict(step=forward, kernels=[("f32_forward_kernel<64>", forward, None, work)], work=work,
                metric="attention_fwd_tflops", unit="TFLOP/s", dtype="f32", bound="mfma",
                peak=PEAK_FP32_TFLOPS,
                config={"workload": "gpt2_small_causal_mha_fwd_fp32", "batch": B, "seq_len": T,
                        "heads": H, "head_dim": D, "storage": "fp32"},
                cpu=("mha", dict(B=B, T=T, H=H, D=D, bf16=False, backward=False)))


def gqa_prefill(torch, capi, d=128):
    import numpy as np
    T, qh, kh = 8192, 24, 4
    p = capi.attention_params(qh, kh, d, 32 if d == 128 else 64, capacity=T)
    gen = torch.Generator(device="cuda").manual_seed(2)
    bf = torch.bfloat16
    qg = (0.5 * torch.randn((T, qh, 2, d), generator=gen, device="cuda")).to(bf)
    k = (0.5 * torch.randn((T, kh, d), generator=gen, device="cuda")).to(bf)
    v = (0.5 * torch.randn((T, kh, d), generator=gen, device="cuda")).to(bf)
    qw = torch.from_numpy(values(np, d, 0.2, 0.3)).cuda()
    kw = torch.from_numpy(values(np, d, 0.8, 0.4)).cuda()
    cache = capi.KvCache(T, kh, d)
    out = torch.empty((T, qh, d), dtype=bf, device="cuda")
    size = capi.lib().pluto_hip_gqa_prefill_workspace_bytes(p, T)
    workspace = torch.empty(size, dtype=torch.uint8, device="cuda")

    def step():
        capi.gqa_prefill(p, qg, k, v, qw, kw, cache, out=out, workspace=workspace)

    work = 4.0 * qh * d * causal_pairs(T)
    return dict(step=step,
                kernels=[("rope table + prepare", step, capi.AUXILIARY_KERNELS, None),
                         ("flash_forward_pipelined_kernel<%d>" % d, step,
                          capi.MAIN_KERNEL | capi.EIGHT_WAVE | capi.FROM_LENGTH, work)],
                work=work,
                metric="gqa_prefill_tflops", unit="TFLOP/s", dtype="bf16", bound="mfma",
                peak=PEAK_BF16_TFLOPS,
                config={"workload": "qwen_gqa_prefill", "batch": 1, "seq_len": T, "query_heads": qh,
                        "kv_heads": kh, "head_dim": d,
                        "kv_cache": "bf16 [1,4,8192,%d], written by the call" % d},
                cpu=("gqa_prefill", dict(T=T, qh=qh, kh=kh, d=d)) if d == 128 else None)


def gqa_prefill_d256(torch, capi):
    """The prefill shape at the head width the model's parameters default to
    (256, rotary width 64): a row after the headline ones, not part of
    --workload all."""
    return gqa_prefill(torch, capi, d=256)


def gqa_prefill_bwd(torch, capi):
    """Backward of the whole-sequence Qwen layer at the prefill shape (the row
    after the headline ones: not part of --workload all)."""
    import numpy as np
    T, qh, kh, d = 8192, 24, 4, 128
    p = capi.attention_params(qh, kh, d, 32, capacity=T)
    gen = torch.Generator(device="cuda").manual_seed(2)
    bf = torch.bfloat16
    qg = (0.5 * torch.randn((T, qh, 2, d), generator=gen, device="cuda")).to(bf)
    k = (0.5 * torch.randn((T, kh, d), generator=gen, device="cuda")).to(bf)
    v = (0.5 * torch.randn((T, kh, d), generator=gen, device="cuda")).to(bf)
    dy = torch.randn((T, qh, d), generator=gen, device="cuda")
    qw = torch.from_numpy(values(np, d, 0.2, 0.3)).cuda()
    kw = torch.from_numpy(values(np, d, 0.8, 0.4)).cuda()

    # the forward pass of the training step leaves the attention output and the
    # row statistics for this call (outside the timed region, like the forward)
    cache = capi.KvCache(T, kh, d)
    saved = capi.gqa_prefill_saved(p, T, cache)
    capi.gqa_prefill(p, qg, k, v, qw, kw, cache, saved=saved)

    def step():
        capi.gqa_prefill_backward(p, qg, k, v, qw, kw, dy, saved=saved)

    work = 10.0 * qh * d * causal_pairs(T)
    return dict(step=step, kernels=[("whole call", step, None, work)], work=work,
                metric="gqa_sequence_backward_tflops", unit="TFLOP/s", dtype="bf16", bound="mfma",
                peak=PEAK_BF16_TFLOPS,
                config={"workload": "qwen_gqa_sequence_backward", "batch": 1, "seq_len": T,
                        "query_heads": qh, "kv_heads": kh, "head_dim": d,
                        "counted": "5 attention GEMMs; attention output and row statistics saved "
                                   "by the forward call"},
                cpu=None)


def gdn_layer_bwd(torch, capi):
    """Backward of the gated delta-net layer (FP32; 128 x 128 heads run in
    64-token chunks on the FP32 matrix cores): a row after the headline ones, not
    part of --workload all."""
    import numpy as np
    B, T, H, dk, dv, K = 1, 2048, 16, 128, 128, 4
    p = capi.delta_params(H, H, dk, dv, K)
    channels = 2 * H * dk + H * dv
    gen = torch.Generator(device="cuda").manual_seed(4)
    bf = torch.bfloat16
    qkv = torch.randn((B, T, channels), generator=gen, device="cuda").to(bf)
    z = torch.randn((B, T, H * dv), generator=gen, device="cuda").to(bf)
    a = torch.randn((B, T, H), generator=gen, device="cuda").to(bf)
    b = torch.randn((B, T, H), generator=gen, device="cuda").to(bf)
    conv = 0.5 * torch.randn((channels, K), generator=gen, device="cuda")
    a_log = torch.zeros(H, device="cuda")
    dt_bias = torch.zeros(H, device="cuda")
    norm = torch.ones(dv, device="cuda")
    dy = torch.randn((B, T, H * dv), generator=gen, device="cuda")

    # every parameter trains: the four parameter gradients are part of the call
    grads = dict(conv_weight=torch.zeros_like(conv), a_log=torch.zeros_like(a_log),
                 dt_bias=torch.zeros_like(dt_bias), norm=torch.zeros_like(norm))

    def step():
        capi.gdn_layer_backward(p, qkv, z, a, b, conv, a_log, dt_bias, norm, dy,
                                parameter_grads=grads)

    # recurrence form, per token, head and state element: 7 FLOPs to repeat the
    # forward (decay, prediction, update, output) and 15 for the reverse sweep
    work = 22.0 * B * T * H * dk * dv
    return dict(step=step, kernels=[("whole call", step, None, work)], work=work,
                metric="gdn_layer_backward_tflops", unit="TFLOP/s", dtype="f32", bound="mfma",
                peak=PEAK_FP32_TFLOPS,
                config={"workload": "gated_delta_net_layer_backward", "batch": B, "seq_len": T,
                        "heads": H, "d_k": dk, "d_v": dv, "conv_kernel": K,
                        "counted": "22 dk dv FLOPs per token and head (recurrence form)"},
                cpu=None)


def gqa_decode(torch, capi):
    import numpy as np
    batch, qh, kh, d, capacity = 32, 24, 4, 128, 32768
    p = capi.attention_params(qh, kh, d, 32, capacity=capacity)
    rng = np.random.default_rng(3)
    lengths = (1024 + np.floor(rng.random(batch) * 31745)).astype(int)
    gen = torch.Generator(device="cuda").manual_seed(3)
    bf = torch.bfloat16
    caches = []
    for L in lengths:
        c = capi.KvCache(capacity, kh, d)
        c.keys[:, :L] = torch.randn((kh, L, d), generator=gen, device="cuda").to(bf)
        c.values[:, :L] = torch.randn((kh, L, d), generator=gen, device="cuda").to(bf)
        c.position = int(L - 1)
        caches.append(c)
    q_gate = torch.randn((batch, qh, 2, d), generator=gen, device="cuda").to(bf)
    k = torch.randn((batch, kh, d), generator=gen, device="cuda").to(bf)
    v = torch.randn((batch, kh, d), generator=gen, device="cuda").to(bf)
    qw = torch.from_numpy(values(np, d, 0.2, 0.3)).cuda()
    kw = torch.from_numpy(values(np, d, 0.8, 0.4)).cuda()
    positions = [int(L - 1) for L in lengths]
    workspace = capi.gqa_decode_workspace(p, positions, 512)
    out = torch.empty((batch, qh, d), dtype=bf, device="cuda")

    def step():
        capi.gqa_decode(p, q_gate, k, v, qw, kw, caches, positions=positions, split_tokens=512,
                        workspace=workspace, out=out, advance=False)

    work = 2.0 * kh * d * 2 * float(lengths.sum())   # K and V bytes of the valid prefix
    return dict(step=step, graph_outputs=lambda: [out],
                kernels=[("counter clear", step, capi.AUXILIARY_KERNELS, None),
                         ("decode_fused_kernel<128,6>", step, capi.MAIN_KERNEL, work)],
                work=work,
                metric="gqa_decode_hbm_gbs", unit="GB/s", dtype="bf16", bound="hbm",
                peak=PEAK_HBM_GBS,
                config={"workload": "qwen_gqa_decode", "batch": batch, "sum_context": int(lengths.sum()),
                        "query_heads": qh, "kv_heads": kh, "head_dim": d, "split_tokens": 512,
                        "kv_cache": "bf16 head-major"},
                cpu=("gqa_decode", dict(lengths=[int(L) for L in lengths], qh=qh, kh=kh, d=d)))


def gdn_scan(torch, capi):
    B, T, H, dk, dv = 2, 16384, 16, 128, 128
    p = capi.delta_params(H, H, dk, dv)
    gen = torch.Generator(device="cuda").manual_seed(4)
    bf = torch.bfloat16
    q = torch.nn.functional.normalize(torch.randn((B, T, H, dk), generator=gen, device="cuda"), dim=-1).to(bf)
    k = torch.nn.functional.normalize(torch.randn((B, T, H, dk), generator=gen, device="cuda"), dim=-1).to(bf)
    v = torch.randn((B, T, H, dv), generator=gen, device="cuda").to(bf)
    beta = torch.sigmoid(torch.randn((B, T, H), generator=gen, device="cuda"))
    g = -torch.nn.functional.softplus(torch.randn((B, T, H), generator=gen, device="cuda"))
    state = torch.zeros((B, H, dk, dv), device="cuda")
    workspace = capi.gdn_scan_workspace(p, B, T, 64)
    out = torch.empty((B, T, H, dv), dtype=bf, device="cuda")
    scale = 1.0 / math.sqrt(dk)

    def scan():
        capi.gdn_scan(p, q, k, v, g, beta, state, q_scale=scale, chunk=64, workspace=workspace,
                      out=out)

    def step():
        state.zero_()
        scan()

    # The sequential kernel bounds the step; it reads K, Q, V, the prepared
    # per-chunk operands and the state, and writes the outputs and the state.
    # Priced against the whole step's algorithmic bytes it gives the fraction
    # of the roofline the step would reach if the preparation were free.
    work = B * T * H * (2 * dk + 2 * dv) * 2.0 + 2.0 * B * T * H * 4 + B * H * dk * dv * 4.0
    return dict(step=step,
                kernels=[("state clear", state.zero_, None, None),
                         ("gdn_chunk_prepare", scan, capi.AUXILIARY_KERNELS, None),
                         ("gdn_chunk_scan", scan, capi.MAIN_KERNEL, work)],
                work=work,
                metric="gated_delta_scan_hbm_gbs", unit="GB/s", dtype="bf16", bound="hbm",
                peak=PEAK_HBM_GBS,
                config={"workload": "gated_delta_net_chunked_scan", "batch": B, "seq_len": T,
                        "heads": H, "d_k": dk, "d_v": dv, "chunk": 64, "state": "fp32"},
                cpu=("gdn_scan", dict(T=T, H=H, dk=dk, dv=dv)))


def gdn_decode(torch, capi):
    """One token of the gated delta-net layer for 32 sequences with their own
    states (the delta-net half of a batched decoder step): a row after the
    headline ones, not part of --workload all."""
    batch, kh, H, dk, dv, K = 32, 16, 48, 128, 128, 4   # the model's 16 key / 48 value heads
    p = capi.delta_params(kh, H, dk, dv, K)
    channels = 2 * kh * dk + H * dv
    gen = torch.Generator(device="cuda").manual_seed(5)
    bf = torch.bfloat16
    states = capi.DeltaNetStep(p, batch=batch)
    qkv = torch.randn((batch, channels), generator=gen, device="cuda").to(bf)
    z = torch.randn((batch, H * dv), generator=gen, device="cuda").to(bf)
    a = torch.randn((batch, H), generator=gen, device="cuda").to(bf)
    b = torch.randn((batch, H), generator=gen, device="cuda").to(bf)
    conv = 0.5 * torch.randn((channels, K), generator=gen, device="cuda")
    a_log = torch.zeros(H, device="cuda")
    dt_bias = torch.zeros(H, device="cuda")
    norm = torch.ones(dv, device="cuda")

    def step():
        states.step(qkv, z, a, b, conv, a_log, dt_bias, norm)

    # every recurrent state is read and written once; so is every convolution state
    work = 2.0 * batch * (H * dk * dv + channels * K) * 4
    return dict(step=step, kernels=[("whole call", step, None, work)], work=work,
                metric="gdn_decode_step_hbm_gbs", unit="GB/s", dtype="f32", bound="hbm",
                peak=PEAK_HBM_GBS,
                config={"workload": "gated_delta_net_decode_step", "batch": batch, "key_heads": kh,
                        "value_heads": H, "d_k": dk, "d_v": dv, "conv_kernel": K,
                        "activations": "bf16", "state": "fp32, one per sequence"},
                cpu=None)


def decode_block(torch, capi):
    """The attention branches of one decoder step for 32 sequences at the model's
    shape (CreateAttentionBranch, qwen/model.cc:174-274, lifted from batch one):
    a full-attention branch (FP8 q|gate, k, v projections from the 5120-wide
    residual stream, cached attention with 24 / 4 heads of 256 over contexts of
    1024..32768 tokens, FP8 output projection) and a delta-net branch (FP8
    q|k|v, z, a, b projections, the gated delta step with 16 / 48 heads of
    128 x 128, FP8 output projection).  Bytes: every weight, every valid K/V row
    and every state once.  A row after the headline ones, not part of
    --workload all."""
    import numpy as np
    batch, width = 32, 5120
    qh, kvh, d, capacity = 24, 4, 256, 32768
    kh, vh, dk, dv, taps = 16, 48, 128, 128, 4
    bf = torch.bfloat16
    gen = torch.Generator(device="cuda").manual_seed(9)

    def matrix(n_in, n_out):
        w = torch.randint(0, 0x7e, (n_out, n_in), generator=gen, device="cuda", dtype=torch.uint8)
        w |= torch.randint(0, 2, (n_out, n_in), generator=gen, device="cuda", dtype=torch.uint8) << 7
        sc = (0.5 + torch.rand(((n_out + 127) // 128, (n_in + 127) // 128), generator=gen,
                               device="cuda")) * (0.004 / math.sqrt(n_in / 5120))
        size = lib_bytes(tokens=batch, input_dim=n_in)
        return dict(w=w, s=sc, ws=torch.empty(size, dtype=torch.uint8, device="cuda"),
                    bytes=float(w.numel() + sc.numel() * 4))

    def lib_bytes(tokens, input_dim):
        return max(capi.lib().pluto_hip_dense_imported_batch_workspace_bytes(tokens, input_dim), 1)

    def project(m, x, out):
        capi.dense_imported_forward_batch(capi.MATRIX_FP8_E4M3, m["w"], m["s"], x, m["ws"], out)

    hidden = torch.randn((batch, width), generator=gen, device="cuda").to(bf)
    # full attention
    q, kv = qh * d, kvh * d
    wq, wk, wv, wo = matrix(width, 2 * q), matrix(width, kv), matrix(width, kv), matrix(q, width)
    p = capi.attention_params(qh, kvh, d, 64, capacity=capacity)
    rng = np.random.default_rng(3)
    lengths = (1024 + np.floor(rng.random(batch) * 31745)).astype(int)
    caches = []
    for L in lengths:
        c = capi.KvCache(capacity, kvh, d)
        c.keys[:, :L] = torch.randn((kvh, L, d), generator=gen, device="cuda").to(bf)
        c.values[:, :L] = torch.randn((kvh, L, d), generator=gen, device="cuda").to(bf)
        caches.append(c)
    positions = [int(L - 1) for L in lengths]
    qn = torch.from_numpy(values(np, d, 0.2, 0.3)).cuda()
    kn = torch.from_numpy(values(np, d, 0.8, 0.4)).cuda()
    q_gate = torch.empty((batch, qh, 2, d), dtype=bf, device="cuda")
    k_new = torch.empty((batch, kvh, d), dtype=bf, device="cuda")
    v_new = torch.empty((batch, kvh, d), dtype=bf, device="cuda")
    attended = torch.empty((batch, qh, d), dtype=bf, device="cuda")
    attention_out = torch.empty((batch, width), dtype=bf, device="cuda")
    decode_ws = capi.gqa_decode_workspace(p, positions, 0)

    def project_many(matrices, x, outs):
        # the projections of one input in one call, as the host's branches run them
        capi.dense_imported_forward_many(capi.MATRIX_FP8_E4M3, [m["w"] for m in matrices],
                                         [m["s"] for m in matrices], x, matrices[0]["ws"], outs)

    def attention_in():
        project_many([wq, wk, wv], hidden,
                     [q_gate.view(batch, -1), k_new.view(batch, -1), v_new.view(batch, -1)])

    def attention_core():
        capi.gqa_decode(p, q_gate, k_new, v_new, qn, kn, caches, positions=positions,
                        workspace=decode_ws, out=attended, advance=False)

    def attention_project():
        project(wo, attended.view(batch, -1), attention_out)

    # delta-net
    keys, vals = kh * dk, vh * dv
    channels = 2 * keys + vals
    wqkv, wz, wa, wb, wout = (matrix(width, channels), matrix(width, vals), matrix(width, vh),
                              matrix(width, vh), matrix(vals, width))
    dp = capi.delta_params(kh, vh, dk, dv, taps)
    states = capi.DeltaNetStep(dp, batch=batch)
    conv = 0.5 * torch.randn((channels, taps), generator=gen, device="cuda")
    a_log, dt_bias, norm = (torch.zeros(vh, device="cuda"), torch.zeros(vh, device="cuda"),
                            torch.ones(dv, device="cuda"))
    qkv = torch.empty((batch, channels), dtype=bf, device="cuda")
    z = torch.empty((batch, vals), dtype=bf, device="cuda")
    a = torch.empty((batch, vh), dtype=bf, device="cuda")
    b = torch.empty((batch, vh), dtype=bf, device="cuda")
    delta_out = torch.empty((batch, width), dtype=bf, device="cuda")
    mixed = [None]

    def delta_in():
        project_many([wqkv, wz, wa, wb], hidden, [qkv, z, a, b])

    def delta_core():
        mixed[0] = states.step(qkv, z, a, b, conv, a_log, dt_bias, norm)

    def delta_project():
        project(wout, mixed[0], delta_out)

    def step():
        attention_in()
        attention_core()
        attention_project()
        delta_in()
        delta_core()
        delta_project()

    kv_bytes = 2.0 * kvh * d * 2 * float(lengths.sum())
    state_bytes = 2.0 * batch * (vh * dk * dv + channels * taps) * 4
    in_a = wq["bytes"] + wk["bytes"] + wv["bytes"]
    in_d = wqkv["bytes"] + wz["bytes"] + wa["bytes"] + wb["bytes"]
    work = kv_bytes + state_bytes + in_a + in_d + wo["bytes"] + wout["bytes"]
    return dict(step=step,
                kernels=[("attention: q|gate, k, v projections", attention_in, None, in_a),
                         ("attention: cached step (decode_fused_kernel<256,6>)", attention_core,
                          None, kv_bytes),
                         ("attention: output projection", attention_project, None, wo["bytes"]),
                         ("delta-net: q|k|v, z, a, b projections", delta_in, None, in_d),
                         ("delta-net: gated delta step", delta_core, None, state_bytes),
                         ("delta-net: output projection", delta_project, None, wout["bytes"])],
                work=work, metric="decoder_attention_branches_hbm_gbs", unit="GB/s", dtype="bf16",
                bound="hbm", peak=PEAK_HBM_GBS,
                config={"workload": "qwen_decoder_step_attention_branches", "batch": batch,
                        "model_width": width, "projections": "fp8_e4m3, 128x128 fp32 block scales",
                        "full_attention": {"query_heads": qh, "kv_heads": kvh, "head_dim": d,
                                           "rotary_dim": 64, "sum_context": int(lengths.sum()),
                                           "kv_cache": "bf16 head-major"},
                        "delta_net": {"key_heads": kh, "value_heads": vh, "d_k": dk, "d_v": dv,
                                      "conv_kernel": taps, "state": "fp32, one per sequence"}},
                cpu=None)


def dense_qkv(torch, capi):
    """The QKV projection in front of the default workload (gpt2.cc:55-71):
    FullyConnectedLayer 768 -> 2304 on 16 x 1024 bf16 rows, forward + backward.
    A row after the headline ones, not part of --workload all."""
    rows, n_in, n_out = 16 * 1024, 768, 2304
    gen = torch.Generator(device="cuda").manual_seed(6)
    x = torch.randn((rows, n_in), generator=gen, device="cuda").to(torch.bfloat16)
    w = torch.randn((n_in, n_out), generator=gen, device="cuda") / math.sqrt(n_in)
    b = torch.zeros(n_out, device="cuda")
    dy = torch.randn((rows, n_out), generator=gen, device="cuda")
    workspace = capi.dense_workspace(x, n_out)
    out = torch.empty((rows, n_out), dtype=torch.bfloat16, device="cuda")

    def forward():
        capi.dense_forward(x, w, b, workspace=workspace, out=out)

    def backward():
        capi.dense_backward(x, w, dy, workspace=workspace)

    def step():
        forward()
        backward()

    product = 2.0 * rows * n_in * n_out
    return dict(step=step, kernels=[("forward", forward, None, product),
                                    ("backward", backward, None, 2 * product)],
                work=3 * product, metric="dense_fwd_bwd_tflops", unit="TFLOP/s", dtype="bf16",
                bound="mfma", peak=PEAK_BF16_TFLOPS,
                config={"workload": "gpt2_small_qkv_projection_fwd_bwd", "rows": rows,
                        "input_dim": n_in, "output_dim": n_out, "storage": "bf16",
                        "accumulate": "fp32", "master_weights": "fp32"},
                cpu=None)


def dense_imported(torch, capi):
    """A frozen FP8 checkpoint projection at decode time (qwen/model.cc:192-227
    builds its projections from imported FullyConnectedLayers): one bf16 token
    of the checkpoint's 5120-wide residual stream times a [12288, 5120] FP8
    E4M3 matrix with 128 x 128 block scales.  Byte-bound: every weight is read
    once.  A row after the headline ones, not part of --workload all."""
    n_in, n_out = 5120, 12288
    gen = torch.Generator(device="cuda").manual_seed(8)
    weights = torch.randint(0, 0x7e, (n_out, n_in), generator=gen, device="cuda", dtype=torch.uint8)
    scales = torch.rand(((n_out + 127) // 128, (n_in + 127) // 128), generator=gen,
                        device="cuda") * 0.01
    x = torch.randn(n_in, generator=gen, device="cuda").to(torch.bfloat16)

    workspace = capi.dense_imported_workspace(n_in, x.device)
    out = torch.empty(n_out, dtype=torch.bfloat16, device="cuda")

    def step():
        capi.dense_imported_forward(capi.MATRIX_FP8_E4M3, weights, scales, x, workspace, out)

    work = float(n_in * n_out + scales.numel() * 4 + n_in * 2 + n_out * 2)
    return dict(step=step, kernels=[("whole call", step, None, work)], work=work,
                metric="imported_projection_gbs", unit="GB/s", dtype="f32", bound="hbm",
                peak=PEAK_HBM_GBS,
                config={"workload": "qwen_imported_fp8_projection_one_token", "input_dim": n_in,
                        "output_dim": n_out, "storage": "fp8_e4m3", "block_scales": "128x128 fp32"},
                cpu=None)


def copy(torch, capi):
    n = 256 * 2 ** 20   # 1 GiB read + 1 GiB written per step
    src = torch.ones(n, dtype=torch.float32, device="cuda")
    dst = torch.empty_like(src)

    def step():
        dst.copy_(src)

    work = 2.0 * n * 4
    return dict(step=step, kernels=[("copy", step, None, work)], work=work, metric="device_copy_gbs",
                unit="GB/s", dtype="f32", bound="hbm", peak=PEAK_HBM_GBS,
                config={"workload": "device_copy_calibration", "bytes_read": n * 4,
                        "bytes_written": n * 4}, cpu=None)


WORKLOADS = {"copy": copy, "gdn_decode": gdn_decode, "decode_block": decode_block, "dense_qkv": dense_qkv, "dense_imported": dense_imported, "mha_train_bf16": mha_train_bf16, "mha_fwd_fp32": mha_fwd_fp32,
             "gqa_prefill": gqa_prefill, "gqa_prefill_d256": gqa_prefill_d256,
             "gqa_prefill_bwd": gqa_prefill_bwd, "gdn_layer_bwd": gdn_layer_bwd,
             "gqa_decode": gqa_decode,
             "gdn_scan": gdn_scan}


# --------------------------------------------------------------------------
# CPU baseline: the scalar oracle on independent units of the same workload.
# Each maker returns (run_unit(i) -> algorithmic work of that unit, number of
# units, description of a unit).
# --------------------------------------------------------------------------

def cpu_units_mha(spec):
    import numpy as np
    from oracle import pyoracle as oracle
    B, T, H, D = spec["B"], spec["T"], spec["H"], spec["D"]
    E = H * D
    rng = np.random.default_rng(1)
    x = rng.standard_normal((T, 3 * E)).astype(np.float32)
    d_out = rng.standard_normal((T, E)).astype(np.float32)
    dtype = oracle.BF16 if spec["bf16"] else oracle.F32
    data = oracle.f32_to_bf16_bits(x).reshape(x.shape) if spec["bf16"] else x
    work = (14.0 if spec["backward"] else 4.0) * D * causal_pairs(T)

    def run(i):
        head = i % H
        out, _, _ = oracle.mha_fwd(data, T, H, dtype, (0, 1), (head, head + 1))
        if spec["backward"]:
            oracle.mha_bwd(data, out, d_out, T, H, dtype, (0, 1), (head, head + 1))
        return work

    return run, B * H, "(sequence, head) units, %s" % (
        "forward+backward" if spec["backward"] else "forward")


def cpu_units_gqa_prefill(spec):
    import numpy as np
    from oracle import pyoracle as oracle
    T, qh, kh, d = spec["T"], spec["qh"], spec["kh"], spec["d"]
    po = oracle.attention_params(qh, kh, d, 32, capacity=T)
    rng = np.random.default_rng(2)
    qg = oracle.bf16_round((0.5 * rng.standard_normal((T, qh, 2, d))).astype(np.float32))
    k = oracle.bf16_round((0.5 * rng.standard_normal((T, kh, d))).astype(np.float32))
    v = oracle.bf16_round((0.5 * rng.standard_normal((T, kh, d))).astype(np.float32))
    qw, kw = values(np, d, 0.2, 0.3), values(np, d, 0.8, 0.4)
    rows = 32   # query rows per unit, taken from evenly spread places of the sequence
    blocks = T // rows

    def run(i):
        head = i % qh
        block = (i * 37 + 11) % blocks
        r0 = block * rows
        oracle.gqa_sequence(po, qg, k, v, qw, kw, rows=(r0, r0 + rows), heads=(head, head + 1))
        return 4.0 * d * sum(r + 1 for r in range(r0, r0 + rows))

    return run, blocks * qh, "(head, %d query rows) units" % rows


def cpu_units_gqa_decode(spec):
    import numpy as np
    from oracle import pyoracle as oracle
    lengths, qh, kh, d = spec["lengths"], spec["qh"], spec["kh"], spec["d"]
    po = oracle.attention_params(qh, kh, d, 32, capacity=max(lengths))
    rng = np.random.default_rng(3)
    longest = max(lengths)
    keys = oracle.bf16_round(rng.standard_normal((kh, longest, d)).astype(np.float32))
    vals = oracle.bf16_round(rng.standard_normal((kh, longest, d)).astype(np.float32))
    q = oracle.bf16_round(rng.standard_normal((qh, d)).astype(np.float32))
    gate = oracle.bf16_round(rng.standard_normal((qh, d)).astype(np.float32))

    def run(i):
        L = lengths[i % len(lengths)]
        oracle.gqa_attend(po, q, gate, np.ascontiguousarray(keys[:, :L]),
                          np.ascontiguousarray(vals[:, :L]))
        return 2.0 * kh * d * 2 * L

    return run, len(lengths), "sequences (attention over the cached rows, all heads)"


def cpu_units_gdn_scan(spec):
    import numpy as np
    from oracle import pyoracle as oracle
    T, H, dk, dv = spec["T"], spec["H"], spec["dk"], spec["dv"]
    tokens = 2048   # tokens per unit: the first `tokens` of one head's chain
    po = oracle.delta_params(H, H, dk, dv)
    rng = np.random.default_rng(4)

    def unit(x):
        return x / np.sqrt((x * x).sum(-1, keepdims=True))

    q = oracle.bf16_round(unit(rng.standard_normal((tokens, H, dk))).astype(np.float32))
    k = oracle.bf16_round(unit(rng.standard_normal((tokens, H, dk))).astype(np.float32))
    v = oracle.bf16_round(rng.standard_normal((tokens, H, dv)).astype(np.float32))
    beta = (1.0 / (1.0 + np.exp(-rng.standard_normal((tokens, H))))).astype(np.float32)
    g = (-np.log1p(np.exp(rng.standard_normal((tokens, H))))).astype(np.float32)
    scale = 1.0 / math.sqrt(dk)
    per_token = (2 * dk + 2 * dv) * 2.0 + 8.0

    def run(i):
        head = i % H
        oracle.gdn_scan(po, q, k, v, g, beta, False, scale, heads=(head, head + 1))
        return per_token * tokens

    return run, 2 * H * (T // tokens), "(head, %d tokens) units of a chain" % tokens


CPU_UNITS = {"mha": cpu_units_mha, "gqa_prefill": cpu_units_gqa_prefill,
             "gqa_decode": cpu_units_gqa_decode, "gdn_scan": cpu_units_gdn_scan}


def cpu_baseline(kind, spec, bound, budget):
    """One thread (as the reference runs), then `threads` threads over
    independent units (the oracle's C code runs outside the interpreter lock).
    Rates are per unit of algorithmic work, so a sample needs no scaling."""
    import concurrent.futures
    run, total, what = CPU_UNITS[kind](spec)
    divisor = 1e12 if bound == "mfma" else 1e9
    unit = "TFLOP/s" if bound == "mfma" else "GB/s"
    done, work, t0 = 0, 0.0, time.perf_counter()
    while done < total and time.perf_counter() - t0 < budget:
        work += run(done)
        done += 1
    seconds = time.perf_counter() - t0
    threads = max(1, min(16, os.cpu_count() or 1))

    def worker(first):
        mine, i = 0.0, first
        start = time.perf_counter()
        while i < total and time.perf_counter() - start < budget:
            mine += run(i)
            i += threads
        return mine, (i - first) // threads

    t1 = time.perf_counter()
    with concurrent.futures.ThreadPoolExecutor(max_workers=threads) as pool:
        results = list(pool.map(worker, range(threads)))
    wall = time.perf_counter() - t1
    many_work = sum(r[0] for r in results)
    many_units = sum(r[1] for r in results)
    return dict(value=float("%.4g" % (work / seconds / divisor)), unit=unit, cores=1, kind="port",
                sample="%d of %d %s of the workload in %.1f s" % (done, total, what, seconds),
                threads=dict(cores=threads, value=float("%.4g" % (many_work / wall / divisor)),
                             sample="%d units in %.1f s" % (many_units, wall)))


def capture_step(torch, w):
    """The step as a HIP graph, or None.  A workload that wants its timed steps
    replayed from a graph lists under "graph_outputs" the tensors a step writes;
    the graph is used only if three replays, with eager steps and
    synchronizations between them, each leave bit for bit what the eager step
    leaves (every kernel here is bitwise repeatable)."""
    outputs = w.get("graph_outputs")
    if outputs is None:
        return None
    w["step"]()
    torch.cuda.synchronize()
    expected = [t.clone() for t in outputs()]
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        w["step"]()
    for _ in range(3):
        for t in outputs():
            t.zero_()
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        if not all(torch.equal(a, b) for a, b in zip(outputs(), expected)):
            return None
        w["step"]()
        torch.cuda.synchronize()
    return graph


def measure(torch, capi, w, steps, warmup, launch="eager", settle_seconds=0.0):
    stream = torch.cuda.current_stream()

    def timed(run, count):
        """`count` calls between two events on the launch stream, themselves just
        inside two synchronizations: the host's wake-up after the last kernel
        (tens of microseconds, 5 % of 20 steps of 0.2 ms) is not charged to the
        steps; the host's own clock over the same bracket is returned too."""
        first, last = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        first.record(stream)
        for _ in range(count):
            run()
        last.record(stream)
        torch.cuda.synchronize()
        return first.elapsed_time(last) / count, (time.perf_counter() - t0) * 1e3 / count

    for _ in range(warmup):
        w["step"]()
    torch.cuda.synchronize()
    graph = capture_step(torch, w) if launch == "graph" else None
    run_step = graph.replay if graph is not None else w["step"]
    w["config"]["launch"] = ("hip graph replay, one per step" if graph is not None
                             else "eager, one launch per kernel")
    # the K steps right after the W warm-up steps: a part that was idle a moment ago
    first_steps_ms, _ = timed(run_step, steps)
    # The part needs some 30 ms of continuous work to reach the clocks it then
    # sustains (the matrix-core kernels run 10-15 % slower until then), far more
    # than a handful of warm-up steps of 0.2 ms: the step runs untimed for
    # `settle_seconds`, then the K steps are timed again.
    settle_until = time.perf_counter() + settle_seconds
    while time.perf_counter() < settle_until:
        for _ in range(50):
            run_step()
        torch.cuda.synchronize()
    w["config"]["settle_s"] = settle_seconds
    ms_per_step, host_ms_per_step = timed(run_step, steps)
    # Every buffer now holds what a complete step leaves, so any one kernel group
    # of the step can run alone on valid inputs.  K split steps: the groups in
    # the step's order, each queued by its own call, an event between them.
    groups = w["kernels"]
    marks = [[torch.cuda.Event(enable_timing=True) for _ in range(len(groups) + 1)]
             for _ in range(steps)]

    def split_step(events):
        events[0].record(stream)
        for (name, fn, mask, work), event in zip(groups, events[1:]):
            with capi.only_kernels(0xffffffff if mask is None else mask):
                fn()
            event.record(stream)

    for _ in range(max(3, warmup)):
        split_step(marks[0])
    torch.cuda.synchronize()
    for events in marks:
        split_step(events)
    torch.cuda.synchronize()
    kernels = {}
    for index, (name, fn, mask, work) in enumerate(groups):
        mean = sum(e[index].elapsed_time(e[index + 1]) for e in marks) / steps
        kernels[name] = (mean, work)
    split_step_ms = marks[0][0].elapsed_time(marks[-1][-1]) / steps
    w["step"]()   # leave complete results behind
    torch.cuda.synchronize()
    counted = {k: v for k, v in kernels.items() if v[1] is not None}
    dominant = max(counted, key=lambda k: counted[k][0])
    dom_ms, dom_work = counted[dominant]
    divisor = 1e12 if w["bound"] == "mfma" else 1e9
    value = w["work"] / (ms_per_step * 1e-3) / divisor
    achieved = dom_work / (dom_ms * 1e-3) / divisor
    return dict(ms_per_step=ms_per_step, host_ms_per_step=host_ms_per_step,
                first_steps_ms=first_steps_ms, split_step_ms=split_step_ms, value=value,
                kernels=kernels, dominant=dominant, achieved=achieved, kernel_ms=dom_ms)


def roofline(name, w, m):
    unit = "TFLOP/s" if w["bound"] == "mfma" else "GB/s"
    line = {"bound": w["bound"], "kernel": m["dominant"], "achieved": round(m["achieved"], 3),
            "peak": w["peak"], "unit": unit, "frac": round(m["achieved"] / w["peak"], 4),
            "traffic": None, "kernel_ms": round(m["kernel_ms"], 4)}
    measured = MEASURED_TRAFFIC_BYTES.get((name, m["dominant"]))
    if measured is not None:
        moved, commit = measured
        line["traffic"] = moved
        line["traffic_commit"] = commit
        if w["bound"] == "hbm":
            # `achieved` and `frac` price the algorithmic bytes; these the bytes moved
            line["algorithmic_bytes"] = w["work"]
            line["moved_bytes"] = moved
            line["frac_moved"] = round(moved / (m["kernel_ms"] * 1e-3) / 1e9 / w["peak"], 4)
    return line


def summary(w, m):
    return {"ms_per_step": round(m["ms_per_step"], 4),
            "host_ms_per_step": round(m["host_ms_per_step"], 4),
            "first_steps_ms": round(m["first_steps_ms"], 4),
            "split_step_ms": round(m["split_step_ms"], 4)}


def main():
    args = parse_args()
    if args.gpus != 1:
        print("bench.py measures one GPU: this build has no multi-GPU path (use --gpus 1)",
              file=sys.stderr)
        sys.exit(2)
    import torch
    from pluto_amd import capi
    assert torch.cuda.is_available(), "bench.py needs a GPU"
    torch.cuda.set_device(0)
    capi.lib()
    head = "mha_train_bf16" if args.workload == "all" else args.workload
    w = WORKLOADS[head](torch, capi)
    m = measure(torch, capi, w, args.steps, args.warmup, args.launch, args.settle_seconds)
    result = {
        "metric": w["metric"], "value": round(m["value"], 3), "unit": w["unit"], "n_gpus": 1,
        "steps": args.steps, "warmup": args.warmup, **summary(w, m),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": w["dtype"], "data": "synthetic", "config": w["config"],
        "roofline": roofline(head, w, m),
        "kernels_ms": {k: round(v[0], 4) for k, v in m["kernels"].items()},
    }
    if not args.no_cpu_baseline and w["cpu"] is not None:
        result["cpu_baseline"] = cpu_baseline(w["cpu"][0], w["cpu"][1], w["bound"], args.cpu_seconds)
    if args.workload == "all":
        others = {}
        for name in NAMES:
            if name == head:
                continue
            del w
            torch.cuda.empty_cache()
            w = WORKLOADS[name](torch, capi)
            mm = measure(torch, capi, w, args.steps, args.warmup, args.launch, args.settle_seconds)
            others[name] = {"metric": w["metric"], "value": round(mm["value"], 3), "unit": w["unit"],
                            **summary(w, mm), "dtype": w["dtype"],
                            "config": w["config"], "roofline": roofline(name, w, mm),
                            "kernels_ms": {k: round(v[0], 4) for k, v in mm["kernels"].items()}}
            if not args.no_cpu_baseline and w["cpu"] is not None:
                others[name]["cpu_baseline"] = cpu_baseline(w["cpu"][0], w["cpu"][1], w["bound"],
                                                            args.cpu_seconds)
        result["workloads"] = others
    print(json.dumps(result))


if __name__ == "__main__":
    main()
