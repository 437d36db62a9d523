#!/usr/bin/env python3
"""Benchmark of the attention hot path on one MI355X.

`python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload NAME]`

A step is one pass of the hot path over one batch of synthetic input that is
already resident in HBM.  The default workload is the configuration the
headline metric is quoted on: GPT-2-small causal attention forward+backward,
bf16 storage, B=16, T=1024, H=12, D=64.  One JSON line is printed.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

PEAK_BF16_TFLOPS = 2500.0   # MI355X dense bf16 MFMA, published
PEAK_HBM_GBS = 8000.0       # MI355X HBM3E, published


def parse_args():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--workload", default="mha_train_bf16",
                    choices=["mha_train_bf16", "mha_fwd_fp32", "gqa_prefill",
                             "gqa_decode", "gdn_scan"])
    ap.add_argument("--no-cpu-baseline", action="store_true")
    return ap.parse_args()


def causal_pairs(T):
    return T * (T + 1) // 2


class EventTimer:
    """HIP events on the stream the kernels are launched on."""

    def __init__(self, torch, stream):
        self.torch, self.stream = torch, stream
        self.pairs = []

    def time(self, fn):
        start = self.torch.cuda.Event(enable_timing=True)
        end = self.torch.cuda.Event(enable_timing=True)
        start.record(self.stream)
        fn()
        end.record(self.stream)
        self.pairs.append((start, end))

    def mean_ms(self):
        return sum(s.elapsed_time(e) for s, e in self.pairs) / max(len(self.pairs), 1)


def mha_train_bf16(args, torch, capi):
    B, T, H, D = 16, 1024, 12, 64
    E = H * D
    gen = torch.Generator(device="cuda").manual_seed(1)
    qkv = torch.randn((B * T, 3 * E), generator=gen, device="cuda").to(torch.bfloat16)
    d_out = torch.randn((B * T, E), generator=gen, device="cuda")
    workspace = capi.mha_backward_workspace(qkv, T, H)
    d_qkv = torch.empty((B * T, 3 * E), dtype=torch.float32, device="cuda")
    state = {}

    def forward():
        state["fwd"] = capi.mha_forward(qkv, T, H)

    def backward():
        out, maxima, normalizers = state["fwd"]
        capi.mha_backward(qkv, out, d_out, maxima, normalizers, T, H, workspace, d_qkv)

    def step():
        forward()
        backward()

    fwd_flops = 4.0 * B * H * D * causal_pairs(T)
    bwd_flops = 10.0 * B * H * D * causal_pairs(T)
    return dict(
        step=step, parts=[("forward", forward, fwd_flops), ("backward", backward, bwd_flops)],
        flops=fwd_flops + bwd_flops, metric="attention_fwd_bwd_tflops", unit="TFLOP/s",
        dtype="bf16", bound="mfma", peak=PEAK_BF16_TFLOPS,
        config={"workload": "gpt2_small_causal_mha_fwd_bwd", "batch": B, "seq_len": T,
                "heads": H, "head_dim": D, "storage": "bf16", "accumulate": "fp32"},
        cpu=("mha", dict(B=B, T=T, H=H, D=D, bf16=True)))


WORKLOADS = {"mha_train_bf16": mha_train_bf16}


def cpu_baseline_mha(spec, budget_units=1):
    """Times the scalar CPU oracle (one thread) on whole (sequence, head) units of
    the same workload and scales to the full size."""
    import numpy as np
    from oracle import pyoracle as oracle
    B, T, H, D = spec["B"], spec["T"], spec["H"], spec["D"]
    E = H * D
    rng = np.random.default_rng(1)
    x = rng.standard_normal((T, 3 * E)).astype(np.float32)   # one sequence is enough
    d_out = rng.standard_normal((T, E)).astype(np.float32)
    bits = oracle.f32_to_bf16_bits(x).reshape(x.shape)
    t0 = time.perf_counter()
    out, _, _ = oracle.mha_fwd(bits, T, H, oracle.BF16, (0, 1), (0, budget_units))
    oracle.mha_bwd(bits, out, d_out, T, H, oracle.BF16, (0, 1), (0, budget_units))
    seconds = time.perf_counter() - t0
    flops = 14.0 * D * causal_pairs(T) * budget_units
    return dict(value=flops / seconds / 1e12, unit="TFLOP/s", cores=1, kind="port",
                sample="%d of %d (sequence, head) units, forward+backward, %.1f s" % (
                    budget_units, B * H, seconds))


def main():
    args = parse_args()
    if args.gpus != 1:
        print("bench.py measures one GPU: this build has no multi-GPU path "
              "(run with --gpus 1)", file=sys.stderr)
        sys.exit(2)
    import torch
    from pluto_amd import capi
    assert torch.cuda.is_available(), "bench.py needs a GPU"
    torch.cuda.set_device(0)
    capi.lib()
    if args.workload not in WORKLOADS:
        print("workload %s is not built yet" % args.workload, file=sys.stderr)
        sys.exit(2)
    w = WORKLOADS[args.workload](args, torch, capi)
    stream = torch.cuda.current_stream()
    for _ in range(args.warmup):
        w["step"]()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        w["step"]()
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    ms_per_step = wall * 1e3 / args.steps
    # Per-part device time with HIP events on the launch stream.
    parts = {}
    for name, fn, work in w["parts"]:
        timer = EventTimer(torch, stream)
        for _ in range(args.steps):
            timer.time(fn)
        torch.cuda.synchronize()
        parts[name] = (timer.mean_ms(), work)
    dominant = max(parts, key=lambda k: parts[k][0])
    dom_ms, dom_work = parts[dominant]
    if w["bound"] == "mfma":
        value = w["flops"] / (ms_per_step * 1e-3) / 1e12
        achieved = dom_work / (dom_ms * 1e-3) / 1e12
        roof_unit = "TFLOP/s"
    else:
        value = w["bytes"] / (ms_per_step * 1e-3) / 1e9
        achieved = dom_work / (dom_ms * 1e-3) / 1e9
        roof_unit = "GB/s"
    result = {
        "metric": w["metric"], "value": round(value, 3), "unit": w["unit"], "n_gpus": 1,
        "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(ms_per_step, 4),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": w["dtype"], "data": "synthetic", "config": w["config"],
        "roofline": {"bound": w["bound"], "kernel": dominant, "achieved": round(achieved, 3),
                     "peak": w["peak"], "unit": roof_unit,
                     "frac": round(achieved / w["peak"], 4), "traffic": None,
                     "kernel_ms": round(dom_ms, 4)},
        "parts_ms": {k: round(v[0], 4) for k, v in parts.items()},
    }
    if not args.no_cpu_baseline:
        kind, spec = w["cpu"]
        result["cpu_baseline"] = cpu_baseline_mha(spec) if kind == "mha" else None
    print(json.dumps(result))


if __name__ == "__main__":
    main()
