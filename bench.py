#!/usr/bin/env python3
"""Benchmark of the causal FlashAttention-2 hot path on one MI355X.

A step is one forward + backward pass of ``flash_attention_v2`` through the real
``torch.autograd`` path on one batch of synthetic input already resident in HBM.  The workload
is BASELINE's headline configuration C3 (B=2, H=32, N=4096, D=128, bf16, causal) unless
``--workload`` names another one.  One JSON line is printed; ``value`` is forward+backward
TFLOP/s with the FlashAttention-2 FLOP convention (fwd = 4*B*H*N^2*D/2, bwd = 2.5 x fwd), and
the forward-only figures and fractions of the dense bf16 MFMA peak are in the same line.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload C3] [--no-cpu-baseline]
"""

from __future__ import annotations

import argparse
import importlib
import json
import os
import pathlib
import statistics
import sys
import time

import torch

ROOT = pathlib.Path(__file__).resolve().parent
sys.path.insert(0, str(ROOT))

# Published dense peaks of MI355X.
PEAK_TFLOPS = {"bf16": 2500.0, "f16": 2500.0}
PEAK_HBM_GBS = 8000.0
METRIC = "causal attn TFLOP/s fwd & fwd+bwd (bf16, D=128) and % of MFMA peak, 1 GPU"


def _load_package():
    pkg = importlib.import_module("flash_attention_triton_amd")
    capi = importlib.import_module("flash-attention-triton_amd._capi")
    workloads = importlib.import_module("flash-attention-triton_amd.workloads")
    if not capi.LIBRARY_PATH.exists():
        importlib.import_module("flash-attention-triton_amd.build").build()
    return pkg, capi, workloads


def _event_time_ms(fn, iters: int) -> list[float]:
    """Per-call GPU time of ``fn`` measured with HIP events on torch's current stream, which is
    the stream the library launches on."""
    times = []
    for _ in range(iters):
        start = torch.cuda.Event(enable_timing=True)
        end = torch.cuda.Event(enable_timing=True)
        start.record()
        fn()
        end.record()
        end.synchronize()
        times.append(start.elapsed_time(end))
    return times


def _kernel_legs(capi, w, q, k, v, d_o, iters: int):
    """Time each C-ABI entry point alone (forward, delta preprocess, backward main)."""
    import math
    import ctypes  # noqa: F401

    fa2 = importlib.import_module("flash-attention-triton_amd.flash_attention_2")
    lib = capi.load()
    b, h, n, d = w.shape
    n_r = math.ceil(n / capi.FA2_MAX_HEADDIM) * capi.FA2_MAX_HEADDIM
    dtype = fa2._COMPUTE_DTYPES[q.dtype]
    scale = 1.0 / math.sqrt(d)
    o = torch.empty_like(q)
    lse = torch.empty((b, h, n_r), device=q.device, dtype=torch.float32)
    delta = torch.empty_like(lse)
    dq, dk, dv = torch.empty_like(q), torch.empty_like(k), torch.empty_like(v)
    s3 = fa2._strides3
    stream = torch.cuda.current_stream().cuda_stream

    def fwd():
        capi.check(lib.fa2_fwd(q.data_ptr(), k.data_ptr(), v.data_ptr(), o.data_ptr(), lse.data_ptr(),
                               b, h, n, n, d, n_r, *s3(q), *s3(k), *s3(v), *s3(o),
                               scale, dtype, capi.FA2_CONFIG_AUTO, stream), "fa2_fwd")

    def pre():
        capi.check(lib.fa2_bwd_preprocess(o.data_ptr(), d_o.data_ptr(), delta.data_ptr(), b, h, n, d, n_r,
                                          *s3(o), *s3(d_o), dtype, stream), "fa2_bwd_preprocess")

    results = {}
    fwd()
    pre()
    torch.cuda.synchronize()
    results["fwd"] = _event_time_ms(fwd, iters)
    results["bwd_preprocess"] = _event_time_ms(pre, iters)
    for det in (1, 0):
        ws_bytes = lib.fa2_bwd_workspace_bytes(b, h, n, n, d, det, capi.FA2_CONFIG_AUTO)
        ws = torch.empty(max(ws_bytes, 1), dtype=torch.uint8, device=q.device)

        def bwd(det=det, ws=ws):
            capi.check(lib.fa2_bwd(q.data_ptr(), k.data_ptr(), v.data_ptr(), d_o.data_ptr(),
                                   lse.data_ptr(), delta.data_ptr(), ws.data_ptr(),
                                   dq.data_ptr(), dk.data_ptr(), dv.data_ptr(),
                                   b, h, n, n, d, n_r, *s3(q), *s3(k), *s3(v), *s3(d_o),
                                   *s3(dq), *s3(dk), *s3(dv), scale, dtype, det,
                                   capi.FA2_CONFIG_AUTO, stream), "fa2_bwd")

        bwd()
        torch.cuda.synchronize()
        results["bwd_deterministic" if det else "bwd_sequence_parallel"] = _event_time_ms(bwd, iters)
    return results


def _cpu_baseline(w, workloads, heads: int):
    """Naive fp32 causal attention (the reference's ground truth) on the host CPU, on the first
    ``heads`` (batch, head) slices of the same seeded workload, forward + backward."""
    from oracle import naive_attention as oracle

    threads = os.cpu_count() or 1
    threads = min(threads, 16)
    torch.set_num_threads(threads)
    q, k, v, d_o = workloads.make_inputs(w, "cpu", heads=heads)
    t0 = time.perf_counter()
    oracle.sliced_forward_backward(q, k, v, d_o, w.softmax_scale, torch.float32, heads=heads)
    dt = time.perf_counter() - t0
    flops = 3.5 * w.fwd_flops * heads / (w.batch * w.nheads)
    return {
        "value": flops / dt / 1e12,
        "unit": "TFLOP/s",
        "cores": torch.get_num_threads(),
        "kind": "port",
        "sample": f"{heads} of {w.batch * w.nheads} (batch, head) slices of {w.name}, fp32 forward+backward "
                  f"through torch autograd, {dt:.2f} s",
        "seconds": dt,
    }


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--workload", default="C3")
    ap.add_argument("--deterministic", action="store_true", help="time the deterministic backward in the step")
    ap.add_argument("--cpu-heads", type=int, default=2, help="(batch, head) slices in the CPU baseline sample")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    args = ap.parse_args()

    if args.gpus != 1:
        print("bench.py measures one GPU: every box of this build has one, and causal attention needs "
              "no exchange between GPUs (batch and heads shard with no communication). Use --gpus 1.",
              file=sys.stderr)
        return 2
    if not torch.cuda.is_available():
        print("bench.py needs a GPU (the HIP kernels have no CPU fallback).", file=sys.stderr)
        return 2

    pkg, capi, workloads = _load_package()
    w = workloads.WORKLOADS[args.workload]
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    props = torch.cuda.get_device_properties(dev)
    q, k, v, d_o = workloads.make_inputs(w, dev)
    q.requires_grad_(True)
    k.requires_grad_(True)
    v.requires_grad_(True)
    scale = w.softmax_scale
    det = bool(args.deterministic)

    def step():
        out = pkg.flash_attention_v2(q, k, v, scale, det)
        return torch.autograd.grad(out, (q, k, v), d_o)

    def fwd_only():
        with torch.no_grad():
            return pkg.flash_attention_v2(q, k, v, scale, det)

    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step()
    torch.cuda.synchronize()
    step_ms = (time.perf_counter() - t0) * 1e3 / args.steps

    for _ in range(max(args.warmup, 1)):
        fwd_only()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        fwd_only()
    torch.cuda.synchronize()
    fwd_ms = (time.perf_counter() - t0) * 1e3 / args.steps

    dtype_name = "bf16" if w.dtype == torch.bfloat16 else "f16"
    peak = PEAK_TFLOPS[dtype_name]
    fwd_bwd_tflops = 3.5 * w.fwd_flops / (step_ms * 1e-3) / 1e12
    fwd_tflops = w.fwd_flops / (fwd_ms * 1e-3) / 1e12

    # Per-kernel legs through the C ABI, timed with HIP events on the launch stream.
    legs = _kernel_legs(capi, w, q.detach(), k.detach(), v.detach(), d_o, max(args.steps, 5))
    leg_ms = {name: statistics.mean(ts) for name, ts in legs.items()}
    # Algorithmic FLOPs: the forward owns 2 GEMMs (1 x fwd_flops), the backward 5 (2.5 x).
    bwd_leg = "bwd_deterministic" if det else "bwd_sequence_parallel"
    dominant = "fwd" if leg_ms["fwd"] >= leg_ms[bwd_leg] else bwd_leg
    dom_flops = w.fwd_flops if dominant == "fwd" else w.bwd_flops
    achieved = dom_flops / (leg_ms[dominant] * 1e-3) / 1e12
    roofline = {
        "kernel": "fa2_fwd (fwd_kernel)" if dominant == "fwd" else f"fa2_bwd ({bwd_leg}: bwd_dkdv_kernel + bwd_dq_kernel)",
        "bound": "mfma",
        "achieved": achieved,
        "peak": peak,
        "unit": "TFLOP/s",
        "frac": achieved / peak,
        "traffic": None,
        "avg_launch_ms": leg_ms[dominant],
    }
    fwd_roofline = {
        "kernel": "fa2_fwd (fwd_kernel)", "bound": "mfma",
        "achieved": w.fwd_flops / (leg_ms["fwd"] * 1e-3) / 1e12, "peak": peak, "unit": "TFLOP/s",
        "frac": w.fwd_flops / (leg_ms["fwd"] * 1e-3) / 1e12 / peak, "traffic": None,
        "avg_launch_ms": leg_ms["fwd"],
    }
    pre_bytes = 2.0 * w.batch * w.nheads * w.seqlen * w.headdim * 2 + w.batch * w.nheads * w.seqlen * 4
    pre_roofline = {
        "kernel": "fa2_bwd_preprocess (bwd_preprocess_kernel)", "bound": "hbm",
        "achieved": pre_bytes / (leg_ms["bwd_preprocess"] * 1e-3) / 1e9, "peak": PEAK_HBM_GBS, "unit": "GB/s",
        "frac": pre_bytes / (leg_ms["bwd_preprocess"] * 1e-3) / 1e9 / PEAK_HBM_GBS, "traffic": None,
        "avg_launch_ms": leg_ms["bwd_preprocess"],
    }

    line = {
        "metric": METRIC,
        "value": fwd_bwd_tflops,
        "unit": "TFLOP/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": step_ms,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": dtype_name,
        "data": "synthetic",
        "config": {
            "workload": f"{w.name}: causal attention fwd+bwd, B={w.batch} H={w.nheads} N={w.seqlen} D={w.headdim}, "
                        f"{dtype_name} q/k/v/dO ~ N(0,{w.qk_std:g}^2) seed 42, layout (B,H,N,D)",
            "deterministic": det,
            "flop_convention": "fwd = 4*B*H*N^2*D/2, bwd = 2.5*fwd",
        },
        "fwd_bwd_tflops": fwd_bwd_tflops,
        "fwd_bwd_frac_of_peak": fwd_bwd_tflops / peak,
        "fwd_tflops": fwd_tflops,
        "fwd_ms": fwd_ms,
        "fwd_frac_of_peak": fwd_tflops / peak,
        "peak_tflops": peak,
        "device": {"name": props.name, "arch": getattr(props, "gcnArchName", ""),
                   "compute_units": props.multi_processor_count,
                   "clock_mhz": getattr(props, "clock_rate", 0) / 1e3},
        "roofline": roofline,
        "roofline_fwd": fwd_roofline,
        "roofline_bwd_preprocess": pre_roofline,
        "kernel_ms": leg_ms,
    }
    if not args.no_cpu_baseline:
        line["cpu_baseline"] = _cpu_baseline(w, workloads, args.cpu_heads)
    print(json.dumps(line))
    return 0


if __name__ == "__main__":
    sys.exit(main())
