#!/usr/bin/env python3
"""Benchmark of the causal FlashAttention-2 hot path on one MI355X.

A step is one forward + backward pass of ``flash_attention_v2`` through the real
``torch.autograd`` path on one batch of synthetic input already resident in HBM.  The workload
is the headline configuration C3 (B=2, H=32, N=4096, D=128, bf16, causal) unless
``--workload`` names another one.  One JSON line is printed; ``value`` is forward+backward
TFLOP/s with the FlashAttention-2 FLOP convention (fwd = 4*B*H*N^2*D/2, bwd = 2.5 x fwd), and
the forward-only figures and fractions of the dense bf16 MFMA peak are in the same line.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload C3] [--no-cpu-baseline]
                    [--no-other-workloads]

After the headline workload's timed region the other BASELINE configurations (and one
short-sequence shape) are timed briefly and reported in ``other_workloads``.
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
CALIBRATION_BYTES = 256 << 20
# HBM bytes per launch come from rocprofv3's FETCH_SIZE / WRITE_SIZE counters (counters cannot be
# read from inside the process): the tracked summary below lists them per kernel for workload C3,
# together with a hash of the kernel sources it was measured on.  Other workloads, or sources that
# have changed since, report null.
TRAFFIC_PROFILE = ROOT / "profiles" / "fwd_bwd_kernels_c3_bf16_hbm_traffic.txt"
KERNEL_SOURCES = ROOT / "flash-attention-triton_amd" / "csrc"
PEAK_HBM_GBS = 8000.0
METRIC = "causal attn TFLOP/s fwd & fwd+bwd (bf16, D=128) and % of MFMA peak, 1 GPU"


def kernel_sources_hash() -> str:
    """sha256 over the kernel sources with comments and white space taken out (names and code): the
    stamp the traffic summary carries.  A change of comments or layout leaves it alone; any change of
    code, which may change the traffic, does not."""
    import hashlib
    import re

    strip = re.compile(r'//[^\n]*|/\*.*?\*/|("(?:\\.|[^"\\])*")', re.S)
    h = hashlib.sha256()
    for path in sorted(list(KERNEL_SOURCES.glob("*.h*")) + list(KERNEL_SOURCES.glob("Makefile"))):
        text = strip.sub(lambda m: m.group(1) or " ", path.read_text())
        h.update(path.name.encode())
        h.update(" ".join(text.split()).encode())
    return h.hexdigest()[:16]


def _measured_traffic(workload: str) -> tuple[dict, str]:
    """{leg: bytes per launch} from the tracked counter summary, and a note saying why it is empty."""
    if workload != "C3":
        return {}, "the counter summary covers workload C3 only"
    if not TRAFFIC_PROFILE.exists():
        return {}, "no counter summary in profiles/"
    stamp, rows = None, {}
    for line in TRAFFIC_PROFILE.read_text().splitlines():
        if line.startswith("kernel-sources-sha256:"):
            stamp = line.split(":", 1)[1].strip()
        if line.startswith("traffic-bytes "):
            _, leg, value = line.split()
            rows[leg] = float(value)
    if stamp != kernel_sources_hash():
        return {}, f"kernel sources changed since the counter summary was taken (summary {stamp}, now {kernel_sources_hash()})"
    return rows, "profiles/" + TRAFFIC_PROFILE.name


class ClockSampler:
    """Samples the shader clock the driver reports (sysfs pp_dpm_sclk, the level marked '*') from
    a background thread while a timed region runs."""

    def __init__(self, period_s: float = 0.002):
        import glob
        import threading

        files = sorted(glob.glob("/sys/class/drm/card*/device/pp_dpm_sclk"))
        self.path = files[0] if files else None
        self.period = period_s
        self.samples: list[float] = []
        self._stop = threading.Event()
        self._thread = threading.Thread(target=self._run, daemon=True)

    def _read(self):
        try:
            with open(self.path) as f:
                for line in f:
                    if "*" in line:
                        return float(line.split(":")[1].lower().replace("mhz", "").replace("*", "").strip())
        except (OSError, ValueError, IndexError):
            return None
        return None

    def _run(self):
        while not self._stop.is_set():
            v = self._read()
            if v is not None:
                self.samples.append(v)
            self._stop.wait(self.period)

    def __enter__(self):
        if self.path:
            self._thread.start()
        return self

    def __exit__(self, *exc):
        self._stop.set()
        if self.path:
            self._thread.join()
        return False

    def summary(self):
        if not self.samples:
            return None
        return {"samples": len(self.samples), "min": min(self.samples), "max": max(self.samples),
                "mean": sum(self.samples) / len(self.samples)}


def _device_clock_mhz(props) -> float:
    """Maximum shader clock: torch's property when it is filled in, else hipDeviceAttributeClockRate."""
    khz = getattr(props, "clock_rate", 0)
    if not khz:
        import ctypes

        try:
            hip = ctypes.CDLL("libamdhip64.so")
            value = ctypes.c_int(0)
            if hip.hipDeviceGetAttribute(ctypes.byref(value), 5, 0) == 0:  # hipDeviceAttributeClockRate, kHz
                khz = value.value
        except OSError:
            khz = 0
    return khz / 1e3


def _cpu_model() -> str:
    try:
        for line in open("/proc/cpuinfo"):
            if line.lower().startswith("model name"):
                return line.split(":", 1)[1].strip()
    except OSError:
        pass
    return "unknown"


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
    for _ in range(3):  # untimed: first launches of a kernel run at clocks that have not settled
        fn()
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

    def fwd(row=capi.FA2_CONFIG_AUTO):
        capi.check(lib.fa2_fwd(q.data_ptr(), k.data_ptr(), v.data_ptr(), o.data_ptr(), lse.data_ptr(),
                               b, h, n, n, d, n_r, *s3(q), *s3(k), *s3(v), *s3(o),
                               scale, dtype, row, stream), "fa2_fwd")

    # The row a forward takes that nothing will differentiate (what `fwd_ms` of the JSON line times).
    forward_only_row = lib.fa2_pick_config_forward_only(dtype, d, n, n)

    def pre():
        capi.check(lib.fa2_bwd_preprocess(o.data_ptr(), d_o.data_ptr(), delta.data_ptr(), b, h, n, d, n_r,
                                          *s3(o), *s3(d_o), dtype, stream), "fa2_bwd_preprocess")

    results = {}
    fwd()
    pre()
    torch.cuda.synchronize()
    results["fwd"] = _event_time_ms(fwd, iters)
    results["fwd_forward_only"] = _event_time_ms(lambda: fwd(forward_only_row), iters)
    fwd()  # leave the log-sum-exp of the forward a backward follows for the backward legs
    results["bwd_preprocess"] = _event_time_ms(pre, iters)
    ws_bytes = lib.fa2_bwd_workspace_bytes(b, h, n, n, d, 0, capi.FA2_CONFIG_AUTO)
    ws = torch.empty(max(ws_bytes, 1), dtype=torch.uint8, device=q.device)

    def bwd(det, want_dq=True, want_dkdv=True):
        capi.check(lib.fa2_bwd(q.data_ptr(), k.data_ptr(), v.data_ptr(), d_o.data_ptr(),
                               lse.data_ptr(), delta.data_ptr(), ws.data_ptr(),
                               dq.data_ptr() if want_dq else None,
                               dk.data_ptr() if want_dkdv else None,
                               dv.data_ptr() if want_dkdv else None,
                               b, h, n, n, d, n_r, *s3(q), *s3(k), *s3(v), *s3(d_o),
                               *s3(dq), *s3(dk), *s3(dv), scale, dtype, det,
                               capi.FA2_CONFIG_AUTO, stream), "fa2_bwd")

    def bwd_fused():
        capi.check(lib.fa2_bwd_fused(q.data_ptr(), k.data_ptr(), v.data_ptr(), o.data_ptr(), d_o.data_ptr(),
                                     lse.data_ptr(), delta.data_ptr(), ws.data_ptr(),
                                     dq.data_ptr(), dk.data_ptr(), dv.data_ptr(),
                                     b, h, n, n, d, n_r, *s3(q), *s3(k), *s3(v), *s3(o), *s3(d_o),
                                     *s3(dq), *s3(dk), *s3(dv), scale, dtype, 0,
                                     capi.FA2_CONFIG_AUTO, stream), "fa2_bwd_fused")

    legs = {
        # What autograd runs: dQ (forming delta on the way) then dK/dV, no preprocess launch.
        "bwd_fused": bwd_fused,
        "bwd_deterministic": lambda: bwd(1),
        "bwd_sequence_parallel": lambda: bwd(0),
        # One kernel each: NULL outputs switch the other kernel off.
        "bwd_dkdv": lambda: bwd(0, want_dq=False),
        "bwd_dq": lambda: bwd(0, want_dkdv=False),
    }
    # The sequence-parallel backward run the reference's way (table rows with dq_atomic: one kernel
    # per key tile, dQ accumulated with fp32 global atomics; never picked automatically): the whole
    # call, i.e. accumulator clear + that kernel + conversion, preprocess not included, so that the
    # figure compares with bwd_deterministic / bwd_sequence_parallel above.
    atomic_rows = {r["headdim_padded"]: r["id"] for r in capi.config_table() if r["dq_atomic"]}
    if d in atomic_rows:
        row = atomic_rows[d]
        ws_atomic = torch.empty(lib.fa2_bwd_workspace_bytes(b, h, n, n, d, 0, row), dtype=torch.uint8, device=q.device)

        def bwd_atomic():
            capi.check(lib.fa2_bwd(q.data_ptr(), k.data_ptr(), v.data_ptr(), d_o.data_ptr(),
                                   lse.data_ptr(), delta.data_ptr(), ws_atomic.data_ptr(),
                                   dq.data_ptr(), dk.data_ptr(), dv.data_ptr(),
                                   b, h, n, n, d, n_r, *s3(q), *s3(k), *s3(v), *s3(d_o),
                                   *s3(dq), *s3(dk), *s3(dv), scale, dtype, 0, row, stream), "fa2_bwd (dq_atomic row)")

        legs["bwd_sequence_parallel_atomic"] = bwd_atomic
    for name, fn in legs.items():
        fn()
        torch.cuda.synchronize()
        results[name] = _event_time_ms(fn, iters)
    return results


def _cpu_baseline(w, workloads, heads: int):
    """Naive fp32 causal attention (the reference's ground truth) on the host CPU, on the first
    ``heads`` (batch, head) slices of the same seeded workload, forward + backward."""
    from oracle import naive_attention as oracle

    # A one-GPU box's share of the host is 16 cores whatever os.cpu_count() shows there.
    threads = min(os.cpu_count() or 1, 16)
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
        "os_cpu_count": os.cpu_count(),
        "cpu_model": _cpu_model(),
        "kind": "port",
        "sample": f"{heads} of {w.batch * w.nheads} (batch, head) slices of {w.name}, fp32 forward+backward "
                  f"through torch autograd, {dt:.2f} s",
        "seconds": dt,
    }


# Workloads timed after the headline one (a few tens of milliseconds each) and reported in
# `other_workloads`: the other four BASELINE configurations and one short-sequence, many-heads shape
# of the kind the reference's own tests use (tests/test_flash_attention_2.py:22-29).
OTHER_WORKLOADS = ("C1", "C2", "C4", "C5", "S512")


def _other_workloads(pkg, workloads, dev, names, budget_ms: float = 60.0) -> dict:
    """Forward and forward+backward time of further workloads through the same public function and
    autograd path as the headline step.  Inputs are drawn on the device (same shapes, dtypes and
    standard deviations as the seeded parity inputs; only timing is taken here)."""
    table = dict(workloads.WORKLOADS)
    table["S512"] = workloads.Workload("S512", 256, 16, 512, 64, torch.bfloat16,
                                       description="short sequences, many heads")
    out = {}
    for name in names:
        w = table[name]
        gen = torch.Generator(device=dev).manual_seed(42)
        q, k, v, d_o = (
            (torch.randn(w.shape, generator=gen, device=dev, dtype=torch.float32) * std).to(w.dtype)
            for std in (w.qk_std, w.qk_std, 1.0, 1.0))
        q.requires_grad_(True)
        k.requires_grad_(True)
        v.requires_grad_(True)

        def step():
            return torch.autograd.grad(pkg.flash_attention_v2(q, k, v, w.softmax_scale, False), (q, k, v), d_o)

        def fwd_only():
            with torch.no_grad():
                return pkg.flash_attention_v2(q, k, v, w.softmax_scale, False)

        def timed(fn):
            # Untimed calls for about a third of the budget, then as many timed calls as fit the rest.
            fn()
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            fn()
            torch.cuda.synchronize()
            once_ms = max((time.perf_counter() - t0) * 1e3, 1e-3)
            n_warm = max(3, int(budget_ms / 3 / once_ms))
            n = max(5, min(2000, int(budget_ms * 2 / 3 / once_ms)))
            for _ in range(n_warm):
                fn()
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            for _ in range(n):
                fn()
            torch.cuda.synchronize()
            return (time.perf_counter() - t0) * 1e3 / n, n

        step_ms, n_step = timed(step)
        fwd_ms, n_fwd = timed(fwd_only)
        peak = PEAK_TFLOPS["bf16" if w.dtype == torch.bfloat16 else "f16"]
        out[name] = {
            "shape": list(w.shape), "dtype": "bf16" if w.dtype == torch.bfloat16 else "f16", "qk_std": w.qk_std,
            "fwd_ms": fwd_ms, "ms_per_step": step_ms, "timed_calls": [n_fwd, n_step],
            "fwd_tflops": w.fwd_flops / (fwd_ms * 1e-3) / 1e12,
            "fwd_frac_of_peak": w.fwd_flops / (fwd_ms * 1e-3) / 1e12 / peak,
            "fwd_bwd_tflops": 3.5 * w.fwd_flops / (step_ms * 1e-3) / 1e12,
            "fwd_bwd_frac_of_peak": 3.5 * w.fwd_flops / (step_ms * 1e-3) / 1e12 / peak,
        }
        del q, k, v, d_o
    return out


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=100)
    ap.add_argument("--warmup", type=int, default=50, help="untimed steps right before the timed ones")
    ap.add_argument("--settle-ms", type=float, default=400.0,
                    help="before the warm-up steps, run untimed steps for at least this long and then until "
                         "their rate has stopped changing (see --settle-max-ms): an idle GPU sits at ~100 MHz, "
                         "its clocks need some hundreds of milliseconds of load, and under its power limit the "
                         "chip keeps getting faster for several seconds as it warms up (on a box that had been "
                         "idle the same 20 steps measured 6 %% slower after 0.4 s of load than after 8 s).  "
                         "0 switches the phase off")
    ap.add_argument("--settle-max-ms", type=float, default=20000.0,
                    help="upper bound of the settle phase; it ends earlier once the rate of half-second windows "
                         "of calls has stopped moving (last three within 0.4 %%, less than 0.3 %% over two seconds)")
    ap.add_argument("--workload", default="C3")
    ap.add_argument("--deterministic", action="store_true", help="time the deterministic backward in the step")
    ap.add_argument("--cpu-heads", type=int, default=64, help="(batch, head) slices in the CPU baseline sample")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-other-workloads", action="store_true",
                    help="skip the block of further workloads timed after the headline one")
    ap.add_argument("--traffic-calibration", action="store_true",
                    help="also launch a plain 256 MiB -> 256 MiB elementwise copy three times, so a hardware-"
                         "counter run of this command holds a kernel of known HBM traffic to scale by")
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

    def settle(fn):
        """Untimed calls until the rate is steady (at least --settle-ms, at most --settle-max-ms).
        Returns what was observed."""
        if args.settle_ms <= 0:
            return {"ms": 0.0, "windows": 0}
        t_begin = time.perf_counter()
        windows = []
        while True:
            t0, calls = time.perf_counter(), 0
            while time.perf_counter() - t0 < 0.5:
                for _ in range(10):
                    fn()
                torch.cuda.synchronize()
                calls += 10
            windows.append((time.perf_counter() - t0) * 1e3 / calls)
            elapsed_ms = (time.perf_counter() - t_begin) * 1e3
            # Steady: the last three windows agree within 0.4 % and the rate has moved by less than
            # 0.3 % over the last two seconds (the warm-up drift is slow: a tenth of a percent a second).
            last = windows[-3:]
            steady = (len(windows) >= 5 and max(last) / min(last) - 1.0 < 0.004
                      and abs(windows[-1] / windows[-5] - 1.0) < 0.003)
            if elapsed_ms >= args.settle_max_ms or (elapsed_ms >= args.settle_ms and steady):
                return {"ms": elapsed_ms, "windows": len(windows), "first_window_ms_per_call": windows[0],
                        "last_window_ms_per_call": windows[-1]}

    settle_step = settle(step)
    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    with ClockSampler() as step_clock:
        t0 = time.perf_counter()
        for _ in range(args.steps):
            step()
        torch.cuda.synchronize()
        step_ms = (time.perf_counter() - t0) * 1e3 / args.steps

    # The same steps with PyTorch's backward engine kept on the calling thread.  By default the
    # engine hands the backward of CUDA tensors to a worker thread and waits for it; at the smallest
    # workloads that hand-off (tens of microseconds of host time) is longer than the kernels.
    # Reported beside ms_per_step, never instead of it.
    with torch.autograd.set_multithreading_enabled(False):
        for _ in range(max(args.warmup, 1)):
            step()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(args.steps):
            step()
        torch.cuda.synchronize()
        step_ms_one_thread = (time.perf_counter() - t0) * 1e3 / args.steps

    settle_fwd = settle(fwd_only)
    for _ in range(max(args.warmup, 1)):
        fwd_only()
    torch.cuda.synchronize()
    with ClockSampler() as fwd_clock:
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
    # FLOPs per launch, counted in causal GEMMs of fwd_flops / 2 each: the forward kernel owns 2
    # (S, PV), the dK/dV kernel 4 (S, dP, dV, dK), the dQ kernel 3 (S, dP, dQ).  The whole backward
    # is priced at the conventional 5 (2.5 x forward) although the two kernels execute 7.
    # The LDS-direct kernels run when the table row has them and the head dimension needs no
    # padding (the bench tensors are contiguous and 16-byte aligned); otherwise the generic ones.
    fa2 = importlib.import_module("flash-attention-triton_amd.flash_attention_2")
    row_id = capi.load().fa2_pick_config(fa2._COMPUTE_DTYPES[w.dtype], w.headdim, w.seqlen, w.seqlen, int(det))
    row = capi.config_table()[row_id]
    kind = "direct_kernel" if row["lds_direct"] and row["headdim_padded"] == w.headdim else "kernel"
    only_row = capi.config_table()[capi.load().fa2_pick_config_forward_only(fa2._COMPUTE_DTYPES[w.dtype], w.headdim,
                                                                           w.seqlen, w.seqlen)]
    kernels = {
        "fwd": (f"fwd_{kind} (fa2_fwd, table row {row['id']}: the forward a backward follows)", 1.0 * w.fwd_flops),
        "fwd_forward_only": (f"fwd_{kind} (fa2_fwd, table row {only_row['id']}: the forward nothing differentiates, "
                             "timed as fwd_ms)", 1.0 * w.fwd_flops),
        "bwd_dkdv": (f"bwd_dkdv_{kind} (fa2_bwd, dK/dV half)", 2.0 * w.fwd_flops),
        "bwd_dq": (f"bwd_dq_{kind} (fa2_bwd, dQ half)", 1.5 * w.fwd_flops),
    }
    dominant = max((name for name in kernels if name != "fwd_forward_only"), key=lambda name: leg_ms[name])
    traffic, traffic_source = _measured_traffic(w.name)

    def mfma_roofline(name):
        label, flops = kernels[name]
        achieved = flops / (leg_ms[name] * 1e-3) / 1e12
        return {"kernel": label, "bound": "mfma", "achieved": achieved, "peak": peak, "unit": "TFLOP/s",
                "frac": achieved / peak, "traffic": traffic.get(name), "traffic_source": traffic_source,
                "flops_per_launch": flops,
                "avg_launch_ms": leg_ms[name]}

    roofline = mfma_roofline(dominant)
    bwd_leg = "bwd_fused"
    bwd_tflops = w.bwd_flops / (leg_ms[bwd_leg] * 1e-3) / 1e12
    pre_bytes = 2.0 * w.batch * w.nheads * w.seqlen * w.headdim * 2 + w.batch * w.nheads * w.seqlen * 4
    pre_roofline = {
        "kernel": "fa2_bwd_preprocess (bwd_preprocess_kernel)", "bound": "hbm",
        "achieved": pre_bytes / (leg_ms["bwd_preprocess"] * 1e-3) / 1e9, "peak": PEAK_HBM_GBS, "unit": "GB/s",
        "frac": pre_bytes / (leg_ms["bwd_preprocess"] * 1e-3) / 1e9 / PEAK_HBM_GBS,
        "traffic": traffic.get("bwd_preprocess"), "bytes_per_launch": pre_bytes,
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
        "ms_per_step_autograd_on_calling_thread": step_ms_one_thread,
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
        # fwd_ms times the public function under torch.no_grad(): for bf16 that is the forward-only
        # table row.  The forward inside the timed step (a backward follows) is the plain row:
        "fwd_in_step_kernel_ms": leg_ms["fwd"],
        "fwd_in_step_frac_of_peak": w.fwd_flops / (leg_ms["fwd"] * 1e-3) / 1e12 / peak,
        "peak_tflops": peak,
        "device": {"name": props.name, "arch": getattr(props, "gcnArchName", ""),
                   "compute_units": props.multi_processor_count,
                   "clock_mhz": _device_clock_mhz(props),
                   "sclk_mhz_during_steps": step_clock.summary(),
                   "sclk_mhz_during_fwd": fwd_clock.summary()},
        # Untimed calls before each timed region (forward + backward steps, then forward only) and how
        # their rate moved meanwhile; see --settle-ms.
        "settle_ms": settle_step["ms"] + settle_fwd["ms"],
        "settle": {"steps": settle_step, "fwd": settle_fwd},
        "roofline": roofline,
        "roofline_fwd": mfma_roofline("fwd_forward_only"),
        "roofline_fwd_in_step": mfma_roofline("fwd"),
        "roofline_bwd_dkdv": mfma_roofline("bwd_dkdv"),
        "roofline_bwd_dq": mfma_roofline("bwd_dq"),
        "bwd_tflops_algorithmic": bwd_tflops,
        "bwd_frac_of_peak": bwd_tflops / peak,
        "roofline_bwd_preprocess": pre_roofline,
        "kernel_ms": leg_ms,
        "table_row": row,
        "table_row_forward_only": only_row,
    }
    if args.traffic_calibration:
        src = torch.ones(CALIBRATION_BYTES // 4, device=dev, dtype=torch.float32)
        dst = torch.empty_like(src)
        for _ in range(3):
            torch.mul(src, 1.0, out=dst)
        torch.cuda.synchronize()
        line["traffic_calibration"] = {"kernel": "torch elementwise mul (fp32, out=)",
                                       "read_bytes": CALIBRATION_BYTES, "write_bytes": CALIBRATION_BYTES}
    if not args.no_other_workloads:
        line["other_workloads"] = _other_workloads(pkg, workloads, dev, [n for n in OTHER_WORKLOADS if n != w.name])
    if not args.no_cpu_baseline:
        line["cpu_baseline"] = _cpu_baseline(w, workloads, args.cpu_heads)
    print(json.dumps(line))
    return 0


if __name__ == "__main__":
    sys.exit(main())
