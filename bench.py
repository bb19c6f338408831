#!/usr/bin/env python3
"""Throughput of the low-precision hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload NAME] [--no-cpu]

Prints ONE JSON line. A "step" is one pass of the hot path over one batch of
synthetic input that is already resident in HBM. The default workload is the 8192^3
blockwise FP8 GEMM. Every time is the median of WINDOWS windows of K steps.
``roofline`` prices the dominant kernel of the workload (algorithmic bytes or flops per
launch / its launch duration, timed with HIP events on the launch stream) against MI355X's
published peak; the HBM-bound workloads rotate their input through more than 512 MB of
copies, so that the 256 MB Infinity Cache cannot serve the reads. ``cpu_baseline`` times the
reference's own pure-PyTorch formulas (oracle/cpu_reference.py) on the host cores over a
bounded sample. ``extra`` carries the same measurements for the other workloads of the
configurations this path is quoted on (shorter runs, no CPU leg).
"""

from __future__ import annotations

import argparse
import json
import os
import sys
import time
from pathlib import Path

ROOT = Path(__file__).resolve().parent
for _p in (ROOT, ROOT / "primus-turbo_amd"):
    if str(_p) not in sys.path:
        sys.path.insert(0, str(_p))

import torch  # noqa: E402

HBM_PEAK_GBS = 8000.0
FP8_PEAK_TFLOPS = 5000.0
FP4_PEAK_TFLOPS = 10100.0


def _events_ms(fn, iters):
    """Average duration (ms) of ``fn`` over ``iters`` back-to-back launches, HIP events on
    torch's current stream (the stream every kernel of this library is launched on)."""
    start = torch.cuda.Event(enable_timing=True)
    stop = torch.cuda.Event(enable_timing=True)
    torch.cuda.synchronize()
    start.record()
    for _ in range(iters):
        fn()
    stop.record()
    stop.synchronize()
    return start.elapsed_time(stop) / iters


def _graph_ms(fn, iters, batch=10):
    """Average duration (ms) of ``fn`` from replays of a HIP graph holding ``batch`` calls: for
    kernels of a few tens of microseconds, which the Python path cannot issue back to back.
    (Timing only: results are checked in eager mode.)"""
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        for _ in range(3):
            fn()
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        for _ in range(batch):
            fn()
    graph.replay()
    reps = max(2, iters // batch)
    return _events_ms(graph.replay, reps) / batch


def _outlier_randn(shape, seed, frac=0.001, mul=100.0):
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(shape, generator=g, dtype=torch.float32)
    g2 = torch.Generator().manual_seed(seed + 1)
    n = max(1, int(x.numel() * frac))
    idx = torch.randperm(x.numel(), generator=g2)[:n]
    x.view(-1)[idx] *= mul
    return x.to(torch.bfloat16)


# ---------------------------------------------------------------------------------------
# workloads
# ---------------------------------------------------------------------------------------
class QuantTensorwise:
    """BASELINE config 0: E4M3 tensorwise quantize + dequantize of a 4096x4096 bf16 tensor."""

    name = "fp8_e4m3_tensorwise_quant_dequant_4096x4096_bf16"
    metric = "quantize+dequantize GB/s (algorithmic bytes)"
    unit = "GB/s"
    dtype = "f32"
    bound = "hbm"
    # rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE of the fused kernel, scaled by a 256 MiB copy in the same
    # run: 32.2 MiB fetched + 16.0 MiB written (the summary is under profiles/)
    traffic = int(48.2 * 1024 * 1024)

    def __init__(self, dev):
        import primus_turbo.pytorch as turbo
        from primus_turbo.pytorch.core.low_precision import ScalingGranularity as G

        self.turbo, self.G = turbo, G
        self.x_cpu = _outlier_randn((4096, 4096), 0)
        self.x = self.x_cpu.to(dev)
        self.n = self.x.numel()
        self.q, self.sinv = turbo.ops.quantize_fp8(self.x, turbo.float8_e4m3, G.TENSORWISE)
        # 20 copies of the 32 MiB input (640 MiB): rotating through them keeps the reads in HBM
        self._ring = [self.x] + [self.x.clone() for _ in range(19)]
        self._pos = 0

    def rotate(self):
        self._pos = (self._pos + 1) % len(self._ring)
        self.x = self._ring[self._pos]

    # bytes: quant reads 2 B + writes 1 B per element, dequant reads 1 B + writes 2 B
    def step_work(self):
        return 6.0 * self.n

    def step(self):
        q, sinv = self.turbo.ops.quantize_fp8(self.x, self.turbo.float8_e4m3, self.G.TENSORWISE)
        return self.turbo.ops.dequantize_fp8(q, torch.bfloat16, self.G.TENSORWISE, scale_inv=sinv)

    dominant_name = "quant_tensorwise_kernel (fused amax + scale + cast)"

    def dominant(self):
        """One launch of the fused kernel through the C entry point with preallocated outputs: the
        kernel runs ~13 us, less than the op's Python path takes to issue it."""
        from primus_turbo import _native as N

        if not hasattr(self, "_dom"):
            lib = N.lib()
            out = torch.empty_like(self.x, dtype=torch.float8_e4m3fn)
            sinv = torch.empty((), dtype=torch.float32, device=self.x.device)
            self._dom = (lib.pt_quantize_fp8_tensorwise_static, out, sinv)
        fn, out, sinv = self._dom
        N.check(fn(N.ptr(self.x), N.dtype_code(self.x.dtype), self.x.numel(), N.ptr(out), N.dtype_code(out.dtype),
                   None, N.ptr(sinv), None, N.stream_of(self.x)))
        return out

    def dominant_work(self):
        return 3.0 * self.n  # bytes per launch

    def check(self):
        import numpy as np

        from oracle import quantize as Q

        oq, osinv = Q.fp8_tensorwise(self.x_cpu.float().numpy(), "e4m3")
        same = np.array_equal(self.q.cpu().view(torch.uint8).numpy(), oq)
        same = same and self.sinv.cpu().view(torch.int32).item() == osinv.view(np.int32).item()
        return bool(same), "bytes and scale_inv bit-exact vs oracle"

    def cpu_baseline(self):
        from oracle import cpu_reference as R

        x = self.x_cpu
        R.quantize_fp8_tensorwise_ref(x, torch.float8_e4m3fn)  # warm-up
        times = []
        t_end = time.perf_counter() + 10.0
        while len(times) < 5 or (time.perf_counter() < t_end and len(times) < 40):
            t0 = time.perf_counter()
            q, _, sinv = R.quantize_fp8_tensorwise_ref(x, torch.float8_e4m3fn)
            R.dequantize_fp8_ref(q, torch.bfloat16, sinv)
            times.append(time.perf_counter() - t0)
        med = sorted(times)[len(times) // 2]
        return dict(
            value=6.0 * self.n / med / 1e9,
            unit="GB/s",
            cores=torch.get_num_threads(),
            kind="port",
            sample=f"full 4096x4096 quantize+dequantize, median of {len(times)} runs, "
            f"{os.cpu_count()} logical CPUs visible",
        )


class QuantTensorwiseLarge(QuantTensorwise):
    """The same quantizer on a 16384 x 16384 bf16 tensor (512 MiB): its rate away from the launch
    ramp of the 32 MiB case. The fused kernel parks 32 MiB in registers across the grid exchange
    and reads the rest a second time, so it moves 5 bytes per element for 3 algorithmic ones."""

    name = "fp8_e4m3_tensorwise_quant_dequant_16384x16384_bf16"
    traffic = None

    def __init__(self, dev, side=16384):
        import primus_turbo.pytorch as turbo
        from primus_turbo.pytorch.core.low_precision import ScalingGranularity as G

        self.turbo, self.G = turbo, G
        g = torch.Generator().manual_seed(3)
        self.x_cpu = torch.randn((side, side), generator=g, dtype=torch.float32).to(torch.bfloat16)
        self.x_cpu.view(-1)[12345] = 300.0
        self.x = self.x_cpu.to(dev)
        self.n = self.x.numel()
        self.q, self.sinv = turbo.ops.quantize_fp8(self.x, turbo.float8_e4m3, G.TENSORWISE)
        self._ring = [self.x, self.x.clone()]
        self._pos = 0

    def check(self):
        import numpy as np

        from oracle import quantize as Q

        # the scale from the whole tensor's abs-max, the bytes of the first and last 256 rows
        amax = np.float32(self.x_cpu.abs().max().item())
        _, osinv = Q.fp8_tensorwise(np.array([amax], dtype=np.float32), "e4m3")
        same = self.sinv.cpu().view(torch.int32).item() == osinv.view(np.int32).item()
        scale = np.float32(448.0) / max(amax, np.float32(1e-12))
        for rows in (slice(0, 256), slice(-256, None)):
            oq, _ = Q.fp8_tensorwise(self.x_cpu[rows].float().numpy(), "e4m3", scale=scale)
            same = same and np.array_equal(self.q[rows].cpu().view(torch.uint8).numpy(), oq)
        return bool(same), "scale_inv and the bytes of the first and last 256 rows bit-exact vs oracle"

    def cpu_baseline(self):
        from oracle import cpu_reference as R

        x = self.x_cpu[:4096, :4096].contiguous()
        t0 = time.perf_counter()
        q, _, sinv = R.quantize_fp8_tensorwise_ref(x, torch.float8_e4m3fn)
        R.dequantize_fp8_ref(q, torch.bfloat16, sinv)
        dt = time.perf_counter() - t0
        return dict(value=6.0 * x.numel() / dt / 1e9, unit="GB/s", cores=torch.get_num_threads(), kind="port",
                    sample=f"a 4096x4096 corner, one run, {os.cpu_count()} logical CPUs visible")


WORKLOADS = {"quant_tensorwise": QuantTensorwise, "quant_tensorwise_16384": QuantTensorwiseLarge}
from bench_quant_workloads import register as _register_quant  # noqa: E402
from bench_workloads import register as _register  # noqa: E402

_register_quant(WORKLOADS)
_register(WORKLOADS)

DEFAULT_ORDER = ["gemm_fp8_blockwise_8192", "gemm_fp8_rowwise", "quant_tensorwise"]

# the other workloads of the configurations the path is quoted on, reported under "extra"
EXTRA_GEMM = ["gemm_fp8_rowwise", "gemm_fp8_blockwise", "gemm_fp8_blockwise_k7168", "grouped_gemm_fp8",
              "grouped_gemm_fp8_down", "gemm_mxfp4", "gemm_mxfp4_n28672", "gemm_mxfp8", "gemm_mxfp8_n28672",
              "grouped_gemm_mxfp8", "grouped_gemm_mxfp8_down", "grouped_gemm_mxfp4", "grouped_gemm_mxfp4_down"]
EXTRA_QUANT = ["hbm_stream", "swiglu_with_probs", "moe_permute", "quant_tensorwise", "quant_tensorwise_16384", "quant_rowwise", "quant_blockwise", "quant_blockwise_dual", "quant_blockwise_weight",
               "quant_grouped", "glu_quant_grouped", "glu_quant_grouped_mxfp8", "quant_mxfp8", "quant_mxfp8_dual", "quant_mxfp4", "quant_mxfp4_dual"]
EXTRA_BUDGET_S = 400.0  # no further extra workload is started after this many seconds of run time


def _median(xs):
    xs = sorted(xs)
    return xs[len(xs) // 2]


def _rotating(wl, fn):
    """``fn`` preceded by the workload's input rotation (HBM-bound workloads only)."""
    rot = getattr(wl, "rotate", None)
    if rot is None:
        return fn

    def call():
        rot()
        return fn()

    return call


def measure(wl, steps, warmup, windows):
    """-> (ms_per_step, value, roofline dict, parity dict); every time a median of ``windows``."""
    step = _rotating(wl, wl.step)
    dominant = _rotating(wl, wl.dominant)
    # Setup ends with the GPU busy: data generation ran on the host while the idle GPU dropped to
    # its low power state, and a handful of sub-millisecond warm-up steps is over before the clocks
    # are back up. (The parity check runs after the timed region for the same reason: its oracle
    # leg keeps the GPU idle.)
    t_spin = time.perf_counter()
    while time.perf_counter() - t_spin < 0.3:
        for _ in range(5):
            step()
        torch.cuda.synchronize()
    for _ in range(warmup):
        step()
    wins = []
    for _ in range(windows):
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(steps):
            step()
        torch.cuda.synchronize()
        wins.append((time.perf_counter() - t0) * 1e3 / steps)
    ms_per_step = _median(wins)
    scale = 1e12 if wl.unit == "TFLOP/s" else 1e9
    value = wl.step_work() / (ms_per_step * 1e-3) / scale

    # dominant kernel, HIP events on the launch stream
    for _ in range(max(3, warmup)):
        dominant()
    timer = _graph_ms if getattr(wl, "graph_dominant", False) else _events_ms
    dom_ms = _median([timer(dominant, max(steps, 20)) for _ in range(windows)])
    achieved = wl.dominant_work() / (dom_ms * 1e-3) / scale
    peak = {"hbm": HBM_PEAK_GBS, "mfma": getattr(wl, "peak", FP8_PEAK_TFLOPS)}[wl.bound]
    roofline = dict(
        bound=wl.bound,
        achieved=round(achieved, 2),
        peak=peak,
        unit="GB/s" if wl.bound == "hbm" else "TFLOP/s",
        frac=round(achieved / peak, 4),
        traffic=getattr(wl, "traffic", None),
        kernel=wl.dominant_name,
        kernel_ms=round(dom_ms, 5),
    )
    if getattr(wl, "rotate", None) is not None:
        roofline["inputs"] = "rotating through copies of the input (> 512 MB): reads come from HBM, not the Infinity Cache"
    kernels = getattr(wl, "kernels", None)
    if kernels is not None:  # further kernels of the step, each alone under HIP events
        per = {}
        for kname, fn, work in kernels():
            for _ in range(3):
                fn()
            kms = _median([_events_ms(fn, max(steps, 20)) for _ in range(windows)])
            per[kname] = dict(kernel_ms=round(kms, 5), achieved=round(work / (kms * 1e-3) / scale, 2),
                              frac=round(work / (kms * 1e-3) / scale / peak, 4))
        roofline["kernels"] = per
    ok, what = wl.check()
    return ms_per_step, value, roofline, dict(ok=ok, what=what)


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--windows", type=int, default=5, help="timed windows of --steps steps; the median is reported")
    ap.add_argument("--workload", default="auto", help="one of: auto, " + ", ".join(WORKLOADS))
    ap.add_argument("--extra", default=None, choices=["all", "gemm", "none"],
                    help="which other workloads to measure into 'extra' (default: all for the default workload, else none)")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--calib-copy", action="store_true",
                    help="also launch one plain elementwise copy of 256 MiB (fp32 x + 0 -> y): the known-size "
                    "kernel that HBM traffic counters of a profiled run are scaled by")
    args = ap.parse_args()
    t_start = time.perf_counter()

    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        print(
            "bench.py: this build measures the one-GPU hot path only; run it with --gpus 1 "
            "(no collectives or sharding are part of it).",
            file=sys.stderr,
        )
        sys.exit(2)
    if not torch.cuda.is_available():
        print("bench.py: no GPU visible; the hot path has no CPU fallback.", file=sys.stderr)
        sys.exit(3)

    name = args.workload
    extra_mode = args.extra or ("all" if name == "auto" else "none")
    if name == "auto":
        name = next(w for w in DEFAULT_ORDER if w in WORKLOADS)
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    wl = WORKLOADS[name](dev)

    if args.calib_copy:
        src = torch.ones(64 << 20, dtype=torch.float32, device=dev)
        dst = torch.empty_like(src)
        torch.add(src, 0.0, out=dst)
        torch.cuda.synchronize()
        del src, dst

    ms_per_step, value, roofline, parity = measure(wl, args.steps, args.warmup, args.windows)
    out = dict(
        metric=wl.metric,
        value=round(value, 2),
        unit=wl.unit,
        n_gpus=1,
        steps=args.steps,
        warmup=args.warmup,
        windows=args.windows,
        ms_per_step=round(ms_per_step, 5),
        higher_is_better=True,
        scaling="weak",
        vs_baseline=None,
        dtype=wl.dtype,
        data="synthetic",
        config=dict(workload=wl.name),
        parity=parity,
        roofline=roofline,
    )
    if not args.no_cpu:
        out["cpu_baseline"] = wl.cpu_baseline()
    del wl
    torch.cuda.empty_cache()

    if extra_mode != "none":
        keys = [k for k in EXTRA_GEMM + (EXTRA_QUANT if extra_mode == "all" else []) if k in WORKLOADS and k != name]
        extra = {}
        for key in keys:
            if time.perf_counter() - t_start > EXTRA_BUDGET_S:
                extra[key] = dict(skipped="time budget of the run spent")
                continue
            w = WORKLOADS[key](dev)
            ms, val, roof, par = measure(w, max(10, args.steps // 2), max(3, args.warmup // 2), args.windows)
            rec = dict(workload=w.name, ms=round(ms, 5), value=round(val, 2), unit=w.unit, bound=roof["bound"],
                       frac=roof["frac"], achieved=roof["achieved"], kernel_ms=roof["kernel_ms"], parity_ok=par["ok"])
            if "kernels" in roof:
                rec["kernels"] = roof["kernels"]
            extra[key] = rec
            del w
            torch.cuda.empty_cache()
        out["extra"] = extra
    out["run_seconds"] = round(time.perf_counter() - t_start, 1)
    print(json.dumps(out))


if __name__ == "__main__":
    main()
