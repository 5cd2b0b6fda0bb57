#!/usr/bin/env python
"""Headline benchmark: forward+backward of the block-dropout matmul at M=N=K=8192 fp16, 64x64 blocks.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--size 8192] [--p 0.5] [--no-sweep] [--no-cpu]

One "step" is one pass of the hot path over one batch of synthetic input already resident in HBM:
kept-block list build, DSD forward Y, SDD backward dX, DSD backward dW (the three launches the
reference's autograd function issues, flash_dropout/functional/blockwise_dropout_matmul_cuda.py:26,46,49).
Prints ONE JSON line.  `value` is the effective dense-equivalent rate 6*M*N*K / t at p = 0.5; the same line
carries the p-sweep (0, 0.25, 0.5, 0.75) with kept-work rates (the reference's FLOP convention,
benchmark/full.py:160-163: 2MNK forward + 4MNK backward, times the kept fraction), the t(p=.5)/t(p=0)
ratio, a roofline object for the dominant kernel (HIP-event timed per launch) and the CPU baseline.
"""
from __future__ import annotations

import argparse
import json
import os
import statistics
import sys
import time
from pathlib import Path

ROOT = Path(__file__).resolve().parent
for _p in (ROOT, ROOT / "sparse-dropout_amd"):
    if str(_p) not in sys.path:
        sys.path.insert(0, str(_p))

PEAK_FP16_TFLOPS = 2500.0  # MI355X dense fp16 MFMA peak

# HBM/fabric bytes per launch of the three GEMM kernels at the headline workload (M=N=K=8192, p=0.5) are not
# measured by this process (a counter run cannot be made from inside it): they are read from the stored summary of
# the rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE runs of this same command, profiles/bench_8192_p50_pmc.txt (its
# "traffic_json:" line), which names the commit it was taken at; the JSON line says so next to the figure.
TRAFFIC_FILE = ROOT / "profiles" / "bench_8192_p50_pmc.txt"


def stored_traffic(kernel: str):
    """(bytes per launch, provenance) of `kernel` from the stored counter summary, or (None, None)."""
    try:
        line = next(l for l in TRAFFIC_FILE.read_text().splitlines() if l.startswith("traffic_json:"))
        doc = json.loads(line[len("traffic_json:"):])
        entry = doc["kernels"][kernel]
        return int(entry["fetch_bytes"] + entry["write_bytes"]), {
            "file": str(TRAFFIC_FILE.relative_to(ROOT)), "taken_at_commit": doc.get("commit"),
            "read_factor": doc.get("read_factor"), "write_factor": doc.get("write_factor")}
    except (OSError, KeyError, ValueError, StopIteration):
        return None, None


METRIC = "fwd+bwd ms & effective TFLOP/s vs p (0–0.75) at 8192³ fp16; % of MFMA peak"


LD_PAD = 0  # extra elements in every leading dimension (--ld-pad; 0 = dense row-major tensors)


def _padded(t, dev):
    import torch

    if LD_PAD == 0:
        return t.to(dev)
    buf = torch.empty(t.shape[0], t.shape[1] + LD_PAD, dtype=t.dtype, device=dev)
    view = buf[:, : t.shape[1]]
    view.copy_(t)
    return view


ZERO_DATA = False  # --zero-data: all-zero operands (same instructions and traffic, no switching activity in the multipliers)


def make_problem(size: int, p: float, bs: int, seed: int = 0):
    import torch

    gen = torch.Generator().manual_seed(seed)
    M = N = K = size
    dev = torch.device("cuda:0")
    x = _padded(torch.randn(M, K, generator=gen).half(), dev)
    w = _padded((torch.randn(N, K, generator=gen) / K ** 0.5).half(), dev)
    dy = _padded(torch.randn(M, N, generator=gen).half(), dev)
    if ZERO_DATA:
        for t in (x, w, dy):
            t.zero_()
    mask = (torch.rand(M // bs, K // bs, generator=gen) < p).to(dev)  # CPU generator: device independent
    return x, w, dy, mask


class Step:
    """The hot path with preallocated outputs, called through the C-ABI shim."""

    def __init__(self, x, w, dy, mask, bs, p):
        import torch

        from flash_dropout.hip import GEMM

        self.ext = GEMM()
        self.x, self.w, self.dy, self.mask, self.bs = x, w, dy, mask, bs
        self.scale = 1.0 / (1.0 - p)
        M, K = x.shape
        N = w.shape[0]
        self.y = torch.empty(M, N + LD_PAD, dtype=x.dtype, device=x.device)[:, :N]
        self.dx = torch.empty(M, K + LD_PAD, dtype=x.dtype, device=x.device)[:, :K]
        self.dw_t = torch.empty(N, K + LD_PAD, dtype=x.dtype, device=x.device)[:, :K].t()  # [K, N] view of [N, K]
        self.lists = self.ext.build_lists(mask)
        kept = int((~mask).sum().item())
        self.kept_area = kept * bs * bs
        self.flops_fwd = 2.0 * self.kept_area * N
        self.flops_total = 6.0 * self.kept_area * N
        self.flops_dense = 6.0 * M * N * K

    def build(self):
        self.lists = self.ext.build_lists(self.mask)

    def fwd(self):
        self.ext.gemm_dsd_lists(self.x, self.w, self.lists, self.bs, self.scale, out=self.y)

    def dx_(self):
        self.ext.gemm_sdd_lists(self.dy, self.w.t(), self.lists, self.bs, self.scale, out=self.dx)

    def dw_(self):
        self.ext.gemm_dsd_lists(self.x.t(), self.dy.t(), self.lists.transposed(), self.bs, self.scale,
                                out=self.dw_t)

    def __call__(self):
        self.build()
        self.fwd()
        self.dx_()
        self.dw_()


def time_steps(step, steps: int, warmup: int) -> float:
    import torch

    for _ in range(warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        step()
    torch.cuda.synchronize()
    return (time.perf_counter() - t0) * 1e3 / steps


def time_kernel_events(fn, reps: int, flush=None) -> float:
    """Average launch duration in ms, HIP events on the launch stream, one pair per launch."""
    import torch

    ev = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(reps)]
    for a, b in ev:
        if flush is not None:
            flush.zero_()
        a.record()
        fn()
        b.record()
    torch.cuda.synchronize()
    return statistics.fmean(a.elapsed_time(b) for a, b in ev)


def looped_with_clock(fn, seconds: float = 2.5):
    """fn launched back to back for `seconds`; rocm-smi polled from a thread meanwhile.  Returns microseconds per
    launch, the median shader clock seen and, from the two, shader cycles per launch."""
    import re
    import subprocess
    import threading
    import time

    import torch

    clocks = []

    def poll():
        time.sleep(0.7)
        for _ in range(3):
            out = subprocess.run(["rocm-smi", "--showclocks"], capture_output=True, text=True).stdout
            m = re.search(r"sclk clock level: \d+: \((\d+)Mhz\)", out)
            if m:
                clocks.append(int(m.group(1)))
            time.sleep(0.3)

    for _ in range(20):
        fn()
    torch.cuda.synchronize()
    th = threading.Thread(target=poll)
    th.start()
    a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    n, t0 = 0, time.time()
    a.record()
    while time.time() - t0 < seconds or th.is_alive():
        for _ in range(50):
            fn()
        n += 50
        torch.cuda.synchronize()
    b.record()
    torch.cuda.synchronize()
    th.join()
    us = a.elapsed_time(b) * 1e3 / n
    mhz = statistics.median(clocks) if clocks else None
    return {"us_per_launch": round(us, 1), "sclk_mhz": mhz,
            "kilocycles_per_launch": round(us * mhz / 1e3, 1) if mhz else None}


def cpu_baseline(size: int, bs: int, p: float, reps: int):
    """The oracle's literal naive path (mask expand + dense linear + autograd backward) on the host
    cores, fp32, same kind of workload at a bounded size."""
    import torch

    from oracle import naive_torch

    gen = torch.Generator().manual_seed(0)
    x = torch.randn(size, size, generator=gen)
    w = torch.randn(size, size, generator=gen) / size ** 0.5
    dy = torch.randn(size, size, generator=gen)
    mask = torch.rand(size // bs, size // bs, generator=gen) < p
    naive_torch.forward_backward(x, w, dy, mask, bs, p)
    ts = []
    for _ in range(reps):
        t0 = time.perf_counter()
        naive_torch.forward_backward(x, w, dy, mask, bs, p)
        ts.append(time.perf_counter() - t0)
    t = statistics.median(ts)
    # per-core figure: the same path on one thread at a size that keeps it to a few seconds
    threads = torch.get_num_threads()
    small = min(size, 2048)
    xs, ws, dys = x[:small, :small].contiguous(), w[:small, :small].contiguous(), dy[:small, :small].contiguous()
    ms_ = mask[: small // bs, : small // bs].contiguous()
    torch.set_num_threads(1)
    try:
        naive_torch.forward_backward(xs, ws, dys, ms_, bs, p)
        t1s = []
        for _ in range(3):
            t0 = time.perf_counter()
            naive_torch.forward_backward(xs, ws, dys, ms_, bs, p)
            t1s.append(time.perf_counter() - t0)
    finally:
        torch.set_num_threads(threads)
    t1 = statistics.median(t1s)
    # the reference's own CPU-runnable case: 1024^3, median of 20 repetitions after 3 warm-ups, all threads
    c1 = min(size, 1024)
    xc, wc, dyc = x[:c1, :c1].contiguous(), w[:c1, :c1].contiguous(), dy[:c1, :c1].contiguous()
    mc = mask[: c1 // bs, : c1 // bs].contiguous()
    for _ in range(3):
        naive_torch.forward_backward(xc, wc, dyc, mc, bs, p)
    tcs = []
    for _ in range(20):
        t0 = time.perf_counter()
        naive_torch.forward_backward(xc, wc, dyc, mc, bs, p)
        tcs.append(time.perf_counter() - t0)
    tc = statistics.median(tcs)
    return {
        "small_case": {"value": round(6.0 * c1 ** 3 / tc / 1e12, 4), "unit": "TFLOP/s", "cores": threads,
                       "sample": f"same path at M=N=K={c1}, median of 20 reps after 3 warm-ups ({tc * 1e3:.2f} ms each)"},
        "one_core": {"value": round(6.0 * small ** 3 / t1 / 1e12, 4), "unit": "TFLOP/s", "cores": 1,
                     "sample": f"same path, torch.set_num_threads(1), M=N=K={small}, median of 3 reps ({t1 * 1e3:.1f} ms each)"},
        "value": round(6.0 * size ** 3 / t / 1e12, 4),
        "unit": "TFLOP/s",
        "cores": threads,
        "kind": "port",
        "sample": f"oracle/naive_torch.py fwd+bwd fp32 at M=N=K={size}, bs={bs}, p={p}, median of {reps} reps "
                  f"({t * 1e3:.1f} ms each; host has {os.cpu_count()} logical cpus); dense-equivalent 6MNK/t",
        "ms": round(t * 1e3, 2),
    }


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--size", type=int, default=8192)
    ap.add_argument("--p", type=float, default=0.5)
    ap.add_argument("--block-size", type=int, default=64)
    ap.add_argument("--no-sweep", action="store_true")
    ap.add_argument("--no-cpu", action="store_true")
    ap.add_argument("--cpu-size", type=int, default=8192)
    ap.add_argument("--copy-calibration", action="store_true",
                    help="also run a plain 128 MiB device copy 3 times (known traffic, for scaling rocprof's FETCH_SIZE / WRITE_SIZE)")
    ap.add_argument("--dense-reference", action="store_true",
                    help="also time the dense products on the same tensors: torch.matmul (hipBLASLt) and this library's sd_gemm")
    ap.add_argument("--zero-data", action="store_true",
                    help="all-zero operands: what the kernels do when the chip's power limit is out of the picture")
    ap.add_argument("--ld-pad", type=int, default=0,
                    help="pad every leading dimension by this many elements (experiment: power-of-two row strides)")
    args = ap.parse_args()
    global LD_PAD, ZERO_DATA
    LD_PAD = args.ld_pad
    ZERO_DATA = args.zero_data
    if args.gpus != 1:
        print("bench.py: this build runs on one GPU; --gpus N with N > 1 is not supported "
              "(the path has no collectives: row blocks would shard over GPUs with one reduction for dW)", file=sys.stderr)
        return 2

    import torch

    import __graft_entry__ as entry

    entry.ensure_built()
    assert torch.cuda.is_available(), "bench.py needs a GPU"
    size, bs = args.size, args.block_size

    if args.copy_calibration:
        src = torch.empty(64 << 20, dtype=torch.float16, device="cuda").normal_()
        dst = torch.empty_like(src)
        for _ in range(3):
            dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst

    # ---- headline: K timed steps at p -----------------------------------------------------
    step = Step(*make_problem(size, args.p, bs), bs, args.p)
    ms = time_steps(step, args.steps, args.warmup)
    value = step.flops_dense / (ms * 1e-3) / 1e12
    kept_tflops = step.flops_total / (ms * 1e-3) / 1e12

    # ---- per-kernel launch durations (HIP events on the launch stream) ---------------------
    reps = max(5, min(args.steps, 20))
    kern_ms = {
        "build_lists": time_kernel_events(step.build, reps),
        "dsd_forward": time_kernel_events(step.fwd, reps),
        "sdd_dx": time_kernel_events(step.dx_, reps),
        "dsd_dw": time_kernel_events(step.dw_, reps),
    }
    dominant = max(("dsd_forward", "sdd_dx", "dsd_dw"), key=lambda k: kern_ms[k])
    achieved = step.flops_fwd / (kern_ms[dominant] * 1e-3) / 1e12  # each GEMM does 2*kept_area*N flops
    headline = size == 8192 and args.p == 0.5 and bs == 64 and LD_PAD == 0 and not ZERO_DATA
    traffic, traffic_source = stored_traffic(dominant) if headline else (None, None)
    roofline = {
        "bound": "mfma",
        "kernel": dominant,
        "achieved": round(achieved, 2),
        "peak": PEAK_FP16_TFLOPS,
        "unit": "TFLOP/s",
        "frac": round(achieved / PEAK_FP16_TFLOPS, 4),
        "traffic": traffic,
        "traffic_unit": "bytes per launch (HBM/fabric reads + writes); not measured by this run: stored rocprofv3 "
                        "FETCH_SIZE/WRITE_SIZE figures of the same command, see traffic_source",
        "traffic_source": traffic_source,
        "flops_per_launch": step.flops_fwd,
        "avg_launch_ms": round(kern_ms[dominant], 4),
        "all_kernels_ms": {k: round(v, 4) for k, v in kern_ms.items()},
        "all_kernels_tflops": {k: round(step.flops_fwd / (kern_ms[k] * 1e-3) / 1e12, 2)
                               for k in ("dsd_forward", "sdd_dx", "dsd_dw")},
    }

    # ---- p sweep (reference protocol: L2-sized buffer zeroed before each call, median) ------
    sweep = []
    ratio = None
    if not args.no_sweep:
        flush = torch.empty(512 << 20, dtype=torch.int8, device="cuda")  # > L2 + MALL
        t_by_p = {}
        sweep_steps = {p: Step(*make_problem(size, p, bs), bs, p) for p in (0.0, 0.25, 0.5, 0.75)}

        def flushed_median(st, n):
            ts = []
            for _ in range(n):
                flush.zero_()
                a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                a.record()
                st()
                b.record()
                torch.cuda.synchronize()
                ts.append(a.elapsed_time(b))
            return statistics.median(ts)

        # One untimed pass over every p first: under this flush-and-synchronise protocol the first second or so
        # of measurements comes out 10-15 % slow whatever is measured, which would flatter whichever p goes later.
        for st in sweep_steps.values():
            for _ in range(3):
                st()
            flushed_median(st, 5)
        for p, st in sweep_steps.items():
            t = flushed_median(st, max(5, args.steps // 2))
            t_by_p[p] = t
            sweep.append({
                "p": p,
                "kept_fraction": round(st.kept_area / (size * size), 4),
                "fwd_bwd_ms": round(t, 4),
                "kept_work_tflops": round(st.flops_total / (t * 1e-3) / 1e12, 2),
                "dense_equiv_tflops": round(st.flops_dense / (t * 1e-3) / 1e12, 2),
                "pct_mfma_peak_kept_work": round(100 * st.flops_total / (t * 1e-3) / 1e12 / PEAK_FP16_TFLOPS, 2),
            })
        ratio = round(t_by_p[0.5] / t_by_p[0.0], 4)
        del flush, sweep_steps

    dense_reference = None
    if args.dense_reference:
        flush = torch.empty(512 << 20, dtype=torch.int8, device="cuda")
        x, w, dy = step.x, step.w, step.dy
        y = torch.empty_like(step.y)
        for _ in range(3):  # library heuristics and kernel loading happen on the first calls
            torch.matmul(x, w.t(), out=y)
            step.ext.gemm(x, w, out=y)
            step.ext.gemm(dy, w.t(), out=step.dx)
        torch.cuda.synchronize()
        dense_reference = {
            "workload": f"one dense product Y = X.W^T at M=N=K={size} on the benchmark's tensors, L2 flushed before each call, "
                        "HIP-event average",
            "torch_matmul_ms": round(time_kernel_events(lambda: torch.matmul(x, w.t(), out=y), reps, flush), 4),
            "sd_gemm_ms": round(time_kernel_events(lambda: step.ext.gemm(x, w, out=y), reps, flush), 4),
            "sd_gemm_dx_layout_ms": round(time_kernel_events(lambda: step.ext.gemm(dy, w.t(), out=step.dx), reps, flush), 4),
            # the same three in a tight loop (no flush) with the shader clock read beside them: the products run the
            # chip into its power limit to different degrees, so milliseconds alone do not compare the kernels
            "looped": {
                "torch_matmul": looped_with_clock(lambda: torch.matmul(x, w.t(), out=y)),
                "sd_gemm": looped_with_clock(lambda: step.ext.gemm(x, w, out=y)),
                "sd_forward_p": looped_with_clock(step.fwd),
            },
        }
        del flush

    out = {
        "metric": METRIC,
        "value": round(value, 2),
        "unit": "TFLOP/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(ms, 4),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f16",
        "data": "synthetic",
        "config": {
            "workload": f"square GEMM sweep M=N=K={size} fp16, 64x64 block mask, fwd DSD + bwd SDD/DSD "
                        f"(list build included), value at p={args.p}",
            "M": size, "N": size, "K": size, "block_size": bs, "p": args.p,
            "value_definition": "dense-equivalent 6*M*N*K / t",
        },
        "kept_work_tflops": round(kept_tflops, 2),
        "pct_mfma_peak_kept_work": round(100 * kept_tflops / PEAK_FP16_TFLOPS, 2),
        "ratio_t_p50_over_t_p0": ratio,
        "sweep": sweep,
        "roofline": roofline,
    }
    if ZERO_DATA:
        out["data"] = "synthetic, all-zero operands (--zero-data)"
    if dense_reference is not None:
        out["dense_reference"] = dense_reference
    if not args.no_cpu:
        out["cpu_baseline"] = cpu_baseline(args.cpu_size, bs, args.p, reps=4)
    print(json.dumps(out))
    return 0


if __name__ == "__main__":
    sys.exit(main())
