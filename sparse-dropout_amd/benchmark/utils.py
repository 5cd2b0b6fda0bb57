"""Event-timed comparison of several methods with named breakpoints.

Protocol of the reference's harness (benchmark/utils.py:40-113): a method is a generator function
that yields a breakpoint name after each phase ("forward", "backward"); every phase is bracketed by
device events; the last-level cache is flushed by zeroing a buffer before each method; methods are
interleaved round-robin for a fixed wall-clock duration after warm-up."""
from __future__ import annotations

import statistics
import time
from collections import defaultdict
from typing import Callable, Iterator

import torch

BenchmarkFn = Callable[[], Iterator[str]]
FLUSH_BYTES = 512 << 20  # larger than L2 (32 MiB) + memory-side cache (256 MiB)


def make_tensor(*size: int, row_major: bool = True, requires_grad: bool = True, dtype=torch.float16,
                scale: float = 1.0) -> torch.Tensor:
    """N(0, scale^2) operand on the GPU, row-major or (as a transposed view) column-major
    (reference: benchmark/utils.py:12-20)."""
    shape = size if row_major else size[::-1]
    t = (torch.randn(shape, device="cuda") * scale).to(dtype)
    t = t if row_major else t.T
    return t.requires_grad_(requires_grad)


class Benchmarker:
    def __init__(self, fns: dict[str, BenchmarkFn], warmup_reps: int = 3, duration: float = 1.0,
                 flush: bool = True) -> None:
        self.fns = fns
        self.warmup_reps = warmup_reps
        self.duration = duration
        self.cache = torch.empty(FLUSH_BYTES, dtype=torch.int8, device="cuda") if flush else None
        self.timings: dict[str, dict[str, list[float]]] = {name: defaultdict(list) for name in fns}

    def _flush(self) -> None:
        if self.cache is not None:
            self.cache.zero_()

    def _once(self, record: bool) -> None:
        pending = []
        for name, fn in self.fns.items():
            self._flush()
            it = iter(fn())
            while True:
                start = torch.cuda.Event(enable_timing=True)
                end = torch.cuda.Event(enable_timing=True)
                start.record()
                try:
                    breakpoint_name = next(it)
                except StopIteration:
                    break
                end.record()
                pending.append((name, breakpoint_name, start, end))
        torch.cuda.synchronize()
        if record:
            for name, bp, start, end in pending:
                self.timings[name][bp].append(start.elapsed_time(end))  # ms

    def run(self) -> int:
        for _ in range(self.warmup_reps):
            self._once(record=False)
        t0, count = time.time(), 0
        while time.time() - t0 < self.duration or count < 3:
            self._once(record=True)
            count += 1
        return count

    def results(self) -> list[dict]:
        rows = []
        for name, bps in self.timings.items():
            total = [sum(ts) for ts in zip(*bps.values())]
            for bp, ts in list(bps.items()) + [("total", total)]:
                rows.append({"method": name, "breakpoint": bp, "median_ms": statistics.median(ts),
                             "min_ms": min(ts), "n": len(ts)})
        return rows


def print_table(rows: list[dict], extra: Callable[[dict], str] | None = None) -> None:
    width = max(len(r["method"]) for r in rows)
    for r in rows:
        tail = f"  {extra(r)}" if extra else ""
        print(f"{r['method']:<{width}}  {r['breakpoint']:<9} median {r['median_ms']:8.4f} ms  "
              f"min {r['min_ms']:8.4f} ms  n={r['n']}{tail}")
