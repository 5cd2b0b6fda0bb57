"""What each part of the DSD step loop costs: the forward product timed on builds of the GEMM kernels with the tile
loads, the fragment reads or the MFMAs compiled out (SD_TIMING_* in csrc/gemm_fast.hip; their results are wrong by
construction, only their time means anything).

    python -m benchmark.decompose [--size 8192] [--p 0 0.5] [--zero-data]

Everything is compiled here (hipcc, a minute or two, in parallel) into a temporary directory: the library's other
sources once, csrc/gemm_fast.hip once per variant.  One child process per variant loads its library and prints
microseconds per launch (median, L2 flushed before each call, after a warm-up pass over every p)."""
from __future__ import annotations

import argparse
import subprocess
import sys
import tempfile
from concurrent.futures import ThreadPoolExecutor
from pathlib import Path

PKG = Path(__file__).resolve().parent.parent
CSRC = PKG / "csrc"
VARIANTS = {
    "everything": [],
    "no tile loads": ["-DSD_TIMING_NO_LOADS"],
    "no fragment reads": ["-DSD_TIMING_NO_READS"],
    "no loads, no reads": ["-DSD_TIMING_NO_LOADS", "-DSD_TIMING_NO_READS"],
    "no MFMAs": ["-DSD_TIMING_NO_MFMA"],
}

CHILD = r"""
import sys, statistics, torch
from pathlib import Path
sys.path.insert(0, sys.argv[1])
from flash_dropout.hip import _loader
_loader.LIB_PATH = Path(sys.argv[2])
from flash_dropout.hip import GEMM
ext = GEMM()
size, zero = int(sys.argv[3]), sys.argv[4] == "1"
ps = [float(v) for v in sys.argv[5:]]
g = torch.Generator(device="cuda").manual_seed(0)
A = torch.randn(size, size, device="cuda", dtype=torch.float16, generator=g)
B = torch.randn(size, size, device="cuda", dtype=torch.float16, generator=g) * size ** -0.5
if zero:
    A.zero_(); B.zero_()
y = torch.empty(size, size, device="cuda", dtype=torch.float16)
flush = torch.empty(512 << 20, dtype=torch.int8, device="cuda")
lists = {p: ext.build_lists(torch.rand(size // 64, size // 64, device="cuda", generator=g) < p) for p in ps}
def med(p, n):
    ts = []
    for _ in range(n):
        flush.zero_()
        a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        a.record(); ext.gemm_dsd_lists(A, B, lists[p], 64, 1.0 / (1.0 - p), out=y); b.record()
        torch.cuda.synchronize()
        ts.append(a.elapsed_time(b))
    return statistics.median(ts) * 1e3
for p in ps: med(p, 15)
print(" ".join(f"p={p}: {med(p, 15):.0f} us" for p in ps))
"""


sys.path.insert(0, str(CSRC))
import build as libbuild  # noqa: E402  (csrc/build.py: compiler, flags, source list)


def compile_one(src: Path, obj: Path, flags: list[str]) -> Path:
    subprocess.run([libbuild.HIPCC, *libbuild.FLAGS, *flags, "-c", str(src), "-o", str(obj)], check=True,
                   stderr=subprocess.DEVNULL)
    return obj


def main() -> None:
    ap = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    ap.add_argument("--size", type=int, default=8192)
    ap.add_argument("--p", type=float, nargs="+", default=[0.0, 0.5])
    ap.add_argument("--zero-data", action="store_true")
    args = ap.parse_args()
    libbuild.write_source_hash()
    with tempfile.TemporaryDirectory() as tmp:
        tmp = Path(tmp)
        jobs = [(s, tmp / (s.stem + ".o"), []) for s in libbuild.sources() if s.name != "gemm_fast.hip"]
        jobs += [(CSRC / "gemm_fast.hip", tmp / f"gemm_fast_{i}.o", flags) for i, flags in enumerate(VARIANTS.values())]
        with ThreadPoolExecutor(8) as pool:
            objs = list(pool.map(lambda j: compile_one(*j), jobs))
        shared, per_variant = objs[:-len(VARIANTS)], objs[-len(VARIANTS):]
        libs = {}
        for name, obj in zip(VARIANTS, per_variant):
            libs[name] = obj.with_suffix(".so")
            subprocess.run([libbuild.HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", str(libs[name]), str(obj),
                            *map(str, shared)], check=True)
        print(f"forward product Y = s (keep . X) W^T, M=N=K={args.size} fp16, {'all-zero' if args.zero_data else 'N(0,1)'} operands")
        for name, lib in libs.items():
            out = subprocess.run([sys.executable, "-c", CHILD, str(PKG), str(lib), str(args.size),
                                  "1" if args.zero_data else "0", *map(str, args.p)],
                                 capture_output=True, text=True, timeout=300)
            print(f"{name:22s} {out.stdout.strip() or out.stderr.strip()[-300:]}", flush=True)


if __name__ == "__main__":
    main()
