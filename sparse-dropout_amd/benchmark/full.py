"""Forward + backward of one dropout-matmul as the drop rate varies (reference: benchmark/full.py).

    python -m benchmark.full --size 8192 --block-size 64 --p 0 0.25 0.5 0.75

Methods: torch dense linear; element dropout + dense ("Dropout + Dense"); the library's dense GEMM;
SparseDrop (mask draw + list build + DSD forward, SDD dX, DSD dW).  TFLOP/s is dense-equivalent
(6*M*N*K / time), the convention of benchmark/full.py:160-163 applied to the whole problem."""
from __future__ import annotations

import argparse

import torch

import flash_dropout.functional as F
from flash_dropout.hip import GEMM

from .utils import Benchmarker, make_tensor, print_table


def f_dense(A, B, dC):
    C = torch.nn.functional.linear(A, B)
    yield "forward"
    C.backward(dC)
    yield "backward"


def f_baseline(A, B, dC, p):
    C = F.vanilla_dropout_matmul(A, B, p)
    yield "forward"
    C.backward(dC)
    yield "backward"


def f_dense_hip(A, B, dC):
    ext = GEMM()
    with torch.no_grad():
        ext.gemm(A, B)
        yield "forward"
        ext.gemm(dC, B.T)
        ext.gemm(A.T, dC.T, transposed_out=True)
        yield "backward"


def f_sparsedrop(A, B, dC, block_size, p):
    C = F.hip_blockwise_dropout_matmul(A, B, block_size, p)
    yield "forward"
    C.backward(dC)
    yield "backward"


def main() -> None:
    ap = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    ap.add_argument("--size", type=int, nargs="+", default=[8192], help="M = N = K, or M N K")
    ap.add_argument("--block-size", type=int, default=64)
    ap.add_argument("--p", type=float, nargs="+", default=[0.0, 0.25, 0.5, 0.75])
    ap.add_argument("--duration", type=float, default=1.0, help="seconds of timed repetitions per drop rate")
    ap.add_argument("--dtype", choices=["float16", "bfloat16"], default="float16")
    args = ap.parse_args()
    M, N, K = args.size * 3 if len(args.size) == 1 else args.size
    dtype = getattr(torch, args.dtype)
    torch.manual_seed(0)
    A = make_tensor(M, K, dtype=dtype)
    B = make_tensor(N, K, dtype=dtype, scale=K ** -0.5)
    dC = make_tensor(M, N, dtype=dtype, requires_grad=False)
    dense_flops = 6.0 * M * N * K
    print(f"M={M} N={N} K={K} block_size={args.block_size} dtype={args.dtype}")
    for p in args.p:
        fns = {
            "Dense (torch)": lambda: f_dense(A, B, dC),
            "Dropout + Dense": lambda: f_baseline(A, B, dC, p),
            "Dense (HIP)": lambda: f_dense_hip(A, B, dC),
            "SparseDrop (HIP)": lambda: f_sparsedrop(A, B, dC, args.block_size, p),
        }
        bench = Benchmarker(fns, duration=args.duration)
        bench.run()
        print(f"--- p = {p}")
        print_table(bench.results(), lambda r: (f"{dense_flops / r['median_ms'] / 1e9:8.1f} TFLOP/s dense-equivalent"
                                                if r["breakpoint"] == "total" else ""))
        A.grad = B.grad = None


if __name__ == "__main__":
    main()
