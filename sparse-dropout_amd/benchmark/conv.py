"""3x3 convolution forward + backward: torch's conv2d, the im2col + GEMM route, and block dropout on the
patch matrix (reference: benchmark/conv.py, which times the dense routes only).

    python -m benchmark.conv --n 128 --c 64 --k 128 --hw 32 --p 0 0.5"""
from __future__ import annotations

import argparse

import torch

import flash_dropout.functional as F

from .utils import Benchmarker, print_table


def f_torch(x, kern, dy, padding):
    y = torch.nn.functional.conv2d(x, kern, padding=padding)
    yield "forward"
    y.backward(dy)
    yield "backward"


def f_im2col(x, kern, dy, padding):
    y = F.im2col_conv2d(x, kern, padding=padding)
    yield "forward"
    y.backward(dy)
    yield "backward"


def f_blockdrop(x, kern, dy, padding, block_size, p):
    y = F.blockwise_dropout_conv2d(x, kern, block_size, p, padding=padding)
    yield "forward"
    y.backward(dy)
    yield "backward"


def main() -> None:
    ap = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    ap.add_argument("--n", type=int, default=128)
    ap.add_argument("--c", type=int, default=64)
    ap.add_argument("--k", type=int, default=128)
    ap.add_argument("--hw", type=int, default=32)
    ap.add_argument("--rs", type=int, default=3)
    ap.add_argument("--block-size", type=int, default=64)
    ap.add_argument("--p", type=float, nargs="+", default=[0.0, 0.5])
    ap.add_argument("--duration", type=float, default=1.0)
    args = ap.parse_args()
    torch.manual_seed(0)
    pad = args.rs // 2
    x = torch.randn(args.n, args.c, args.hw, args.hw, device="cuda").half().requires_grad_()
    kern = (torch.randn(args.k, args.c, args.rs, args.rs, device="cuda") * (args.c * args.rs ** 2) ** -0.5).half().requires_grad_()
    dy = torch.randn(args.n, args.k, args.hw, args.hw, device="cuda").half().contiguous(memory_format=torch.channels_last)
    fns = {"conv2d (torch)": lambda: f_torch(x, kern, dy, pad), "im2col + GEMM (HIP)": lambda: f_im2col(x, kern, dy, pad)}
    for p in args.p:
        fns[f"block dropout p={p} (HIP)"] = lambda p=p: f_blockdrop(x, kern, dy, pad, args.block_size, p)
    bench = Benchmarker(fns, duration=args.duration)
    bench.run()
    print(f"input {tuple(x.shape)} kernel {tuple(kern.shape)} pad {pad} block_size {args.block_size}")
    print_table(bench.results())


if __name__ == "__main__":
    main()
