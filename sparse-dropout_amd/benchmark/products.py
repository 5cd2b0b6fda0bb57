"""Single products on model shapes: forward (DSD), dX (SDD) and dW (DSD on transposed views) of a block-dropout linear
layer at a few drop rates, beside ``torch.matmul`` on the same operands.  L2 flushed before every call, median of 20.

    python -m benchmark.products                      # the shapes below
    python -m benchmark.products --shape 4096 1024 4096 --p 0 0.5

Prints microseconds per product and the kernel each call ran on (``GEMM.last_kernel_detail``).
"""
from __future__ import annotations

import argparse

import torch

from flash_dropout.hip import GEMM

# tokens M, output features N, input features K
SHAPES = {
    "gpt-ffn up": (4096, 4096, 1024),
    "gpt-ffn down": (4096, 1024, 4096),
    "vit-ffn up": (16384, 1536, 384),
    "vit-ffn down": (16384, 384, 1536),
    "2048^3": (2048, 2048, 2048),
    "4096^3": (4096, 4096, 4096),
}
FLUSH_BYTES = 512 << 20


def median_us(f, flush: torch.Tensor, n: int = 20) -> float:
    for _ in range(3):
        f()
    ts = []
    for _ in range(n):
        flush.zero_()
        a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        a.record()
        f()
        b.record()
        torch.cuda.synchronize()
        ts.append(a.elapsed_time(b))
    return sorted(ts)[len(ts) // 2] * 1e3


def main() -> None:
    ap = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    ap.add_argument("--shape", type=int, nargs=3, metavar=("M", "N", "K"), help="one shape instead of the built-in list")
    ap.add_argument("--p", type=float, nargs="+", default=[0.0, 0.5])
    ap.add_argument("--dtype", choices=["float16", "bfloat16"], default="float16")
    ap.add_argument("--tile-policy", choices=sorted(GEMM.TILE_POLICIES), default="auto",
                    help="force a workgroup shape (to check what the library picks by itself)")
    args = ap.parse_args()
    ext = GEMM()
    ext.set_tile_policy(args.tile_policy)
    dtype = getattr(torch, args.dtype)
    flush = torch.empty(FLUSH_BYTES, dtype=torch.int8, device="cuda")
    gen = torch.Generator(device="cuda").manual_seed(0)
    shapes = {"x".join(map(str, args.shape)): tuple(args.shape)} if args.shape else SHAPES
    for name, (M, N, K) in shapes.items():
        x = torch.randn(M, K, device="cuda", dtype=dtype, generator=gen)
        w = torch.randn(N, K, device="cuda", dtype=dtype, generator=gen) * K ** -0.5
        dy = torch.randn(M, N, device="cuda", dtype=dtype, generator=gen)
        t = [median_us(f, flush) for f in (lambda: torch.matmul(x, w.t()), lambda: torch.matmul(dy, w),
                                           lambda: torch.matmul(dy.t(), x))]
        print(f"{name:13s} M={M} N={N} K={K}   torch.matmul: forward {t[0]:.0f}  dX {t[1]:.0f}  dW {t[2]:.0f}  sum {sum(t):.0f} us",
              flush=True)
        for p in args.p:
            mask = torch.rand(-(-M // 64), -(-K // 64), device="cuda", generator=gen) < p
            lists = ext.build_lists(mask)
            lt = lists.transposed()
            s = 1 / (1 - p)
            y = torch.empty(M, N, device="cuda", dtype=dtype)
            dx = torch.empty(M, K, device="cuda", dtype=dtype)
            dwt = torch.empty(N, K, device="cuda", dtype=dtype).t()
            t, routes = [], []
            for f in (lambda: ext.gemm_dsd_lists(x, w, lists, 64, s, out=y),
                      lambda: ext.gemm_sdd_lists(dy, w.t(), lists, 64, s, out=dx, keep_hint=1 - p),
                      lambda: ext.gemm_dsd_lists(x.t(), dy.t(), lt, 64, s, out=dwt)):
                t.append(median_us(f, flush))
                routes.append(ext.last_kernel_detail())
            print(f"   block dropout p={p:<4}: forward {t[0]:.0f}  dX {t[1]:.0f}  dW {t[2]:.0f}  sum {sum(t):.0f} us   "
                  f"[{' | '.join(routes)}]", flush=True)


if __name__ == "__main__":
    main()
