"""The three products at 8192^3 on masks that keep half of the blocks in different arrangements: what a launch costs
follows how the kept tiles sit in a workgroup's 4 row blocks, not only how many there are.

    python -m benchmark.masks                         # times, L2 flushed before every call, median of 12
    python -m benchmark.masks --only dx --mask checkerboard --launches 6     # a few launches of one product, for
                                                      # rocprofv3 --pmc FETCH_SIZE -- python -m benchmark.masks ...

Masks (True = dropped, 128 x 128 blocks of 64): "bernoulli" (p = 0.5), "checkerboard" (every workgroup of the dX kernel
gets the same 6 columns x 2 tiles), "rows" (row blocks 2 and 3 of every four dropped), "columns" (every other column
block dropped: the kept tiles form dense 4 x 4 groups), "none" (nothing dropped).
"""
from __future__ import annotations

import argparse

import torch

from flash_dropout.hip import GEMM

SIZE = 8192
MASKS = ("bernoulli", "checkerboard", "rows", "columns", "none")


def make_mask(name: str, gen: torch.Generator) -> torch.Tensor:
    nb = SIZE // 64
    i = torch.arange(nb, device="cuda")
    if name == "bernoulli":
        return torch.rand(nb, nb, device="cuda", generator=gen) < 0.5
    if name == "checkerboard":
        return (i[:, None] + i[None, :]) % 2 == 0
    if name == "rows":
        return (i[:, None] % 4 >= 2).expand(nb, nb).contiguous()
    if name == "columns":
        return (i[None, :] % 2 == 0).expand(nb, nb).contiguous()
    return torch.zeros(nb, nb, dtype=torch.bool, device="cuda")


def main() -> None:
    ap = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    ap.add_argument("--mask", nargs="+", choices=MASKS, default=list(MASKS))
    ap.add_argument("--only", choices=["forward", "dx", "dw"], help="one product only")
    ap.add_argument("--launches", type=int, default=0, help="this many flushed launches per product and no timing")
    args = ap.parse_args()
    ext = GEMM()
    gen = torch.Generator(device="cuda").manual_seed(0)
    x = torch.randn(SIZE, SIZE, device="cuda", dtype=torch.float16, generator=gen)
    w = torch.randn(SIZE, SIZE, device="cuda", dtype=torch.float16, generator=gen) * SIZE ** -0.5
    dy = torch.randn(SIZE, SIZE, device="cuda", dtype=torch.float16, generator=gen)
    flush = torch.empty(512 << 20, dtype=torch.int8, device="cuda")
    y, dx = torch.empty_like(x), torch.empty_like(x)
    dwt = torch.empty_like(x).t()

    def run(f, n):
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

    for rnd in range(1 if args.launches else 2):  # the first pass over the masks is warm-up
        for name in args.mask:
            mask = make_mask(name, gen)
            lists = ext.build_lists(mask)
            lt = lists.transposed()
            keep = 1.0 - mask.float().mean().item()
            products = {
                "forward": lambda: ext.gemm_dsd_lists(x, w, lists, 64, 2.0, out=y),
                "dx": lambda: ext.gemm_sdd_lists(dy, w.t(), lists, 64, 2.0, out=dx, keep_hint=keep),
                "dw": lambda: ext.gemm_dsd_lists(x.t(), dy.t(), lt, 64, 2.0, out=dwt),
            }
            if args.only:
                products = {args.only: products[args.only]}
            if args.launches:
                for f in products.values():
                    run(f, args.launches)
                continue
            for f in products.values():
                run(f, 3)
            t = {k: run(f, 12) for k, f in products.items()}
            if rnd:
                print(f"{name:13s} kept {keep:.3f}: " + "  ".join(f"{k} {v:.0f}" for k, v in t.items()) + " us", flush=True)


if __name__ == "__main__":
    main()
