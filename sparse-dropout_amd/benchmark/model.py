"""Whole-model forward + backward time as the drop rate varies (reference: benchmark/model.py:119-229).

    python -m benchmark.model --model mlp mlp-784 vit-ffn gpt-ffn --p 0 0.1 0.3 0.5 0.7

Models are built from ``DropoutMM`` the way the reference's evaluation models are:
  mlp      flattened 32x32 images -> [hidden]*layers -> 10 classes padded to 128, ReLU between, dropout on
           the input of every linear but the first (eval/mlp/model.py: BasicNet); batch 1024, hidden 1024
  mlp-784  the same on 4096 unresized 28x28 images with 10 unpadded classes: 784 -> 1024 -> 1024 -> 10
  vit-ffn  one transformer feed-forward block on 64x256 tokens: 384 -> 1536 -> GELU -> 384, dropout on the
           inputs of both linears
  gpt-ffn  the feed-forward block of the reference's GPT (benchmark/model.py:96-112: n_embed 1024, context 128,
           batch 32; eval/llm/model.py:58-66: 1024 -> 4096 -> GELU -> 1024) on its 32x128 = 4096 tokens
Each is timed with variant "none" (dense), "vanilla" (element dropout + dense), "blockwise[hip]" and
"blockwise[hip-fused]": the same layers as one autograd function whose GEMM stores apply the activation and
its derivative (no activation kernels in either direction)."""
from __future__ import annotations

import argparse
import statistics
import time

import torch
from torch import nn

import flash_dropout.functional as F
from flash_dropout.layers import DropoutMM

from .utils import FLUSH_BYTES


class Mlp(nn.Module):
    def __init__(self, variant, p, block_size, in_dim=1024, hidden=1024, layers=2, classes=128):
        super().__init__()
        dims = [in_dim] + [hidden] * layers + [classes]
        self.linears = nn.ModuleList(
            DropoutMM(dims[i], dims[i + 1], p=p if i else 0.0, variant=variant if i else "none",
                      block_size=block_size) for i in range(len(dims) - 1))

    def forward(self, x):
        x = x.flatten(1)
        for i, lin in enumerate(self.linears):
            x = lin(x if i == 0 else torch.relu(x))
        return x


class VitFfn(nn.Module):
    def __init__(self, variant, p, block_size, dim=384, hidden=1536):
        super().__init__()
        self.up = DropoutMM(dim, hidden, p=p, variant=variant, block_size=block_size)
        self.down = DropoutMM(hidden, dim, p=p, variant=variant, block_size=block_size)

    def forward(self, x):
        return self.down(nn.functional.gelu(self.up(x)))


class FusedStack(nn.Module):
    """The layers of ``Mlp`` / ``VitFfn`` (same shapes, same initialisation) run through
    ``hip_blockwise_dropout_mlp``: activation and activation gradient in the GEMM epilogues."""

    def __init__(self, dims, ps, activation, block_size):
        super().__init__()
        self.linears = nn.ModuleList(DropoutMM(dims[i], dims[i + 1], p=ps[i], variant="none")
                                     for i in range(len(dims) - 1))  # parameter holders
        self.ps, self.activation, self.block_size = tuple(ps), activation, block_size

    def forward(self, x):
        lead = x.shape[:-1] if x.dim() == 3 else None
        x2 = x.flatten(1) if lead is None else x.reshape(-1, x.shape[-1])
        y = F.hip_blockwise_dropout_mlp(x2, [l.weight for l in self.linears], self.block_size, self.ps, self.activation)
        return y if lead is None else y.reshape(*lead, y.shape[-1])


def fused_variant(name, p, block_size):
    if name == "mlp":
        return FusedStack([1024, 1024, 1024, 128], [0.0, p, p], "relu", block_size)
    if name == "mlp-784":
        return FusedStack([784, 1024, 1024, 10], [0.0, p, p], "relu", block_size)
    if name == "gpt-ffn":
        return FusedStack([1024, 4096, 1024], [p, p], "gelu", block_size)
    return FusedStack([384, 1536, 384], [p, p], "gelu", block_size)


class Mlp784(Mlp):
    """28 x 28 images without the reference's resize and class padding: 784 -> 1024 -> 1024 -> 10, so the first
    product has a ragged reduction (784 = 12 * 64 + 16) and the last one 10 output columns."""

    def __init__(self, variant, p, block_size):
        super().__init__(variant, p, block_size, in_dim=784, hidden=1024, layers=2, classes=10)


class GptFfn(VitFfn):
    """The feed-forward block of the reference's GPT configuration: 1024 -> 4096 -> GELU -> 1024."""

    def __init__(self, variant, p, block_size):
        super().__init__(variant, p, block_size, dim=1024, hidden=4096)


MODELS = {
    "gpt-ffn": (GptFfn, lambda: torch.randn(32, 128, 1024)),
    "mlp": (Mlp, lambda: torch.rand(1024, 1, 32, 32)),
    "mlp-784": (Mlp784, lambda: torch.rand(4096, 1, 28, 28)),
    "vit-ffn": (VitFfn, lambda: torch.randn(64, 256, 384)),
}


def time_model(model: nn.Module, x: torch.Tensor, warmup: float, rep: float, graph: bool = False) -> list[float]:
    """fwd+bwd milliseconds per repetition, cache flushed before each (benchmark/model.py:119-142).
    With ``graph`` the step is captured once in a HIP graph and replayed: no Python or launch path in the
    timed region (block-dropout masks still change from replay to replay, they are drawn from device state)."""
    cache = torch.empty(FLUSH_BYTES, dtype=torch.int8, device="cuda")

    def step():
        model(x).float().square().mean().backward()

    f = step
    if graph:
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            for _ in range(3):
                step()
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()
        for prm in model.parameters():
            prm.grad = None
        captured = torch.cuda.CUDAGraph()
        with torch.cuda.graph(captured):
            step()
        f = captured.replay

    for _ in range(10):
        f()
    t0 = time.time()
    while time.time() - t0 < warmup:
        f()
        torch.cuda.synchronize()
    timings, t0 = [], time.time()
    while time.time() - t0 < rep or len(timings) < 5:
        cache.zero_()
        a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        a.record()
        f()
        b.record()
        torch.cuda.synchronize()
        timings.append(a.elapsed_time(b))
    return timings


def main() -> None:
    ap = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    ap.add_argument("--model", nargs="+", choices=sorted(MODELS), default=sorted(MODELS))
    ap.add_argument("--p", type=float, nargs="+", default=[0.0, 0.1, 0.3, 0.5, 0.7])
    ap.add_argument("--block-size", type=int, default=64)
    ap.add_argument("--rep", type=float, default=0.3, help="seconds of timed repetitions per point")
    ap.add_argument("--graph", action="store_true", help="capture the step in a HIP graph and time replays")
    args = ap.parse_args()
    torch.manual_seed(0)
    for name in args.model:
        cls, make_x = MODELS[name]
        x = make_x().cuda().half()
        print(f"=== {name}  input {tuple(x.shape)}  block_size {args.block_size}{'  (graph replay)' if args.graph else ''}")
        for variant, ps in (("none", [0.0]), ("vanilla", [0.5]), ("blockwise[hip]", args.p),
                            ("blockwise[hip-fused]", args.p)):
            for p in ps:
                model = (fused_variant(name, p, args.block_size) if variant.endswith("fused]")
                         else cls(variant, p, args.block_size)).cuda().half().train()
                ts = time_model(model, x, warmup=0.2, rep=args.rep, graph=args.graph)
                sem = statistics.stdev(ts) / len(ts) ** 0.5 if len(ts) > 1 else 0.0
                print(f"{variant:<21} p={p:<4} median {statistics.median(ts):8.4f} ms  "
                      f"mean {statistics.mean(ts):8.4f} +- {1.96 * sem:.4f}  n={len(ts)}")


if __name__ == "__main__":
    main()
