"""``DropoutMM``: a bias-free linear layer with dropout on its input
(reference: flash_dropout/layers/dropout_mm.py:10-65)."""
from __future__ import annotations

import math

import torch
from torch import nn

from .. import functional as F

_BLOCKWISE = {
    "blockwise[naive]": F.naive_blockwise_dropout_matmul,
    "blockwise[hip]": F.hip_blockwise_dropout_matmul,
    # the reference's backend names keep working and run the HIP kernels
    "blockwise[cuda]": F.cuda_blockwise_dropout_matmul,
    "blockwise[triton]": F.triton_blockwise_dropout_matmul,
}
VARIANTS = ("none", "vanilla", *_BLOCKWISE)


class DropoutMM(nn.Module):
    """y = dropout(x) @ W.T, W of shape (out_features, in_features), no bias.

    ``variant``: "none" (no dropout), "vanilla" (element-wise dropout), or one of the block-wise
    variants, which need ``block_size=`` in ``kwargs``.  In eval mode every variant is a plain
    linear.  Leading dims are flattened first, so blocks span consecutive rows of the
    (batch*seq, features) matrix (dropout_mm.py:41-42).
    """

    __constants__ = ["in_features", "out_features"]

    def __init__(self, in_features: int, out_features: int, p: float = 0.1, variant: str = "vanilla",
                 **kwargs) -> None:
        super().__init__()
        self.in_features = in_features
        self.out_features = out_features
        self.p = p
        self.variant = variant
        self.kwargs = kwargs
        self.weight = nn.Parameter(torch.empty(out_features, in_features))
        self.reset_parameters()

    def reset_parameters(self) -> None:
        # same initialisation as the reference (dropout_mm.py:34-35)
        nn.init.kaiming_uniform_(self.weight, a=math.sqrt(5))

    def forward(self, input: torch.Tensor) -> torch.Tensor:
        if not self.training:
            return nn.functional.linear(input, self.weight)
        lead = input.shape[:-1]
        x2 = input.reshape(-1, input.shape[-1])
        if self.variant == "none":
            y2 = nn.functional.linear(x2, self.weight)
        elif self.variant == "vanilla":
            y2 = F.vanilla_dropout_matmul(x2, self.weight, self.p)
        elif self.variant in _BLOCKWISE:
            y2 = _BLOCKWISE[self.variant](x2, self.weight, self.kwargs["block_size"], self.p)
        else:
            raise ValueError(f"Unknown variant {self.variant}")
        return y2.reshape(*lead, self.out_features)

    def extra_repr(self) -> str:
        return (f"in_features={self.in_features}, out_features={self.out_features}, p={self.p}, "
                f"variant={self.variant!r}")
