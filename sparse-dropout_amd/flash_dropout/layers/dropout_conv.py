"""``DropoutConv2d``: a bias-free 2-D convolution with dropout on its input
(reference: flash_dropout/layers/dropout_conv.py:10-101).

The reference stops at "none" / "im2col" / "vanilla" / "vanilla_2d" and leaves the block-wise
variants commented out (:86-99) with no error for unknown names; here the block-wise variants run
(block dropout on the im2col patch matrix) and an unknown variant raises.
"""
from __future__ import annotations

import math

import torch
from torch import nn

from .. import functional as F

VARIANTS = ("none", "im2col", "vanilla", "vanilla_2d", "blockwise[naive]", "blockwise[hip]",
            "blockwise[cuda]", "blockwise[triton]")


class DropoutConv2d(nn.Module):
    __constants__ = ["stride", "padding", "dilation", "in_channels", "out_channels", "kernel_size",
                     "p", "variant"]

    def __init__(self, in_channels: int, out_channels: int, kernel_size: tuple[int, int],
                 stride: tuple[int, int] = (1, 1), padding: tuple[int, int] = (0, 0),
                 dilation: tuple[int, int] = (1, 1), p: float = 0.1, variant: str = "vanilla",
                 **kwargs) -> None:
        super().__init__()
        self.in_channels = in_channels
        self.out_channels = out_channels
        self.kernel_size = tuple(kernel_size)
        self.stride = tuple(stride)
        self.padding = tuple(padding)
        self.dilation = tuple(dilation)
        self.p = p
        self.variant = variant
        self.kwargs = kwargs
        self.weight = nn.Parameter(torch.empty(out_channels, in_channels, *self.kernel_size))
        self.reset_parameters()

    def reset_parameters(self) -> None:
        nn.init.kaiming_uniform_(self.weight, a=math.sqrt(5))

    def _conv(self, x: torch.Tensor) -> torch.Tensor:
        return nn.functional.conv2d(x, self.weight, stride=self.stride, padding=self.padding,
                                    dilation=self.dilation)

    def forward(self, input: torch.Tensor) -> torch.Tensor:
        if not self.training:
            return self._conv(input)
        geom = dict(padding=self.padding, stride=self.stride, dilation=self.dilation)
        v = self.variant
        if v == "none":
            return self._conv(input)
        if v == "im2col":
            return F.im2col_conv2d(input, self.weight, **geom)
        if v == "vanilla":
            return self._conv(nn.functional.dropout(input, p=self.p))
        if v == "vanilla_2d":
            return self._conv(nn.functional.dropout2d(input, p=self.p))
        if v == "blockwise[naive]":
            return F.naive_blockwise_dropout_conv2d(input, self.weight, self.kwargs["block_size"], self.p, **geom)
        if v in ("blockwise[hip]", "blockwise[cuda]", "blockwise[triton]"):
            return F.blockwise_dropout_conv2d(input, self.weight, self.kwargs["block_size"], self.p, **geom)
        raise ValueError(f"Unknown variant {self.variant}")

    def extra_repr(self) -> str:
        return (f"{self.in_channels}, {self.out_channels}, kernel_size={self.kernel_size}, "
                f"stride={self.stride}, padding={self.padding}, dilation={self.dilation}, p={self.p}, "
                f"variant={self.variant!r}")
