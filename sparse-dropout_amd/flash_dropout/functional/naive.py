"""Block dropout followed by a dense linear, in plain torch ops on whatever device the input is on.

The "Block dropout + Dense" comparison line of the reference (flash_dropout/functional/naive.py:8-32):
no work is skipped.  Unlike the reference, M and K need not be multiples of the block size (the mask
is ceil-shaped, so edge blocks are simply smaller).
"""
from __future__ import annotations

import torch
import torch.nn.functional as F

from ..hip.binding_gemm import _block_size
from .utils import blockwise_dropout_mask


def blockwise_dropout_matmul_mask(input: torch.Tensor, mask: torch.Tensor, block_size, p: float,
                                  weight: torch.Tensor) -> torch.Tensor:
    if not 0 <= p < 1:
        raise ValueError("Dropout probability must be in [0, 1)")
    bs = _block_size(block_size)
    M, K = input.shape
    keep = (~mask).repeat_interleave(bs, 0).repeat_interleave(bs, 1)[:M, :K]
    return F.linear(input * keep.to(input.dtype) / (1 - p), weight)


def blockwise_dropout_matmul(input: torch.Tensor, weight: torch.Tensor, block_size, p: float):
    mask = blockwise_dropout_mask(input, block_size, p)
    return blockwise_dropout_matmul_mask(input, mask, block_size, p, weight)
