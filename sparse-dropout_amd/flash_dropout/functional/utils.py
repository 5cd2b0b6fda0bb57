"""Mask helpers (reference: flash_dropout/functional/utils.py)."""
from __future__ import annotations

from math import ceil

import torch

from ..hip.binding_gemm import GEMM, KeptLists, _block_size


def blockwise_dropout_mask(x: torch.Tensor, block_size, p: float) -> torch.Tensor:
    """Bernoulli block mask for the last two dims of ``x``; True = dropped.

    Same definition as the reference (utils.py:11-16): ``rand(ceil(m/bs), ceil(k/bs)) < p`` drawn
    from the generator of ``x``'s device, leading dims kept as batch dims.
    """
    bs = _block_size(block_size)
    *batch, m, k = x.shape
    return torch.rand(*batch, ceil(m / bs), ceil(k / bs), device=x.device) < p


def kept_block_lists(mask: torch.Tensor) -> KeptLists:
    """Compacted kept-block lists (CSR + CSC, int32) of a 2D block mask, built on the GPU."""
    return GEMM().build_lists(mask)


def kept_block_table(mask: torch.Tensor) -> torch.Tensor:
    """[nnz, 2] int64 (row_blk, col_blk) of kept blocks in row-major order — what the reference gets
    from ``torch.nonzero(~mask)`` (blockwise_dropout_matmul_triton.py:48) — from the HIP lists."""
    lists = kept_block_lists(mask)
    nnz = lists.nnz()
    widths = (lists.row_ptr[1:] - lists.row_ptr[:-1]).to(torch.int64)
    rows = torch.repeat_interleave(torch.arange(mask.shape[0], device=mask.device), widths,
                                   output_size=nnz)
    return torch.stack([rows, lists.col_idx[:nnz].to(torch.int64)], dim=1)


def mask_to_increment_table(mask: torch.Tensor, BLOCK_K: int):
    """(table, row_indices, row_widths) as the reference defines them (utils.py:19-69): per kept
    block the number of elements to advance along K from the previous kept block of its row (the
    first of a row counts from 0), the start of each row in ``table``, and each row's length."""
    g = GEMM()
    return g.increment_table(g.build_lists(mask), BLOCK_K)


def min_dtype(a_dtype: torch.dtype, b_dtype: torch.dtype) -> torch.dtype:
    """The narrower of two float dtypes (utils.py:84-88)."""
    return a_dtype if torch.finfo(a_dtype).bits < torch.finfo(b_dtype).bits else b_dtype
