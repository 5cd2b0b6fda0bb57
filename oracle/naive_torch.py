"""Second witness + CPU baseline: the reference's naive PyTorch path, restated on torch CPU.

TEST INFRASTRUCTURE ONLY (same rule as sparsedrop_oracle.py: never imported by the product).

Follows flash_dropout/functional/naive.py:8-25 step for step — copy X, look at it as a grid of
block_size x block_size tiles, zero the dropped tiles, divide the kept tiles by (1-p), then a
dense linear — and lets torch autograd produce dX and dW, which is how the reference's own
parity test builds its expected values (test/test_cuda.py:37-43).  Like the reference it needs
M and K to be multiples of the block size.  The numpy oracle's closed forms are checked
against this in tests/test_oracle.py, and bench.py times it as the reported CPU baseline.
"""
from __future__ import annotations

import torch


def masked_scaled_input(x: torch.Tensor, mask: torch.Tensor, block_size: int, p: float) -> torch.Tensor:
    """(keep ⊙ X)/(1-p) built with tile indexing as in naive.py:18-23 (differentiable w.r.t. x)."""
    if not 0 <= p < 1:
        raise ValueError("Dropout probability must be in [0, 1)")
    m, k = x.shape
    if m % block_size or k % block_size:
        raise ValueError("the naive path needs M and K to be multiples of block_size")
    xs = x.clone()
    tiles = xs.view(m // block_size, block_size, k // block_size, block_size).transpose(1, 2)
    tiles[mask] = 0
    tiles[~mask] /= 1 - p
    return xs


def forward(x: torch.Tensor, w: torch.Tensor, mask: torch.Tensor, block_size: int, p: float) -> torch.Tensor:
    return torch.nn.functional.linear(masked_scaled_input(x, mask, block_size, p), w)


def forward_backward(x, w, dy, mask, block_size: int, p: float):
    """Returns (Y, dX, dW) via autograd, fp32 or fp64 as given."""
    x = x.detach().clone().requires_grad_()
    w = w.detach().clone().requires_grad_()
    y = forward(x, w, mask, block_size, p)
    y.backward(dy)
    return y.detach(), x.grad, w.grad
