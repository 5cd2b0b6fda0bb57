"""Block-dropout matmul on the HIP kernels, as an autograd Function.

Counterpart of the reference's ``BlockwiseDropoutMatmulCUDA``
(flash_dropout/functional/blockwise_dropout_matmul_cuda.py:7-59):

    forward   Y  = gemm_dsd(X, W, mask)            (:26)
    backward  dX = gemm_sdd(dY, W.T, mask)         (:46)
              dW = gemm_dsd(X.T, dY.T, mask.T).T   (:49-51)

Differences that matter to a caller: the kept-block lists are built once on the GPU in forward and
reused by both backward products (no per-iteration mask reads, no host sync); without a given mask
the Bernoulli draw happens inside the list-building launch; dW comes back as a contiguous [N, K]
tensor instead of a transposed view; bf16 works as well as fp16; shapes need not be multiples of
anything; block sizes that are multiples of 64 all run on the 64-block kernels; launches go to
torch's current stream.
"""
from __future__ import annotations

import torch

from ..hip.binding_gemm import GEMM, KeptLists, _block_size, as_matrix


class BlockwiseDropoutMatmulHIP(torch.autograd.Function):
    @staticmethod
    def forward(ctx, input: torch.Tensor, weight: torch.Tensor, mask: torch.Tensor | None,
                block_size: int, p: float, seed: int | None = None):
        ext = GEMM()
        # mask given, or drawn in the list-building launch (reference: blockwise_dropout_mask, …_cuda.py:24);
        # C (M N) = A (M K sparse) * B (N K); one library call for mask, lists and product
        out, mask, lists, kernel_bs = ext.dropout_matmul_forward(input, weight, block_size, p, mask, seed)
        ctx.save_for_backward(input, weight, mask, lists.row_ptr, lists.col_idx, lists.col_ptr,
                              lists.row_idx)
        ctx.block_size = kernel_bs
        ctx.list_shape = lists.shape
        ctx.p = p
        return out

    @staticmethod
    def backward(ctx, grad_output: torch.Tensor):
        input, weight, mask, row_ptr, col_idx, col_ptr, row_idx = ctx.saved_tensors
        lists = KeptLists(row_ptr, col_idx, col_ptr, row_idx, ctx.list_shape)
        ext = GEMM()
        if grad_output.dtype != input.dtype:
            grad_output = grad_output.to(input.dtype)
        grad_output = as_matrix(grad_output)  # expanded (stride 0) and doubly strided gradients are laid out first
        # dA (M K sparse) = dC (M N) * B.T (K N), the mask over the output; dB.T (K N) = A.T (K M sparse) * dC.T (N M),
        # written straight into a row-major [N, K] (reference: …_cuda.py:46-51); one library call for both
        grad_input, grad_weight = ext.dropout_matmul_backward(grad_output, weight, input, lists, ctx.block_size, ctx.p,
                                                              ctx.needs_input_grad[0], ctx.needs_input_grad[1])
        return grad_input, grad_weight, None, None, None, None


def _apply_outside_autocast(function, *args):
    """``function.apply(*args)`` with autocast off inside, as ``custom_fwd(cast_inputs=...)`` arranges in the
    reference (…_cuda.py:9); the context is only entered when autocast is on (it costs microseconds per call)."""
    if torch.is_autocast_enabled("cuda"):
        with torch.autocast("cuda", enabled=False):
            return function.apply(*args)
    return function.apply(*args)


def _prepare(input: torch.Tensor, weight: torch.Tensor):
    """Autocast contract of the reference (``custom_fwd(cast_inputs=torch.float16)``, …_cuda.py:9):
    under autocast the operands are cast to the autocast dtype; outside it they must already be
    float16 / bfloat16."""
    if input.dim() != 2 or weight.dim() != 2:
        raise ValueError("input must be [M, K] and weight [N, K]")
    if torch.is_autocast_enabled("cuda"):
        dt = torch.get_autocast_dtype("cuda")
        input, weight = input.to(dt), weight.to(dt)
    return as_matrix(input), as_matrix(weight)


def blockwise_dropout_matmul_mask(input: torch.Tensor, mask: torch.Tensor, block_size, p: float,
                                  weight: torch.Tensor) -> torch.Tensor:
    """Same as :func:`blockwise_dropout_matmul` with the mask given (True = dropped); argument order
    of the reference's naive counterpart (functional/naive.py:8-14)."""
    if not 0 <= p < 1:
        raise ValueError("Dropout probability must be in [0, 1)")
    bs = _block_size(block_size)
    input, weight = _prepare(input, weight)
    return _apply_outside_autocast(BlockwiseDropoutMatmulHIP, input, weight, mask, bs, float(p))


def blockwise_dropout_matmul(input: torch.Tensor, weight: torch.Tensor, block_size, p: float,
                             seed: int | None = None) -> torch.Tensor:
    """``(keep ⊙ input)/(1-p) @ weight.T`` with a fresh block mask (reference: …_cuda.py:56-59).

    The mask is drawn on the device inside the list-building launch; ``seed`` pins it (the same mask
    comes back from ``GEMM().random_lists(mask_shape, p, seed)``), otherwise it comes from the
    device-resident generator state, which starts at ``torch.initial_seed()`` and advances by one per
    call on the stream: nothing about the draw is a launch argument, so a captured graph draws a new
    mask at every replay."""
    if not 0 <= p < 1:
        raise ValueError("Dropout probability must be in [0, 1)")
    bs = _block_size(block_size)
    input, weight = _prepare(input, weight)
    return _apply_outside_autocast(BlockwiseDropoutMatmulHIP, input, weight, None, bs, float(p), seed)
