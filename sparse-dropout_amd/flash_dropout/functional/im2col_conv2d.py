"""2-D convolution as im2col + matmul, dense and with block dropout on the patch matrix.

Reference: flash_dropout/functional/im2col_conv2d.py:5-27 — ``F.unfold`` to (N, C*R*S, P*Q), permute
to (N, P*Q, C*R*S), ``F.linear`` with ``kernel.view(K, -1)``, back to (N, K, P, Q).  Here the patch
matrix [N*P*Q, C*R*S] (same column order c*R*S + r*S + s) is produced by the HIP gather kernel and
multiplied by the HIP GEMMs; the result is returned, like the reference's, as an (N, K, P, Q) view
of an (N, P*Q, K) buffer.

The block-dropout variant is the one the reference left as comments in its conv layer
(flash_dropout/layers/dropout_conv.py:86-99): one Bernoulli per block_size x block_size tile of the
patch matrix; dropped tiles are neither gathered nor multiplied.
"""
from __future__ import annotations

from math import ceil

import torch
import torch.nn.functional as F

from ..hip.binding_gemm import GEMM, KeptLists, _block_size


# Use the implicit-GEMM forward (sd_conv2d_dsd_lists) where the library takes the geometry.  Module-level
# switch so that tests and benchmarks can compare both routes.
IMPLICIT_FORWARD = True
# Use the one-launch input gradient (sd_conv2d_dx) where the library takes the geometry.
FUSED_INPUT_GRADIENT = True

# Which route each product of the calling process's last convolution took: "implicit" / "fused" (no patch matrix in
# memory: sd_conv2d_dsd_lists, sd_conv2d_dw_lists, sd_conv2d_dx) or "explicit" (im2col / col2im around the GEMMs, taken
# when the library does not take the geometry or a switch above is off).  Read it with conv_last_routes().
_last_routes = {"forward": None, "dx": None, "dw": None}


def conv_last_routes() -> dict:
    """{"forward": ..., "dx": ..., "dw": ...} of the last convolution run through this module ("implicit", "fused" or
    "explicit"; None for a product that was not computed): nothing falls back to the patch matrix unseen."""
    return dict(_last_routes)


def _mask_on_64_grid(mask: torch.Tensor, block_size: int, rows: int, cols: int) -> torch.Tensor:
    """A mask at a block size that is a multiple of 64 as the mask of the same elements at block size 64 (every
    entry repeated, cropped to the 64 grid of a rows x cols matrix)."""
    f = block_size // 64
    if f == 1:
        return mask
    m = mask.repeat_interleave(f, 0).repeat_interleave(f, 1)
    return m[: ceil(rows / 64), : ceil(cols / 64)].contiguous()



def _pair(v) -> tuple[int, int]:
    if isinstance(v, int):
        return (v, v)
    a, b = v
    return (int(a), int(b))


def _to_matrix_grad(grad_output: torch.Tensor, dtype) -> torch.Tensor:
    """(N, K, P, Q) gradient -> [N*P*Q, K] row-major (free when it is channels-last in memory)."""
    n, k, p, q = grad_output.shape
    dy2 = grad_output.to(dtype).permute(0, 2, 3, 1).reshape(n * p * q, k)
    if dy2.stride(1) != 1 or dy2.stride(0) < k:  # e.g. the expanded (stride 0) gradient of a sum()
        dy2 = dy2.contiguous()
    return dy2


class _Im2colConv2d(torch.autograd.Function):
    @staticmethod
    def forward(ctx, input, kernel, mask, block_size, p, padding, stride, dilation, seed=None):
        ext = GEMM()
        n, c, h, w = input.shape
        k, _, r, s = kernel.shape
        po, qo = ext.conv_out_hw(h, w, r, s, padding, stride, dilation)
        w2 = kernel.reshape(k, c * r * s)
        kernel_bs = block_size
        if block_size:  # block dropout: mask given, or drawn in the list-building launch
            mask, lists, kernel_bs = ext.kept_lists(n * po * qo, c * r * s, block_size, mask, p, seed,
                                                    input.device)
            # implicit GEMM where the library takes the geometry: no patch matrix in the forward, and the
            # input is what is kept for the backward (the patch matrix is 9x its size for a 3x3 kernel)
            y2 = ext.conv2d_dsd_lists(input, w2, lists, kernel_bs, 1.0 / (1.0 - p), (r, s), padding, stride,
                                      dilation) if IMPLICIT_FORWARD else None
            ctx.implicit = y2 is not None
            _last_routes.update(forward="implicit" if ctx.implicit else "explicit", dx=None, dw=None)
            if y2 is None:
                cols = ext.im2col(input, (r, s), padding, stride, dilation, lists, kernel_bs)
                y2 = ext.gemm_dsd_lists(cols, w2, lists, kernel_bs, 1.0 / (1.0 - p))
            ctx.save_for_backward(input if ctx.implicit else cols, w2, mask, lists.row_ptr, lists.col_idx,
                                  lists.col_ptr, lists.row_idx)
            ctx.list_shape = lists.shape
        else:
            y2 = ext.conv2d_dsd_lists(input, w2, None, 0, 1.0, (r, s), padding, stride,
                                      dilation) if IMPLICIT_FORWARD else None
            ctx.implicit = y2 is not None
            _last_routes.update(forward="implicit" if ctx.implicit else "explicit", dx=None, dw=None)
            if y2 is None:
                cols = ext.im2col(input, (r, s), padding, stride, dilation)
                y2 = ext.gemm(cols, w2)
            ctx.save_for_backward(input if ctx.implicit else cols, w2)
        ctx.geom = (tuple(input.shape), tuple(kernel.shape), padding, stride, dilation, block_size, kernel_bs, p,
                    input.is_contiguous(memory_format=torch.channels_last) and not input.is_contiguous())
        return y2.view(n, po * qo, k).permute(0, 2, 1).view(n, k, po, qo)

    @staticmethod
    def backward(ctx, grad_output):
        ext = GEMM()
        x_shape, k_shape, padding, stride, dilation, block_size, kernel_bs, p, ch_last = ctx.geom
        r, s = k_shape[2], k_shape[3]
        saved = ctx.saved_tensors
        cols, w2 = saved[0], saved[1]
        dy2 = _to_matrix_grad(grad_output, cols.dtype)
        dx = dk = None
        if len(saved) > 2:
            mask = saved[2]
            lists = KeptLists(saved[3], saved[4], saved[5], saved[6], ctx.list_shape)
            scale = 1.0 / (1.0 - p)
            if ctx.needs_input_grad[0]:
                if FUSED_INPUT_GRADIENT and block_size % 64 == 0:
                    # the kernel works on 64 x 64 blocks: a mask at a larger multiple of 64 is the same element mask
                    m64 = _mask_on_64_grid(mask, block_size, dy2.shape[0], w2.shape[1])
                    dx = ext.conv2d_dx(dy2, w2, x_shape, (r, s), padding, stride, dilation, m64, 64, scale, ch_last)
                _last_routes["dx"] = "fused" if dx is not None else "explicit"
                if dx is None:
                    # col2im skips the dropped blocks, so the SDD need not zero them
                    dcols = ext.gemm_sdd_lists(dy2, w2.t(), lists, kernel_bs, scale, kept_only=True,
                                                keep_hint=1.0 / scale)
                    dx = ext.col2im(dcols, x_shape, (r, s), padding, stride, dilation, mask, block_size, ch_last)
            if ctx.needs_input_grad[1]:
                if ctx.implicit:  # the forward kept the input, not the patch matrix
                    dk = ext.conv2d_dw_lists(cols, dy2, lists, kernel_bs, scale, (r, s), padding, stride, dilation)
                    if dk is None:  # gather the kept blocks now
                        cols = ext.im2col(cols, (r, s), padding, stride, dilation, lists, kernel_bs)
                _last_routes["dw"] = "implicit" if dk is not None else "explicit"
                if dk is None:
                    dk = ext.gemm_dsd_lists(cols.t(), dy2.t(), lists.transposed(), kernel_bs, scale,
                                            transposed_out=True).t()
                dk = dk.reshape(k_shape)
        else:
            if ctx.needs_input_grad[0]:
                if FUSED_INPUT_GRADIENT:
                    dx = ext.conv2d_dx(dy2, w2, x_shape, (r, s), padding, stride, dilation, channels_last=ch_last)
                _last_routes["dx"] = "fused" if dx is not None else "explicit"
                if dx is None:
                    dcols = ext.gemm(dy2, w2.t())
                    dx = ext.col2im(dcols, x_shape, (r, s), padding, stride, dilation, channels_last=ch_last)
            if ctx.needs_input_grad[1]:
                if ctx.implicit:
                    dk = ext.conv2d_dw_lists(cols, dy2, None, 0, 1.0, (r, s), padding, stride, dilation)
                    if dk is None:
                        cols = ext.im2col(cols, (r, s), padding, stride, dilation)
                _last_routes["dw"] = "implicit" if dk is not None else "explicit"
                if dk is None:
                    dk = ext.gemm(cols.t(), dy2.t(), transposed_out=True).t()
                dk = dk.reshape(k_shape)
        return dx, dk, None, None, None, None, None, None, None


def _apply_outside_autocast(function, *args):
    """``function.apply(*args)`` with autocast off inside, as ``custom_fwd(cast_inputs=...)`` arranges in the
    reference (…_cuda.py:9); the context is only entered when autocast is on (it costs microseconds per call)."""
    if torch.is_autocast_enabled("cuda"):
        with torch.autocast("cuda", enabled=False):
            return function.apply(*args)
    return function.apply(*args)


def _prepare(input: torch.Tensor, kernel: torch.Tensor):
    if input.dim() != 4 or kernel.dim() != 4:
        raise ValueError("input must be (N, C, H, W) and kernel (K, C, R, S)")
    if input.shape[1] != kernel.shape[1]:
        raise ValueError(f"channel mismatch: input {input.shape[1]}, kernel {kernel.shape[1]}")
    if torch.is_autocast_enabled("cuda"):
        dt = torch.get_autocast_dtype("cuda")
        input, kernel = input.to(dt), kernel.to(dt)
    return input, kernel.contiguous()


def im2col_conv2d(input: torch.Tensor, kernel: torch.Tensor, padding=(0, 0), stride=(1, 1),
                  dilation=(1, 1)) -> torch.Tensor:
    """Dense convolution through the patch matrix (reference: im2col_conv2d.py:5-27)."""
    input, kernel = _prepare(input, kernel)
    return _apply_outside_autocast(_Im2colConv2d, input, kernel, None, 0, 0.0, _pair(padding), _pair(stride), _pair(dilation))


def conv_patch_matrix_shape(input_shape, kernel_shape, padding=(0, 0), stride=(1, 1), dilation=(1, 1)):
    """(N*P*Q, C*R*S): the matrix the block mask of the conv variant is drawn over."""
    n, c, h, w = input_shape
    _, _, r, s = kernel_shape
    po, qo = GEMM.conv_out_hw(h, w, r, s, _pair(padding), _pair(stride), _pair(dilation))
    return n * po * qo, c * r * s


def blockwise_dropout_conv2d_mask(input, mask, block_size, p: float, kernel, padding=(0, 0),
                                  stride=(1, 1), dilation=(1, 1)) -> torch.Tensor:
    """Block-dropout convolution with the mask given: ``mask`` is bool
    [ceil(N*P*Q/bs), ceil(C*R*S/bs)], True = dropped."""
    if not 0 <= p < 1:
        raise ValueError("Dropout probability must be in [0, 1)")
    bs = _block_size(block_size)
    if bs % 64:
        raise NotImplementedError(f"block_size {bs}: the convolution takes multiples of 64 (the matmul also 32)")
    input, kernel = _prepare(input, kernel)
    return _apply_outside_autocast(_Im2colConv2d, input, kernel, mask, bs, float(p), _pair(padding), _pair(stride), _pair(dilation))


def blockwise_dropout_conv2d(input, kernel, block_size, p: float, padding=(0, 0), stride=(1, 1),
                             dilation=(1, 1), seed: int | None = None) -> torch.Tensor:
    """Block-dropout convolution with a fresh mask over the patch matrix, drawn on the device inside the
    list-building launch (``seed`` pins it, as for the matmul)."""
    if not 0 <= p < 1:
        raise ValueError("Dropout probability must be in [0, 1)")
    bs = _block_size(block_size)
    if bs % 64:
        raise NotImplementedError(f"block_size {bs}: the convolution takes multiples of 64 (the matmul also 32)")
    input, kernel = _prepare(input, kernel)
    return _apply_outside_autocast(_Im2colConv2d, input, kernel, None, bs, float(p), _pair(padding), _pair(stride),
                                   _pair(dilation), seed)


def naive_blockwise_dropout_conv2d_mask(input, mask, block_size, p: float, kernel, padding=(0, 0),
                                        stride=(1, 1), dilation=(1, 1)) -> torch.Tensor:
    """The same function in plain torch ops (unfold, expanded mask, dense linear); no work skipped."""
    from .naive import blockwise_dropout_matmul_mask

    n, c, h, w = input.shape
    k, _, r, s = kernel.shape
    po, qo = GEMM.conv_out_hw(h, w, r, s, _pair(padding), _pair(stride), _pair(dilation))
    cols = F.unfold(input, (r, s), dilation=_pair(dilation), padding=_pair(padding), stride=_pair(stride))
    cols = cols.permute(0, 2, 1).reshape(n * po * qo, c * r * s)
    y2 = blockwise_dropout_matmul_mask(cols, mask, block_size, p, kernel.reshape(k, -1))
    return y2.view(n, po * qo, k).permute(0, 2, 1).reshape(n, k, po, qo)


def naive_blockwise_dropout_conv2d(input, kernel, block_size, p: float, padding=(0, 0), stride=(1, 1),
                                   dilation=(1, 1)) -> torch.Tensor:
    bs = _block_size(block_size)
    rows, ncols = conv_patch_matrix_shape(input.shape, kernel.shape, padding, stride, dilation)
    mask = torch.rand(ceil(rows / bs), ceil(ncols / bs), device=input.device) < p
    return naive_blockwise_dropout_conv2d_mask(input, mask, bs, p, kernel, padding, stride, dilation)
