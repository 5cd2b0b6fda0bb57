"""A stack of dropout-linear layers with an activation between consecutive ones, as ONE autograd function whose
GEMM epilogues do the activation work.

The reference's models interleave exactly this (eval/mlp/model.py:31-40: DropoutMM, ReLU, DropoutMM, ..., DropoutMM;
eval/llm/model.py:62-66: DropoutMM, GELU, DropoutMM) as separate modules, i.e. one elementwise kernel per
activation in forward and one in backward, each a full pass over the hidden activations.  Here

    forward   h_{i+1} = act(s_i (keep_i ⊙ h_i) W_i^T)     the activation is applied to the fp32 accumulator in the
                                                            DSD kernel's store (sd_gemm_dsd_lists_act)
    backward  g_{i-1} = (s_i (g_i W_i) ⊙ keep_i) ⊙ act'     the derivative is multiplied in the SDD kernel's store
                                                            (sd_gemm_sdd_lists_actgrad); g_i is the gradient with
                                                            respect to layer i's pre-activation
              dW_i    = s_i g_i^T (keep_i ⊙ h_i)

so no activation kernel is launched in either direction.  ReLU's derivative is read off the activated tensor
(already kept as the next layer's input); GELU keeps the pre-activation as well.
"""
from __future__ import annotations

import torch

from ..hip.binding_gemm import GEMM, KeptLists, _activation, _block_size, as_matrix
from .blockwise_dropout_matmul_hip import _apply_outside_autocast


class BlockwiseDropoutMLPHIP(torch.autograd.Function):
    @staticmethod
    def forward(ctx, input: torch.Tensor, block_size: int, ps: tuple, activation, seed, masks, *weights):
        ext = GEMM()
        n = len(weights)
        h = input
        saved, shapes, kbs = [input], [], []
        for i, w in enumerate(weights):
            p = ps[i]
            last = i + 1 == n
            if i == 0 and p == 0.0 and masks is None and not ctx.needs_input_grad[0]:
                # a first layer without dropout whose input needs no gradient (the reference's models start with one,
                # eval/mlp/model.py:31-33): the dense product with the same fused store, no mask and no lists
                out, pre = ext.gemm_act(h, w, None if last else activation,
                                        want_pre=(not last and activation == "gelu"))
                empty = out.new_empty(0)
                saved += [w, empty, empty, empty, empty, empty, pre if pre is not None else empty]
                if not last:
                    saved.append(out)
                shapes.append(None)
                kbs.append(0)
                h = out
                continue
            # mask, lists and product in one library call (one launch for small layers)
            out, mask, lists, kernel_bs, pre = ext.dropout_matmul_forward_act(
                h, w, block_size, p, None if masks is None else masks[i], None if seed is None else seed + i,
                activation=None if last else activation, want_pre=(not last and activation == "gelu"))
            if last or activation is None:
                pre = None
            # per layer: weight, mask, the four list arrays, what the activation's derivative is evaluated at
            # (GELU: the pre-activation; ReLU: nothing extra, the activated output is the next layer's input)
            saved += [w, mask, lists.row_ptr, lists.col_idx, lists.col_ptr, lists.row_idx]
            saved.append(pre if pre is not None else out.new_empty(0))
            if not last:
                saved.append(out)
            shapes.append(lists.shape)
            kbs.append(kernel_bs)
            h = out
        ctx.save_for_backward(*saved)
        ctx.n, ctx.ps, ctx.activation, ctx.shapes, ctx.kbs = n, ps, activation, shapes, kbs
        return h

    @staticmethod
    def backward(ctx, grad_output: torch.Tensor):
        ext = GEMM()
        t = ctx.saved_tensors
        n, act = ctx.n, ctx.activation
        # unpack: input, then per layer (w, mask, row_ptr, col_idx, col_ptr, row_idx, pre, [out])
        hs, layers, pos = [t[0]], [], 1
        for i in range(n):
            w, _, rp, ci, cp, ri, pre = t[pos:pos + 7]
            pos += 7
            layers.append((w, KeptLists(rp, ci, cp, ri, ctx.shapes[i]) if ctx.shapes[i] is not None else None, pre))
            if i + 1 < n:
                hs.append(t[pos])
                pos += 1
        g = grad_output if grad_output.dtype == hs[0].dtype else grad_output.to(hs[0].dtype)
        g = as_matrix(g)
        grads_w = [None] * n
        for i in reversed(range(n)):
            w, lists, _ = layers[i]
            need_w = ctx.needs_input_grad[6 + i]
            need_in = i > 0 or ctx.needs_input_grad[0]
            if lists is None:  # the dense first layer: only its weight gradient is wanted, dW = g^T . h
                if need_w:
                    if w.shape[0] % 8:
                        # the library's kernels take gradients whose width is a multiple of 8 (the 16 bytes of a
                        # lane's load): zero columns up to the next one, as the dropout layers' narrow heads do
                        n8 = -(-w.shape[0] // 8) * 8
                        gp = g.new_zeros(g.shape[0], n8)
                        gp[:, : w.shape[0]] = g
                        grads_w[i] = ext.gemm(gp.t(), hs[i].t())[: w.shape[0]]
                    else:
                        grads_w[i] = ext.gemm(g.t(), hs[i].t())
                break
            at = None
            if i > 0 and need_in and act is not None:
                prev_pre = layers[i - 1][2]
                at = prev_pre if prev_pre.numel() else hs[i]  # GELU: pre-activation; ReLU: the activated input
            # both gradients of the layer in one library call (one launch for small layers), the activation's
            # derivative riding on the dX store
            dx, dw = ext.dropout_matmul_backward(g, w, hs[i], lists, ctx.kbs[i], ctx.ps[i], need_dx=need_in,
                                                 need_dw=need_w, activation=act if at is not None else None, act_at=at)
            if need_w:
                grads_w[i] = dw
            if not need_in:
                break
            g = dx
        grad_in = g if ctx.needs_input_grad[0] else None
        return (grad_in, None, None, None, None, None, *grads_w)


def blockwise_dropout_mlp(input: torch.Tensor, weights, block_size, p, activation: str | None = "relu",
                          masks=None, seed: int | None = None) -> torch.Tensor:
    """``W_n drop(act(... W_2 drop(act(W_1 drop(x))) ...))``: every layer drops blocks of its INPUT with
    probability p (a number, or one per layer; 0 keeps everything) and scales by 1/(1-p), ``activation``
    ("relu", "gelu" or None) sits between consecutive layers, none after the last.  ``masks`` (one bool mask per
    layer, True = dropped) pins the masks, ``seed`` pins the draws (layer i uses seed + i); otherwise they come
    from the device-resident generator.  ``input`` is [M, K], ``weights[i]`` is [out_i, in_i].

    With the device-resident generator a first layer with p = 0 whose input needs no gradient draws nothing (it runs as
    a dense product): the following layers then use the generator's draws 0, 1, ...; when the input does require a
    gradient that layer draws its (all kept) mask as well and the others use the draws 1, 2, ....  Results are valid
    either way; pass ``seed`` or ``masks`` where a run must not depend on it."""
    weights = list(weights)
    if not weights:
        raise ValueError("at least one layer is needed")
    ps = tuple(float(p) for _ in weights) if isinstance(p, (int, float)) else tuple(float(v) for v in p)
    if len(ps) != len(weights) or any(not 0 <= v < 1 for v in ps):
        raise ValueError("p must be one probability in [0, 1), or one per layer")
    _activation(activation)
    if masks is not None and len(masks) != len(weights):
        raise ValueError("one mask per layer is needed")
    bs = _block_size(block_size)
    if input.dim() != 2 or any(w.dim() != 2 for w in weights):
        raise ValueError("input must be [M, K] and every weight [out, in]")
    tensors = [input, *weights]
    if torch.is_autocast_enabled("cuda"):  # the autocast contract of the single layer (…_cuda.py:9)
        dt = torch.get_autocast_dtype("cuda")
        tensors = [t.to(dt) for t in tensors]
    x, *ws = (as_matrix(t) for t in tensors)
    return _apply_outside_autocast(BlockwiseDropoutMLPHIP, x, bs, ps, activation, seed,
                                   None if masks is None else tuple(masks), *ws)
