"""CPU oracle for the SparseDrop hot path (block-wise dropout fused into matmul).

TEST INFRASTRUCTURE ONLY.  Nothing that ships (the ``flash_dropout`` package, the
C-ABI library) may import this module; it exists so that tests, the smoke check and
the ``cpu_baseline`` leg of the benchmark have an independent statement of what the
HIP kernels must compute.  Everything is plain numpy, written from the reference's
definitions (paths relative to the reference checkout):

  mask polarity / shape      flash_dropout/functional/utils.py:11-16   (True = dropped, ceil shapes)
  increment table            flash_dropout/functional/utils.py:19-69   (docstring known answer :36-56)
  kept-block table           flash_dropout/functional/blockwise_dropout_matmul_triton.py:48
  forward                    flash_dropout/functional/naive.py:8-25
  backward operand algebra   flash_dropout/functional/blockwise_dropout_matmul_cuda.py:44-53
  gemm_dsd / gemm_sdd        flash_dropout/cuda/src/matmul_dsd.cuh:47-66, matmul_sdd.cuh:44-65
  SDD reference recipe       flash_dropout/cuda/binding_gemm.py:122-129
  im2col conv                flash_dropout/functional/im2col_conv2d.py:5-27  (column = c*R*S + r*S + s)

Parity status of each function (what pins it is in tests/test_oracle.py):
  compact_csr / compact_csc / kept_table   pinned: numpy.nonzero identity, hand cases, brute force
  mask_to_increment_table                  pinned: the reference's docstring known answer
  gemm_dsd / gemm_sdd / dsd_forward /
  sdd_dx / dsd_dw                          pinned: brute-force loops on tiny inputs, p=0 == dense,
                                           single-kept-block closed form, torch autograd of the
                                           literal naive.py restatement (oracle/naive_torch.py)
  im2col / col2im / conv2d_blockdrop       pinned: torch F.unfold / F.fold / F.conv2d library routines
  philox4x32_10 / random_mask              pinned: the Random123 known-answer vectors for Philox4x32-10
                                           (zeros, all ones, digits of pi); the mask on top of it is the
                                           reference's definition ``uniform < p`` (utils.py:15) on a 24-bit
                                           uniform, checked for polarity, p=0 and the empirical rate.  The
                                           reference draws from torch's generator instead: equality of the
                                           random STREAM is not part of the contract (parity is defined for
                                           a given mask), only the distribution is
  split_mask                               pinned: expand_keep identity (same element mask at both sizes)
  merge_mask_quads / compact_csr_quads     pinned: expand_keep identity (the 64-grid mask with its quadrant bits
                                           expands to the same element mask as the block-size-32 mask), hand case
  act_apply / act_grad / dsd_forward_act /
  sdd_dx_actgrad / mlp_forward_backward    pinned: torch's relu / gelu (erf form) and their autograd derivatives;
                                           the MLP against torch autograd through the literal naive.py
                                           restatement with torch activations in between (the composition the
                                           reference's models make, eval/mlp/model.py:31-40, eval/llm/model.py:58-66)
No function here is "parity unpinned".
"""
from __future__ import annotations

import math

import numpy as np

__all__ = [
    "mask_shape",
    "expand_keep",
    "compact_csr",
    "compact_csc",
    "kept_table",
    "mask_to_increment_table",
    "philox4x32_10",
    "random_mask",
    "split_mask",
    "merge_mask_quads",
    "compact_csr_quads",
    "gemm_dsd",
    "gemm_sdd",
    "dsd_forward",
    "sdd_dx",
    "dsd_dw",
    "act_apply",
    "act_grad",
    "dsd_forward_act",
    "sdd_dx_actgrad",
    "mlp_forward_backward",
    "conv_out_hw",
    "im2col",
    "col2im",
    "conv2d_blockdrop",
]


# --------------------------------------------------------------------------------------
# mask + compaction (integer work; bit-exact contract)
# --------------------------------------------------------------------------------------
_PHILOX_M0, _PHILOX_M1 = 0xD2511F53, 0xCD9E8D57
_PHILOX_W0, _PHILOX_W1 = 0x9E3779B9, 0xBB67AE85


def philox4x32_10(counter, key) -> np.ndarray:
    """Philox4x32 with 10 rounds (Salmon, Moraes, Dror, Shaw: "Parallel random numbers: as easy as
    1, 2, 3", SC'11, the generator family torch uses on GPUs).  ``counter`` is [..., 4] and ``key``
    [..., 2] (broadcast), uint32 words; returns [..., 4] uint32.

    One round: (hi0, lo0) = M0*c0, (hi1, lo1) = M1*c2 as 64-bit products;
    c <- (hi1 ^ c1 ^ k0, lo1, hi0 ^ c3 ^ k1, lo0); the key is bumped by (W0, W1) between rounds.
    """
    c = np.array(counter, dtype=np.uint64) & 0xFFFFFFFF
    k = np.array(key, dtype=np.uint64) & 0xFFFFFFFF
    c0, c1, c2, c3 = (c[..., i] for i in range(4))
    k0, k1 = k[..., 0], k[..., 1]
    for _ in range(10):
        p0 = _PHILOX_M0 * c0  # < 2^64: fits uint64 exactly
        p1 = _PHILOX_M1 * c2
        c0, c1, c2, c3 = ((p1 >> 32) ^ c1 ^ k0, p1 & 0xFFFFFFFF, (p0 >> 32) ^ c3 ^ k1, p0 & 0xFFFFFFFF)
        k0 = (k0 + _PHILOX_W0) & 0xFFFFFFFF
        k1 = (k1 + _PHILOX_W1) & 0xFFFFFFFF
    return np.stack(np.broadcast_arrays(c0, c1, c2, c3), axis=-1).astype(np.uint32)


def random_mask(shape: tuple[int, int], p: float, seed: int, offset: int = 0) -> np.ndarray:
    """The block mask the library draws for (seed, offset): bool [mb, kb], True = dropped with
    probability p — the reference's ``torch.rand(mb, kb) < p`` (utils.py:15) on a counter-based stream.

    Entry e = i*kb + j takes word e % 4 of philox4x32_10(counter=(lo32(e//4), hi32(e//4),
    lo32(offset), hi32(offset)), key=(lo32(seed), hi32(seed))); its top 24 bits make a uniform in
    [0, 1) (exact in float32), compared with float32(p)."""
    mb, kb = shape
    e = np.arange(mb * kb, dtype=np.uint64)
    blk = e >> np.uint64(2)
    ctr = np.stack([blk & 0xFFFFFFFF, blk >> np.uint64(32),
                    np.full_like(blk, offset & 0xFFFFFFFF), np.full_like(blk, (offset >> 32) & 0xFFFFFFFF)], axis=-1)
    words = philox4x32_10(ctr, [seed & 0xFFFFFFFF, (seed >> 32) & 0xFFFFFFFF])
    w = words[np.arange(mb * kb), (e & np.uint64(3)).astype(np.int64)]
    u = (w >> np.uint32(8)).astype(np.float32) * np.float32(2.0 ** -24)
    return (u < np.float32(p)).reshape(mb, kb)


def split_mask(mask: np.ndarray, split: int, grid: tuple[int, int] | None = None) -> np.ndarray:
    """Block splitting: every entry repeated split x split times, cropped to ``grid``.  A mask at
    block size bs*split over an [m, k] matrix and its split at block size bs with
    grid = mask_shape(m, k, bs) expand to the same element mask (naive.py:18-23 zeroes whole tiles)."""
    mask = np.asarray(mask, dtype=bool)
    out = np.repeat(np.repeat(mask, split, axis=0), split, axis=1)
    if grid is not None:
        assert (mask.shape[0] - 1) * split < grid[0] <= mask.shape[0] * split, (mask.shape, split, grid)
        assert (mask.shape[1] - 1) * split < grid[1] <= mask.shape[1] * split, (mask.shape, split, grid)
        out = out[: grid[0], : grid[1]]
    return out

def merge_mask_quads(mask: np.ndarray) -> tuple[np.ndarray, np.ndarray]:
    """A block-size-32 mask on the 64 grid: (mask64, quads).  mask64[i, j] is True (dropped) when all of the (up to)
    four entries (2i + a, 2j + b) are; quads[i, j] has bit 2a + b set when entry (2i + a, 2j + b) exists and is
    kept.  This is the report's block splitting read downwards (report.pdf section 3.3): the kernels' 64 x 64 tile
    covers four logical blocks."""
    mask = np.asarray(mask, dtype=bool)
    mb, kb = mask.shape
    ob, ok = (mb + 1) // 2, (kb + 1) // 2
    padded = np.ones((2 * ob, 2 * ok), dtype=bool)
    padded[:mb, :kb] = mask
    quads = np.zeros((ob, ok), dtype=np.uint8)
    for a in range(2):
        for b in range(2):
            quads |= (~padded[a::2, b::2]).astype(np.uint8) << (2 * a + b)
    return quads == 0, quads


def compact_csr_quads(mask: np.ndarray) -> tuple[np.ndarray, np.ndarray]:
    """CSR list of merge_mask_quads(mask) with each entry's quadrant bits in bits 28-31, as int32 (the encoding
    of the library's lists for block size 32).  For the list by columns call it on mask.T."""
    mask64, quads = merge_mask_quads(mask)
    row_ptr, col_idx = compact_csr(mask64)
    rows = np.repeat(np.arange(mask64.shape[0]), np.diff(row_ptr))
    enc = col_idx.astype(np.uint32) | (quads[rows, col_idx].astype(np.uint32) << 28)
    return row_ptr, enc.view(np.int32)


def mask_shape(m: int, k: int, block_size: int) -> tuple[int, int]:
    """Shape of the block mask of an [m, k] matrix (utils.py:13-14: ceil on both axes)."""
    return (math.ceil(m / block_size), math.ceil(k / block_size))


def expand_keep(mask: np.ndarray, block_size: int, m: int, k: int) -> np.ndarray:
    """Element-granular KEEP matrix [m, k] from the block mask (True = dropped, utils.py:15).

    Each mask entry covers a block_size x block_size tile; tiles on the bottom / right edge
    are cropped, which is what a ceil-shaped mask means for a matrix that is not a multiple
    of the block size.
    """
    mask = np.asarray(mask, dtype=bool)
    assert mask.shape == mask_shape(m, k, block_size), (mask.shape, (m, k, block_size))
    keep = ~mask
    return np.repeat(np.repeat(keep, block_size, axis=0), block_size, axis=1)[:m, :k]


def compact_csr(mask: np.ndarray) -> tuple[np.ndarray, np.ndarray]:
    """Per-row-block list of kept column blocks.

    row_ptr[int32, Mb+1], col_idx[int32, nnz]; row r's kept blocks are
    col_idx[row_ptr[r]:row_ptr[r+1]], ascending.  Concatenated this is exactly the
    second column of nonzero(~mask) (blockwise_dropout_matmul_triton.py:48).
    """
    keep = ~np.asarray(mask, dtype=bool)
    widths = keep.sum(axis=1)
    row_ptr = np.zeros(keep.shape[0] + 1, dtype=np.int32)
    np.cumsum(widths, out=row_ptr[1:])
    col_idx = np.nonzero(keep)[1].astype(np.int32)
    return row_ptr, col_idx


def compact_csc(mask: np.ndarray) -> tuple[np.ndarray, np.ndarray]:
    """Per-column-block list of kept row blocks (the CSR of mask.T): col_ptr[Kb+1], row_idx[nnz].

    This is the skip list of the weight-gradient product, which the reference expresses as
    gemm_dsd(X.T, dY.T, mask.T) (blockwise_dropout_matmul_cuda.py:49-51).
    """
    return compact_csr(np.asarray(mask, dtype=bool).T)


def kept_table(mask: np.ndarray) -> np.ndarray:
    """[nnz, 2] int64 (row_blk, col_blk) of kept blocks in row-major order (…_triton.py:48)."""
    r, c = np.nonzero(~np.asarray(mask, dtype=bool))
    return np.stack([r, c], axis=1).astype(np.int64)


def mask_to_increment_table(mask: np.ndarray, block_k: int):
    """Pointer-increment table of utils.py:19-69.

    offsets = kept column index * block_k in row-major order; table = first difference of
    offsets, except that each row's first entry is the absolute offset (utils.py:63-67).
    Rows whose start index is past the end of the table (trailing rows with nothing kept)
    are skipped when patching, as the reference does (:64-67).  A row with nothing kept that
    is *followed* by a non-empty row shares its start index with that row, so the patch
    lands on the next row's first entry — which is that entry's absolute offset, as wanted.
    Returns (table[int64, nnz], row_indices[int64, Mb], row_widths[int64, Mb]).
    """
    keep = ~np.asarray(mask, dtype=bool)
    row_widths = keep.sum(axis=1).astype(np.int64)
    row_indices = np.zeros(keep.shape[0], dtype=np.int64)
    row_indices[1:] = np.cumsum(row_widths[:-1])
    offsets = np.nonzero(keep)[1].astype(np.int64) * block_k
    table = np.diff(offsets, prepend=np.int64(0))
    in_range = row_indices[row_indices < len(table)]
    table[in_range] = offsets[in_range]
    return table, row_indices, row_widths


# --------------------------------------------------------------------------------------
# the three products
# --------------------------------------------------------------------------------------
def gemm_dsd(a, b, mask, block_size: int, scale: float, dtype=np.float64) -> np.ndarray:
    """C[M,N] = scale * (A ⊙ keep) @ B.T with A[M,K], B[N,K], mask over A (matmul_dsd.cuh:47-66)."""
    a = np.asarray(a, dtype=dtype)
    b = np.asarray(b, dtype=dtype)
    m, k = a.shape
    keep = expand_keep(mask, block_size, m, k)
    return (np.where(keep, a, 0) @ b.T) * dtype(scale)


def gemm_sdd(a, b, mask, block_size: int, scale: float, dtype=np.float64) -> np.ndarray:
    """C[M,N] = scale * (A @ B.T) ⊙ keep with mask over the OUTPUT (matmul_sdd.cuh:44-65).

    Dropped tiles are exactly zero (the kernel writes cleared accumulators)."""
    a = np.asarray(a, dtype=dtype)
    b = np.asarray(b, dtype=dtype)
    m, n = a.shape[0], b.shape[0]
    keep = expand_keep(mask, block_size, m, n)
    return np.where(keep, (a @ b.T) * dtype(scale), 0)


def dsd_forward(x, w, mask, block_size: int, p: float, dtype=np.float64) -> np.ndarray:
    """Y = (keep ⊙ X)/(1-p) @ W.T  (naive.py:8-25)."""
    assert 0 <= p < 1
    return gemm_dsd(x, w, mask, block_size, 1.0 / (1.0 - p), dtype)


def sdd_dx(dy, w, mask, block_size: int, p: float, dtype=np.float64) -> np.ndarray:
    """dX = (dY @ W) ⊙ keep /(1-p): gemm_sdd(dY, W.T, mask)  (…_cuda.py:46)."""
    assert 0 <= p < 1
    w = np.asarray(w, dtype=dtype)
    return gemm_sdd(dy, w.T, mask, block_size, 1.0 / (1.0 - p), dtype)


def dsd_dw(dy, x, mask, block_size: int, p: float, dtype=np.float64) -> np.ndarray:
    """dW[N,K] = dY.T @ (keep ⊙ X)/(1-p): gemm_dsd(X.T, dY.T, mask.T).T  (…_cuda.py:49-51)."""
    assert 0 <= p < 1
    x = np.asarray(x, dtype=dtype)
    dy = np.asarray(dy, dtype=dtype)
    mask = np.asarray(mask, dtype=bool)
    return gemm_dsd(x.T, dy.T, mask.T, block_size, 1.0 / (1.0 - p), dtype).T


# --------------------------------------------------------------------------------------
# activations between dropout-linear layers (what the fused epilogues compute)
# --------------------------------------------------------------------------------------
_erf = np.vectorize(math.erf, otypes=[np.float64])


def act_apply(x, act: str | None) -> np.ndarray:
    """relu(x) = max(x, 0); gelu(x) = x * Phi(x), the exact (erf) form that torch.nn.GELU() defaults to
    (the reference's models: nn.ReLU eval/mlp/model.py:29, nn.GELU eval/llm/model.py:59)."""
    x = np.asarray(x, dtype=np.float64)
    if act in (None, "none"):
        return x
    if act == "relu":
        return np.maximum(x, 0.0)
    if act == "gelu":
        return 0.5 * x * (1.0 + _erf(x / math.sqrt(2.0)))
    raise ValueError(f"unknown activation {act!r}")


def act_grad(x, act: str | None) -> np.ndarray:
    """d act(x) / dx: relu' = [x > 0]; gelu' = Phi(x) + x * phi(x)."""
    x = np.asarray(x, dtype=np.float64)
    if act in (None, "none"):
        return np.ones_like(x)
    if act == "relu":
        return (x > 0).astype(np.float64)
    if act == "gelu":
        return 0.5 * (1.0 + _erf(x / math.sqrt(2.0))) + x * np.exp(-0.5 * x * x) / math.sqrt(2.0 * math.pi)
    raise ValueError(f"unknown activation {act!r}")


def dsd_forward_act(x, w, mask, block_size: int, p: float, act: str | None, dtype=np.float64):
    """(act(Y), Y) with Y = dsd_forward(...): the activation follows the dropout-linear layer
    (eval/mlp/model.py:33-34: ``x = self.in_proj(x); x = self.act(x)``)."""
    pre = dsd_forward(x, w, mask, block_size, p, np.float64)
    return act_apply(pre, act).astype(dtype), pre.astype(dtype)


def sdd_dx_actgrad(dy, w, mask, block_size: int, p: float, act: str | None, act_at, dtype=np.float64):
    """Input gradient of a dropout-linear layer whose input was act(act_at), taken one step further to the
    gradient with respect to act_at: sdd_dx(...) * act'(act_at) (chain rule through eval/mlp/model.py:34)."""
    dx = sdd_dx(dy, w, mask, block_size, p, np.float64)
    return (dx * act_grad(act_at, act)).astype(dtype)


def mlp_forward_backward(x, weights, masks, block_size: int, p: float, act: str | None, dy, dtype=np.float64,
                         hidden_dtype=None):
    """The reference's MLPs (eval/mlp/model.py:31-40; eval/llm/model.py:62-66): dropout-linear layers with an
    activation between consecutive ones (none after the last).  Returns (out, dx, [dW_i]) for the upstream
    gradient dy, by the chain rule over dsd_forward / sdd_dx / dsd_dw.

    ``hidden_dtype`` (e.g. np.float16): hidden tensors are stored in that type between layers, as they are under
    the reference's autocast contract (blockwise_dropout_matmul_cuda.py:9): the pre-activation and the activated
    tensor are each rounded once, the next layer and the activation's derivative see the rounded values, and the
    backward is the exact chain rule of that computation with the roundings taken as identities.  Without it
    nothing is rounded.  (It matters for ReLU: a rounding upstream moves pre-activations near zero across the
    kink, which a comparison must not count as an error of the products.)"""
    rnd = (lambda a: a) if hidden_dtype is None else (lambda a: a.astype(hidden_dtype).astype(np.float64))
    ps = [float(p)] * len(weights) if np.isscalar(p) else [float(v) for v in p]  # one drop rate, or one per layer
    assert len(ps) == len(weights)
    h = np.asarray(x, dtype=np.float64)
    inputs, pres = [], []
    for i, (w, m) in enumerate(zip(weights, masks)):
        inputs.append(h)
        pre = dsd_forward(h, np.asarray(w, dtype=np.float64), m, block_size, ps[i], np.float64)
        if i + 1 < len(weights):
            pres.append(rnd(pre))
            h = rnd(act_apply(pre, act))
        else:
            pres.append(pre)
            h = pre
    out = h
    g = np.asarray(dy, dtype=np.float64)  # gradient with respect to the current layer's pre-activation
    dws = [None] * len(weights)
    for i in reversed(range(len(weights))):
        w = np.asarray(weights[i], dtype=np.float64)
        dws[i] = dsd_dw(g, inputs[i], masks[i], block_size, ps[i], np.float64).astype(dtype)
        g = sdd_dx(g, w, masks[i], block_size, ps[i], np.float64)
        if i > 0:
            # ReLU's derivative can be read off either tensor (same sign); GELU's is evaluated at the stored
            # pre-activation
            g = g * act_grad(inputs[i] if act == "relu" else pres[i - 1], act)
    return out.astype(dtype), g.astype(dtype), dws


# --------------------------------------------------------------------------------------
# conv via im2col
# --------------------------------------------------------------------------------------
def conv_out_hw(h, w, r, s, padding, stride, dilation) -> tuple[int, int]:
    """Output extent P, Q (im2col_conv2d.py:14-15)."""
    p_ = (h + 2 * padding[0] - dilation[0] * (r - 1) - 1) // stride[0] + 1
    q_ = (w + 2 * padding[1] - dilation[1] * (s - 1) - 1) // stride[1] + 1
    return p_, q_


def im2col(x, r: int, s: int, padding=(0, 0), stride=(1, 1), dilation=(1, 1)) -> np.ndarray:
    """[N*P*Q, C*R*S] patch matrix; row = (n, p, q), column = c*R*S + rr*S + ss
    (F.unfold order, im2col_conv2d.py:17-20).  Out-of-image taps read zero."""
    x = np.asarray(x)
    n, c, h, w = x.shape
    p_, q_ = conv_out_hw(h, w, r, s, padding, stride, dilation)
    xp = np.zeros((n, c, h + 2 * padding[0], w + 2 * padding[1]), dtype=x.dtype)
    xp[:, :, padding[0]:padding[0] + h, padding[1]:padding[1] + w] = x
    cols = np.zeros((n, p_, q_, c, r, s), dtype=x.dtype)
    for rr in range(r):
        for ss in range(s):
            h0 = rr * dilation[0]
            w0 = ss * dilation[1]
            patch = xp[:, :, h0:h0 + (p_ - 1) * stride[0] + 1:stride[0],
                       w0:w0 + (q_ - 1) * stride[1] + 1:stride[1]]  # n c p q
            cols[:, :, :, :, rr, ss] = patch.transpose(0, 2, 3, 1)
    return cols.reshape(n * p_ * q_, c * r * s)


def col2im(cols, x_shape, r: int, s: int, padding=(0, 0), stride=(1, 1), dilation=(1, 1)) -> np.ndarray:
    """Adjoint of im2col: scatter-add a [N*P*Q, C*R*S] matrix back to [N,C,H,W]."""
    n, c, h, w = x_shape
    p_, q_ = conv_out_hw(h, w, r, s, padding, stride, dilation)
    cols = np.asarray(cols).reshape(n, p_, q_, c, r, s)
    xp = np.zeros((n, c, h + 2 * padding[0], w + 2 * padding[1]), dtype=cols.dtype)
    for rr in range(r):
        for ss in range(s):
            h0 = rr * dilation[0]
            w0 = ss * dilation[1]
            xp[:, :, h0:h0 + (p_ - 1) * stride[0] + 1:stride[0],
               w0:w0 + (q_ - 1) * stride[1] + 1:stride[1]] += cols[:, :, :, :, rr, ss].transpose(0, 3, 1, 2)
    return xp[:, :, padding[0]:padding[0] + h, padding[1]:padding[1] + w]


def conv2d_blockdrop(x, kernel, mask, block_size: int, p: float, padding=(0, 0), stride=(1, 1),
                     dilation=(1, 1), dy=None, dtype=np.float64):
    """Block dropout applied to the im2col matrix, then the linear layer, then back to NKPQ.

    The reference never finished this variant (layers/dropout_conv.py:86-99 are comments), so
    the oracle is *defined* by composition: im2col (im2col_conv2d.py:17-20) -> dsd_forward
    (naive.py:8-25) -> reshape (im2col_conv2d.py:24-25).  ``mask`` is over [N*P*Q, C*R*S].
    With ``dy`` [N,K,P,Q] also returns (dx [N,C,H,W], dkernel [K,C,R,S]).
    """
    x = np.asarray(x, dtype=dtype)
    kernel = np.asarray(kernel, dtype=dtype)
    n, c, h, w = x.shape
    kk, _, r, s = kernel.shape
    p_, q_ = conv_out_hw(h, w, r, s, padding, stride, dilation)
    cols = im2col(x, r, s, padding, stride, dilation)
    w2 = kernel.reshape(kk, c * r * s)
    y2 = dsd_forward(cols, w2, mask, block_size, p, dtype)  # [N*P*Q, K]
    y = y2.reshape(n, p_ * q_, kk).transpose(0, 2, 1).reshape(n, kk, p_, q_)
    if dy is None:
        return y
    dy2 = np.asarray(dy, dtype=dtype).reshape(n, kk, p_ * q_).transpose(0, 2, 1).reshape(n * p_ * q_, kk)
    dcols = sdd_dx(dy2, w2, mask, block_size, p, dtype)
    dx = col2im(dcols, x.shape, r, s, padding, stride, dilation)
    dw2 = dsd_dw(dy2, cols, mask, block_size, p, dtype)
    return y, dx, dw2.reshape(kernel.shape)
