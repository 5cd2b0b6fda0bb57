"""Python face of the C ABI: the counterpart of the reference's ``flash_dropout/cuda/binding_gemm.py``.

``GEMM`` keeps the reference's three methods with the same argument meaning
(binding_gemm.py:26-47: ``gemm(A, B)``, ``gemm_dsd(A, B, mask, block_size, scale)``,
``gemm_sdd(A, B, mask, block_size, scale)``; A is [M, K], B is [N, K], each row- or column-major,
result a new row-major [M, N] tensor) and adds what the HIP path needs on top: the kept-block list
builder, list-taking GEMMs (so forward and backward share one list build), and im2col / col2im.

torch is plumbing here: it owns device memory and the stream; every computation is a call into
libsparsedrop.so with raw pointers.  Tensors must live on the GPU; there is no CPU path.
"""
from __future__ import annotations

import contextlib
from dataclasses import dataclass
from functools import cache
from math import ceil

import torch

from . import _loader

SD_F16, SD_BF16 = 0, 1
_DTYPES = {torch.float16: SD_F16, torch.bfloat16: SD_BF16}
ACTIVATIONS = {None: 0, "none": 0, "relu": 1, "gelu": 2}  # enum sd_act


def _activation(act) -> int:
    if act not in ACTIVATIONS:
        raise ValueError(f"activation {act!r}: expected one of {sorted(k for k in ACTIVATIONS if k)} or None")
    return ACTIVATIONS[act]


class SparseDropError(RuntimeError):
    """A libsparsedrop call returned a non-zero status."""


@dataclass
class KeptLists:
    """Compacted kept-block lists of one block mask (True = dropped), all int32 on the mask's device.

    CSR: kept column blocks of row block r are ``col_idx[row_ptr[r]:row_ptr[r+1]]`` (ascending);
    CSC: kept row blocks of column block c are ``row_idx[col_ptr[c]:col_ptr[c+1]]``.
    ``col_idx`` / ``row_idx`` have capacity Mb*Kb; only the first nnz entries are meaningful.
    """

    row_ptr: torch.Tensor
    col_idx: torch.Tensor
    col_ptr: torch.Tensor
    row_idx: torch.Tensor
    shape: tuple[int, int]

    def nnz(self) -> int:
        """Number of kept blocks (synchronises with the device)."""
        return int(self.row_ptr[-1].item())

    def transposed(self) -> "KeptLists":
        """Lists of mask.T: CSR and CSC swap roles."""
        return KeptLists(self.col_ptr, self.row_idx, self.row_ptr, self.col_idx,
                         (self.shape[1], self.shape[0]))


_NO_GUARD = contextlib.nullcontext()

# torch keeps a fast accessor for the raw current-stream handle (an order of magnitude cheaper than building
# a Stream object per launch); fall back to the public API where it is missing
_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None) or (
    lambda index: torch.cuda.current_stream(index).cuda_stream)


def _device(device) -> torch.device:
    dev = torch.device("cuda") if device is None else torch.device(device)
    if dev.index is None:
        dev = torch.device("cuda", torch.cuda.current_device())
    return dev


def _guard(dev: torch.device):
    """Makes ``dev`` the current device for a launch; free when it already is."""
    return _NO_GUARD if dev.index == torch.cuda.current_device() else torch.cuda.device(dev)


def _block_size(block_size) -> int:
    """int, or a (bm, bk) pair with bm == bk (the reference's configs pass (128, 128) tuples,
    eval/mlp/config.py:26, while its kernels take an int, gemm_binding.cu:82-83)."""
    if isinstance(block_size, (tuple, list)):
        if len(block_size) != 2 or block_size[0] != block_size[1]:
            raise ValueError(f"block_size must be an int or a pair of equal ints, got {block_size!r}")
        block_size = block_size[0]
    if int(block_size) != block_size or block_size <= 0:
        raise ValueError(f"block_size must be a positive integer, got {block_size!r}")
    return int(block_size)


def _list_grid_size(bs: int) -> int:
    """Edge of the blocks the kept-block lists are over: 64 for an odd multiple of 32 (the lists then carry, in the
    top four bits of every entry, which of the entry's four 32-blocks are kept), else the block size."""
    return 64 if bs % 64 == 32 else bs


def _check_operand(name: str, x: torch.Tensor) -> None:
    # same rules as the reference's check_operand + dtype checks (gemm_binding.cu:18-22, 87-89)
    if not isinstance(x, torch.Tensor):
        raise TypeError(f"{name} must be a tensor")
    if not x.is_cuda:
        raise ValueError(f"{name} must be on the GPU (got {x.device})")
    if x.dim() != 2:
        raise ValueError(f"{name} must be 2D (got {x.dim()}D)")
    if x.dtype not in _DTYPES:
        raise TypeError(f"{name} must be float16 or bfloat16 (got {x.dtype})")
    if x.numel() and x.stride(0) != 1 and x.stride(1) != 1:
        raise ValueError(f"{name} must be row or column major (strides {x.stride()})")


def _mat(x: torch.Tensor):
    """(pointer, row stride, column stride) in elements.  The stride of an extent-1 dimension is arbitrary in
    torch and normalised here; a zero stride over a real extent (an expanded tensor) is not a matrix in memory."""
    sr, sc = x.stride()
    rows, cols = x.shape
    if (rows > 1 and sr == 0) or (cols > 1 and sc == 0):
        raise ValueError(f"operand is an expanded view (strides {x.stride()}): call .contiguous() first")
    if rows <= 1 and sc == 1:
        sr = max(cols, 1)
    if cols <= 1 and sr == 1:
        sc = max(rows, 1)
    return x.data_ptr(), max(sr, 1), max(sc, 1)


def as_matrix(x: torch.Tensor) -> torch.Tensor:
    """``x`` itself when it is a row- or column-major matrix in memory (unit stride along one index, the other
    stride at least the contiguous extent), else a contiguous copy: expanded gradients (stride 0, e.g. from
    ``y.sum(0)``), overlapping or doubly strided views."""
    rows, cols = x.shape
    sr, sc = x.stride()
    if sc == 1 and (rows <= 1 or sr >= cols):
        return x
    if sr == 1 and (cols <= 1 or sc >= rows):
        return x
    return x.contiguous()


def _check_mask(mask: torch.Tensor, shape: tuple[int, int], like: torch.Tensor) -> torch.Tensor:
    if mask.dtype != torch.bool:
        raise TypeError(f"Mask must be bool (got {mask.dtype})")
    if mask.device != like.device:
        raise ValueError("mask must be on the same device as the operands")
    if tuple(mask.shape) != shape:
        raise ValueError(f"mask shape {tuple(mask.shape)} does not match blocks {shape}")
    if mask.numel() and mask.stride(0) != 1 and mask.stride(1) != 1:
        mask = mask.contiguous()
    return mask


def _mask_strides(mask: torch.Tensor):
    sr, sc = mask.stride()
    if sr != 1 and sc != 1:  # only possible for degenerate shapes
        sr, sc = mask.shape[1], 1
    return max(sr, 1), max(sc, 1)


@cache
class GEMM:
    """Process-wide handle on libsparsedrop.so (the reference caches its JIT-built module the same
    way, binding_gemm.py:7)."""

    def __init__(self) -> None:
        self.lib = _loader.load()
        self._rng: dict[int, tuple[int, torch.Tensor]] = {}  # device index -> (torch seed it follows, state)

    def last_kernel(self) -> str:
        """"specialised" or "generic": the kernel family this thread's last GEMM call ran on."""
        return self.lib.sd_last_kernel().decode()

    def last_kernel_detail(self) -> str:
        """Kernel, workgroup shape and reduction splits of this thread's last launch, e.g. "sdd:big"."""
        return self.lib.sd_last_kernel_detail().decode()

    TILE_POLICIES = {"auto": 0, "big": 1, "mid": 2}

    def set_tile_policy(self, policy: str) -> str:
        """Workgroup shape of the specialised DSD / dense kernels for every later call of the process:
        "auto" (from the shape), "big" (256 x 256 output tiles) or "mid" (128 x 128).  Returns the
        previous setting.  A tuning and test hook."""
        if policy not in self.TILE_POLICIES:
            raise ValueError(f"tile policy {policy!r}: expected one of {sorted(self.TILE_POLICIES)}")
        prev = self.lib.sd_set_tile_policy(self.TILE_POLICIES[policy])
        return {v: k for k, v in self.TILE_POLICIES.items()}[prev]

    # ------------------------------------------------------------------ plumbing
    def _call(self, fn, *args) -> None:
        rc = fn(*args)
        if rc != 0:
            msg = self.lib.sd_last_error().decode(errors="replace")
            exc = {1: ValueError, 2: NotImplementedError}.get(rc, SparseDropError)
            raise exc(f"{fn.__name__}: {msg}")

    @staticmethod
    def _stream(t: torch.Tensor) -> int:
        """Raw handle of torch's current stream on the tensor's device (what the launches go to)."""
        return _raw_stream(t.device.index)

    def _check_pair(self, A, B):
        _check_operand("A", A)
        _check_operand("B", B)
        if A.dtype != B.dtype:
            raise TypeError(f"A and B must have the same dtype ({A.dtype} vs {B.dtype})")
        if A.device != B.device:
            raise ValueError("A and B must be on the same device")
        if A.shape[1] != B.shape[1]:
            raise ValueError(f"reduction dims differ: A {tuple(A.shape)}, B {tuple(B.shape)}")

    @staticmethod
    def _out(A, B, out, transposed_out):
        M, N = A.shape[0], B.shape[0]
        if out is None:
            if transposed_out:
                return torch.empty((N, M), dtype=A.dtype, device=A.device).t()
            return torch.empty((M, N), dtype=A.dtype, device=A.device)
        if tuple(out.shape) != (M, N) or out.dtype != A.dtype or out.device != A.device:
            raise ValueError("out has the wrong shape, dtype or device")
        _check_operand("out", out)
        return out

    # ------------------------------------------------------------------ reference methods
    def gemm(self, A: torch.Tensor, B: torch.Tensor, out=None, transposed_out=False) -> torch.Tensor:
        """Dense ``A @ B.T`` (reference: binding_gemm.py:26-27)."""
        self._check_pair(A, B)
        C = self._out(A, B, out, transposed_out)
        if A.shape[0] == 0 or B.shape[0] == 0:
            return C
        ws, ws_ptr, ws_bytes = self._splitk_scratch(A, B, 0, 0)
        with _guard(A.device):
            self._call(self.lib.sd_gemm, *_mat(A), *_mat(B), *_mat(C), A.shape[0], B.shape[0],
                       A.shape[1], _DTYPES[A.dtype], ws_ptr, ws_bytes, self._stream(A))
        return C

    def _splitk_scratch(self, A, B, bs, sparse):
        """fp32 scratch for a split reduction, when the library wants one for this shape."""
        nbytes = self.lib.sd_splitk_workspace_bytes(A.shape[0], B.shape[0], A.shape[1], bs, sparse)
        if nbytes <= 0:
            return None, None, 0
        ws = torch.empty(nbytes // 4, dtype=torch.float32, device=A.device)
        return ws, ws.data_ptr(), nbytes


    def _masked(self, fn, mask_cols, A, B, mask, block_size, scale, out, transposed_out):
        self._check_pair(A, B)
        bs = _block_size(block_size)
        M, N, K = A.shape[0], B.shape[0], A.shape[1]
        mb, cb = ceil(M / bs), ceil((K if mask_cols == "K" else N) / bs)
        mask = _check_mask(mask, (mb, cb), A)
        C = self._out(A, B, out, transposed_out)
        if M == 0 or N == 0:
            return C
        if bs > 64 and bs % 32 == 0 or bs == 32:  # the 64-granular list: the library splits / merges the mask
            ws_bytes = self.lib.sd_workspace_bytes(ceil(M / 64), ceil((K if mask_cols == "K" else N) / 64))
        else:
            ws_bytes = self.lib.sd_workspace_bytes(mb, cb)
        ws_bytes = (ws_bytes + 15) // 16 * 16
        if mask_cols == "K":
            ws_bytes += self.lib.sd_splitk_workspace_bytes(M, N, K, bs, 1)
        ws = torch.empty((ws_bytes + 3) // 4, dtype=torch.int32, device=A.device)
        with _guard(A.device):
            self._call(fn, *_mat(A), *_mat(B), *_mat(C), mask.data_ptr(), *_mask_strides(mask),
                       M, N, K, bs, float(scale), _DTYPES[A.dtype], ws.data_ptr(), ws_bytes,
                       self._stream(A))
        return C

    def gemm_dsd(self, A, B, mask, block_size, scale, out=None, transposed_out=False) -> torch.Tensor:
        """``scale * (A ⊙ keep) @ B.T`` with ``mask`` [ceil(M/bs), ceil(K/bs)] over A, True = dropped
        (reference: binding_gemm.py:29-37)."""
        return self._masked(self.lib.sd_gemm_dsd, "K", A, B, mask, block_size, scale, out, transposed_out)

    def gemm_dsd_noalloc(self, A, B, mask, block_size, scale, out: torch.Tensor) -> torch.Tensor:
        """:meth:`gemm_dsd` into the caller's ``out`` through the entry point that allocates nothing: the
        kept-block list goes into an array inside the library (about 2**18 mask blocks at most), so calls
        that overlap on one GPU race on it."""
        self._check_pair(A, B)
        bs = _block_size(block_size)
        M, N, K = A.shape[0], B.shape[0], A.shape[1]
        mask = _check_mask(mask, (ceil(M / bs), ceil(K / bs)), A)
        C = self._out(A, B, out, False)
        with _guard(A.device):
            self._call(self.lib.sd_gemm_dsd_noalloc, *_mat(A), *_mat(B), *_mat(C), mask.data_ptr(),
                       *_mask_strides(mask), M, N, K, bs, float(scale), _DTYPES[A.dtype], self._stream(A))
        return C

    def gemm_sdd(self, A, B, mask, block_size, scale, out=None, transposed_out=False) -> torch.Tensor:
        """``scale * (A @ B.T) ⊙ keep`` with ``mask`` [ceil(M/bs), ceil(N/bs)] over the output; dropped
        tiles are written as zeros (reference: binding_gemm.py:39-47)."""
        return self._masked(self.lib.sd_gemm_sdd, "N", A, B, mask, block_size, scale, out, transposed_out)

    # ------------------------------------------------------------------ lists
    @staticmethod
    def _list_grid(mb, kb, split, grid):
        split = int(split)
        if split <= 0:  # a mask of block size 32 * sub: its 32-blocks merged two by two onto the 64 grid
            sub = -split if split else 1
            full = ((mb * sub + 1) // 2, (kb * sub + 1) // 2)
            out_mb, out_kb = full if grid is None else (int(grid[0]), int(grid[1]))
            if not ((mb - 1) * sub < 2 * out_mb and out_mb <= full[0] and (kb - 1) * sub < 2 * out_kb and out_kb <= full[1]):
                raise ValueError(f"grid {(out_mb, out_kb)} of 64-blocks does not match a {(mb, kb)} mask at block size {32 * sub}")
            return split, out_mb, out_kb
        out_mb, out_kb = (mb * split, kb * split) if grid is None else (int(grid[0]), int(grid[1]))
        if not ((mb - 1) * split < out_mb <= mb * split and (kb - 1) * split < out_kb <= kb * split):
            raise ValueError(f"grid {(out_mb, out_kb)} does not match a {(mb, kb)} mask split by {split}")
        return split, out_mb, out_kb

    @staticmethod
    def _list_buffers(out_mb, out_kb, dev):
        # one allocation: row_ptr | col_ptr | col_idx | row_idx
        buf = torch.empty(out_mb + 1 + out_kb + 1 + 2 * out_mb * out_kb, dtype=torch.int32, device=dev)
        return torch.split(buf, [out_mb + 1, out_kb + 1, out_mb * out_kb, out_mb * out_kb])

    def build_lists(self, mask: torch.Tensor, split: int = 1, grid=None) -> KeptLists:
        """Mask -> CSR + CSC kept-block lists in one launch, no host synchronisation.

        ``split`` > 1 lists the mask with every entry repeated split x split times, cropped to
        ``grid`` = (rows, cols) of the finer block grid (default: uncropped): a mask drawn at block
        size 64*split then drives the 64-block kernels.  ``split`` = 0 goes the other way for a mask at block
        size 32: it is listed on the 64 grid, an entry kept when any of its four 32-blocks is, and bits 28-31 of
        the entry say which (bit 2a + b: row half a, column half b; in ``row_idx`` with the halves swapped, as
        the list of the transposed mask needs them); the ``*_lists`` calls take such lists with block size 32."""
        if mask.dim() != 2 or mask.dtype != torch.bool or not mask.is_cuda:
            raise ValueError("mask must be a 2D bool tensor on the GPU")
        mb, kb = mask.shape
        if mb == 0 or kb == 0:
            raise ValueError("mask must be non-empty")
        split, out_mb, out_kb = self._list_grid(mb, kb, split, grid)
        if mask.stride(0) != 1 and mask.stride(1) != 1:
            mask = mask.contiguous()
        row_ptr, col_ptr, col_idx, row_idx = self._list_buffers(out_mb, out_kb, mask.device)
        with _guard(mask.device):
            self._call(self.lib.sd_build_lists_split, mask.data_ptr(), mb, kb, *_mask_strides(mask),
                       split, out_mb, out_kb, row_ptr.data_ptr(), col_idx.data_ptr(), col_ptr.data_ptr(),
                       row_idx.data_ptr(), self._stream(mask))
        return KeptLists(row_ptr, col_idx, col_ptr, row_idx, (out_mb, out_kb))

    def manual_seed(self, seed: int, device=None) -> None:
        """(Re)starts the device-resident mask generator of ``device`` at (seed, offset 0).  Without this
        call the generator starts from ``torch.initial_seed()`` at first use and restarts whenever that
        value changes (``torch.manual_seed`` with a new seed).

        The state is ONE int64[4] tensor per device for the life of the process, reseeded in place by a copy
        on the current stream: reseeding is ordered with the draws on that stream, and a captured graph (which
        holds the tensor's address) follows a later reseed instead of reading freed memory."""
        dev = _device(device)
        seed = int(seed) & (2 ** 64 - 1)
        as_i64 = seed if seed < 2 ** 63 else seed - 2 ** 64
        host = torch.tensor([as_i64, 0, 0, 0], dtype=torch.int64)
        entry = self._rng.get(dev.index)
        if entry is None:
            state = host.to(dev)
        else:
            state = entry[1]
            with _guard(dev):
                state.copy_(host)
        self._rng[dev.index] = (torch.initial_seed(), state)

    def rng_state(self, device=None) -> torch.Tensor:
        """int64[4] device tensor {seed, offset, 0, 0} behind the draws that are given no explicit seed; every
        such draw advances the offset by one on the stream it runs on.  Create it (one draw, or
        :meth:`manual_seed`) before capturing a graph: the first use copies the seed from the host.  The same
        tensor is returned for the life of the process."""
        dev = _device(device)
        entry = self._rng.get(dev.index)
        if entry is None or entry[0] != torch.initial_seed():
            self.manual_seed(torch.initial_seed(), dev)
            entry = self._rng[dev.index]
        return entry[1]

    def random_lists(self, shape, p: float, seed: int | None = None, offset: int = 0, device=None,
                     split: int = 1, grid=None):
        """Draws a Bernoulli(p) block mask of ``shape`` on the device (True = dropped) and lists it in
        the same launch: (mask, lists).  The mask is a pure function of (seed, offset, shape[1]) —
        Philox4x32-10, one 32-bit word per entry — not torch's generator stream.  With ``seed=None``
        seed and offset come from the device-resident state (:meth:`rng_state`), which the call
        advances: the form that survives graph capture."""
        mb, kb = int(shape[0]), int(shape[1])
        if mb <= 0 or kb <= 0:
            raise ValueError("mask must be non-empty")
        if not 0.0 <= p < 1.0:
            raise ValueError(f"p must be in [0, 1), got {p}")
        split, out_mb, out_kb = self._list_grid(mb, kb, split, grid)
        dev = _device(device)
        state = self.rng_state(dev) if seed is None else None
        mask = torch.empty((mb, kb), dtype=torch.bool, device=dev)
        row_ptr, col_ptr, col_idx, row_idx = self._list_buffers(out_mb, out_kb, dev)
        tail = (mb, kb, mask.data_ptr(), split, out_mb, out_kb, row_ptr.data_ptr(), col_idx.data_ptr(),
                col_ptr.data_ptr(), row_idx.data_ptr(), self._stream(mask))
        with _guard(dev):
            if state is None:
                self._call(self.lib.sd_random_lists, int(seed) & (2 ** 64 - 1), int(offset) & (2 ** 64 - 1),
                           float(p), *tail)
            else:
                self._call(self.lib.sd_random_lists_state, state.data_ptr(), float(p), *tail)
        return mask, KeptLists(row_ptr, col_idx, col_ptr, row_idx, (out_mb, out_kb))

    def kept_lists(self, rows: int, cols: int, block_size, mask: torch.Tensor | None = None,
                   p: float = 0.0, seed: int | None = None, device=None):
        """Lists for a [rows, cols] matrix masked in block_size tiles -> (mask, lists, kernel block size).

        The mask is the given one, or drawn on the device (Bernoulli(p); ``seed`` pins it, otherwise the
        device-resident generator state is used and advanced, which follows ``torch.manual_seed``).  A block size
        that is a larger multiple of 64 is listed at 64 granularity, which is what the fast kernels
        take: pass the returned block size, not the logical one, to the ``*_lists`` calls."""
        bs = _block_size(block_size)
        shape = (ceil(rows / bs), ceil(cols / bs))
        split, grid, kernel_bs = 1, None, bs
        if bs > 64 and bs % 64 == 0:
            split, grid, kernel_bs = bs // 64, (ceil(rows / 64), ceil(cols / 64)), 64
        elif bs % 64 == 32:  # 32, 96, 160, ...: the 32-blocks merged two by two onto the 64 grid; the *_lists calls
            # are told so by block size 32
            split, grid, kernel_bs = -(bs // 32), (ceil(rows / 64), ceil(cols / 64)), 32
        if mask is None:
            mask, lists = self.random_lists(shape, p, seed, 0, device, split, grid)
        else:
            if tuple(mask.shape) != shape:
                raise ValueError(f"mask shape {tuple(mask.shape)} != {shape} for a [{rows}, {cols}] matrix "
                                 f"in blocks of {bs}")
            lists = self.build_lists(mask, split, grid)
        return mask, lists, kernel_bs

    def increment_table(self, lists: KeptLists, block_k: int):
        """(table, row_indices, row_widths) of the reference's ``mask_to_increment_table``
        (functional/utils.py:19-69), int64.  Reads nnz back to size ``table`` (one sync), as the
        reference's ``nonzero`` does."""
        mb = lists.shape[0]
        dev = lists.row_ptr.device
        table = torch.empty(lists.col_idx.numel(), dtype=torch.int64, device=dev)
        row_indices = torch.empty(mb, dtype=torch.int64, device=dev)
        row_widths = torch.empty(mb, dtype=torch.int64, device=dev)
        with _guard(dev):
            self._call(self.lib.sd_increment_table, lists.row_ptr.data_ptr(), lists.col_idx.data_ptr(),
                       mb, int(block_k), table.data_ptr(), row_indices.data_ptr(),
                       row_widths.data_ptr(), self._stream(table))
        return table[: lists.nnz()], row_indices, row_widths

    def _listed(self, fn, mask_cols, A, B, lists, block_size, scale, out, transposed_out):
        self._check_pair(A, B)
        bs = _block_size(block_size)
        M, N, K = A.shape[0], B.shape[0], A.shape[1]
        lg = _list_grid_size(bs)
        want = (ceil(M / lg), ceil((K if mask_cols == "K" else N) / lg))
        if tuple(lists.shape) != want:
            raise ValueError(f"lists are for a {lists.shape} mask, operands need {want}")
        C = self._out(A, B, out, transposed_out)
        if M == 0 or N == 0:
            return C
        extra = ()
        if mask_cols == "K":  # DSD may split a long reduction
            ws, ws_ptr, ws_bytes = self._splitk_scratch(A, B, bs, 1)
            extra = (ws_ptr, ws_bytes)
        with _guard(A.device):
            self._call(fn, *_mat(A), *_mat(B), *_mat(C), lists.row_ptr.data_ptr(),
                       lists.col_idx.data_ptr(), M, N, K, bs, float(scale), _DTYPES[A.dtype],
                       *extra, self._stream(A))
        return C

    def gemm_dsd_lists(self, A, B, lists: KeptLists, block_size, scale, out=None, transposed_out=False):
        return self._listed(self.lib.sd_gemm_dsd_lists, "K", A, B, lists, block_size, scale, out, transposed_out)

    def gemm_sdd_lists(self, A, B, lists: KeptLists, block_size, scale, out=None, transposed_out=False,
                       kept_only=False, keep_hint: float | None = None):
        """``kept_only``: dropped tiles of the result are left as they are (uninitialised for a fresh buffer)
        instead of being zeroed, for a consumer that never reads them (:meth:`col2im` with the mask).
        ``keep_hint``: expected fraction of kept blocks (1 - p) when the caller knows it; it only steers the
        choice of workgroup shape (the lists live on the device), never the result."""
        self._check_pair(A, B)
        bs = _block_size(block_size)
        M, N, K = A.shape[0], B.shape[0], A.shape[1]
        lg = _list_grid_size(bs)
        want = (ceil(M / lg), ceil(N / lg))
        if tuple(lists.shape) != want:
            raise ValueError(f"lists are for a {lists.shape} mask, operands need {want}")
        C = self._out(A, B, out, transposed_out)
        if M == 0 or N == 0:
            return C
        with _guard(A.device):
            self._call(self.lib.sd_gemm_sdd_lists_ex, *_mat(A), *_mat(B), *_mat(C), lists.row_ptr.data_ptr(),
                       lists.col_idx.data_ptr(), M, N, K, bs, float(scale), _DTYPES[A.dtype],
                       1 if kept_only else 0, -1.0 if keep_hint is None else float(keep_hint), self._stream(A))
        return C

    # ------------------------------------------------------------------ products with a fused activation
    def gemm_dsd_lists_act(self, A, B, lists: KeptLists, block_size, scale, act, want_pre: bool = False):
        """``act(scale * (A ⊙ keep) @ B.T)`` with the activation ("relu", "gelu" in its erf form, or None) applied
        to the fp32 accumulator in the kernel's store -> (activated, pre-activation or None).  The pre-activation
        is what the GELU backward is evaluated at; ReLU's can use the activated tensor."""
        self._check_pair(A, B)
        bs = _block_size(block_size)
        code = _activation(act)
        M, N, K = A.shape[0], B.shape[0], A.shape[1]
        lg = _list_grid_size(bs)
        want = (ceil(M / lg), ceil(K / lg))
        if tuple(lists.shape) != want:
            raise ValueError(f"lists are for a {lists.shape} mask, operands need {want}")
        C = torch.empty((M, N), dtype=A.dtype, device=A.device)
        pre = torch.empty((M, N), dtype=A.dtype, device=A.device) if (want_pre and code) else None
        if M == 0 or N == 0:
            return C, pre
        ws, ws_ptr, ws_bytes = self._splitk_scratch(A, B, bs, 1)
        with _guard(A.device):
            self._call(self.lib.sd_gemm_dsd_lists_act, *_mat(A), *_mat(B), *_mat(C), lists.row_ptr.data_ptr(),
                       lists.col_idx.data_ptr(), M, N, K, bs, float(scale), _DTYPES[A.dtype], code,
                       *(_mat(pre) if pre is not None else (None, 0, 0)), ws_ptr, ws_bytes, self._stream(A))
        return C, (pre if code else (C if want_pre else None))

    def gemm_act(self, A, B, act, want_pre: bool = False):
        """``act(A @ B.T)``, the dense product with the activation in the kernel's store -> (activated,
        pre-activation or None): a layer without dropout inside a fused stack."""
        self._check_pair(A, B)
        code = _activation(act)
        M, N, K = A.shape[0], B.shape[0], A.shape[1]
        C = torch.empty((M, N), dtype=A.dtype, device=A.device)
        pre = torch.empty((M, N), dtype=A.dtype, device=A.device) if (want_pre and code) else None
        if M == 0 or N == 0:
            return C, pre
        if K == 0:
            return C.zero_(), (pre.zero_() if pre is not None else None)
        ws, ws_ptr, ws_bytes = self._splitk_scratch(A, B, 0, 0)
        with _guard(A.device):
            self._call(self.lib.sd_gemm_act, *_mat(A), *_mat(B), *_mat(C), M, N, K, _DTYPES[A.dtype], code,
                       *(_mat(pre) if pre is not None else (None, 0, 0)), ws_ptr, ws_bytes, self._stream(A))
        return C, (pre if code else (C if want_pre else None))

    def gemm_sdd_lists_actgrad(self, A, B, lists: KeptLists, block_size, scale, act, act_at: torch.Tensor,
                               keep_hint: float | None = None):
        """``scale * (A @ B.T) ⊙ keep ⊙ act'(act_at)``: the input gradient of a layer whose input was
        ``act(act_at)``, carried through to ``act_at`` in the kernel's store.  ``act_at`` is [M, N] like the
        result; for "relu" it may be the activated tensor itself."""
        self._check_pair(A, B)
        bs = _block_size(block_size)
        code = _activation(act)
        M, N, K = A.shape[0], B.shape[0], A.shape[1]
        lg = _list_grid_size(bs)
        want = (ceil(M / lg), ceil(N / lg))
        if tuple(lists.shape) != want:
            raise ValueError(f"lists are for a {lists.shape} mask, operands need {want}")
        if code:
            _check_operand("act_at", act_at)
            if tuple(act_at.shape) != (M, N) or act_at.dtype != A.dtype or act_at.device != A.device:
                raise ValueError(f"act_at must be a [{M}, {N}] {A.dtype} tensor on {A.device}")
        C = torch.empty((M, N), dtype=A.dtype, device=A.device)
        if M == 0 or N == 0:
            return C
        with _guard(A.device):
            self._call(self.lib.sd_gemm_sdd_lists_actgrad, *_mat(A), *_mat(B), *_mat(C), lists.row_ptr.data_ptr(),
                       lists.col_idx.data_ptr(), M, N, K, bs, float(scale), _DTYPES[A.dtype], code,
                       *(_mat(act_at) if code else (None, 0, 0)), -1.0 if keep_hint is None else float(keep_hint),
                       self._stream(A))
        return C

    # ------------------------------------------------------------------ the autograd function's two calls
    def dropout_matmul_forward(self, x: torch.Tensor, w: torch.Tensor, block_size, p: float,
                               mask: torch.Tensor | None = None, seed: int | None = None):
        """Mask (given, or drawn on the device: pinned by ``seed``, else from the device-resident generator),
        kept-block lists and ``Y = (keep ⊙ x)/(1-p) @ w.T`` in one library call - and, for small layers, one
        launch -> (y, mask, lists, kernel block size).  The lists are at the granularity the kernels run at (64
        for block sizes that are multiples of 64) and serve :meth:`dropout_matmul_backward`."""
        return self.dropout_matmul_forward_act(x, w, block_size, p, mask, seed)[:4]

    def dropout_matmul_forward_act(self, x: torch.Tensor, w: torch.Tensor, block_size, p: float,
                                   mask: torch.Tensor | None = None, seed: int | None = None,
                                   activation: str | None = None, want_pre: bool = False):
        """:meth:`dropout_matmul_forward` with the activation ("relu", "gelu" or None) applied in the product's
        store -> (activated y, mask, lists, kernel block size, pre-activation or None)."""
        self._check_pair(x, w)
        code = _activation(activation)
        bs = _block_size(block_size)
        if not 0.0 <= p < 1.0:
            raise ValueError(f"p must be in [0, 1), got {p}")
        M, K, N = x.shape[0], x.shape[1], w.shape[0]
        g = 64 if bs % 32 == 0 else bs
        mb, kb, out_mb, out_kb = ceil(M / bs), ceil(K / bs), ceil(M / g), ceil(K / g)
        if mb == 0 or kb == 0:
            raise ValueError("mask must be non-empty")
        dev = x.device
        state = None
        if mask is None:
            mask = torch.empty((mb, kb), dtype=torch.bool, device=dev)
            given = (None, 0, 0)
            if seed is None:
                state = self.rng_state(dev)
        else:
            mask = _check_mask(mask, (mb, kb), x)
            given = (mask.data_ptr(), *_mask_strides(mask))
        row_ptr, col_ptr, col_idx, row_idx = self._list_buffers(out_mb, out_kb, dev)
        y = torch.empty((M, N), dtype=x.dtype, device=dev)
        pre = torch.empty((M, N), dtype=x.dtype, device=dev) if (want_pre and code) else None
        ws, ws_ptr, ws_bytes = self._splitk_scratch(x, w, g, 1)
        with _guard(dev):
            self._call(self.lib.sd_dropout_matmul_forward_act, *_mat(x), *_mat(w), *_mat(y), *given,
                       None if state is None else state.data_ptr(), (int(seed) & (2 ** 64 - 1)) if seed is not None else 0,
                       0, float(p), mask.data_ptr(), row_ptr.data_ptr(), col_idx.data_ptr(), col_ptr.data_ptr(),
                       row_idx.data_ptr(), M, N, K, bs, _DTYPES[x.dtype], code,
                       *(_mat(pre) if pre is not None else (None, 0, 0)), ws_ptr, ws_bytes, self._stream(x))
        # block size 32 stays 32 for the backward call: it says that the lists carry quadrant bits
        return (y, mask, KeptLists(row_ptr, col_idx, col_ptr, row_idx, (out_mb, out_kb)), (32 if bs % 64 == 32 else g),
                pre if code else (y if want_pre else None))

    def dropout_matmul_backward(self, dy: torch.Tensor, w: torch.Tensor, x: torch.Tensor, lists: KeptLists,
                                block_size, p: float, need_dx: bool = True, need_dw: bool = True,
                                activation: str | None = None, act_at: torch.Tensor | None = None):
        """``dX = (dy @ w) ⊙ keep / (1-p)`` and ``dW = dy.T @ (keep ⊙ x) / (1-p)`` (a contiguous [N, K] tensor) in
        one library call - and, for small layers, one launch; either may be skipped -> (dx or None, dw or None).
        With ``activation`` dX is also multiplied by the activation's derivative at ``act_at`` ([M, K]: the
        pre-activation, or for ReLU the activated tensor), as :meth:`gemm_sdd_lists_actgrad` does."""
        self._check_pair(x, w)
        _check_operand("dy", dy)
        bs = _block_size(block_size)
        M, K, N = x.shape[0], x.shape[1], w.shape[0]
        if tuple(dy.shape) != (M, N) or dy.dtype != x.dtype or dy.device != x.device:
            raise ValueError(f"dy must be a [{M}, {N}] {x.dtype} tensor on {x.device}")
        g = 64 if bs % 32 == 0 else bs
        if tuple(lists.shape) != (ceil(M / g), ceil(K / g)):
            raise ValueError(f"lists are for a {lists.shape} mask, operands need {(ceil(M / g), ceil(K / g))}")
        if N % 8 and N > 0 and M > 0 and K > 0 and (need_dx or need_dw):
            # An output width that is not a multiple of 8 (a 10-class head) would put 16-byte loads across row
            # ends in both products.  Zero-padded copies of dY and W (the reference pads its head to 128 outputs
            # up front, eval/mlp/model.py:22-24,40) keep them on the specialised kernels: the extra columns of dY
            # are zeros, so dX is unchanged, and the extra rows of dW are dropped.
            n_pad = (N + 7) // 8 * 8
            dy_pad = dy.new_zeros((M, n_pad))
            dy_pad[:, :N] = dy
            w_pad = w.new_zeros((n_pad, K))
            if need_dx:
                w_pad[:N] = w
            dx, dw = self.dropout_matmul_backward(dy_pad, w_pad, x, lists, bs, p, need_dx, need_dw, activation, act_at)
            return dx, (dw[:N] if dw is not None else None)
        dx = torch.empty((M, K), dtype=x.dtype, device=x.device) if need_dx else None
        dw = torch.empty((N, K), dtype=x.dtype, device=x.device) if need_dw else None
        if not (need_dx or need_dw) or M == 0 or K == 0:
            return dx, dw
        if N == 0:
            return (dx.zero_() if need_dx else None), dw
        ws_ptr, ws_bytes, ws = None, 0, None
        if need_dw:  # the weight gradient of a tall activation matrix splits its reduction over workgroups
            ws, ws_ptr, ws_bytes = self._splitk_scratch(x.t(), dy.t(), g, 1)
        act = _activation(activation) if need_dx else 0
        if act:
            if act_at is None or tuple(act_at.shape) != (M, K) or act_at.dtype != x.dtype or act_at.device != x.device:
                raise ValueError(f"act_at must be a [{M}, {K}] {x.dtype} tensor on {x.device}")
            _check_operand("act_at", act_at)
        with _guard(x.device):
            self._call(self.lib.sd_dropout_matmul_backward_act, *_mat(dy), *_mat(w), *_mat(x),
                       *(_mat(dx) if need_dx else (None, 0, 0)), *(_mat(dw) if need_dw else (None, 0, 0)),
                       lists.row_ptr.data_ptr(), lists.col_idx.data_ptr(), lists.col_ptr.data_ptr(),
                       lists.row_idx.data_ptr(), M, N, K, bs, float(p), _DTYPES[x.dtype],
                       act, *(_mat(act_at) if act else (None, 0, 0)), ws_ptr, ws_bytes, self._stream(x))
        return dx, dw

    # ------------------------------------------------------------------ conv feed
    @staticmethod
    def conv_out_hw(h, w, r, s, padding, stride, dilation):
        # reference: functional/im2col_conv2d.py:14-15
        p = (h + 2 * padding[0] - dilation[0] * (r - 1) - 1) // stride[0] + 1
        q = (w + 2 * padding[1] - dilation[1] * (s - 1) - 1) // stride[1] + 1
        return p, q

    def im2col(self, x: torch.Tensor, kernel_size, padding=(0, 0), stride=(1, 1), dilation=(1, 1),
               lists: KeptLists | None = None, block_size=None,
               out: torch.Tensor | None = None) -> torch.Tensor:
        """[N*P*Q, C*R*S] patch matrix in F.unfold column order.  With ``lists`` (over the block mask
        of that matrix) only kept blocks are written; the rest of the buffer is left as it was
        (uninitialised for a fresh one).  ``out`` may be any 2D view with unit column stride."""
        if x.dim() != 4 or not x.is_cuda or x.dtype not in _DTYPES:
            raise ValueError("x must be a 4D float16/bfloat16 tensor on the GPU")
        n, c, h, w = x.shape
        r, s = kernel_size
        p, q = self.conv_out_hw(h, w, r, s, padding, stride, dilation)
        if p <= 0 or q <= 0:
            raise ValueError("kernel does not fit the padded image")
        if out is None:
            cols = torch.empty((n * p * q, c * r * s), dtype=x.dtype, device=x.device)
        else:
            cols = out
            if (tuple(cols.shape) != (n * p * q, c * r * s) or cols.dtype != x.dtype
                    or cols.device != x.device or cols.stride(1) != 1):
                raise ValueError(f"out must be a [{n * p * q}, {c * r * s}] {x.dtype} view on {x.device} "
                                 "with unit column stride")
        rp = ci = None
        bs = 0
        if lists is not None:
            bs = _block_size(block_size)
            want = (ceil(n * p * q / bs), ceil(c * r * s / bs))
            if tuple(lists.shape) != want:
                raise ValueError(f"lists are for a {lists.shape} mask, patch matrix needs {want}")
            rp, ci = lists.row_ptr.data_ptr(), lists.col_idx.data_ptr()
        with _guard(x.device):
            self._call(self.lib.sd_im2col, x.data_ptr(), *x.stride(), cols.data_ptr(), cols.stride(0),
                       n, c, h, w, r, s, *padding, *stride, *dilation, rp, ci, bs, _DTYPES[x.dtype],
                       self._stream(x))
        return cols

    def conv2d_dsd_lists(self, x: torch.Tensor, weight2d: torch.Tensor, lists: KeptLists | None, block_size,
                         scale: float, kernel_size, padding=(0, 0), stride=(1, 1),
                         dilation=(1, 1)) -> torch.Tensor | None:
        """Implicit-GEMM forward of the block-dropout convolution: the [N*P*Q, K] product of the patch matrix
        (never materialised) with ``weight2d`` [K, C*R*S] over the kept blocks of ``lists`` (None: all of them,
        the dense convolution).  Returns None when the library does not take the geometry (the caller then
        goes through :meth:`im2col`)."""
        if x.dim() != 4 or not x.is_cuda or x.dtype not in _DTYPES:
            raise ValueError("x must be a 4D float16/bfloat16 tensor on the GPU")
        n, c, h, w = x.shape
        r, s = kernel_size
        p, q = self.conv_out_hw(h, w, r, s, padding, stride, dilation)
        if p <= 0 or q <= 0:
            raise ValueError("kernel does not fit the padded image")
        if (weight2d.dim() != 2 or weight2d.shape[1] != c * r * s or weight2d.dtype != x.dtype
                or weight2d.device != x.device or weight2d.stride(1) != 1):
            raise ValueError(f"weight2d must be a [K, {c * r * s}] {x.dtype} matrix on {x.device} with unit column stride")
        bs, rp, ci = 0, None, None
        if lists is not None:
            bs = _block_size(block_size)
            want = (ceil(n * p * q / bs), ceil(c * r * s / bs))
            if tuple(lists.shape) != want:
                raise ValueError(f"lists are for a {lists.shape} mask, patch matrix needs {want}")
            rp, ci = lists.row_ptr.data_ptr(), lists.col_idx.data_ptr()
        k = weight2d.shape[0]
        y = torch.empty((n * p * q, k), dtype=x.dtype, device=x.device)
        with _guard(x.device):
            rc = self.lib.sd_conv2d_dsd_lists(x.data_ptr(), *x.stride(), weight2d.data_ptr(), weight2d.stride(0),
                                              y.data_ptr(), y.stride(0), n, c, h, w, k, r, s, *padding, *stride,
                                              *dilation, rp, ci, bs, float(scale), _DTYPES[x.dtype],
                                              self._stream(x))
        if rc == 2:  # geometry not taken: nothing was launched
            return None
        if rc != 0:
            msg = self.lib.sd_last_error().decode(errors="replace")
            raise {1: ValueError}.get(rc, SparseDropError)(f"sd_conv2d_dsd_lists: {msg}")
        return y

    def conv2d_dw_lists(self, x: torch.Tensor, dy2d: torch.Tensor, lists: KeptLists | None, block_size,
                        scale: float, kernel_size, padding=(0, 0), stride=(1, 1),
                        dilation=(1, 1)) -> torch.Tensor | None:
        """Implicit-GEMM weight gradient of the block-dropout convolution: [K, C*R*S] from the input ``x`` and
        the output gradient ``dy2d`` [N*P*Q, K], over the kept blocks of ``lists`` (the lists of the patch
        matrix's mask; None = dense), without the patch matrix.  Returns None when the library does not take
        the geometry."""
        if x.dim() != 4 or not x.is_cuda or x.dtype not in _DTYPES:
            raise ValueError("x must be a 4D float16/bfloat16 tensor on the GPU")
        n, c, h, w = x.shape
        r, s = kernel_size
        p, q = self.conv_out_hw(h, w, r, s, padding, stride, dilation)
        if p <= 0 or q <= 0:
            raise ValueError("kernel does not fit the padded image")
        if (dy2d.dim() != 2 or dy2d.shape[0] != n * p * q or dy2d.dtype != x.dtype or dy2d.device != x.device
                or dy2d.stride(1) != 1):
            raise ValueError(f"dy2d must be a [{n * p * q}, K] {x.dtype} matrix on {x.device} with unit column stride")
        bs, cp, ri = 0, None, None
        if lists is not None:
            bs = _block_size(block_size)
            want = (ceil(n * p * q / bs), ceil(c * r * s / bs))
            if tuple(lists.shape) != want:
                raise ValueError(f"lists are for a {lists.shape} mask, patch matrix needs {want}")
            cp, ri = lists.col_ptr.data_ptr(), lists.row_idx.data_ptr()
        k = dy2d.shape[1]
        dw = torch.empty((k, c * r * s), dtype=x.dtype, device=x.device)
        nbytes = self.lib.sd_conv2d_dw_workspace_bytes(n, c, k, r, s, p, q)
        ws = torch.empty(nbytes // 4, dtype=torch.float32, device=x.device) if nbytes > 0 else None
        with _guard(x.device):
            rc = self.lib.sd_conv2d_dw_lists(x.data_ptr(), *x.stride(), dy2d.data_ptr(), dy2d.stride(0),
                                             dw.data_ptr(), dw.stride(0), n, c, h, w, k, r, s, *padding, *stride,
                                             *dilation, cp, ri, bs, float(scale), _DTYPES[x.dtype],
                                             ws.data_ptr() if ws is not None else None, nbytes, self._stream(x))
        if rc == 2:  # geometry not taken: nothing was launched
            return None
        if rc != 0:
            msg = self.lib.sd_last_error().decode(errors="replace")
            raise {1: ValueError}.get(rc, SparseDropError)(f"sd_conv2d_dw_lists: {msg}")
        return dw

    def conv2d_dx(self, dy2d: torch.Tensor, weight2d: torch.Tensor, x_shape, kernel_size, padding=(0, 0),
                  stride=(1, 1), dilation=(1, 1), mask: torch.Tensor | None = None, block_size=None,
                  scale: float = 1.0, channels_last: bool = False) -> torch.Tensor | None:
        """Input gradient of the (block-dropout) convolution in one launch: ``dy2d`` [N*P*Q, K] and
        ``weight2d`` [K, C*R*S] -> [N, C, H, W], the patch matrix's gradient never in memory.  ``mask`` is the
        block mask of the patch matrix (True = dropped).  Returns None when the library does not take the
        geometry (the caller then goes through :meth:`gemm_sdd_lists` and :meth:`col2im`)."""
        n, c, h, w = x_shape
        r, s = kernel_size
        p, q = self.conv_out_hw(h, w, r, s, padding, stride, dilation)
        if (dy2d.dim() != 2 or not dy2d.is_cuda or dy2d.dtype not in _DTYPES or dy2d.stride(1) != 1
                or dy2d.shape[0] != n * p * q):
            raise ValueError(f"dy2d must be a row-major [{n * p * q}, K] float16/bfloat16 matrix on the GPU")
        k = dy2d.shape[1]
        if (tuple(weight2d.shape) != (k, c * r * s) or weight2d.dtype != dy2d.dtype or weight2d.device != dy2d.device
                or weight2d.stride(1) != 1):
            raise ValueError(f"weight2d must be a [{k}, {c * r * s}] {dy2d.dtype} matrix with unit column stride")
        mp, msr, msc, bs = None, 0, 0, 64
        if mask is not None:
            bs = _block_size(block_size)
            mask = _check_mask(mask, (ceil(n * p * q / bs), ceil(c * r * s / bs)), dy2d)
            mp = mask.data_ptr()
            msr, msc = _mask_strides(mask)
        fmt = torch.channels_last if channels_last else torch.contiguous_format
        dx = torch.empty((n, c, h, w), dtype=dy2d.dtype, device=dy2d.device, memory_format=fmt)
        with _guard(dy2d.device):
            rc = self.lib.sd_conv2d_dx(dy2d.data_ptr(), dy2d.stride(0), weight2d.data_ptr(), weight2d.stride(0),
                                       dx.data_ptr(), *dx.stride(), mp, msr, msc, n, c, h, w, k, r, s, *padding,
                                       *stride, *dilation, bs, float(scale), _DTYPES[dy2d.dtype], self._stream(dy2d))
        if rc == 2:  # geometry not taken: nothing was launched
            return None
        if rc != 0:
            msg = self.lib.sd_last_error().decode(errors="replace")
            raise {1: ValueError}.get(rc, SparseDropError)(f"sd_conv2d_dx: {msg}")
        return dx

    def col2im(self, cols: torch.Tensor, x_shape, kernel_size, padding=(0, 0), stride=(1, 1),
               dilation=(1, 1), mask: torch.Tensor | None = None, block_size=None,
               channels_last: bool = False) -> torch.Tensor:
        """Adjoint of :meth:`im2col`: [N*P*Q, C*R*S] -> [N, C, H, W] (scatter-add expressed as a gather).
        With ``mask`` dropped blocks of ``cols`` are not read."""
        n, c, h, w = x_shape
        r, s = kernel_size
        if cols.dim() != 2 or not cols.is_cuda or cols.dtype not in _DTYPES or cols.stride(1) != 1:
            raise ValueError("cols must be a row-major 2D float16/bfloat16 tensor on the GPU")
        p, q = self.conv_out_hw(h, w, r, s, padding, stride, dilation)
        if tuple(cols.shape) != (n * p * q, c * r * s):
            raise ValueError(f"cols shape {tuple(cols.shape)} != {(n * p * q, c * r * s)}")
        fmt = torch.channels_last if channels_last else torch.contiguous_format
        dx = torch.empty((n, c, h, w), dtype=cols.dtype, device=cols.device, memory_format=fmt)
        mp, msr, msc, bs = None, 0, 0, 0
        if mask is not None:
            bs = _block_size(block_size)
            mask = _check_mask(mask, (ceil(n * p * q / bs), ceil(c * r * s / bs)), cols)
            mp = mask.data_ptr()
            msr, msc = _mask_strides(mask)
        with _guard(cols.device):
            self._call(self.lib.sd_col2im, cols.data_ptr(), cols.stride(0), dx.data_ptr(), *dx.stride(),
                       n, c, h, w, r, s, *padding, *stride, *dilation, mp, msr, msc, bs,
                       _DTYPES[cols.dtype], self._stream(cols))
        return dx
