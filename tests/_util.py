"""Shared helpers for the GPU parity tests."""
import numpy as np
import torch

# parity bar for floating point outputs: relative Frobenius error against the fp32/fp64 oracle
# evaluated on the same fp16/bf16-rounded inputs
REL_FRO_TOL = 1e-2


def rel_fro(got, ref) -> float:
    got = got.detach().double().cpu().numpy() if isinstance(got, torch.Tensor) else np.asarray(got, dtype=np.float64)
    ref = ref.detach().double().cpu().numpy() if isinstance(ref, torch.Tensor) else np.asarray(ref, dtype=np.float64)
    assert got.shape == ref.shape, (got.shape, ref.shape)
    den = np.linalg.norm(ref)
    num = np.linalg.norm(got - ref)
    if den == 0:
        return 0.0 if num == 0 else float("inf")
    return float(num / den)


def to_np(t: torch.Tensor, dtype=np.float32):
    return t.detach().float().cpu().numpy().astype(dtype)


def make_operand(rows, cols, dtype, device, row_major=True, scale=1.0, gen=None):
    """[rows, cols] N(0, scale^2) tensor, row-major or (as a transposed view) column-major."""
    if row_major:
        t = torch.randn(rows, cols, generator=gen) * scale
        return t.to(dtype).to(device)
    t = torch.randn(cols, rows, generator=gen) * scale
    return t.to(dtype).to(device).t()


def cpu_mask(shape, p, gen):
    """Block mask drawn on the CPU generator (device independent), True = dropped."""
    return torch.rand(*shape, generator=gen) < p


def max_tile_rel_fro(got, ref, tile: int = 64) -> float:
    """Largest relative Frobenius error over the tile x tile tiles of a matrix (the kernels' unit of work:
    one wrong, missing or half-computed tile moves the whole-matrix error of a large output by less than the
    parity bar, but not its own tile's).  A tile whose reference is all zeros (a dropped SDD tile, a row block
    with nothing kept) must be exactly zero, else the result is inf.  Tensors with more than two dimensions are
    viewed as [prod(leading), last]."""
    got = got.detach().double().cpu().numpy() if isinstance(got, torch.Tensor) else np.asarray(got, dtype=np.float64)
    ref = ref.detach().double().cpu().numpy() if isinstance(ref, torch.Tensor) else np.asarray(ref, dtype=np.float64)
    assert got.shape == ref.shape, (got.shape, ref.shape)
    if got.size == 0:
        return 0.0
    got = got.reshape(-1, got.shape[-1])
    ref = ref.reshape(-1, ref.shape[-1])
    r0 = np.arange(0, got.shape[0], tile)
    c0 = np.arange(0, got.shape[1], tile)
    tiles = lambda a: np.add.reduceat(np.add.reduceat(a, r0, axis=0), c0, axis=1)
    num = np.sqrt(tiles((got - ref) ** 2))
    den = np.sqrt(tiles(ref ** 2))
    with np.errstate(divide="ignore", invalid="ignore"):
        rel = np.where(den > 0, num / den, np.where(num > 0, np.inf, 0.0))
    return float(rel.max())
