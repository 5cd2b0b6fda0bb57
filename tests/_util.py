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
