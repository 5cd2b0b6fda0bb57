"""Kernel (a): block mask -> compacted kept-block lists, through the C ABI.  Bit-exact contract."""
import json
from pathlib import Path

import numpy as np
import pytest
import torch

from oracle import sparsedrop_oracle as O

pytestmark = pytest.mark.gpu
GOLDEN = Path(__file__).parent / "golden"
CASES = json.loads((GOLDEN / "compaction_cases.json").read_text())


def _lists_np(lists):
    nnz = lists.nnz()
    return (lists.row_ptr.cpu().numpy(), lists.col_idx[:nnz].cpu().numpy(),
            lists.col_ptr.cpu().numpy(), lists.row_idx[:nnz].cpu().numpy())


@pytest.mark.parametrize("name", sorted(CASES))
def test_known_answers(name):
    from flash_dropout.hip import GEMM

    c = CASES[name]
    g = GEMM()
    mask = torch.tensor(c["mask"], dtype=torch.bool, device="cuda")
    lists = g.build_lists(mask)
    rp, ci, cp, ri = _lists_np(lists)
    assert rp.dtype == np.int32 and ci.dtype == np.int32
    assert rp.tolist() == c["row_ptr"] and ci.tolist() == c["col_idx"]
    assert cp.tolist() == c["col_ptr"] and ri.tolist() == c["row_idx"]
    table, row_indices, row_widths = g.increment_table(lists, c["block_k"])
    assert table.dtype == torch.int64
    assert table.cpu().tolist() == c["table"]
    assert row_indices.cpu().tolist() == c["row_indices"]
    assert row_widths.cpu().tolist() == c["row_widths"]


@pytest.mark.parametrize("shape,p", [((16, 16), 0.5), ((128, 128), 0.5), ((128, 128), 0.0), ((128, 128), 1.0),
                                     ((64, 13), 0.5), ((256, 6), 0.3), ((2048, 9), 0.5), ((1, 1), 0.0),
                                     ((1, 300), 0.7), ((300, 1), 0.7), ((65, 129), 0.25), ((1000, 700), 0.9)])
@pytest.mark.parametrize("col_major", [False, True])
def test_random_masks_bit_exact(shape, p, col_major):
    import flash_dropout.functional as F

    gen = torch.Generator().manual_seed(shape[0] * 1000 + shape[1])
    mask_cpu = torch.rand(*shape, generator=gen) < p
    mask = mask_cpu.t().contiguous().cuda().t() if col_major else mask_cpu.cuda()
    assert tuple(mask.shape) == shape
    lists = F.kept_block_lists(mask)
    rp, ci, cp, ri = _lists_np(lists)
    erp, eci = O.compact_csr(mask_cpu.numpy())
    ecp, eri = O.compact_csc(mask_cpu.numpy())
    assert np.array_equal(rp, erp) and np.array_equal(ci, eci)
    assert np.array_equal(cp, ecp) and np.array_equal(ri, eri)
    # the library identity the reference relies on (blockwise_dropout_matmul_triton.py:48)
    nz = torch.nonzero(~mask, as_tuple=False)
    assert torch.equal(F.kept_block_table(mask), nz)
    # transposed view swaps CSR and CSC
    t = lists.transposed()
    assert t.shape == (shape[1], shape[0]) and t.row_ptr is lists.col_ptr


def test_large_mask_uses_multi_launch_path():
    import flash_dropout.functional as F

    gen = torch.Generator().manual_seed(7)
    mask_cpu = torch.rand(1500, 400, generator=gen) < 0.6  # 600k entries > fused limit
    lists = F.kept_block_lists(mask_cpu.cuda())
    rp, ci, cp, ri = _lists_np(lists)
    erp, eci = O.compact_csr(mask_cpu.numpy())
    ecp, eri = O.compact_csc(mask_cpu.numpy())
    assert np.array_equal(rp, erp) and np.array_equal(ci, eci)
    assert np.array_equal(cp, ecp) and np.array_equal(ri, eri)


@pytest.mark.parametrize("shape,p,bk", [((16, 16), 0.5, 64), ((40, 70), 0.8, 128), ((9, 3), 0.95, 16)])
def test_increment_table_vs_oracle(shape, p, bk):
    import flash_dropout.functional as F

    gen = torch.Generator().manual_seed(11)
    mask_cpu = torch.rand(*shape, generator=gen) < p
    table, ri, rw = F.mask_to_increment_table(mask_cpu.cuda(), bk)
    et, eri, erw = O.mask_to_increment_table(mask_cpu.numpy(), bk)
    assert np.array_equal(table.cpu().numpy(), et)
    assert np.array_equal(ri.cpu().numpy(), eri)
    assert np.array_equal(rw.cpu().numpy(), erw)


@pytest.mark.parametrize("shape", [(1, 1), (2, 2), (5, 7), (16, 24), (63, 33), (256, 256), (600, 500)])
@pytest.mark.parametrize("p", [0.0, 0.5, 0.9])
def test_merged_lists_of_a_block_size_32_mask_bit_exact(shape, p):
    """split = 0: a mask at block size 32 listed on the 64 grid with the quadrant keep bits in bits 28-31 of every
    entry, against the oracle's encoding, for the list by rows and (transposed bits) by columns; masks larger than
    2^18 listed entries take the multi-launch builder."""
    from flash_dropout.hip import GEMM

    ext = GEMM()
    gen = torch.Generator().manual_seed(shape[0] * 1000 + shape[1])
    mask = torch.rand(*shape, generator=gen) < p
    lists = ext.build_lists(mask.cuda(), split=0)
    assert lists.shape == ((shape[0] + 1) // 2, (shape[1] + 1) // 2)
    rp, ci = O.compact_csr_quads(mask.numpy())
    assert np.array_equal(lists.row_ptr.cpu().numpy(), rp)
    assert np.array_equal(lists.col_idx[: lists.nnz()].cpu().numpy(), ci)
    cp, ri = O.compact_csr_quads(mask.numpy().T)
    assert np.array_equal(lists.col_ptr.cpu().numpy(), cp)
    assert np.array_equal(lists.row_idx[: lists.nnz()].cpu().numpy(), ri)
    # the same from a drawn mask
    drawn, lists = ext.random_lists(shape, p, seed=9, split=0)
    want = O.random_mask(shape, p, 9)
    assert np.array_equal(drawn.cpu().numpy(), want)
    rp, ci = O.compact_csr_quads(want)
    assert np.array_equal(lists.row_ptr.cpu().numpy(), rp)
    assert np.array_equal(lists.col_idx[: lists.nnz()].cpu().numpy(), ci)


@pytest.mark.parametrize("rows,cols,bs", [(96, 96, 96), (100, 130, 96), (1000, 784, 96), (4096, 4096, 160), (70, 700, 224),
                                          (8192, 8192, 96)])
@pytest.mark.parametrize("p", [0.0, 0.5, 0.9])
def test_merged_lists_of_odd_multiples_of_32_bit_exact(rows, cols, bs, p):
    """split = -k: a mask at block size 32 * k (96, 160, 224) over a [rows, cols] matrix, listed on the matrix's grid of
    64-blocks with the quadrant keep bits: against the oracle's composition (every mask entry repeated k x k times onto
    the grid of 32-blocks, that grid merged two by two), by rows and by columns, for a stored and a drawn mask."""
    from flash_dropout.hip import GEMM

    ext = GEMM()
    k = bs // 32
    shape = O.mask_shape(rows, cols, bs)
    grid64 = O.mask_shape(rows, cols, 64)
    gen = torch.Generator().manual_seed(rows + cols + bs)
    mask = torch.rand(*shape, generator=gen) < p

    def want(m):
        # the mask's 32-blocks, as far as the 64 grid reaches (a 32-block past the matrix but inside the mask's last
        # entry keeps that entry's value)
        m32 = O.split_mask(m, k, (min(shape[0] * k, 2 * grid64[0]), min(shape[1] * k, 2 * grid64[1])))
        return O.compact_csr_quads(m32), O.compact_csr_quads(m32.T)

    def check(lists, m):
        (rp, ci), (cp, ri) = want(m)
        assert lists.shape == grid64
        assert np.array_equal(lists.row_ptr.cpu().numpy(), rp)
        assert np.array_equal(lists.col_idx[: lists.nnz()].cpu().numpy(), ci)
        assert np.array_equal(lists.col_ptr.cpu().numpy(), cp)
        assert np.array_equal(lists.row_idx[: lists.nnz()].cpu().numpy(), ri)

    check(ext.build_lists(mask.cuda(), split=-k, grid=grid64), mask.numpy())
    check(ext.build_lists(mask.t().contiguous().cuda().t(), split=-k, grid=grid64), mask.numpy())  # column-major mask
    drawn, lists = ext.random_lists(shape, p, seed=11, split=-k, grid=grid64)
    assert np.array_equal(drawn.cpu().numpy(), O.random_mask(shape, p, 11))
    check(lists, O.random_mask(shape, p, 11))
    # the element mask is the one of the block size: what makes the composition the right oracle
    m32 = O.split_mask(mask.numpy(), k, O.mask_shape(rows, cols, 32))
    assert np.array_equal(O.expand_keep(m32, 32, rows, cols), O.expand_keep(mask.numpy(), bs, rows, cols))
