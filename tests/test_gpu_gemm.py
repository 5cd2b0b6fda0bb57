"""Kernels (b)(c)(d) through the C ABI: gemm / gemm_dsd / gemm_sdd against the CPU oracle.

Mirrors the structure of the reference's own parity test (test/test_cuda.py:23-57): same shape grid,
same p grid, one mask tensor handed to both sides, three outputs (C, dA, dB) checked — with the
tolerance the north star states (relative Frobenius error <= 1e-2 against the fp32 oracle on the
fp16-rounded inputs) in addition to the reference's own assert_close(atol=0.2, rtol=0.01).
"""
from itertools import product

import numpy as np
import pytest
import torch

from _util import REL_FRO_TOL, max_tile_rel_fro, cpu_mask, make_operand, rel_fro, to_np
from oracle import sparsedrop_oracle as O

pytestmark = pytest.mark.gpu


@pytest.fixture(autouse=True, params=["auto", "big", "mid"])
def tile_policy(request):
    """Every test of this file runs with the DSD workgroup shape chosen from the problem shape and with
    each of the two shapes forced, so both are checked on every shape and edge case below."""
    from flash_dropout.hip import GEMM

    ext = GEMM()
    prev = ext.set_tile_policy(request.param)
    yield request.param
    ext.set_tile_policy(prev)


def _three_products(A, B, dC, mask, bs, p):
    """The three calls exactly as the reference's autograd function issues them."""
    from flash_dropout.hip import GEMM

    ext = GEMM()
    s = 1 / (1 - p)
    C = ext.gemm_dsd(A, B, mask, bs, s)
    dA = ext.gemm_sdd(dC, B.T, mask, bs, s)
    dB = ext.gemm_dsd(A.T, dC.T, mask.T, bs, s).T
    return C, dA, dB


def _oracle_products(A, B, dC, mask, bs, p, dtype=np.float32):
    a, b, dc, mk = to_np(A, dtype), to_np(B, dtype), to_np(dC, dtype), mask.cpu().numpy()
    return (O.dsd_forward(a, b, mk, bs, p, dtype), O.sdd_dx(dc, b, mk, bs, p, dtype),
            O.dsd_dw(dc, a, mk, bs, p, dtype))


def _check(got, ref, what, atol=0.2, rtol=0.01):
    err = max_tile_rel_fro(got, ref)
    assert err <= REL_FRO_TOL, f"{what}: largest per-tile relative Frobenius error {err:.3e}"
    torch.testing.assert_close(got.float().cpu(), torch.from_numpy(np.asarray(ref, dtype=np.float32)),
                               atol=atol, rtol=rtol)


# the reference's grid (test/test_cuda.py:12-20)
REF_MNKS = [(128, 128, 128), (512, 512, 512), (1024, 1024, 1024), (2048, 2048, 2048)]
REF_PS = [0.0, 0.1, 0.2, 0.5, 0.9, 0.99, 0.999]


@pytest.mark.parametrize("mnk,block_size,p", list(product(REF_MNKS, [128], REF_PS)))
def test_reference_grid(mnk, block_size, p):
    M, N, K = mnk
    gen = torch.Generator().manual_seed(0)
    A = make_operand(M, K, torch.float16, "cuda", gen=gen)
    B = make_operand(N, K, torch.float16, "cuda", gen=gen)
    dC = make_operand(M, N, torch.float16, "cuda", gen=gen)
    mask = cpu_mask((M // block_size, K // block_size), p, gen).cuda()
    C, dA, dB = _three_products(A, B, dC, mask, block_size, p)
    rC, rdA, rdB = _oracle_products(A, B, dC, mask, block_size, p)
    # p = 0.999 scales by 1000: the absolute tolerance scales with it, as values do
    atol = 0.2 * max(1.0, (1 / (1 - p)) / 10)
    _check(C, rC, "C", atol)
    _check(dB, rdB, "dB", atol)
    _check(dA, rdA, "dA", atol)
    keep = O.expand_keep(mask.cpu().numpy(), block_size, M, K)
    assert (dA.cpu().numpy()[~keep] == 0).all(), "dropped dX tiles must be exactly zero"


@pytest.mark.parametrize("mnk", [(256, 256, 256), (1024, 1024, 1024), (2048, 2048, 2048)])
@pytest.mark.parametrize("p", [0.0, 0.25, 0.5, 0.75])
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_block64_square(mnk, p, dtype):
    M, N, K = mnk
    bs = 64
    gen = torch.Generator().manual_seed(1)
    A = make_operand(M, K, dtype, "cuda", gen=gen)
    B = make_operand(N, K, dtype, "cuda", scale=K ** -0.5, gen=gen)
    dC = make_operand(M, N, dtype, "cuda", gen=gen)
    mask = cpu_mask((M // bs, K // bs), p, gen).cuda()
    C, dA, dB = _three_products(A, B, dC, mask, bs, p)
    rC, rdA, rdB = _oracle_products(A, B, dC, mask, bs, p)
    for got, ref, what in ((C, rC, "C"), (dA, rdA, "dA"), (dB, rdB, "dB")):
        assert max_tile_rel_fro(got, ref) <= REL_FRO_TOL, what


LAYOUTS = list(product([True, False], repeat=3))  # A row-major?, B row-major?, mask row-major?


@pytest.mark.parametrize("a_rm,b_rm,m_rm", LAYOUTS)
@pytest.mark.parametrize("out_t", [False, True])
def test_all_majorness_combinations(a_rm, b_rm, m_rm, out_t):
    """The four operand layouts of the reference's manual script (binding_gemm.py:88-99) x mask layout
    x output layout, for dense, DSD and SDD."""
    from flash_dropout.hip import GEMM

    ext = GEMM()
    M, N, K, bs, p = 256, 384, 512, 64, 0.4
    gen = torch.Generator().manual_seed(2)
    A = make_operand(M, K, torch.float16, "cuda", row_major=a_rm, gen=gen)
    B = make_operand(N, K, torch.float16, "cuda", row_major=b_rm, gen=gen)
    a, b = to_np(A), to_np(B)
    got = ext.gemm(A, B, transposed_out=out_t)
    assert got.shape == (M, N) and (got.stride(0) == 1) == out_t
    assert max_tile_rel_fro(got, a @ b.T) <= REL_FRO_TOL
    mk = cpu_mask((M // bs, K // bs), p, gen)
    mask = mk.cuda() if m_rm else mk.t().contiguous().cuda().t()
    got = ext.gemm_dsd(A, B, mask, bs, 1 / (1 - p), transposed_out=out_t)
    assert max_tile_rel_fro(got, O.gemm_dsd(a, b, mk.numpy(), bs, 1 / (1 - p), np.float32)) <= REL_FRO_TOL
    mk = cpu_mask((M // bs, N // bs), p, gen)
    mask = mk.cuda() if m_rm else mk.t().contiguous().cuda().t()
    got = ext.gemm_sdd(A, B, mask, bs, 1 / (1 - p), transposed_out=out_t)
    ref = O.gemm_sdd(a, b, mk.numpy(), bs, 1 / (1 - p), np.float32)
    assert max_tile_rel_fro(got, ref) <= REL_FRO_TOL
    assert (got.cpu().numpy()[ref == 0] == 0).all()


@pytest.mark.parametrize("M,N,K,bs", [
    (4096, 1024, 784, 64),   # MLP layer 1: K tail 784 = 12*64 + 16
    (4096, 10, 1024, 64),    # MLP layer 3: N tail 10 (dY leading dimension 10: unaligned loads)
    (1000, 130, 200, 64),    # tails everywhere
    (100, 70, 50, 64),       # smaller than one block
    (16384, 1536, 384, 64),  # transformer MLP up-projection
    (16384, 384, 1536, 64),  # transformer MLP down-projection
    (512, 512, 512, 256),    # large block
    (300, 200, 500, 128),
    (16384, 128, 576, 64),   # conv patch matrix (8 images): dW = 576 x 128 over a 16384-long reduction, split over workgroups
    (73728, 64, 128, 64),    # dW reduction of 1152 blocks: more than one workgroup's step table, only reachable split
    (4096, 320, 192, 64),    # N = 256 + 64: the second column tile overhangs
])
@pytest.mark.parametrize("p", [0.0, 0.5])
def test_tails_and_model_shapes(M, N, K, bs, p):
    gen = torch.Generator().manual_seed(3)
    A = make_operand(M, K, torch.float16, "cuda", gen=gen)
    B = make_operand(N, K, torch.float16, "cuda", scale=K ** -0.5, gen=gen)
    dC = make_operand(M, N, torch.float16, "cuda", gen=gen)
    mask = cpu_mask(O.mask_shape(M, K, bs), p, gen).cuda()
    C, dA, dB = _three_products(A, B, dC, mask, bs, p)
    rC, rdA, rdB = _oracle_products(A, B, dC, mask, bs, p)
    for got, ref, what in ((C, rC, "C"), (dA, rdA, "dA"), (dB, rdB, "dB")):
        assert max_tile_rel_fro(got, ref) <= REL_FRO_TOL, what
    keep = O.expand_keep(mask.cpu().numpy(), bs, M, K)
    assert (dA.cpu().numpy()[~keep] == 0).all()


def test_degenerate_masks():
    M, N, K, bs = 256, 128, 320, 64
    gen = torch.Generator().manual_seed(4)
    A = make_operand(M, K, torch.float16, "cuda", gen=gen)
    B = make_operand(N, K, torch.float16, "cuda", gen=gen)
    dC = make_operand(M, N, torch.float16, "cuda", gen=gen)
    masks = {
        "row_dropped": torch.zeros(4, 5, dtype=torch.bool),
        "col_dropped": torch.zeros(4, 5, dtype=torch.bool),
        "all_dropped": torch.ones(4, 5, dtype=torch.bool),
        "none_dropped": torch.zeros(4, 5, dtype=torch.bool),
        "last_row_dropped": torch.zeros(4, 5, dtype=torch.bool),
    }
    masks["row_dropped"][1, :] = True
    masks["col_dropped"][:, 2] = True
    masks["last_row_dropped"][3, :] = True
    for name, mk in masks.items():
        C, dA, dB = _three_products(A, B, dC, mk.cuda(), bs, 0.5)
        rC, rdA, rdB = _oracle_products(A, B, dC, mk, bs, 0.5)
        for got, ref, what in ((C, rC, "C"), (dA, rdA, "dA"), (dB, rdB, "dB")):
            assert max_tile_rel_fro(got, ref) <= REL_FRO_TOL, (name, what)
    C, dA, dB = _three_products(A, B, dC, masks["all_dropped"].cuda(), bs, 0.5)
    assert (C == 0).all() and (dA == 0).all() and (dB == 0).all()
    C, _, _ = _three_products(A, B, dC, masks["row_dropped"].cuda(), bs, 0.5)
    assert (C[64:128] == 0).all()


def test_lists_entry_points_match_mask_entry_points():
    from flash_dropout.hip import GEMM

    ext = GEMM()
    M, N, K, bs, p = 512, 256, 384, 64, 0.5
    gen = torch.Generator().manual_seed(5)
    A = make_operand(M, K, torch.float16, "cuda", gen=gen)
    B = make_operand(N, K, torch.float16, "cuda", gen=gen)
    dC = make_operand(M, N, torch.float16, "cuda", gen=gen)
    mask = cpu_mask((M // bs, K // bs), p, gen).cuda()
    lists = ext.build_lists(mask)
    s = 1 / (1 - p)
    assert torch.equal(ext.gemm_dsd_lists(A, B, lists, bs, s), ext.gemm_dsd(A, B, mask, bs, s))
    assert torch.equal(ext.gemm_sdd_lists(dC, B.T, lists, bs, s), ext.gemm_sdd(dC, B.T, mask, bs, s))
    dW = ext.gemm_dsd_lists(A.T, dC.T, lists.transposed(), bs, s, transposed_out=True).T
    assert dW.is_contiguous()
    # the row-major [K, N] result of the mask form comes from a different kernel (other summation order)
    assert rel_fro(dW, ext.gemm_dsd(A.T, dC.T, mask.T, bs, s).T.float()) <= 1e-3
    assert torch.equal(dW, ext.gemm_dsd(A.T, dC.T, mask.T, bs, s, transposed_out=True).T)


def test_errors_through_the_shim():
    from flash_dropout.hip import GEMM

    ext = GEMM()
    A = torch.randn(128, 128, device="cuda", dtype=torch.float16)
    mask = torch.zeros(2, 2, dtype=torch.bool, device="cuda")
    with pytest.raises(TypeError, match="float16 or bfloat16"):
        ext.gemm_dsd(A.float(), A.float(), mask, 64, 1.0)
    with pytest.raises(TypeError, match="Mask must be bool"):
        ext.gemm_dsd(A, A, mask.to(torch.uint8), 64, 1.0)
    with pytest.raises(ValueError, match="mask shape"):
        ext.gemm_dsd(A, A, torch.zeros(1, 2, dtype=torch.bool, device="cuda"), 64, 1.0)
    with pytest.raises(ValueError, match="row or column major"):
        ext.gemm(A[::2, ::2], A[:64, :64])
    with pytest.raises(NotImplementedError, match="multiples of 32"):
        ext.gemm_dsd(A, A, torch.zeros(3, 3, dtype=torch.bool, device="cuda"), 48, 1.0)
    with pytest.raises(ValueError, match="reduction dims"):
        ext.gemm(A, A[:, :64])


def test_runs_on_the_current_stream():
    from flash_dropout.hip import GEMM

    ext = GEMM()
    gen = torch.Generator().manual_seed(6)
    A = make_operand(512, 512, torch.float16, "cuda", gen=gen)
    B = make_operand(512, 512, torch.float16, "cuda", gen=gen)
    mask = cpu_mask((8, 8), 0.5, gen).cuda()
    ref = ext.gemm_dsd(A, B, mask, 64, 2.0)
    torch.cuda.synchronize()
    side = torch.cuda.Stream()
    with torch.cuda.stream(side):
        got = ext.gemm_dsd(A, B, mask, 64, 2.0)
    side.synchronize()
    assert torch.equal(got, ref)


@pytest.mark.parametrize("p", [0.0, 0.5])
def test_full_size_8192_sampled_against_oracle(p):
    """Headline size: the oracle is evaluated on sampled row/column blocks only (it is linear in rows
    of A and of B, so any sub-block of the output is an independent oracle problem)."""
    M = N = K = 8192
    bs = 64
    gen = torch.Generator().manual_seed(8)
    A = make_operand(M, K, torch.float16, "cuda", gen=gen)
    B = make_operand(N, K, torch.float16, "cuda", scale=K ** -0.5, gen=gen)
    dC = make_operand(M, N, torch.float16, "cuda", gen=gen)
    mask = cpu_mask((M // bs, K // bs), p, gen).cuda()
    C, dA, dB = _three_products(A, B, dC, mask, bs, p)
    mk = mask.cpu().numpy()
    rows = np.r_[0:64, 4032:4160, 8128:8192]       # row blocks 0, 63, 64, 127
    cols = np.r_[64:128, 5000:5100, 8100:8192]
    a, b, dc = to_np(A), to_np(B), to_np(dC)
    s = np.float32(1 / (1 - p))
    keep = O.expand_keep(mk, bs, M, K)
    # Y[rows, cols]
    ref = (np.where(keep[rows], a[rows], 0) @ b[cols].T) * s
    assert max_tile_rel_fro(C.cpu().numpy()[np.ix_(rows, cols)], ref) <= REL_FRO_TOL
    # dX[rows, cols]
    ref = np.where(keep[np.ix_(rows, cols)], (dc[rows] @ b[:, cols]) * s, 0)
    got = dA.cpu().numpy()[np.ix_(rows, cols)]
    assert max_tile_rel_fro(got, ref) <= REL_FRO_TOL
    assert (dA.cpu().numpy()[~keep] == 0).all()
    # dW[rows (of N), cols (of K)]
    ref = (dc[:, rows].T @ np.where(keep[:, cols], a[:, cols], 0)) * s
    assert max_tile_rel_fro(dB.cpu().numpy()[np.ix_(rows, cols)], ref) <= REL_FRO_TOL
    if p == 0.0:
        from flash_dropout.hip import GEMM

        # size-independent property: with nothing dropped DSD/SDD are the dense product (the kernels
        # may sum in a different order, so to rounding rather than bit for bit)
        ext = GEMM()
        assert rel_fro(C, ext.gemm(A, B).float()) <= 1e-3
        assert rel_fro(dA, ext.gemm(dC, B.T).float()) <= 1e-3


@pytest.mark.parametrize("size,p", [(4096, 0.0), (4096, 0.25), (4096, 0.5), (4096, 0.75),
                                    (8192, 0.0), (8192, 0.25), (8192, 0.5), (8192, 0.75)])
def test_square_sweep_sizes_against_the_full_oracle(size, p, tile_policy):
    """The square sweep's larger sizes at every drop rate of the benchmark, every 64 x 64 tile of Y, dX and dW against
    the fp32 oracle: 4096^3 sits at the boundary between the two workgroup shapes, 8192^3 is the headline size."""
    if tile_policy != "auto":
        pytest.skip("full-size oracle runs once, under the shape policy the library picks itself")
    M = N = K = size
    bs = 64
    gen = torch.Generator().manual_seed(9)
    A = make_operand(M, K, torch.float16, "cuda", gen=gen)
    B = make_operand(N, K, torch.float16, "cuda", scale=K ** -0.5, gen=gen)
    dC = make_operand(M, N, torch.float16, "cuda", gen=gen)
    mask = cpu_mask((M // bs, K // bs), p, gen).cuda()
    C, dA, dB = _three_products(A, B, dC, mask, bs, p)
    from flash_dropout.hip import GEMM

    assert GEMM().last_kernel() == "specialised"
    rC, rdA, rdB = _oracle_products(A, B, dC, mask, bs, p)
    for got, ref, what in ((C, rC, "C"), (dA, rdA, "dA"), (dB, rdB, "dB")):
        err = max_tile_rel_fro(got, ref)
        assert err <= REL_FRO_TOL, f"{what}: largest per-tile relative Frobenius error {err:.3e}"


@pytest.mark.parametrize("dtype,bs", [(torch.bfloat16, 64), (torch.float16, 32), (torch.bfloat16, 32)])
def test_4096_bf16_and_block_size_32_against_the_full_oracle(dtype, bs, tile_policy):
    """bf16 and a mask of block size 32 at 4096^3, p = 0.5: every 64 x 64 tile of the three products against the
    fp32 oracle on the same rounded inputs, dropped 32 x 32 blocks of dX exactly zero."""
    if tile_policy != "auto":
        pytest.skip("full-size oracle runs once, under the shape policy the library picks itself")
    M = N = K = 4096
    p = 0.5
    gen = torch.Generator().manual_seed(10)
    A = make_operand(M, K, dtype, "cuda", gen=gen)
    B = make_operand(N, K, dtype, "cuda", scale=K ** -0.5, gen=gen)
    dC = make_operand(M, N, dtype, "cuda", gen=gen)
    mask = cpu_mask((M // bs, K // bs), p, gen).cuda()
    C, dA, dB = _three_products(A, B, dC, mask, bs, p)
    from flash_dropout.hip import GEMM

    assert GEMM().last_kernel() == "specialised"
    rC, rdA, rdB = _oracle_products(A, B, dC, mask, bs, p)
    for got, ref, what in ((C, rC, "C"), (dA, rdA, "dA"), (dB, rdB, "dB")):
        err = max_tile_rel_fro(got, ref, tile=bs)
        assert err <= REL_FRO_TOL, f"{what}: largest per-tile relative Frobenius error {err:.3e}"
    keep = O.expand_keep(mask.cpu().numpy(), bs, M, K)
    assert (dA.float().cpu().numpy()[~keep] == 0).all(), "dropped dX blocks must be exactly zero"


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_quadrant_masks_on_the_256_tile_kernels_leave_out_the_dropped_quadrants(dtype, tile_policy):
    """Masks of block size 32 on aligned operands under the 256 x 256 workgroup shape: the kernels that alternate
    memory and compute phases take them (not the ragged-edge instances) and leave out the MFMAs of dropped 32 x 32
    quadrants.  Structured masks - one quadrant per 64-tile kept, a checkerboard of quadrants, whole 32-rows and
    32-columns dropped, nearly everything dropped - against the oracle per 32 x 32 block; dropped blocks of dX
    exactly zero."""
    from flash_dropout.hip import GEMM

    if tile_policy != "big":
        pytest.skip("the 256 x 256 shape is what this test is about")
    ext = GEMM()
    M, N, K = 768, 512, 640
    gen = torch.Generator().manual_seed(21)
    A = make_operand(M, K, dtype, "cuda", gen=gen)
    B = make_operand(N, K, dtype, "cuda", scale=K ** -0.5, gen=gen)
    dC = make_operand(M, N, dtype, "cuda", gen=gen)
    mb, kb = M // 32, K // 32
    masks = {f"bernoulli_{p}": cpu_mask((mb, kb), p, gen) for p in (0.3, 0.7, 0.95)}
    for qi in range(4):  # one quadrant of every 64-tile kept
        m = torch.ones(mb, kb, dtype=torch.bool)
        m[qi // 2::2, qi % 2::2] = False
        masks[f"only_quadrant_{qi}"] = m
    m = torch.zeros(mb, kb, dtype=torch.bool)
    m[::2, ::2] = True
    m[1::2, 1::2] = True
    masks["checkerboard"] = m
    m = torch.zeros(mb, kb, dtype=torch.bool)
    m[1::2, :] = True
    masks["odd_32_rows_dropped"] = m
    m = torch.zeros(mb, kb, dtype=torch.bool)
    m[:, ::2] = True
    masks["even_32_columns_dropped"] = m
    m = torch.ones(mb, kb, dtype=torch.bool)
    m[mb - 1, kb - 1] = False
    masks["single_last_quadrant"] = m
    masks["none_dropped"] = torch.zeros(mb, kb, dtype=torch.bool)
    a, b, dc = to_np(A), to_np(B), to_np(dC)
    for name, mk in masks.items():
        _, lists, kbs = ext.kept_lists(M, K, 32, mask=mk.cuda())
        C = ext.gemm_dsd_lists(A, B, lists, kbs, 2.0)
        assert ext.last_kernel_detail().startswith("dsd:big splits"), (name, ext.last_kernel_detail())
        dA = ext.gemm_sdd_lists(dC, B.T, lists, kbs, 2.0)
        assert ext.last_kernel_detail() == "sdd:big", (name, ext.last_kernel_detail())
        dB = ext.gemm_dsd_lists(A.T, dC.T, lists.transposed(), kbs, 2.0).T
        assert ext.last_kernel_detail().startswith("dsd:big:strided splits"), (name, ext.last_kernel_detail())
        mkn = mk.numpy()
        for got, ref, what in ((C, O.gemm_dsd(a, b, mkn, 32, 2.0, np.float32), "C"),
                               (dA, O.gemm_sdd(dc, b.T, mkn, 32, 2.0, np.float32), "dA"),
                               (dB, O.gemm_dsd(a.T, dc.T, mkn.T, 32, 2.0, np.float32).T, "dB")):
            assert max_tile_rel_fro(got, ref, tile=32) <= REL_FRO_TOL, (name, what)
        keep = O.expand_keep(mkn, 32, M, K)
        assert (dA.float().cpu().numpy()[~keep] == 0).all(), name


@pytest.mark.parametrize("M,N,K", [(128, 64, 64), (256, 192, 128), (384, 320, 192), (1024, 448, 1024),
                                   (2048, 2048, 2048), (4096, 1024, 1024)])
@pytest.mark.parametrize("p", [0.0, 0.5, 0.9])
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_loops_with_several_steps_in_flight(M, N, K, p, dtype, tile_policy):
    """Aligned products too small for the 256 x 256 shapes run loops that keep two or three steps in flight: fewer
    steps than stages (K = 64, 128, 192), column tiles that overhang N (N = 64 mod 128), steps in which a wave keeps
    nothing (p = 0.9), and the routes themselves."""
    from flash_dropout.hip import GEMM

    ext = GEMM()
    gen = torch.Generator().manual_seed(M + N + K)
    A = make_operand(M, K, dtype, "cuda", gen=gen)
    B = make_operand(N, K, dtype, "cuda", scale=K ** -0.5, gen=gen)
    dC = make_operand(M, N, dtype, "cuda", gen=gen)
    mk = cpu_mask((M // 64, K // 64), p, gen)
    lists = ext.build_lists(mk.cuda())
    s = 1 / (1 - p)
    C = ext.gemm_dsd_lists(A, B, lists, 64, s)
    routes = [ext.last_kernel_detail()]
    dA = ext.gemm_sdd_lists(dC, B.T, lists, 64, s, keep_hint=1 - p)
    routes.append(ext.last_kernel_detail())
    dB = ext.gemm_dsd_lists(A.T, dC.T, lists.transposed(), 64, s).T
    routes.append(ext.last_kernel_detail())
    if tile_policy == "auto" and (M, N, K) == (2048, 2048, 2048):
        assert routes == ["dsd:mid splits=1", "sdd:small", "dsd:mid:strided splits=1"], routes
    if tile_policy == "mid":
        assert routes[1] == "sdd:mid", routes
    rC, rdA, rdB = _oracle_products(A, B, dC, mk, 64, p)
    for got, ref, what in ((C, rC, "C"), (dA, rdA, "dA"), (dB, rdB, "dB")):
        assert max_tile_rel_fro(got, ref) <= REL_FRO_TOL, (what, routes)
    keep = O.expand_keep(mk.numpy(), 64, M, K)
    assert (dA.float().cpu().numpy()[~keep] == 0).all()


def _structured_masks(mb, cb, gen):
    """Masks that steer the grouped SDD kernel through its branches: groups cut by the 6-active-column
    limit, by the 16-kept-tile limit, long runs of all-dropped columns, single tiles, ragged row quads."""
    masks = {}
    for p in (0.05, 0.3, 0.9, 0.97):
        masks[f"bernoulli_{p}"] = cpu_mask((mb, cb), p, gen)
    m = torch.ones(mb, cb, dtype=torch.bool)
    m[:, ::2] = False
    masks["every_other_column_kept"] = m            # 4 kept per active column: cut at 16 tiles
    m = torch.ones(mb, cb, dtype=torch.bool)
    m[::4, :] = False
    masks["one_row_of_each_quad_kept"] = m          # 1 kept per column: cut at 6 active columns
    m = torch.ones(mb, cb, dtype=torch.bool)
    m[0, 0] = False
    masks["single_first_tile"] = m
    m = torch.ones(mb, cb, dtype=torch.bool)
    m[mb - 1, cb - 1] = False
    masks["single_last_tile"] = m
    m = torch.ones(mb, cb, dtype=torch.bool)
    m[:, cb - 1] = False
    masks["last_column_only"] = m
    m = torch.zeros(mb, cb, dtype=torch.bool)
    m[:, 3: cb - 2] = True
    masks["gap_in_the_middle"] = m
    masks["all_dropped"] = torch.ones(mb, cb, dtype=torch.bool)
    masks["none_dropped"] = torch.zeros(mb, cb, dtype=torch.bool)
    return masks


@pytest.mark.parametrize("M,N,K", [(576, 256, 1216), (256, 128, 4480)])
def test_sdd_column_groups(M, N, K):
    """dX = (dY . W) (.) keep on shapes whose block grid is not a multiple of the 4-row quads (9 row blocks)
    or of any group width (19 / 70 column blocks), under structured masks."""
    from flash_dropout.hip import GEMM

    ext = GEMM()
    gen = torch.Generator().manual_seed(11)
    dC = make_operand(M, N, torch.float16, "cuda", gen=gen)
    B = make_operand(N, K, torch.float16, "cuda", scale=N ** -0.5, gen=gen)
    dc, b = to_np(dC), to_np(B)
    for name, mk in _structured_masks(M // 64, K // 64, gen).items():
        got = ext.gemm_sdd(dC, B.T, mk.cuda(), 64, 2.0)
        ref = O.gemm_sdd(dc, b.T, mk.numpy(), 64, 2.0, np.float32)
        assert max_tile_rel_fro(got, ref) <= REL_FRO_TOL, name
        keep = O.expand_keep(mk.numpy(), 64, M, K)
        assert (got.cpu().numpy()[~keep] == 0).all(), name


@pytest.mark.parametrize("M,N,K", [(1000, 256, 512), (19700 // 4, 384, 768), (70, 128, 192), (4097, 512, 256),
                                   (8200, 128, 576),
                                   # feature dimensions that are multiples of 8 but not of 64
                                   (4096, 1024, 784), (1000, 1000, 1000), (70, 72, 200), (256, 264, 72),
                                   (300, 8, 8), (8200, 72, 200), (130, 320, 56), (64, 64, 4104)])
@pytest.mark.parametrize("p", [0.0, 0.5])
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_ragged_shapes_stay_on_the_specialised_kernels(M, N, K, p, dtype):
    """M (batch x sequence) is rarely a multiple of 64, and feature counts such as 784 or 1000 are not either:
    forward, dX and dW all run on the specialised kernels with ragged last blocks along any of M, N, K
    (any M; N and K multiples of 8, the 16 bytes of one load), and match the oracle."""
    from flash_dropout.hip import GEMM

    ext = GEMM()
    gen = torch.Generator().manual_seed(M + N)
    A = make_operand(M, K, dtype, "cuda", gen=gen)
    B = make_operand(N, K, dtype, "cuda", scale=K ** -0.5, gen=gen)
    dC = make_operand(M, N, dtype, "cuda", gen=gen)
    mk = cpu_mask(O.mask_shape(M, K, 64), p, gen)
    lists = ext.build_lists(mk.cuda())
    s = 1 / (1 - p)
    C = ext.gemm_dsd_lists(A, B, lists, 64, s)
    assert ext.last_kernel() == "specialised"
    dA = ext.gemm_sdd_lists(dC, B.T, lists, 64, s)
    assert ext.last_kernel() == "specialised"
    dB = ext.gemm_dsd_lists(A.T, dC.T, lists.transposed(), 64, s, transposed_out=True).T
    assert ext.last_kernel() == "specialised"
    dBt = ext.gemm_dsd_lists(A.T, dC.T, lists.transposed(), 64, s)  # [K, N] row-major
    assert ext.last_kernel() == "specialised"
    rC, rdA, rdB = _oracle_products(A, B, dC, mk, 64, p)
    for got, ref, what in ((C, rC, "C"), (dA, rdA, "dA"), (dB, rdB, "dB"), (dBt, rdB.T, "dBt")):
        assert tuple(got.shape) == ref.shape, what
        assert max_tile_rel_fro(got, ref) <= REL_FRO_TOL, what
    keep = O.expand_keep(mk.numpy(), 64, M, K)
    assert (to_np(dA)[~keep] == 0).all()
    # the dense products on the same ragged shape
    assert max_tile_rel_fro(ext.gemm(A, B), to_np(A) @ to_np(B).T) <= REL_FRO_TOL
    assert ext.last_kernel() == "specialised"
    assert max_tile_rel_fro(ext.gemm(A.T, dC.T, transposed_out=True), to_np(A).T @ to_np(dC)) <= REL_FRO_TOL
    assert ext.last_kernel() == "specialised"


@pytest.mark.parametrize("M,N,K", [(8192, 8192, 8192), (16384, 1536, 384), (16384, 384, 1536), (131072, 128, 576)])
def test_baseline_shapes_run_on_the_specialised_kernels(M, N, K):
    """The benchmark configurations must not fall back to the generic kernel (shapes only: tiny launches
    on uninitialised operands)."""
    from flash_dropout.hip import GEMM

    ext = GEMM()
    A = torch.empty(M, K, dtype=torch.float16, device="cuda").zero_()
    B = torch.empty(N, K, dtype=torch.float16, device="cuda").zero_()
    dC = torch.empty(M, N, dtype=torch.float16, device="cuda").zero_()
    mask = torch.rand(M // 64, K // 64, device="cuda") < 0.5
    lists = ext.build_lists(mask)
    ext.gemm_dsd_lists(A, B, lists, 64, 2.0)
    assert ext.last_kernel() == "specialised"
    ext.gemm_sdd_lists(dC, B.T, lists, 64, 2.0)
    assert ext.last_kernel() == "specialised"
    ext.gemm_dsd_lists(A.T, dC.T, lists.transposed(), 64, 2.0, transposed_out=True)
    assert ext.last_kernel() == "specialised"
    # and the reference-style calls with a block size of 128
    mask128 = torch.rand(-(-M // 128), -(-K // 128), device="cuda") < 0.5
    ext.gemm_dsd(A, B, mask128, 128, 2.0)
    assert ext.last_kernel() == "specialised"
    ext.gemm_sdd(dC, B.T, mask128, 128, 2.0)
    assert ext.last_kernel() == "specialised"
    ext.gemm_dsd(A.T, dC.T, mask128.T, 128, 2.0)
    assert ext.last_kernel() == "specialised"


def test_sdd_shape_choice_follows_the_keep_hint_not_the_scale(tile_policy):
    """The SDD launcher picks its workgroup shape from the caller's estimate of the kept fraction, never from
    `scale`: a 3072 x 3072 output gives the large shape 144 workgroups when groups are 4 column blocks wide
    (kept fraction unknown or high) and 96 when they are 6 wide (a quarter kept), which is under the limit below
    which the small shape runs.  scale = 1.0 with a 75 %-dropped mask must still take the hint."""
    if tile_policy != "auto":
        pytest.skip("the choice under test is the automatic one")
    from flash_dropout.hip import GEMM

    ext = GEMM()
    M = N = 3072
    K = 128
    gen = torch.Generator().manual_seed(13)
    dC = make_operand(M, K, torch.float16, "cuda", gen=gen)
    B = make_operand(N, K, torch.float16, "cuda", row_major=False, scale=K ** -0.5, gen=gen)  # W.T as in backward
    mk = cpu_mask((M // 64, N // 64), 0.75, gen)
    lists = ext.build_lists(mk.cuda())
    ref = O.gemm_sdd(to_np(dC), to_np(B), mk.numpy(), 64, 1.0, np.float32)
    got = ext.gemm_sdd_lists(dC, B, lists, 64, 1.0, keep_hint=0.25)
    assert ext.last_kernel_detail() == "sdd:mid"
    assert max_tile_rel_fro(got, ref) <= REL_FRO_TOL
    got = ext.gemm_sdd_lists(dC, B, lists, 64, 4.0)  # no hint: counted as everything kept, whatever the scale
    assert ext.last_kernel_detail() == "sdd:big"
    assert max_tile_rel_fro(got, 4.0 * ref) <= REL_FRO_TOL
    got = ext.gemm_sdd_lists(dC, B, lists, 64, 1.0, keep_hint=0.9)
    assert ext.last_kernel_detail() == "sdd:big"
    with pytest.raises(ValueError, match="keep_hint"):
        ext.gemm_sdd_lists(dC, B, lists, 64, 1.0, keep_hint=1.5)


@pytest.mark.parametrize("M,N,K", [(512, 256, 576), (1000, 128, 200), (4096, 64, 4104)])
def test_sdd_kept_only_leaves_dropped_tiles_untouched(M, N, K):
    """sd_gemm_sdd_lists_kept: kept tiles equal the ordinary call's, dropped tiles keep what the buffer held."""
    from flash_dropout.hip import GEMM

    ext = GEMM()
    gen = torch.Generator().manual_seed(3)
    dC = make_operand(M, N, torch.float16, "cuda", gen=gen)
    B = make_operand(N, K, torch.float16, "cuda", scale=N ** -0.5, gen=gen)
    mk = cpu_mask(O.mask_shape(M, K, 64), 0.5, gen)
    lists = ext.build_lists(mk.cuda())
    full = ext.gemm_sdd_lists(dC, B.T, lists, 64, 2.0)
    sentinel = 123.0
    out = torch.full((M, K), sentinel, dtype=torch.float16, device="cuda")
    got = ext.gemm_sdd_lists(dC, B.T, lists, 64, 2.0, out=out, kept_only=True)
    keep = torch.from_numpy(O.expand_keep(mk.numpy(), 64, M, K)).cuda()
    assert torch.equal(got[keep], full[keep])
    assert (got[~keep] == sentinel).all()


# ---- block size 32: four mask blocks per 64 x 64 tile of the kernels -------------------------------------------
@pytest.mark.parametrize("mnk,p", list(product(REF_MNKS, REF_PS)))
def test_reference_grid_at_block_size_32(mnk, p):
    """The reference's shape and drop-rate grid (test/test_cuda.py:12-20) at block size 32, which its Triton path
    takes (flash_dropout/triton/utils.py:6-19): Y, dX and dW against the oracle, dropped 32-blocks of dX exactly
    zero."""
    M, N, K = mnk
    bs = 32
    gen = torch.Generator().manual_seed(20)
    A = make_operand(M, K, torch.float16, "cuda", gen=gen)
    # weights scaled as a layer's are: with N(0, 1) weights the kept blocks at p = 0.999 (scale 1000) overflow fp16
    B = make_operand(N, K, torch.float16, "cuda", scale=K ** -0.5, gen=gen)
    dC = make_operand(M, N, torch.float16, "cuda", gen=gen)
    mask = cpu_mask((M // bs, K // bs), p, gen).cuda()
    C, dA, dB = _three_products(A, B, dC, mask, bs, p)
    rC, rdA, rdB = _oracle_products(A, B, dC, mask, bs, p)
    atol = 0.2 * max(1.0, (1 / (1 - p)) / 10)
    _check(C, rC, "C", atol)
    _check(dB, rdB, "dB", atol)
    _check(dA, rdA, "dA", atol)
    keep = O.expand_keep(mask.cpu().numpy(), bs, M, K)
    assert (dA.cpu().numpy()[~keep] == 0).all(), "dropped dX blocks must be exactly zero"


@pytest.mark.parametrize("M,N,K", [(1000, 136, 200), (100, 70, 50), (4096, 10, 1024), (4096, 1024, 784), (96, 64, 160),
                                   (16384, 384, 1536)])
@pytest.mark.parametrize("p", [0.3, 0.75])
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_block_size_32_on_ragged_and_model_shapes(M, N, K, p, dtype):
    """Block size 32 where the 32-grid has an odd number of blocks, the shape is ragged against both grids, or
    the operands force the generic kernel (K = 50): mask forms and list forms, all three products."""
    from flash_dropout.hip import GEMM

    ext = GEMM()
    gen = torch.Generator().manual_seed(M + K)
    A = make_operand(M, K, dtype, "cuda", gen=gen)
    B = make_operand(N, K, dtype, "cuda", scale=K ** -0.5, gen=gen)
    dC = make_operand(M, N, dtype, "cuda", gen=gen)
    mk = cpu_mask(O.mask_shape(M, K, 32), p, gen)
    C, dA, dB = _three_products(A, B, dC, mk.cuda(), 32, p)
    rC, rdA, rdB = _oracle_products(A, B, dC, mk, 32, p)
    for got, ref, what in ((C, rC, "C"), (dA, rdA, "dA"), (dB, rdB, "dB")):
        assert max_tile_rel_fro(got, ref, tile=32) <= REL_FRO_TOL, what
    keep = O.expand_keep(mk.numpy(), 32, M, K)
    assert (to_np(dA)[~keep] == 0).all()
    # the list forms on lists built once (block size 32 tells them that the lists carry quadrant bits)
    lists = ext.build_lists(mk.cuda(), split=0)
    s = 1 / (1 - p)
    assert torch.equal(ext.gemm_dsd_lists(A, B, lists, 32, s), C)
    assert torch.equal(ext.gemm_sdd_lists(dC, B.T, lists, 32, s), dA)
    dBl = ext.gemm_dsd_lists(A.T, dC.T, lists.transposed(), 32, s, transposed_out=True).T
    assert max_tile_rel_fro(dBl, rdB, tile=32) <= REL_FRO_TOL


# ---- odd multiples of 32 (96, 160): the mask split to its 32-blocks, those merged onto the kernels' 64 grid ----------
@pytest.mark.parametrize("mnk,p", list(product(REF_MNKS, REF_PS)))
@pytest.mark.parametrize("bs", [96, 160])
def test_reference_grid_at_odd_multiples_of_32(mnk, p, bs, tile_policy):
    """The reference's shape and drop-rate grid at block sizes 96 and 160, which its Triton path takes (any block size
    its 32-wide tiles divide, flash_dropout/triton/utils.py:6-19): Y, dX and dW against the oracle at that block size
    (the shapes are not multiples of it: the mask's last row and column of blocks are cropped), dropped blocks of dX
    exactly zero."""
    if tile_policy == "big":
        pytest.skip("two shape policies are enough here")
    M, N, K = mnk
    gen = torch.Generator().manual_seed(24)
    A = make_operand(M, K, torch.float16, "cuda", gen=gen)
    B = make_operand(N, K, torch.float16, "cuda", scale=K ** -0.5, gen=gen)
    dC = make_operand(M, N, torch.float16, "cuda", gen=gen)
    mask = cpu_mask(O.mask_shape(M, K, bs), p, gen).cuda()
    C, dA, dB = _three_products(A, B, dC, mask, bs, p)
    rC, rdA, rdB = _oracle_products(A, B, dC, mask, bs, p)
    atol = 0.2 * max(1.0, (1 / (1 - p)) / 10)
    _check(C, rC, "C", atol)
    _check(dB, rdB, "dB", atol)
    _check(dA, rdA, "dA", atol)
    keep = O.expand_keep(mask.cpu().numpy(), bs, M, K)
    assert (dA.cpu().numpy()[~keep] == 0).all(), "dropped dX blocks must be exactly zero"


@pytest.mark.parametrize("M,N,K,bs", [(1000, 136, 200, 96), (100, 70, 50, 96), (4096, 1024, 784, 160), (130, 64, 290, 96),
                                      (16384, 384, 1536, 224)])
def test_odd_multiples_of_32_on_ragged_and_model_shapes(M, N, K, bs):
    """Ragged shapes (against the block size, the 64 grid and the 32 grid), the generic kernel (K = 50) and a model
    shape: mask forms and list forms of all three products at block sizes 96, 160 and 224."""
    from flash_dropout.hip import GEMM

    ext = GEMM()
    p = 0.4
    gen = torch.Generator().manual_seed(M + K + bs)
    A = make_operand(M, K, torch.float16, "cuda", gen=gen)
    B = make_operand(N, K, torch.float16, "cuda", scale=K ** -0.5, gen=gen)
    dC = make_operand(M, N, torch.float16, "cuda", gen=gen)
    mk = cpu_mask(O.mask_shape(M, K, bs), p, gen)
    C, dA, dB = _three_products(A, B, dC, mk.cuda(), bs, p)
    rC, rdA, rdB = _oracle_products(A, B, dC, mk, bs, p)
    for got, ref, what in ((C, rC, "C"), (dA, rdA, "dA"), (dB, rdB, "dB")):
        assert max_tile_rel_fro(got, ref, tile=32) <= REL_FRO_TOL, what
    keep = O.expand_keep(mk.numpy(), bs, M, K)
    assert (to_np(dA)[~keep] == 0).all()
    # the list forms on lists built once: block size 32 tells them that the lists carry quadrant bits
    lists = ext.build_lists(mk.cuda(), split=-(bs // 32), grid=(-(-M // 64), -(-K // 64)))
    s = 1 / (1 - p)
    assert torch.equal(ext.gemm_dsd_lists(A, B, lists, 32, s), C)
    assert torch.equal(ext.gemm_sdd_lists(dC, B.T, lists, 32, s), dA)
