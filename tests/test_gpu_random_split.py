"""On-device mask draw fused with the list build, and block splitting (a logical block size that is a
larger multiple of 64 listed at 64 granularity), through the C ABI and the functional API."""
import numpy as np
import pytest
import torch

from _util import REL_FRO_TOL, max_tile_rel_fro, cpu_mask, rel_fro
from oracle import sparsedrop_oracle as O

pytestmark = pytest.mark.gpu


def make_operand(shape, dtype, gen, scale=1.0):
    return (torch.randn(*shape, generator=gen) * scale).to(dtype)


def _lists_np(lists):
    nnz = lists.nnz()
    return (lists.row_ptr.cpu().numpy(), lists.col_idx[:nnz].cpu().numpy(),
            lists.col_ptr.cpu().numpy(), lists.row_idx[:nnz].cpu().numpy())


def _assert_lists(lists, mask_np):
    rp, ci, cp, ri = _lists_np(lists)
    want_rp, want_ci = O.compact_csr(mask_np)
    want_cp, want_ri = O.compact_csc(mask_np)
    assert lists.shape == mask_np.shape
    assert np.array_equal(rp, want_rp) and np.array_equal(ci, want_ci)
    assert np.array_equal(cp, want_cp) and np.array_equal(ri, want_ri)


@pytest.mark.parametrize("shape,p,seed,offset", [
    ((16, 16), 0.5, 0, 0),
    ((128, 128), 0.5, 1234, 0),
    ((37, 53), 0.25, (5 << 32) | 9, (1 << 32) | 2),
    ((1, 1), 0.5, 3, 0),
    ((3, 700), 0.75, 2 ** 63 + 5, 7),
    ((128, 128), 0.0, 1, 0),
    ((600, 600), 0.5, 99, 1),          # more than 2^18 entries: the multi-launch builder
])
def test_random_lists_bit_exact(shape, p, seed, offset):
    from flash_dropout.hip import GEMM

    mask, lists = GEMM().random_lists(shape, p, seed, offset)
    want = O.random_mask(shape, p, seed, offset)
    assert mask.dtype == torch.bool and tuple(mask.shape) == shape
    assert np.array_equal(mask.cpu().numpy(), want)
    _assert_lists(lists, want)


@pytest.mark.parametrize("shape,split,grid", [
    ((4, 6), 2, None), ((4, 6), 2, (7, 11)), ((5, 3), 3, (13, 7)), ((64, 64), 2, (128, 127)),
    ((300, 300), 2, (599, 600)),       # multi-launch builder
])
def test_split_lists_bit_exact(shape, split, grid):
    from flash_dropout.hip import GEMM

    gen = torch.Generator().manual_seed(4)
    mask = cpu_mask(shape, 0.5, gen)
    want = O.split_mask(mask.numpy(), split, grid)
    _assert_lists(GEMM().build_lists(mask.cuda(), split, grid), want)
    _assert_lists(GEMM().build_lists(mask.t().contiguous().t().cuda(), split, grid), want)  # column-major mask
    # drawn + split in one launch
    m2, l2 = GEMM().random_lists(shape, 0.5, 77, split=split, grid=grid)
    _assert_lists(l2, O.split_mask(O.random_mask(shape, 0.5, 77), split, grid))
    assert np.array_equal(m2.cpu().numpy(), O.random_mask(shape, 0.5, 77))


def test_split_grid_is_validated():
    from flash_dropout.hip import GEMM

    mask = torch.zeros(4, 4, dtype=torch.bool, device="cuda")
    with pytest.raises(ValueError):
        GEMM().build_lists(mask, 2, (6, 8))   # 6 rows would not touch the last mask row
    with pytest.raises(ValueError):
        GEMM().build_lists(mask, 2, (8, 9))


@pytest.mark.parametrize("m,n,k,bs", [(512, 512, 512, 128), (384, 256, 640, 128), (200, 136, 328, 128),
                                      (768, 256, 384, 192), (1024, 512, 1024, 256)])
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_mask_entry_points_with_larger_blocks(m, n, k, bs, dtype):
    """gemm_dsd / gemm_sdd with the reference's own block size (128, matmul_dsd.cuh:92-93) and other
    multiples of 64 against the oracle at that block size."""
    from flash_dropout.hip import GEMM

    ext = GEMM()
    gen = torch.Generator().manual_seed(m + n + bs)
    a = make_operand((m, k), dtype, gen)
    b = make_operand((n, k), dtype, gen, scale=k ** -0.5)
    mask = cpu_mask(O.mask_shape(m, k, bs), 0.5, gen)
    got = ext.gemm_dsd(a.cuda(), b.cuda(), mask.cuda(), bs, 2.0)
    want = O.gemm_dsd(a.float().numpy(), b.float().numpy(), mask.numpy(), bs, 2.0)
    assert max_tile_rel_fro(got, want) <= REL_FRO_TOL
    # SDD: A [m, k] x B [n, k] with the mask over the [m, n] result
    mask_c = cpu_mask(O.mask_shape(m, n, bs), 0.5, gen)
    got = ext.gemm_sdd(a.cuda(), b.cuda(), mask_c.cuda(), bs, 2.0)
    want = O.gemm_sdd(a.float().numpy(), b.float().numpy(), mask_c.numpy(), bs, 2.0)
    assert max_tile_rel_fro(got, want) <= REL_FRO_TOL
    keep = torch.from_numpy(O.expand_keep(mask_c.numpy(), bs, m, n))
    assert bool((got.cpu()[~keep] == 0).all())  # dropped tiles are exact zeros


@pytest.mark.parametrize("bs", [64, 128])
@pytest.mark.parametrize("p", [0.0, 0.5])
def test_functional_draws_its_mask_on_the_device(bs, p):
    """blockwise_dropout_matmul(seed=...) uses the mask random_lists returns for that seed; forward and
    both gradients match the oracle under that mask."""
    import flash_dropout.functional as F
    from flash_dropout.hip import GEMM

    m, n, k = 512, 256, 768
    gen = torch.Generator().manual_seed(8)
    x = make_operand((m, k), torch.float16, gen)
    w = make_operand((n, k), torch.float16, gen, scale=k ** -0.5)
    dy = make_operand((m, n), torch.float16, gen)
    xg, wg = x.cuda().requires_grad_(), w.cuda().requires_grad_()
    y = F.hip_blockwise_dropout_matmul(xg, wg, bs, p, seed=4242)
    y.backward(dy.cuda())
    mask = O.random_mask(O.mask_shape(m, k, bs), p, 4242)
    dev_mask, _ = GEMM().random_lists(O.mask_shape(m, k, bs), p, 4242)
    assert np.array_equal(dev_mask.cpu().numpy(), mask)
    xf, wf, dyf = x.float().numpy(), w.float().numpy(), dy.float().numpy()
    assert max_tile_rel_fro(y, O.dsd_forward(xf, wf, mask, bs, p)) <= REL_FRO_TOL
    assert max_tile_rel_fro(xg.grad, O.sdd_dx(dyf, wf, mask, bs, p)) <= REL_FRO_TOL
    assert max_tile_rel_fro(wg.grad, O.dsd_dw(dyf, xf, mask, bs, p)) <= REL_FRO_TOL


def test_functional_mask_follows_torch_seed():
    import flash_dropout.functional as F
    from flash_dropout.hip import GEMM

    x = torch.ones(256, 256, dtype=torch.float16, device="cuda")
    w = torch.eye(256, dtype=torch.float16, device="cuda")
    torch.manual_seed(3)
    a = F.hip_blockwise_dropout_matmul(x, w, 64, 0.5)
    b = F.hip_blockwise_dropout_matmul(x, w, 64, 0.5)
    assert not torch.equal(a, b)        # consecutive calls draw different masks
    torch.manual_seed(4)                # a new torch seed restarts the device generator from it
    c = F.hip_blockwise_dropout_matmul(x, w, 64, 0.5)
    assert not torch.equal(a, c)
    torch.manual_seed(3)
    a2 = F.hip_blockwise_dropout_matmul(x, w, 64, 0.5)
    assert torch.equal(a, a2)           # same seed, same first mask
    keep = torch.from_numpy(O.expand_keep(O.random_mask((4, 4), 0.5, 3, offset=0), 64, 256, 256)).cuda()
    assert torch.equal(a != 0, keep)    # and it is draw 0 of seed 3
    ext = GEMM()
    ext.manual_seed(77)                 # explicit restart, independent of torch's seed
    m0, _ = ext.random_lists((5, 7), 0.4)
    m1, _ = ext.random_lists((5, 7), 0.4)
    assert ext.rng_state().tolist() == [77, 2, 0, 0]
    assert np.array_equal(m0.cpu().numpy(), O.random_mask((5, 7), 0.4, 77, offset=0))
    assert np.array_equal(m1.cpu().numpy(), O.random_mask((5, 7), 0.4, 77, offset=1))
    # large mask: the multi-launch builder reads the same state in all of its kernels
    m2, l2 = ext.random_lists((600, 600), 0.5)
    want = O.random_mask((600, 600), 0.5, 77, offset=2)
    assert np.array_equal(m2.cpu().numpy(), want)
    _assert_lists(l2, want)
    assert ext.rng_state().tolist() == [77, 3, 0, 0]


def test_graph_replays_draw_fresh_masks():
    """A captured forward + backward step replays correctly and every replay draws a new mask: nothing
    about the draw is a launch argument.  Replays are separated by eager work and synchronisation, and
    each is checked against the oracle under the mask it must have drawn."""
    import flash_dropout.functional as F
    from flash_dropout.hip import GEMM

    ext = GEMM()
    m, n, k, p = 512, 256, 384, 0.5
    gen = torch.Generator().manual_seed(21)
    x = make_operand((m, k), torch.float16, gen)
    w = make_operand((n, k), torch.float16, gen, scale=k ** -0.5)
    dy = make_operand((m, n), torch.float16, gen)
    xg, wg, dyg = x.cuda().requires_grad_(), w.cuda().requires_grad_(), dy.cuda()
    ext.manual_seed(5)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):       # warm-up on the capture stream: kernels configured, state created
        for _ in range(2):
            F.hip_blockwise_dropout_matmul(xg, wg, 64, p).backward(dyg)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    xg.grad = wg.grad = None
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        y = F.hip_blockwise_dropout_matmul(xg, wg, 64, p)
        y.backward(dyg)
    torch.cuda.synchronize()
    first = int(ext.rng_state()[1].item())   # capture itself does not run the kernels
    assert first == 2
    xf, wf, dyf = x.float().numpy(), w.float().numpy(), dy.float().numpy()
    seen = []
    for r in range(3):
        graph.replay()
        torch.cuda.synchronize()
        mask = O.random_mask(O.mask_shape(m, k, 64), p, 5, offset=first + r)
        assert max_tile_rel_fro(y, O.dsd_forward(xf, wf, mask, 64, p)) <= REL_FRO_TOL, r
        assert max_tile_rel_fro(xg.grad, O.sdd_dx(dyf, wf, mask, 64, p)) <= REL_FRO_TOL, r
        assert max_tile_rel_fro(wg.grad, O.dsd_dw(dyf, xf, mask, 64, p)) <= REL_FRO_TOL, r
        seen.append(mask)
        # eager work between replays
        eager = F.hip_blockwise_dropout_matmul_mask(xg.detach(), torch.from_numpy(mask).cuda(), 64, p, wg.detach())
        assert rel_fro(eager, y) <= 1e-3
        torch.cuda.synchronize()
    assert not np.array_equal(seen[0], seen[1]) and not np.array_equal(seen[1], seen[2])
    assert int(ext.rng_state()[1].item()) == first + 3


def test_conv_with_larger_blocks_and_device_mask():
    import flash_dropout.functional as F

    gen = torch.Generator().manual_seed(6)
    x = torch.randn(4, 32, 16, 16, generator=gen).half()
    kern = ((torch.rand(64, 32, 3, 3, generator=gen) * 2 - 1) * (32 * 9) ** -0.5).half()
    rows, ncols = 4 * 16 * 16, 32 * 9
    bs, p = 128, 0.5
    mask = O.random_mask(O.mask_shape(rows, ncols, bs), p, 31)
    xg, kg = x.cuda().requires_grad_(), kern.cuda().requires_grad_()
    y = F.blockwise_dropout_conv2d(xg, kg, bs, p, padding=(1, 1), seed=31)
    dy = torch.randn(y.shape, generator=gen).half()
    y.backward(dy.cuda())
    geo = dict(padding=(1, 1), stride=(1, 1), dilation=(1, 1))
    want_y, want_dx, want_dk = O.conv2d_blockdrop(x.float().numpy(), kern.float().numpy(), mask, bs, p,
                                                  dy=dy.float().numpy(), **geo)
    assert max_tile_rel_fro(y, want_y) <= REL_FRO_TOL
    assert max_tile_rel_fro(xg.grad, want_dx) <= REL_FRO_TOL
    assert max_tile_rel_fro(kg.grad, want_dk) <= REL_FRO_TOL


def test_reseeding_after_capture_is_followed_by_the_graph():
    """The generator state is one tensor per device for the life of the process, reseeded in place: a graph
    captured before manual_seed() keeps a valid address and its next replay draws from the new seed at offset 0
    (it used to keep reading the freed old state)."""
    from flash_dropout.hip import GEMM

    ext = GEMM()
    shape, p = (24, 40), 0.5
    ext.manual_seed(3)
    state = ext.rng_state()
    ptr = state.data_ptr()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        ext.random_lists(shape, p)  # warm-up on the capture stream
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        mask, lists = ext.random_lists(shape, p)
    graph.replay()
    torch.cuda.synchronize()
    assert np.array_equal(mask.cpu().numpy(), O.random_mask(shape, p, 3, offset=1))
    ext.manual_seed(7)
    assert ext.rng_state().data_ptr() == ptr, "reseeding must not move the state a graph has captured"
    graph.replay()
    torch.cuda.synchronize()
    assert np.array_equal(mask.cpu().numpy(), O.random_mask(shape, p, 7, offset=0))
    rp, ci = O.compact_csr(O.random_mask(shape, p, 7, offset=0))
    assert np.array_equal(lists.row_ptr.cpu().numpy(), rp)
    assert np.array_equal(lists.col_idx[: lists.nnz()].cpu().numpy(), ci)
    graph.replay()
    torch.cuda.synchronize()
    assert np.array_equal(mask.cpu().numpy(), O.random_mask(shape, p, 7, offset=1))
    # torch.manual_seed with a new seed restarts the generator in the same tensor as well
    torch.manual_seed(1234)
    assert ext.rng_state().data_ptr() == ptr
    graph.replay()
    torch.cuda.synchronize()
    assert np.array_equal(mask.cpu().numpy(), O.random_mask(shape, p, 1234, offset=0))
