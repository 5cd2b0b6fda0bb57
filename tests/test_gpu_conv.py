"""Kernel (e): im2col gather / col2im and the conv path built on them, against the CPU oracle."""
import numpy as np
import pytest
import torch

from _util import REL_FRO_TOL, max_tile_rel_fro, cpu_mask, rel_fro, to_np
from oracle import sparsedrop_oracle as O

pytestmark = pytest.mark.gpu

GEOMS = [
    dict(n=2, c=3, h=8, w=8, r=3, s=3, padding=(1, 1), stride=(1, 1), dilation=(1, 1)),
    dict(n=3, c=5, h=13, w=9, r=3, s=2, padding=(0, 1), stride=(2, 1), dilation=(1, 2)),
    dict(n=4, c=64, h=16, w=16, r=3, s=3, padding=(1, 1), stride=(1, 1), dilation=(1, 1)),
    dict(n=2, c=16, h=10, w=10, r=1, s=1, padding=(0, 0), stride=(1, 1), dilation=(1, 1)),
    dict(n=1, c=8, h=12, w=12, r=5, s=5, padding=(2, 2), stride=(2, 2), dilation=(1, 1)),
    # P*Q a multiple of 64 and C*R*S a multiple of 8: the patch-staged im2col kernel
    dict(n=2, c=24, h=24, w=24, r=3, s=3, padding=(1, 1), stride=(1, 1), dilation=(1, 1)),   # 216 columns: ragged tile
    dict(n=2, c=8, h=32, w=32, r=3, s=3, padding=(1, 1), stride=(2, 2), dilation=(1, 1)),
    dict(n=1, c=16, h=16, w=16, r=3, s=3, padding=(2, 2), stride=(1, 1), dilation=(2, 2)),
    dict(n=2, c=8, h=16, w=16, r=5, s=5, padding=(2, 2), stride=(1, 1), dilation=(1, 1)),
    dict(n=1, c=32, h=8, w=128, r=1, s=7, padding=(0, 3), stride=(1, 1), dilation=(1, 1)),   # a 64-row group inside one image row
]


def _geo(cfg):
    return dict(padding=cfg["padding"], stride=cfg["stride"], dilation=cfg["dilation"])


@pytest.mark.parametrize("cfg", GEOMS)
@pytest.mark.parametrize("channels_last", [False, True])
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_im2col_bit_exact(cfg, channels_last, dtype):
    from flash_dropout.hip import GEMM

    gen = torch.Generator().manual_seed(0)
    x = torch.randn(cfg["n"], cfg["c"], cfg["h"], cfg["w"], generator=gen).to(dtype)
    xg = x.cuda()
    if channels_last:
        xg = xg.contiguous(memory_format=torch.channels_last)
    cols = GEMM().im2col(xg, (cfg["r"], cfg["s"]), **_geo(cfg))
    ref = O.im2col(x.float().numpy(), cfg["r"], cfg["s"], **_geo(cfg))
    assert cols.shape == ref.shape
    assert np.array_equal(cols.float().cpu().numpy(), ref)  # a gather: bit exact


@pytest.mark.parametrize("cfg", [
    GEOMS[2],                                                                                   # patch-staged kernel
    dict(n=4, c=64, h=12, w=12, r=3, s=3, padding=(1, 1), stride=(1, 1), dilation=(1, 1)),      # P*Q = 144: tile-turning kernel
    dict(n=4, c=24, h=16, w=16, r=3, s=3, padding=(1, 1), stride=(1, 1), dilation=(1, 1)),      # 216 columns: ragged last block
])
@pytest.mark.parametrize("bs", [64, 128])
def test_im2col_writes_only_kept_blocks(cfg, bs):
    from flash_dropout.hip import GEMM

    ext = GEMM()
    gen = torch.Generator().manual_seed(1)
    x = torch.randn(cfg["n"], cfg["c"], cfg["h"], cfg["w"], generator=gen).half().cuda()
    ks = (cfg["r"], cfg["s"])
    p_, q_ = O.conv_out_hw(cfg["h"], cfg["w"], *ks, **_geo(cfg))
    rows, ncols = cfg["n"] * p_ * q_, cfg["c"] * cfg["r"] * cfg["s"]
    mask = cpu_mask(O.mask_shape(rows, ncols, bs), 0.5, gen)
    lists = ext.build_lists(mask.cuda())
    full = ext.im2col(x, ks, **_geo(cfg))
    part = torch.full((rows, ncols), 7.0, dtype=torch.float16, device="cuda")
    ext.im2col(x, ks, lists=lists, block_size=bs, out=part, **_geo(cfg))
    keep = torch.from_numpy(O.expand_keep(mask.numpy(), bs, rows, ncols)).cuda()
    assert torch.equal(part[keep], full[keep])
    assert bool((part[~keep] == 7.0).all())  # dropped blocks are not touched


@pytest.mark.parametrize("cfg", GEOMS)
@pytest.mark.parametrize("channels_last", [False, True])
def test_col2im_vs_oracle(cfg, channels_last):
    from flash_dropout.hip import GEMM

    gen = torch.Generator().manual_seed(2)
    p_, q_ = O.conv_out_hw(cfg["h"], cfg["w"], cfg["r"], cfg["s"], **_geo(cfg))
    rows, ncols = cfg["n"] * p_ * q_, cfg["c"] * cfg["r"] * cfg["s"]
    g = torch.randn(rows, ncols, generator=gen).half()
    shape = (cfg["n"], cfg["c"], cfg["h"], cfg["w"])
    dx = GEMM().col2im(g.cuda(), shape, (cfg["r"], cfg["s"]), channels_last=channels_last, **_geo(cfg))
    ref = O.col2im(g.float().numpy(), shape, cfg["r"], cfg["s"], **_geo(cfg))
    assert dx.shape == shape
    assert rel_fro(dx, ref) <= 2e-3  # fp32 sum of <= R*S fp16 values, one rounding
    # with a mask: dropped blocks count as zero and are not read
    mask = cpu_mask(O.mask_shape(rows, ncols, 64), 0.5, gen)
    keep = O.expand_keep(mask.numpy(), 64, rows, ncols)
    dxm = GEMM().col2im(g.cuda(), shape, (cfg["r"], cfg["s"]), mask=mask.cuda(), block_size=64, **_geo(cfg))
    refm = O.col2im(np.where(keep, g.float().numpy(), 0), shape, cfg["r"], cfg["s"], **_geo(cfg))
    assert rel_fro(dxm, refm) <= 2e-3


@pytest.mark.parametrize("cfg", [
    dict(n=8, c=64, h=32, w=32, k=128, r=3, s=3, padding=(1, 1), stride=(1, 1), dilation=(1, 1)),
    dict(n=4, c=24, h=17, w=15, k=40, r=3, s=3, padding=(1, 0), stride=(2, 1), dilation=(1, 1)),
])
@pytest.mark.parametrize("p", [0.0, 0.5])
def test_blockdrop_conv_forward_backward(cfg, p):
    """Reduced-batch version of the conv configuration (same 64->128 3x3 stride 1 pad 1 layer, 8 images
    instead of 128) plus a ragged geometry: forward, dx and dkernel against the oracle."""
    import flash_dropout.functional as F

    gen = torch.Generator().manual_seed(5)
    x = torch.randn(cfg["n"], cfg["c"], cfg["h"], cfg["w"], generator=gen).half()
    fan_in = cfg["c"] * cfg["r"] * cfg["s"]
    k = ((torch.rand(cfg["k"], cfg["c"], cfg["r"], cfg["s"], generator=gen) * 2 - 1) * fan_in ** -0.5).half()
    p_, q_ = O.conv_out_hw(cfg["h"], cfg["w"], cfg["r"], cfg["s"], **_geo(cfg))
    rows = cfg["n"] * p_ * q_
    mask = cpu_mask(O.mask_shape(rows, fan_in, 64), p, gen)
    dy = torch.randn(cfg["n"], cfg["k"], p_, q_, generator=gen).half()

    xg, kg = x.cuda().requires_grad_(), k.cuda().requires_grad_()
    y = F.blockwise_dropout_conv2d_mask(xg, mask.cuda(), 64, p, kg, **_geo(cfg))
    assert y.shape == dy.shape
    y.backward(dy.cuda())
    ry, rdx, rdk = O.conv2d_blockdrop(to_np(x), to_np(k), mask.numpy(), 64, p, dy=to_np(dy), dtype=np.float32, **_geo(cfg))
    assert max_tile_rel_fro(y, ry) <= REL_FRO_TOL
    assert max_tile_rel_fro(xg.grad, rdx) <= REL_FRO_TOL
    assert max_tile_rel_fro(kg.grad, rdk) <= REL_FRO_TOL


IMPLICIT_GEOMS = [
    # (geometry, taken by the implicit kernel)
    (dict(n=4, c=64, h=32, w=32, k=128, r=3, s=3, padding=(1, 1), stride=(1, 1), dilation=(1, 1)), True),   # the conv configuration's layer
    (dict(n=2, c=16, h=16, w=16, k=40, r=3, s=3, padding=(1, 1), stride=(1, 1), dilation=(1, 1)), True),    # 144 columns, 40 outputs: ragged both ways; 4 output rows per block
    (dict(n=3, c=8, h=32, w=32, k=64, r=5, s=5, padding=(2, 2), stride=(1, 1), dilation=(1, 1)), True),     # 25 taps
    (dict(n=2, c=64, h=32, w=32, k=256, r=1, s=1, padding=(0, 0), stride=(1, 1), dilation=(1, 1)), True),   # 1x1: one reduction block, two column tiles
    (dict(n=2, c=32, h=16, w=64, k=64, r=3, s=3, padding=(1, 1), stride=(1, 1), dilation=(1, 1)), True),    # one output row per block
    (dict(n=5, c=24, h=32, w=8, k=72, r=3, s=3, padding=(1, 1), stride=(1, 1), dilation=(1, 1)), True),     # 8 output rows per block
    (dict(n=2, c=16, h=36, w=32, k=64, r=5, s=1, padding=(0, 0), stride=(1, 1), dilation=(1, 1)), True),    # no padding: P = 32 from H = 36
    (dict(n=2, c=16, h=16, w=16, k=64, r=3, s=3, padding=(2, 2), stride=(1, 1), dilation=(1, 1)), False),   # Q = 18
    (dict(n=2, c=8, h=32, w=32, k=64, r=3, s=3, padding=(1, 1), stride=(2, 2), dilation=(1, 1)), True),     # stride 2: 16 x 16 outputs
    (dict(n=2, c=24, h=32, w=32, k=64, r=3, s=3, padding=(2, 2), stride=(1, 1), dilation=(2, 2)), True),    # dilation 2
    (dict(n=3, c=16, h=32, w=32, k=72, r=3, s=3, padding=(1, 1), stride=(2, 1), dilation=(1, 1)), True),    # stride 2 down, 1 across
    (dict(n=2, c=40, h=64, w=16, k=64, r=5, s=3, padding=(4, 1), stride=(2, 2), dilation=(2, 1)), True),    # stride and dilation, Q = 8
    (dict(n=1, c=16, h=8, w=16, k=64, r=3, s=3, padding=(1, 1), stride=(1, 1), dilation=(1, 1)), True),     # P*Q = 128: every 64-position block with its own input rows, half a workgroup
    (dict(n=5, c=32, h=8, w=8, k=64, r=3, s=3, padding=(1, 1), stride=(1, 1), dilation=(1, 1)), True),      # 8 x 8 images: a workgroup's four blocks are four images, the last workgroup has one
    (dict(n=3, c=72, h=12, w=16, k=136, r=3, s=3, padding=(1, 1), stride=(1, 1), dilation=(1, 1)), True),   # P*Q = 192: blocks of 4 rows, three per image, 648 columns
    (dict(n=1, c=256, h=32, w=32, k=64, r=3, s=3, padding=(1, 1), stride=(1, 1), dilation=(1, 1)), True),   # too many channels for one copy of the input rows: a copy per step
    (dict(n=2, c=136, h=16, w=16, k=192, r=3, s=3, padding=(1, 1), stride=(1, 1), dilation=(1, 1)), True),  # the same with 1224 columns (ragged), two column tiles
]


@pytest.fixture(params=["auto", "big"])
def copy_form(request):
    """The implicit forward keeps a copy of the input rows per step, or one copy of all channels' rows for the
    whole kernel where only that fits; the large-tile policy prefers the latter, so both run where both fit."""
    from flash_dropout.hip import GEMM

    ext = GEMM()
    prev = ext.set_tile_policy(request.param)
    yield request.param
    ext.set_tile_policy(prev)


@pytest.mark.parametrize("cfg,taken", IMPLICIT_GEOMS)
@pytest.mark.parametrize("p", [0.0, 0.5])
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_implicit_gemm_conv_forward(cfg, taken, p, dtype, copy_form):
    """sd_conv2d_dsd_lists (no patch matrix) against the oracle and against im2col + DSD on the same lists;
    geometries it does not take must come back as None with nothing written."""
    from flash_dropout.hip import GEMM

    ext = GEMM()
    gen = torch.Generator().manual_seed(cfg["c"] + cfg["k"])
    x = torch.randn(cfg["n"], cfg["c"], cfg["h"], cfg["w"], generator=gen).to(dtype)
    fan_in = cfg["c"] * cfg["r"] * cfg["s"]
    k = ((torch.rand(cfg["k"], cfg["c"], cfg["r"], cfg["s"], generator=gen) * 2 - 1) * fan_in ** -0.5).to(dtype)
    p_, q_ = O.conv_out_hw(cfg["h"], cfg["w"], cfg["r"], cfg["s"], **_geo(cfg))
    rows = cfg["n"] * p_ * q_
    mask = cpu_mask(O.mask_shape(rows, fan_in, 64), p, gen)
    lists = ext.build_lists(mask.cuda())
    xg, w2 = x.cuda(), k.cuda().reshape(cfg["k"], fan_in)
    s = 1 / (1 - p)
    y = ext.conv2d_dsd_lists(xg, w2, lists, 64, s, (cfg["r"], cfg["s"]), **_geo(cfg))
    if not taken:
        assert y is None
        return
    assert y is not None and tuple(y.shape) == (rows, cfg["k"])
    assert ext.last_kernel() == "specialised"
    cols = ext.im2col(xg, (cfg["r"], cfg["s"]), **_geo(cfg))
    explicit = ext.gemm_dsd_lists(cols, w2, lists, 64, s)
    assert rel_fro(y, to_np(explicit)) <= 1e-3
    ry = O.conv2d_blockdrop(to_np(x), to_np(k), mask.numpy(), 64, p, dtype=np.float32, **_geo(cfg))
    ry2 = np.transpose(ry, (0, 2, 3, 1)).reshape(rows, cfg["k"])
    assert max_tile_rel_fro(y, ry2) <= REL_FRO_TOL


@pytest.mark.parametrize("cfg,taken", [g for g in IMPLICIT_GEOMS if g[1]][:5] + IMPLICIT_GEOMS[-2:])
def test_implicit_gemm_conv_dense(cfg, taken, copy_form):
    """No lists = every block kept: the dense convolution, against torch's conv2d in fp32."""
    from flash_dropout.hip import GEMM

    ext = GEMM()
    gen = torch.Generator().manual_seed(2)
    x = torch.randn(cfg["n"], cfg["c"], cfg["h"], cfg["w"], generator=gen).half()
    fan_in = cfg["c"] * cfg["r"] * cfg["s"]
    k = ((torch.rand(cfg["k"], cfg["c"], cfg["r"], cfg["s"], generator=gen) * 2 - 1) * fan_in ** -0.5).half()
    y = ext.conv2d_dsd_lists(x.cuda(), k.cuda().reshape(cfg["k"], fan_in), None, 0, 1.0, (cfg["r"], cfg["s"]), **_geo(cfg))
    assert y is not None
    ref = torch.nn.functional.conv2d(x.float(), k.float(), padding=cfg["padding"])
    n, kk, p_, q_ = ref.shape
    assert max_tile_rel_fro(y, ref.permute(0, 2, 3, 1).reshape(n * p_ * q_, kk).numpy()) <= REL_FRO_TOL


@pytest.mark.parametrize("cfg,fwd_taken", IMPLICIT_GEOMS)
@pytest.mark.parametrize("p", [0.0, 0.5])
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_implicit_gemm_conv_weight_gradient(cfg, fwd_taken, p, dtype):
    """sd_conv2d_dw_lists (no patch matrix) against the oracle and against im2col + DSD on the transposed
    operands; it takes every geometry the forward takes (and some more: P*Q only has to be a multiple of 64)."""
    from flash_dropout.hip import GEMM

    ext = GEMM()
    gen = torch.Generator().manual_seed(cfg["c"] * 3 + cfg["k"])
    x = torch.randn(cfg["n"], cfg["c"], cfg["h"], cfg["w"], generator=gen).to(dtype)
    fan_in = cfg["c"] * cfg["r"] * cfg["s"]
    p_, q_ = O.conv_out_hw(cfg["h"], cfg["w"], cfg["r"], cfg["s"], **_geo(cfg))
    rows = cfg["n"] * p_ * q_
    dy2 = torch.randn(rows, cfg["k"], generator=gen).to(dtype)
    mask = cpu_mask(O.mask_shape(rows, fan_in, 64), p, gen)
    lists = ext.build_lists(mask.cuda())
    s = 1 / (1 - p)
    xg, dyg = x.cuda(), dy2.cuda()
    dw = ext.conv2d_dw_lists(xg, dyg, lists, 64, s, (cfg["r"], cfg["s"]), **_geo(cfg))
    if dw is None:
        assert not fwd_taken
        return
    assert tuple(dw.shape) == (cfg["k"], fan_in)
    cols = ext.im2col(xg, (cfg["r"], cfg["s"]), **_geo(cfg))
    explicit = ext.gemm_dsd_lists(cols.t(), dyg.t(), lists.transposed(), 64, s, transposed_out=True).t()
    assert rel_fro(dw, to_np(explicit)) <= 2e-3
    ref = O.dsd_dw(to_np(dy2), O.im2col(to_np(x), cfg["r"], cfg["s"], **_geo(cfg)), mask.numpy(), 64, p, np.float32)
    assert max_tile_rel_fro(dw, ref) <= REL_FRO_TOL
    if p == 0.0:  # and without lists: the dense weight gradient
        dense = ext.conv2d_dw_lists(xg, dyg, None, 0, 1.0, (cfg["r"], cfg["s"]), **_geo(cfg))
        assert dense is not None and max_tile_rel_fro(dense, ref) <= REL_FRO_TOL


DX_GEOMS = [
    (dict(n=4, c=64, h=32, w=32, k=128, r=3, s=3, padding=(1, 1), stride=(1, 1), dilation=(1, 1)), True),   # the conv configuration's layer
    (dict(n=2, c=16, h=16, w=16, k=64, r=3, s=3, padding=(1, 1), stride=(1, 1), dilation=(1, 1)), True),    # 144 columns: ragged last block
    (dict(n=2, c=16, h=33, w=33, k=128, r=2, s=2, padding=(0, 0), stride=(1, 1), dilation=(1, 1)), True),   # 2x2 on a 33 x 33 image: one block column, 18 open channels
    (dict(n=2, c=64, h=32, w=32, k=128, r=1, s=1, padding=(0, 0), stride=(1, 1), dilation=(1, 1)), True),   # 1x1: 66 open channels per block column, so the band shrinks to one input row for the ring to fit
    (dict(n=2, c=32, h=16, w=64, k=64, r=3, s=3, padding=(1, 1), stride=(1, 1), dilation=(1, 1)), True),    # one output row per block
    (dict(n=3, c=24, h=32, w=8, k=128, r=3, s=3, padding=(1, 1), stride=(1, 1), dilation=(1, 1)), True),    # 8 output rows per block
    (dict(n=2, c=16, h=34, w=32, k=64, r=3, s=1, padding=(0, 0), stride=(1, 1), dilation=(1, 1)), True),    # no padding, H not a multiple of the band
    (dict(n=2, c=8, h=16, w=16, k=64, r=5, s=5, padding=(2, 2), stride=(1, 1), dilation=(1, 1)), True),     # 25 taps, 4 output rows per block
    (dict(n=2, c=128, h=16, w=16, k=256, r=3, s=3, padding=(1, 1), stride=(1, 1), dilation=(1, 1)), True),  # K_out = 256: the instance with the longer reduction
    (dict(n=2, c=24, h=16, w=16, k=192, r=5, s=3, padding=(2, 1), stride=(1, 1), dilation=(1, 1)), True),   # K_out = 192, 15 taps
    (dict(n=2, c=16, h=32, w=32, k=256, r=1, s=1, padding=(0, 0), stride=(1, 1), dilation=(1, 1)), True),   # 1x1 with K_out = 256: that instance's LDS holds the 66-slot ring
    (dict(n=1, c=16, h=32, w=32, k=320, r=3, s=3, padding=(1, 1), stride=(1, 1), dilation=(1, 1)), False),  # K_out = 320
    (dict(n=2, c=40, h=32, w=32, k=128, r=2, s=2, padding=(0, 0), stride=(1, 1), dilation=(1, 1)), False),  # Q = 31
    (dict(n=3, c=8, h=32, w=32, k=64, r=5, s=5, padding=(2, 2), stride=(1, 1), dilation=(1, 1)), True),     # 5 taps high on 2-row blocks: the band shrinks to two input rows
    (dict(n=2, c=16, h=16, w=16, k=40, r=3, s=3, padding=(1, 1), stride=(1, 1), dilation=(1, 1)), False),   # K_out = 40
    (dict(n=2, c=8, h=32, w=32, k=64, r=3, s=3, padding=(1, 1), stride=(2, 2), dilation=(1, 1)), True),     # stride 2: three of four taps fall between outputs
    (dict(n=2, c=24, h=32, w=32, k=64, r=3, s=3, padding=(2, 2), stride=(1, 1), dilation=(2, 2)), True),    # dilation 2
    (dict(n=3, c=16, h=32, w=32, k=128, r=3, s=3, padding=(1, 1), stride=(2, 1), dilation=(1, 1)), True),   # stride 2 down, 1 across
    (dict(n=2, c=40, h=64, w=16, k=64, r=5, s=3, padding=(4, 1), stride=(2, 2), dilation=(2, 1)), True),    # stride and dilation, Q = 8
]


@pytest.mark.parametrize("cfg,taken", DX_GEOMS)
@pytest.mark.parametrize("p", [0.0, 0.5])
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("channels_last", [False, True])
def test_fused_conv_input_gradient(cfg, taken, p, dtype, channels_last):
    """sd_conv2d_dx (kept tiles of dY.W formed and folded in LDS) against the oracle's dx and against the
    two-kernel route; run twice, the result must be bitwise the same (one owner and one order per sum)."""
    from flash_dropout.hip import GEMM

    ext = GEMM()
    gen = torch.Generator().manual_seed(cfg["c"] * 5 + cfg["k"])
    shape = (cfg["n"], cfg["c"], cfg["h"], cfg["w"])
    fan_in = cfg["c"] * cfg["r"] * cfg["s"]
    kern = ((torch.rand(cfg["k"], cfg["c"], cfg["r"], cfg["s"], generator=gen) * 2 - 1) * fan_in ** -0.5).to(dtype)
    p_, q_ = O.conv_out_hw(cfg["h"], cfg["w"], cfg["r"], cfg["s"], **_geo(cfg))
    rows = cfg["n"] * p_ * q_
    dy2 = torch.randn(rows, cfg["k"], generator=gen).to(dtype)
    mask = cpu_mask(O.mask_shape(rows, fan_in, 64), p, gen)
    s = 1 / (1 - p)
    w2 = kern.cuda().reshape(cfg["k"], fan_in)
    dx = ext.conv2d_dx(dy2.cuda(), w2, shape, (cfg["r"], cfg["s"]), mask=mask.cuda(), block_size=64, scale=s,
                       channels_last=channels_last, **_geo(cfg))
    if not taken:
        assert dx is None
        return
    assert dx is not None and tuple(dx.shape) == shape
    again = ext.conv2d_dx(dy2.cuda(), w2, shape, (cfg["r"], cfg["s"]), mask=mask.cuda(), block_size=64, scale=s,
                          channels_last=channels_last, **_geo(cfg))
    assert torch.equal(dx, again)
    lists = ext.build_lists(mask.cuda())
    dcols = ext.gemm_sdd_lists(dy2.cuda(), w2.t(), lists, 64, s)
    two_step = ext.col2im(dcols, shape, (cfg["r"], cfg["s"]), mask=mask.cuda(), block_size=64, **_geo(cfg))
    assert rel_fro(dx, to_np(two_step)) <= 2e-3
    ref = O.col2im(O.sdd_dx(to_np(dy2), to_np(w2.cpu()), mask.numpy(), 64, p, np.float32), shape, cfg["r"], cfg["s"],
                   **_geo(cfg))
    assert max_tile_rel_fro(dx, ref) <= REL_FRO_TOL
    if p == 0.0:  # no mask: the dense input gradient
        dense = ext.conv2d_dx(dy2.cuda(), w2, shape, (cfg["r"], cfg["s"]), **_geo(cfg))
        assert dense is not None and max_tile_rel_fro(dense, ref) <= REL_FRO_TOL


@pytest.mark.parametrize("stride,dilation,padding", [((1, 1), (1, 1), (1, 1)), ((2, 2), (1, 1), (1, 1)),
                                                     ((1, 1), (2, 2), (2, 2))])
def test_implicit_and_explicit_conv_routes_agree(stride, dilation, padding):
    """The autograd function with the implicit forward (input kept, kept patch blocks re-gathered for the weight
    gradient, fused input gradient) and with the explicit one (patch matrix kept) give the same three results,
    also for a strided and for a dilated convolution."""
    import sys

    import flash_dropout.functional as F

    mod = sys.modules["flash_dropout.functional.im2col_conv2d"]  # the package re-exports a function of that name
    gen = torch.Generator().manual_seed(9)
    x = torch.randn(4, 64, 32, 32, generator=gen).half().cuda()
    k = (torch.randn(128, 64, 3, 3, generator=gen) * 0.04).half().cuda()
    p_, q_ = O.conv_out_hw(32, 32, 3, 3, padding=padding, stride=stride, dilation=dilation)
    dy = torch.randn(4, 128, p_, q_, generator=gen).half().cuda()
    mask = (torch.rand(4 * p_ * q_ // 64, 9, generator=gen) < 0.5).cuda()
    out = {}
    for implicit in (True, False):
        prev, mod.IMPLICIT_FORWARD = mod.IMPLICIT_FORWARD, implicit
        prev_dx, mod.FUSED_INPUT_GRADIENT = mod.FUSED_INPUT_GRADIENT, implicit
        try:
            xg, kg = x.clone().requires_grad_(), k.clone().requires_grad_()
            y = F.blockwise_dropout_conv2d_mask(xg, mask, 64, 0.5, kg, padding=padding, stride=stride,
                                                dilation=dilation)
            y.backward(dy)
            out[implicit] = (y.detach(), xg.grad, kg.grad)
        finally:
            mod.IMPLICIT_FORWARD = prev
            mod.FUSED_INPUT_GRADIENT = prev_dx
    for a, b, what in zip(out[True], out[False], ("y", "dx", "dk")):
        assert rel_fro(a, to_np(b)) <= 1e-3, what


@pytest.mark.parametrize("dropout", [True, False])
def test_conv_backward_takes_an_expanded_gradient(dropout):
    """out.sum().backward() hands the backward a gradient with all strides zero; it must be laid out before the
    kernels see it (the result is then the gradient of the sum: compare with a materialised gradient of ones)."""
    import flash_dropout.functional as F

    gen = torch.Generator().manual_seed(3)
    x = torch.randn(4, 16, 16, 16, generator=gen).half().cuda()
    k = (torch.randn(64, 16, 3, 3, generator=gen) * 0.08).half().cuda()
    mask = (torch.rand(16, 3, generator=gen) < 0.5).cuda()
    grads = []
    for expanded in (True, False):
        xg, kg = x.clone().requires_grad_(), k.clone().requires_grad_()
        if dropout:
            out = F.blockwise_dropout_conv2d_mask(xg, mask, 64, 0.5, kg, padding=(1, 1))
        else:
            out = F.im2col_conv2d(xg, kg, padding=(1, 1), stride=(1, 1), dilation=(1, 1))
        if expanded:
            out.sum().backward()
        else:
            out.backward(torch.ones_like(out))
        grads.append((xg.grad, kg.grad))
    assert torch.equal(grads[0][0], grads[1][0]) and torch.equal(grads[0][1], grads[1][1])
    assert grads[0][0].abs().sum().item() > 0


def test_dense_im2col_conv_matches_conv2d():
    """The reference's implied check for its im2col path: equal to F.conv2d (benchmark/conv.py:20-75)."""
    import flash_dropout.functional as F

    torch.manual_seed(6)
    x = torch.randn(4, 32, 20, 20, device="cuda", dtype=torch.float16, requires_grad=True)
    k = (torch.randn(48, 32, 3, 3, device="cuda", dtype=torch.float16) * 0.06).requires_grad_()
    y = F.im2col_conv2d(x, k, padding=(1, 1), stride=(1, 1), dilation=(1, 1))
    dy = torch.randn_like(y)
    y.backward(dy)
    xr, kr = x.detach().float().requires_grad_(), k.detach().float().requires_grad_()
    yr = torch.nn.functional.conv2d(xr, kr, padding=1)
    yr.backward(dy.float())
    assert max_tile_rel_fro(y, yr) <= REL_FRO_TOL
    assert max_tile_rel_fro(x.grad, xr.grad) <= REL_FRO_TOL
    assert max_tile_rel_fro(k.grad, kr.grad) <= REL_FRO_TOL


def test_conv_layer_variants_on_gpu():
    from flash_dropout.layers import DropoutConv2d

    torch.manual_seed(7)
    x = torch.randn(4, 16, 12, 12, device="cuda", dtype=torch.float16)
    for variant in ("im2col", "blockwise[hip]", "blockwise[naive]"):
        conv = DropoutConv2d(16, 32, (3, 3), padding=(1, 1), p=0.0, variant=variant, block_size=64).cuda().half()
        ref = torch.nn.functional.conv2d(x, conv.weight, padding=1)
        assert max_tile_rel_fro(conv(x), ref) <= REL_FRO_TOL, variant
    conv = DropoutConv2d(16, 32, (3, 3), padding=(1, 1), p=0.5, variant="blockwise[hip]", block_size=64).cuda().half()
    y = conv(x)
    y.float().sum().backward()
    assert y.shape == (4, 32, 12, 12) and conv.weight.grad is not None


def test_full_size_conv_config_against_the_full_oracle():
    """The full conv configuration ([128,64,32,32] -> patch matrix [131072 x 576], 3x3 64->128, p = 0.5) at full
    batch: forward, input gradient and weight gradient (2048 row blocks, the reduction split over workgroups)
    against the fp32 oracle, every tile; plus the adjoint identity <im2col(x), g> == <x, col2im(g)>."""
    import flash_dropout.functional as F
    from flash_dropout.hip import GEMM

    ext = GEMM()
    gen = torch.Generator().manual_seed(8)
    geo = dict(padding=(1, 1), stride=(1, 1), dilation=(1, 1))
    x = torch.randn(128, 64, 32, 32, generator=gen).half()
    k = ((torch.rand(128, 64, 3, 3, generator=gen) * 2 - 1) * 576 ** -0.5).half()
    mask = cpu_mask((2048, 9), 0.5, gen)
    dy = torch.randn(128, 128, 32, 32, generator=gen).half()
    xg, kg = x.cuda().requires_grad_(), k.cuda().requires_grad_()
    y = F.blockwise_dropout_conv2d_mask(xg, mask.cuda(), 64, 0.5, kg, **geo)
    y.backward(dy.cuda())
    # none of the three products went through a patch matrix
    assert F.conv_last_routes() == {"forward": "implicit", "dx": "fused", "dw": "implicit"}
    ry, rdx, rdk = O.conv2d_blockdrop(to_np(x), to_np(k), mask.numpy(), 64, 0.5, dy=to_np(dy), dtype=np.float32, **geo)
    # in the products' own layouts, so that a tile of the check is a tile of the kernels
    as_rows = lambda t: t.permute(0, 2, 3, 1).reshape(-1, t.shape[1])
    assert max_tile_rel_fro(as_rows(y.detach().cpu()), as_rows(torch.from_numpy(ry))) <= REL_FRO_TOL
    assert max_tile_rel_fro(xg.grad, rdx) <= REL_FRO_TOL
    assert max_tile_rel_fro(kg.grad.reshape(128, 576), rdk.reshape(128, 576)) <= REL_FRO_TOL
    xs = x[:16].cuda()
    cols = ext.im2col(xs, (3, 3), **geo)
    g = torch.randn(cols.shape, generator=gen).half().cuda()
    lhs = (cols.double() * g.double()).sum().item()
    rhs = (xs.double() * ext.col2im(g, xs.shape, (3, 3), **geo).double()).sum().item()
    assert abs(lhs - rhs) <= 2e-3 * max(abs(lhs), (cols.double().norm() * g.double().norm()).item() * 1e-2)


@pytest.mark.parametrize("bs,dx_route", [(64, "fused"), (128, "fused"), (192, "fused")])
def test_conv_routes_are_reported_and_block_sizes_above_64_stay_fused(bs, dx_route):
    """Which route a convolution's products took is visible (conv_last_routes), a geometry the fused kernels do not take
    reports the patch-matrix route, and masks at block sizes 128 and 192 run the fused input gradient too (as the
    mask of the same elements at block size 64): results against the oracle at that block size."""
    import sys

    import flash_dropout.functional as F

    mod = sys.modules["flash_dropout.functional.im2col_conv2d"]  # the package re-exports a function of that name

    gen = torch.Generator().manual_seed(12)
    geo = dict(padding=(1, 1), stride=(1, 1), dilation=(1, 1))
    x = torch.randn(8, 64, 32, 32, generator=gen).half()
    k = ((torch.rand(128, 64, 3, 3, generator=gen) * 2 - 1) * 576 ** -0.5).half()
    dy = torch.randn(8, 128, 32, 32, generator=gen).half()
    mask = cpu_mask(O.mask_shape(8 * 32 * 32, 576, bs), 0.5, gen)
    xg, kg = x.cuda().requires_grad_(), k.cuda().requires_grad_()
    y = F.blockwise_dropout_conv2d_mask(xg, mask.cuda(), bs, 0.5, kg, **geo)
    y.backward(dy.cuda())
    assert F.conv_last_routes() == {"forward": "implicit", "dx": dx_route, "dw": "implicit"}
    ry, rdx, rdk = O.conv2d_blockdrop(to_np(x), to_np(k), mask.numpy(), bs, 0.5, dy=to_np(dy), dtype=np.float32, **geo)
    assert max_tile_rel_fro(y, ry) <= REL_FRO_TOL
    assert max_tile_rel_fro(xg.grad, rdx) <= REL_FRO_TOL
    assert max_tile_rel_fro(kg.grad, rdk) <= REL_FRO_TOL
    if bs == 64:
        # Q = 18 is a geometry none of the fused kernels takes; and the switches force the patch-matrix route
        x2 = torch.randn(2, 16, 16, 16, generator=gen).half().cuda().requires_grad_()
        k2 = (torch.randn(64, 16, 3, 3, generator=gen) * 144 ** -0.5).half().cuda().requires_grad_()
        F.im2col_conv2d(x2, k2, padding=(2, 2)).sum().backward()
        assert F.conv_last_routes() == {"forward": "explicit", "dx": "explicit", "dw": "explicit"}
        old = mod.IMPLICIT_FORWARD, mod.FUSED_INPUT_GRADIENT
        try:
            mod.IMPLICIT_FORWARD = mod.FUSED_INPUT_GRADIENT = False
            xg.grad = kg.grad = None
            F.blockwise_dropout_conv2d_mask(xg, mask.cuda(), bs, 0.5, kg, **geo).backward(dy.cuda())
            assert F.conv_last_routes() == {"forward": "explicit", "dx": "explicit", "dw": "explicit"}
            assert max_tile_rel_fro(xg.grad, rdx) <= REL_FRO_TOL
        finally:
            mod.IMPLICIT_FORWARD, mod.FUSED_INPUT_GRADIENT = old
