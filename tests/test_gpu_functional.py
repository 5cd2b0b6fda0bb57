"""The public API on the GPU: autograd function, layers, autocast — against the CPU oracle."""
import json
from pathlib import Path

import numpy as np
import pytest
import torch

from _util import REL_FRO_TOL, max_tile_rel_fro, cpu_mask, rel_fro, to_np
from oracle import naive_torch
from oracle import sparsedrop_oracle as O

pytestmark = pytest.mark.gpu
GOLDEN = Path(__file__).parent / "golden"


def _fwd_bwd(x, w, dy, mask, bs, p):
    import flash_dropout.functional as F

    x = x.detach().clone().requires_grad_()
    w = w.detach().clone().requires_grad_()
    y = F.hip_blockwise_dropout_matmul_mask(x, mask, bs, p, w)
    y.backward(dy)
    return y.detach(), x.grad, w.grad


def test_cfg1_cpu_reference_configuration():
    """X[1024x1024] ~N(0,1), W ~N(0,1/1024), 64x64 blocks, keep 0.5, seed 0, committed mask fixture.
    Expected values come from autograd through the literal naive restatement in fp32, the HIP path
    runs on the fp16-rounded tensors (the reference's own test does the same, test/test_cuda.py:45-51)."""
    fx = json.loads((GOLDEN / "cfg1_mask.json").read_text())
    mask = torch.tensor([[ch == "1" for ch in row] for row in fx["rows"]])
    torch.manual_seed(0)
    x = torch.randn(1024, 1024)
    w = torch.randn(1024, 1024) / 32
    dy = torch.randn(1024, 1024)
    xh, wh, dyh = x.half(), w.half(), dy.half()
    ry, rdx, rdw = naive_torch.forward_backward(xh.float(), wh.float(), dyh.float(), mask, 64, 0.5)
    y, dx, dw = _fwd_bwd(xh.cuda(), wh.cuda(), dyh.cuda(), mask.cuda(), 64, 0.5)
    assert y.dtype == torch.float16 and dw.is_contiguous() and dw.shape == (1024, 1024)
    assert max_tile_rel_fro(y, ry) <= REL_FRO_TOL
    assert max_tile_rel_fro(dx, rdx) <= REL_FRO_TOL
    assert max_tile_rel_fro(dw, rdw) <= REL_FRO_TOL
    # and against the unrounded fp32 problem the reference's tolerances still hold
    fy, fdx, fdw = naive_torch.forward_backward(x, w, dy, mask, 64, 0.5)
    torch.testing.assert_close(y.float().cpu(), fy, atol=0.2, rtol=0.01)
    torch.testing.assert_close(dw.float().cpu(), fdw, atol=0.2, rtol=0.01)
    torch.testing.assert_close(dx.float().cpu(), fdx, atol=0.2, rtol=0.01)


@pytest.mark.parametrize("p", [0.1, 0.3, 0.5])
def test_cfg4_transformer_mlp(p):
    """64x256 tokens -> X[16384x384]; Linear 384->1536, GELU, 1536->384; block dropout on both inputs."""
    import flash_dropout.functional as F

    gen = torch.Generator().manual_seed(4)
    x = torch.randn(16384, 384, generator=gen).half()
    w1 = (torch.rand(1536, 384, generator=gen) * 2 - 1).mul(384 ** -0.5).half()
    w2 = (torch.rand(384, 1536, generator=gen) * 2 - 1).mul(1536 ** -0.5).half()
    m1 = cpu_mask((256, 6), p, gen)
    m2 = cpu_mask((256, 24), p, gen)
    dy = torch.randn(16384, 384, generator=gen).half()

    xg, w1g, w2g = (t.cuda().requires_grad_() for t in (x, w1, w2))
    h = F.hip_blockwise_dropout_matmul_mask(xg, m1.cuda(), 64, p, w1g)
    a = torch.nn.functional.gelu(h)
    y = F.hip_blockwise_dropout_matmul_mask(a, m2.cuda(), 64, p, w2g)
    y.backward(dy.cuda())

    # oracle: same graph in fp32 with the naive restatement
    xr, w1r, w2r = (t.float().requires_grad_() for t in (x, w1, w2))
    hr = naive_torch.forward(xr, w1r, m1, 64, p)
    ar = torch.nn.functional.gelu(hr)
    yr = naive_torch.forward(ar, w2r, m2, 64, p)
    yr.backward(dy.float())
    assert max_tile_rel_fro(h, hr) <= REL_FRO_TOL
    assert max_tile_rel_fro(y, yr) <= REL_FRO_TOL
    assert max_tile_rel_fro(xg.grad, xr.grad) <= REL_FRO_TOL
    assert max_tile_rel_fro(w1g.grad, w1r.grad) <= REL_FRO_TOL
    assert max_tile_rel_fro(w2g.grad, w2r.grad) <= REL_FRO_TOL


def test_cfg3_mlp_on_28x28_images_through_layers():
    """X[4096x784] uniform[0,1]; 784->1024->1024->10 with ReLU; block dropout p=0.5 on each hidden
    input (layers 2 and 3) and, to exercise the K tail 784 = 12*64+16, on layer 1 as well.

    Parity is judged layer by layer on identical inputs: each layer's fp16 input and upstream gradient
    are taken from the GPU run and handed to the oracle, so the 1e-2 bar applies to every product and
    is not blurred by fp16 rounding accumulating through three layers and two ReLUs."""
    from flash_dropout.layers import DropoutMM

    torch.manual_seed(3)
    dims = [784, 1024, 1024, 10]
    layers = [DropoutMM(dims[i], dims[i + 1], p=0.5, variant="blockwise[hip]", block_size=64) for i in range(3)]
    x = torch.rand(4096, 784).half()
    dy = torch.randn(4096, 10).half()
    mods = [l.cuda().half() for l in layers]

    # restart the device-resident mask generator so that the masks the layers draw can be re-drawn for
    # the oracle: draw number i since the restart uses (seed, offset i)
    from flash_dropout.hip import GEMM
    GEMM().manual_seed(123)
    ins, outs = [], []
    h = x.cuda().requires_grad_()
    for i, l in enumerate(mods):
        h.retain_grad()
        ins.append(h)
        h = l(h)
        h.retain_grad()
        outs.append(h)
        if i < 2:
            h = torch.relu(h)
    h.backward(dy.cuda())

    masks = [O.random_mask((64, -(-dims[i] // 64)), 0.5, 123, offset=i) for i in range(3)]
    for i, l in enumerate(mods):
        a, g, w = to_np(ins[i]), to_np(outs[i].grad), to_np(l.weight)
        assert max_tile_rel_fro(outs[i], O.dsd_forward(a, w, masks[i], 64, 0.5, np.float32)) <= REL_FRO_TOL, f"Y{i}"
        assert max_tile_rel_fro(ins[i].grad, O.sdd_dx(g, w, masks[i], 64, 0.5, np.float32)) <= REL_FRO_TOL, f"dX{i}"
        assert max_tile_rel_fro(l.weight.grad, O.dsd_dw(g, a, masks[i], 64, 0.5, np.float32)) <= REL_FRO_TOL, f"dW{i}"
        assert l.weight.grad.shape == l.weight.shape


def test_layer_eval_and_3d_inputs_and_bf16():
    from flash_dropout.layers import DropoutMM

    torch.manual_seed(0)
    layer = DropoutMM(384, 256, p=0.3, variant="blockwise[cuda]", block_size=(64, 64)).cuda().bfloat16()
    x = torch.randn(8, 256, 384, device="cuda", dtype=torch.bfloat16)
    layer.eval()
    assert torch.equal(layer(x), torch.nn.functional.linear(x, layer.weight))
    layer.train()
    from flash_dropout.hip import GEMM
    GEMM().manual_seed(9)
    y = layer(x)
    assert y.shape == (8, 256, 256) and y.dtype == torch.bfloat16
    mask = O.random_mask((32, 6), 0.3, 9, offset=0)  # first draw after the restart
    ref = O.dsd_forward(to_np(x.reshape(-1, 384)), to_np(layer.weight), mask, 64, 0.3, np.float32)
    assert max_tile_rel_fro(y.reshape(-1, 256), ref) <= REL_FRO_TOL


def test_autocast_contract():
    import flash_dropout.functional as F

    torch.manual_seed(1)
    x = torch.randn(256, 256, device="cuda", requires_grad=True)
    w = torch.randn(128, 256, device="cuda", requires_grad=True)
    mask = torch.rand(4, 4, device="cuda") < 0.5
    with pytest.raises(TypeError, match="float16 or bfloat16"):
        F.hip_blockwise_dropout_matmul_mask(x, mask, 64, 0.5, w)
    for dt in (torch.float16, torch.bfloat16):
        x.grad = w.grad = None
        with torch.autocast("cuda", dtype=dt):
            y = F.hip_blockwise_dropout_matmul_mask(x, mask, 64, 0.5, w)
        assert y.dtype == dt
        y.float().sum().backward()
        assert x.grad.dtype == torch.float32 and w.grad.dtype == torch.float32
        ref = O.dsd_forward(to_np(x.to(dt)), to_np(w.to(dt)), mask.cpu().numpy(), 64, 0.5, np.float32)
        assert max_tile_rel_fro(y, ref) <= REL_FRO_TOL
        ones = np.ones((256, 128), dtype=np.float32)
        assert max_tile_rel_fro(x.grad, O.sdd_dx(ones, to_np(w.to(dt)), mask.cpu().numpy(), 64, 0.5, np.float32)) <= REL_FRO_TOL
        assert max_tile_rel_fro(w.grad, O.dsd_dw(ones, to_np(x.to(dt)), mask.cpu().numpy(), 64, 0.5, np.float32)) <= REL_FRO_TOL


def test_public_names_and_p_range():
    import flash_dropout.functional as F

    for name in ("cuda_blockwise_dropout_matmul", "triton_blockwise_dropout_matmul", "im2col_conv2d",
                 "naive_blockwise_dropout_matmul", "vanilla_dropout_matmul"):
        assert callable(getattr(F, name))
    x = torch.randn(128, 128, device="cuda", dtype=torch.float16)
    with pytest.raises(ValueError, match=r"\[0, 1\)"):
        F.cuda_blockwise_dropout_matmul(x, x, 64, 1.0)
    y = F.cuda_blockwise_dropout_matmul(x, x, 64, 0.0)
    assert max_tile_rel_fro(y, to_np(x) @ to_np(x).T) <= REL_FRO_TOL
    # statistical sanity of the fresh mask: about p of the blocks are dropped
    big = torch.ones(4096, 4096, device="cuda", dtype=torch.float16)
    eye = torch.eye(4096, device="cuda", dtype=torch.float16)
    torch.manual_seed(0)
    out = F.cuda_blockwise_dropout_matmul(big, eye, 64, 0.25)
    frac_dropped = (out == 0).float().mean().item()
    assert abs(frac_dropped - 0.25) < 0.03
    assert torch.all((out == 0) | (out == torch.tensor(1 / 0.75, dtype=torch.float16, device="cuda")))


def test_backward_takes_an_expanded_gradient():
    """y.sum(0).sum().backward() hands the backward a gradient with strides (0, 1); it is laid out before the
    kernels see it, and the result is the gradient of a materialised all-ones dY."""
    import flash_dropout.functional as F

    gen = torch.Generator().manual_seed(12)
    x = torch.randn(256, 192, generator=gen).half().cuda()
    w = (torch.randn(128, 192, generator=gen) * 192 ** -0.5).half().cuda()
    mask = cpu_mask((4, 3), 0.5, gen).cuda()
    grads = []
    for expanded in (True, False):
        xg, wg = x.clone().requires_grad_(), w.clone().requires_grad_()
        y = F.hip_blockwise_dropout_matmul_mask(xg, mask, 64, 0.5, wg)
        if expanded:
            y.sum(0).sum().backward()
        else:
            y.backward(torch.ones_like(y))
        grads.append((xg.grad, wg.grad))
    assert torch.equal(grads[0][0], grads[1][0]) and torch.equal(grads[0][1], grads[1][1])
    ones = np.ones((256, 128), dtype=np.float32)
    assert max_tile_rel_fro(grads[0][0], O.sdd_dx(ones, to_np(w), mask.cpu().numpy(), 64, 0.5, np.float32)) <= REL_FRO_TOL
    assert max_tile_rel_fro(grads[0][1], O.dsd_dw(ones, to_np(x), mask.cpu().numpy(), 64, 0.5, np.float32)) <= REL_FRO_TOL


def test_narrow_head_stays_on_the_specialised_kernels():
    """The 10-class head of the MLP configuration (1024 -> 10): forward, input gradient and weight gradient all run
    on the specialised kernels (the backward pads the 10 output columns to 16 with zeros, as the reference pads its
    head to 128, eval/mlp/model.py:22-24,40) and match the oracle."""
    import flash_dropout.functional as F
    from flash_dropout.hip import GEMM

    ext = GEMM()
    gen = torch.Generator().manual_seed(14)
    M, K, N, p = 4096, 1024, 10, 0.5
    x = torch.rand(M, K, generator=gen).half()
    w = ((torch.rand(N, K, generator=gen) * 2 - 1) * K ** -0.5).half()
    dy = torch.randn(M, N, generator=gen).half()
    mask = cpu_mask((M // 64, K // 64), p, gen)
    a, b, g, mk = to_np(x), to_np(w), to_np(dy), mask.numpy()
    # the library calls the autograd function makes (its backward runs on autograd's own thread, and which kernel
    # ran is recorded per thread)
    y, _, lists, g_bs = ext.dropout_matmul_forward(x.cuda(), w.cuda(), 64, p, mask=mask.cuda())
    assert ext.last_kernel() == "specialised"
    dx, none = ext.dropout_matmul_backward(dy.cuda(), w.cuda(), x.cuda(), lists, g_bs, p, need_dw=False)
    assert none is None and ext.last_kernel() == "specialised" and ext.last_kernel_detail().startswith("sdd:")
    none, dw = ext.dropout_matmul_backward(dy.cuda(), w.cuda(), x.cuda(), lists, g_bs, p, need_dx=False)
    assert none is None and ext.last_kernel() == "specialised" and ext.last_kernel_detail().startswith("dsd:")
    assert dw.shape == (N, K)
    ry, rdx, rdw = (O.dsd_forward(a, b, mk, 64, p, np.float32), O.sdd_dx(g, b, mk, 64, p, np.float32),
                    O.dsd_dw(g, a, mk, 64, p, np.float32))
    for got, ref in ((y, ry), (dx, rdx), (dw, rdw)):
        assert max_tile_rel_fro(got, ref) <= REL_FRO_TOL
    # and through autograd
    xg, wg = x.cuda().requires_grad_(), w.cuda().requires_grad_()
    F.hip_blockwise_dropout_matmul_mask(xg, mask.cuda(), 64, p, wg).backward(dy.cuda())
    assert wg.grad.shape == (N, K)
    assert max_tile_rel_fro(xg.grad, rdx) <= REL_FRO_TOL
    assert max_tile_rel_fro(wg.grad, rdw) <= REL_FRO_TOL


@pytest.mark.parametrize("bs", [64, 128])
def test_fused_forward_and_backward_calls_match_the_separate_ones(bs):
    """sd_dropout_matmul_forward / _backward (mask, lists and product in one library call; both gradients in one)
    against the calls they bundle, bit for bit, with a given mask, a seeded draw and the device-resident generator."""
    from flash_dropout.hip import GEMM

    ext = GEMM()
    gen = torch.Generator().manual_seed(15)
    M, K, N, p = 640, 448, 200, 0.3
    x = torch.randn(M, K, generator=gen).half().cuda()
    w = (torch.randn(N, K, generator=gen) * K ** -0.5).half().cuda()
    dy = torch.randn(M, N, generator=gen).half().cuda()
    s = 1 / (1 - p)
    # given mask
    mask = cpu_mask(O.mask_shape(M, K, bs), p, gen).cuda()
    y, m2, lists, g = ext.dropout_matmul_forward(x, w, bs, p, mask=mask)
    assert g == 64 and torch.equal(m2, mask)
    assert torch.equal(y, ext.gemm_dsd(x, w, mask, bs, s))
    dx, dw = ext.dropout_matmul_backward(dy, w, x, lists, g, p)
    assert torch.equal(dx, ext.gemm_sdd(dy, w.t(), mask, bs, s))
    assert dw.is_contiguous() and torch.equal(dw, ext.gemm_dsd(x.t(), dy.t(), mask.t(), bs, s, transposed_out=True).t())
    only_dx, none = ext.dropout_matmul_backward(dy, w, x, lists, g, p, need_dw=False)
    assert none is None and torch.equal(only_dx, dx)
    # seeded draw: the mask of the oracle's generator
    y, m3, lists, g = ext.dropout_matmul_forward(x, w, bs, p, seed=77)
    want = O.random_mask(O.mask_shape(M, K, bs), p, 77)
    assert np.array_equal(m3.cpu().numpy(), want)
    assert max_tile_rel_fro(y, O.dsd_forward(to_np(x), to_np(w), want, bs, p, np.float32)) <= REL_FRO_TOL
    # device-resident generator: follows manual_seed and advances
    ext.manual_seed(5)
    _, m4, _, _ = ext.dropout_matmul_forward(x, w, bs, p)
    _, m5, _, _ = ext.dropout_matmul_forward(x, w, bs, p)
    assert np.array_equal(m4.cpu().numpy(), O.random_mask(O.mask_shape(M, K, bs), p, 5, offset=0))
    assert np.array_equal(m5.cpu().numpy(), O.random_mask(O.mask_shape(M, K, bs), p, 5, offset=1))


@pytest.mark.parametrize("M,K,N,bs,dtype,merged", [
    (1024, 1024, 1024, 64, torch.float16, True),      # aligned
    (4096, 784, 1024, 64, torch.float16, True),       # ragged K
    (2048, 512, 384, 128, torch.bfloat16, True),      # bf16, a mask at block size 128 listed on the 64 grid
    (1000, 520, 264, 32, torch.float16, True),        # ragged everywhere, block size 32 (quadrant keep bits)
    (256, 4096, 256, 64, torch.float16, True),        # few output tiles, long reduction: split over workgroups
    (8192, 2048, 4352, 64, torch.float16, False),     # 544 workgroups: the list build stays a launch of its own
])
def test_forward_that_builds_its_lists_in_the_same_launch(M, K, N, bs, dtype, merged):
    """sd_dropout_matmul_forward_act on a small layer is ONE launch (forward_lists_kernel): the product's workgroups
    take their keep bits from the mask source, other workgroups of the grid write the lists and the drawn mask.  Mask,
    lists, product and pre-activation must be, bit for bit, what the list build and the list-driven product give as
    launches of their own, for a stored mask, a seeded draw and the device-resident generator."""
    from flash_dropout.hip import GEMM

    ext = GEMM()
    gen = torch.Generator().manual_seed(29)
    p = 0.5
    x = torch.randn(M, K, generator=gen).to(dtype).cuda()
    w = (torch.randn(N, K, generator=gen) * K ** -0.5).to(dtype).cuda()
    s = 1 / (1 - p)
    split = 0 if bs == 32 else max(bs // 64, 1)
    grid = (-(-M // 64), -(-K // 64))

    def same_lists(a, b):
        nnz = b.nnz()
        assert a.shape == b.shape and a.nnz() == nnz
        assert torch.equal(a.row_ptr, b.row_ptr) and torch.equal(a.col_ptr, b.col_ptr)
        assert torch.equal(a.col_idx[:nnz], b.col_idx[:nnz]) and torch.equal(a.row_idx[:nnz], b.row_idx[:nnz])

    def check(y, pre, mask, lists, g, act):
        assert ext.last_kernel_detail().startswith("dsd+lists:") == merged, ext.last_kernel_detail()
        want_lists = ext.build_lists(mask, split, grid) if bs != 64 else ext.build_lists(mask)
        same_lists(lists, want_lists)
        want_y, want_pre = ext.gemm_dsd_lists_act(x, w, want_lists, g, s, act, want_pre=pre is not None)
        assert not ext.last_kernel_detail().startswith("dsd+lists:")
        assert torch.equal(y, want_y)
        if pre is not None:
            assert torch.equal(pre, want_pre)

    # a stored mask, plain and with the activation in the store
    mask = cpu_mask(O.mask_shape(M, K, bs), p, gen).cuda()
    y, m, lists, g = ext.dropout_matmul_forward(x, w, bs, p, mask=mask)
    check(y, None, mask, lists, g, None)
    y, m, lists, g, pre = ext.dropout_matmul_forward_act(x, w, bs, p, mask=mask, activation="gelu", want_pre=True)
    check(y, pre, mask, lists, g, "gelu")
    if M * K * N <= 1 << 31:
        assert max_tile_rel_fro(pre, O.dsd_forward(to_np(x), to_np(w), mask.cpu().numpy(), bs, p, np.float32)) <= REL_FRO_TOL
    # a seeded draw: the oracle's mask, stored for the caller
    y, m, lists, g, pre = ext.dropout_matmul_forward_act(x, w, bs, p, seed=91, activation="relu")
    assert pre is None and np.array_equal(m.cpu().numpy(), O.random_mask(O.mask_shape(M, K, bs), p, 91))
    check(y, None, m, lists, g, "relu")
    # the device-resident generator: every workgroup of the launch reads the state before the last one moves it on
    ext.manual_seed(12)
    for offset in range(3):
        y, m, lists, g = ext.dropout_matmul_forward(x, w, bs, p)
        assert np.array_equal(m.cpu().numpy(), O.random_mask(O.mask_shape(M, K, bs), p, 12, offset=offset))
        check(y, None, m, lists, g, None)


@pytest.mark.parametrize("p", [0.0, 0.95])
@pytest.mark.parametrize("bs", [32, 64])
def test_forward_with_its_lists_at_the_ends_of_the_drop_range(p, bs):
    """The single-launch forward with nothing dropped, with nearly everything dropped (row blocks without a kept block,
    workgroups without a step) and with the mask stored column-major: bit for bit what the separate launches give."""
    from flash_dropout.hip import GEMM

    ext = GEMM()
    gen = torch.Generator().manual_seed(31)
    M, K, N = 1000, 520, 264
    x = torch.randn(M, K, generator=gen).half().cuda()
    w = (torch.randn(N, K, generator=gen) * K ** -0.5).half().cuda()
    s = 1 / (1 - p)
    mask = cpu_mask(O.mask_shape(M, K, bs), p, gen).cuda()
    for stored in (mask, mask.t().contiguous().t()):  # row-major, column-major
        y, m, lists, g = ext.dropout_matmul_forward(x, w, bs, p, mask=stored)
        assert ext.last_kernel_detail().startswith("dsd+lists:")
        want = ext.build_lists(mask, 0, (-(-M // 64), -(-K // 64))) if bs == 32 else ext.build_lists(mask)
        nnz = want.nnz()
        assert lists.nnz() == nnz and torch.equal(lists.row_ptr, want.row_ptr) and torch.equal(lists.col_ptr, want.col_ptr)
        assert torch.equal(lists.col_idx[:nnz], want.col_idx[:nnz]) and torch.equal(lists.row_idx[:nnz], want.row_idx[:nnz])
        assert torch.equal(y, ext.gemm_dsd_lists(x, w, want, g, s))
        assert max_tile_rel_fro(y, O.dsd_forward(to_np(x), to_np(w), mask.cpu().numpy(), bs, p, np.float32)) <= REL_FRO_TOL
    y, m, lists, g = ext.dropout_matmul_forward(x, w, bs, p, seed=5)
    assert np.array_equal(m.cpu().numpy(), O.random_mask(O.mask_shape(M, K, bs), p, 5))
    assert max_tile_rel_fro(y, O.dsd_forward(to_np(x), to_np(w), m.cpu().numpy(), bs, p, np.float32)) <= REL_FRO_TOL


@pytest.mark.parametrize("M,K,N,bs,dtype,paired", [
    (1024, 1024, 1024, 64, torch.float16, True),      # aligned, both products on a fraction of the chip
    (4096, 784, 1024, 64, torch.float16, True),       # ragged K, weight gradient with a split reduction
    (2048, 512, 384, 128, torch.bfloat16, True),      # bf16, block size listed at 64
    (1000, 520, 264, 32, torch.float16, True),        # ragged everywhere, block size 32 (quadrant keep bits)
    (16384, 1536, 384, 64, torch.float16, False),     # dX wants the big workgroup shape, dW the small one: two launches
])
def test_both_gradients_in_one_launch_match_the_two_launches(M, K, N, bs, dtype, paired):
    """sd_dropout_matmul_backward puts dX and dW of a small layer into a single launch (backward_pair_kernel): the
    result must be what the two products give by themselves, bit for bit, and what the oracle gives, per tile."""
    from flash_dropout.hip import GEMM

    ext = GEMM()
    gen = torch.Generator().manual_seed(23)
    p = 0.5
    x = torch.randn(M, K, generator=gen).to(dtype).cuda()
    w = (torch.randn(N, K, generator=gen) * K ** -0.5).to(dtype).cuda()
    dy = torch.randn(M, N, generator=gen).to(dtype).cuda()
    mask = cpu_mask(O.mask_shape(M, K, bs), p, gen)
    g = 64 if bs % 64 == 0 else bs
    lists = ext.build_lists(mask.cuda(), split=0 if bs == 32 else bs // 64) if bs != 64 else ext.build_lists(mask.cuda())
    s = 1 / (1 - p)
    dx, dw = ext.dropout_matmul_backward(dy, w, x, lists, g, p)
    detail = ext.last_kernel_detail()
    assert detail.startswith("pair:") == paired, detail
    assert torch.equal(dx, ext.gemm_sdd(dy, w.t(), mask.cuda(), bs, s))
    assert torch.equal(dw, ext.gemm_dsd(x.t(), dy.t(), mask.t().cuda(), bs, s, transposed_out=True).t())
    if M * K * N <= 1 << 31:
        assert max_tile_rel_fro(dx, O.sdd_dx(to_np(dy), to_np(w), mask.numpy(), bs, p, np.float32)) <= REL_FRO_TOL
        assert max_tile_rel_fro(dw, O.dsd_dw(to_np(dy), to_np(x), mask.numpy(), bs, p, np.float32)) <= REL_FRO_TOL


@pytest.mark.parametrize("N,single", [(8192, True), (8448, False)])
def test_single_launch_forward_and_backward_at_the_workgroup_limit_against_the_oracle(N, single):
    """The forward that builds its lists in the same launch and the backward that runs both gradients in one are
    taken up to 512 workgroups per product.  4096 x 4096 x 8192 is the largest square-ish layer under that limit
    (16 x 32 = 512 tiles of 256 x 256 for the forward and for the weight gradient), N = 8448 the first over it: both
    sides of the switch, every 64 x 64 tile of Y, dX and dW against the fp32 oracle."""
    from flash_dropout.hip import GEMM

    ext = GEMM()
    gen = torch.Generator().manual_seed(41)
    M, K, bs, p = 4096, 4096, 64, 0.5
    x = torch.randn(M, K, generator=gen).half().cuda()
    w = (torch.randn(N, K, generator=gen) * K ** -0.5).half().cuda()
    dy = torch.randn(M, N, generator=gen).half().cuda()
    mask = cpu_mask(O.mask_shape(M, K, bs), p, gen)
    y, m, lists, g = ext.dropout_matmul_forward(x, w, bs, p, mask=mask.cuda())
    assert ext.last_kernel_detail().startswith("dsd+lists:") == single, ext.last_kernel_detail()
    dx, dw = ext.dropout_matmul_backward(dy, w, x, lists, g, p)
    assert ext.last_kernel_detail().startswith("pair:") == single, ext.last_kernel_detail()
    xn, wn, dyn, mk = to_np(x), to_np(w), to_np(dy), mask.numpy()
    for got, ref, what in ((y, O.dsd_forward(xn, wn, mk, bs, p, np.float32), "y"),
                           (dx, O.sdd_dx(dyn, wn, mk, bs, p, np.float32), "dx"),
                           (dw, O.dsd_dw(dyn, xn, mk, bs, p, np.float32), "dw")):
        err = max_tile_rel_fro(got, ref)
        assert err <= REL_FRO_TOL, f"{what}: largest per-tile relative Frobenius error {err:.3e}"
    keep = O.expand_keep(mk, bs, M, K)
    assert (dx.cpu().numpy()[~keep] == 0).all(), "dropped dX tiles must be exactly zero"


@pytest.mark.parametrize("act", ["relu", "gelu"])
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_fused_activation_products_against_the_oracle(act, dtype):
    """sd_gemm_dsd_lists_act (activation on the fp32 accumulator in the store, pre-activation kept on request) and
    sd_gemm_sdd_lists_actgrad (derivative multiplied in the store, dropped tiles exactly zero) against the oracle's
    closed forms, on a shape with ragged edges in every dimension."""
    from flash_dropout.hip import GEMM

    ext = GEMM()
    gen = torch.Generator().manual_seed(16)
    M, K, N, p = 1000, 456, 328, 0.5
    x = torch.randn(M, K, generator=gen).to(dtype)
    w = (torch.randn(N, K, generator=gen) * K ** -0.5).to(dtype)
    mk = cpu_mask(O.mask_shape(M, K, 64), p, gen)
    lists = ext.build_lists(mk.cuda())
    s = 1 / (1 - p)
    y, pre = ext.gemm_dsd_lists_act(x.cuda(), w.cuda(), lists, 64, s, act, want_pre=True)
    assert ext.last_kernel() == "specialised"
    ry, rpre = O.dsd_forward_act(to_np(x), to_np(w), mk.numpy(), 64, p, act, np.float32)
    assert max_tile_rel_fro(pre, rpre) <= REL_FRO_TOL
    assert max_tile_rel_fro(y, ry) <= REL_FRO_TOL
    if act == "relu":
        assert (y >= 0).all()
    # input gradient carried to the previous pre-activation: dX[M, K] * act'(at[M, K])
    dy = torch.randn(M, N, generator=gen).to(dtype)
    at = torch.randn(M, K, generator=gen).to(dtype)
    dx = ext.gemm_sdd_lists_actgrad(dy.cuda(), w.cuda().t(), lists, 64, s, act, at.cuda(), keep_hint=1 - p)
    assert ext.last_kernel() == "specialised"
    rdx = O.sdd_dx_actgrad(to_np(dy), to_np(w), mk.numpy(), 64, p, act, to_np(at), np.float32)
    assert max_tile_rel_fro(dx, rdx) <= REL_FRO_TOL
    keep = O.expand_keep(mk.numpy(), 64, M, K)
    assert (to_np(dx)[~keep] == 0).all()
    # act = None is the plain product
    y0, none = ext.gemm_dsd_lists_act(x.cuda(), w.cuda(), lists, 64, s, None)
    assert none is None and torch.equal(y0, ext.gemm_dsd_lists(x.cuda(), w.cuda(), lists, 64, s))


@pytest.mark.parametrize("act,dims,rows", [("relu", (784, 1024, 1024, 10), 4096), ("gelu", (384, 1536, 384), 16384),
                                            (None, (192, 128, 72), 300)])
def test_fused_mlp_against_the_oracle_and_the_unfused_layers(act, dims, rows):
    """The MLP-on-images and transformer-FFN configurations as one autograd function with fused activation
    epilogues: output, input gradient and every weight gradient against the oracle's chain rule under the same
    masks, and against the unfused composition (separate layers + torch activations)."""
    import flash_dropout.functional as F

    gen = torch.Generator().manual_seed(17)
    p = 0.5
    x = (torch.rand(rows, dims[0], generator=gen) if act == "relu" else torch.randn(rows, dims[0], generator=gen)).half()
    ws = [((torch.rand(dims[i + 1], dims[i], generator=gen) * 2 - 1) * dims[i] ** -0.5).half() for i in range(len(dims) - 1)]
    masks = [cpu_mask(O.mask_shape(rows, dims[i], 64), p, gen) for i in range(len(ws))]
    dy = torch.randn(rows, dims[-1], generator=gen).half()
    xg = x.cuda().requires_grad_()
    wg = [w.cuda().requires_grad_() for w in ws]
    out = F.hip_blockwise_dropout_mlp(xg, wg, 64, p, act, masks=[m.cuda() for m in masks])
    out.backward(dy.cuda())
    # hidden tensors live in fp16 between the layers, in the oracle as on the device
    rout, rdx, rdws = O.mlp_forward_backward(to_np(x), [to_np(w) for w in ws], [m.numpy() for m in masks], 64, p, act,
                                             to_np(dy), np.float32, hidden_dtype=np.float16)
    assert max_tile_rel_fro(out, rout) <= REL_FRO_TOL
    assert max_tile_rel_fro(xg.grad, rdx) <= REL_FRO_TOL
    for got, ref in zip(wg, rdws):
        assert got.grad.shape == ref.shape
        assert max_tile_rel_fro(got.grad, ref) <= REL_FRO_TOL
    # the unfused composition (it rounds the hidden pre-activations to fp16 before activating them)
    x2 = x.cuda().requires_grad_()
    w2 = [w.cuda().requires_grad_() for w in ws]
    f = {"relu": torch.relu, "gelu": torch.nn.functional.gelu, None: lambda t: t}[act]
    h = x2
    for i, w in enumerate(w2):
        h = F.hip_blockwise_dropout_matmul_mask(h, masks[i].cuda(), 64, p, w)
        if i + 1 < len(w2):
            h = f(h)
    h.backward(dy.cuda())
    assert rel_fro(out, h.float()) <= 2e-3
    assert rel_fro(xg.grad, x2.grad.float()) <= 4e-3
    for a, b in zip(wg, w2):
        assert rel_fro(a.grad, b.grad.float()) <= 4e-3


@pytest.mark.parametrize("act", ["relu", "gelu"])
def test_dense_product_with_fused_activation_and_the_stack_that_starts_with_one(act):
    """sd_gemm_act against act(A . B^T) from the oracle, and the fused MLP whose first layer has p = 0 (the dense
    fused product, no mask, no lists) against the same stack run with explicit masks (the list path the oracle
    test above pins)."""
    import flash_dropout.functional as F
    from flash_dropout.hip import GEMM

    ext = GEMM()
    gen = torch.Generator().manual_seed(29)
    rows, dims = 520, [200, 320, 264, 72]
    x = torch.randn(rows, dims[0], generator=gen).half()
    ws = [(torch.randn(dims[i + 1], dims[i], generator=gen) * dims[i] ** -0.5).half() for i in range(3)]
    y, pre = ext.gemm_act(x.cuda(), ws[0].cuda(), act, want_pre=True)
    ref_pre = to_np(x).astype(np.float64) @ to_np(ws[0]).astype(np.float64).T
    assert max_tile_rel_fro(pre, ref_pre.astype(np.float32)) <= REL_FRO_TOL
    assert max_tile_rel_fro(y, O.act_apply(ref_pre, act).astype(np.float32)) <= REL_FRO_TOL
    assert ext.last_kernel() == "specialised"
    ps, seed = [0.0, 0.5, 0.5], 31
    masks = [torch.zeros(O.mask_shape(rows, dims[0], 64), dtype=torch.bool)] + [
        torch.from_numpy(O.random_mask(O.mask_shape(rows, dims[i], 64), 0.5, seed + i)) for i in (1, 2)]
    dy = torch.randn(rows, dims[-1], generator=gen).half().cuda()
    grads = []
    for kw in ({"seed": seed}, {"masks": [m.cuda() for m in masks]}):
        wg = [w.cuda().requires_grad_() for w in ws]
        out = F.hip_blockwise_dropout_mlp(x.cuda(), wg, 64, ps, act, **kw)
        out.backward(dy)
        grads.append((out.detach(), [w.grad for w in wg]))
    (o1, g1), (o2, g2) = grads
    assert rel_fro(o1, o2.float()) <= 1e-3
    for a, b in zip(g1, g2):
        assert a.shape == b.shape and rel_fro(a, b.float()) <= 1e-3


@pytest.mark.parametrize("act", ["relu", "gelu"])
def test_dense_first_layer_takes_a_transposed_weight_view_and_a_narrow_output(act):
    """The fused MLP's dense first layer (p = 0, input without gradient) with its weight given as a transposed view (the
    operand layout of the input gradient: the activation then runs on the generic kernel's store), and a one-layer
    stack whose output width is not a multiple of 8 (its weight gradient goes through zero-padded columns, inside
    the library): both against the oracle."""
    import flash_dropout.functional as F

    gen = torch.Generator().manual_seed(37)
    rows, dims = 384, [200, 320, 72]
    x = torch.randn(rows, dims[0], generator=gen).half()
    w0 = (torch.randn(dims[0], dims[1], generator=gen) * dims[0] ** -0.5).half()   # stored [in, out]: used as w0.t()
    w1 = (torch.randn(dims[2], dims[1], generator=gen) * dims[1] ** -0.5).half()
    dy = torch.randn(rows, dims[2], generator=gen).half()
    seed = 5
    w0g, w1g = w0.cuda().requires_grad_(), w1.cuda().requires_grad_()
    out = F.hip_blockwise_dropout_mlp(x.cuda(), [w0g.t(), w1g], 64, [0.0, 0.5], act, seed=seed)
    out.backward(dy.cuda())
    masks = [np.zeros(O.mask_shape(rows, dims[0], 64), dtype=bool), O.random_mask(O.mask_shape(rows, dims[1], 64), 0.5, seed + 1)]
    ry, _, rdw = O.mlp_forward_backward(to_np(x), [to_np(w0).T.copy(), to_np(w1)], masks, 64, [0.0, 0.5], act, to_np(dy),
                                        hidden_dtype=np.float16)
    assert max_tile_rel_fro(out, ry) <= REL_FRO_TOL
    assert max_tile_rel_fro(w0g.grad.t(), rdw[0]) <= REL_FRO_TOL
    assert max_tile_rel_fro(w1g.grad, rdw[1]) <= REL_FRO_TOL
    # one dense layer, 10 outputs
    w = (torch.randn(10, dims[0], generator=gen) * dims[0] ** -0.5).half().cuda().requires_grad_()
    g10 = torch.randn(rows, 10, generator=gen).half()
    F.hip_blockwise_dropout_mlp(x.cuda(), [w], 64, 0.0, act).backward(g10.cuda())
    assert w.grad.shape == (10, dims[0])
    assert max_tile_rel_fro(w.grad, to_np(g10).T @ to_np(x)) <= REL_FRO_TOL


@pytest.mark.parametrize("name", ["mlp", "mlp-784", "vit-ffn", "gpt-ffn"])
def test_model_harness_runs_every_variant(name):
    """benchmark/model.py (the reference's benchmark/model.py:119-229 protocol): every variant of every model
    steps forward and backward, eagerly and as a replayed graph, and the fused stack agrees with the layer-by-layer
    model when both are given the same weights and no dropout."""
    from benchmark import model as bm

    cls, make_x = bm.MODELS[name]
    torch.manual_seed(0)
    x = make_x().cuda().half()
    for variant in ("none", "vanilla", "blockwise[hip]", "blockwise[hip-fused]"):
        net = (bm.fused_variant(name, 0.5, 64) if variant.endswith("fused]") else cls(variant, 0.5, 64)).cuda().half().train()
        ts = bm.time_model(net, x, warmup=0.0, rep=0.0, graph=False)
        assert len(ts) >= 5 and all(t > 0 for t in ts)
    fused = bm.fused_variant(name, 0.5, 64).cuda().half().train()
    assert len(bm.time_model(fused, x, warmup=0.0, rep=0.0, graph=True)) >= 5
    # p = 0: the fused stack is the dense model
    fused0 = bm.fused_variant(name, 0.0, 64).cuda().half().train()
    plain = cls("none", 0.0, 64).cuda().half().train()
    mods = list(plain.linears) if hasattr(plain, "linears") else [plain.up, plain.down]
    for a, b in zip(fused0.linears, mods):
        b.weight.data.copy_(a.weight.data)
    assert rel_fro(fused0(x), plain(x).float()) <= 3e-3


@pytest.mark.parametrize("bs", [32, 96, 160])
def test_odd_multiples_of_32_through_autograd_and_the_fused_mlp(bs):
    """block_size = 32, 96, 160 end to end: the single layer's autograd function (one library call per direction)
    and the fused MLP, against the oracle under the masks the library drew."""
    import flash_dropout.functional as F
    from flash_dropout.hip import GEMM

    gen = torch.Generator().manual_seed(18)
    M, K, N, p = 480, 352, 264, 0.5
    x = torch.randn(M, K, generator=gen).half()
    w = (torch.randn(N, K, generator=gen) * K ** -0.5).half()
    dy = torch.randn(M, N, generator=gen).half()
    xg, wg = x.cuda().requires_grad_(), w.cuda().requires_grad_()
    y = F.hip_blockwise_dropout_matmul(xg, wg, bs, p, seed=123)
    y.backward(dy.cuda())
    mask = O.random_mask(O.mask_shape(M, K, bs), p, 123)
    assert max_tile_rel_fro(y, O.dsd_forward(to_np(x), to_np(w), mask, bs, p, np.float32), tile=32) <= REL_FRO_TOL
    assert max_tile_rel_fro(xg.grad, O.sdd_dx(to_np(dy), to_np(w), mask, bs, p, np.float32), tile=32) <= REL_FRO_TOL
    assert max_tile_rel_fro(wg.grad, O.dsd_dw(to_np(dy), to_np(x), mask, bs, p, np.float32), tile=32) <= REL_FRO_TOL
    # the mask form that allocates nothing takes it too
    ext = GEMM()
    out = torch.empty(M, N, dtype=torch.float16, device="cuda")
    ext.gemm_dsd_noalloc(x.cuda(), w.cuda(), torch.from_numpy(mask).cuda(), bs, 1 / (1 - p), out)
    assert torch.equal(out, y.detach())
    # fused MLP, ReLU, given masks
    dims = (352, 264, 96)
    ws = [((torch.rand(dims[i + 1], dims[i], generator=gen) * 2 - 1) * dims[i] ** -0.5).half() for i in range(2)]
    masks = [cpu_mask(O.mask_shape(M, dims[i], bs), p, gen) for i in range(2)]
    dy2 = torch.randn(M, dims[-1], generator=gen).half()
    xg = x.cuda().requires_grad_()
    wgs = [t.cuda().requires_grad_() for t in ws]
    out = F.hip_blockwise_dropout_mlp(xg, wgs, bs, p, "relu", masks=[m.cuda() for m in masks])
    out.backward(dy2.cuda())
    rout, rdx, rdws = O.mlp_forward_backward(to_np(x), [to_np(t) for t in ws], [m.numpy() for m in masks], bs, p,
                                             "relu", to_np(dy2), np.float32, hidden_dtype=np.float16)
    assert max_tile_rel_fro(out, rout, tile=32) <= REL_FRO_TOL
    assert max_tile_rel_fro(xg.grad, rdx, tile=32) <= REL_FRO_TOL
    for got, ref in zip(wgs, rdws):
        assert max_tile_rel_fro(got.grad, ref, tile=32) <= REL_FRO_TOL
