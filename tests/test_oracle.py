"""Pins the CPU oracle (oracle/sparsedrop_oracle.py) before anything is compared against it.

What pins what:
  * compaction + increment table: the literal known answers in tests/golden/compaction_cases.json
    (case "reference_docstring" is the example in the reference's own docstring,
    flash_dropout/functional/utils.py:36-56), the numpy.nonzero identity, and a pure-Python loop.
  * the three products: triple-loop brute force on tiny inputs, reduction to a dense matmul at p=0,
    the single-kept-block closed form, exact zeros in dropped SDD tiles, and torch autograd through a
    literal restatement of the reference's naive path (oracle/naive_torch.py) — chosen so that a
    transposed operand, a wrong mask polarity, a dropped 1/(1-p) or a mask applied on the wrong side
    fails at least one of them.
  * conv: torch's own F.unfold / F.fold / F.conv2d.
"""
import json
from pathlib import Path

import numpy as np
import pytest
import torch

from oracle import naive_torch
from oracle import sparsedrop_oracle as O

GOLDEN = Path(__file__).parent / "golden"
CASES = json.loads((GOLDEN / "compaction_cases.json").read_text())


# ------------------------------------------------------------------ compaction
@pytest.mark.parametrize("name", sorted(CASES))
def test_compaction_known_answers(name):
    c = CASES[name]
    mask = np.array(c["mask"], dtype=bool)
    row_ptr, col_idx = O.compact_csr(mask)
    col_ptr, row_idx = O.compact_csc(mask)
    assert row_ptr.dtype == np.int32 and col_idx.dtype == np.int32
    assert row_ptr.tolist() == c["row_ptr"]
    assert col_idx.tolist() == c["col_idx"]
    assert col_ptr.tolist() == c["col_ptr"]
    assert row_idx.tolist() == c["row_idx"]
    table, row_indices, row_widths = O.mask_to_increment_table(mask, c["block_k"])
    assert table.tolist() == c["table"]
    assert row_indices.tolist() == c["row_indices"]
    assert row_widths.tolist() == c["row_widths"]
    # offsets of the docstring = running position implied by the table
    offs = []
    for r in range(mask.shape[0]):
        pos = 0
        for i in range(row_indices[r], row_indices[r] + row_widths[r]):
            pos = table[i] if i == row_indices[r] else pos + table[i]
            offs.append(int(pos))
    assert offs == c["offsets"]


def _loop_lists(mask):
    rp, ci = [0], []
    for r in range(mask.shape[0]):
        for c in range(mask.shape[1]):
            if not mask[r, c]:
                ci.append(c)
        rp.append(len(ci))
    return rp, ci


@pytest.mark.parametrize("shape,p,seed", [((16, 16), 0.5, 0), ((7, 13), 0.3, 1), ((64, 9), 0.9, 2),
                                          ((1, 200), 0.5, 3), ((130, 1), 0.5, 4), ((5, 5), 0.0, 5),
                                          ((5, 5), 1.0, 6)])
def test_compaction_vs_loops_and_nonzero(shape, p, seed):
    rng = np.random.default_rng(seed)
    mask = rng.random(shape) < p
    row_ptr, col_idx = O.compact_csr(mask)
    rp, ci = _loop_lists(mask)
    assert row_ptr.tolist() == rp and col_idx.tolist() == ci
    col_ptr, row_idx = O.compact_csc(mask)
    rp, ci = _loop_lists(mask.T)
    assert col_ptr.tolist() == rp and row_idx.tolist() == ci
    tab = O.kept_table(mask)
    assert tab.dtype == np.int64
    nz = torch.nonzero(~torch.from_numpy(mask), as_tuple=False).numpy()
    assert np.array_equal(tab, nz)
    assert np.array_equal(tab[:, 1], col_idx)


def test_cfg1_mask_fixture():
    fx = json.loads((GOLDEN / "cfg1_mask.json").read_text())
    mask = np.array([[ch == "1" for ch in row] for row in fx["rows"]])
    assert mask.shape == (16, 16)
    # regenerating with the documented draw order gives the stored bits
    torch.manual_seed(0)
    torch.randn(1024, 1024), torch.randn(1024, 1024), torch.randn(1024, 1024)
    again = (torch.rand(16, 16) < 0.5).numpy()
    assert np.array_equal(mask, again)
    assert O.mask_shape(1024, 1024, 64) == (16, 16)


def test_mask_shape_is_ceil():
    assert O.mask_shape(784, 784, 64) == (13, 13)
    assert O.mask_shape(4096, 10, 64) == (64, 1)
    keep = O.expand_keep(np.array([[False, True], [True, False]]), 4, 6, 5)
    assert keep.shape == (6, 5)
    assert keep[:4, :4].all() and not keep[:4, 4:].any() and not keep[4:, :4].any() and keep[4:, 4:].all()


# ------------------------------------------------------------------ products
def _brute_dsd(a, b, mask, bs, scale):
    m, k = a.shape
    n = b.shape[0]
    out = np.zeros((m, n))
    for i in range(m):
        for j in range(n):
            acc = 0.0
            for kk in range(k):
                if not mask[i // bs, kk // bs]:
                    acc += a[i, kk] * b[j, kk]
            out[i, j] = acc * scale
    return out


def _brute_sdd(a, b, mask, bs, scale):
    m, k = a.shape
    n = b.shape[0]
    out = np.zeros((m, n))
    for i in range(m):
        for j in range(n):
            if mask[i // bs, j // bs]:
                continue
            out[i, j] = scale * sum(a[i, kk] * b[j, kk] for kk in range(k))
    return out


@pytest.mark.parametrize("m,n,k,bs", [(8, 6, 8, 2), (12, 5, 16, 4), (7, 3, 10, 4)])
def test_products_bruteforce(m, n, k, bs):
    rng = np.random.default_rng(m * 100 + k)
    a, b = rng.standard_normal((m, k)), rng.standard_normal((n, k))
    mask = rng.random(O.mask_shape(m, k, bs)) < 0.5
    np.testing.assert_allclose(O.gemm_dsd(a, b, mask, bs, 1.7), _brute_dsd(a, b, mask, bs, 1.7), rtol=1e-12, atol=1e-12)
    mask_o = rng.random(O.mask_shape(m, n, bs)) < 0.5
    got = O.gemm_sdd(a, b, mask_o, bs, 2.5)
    np.testing.assert_allclose(got, _brute_sdd(a, b, mask_o, bs, 2.5), rtol=1e-12, atol=1e-12)
    assert (got[~O.expand_keep(mask_o, bs, m, n)] == 0).all()


def test_p0_is_dense_and_single_block_closed_form():
    rng = np.random.default_rng(0)
    x, w, dy = rng.standard_normal((8, 12)), rng.standard_normal((5, 12)), rng.standard_normal((8, 5))
    none = np.zeros((2, 3), dtype=bool)
    np.testing.assert_allclose(O.dsd_forward(x, w, none, 4, 0.0), x @ w.T, rtol=1e-13)
    np.testing.assert_allclose(O.sdd_dx(dy, w, none, 4, 0.0), dy @ w, rtol=1e-13)
    np.testing.assert_allclose(O.dsd_dw(dy, x, none, 4, 0.0), dy.T @ x, rtol=1e-13)
    one = np.ones((2, 3), dtype=bool)
    one[1, 2] = False  # only block (1,2) kept: rows 4..8, cols 8..12
    p = 0.75
    y = O.dsd_forward(x, w, one, 4, p)
    assert (y[:4] == 0).all()
    np.testing.assert_allclose(y[4:], 4.0 * x[4:, 8:] @ w[:, 8:].T, rtol=1e-13)
    dx = O.sdd_dx(dy, w, one, 4, p)
    assert (dx[:4] == 0).all() and (dx[:, :8] == 0).all()
    np.testing.assert_allclose(dx[4:, 8:], 4.0 * dy[4:] @ w[:, 8:], rtol=1e-13)
    dw = O.dsd_dw(dy, x, one, 4, p)
    assert (dw[:, :8] == 0).all()
    np.testing.assert_allclose(dw[:, 8:], 4.0 * dy[4:].T @ x[4:, 8:], rtol=1e-13)


@pytest.mark.parametrize("p", [0.0, 0.3, 0.9])
def test_products_vs_autograd_of_naive_restatement(p):
    torch.manual_seed(1)
    m, n, k, bs = 32, 24, 48, 8
    x = torch.randn(m, k, dtype=torch.float64)
    w = torch.randn(n, k, dtype=torch.float64)
    dy = torch.randn(m, n, dtype=torch.float64)
    mask = torch.rand(m // bs, k // bs) < p
    y, dx, dw = naive_torch.forward_backward(x, w, dy, mask, bs, p)
    mk = mask.numpy()
    np.testing.assert_allclose(O.dsd_forward(x.numpy(), w.numpy(), mk, bs, p), y.numpy(), rtol=1e-12, atol=1e-12)
    np.testing.assert_allclose(O.sdd_dx(dy.numpy(), w.numpy(), mk, bs, p), dx.numpy(), rtol=1e-12, atol=1e-12)
    np.testing.assert_allclose(O.dsd_dw(dy.numpy(), x.numpy(), mk, bs, p), dw.numpy(), rtol=1e-12, atol=1e-12)


def test_backward_formulas_match_reference_operand_algebra():
    # dX = gemm_sdd(dY, W.T, mask), dW = gemm_dsd(X.T, dY.T, mask.T).T (blockwise_dropout_matmul_cuda.py:46-51)
    rng = np.random.default_rng(3)
    x, w, dy = rng.standard_normal((16, 8)), rng.standard_normal((12, 8)), rng.standard_normal((16, 12))
    mask = rng.random((4, 2)) < 0.5
    s = 1 / (1 - 0.4)
    np.testing.assert_allclose(O.sdd_dx(dy, w, mask, 4, 0.4), O.gemm_sdd(dy, w.T, mask, 4, s), rtol=1e-13)
    np.testing.assert_allclose(O.dsd_dw(dy, x, mask, 4, 0.4), O.gemm_dsd(x.T, dy.T, mask.T, 4, s).T, rtol=1e-13)


# ------------------------------------------------------------------ conv
CONV_CASES = [
    dict(n=2, c=3, h=8, w=8, k=4, r=3, s=3, padding=(1, 1), stride=(1, 1), dilation=(1, 1)),
    dict(n=1, c=2, h=9, w=7, k=3, r=3, s=2, padding=(0, 1), stride=(2, 1), dilation=(1, 2)),
    dict(n=2, c=4, h=6, w=6, k=2, r=1, s=1, padding=(0, 0), stride=(1, 1), dilation=(1, 1)),
]


@pytest.mark.parametrize("cfg", CONV_CASES)
def test_im2col_matches_unfold_and_fold(cfg):
    torch.manual_seed(0)
    x = torch.randn(cfg["n"], cfg["c"], cfg["h"], cfg["w"], dtype=torch.float64)
    geo = dict(padding=cfg["padding"], stride=cfg["stride"], dilation=cfg["dilation"])
    cols = O.im2col(x.numpy(), cfg["r"], cfg["s"], **geo)
    ref = torch.nn.functional.unfold(x, (cfg["r"], cfg["s"]), **geo).permute(0, 2, 1)
    ref = ref.reshape(-1, cfg["c"] * cfg["r"] * cfg["s"]).numpy()
    assert np.array_equal(cols, ref)
    p_, q_ = O.conv_out_hw(cfg["h"], cfg["w"], cfg["r"], cfg["s"], **geo)
    g = torch.randn(cols.shape, dtype=torch.float64)
    back = O.col2im(g.numpy(), x.shape, cfg["r"], cfg["s"], **geo)
    fold_in = g.reshape(cfg["n"], p_ * q_, -1).permute(0, 2, 1)
    ref_back = torch.nn.functional.fold(fold_in, (cfg["h"], cfg["w"]), (cfg["r"], cfg["s"]), **geo).numpy()
    np.testing.assert_allclose(back, ref_back, rtol=1e-13, atol=1e-13)


@pytest.mark.parametrize("cfg", CONV_CASES)
def test_conv_p0_matches_conv2d_with_grads(cfg):
    torch.manual_seed(1)
    x = torch.randn(cfg["n"], cfg["c"], cfg["h"], cfg["w"], dtype=torch.float64, requires_grad=True)
    k = torch.randn(cfg["k"], cfg["c"], cfg["r"], cfg["s"], dtype=torch.float64, requires_grad=True)
    geo = dict(padding=cfg["padding"], stride=cfg["stride"], dilation=cfg["dilation"])
    y_ref = torch.nn.functional.conv2d(x, k, **geo)
    dy = torch.randn_like(y_ref)
    y_ref.backward(dy)
    rows = y_ref.shape[0] * y_ref.shape[2] * y_ref.shape[3]
    mask = np.zeros(O.mask_shape(rows, cfg["c"] * cfg["r"] * cfg["s"], 4), dtype=bool)
    y, dx, dk = O.conv2d_blockdrop(x.detach().numpy(), k.detach().numpy(), mask, 4, 0.0, dy=dy.numpy(), **geo)
    np.testing.assert_allclose(y, y_ref.detach().numpy(), rtol=1e-12, atol=1e-12)
    np.testing.assert_allclose(dx, x.grad.numpy(), rtol=1e-12, atol=1e-12)
    np.testing.assert_allclose(dk, k.grad.numpy(), rtol=1e-12, atol=1e-12)


def test_conv_blockdrop_vs_autograd_composition():
    torch.manual_seed(2)
    n, c, h, w, kk, r, s, bs, p = 2, 4, 8, 8, 6, 3, 3, 4, 0.5
    geo = dict(padding=(1, 1), stride=(1, 1), dilation=(1, 1))
    x = torch.randn(n, c, h, w, dtype=torch.float64, requires_grad=True)
    k = torch.randn(kk, c, r, s, dtype=torch.float64, requires_grad=True)
    rows, ncols = n * h * w, c * r * s
    mask = torch.rand(rows // bs, ncols // bs) < p
    cols = torch.nn.functional.unfold(x, (r, s), **geo).permute(0, 2, 1).reshape(rows, ncols)
    y2 = naive_torch.forward(cols, k.reshape(kk, -1), mask, bs, p)
    y_ref = y2.view(n, h * w, kk).permute(0, 2, 1).reshape(n, kk, h, w)
    dy = torch.randn_like(y_ref)
    y_ref.backward(dy)
    y, dx, dk = O.conv2d_blockdrop(x.detach().numpy(), k.detach().numpy(), mask.numpy(), bs, p, dy=dy.numpy(), **geo)
    np.testing.assert_allclose(y, y_ref.detach().numpy(), rtol=1e-12, atol=1e-12)
    np.testing.assert_allclose(dx, x.grad.numpy(), rtol=1e-12, atol=1e-12)
    np.testing.assert_allclose(dk, k.grad.numpy(), rtol=1e-12, atol=1e-12)


# ---- on-device mask draw and block splitting ---------------------------------------------------
# Known answers of Philox4x32-10 from the Random123 distribution's kat_vectors (counter, key, output).
PHILOX_KAT = [
    ([0x00000000] * 4, [0x00000000] * 2, [0x6627E8D5, 0xE169C58D, 0xBC57AC4C, 0x9B00DBD8]),
    ([0xFFFFFFFF] * 4, [0xFFFFFFFF] * 2, [0x408F276D, 0x41C83B0E, 0xA20BC7C6, 0x6D5451FD]),
    ([0x243F6A88, 0x85A308D3, 0x13198A2E, 0x03707344], [0xA4093822, 0x299F31D0],
     [0xD16CFE09, 0x94FDCCEB, 0x5001E420, 0x24126EA1]),
]


@pytest.mark.parametrize("counter,key,want", PHILOX_KAT)
def test_philox_known_answers(counter, key, want):
    assert O.philox4x32_10(counter, key).tolist() == want


def test_philox_is_vectorised_consistently():
    ctr = np.array([k[0] for k in PHILOX_KAT], dtype=np.uint64)
    one_key = O.philox4x32_10(ctr, PHILOX_KAT[2][1])
    assert one_key[2].tolist() == PHILOX_KAT[2][2]
    assert one_key[0].tolist() == O.philox4x32_10(PHILOX_KAT[0][0], PHILOX_KAT[2][1]).tolist()


def test_random_mask_definition():
    shape = (37, 53)
    # entry e uses word e % 4 of block e // 4: recompute a few entries by hand
    m = O.random_mask(shape, 0.4, seed=(5 << 32) | 9, offset=(1 << 32) | 2)
    for e in (0, 1, 5, 702, 37 * 53 - 1):
        w = O.philox4x32_10([e // 4, 0, 2, 1], [9, 5])[e % 4]
        assert m.reshape(-1)[e] == (np.float32(w >> 8) * np.float32(2.0 ** -24) < np.float32(0.4))
    assert m.dtype == bool and m.shape == shape
    assert not O.random_mask(shape, 0.0, 1).any()                 # p = 0 keeps everything
    assert O.random_mask(shape, 1.0 - 2.0 ** -24, 1).mean() > 0.999  # True means dropped
    big = O.random_mask((512, 512), 0.3, seed=11)
    assert abs(big.mean() - 0.3) < 4 * (0.3 * 0.7 / big.size) ** 0.5
    assert (O.random_mask((512, 512), 0.3, seed=12) != big).any()
    assert (O.random_mask((512, 512), 0.3, seed=11, offset=1) != big).any()
    # rows are independent: no visible correlation between neighbouring entries
    assert abs(np.corrcoef(big[:, :-1].ravel(), big[:, 1:].ravel())[0, 1]) < 0.02


@pytest.mark.parametrize("m,k,bs,split", [(256, 384, 128, 2), (200, 130, 128, 2), (70, 500, 192, 3), (64, 64, 64, 1)])
def test_split_mask_expands_to_the_same_elements(m, k, bs, split):
    rng = np.random.default_rng(0)
    mask = rng.random(O.mask_shape(m, k, bs)) < 0.5
    fine = O.split_mask(mask, split, O.mask_shape(m, k, bs // split))
    assert fine.shape == O.mask_shape(m, k, bs // split)
    assert np.array_equal(O.expand_keep(mask, bs, m, k), O.expand_keep(fine, bs // split, m, k))


@pytest.mark.parametrize("act", ["relu", "gelu"])
def test_activations_match_torch_and_its_autograd(act):
    """act_apply / act_grad against the library routines (torch.relu, torch's erf-form gelu) and their autograd
    derivatives, over a range that covers both tails and the origin."""
    x = torch.linspace(-6, 6, 1201, dtype=torch.float64, requires_grad=True)
    y = torch.relu(x) if act == "relu" else torch.nn.functional.gelu(x)
    y.sum().backward()
    np.testing.assert_allclose(O.act_apply(x.detach().numpy(), act), y.detach().numpy(), rtol=1e-12, atol=1e-14)
    np.testing.assert_allclose(O.act_grad(x.detach().numpy(), act), x.grad.numpy(), rtol=1e-12, atol=1e-14)
    # known values: gelu(0) = 0, gelu'(0) = 1/2, relu'(0) = 0 (torch's convention)
    assert O.act_apply(np.zeros(1), act)[0] == 0.0
    assert O.act_grad(np.zeros(1), act)[0] == (0.5 if act == "gelu" else 0.0)


@pytest.mark.parametrize("act", ["relu", "gelu", None])
def test_mlp_chain_rule_vs_autograd_of_the_naive_restatement(act):
    """mlp_forward_backward, dsd_forward_act and sdd_dx_actgrad against torch autograd through the literal
    restatement of the reference's naive layer with torch activations in between: the composition the
    reference's models make (eval/mlp/model.py:31-40)."""
    from oracle import naive_torch

    gen = torch.Generator().manual_seed(31)
    bs, p = 4, 0.4
    dims = [16, 24, 12, 8]
    m = 20
    x = torch.randn(m, dims[0], generator=gen, dtype=torch.float64, requires_grad=True)
    ws = [torch.randn(dims[i + 1], dims[i], generator=gen, dtype=torch.float64, requires_grad=True) for i in range(3)]
    masks = [torch.rand(m // bs, dims[i] // bs, generator=gen) < p for i in range(3)]
    dy = torch.randn(m, dims[-1], generator=gen, dtype=torch.float64)
    f = {"relu": torch.relu, "gelu": torch.nn.functional.gelu, None: lambda t: t}[act]
    h = x
    pres = []
    for i in range(3):
        pre = naive_torch.forward(h, ws[i], masks[i], bs, p)
        pres.append(pre)
        h = f(pre) if i < 2 else pre
    h.backward(dy)
    out, dx, dws = O.mlp_forward_backward(x.detach().numpy(), [w.detach().numpy() for w in ws],
                                          [mk.numpy() for mk in masks], bs, p, act, dy.numpy())
    np.testing.assert_allclose(out, h.detach().numpy(), rtol=1e-10, atol=1e-12)
    np.testing.assert_allclose(dx, x.grad.numpy(), rtol=1e-10, atol=1e-12)
    for got, w in zip(dws, ws):
        np.testing.assert_allclose(got, w.grad.numpy(), rtol=1e-10, atol=1e-12)
    # the two fused products on their own: layer 0's activated output, and layer 1's input gradient carried to
    # layer 0's pre-activation
    y0, pre0 = O.dsd_forward_act(x.detach().numpy(), ws[0].detach().numpy(), masks[0].numpy(), bs, p, act)
    np.testing.assert_allclose(pre0, pres[0].detach().numpy(), rtol=1e-10, atol=1e-12)
    np.testing.assert_allclose(y0, f(pres[0]).detach().numpy(), rtol=1e-10, atol=1e-12)
    dpre1 = torch.randn(m, dims[2], generator=gen, dtype=torch.float64)
    x0 = pres[0].detach().clone().requires_grad_()
    naive_torch.forward(f(x0), ws[1].detach(), masks[1], bs, p).backward(dpre1)
    got = O.sdd_dx_actgrad(dpre1.numpy(), ws[1].detach().numpy(), masks[1].numpy(), bs, p, act, pres[0].detach().numpy())
    np.testing.assert_allclose(got, x0.grad.numpy(), rtol=1e-10, atol=1e-12)
    # a drop rate per layer (the reference's models start with a layer that drops nothing)
    ps = [0.0, 0.4, 0.25]
    pmasks = [torch.rand(m // bs, dims[i] // bs, generator=gen) < ps[i] for i in range(3)]
    x.grad = None
    for w in ws:
        w.grad = None
    h = x
    for i in range(3):
        h = naive_torch.forward(h, ws[i], pmasks[i], bs, ps[i])
        h = f(h) if i < 2 else h
    h.backward(dy)
    out, dx, dws = O.mlp_forward_backward(x.detach().numpy(), [w.detach().numpy() for w in ws],
                                          [mk.numpy() for mk in pmasks], bs, ps, act, dy.numpy())
    np.testing.assert_allclose(out, h.detach().numpy(), rtol=1e-10, atol=1e-12)
    np.testing.assert_allclose(dx, x.grad.numpy(), rtol=1e-10, atol=1e-12)
    for got, w in zip(dws, ws):
        np.testing.assert_allclose(got, w.grad.numpy(), rtol=1e-10, atol=1e-12)


@pytest.mark.parametrize("act", ["relu", "gelu"])
def test_mlp_with_hidden_tensors_stored_in_fp16(act):
    """mlp_forward_backward(hidden_dtype=float16) against torch autograd of the same computation: hidden tensors
    rounded to fp16 in value, identity in gradient (a straight-through rounding), GELU's derivative evaluated at
    the rounded pre-activation."""
    from oracle import naive_torch

    gen = torch.Generator().manual_seed(32)
    bs, p, m = 4, 0.25, 24
    dims = [16, 32, 8]
    x = torch.randn(m, dims[0], generator=gen, dtype=torch.float64, requires_grad=True)
    ws = [torch.randn(dims[i + 1], dims[i], generator=gen, dtype=torch.float64, requires_grad=True) for i in range(2)]
    masks = [torch.rand(m // bs, dims[i] // bs, generator=gen) < p for i in range(2)]
    dy = torch.randn(m, dims[-1], generator=gen, dtype=torch.float64)
    st = lambda t: t + (t.half().double() - t).detach()  # rounded value, identity gradient
    f = {"relu": torch.relu, "gelu": torch.nn.functional.gelu}[act]
    pre = naive_torch.forward(x, ws[0], masks[0], bs, p)
    # the activated tensor is act(exact pre) rounded; its derivative is taken at the rounded pre-activation (GELU)
    # or read off the rounded activated tensor (ReLU): spelled out with a custom function
    class Act(torch.autograd.Function):
        @staticmethod
        def forward(ctx, t):
            ctx.save_for_backward(t)
            return f(t).half().double()

        @staticmethod
        def backward(ctx, g):
            (t,) = ctx.saved_tensors
            at = t.half().double() if act == "gelu" else f(t).half().double()
            return g * torch.from_numpy(O.act_grad(at.numpy(), act))
    h = Act.apply(pre)
    out = naive_torch.forward(h, ws[1], masks[1], bs, p)
    out.backward(dy)
    rout, rdx, rdws = O.mlp_forward_backward(x.detach().numpy(), [w.detach().numpy() for w in ws],
                                             [mk.numpy() for mk in masks], bs, p, act, dy.numpy(),
                                             hidden_dtype=np.float16)
    np.testing.assert_allclose(rout, out.detach().numpy(), rtol=1e-10, atol=1e-12)
    np.testing.assert_allclose(rdx, x.grad.numpy(), rtol=1e-10, atol=1e-12)
    for got, w in zip(rdws, ws):
        np.testing.assert_allclose(got, w.grad.numpy(), rtol=1e-10, atol=1e-12)


@pytest.mark.parametrize("shape", [(4, 6), (5, 7), (1, 1), (9, 2)])
def test_merged_mask_expands_to_the_same_elements(shape):
    """merge_mask_quads / compact_csr_quads: a block-size-32 mask and its 64-grid form with quadrant bits describe
    the same element mask (expand_keep identity), and the encoded list decodes back to mask and bits."""
    rng = np.random.default_rng(sum(shape))
    mask = rng.random(shape) < 0.5
    m, k = shape[0] * 32 - 5, shape[1] * 32 - 9  # ragged last blocks
    mask64, quads = O.merge_mask_quads(mask)
    assert mask64.shape == ((shape[0] + 1) // 2, (shape[1] + 1) // 2)
    keep = O.expand_keep(mask, 32, m, k)
    rebuilt = np.zeros_like(keep)
    for i in range(mask64.shape[0]):
        for j in range(mask64.shape[1]):
            for a in range(2):
                for b in range(2):
                    if quads[i, j] >> (2 * a + b) & 1:
                        rebuilt[64 * i + 32 * a: 64 * i + 32 * a + 32, 64 * j + 32 * b: 64 * j + 32 * b + 32] = True
    assert np.array_equal(rebuilt, keep)
    assert np.array_equal(mask64, quads == 0)
    row_ptr, enc = O.compact_csr_quads(mask)
    rp, ci = O.compact_csr(mask64)
    assert np.array_equal(row_ptr, rp)
    assert np.array_equal(enc.view(np.uint32) & 0x0FFFFFFF, ci)
    rows = np.repeat(np.arange(mask64.shape[0]), np.diff(rp))
    assert np.array_equal(enc.view(np.uint32) >> 28, quads[rows, ci])


def test_merged_mask_hand_case():
    # rows 0-1 x cols 0-1 -> entry (0, 0): kept are (0, 1) and (1, 0): bits 1 and 2; entry (0, 1) covers column 2 only
    mask = np.array([[1, 0, 1], [0, 1, 0]], dtype=bool)
    mask64, quads = O.merge_mask_quads(mask)
    assert mask64.tolist() == [[False, False]]
    assert quads.tolist() == [[0b0110, 0b0100]]
    row_ptr, enc = O.compact_csr_quads(mask)
    assert row_ptr.tolist() == [0, 2]
    assert enc.view(np.uint32).tolist() == [0 | (0b0110 << 28), 1 | (0b0100 << 28)]
