"""CPU-side checks: the C-ABI library loads and exports what include/sparsedrop.h declares, host-side
argument validation (which runs before any GPU call), and the layer/host logic."""
import ctypes
import re
from pathlib import Path

import pytest
import torch

ROOT = Path(__file__).resolve().parent.parent


def _declared_symbols():
    text = (ROOT / "include" / "sparsedrop.h").read_text()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(sd_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    from flash_dropout.hip import _loader

    lib = _loader.load()
    declared = _declared_symbols()
    assert len(declared) >= 12
    for name in declared:
        assert hasattr(lib, name), f"{name} declared in include/sparsedrop.h but not exported"
    # and the ctypes table covers exactly the header
    assert sorted(_loader.SIGNATURES) == declared
    assert lib.sd_version() >= 100


def test_workspace_bytes():
    from flash_dropout.hip import _loader

    lib = _loader.load()
    # split-K scratch: wanted for a long reduction over few tiles, not for a square problem
    assert lib.sd_splitk_workspace_bytes(576, 128, 131072, 64, 1) >= 2 * 576 * 128 * 4
    assert lib.sd_splitk_workspace_bytes(8192, 8192, 8192, 64, 1) == 0
    assert lib.sd_splitk_workspace_bytes(64, 64, 512, 64, 0) == 0
    assert lib.sd_workspace_bytes(128, 128) >= (129 + 128 * 128) * 4
    assert lib.sd_workspace_bytes(1, 1) >= 12
    assert lib.sd_workspace_bytes(-1, 4) == 0


def test_host_validation_rejects_bad_arguments_without_touching_the_gpu():
    from flash_dropout.hip import _loader

    lib = _loader.load()
    fake = ctypes.c_void_p(0x1000)
    # neither stride is 1
    rc = lib.sd_gemm(fake, 2, 2, fake, 8, 1, fake, 8, 1, 8, 8, 8, 0, None, 0, None)
    assert rc == 1 and b"row or column major" in lib.sd_last_error()
    # bad dtype
    rc = lib.sd_gemm(fake, 8, 1, fake, 8, 1, fake, 8, 1, 8, 8, 8, 7, None, 0, None)
    assert rc == 1 and b"dtype" in lib.sd_last_error()
    # row stride shorter than the row
    rc = lib.sd_gemm(fake, 4, 1, fake, 8, 1, fake, 8, 1, 8, 8, 8, 0, None, 0, None)
    assert rc == 1 and b"row stride" in lib.sd_last_error()
    # unsupported block size
    rc = lib.sd_gemm_dsd_lists(fake, 96, 1, fake, 96, 1, fake, 96, 1, fake, fake, 96, 96, 96, 48, 1.0, 0, None, 0, None)
    assert rc == 2 and b"multiples of 32" in lib.sd_last_error()
    # workspace too small
    rc = lib.sd_gemm_dsd(fake, 128, 1, fake, 128, 1, fake, 128, 1, fake, 2, 1, 128, 128, 128, 64, 2.0, 0, fake, 8, None)
    assert rc == 1 and b"workspace too small" in lib.sd_last_error()
    # null list
    rc = lib.sd_gemm_sdd_lists(fake, 128, 1, fake, 128, 1, fake, 128, 1, None, None, 128, 128, 128, 64, 2.0, 0, None)
    assert rc == 1 and b"null list" in lib.sd_last_error()
    # build_lists argument checks
    rc = lib.sd_build_lists(fake, 4, 4, 4, 1, None, None, None, None, None)
    assert rc == 1 and b"nothing to build" in lib.sd_last_error()
    rc = lib.sd_build_lists(fake, 0, 4, 4, 1, fake, fake, None, None, None)
    assert rc == 1 and b"non-empty" in lib.sd_last_error()
    # conv geometry
    rc = lib.sd_im2col(fake, 1, 1, 1, 1, fake, 4, 1, 1, 2, 2, 3, 3, 0, 0, 1, 1, 1, 1, None, None, 0, 0, None)
    assert rc == 1 and b"does not fit" in lib.sd_last_error()
    rc = lib.sd_im2col(fake, 1, 1, 1, 1, fake, 4, 1, 1, 4, 4, 3, 3, 0, 0, 1, 1, 1, 1, None, None, 0, 0, None)
    assert rc == 1 and b"cols_ld" in lib.sd_last_error()
    # the implicit-GEMM conv entry points: argument errors are reported (1), geometries without a kernel are
    # declined (2) -- both before anything is launched
    # x [1, 8, 4, 4], 3x3 without padding: P = Q = 2
    conv = [1, 8, 4, 4, 64, 3, 3, 0, 0, 1, 1, 1, 1]  # n, c, h, w, k_out, r, s, pads, strides, dilations
    rc = lib.sd_conv2d_dsd_lists(fake, 128, 16, 4, 1, fake, 72, None, 64, *conv, None, None, 64, 1.0, 0, None)
    assert rc == 1 and b"null pointer" in lib.sd_last_error()
    rc = lib.sd_conv2d_dsd_lists(fake, 128, 16, 4, 1, fake, 72, fake, 64, *conv, fake, None, 64, 1.0, 0, None)
    assert rc == 1 and b"both be given" in lib.sd_last_error()
    rc = lib.sd_conv2d_dsd_lists(fake, 128, 16, 4, 1, fake, 8, fake, 64, *conv, None, None, 64, 1.0, 0, None)
    assert rc == 1 and b"leading dimensions" in lib.sd_last_error()
    rc = lib.sd_conv2d_dsd_lists(fake, 128, 16, 4, 1, fake, 72, fake, 64, *conv, None, None, 64, 1.0, 0, None)
    assert rc == 2  # P * Q = 4 is not a multiple of 64
    rc = lib.sd_conv2d_dx(fake, 64, fake, 72, None, 128, 16, 4, 1, None, 0, 0, *conv, 64, 1.0, 0, None)
    assert rc == 1 and b"null pointer" in lib.sd_last_error()
    rc = lib.sd_conv2d_dx(fake, 64, fake, 72, fake, 128, 16, 4, 1, None, 0, 0, *conv[:9], 0, 1, 1, 1, 64, 1.0, 0, None)
    assert rc == 1 and b"strides" in lib.sd_last_error()
    rc = lib.sd_conv2d_dx(fake, 64, fake, 72, fake, 128, 16, 4, 1, fake, 1, 1, *conv, 128, 1.0, 0, None)
    assert rc == 2  # a mask at another block size than 64
    rc = lib.sd_conv2d_dw_lists(fake, 128, 16, 4, 1, fake, 64, None, 72, *conv, None, None, 64, 1.0, 0, None, 0, None)
    assert rc == 1 and b"null pointer" in lib.sd_last_error()
    assert lib.sd_conv2d_dw_workspace_bytes(128, 64, 128, 3, 3, 32, 32) >= 2 * 576 * 128 * 4
    assert lib.sd_conv2d_dw_workspace_bytes(0, 64, 128, 3, 3, 32, 32) == 0


def test_python_shim_rejects_cpu_and_fp32_operands():
    from flash_dropout.hip import GEMM

    g = GEMM()
    a = torch.randn(64, 64, dtype=torch.float16)
    with pytest.raises(ValueError, match="GPU"):
        g.gemm(a, a)
    with pytest.raises(ValueError, match="GPU"):
        g.build_lists(torch.zeros(2, 2, dtype=torch.bool))


def test_block_size_int_or_equal_pair():
    from flash_dropout.hip.binding_gemm import _block_size

    assert _block_size(64) == 64
    assert _block_size((128, 128)) == 128
    with pytest.raises(ValueError):
        _block_size((64, 128))
    with pytest.raises(ValueError):
        _block_size(0)


def test_mask_helper_matches_reference_definition():
    import flash_dropout.functional as F

    x = torch.empty(3, 784, 100)
    torch.manual_seed(5)
    m = F.blockwise_dropout_mask(x, 64, 0.5)
    torch.manual_seed(5)
    again = torch.rand(3, 13, 2) < 0.5
    assert m.dtype == torch.bool and torch.equal(m, again)
    assert not F.blockwise_dropout_mask(x, (64, 64), 0.0).any()


def test_dropout_mm_layer_host_logic():
    from flash_dropout.layers import DropoutMM

    torch.manual_seed(0)
    layer = DropoutMM(16, 8, p=0.5, variant="blockwise[naive]", block_size=4)
    assert layer.weight.shape == (8, 16) and not hasattr(layer, "bias")
    x = torch.randn(2, 3, 16)
    layer.eval()
    assert torch.allclose(layer(x), torch.nn.functional.linear(x, layer.weight))
    layer.train()
    y = layer(x)
    assert y.shape == (2, 3, 8)
    for variant in ("none", "vanilla"):
        assert DropoutMM(16, 8, variant=variant)(x).shape == (2, 3, 8)
    bad = DropoutMM(16, 8, variant="nope")
    with pytest.raises(ValueError, match="Unknown variant"):
        bad(x)
    # p = 0 block dropout is a plain linear
    l0 = DropoutMM(16, 8, p=0.0, variant="blockwise[naive]", block_size=4)
    assert torch.allclose(l0(x), torch.nn.functional.linear(x, l0.weight), atol=1e-6)


def test_naive_variant_matches_oracle_with_tails():
    import numpy as np

    import flash_dropout.functional as F
    from oracle import sparsedrop_oracle as O

    torch.manual_seed(0)
    x, w = torch.randn(10, 14, dtype=torch.float64), torch.randn(5, 14, dtype=torch.float64)
    mask = torch.rand(3, 4) < 0.5
    y = F.naive_blockwise_dropout_matmul_mask(x, mask, 4, 0.25, w)
    np.testing.assert_allclose(y.numpy(), O.dsd_forward(x.numpy(), w.numpy(), mask.numpy(), 4, 0.25), rtol=1e-12)


def test_dropout_conv_layer_host_logic():
    from flash_dropout.layers import DropoutConv2d

    torch.manual_seed(0)
    x = torch.randn(2, 3, 8, 8)
    conv = DropoutConv2d(3, 4, (3, 3), padding=(1, 1), p=0.0, variant="blockwise[naive]", block_size=4)
    ref = torch.nn.functional.conv2d(x, conv.weight, padding=(1, 1))
    assert torch.allclose(conv(x), ref, atol=1e-5)
    conv.eval()
    assert torch.allclose(conv(x), ref, atol=1e-6)
    for variant in ("none", "vanilla", "vanilla_2d"):
        assert DropoutConv2d(3, 4, (3, 3), padding=(1, 1), variant=variant)(x).shape == (2, 4, 8, 8)
    with pytest.raises(ValueError, match="Unknown variant"):
        DropoutConv2d(3, 4, (3, 3), variant="nope")(x)


@pytest.mark.parametrize("kind", [0, 1])
def test_tile_map_is_a_bijection_onto_the_tile_grid(kind):
    """The workgroup-to-tile map of the specialised kernels (the counterpart of the reference's
    threadblock_swizzle, gemm.cuh:84-97) must hit every tile of the grid exactly once, for every grid up to
    40 x 40 — totals that are not multiples of the 8 XCDs and tile-row counts that are not multiples of the
    group height included."""
    from flash_dropout.hip import _loader

    lib = _loader.load()
    tm, tn = ctypes.c_int32(), ctypes.c_int32()
    for tiles_m in range(1, 41):
        for tiles_n in range(1, 41):
            seen = set()
            for b in range(tiles_m * tiles_n):
                assert lib.sd_tile_of_block(kind, b, tiles_m, tiles_n, ctypes.byref(tm), ctypes.byref(tn)) == 0
                assert 0 <= tm.value < tiles_m and 0 <= tn.value < tiles_n, (tiles_m, tiles_n, b)
                seen.add((tm.value, tn.value))
            assert len(seen) == tiles_m * tiles_n, (tiles_m, tiles_n)
    # outside the grid: an error, not a tile
    assert lib.sd_tile_of_block(kind, 12, 3, 4, ctypes.byref(tm), ctypes.byref(tn)) == 1
    assert lib.sd_tile_of_block(2, 0, 3, 4, ctypes.byref(tm), ctypes.byref(tn)) == 1


def test_tile_map_keeps_an_xcd_on_a_compact_patch():
    """What the map is for: the 32 workgroups an XCD holds at a time (launch indices x, x+8, x+16, ...) cover
    at most 8 tile rows x 4+1 tile columns of a large grid, not a scattered set."""
    from flash_dropout.hip import _loader

    lib = _loader.load()
    tm, tn = ctypes.c_int32(), ctypes.c_int32()
    tiles_m = tiles_n = 32
    for x in range(8):
        rows, cols = set(), set()
        for i in range(32):
            lib.sd_tile_of_block(0, x + 8 * i, tiles_m, tiles_n, ctypes.byref(tm), ctypes.byref(tn))
            rows.add(tm.value)
            cols.add(tn.value)
        assert len(rows) <= 8 and len(cols) <= 5, (x, sorted(rows), sorted(cols))


def test_loader_refuses_a_library_built_from_other_sources(monkeypatch):
    from flash_dropout.hip import _loader

    lib = _loader.load()
    assert lib.sd_source_hash().decode() == _loader.source_hash()
    monkeypatch.setattr(_loader, "source_hash", lambda: "0" * 16)
    with pytest.raises(RuntimeError, match="built from other sources"):
        _loader.load.__wrapped__()


def test_as_matrix_lays_out_expanded_and_strided_views():
    from flash_dropout.hip.binding_gemm import _mat, as_matrix

    a = torch.zeros(6, 8)
    at = a.t()
    assert as_matrix(a) is a and as_matrix(at) is at
    assert as_matrix(a[:, :4]) is not None and as_matrix(a[:, :4]).data_ptr() == a.data_ptr()  # row stride 8 >= 4
    e = torch.zeros(1, 8).expand(6, 8)  # strides (0, 1): what y.sum(0) hands to backward
    assert as_matrix(e).stride() == (8, 1)
    assert as_matrix(a[::2, ::2]).stride() == (4, 1)
    with pytest.raises(ValueError, match="expanded view"):
        _mat(e)
    assert _mat(torch.zeros(1, 8))[1:] == (8, 1)


@pytest.mark.parametrize("name", ["mfma_ceiling.hip", "lds_load_ceiling.hip"])
def test_ceiling_probes_compile_for_gfx950(name, tmp_path):
    """The stand-alone measurement programs under benchmark/ are only ever run on a GPU box by hand: keep them
    compiling (device code for gfx950, no GPU needed)."""
    import shutil
    import subprocess

    hipcc = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    src = Path(__file__).resolve().parent.parent / "sparse-dropout_amd" / "benchmark" / name
    proc = subprocess.run([hipcc, "--offload-arch=gfx950", "-O3", "-w", "-Xclang", "-target-feature", "-Xclang",
                           "-packed-fp32-ops", "-c", str(src), "-o", str(tmp_path / "probe.o")],
                          capture_output=True, text=True)
    assert proc.returncode == 0, proc.stderr[-2000:]


