"""sd_gemm_dsd_noalloc (the entry point that allocates nothing) against sd_gemm_dsd, through the C ABI.

Two calls in a row share the library's built-in scratch array; the second has a smaller input, so
anything stale from the first call that leaked into it would show.  Run last: a failure here must not
hide the other GPU tests."""
import ctypes

import numpy as np
import pytest
import torch

from _util import REL_FRO_TOL, cpu_mask, make_operand, max_tile_rel_fro, to_np
from oracle import sparsedrop_oracle as O

pytestmark = pytest.mark.gpu


def _raw_call(lib, name, A, B, C, mask, M, N, K, bs, scale, tail):
    fn = getattr(lib, name)
    rc = fn(A.data_ptr(), A.stride(0), A.stride(1), B.data_ptr(), B.stride(0), B.stride(1),
            C.data_ptr(), C.stride(0), C.stride(1), mask.data_ptr(), mask.stride(0), mask.stride(1),
            M, N, K, bs, ctypes.c_float(scale), 0, *tail)
    assert rc == 0, lib.sd_last_error().decode()


@pytest.mark.parametrize("dtype", [torch.float16])
def test_noalloc_matches_workspace_form_on_two_calls_in_a_row(dtype):
    from flash_dropout.hip import GEMM

    ext = GEMM()
    lib = ext.lib
    assert lib.sd_noalloc_scratch_bytes() >= 1 << 20
    stream = torch.cuda.current_stream().cuda_stream
    gen = torch.Generator().manual_seed(21)
    # the second problem is smaller in every dimension, and has another block size (listed at 64 granularity)
    for (M, N, K, bs, p) in [(2048, 512, 1536, 64, 0.5), (700, 136, 392, 128, 0.3)]:
        A = make_operand(M, K, dtype, "cuda", gen=gen)
        B = make_operand(N, K, dtype, "cuda", scale=K ** -0.5, gen=gen)
        mk = cpu_mask(O.mask_shape(M, K, bs), p, gen)
        mask = mk.cuda()
        scale = 1 / (1 - p)
        ws_bytes = (lib.sd_workspace_bytes(-(-M // 64), -(-K // 64)) + 15) // 16 * 16
        ws = torch.empty(ws_bytes // 4, dtype=torch.int32, device="cuda")
        want = torch.full((M, N), float("nan"), dtype=dtype, device="cuda")
        got = torch.full((M, N), float("nan"), dtype=dtype, device="cuda")
        _raw_call(lib, "sd_gemm_dsd", A, B, want, mask, M, N, K, bs, scale, (ws.data_ptr(), ws_bytes, stream))
        _raw_call(lib, "sd_gemm_dsd_noalloc", A, B, got, mask, M, N, K, bs, scale, (stream,))
        torch.cuda.synchronize()
        assert torch.equal(got, want), (M, N, K, bs)
        ref = O.gemm_dsd(to_np(A), to_np(B), mk.numpy(), bs, scale, np.float32)
        assert max_tile_rel_fro(got, ref) <= REL_FRO_TOL


def test_noalloc_rejects_what_does_not_fit_and_allocates_nothing():
    from flash_dropout.hip import GEMM

    ext = GEMM()
    gen = torch.Generator().manual_seed(22)
    M, N, K, bs = 512, 256, 384, 64
    A = make_operand(M, K, torch.float16, "cuda", gen=gen)
    B = make_operand(N, K, torch.float16, "cuda", gen=gen)
    mask = cpu_mask((M // bs, K // bs), 0.5, gen).cuda()
    out = torch.empty(M, N, dtype=torch.float16, device="cuda")
    ext.gemm_dsd_noalloc(A, B, mask, bs, 2.0, out)  # first use on this device done
    torch.cuda.synchronize()
    before = torch.cuda.memory_stats()["allocation.all.allocated"]
    free_before, _ = torch.cuda.mem_get_info()
    ext.gemm_dsd_noalloc(A, B, mask, bs, 2.0, out)
    torch.cuda.synchronize()
    assert torch.cuda.memory_stats()["allocation.all.allocated"] == before
    assert torch.cuda.mem_get_info()[0] == free_before
    assert torch.equal(out, ext.gemm_dsd(A, B, mask, bs, 2.0))
    # a grid whose list does not fit the built-in array: rejected on the host, nothing launched (the operand
    # pointers are never dereferenced, so a small tensor stands in for the huge matrix)
    big = 64 * 1024
    rc = ext.lib.sd_gemm_dsd_noalloc(A.data_ptr(), big, 1, B.data_ptr(), big, 1, out.data_ptr(), N, 1,
                                     mask.data_ptr(), big // 64, 1, big, N, big, 64, ctypes.c_float(2.0), 0, None)
    assert rc == 1 and b"scratch" in ext.lib.sd_last_error()


def test_noalloc_under_graph_capture_after_a_first_call():
    """What the entry point is for: captured in a HIP graph (after one eager call on the device, which does the
    one-time symbol lookup and kernel set-up) and replayed on changing inputs, with eager work and synchronisations
    between the replays; every replay against sd_gemm_dsd on the same inputs."""
    from flash_dropout.hip import GEMM

    ext = GEMM()
    gen = torch.Generator().manual_seed(23)
    M, N, K, bs, p = 1024, 384, 768, 64, 0.5
    A = make_operand(M, K, torch.float16, "cuda", gen=gen)
    B = make_operand(N, K, torch.float16, "cuda", scale=K ** -0.5, gen=gen)
    mask = cpu_mask((M // bs, K // bs), p, gen).cuda()
    out = torch.empty(M, N, dtype=torch.float16, device="cuda")
    ext.gemm_dsd_noalloc(A, B, mask, bs, 2.0, out)  # first use on this device, outside the capture
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        ext.gemm_dsd_noalloc(A, B, mask, bs, 2.0, out)
    for rep in range(3):
        A.copy_(make_operand(M, K, torch.float16, "cuda", gen=gen))          # eager work between the replays
        mask.copy_(cpu_mask((M // bs, K // bs), p, gen).cuda())
        out.fill_(float("nan"))
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out, ext.gemm_dsd(A, B, mask, bs, 2.0)), rep
