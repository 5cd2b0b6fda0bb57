"""The drop-in binding stub published with the integration notes really is a working binding: extract the
code block, point it at the built library and run the reference's three-call sequence through it."""
import re
from pathlib import Path

import numpy as np
import pytest
import torch

from _util import REL_FRO_TOL, max_tile_rel_fro, rel_fro, to_np
from oracle import sparsedrop_oracle as O

pytestmark = pytest.mark.gpu
ROOT = Path(__file__).resolve().parent.parent


def test_integration_stub_runs_the_reference_call_sequence():
    from flash_dropout.hip import _loader

    text = (ROOT / "INTEGRATION.md").read_text()
    code = re.search(r"```python\n(.*?)```", text, flags=re.S).group(1)
    ns = {}
    exec(compile(code, "INTEGRATION.md", "exec"), ns)
    ext = ns["GEMM"](str(_loader.LIB_PATH))
    gen = torch.Generator().manual_seed(0)
    M, N, K, bs, p = 512, 256, 384, 128, 0.3
    A = torch.randn(M, K, generator=gen).half().cuda()
    B = torch.randn(N, K, generator=gen).half().cuda()
    dC = torch.randn(M, N, generator=gen).half().cuda()
    mask = (torch.rand(M // bs, K // bs, generator=gen) < p).cuda()
    s = 1 / (1 - p)
    # flash_dropout/functional/blockwise_dropout_matmul_cuda.py:26,46,49-51
    C = ext.gemm_dsd(A, B, mask, bs, s)
    dA = ext.gemm_sdd(dC, B.T, mask, bs, s)
    dB = ext.gemm_dsd(A.T, dC.T, mask.T, bs, s).T
    a, b, dc, mk = to_np(A), to_np(B), to_np(dC), mask.cpu().numpy()
    assert max_tile_rel_fro(C, O.dsd_forward(a, b, mk, bs, p, np.float32)) <= REL_FRO_TOL
    assert max_tile_rel_fro(dA, O.sdd_dx(dc, b, mk, bs, p, np.float32)) <= REL_FRO_TOL
    assert max_tile_rel_fro(dB, O.dsd_dw(dc, a, mk, bs, p, np.float32)) <= REL_FRO_TOL
    assert max_tile_rel_fro(ext.gemm(A, B), a @ b.T) <= REL_FRO_TOL
    with pytest.raises(RuntimeError, match="row or column major"):
        ext.gemm(A[::2, ::2], B[::2, ::2])
