"""ctypes loader for libsparsedrop.so (the C ABI declared in include/sparsedrop.h).

The library is built ahead of time by ``sparse-dropout_amd/csrc/build.py``; there is no JIT step and
no fallback: if the shared object is missing, or was built from other sources than the ones next to it,
loading raises.
"""
from __future__ import annotations

import ctypes
from ctypes import c_char_p, c_double, c_float, c_int, c_int64, c_uint64, c_void_p
import hashlib
from functools import lru_cache
from pathlib import Path

LIB_PATH = Path(__file__).resolve().parent.parent / "_lib" / "libsparsedrop.so"

_mat = [c_void_p, c_int64, c_int64]  # ptr, stride_r, stride_c

# name -> (restype, argtypes); mirrors include/sparsedrop.h declaration by declaration
SIGNATURES = {
    "sd_version": (c_int, []),
    "sd_last_error": (c_char_p, []),
    "sd_source_hash": (c_char_p, []),
    "sd_last_kernel": (c_char_p, []),
    "sd_last_kernel_detail": (c_char_p, []),
    "sd_tile_of_block": (c_int, [c_int, c_int64, c_int64, c_int64, c_void_p, c_void_p]),
    "sd_set_tile_policy": (c_int, [c_int]),
    "sd_workspace_bytes": (c_int64, [c_int64, c_int64]),
    "sd_build_lists": (c_int, [c_void_p, c_int64, c_int64, c_int64, c_int64,
                               c_void_p, c_void_p, c_void_p, c_void_p, c_void_p]),
    "sd_build_lists_split": (c_int, [c_void_p, c_int64, c_int64, c_int64, c_int64, c_int64, c_int64, c_int64,
                                     c_void_p, c_void_p, c_void_p, c_void_p, c_void_p]),
    "sd_random_lists": (c_int, [c_uint64, c_uint64, c_float, c_int64, c_int64, c_void_p, c_int64, c_int64,
                                c_int64, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p]),
    "sd_random_lists_state": (c_int, [c_void_p, c_float, c_int64, c_int64, c_void_p, c_int64, c_int64,
                                      c_int64, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p]),
    "sd_increment_table": (c_int, [c_void_p, c_void_p, c_int64, c_int64,
                                   c_void_p, c_void_p, c_void_p, c_void_p]),
    "sd_splitk_workspace_bytes": (c_int64, [c_int64, c_int64, c_int64, c_int64, c_int]),
    "sd_gemm": (c_int, [*_mat, *_mat, *_mat, c_int64, c_int64, c_int64, c_int, c_void_p, c_int64, c_void_p]),
    "sd_gemm_dsd": (c_int, [*_mat, *_mat, *_mat, *_mat, c_int64, c_int64, c_int64, c_int64,
                            c_float, c_int, c_void_p, c_int64, c_void_p]),
    "sd_noalloc_scratch_bytes": (c_int64, []),
    "sd_gemm_dsd_noalloc": (c_int, [*_mat, *_mat, *_mat, *_mat, c_int64, c_int64, c_int64, c_int64,
                                    c_float, c_int, c_void_p]),
    "sd_gemm_sdd": (c_int, [*_mat, *_mat, *_mat, *_mat, c_int64, c_int64, c_int64, c_int64,
                            c_float, c_int, c_void_p, c_int64, c_void_p]),
    "sd_gemm_dsd_lists": (c_int, [*_mat, *_mat, *_mat, c_void_p, c_void_p, c_int64, c_int64,
                                  c_int64, c_int64, c_float, c_int, c_void_p, c_int64, c_void_p]),
    "sd_gemm_sdd_lists": (c_int, [*_mat, *_mat, *_mat, c_void_p, c_void_p, c_int64, c_int64,
                                  c_int64, c_int64, c_float, c_int, c_void_p]),
    "sd_gemm_sdd_lists_ex": (c_int, [*_mat, *_mat, *_mat, c_void_p, c_void_p, c_int64, c_int64,
                                     c_int64, c_int64, c_float, c_int, c_int, c_float, c_void_p]),
    "sd_gemm_dsd_lists_act": (c_int, [*_mat, *_mat, *_mat, c_void_p, c_void_p, c_int64, c_int64, c_int64, c_int64,
                                      c_float, c_int, c_int, *_mat, c_void_p, c_int64, c_void_p]),
    "sd_gemm_sdd_lists_actgrad": (c_int, [*_mat, *_mat, *_mat, c_void_p, c_void_p, c_int64, c_int64, c_int64, c_int64,
                                          c_float, c_int, c_int, *_mat, c_float, c_void_p]),
    "sd_gemm_sdd_lists_kept": (c_int, [*_mat, *_mat, *_mat, c_void_p, c_void_p, c_int64, c_int64,
                                  c_int64, c_int64, c_float, c_int, c_void_p]),
    "sd_dropout_matmul_forward": (c_int, [*_mat, *_mat, *_mat, *_mat, c_void_p, c_uint64, c_uint64, c_double, c_void_p,
                                          c_void_p, c_void_p, c_void_p, c_void_p, c_int64, c_int64, c_int64, c_int64,
                                          c_int, c_void_p, c_int64, c_void_p]),
    "sd_dropout_matmul_forward_act": (c_int, [*_mat, *_mat, *_mat, *_mat, c_void_p, c_uint64, c_uint64, c_double,
                                              c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int64, c_int64,
                                              c_int64, c_int64, c_int, c_int, *_mat, c_void_p, c_int64, c_void_p]),
    "sd_gemm_act": (c_int, [*_mat, *_mat, *_mat, c_int64, c_int64, c_int64, c_int, c_int, *_mat, c_void_p, c_int64,
                            c_void_p]),
    "sd_dropout_matmul_backward": (c_int, [*_mat, *_mat, *_mat, *_mat, *_mat, c_void_p, c_void_p, c_void_p, c_void_p,
                                           c_int64, c_int64, c_int64, c_int64, c_double, c_int, c_void_p, c_int64,
                                           c_void_p]),
    "sd_dropout_matmul_backward_act": (c_int, [*_mat, *_mat, *_mat, *_mat, *_mat, c_void_p, c_void_p, c_void_p,
                                               c_void_p, c_int64, c_int64, c_int64, c_int64, c_double, c_int,
                                               c_int, *_mat, c_void_p, c_int64, c_void_p]),
    "sd_conv2d_dsd_lists": (c_int, [c_void_p, c_int64, c_int64, c_int64, c_int64, c_void_p, c_int64, c_void_p, c_int64,
                                    c_int64, c_int64, c_int64, c_int64, c_int64, c_int64, c_int64,
                                    c_int64, c_int64, c_int64, c_int64, c_int64, c_int64,
                                    c_void_p, c_void_p, c_int64, c_float, c_int, c_void_p]),
    "sd_conv2d_dx": (c_int, [c_void_p, c_int64, c_void_p, c_int64, c_void_p, c_int64, c_int64, c_int64, c_int64,
                             c_void_p, c_int64, c_int64,
                             c_int64, c_int64, c_int64, c_int64, c_int64, c_int64, c_int64,
                             c_int64, c_int64, c_int64, c_int64, c_int64, c_int64,
                             c_int64, c_float, c_int, c_void_p]),
    "sd_conv2d_dw_workspace_bytes": (c_int64, [c_int64] * 7),
    "sd_conv2d_dw_lists": (c_int, [c_void_p, c_int64, c_int64, c_int64, c_int64, c_void_p, c_int64, c_void_p, c_int64,
                                   c_int64, c_int64, c_int64, c_int64, c_int64, c_int64, c_int64,
                                   c_int64, c_int64, c_int64, c_int64, c_int64, c_int64,
                                   c_void_p, c_void_p, c_int64, c_float, c_int, c_void_p, c_int64, c_void_p]),
    "sd_im2col": (c_int, [c_void_p, c_int64, c_int64, c_int64, c_int64, c_void_p, c_int64,
                          *([c_int64] * 12), c_void_p, c_void_p, c_int64, c_int, c_void_p]),
    "sd_col2im": (c_int, [c_void_p, c_int64, c_void_p, c_int64, c_int64, c_int64, c_int64,
                          *([c_int64] * 12), c_void_p, c_int64, c_int64, c_int64, c_int, c_void_p]),
}


def source_hash() -> str | None:
    """Hash of the sources the library is built from (the same function as build.py's), or None when the
    sources are not there (an installed library without its source tree)."""
    csrc = LIB_PATH.parent.parent.parent / "csrc"
    include = csrc.parent.parent / "include"
    hips = sorted(csrc.glob("*.hip"))
    if not hips:
        return None
    files = [*hips, *sorted(csrc.glob("*.h")), *sorted(include.glob("*.h"))]
    h = hashlib.sha256()
    for f in files:
        h.update(f.name.encode())
        h.update(f.read_bytes())
    return h.hexdigest()[:16]


@lru_cache(maxsize=None)
def load() -> ctypes.CDLL:
    if not LIB_PATH.exists():
        raise RuntimeError(
            f"{LIB_PATH} not found: build it with `python sparse-dropout_amd/csrc/build.py` "
            "(hipcc, gfx950). There is no fallback implementation."
        )
    lib = ctypes.CDLL(str(LIB_PATH))
    for name, (res, args) in SIGNATURES.items():
        fn = getattr(lib, name)  # AttributeError here = header and library disagree
        fn.restype = res
        fn.argtypes = args
    built, now = lib.sd_source_hash().decode(), source_hash()
    if now is not None and built != now:
        raise RuntimeError(
            f"{LIB_PATH} was built from other sources (library {built}, tree {now}): rebuild it with "
            "`python sparse-dropout_amd/csrc/build.py`"
        )
    return lib
