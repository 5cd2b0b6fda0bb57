"""SparseDrop for MI355X: block-wise dropout fused into matmul, on hand-written gfx950 HIP kernels.

Same public surface as the reference ``flash_dropout`` package (``flash_dropout.functional``,
``flash_dropout.layers``); the kernels live in ``_lib/libsparsedrop.so`` behind a C ABI
(``include/sparsedrop.h``) and are reached through ``flash_dropout.hip.binding_gemm.GEMM``.
"""

__version__ = "0.1.0"
