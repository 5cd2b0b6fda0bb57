from .binding_gemm import GEMM, KeptLists, SparseDropError  # noqa: F401
