"""Public functional API.  The five names of the reference (flash_dropout/functional/__init__.py:1-9)
are kept; ``cuda_blockwise_dropout_matmul`` and ``triton_blockwise_dropout_matmul`` both resolve to
the HIP implementation (there is one kernel backend here, not three)."""
from .blockwise_dropout_matmul_hip import blockwise_dropout_matmul as hip_blockwise_dropout_matmul
from .blockwise_dropout_matmul_hip import blockwise_dropout_matmul_mask as hip_blockwise_dropout_matmul_mask
from .blockwise_dropout_mlp_hip import blockwise_dropout_mlp as hip_blockwise_dropout_mlp
from .im2col_conv2d import (
    blockwise_dropout_conv2d,
    blockwise_dropout_conv2d_mask,
    conv_last_routes,
    conv_patch_matrix_shape,
    im2col_conv2d,
    naive_blockwise_dropout_conv2d,
    naive_blockwise_dropout_conv2d_mask,
)
from .naive import blockwise_dropout_matmul as naive_blockwise_dropout_matmul
from .naive import blockwise_dropout_matmul_mask as naive_blockwise_dropout_matmul_mask
from .utils import blockwise_dropout_mask, kept_block_lists, kept_block_table, mask_to_increment_table
from .vanilla import dropout_matmul as vanilla_dropout_matmul

cuda_blockwise_dropout_matmul = hip_blockwise_dropout_matmul
triton_blockwise_dropout_matmul = hip_blockwise_dropout_matmul
