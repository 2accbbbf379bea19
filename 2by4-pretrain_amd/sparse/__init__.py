"""`sparse`: drop-in for the 2:4 sparse hot path of huyz2023/2by4-pretrain on MI355X (gfx950).

Same names as the reference package (sparse/__init__.py:1-25) for everything on the 2:4 path;
every operator runs a hand-written HIP kernel from lib2by4_gfx950.so and raises if that library
is missing -- there is no CPU or PyTorch fallback.
"""
from .semi_structured import (SparseSemiStructuredTensor, to_sparse_semi_structured, to_sparse_semi_structured_pair,
                              to_sparse_semi_structured_with_row_sums, mvue_device_state)
from .transposable_semi_structured import TransposableSparse, mask_select, transposable_mask_
from .decay import masked_add_
from .adamw import MaskedDecayAdamW
from .adamw_step import AdamW_STEP
from .dense_ops import (soft_threshold24, sparse24, MVUE24_approx,
                        soft_threshold24_triton, sparse24_triton, MVUE24_approx_triton,
                        soft_threshold24_torch, sparse24_torch, MVUE24_approx_torch)
from .sparse_linear_transpose import SparseLinearTranspose, sparse_linear_transpose
from .sparse_semi_structured_linear import sparse_semi_structured_linear
from .GELUglu import GELUglu, gelu_glu
from .sparse_ops import MyLinear, SparseLinear, SoftThreshold, SoftThresholdLinear, Sparse24

__all__ = [
    "SparseSemiStructuredTensor", "to_sparse_semi_structured", "to_sparse_semi_structured_pair",
    "to_sparse_semi_structured_with_row_sums", "mvue_device_state",
    "TransposableSparse", "mask_select", "transposable_mask_",
    "masked_add_", "MaskedDecayAdamW", "AdamW_STEP",
    "soft_threshold24", "sparse24", "MVUE24_approx",
    "soft_threshold24_triton", "sparse24_triton", "MVUE24_approx_triton",
    "soft_threshold24_torch", "sparse24_torch", "MVUE24_approx_torch",
    "SparseLinearTranspose", "sparse_linear_transpose",
    "sparse_semi_structured_linear",
    "GELUglu", "gelu_glu",
    "MyLinear", "SparseLinear", "SoftThreshold", "SoftThresholdLinear", "Sparse24",
]
