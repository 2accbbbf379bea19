"""Dense-shaped 2:4 operators (sparse/triton_ops.py of huyz2023/2by4-pretrain), on HIP kernels.

    soft_threshold24(dense)        -> (sparse, mask)   S-STE soft threshold   (triton_ops.py:198-227)
    sparse24(dense)                -> (sparse, mask)   magnitude pruning      (triton_ops.py:125-154)
    MVUE24_approx(dense, rand=None)-> sparse           MVUE24 estimator       (triton_ops.py:55-81)

Outputs have the input's shape, dtype and strides; the mask is returned in the dense dtype
(1.0 / 0.0), as the reference does.  The reference's `*_triton` names are kept as aliases.

The reference's `*_torch` forms (sparse/legacy.py:26-40, :96-117, :227-268: the same three operators
written with argsort / multinomial over the flattened tensor, any shape, int32 mask) are kept as
names on top of the same kernels: the tensor is viewed as rows of its last dimension, groups of 4
run along the flattened storage exactly as `reshape(group, 4)` cuts them.
"""
import torch

from . import _native as N

__all__ = ["soft_threshold24", "sparse24", "MVUE24_approx",
           "soft_threshold24_triton", "sparse24_triton", "MVUE24_approx_triton",
           "soft_threshold24_torch", "sparse24_torch", "MVUE24_approx_torch"]


def _prepare(dense):
    if dense.dim() != 2:
        raise RuntimeError(f"Expected 2-dimensional dense tensor, got {dense.dim()}-dimensional tensor")
    if not dense.is_cuda:
        raise RuntimeError(f"Expected a GPU tensor, got device {dense.device}")
    if dense.dtype not in (torch.float16, torch.bfloat16, torch.float32):
        raise RuntimeError(f"Invalid datatype {dense.dtype} of dense matrix")
    src = N.as_matrix(dense)
    layout, ld = N.layout_of(src)
    return src, layout, ld


def _like(src, dtype=None):
    return torch.empty_strided(src.shape, src.stride(), dtype=dtype or src.dtype, device=src.device)


def soft_threshold24(dense):
    src, layout, ld = _prepare(dense)
    m, k = src.shape
    sparse, mask = _like(src), _like(src)
    N.check(N.lib().tf24_soft_threshold24(src.data_ptr(), N.dtype_code(src.dtype), layout, ld, m, k,
                                          sparse.data_ptr(), mask.data_ptr(), N.stream_ptr()))
    return sparse, mask


def sparse24(dense):
    src, layout, ld = _prepare(dense)
    m, k = src.shape
    sparse, mask = _like(src), _like(src)
    N.check(N.lib().tf24_sparse24_dense(src.data_ptr(), N.dtype_code(src.dtype), layout, ld, m, k,
                                        sparse.data_ptr(), mask.data_ptr(), N.stream_ptr()))
    return sparse, mask


def MVUE24_approx(dense, rand=None):
    src, layout, ld = _prepare(dense)
    m, k = src.shape
    if rand is None:
        rand = _like(src, torch.float32).uniform_()
    rand = N.as_matrix(rand.float(), like=src)
    sparse = _like(src)
    N.check(N.lib().tf24_mvue24_dense(src.data_ptr(), N.dtype_code(src.dtype), layout, ld, m, k,
                                      rand.data_ptr(), N.layout_of(rand)[1], sparse.data_ptr(), N.stream_ptr()))
    return sparse


soft_threshold24_triton = soft_threshold24
sparse24_triton = sparse24
MVUE24_approx_triton = MVUE24_approx


def _as_rows(weight):
    """Contiguous 2-d view [rows, cols] of a tensor of any shape whose groups of 4 along the flattened
    storage are the groups of 4 along cols."""
    if weight.numel() % 8:
        raise RuntimeError(f"number of elements {weight.numel()} must be a multiple of 8")
    flat = weight.contiguous()
    cols = flat.shape[-1] if flat.dim() >= 2 and flat.shape[-1] % 8 == 0 else 8
    return flat.view(-1, cols)


def sparse24_torch(weight):
    """legacy.py:26-40: (weight * mask, mask) with an int32 mask of weight's shape."""
    sparse, mask = sparse24(_as_rows(weight))
    return sparse.view(weight.shape), mask.view(weight.shape).to(torch.int32)


def soft_threshold24_torch(weight):
    """legacy.py:96-117: (soft-thresholded weight, int32 mask)."""
    sparse, mask = soft_threshold24(_as_rows(weight))
    return sparse.view(weight.shape), mask.view(weight.shape).to(torch.int32)


def MVUE24_approx_torch(weight, rand=None):
    """legacy.py:227-268: the MVUE24 estimate of weight, same shape."""
    rows = _as_rows(weight)
    if rand is not None:
        rand = rand.contiguous().view(rows.shape)
    return MVUE24_approx(rows, rand).view(weight.shape)
