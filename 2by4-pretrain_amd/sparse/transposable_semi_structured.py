"""TransposableSparse: transposable 2:4 mask search (mask valid for W and for W.T).

Mirrors sparse/transposable_semi_structured.py:97-200 of huyz2023/2by4-pretrain: a module whose
forward returns `(sparse, mask)` -- the pruned matrix and a bool mask -- choosing for every
aligned 4x4 block the first of the 90 row-and-column 2:4 patterns with the largest sum of
|entries| (entries when abs=False).  The pattern table is a closed form evaluated inside the HIP
kernel, so the module holds no table; `mask_pattern` is kept as a lazily built attribute for
code that inspects it.
"""
import itertools

import torch
from torch import Tensor, nn

from . import _native as N

__all__ = ["TransposableSparse", "mask_select", "transposable_mask_"]

_PAIRS = ((0, 1), (0, 2), (0, 3), (1, 2), (1, 3), (2, 3))


def _pattern_table():
    rows = []
    for qs in itertools.product(range(6), repeat=4):
        mat = [[1 if c in _PAIRS[q] else 0 for c in range(4)] for q in qs]
        if all(sum(mat[r][c] for r in range(4)) == 2 for c in range(4)):
            rows.append([b for row in mat for b in row])
    return torch.tensor(sorted(rows, reverse=True), dtype=torch.float32)


def _check_dense(dense: Tensor):
    if dense.dim() != 2:
        raise RuntimeError(f"Expected 2-dimensional dense tensor, got {dense.dim()}-dimensional tensor")
    if not dense.is_cuda:
        raise RuntimeError(f"Expected a GPU tensor, got device {dense.device}")
    m, k = dense.shape
    if dense.dtype not in (torch.float16, torch.bfloat16, torch.float32):
        raise RuntimeError(f"Invalid datatype {dense.dtype} of dense matrix")
    if m % 32 != 0:
        raise RuntimeError(f"Number rows columns of dense matrix {m} must be divisible by 32")
    if k % 64 != 0:
        raise RuntimeError(f"Number of columns of dense matrix {k} must be divisible by {64}")


def _to_transposable_sparse_semi_structured(dense: Tensor, abs: bool = True):
    _check_dense(dense)
    m, k = dense.shape
    src = N.as_matrix(dense)
    layout, ld = N.layout_of(src)
    sparse = torch.empty_strided(src.shape, src.stride(), dtype=src.dtype, device=src.device)
    mask = torch.empty_strided(src.shape, src.stride(), dtype=torch.bool, device=src.device)
    N.check(N.lib().tf24_transposable_mask(src.data_ptr(), N.dtype_code(src.dtype), layout, ld, m, k, int(bool(abs)),
                                           sparse.data_ptr(), mask.data_ptr(), N.stream_ptr()))
    return sparse, mask


def transposable_mask_(dense: Tensor, mask: Tensor, abs: bool = True) -> Tensor:
    """The transposable mask of `dense` written INTO `mask` (bool, same shape, strides and device); the pruned
    matrix is not produced.  What a training layer needs at a mask refresh: the buffer every other user of
    the mask already points to (the compression of W and W^T, the masked decay, a recorded HIP graph) is
    updated in place, and the 2 bytes per element of the `sparse` output are never written."""
    _check_dense(dense)
    if (mask.dtype != torch.bool or mask.shape != dense.shape or mask.device != dense.device or mask.stride() != dense.stride()
            or N.layout_of(dense) is None or dense.data_ptr() % 16 or N.layout_of(dense)[1] % 8):
        raise RuntimeError("transposable_mask_: mask must be a bool tensor with the shape, strides and device of a dense "
                           "row- or column-major matrix (16-byte aligned, leading dimension a multiple of 8)")
    m, k = dense.shape
    layout, ld = N.layout_of(dense)
    N.check(N.lib().tf24_transposable_mask(dense.data_ptr(), N.dtype_code(dense.dtype), layout, ld, m, k, int(bool(abs)),
                                           None, mask.data_ptr(), N.stream_ptr()))
    return mask


class TransposableSparse(nn.Module):
    r"""
    :return sparse, mask
    """

    def __init__(self, abs: bool = True):
        super().__init__()
        self.abs = abs
        self._mask_pattern = None

    @property
    def mask_pattern(self):
        if self._mask_pattern is None:
            self._mask_pattern = _pattern_table()
        return self._mask_pattern

    def forward(self, x: Tensor):
        return _to_transposable_sparse_semi_structured(x, self.abs)


def mask_select(x: Tensor, abs: bool = True):
    """Functional form: (sparse, mask) of the transposable search."""
    return _to_transposable_sparse_semi_structured(x, abs)
