"""masked_add_: fused masked decay (sparse/decay.py:27-37 of huyz2023/2by4-pretrain).

Equivalent to grad.add_(p_data * (1 - p_mask), alpha=alpha): where the mask is zero the gradient
receives alpha * p, elsewhere it is untouched.  In place, returns None.
"""
import torch

from . import _native as N

__all__ = ["masked_add_"]


def masked_add_(grad: torch.Tensor, p_data: torch.Tensor, p_mask: torch.Tensor, alpha: float = 0):
    assert grad.is_cuda and p_data.is_cuda and p_mask.is_cuda
    assert (grad.layout, p_data.layout, p_mask.layout) == (torch.strided, torch.strided, torch.strided)
    assert grad.stride() == p_data.stride() == p_mask.stride()
    n = grad.numel()
    if n == 0:
        return
    # like the reference kernel, storage is indexed linearly: the tensors must cover it densely
    dense_in_memory = grad.is_contiguous() or (grad.dim() == 2 and grad.t().is_contiguous())
    if not dense_in_memory:
        raise RuntimeError("masked_add_: tensors must be dense in memory (contiguous in some dimension order)")
    N.check(N.lib().tf24_masked_add(grad.data_ptr(), N.dtype_code(grad.dtype), p_data.data_ptr(), N.dtype_code(p_data.dtype),
                                    p_mask.data_ptr(), N.dtype_code(p_mask.dtype), n, float(alpha), N.stream_ptr()))
