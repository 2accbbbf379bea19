"""sparse_semi_structured_linear: the matmul entry point behind the tensor dispatch.

The reference binds its CUTLASS kernel under this name
(sparse/sparse_semi_structured_linear.py:4-5 -> csrc/mySparseSemiStructuredLinear_cuda.cu:498):
    sparse_semi_structured_linear(input, weight, meta, bias_opt, activation_opt) -> input . W^T (+bias)
with `weight`/`meta` the compressed values and metadata.  Here `weight` may also be a
SparseSemiStructuredTensor (then `meta` is omitted), which keeps the operand in the panel layout
the fast kernel streams.  Extra keywords: `out_dtype` (fp8 operands: float32 default, bfloat16 or
float16 allowed) and `scale` (multiplies the float32 accumulator before bias/activation, e.g. the
product of the per-tensor dequantisation scales of fp8 operands).
"""
from typing import Optional

import torch

from . import _native as N
from .semi_structured import SparseSemiStructuredTensor, _spmm

__all__ = ["sparse_semi_structured_linear"]

_ACTIVATIONS = {None: N.ACT_NONE, "none": N.ACT_NONE, "relu": N.ACT_RELU, "silu": N.ACT_SILU, "gelu": N.ACT_GELU}


def sparse_semi_structured_linear(input: torch.Tensor, weight, meta: Optional[torch.Tensor] = None,
                                  bias: Optional[torch.Tensor] = None, activation: Optional[str] = None,
                                  out_dtype: Optional[torch.dtype] = None, scale: float = 1.0) -> torch.Tensor:
    if activation not in _ACTIVATIONS:
        raise RuntimeError(f"activation {activation!r} is not supported (none, relu, silu, gelu)")
    if not isinstance(weight, SparseSemiStructuredTensor):
        if meta is None:
            raise RuntimeError("sparse_semi_structured_linear: metadata tensor missing")
        m, half = weight.shape
        weight = SparseSemiStructuredTensor(None, original_shape=torch.Size([m, 2 * half]), sparse_tensor_cutlass=weight,
                                            meta_tensor_cutlass=meta, dtype=weight.dtype)
    shape = input.shape
    x2d = input.reshape(-1, shape[-1])
    rows = x2d.shape[0]
    padded = weight._pad_tensor_for_matmul(x2d)
    if out_dtype is None:
        out_dtype = weight._out_dtype()
    out = _spmm(weight, padded, False, bias=bias, out_dtype=out_dtype, scale=scale, activation=_ACTIVATIONS[activation])
    return out[:rows].view(*shape[:-1], -1)
