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


# Panel-layout copies of operands that arrive as canonical (values, meta) tensors through the
# functional entry point: the tiled kernel streams the panel form only, and a fresh wrapper per call
# would repack (one full pass over the operand, two allocations) before every product.  Keyed on
# the storage identity of the two tensors; `_version` catches in-place updates.  A handful of
# entries: a caller alternates between a few weights at most.
_PANEL_CACHE = {}
_PANEL_CACHE_ENTRIES = 8


def _wrapper_for(values, meta):
    key = (values.data_ptr(), meta.data_ptr(), tuple(values.shape), values.dtype)
    stamp = (values._version, meta._version)
    hit = _PANEL_CACHE.get(key)
    if hit is not None and hit[0] == stamp:
        return hit[1]
    m, half = values.shape
    wrapper = SparseSemiStructuredTensor(None, original_shape=torch.Size([m, 2 * half]), sparse_tensor_cutlass=values,
                                         meta_tensor_cutlass=meta, dtype=values.dtype)
    if len(_PANEL_CACHE) >= _PANEL_CACHE_ENTRIES:
        _PANEL_CACHE.pop(next(iter(_PANEL_CACHE)))
    # the entry holds the tensors themselves, so their addresses cannot be reused while it lives
    _PANEL_CACHE[key] = (stamp, wrapper, values, meta)
    return wrapper


def sparse_semi_structured_linear(input: torch.Tensor, weight, meta: Optional[torch.Tensor] = None,
                                  bias_opt: Optional[torch.Tensor] = None, activation_opt: Optional[str] = None,
                                  out_dtype: Optional[torch.dtype] = None, scale: float = 1.0,
                                  bias: Optional[torch.Tensor] = None, activation: Optional[str] = None) -> torch.Tensor:
    """Positional order and the keywords `bias_opt` / `activation_opt` are the reference's
    (sparse_semi_structured_linear.py:4); `bias` / `activation` are accepted as well, because the
    reference's own dispatch calls the function with `bias=` (semi_structured.py:433-438, :510-515)."""
    if bias is not None:
        if bias_opt is not None:
            raise TypeError("sparse_semi_structured_linear: both bias_opt and bias given")
        bias_opt = bias
    if activation is not None:
        if activation_opt is not None:
            raise TypeError("sparse_semi_structured_linear: both activation_opt and activation given")
        activation_opt = activation
    if activation_opt not in _ACTIVATIONS:
        raise RuntimeError(f"activation {activation_opt!r} is not supported (none, relu, silu, gelu)")
    if not isinstance(weight, SparseSemiStructuredTensor):
        if meta is None:
            raise RuntimeError("sparse_semi_structured_linear: metadata tensor missing")
        weight = _wrapper_for(weight, meta)
    shape = input.shape
    x2d = input.reshape(-1, shape[-1])
    rows = x2d.shape[0]
    padded = weight._pad_tensor_for_matmul(x2d)
    if out_dtype is None:
        out_dtype = weight._out_dtype()
    out = _spmm(weight, padded, False, bias=bias_opt, out_dtype=out_dtype, scale=scale, activation=_ACTIVATIONS[activation_opt])
    return out[:rows].view(*shape[:-1], -1)
