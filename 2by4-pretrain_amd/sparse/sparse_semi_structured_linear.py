"""sparse_semi_structured_linear: the matmul entry point behind the tensor dispatch.

The reference binds its CUTLASS kernel under this name
(sparse/sparse_semi_structured_linear.py:4-5 -> csrc/mySparseSemiStructuredLinear_cuda.cu:498):
    sparse_semi_structured_linear(input, weight, meta, bias_opt, activation_opt) -> input . W^T (+bias)
with `weight`/`meta` the compressed values and metadata.  Here `weight` may also be a
SparseSemiStructuredTensor (then `meta` is omitted), which keeps the operand in the panel layout
the fast kernel streams; a raw (weight, meta) pair is repacked to that layout on every call.  Extra keywords: `out_dtype` (fp8 operands: float32 default, bfloat16 or
float16 allowed) and `scale` (multiplies the float32 accumulator before bias/activation, e.g. the
product of the per-tensor dequantisation scales of fp8 operands).
"""
from typing import Optional

import torch

from . import _native as N
from .semi_structured import SparseSemiStructuredTensor, _spmm

__all__ = ["sparse_semi_structured_linear"]

_ACTIVATIONS = {None: N.ACT_NONE, "none": N.ACT_NONE, "relu": N.ACT_RELU, "silu": N.ACT_SILU, "gelu": N.ACT_GELU}


_META_LAYOUTS = {"canonical": N.COMPRESSED_CANONICAL, "cutlass": N.COMPRESSED_CUTLASS}


def _borrowed_wrapper(values, meta, meta_layout):
    """A wrapper around the caller's (values, meta) tensors for one product.  Nothing is memoised across
    calls: the caller may rewrite the tensors in ways no version counter records (`.data`, kernels that
    write through raw pointers, graph replays), so the panel copy the fast kernel streams is made per
    call.  A caller who multiplies by the same operand repeatedly passes a SparseSemiStructuredTensor,
    which owns its storage and keeps the panel copy."""
    if meta_layout is None:
        layout = N.COMPRESSED_CUTLASS if SparseSemiStructuredTensor._CUTLASS_METADATA else N.COMPRESSED_CANONICAL
    elif meta_layout in _META_LAYOUTS:
        layout = _META_LAYOUTS[meta_layout]
    else:
        raise RuntimeError(f"meta_layout {meta_layout!r} is not supported (canonical, cutlass)")
    m, half = values.shape
    wrapper = SparseSemiStructuredTensor(None, original_shape=torch.Size([m, 2 * half]), sparse_tensor_cutlass=values,
                                         meta_tensor_cutlass=meta, dtype=values.dtype)
    wrapper._set_storage(values.contiguous().view(-1), meta.contiguous().view(-1), (m, 2 * half), layout)
    return wrapper


def sparse_semi_structured_linear(input: torch.Tensor, weight, meta: Optional[torch.Tensor] = None,
                                  bias_opt: Optional[torch.Tensor] = None, activation_opt: Optional[str] = None,
                                  out_dtype: Optional[torch.dtype] = None, scale: float = 1.0,
                                  bias: Optional[torch.Tensor] = None, activation: Optional[str] = None,
                                  meta_layout: Optional[str] = None) -> torch.Tensor:
    """Positional order and the keywords `bias_opt` / `activation_opt` are the reference's
    (sparse_semi_structured_linear.py:4); `bias` / `activation` are accepted as well, because the
    reference's own dispatch calls the function with `bias=` (semi_structured.py:433-438, :510-515).
    `meta_layout` says how a `meta` tensor is ordered: "cutlass" = the reference's reordered words (what
    its binding takes, csrc .cu:826-851), "canonical" = the plain nibble stream; default: the class flag
    SparseSemiStructuredTensor._CUTLASS_METADATA."""
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
    borrowed = False
    if not isinstance(weight, SparseSemiStructuredTensor):
        if meta is None:
            raise RuntimeError("sparse_semi_structured_linear: metadata tensor missing")
        weight = _borrowed_wrapper(weight, meta, meta_layout)
        borrowed = True
    shape = input.shape
    x2d = input.reshape(-1, shape[-1])
    rows = x2d.shape[0]
    padded = weight._pad_tensor_for_matmul(x2d)
    if out_dtype is None:
        out_dtype = weight._out_dtype()
    out = _spmm(weight, padded, False, bias=bias_opt, out_dtype=out_dtype, scale=scale, activation=_ACTIVATIONS[activation_opt],
                keep_panel=not borrowed)
    return out[:rows].view(*shape[:-1], -1)
