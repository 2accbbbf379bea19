"""GELUglu / gelu_glu: out = gelu_tanh(gate) * x for an input whose last dimension is [x | gate].

Mirror of the reference module (sparse/GELUglu.py:156-243): an autograd function over a 3-d input
and the nn.Module around it.  Inputs whose last dimension is contiguous take the row-major kernel
(:161-177); inputs stored with the last dimension strided (a transposed 2-d view: :178-197) take
the column-major one and, like the reference, return an output stored the same way.
"""
import torch
from torch import autograd

from . import _native as N

__all__ = ["GELUglu", "gelu_glu"]


def _as_2d(t):
    """(2-d view [rows, cols], layout, ld) the kernels can address, copying when neither
    dimension of the flattened tensor is contiguous."""
    t2 = t.reshape(-1, t.shape[-1])
    lay = N.layout_of(t2)
    if lay is None:
        t2 = t2.contiguous()
        lay = N.layout_of(t2)
    return t2, lay[0], lay[1]


def _ld(t, layout):
    return t.stride(0) if layout == N.ROW_MAJOR else t.stride(1)


def _empty_like_layout(rows, cols, layout, like):
    if layout == N.ROW_MAJOR:
        return torch.empty((rows, cols), dtype=like.dtype, device=like.device)
    return torch.empty((cols, rows), dtype=like.dtype, device=like.device).t()


class gelu_glu(autograd.Function):
    @staticmethod
    def forward(ctx, input):
        assert input.dim() == 3, 'input must be 3D'
        if not input.is_cuda:
            raise RuntimeError("gelu_glu: only CUDA tensors are supported")
        if input.shape[-1] % 2:
            raise RuntimeError(f"gelu_glu: the last dimension ({input.shape[-1]}) must be even")
        x2, layout, ld = _as_2d(input)
        rows, cols = x2.shape
        out = _empty_like_layout(rows, cols // 2, layout, x2)
        N.check(N.lib().tf24_gelu_glu_forward(x2.data_ptr(), N.dtype_code(x2.dtype), layout, ld, rows, cols,
                                              out.data_ptr(), _ld(out, layout), N.stream_ptr()))
        ctx.save_for_backward(x2)
        ctx.layout, ctx.shape = layout, input.shape
        return out.view(*input.shape[:-1], cols // 2)

    @staticmethod
    def backward(ctx, grad_output):
        assert grad_output.dim() == 3, 'grad_output must be 3D'
        (x2,) = ctx.saved_tensors
        layout = ctx.layout
        rows, cols = x2.shape
        go = grad_output.reshape(rows, cols // 2).to(x2.dtype)
        want = _empty_like_layout(rows, cols // 2, layout, x2)
        if go.stride() != want.stride():          # bring the gradient to the layout of the forward output
            want.copy_(go)
            go = want
        grad_in = _empty_like_layout(rows, cols, layout, x2)
        N.check(N.lib().tf24_gelu_glu_backward(go.data_ptr(), _ld(go, layout), x2.data_ptr(), N.dtype_code(x2.dtype), layout,
                                               _ld(x2, layout), rows, cols, grad_in.data_ptr(), _ld(grad_in, layout),
                                               N.stream_ptr()))
        return grad_in.view(ctx.shape)


class GELUglu(torch.nn.Module):
    def __init__(self):
        super().__init__()

    def forward(self, x):
        return gelu_glu.apply(x)
