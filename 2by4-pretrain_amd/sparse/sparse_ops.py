"""Linear modules built on the dense-shaped 2:4 operators.

    MyLinear, my_linear          plain linear as an autograd.Function          (sparse/sparse_ops.py:8-46)
    SparseLinear, sparse_linear  same forward; dX uses an MVUE24 estimate of W  (sparse/sparse_ops.py:49-87)
    SoftThreshold                S-STE: soft-thresholded 2:4 weight x scale,
                                 straight-through gradient                      (README.md:233-243)
    SoftThresholdLinear          nn.Linear on SoftThreshold with the frozen
                                 scale of README.md:245-266 (the README calls
                                 this class SparseLinear as well)
    Sparse24                     STE magnitude pruning of the STEP recipe       (README.md:286-295)

The matrix products are torch's dense ones, as in the reference: only the pruning operators run
this package's kernels.
"""
import torch
import torch.nn.functional as F
from torch import autograd, nn
from torch.amp import custom_bwd, custom_fwd

from .dense_ops import MVUE24_approx, soft_threshold24, sparse24

__all__ = ["MyLinear", "my_linear", "SparseLinear", "sparse_linear", "SoftThreshold", "SoftThresholdLinear", "Sparse24"]


def _forward(ctx, input, weight, bias):
    ctx.save_for_backward(input, weight, bias)
    ctx.shape = input.shape
    out = torch.mm(input.view(-1, input.shape[-1]), weight.t()).view(*input.shape[:-1], -1)
    return out if bias is None else out + bias


def _backward(ctx, grad_output, weight_for_dx):
    input, weight, bias = ctx.saved_tensors
    grad_input = grad_weight = grad_bias = None
    g2 = grad_output.reshape(-1, grad_output.shape[-1])
    if ctx.needs_input_grad[0]:
        grad_input = torch.mm(g2, weight_for_dx(weight)).view(ctx.shape)
    if ctx.needs_input_grad[1]:
        grad_weight = torch.mm(g2.t(), input.view(-1, input.shape[-1]))
    if ctx.needs_input_grad[2]:
        grad_bias = g2.sum(0)
    return grad_input, grad_weight, grad_bias


class my_linear(autograd.Function):
    @staticmethod
    @custom_fwd(device_type="cuda")
    def forward(ctx, input, weight, bias):
        return _forward(ctx, input, weight, bias)

    @staticmethod
    @custom_bwd(device_type="cuda")
    def backward(ctx, grad_output):
        return _backward(ctx, grad_output, lambda w: w)


class sparse_linear(autograd.Function):
    """dX = dY . MVUE24(W^T)^T: the weight is pruned 2:4 along its output axis, unbiasedly."""

    @staticmethod
    @custom_fwd(device_type="cuda")
    def forward(ctx, input, weight, bias):
        return _forward(ctx, input, weight, bias)

    @staticmethod
    @custom_bwd(device_type="cuda")
    def backward(ctx, grad_output):
        return _backward(ctx, grad_output, lambda w: MVUE24_approx(w.t()).t())


class MyLinear(nn.Linear):
    def forward(self, x):
        return my_linear.apply(x, self.weight, self.bias)


class SparseLinear(nn.Linear):
    def forward(self, x):
        return sparse_linear.apply(x, self.weight, self.bias)


class SoftThreshold(autograd.Function):
    @staticmethod
    def forward(ctx, weight, scale):
        weight_sparse, _ = soft_threshold24(weight.detach())
        return weight_sparse * scale

    @staticmethod
    def backward(ctx, grad_output):
        return grad_output, None


class SoftThresholdLinear(nn.Linear):
    def __init__(self, in_features: int, out_features: int, bias: bool = True, device=None, dtype=None):
        super().__init__(in_features, out_features, bias=bias, device=device, dtype=dtype)
        self.register_buffer("scale", torch.tensor(0.0))

    def get_sparse_weights(self):
        return SoftThreshold.apply(self.weight, self.scale)

    @torch.no_grad()
    def init_scale(self):
        """scale = <w, S(w)> / <S(w), S(w)>: the least-squares fit of scale * S(w) to w."""
        weight = self.weight.detach()
        weight_sparse, _ = soft_threshold24(weight)
        ws = torch.flatten(weight_sparse).float()
        scale = torch.dot(torch.flatten(weight).float(), ws) / torch.dot(ws, ws)
        self.scale.copy_(scale)
        self.weight.scale = self.scale

    def forward(self, x):
        return F.linear(x, self.get_sparse_weights(), self.bias)


class Sparse24(autograd.Function):
    @staticmethod
    def forward(ctx, weight):
        weight_sparse, _ = sparse24(weight)
        return weight_sparse

    @staticmethod
    def backward(ctx, grad_output):
        return grad_output
