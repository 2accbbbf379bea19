"""SparseLinearTranspose / sparse_linear_transpose: 2:4 sparse training linear layer.

The reference defines these only in its README (README.md:125-200): an nn.Linear whose
weight carries a transposable 2:4 mask (refreshed every `freq` optimizer steps), two compressed
copies (W and W.T) rebuilt once per optimizer step, and an autograd function computing
    y  = x . W_sparse^T           (2:4 spMM)
    dX = dY . W_sparse_T^T        (2:4 spMM on the transposed copy)
    dW = MVUE24(dY^T) . x         (2:4 spMM with the gradient pruned along the token axis)
    db = sum(dY)
State lives as attributes on the weight Parameter, exactly as in the README: freq, cnt, counter,
step, mask, weight_sparse, weight_sparse_T, mode.
"""
import torch
import torch.nn.functional as F
from torch import autograd, nn

from .semi_structured import (SparseSemiStructuredTensor, _dense_times_sparse_t, _spmm, to_sparse_semi_structured,
                              to_sparse_semi_structured_pair, to_sparse_semi_structured_with_row_sums)
from .transposable_semi_structured import TransposableSparse, transposable_mask_

__all__ = ["SparseLinearTranspose", "sparse_linear_transpose"]


class sparse_linear_transpose(autograd.Function):
    """README.md:168-200.  The reference decorates forward with custom_fwd(cast_inputs=torch.float16): the
    arguments are cast and both passes run with autocast off.  That also casts the float32 master
    `weight` on every call although forward only uses its compressed copies; here the activations
    and the bias are cast to the compressed copies' dtype and `weight` is left alone.  dW leaves the
    matmul in the master weight's dtype instead of float16 followed by autograd's cast.  Neither pass
    enters an autocast context: every tensor operation in them is an explicit cast, a view or a call
    into the library, none of which autocast touches (three context managers per layer and step are
    12 us of host time; the one reduction that autocast would promote keeps its own guard)."""

    # True: a 3-d grad_output whose strides are all zero is replaced by ones, as the reference does
    # (README.md:186-187); False (default): its values are used
    ones_for_expanded_grad = False

    @staticmethod
    def forward(ctx, input, weight, weight_sparse, weight_sparse_T, bias):
        compute = weight_sparse.dtype
        if input.dtype != compute:
            input = input.to(compute)
        if bias is not None and bias.dtype != compute:
            bias = bias.to(compute)
        ctx.save_for_backward(input, weight_sparse_T, bias)
        shape = ctx.shape = input.shape
        ctx.weight_dtype = weight.dtype
        if len(shape) != 2:
            input = input.view(-1, shape[-1])
        # = torch.mm(input, weight_sparse.t()) / torch.addmm(bias, input, weight_sparse.t()) (README.md:176-179)
        # called directly; the bias is added in the matmul epilogue
        output = _dense_times_sparse_t(input, weight_sparse, bias)
        return output if len(shape) == 2 else output.view(*shape[:-1], -1)

    @staticmethod
    def backward(ctx, grad_output):
        input, weight_T, bias = ctx.saved_tensors
        grad_input = grad_weight = grad_bias = None
        # An expanded scalar gradient (all strides 0: the layer's output fed straight into .sum()) is
        # materialised with its values.  The reference replaces a 3-d one by ones (README.md:186-187), which
        # is the same thing after a plain .sum() and drops the factor when the sum is scaled (a loss scale,
        # a weight on the term); the class attribute `ones_for_expanded_grad` switches that behaviour on
        # for training scripts tuned against it.
        if sparse_linear_transpose.ones_for_expanded_grad and grad_output.dim() == 3 and grad_output.stride() == (0, 0, 0):
            grad_output = torch.ones_like(grad_output, memory_format=torch.contiguous_format)
        if grad_output.dim() != 2:
            grad_output = grad_output.reshape(-1, grad_output.shape[-1])
        if grad_output.stride(-1) != 1 or grad_output.stride(0) < grad_output.shape[-1]:
            grad_output = grad_output.contiguous()
        if grad_output.dtype != input.dtype:
            grad_output = grad_output.to(input.dtype)
        needs = ctx.needs_input_grad
        if needs[0]:
            grad_input = _dense_times_sparse_t(grad_output, weight_T)      # = torch.mm(grad_output, weight_T.t())
            if len(ctx.shape) != 2:
                grad_input = grad_input.view(ctx.shape)
        if needs[1]:
            if input.dim() != 2:
                input = input.view(-1, input.shape[-1])
            if needs[4]:
                # MVUE24(dY^T) and grad_bias = dY.sum(0) (README.md:193-197) from one read of dY
                grad_sparse, grad_bias = to_sparse_semi_structured_with_row_sums(grad_output.t(), MVUE24=True, dtype=grad_output.dtype)
            else:
                grad_sparse = to_sparse_semi_structured(grad_output.t(), MVUE24=True, dtype=grad_output.dtype)
            grad_weight = _spmm(grad_sparse, input, True, out_dtype=ctx.weight_dtype)
        elif needs[4]:
            with torch.autocast(device_type="cuda", enabled=False):      # (autocast would promote the sum to float32)
                grad_bias = grad_output.sum(0)
        return grad_input, grad_weight, None, None, grad_bias


class SparseLinearTranspose(nn.Linear):
    def __init__(self, in_features: int, out_features: int, bias: bool = True, func=lambda step: 'dense', **kwargs):
        super().__init__(in_features, out_features, bias=bias, **kwargs)
        self.weight.freq = 40      # mask refresh period, in optimizer steps
        self.weight.cnt = 0        # forward passes since the last optimizer step
        self.weight.counter = 0    # optimizer steps
        self.weight.step = 0       # forward passes in training mode
        self.weight.mask = torch.ones_like(self.weight, dtype=torch.bool)
        self.weight.weight_sparse = None
        self.weight.weight_sparse_T = None
        self.weight.mode = 'sparse'
        self.func = func
        self.transposable_sparse = TransposableSparse(abs=True)
        SparseSemiStructuredTensor._FORCE_CUTLASS = True

    def forward(self, x):
        w = self.weight
        if w.mode == 'dense':
            x = F.linear(x, w, self.bias)
        else:
            if w.mask.device != w.device:
                w.mask = w.mask.to(device=w.device)
            if w.counter % w.freq == 0 and w.cnt == 0:
                # = `_, w.mask = self.transposable_sparse(w)` (README.md:149-150) with the mask rewritten in place
                # where the buffer fits: whoever holds the tensor (the masked decay, a recorded graph) sees the
                # new mask, and the unused pruned copy of w is not written
                m = w.mask
                if (torch.is_tensor(m) and m.dtype == torch.bool and m.shape == w.shape and m.stride() == w.stride()
                        and m.device == w.device and w.is_contiguous() and w.data_ptr() % 16 == 0 and w.shape[1] % 8 == 0
                        and self.transposable_sparse.abs):
                    transposable_mask_(w.detach(), m, abs=True)
                else:
                    _, w.mask = self.transposable_sparse(w)
            if w.cnt == 0:
                # = to_sparse_semi_structured(w, mask=w.mask), to_sparse_semi_structured(w.T, mask=w.mask.T)
                # (README.md:165-166), from one read of w and the mask
                w.weight_sparse, w.weight_sparse_T = to_sparse_semi_structured_pair(w, w.mask, dtype=torch.float16)
            # (the README wraps this call in torch.autocast(dtype=float16) for the function's custom_fwd to cast its
            # arguments; the function here casts them itself, to the compressed copies' dtype)
            x = sparse_linear_transpose.apply(x, w, w.weight_sparse, w.weight_sparse_T, self.bias)
        if self.training:
            if w.cnt == 0:
                w.counter += 1
            w.step += 1
            w.cnt += 1
        return x
