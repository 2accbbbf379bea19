"""Oracle: the 2:4 sparse matmul, as a dense masked float32 product.

TEST INFRASTRUCTURE ONLY -- never imported by the shipped package.

The reference computes out[M,N] = input[M,K] . W_sparse^T (+ bias[N]) with float32 accumulation
(csrc/mySparseSemiStructuredLinear_cuda.cu:498-817, via CUTLASS SparseGemm).  CUTLASS is an
un-vendored submodule, so the GEMM's own rounding is not reproducible; the definition used
here is the mathematical one the task states: X.float() @ W_masked.float().T.
"""
import torch


def spmm_ref(x, w_masked_dense, bias=None):
    """x [M,K], w_masked_dense [N,K] (already pruned, zeros in place) -> float32 [M,N]."""
    out = x.float() @ w_masked_dense.float().t()
    if bias is not None:
        out = out + bias.float()
    return out


def linear_ref(x, w_masked_dense, bias=None):
    """N-d input variant (semi_structured.py:498-524)."""
    shape = x.shape
    return spmm_ref(x.reshape(-1, shape[-1]), w_masked_dense, bias).reshape(*shape[:-1], -1)


def spmm_ref_int(x, w_masked_dense, bias=None, relu=False):
    """The int8 product of the reference (.cu:594-637: int8 x int8, int32 accumulate, int32 bias and
    output, optional ReLU), evaluated exactly in int64.  x [M,K] int8, w_masked_dense [N,K] int8
    -> int32 [M,N]; raises if a result leaves the int32 range (the accumulator would wrap)."""
    out = x.long() @ w_masked_dense.long().t()
    if bias is not None:
        out = out + bias.long()
    if relu:
        out = out.clamp_min(0)
    if out.abs().max() >= 2 ** 31:
        raise RuntimeError("int32 accumulator overflow in the test data")
    return out.int()
