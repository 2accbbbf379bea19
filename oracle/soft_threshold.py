"""Oracle: S-STE soft threshold on 2:4 groups.

TEST INFRASTRUCTURE ONLY -- never imported by the shipped package.

Follows sparse/utils.py:72-90 (`_soft_threshold`) and the wrapper sparse/triton_ops.py:157-227:
magnitude mask, threshold = second smallest |a| of the group (the min/max network of
utils.py:83-84), kept values shrunk towards zero by the threshold, outputs dense-shaped and
pre-zeroed with only kept positions written, the mask in the dense dtype.
Arithmetic is float32 on upcast inputs, rounded once to the dense dtype.
"""
import torch

from .semi_structured import _groups, prune24_mask


def soft_threshold24(dense):
    """Returns (sparse, mask), both of dense's shape and dtype."""
    a = _groups(dense.float())
    a0, a1, a2, a3 = a.abs().unbind(-1)
    thr = torch.minimum(
        torch.maximum(torch.minimum(a0, a1), torch.minimum(a2, a3)),
        torch.minimum(torch.maximum(a0, a1), torch.maximum(a2, a3)),
    ).unsqueeze(-1)
    shrunk = torch.where(a > 0, a - thr, a + thr).reshape(dense.shape)
    mask = prune24_mask(dense)
    sparse = torch.where(mask, shrunk, torch.zeros_like(shrunk)).to(dense.dtype)
    return sparse, mask.to(dense.dtype)
