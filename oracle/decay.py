"""Oracle: masked decay.

TEST INFRASTRUCTURE ONLY -- never imported by the shipped package.

Follows sparse/decay.py:7-37: where mask == 0, grad += p * alpha; other elements untouched.
Evaluated in float32 as two rounded operations (product, then sum), no fused multiply-add,
and rounded once to grad's dtype.
"""
import torch


def masked_add(grad, p, mask, alpha=0.0):
    """Out-of-place restatement: returns the new grad (same dtype as grad)."""
    prod = p.float() * torch.tensor(alpha, dtype=torch.float32)
    new = (grad.float() + prod).to(grad.dtype)
    return torch.where(mask != 0, grad, new)
