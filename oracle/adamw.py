"""Oracle: AdamW step preceded by the masked decay.

TEST INFRASTRUCTURE ONLY -- never imported by the shipped package.

Follows sparse/adamw.py:70-113 (p *= 1 - lr*wd; exp_avg = exp_avg*b1 + (1-b1)*g;
exp_avg_sq = exp_avg_sq*b2 + (1-b2)*g*g; denom = sqrt(exp_avg_sq)/sqrt(bc2) + eps;
p += -(lr/bc1) * exp_avg/denom) on a gradient that first received the decay term of
sparse/decay.py:27-37 (README.md:205-213).  float32 tensor arithmetic with Python-float scalars,
one torch operation per rounded step.

Pinned by: closed forms at step 1 (exp_avg = (1-b1)*g, exp_avg_sq = (1-b2)*g*g, so the update is
-lr * g / (|g| + eps*...) ~ -lr*sign(g)), equality with torch.optim.AdamW (an independent
implementation of the same algorithm) to float32 rounding over several steps, and the masked
decay's own vectors.  Tolerance-level parity: torch's in-place ops may contract multiply-adds.
"""
import math

import torch

from .decay import masked_add


def adamw_masked_decay(p, grad, exp_avg, exp_avg_sq, mask, step, lr=1e-3, betas=(0.9, 0.999), eps=1e-8,
                       weight_decay=1e-2, alpha=0.0):
    """Out-of-place: returns (p, exp_avg, exp_avg_sq) after update number `step` (>= 1)."""
    beta1, beta2 = betas
    g = grad.float()
    if mask is not None:
        g = masked_add(g, p, mask, alpha)
    p = p * (1 - lr * weight_decay)
    exp_avg = exp_avg * beta1 + (1 - beta1) * g
    exp_avg_sq = exp_avg_sq * beta2 + ((1 - beta2) * g) * g
    bc1, bc2 = 1 - beta1 ** step, 1 - beta2 ** step
    denom = exp_avg_sq.sqrt() / math.sqrt(bc2) + eps
    p = p + (-(lr / bc1)) * (exp_avg / denom)
    return p, exp_avg, exp_avg_sq
