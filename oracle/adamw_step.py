"""Oracle: the STEP optimizer's per-tensor update and its variance-change statistic.

TEST INFRASTRUCTURE ONLY -- never imported by the shipped package.

Follows sparse/adamw_step.py:84-148 (decay, moments, the two denominators, the parameter update)
and :124-129, :152-158 (variance change v_t - v_{t-1}; Z_t = mean|.| for option 1, exp(mean(log|.|))
for option 2).  float32 tensor arithmetic with Python-float scalars, one torch operation per rounded
step.  The phase logic (sliding window of length int(1/(1-beta2)), switch when its mean falls below
eps or the step count passes T_max, :159-194) is host code of the optimizer class and is tested there.

Pinned by: phase 1 equals torch.optim.AdamW (with and without amsgrad), an independent implementation;
phase 2 with eps = 0 and the frozen variance set to v_t / bc2 must give the same update as phase 1 with
eps = 0 (sqrt(v/bc2) = sqrt(v)/sqrt(bc2)); at step 1 from zero state the variance change is
(1 - beta2) * g^2, so Z_1 = (1 - beta2) * mean(g^2) (option 1) or (1 - beta2) * geometric mean of g^2
(option 2).  Tolerance-level parity: torch's in-place ops may contract multiply-adds.
"""
import math

import torch


def adamw_step_update(p, grad, exp_avg, exp_avg_sq, step, lr=1e-3, betas=(0.9, 0.999), eps=1e-8, weight_decay=1e-2,
                      max_exp_avg_sq=None, precond_variance=None):
    """Out-of-place: returns (p, exp_avg, exp_avg_sq, max_exp_avg_sq, variance_change)."""
    beta1, beta2 = betas
    g = grad.float()
    p = p * (1 - lr * weight_decay)
    exp_avg = exp_avg * beta1 + (1 - beta1) * g
    new_sq = exp_avg_sq * beta2 + ((1 - beta2) * g) * g
    change = new_sq - exp_avg_sq
    bc1, bc2 = 1 - beta1 ** step, 1 - beta2 ** step
    if precond_variance is not None:
        denom = precond_variance.sqrt() + math.sqrt(eps) * math.sqrt(math.sqrt(eps))
    elif max_exp_avg_sq is not None:
        max_exp_avg_sq = torch.maximum(max_exp_avg_sq, new_sq)
        denom = max_exp_avg_sq.sqrt() / math.sqrt(bc2) + eps
    else:
        denom = new_sq.sqrt() / math.sqrt(bc2) + eps
    p = p + (-(lr / bc1)) * (exp_avg / denom)
    return p, exp_avg, new_sq, max_exp_avg_sq, change


def variance_change_statistic(changes, option=1):
    """Z_t over the variance changes of all tracked tensors (float64 accumulation)."""
    flat = torch.cat([c.reshape(-1) for c in changes]).double().abs()
    if option == 1:
        return flat.mean().item()
    return math.exp(flat.log().mean().item()) if (flat > 0).all() else 0.0
