"""Oracle: MVUE24 (minimum-variance unbiased 2:4 estimator) driven by a supplied U(0,1) tensor.

TEST INFRASTRUCTURE ONLY -- never imported by the shipped package.

Follows sparse/utils.py:5-59 (= _semi_structured_conversions.py:374-428) operation by
operation, in float32, in the written order.  The reference draws its two uniforms per
group from an in-kernel philox stream seeded by Python's `random`
(_semi_structured_conversions.py:536-542, :1076), which cannot be reproduced; here group g
of row r takes r0 = U[r, 4g] and r1 = U[r, 4g+1] from a caller-supplied tensor of the dense
shape.
"""
import torch

from .semi_structured import _groups, compress24

_EPS = 1.19209e-07  # utils.py:7, rounded to float32 when used


def _terms(dense):
    x = _groups(dense.float())
    eps = torch.tensor(_EPS, dtype=torch.float32)
    a = x.abs() + eps                                   # a_i
    a0, a1, a2, a3 = a.unbind(-1)
    total = ((a0 + a1) + a2) + a3                       # utils.py:12
    t = a / total.unsqueeze(-1)                         # t_i
    s = total.unsqueeze(-1) - a                         # s_i
    kk = t / s                                          # k_i
    k0, k1, k2, k3 = kk.unbind(-1)
    ksum = ((k0 + k1) + k2) + k3
    p = t + a * (ksum.unsqueeze(-1) - kk)               # p_i, utils.py:31-34 (mul then add)
    return x, a, t, p


def mvue24_probabilities(dense):
    """Inclusion probabilities p_i [m, k] float32 (sum to 2 within each group)."""
    _, _, _, p = _terms(dense)
    return p.reshape(dense.shape)


def _mvue(dense, rand):
    x, a, t, p = _terms(dense)
    u = _groups(rand.float())
    r0, r1 = u[..., 0], u[..., 1]
    t0, t1, t2, _ = t.unbind(-1)
    a0, a1, a2, a3 = a.unbind(-1)
    m0 = r0 <= t0
    m1 = (r0 <= (t0 + t1)) & ~m0
    m2 = (r0 <= ((t0 + t1) + t2)) & ~m1 & ~m0
    m3 = ~m2 & ~m1 & ~m0
    zero = torch.zeros((), dtype=torch.float32)
    d0 = torch.where(m0, zero, a0)                      # utils.py:41-44: (~m) * a
    d1 = torch.where(m1, zero, a1)
    d2 = torch.where(m2, zero, a2)
    d3 = torch.where(m3, zero, a3)
    dsum = ((d0 + d1) + d2) + d3
    tt = r1 * dsum
    e0 = tt <= d0
    e1 = (tt <= (d0 + d1)) & ~e0
    e2 = (tt <= ((d0 + d1) + d2)) & ~e1 & ~e0
    e3 = ~e2 & ~e1 & ~e0
    mask = torch.stack((m0 | e0, m1 | e1, m2 | e2, m3 | e3), dim=-1)
    scaled = x / p                                      # utils.py:54-57
    return scaled.reshape(dense.shape), mask.reshape(dense.shape)


def mvue24(dense, rand, out_dtype=torch.float16):
    """MVUE-prune and compress: (values [m,k/2] out_dtype, canonical meta, mask bool [m,k]).

    The kept value is x_i / p_i in float32, rounded once to out_dtype; encoding is the same
    nibble scheme as the magnitude path (_semi_structured_conversions.py:534-604).
    """
    scaled, mask = _mvue(dense, rand)
    values, meta = compress24(dense, mask=mask, out_dtype=out_dtype, source=scaled)
    return values, meta, mask


def mvue24_dense(dense, rand):
    """Dense-shaped twin (triton_ops.py:10-81): rescaled kept values, zeros elsewhere, in the
    dense dtype."""
    scaled, mask = _mvue(dense, rand)
    return torch.where(mask, scaled, torch.zeros_like(scaled)).to(dense.dtype)
