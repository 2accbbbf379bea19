"""Oracle: GELU-GLU forward and backward.

TEST INFRASTRUCTURE ONLY -- never imported by the shipped package.

Follows sparse/GELUglu.py: the input's last dimension holds [x | gate]; forward :29-43
(gate_cube, inner = beta*(gate + kappa*gate^3), tanh through exp :8-13, gate_gelu =
0.5*gate*(tanh + 1), out = gate_gelu * x), backward :104-119 (grad_x = grad_out * gate_gelu,
grad_gate = grad_out * x * (0.5*(1 + tanh) + 0.5*gate*(1 - tanh^2)*beta*(1 + 3*kappa*gate^2))).
Evaluated in float64 (the reference evaluates in the storage type; the GPU kernel in float32), so
parity is tolerance-level by construction.

Pinned by: forward equals torch.nn.functional.gelu(gate, approximate='tanh') * x (a library routine
for the same formula) and backward equals torch.autograd's gradient of that expression -- a wrong
sign, a dropped factor or swapped halves fails one of the two.
"""
import torch

BETA = 0.7978845608028654
KAPPA = 0.044715


def _tanh(v):
    neg = (torch.exp(v * 2) - 1) / (torch.exp(v * 2) + 1)
    pos = (1 - torch.exp(-2 * v)) / (1 + torch.exp(-2 * v))
    return torch.where(v > 0, pos, neg)


def gelu_glu_forward(inp):
    """inp [..., 2h] -> [..., h], float64."""
    v = inp.double()
    h = v.shape[-1] // 2
    x, gate = v[..., :h], v[..., h:]
    inner = BETA * (gate + KAPPA * gate * gate * gate)
    return 0.5 * gate * (_tanh(inner) + 1) * x


def gelu_glu_backward(grad_out, inp):
    """grad of gelu_glu_forward w.r.t. inp, float64 [..., 2h]."""
    v, go = inp.double(), grad_out.double()
    h = v.shape[-1] // 2
    x, gate = v[..., :h], v[..., h:]
    inner = BETA * (gate + KAPPA * gate * gate * gate)
    th = _tanh(inner)
    gate_gelu = 0.5 * gate * (th + 1)
    grad_x = go * gate_gelu
    grad_gate = (go * x) * (0.5 * (1 + th) + 0.5 * gate * (1 - th * th) * BETA * (1 + KAPPA * 3 * gate * gate))
    return torch.cat([grad_x, grad_gate], dim=-1)
