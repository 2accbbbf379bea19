"""AdamW with the masked decay of the 2:4 recipe folded into the update (one HIP kernel per tensor).

The reference trains with its AdamW (sparse/adamw.py:9-115) after a loop that adds the decay term
to the gradients of masked weights (README.md:205-213):

    p.grad = p.grad.float(); masked_add_(p.grad.data, p.data, p.mask, alpha=alpha); p.cnt = 0

MaskedDecayAdamW does both in one pass per parameter: for a parameter that carries a `mask` and is
in 'sparse' mode the gradient seen by the update is grad + alpha * p where the mask is zero, then
the update of sparse/adamw.py:70-113 (decoupled weight decay, bias-corrected moments, no amsgrad).
The stored gradient is not modified; `cnt` is reset as the loop above does.  Parameters and moments
are float32; gradients may be float32, float16 or bfloat16.

capturable=True keeps every parameter's step count in device memory (an int64 tensor, advanced by a
device operation), as torch's own optimizers do under that name: a step recorded into a HIP graph then
replays with the count of the replay.  Hyper-parameters are read on the host at every call, so a
recording holds the values of its time.
"""
import torch
from torch.optim.optimizer import Optimizer

from . import _native as N

__all__ = ["MaskedDecayAdamW"]


class MaskedDecayAdamW(Optimizer):
    def __init__(self, params, lr=1e-3, betas=(0.9, 0.999), eps=1e-8, weight_decay=1e-2, alpha=0.0, capturable=False):
        if not 0.0 <= lr:
            raise ValueError("Invalid learning rate: {}".format(lr))
        if not 0.0 <= eps:
            raise ValueError("Invalid epsilon value: {}".format(eps))
        if not 0.0 <= betas[0] < 1.0:
            raise ValueError("Invalid beta parameter at index 0: {}".format(betas[0]))
        if not 0.0 <= betas[1] < 1.0:
            raise ValueError("Invalid beta parameter at index 1: {}".format(betas[1]))
        super().__init__(params, dict(lr=lr, betas=betas, eps=eps, weight_decay=weight_decay, alpha=alpha,
                                      capturable=bool(capturable)))

    def _check(self, p, capturable=False):
        """Once per parameter: what the kernel assumes about it (flat float32 storage shared by the moments)."""
        if p.dtype != torch.float32 or not p.is_cuda:
            raise RuntimeError("MaskedDecayAdamW: parameters must be float32 GPU tensors")
        if not (p.is_contiguous() or (p.dim() == 2 and p.t().is_contiguous())):
            raise RuntimeError("MaskedDecayAdamW: parameters must be dense in memory")
        state = self.state[p]
        state["step"] = torch.zeros((), dtype=torch.int64, device=p.device) if capturable else 0
        state["exp_avg"] = torch.zeros_like(p, memory_format=torch.preserve_format)
        state["exp_avg_sq"] = torch.zeros_like(p, memory_format=torch.preserve_format)
        return state

    @torch.no_grad()
    def step(self, closure=None):
        loss = None
        if closure is not None:
            with torch.enable_grad():
                loss = closure()
        host_step, device_step = N.lib().tf24_adamw_masked_decay, N.lib().tf24_adamw_masked_decay_device_step
        stream = N.stream_ptr()
        for group in self.param_groups:
            beta1, beta2 = group["betas"]
            lr, eps, wd, alpha = float(group["lr"]), float(group["eps"]), float(group["weight_decay"]), float(group["alpha"])
            for p in group["params"]:
                grad = p.grad
                if grad is None:
                    continue
                state = self.state[p]
                if not state:
                    state = self._check(p, group.get("capturable", False))
                if grad.is_sparse or grad.stride() != p.stride():
                    raise RuntimeError("MaskedDecayAdamW: the gradient must be dense with the parameter's strides")
                state["step"] += 1
                mask = getattr(p, "mask", None)
                mask_ptr, mask_code = None, N.U8
                if mask is not None and torch.is_tensor(mask) and getattr(p, "mode", "sparse") == "sparse":
                    if mask.stride() != p.stride() or mask.device != p.device:
                        raise RuntimeError("MaskedDecayAdamW: mask must have the parameter's strides and device")
                    mask_ptr, mask_code = mask.data_ptr(), N.dtype_code(mask.dtype)
                    p.cnt = 0
                on_device = torch.is_tensor(state["step"])
                N.check((device_step if on_device else host_step)(
                    p.data_ptr(), grad.data_ptr(), N.dtype_code(grad.dtype), state["exp_avg"].data_ptr(),
                    state["exp_avg_sq"].data_ptr(), mask_ptr, mask_code, p.numel(), lr, float(beta1), float(beta2),
                    eps, wd, alpha, state["step"].data_ptr() if on_device else state["step"], stream))
        return loss
