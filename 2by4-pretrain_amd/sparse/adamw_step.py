"""AdamW_STEP: the optimizer of the STEP recipe (learn 2:4 masks after a preconditioning phase).

Mirror of the reference class (sparse/adamw_step.py:9-213; used as in README.md:271-329): phase 1
is AdamW on dense weights while the change of the second moment is watched; when its windowed mean
Z falls below eps -- or the step count passes T_max -- every parameter that carries a `mask`
attribute ('dense' / 'sparse', a string here, unlike the boolean mask of the 2:4 layers) is switched
to 'sparse', its second moment is frozen as `preconditioned_variance`, and phase 2 divides by that
frozen variance instead.  Same constructor, attributes (`mask`, `sliding_window`, `T_omega`, `eps`,
`T_min`, `T_max`, `t`, `option`) and state keys; one HIP kernel per tensor does the whole update and
leaves the variance-change terms as per-block partial sums, so `exp_avg_sq_last` is never
materialised (the state key exists, as an empty tensor, for code that lists the keys).
"""
import math

import torch
from torch.optim.optimizer import Optimizer

from . import _native as N

__all__ = ["AdamW_STEP"]


class AdamW_STEP(Optimizer):
    def __init__(self, params, lr=1e-3, betas=(0.9, 0.999), eps=1e-8, weight_decay=1e-2, amsgrad=False,
                 clipping=(None, None), option=1):
        if not 0.0 <= lr:
            raise ValueError("Invalid learning rate: {}".format(lr))
        if not 0.0 <= eps:
            raise ValueError("Invalid epsilon value: {}".format(eps))
        if not 0.0 <= betas[0] < 1.0:
            raise ValueError("Invalid beta parameter at index 0: {}".format(betas[0]))
        if not 0.0 <= betas[1] < 1.0:
            raise ValueError("Invalid beta parameter at index 1: {}".format(betas[1]))
        if option not in [1, 2]:
            raise ValueError("Invalid option: {}".format(option))
        super().__init__(params, dict(lr=lr, betas=betas, eps=eps, weight_decay=weight_decay, amsgrad=amsgrad))
        self.mask = 'dense'
        self.sliding_window = []
        self.T_omega = int(1 / (1 - betas[1]))
        self.eps = eps
        self.T_min, self.T_max = clipping
        self.t = 0
        self.option = option

    def __setstate__(self, state):
        super().__setstate__(state)
        for group in self.param_groups:
            group.setdefault('amsgrad', False)

    def _init_state(self, p, amsgrad):
        if p.dtype != torch.float32 or not p.is_cuda:
            raise RuntimeError("AdamW_STEP: parameters must be float32 GPU tensors")
        if not (p.is_contiguous() or (p.dim() == 2 and p.t().is_contiguous())):
            raise RuntimeError("AdamW_STEP: parameters must be dense in memory")
        state = self.state[p]
        state['step'] = 0
        state['exp_avg'] = torch.zeros_like(p, memory_format=torch.preserve_format)
        state['exp_avg_sq'] = torch.zeros_like(p, memory_format=torch.preserve_format)
        if hasattr(p, 'mask'):
            assert p.mask == 'dense'
            state['exp_avg_sq_last'] = torch.empty(0, dtype=p.dtype, device=p.device)
        if amsgrad:
            state['max_exp_avg_sq'] = torch.zeros_like(p, memory_format=torch.preserve_format)
        return state

    @torch.no_grad()
    def step(self, closure=None):
        loss = None
        if closure is not None:
            with torch.enable_grad():
                loss = closure()
        self.t += 1
        lib, stream = N.lib(), N.stream_ptr()
        watching = self.mask == 'dense'
        partials, tracked_elements = [], 0
        for group in self.param_groups:
            beta1, beta2 = group['betas']
            amsgrad = group['amsgrad']
            lr, eps, wd = float(group['lr']), float(group['eps']), float(group['weight_decay'])
            for p in group['params']:
                grad = p.grad
                if grad is None:
                    continue
                if grad.is_sparse:
                    raise RuntimeError('Adam does not support sparse gradients, please consider SparseAdam instead')
                state = self.state[p]
                if len(state) == 0:
                    state = self._init_state(p, amsgrad)
                if grad.stride() != p.stride():
                    raise RuntimeError("AdamW_STEP: the gradient must have the parameter's strides")
                state['step'] += 1
                tracked = hasattr(p, 'mask')
                z_ptr, z_option, precond = None, 0, None
                if tracked and watching:
                    assert p.mask == 'dense'
                    z = torch.empty((lib.tf24_adamw_step_partials(p.numel()),), dtype=torch.float32, device=p.device)
                    partials.append(z)
                    tracked_elements += p.numel()
                    z_ptr, z_option = z.data_ptr(), self.option
                elif tracked:
                    assert p.mask == 'sparse'
                    precond = state['preconditioned_variance'].data_ptr()
                N.check(lib.tf24_adamw_step(
                    p.data_ptr(), grad.data_ptr(), N.dtype_code(grad.dtype), state['exp_avg'].data_ptr(),
                    state['exp_avg_sq'].data_ptr(), state['max_exp_avg_sq'].data_ptr() if amsgrad else None, precond,
                    p.numel(), lr, float(beta1), float(beta2), eps, wd, state['step'], z_ptr, z_option, stream))
        if watching:
            self._watch_variance(partials, tracked_elements)
        return loss

    def _watch_variance(self, partials, count):
        """Z_t, its window, and the switch to phase 2 (reference :150-194)."""
        if count == 0:
            raise RuntimeError("AdamW_STEP: no parameter carries a `mask` attribute, there is nothing to watch")
        total = torch.cat(partials).double().sum() / count
        z_t = total if self.option == 1 else torch.exp(total)
        self.sliding_window.append(z_t.float())
        while len(self.sliding_window) > self.T_omega:
            self.sliding_window.pop(0)
        average_z = torch.mean(torch.stack(self.sliding_window))
        if (self.T_max is not None) and (self.T_min is not None):
            if (self.t > self.T_max) or (average_z < self.eps and self.t > self.T_min):
                self.mask = 'sparse'
        elif average_z < self.eps:
            self.mask = 'sparse'
        if self.mask == 'sparse':
            print('Auto Switch Between two Phases...', flush=True)
            for group in self.param_groups:
                for p in group['params']:
                    if hasattr(p, 'mask'):
                        assert p.mask == 'dense'
                        p.mask = 'sparse'
                        state = self.state[p]
                        source = state['max_exp_avg_sq'] if group['amsgrad'] else state['exp_avg_sq']
                        state['preconditioned_variance'] = source.clone(memory_format=torch.preserve_format)
