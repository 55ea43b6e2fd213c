"""LookSAM: AdamW whose gradients are periodically nudged along a stored
sharpness direction.

Drop-in for the reference class (grokking_optimizers/looksam.py:20-247): same
constructor arguments and defaults, `step()` is a plain AdamW step (one fused
launch), `sam_step()` perturbs the parameters along the gradient, re-evaluates
the loss there, restores them, stores v = (g_sam - g)/|g_sam - g| per parameter
and adds alpha*|g|*v to the gradient.  The four tensor passes run through
`_ops.looksam_*`; norms are reduced on the device.
"""
from typing import Callable, Iterable, Optional, Tuple

import torch
from torch.optim import Optimizer

from grokking_optimizers import _ops
from grokking_optimizers._adamw_helper import adamw_step
from grokking_optimizers._common import check_hyper, gather, run_closure


class LookSAM(Optimizer):
    _BUFFERS = ("exp_avg", "exp_avg_sq", "sam_direction")

    def __init__(self, params: Iterable, lr: float = 1e-3, betas: Tuple[float, float] = (0.9, 0.98), eps: float = 1e-8,
                 weight_decay: float = 1.0, rho: float = 0.05, k: int = 5, alpha: float = 0.7) -> None:
        check_hyper(lr, eps, betas)
        if rho < 0.0:
            raise ValueError(f"Invalid rho value: {rho}")
        if k < 1:
            raise ValueError(f"Invalid k value: {k}")
        super().__init__(params, dict(lr=lr, betas=betas, eps=eps, weight_decay=weight_decay, rho=rho, k=k, alpha=alpha))
        self._global_step: int = 0

    @torch.no_grad()
    def step(self, closure=None) -> Optional[float]:
        loss = run_closure(closure)
        self._global_step += 1
        for group in self.param_groups:
            s = gather(self, group, self._BUFFERS)
            if s["params"]:
                adamw_step(s["params"], s["grads"], s["exp_avg"], s["exp_avg_sq"], s["steps"], group["lr"], group["betas"][0],
                           group["betas"][1], group["eps"], group["weight_decay"])
        return loss

    @torch.no_grad()
    def sam_step(self, model: torch.nn.Module, train_x, train_y, criterion: Callable) -> None:
        work = []
        for group in self.param_groups:
            s = gather(self, group, self._BUFFERS, count_steps=False)
            if not s["params"]:
                continue
            grads = [g.clone() for g in s["grads"]]
            backups = _ops.looksam_perturb_all(s["params"], grads, group["rho"])
            work.append((s["params"], grads, s["sam_direction"], backups, group))
        model.zero_grad()
        with torch.enable_grad():
            criterion(model(train_x), train_y).backward()
        for params, grads, dirs, backups, group in work:
            sam_grads = [p.grad.clone() for p in params]
            _ops.looksam_restore_all(params, backups)
            _ops.looksam_compute_directions(dirs, sam_grads, grads)
            _ops.looksam_adjust_grads(grads, dirs, group["alpha"])
            for p, g in zip(params, grads):
                p.grad.copy_(g)

    @property
    def global_step(self) -> int:
        return self._global_step

    def should_sam_step(self) -> bool:
        return self._global_step % self.param_groups[0]["k"] == 0
