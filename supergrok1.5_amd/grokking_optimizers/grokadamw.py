"""GrokAdamW: AdamW on g + lamb * EMA(g), with global-norm clipping.

Drop-in for the reference class (grokking_optimizers/grokadamw.py:21-144): same
constructor arguments and defaults (`gamma` and `decay` are accepted and unused,
as there), same state (`step`, `exp_avg`, `exp_avg_sq`, `ema`, fp32).  One call
of `_ops.grokadamw_fused_step` per parameter group.
"""
from typing import Iterable, Optional, Tuple

import torch
from torch.optim import Optimizer

from grokking_optimizers import _ops
from grokking_optimizers._common import check_hyper, gather, run_closure


class GrokAdamW(Optimizer):
    def __init__(self, params: Iterable, lr: float = 1e-3, betas: Tuple[float, float] = (0.9, 0.98), eps: float = 1e-8,
                 weight_decay: float = 1.0, alpha: float = 0.98, lamb: float = 5.0, gamma: float = 0.1, decay: float = 0.1,
                 grad_clip: float = 1.0) -> None:
        check_hyper(lr, eps, betas)
        if not 0.0 <= alpha < 1.0:
            raise ValueError(f"Invalid alpha parameter: {alpha}")
        super().__init__(params, dict(lr=lr, betas=betas, eps=eps, weight_decay=weight_decay, alpha=alpha, lamb=lamb,
                                      gamma=gamma, decay=decay, grad_clip=grad_clip))

    @torch.no_grad()
    def step(self, closure=None) -> Optional[float]:
        loss = run_closure(closure)
        for group in self.param_groups:
            s = gather(self, group, ("exp_avg", "exp_avg_sq", "ema"))
            if not s["params"]:
                continue
            _ops.grokadamw_fused_step(s["params"], s["grads"], s["exp_avg"], s["exp_avg_sq"], s["ema"], s["steps"], group["alpha"],
                                      group["lamb"], group["betas"][0], group["betas"][1], group["lr"], group["weight_decay"],
                                      group["eps"], group["grad_clip"])
        return loss
