"""Lion: sign of the interpolated momentum, decoupled weight decay.

Drop-in for the reference class (grokking_optimizers/lion.py:17-101): same
constructor arguments and defaults, one fp32 `exp_avg` per parameter, no step
counter.  One call of `_ops.lion_fused_step` per parameter group.
"""
from typing import Iterable, Optional, Tuple

import torch
from torch.optim import Optimizer

from grokking_optimizers import _ops
from grokking_optimizers._common import check_hyper, run_closure


class Lion(Optimizer):
    def __init__(self, params: Iterable, lr: float = 1e-4, betas: Tuple[float, float] = (0.9, 0.99),
                 weight_decay: float = 3.0) -> None:
        check_hyper(lr, None, betas)
        super().__init__(params, dict(lr=lr, betas=betas, weight_decay=weight_decay))

    @torch.no_grad()
    def step(self, closure=None) -> Optional[float]:
        loss = run_closure(closure)
        for group in self.param_groups:
            ps, gs, ms = [], [], []
            for p in group["params"]:
                if p.grad is None:
                    continue
                st = self.state[p]
                if len(st) == 0:
                    st["exp_avg"] = torch.zeros_like(p, dtype=torch.float32)
                ps.append(p)
                gs.append(p.grad)
                ms.append(st["exp_avg"])
            if ps:
                _ops.lion_fused_step(ps, gs, ms, group["lr"], group["betas"][0], group["betas"][1], group["weight_decay"])
        return loss
