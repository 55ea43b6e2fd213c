"""Prodigy: Adam whose step size estimate d_lr grows with the distance travelled.

Drop-in for the reference class (grokking_optimizers/prodigy.py:17-136): same
constructor arguments and defaults, state `step`, `exp_avg`, `exp_avg_sq`, `s`
(fp32) and `param_init` (fp32 copy of the initial value), `d_lr` starting at
1e-6 and fed back through `_ops.prodigy_fused_step`, which returns its update.
"""
from typing import Iterable, Optional, Tuple

import torch
from torch.optim import Optimizer

from grokking_optimizers import _ops
from grokking_optimizers._common import check_hyper, gather, run_closure


class Prodigy(Optimizer):
    def __init__(self, params: Iterable, lr: float = 1.0, betas: Tuple[float, float] = (0.9, 0.999), eps: float = 1e-8,
                 weight_decay: float = 1.0) -> None:
        check_hyper(lr, eps, betas)
        super().__init__(params, dict(lr=lr, betas=betas, eps=eps, weight_decay=weight_decay))
        self._d_lr: float = 1e-6

    @torch.no_grad()
    def step(self, closure=None) -> Optional[float]:
        loss = run_closure(closure)

        def keep_init(p, st):
            st["param_init"] = p.detach().clone().float()

        for group in self.param_groups:
            s = gather(self, group, ("exp_avg", "exp_avg_sq", "s"), extra_init=keep_init)
            if not s["params"]:
                continue
            inits = [self.state[p]["param_init"] for p in s["params"]]
            self._d_lr = _ops.prodigy_fused_step(s["params"], s["grads"], s["exp_avg"], s["exp_avg_sq"], s["s"], inits, s["steps"],
                                                 self._d_lr, group["betas"][0], group["betas"][1], group["lr"],
                                                 group["weight_decay"], group["eps"])
        return loss

    @property
    def d_lr(self) -> float:
        return self._d_lr
