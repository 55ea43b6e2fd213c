"""Grokfast: EMA low-pass filter of the gradient, amplification, AdamW.

Drop-in for the reference class (grokking_optimizers/grokfast.py:30-145):
same constructor arguments and defaults, same per-parameter state
(`step`, `ema`, `exp_avg`, `exp_avg_sq`, all fp32), `p.grad` overwritten with
the amplified gradient.  The whole step is ONE fused kernel launch over all
parameters (`_ops.grokfast_adamw_fused_step`); `fused=False` keeps the
reference's two-phase sequence (`_ops.grokfast_fused_step`, then AdamW).
"""
from typing import Iterable, Optional, Tuple

import torch
from torch.optim import Optimizer

from grokking_optimizers import _ops
from grokking_optimizers._adamw_helper import adamw_step


class Grokfast(Optimizer):
    def __init__(self, params: Iterable, lr: float = 1e-3, betas: Tuple[float, float] = (0.9, 0.98),
                 eps: float = 1e-8, weight_decay: float = 1.0, grokfast_alpha: float = 0.98,
                 grokfast_lamb: float = 2.0, fused: bool = True) -> None:
        if lr < 0.0:
            raise ValueError(f"Invalid learning rate: {lr}")
        if eps < 0.0:
            raise ValueError(f"Invalid epsilon value: {eps}")
        if not 0.0 <= betas[0] < 1.0:
            raise ValueError(f"Invalid beta parameter at index 0: {betas[0]}")
        if not 0.0 <= betas[1] < 1.0:
            raise ValueError(f"Invalid beta parameter at index 1: {betas[1]}")
        if not 0.0 <= grokfast_alpha < 1.0:
            raise ValueError(f"Invalid grokfast_alpha: {grokfast_alpha}")
        self.fused = fused
        super().__init__(params, dict(lr=lr, betas=betas, eps=eps, weight_decay=weight_decay,
                                      grokfast_alpha=grokfast_alpha, grokfast_lamb=grokfast_lamb))

    @torch.no_grad()
    def step(self, closure=None) -> Optional[float]:
        loss = None
        if closure is not None:
            with torch.enable_grad():
                loss = closure()
        for group in self.param_groups:
            ps, gs, emas, ms, vs, ts = [], [], [], [], [], []
            for p in group["params"]:
                if p.grad is None:
                    continue
                st = self.state[p]
                if len(st) == 0:
                    st["step"] = 0
                    for k in ("ema", "exp_avg", "exp_avg_sq"):
                        st[k] = torch.zeros_like(p, dtype=torch.float32)
                st["step"] += 1
                ps.append(p)
                gs.append(p.grad)
                emas.append(st["ema"])
                ms.append(st["exp_avg"])
                vs.append(st["exp_avg_sq"])
                ts.append(st["step"])
            if not ps:
                continue
            b1, b2 = group["betas"]
            if self.fused:
                _ops.grokfast_adamw_fused_step(ps, gs, emas, ms, vs, ts, group["grokfast_alpha"],
                                               group["grokfast_lamb"], group["lr"], b1, b2, group["eps"],
                                               group["weight_decay"])
            else:
                _ops.grokfast_fused_step(gs, emas, group["grokfast_alpha"], group["grokfast_lamb"])
                adamw_step(ps, gs, ms, vs, ts, group["lr"], b1, b2, group["eps"], group["weight_decay"])
        return loss
