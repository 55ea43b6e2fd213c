"""Muon: momentum + Newton-Schulz orthogonalisation for 2-D parameters, AdamW
for the rest.  Drop-in for the reference class (grokking_optimizers/muon.py):
2-D parameters go to `_ops.muon_fused_step` with an fp32 momentum buffer
(muon.py:145-147 there); everything else takes `adamw_step`."""
from typing import Iterable, Optional, Tuple

import torch
from torch.optim import Optimizer

from grokking_optimizers import _ops
from grokking_optimizers._adamw_helper import adamw_step
from grokking_optimizers._common import check_ranges


class Muon(Optimizer):
    """Args (as the reference, muon.py:45-56 there): params_2d, params_1d=None, lr=0.02,
    momentum=0.95, weight_decay=1.0, adamw_lr=1e-3, adamw_betas=(0.9, 0.98),
    adamw_eps=1e-8, ns_steps=5.  Group 0 holds the 2-D parameters (Muon),
    group 1 the others (AdamW, same weight decay)."""

    def __init__(self, params_2d: Iterable, params_1d: Optional[Iterable] = None, lr: float = 0.02,
                 momentum: float = 0.95, weight_decay: float = 1.0, adamw_lr: float = 1e-3,
                 adamw_betas: Tuple[float, float] = (0.9, 0.98), adamw_eps: float = 1e-8, ns_steps: int = 5) -> None:
        check_ranges((("learning rate", lr, 0.0, None), ("AdamW learning rate", adamw_lr, 0.0, None), ("momentum", momentum, 0.0, 1.0),
                      ("AdamW beta at index 0", adamw_betas[0], 0.0, 1.0), ("AdamW beta at index 1", adamw_betas[1], 0.0, 1.0),
                      ("ns_steps", ns_steps, 1, None)))
        groups = [dict(params=list(params_2d), lr=lr, momentum=momentum, weight_decay=weight_decay,
                       ns_steps=ns_steps, group_type="muon")]
        one_d = list(params_1d) if params_1d is not None else []
        if one_d:
            groups.append(dict(params=one_d, lr=adamw_lr, betas=adamw_betas, eps=adamw_eps,
                               weight_decay=weight_decay, group_type="adamw"))
        super().__init__(groups, dict(lr=lr, momentum=momentum, weight_decay=weight_decay, ns_steps=ns_steps,
                                      group_type="muon"))

    @torch.no_grad()
    def step(self, closure=None) -> Optional[float]:
        loss = None
        if closure is not None:
            with torch.enable_grad():
                loss = closure()
        for group in self.param_groups:
            if group.get("group_type", "muon") == "muon":
                self._step_muon(group)
            else:
                self._step_adamw(group)
        return loss

    def _step_muon(self, group) -> None:
        ps, gs, bufs = [], [], []
        for p in group["params"]:
            if p.grad is None:
                continue
            st = self.state[p]
            if len(st) == 0:
                st["momentum_buffer"] = torch.zeros_like(p, dtype=torch.float32)
            ps.append(p)
            gs.append(p.grad)
            bufs.append(st["momentum_buffer"])
        if ps:
            _ops.muon_fused_step(ps, gs, bufs, group["momentum"], group["lr"], group["weight_decay"], group["ns_steps"])

    def _step_adamw(self, group) -> None:
        ps, gs, ms, vs, ts = [], [], [], [], []
        for p in group["params"]:
            if p.grad is None:
                continue
            st = self.state[p]
            if len(st) == 0:
                st["step"] = 0
                st["exp_avg"] = torch.zeros_like(p, dtype=torch.float32)
                st["exp_avg_sq"] = torch.zeros_like(p, dtype=torch.float32)
            st["step"] += 1
            ps.append(p)
            gs.append(p.grad)
            ms.append(st["exp_avg"])
            vs.append(st["exp_avg_sq"])
            ts.append(st["step"])
        if ps:
            b1, b2 = group.get("betas", (0.9, 0.98))
            adamw_step(ps, gs, ms, vs, ts, group["lr"], b1, b2, group.get("eps", 1e-8), group["weight_decay"])
