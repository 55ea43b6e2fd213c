"""NeuralGrok: Adam on gradients rescaled by a small learned amplifier MLP.

Drop-in for the reference classes (grokking_optimizers/neuralgrok.py:22-243):
`_Amplifier` (Linear(1,H), ReLU, [Linear(H,H), ReLU]*, Linear(H,1)) and
`NeuralGrok` with the same constructor arguments, defaults and helper methods.
As in the reference, the fused step evaluates only the first and the last Linear
of the amplifier; with num_layers=2 that is the whole network.
"""
from typing import Iterable, List, Optional, Tuple

import torch
import torch.nn as nn
from torch.optim import Optimizer

from grokking_optimizers import _ops
from grokking_optimizers._common import check_hyper, gather, run_closure


class _Amplifier(nn.Module):
    def __init__(self, num_layers: int = 3, hidden_dim: int = 128) -> None:
        super().__init__()
        if num_layers < 2:
            raise ValueError("num_layers must be >= 2 (input + output layer)")
        self.hidden_dim = hidden_dim
        layers: List[nn.Module] = [nn.Linear(1, hidden_dim), nn.ReLU()]
        for _ in range(num_layers - 2):
            layers += [nn.Linear(hidden_dim, hidden_dim), nn.ReLU()]
        layers.append(nn.Linear(hidden_dim, 1))
        self.net = nn.Sequential(*layers)

    def forward(self, x):
        return self.net(x)

    def get_weights(self):
        first, last = self.net[0], self.net[-1]
        return tuple(t.detach().float().contiguous() for t in (first.weight, first.bias, last.weight, last.bias))


class NeuralGrok(Optimizer):
    def __init__(self, params: Iterable, lr: float = 1e-3, betas: Tuple[float, float] = (0.9, 0.98), eps: float = 1e-8,
                 weight_decay: float = 1.0, alpha: float = 10.0, beta: float = 4.0, num_layers: int = 3, hidden_dim: int = 128,
                 inner_steps: int = 1, grad_clip: float = 1.0) -> None:
        check_hyper(lr, eps, betas)
        self.amplifier = _Amplifier(num_layers=num_layers, hidden_dim=hidden_dim)
        super().__init__(params, dict(lr=lr, betas=betas, eps=eps, weight_decay=weight_decay, alpha=alpha, beta=beta,
                                      inner_steps=inner_steps, grad_clip=grad_clip))
        self._meta_weights_dirty = True
        self._cached_meta_weights = None

    @torch.no_grad()
    def step(self, closure=None) -> Optional[float]:
        loss = run_closure(closure)
        if self._meta_weights_dirty or self._cached_meta_weights is None:
            self._cached_meta_weights = self.amplifier.get_weights()
            self._meta_weights_dirty = False
        for group in self.param_groups:
            s = gather(self, group, ("exp_avg", "exp_avg_sq"))
            if not s["params"]:
                continue
            dev = s["params"][0].device
            W1, b1, W2, b2 = (w.to(dev) for w in self._cached_meta_weights)
            _ops.neuralgrok_fused_step(s["params"], s["grads"], s["exp_avg"], s["exp_avg_sq"], s["steps"], W1, b1, W2, b2,
                                       group["alpha"], group["beta"], self.amplifier.hidden_dim, group["betas"][0],
                                       group["betas"][1], group["lr"], group["weight_decay"], group["eps"], group["grad_clip"])
        return loss

    def mark_amplifier_dirty(self) -> None:
        """Call after the amplifier's weights changed so the next step re-extracts them."""
        self._meta_weights_dirty = True

    def get_amplifier(self) -> _Amplifier:
        return self.amplifier

    def get_amplifier_optimizer(self, lr: float = 1e-4) -> torch.optim.Adam:
        return torch.optim.Adam(self.amplifier.parameters(), lr=lr)
