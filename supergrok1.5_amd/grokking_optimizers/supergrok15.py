"""SuperGrok v1.5: Adam + mu EMA + a 2->H->1 sharpness meta-net, sigmoid-gated
lambda, progressive weight decay.  Drop-in for the reference class
(grokking_optimizers/supergrok15.py:67-305): same constructor arguments and
defaults, flat fp32 state lists, and the same `_ops.supergrok15_fused_step`
call (supergrok15.py:289-303 there) -- which here is one batched launch with
the gradient-norm clip reduced on the device instead of a host sync.

As in the reference, `_flat_steps` is passed by value through pybind, so the
bias corrections seen by the kernel are those of step 1 on every call.
"""
from typing import Optional

import torch
import torch.nn as nn
from torch.optim import Optimizer

from grokking_optimizers import _ops
from grokking_optimizers._meta_training import MetaTraining, ScheduledTraining
from grokking_optimizers._schedule import GrokSchedule


class SharpnessMetaNet(nn.Module):
    """output = grad + rescale * MLP([grad, sharpness]),  MLP = Linear(2,H) -> GELU -> Linear(H,1).
    rescale starts at 0, weights N(0, 0.01), biases 0 (reference: supergrok15.py:25-64)."""

    def __init__(self, hidden_dim: int = 32):
        super().__init__()
        self.hidden_dim = hidden_dim
        self.net = nn.Sequential(nn.Linear(2, hidden_dim), nn.GELU(), nn.Linear(hidden_dim, 1))
        self.rescale = nn.Parameter(torch.zeros(1))
        with torch.no_grad():
            for lin in (self.net[0], self.net[2]):
                lin.weight.normal_(0, 0.01)
                lin.bias.zero_()

    def forward(self, grad: torch.Tensor, sharpness: torch.Tensor) -> torch.Tensor:
        if grad.numel() == 0:
            return grad
        x = torch.stack([grad.reshape(-1), sharpness.reshape(-1)], dim=1)
        return (grad.reshape(-1, 1) + self.rescale * self.net(x)).reshape(grad.shape)

    def get_weights(self):
        return (self.net[0].weight.data.contiguous(), self.net[0].bias.data.contiguous(),
                self.net[2].weight.data.contiguous(), self.net[2].bias.data.contiguous(),
                self.rescale.data.item())


class SuperGrok15(GrokSchedule, MetaTraining, ScheduledTraining, Optimizer):
    def __init__(self, params, lr: float = 1e-3, betas: tuple = (0.9, 0.999), eps: float = 1e-8,
                 weight_decay: float = 1.0, alpha_init: float = 0.98, lamb: float = 2.0, gamma: float = 0.1,
                 gamma_alpha: float = 0.0, kappa: float = 0.1, warmup_steps: int = 100, warmup_ramp: int = 100,
                 gradient_clipping: float = 1.0, meta_net: Optional[nn.Module] = None, meta_hidden_dim: int = 32,
                 alpha_update_freq: int = 100, zero_loss_threshold: float = 1e-4, zero_acc_threshold: float = 0.995,
                 sam_rho: float = 0.05, gate_scale: float = 20.0, gate_thresh: float = 0.8, sam_freq_min: int = 3,
                 sam_freq_max: int = 20, sam_scale: float = 20.0, sam_thresh: float = 0.85, bilevel_freq_min: int = 5,
                 bilevel_freq_max: int = 30, bilevel_scale: float = 20.0, bilevel_thresh: float = 0.9,
                 wd_ramp: float = 4.0, wd_scale: float = 20.0, wd_thresh: float = 0.9,
                 sam_enable_threshold: float = 0.0):
        Optimizer.__init__(self, params, dict(lr=lr, betas=betas, eps=eps, weight_decay=weight_decay))
        # None: whatever `_ops.supergrok15_set_gelu_mode` last selected for the process ("erf" unless changed); "erf" / "sigmoid":
        # this instance's own form (the reference's CPU path / its GPU kernel), whatever other instances use
        self.gelu_mode = None
        for k, v in dict(alpha_init=alpha_init, lamb=lamb, gamma=gamma, gamma_alpha=gamma_alpha, kappa=kappa,
                         warmup_steps=warmup_steps, warmup_ramp=max(1, warmup_ramp),
                         gradient_clipping=gradient_clipping, alpha_update_freq=alpha_update_freq,
                         zero_loss_threshold=zero_loss_threshold, zero_acc_threshold=zero_acc_threshold,
                         sam_rho=sam_rho, meta_hidden_dim=meta_hidden_dim, gate_scale=gate_scale,
                         gate_thresh=gate_thresh, sam_freq_min=sam_freq_min, sam_freq_max=sam_freq_max,
                         sam_scale=sam_scale, sam_thresh=sam_thresh, bilevel_freq_min=bilevel_freq_min,
                         bilevel_freq_max=bilevel_freq_max, bilevel_scale=bilevel_scale,
                         bilevel_thresh=bilevel_thresh, wd_ramp=wd_ramp, wd_scale=wd_scale, wd_thresh=wd_thresh,
                         sam_enable_threshold=sam_enable_threshold).items():
            setattr(self, k, v)
        self.meta_net = SharpnessMetaNet(meta_hidden_dim) if meta_net is None else meta_net
        self._flat_params = [p for g in self.param_groups for p in g["params"]]
        if self._flat_params:
            self.meta_net = self.meta_net.to(self._flat_params[0].device)
        self._global_step = 0
        self._cached_alpha = alpha_init
        self._cached_train_acc = 0.0
        self._flat_layer_beta1s, self._flat_layer_alphas = self._layer_tables(self.param_groups, gamma, gamma_alpha)
        self._flat_steps = [0] * len(self._flat_params)
        self._param_to_idx = {id(p): i for i, p in enumerate(self._flat_params)}
        self._num_params = len(self._flat_params)
        self._flat_param_data = [p.data for p in self._flat_params]
        self._flat_exp_avgs, self._flat_exp_avg_sqs, self._flat_mus, self._flat_sharpness = [], [], [], []
        self._state_initialized = False
        self._weights_dirty = True
        self._cached_weights = None

    def _ensure_state(self):
        if self._state_initialized:
            return
        for p in self._flat_params:
            mk = lambda: torch.zeros(p.data.numel(), dtype=torch.float32, device=p.device)
            self._flat_exp_avgs.append(mk())
            self._flat_exp_avg_sqs.append(mk())
            self._flat_mus.append(mk())
            self._flat_sharpness.append(mk())
        self._state_initialized = True

    @torch.no_grad()
    def step(self, closure=None, train_loss=None, val_loss=None, train_acc=None):
        loss = None
        if closure is not None:
            with torch.enable_grad():
                loss = closure()
        self._ensure_state()
        self._global_step += 1
        if train_acc is not None:
            self._cached_train_acc = train_acc
        self._maybe_update_alpha(train_loss, val_loss, train_acc)
        alpha = self._cached_alpha
        layer_alphas = [max(0.0, min(1.0, alpha * f)) for f in self._flat_layer_alphas]
        group = self.param_groups[0]
        grads = [p.grad.data if p.grad is not None else torch.Tensor() for p in self._flat_params]
        if self._weights_dirty:
            self._cached_weights = self.meta_net.get_weights()
            self._weights_dirty = False
        W1, b1, W2, b2, rescale = self._cached_weights
        # sharpness is kept in fp32; hand the kernel the gradient's element type
        sharp = [s if (g.numel() == 0 or s.dtype == g.dtype) else s.to(g.dtype)
                 for s, g in zip(self._flat_sharpness, grads)]
        if self.gelu_mode is not None:        # this optimizer's own choice of the meta-net's GELU form, set right before its call
            _ops.supergrok15_set_gelu_mode(self.gelu_mode)
        _ops.supergrok15_fused_step(
            self._flat_param_data, grads, self._flat_exp_avgs, self._flat_exp_avg_sqs, self._flat_mus, sharp,
            self._flat_steps, layer_alphas, self._flat_layer_beta1s, W1, b1, W2, b2, rescale, self.meta_hidden_dim,
            group["betas"][1], group["lr"], self._get_effective_wd(group["weight_decay"]), group["eps"],
            self.lamb, self._get_ramp_factor(), self._get_gate_signal(), self.gradient_clipping)
        return loss

    # sam_step comes from MetaTraining (supergrok15.py:307-352 of the reference)

    def bilevel_step(self, model, train_x, train_y, val_x, val_y, criterion, meta_optimizer):
        """Bilevel meta-net update on the validation batch with the cached sharpness (supergrok15.py:354-413 there)."""
        return self._meta_update(model, val_x, val_y, criterion, meta_optimizer)

    # sam_meta_step, get_cached_alpha, get_effective_wd and step_full come from ScheduledTraining
