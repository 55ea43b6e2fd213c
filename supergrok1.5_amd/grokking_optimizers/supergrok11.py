"""SuperGrok v1.1: Adam + mu EMA + the 2->H->1 sharpness meta-net, with
lambda gated per parameter by the cosine similarity between the smart gradient
and mu.  Drop-in for the reference class (grokking_optimizers/supergrok11.py:
14-302): same constructor arguments and defaults, flat fp32 state lists, the
same `_ops.supergrok11_fused_step` call - which here is three launches for all
parameters with the clip norm and every cosine gate reduced on the device (the
reference syncs the host once per parameter for the gate).

As in the reference, `_flat_steps` is passed by value through pybind, so the
bias corrections seen by the kernel are those of step 1 on every call.
"""
import math
from typing import Optional

import torch
import torch.nn as nn
from torch.optim import Optimizer

from grokking_optimizers import _ops
from grokking_optimizers._meta_training import MetaTraining
from grokking_optimizers._schedule import GrokSchedule
from grokking_optimizers.supergrok15 import SharpnessMetaNet


class SuperGrok11(MetaTraining, Optimizer):
    def __init__(self, params, lr: float = 1e-3, betas: tuple = (0.9, 0.999), eps: float = 1e-8, weight_decay: float = 1.0,
                 alpha_init: float = 0.98, lamb: float = 5.0, gamma: float = 0.1, gamma_alpha: float = 0.0, kappa: float = 0.1,
                 warmup_steps: int = 100, warmup_ramp: int = 100, gradient_clipping: float = 1.0,
                 meta_net: Optional[nn.Module] = None, meta_hidden_dim: int = 32, gate_temperature: float = 5.0,
                 alpha_update_freq: int = 50, meta_update_freq: int = 5, zero_loss_threshold: float = 1e-4,
                 zero_acc_threshold: float = 0.995, sam_rho: float = 0.05, sam_enable_threshold: float = 0.0):
        super().__init__(params, dict(lr=lr, betas=betas, eps=eps, weight_decay=weight_decay))
        self.gelu_mode = None      # None: the process-wide form of `_ops.supergrok15_set_gelu_mode`; "erf" / "sigmoid": this instance's own
        for k, v in dict(alpha_init=alpha_init, lamb=lamb, gamma=gamma, gamma_alpha=gamma_alpha, kappa=kappa,
                         warmup_steps=warmup_steps, warmup_ramp=max(1, warmup_ramp), gradient_clipping=gradient_clipping,
                         meta_hidden_dim=meta_hidden_dim, gate_temperature=gate_temperature, alpha_update_freq=alpha_update_freq,
                         meta_update_freq=meta_update_freq, zero_loss_threshold=zero_loss_threshold,
                         zero_acc_threshold=zero_acc_threshold, sam_rho=sam_rho, sam_enable_threshold=sam_enable_threshold).items():
            setattr(self, k, v)
        self.meta_net = SharpnessMetaNet(meta_hidden_dim) if meta_net is None else meta_net
        self._flat_params = [p for g in self.param_groups for p in g["params"]]
        if self._flat_params:
            self.meta_net = self.meta_net.to(self._flat_params[0].device)
        self._global_step = 0
        self._cached_alpha = alpha_init
        self._cached_train_acc = 0.0
        self._flat_layer_beta1s, self._flat_layer_alphas = GrokSchedule._layer_tables(self.param_groups, gamma, gamma_alpha)
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
            for lst in (self._flat_exp_avgs, self._flat_exp_avg_sqs, self._flat_mus, self._flat_sharpness):
                lst.append(torch.zeros(p.data.numel(), dtype=torch.float32, device=p.device))
        self._state_initialized = True

    def _update_alpha(self, train_loss, val_loss, train_acc):
        GrokSchedule._update_alpha(self, train_loss, val_loss, train_acc)

    def _get_ramp_factor(self):
        return GrokSchedule._get_ramp_factor(self)

    def _get_effective_sam_freq(self):
        """999999 (off) below sam_enable_threshold, else 1: the training loop decides the actual frequency."""
        return 999999 if self._cached_train_acc < self.sam_enable_threshold else 1

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
        if self._global_step % self.alpha_update_freq == 0 or self._global_step == 1:
            self._update_alpha(train_loss, val_loss, train_acc)
        layer_alphas = [max(0.0, min(1.0, self._cached_alpha * f)) for f in self._flat_layer_alphas]
        group = self.param_groups[0]
        grads = [p.grad.data if p.grad is not None else torch.Tensor() for p in self._flat_params]
        if self._weights_dirty:
            self._cached_weights = self.meta_net.get_weights()
            self._weights_dirty = False
        W1, b1, W2, b2, rescale = self._cached_weights
        sharp = [s if (g.numel() == 0 or s.dtype == g.dtype) else s.to(g.dtype) for s, g in zip(self._flat_sharpness, grads)]
        if self.gelu_mode is not None:        # this optimizer's own choice of the meta-net's GELU form, set right before its call
            _ops.supergrok15_set_gelu_mode(self.gelu_mode)
        _ops.supergrok11_fused_step(
            self._flat_param_data, grads, self._flat_exp_avgs, self._flat_exp_avg_sqs, self._flat_mus, sharp, self._flat_steps,
            layer_alphas, self._flat_layer_beta1s, W1, b1, W2, b2, rescale, self.meta_hidden_dim, group["betas"][1], group["lr"],
            group["weight_decay"], group["eps"], self.lamb, self._get_ramp_factor(), self.gate_temperature, self.gradient_clipping)
        return loss

    def meta_step(self, model, val_x, val_y, criterion, meta_optimizer):
        """Bilevel meta-net update on the validation batch (supergrok11.py:236-285 of the reference)."""
        return self._meta_update(model, val_x, val_y, criterion, meta_optimizer)
