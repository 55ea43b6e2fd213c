"""SuperGrok v2: Adam driven by a per-tensor meta-network (magnitude sort ->
bidirectional Mamba-3 scan -> per-element GRU -> 4-head PEER routing -> expert
MLP) with mu EMA, sigmoid-gated lambda and progressive weight decay.

Drop-in for the optimizer step of the reference class
(grokking_optimizers/supergrok2.py:40-472): same constructor arguments and
defaults, the same flat state lists and shapes (:202-221 there), the same
per-tensor scalars (beta1_i, alpha_i, bias corrections in Python double,
lambda_eff = lamb*ramp*gate, progressive wd) and the same 51-argument
`_ops.supergrok2_mamba_peer_batched_step` call (:373-423 there), followed by
expert recycling every `recycle_interval` steps.

Differences, all on the host side:
  * the per-tensor norm clip is applied with device-side scale factors
    (torch._foreach_norm) instead of two host syncs per tensor; a gradient whose
    norm is below the threshold is multiplied by exactly 1.0;
  * non-finite gradient entries are zeroed inside the kernel (the reference
    does it both on the host and in the kernel);
  * after a recycling event the cached weight tensors are rebuilt, so re-drawn
    product keys are seen by the next step (the reference keeps using stale
    stacked copies until its cache is next invalidated);
  * parameters must live on the GPU: there is no Python fallback path.
`sam_step`, `bilevel_step`, `sam_meta_step` and `step_full` are there too: the SAM
probe through the fused perturb / sharpness ops, the bilevel update with the
meta-net differentiated in HIP (grokking_optimizers/_bilevel.py).
"""
from typing import Optional

import torch
import torch.nn as nn
from torch.optim import Optimizer

from grokking_optimizers import _ops
from grokking_optimizers._meta_training import MetaTraining, ScheduledTraining
from grokking_optimizers._schedule import GrokSchedule
from grokking_optimizers.mamba3_peer_metanet import Mamba3PEERMetaNet


class SuperGrok2(GrokSchedule, MetaTraining, ScheduledTraining, Optimizer):
    def __init__(self, params, lr: float = 1e-3, betas: tuple = (0.9, 0.999), eps: float = 1e-8,
                 weight_decay: float = 1.0, alpha_init: float = 0.98, lamb: float = 2.0, gamma: float = 0.1,
                 gamma_alpha: float = 0.0, kappa: float = 0.1, warmup_steps: int = 100, warmup_ramp: int = 100,
                 gradient_clipping: float = 1.0, meta_net: Optional[nn.Module] = None, d_model: int = 8,
                 d_state: int = 16, mamba_expand: int = 2, num_peer_heads: int = 4, num_experts: int = 144,
                 expert_hidden: int = 16, gru_hidden: int = 4, meta_rescale: float = 0.1, recycle_interval: int = 100,
                 recycle_threshold: float = 0.001, alpha_update_freq: int = 100, zero_loss_threshold: float = 1e-4,
                 zero_acc_threshold: float = 0.995, sam_rho: float = 0.05, gate_scale: float = 20.0,
                 gate_thresh: float = 0.8, sam_freq_min: int = 3, sam_freq_max: int = 20, sam_scale: float = 20.0,
                 sam_thresh: float = 0.85, bilevel_freq_min: int = 5, bilevel_freq_max: int = 30,
                 bilevel_scale: float = 20.0, bilevel_thresh: float = 0.9, wd_ramp: float = 4.0, wd_scale: float = 20.0,
                 wd_thresh: float = 0.9, sam_enable_threshold: float = 0.0, bilevel_checkpoint_interval: int = 1):
        Optimizer.__init__(self, params, dict(lr=lr, betas=betas, eps=eps, weight_decay=weight_decay))
        for k, v in dict(alpha_init=alpha_init, sam_enable_threshold=sam_enable_threshold, lamb=lamb, gamma=gamma,
                         gamma_alpha=gamma_alpha, kappa=kappa, warmup_steps=warmup_steps,
                         warmup_ramp=max(1, warmup_ramp), gradient_clipping=gradient_clipping,
                         alpha_update_freq=alpha_update_freq, zero_loss_threshold=zero_loss_threshold,
                         zero_acc_threshold=zero_acc_threshold, sam_rho=sam_rho, d_model=d_model, d_state=d_state,
                         num_experts=num_experts, expert_hidden=expert_hidden, gru_hidden=gru_hidden,
                         meta_rescale=meta_rescale, gate_scale=gate_scale, gate_thresh=gate_thresh,
                         sam_freq_min=sam_freq_min, sam_freq_max=sam_freq_max, sam_scale=sam_scale,
                         sam_thresh=sam_thresh, bilevel_freq_min=bilevel_freq_min, bilevel_freq_max=bilevel_freq_max,
                         bilevel_scale=bilevel_scale, bilevel_thresh=bilevel_thresh, wd_ramp=wd_ramp,
                         wd_scale=wd_scale, wd_thresh=wd_thresh,
                         bilevel_checkpoint_interval=max(1, bilevel_checkpoint_interval)).items():
            setattr(self, k, v)
        if meta_net is None:
            meta_net = Mamba3PEERMetaNet(d_model=d_model, d_state=d_state, mamba_expand=mamba_expand,
                                         num_peer_heads=num_peer_heads, num_experts=num_experts,
                                         expert_hidden=expert_hidden, gru_hidden=gru_hidden, rescale=meta_rescale,
                                         recycle_interval=recycle_interval, recycle_threshold=recycle_threshold)
        self.meta_net = meta_net
        self._flat_params = [p for g in self.param_groups for p in g["params"]]
        if self._flat_params:
            self.meta_net = self.meta_net.to(self._flat_params[0].device)
        self._global_step = 0
        self._step_counter = 0
        self._cached_alpha = alpha_init
        self._cached_train_acc = 0.0
        self._flat_layer_beta1s, self._flat_layer_alphas = self._layer_tables(self.param_groups, gamma, gamma_alpha)
        self._flat_steps = [0] * len(self._flat_params)
        self._param_to_idx = {id(p): i for i, p in enumerate(self._flat_params)}
        self._num_params = len(self._flat_params)
        self._flat_param_data = [p.data for p in self._flat_params]
        self._flat_exp_avgs, self._flat_exp_avg_sqs, self._flat_mus, self._flat_sharpness = [], [], [], []
        self._flat_gru_states, self._flat_mamba_fwd_states, self._flat_mamba_bwd_states = [], [], []
        self._state_initialized = False
        self._weights_dirty = True
        self._cached_weights = None

    def _ensure_state(self):
        if self._state_initialized:
            return
        for p in self._flat_params:
            n = p.data.numel()
            mk = lambda *s: torch.zeros(*s, dtype=torch.float32, device=p.device)
            self._flat_exp_avgs.append(mk(n))
            self._flat_exp_avg_sqs.append(mk(n))
            self._flat_mus.append(mk(n))
            self._flat_sharpness.append(mk(n))
            self._flat_gru_states.append(mk(n, self.gru_hidden))
            self._flat_mamba_fwd_states.append(None)     # created on first use, as in the reference
            self._flat_mamba_bwd_states.append(None)
        self._state_initialized = True

    def _clip(self, grads):
        """grad * clip/(norm+1e-12) where norm > clip, non-finite entries zeroed (reference: supergrok2.py:316-321):
        three launches for all tensors, norms reduced on the device, no host syncs."""
        return _ops.supergrok2_clip_grads([g.contiguous() for g in grads], float(self.gradient_clipping))

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

        group = self.param_groups[0]
        lr, beta2, eps = group["lr"], group["betas"][1], group["eps"]
        wd_eff = self._get_effective_wd(group["weight_decay"])
        lamb_eff = self.lamb * self._get_ramp_factor() * self._get_gate_signal()

        active = [i for i, p in enumerate(self._flat_params) if p.grad is not None]
        if not active:
            return loss
        mn = self.meta_net
        if not self._flat_params[active[0]].is_cuda:
            raise RuntimeError("SuperGrok2 on MI355X needs GPU parameters: the fused step has no CPU path")
        alphas, lambs, beta1s, bc1s, bc2s = [], [], [], [], []
        for i in active:
            p = self._flat_params[i]
            self._flat_steps[i] += 1
            t, b1 = self._flat_steps[i], self._flat_layer_beta1s[i]
            alphas.append(float(max(0.0, min(1.0, self._cached_alpha * self._flat_layer_alphas[i]))))
            lambs.append(float(lamb_eff))
            beta1s.append(float(b1))
            bc1s.append(float(1.0 - b1 ** t))
            bc2s.append(float(1.0 - beta2 ** t))
            if self._flat_mamba_fwd_states[i] is None:
                shape = (mn.mamba_fwd.d_inner, mn.d_state)
                self._flat_mamba_fwd_states[i] = torch.zeros(*shape, dtype=torch.float32, device=p.device)
                self._flat_mamba_bwd_states[i] = torch.zeros(*shape, dtype=torch.float32, device=p.device)
        grads = self._clip([self._flat_params[i].grad.data for i in active])
        grads = [g.contiguous() for g in grads]
        if self._weights_dirty:
            self._cached_weights = mn.flat_weights()
            self._weights_dirty = False
        sharp = [self._flat_sharpness[i].to(g.dtype) for i, g in zip(active, grads)]
        pick = lambda lst: [lst[i] for i in active]
        _ops.supergrok2_mamba_peer_batched_step(
            [self._flat_params[i].data for i in active], grads, sharp, pick(self._flat_exp_avgs),
            pick(self._flat_exp_avg_sqs), pick(self._flat_mus), pick(self._flat_gru_states),
            pick(self._flat_mamba_fwd_states), pick(self._flat_mamba_bwd_states), *self._cached_weights,
            alphas, lambs, beta1s, bc1s, bc2s, float(mn.rescale), float(beta2), float(lr), float(wd_eff), float(eps),
            mn.d_model, mn.d_state, mn.mamba_fwd.d_inner, mn.gru_hidden, mn.num_peer_heads, mn.pk_dim,
            mn.expert_hidden, mn.num_experts, mn.expert_counts)
        self._step_counter += 1
        if mn.recycle_interval > 0 and self._step_counter % mn.recycle_interval == 0:
            if mn._recycle_dead_experts():
                self._weights_dirty = True
        return loss

    # sam_step comes from MetaTraining (supergrok2.py:474-514 of the reference); sam_meta_step, step_full and the
    # getters from ScheduledTraining.

    def bilevel_step(self, model, train_x, train_y, val_x, val_y, criterion, meta_optimizer):
        """One meta-optimizer step on  -sum_p <smart_grad_p, val_grad_p / |val_grad_p|>  where smart_grad is the
        meta-net's differentiable output (soft top-4 routing) on the training gradient, cached sharpness and
        persistent states of every parameter (reference: supergrok2.py:516-1371).  The meta-net runs in HIP forward and
        backward, for all parameters in one pass; .grad of the model is restored.
        Returns the validation loss."""
        from grokking_optimizers import _bilevel
        self._ensure_state()
        named = list(model.named_parameters())
        saved = {n: p.grad.detach().clone() for n, p in named if p.grad is not None}
        picked = [(n, p, self._param_to_idx[id(p)]) for n, p in named
                  if n in saved and id(p) in self._param_to_idx and saved[n].numel() > 0]
        if not picked:
            return 0.0
        model.zero_grad()
        with torch.enable_grad():
            val_loss = criterion(model(val_x), val_y)
            val_loss.backward()
        meta_optimizer.zero_grad()
        grads, sharps, grus, mf, mb, cots = [], [], [], [], [], []
        for n, p, i in picked:
            if p.grad is None:
                continue
            vg = p.grad.detach().float()
            norm = vg.norm()
            grads.append(saved[n].reshape(-1).float().contiguous())
            sharps.append(self._flat_sharpness[i].reshape(-1).float().contiguous())
            grus.append(self._flat_gru_states[i])
            mf.append(self._flat_mamba_fwd_states[i])
            mb.append(self._flat_mamba_bwd_states[i])
            cots.append(-torch.where(norm > 1e-12, vg / norm, vg).reshape(-1))
        if grads:
            _bilevel.accumulate_meta_gradients(self.meta_net, grads, sharps, grus, mf, mb, cots)
            meta_optimizer.step()
            self._weights_dirty = True
        for n, p in named:
            p.grad = saved.get(n)
        return float(val_loss.item())
