"""Training-loop helpers shared by SuperGrok v1.1 and v1.5: the SAM sharpness
probe and the one-step bilevel update of the sharpness meta-net
(reference: grokking_optimizers/supergrok15.py:307-413 and
supergrok11.py:196-285, the same code in both classes).

The elementwise work runs through `_ops`: the global gradient norm and the
ascent step p + rho*g/|g| in `supergrok15_sam_perturb_all` (norm reduced on the
device, no host sync), |g_sam - g| in `supergrok15_sharpness_restore_all`.
Forward/backward passes are the caller's model under torch autograd.

One deliberate difference: the reference builds the perturbed parameters from
detached tensors and then calls `backward()`, which leaves nothing to
differentiate; here the perturbed copies require grad and the SAM gradient is
taken with respect to them.
"""
import torch
import torch.nn as nn

from grokking_optimizers import _ops

# expected on self: _ensure_state(), _param_to_idx, _flat_sharpness, sam_rho, meta_net, _weights_dirty


class MetaTraining:
    def sam_step(self, model, train_x, train_y, criterion):
        """sharpness[p] <- |grad at (params + rho*g/|g|) - g| for every parameter with a gradient; returns the
        loss at the perturbed point.  Parameters and their .grad are left as they were."""
        self._ensure_state()
        named = list(model.named_parameters())
        names = [n for n, p in named if p.grad is not None and p.grad.numel() > 0]
        if not names:
            return 0.0
        by_name = dict(named)
        grads = [by_name[n].grad.detach().clone() for n in names]
        perturbed = {n: p.detach() for n, p in named}
        moved = [by_name[n].detach().clone() for n in names]
        with torch.no_grad():
            originals = _ops.supergrok15_sam_perturb_all(moved, grads, self.sam_rho)
        for n, t in zip(names, moved):
            perturbed[n] = t.requires_grad_(True)
        with torch.enable_grad():
            sam_loss = criterion(torch.func.functional_call(model, perturbed, (train_x,)), train_y)
            sam_grads = torch.autograd.grad(sam_loss, moved, allow_unused=True)
        keep = [k for k, n in enumerate(names) if sam_grads[k] is not None and id(by_name[n]) in self._param_to_idx]
        if keep:
            sg = [sam_grads[k].detach().contiguous() for k in keep]
            ng = [grads[k] for k in keep]
            sharp = [torch.empty_like(g) for g in ng]
            with torch.no_grad():
                # also puts the original values back into the scratch copies; only the sharpness is used
                _ops.supergrok15_sharpness_restore_all([moved[k].detach() for k in keep], sharp, [originals[k] for k in keep], sg, ng)
            for k, s in zip(keep, sharp):
                self._flat_sharpness[self._param_to_idx[id(by_name[names[k]])]] = s.reshape(-1).float()
        return float(sam_loss.item())

    def _meta_update(self, model, val_x, val_y, criterion, meta_optimizer):
        """One meta-net step on  -sum_p <smart_grad_p, val_grad_p/|val_grad_p|>  (alignment of the meta-net's output
        with the validation gradient); .grad of the model is restored afterwards."""
        self._ensure_state()
        named = list(model.named_parameters())
        saved = {n: p.grad.detach().clone() for n, p in named if p.grad is not None}
        names = [n for n, _ in named if n in saved]
        smart = {}
        if names:
            by_name = dict(named)
            flat_g, flat_s = [], []
            for n in names:
                idx = self._param_to_idx.get(id(by_name[n]))
                flat_g.append(saved[n].reshape(-1).float())
                flat_s.append(self._flat_sharpness[idx].reshape(-1) if idx is not None
                              else torch.zeros(saved[n].numel(), device=saved[n].device))
            with torch.enable_grad():
                out = self.meta_net(torch.cat(flat_g), torch.cat(flat_s))
            off = 0
            for n in names:
                k = saved[n].numel()
                smart[n] = out[off:off + k].reshape(saved[n].shape)
                off += k
        model.zero_grad()
        with torch.enable_grad():
            val_loss = criterion(model(val_x), val_y)
            val_loss.backward()
        meta_optimizer.zero_grad()
        with torch.enable_grad():
            meta_loss = torch.zeros((), device=val_x.device)
            for n, p in named:
                if n in smart and p.grad is not None:
                    vg = p.grad.detach().float()
                    norm = vg.norm()
                    meta_loss = meta_loss - (smart[n] * (vg / norm if norm > 1e-12 else vg)).sum()
            if meta_loss.requires_grad:
                meta_loss.backward()
                meta_optimizer.step()
        self._weights_dirty = True
        for n, p in named:
            p.grad = saved.get(n)
        return float(val_loss.item())

    def get_global_step(self):
        return self._global_step


class ScheduledTraining:
    """The training-loop entry points SuperGrok v1.5 and v2 share (reference: supergrok15.py:415-478 and
    supergrok2.py:1373-1440): expects sam_step, bilevel_step, step, the adaptive-frequency getters of GrokSchedule
    and meta_net on self."""

    def sam_meta_step(self, model, train_x, train_y, val_x, val_y, criterion, meta_optimizer):
        return (self.sam_step(model, train_x, train_y, criterion),
                self.bilevel_step(model, train_x, train_y, val_x, val_y, criterion, meta_optimizer))

    def get_cached_alpha(self):
        return self._cached_alpha

    def get_effective_wd(self):
        return self._get_effective_wd(self.param_groups[0]["weight_decay"]) if self.param_groups else 0.0

    def step_full(self, model, train_x, train_y, val_x, val_y, criterion=None):
        """Forward + backward + (at their adaptive frequencies) SAM probe and bilevel update + optimizer step;
        returns the metrics it computed.  Unlike the reference, errors of the SAM probe and of the bilevel update
        are not swallowed."""
        criterion = nn.CrossEntropyLoss() if criterion is None else criterion
        if not hasattr(self, "_auto_meta_opt"):
            self._auto_meta_opt = torch.optim.Adam(self.meta_net.parameters(), lr=1e-4)
        model.zero_grad()
        logits = model(train_x)
        loss = criterion(logits, train_y)
        loss.backward()
        metrics = {}
        step_num = self._global_step + 1
        if step_num % self._get_effective_sam_freq() == 0:
            metrics["sam_loss"] = self.sam_step(model, train_x, train_y, criterion)
        if step_num % self._get_effective_bilevel_freq() == 0:
            metrics["val_loss"] = self.bilevel_step(model, train_x, train_y, val_x, val_y, criterion, self._auto_meta_opt)
        kw = {}
        if step_num % self.alpha_update_freq == 0 or step_num == 1:
            with torch.no_grad():
                kw["train_loss"] = metrics["train_loss"] = float(loss.item())
                kw["train_acc"] = metrics["train_acc"] = float((logits.detach().argmax(-1) == train_y).float().mean().item())
                if step_num % self.alpha_update_freq == 0:
                    kw["val_loss"] = float(criterion(model(val_x), val_y).item())
                    metrics.setdefault("val_loss", kw["val_loss"])
        self.step(**kw)
        return metrics
