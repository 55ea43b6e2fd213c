"""Host-side schedules shared by SuperGrok v1.5 and v2: alpha from the
train/val gap, warm-up ramp, sigmoid gates for lambda, weight decay and the
SAM / bilevel frequencies (reference: grokking_optimizers/supergrok2.py:222-268
and supergrok15.py:201-247, identical formulas in both classes)."""
import math


class GrokSchedule:
    # attributes expected on self: alpha_init, kappa, warmup_steps, warmup_ramp, zero_loss_threshold,
    # zero_acc_threshold, gate_scale/thresh, wd_ramp/scale/thresh, sam_*, bilevel_*, sam_enable_threshold,
    # _global_step, _cached_alpha, _cached_train_acc

    @staticmethod
    def _sigmoid(scale, value, thresh):
        return 1.0 / (1.0 + math.exp(-scale * (value - thresh)))

    def _update_alpha(self, train_loss, val_loss, train_acc):
        if train_loss is None and train_acc is None:
            return
        memorized = (train_acc is not None and train_acc >= self.zero_acc_threshold) or \
                    (train_loss is not None and train_loss < self.zero_loss_threshold)
        if memorized:
            signal = 10.0
        elif val_loss is not None and train_loss is not None and train_loss > 1e-12:
            signal = max(0.0, (val_loss - train_loss) / train_loss)
        else:
            signal = 0.0
        self._cached_alpha = self.alpha_init * math.exp(-self.kappa * signal)

    def _maybe_update_alpha(self, train_loss, val_loss, train_acc):
        """Refresh alpha on step 1, every alpha_update_freq steps, and whenever the run looks memorized."""
        if self._global_step % self.alpha_update_freq == 0 or self._global_step == 1:
            self._update_alpha(train_loss, val_loss, train_acc)
        elif train_acc is not None and train_acc >= self.zero_acc_threshold:
            self._update_alpha(train_loss, val_loss, train_acc)
        elif train_loss is not None and train_loss < self.zero_loss_threshold:
            self._update_alpha(train_loss, val_loss, train_acc)

    def _get_ramp_factor(self):
        if self._global_step <= self.warmup_steps:
            return 0.0
        return min(1.0, (self._global_step - self.warmup_steps) / self.warmup_ramp)

    def _get_effective_wd(self, base_wd):
        return base_wd * (1.0 + self.wd_ramp * self._sigmoid(self.wd_scale, self._cached_train_acc, self.wd_thresh))

    def _get_gate_signal(self):
        return self._sigmoid(self.gate_scale, self._cached_train_acc, self.gate_thresh)

    def _freq(self, fmin, fmax, scale, thresh):
        heat = self._sigmoid(scale, self._cached_train_acc, thresh)
        return max(1, round(fmax - (fmax - fmin) * heat))

    def _get_effective_sam_freq(self):
        if self._cached_train_acc < self.sam_enable_threshold:
            return 999999
        return self._freq(self.sam_freq_min, self.sam_freq_max, self.sam_scale, self.sam_thresh)

    def _get_effective_bilevel_freq(self):
        return self._freq(self.bilevel_freq_min, self.bilevel_freq_max, self.bilevel_scale, self.bilevel_thresh)

    @staticmethod
    def _layer_tables(param_groups, gamma, gamma_alpha):
        """Per-parameter beta1_i = beta1 (1-gamma)^i and alpha factor (1-gamma_alpha)^(max_idx-i)."""
        n = sum(len(g["params"]) for g in param_groups)
        beta1s, alphas, idx = [], [], 0
        for g in param_groups:
            for _ in g["params"]:
                beta1s.append(g["betas"][0] * ((1.0 - gamma) ** idx))
                alphas.append(1.0 if gamma_alpha == 0.0 else (1.0 - gamma_alpha) ** (max(n - 1, 1) - idx))
                idx += 1
        return beta1s, alphas
