"""AdamW over a list of tensors with ATen ops: the update Muon applies to its
non-2D parameter group (reference: grokking_optimizers/_adamw_helper.py:12-22;
decay first, bias corrections in Python double, denom = sqrt(v/bc2) + eps)."""
import torch


@torch.no_grad()
def adamw_step(params, grads, exp_avgs, exp_avg_sqs, steps, lr, beta1, beta2, eps, wd):
    for p, g, m, v, t in zip(params, grads, exp_avgs, exp_avg_sqs, steps):
        bc1, bc2 = 1.0 - beta1 ** t, 1.0 - beta2 ** t
        m.mul_(beta1).add_(g, alpha=1 - beta1)
        v.mul_(beta2).addcmul_(g, g, value=1 - beta2)
        denom = (v / bc2).sqrt().add_(eps)
        p.mul_(1 - lr * wd)
        p.addcdiv_(m, denom, value=-(lr / bc1))
