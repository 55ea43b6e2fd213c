"""AdamW over a list of tensors: the update Muon applies to its non-2D parameter
group and LookSAM applies in `step()` (reference:
grokking_optimizers/_adamw_helper.py:12-22; decay first, bias corrections in
Python double, denom = sqrt(v/bc2) + eps).  One fused launch over all tensors
(`_ops.adamw_fused_step`) instead of six ATen calls per tensor."""
import torch

from grokking_optimizers import _ops


@torch.no_grad()
def adamw_step(params, grads, exp_avgs, exp_avg_sqs, steps, lr, beta1, beta2, eps, wd):
    if params:
        _ops.adamw_fused_step(list(params), list(grads), list(exp_avgs), list(exp_avg_sqs), [int(t) for t in steps],
                              float(lr), float(beta1), float(beta2), float(eps), float(wd))
