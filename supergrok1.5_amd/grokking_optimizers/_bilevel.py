"""Differentiable pieces of the SuperGrok v2 meta-net used by bilevel training
(reference: Mamba3PEERMetaNet.forward_for_bilevel,
grokking_optimizers/mamba3_peer_metanet.py:372-436, driven from
grokking_optimizers/supergrok2.py:516-1371).

The sequential part - magnitude sort and bidirectional Mamba-3 scan - runs in
HIP, forward and backward (`ScanContexts`, over sg2_bilevel_forward /
sg2_bilevel_backward); what follows per element (GRU, soft top-4 PEER routing,
expert MLPs) is dense tensor algebra and is left to torch autograd.
"""
import torch

from grokking_optimizers import _cabi

GROUP_ROWS = 16


def compose_coefficients(Win, bin_, in_proj, dt_W, dt_b, Bp, Cp):
    """[5, 16, 3] coefficient triples (c_g, c_s, c_0) of x-branch, z, dt_raw, B, C as affine functions of an
    element's (gradient, sharpness): the same composition include/sg2_compose.h performs on the device, as
    differentiable torch algebra (float64), used to carry the coefficient gradients back to the raw weights."""
    f = torch.float64
    src = torch.cat([Win.to(f), bin_.to(f).unsqueeze(1)], dim=1)            # [d_model, 3]
    di = dt_W.shape[0]
    xb = in_proj.to(f)[:di] @ src                                            # [d_inner, 3]
    z = in_proj.to(f)[di:] @ src
    dt = dt_W.to(f) @ xb
    dt = dt + torch.stack([torch.zeros_like(dt_b, dtype=f), torch.zeros_like(dt_b, dtype=f), dt_b.to(f)], dim=1)
    return torch.stack([xb, z, dt, Bp.to(f) @ xb, Cp.to(f) @ xb], dim=0)


class ScanContexts(torch.autograd.Function):
    """(fwd_ctx, bwd_ctx) of every element of a list of tensors as a function of the 20 scan weights
    (input_proj W, b; then in_proj, dt_W, dt_b, B_proj, C_proj, A_log, D, rope_freq, out_proj for each direction)."""

    @staticmethod
    def forward(ctx, plan, *scan_weights):
        out = plan.forward()
        ctx.plan = plan
        ctx.save_for_backward(*scan_weights)
        return out

    @staticmethod
    def backward(ctx, d_out):
        W = ctx.saved_tensors
        blk = ctx.plan.backward(d_out).double()                              # [2, SG2_BWD_STRIDE]
        grads = [None] * 20
        d_in_W = torch.zeros_like(W[0], dtype=torch.float64)
        d_in_b = torch.zeros_like(W[1], dtype=torch.float64)
        for d in range(2):
            base = 2 + 9 * d
            in_proj, dt_W, dt_b, Bp, Cp, A_log, D, rope, out_proj = W[base:base + 9]
            o = 0
            dcomp = blk[d, o:o + 5 * GROUP_ROWS * 3].reshape(5, GROUP_ROWS, 3); o += 5 * GROUP_ROWS * 3
            d_alog = blk[d, o:o + A_log.numel()].reshape(A_log.shape); o += A_log.numel()
            d_rope = blk[d, o:o + rope.numel()].reshape(rope.shape); o += rope.numel()
            d_D = blk[d, o:o + D.numel()].reshape(D.shape); o += D.numel()
            d_out_proj = blk[d, o:o + out_proj.numel()].reshape(out_proj.shape)
            with torch.enable_grad():
                raw = [t.detach().double().requires_grad_(True) for t in (W[0], W[1], in_proj, dt_W, dt_b, Bp, Cp)]
                comp = compose_coefficients(*raw)
                g = torch.autograd.grad(comp, raw, grad_outputs=dcomp)
            d_in_W += g[0]
            d_in_b += g[1]
            grads[base:base + 9] = [g[2], g[3], g[4], g[5], g[6], d_alog, d_D, d_rope, d_out_proj]
        grads[0], grads[1] = d_in_W, d_in_b
        return (None,) + tuple(gr.to(w.dtype) for gr, w in zip(grads, W))


def scan_contexts(weights33, scan_params, grads, sharps, mamba_fwd, mamba_bwd, dims=None):
    """weights33: the 33 flat fp32 weight tensors in `_ops` order (values); scan_params: the 20 tensors, in the
    order ScanContexts documents, that gradients should flow to.  Returns [2, sum numel, d_model]."""
    plan = _cabi.Sg2Bilevel(weights33, grads, sharps, mamba_fwd, mamba_bwd, dims)
    return ScanContexts.apply(plan, *scan_params)
