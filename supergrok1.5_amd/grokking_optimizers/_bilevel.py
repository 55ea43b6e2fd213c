"""Differentiable pieces of the SuperGrok v2 meta-net used by bilevel training
(reference: Mamba3PEERMetaNet.forward_for_bilevel,
grokking_optimizers/mamba3_peer_metanet.py:372-436, driven from
grokking_optimizers/supergrok2.py:516-1371).

The optimizer's bilevel update (`accumulate_meta_gradients`) runs in HIP end to
end: sort + bidirectional Mamba-3 scan (sg2_bilevel_forward), per-element GRU /
soft top-4 PEER routing / expert MLPs forward and backward in one pass
(sg2_bilevel_elem), then the exact adjoint of the scan down to the gradients
of the scan's weights (sg2_bilevel_backward).
`forward_for_bilevel` is the module-level differentiable forward of one tensor
over the same kernels: the scan as one autograd Function (ScanContexts), the
per-element part as another (SoftElements over sg2_bilevel_elem).  `forward`
(hard top-1 routing, no gradients) is one call of sg2_meta_forward.  `per_element`
restates the per-element part in torch ops: the tests check sg2_bilevel_elem
against it, and it serves meta-nets whose routing sizes (heads, keys, experts)
the per-element bilevel kernel is not built for.  Scan blocks up to the default
(d_model 8, d_state 16, d_inner 16) run in HIP, smaller ones embedded; larger ones
take the scan blocks' own torch forward (chunked, on the GPU) under autograd.
"""
import torch

from grokking_optimizers import _cabi

def split_flat(flat, params):
    """Views of one flat gradient tensor, one per parameter, in order (no copies, no kernels)."""
    out, o = [], 0
    for p in params:
        out.append(flat[o:o + p.numel()].view(p.shape))
        o += p.numel()
    assert o == flat.numel()
    return out


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
        return (None,) + tuple(gr.to(w.dtype) for gr, w in zip(split_flat(ctx.plan.backward(d_out), W), W))


def scan_parameters(mn):
    """The 20 scan parameters of a Mamba3PEERMetaNet in the order ScanContexts expects."""
    out = [mn.input_proj.weight, mn.input_proj.bias]
    for blk in (mn.mamba_fwd, mn.mamba_bwd):
        out += [blk.in_proj.weight, blk.dt_proj.weight, blk.dt_proj.bias, blk.B_proj.weight, blk.C_proj.weight,
                blk.A_log, blk.D, blk.rope_freq, blk.out_proj.weight]
    return out


def meta_dims(mn):
    return dict(d_model=mn.d_model, d_state=mn.d_state, d_inner=mn.mamba_fwd.d_inner, gru_hidden=mn.gru_hidden,
                num_heads=mn.num_peer_heads, pk_dim=mn.pk_dim, expert_hidden=mn.expert_hidden, num_experts=mn.num_experts)


def make_plan(mn, grads, sharps, mamba_fwd, mamba_bwd):
    dev = grads[0].device
    if dev.type != "cuda":
        raise RuntimeError("the bilevel path of SuperGrok v2 needs GPU tensors: there is no CPU path")
    shape = (mn.mamba_fwd.d_inner, mn.d_state)
    zero = lambda m: torch.zeros(*shape, dtype=torch.float32, device=dev) if m is None else m
    return _cabi.Sg2Bilevel(mn.flat_weights(), [g.reshape(-1) for g in grads], [s.reshape(-1).to(g.dtype) for s, g in zip(sharps, grads)],
                            [zero(m) for m in mamba_fwd], [zero(m) for m in mamba_bwd], meta_dims(mn))


def per_element(mn, g, s, ctx_f, ctx_b, gru_state, topk=4):
    """GRU, soft top-k product-key routing (softmax of 10 x the k best scores of each sub-key, k*k experts per head)
    and the expert MLPs for N elements: smart gradient [N] and new GRU state
    (reference: Mamba3PEERMetaNet.forward_for_bilevel, mamba3_peer_metanet.py:395-436; GRU :178-192).
    topk=0: the hard top-1 routing of the optimizer step (Mamba3PEERMetaNet.forward, :319-367 there)."""
    gru = mn.gru
    xin = torch.cat([g.unsqueeze(-1), s.unsqueeze(-1), ctx_f, ctx_b], dim=-1)
    xh = torch.cat([xin, gru_state], dim=-1)
    z = torch.sigmoid(gru.W_z(xh))
    r = torch.sigmoid(gru.W_r(xh))
    cand = torch.tanh(gru.W_h(torch.cat([xin, r * gru_state], dim=-1)))
    h_new = (1 - z) * gru_state + z * cand
    pin = torch.cat([h_new, ctx_f, ctx_b, g.unsqueeze(-1), s.unsqueeze(-1)], dim=-1)
    N, half, pk = g.numel(), mn.d_model // 2, mn.pk_dim
    W1, b1 = mn.expert_W1.squeeze(-1), mn.expert_b1
    W2, b2 = mn.expert_W2.squeeze(1), mn.expert_b2.squeeze(-1)
    total = torch.zeros(N, device=g.device, dtype=torch.float32)
    for h in range(mn.num_peer_heads):
        q = mn.peer_queries[h](pin)
        if topk == 0:
            e = (q[:, :half] @ mn.product_keys_A[h].T).argmax(dim=-1) * pk + (q[:, half:] @ mn.product_keys_B[h].T).argmax(dim=-1)
            total = total + (W2[e] * torch.relu(W1[e] * g.unsqueeze(-1) + b1[e])).sum(-1) + b2[e]
            continue
        va, ia = (q[:, :half] @ mn.product_keys_A[h].T).topk(topk, dim=-1)
        vb, ib = (q[:, half:] @ mn.product_keys_B[h].T).topk(topk, dim=-1)
        wa, wb = torch.softmax(va * 10.0, dim=-1), torch.softmax(vb * 10.0, dim=-1)
        idx = (ia.unsqueeze(2) * pk + ib.unsqueeze(1)).reshape(N, -1)
        route = (wa.unsqueeze(2) * wb.unsqueeze(1)).reshape(N, -1)
        act = torch.relu(W1[idx] * g.reshape(N, 1, 1) + b1[idx])
        out = (W2[idx] * act).sum(-1) + b2[idx]
        total = total + (route * out).sum(dim=1)
    return g + mn.rescale * (total / mn.num_peer_heads), h_new


class SoftElements(torch.autograd.Function):
    """(smart_grad, new GRU state) of N elements from their two contexts, soft top-4 routing, through sg2_bilevel_elem
    (forward and backward are the same fused kernel: the forward call runs it with a zero cotangent).  Gradients
    reach the contexts and the 42 - 20 = 22 parameter tensors of the per-element part; the gradient, the sharpness
    and the old GRU state are data, and the new GRU state is returned without a gradient path (nothing in the
    reference differentiates through it)."""

    @staticmethod
    def forward(ctx, weights33, dims, rescale, g, s, h, contexts, *elem_params):
        smart, _, _, h_new = _cabi.bilevel_elem(weights33, g, s, contexts, h, torch.zeros_like(g), rescale, dims, want_gru=True)
        ctx.args = (weights33, dims, rescale)
        ctx.save_for_backward(g, s, h, contexts, *elem_params)
        ctx.mark_non_differentiable(h_new)
        return smart, h_new

    @staticmethod
    def backward(ctx, d_smart, _d_h):
        weights33, dims, rescale = ctx.args
        g, s, h, contexts = ctx.saved_tensors[:4]
        params = ctx.saved_tensors[4:]
        _, d_ctx, blk = _cabi.bilevel_elem(weights33, g, s, contexts, h, d_smart.contiguous(), rescale, dims, want_smart=False)
        return (None, None, None, None, None, None, d_ctx) + tuple(gr.to(p.dtype) for gr, p in zip(split_flat(blk, params), params))


def elem_kernel_fits(mn):
    """Whether sg2_bilevel_elem can run this net's per-element part: its routing sizes as built (4 heads, 12 x 12
    keys, 144 experts); context width, GRU width and expert width up to its own (smaller ones run embedded)."""
    d = meta_dims(mn)
    return ((d["num_heads"], d["pk_dim"], d["num_experts"]) == (4, 12, 144) and d["d_model"] <= _cabi.BILEVEL_SCAN_BLOCK[0]
            and d["gru_hidden"] <= _cabi.BILEVEL_GRU_HIDDEN and d["expert_hidden"] <= _cabi.BILEVEL_EXPERT_WIDTH)


def scan_kernels_fit(mn):
    """Whether the scan kernels of the bilevel pass can run this net's scan block (up to d_model 8, d_state 16,
    d_inner 16; smaller ones run embedded)."""
    dm, ds, di = _cabi.BILEVEL_SCAN_BLOCK
    return mn.d_model <= dm and mn.d_state <= ds and mn.mamba_fwd.d_inner <= di


TORCH_SCAN_LIMIT = 1 << 30      # numel * d_inner * d_state of one tensor on the torch-operation scan (4 GiB per coefficient array)


def torch_contexts(mn, g, s, mamba_fwd_state, mamba_bwd_state):
    """The two contexts of one tensor ([2, N, d_model], element order) and the new Mamba states through the scan
    blocks' own torch forward (Mamba3ScanBlock.forward, chunked), differentiable by autograd: the bilevel pass of
    scan blocks larger than its kernels are built for.  Same sort as the kernels: stable, by |g| with non-finite
    entries taken as 0."""
    n = g.numel()
    if n * mn.mamba_fwd.d_inner * mn.d_state > TORCH_SCAN_LIMIT:
        raise RuntimeError("the bilevel pass of a scan block larger than d_model 8, d_state 16, d_inner 16 runs in torch operations and "
                           "holds numel * d_inner * d_state floats per coefficient: %d elements exceed its limit of %d"
                           % (n, TORCH_SCAN_LIMIT // (mn.mamba_fwd.d_inner * mn.d_state)))
    g = torch.where(torch.isfinite(g), g, torch.zeros_like(g))
    s = torch.where(torch.isfinite(s), s, torch.zeros_like(s))
    perm = torch.sort(g.abs(), stable=True).indices
    x = mn.input_proj(torch.stack([g[perm], s[perm]], dim=-1))
    fwd, new_f = mn.mamba_fwd(x, mamba_fwd_state)
    bwd, new_b = mn.mamba_bwd(x.flip(0), mamba_bwd_state)
    inv = torch.empty_like(perm)
    inv[perm] = torch.arange(n, device=g.device)
    return torch.stack([fwd[inv], bwd.flip(0)[inv]]), new_f.detach(), new_b.detach()


def forward(mn, grad, sharpness, gru_state, mamba_fwd_state=None, mamba_bwd_state=None):
    """The step's own forward (hard top-1 routing) as a module call, for callers that use the meta-net outside the
    fused step: same return values as the reference's Mamba3PEERMetaNet.forward, computed by one call of
    sg2_meta_forward (sort, scan, GRU, routing, experts in HIP).  No gradient path: bilevel training differentiates
    forward_for_bilevel."""
    dev = grad.device
    if dev.type != "cuda":
        raise RuntimeError("the SuperGrok v2 meta-net needs GPU tensors: there is no CPU path")
    g = grad.reshape(-1).float().contiguous()
    s = sharpness.reshape(-1).float().contiguous()
    shape = (mn.mamba_fwd.d_inner, mn.d_state)
    state = lambda m: torch.zeros(*shape, dtype=torch.float32, device=dev) if m is None else m.detach().float().contiguous().clone()
    mf, mb = state(mamba_fwd_state), state(mamba_bwd_state)
    smart, h_new = _cabi.meta_forward(mn.flat_weights(), [g], [s], [gru_state], [mf], [mb], float(mn.rescale), meta_dims(mn),
                                      expert_counts=mn.expert_counts if mn.training else None)
    return smart.reshape(grad.shape).to(grad.dtype), h_new, mf, mb


def forward_for_bilevel(mn, grad, sharpness, gru_state, mamba_fwd_state=None, mamba_bwd_state=None):
    """Differentiable forward of one tensor, the reference's return values: (smart_grad, new_gru, new_mamba_fwd_state,
    new_mamba_bwd_state); gradients reach every parameter of `mn` (the new states are plain tensors: nothing in
    the reference differentiates through them)."""
    g = grad.reshape(-1).float()
    s = sharpness.reshape(-1).float()
    if g.device.type != "cuda":
        raise RuntimeError("the bilevel path of SuperGrok v2 needs GPU tensors: there is no CPU path")
    if scan_kernels_fit(mn):
        plan = make_plan(mn, [g], [s], [mamba_fwd_state], [mamba_bwd_state])
        ctx = ScanContexts.apply(plan, *scan_parameters(mn))
        new_f, new_b, weights33 = plan.mf[0], plan.mb[0], plan.weights
    else:
        ctx, new_f, new_b = torch_contexts(mn, g, s, mamba_fwd_state, mamba_bwd_state)
        weights33 = None
    if elem_kernel_fits(mn):
        smart, h_new = SoftElements.apply(mn.flat_weights() if weights33 is None else weights33, meta_dims(mn), float(mn.rescale),
                                          g.contiguous(), s.contiguous(), gru_state.detach().float().contiguous(), ctx, *elem_parameters(mn))
    else:
        smart, h_new = per_element(mn, g, s, ctx[0], ctx[1], gru_state.float())
    return smart.reshape(grad.shape).to(grad.dtype), h_new, new_f, new_b


def elem_parameters(mn):
    """The parameters of the per-element part in the order of sg2_bilevel_elem's gradient block."""
    out = []
    for lin in (mn.gru.W_z, mn.gru.W_r, mn.gru.W_h):
        out += [lin.weight, lin.bias]
    out += [q.weight for q in mn.peer_queries] + list(mn.product_keys_A) + list(mn.product_keys_B)
    return out + [mn.expert_W1, mn.expert_b1, mn.expert_W2, mn.expert_b2]


def _add_grads(params, flat):
    """p.grad (+)= its slice of `flat`; a parameter without a gradient gets a view of the flat tensor."""
    for p, gr in zip(params, split_flat(flat, params)):
        if p.requires_grad:
            gr = gr if gr.dtype == p.dtype else gr.to(p.dtype)
            p.grad = gr if p.grad is None else p.grad + gr


def accumulate_meta_gradients(mn, grads, sharps, gru_states, mamba_fwd, mamba_bwd, cotangents):
    """Adds the gradient of  sum_p <smart_grad_p, cotangent_p>  with respect to every parameter of `mn` to its
    .grad, for a list of tensors at once, all in HIP: scan forward (sg2_bilevel_forward), per-element forward and
    backward (sg2_bilevel_elem), scan adjoint (sg2_bilevel_backward).  Returns the smart gradients (flat, packed)."""
    if not scan_kernels_fit(mn):
        # a scan block larger than the bilevel kernels are built for: tensor by tensor through the autograd form
        params = [p for p in mn.parameters() if p.requires_grad]
        smarts = []
        for g, s, h, f, b, c in zip(grads, sharps, gru_states, mamba_fwd, mamba_bwd, cotangents):
            with torch.enable_grad():
                smart = forward_for_bilevel(mn, g.reshape(-1), s.reshape(-1), h, f, b)[0].float()
                got = torch.autograd.grad((smart * c.reshape(-1).float()).sum(), params, allow_unused=True)
            for p, gr in zip(params, got):
                if gr is not None:
                    p.grad = gr if p.grad is None else p.grad + gr
            smarts.append(smart.detach())
        return torch.cat(smarts)
    plan = make_plan(mn, grads, sharps, mamba_fwd, mamba_bwd)
    g_all = torch.cat([g.reshape(-1).float() for g in grads])
    s_all = torch.cat([s.reshape(-1).float() for s in sharps])
    h_all = torch.cat([h.float() for h in gru_states])
    c_all = torch.cat([c.reshape(-1).float() for c in cotangents])
    if not elem_kernel_fits(mn):
        # routing sizes the per-element kernel is not built for: the scan and its adjoint in HIP, the per-element part
        # and its derivative as torch operations on the GPU
        with torch.enable_grad():
            ctx = ScanContexts.apply(plan, *scan_parameters(mn))
            smart, _ = per_element(mn, g_all, s_all, ctx[0], ctx[1], h_all)
            params = [p for p in mn.parameters() if p.requires_grad]
            for p, gr in zip(params, torch.autograd.grad((smart * c_all).sum(), params, allow_unused=True)):
                if gr is not None:
                    p.grad = gr if p.grad is None else p.grad + gr
        return smart.detach()
    ctx = plan.forward()
    smart, d_ctx, blk = _cabi.bilevel_elem(plan.weights, g_all, s_all, ctx, h_all, c_all, float(mn.rescale), meta_dims(mn))
    _add_grads(elem_parameters(mn), blk)
    _add_grads(scan_parameters(mn), plan.backward(d_ctx))
    return smart


def scan_contexts(weights33, scan_params, grads, sharps, mamba_fwd, mamba_bwd, dims=None):
    """weights33: the 33 flat fp32 weight tensors in `_ops` order (values); scan_params: the 20 tensors, in the
    order ScanContexts documents, that gradients should flow to.  Returns [2, sum numel, d_model]."""
    plan = _cabi.Sg2Bilevel(weights33, grads, sharps, mamba_fwd, mamba_bwd, dims)
    return ScanContexts.apply(plan, *scan_params)
