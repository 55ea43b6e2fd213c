"""The reference's bilevel entry points through `_ops`
(supergrok2_bilevel_fwd_save_batched / supergrok2_bilevel_backward_batched / supergrok2_bilevel_fwd_save /
supergrok2_bilevel_backward, with the argument lists of csrc/ops.h:232-371 of the reference), driven the way the reference's own caller drives them
(grokking_optimizers/supergrok2.py:646-1040 there): packed buffers allocated by the caller, out_proj / unsort / GRU /
soft top-4 routing / experts in torch between the two calls, input_proj gradients from d_x_sorted afterwards.
Checked against float64 autograd through the restatement of the whole differentiable forward
(ref_fp64.forward_for_bilevel, pinned on the CPU by tests/test_oracle_sg2_pins.py): every one of the 42 parameter
gradients within 2e-4 of its largest entry."""
import copy

import numpy as np
import pytest
import torch

import ref_fp64

pytestmark = pytest.mark.gpu


def _meta_net(seed, dev):
    from grokking_optimizers import Mamba3PEERMetaNet
    torch.manual_seed(seed)
    mn = Mamba3PEERMetaNet()
    with torch.no_grad():       # the initial keys and experts are nearly silent: give every part a visible gradient
        for p in mn.parameters():
            if p.dim() > 0 and float(p.abs().max()) < 0.05:
                p.add_(torch.randn_like(p) * 0.2)
    return mn.to(dev)


def _flat64(mn):
    blk = lambda b: [b.in_proj.weight, b.dt_proj.weight, b.dt_proj.bias, b.B_proj.weight, b.C_proj.weight, b.A_log, b.D,
                     b.rope_freq, b.out_proj.weight]
    E = mn.num_experts
    return ([mn.input_proj.weight, mn.input_proj.bias] + blk(mn.mamba_fwd) + blk(mn.mamba_bwd) +
            [mn.gru.W_z.weight, mn.gru.W_z.bias, mn.gru.W_r.weight, mn.gru.W_r.bias, mn.gru.W_h.weight, mn.gru.W_h.bias] +
            [torch.stack([q.weight for q in mn.peer_queries]), torch.stack(list(mn.product_keys_A)), torch.stack(list(mn.product_keys_B))] +
            [mn.expert_W1.reshape(E, -1), mn.expert_b1, mn.expert_W2.reshape(E, -1), mn.expert_b2.reshape(-1)])


MAMBA = ("in_proj", "dt_proj_W", "dt_proj_b", "B_proj", "C_proj", "A_log", "D", "rope_freq")


def _mamba_args(w, tag, with_out):
    names = MAMBA + (("out_proj",) if with_out else ())
    return [w[f"mamba_{tag}_{n}"] for n in names]


def test_reference_batched_bilevel_entry_points():
    from grokking_optimizers import _bilevel, _ops
    dev = torch.device("cuda:0")
    mn = _meta_net(5, dev)
    mn64 = copy.deepcopy(mn).double().cpu()
    gen = torch.Generator().manual_seed(23)
    Ns = [150, 99, 1300, 64]
    data = [dict(g=torch.randn(n, generator=gen) * 0.5, s=torch.rand(n, generator=gen) * 0.3, h=torch.randn(n, 4, generator=gen) * 0.5,
                 hf=torch.randn(16, 16, generator=gen) * 0.3, hb=torch.randn(16, 16, generator=gen) * 0.3, R=torch.randn(n, generator=gen))
            for n in Ns]
    # ---- float64 reference: gradient of sum_p <smart_p, R_p> with respect to all 42 parameters
    dims = dict(d_model=8, num_heads=4, pk_dim=12)
    for d in data:
        smart, _, _, _ = ref_fp64.forward_for_bilevel(_flat64(mn64), d["g"].double(), d["s"].double(), d["h"].double(), d["hf"].double(),
                                                      d["hb"].double(), mn64.rescale, dims)
        (smart * d["R"].double()).sum().backward()
        d["smart64"] = smart.detach()
    ref = {n: p.grad.clone() for n, p in mn64.named_parameters()}

    # ---- the reference caller's sequence
    w = mn.get_weights()
    w = {k: (v.to(dev) if torch.is_tensor(v) else v) for k, v in w.items()}
    d_model, d_state, d_inner = 8, 16, 16
    total, P = sum(Ns), len(Ns)
    z = lambda *s: torch.zeros(*s, device=dev)
    fwd_scan, bwd_scan = z(total, d_inner), z(total, d_inner)
    saved = [z(total, d_inner, d_state)] + [z(total, d_inner) for _ in range(3)] + [z(total, d_inner, d_state)] + [z(total, d_inner) for _ in range(3)]
    x_sorted, offsets_t = z(total, d_model), torch.zeros(P + 1, dtype=torch.int32, device=dev)
    sort_idx = torch.zeros(total, dtype=torch.int32, device=dev)
    init_f = torch.stack([d["hf"] for d in data]).to(dev)
    init_b = torch.stack([d["hb"] for d in data]).to(dev)
    init_f0, init_b0 = init_f.clone(), init_b.clone()
    grads = [d["g"].to(dev) for d in data]
    sharps = [d["s"].to(dev) for d in data]
    print("fwd_save_batched", Ns, flush=True)
    _ops.supergrok2_bilevel_fwd_save_batched(grads, sharps, w["input_proj_W"], w["input_proj_b"], *_mamba_args(w, "fwd", True),
                                             *_mamba_args(w, "bwd", True), d_model, d_state, d_inner, fwd_scan, bwd_scan, *saved,
                                             x_sorted, offsets_t, sort_idx, init_f, init_b, 1)
    torch.cuda.synchronize()
    assert torch.equal(init_f, init_f0) and torch.equal(init_b, init_b0)         # the caller's states are not touched
    offs = np.concatenate([[0], np.cumsum(Ns)])
    assert np.array_equal(offsets_t.cpu().numpy(), offs)
    for i, d in enumerate(data):                                                  # sort order and x_sorted
        a, b = int(offs[i]), int(offs[i + 1])
        want = torch.sort(d["g"].abs(), stable=True).indices
        assert torch.equal(sort_idx[a:b].cpu().long(), want)
        xs = torch.stack([d["g"][want], d["s"][want]], -1) @ w["input_proj_W"].cpu().T + w["input_proj_b"].cpu()
        assert torch.allclose(x_sorted[a:b].cpu(), xs, rtol=1e-5, atol=1e-6)

    # between the calls: out_proj, unsort, GRU, soft routing, experts in torch (fp32, autograd), as the caller does
    for p in mn.parameters():
        p.grad = None
    fs = fwd_scan.clone().requires_grad_(True)
    bs = bwd_scan.clone().requires_grad_(True)
    loss = torch.zeros((), device=dev)
    smarts = []
    for i, d in enumerate(data):
        a, b = int(offs[i]), int(offs[i + 1])
        unsort = sort_idx[a:b].long().argsort()
        ctx_f = (fs[a:b] @ mn.mamba_fwd.out_proj.weight.T)[unsort]
        ctx_b = (bs[a:b] @ mn.mamba_bwd.out_proj.weight.T).flip(0)[unsort]
        smart, _ = _bilevel.per_element(mn, grads[i], sharps[i], ctx_f, ctx_b, d["h"].to(dev))
        loss = loss + (smart * d["R"].to(dev)).sum()
        smarts.append(smart.detach())
        err = (smart.detach().double().cpu() - d["smart64"]).abs()
        assert bool((err <= 1e-4 * d["smart64"].abs() + 1e-6).all()), ("smart", i, float(err.max()))
    loss.backward()

    d_mamba = [torch.zeros_like(t) for t in _mamba_args(w, "fwd", False) + _mamba_args(w, "bwd", False)]
    d_x_sorted = z(total, d_model)
    print("backward_batched", flush=True)
    _ops.supergrok2_bilevel_backward_batched(fs.grad.contiguous(), bs.grad.contiguous(), x_sorted, *saved, offsets_t,
                                             *_mamba_args(w, "fwd", False), *_mamba_args(w, "bwd", False), *d_mamba, d_x_sorted,
                                             init_f, init_b, d_model, d_state, d_inner, P, 1)
    torch.cuda.synchronize()
    # input_proj from d_x_sorted, as the caller does
    dW, db = z(d_model, 2), z(d_model)
    for i, d in enumerate(data):
        a, b = int(offs[i]), int(offs[i + 1])
        unsort = sort_idx[a:b].long().argsort()
        dxu = d_x_sorted[a:b].index_select(0, unsort)
        dW.addmm_(dxu.T, torch.stack([grads[i], sharps[i]], -1))
        db.add_(dxu.sum(0))

    got = {"input_proj.weight": dW, "input_proj.bias": db}
    tags = {"in_proj": "in_proj.weight", "dt_proj_W": "dt_proj.weight", "dt_proj_b": "dt_proj.bias", "B_proj": "B_proj.weight",
            "C_proj": "C_proj.weight", "A_log": "A_log", "D": "D", "rope_freq": "rope_freq"}
    for k, tag in enumerate(("fwd", "bwd")):
        for q, n in enumerate(MAMBA):
            got[f"mamba_{tag}.{tags[n]}"] = d_mamba[k * 8 + q]
    for n, p in mn.named_parameters():
        if n not in got:
            got[n] = p.grad if p.grad is not None else torch.zeros_like(p)
    worst = {}
    for n, r in ref.items():
        g = got[n].double().cpu().reshape(r.shape)
        scale = float(r.abs().max())
        worst[n] = round(float((g - r).abs().max()) / (2e-4 * scale + 1e-12), 3)
    print("worst gradient tolerance ratios", worst, flush=True)
    assert max(worst.values()) <= 1.0, worst
    # a second backward call on the same buffers has nothing to restart from
    with pytest.raises(RuntimeError, match="already run"):
        _ops.supergrok2_bilevel_backward_batched(fs.grad.contiguous(), bs.grad.contiguous(), x_sorted, *saved, offsets_t,
                                                 *_mamba_args(w, "fwd", False), *_mamba_args(w, "bwd", False), *d_mamba, d_x_sorted,
                                                 init_f, init_b, d_model, d_state, d_inner, P, 1)


def _single_tensor_pass(mn, w, d, dev, acc):
    """One parameter through supergrok2_bilevel_fwd_save -> the caller's torch forward of the per-element part ->
    supergrok2_bilevel_backward, as grokking_optimizers/supergrok2.py:1030-1290 of the reference does it.  `acc`: the
    dict of gradient accumulators (the d_* arguments).  Returns the smart gradient."""
    from grokking_optimizers import _ops
    n = d["g"].numel()
    d_model, d_state, d_inner, gh, H, topk, pk, eh, E = 8, 16, 16, 4, 4, 4, 12, 16, 144
    num_active, half = topk * topk, d_model // 2
    g, s = d["g"].to(dev), d["s"].to(dev)
    z = lambda *sh: torch.zeros(*sh, device=dev)
    fs, bs, ff, fb = z(n, d_inner), z(n, d_inner), z(d_inner, d_state), z(d_inner, d_state)
    saved = [z(n, d_inner, d_state)] + [z(n, d_inner) for _ in range(3)] + [z(n, d_inner, d_state)] + [z(n, d_inner) for _ in range(3)]
    xs, si = z(n, d_model), torch.zeros(n, dtype=torch.int32, device=dev)
    hf, hb = d["hf"].to(dev), d["hb"].to(dev)
    _ops.supergrok2_bilevel_fwd_save(g, s, w["input_proj_W"], w["input_proj_b"], *_mamba_args(w, "fwd", True), *_mamba_args(w, "bwd", True),
                                     d_model, d_state, d_inner, fs, bs, ff, fb, *saved, xs, si, hf, hb, 1)
    with torch.no_grad():
        unsort = si.long().argsort()
        fwd_ctx = (fs @ w["mamba_fwd_out_proj"].T)[unsort]
        bwd_ctx = (bs @ w["mamba_bwd_out_proj"].T).flip(0)[unsort]
        gru_inp = torch.cat([g[:, None], s[:, None], fwd_ctx, bwd_ctx], -1)
        h_old = d["h"].to(dev)
        xh = torch.cat([gru_inp, h_old], -1)
        z_gate = torch.sigmoid(xh @ w["gru_Wz"].T + w["gru_bz"])
        r_gate = torch.sigmoid(xh @ w["gru_Wr"].T + w["gru_br"])
        h_tilde = torch.tanh(torch.cat([gru_inp, r_gate * h_old], -1) @ w["gru_Wh"].T + w["gru_bh"])
        h_new = (1 - z_gate) * h_old + z_gate * h_tilde
        peer_inp = torch.cat([h_new, fwd_ctx, bwd_ctx, g[:, None], s[:, None]], -1)
        Wq = torch.stack([q.weight for q in mn.peer_queries])
        KA, KB = torch.stack(list(mn.product_keys_A)), torch.stack(list(mn.product_keys_B))
        W1, b1 = mn.expert_W1.reshape(E, eh), mn.expert_b1
        W2, b2 = mn.expert_W2.reshape(E, eh), mn.expert_b2.reshape(E)
        e_idx = torch.zeros(n, H, num_active, dtype=torch.int32, device=dev)
        r_w, z_hid = z(n, H, num_active), z(n, H, num_active, eh)
        sc_a, sc_b = z(n, H, pk), z(n, H, pk)
        ta, tb = torch.zeros(n, H, topk, dtype=torch.int32, device=dev), torch.zeros(n, H, topk, dtype=torch.int32, device=dev)
        so_a, so_b = z(n, H, topk), z(n, H, topk)
        total = z(n)
        for h in range(H):
            q = peer_inp @ Wq[h].T
            scores_a, scores_b = q[:, :half] @ KA[h].T, q[:, half:] @ KB[h].T
            sc_a[:, h], sc_b[:, h] = scores_a, scores_b
            va, ia = scores_a.topk(topk, dim=-1)
            vb, ib = scores_b.topk(topk, dim=-1)
            ta[:, h], tb[:, h] = ia.int(), ib.int()
            sa, sb = torch.softmax(va * 10.0, -1), torch.softmax(vb * 10.0, -1)
            so_a[:, h], so_b[:, h] = sa, sb
            idx = (ia.unsqueeze(2) * pk + ib.unsqueeze(1)).reshape(n, num_active)
            rw = (sa.unsqueeze(2) * sb.unsqueeze(1)).reshape(n, num_active)
            e_idx[:, h], r_w[:, h] = idx.int(), rw
            zz = torch.relu(W1[idx] * g[:, None, None] + b1[idx])
            z_hid[:, h] = zz
            total = total + (rw * ((W2[idx] * zz).sum(-1) + b2[idx])).sum(-1) / H
        smart = g + mn.rescale * total
    d_smart = d["R"].to(dev)
    A = acc
    _ops.supergrok2_bilevel_backward(
        d_smart, g, s, float(mn.rescale), si, xs, fs, bs, *saved, gru_inp.contiguous(), h_old.contiguous(), z_gate.contiguous(),
        r_gate.contiguous(), h_tilde.contiguous(), peer_inp.contiguous(), e_idx, r_w, z_hid, sc_a, sc_b, ta, tb, so_a, so_b,
        *_mamba_args(w, "fwd", True), *_mamba_args(w, "bwd", True), w["gru_Wz"], w["gru_Wr"], w["gru_Wh"], Wq.contiguous(), KA.contiguous(),
        KB.contiguous(), W1.contiguous(), W2.contiguous(), b1, b2.contiguous(), w["input_proj_W"], hf, hb,
        *[A["mamba_fwd." + k] for k in MAMBA_PARAMS], A["mamba_fwd.out_proj.weight"],
        *[A["mamba_bwd." + k] for k in MAMBA_PARAMS], A["mamba_bwd.out_proj.weight"],
        A["gru.W_z.weight"], A["gru.W_z.bias"], A["gru.W_r.weight"], A["gru.W_r.bias"], A["gru.W_h.weight"], A["gru.W_h.bias"],
        A["peer_queries"], A["product_keys_A"], A["product_keys_B"], A["expert_W1"], A["expert_b1"], A["expert_W2"], A["expert_b2"],
        A["input_proj.weight"], A["input_proj.bias"], d_model, d_state, d_inner, gh, 2 + 2 * d_model, H, topk, pk, eh, gh + 2 * d_model + 2, E, 1)
    return smart, (fs, bs, ff, fb, si, saved, xs)


MAMBA_PARAMS = ("in_proj.weight", "dt_proj.weight", "dt_proj.bias", "B_proj.weight", "C_proj.weight", "A_log", "D", "rope_freq")


def test_reference_single_tensor_bilevel_pair():
    """supergrok2_bilevel_fwd_save + supergrok2_bilevel_backward (one tensor, every weight of the meta-net), three
    parameters in turn accumulating into one set of d_* tensors like the reference's loop, two of them interleaved
    (forward A, forward B, backward A, backward B: each backward call must find its own forward call).  All 42
    gradients against float64 autograd; the scan outputs and final states of the forward call against the float64 scan."""
    from grokking_optimizers import _ops
    dev = torch.device("cuda:0")
    mn = _meta_net(9, dev)
    mn64 = copy.deepcopy(mn).double().cpu()
    w = {k: (v.to(dev) if torch.is_tensor(v) else v) for k, v in mn.get_weights().items()}
    w["gru_Wz"], w["gru_bz"] = mn.gru.W_z.weight.detach(), mn.gru.W_z.bias.detach()
    w["gru_Wr"], w["gru_br"] = mn.gru.W_r.weight.detach(), mn.gru.W_r.bias.detach()
    w["gru_Wh"], w["gru_bh"] = mn.gru.W_h.weight.detach(), mn.gru.W_h.bias.detach()
    gen = torch.Generator().manual_seed(3)
    data = [dict(g=torch.randn(n, generator=gen) * 0.5, s=torch.rand(n, generator=gen) * 0.3, h=torch.randn(n, 4, generator=gen) * 0.5,
                 hf=torch.randn(16, 16, generator=gen) * 0.3, hb=torch.randn(16, 16, generator=gen) * 0.3, R=torch.randn(n, generator=gen))
            for n in (700, 150, 64)]
    dims = dict(d_model=8, num_heads=4, pk_dim=12)
    for d in data:
        smart, _, _, _ = ref_fp64.forward_for_bilevel(_flat64(mn64), d["g"].double(), d["s"].double(), d["h"].double(), d["hf"].double(),
                                                      d["hb"].double(), mn64.rescale, dims)
        (smart * d["R"].double()).sum().backward()
        d["smart64"] = smart.detach()
    ref = {n: p.grad.clone() for n, p in mn64.named_parameters()}
    acc = {n: torch.zeros_like(p) for n, p in mn.named_parameters() if not n.startswith(("peer_queries", "product_keys"))}
    acc["peer_queries"] = torch.zeros(4, 8, 22, device=dev)
    acc["product_keys_A"], acc["product_keys_B"] = torch.zeros(4, 12, 4, device=dev), torch.zeros(4, 12, 4, device=dev)
    for k, d in enumerate(data):
        print("single-tensor pair, parameter", k, flush=True)
        smart, (fs, bs, ff, fb, si, saved, xs) = _single_tensor_pass(mn, w, d, dev, acc)
        err = (smart.double().cpu() - d["smart64"]).abs()
        assert bool((err <= 1e-4 * d["smart64"].abs() + 1e-6).all()), ("smart", k, float(err.max()))
        if k == 0:       # the forward call's own outputs against the float64 scan
            g, s = d["g"], d["s"]
            perm = torch.sort(g.abs(), stable=True).indices
            assert torch.equal(si.cpu().long(), perm)
            W = [t.double().cpu() for t in mn.flat_weights()]
            x = torch.stack([g.double()[perm], s.double()[perm]], -1) @ W[0].T + W[1]
            eye = torch.eye(16, dtype=torch.float64)           # identity out_proj: scan_block then returns the gated output itself
            fo, hF = ref_fp64.scan_block(x, W[2:10] + [eye], d["hf"].double())
            bo, hB = ref_fp64.scan_block(x.flip(0), W[11:19] + [eye], d["hb"].double())
            for name, got, want in (("fwd_scan_out", fs, fo), ("bwd_scan_out", bs, bo), ("fwd_final_state", ff, hF), ("bwd_final_state", fb, hB)):
                e2 = (got.double().cpu() - want).abs()
                assert bool((e2 <= 1e-4 * want.abs() + 1e-6).all()), (name, float(e2.max()))
    torch.cuda.synchronize()
    got = dict(acc)
    for h in range(4):
        got["peer_queries.%d.weight" % h] = acc["peer_queries"][h]
        got["product_keys_A.%d" % h], got["product_keys_B.%d" % h] = acc["product_keys_A"][h], acc["product_keys_B"][h]
    worst = {}
    for n, r in ref.items():
        gg = got[n].double().cpu().reshape(r.shape)
        scale = float(r.abs().max())
        worst[n] = round(float((gg - r).abs().max()) / (2e-4 * scale + 1e-12), 3)
    print("single-tensor pair: worst gradient tolerance ratios", worst, flush=True)
    assert max(worst.values()) <= 1.0, worst


def test_bilevel_pairs_do_not_see_each_other():
    """Two forward calls before either backward call (two optimizers in one process): each backward call claims the
    forward call that filled ITS buffers; a second backward call on the same buffers, or one on buffers no forward
    call has filled, is refused."""
    from grokking_optimizers import _ops
    dev = torch.device("cuda:0")
    mn = _meta_net(4, dev)
    w = {k: (v.to(dev) if torch.is_tensor(v) else v) for k, v in mn.get_weights().items()}
    gen = torch.Generator().manual_seed(6)
    z = lambda *sh: torch.zeros(*sh, device=dev)

    def forward(n):
        g, s = (torch.randn(n, generator=gen) * 0.5).to(dev), (torch.rand(n, generator=gen) * 0.3).to(dev)
        bufs = dict(fs=z(n, 16), bs=z(n, 16), saved=[z(n, 16, 16)] + [z(n, 16) for _ in range(3)] + [z(n, 16, 16)] + [z(n, 16) for _ in range(3)],
                    xs=z(n, 8), off=torch.zeros(2, dtype=torch.int32, device=dev), si=torch.zeros(n, dtype=torch.int32, device=dev),
                    f0=z(1, 16, 16), b0=z(1, 16, 16), n=n)
        _ops.supergrok2_bilevel_fwd_save_batched([g], [s], w["input_proj_W"], w["input_proj_b"], *_mamba_args(w, "fwd", True),
                                                 *_mamba_args(w, "bwd", True), 8, 16, 16, bufs["fs"], bufs["bs"], *bufs["saved"], bufs["xs"],
                                                 bufs["off"], bufs["si"], bufs["f0"], bufs["b0"], 1)
        return bufs

    def backward(bufs, seed):
        gg = torch.Generator().manual_seed(seed)
        dfs, dbs = torch.randn(bufs["n"], 16, generator=gg).to(dev), torch.randn(bufs["n"], 16, generator=gg).to(dev)
        d_mamba = [torch.zeros_like(t) for t in _mamba_args(w, "fwd", False) + _mamba_args(w, "bwd", False)]
        dx = z(bufs["n"], 8)
        _ops.supergrok2_bilevel_backward_batched(dfs, dbs, bufs["xs"], *bufs["saved"], bufs["off"], *_mamba_args(w, "fwd", False),
                                                 *_mamba_args(w, "bwd", False), *d_mamba, dx, bufs["f0"], bufs["b0"], 8, 16, 16, 1, 1)
        torch.cuda.synchronize()
        return d_mamba, dx

    a_alone = forward(900)
    ga, xa = backward(a_alone, 1)
    gen = torch.Generator().manual_seed(6)          # the same inputs again for A, then B before A's backward call
    a, b = forward(900), forward(333)
    ga2, xa2 = backward(a, 1)
    gb, xb = backward(b, 2)
    assert torch.equal(xa, xa2) and all(torch.equal(p, q) for p, q in zip(ga, ga2))
    assert xb.shape[0] == 333 and bool(torch.isfinite(xb).all())
    with pytest.raises(RuntimeError, match="already run|no supergrok2_bilevel_fwd_save_batched"):
        backward(a, 1)
    fresh = dict(a, saved=[z(900, 16, 16)] + a["saved"][1:])
    with pytest.raises(RuntimeError, match="no supergrok2_bilevel_fwd_save_batched"):
        backward(fresh, 1)


@pytest.mark.parametrize("interval", [1, 4])
def test_forward_save_fills_the_per_step_buffers(interval):
    """The buffers the reference's forward-save kernels leave for its own backward pass
    (csrc/supergrok2_mamba_peer_backward_kernels.cu:950-1008; sizes as grokking_optimizers/supergrok2.py:667-681
    allocates them): x-branch, z and dt of every scan step and the state after every step -- or, with a checkpoint
    interval, after every interval-th step of a tensor's scan and after its last one, at that tensor's checkpoint
    offset -- in the order of each direction's own scan, against the float64 recurrence.  The first four floats of
    fwd_saved_states carry the call's ticket instead of state entries."""
    from grokking_optimizers import _ops
    dev = torch.device("cuda:0")
    mn = _meta_net(9, dev)
    mn64 = copy.deepcopy(mn).double().cpu()
    gen = torch.Generator().manual_seed(41)
    Ns = [150, 31, 1300, 64, 5]
    data = [dict(g=torch.randn(n, generator=gen) * 0.5, s=torch.rand(n, generator=gen) * 0.3,
                 hf=torch.randn(16, 16, generator=gen) * 0.3, hb=torch.randn(16, 16, generator=gen) * 0.3) for n in Ns]
    w = {k: (v.to(dev) if torch.is_tensor(v) else v) for k, v in mn.get_weights().items()}
    d_model, d_state, d_inner = 8, 16, 16
    total, P = sum(Ns), len(Ns)
    ck = [n if interval <= 1 else (n + interval - 1) // interval for n in Ns]
    z = lambda *s: torch.full(s, float("nan"), device=dev)          # whatever is not written stays NaN
    fwd_scan, bwd_scan = z(total, d_inner), z(total, d_inner)
    saved = [z(sum(ck), d_inner, d_state)] + [z(total, d_inner) for _ in range(3)] + [z(sum(ck), d_inner, d_state)] + [z(total, d_inner) for _ in range(3)]
    x_sorted, offsets_t = z(total, d_model), torch.zeros(P + 1, dtype=torch.int32, device=dev)
    sort_idx = torch.zeros(total, dtype=torch.int32, device=dev)
    print("fwd_save_batched with checkpoint interval", interval, flush=True)
    _ops.supergrok2_bilevel_fwd_save_batched([d["g"].to(dev) for d in data], [d["s"].to(dev) for d in data], w["input_proj_W"],
                                             w["input_proj_b"], *_mamba_args(w, "fwd", True), *_mamba_args(w, "bwd", True), d_model, d_state,
                                             d_inner, fwd_scan, bwd_scan, *saved, x_sorted, offsets_t, sort_idx,
                                             torch.stack([d["hf"] for d in data]).to(dev), torch.stack([d["hb"] for d in data]).to(dev), interval)
    torch.cuda.synchronize()
    got = [t.double().cpu() for t in saved]
    W64 = _flat64(mn64)
    offs, coffs = np.concatenate([[0], np.cumsum(Ns)]), np.concatenate([[0], np.cumsum(ck)])

    def close(a, b, what):
        assert bool(torch.isfinite(a).all()), what
        err = (a - b).abs()
        tol = 1e-4 * torch.maximum(a.abs(), b.abs()) + 1e-6
        assert bool((err <= tol).all()), (what, float((err / tol).max()))
    for i, d in enumerate(data):
        a, b, ca, cb = int(offs[i]), int(offs[i + 1]), int(coffs[i]), int(coffs[i + 1])
        perm = torch.sort(d["g"].abs(), stable=True).indices
        x = torch.stack([d["g"][perm], d["s"][perm]], -1).double() @ W64[0].detach().T + W64[1].detach()
        for k, (xs, w9, h0) in enumerate(((x, W64[2:11], d["hf"]), (x.flip(0), W64[11:20], d["hb"]))):
            xb, zz, dt, states = ref_fp64.scan_block_trace(xs, [t.detach() for t in w9], h0.double())
            close(got[4 * k + 1][a:b], xb, ("x_branch", i, k))
            close(got[4 * k + 2][a:b], zz, ("z", i, k))
            close(got[4 * k + 3][a:b], dt, ("dt", i, k))
            n = Ns[i]
            steps = list(range(n)) if interval <= 1 else [min((q + 1) * interval, n) - 1 for q in range(cb - ca)]
            have, want = got[4 * k][ca:cb].clone(), states[steps]
            if k == 0 and i == 0:
                have.view(-1)[:4] = want.reshape(-1)[:4]          # the ticket of the call
            close(have, want, ("states", i, k))
    ticket = saved[0].view(-1)[:4].view(torch.int32).cpu()
    assert int(ticket[0]) == 0x5347324B
