"""Bilevel path of SuperGrok v2, sequential part: the HIP forward (sort + bidirectional scan, through
sg2_bilevel_forward) and the HIP adjoint (sg2_bilevel_backward) against float64 autograd through the
independent torch restatement of the scan (ref_fp64.scan_block, written from
grokking_optimizers/mamba3_peer_metanet.py:90-160 of the reference).

The loss is sum(ctx * R) for a fixed random R, so every context entry of every element carries a gradient.
Gates: contexts within |a-b| <= 1e-4*max(|a|,|b|) + 1e-7; each weight gradient within 2e-4 of the largest
entry of that gradient (fp32 sums over all elements against float64)."""
import numpy as np
import pytest
import torch

import ref_fp64
import workloads as wl

pytestmark = pytest.mark.gpu

NAMES = ["input_proj.W", "input_proj.b"] + [d + n for d in ("fwd.", "bwd.") for n in
         ("in_proj", "dt_W", "dt_b", "B_proj", "C_proj", "A_log", "D", "rope_freq", "out_proj")]


def _reference(W, grads, sharps, mf, mb, R):
    Wd = [w.detach().double().cpu().requires_grad_(True) for w in W[:20]]
    loss = torch.zeros((), dtype=torch.float64)
    ctx = []
    off = 0
    for g, s, hf, hb in zip(grads, sharps, mf, mb):
        g, s = g.reshape(-1).double().cpu(), s.reshape(-1).double().cpu()
        n = g.numel()
        perm = torch.sort(g.abs().float(), stable=True).indices
        x = torch.stack([g[perm], s[perm]], -1) @ Wd[0].T + Wd[1]
        fo, _ = ref_fp64.scan_block(x, Wd[2:11], hf.double().cpu())
        bo, _ = ref_fp64.scan_block(x.flip(0), Wd[11:20], hb.double().cpu())
        unsort = torch.argsort(perm)
        cf, cb = fo[unsort], bo.flip(0)[unsort]
        loss = loss + (cf * R[0, off:off + n]).sum() + (cb * R[1, off:off + n]).sum()
        ctx.append((cf.detach(), cb.detach()))
        off += n
    loss.backward()
    return ctx, [w.grad for w in Wd]


def _case(shapes, seed, sharp, state_std, chunk_len=None, a_log=None, window=None):
    from grokking_optimizers import _bilevel, _cabi
    dev = torch.device("cuda:0")
    if chunk_len is not None:
        assert _cabi.lib().sg2_set_chunk_len(chunk_len) == 0
    if window is not None:
        assert _cabi.lib().sg2_set_scan_window(window) == 0
    try:
        W = wl.meta_weights(seed)
        if a_log is not None:
            for base in (2, 11):
                W[base + 5].fill_(a_log)
        W = [w.to(dev) for w in W]
        grads = [g.to(dev) for g in wl.make_grads(shapes, seed=seed + 1, std=0.5)]
        sharps = [(g.abs() * 0.5).to(dev) if sharp else torch.zeros_like(g, device=dev)
                  for g in wl.make_grads(shapes, seed=seed + 2, std=0.5)]
        gen = torch.Generator().manual_seed(seed + 3)
        mf = [(torch.randn(16, 16, generator=gen) * state_std).to(dev) for _ in shapes]
        mb = [(torch.randn(16, 16, generator=gen) * state_std).to(dev) for _ in shapes]
        total = sum(g.numel() for g in grads)
        R = torch.randn(2, total, 8, generator=gen, dtype=torch.float64)
        params = [w.clone().requires_grad_(True) for w in W[:20]]
        print("bilevel case shapes", shapes, "seed", seed, "sharp", sharp, "chunk", chunk_len, flush=True)
        ctx = _bilevel.scan_contexts(W, params, grads, sharps, mf, mb)
        (ctx.double() * R.to(dev)).sum().backward()
        torch.cuda.synchronize()
        for m0, m1 in zip(mf + mb, [m.clone() for m in mf + mb]):
            assert torch.equal(m0, m1)
        ref_ctx, ref_grads = _reference(W, grads, sharps, mf, mb, R)
        off = 0
        for (cf, cb), g in zip(ref_ctx, grads):
            n = g.numel()
            for d, ref in ((0, cf), (1, cb)):
                got = ctx[d, off:off + n].detach().double().cpu()
                err = (got - ref).abs()
                tol = 1e-4 * torch.maximum(got.abs(), ref.abs()) + 1e-7
                assert bool((err <= tol).all()), ("ctx", d, n, float((err / tol).max()))
            off += n
        worst = {}
        for name, p, ref in zip(NAMES, params, ref_grads):
            got = p.grad.double().cpu()
            scale = float(ref.abs().max())
            ratio = float((got - ref).abs().max()) / (2e-4 * scale + 1e-12)
            worst[name] = round(ratio, 3)
            assert ratio <= 1.0, (name, ratio, scale)
        print("worst gradient tolerance ratios", worst, flush=True)
    finally:
        if chunk_len is not None:
            _cabi.lib().sg2_set_chunk_len(0)
        if window is not None:
            _cabi.lib().sg2_set_scan_window(-1)


def test_small_tensors_with_sharpness_and_carried_states():
    _case([(300,), (70,), (1,), (129,), (5, 13)], seed=11, sharp=True, state_std=0.3)


def test_ragged_tile_ends():
    """Lengths that end 1..7 steps after a multiple of 32 or 64 (the forward pass keeps a state every 32 steps, and the
    last steps of a tensor run through its scalar tail loop)."""
    _case([(99,), (33,), (97,), (39,), (64 + 32,), (32,), (31,), (64 + 39,)], seed=15, sharp=True, state_std=0.3)


def test_zero_sharpness_and_zero_states():
    _case([(200,), (64,), (65,)], seed=12, sharp=False, state_std=0.0)


def test_automatic_chunk_length_on_longer_tensors():
    """5000 + 3000 elements at the chunk length the library picks by itself (several chunks per tensor, partial last
    tiles): the chunk-parallel adjoint (summaries, prefix, replay) against float64 autograd."""
    _case([(5000,), (3000,)], seed=14, sharp=True, state_std=0.3)


def test_barely_contracting_poles_walk_the_whole_chunk():
    """A_log = -12: A_bar stays within 1e-5 of 1, so neither the forward nor the adjoint summary contracts within a
    block; both walk every block of the chunk (chunk length 512, window 256)."""
    _case([(3000,), (1500,)], seed=16, sharp=True, state_std=0.3, chunk_len=512, a_log=-12.0)


def test_slow_poles_need_several_summary_blocks():
    """A_log = -2 (A = -0.135, the slowest pole of the optimizer's own initialisation is -1): with blocks of 64 steps
    the 2x2 part falls below 2^-100 only after several of them, so the block walk of both summary kernels composes
    maps (chunk length 1024, window 64)."""
    _case([(5000,), (2100,)], seed=17, sharp=True, state_std=0.3, chunk_len=1024, a_log=-2.0, window=64)


def test_several_chunks():
    """Chunk length 64: the forward pass runs summaries, chunk prefix and replay; the adjoint crosses chunk borders."""
    _case([(1000,), (257,), (640,)], seed=13, sharp=True, state_std=0.3, chunk_len=64)


# ---------------------------------------------------------------------------------------------------------------
# whole meta-net: differentiable forward (soft top-4 routing) and the optimizer's bilevel_step
# ---------------------------------------------------------------------------------------------------------------
def _ref_forward_for_bilevel(mn, grad, sharp, gru_state, hf, hb):
    """float64 CPU statement of Mamba3PEERMetaNet.forward_for_bilevel (mamba3_peer_metanet.py:372-436 of the
    reference) on a double copy `mn` of the module: ref_fp64.forward_for_bilevel (pinned by the closed forms of
    tests/test_oracle_sg2_pins.py) over the module's own parameters, so that autograd reaches them."""
    blk = lambda b: [b.in_proj.weight, b.dt_proj.weight, b.dt_proj.bias, b.B_proj.weight, b.C_proj.weight, b.A_log, b.D,
                     b.rope_freq, b.out_proj.weight]
    E = mn.num_experts
    W = ([mn.input_proj.weight, mn.input_proj.bias] + blk(mn.mamba_fwd) + blk(mn.mamba_bwd) +
         [mn.gru.W_z.weight, mn.gru.W_z.bias, mn.gru.W_r.weight, mn.gru.W_r.bias, mn.gru.W_h.weight, mn.gru.W_h.bias] +
         [torch.stack([q.weight for q in mn.peer_queries]), torch.stack(list(mn.product_keys_A)),
          torch.stack(list(mn.product_keys_B))] +
         [mn.expert_W1.reshape(E, -1), mn.expert_b1, mn.expert_W2.reshape(E, -1), mn.expert_b2.reshape(-1)])
    dims = dict(d_model=mn.d_model, num_heads=mn.num_peer_heads, pk_dim=mn.pk_dim)
    return ref_fp64.forward_for_bilevel(W, grad, sharp, gru_state, hf, hb, mn.rescale, dims)


def _meta_net(seed, dev, **kw):
    from grokking_optimizers import Mamba3PEERMetaNet
    torch.manual_seed(seed)
    mn = Mamba3PEERMetaNet(**kw)
    with torch.no_grad():       # the initial keys and experts are nearly silent: give every part a visible gradient
        for p in mn.parameters():
            if p.dim() > 0 and float(p.abs().max()) < 0.05:
                p.add_(torch.randn_like(p) * 0.2)
    return mn.to(dev)


def _grad_ratios(named_got, named_ref, rel):
    worst = {}
    for (n, got), (_, ref) in zip(named_got, named_ref):
        got = torch.zeros_like(ref) if got is None else got.double().cpu()
        scale = float(ref.abs().max())
        worst[n] = round(float((got - ref).abs().max()) / (rel * scale + 1e-12), 3)
    return worst


def test_differentiable_forward_of_the_whole_meta_net():
    """smart gradient, new GRU state and the gradient of <smart, R> with respect to every parameter of the meta-net,
    one tensor at a time through the autograd form (HIP scan + torch per-element part), against the float64
    statement; then the all-HIP accumulation over the three tensors at once (sg2_bilevel_forward, sg2_bilevel_elem,
    sg2_bilevel_backward) against the sum of the float64 gradients and the float64 smart gradients."""
    import copy
    from grokking_optimizers import _bilevel
    dev = torch.device("cuda:0")
    mn = _meta_net(5, dev)
    mn64 = copy.deepcopy(mn).double().cpu()
    gen = torch.Generator().manual_seed(17)
    shapes = [(150,), (9, 11), (64,)]
    data = []
    for shp in shapes:
        n = int(np.prod(shp))
        data.append(dict(g=torch.randn(n, generator=gen) * 0.5, s=torch.rand(n, generator=gen) * 0.3,
                         h=torch.randn(n, 4, generator=gen) * 0.5, hf=torch.randn(16, 16, generator=gen) * 0.3,
                         hb=torch.randn(16, 16, generator=gen) * 0.3, R=torch.randn(n, generator=gen)))
    print("whole meta-net forward, shapes", shapes, flush=True)
    ref_sum, ref_smart = None, []
    for k, d in enumerate(data):
        mn.zero_grad()
        mn64.zero_grad()
        smart, hn, nf, nb = mn.forward_for_bilevel(d["g"].to(dev), d["s"].to(dev), d["h"].to(dev), d["hf"].to(dev), d["hb"].to(dev))
        (smart * d["R"].to(dev)).sum().backward()
        rs, rh, rf, rb = _ref_forward_for_bilevel(mn64, d["g"].double(), d["s"].double(), d["h"].double(), d["hf"].double(), d["hb"].double())
        (rs * d["R"].double()).sum().backward()
        for name, got, ref in (("smart", smart, rs), ("gru", hn, rh), ("mamba_fwd", nf, rf), ("mamba_bwd", nb, rb)):
            got, ref = got.detach().double().cpu(), ref.detach()
            err, tol = (got - ref).abs(), 1e-4 * torch.maximum(got.abs(), ref.abs()) + 1e-7
            assert bool((err <= tol).all()), (name, k, float((err / tol).max()))
        ref_smart.append(rs.detach())
        ref_named = [(n, p.grad.clone()) for n, p in mn64.named_parameters()]
        w = _grad_ratios([(n, p.grad) for n, p in mn.named_parameters()], ref_named, 2e-4)
        print("tensor", k, "worst gradient ratios", w, flush=True)
        assert max(w.values()) <= 1.0, w
        ref_sum = ref_named if ref_sum is None else [(n, a + b) for (n, a), (_, b) in zip(ref_sum, ref_named)]
    mn.zero_grad()
    print("all-HIP accumulation over the three tensors", flush=True)
    smart = _bilevel.accumulate_meta_gradients(mn, [d["g"].to(dev) for d in data], [d["s"].to(dev) for d in data],
                                               [d["h"].to(dev) for d in data], [d["hf"].to(dev) for d in data],
                                               [d["hb"].to(dev) for d in data], [d["R"].to(dev) for d in data])
    got, ref = smart.double().cpu(), torch.cat(ref_smart)
    err, tol = (got - ref).abs(), 1e-4 * torch.maximum(got.abs(), ref.abs()) + 1e-7
    assert bool((err <= tol).all()), ("smart", float((err / tol).max()))
    w = _grad_ratios([(n, p.grad) for n, p in mn.named_parameters()], ref_sum, 2e-4)
    print("all-HIP accumulation, worst gradient ratios", w, flush=True)
    assert max(w.values()) <= 1.0, w


@pytest.mark.parametrize("case", ["zero_biases_small_gradients", "thresholds_at_the_gradient_scale"])
def test_expert_gradients_around_the_unit_thresholds(case):
    """The expert part of the all-HIP accumulation works per interval between an expert's sorted unit thresholds
    -b1 / W1: sums next to g = 0 through matrix instructions, the others through atomics.  Two corners against the
    float64 statement.  (1) The module's own initial experts (b1 = 0, every threshold exactly 0, all tied) with
    gradients of 1e-3: every element sits next to zero, on one side or the other.  (2) Thresholds spread over the
    range of the gradients themselves, a few units with W1 = 0 (no threshold) and a few thresholds shared by several
    units: most elements lie beyond the intervals next to zero of some of their experts."""
    import copy
    from grokking_optimizers import _bilevel
    dev = torch.device("cuda:0")
    mn = _meta_net(21, dev)
    gen = torch.Generator().manual_seed(22)
    gstd = 1e-3
    with torch.no_grad():
        E, EH = mn.num_experts, mn.expert_W1.shape[1]
        w1 = (torch.randn(E, EH, 1, generator=gen) * 0.5)
        if case == "zero_biases_small_gradients":
            b1 = torch.zeros(E, EH)
        else:
            theta = torch.randn(E, EH, generator=gen) * 2.0 * gstd          # thresholds where the gradients are
            theta[:, 3] = theta[:, 2]                                       # two units share a threshold
            theta[:, 5] = 0.0
            w1[:, 7, 0] = 0.0                                               # no threshold: active by the sign of b1 alone
            w1[:, 8, 0] = 0.0
            b1 = -theta * w1[:, :, 0]
            b1[:, 7] = 0.3
            b1[:, 8] = -0.3
        mn.expert_W1.copy_(w1.to(dev))
        mn.expert_b1.copy_(b1.to(dev))
    mn64 = copy.deepcopy(mn).double().cpu()
    shapes = [(700,), (33, 9), (130,)]
    data = []
    for shp in shapes:
        n = int(np.prod(shp))
        data.append(dict(g=torch.randn(n, generator=gen) * gstd, s=torch.rand(n, generator=gen) * gstd,
                         h=torch.randn(n, 4, generator=gen) * 0.5, hf=torch.randn(16, 16, generator=gen) * 0.3,
                         hb=torch.randn(16, 16, generator=gen) * 0.3, R=torch.randn(n, generator=gen)))
    print("expert thresholds:", case, "shapes", shapes, flush=True)
    ref_sum, ref_smart = None, []
    for d in data:
        mn64.zero_grad()
        rs, _, _, _ = _ref_forward_for_bilevel(mn64, d["g"].double(), d["s"].double(), d["h"].double(), d["hf"].double(), d["hb"].double())
        (rs * d["R"].double()).sum().backward()
        ref_smart.append(rs.detach())
        ref_named = [(n, p.grad.clone()) for n, p in mn64.named_parameters()]
        ref_sum = ref_named if ref_sum is None else [(n, a + b) for (n, a), (_, b) in zip(ref_sum, ref_named)]
    mn.zero_grad()
    smart = _bilevel.accumulate_meta_gradients(mn, [d["g"].to(dev) for d in data], [d["s"].to(dev) for d in data],
                                               [d["h"].to(dev) for d in data], [d["hf"].to(dev) for d in data],
                                               [d["hb"].to(dev) for d in data], [d["R"].to(dev) for d in data])
    got, ref = smart.double().cpu(), torch.cat(ref_smart)
    err, tol = (got - ref).abs(), 1e-4 * torch.maximum(got.abs(), ref.abs()) + 1e-7
    assert bool((err <= tol).all()), ("smart", float((err / tol).max()))
    w = _grad_ratios([(n, p.grad) for n, p in mn.named_parameters()], ref_sum, 2e-4)
    print("worst gradient ratios", w, flush=True)
    assert max(w.values()) <= 1.0, w
    for n in ("expert_W1", "expert_b1", "expert_W2", "expert_b2"):
        assert float(dict(ref_sum)[n].abs().max()) > 0.0, n          # the comparison is not vacuous


@pytest.mark.parametrize("kw", [dict(expert_hidden=4), dict(d_model=4, d_state=8, gru_hidden=2, expert_hidden=6),
                                dict(d_model=6, d_state=10, gru_hidden=3, num_peer_heads=2, num_experts=25),
                                dict(d_model=16, d_state=32)],
                         ids=["experts_of_width_4", "smaller_net_embedded", "other_routing_sizes", "large_scan_block"])
def test_accumulation_at_other_meta_net_sizes(kw):
    """The bilevel accumulation at sizes other than the defaults, smart gradients and the gradients of every
    parameter against float64 autograd:
    * expert_hidden = 4, the width the reference's training harness constructs the optimizer with
      (grokking_race_v2.py:1583 -> :775): the per-element kernel runs the narrow experts embedded in its own width;
    * a smaller scan block, GRU and expert width: scan kernels and per-element kernel both run the net embedded;
    * other routing sizes (heads, keys, experts): the scan and its adjoint in HIP (embedded block), the per-element
      part as torch operations;
    * the largest scan block the reference admits (d_model 16, d_state 32, d_inner 32), which the bilevel kernels are
      not built for: the scan blocks' own chunked torch forward under autograd, on the GPU.
    Then one tensor through the module's forward_for_bilevel (the autograd form over the same kernels)."""
    import copy
    from grokking_optimizers import _bilevel
    dev = torch.device("cuda:0")
    mn = _meta_net(8, dev, **kw)
    assert mn.expert_W1.shape[1] == kw.get("expert_hidden", 16)
    mn64 = copy.deepcopy(mn).double().cpu()
    gh, di, ds = mn.gru_hidden, mn.mamba_fwd.d_inner, mn.d_state
    gen = torch.Generator().manual_seed(23)
    data = []
    for n in (200, 77, 1300):
        data.append(dict(g=torch.randn(n, generator=gen) * 0.5, s=torch.rand(n, generator=gen) * 0.3,
                         h=torch.randn(n, gh, generator=gen) * 0.5, hf=torch.randn(di, ds, generator=gen) * 0.3,
                         hb=torch.randn(di, ds, generator=gen) * 0.3, R=torch.randn(n, generator=gen)))
    print("bilevel accumulation", kw, "per-element kernel:", _bilevel.elem_kernel_fits(mn), flush=True)
    assert _bilevel.elem_kernel_fits(mn) == ("num_experts" not in kw and kw.get("d_model", 8) <= 8)
    assert _bilevel.scan_kernels_fit(mn) == (kw.get("d_model", 8) <= 8)
    mn64.zero_grad()
    ref_smart = []
    for d in data:
        rs, _, _, _ = _ref_forward_for_bilevel(mn64, d["g"].double(), d["s"].double(), d["h"].double(), d["hf"].double(), d["hb"].double())
        (rs * d["R"].double()).sum().backward()
        ref_smart.append(rs.detach())
    ref_named = [(n, p.grad.clone()) for n, p in mn64.named_parameters()]
    mn.zero_grad()
    smart = _bilevel.accumulate_meta_gradients(mn, [d["g"].to(dev) for d in data], [d["s"].to(dev) for d in data],
                                               [d["h"].to(dev) for d in data], [d["hf"].to(dev) for d in data],
                                               [d["hb"].to(dev) for d in data], [d["R"].to(dev) for d in data])
    got, ref = smart.double().cpu(), torch.cat(ref_smart)
    err, tol = (got - ref).abs(), 1e-4 * torch.maximum(got.abs(), ref.abs()) + 1e-7
    assert bool((err <= tol).all()), ("smart", float((err / tol).max()))
    for n, p in mn.named_parameters():
        assert p.grad is not None and p.grad.shape == p.shape, n
    w = _grad_ratios([(n, p.grad) for n, p in mn.named_parameters()], ref_named, 2e-4)
    print(kw, "worst gradient ratios", w, flush=True)
    assert max(w.values()) <= 1.0, w

    d = data[0]
    mn.zero_grad()
    mn64.zero_grad()
    smart, hn, nf, nb = mn.forward_for_bilevel(d["g"].to(dev), d["s"].to(dev), d["h"].to(dev), d["hf"].to(dev), d["hb"].to(dev))
    (smart * d["R"].to(dev)).sum().backward()
    rs, rh, rf, rb = _ref_forward_for_bilevel(mn64, d["g"].double(), d["s"].double(), d["h"].double(), d["hf"].double(), d["hb"].double())
    (rs * d["R"].double()).sum().backward()
    for name, got, ref in (("smart", smart, rs), ("gru", hn, rh), ("mamba_fwd", nf, rf), ("mamba_bwd", nb, rb)):
        got, ref = got.detach().double().cpu(), ref.detach()
        assert got.shape == ref.shape, (name, got.shape, ref.shape)
        err, tol = (got - ref).abs(), 1e-4 * torch.maximum(got.abs(), ref.abs()) + 1e-7
        assert bool((err <= tol).all()), (name, float((err / tol).max()))
    w = _grad_ratios([(n, p.grad) for n, p in mn.named_parameters()], [(n, p.grad.clone()) for n, p in mn64.named_parameters()], 2e-4)
    print(kw, "forward_for_bilevel, worst gradient ratios", w, flush=True)
    assert max(w.values()) <= 1.0, w


def test_optimizer_bilevel_step_and_step_full():
    """SuperGrok2.bilevel_step changes the meta-net along the gradient the accumulation returns, restores the model's
    gradients and reports the validation loss; step_full with SAM and bilevel at every step runs and learns."""
    import copy
    from grokking_optimizers import SuperGrok2, _bilevel
    dev = torch.device("cuda:0")
    torch.manual_seed(3)
    model = torch.nn.Sequential(torch.nn.Linear(12, 24), torch.nn.ReLU(), torch.nn.Linear(24, 5)).to(dev)
    opt = SuperGrok2(model.parameters(), lr=1e-2, meta_net=_meta_net(8, dev), sam_freq_min=1, sam_freq_max=1,
                     bilevel_freq_min=1, bilevel_freq_max=1, alpha_update_freq=2)
    xs, ys = torch.randn(64, 12, device=dev), torch.randint(0, 5, (64,), device=dev)
    xv, yv = torch.randn(32, 12, device=dev), torch.randint(0, 5, (32,), device=dev)
    crit = torch.nn.CrossEntropyLoss()
    print("bilevel_step on a 2-layer model", flush=True)
    model.zero_grad()
    crit(model(xs), ys).backward()
    opt.step()                  # GRU and Mamba states away from zero (a zero GRU state hides the reset gate)
    model.zero_grad()
    crit(model(xs), ys).backward()
    sam_loss = opt.sam_step(model, xs, ys, crit)
    assert sam_loss > 0 and any(float(s.abs().max()) > 0 for s in opt._flat_sharpness)
    before_grads = [p.grad.clone() for p in model.parameters()]
    before_meta = copy.deepcopy(opt.meta_net.state_dict())
    # expected meta gradient, from the same pieces
    model.zero_grad()
    crit(model(xv), yv).backward()
    cots = []
    for p in model.parameters():
        vg = p.grad.detach().float()
        cots.append(-(vg / vg.norm()).reshape(-1))
    probe = copy.deepcopy(opt.meta_net)
    _bilevel.accumulate_meta_gradients(probe, [g.reshape(-1) for g in before_grads], opt._flat_sharpness, opt._flat_gru_states,
                                       opt._flat_mamba_fwd_states, opt._flat_mamba_bwd_states, cots)
    for p, g in zip(model.parameters(), before_grads):
        p.grad = g.clone()
    meta_opt = torch.optim.SGD(opt.meta_net.parameters(), lr=0.5)
    val = opt.bilevel_step(model, xs, ys, xv, yv, crit, meta_opt)
    assert abs(val - float(crit(model(xv), yv).detach())) < 1e-5
    for p, g in zip(model.parameters(), before_grads):
        assert torch.equal(p.grad, g)
    moved = 0
    for (n, p), q in zip(opt.meta_net.named_parameters(), probe.parameters()):
        want = before_meta[n] - 0.5 * (q.grad if q.grad is not None else torch.zeros_like(p))
        scale = float(q.grad.abs().max()) if q.grad is not None else 0.0
        assert float((p.detach() - want).abs().max()) <= 0.5 * 2e-4 * scale + 1e-7, n      # atomics: order of sums differs
        moved += int(scale > 0)
    assert moved == len(list(opt.meta_net.parameters())), moved
    losses = []
    for it in range(12):
        m = opt.step_full(model, xs, ys, xv, yv, crit)
        assert "sam_loss" in m and "val_loss" in m
        with torch.no_grad():
            losses.append(float(crit(model(xs), ys)))
    print("step_full losses", [round(v, 4) for v in losses], flush=True)
    assert all(np.isfinite(losses)) and losses[-1] < losses[0]


@pytest.mark.parametrize("kw", [dict(), dict(expert_hidden=4), dict(d_model=4, d_state=8, gru_hidden=3, num_peer_heads=2, num_experts=25, expert_hidden=6)])
def test_module_forward_matches_the_float64_step(kw):
    """Mamba3PEERMetaNet.forward (hard top-1 routing; one call of sg2_meta_forward: sort, scan, GRU, routing and experts
    in HIP, at the default sizes and at others) against the float64 restatement of the step: smart gradient, new GRU
    state, both new Mamba states; expert choices may differ only at near-ties, which the tolerance on smart (1e-4 of
    its scale) would expose.  The caller's states are not modified."""
    dev = torch.device("cuda:0")
    mn = _meta_net(21, dev, **kw)
    gen = torch.Generator().manual_seed(22)
    n = 333
    di, ds, gh = mn.mamba_fwd.d_inner, mn.d_state, mn.gru_hidden
    g, s = torch.randn(n, generator=gen) * 0.5, torch.rand(n, generator=gen) * 0.3
    h = torch.randn(n, gh, generator=gen) * 0.5
    hf, hb = torch.randn(di, ds, generator=gen) * 0.3, torch.randn(di, ds, generator=gen) * 0.3
    print("module forward, N", n, kw, flush=True)
    hf_dev, hb_dev, h_dev = hf.to(dev), hb.to(dev), h.to(dev)
    assert mn.training and int(mn.expert_counts.sum()) == 0
    smart, hn, nf, nb = mn(g.to(dev), s.to(dev), h_dev, hf_dev, hb_dev)
    assert torch.equal(hf_dev.cpu(), hf) and torch.equal(hb_dev.cpu(), hb) and torch.equal(h_dev.cpu(), h)
    # a module in training mode counts the winners (one per head and element), one in eval mode does not
    assert int(mn.expert_counts.sum()) == n * mn.num_peer_heads
    mn.eval()
    again = mn(g.to(dev), s.to(dev), h_dev, hf_dev, hb_dev)
    assert int(mn.expert_counts.sum()) == n * mn.num_peer_heads and torch.equal(again[0], smart)
    mn.train()
    assert mn.has_cuda_bilevel
    dims = dict(d_model=mn.d_model, gru_hidden=gh, num_heads=mn.num_peer_heads, pk_dim=mn.pk_dim)
    sc = dict(rescale=mn.rescale, alpha=0.0, lamb_eff=0.0, beta1=0.9, beta2=0.999, bc1=1.0, bc2=1.0, eps=1e-8, lr=0.0, wd_eff=0.0)
    z = torch.zeros(n)
    import workloads as wl
    full = dict(d_model=mn.d_model, d_state=ds, d_inner=di, gru_hidden=gh, num_heads=mn.num_peer_heads, pk_dim=mn.pk_dim,
                expert_hidden=mn.expert_hidden, num_experts=mn.num_experts)
    W = [w.cpu().reshape(shape) for w, shape in zip(mn.flat_weights(), wl.meta_weight_shapes(full))]
    ref = ref_fp64.step(W, z, g, s, z, z, z, h, hf, hb, sc, dims)
    for name, got, want in (("smart", smart, ref["smart"]), ("gru", hn, ref["gru"]), ("mamba_fwd", nf, ref["mamba_fwd"]),
                            ("mamba_bwd", nb, ref["mamba_bwd"])):
        got = got.detach().double().cpu()
        assert float((got - want).abs().max()) <= 1e-4 * float(want.abs().max()) + 1e-7, (name, kw)
