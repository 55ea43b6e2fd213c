"""GPU parity of the Grokfast and SuperGrok v1.5 fused steps (HIP, through the
`_ops` extension and the C ABI behind it) with the CPU checker and with the
golden vectors written by the reference's own CPU code.
Tolerance: |a-b| <= 1e-4*max(|a|,|b|) + 1e-7 (fp32)."""
import os

import numpy as np
import pytest
import torch

import workloads as wl
from helpers import rel_close
from oracle import oracle as orc

pytestmark = pytest.mark.gpu
GOLD = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
REL, FLOOR = 1e-4, 1e-7
f32 = lambda v: float(np.float32(v))


def _ops():
    from grokking_optimizers import _ops
    return _ops


def _close(a, b, what):
    ok, r = rel_close(a.detach().float().cpu().numpy().reshape(-1), np.asarray(b).reshape(-1), REL, FLOOR)
    assert ok, (what, r)


def test_grokfast_golden_and_adamw_fused():
    ops = _ops()
    z = np.load(os.path.join(GOLD, "ref_grokfast.npz"))
    n, steps = int(z["n"]), int(z["steps"])
    emas = [torch.zeros(z[f"g_in_0_{i}"].shape, device="cuda") for i in range(n)]
    for t in range(steps):
        grads = [torch.from_numpy(z[f"g_in_{t}_{i}"]).cuda() for i in range(n)]
        ops.grokfast_fused_step(grads, emas, float(z["alpha"]), float(z["lamb"]))
        for i in range(n):
            _close(grads[i], z[f"g_out_{t}_{i}"], ("grad", t, i))
            _close(emas[i], z[f"ema_{t}_{i}"], ("ema", t, i))


def test_grokfast_config1_100_chained_steps():
    """Config 1: 14-tensor transformer set, alpha .98, lamb 2, AdamW lr 1e-3 betas (.9,.98) wd 1: 1 step from
    zero state is step 1 of the chain; the class is driven for 100 steps against the CPU checker."""
    from grokking_optimizers import Grokfast
    shapes = wl.shared14_shapes()
    p0 = wl.make_params(shapes, seed=0)
    params = [torch.nn.Parameter(p.clone().cuda()) for p in p0]
    opt = Grokfast(params, lr=1e-3, betas=(0.9, 0.98), eps=1e-8, weight_decay=1.0, grokfast_alpha=0.98, grokfast_lamb=2.0)
    ref = [p.numpy().reshape(-1).copy() for p in p0]
    st = [[np.zeros_like(r) for _ in range(3)] for r in ref]         # ema, exp_avg, exp_avg_sq
    for t in range(1, 101):
        grads = wl.make_grads(shapes, seed=t)
        for p, g in zip(params, grads):
            p.grad = g.clone().cuda()
        opt.step()
        for i, g in enumerate(grads):
            gi = g.numpy().reshape(-1).copy()
            orc.grokfast_adamw(ref[i], gi, st[i][0], st[i][1], st[i][2], t, f32(0.98), f32(2.0), 1e-3, 0.9, 0.98, 1e-8, 1.0)
            if t in (1, 2, 50, 100):
                _close(params[i], ref[i], ("param", t, i))
                _close(params[i].grad, gi, ("amplified grad", t, i))
                _close(opt.state[params[i]]["ema"], st[i][0], ("ema", t, i))
                _close(opt.state[params[i]]["exp_avg_sq"], st[i][2], ("exp_avg_sq", t, i))
    # the unfused two-phase sequence of the reference gives the same result
    params2 = [torch.nn.Parameter(p.clone().cuda()) for p in p0]
    opt2 = Grokfast(params2, fused=False)
    for t in range(1, 4):
        for p, g in zip(params2, wl.make_grads(shapes, seed=t)):
            p.grad = g.clone().cuda()
        opt2.step()
    params3 = [torch.nn.Parameter(p.clone().cuda()) for p in p0]
    opt3 = Grokfast(params3, fused=True)
    for t in range(1, 4):
        for p, g in zip(params3, wl.make_grads(shapes, seed=t)):
            p.grad = g.clone().cuda()
        opt3.step()
    for a, b in zip(params2, params3):
        _close(a, b.detach().cpu().numpy(), "fused vs two-phase")


def test_grokfast_half_dtypes_and_empty():
    ops = _ops()
    for dt in (torch.float16, torch.bfloat16):
        g = (torch.randn(1000, generator=torch.Generator().manual_seed(1)) * 1e-2).to(dt)
        ema = torch.randn(1000, generator=torch.Generator().manual_seed(2)) * 1e-2
        gd, ed = g.cuda(), ema.cuda()
        ops.grokfast_fused_step([gd, torch.Tensor(), torch.zeros(0, device="cuda")], [ed, torch.Tensor(), torch.zeros(0, device="cuda")], 0.98, 2.0)
        e2 = ema.numpy().copy()
        g2 = g.float().numpy().copy()
        orc.grokfast_ema(g2, e2, f32(0.98), f32(2.0))
        assert torch.equal(gd.cpu(), torch.from_numpy(g2).to(dt))
        _close(ed, e2, "ema")
    with pytest.raises(RuntimeError, match="requires CUDA tensors"):
        ops.grokfast_fused_step([torch.zeros(4)], [torch.zeros(4)], 0.98, 2.0)


def _sg15_net(H, seed):
    gen = torch.Generator().manual_seed(seed)
    return (torch.randn(H, 2, generator=gen) * 0.5, torch.randn(H, generator=gen) * 0.1,
            torch.randn(1, H, generator=gen) * 0.5, torch.randn(1, generator=gen) * 0.1)


def test_sg15_reference_golden_through_ops():
    ops = _ops()
    z = np.load(os.path.join(GOLD, "ref_sg15.npz"))
    P, steps, H = int(z["n"]), int(z["steps"]), int(z["H"])
    cu = lambda k: torch.from_numpy(z[k]).cuda()
    W1, b1, W2, b2 = cu("W1"), cu("b1"), cu("W2"), cu("b2")
    params = [cu(f"p_in_{i}") for i in range(P)]
    eas, easqs, mus = ([torch.zeros_like(p) for p in params] for _ in range(3))
    for t in range(steps):
        grads = [cu(f"g_in_{t}_{i}") for i in range(P)]
        sharps = [cu(f"s_in_{t}_{i}") for i in range(P)]
        ops.supergrok15_fused_step(params, grads, eas, easqs, mus, sharps, [t] * P, [float(a) for a in z["alphas"]],
                                   [float(b) for b in z["beta1s"]], W1, b1, W2, b2, float(z["rescale"]), H,
                                   float(z["beta2"]), float(z["lr"]), float(z["wd_eff"]), float(z["eps"]), float(z["lamb"]),
                                   float(z["ramp"]), float(z["gate"]), float(z["clip"]))
        for i in range(P):
            for name, arr in (("p", params[i]), ("ea", eas[i]), ("easq", easqs[i]), ("mu", mus[i]), ("g_out", grads[i])):
                _close(arr, z[f"{name}_{t}_{i}"], (name, t, i))


@pytest.mark.parametrize("gelu", ["erf", "sigmoid"])
def test_sg15_config2_steps_vs_checker(gelu):
    """Config 2: 14-tensor set, H=32, heavy-tailed grads (clip active), sharpness from a second grad set via the
    SAM helper kernels, progressive wd / gate from train_acc = t/100."""
    ops = _ops()
    ops.supergrok15_set_gelu_mode(gelu)
    try:
        shapes = wl.shared14_shapes()
        P, H = len(shapes), 32
        gen = torch.Generator().manual_seed(3)
        W1, b1 = torch.randn(H, 2, generator=gen) * 0.01, torch.zeros(H)
        W2, b2 = torch.randn(1, H, generator=gen) * 0.01, torch.zeros(1)
        p0 = [p.reshape(-1) for p in wl.make_params(shapes, seed=0)]
        params = [p.clone().cuda() for p in p0]
        eas, easqs, mus, sharps = ([torch.zeros_like(p) for p in params] for _ in range(4))
        rp = [p.numpy().copy() for p in p0]
        rea, reasq, rmu = ([np.zeros_like(p) for p in rp] for _ in range(3))
        sig = lambda x: 1.0 / (1.0 + np.exp(-x))
        for t in range(1, 13):
            g = [x.reshape(-1) for x in wl.make_grads(shapes, seed=100 + t, tail_frac=0.01, tail="normal")]
            gs = [x.reshape(-1) for x in wl.make_grads(shapes, seed=200 + t, tail_frac=0.01, tail="normal")]
            gd, gsd = [x.clone().cuda() for x in g], [x.clone().cuda() for x in gs]
            backups = [p.clone() for p in params]
            ops.supergrok15_sharpness_restore_all(params, sharps, backups, gsd, gd)      # sharp = |g_sam - g|
            rs = [np.abs(a.numpy() - b.numpy()) for a, b in zip(gs, g)]
            acc = t / 100.0
            wd_eff, gate = f32(1.0 * (1 + 4 * sig(20 * (acc - 0.9)))), f32(sig(20 * (acc - 0.8)))
            alphas, beta1s = [0.98] * P, [0.9 * 0.9 ** i for i in range(P)]
            ops.supergrok15_fused_step(params, gd, eas, easqs, mus, sharps, [t - 1] * P, alphas, beta1s, W1.cuda(), b1.cuda(),
                                       W2.cuda(), b2.cuda(), 0.1, H, 0.999, 1e-3, wd_eff, 1e-8, 2.0, 1.0, gate, 1.0)
            step = np.float32(t)
            pt = [dict(alpha=f32(0.98), beta1=f32(b), bc1=f32(np.float32(1) - np.power(np.float32(b), step)),
                       bc2=f32(np.float32(1) - np.power(np.float32(0.999), step))) for b in beta1s]
            gn = [x.numpy().copy() for x in g]
            coef, on = orc.sg15_step(rp, gn, rs, rea, reasq, rmu, (W1.numpy(), b1.numpy(), W2.numpy(), b2.numpy(), f32(0.1)), pt,
                                     f32(np.float32(1.0) * np.float32(gate) * np.float32(2.0)), f32(0.999), f32(1e-3), wd_eff,
                                     f32(1e-8), f32(1.0), 0 if gelu == "erf" else 1)
            assert on == 1                                     # ||g|| ~ 6.5 > 1: the clip is active
            for i in range(P):
                _close(sharps[i], rs[i], ("sharp", t, i))
                _close(gd[i], gn[i], ("clipped grad", t, i))
                _close(params[i], rp[i], ("param", t, i))
                _close(eas[i], rea[i], ("exp_avg", t, i))
                _close(easqs[i], reasq[i], ("exp_avg_sq", t, i))
                _close(mus[i], rmu[i], ("mu", t, i))
    finally:
        ops.supergrok15_set_gelu_mode("erf")


def test_sg15_sam_perturb_golden_and_class():
    ops = _ops()
    z = np.load(os.path.join(GOLD, "ref_sg15.npz"))
    P = int(z["n"])
    ps = [torch.from_numpy(z[f"sam_p_in_{i}"]).cuda() for i in range(P)]
    gs = [torch.from_numpy(z[f"sam_g_{i}"]).cuda() for i in range(P)]
    backups = ops.supergrok15_sam_perturb_all(ps, gs, 0.05)
    for i in range(P):
        _close(ps[i], z[f"sam_p_out_{i}"], ("perturbed", i))
        assert torch.equal(backups[i].cpu(), torch.from_numpy(z[f"sam_backup_{i}"]))
    # class: 3 steps run, steps list stays at zero (by-value list through pybind, as in the reference)
    from grokking_optimizers import SuperGrok15
    w = [torch.nn.Parameter(torch.randn(64, 32, device="cuda") * 0.02), torch.nn.Parameter(torch.zeros(32, device="cuda"))]
    opt = SuperGrok15(w, warmup_steps=0, warmup_ramp=1)
    opt.meta_net.rescale.data.fill_(0.1)
    before = [p.detach().clone() for p in w]
    for t in range(3):
        for p in w:
            p.grad = torch.randn_like(p) * 1e-3
        opt.step(train_acc=0.9)
    assert opt._flat_steps == [0, 0]
    assert all(bool(torch.isfinite(p).all()) and not torch.equal(p, b) for p, b in zip(w, before))
