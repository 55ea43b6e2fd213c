"""The optimizer classes around the remaining fused steps, driven like the
reference's training loops drive them (tiny model on the GPU), against the CPU
checker (oracle/family_oracle.py), torch.optim.AdamW and torch autograd."""
import copy

import numpy as np
import pytest
import torch
import torch.nn as nn

from helpers import rel_close
from oracle import family_oracle as fo

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _model(seed=0):
    torch.manual_seed(seed)
    return nn.Sequential(nn.Linear(6, 16), nn.Tanh(), nn.Linear(16, 3)).to(DEV)


def _batch(seed):
    g = torch.Generator().manual_seed(seed)
    return torch.randn(32, 6, generator=g).to(DEV), torch.randint(0, 3, (32,), generator=g).to(DEV)


def _np(ts):
    return [t.detach().float().cpu().numpy().reshape(-1).copy() for t in ts]


def _assert_close(tag, got, want, rel=1e-4, floor=1e-7):
    for i, (a, b) in enumerate(zip(got, want)):
        ok, worst = rel_close(a, b, rel, floor)
        assert ok, (tag, i, worst)


def _assert_equal(tag, got, want):
    for i, (a, b) in enumerate(zip(got, want)):
        assert np.array_equal(a, b), (tag, i)


def _drive(opt, model, steps, mirror):
    """steps x (backward, hand the same grads to the checker `mirror(params, grads, t)`, optimizer step, compare params)"""
    crit = nn.CrossEntropyLoss()
    ps = list(model.parameters())
    ref = _np(ps)
    for t in range(1, steps + 1):
        x, y = _batch(100 + t)
        model.zero_grad()
        crit(model(x), y).backward()
        grads = _np([p.grad for p in ps])
        mirror(ref, grads, t)
        opt.step()
        torch.cuda.synchronize()
        _assert_close("params step %d" % t, _np(ps), ref)


def test_grokadamw_class():
    from grokking_optimizers import GrokAdamW
    m = _model()
    opt = GrokAdamW(m.parameters(), lr=1e-2, grad_clip=0.5)
    n = len(list(m.parameters()))
    st = [[np.zeros(p.numel(), np.float32) for p in m.parameters()] for _ in range(3)]
    _drive(opt, m, 4, lambda p, g, t: fo.grokadamw_step(p, g, st[0], st[1], st[2], [t] * n, 0.98, 5.0, 0.9, 0.98, 1e-2, 1.0, 1e-8, 0.5))
    assert opt.state[next(iter(m.parameters()))]["step"] == 4
    with pytest.raises(ValueError):
        GrokAdamW(m.parameters(), alpha=1.5)


def test_lion_and_prodigy_classes():
    from grokking_optimizers import Lion, Prodigy
    m = _model(1)
    st = [np.zeros(p.numel(), np.float32) for p in m.parameters()]
    _drive(Lion(m.parameters(), lr=1e-3), m, 4, lambda p, g, t: fo.lion_step(p, g, st, 1e-3, 0.9, 0.99, 3.0))
    m = _model(2)
    n = len(list(m.parameters()))
    opt = Prodigy(m.parameters(), lr=1e-3, weight_decay=0.0)
    s3 = [[np.zeros(p.numel(), np.float32) for p in m.parameters()] for _ in range(3)]
    p0 = _np(m.parameters())
    box = {"d": 1e-6}

    def mirror(p, g, t):
        box["d"] = fo.prodigy_step(p, g, s3[0], s3[1], s3[2], p0, [t] * n, box["d"], 0.9, 0.999, 1e-3, 0.0, 1e-8)
    _drive(opt, m, 4, mirror)
    assert abs(opt.d_lr - box["d"]) <= 1e-4 * box["d"]


def test_neuralgrok_class():
    from grokking_optimizers import NeuralGrok
    m = _model(3)
    torch.manual_seed(5)
    opt = NeuralGrok(m.parameters(), lr=1e-3, num_layers=2, hidden_dim=16)
    W = [w.cpu().numpy() for w in opt.amplifier.get_weights()]
    n = len(list(m.parameters()))
    st = [[np.zeros(p.numel(), np.float32) for p in m.parameters()] for _ in range(2)]
    _drive(opt, m, 3, lambda p, g, t: fo.neuralgrok_step(p, g, st[0], st[1], [t] * n, *W, 10.0, 4.0, 0.9, 0.98, 1e-3, 1.0, 1e-8, 1.0))
    # a changed amplifier only takes effect after mark_amplifier_dirty()
    with torch.no_grad():
        opt.amplifier.net[0].weight.mul_(2.0)
    opt.mark_amplifier_dirty()
    W2 = [w.cpu().numpy() for w in opt.amplifier.get_weights()]
    ref = _np(m.parameters())
    x, y = _batch(7)
    m.zero_grad()
    nn.CrossEntropyLoss()(m(x), y).backward()
    g = _np([p.grad for p in m.parameters()])
    fo.neuralgrok_step(ref, g, st[0], st[1], [4] * n, *W2, 10.0, 4.0, 0.9, 0.98, 1e-3, 1.0, 1e-8, 1.0)
    opt.step()
    _assert_close("after dirty", _np(m.parameters()), ref)
    assert isinstance(opt.get_amplifier_optimizer(), torch.optim.Adam)


def test_supergrok11_class():
    from grokking_optimizers import SuperGrok11
    m = _model(4)
    torch.manual_seed(6)
    opt = SuperGrok11(m.parameters(), lr=1e-3, warmup_steps=1, warmup_ramp=2, meta_hidden_dim=8)
    with torch.no_grad():
        opt.meta_net.rescale.fill_(0.3)
        opt.meta_net.net[0].weight.normal_(0, 0.5)
        opt.meta_net.net[2].weight.normal_(0, 0.5)
    W1, b1, W2, b2, rescale = opt.meta_net.get_weights()
    W = [w.cpu().numpy() for w in (W1, b1, W2, b2)]
    ps = list(m.parameters())
    n = len(ps)
    st = [[np.zeros(p.numel(), np.float32) for p in ps] for _ in range(3)]
    sharp = [np.zeros(p.numel(), np.float32) for p in ps]
    beta1s = [0.9 * 0.9 ** i for i in range(n)]

    def mirror(p, g, t):
        ramp = 0.0 if t <= 1 else min(1.0, (t - 1) / 2)
        # the class sees step-1 bias corrections on every call (steps travel by value)
        fo.sg11_step(p, g, st[0], st[1], st[2], sharp, [0] * n, [0.98] * n, beta1s, *W, rescale, 0.999, 1e-3, 1.0, 1e-8, 5.0, ramp,
                     5.0, 1.0)
    _drive(opt, m, 4, mirror)
    assert opt.get_global_step() == 4 and opt._flat_steps == [0] * n


def test_looksam_class():
    from grokking_optimizers import LookSAM
    m = _model(5)
    ref_m = copy.deepcopy(m)
    opt = LookSAM(m.parameters(), lr=1e-3, k=2)
    ref = torch.optim.AdamW(ref_m.parameters(), lr=1e-3, betas=(0.9, 0.98), eps=1e-8, weight_decay=1.0)
    crit = nn.CrossEntropyLoss()
    for t in range(3):
        x, y = _batch(200 + t)
        for mm, oo in ((m, opt), (ref_m, ref)):
            mm.zero_grad()
            crit(mm(x), y).backward()
            oo.step()
        _assert_close("adamw %d" % t, _np(m.parameters()), _np(ref_m.parameters()), rel=2e-5)
    assert opt.global_step == 3 and not opt.should_sam_step()
    # sam_step: parameters unchanged, directions unit-norm, gradients moved by alpha*|g|*v
    x, y = _batch(300)
    m.zero_grad()
    crit(m(x), y).backward()
    before_p, before_g = _np(m.parameters()), _np([p.grad for p in m.parameters()])
    opt.sam_step(m, x, y, crit)
    torch.cuda.synchronize()
    _assert_equal("params restored", _np(m.parameters()), before_p)
    for p, g0 in zip(m.parameters(), before_g):
        v = opt.state[p]["sam_direction"].cpu().numpy().reshape(-1)
        assert abs(np.linalg.norm(v.astype(np.float64)) - 1.0) < 1e-5
        want = g0 + 0.7 * np.linalg.norm(g0.astype(np.float64)) * v
        ok, worst = rel_close(p.grad.cpu().numpy().reshape(-1), want, 1e-4, 1e-7)
        assert ok, worst
    # the stored direction is the normalised gradient difference at the perturbed point
    mm = copy.deepcopy(m)
    gn = np.sqrt(sum((g.astype(np.float64) ** 2).sum() for g in before_g))
    with torch.no_grad():
        for p, g0 in zip(mm.parameters(), before_g):
            p.add_(torch.from_numpy(g0).to(DEV).reshape(p.shape), alpha=0.05 / (gn + 1e-12))
    mm.zero_grad()
    crit(mm(x), y).backward()
    for p, pm, g0 in zip(m.parameters(), mm.parameters(), before_g):
        d = pm.grad.cpu().numpy().reshape(-1).astype(np.float64) - g0
        assert np.allclose(opt.state[p]["sam_direction"].cpu().numpy().reshape(-1), d / np.linalg.norm(d), rtol=2e-3, atol=2e-4)


def test_supergrok15_sam_and_bilevel_steps():
    from grokking_optimizers import SuperGrok15
    m = _model(6)
    opt = SuperGrok15(m.parameters(), lr=1e-3, meta_hidden_dim=8)
    crit = nn.CrossEntropyLoss()
    x, y = _batch(400)
    m.zero_grad()
    crit(m(x), y).backward()
    p0, g0 = _np(m.parameters()), _np([p.grad for p in m.parameters()])
    loss = opt.sam_step(m, x, y, crit)
    assert np.isfinite(loss)
    _assert_equal("params untouched", _np(m.parameters()), p0)
    _assert_equal("grads untouched", _np([p.grad for p in m.parameters()]), g0)
    # independent evaluation of |grad(p + rho g/|g|) - grad(p)|
    mm = copy.deepcopy(m)
    gn = np.sqrt(sum((g.astype(np.float64) ** 2).sum() for g in g0))
    with torch.no_grad():
        for p, g in zip(mm.parameters(), g0):
            p.add_(torch.from_numpy(g).to(DEV).reshape(p.shape), alpha=0.05 / (gn + 1e-12))
    mm.zero_grad()
    crit(mm(x), y).backward()
    for i, (pm, g) in enumerate(zip(mm.parameters(), g0)):
        want = np.abs(pm.grad.cpu().numpy().reshape(-1) - g)
        got = opt._flat_sharpness[i].cpu().numpy()
        assert np.allclose(got, want, rtol=2e-3, atol=1e-6 * max(1.0, np.abs(want).max() / 1e-6) * 1e-2 + 1e-9), i
    # bilevel step: meta-net moves, model gradients are put back
    vx, vy = _batch(401)
    meta_opt = torch.optim.Adam(opt.meta_net.parameters(), lr=1e-2)
    w_before = [w.detach().clone() for w in opt.meta_net.parameters()]
    val = opt.bilevel_step(m, x, y, vx, vy, crit, meta_opt)
    assert np.isfinite(val) and opt._weights_dirty
    assert any(not torch.equal(a, b) for a, b in zip(w_before, opt.meta_net.parameters()))
    _assert_equal("grads restored", _np([p.grad for p in m.parameters()]), g0)
    opt.step(train_loss=1.0, val_loss=1.2, train_acc=0.5)
    metrics = opt.step_full(m, x, y, vx, vy, crit)
    assert isinstance(metrics, dict) and opt.get_global_step() == 2
