"""The measured configurations at their stated length, against the CPU checkers after EVERY step, with the worst
tolerance ratio of each step printed so that drift over a chained run is visible:
  config 2  SuperGrok v1.5, 14-tensor set, 100 steps (SAM sharpness, clip active, progressive wd / gate)
  config 3  SuperGrok v2 through SuperGrok2.step, 14-tensor set, 50 steps, expert recycling every 10 steps
  config 5  Muon, one step over all 12 + 12 bf16 matrices
Gates as everywhere: integers bit-exact, fp32 state within 1e-4 relative (floors far below each state's scale);
config 3 additionally asserts what the design claims: every float of the v2 step equals the checker bit for bit."""
import math

import numpy as np
import pytest
import torch

import workloads as wl
from helpers import rel_close
from oracle import muon_oracle
from oracle import oracle as orc

pytestmark = pytest.mark.gpu

f32 = lambda v: float(np.float32(v))
# |a-b| <= 1e-4 max(|a|,|b|) + floor; the floor is about 1e-5 of each state's own scale (parameters 0.02, first
# moments 1e-5 .. 1e-4, second moments 1e-11 .. 1e-9) so that it only covers entries passing through zero
FLOORS = dict(param=1e-7, exp_avg=1e-10, exp_avg_sq=1e-16, mu=1e-10, gru=1e-8, mamba_fwd=1e-9, mamba_bwd=1e-9)


def test_config3_v2_fifty_steps_with_recycling_on_the_14_tensor_set():
    from concurrent.futures import ThreadPoolExecutor
    from grokking_optimizers import SuperGrok2, _cabi
    shapes = wl.shared14_shapes()
    P = len(shapes)
    p0 = wl.make_params(shapes, seed=0)
    params = [torch.nn.Parameter(p.clone().cuda()) for p in p0]
    opt = SuperGrok2(params, warmup_steps=0, warmup_ramp=1, recycle_interval=10, gradient_clipping=1.0)
    mn = opt.meta_net
    mn.load_flat_weights([w.cuda() for w in wl.meta_weights(7)])       # N(0, 0.1), drawn in `_ops` argument order
    ref = []
    for p in p0:
        n = p.numel()
        ref.append(dict(param=p.numpy().reshape(-1).copy(), exp_avg=np.zeros(n, np.float32), exp_avg_sq=np.zeros(n, np.float32),
                        mu=np.zeros(n, np.float32), gru=np.zeros((n, 4), np.float32), mamba_fwd=np.zeros((16, 16), np.float32),
                        mamba_bwd=np.zeros((16, 16), np.float32)))
    chunk_len = _cabi.chunk_len_for([wl.numel(s) for s in shapes])
    window = _cabi.lib().sg2_get_scan_window()
    sig = lambda s, v, th: 1.0 / (1.0 + math.exp(-s * (v - th)))
    counts = np.zeros(144, np.int32)
    recycled = 0
    acc = 0.85                              # gate and progressive weight decay both active
    for t in range(1, 51):
        W = [w.detach().cpu().numpy() for w in mn.flat_weights()]      # the weights in force for this step
        grads = wl.make_grads(shapes, seed=1 + t)
        for p, g in zip(params, grads):
            p.grad = g.clone().cuda()
        print("config 3 step", t, flush=True)
        opt.step(train_acc=acc)
        lamb_eff = 2.0 * min(1.0, t / 1) * sig(20.0, acc, 0.8)
        wd_eff = 1.0 * (1.0 + 4.0 * sig(20.0, acc, 0.9))
        step_counts = [np.zeros(144, np.int32) for _ in range(P)]

        def one(i):
            b1 = 0.9 * (0.9 ** i)
            sc = dict(alpha=f32(0.98), lamb_eff=f32(lamb_eff), beta1=f32(b1), bc1=f32(1.0 - b1 ** t), bc2=f32(1.0 - 0.999 ** t),
                      rescale=f32(0.1), beta2=f32(0.999), lr=f32(1e-3), wd_eff=f32(wd_eff), eps=f32(1e-8))
            gn = np.ascontiguousarray(grads[i].numpy().reshape(-1))    # ||g|| < 1: the per-tensor clip multiplies by exactly 1
            orc.sg2_step(W, ref[i], gn, np.zeros_like(gn), sc, chunk_len=chunk_len, window=window, expert_counts=step_counts[i])
        with ThreadPoolExecutor(8) as ex:
            list(ex.map(one, range(P)))
        worst = {}
        for i in range(P):
            got = dict(param=params[i].detach(), exp_avg=opt._flat_exp_avgs[i], exp_avg_sq=opt._flat_exp_avg_sqs[i], mu=opt._flat_mus[i],
                       gru=opt._flat_gru_states[i], mamba_fwd=opt._flat_mamba_fwd_states[i], mamba_bwd=opt._flat_mamba_bwd_states[i])
            for k, v in got.items():
                a = v.cpu().numpy().reshape(ref[i][k].shape)
                ok, r = rel_close(a, ref[i][k], 1e-4, FLOORS[k])
                worst[k] = max(worst.get(k, 0.0), r)
                assert ok, (k, t, i, r)
                assert np.array_equal(a, ref[i][k]), "step %d tensor %d: %s is not bit-identical to the checker" % (t, i, k)
        print("  worst tolerance ratios", {k: round(v, 4) for k, v in worst.items()}, flush=True)
        counts += sum(step_counts)
        if t % 10 == 0:
            assert int(mn.expert_counts.sum()) == 0                # the recycling decision ran and reset the counters
            after = [w.detach().cpu().numpy() for w in mn.flat_weights()]
            changed = any(not np.array_equal(a, b) for a, b in zip(after, W))
            recycled += int(changed)
            print("  recycling at step", t, "changed weights:", changed, "dead experts before:",
                  int((counts / max(1, counts.sum()) < 0.001).sum()), flush=True)
            counts[:] = 0
        else:
            assert np.array_equal(mn.expert_counts.cpu().numpy(), counts)
    assert recycled >= 1, "no recycling event changed the experts in 50 steps"
    assert opt._flat_steps == [50] * P


def test_config2_v15_hundred_steps():
    from grokking_optimizers import _ops as ops
    ops.supergrok15_set_gelu_mode("erf")
    shapes = wl.shared14_shapes()
    P, H = len(shapes), 32
    gen = torch.Generator().manual_seed(3)
    W1, b1 = torch.randn(H, 2, generator=gen) * 0.01, torch.zeros(H)
    W2, b2 = torch.randn(1, H, generator=gen) * 0.01, torch.zeros(1)
    Wd = [w.cuda() for w in (W1, b1, W2, b2)]
    p0 = [p.reshape(-1) for p in wl.make_params(shapes, seed=0)]
    params = [p.clone().cuda() for p in p0]
    eas, easqs, mus, sharps = ([torch.zeros_like(p) for p in params] for _ in range(4))
    rp = [p.numpy().copy() for p in p0]
    rea, reasq, rmu = ([np.zeros_like(p) for p in rp] for _ in range(3))
    sig = lambda x: 1.0 / (1.0 + np.exp(-x))
    floors = dict(sharp=1e-9, grad=1e-9, param=1e-7, exp_avg=1e-10, exp_avg_sq=1e-16, mu=1e-10)
    overall = {}
    for t in range(1, 101):
        g = [x.reshape(-1) for x in wl.make_grads(shapes, seed=100 + t, tail_frac=0.01, tail="normal")]
        gs = [x.reshape(-1) for x in wl.make_grads(shapes, seed=200 + t, tail_frac=0.01, tail="normal")]
        gd, gsd = [x.clone().cuda() for x in g], [x.clone().cuda() for x in gs]
        backups = [p.clone() for p in params]
        ops.supergrok15_sharpness_restore_all(params, sharps, backups, gsd, gd)      # sharp = |g_sam - g|
        rs = [np.abs(a.numpy() - b.numpy()) for a, b in zip(gs, g)]
        acc = t / 100.0
        wd_eff, gate = f32(1.0 * (1 + 4 * sig(20 * (acc - 0.9)))), f32(sig(20 * (acc - 0.8)))
        alphas, beta1s = [0.98] * P, [0.9 * 0.9 ** i for i in range(P)]
        ops.supergrok15_fused_step(params, gd, eas, easqs, mus, sharps, [t - 1] * P, alphas, beta1s, *Wd, 0.1, H, 0.999, 1e-3,
                                   wd_eff, 1e-8, 2.0, 1.0, gate, 1.0)
        step = np.float32(t)
        pt = [dict(alpha=f32(0.98), beta1=f32(b), bc1=f32(np.float32(1) - np.power(np.float32(b), step)),
                   bc2=f32(np.float32(1) - np.power(np.float32(0.999), step))) for b in beta1s]
        gn = [x.numpy().copy() for x in g]
        coef, on = orc.sg15_step(rp, gn, rs, rea, reasq, rmu, (W1.numpy(), b1.numpy(), W2.numpy(), b2.numpy(), f32(0.1)), pt,
                                 f32(np.float32(1.0) * np.float32(gate) * np.float32(2.0)), f32(0.999), f32(1e-3), wd_eff,
                                 f32(1e-8), f32(1.0), 0)
        assert on == 1                                     # ||g|| ~ 6.5 > 1: the clip is active
        worst = {}
        for i in range(P):
            for name, got, want in (("sharp", sharps[i], rs[i]), ("grad", gd[i], gn[i]), ("param", params[i], rp[i]),
                                    ("exp_avg", eas[i], rea[i]), ("exp_avg_sq", easqs[i], reasq[i]), ("mu", mus[i], rmu[i])):
                ok, r = rel_close(got.cpu().numpy(), want, 1e-4, floors[name])
                worst[name] = max(worst.get(name, 0.0), r)
                assert ok, (name, t, i, r)
        if t % 10 == 0 or t == 1:
            print("config 2 step", t, "worst tolerance ratios", {k: round(v, 4) for k, v in worst.items()}, flush=True)
        for k, v in worst.items():
            overall[k] = max(overall.get(k, 0.0), v)
    print("config 2, 100 steps, worst tolerance ratios overall", {k: round(v, 4) for k, v in overall.items()}, flush=True)


def test_config5_muon_one_step_over_all_24_matrices():
    """12 x [1024,4096] + 12 x [4096,1024] bf16 parameters, one step.  Gates: momentum buffer within 1e-4;
    updated bf16 parameters within one bf16 spacing of the fp32-iteration result rounded to bf16, except entries so
    close to zero that one spacing is below the deviation of the update itself (their fraction is reported and must
    stay below 5e-3; every entry is within one spacing + 2% of the largest update entry)."""
    from grokking_optimizers import _ops as ops
    shapes = [(1024, 4096)] * 12 + [(4096, 1024)] * 12
    gen = torch.Generator().manual_seed(0)
    momentum, lr, wd, ns = 0.95, 0.02, 1.0, 5
    p0 = [(torch.randn(*s, generator=gen) * 0.02).to(torch.bfloat16) for s in shapes]
    g0 = [(torch.randn(*s, generator=gen) * 1e-3).to(torch.bfloat16) for s in shapes]
    params = [p.clone().cuda() for p in p0]
    grads = [g.cuda() for g in g0]
    bufs = [torch.zeros(s, device="cuda") for s in shapes]
    print("config 5: muon step over 24 matrices", flush=True)
    ops.muon_fused_step(params, grads, bufs, momentum, lr, wd, ns)
    torch.cuda.synchronize()
    bf = lambda a: torch.from_numpy(np.ascontiguousarray(a)).to(torch.bfloat16).float().numpy()
    worst_frac = 0.0
    for i, s in enumerate(shapes):
        old = p0[i].float().numpy()
        rb = np.zeros(s, np.float32)
        tall = s[0] > s[1]
        # the iteration on the Gram matrix of the smaller dimension is the same product re-associated: run the fp32
        # restatement on the transpose of a tall matrix (4x fewer flops on the host), and transpose back
        if tall:
            newT, XT = muon_oracle.muon_step(old.T.copy(), g0[i].float().numpy().T.copy(), rb.T.copy(), momentum, lr, wd, ns)
            new_p, X = newT.T, XT.T
            rb = (np.float32(momentum) * rb + g0[i].float().numpy())
        else:
            new_p, X = muon_oracle.muon_step(old, g0[i].float().numpy(), rb, momentum, lr, wd, ns)
        ok, r = rel_close(bufs[i].cpu().numpy(), rb, 1e-4, 1e-9)
        assert ok, ("buf", i, r)
        got = params[i].float().cpu().numpy()
        want = bf(new_p)
        # spacing of bf16 at |want| (8 significant bits): 2^(floor(log2|want|) - 7)
        _, e = np.frexp(np.maximum(np.abs(want), 2.0 ** -120))
        ulp = np.ldexp(1.0, e - 8)
        diff = np.abs(got - want)
        d = diff / ulp
        frac = float((d > 1.0).mean())
        upd_max = float(np.abs(0.2 * lr * X).max())
        # the only entries that can be off by more than one spacing are those so close to zero that the spacing is
        # below the bf16-vs-fp32 deviation of the update itself (bounded here by 2% of the largest update entry)
        assert bool((diff <= ulp + 0.02 * upd_max).all()), ("param", i, float((diff - ulp).max()), upd_max)
        print("  matrix %2d %s: rounded differently %.2e, beyond one spacing %.2e (all within one spacing + %.1e)"
              % (i, s, float((diff > 0).mean()), frac, 0.02 * upd_max), flush=True)
        worst_frac = max(worst_frac, frac)
    print("config 5 worst fraction of entries beyond one bf16 spacing: %.3e" % worst_frac, flush=True)
    # N(0, 0.02) parameters: about 0.5% of the entries lie below 1.3e-4, where one bf16 spacing is under 1e-6
    assert worst_frac <= 5e-3
