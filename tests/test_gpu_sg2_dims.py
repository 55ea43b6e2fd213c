"""The batched step at meta-net dimensions other than the two sets the kernels are specialised for, against the CPU
checker: what the reference's training harness passes (expert_hidden = 4), small and medium scan blocks (run embedded
in a compiled scan geometry: the checker runs on the embedded net, tests/sg2_harness.embed_in_geometry, whose
equivalence with the original is pinned in tests/test_oracle_sg2_dims.py), other GRU / head / sub-key / expert sizes
(the run-time-dimension per-element kernel).  Gates as everywhere: permutation, expert indices and counts bit-exact,
floats within 1e-4 relative."""
import math

import numpy as np
import pytest
import torch

import workloads as wl
from dims_cases import CASES
from helpers import rel_close
from oracle import oracle as orc
from sg2_harness import Sg2Case, embed_in_geometry, per_tensor_scalars, shared_scalars

pytestmark = pytest.mark.gpu

REL, FLOOR = 1e-4, 1e-7


@pytest.fixture(autouse=True)
def _default_chunk():
    from grokking_optimizers import _cabi
    _cabi.lib().sg2_set_chunk_len(0)
    _cabi.lib().sg2_set_scan_window(-1)
    yield
    _cabi.lib().sg2_set_chunk_len(0)
    _cabi.lib().sg2_set_scan_window(-1)


@pytest.mark.parametrize("name", sorted(CASES))
def test_step_matches_checker_at_these_dims(name):
    from grokking_optimizers import _cabi
    dims = CASES[name]
    shapes = [(1,), (63,), (300,), (70, 90), (0,), (5000,), (64,)]
    dtypes = [torch.float32] * 5 + [torch.bfloat16, torch.float16]
    for cl, std in ((256, 0.2), (0, 0.1)):
        assert _cabi.lib().sg2_set_chunk_len(cl) == 0
        case = Sg2Case(shapes, dtypes=dtypes, seed=3 + cl, random_state=True, dims=dims, weights=wl.meta_weights(17, dims, std=std))
        for t in (1, 2):
            grads = wl.make_grads(shapes, seed=10 + t, std=0.02, tail_frac=0.005, tail="student3")
            sharps = [g.abs() * 0.5 for g in wl.make_grads(shapes, seed=500 + t, std=0.02)]
            pt, sh = per_tensor_scalars(case.P, t, 2.0), shared_scalars(4.5)
            print(name, "chunk", cl, "step", t, flush=True)
            case.gpu_step(grads, sharps, pt, sh)
            dbg = case.oracle_step(grads, sharps, pt, sh, cl or None)
            worst = case.compare(dbg, REL, FLOOR)
            print("  worst tolerance ratios", worst, flush=True)
        used = int((case.counts_np > 0).sum())
        print("  experts used:", used, "of", dims["num_experts"], flush=True)


@pytest.mark.parametrize("kw", [dict(expert_hidden=4), dict(d_model=4, d_state=8), dict(gru_hidden=8, num_peer_heads=2, num_experts=36, expert_hidden=8)])
def test_class_steps_at_these_dims(kw):
    """SuperGrok2(...).step() with non-default meta-net sizes, three steps against the checker (the reference's harness
    constructs the optimizer with expert_hidden = 4)."""
    from grokking_optimizers import SuperGrok2, _cabi
    shapes = [(300,), (40, 64), (3000,)]
    P = len(shapes)
    p0 = wl.make_params(shapes, seed=0)
    params = [torch.nn.Parameter(p.clone().cuda()) for p in p0]
    torch.manual_seed(5)
    opt = SuperGrok2(params, warmup_steps=0, warmup_ramp=1, recycle_interval=0, gradient_clipping=1.0, **kw)
    mn = opt.meta_net
    with torch.no_grad():
        for p in mn.parameters():            # away from the near-zero initial keys and experts: routing spreads, experts contribute
            if p.dim() > 0 and float(p.abs().max()) < 0.05:
                p.add_(torch.randn_like(p) * 0.2)
    opt._weights_dirty = True
    dims = dict(d_model=mn.d_model, d_state=mn.d_state, d_inner=mn.mamba_fwd.d_inner, gru_hidden=mn.gru_hidden, num_heads=mn.num_peer_heads,
                pk_dim=mn.pk_dim, expert_hidden=mn.expert_hidden, num_experts=mn.num_experts)
    W, odims = embed_in_geometry([w.detach().cpu().reshape(s) for w, s in zip(mn.flat_weights(), wl.meta_weight_shapes(dims))], dims)
    W = [w.numpy() for w in W]
    DI, DS = odims["d_inner"], odims["d_state"]
    ref = []
    for p in p0:
        n = p.numel()
        ref.append(dict(param=p.numpy().reshape(-1).copy(), exp_avg=np.zeros(n, np.float32), exp_avg_sq=np.zeros(n, np.float32),
                        mu=np.zeros(n, np.float32), gru=np.zeros((n, dims["gru_hidden"]), np.float32),
                        mamba_fwd=np.zeros((DI, DS), np.float32), mamba_bwd=np.zeros((DI, DS), np.float32)))
    chunk_len = _cabi.chunk_len_for([wl.numel(s) for s in shapes])
    window = _cabi.lib().sg2_get_scan_window()
    f32 = lambda v: float(np.float32(v))
    sig = lambda s, v, th: 1.0 / (1.0 + math.exp(-s * (v - th)))
    acc = 0.85
    counts = np.zeros(dims["num_experts"], np.int32)
    for t in (1, 2, 3):
        grads = wl.make_grads(shapes, seed=1 + t)
        for p, g in zip(params, grads):
            p.grad = g.clone().cuda()
        opt.step(train_acc=acc)
        lamb_eff = 2.0 * min(1.0, t / 1) * sig(20.0, acc, 0.8)
        wd_eff = 1.0 * (1.0 + 4.0 * sig(20.0, acc, 0.9))
        for i in range(P):
            b1 = 0.9 * (0.9 ** i)
            sc = dict(alpha=f32(0.98), lamb_eff=f32(lamb_eff), beta1=f32(b1), bc1=f32(1.0 - b1 ** t), bc2=f32(1.0 - 0.999 ** t),
                      rescale=f32(0.1), beta2=f32(0.999), lr=f32(1e-3), wd_eff=f32(wd_eff), eps=f32(1e-8))
            gn = np.ascontiguousarray(grads[i].numpy().reshape(-1))
            orc.sg2_step(W, ref[i], gn, np.zeros_like(gn), sc, dims=odims, chunk_len=chunk_len, window=window, expert_counts=counts)
        di, ds = dims["d_inner"], dims["d_state"]
        for i in range(P):
            got = dict(param=params[i].detach(), exp_avg=opt._flat_exp_avgs[i], exp_avg_sq=opt._flat_exp_avg_sqs[i], mu=opt._flat_mus[i],
                       gru=opt._flat_gru_states[i], mamba_fwd=opt._flat_mamba_fwd_states[i], mamba_bwd=opt._flat_mamba_bwd_states[i])
            for k, v in got.items():
                want = ref[i][k][:di, :ds] if k.startswith("mamba") else ref[i][k]
                ok, r = rel_close(v.cpu().numpy().reshape(want.shape), want, REL, 1e-9)
                assert ok, (kw, t, i, k, r)
        assert np.array_equal(mn.expert_counts.cpu().numpy(), counts), (kw, t)
    print(kw, "experts used:", int((counts > 0).sum()), "of", dims["num_experts"], flush=True)
