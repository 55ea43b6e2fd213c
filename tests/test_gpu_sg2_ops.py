"""The SuperGrok v2 step through the torch extension `_ops` (the reference's
pybind surface) and through the optimizer class, against the C ABI driven
directly and against the CPU checker."""
import numpy as np
import pytest
import torch

import workloads as wl
from helpers import DIMS
from sg2_harness import Sg2Case, per_tensor_scalars, shared_scalars, to_np
from oracle import oracle as orc
from grokking_optimizers import _cabi
from helpers import rel_close

pytestmark = pytest.mark.gpu


def test_ops_entry_is_bitwise_the_c_abi():
    from grokking_optimizers import _ops
    shapes = [(300,), (40, 64), (3000,), (0,)]
    a = Sg2Case(shapes, seed=1, random_state=True)
    b = Sg2Case(shapes, seed=1, random_state=True)
    grads = wl.make_grads(shapes, seed=2)
    sharps = [g.abs() for g in wl.make_grads(shapes, seed=3)]
    pt, sh = per_tensor_scalars(len(shapes), 2, lamb_eff=2.0), shared_scalars(wd_eff=4.5)
    a.gpu_step(grads, sharps, pt, sh)
    g = b.gpu
    dev = "cuda"
    _ops.supergrok2_mamba_peer_batched_step(
        [s["param"] for s in g], [x.reshape(-1).to(dev) for x in grads], [x.reshape(-1).to(dev) for x in sharps],
        [s["exp_avg"] for s in g], [s["exp_avg_sq"] for s in g], [s["mu"] for s in g], [s["gru"] for s in g],
        [s["mamba_fwd"] for s in g], [s["mamba_bwd"] for s in g], *b.Wgpu,
        [x["alpha"] for x in pt], [x["lamb_eff"] for x in pt], [x["beta1"] for x in pt], [x["bc1"] for x in pt],
        [x["bc2"] for x in pt], sh["rescale"], sh["beta2"], sh["lr"], sh["wd_eff"], sh["eps"],
        DIMS["d_model"], DIMS["d_state"], DIMS["d_inner"], DIMS["gru_hidden"], DIMS["num_heads"], DIMS["pk_dim"],
        DIMS["expert_hidden"], DIMS["num_experts"], b.counts_gpu)
    torch.cuda.synchronize()
    for sa, sb in zip(a.gpu, b.gpu):
        for k in sa:
            assert torch.equal(sa[k], sb[k]), k
    assert torch.equal(a.counts_gpu, b.counts_gpu)
    # single-tensor entry point, empty Mamba state = start from zero and do not carry
    c = Sg2Case([(500,)], seed=4)
    s = c.gpu[0]
    gg = wl.make_grads([(500,)], seed=5)[0].cuda()
    empty = torch.zeros(0, device=dev)
    _ops.supergrok2_mamba_peer_step(
        s["param"], gg, torch.zeros_like(gg), s["exp_avg"], s["exp_avg_sq"], s["mu"], s["gru"], empty, empty, *c.Wgpu,
        sh["rescale"], pt[0]["alpha"], pt[0]["lamb_eff"], pt[0]["beta1"], sh["beta2"], sh["lr"], sh["wd_eff"], sh["eps"],
        pt[0]["bc1"], pt[0]["bc2"], DIMS["d_model"], DIMS["d_state"], DIMS["d_inner"], DIMS["gru_hidden"], DIMS["num_heads"],
        DIMS["pk_dim"], DIMS["expert_hidden"], DIMS["num_experts"], c.counts_gpu)
    assert int(c.counts_gpu.sum()) == 4 * 500 and bool(torch.isfinite(s["param"]).all())
    with pytest.raises(RuntimeError, match="requires CUDA tensors"):
        _ops.supergrok2_mamba_peer_batched_step(
            [torch.zeros(4)], [torch.zeros(4)], [torch.zeros(4)], [torch.zeros(4)], [torch.zeros(4)], [torch.zeros(4)],
            [torch.zeros(4, 4)], [torch.zeros(16, 16)], [torch.zeros(16, 16)], *[w.cpu() for w in c.Wgpu],
            [0.98], [0.0], [0.9], [0.1], [0.001], 0.1, 0.999, 1e-3, 1.0, 1e-8, 8, 16, 16, 4, 4, 12, 16, 144,
            torch.zeros(144, dtype=torch.int32))


def test_supergrok2_class_against_checker_with_recycling():
    """SuperGrok2.step for 6 steps (lambda gate active, recycling every 2 steps) vs the CPU checker driven
    with the scalars the class is specified to compute."""
    import math
    from grokking_optimizers import SuperGrok2
    torch.manual_seed(0)
    shapes = [(700,), (32, 40), (5,)]
    p0 = wl.make_params(shapes, seed=3)
    params = [torch.nn.Parameter(p.clone().cuda()) for p in p0]
    opt = SuperGrok2(params, warmup_steps=0, warmup_ramp=1, recycle_interval=2, gradient_clipping=1.0)
    mn = opt.meta_net
    with torch.no_grad():                      # N(0,0.1) meta-weights so that routing is non-trivial
        gen = torch.Generator().manual_seed(7)
        for prm in mn.parameters():
            prm.copy_((torch.randn(prm.shape, generator=gen) * 0.1).to(prm.device))
    ref = []
    for p in p0:
        n = p.numel()
        ref.append(dict(param=p.numpy().reshape(-1).copy(), exp_avg=np.zeros(n, np.float32), exp_avg_sq=np.zeros(n, np.float32),
                        mu=np.zeros(n, np.float32), gru=np.zeros((n, 4), np.float32), mamba_fwd=np.zeros((16, 16), np.float32),
                        mamba_bwd=np.zeros((16, 16), np.float32)))
    counts = np.zeros(144, np.int32)
    sig = lambda s, v, th: 1.0 / (1.0 + math.exp(-s * (v - th)))
    f32 = lambda v: float(np.float32(v))
    for t in range(1, 7):
        acc = 0.85
        W = [w.detach().cpu().numpy() for w in mn.flat_weights()]      # weights in force for this step
        grads = wl.make_grads(shapes, seed=10 + t)
        for p, g in zip(params, grads):
            p.grad = g.clone().cuda()
        before = mn.expert_counts.clone()
        opt.step(train_acc=acc)
        lamb_eff = 2.0 * min(1.0, t / 1) * sig(20.0, acc, 0.8)
        wd_eff = 1.0 * (1.0 + 4.0 * sig(20.0, acc, 0.9))
        step_counts = np.zeros(144, np.int32)
        for i, g in enumerate(grads):
            gn = g.numpy().reshape(-1)
            gi = gn                                     # ||g|| << 1: the per-tensor clip multiplies by exactly 1.0
            b1 = 0.9 * (0.9 ** i)
            sc = dict(alpha=f32(0.98), lamb_eff=f32(lamb_eff), beta1=f32(b1), bc1=f32(1.0 - b1 ** t), bc2=f32(1.0 - 0.999 ** t),
                      rescale=f32(0.1), beta2=f32(0.999), lr=f32(1e-3), wd_eff=f32(wd_eff), eps=f32(1e-8))
            orc.sg2_step(W, ref[i], np.ascontiguousarray(gi, np.float32), np.zeros_like(gn), sc, chunk_len=_cabi.chunk_len_for([g_.numel() for g_ in grads]),
                         window=_cabi.lib().sg2_get_scan_window(), expert_counts=step_counts)
        for i, p in enumerate(params):
            ok, r = rel_close(p.detach().cpu().numpy().reshape(-1), ref[i]["param"], 1e-4, 1e-7)
            assert ok, ("param", t, i, r)
            ok, r = rel_close(opt._flat_gru_states[i].cpu().numpy(), ref[i]["gru"], 1e-4, 1e-7)
            assert ok, ("gru", t, i, r)
            ok, r = rel_close(opt._flat_mamba_fwd_states[i].cpu().numpy(), ref[i]["mamba_fwd"], 1e-4, 1e-7)
            assert ok, ("mamba_fwd", t, i, r)
        counts += step_counts
        if t % 2 == 0:
            assert int(mn.expert_counts.sum()) == 0            # recycling ran and reset the counters
            counts[:] = 0
        else:
            assert np.array_equal(mn.expert_counts.cpu().numpy(), counts)
    assert opt._flat_steps == [6, 6, 6]


def test_class_clip_matches_formula():
    from grokking_optimizers import SuperGrok2
    p = torch.nn.Parameter(torch.zeros(1000, device="cuda"))
    opt = SuperGrok2([p], gradient_clipping=0.5)
    g_big, g_small = torch.randn(1000, device="cuda"), torch.randn(1000, device="cuda") * 1e-3
    out = opt._clip([g_big, g_small])
    want = g_big * (0.5 / (g_big.norm() + 1e-12))
    assert torch.allclose(out[0], want, rtol=1e-6, atol=0) and torch.equal(out[1], g_small)
    # against the CPU checker, with non-finite entries, several tiles and 16-bit gradients
    import numpy as np
    from oracle import family_oracle as fo
    r = np.random.RandomState(4)
    cases = [r.randn(9000).astype(np.float32), (r.randn(5000) * 1e-4).astype(np.float32), r.randn(4096).astype(np.float32),
             r.randn(70).astype(np.float32), r.randn(1).astype(np.float32) * 3]
    cases[2][100] = np.nan
    cases[3][7] = -np.inf
    got = opt._clip([torch.from_numpy(c).cuda() for c in cases])
    for a, b in zip(got, fo.sg2_clip(cases, 0.5)):
        assert np.allclose(a.cpu().numpy(), b, rtol=1e-6, atol=0)
    h = [torch.from_numpy(c).cuda().to(torch.bfloat16) for c in cases[:2]]
    got = opt._clip(h)
    want = fo.sg2_clip([x.float().cpu().numpy() for x in h], 0.5)
    for a, b in zip(got, want):
        assert a.dtype == torch.bfloat16 and np.allclose(a.float().cpu().numpy(), b, rtol=2 ** -7, atol=0)
