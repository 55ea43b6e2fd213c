"""The batched step at the second geometry the kernels are built for (d_model=16, d_state=32, d_inner=32: 512-lane
scan workgroups, 16 RoPE pairs per column) against the CPU checker: integers bit-exact, floats within 1e-4 relative,
and additionally bit for bit, which is what sharing include/sg_math.h with the checker is meant to give."""
import numpy as np
import pytest
import torch

import workloads as wl
from sg2_harness import Sg2Case, per_tensor_scalars, shared_scalars

pytestmark = pytest.mark.gpu

LARGE = dict(wl.DEFAULT_DIMS, d_model=16, d_state=32, d_inner=32)
REL, FLOOR = 1e-4, 1e-7


@pytest.fixture(autouse=True)
def _default_chunk():
    from grokking_optimizers import _cabi
    _cabi.lib().sg2_set_chunk_len(0)
    _cabi.lib().sg2_set_scan_window(-1)
    yield
    _cabi.lib().sg2_set_chunk_len(0)
    _cabi.lib().sg2_set_scan_window(-1)


def _steps(case, steps, chunk_len, sharp=True, lamb_eff=2.0, wd_eff=4.5):
    for t in range(1, steps + 1):
        grads = wl.make_grads(case.shapes, seed=10 + t, tail_frac=0.005, tail="student3")
        sharps = [g.abs() * 0.5 for g in wl.make_grads(case.shapes, seed=500 + t)] if sharp else [torch.zeros_like(g) for g in grads]
        pt, sh = per_tensor_scalars(case.P, t, lamb_eff), shared_scalars(wd_eff)
        print("large geometry step", t, "chunk", chunk_len, [tuple(s) for s in case.shapes], flush=True)
        case.gpu_step(grads, sharps, pt, sh)
        dbg = case.oracle_step(grads, sharps, pt, sh, chunk_len)
        print("  worst tolerance ratios", case.compare(dbg, REL, FLOOR), flush=True)
        ctx = case.step_fn.ctx.cpu().numpy()
        for i in range(case.P):
            a, b = int(case.offsets[i]), int(case.offsets[i + 1])
            if a == b:
                continue
            for d in range(2):
                assert np.array_equal(ctx[d, a:b], dbg[i]["ctx"][d]), "tensor %d: context %d not bit-identical" % (i, d)
            for k in ("exp_avg", "exp_avg_sq", "mu", "gru", "mamba_fwd", "mamba_bwd"):
                got = case.gpu[i][k].cpu().numpy().reshape(case.np[i][k].shape)
                assert np.array_equal(got, case.np[i][k]), "tensor %d: %s not bit-identical" % (i, k)


def test_ragged_tensors_several_chunks():
    """Chunk lengths 64 and 256 (summaries, adaptive window, chunk prefix) on ragged sizes, random carried state."""
    from grokking_optimizers import _cabi
    shapes = [(1,), (63,), (300,), (70, 90), (0,), (5000,), (64,)]
    for cl, win in ((64, -1), (256, 64)):
        assert _cabi.lib().sg2_set_chunk_len(cl) == 0 and _cabi.lib().sg2_set_scan_window(win) == 0
        case = Sg2Case(shapes, seed=cl, random_state=True, dims=LARGE)
        _steps(case, 2, cl)


def test_default_chunk_and_16_bit_parameters():
    shapes = [(300,), (1500,), (1500,), (40000,)]
    dtypes = [torch.float32, torch.float16, torch.bfloat16, torch.float32]
    case = Sg2Case(shapes, dtypes=dtypes, seed=4, random_state=True, dims=LARGE)
    _steps(case, 2, None)
    case = Sg2Case([(2000,), (100,)], seed=5, dims=LARGE)
    _steps(case, 1, None, sharp=False, lamb_eff=0.0, wd_eff=1.0)      # all-zero sharpness: the kernels skip that term


def test_module_initialised_weights():
    """Mamba3PEERMetaNet(d_model=16, d_state=32) as constructed: slow poles, the walk over several summary blocks."""
    from grokking_optimizers import _cabi
    from grokking_optimizers.mamba3_peer_metanet import Mamba3PEERMetaNet
    torch.manual_seed(0)
    mn = Mamba3PEERMetaNet(d_model=16, d_state=32)
    W = [w.detach().float().contiguous() for w in mn.flat_weights()]
    assert _cabi.lib().sg2_set_chunk_len(2048) == 0
    case = Sg2Case([(9000,), (3000,)], seed=2, weights=W, dims=LARGE)
    _steps(case, 2, 2048)


def test_optimizer_class_with_large_meta_net():
    """SuperGrok2(d_model=16, d_state=32): three steps through the class and `_ops`, against the checker."""
    from grokking_optimizers import SuperGrok2, _cabi
    from oracle import oracle as orc
    f32 = lambda v: float(np.float32(v))
    shapes = [(50, 60), (700,), (33,)]
    p0 = wl.make_params(shapes, seed=0)
    params = [torch.nn.Parameter(p.clone().cuda()) for p in p0]
    opt = SuperGrok2(params, warmup_steps=0, warmup_ramp=1, d_model=16, d_state=32)
    mn = opt.meta_net
    mn.load_flat_weights([w.cuda() for w in wl.meta_weights(7, LARGE)])
    ref = [dict(param=p.numpy().reshape(-1).copy(), exp_avg=np.zeros(p.numel(), np.float32), exp_avg_sq=np.zeros(p.numel(), np.float32),
                mu=np.zeros(p.numel(), np.float32), gru=np.zeros((p.numel(), 4), np.float32), mamba_fwd=np.zeros((32, 32), np.float32),
                mamba_bwd=np.zeros((32, 32), np.float32)) for p in p0]
    chunk_len = _cabi.chunk_len_for([wl.numel(s) for s in shapes])
    window = _cabi.lib().sg2_get_scan_window()
    W = [w.detach().cpu().numpy() for w in mn.flat_weights()]
    for t in range(1, 4):
        grads = wl.make_grads(shapes, seed=1 + t)
        for p, g in zip(params, grads):
            p.grad = g.clone().cuda()
        print("class step", t, flush=True)
        opt.step(train_acc=0.0)
        for i in range(len(shapes)):
            b1 = 0.9 * (0.9 ** i)
            sc = dict(alpha=f32(0.98), lamb_eff=f32(2.0 / (1.0 + np.exp(16.0))), beta1=f32(b1), bc1=f32(1.0 - b1 ** t), bc2=f32(1.0 - 0.999 ** t),
                      rescale=f32(0.1), beta2=f32(0.999), lr=f32(1e-3), wd_eff=f32(1.0 * (1.0 + 4.0 / (1.0 + np.exp(18.0)))), eps=f32(1e-8))
            gn = np.ascontiguousarray(grads[i].numpy().reshape(-1))
            orc.sg2_step(W, ref[i], gn, np.zeros_like(gn), sc, dims=LARGE, chunk_len=chunk_len, window=window)
            from helpers import rel_close
            for k, v in dict(param=params[i].detach(), exp_avg=opt._flat_exp_avgs[i], gru=opt._flat_gru_states[i],
                             mamba_fwd=opt._flat_mamba_fwd_states[i]).items():
                ok, r = rel_close(v.cpu().numpy().reshape(ref[i][k].shape), ref[i][k], 1e-4, 1e-7)
                assert ok, (k, t, i, r)


def test_bilevel_pass_refuses_the_large_geometry():
    from grokking_optimizers import _cabi
    g = [torch.zeros(100, device="cuda")]
    st = [torch.zeros(32, 32, device="cuda")]
    with pytest.raises(RuntimeError, match="bilevel pass are built for blocks up to"):
        _cabi.Sg2Bilevel([w.cuda() for w in wl.meta_weights(7, LARGE)], g, g, st, st, dims=LARGE)
