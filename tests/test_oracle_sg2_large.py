"""The CPU checker at the second geometry the step kernels are built for (d_model=16, d_state=32, d_inner=32: the
largest scan block csrc/supergrok2_mamba_peer_kernels.cu:36-42 of the reference admits): its fp64 policy against
the independent torch restatement (tests/ref_fp64.py, written from the Python module, which takes its sizes from
the weight shapes), its fp32 policy against the fp64 one, and chunked against sequential evaluation."""
import numpy as np
import pytest
import torch

import ref_fp64
import workloads as wl
from helpers import copy_state, default_scalars, f32_scalars, random_state_np, rel_close, weights_np
from oracle import oracle as orc

LARGE = dict(wl.DEFAULT_DIMS, d_model=16, d_state=32, d_inner=32)


def _grad(n, seed, std=1e-3):
    return (np.random.RandomState(seed).randn(n) * std).astype(np.float32)


def _run(W, st, g, s, sc, precision, chunk_len=0, window=0):
    st = copy_state(st)
    dbg = orc.sg2_step(W, st, g, s, f32_scalars(sc), dims=LARGE, precision=precision, chunk_len=chunk_len, window=window, debug=True)
    return st, dbg


@pytest.mark.parametrize("n,seed", [(1, 0), (7, 1), (200, 2)])
def test_f64_checker_matches_independent_restatement(n, seed):
    W = weights_np(dims=LARGE)
    st = random_state_np(n, seed, LARGE)
    g, s = _grad(n, 100 + seed), np.abs(_grad(n, 200 + seed))
    sc = f32_scalars(default_scalars(i=2, step=3, lamb_eff=2.0, wd_eff=4.5))
    new, dbg = _run(W, st, g, s, sc, 64)
    t = lambda a: torch.from_numpy(np.asarray(a))
    ref = ref_fp64.step([t(w) for w in W], t(st["param"]), t(g), t(s), t(st["exp_avg"]), t(st["exp_avg_sq"]),
                        t(st["mu"]), t(st["gru"]), t(st["mamba_fwd"]), t(st["mamba_bwd"]), sc, LARGE)
    assert np.array_equal(dbg["perm"], ref["perm"].numpy().astype(np.int32))
    assert np.array_equal(dbg["expert_idx"], ref["expert_idx"].numpy().astype(np.int32))
    for k in ("param", "exp_avg", "exp_avg_sq", "mu", "gru", "mamba_fwd", "mamba_bwd"):
        ok, ratio = rel_close(new[k], ref[k].numpy().reshape(new[k].shape), rel=2e-7, floor=1e-12)
        assert ok, (k, ratio)
    for d, key in enumerate(("ctx_f", "ctx_b")):
        assert dbg["ctx"][d].shape == (n, 16)
        ok, ratio = rel_close(dbg["ctx"][d], ref[key].numpy(), rel=2e-7, floor=1e-10)
        assert ok, (key, ratio)


@pytest.mark.parametrize("n", [16, 300, 1024])
def test_f32_policy_close_to_f64(n):
    W = weights_np(dims=LARGE)
    st = random_state_np(n, n, LARGE)
    g, s = _grad(n, n + 1), np.abs(_grad(n, n + 2))
    sc = default_scalars(i=1, step=2, lamb_eff=2.0, wd_eff=4.5)
    a, da = _run(W, st, g, s, sc, 32)
    b, db = _run(W, st, g, s, sc, 64)
    assert np.array_equal(da["perm"], db["perm"])
    mism = da["expert_idx"] != db["expert_idx"]
    assert (db["margin"].min(-1)[mism] < 1e-5).all()       # a routing flip is only legitimate at a near-tie
    good = ~mism.any(-1)
    for k in ("exp_avg", "exp_avg_sq", "mu", "param"):
        ok, ratio = rel_close(a[k][good], b[k][good], rel=2e-5, floor=1e-9)
        assert ok, (k, ratio)
    ok, ratio = rel_close(a["gru"], b["gru"], rel=2e-5, floor=1e-6)
    assert ok, ratio
    for k in ("mamba_fwd", "mamba_bwd"):
        ok, ratio = rel_close(a[k], b[k], rel=1e-4, floor=1e-6)
        assert ok, (k, ratio)


@pytest.mark.parametrize("n,chunk,window", [(1000, 64, 0), (1000, 256, 64), (700, 1, 0)])
def test_chunked_scan_matches_sequential(n, chunk, window):
    W = weights_np(dims=LARGE)
    st = random_state_np(n, 5, LARGE)
    g, s = _grad(n, 6), np.abs(_grad(n, 7))
    sc = default_scalars(i=0, step=1)
    a, da = _run(W, st, g, s, sc, 64, chunk_len=0)
    b, db = _run(W, st, g, s, sc, 64, chunk_len=chunk, window=window)
    for k in ("param", "gru", "mamba_fwd", "mamba_bwd"):
        ok, ratio = rel_close(a[k], b[k], rel=1e-9, floor=1e-12)
        assert ok, (k, ratio)
    assert np.array_equal(da["expert_idx"], db["expert_idx"])
