"""The CPU checker at meta-net dimensions other than the defaults, and the embedding of a small scan block in a
compiled scan geometry (tests/sg2_harness.embed_in_geometry: what the library does on the device for such blocks).

  * the float64 policy at run-time dimensions against the independently written torch restatement of the reference's
    Python forward (tests/ref_fp64.py), which takes the same dimensions: an indexing mistake that only shows when
    d_inner != d_state, d_model is odd or num_experts < pk_dim^2 fails here;
  * the embedded net against the original: the same function.  Float64: to rounding of the chains (the embedding only
    adds terms with a zero factor).  fp32: the embedded run groups the gates' shared reciprocals and decides its
    summary walk over more lanes, so a few last bits differ; 2e-5 relative."""
import numpy as np
import pytest
import torch

import workloads as wl
from dims_cases import CASES
from helpers import copy_state, default_scalars, f32_scalars, random_state_np, rel_close
from oracle import oracle as orc
import ref_fp64
from sg2_harness import embed_in_geometry


def _grad(n, seed, std=1e-3):
    return (np.random.RandomState(seed).randn(n) * std).astype(np.float32)


def _run(W, st, g, s, sc, dims, precision, chunk_len=0, window=0, counts=None):
    st = copy_state(st)
    dbg = orc.sg2_step(W, st, g, s, sc, dims=dims, precision=precision, chunk_len=chunk_len, window=window,
                       expert_counts=counts, debug=True)
    return st, dbg


@pytest.mark.parametrize("name", sorted(CASES))
def test_f64_checker_matches_independent_restatement_at_these_dims(name):
    dims = CASES[name]
    n = 150
    W = [w.numpy() for w in wl.meta_weights(11, dims, std=0.3)]
    st = random_state_np(n, 5, dims)
    g, s = _grad(n, 1, 0.05), np.abs(_grad(n, 2, 0.05))
    sc = f32_scalars(default_scalars(i=2, step=3, lamb_eff=2.0, wd_eff=4.5))
    new, dbg = _run(W, st, g, s, sc, dims, 64)
    t = lambda a: torch.from_numpy(np.asarray(a))
    ref = ref_fp64.step([t(w) for w in W], t(st["param"]), t(g), t(s), t(st["exp_avg"]), t(st["exp_avg_sq"]), t(st["mu"]),
                        t(st["gru"]), t(st["mamba_fwd"]), t(st["mamba_bwd"]), sc, dims)
    assert np.array_equal(dbg["perm"], ref["perm"].numpy().astype(np.int32))
    mism = dbg["expert_idx"] != ref["expert_idx"].numpy().astype(np.int32)
    assert not mism.any(), int(mism.sum())
    for k in ("param", "exp_avg", "exp_avg_sq", "mu", "gru", "mamba_fwd", "mamba_bwd"):
        ok, ratio = rel_close(new[k], ref[k].numpy().reshape(new[k].shape), rel=2e-7, floor=1e-12)
        assert ok, (k, ratio)
    for d, key in ((0, "ctx_f"), (1, "ctx_b")):
        ok, ratio = rel_close(dbg["ctx"][d], ref[key].numpy(), rel=2e-7, floor=1e-10)
        assert ok, (key, ratio)
    assert int(dbg["expert_idx"].max()) < dims["num_experts"]


@pytest.mark.parametrize("name", sorted(CASES))
@pytest.mark.parametrize("precision", [64, 32])
def test_embedded_net_computes_the_same_function(name, precision):
    dims = CASES[name]
    Wt = wl.meta_weights(13, dims, std=0.2)
    eW, edims = embed_in_geometry(Wt, dims)
    n = 700
    st = random_state_np(n, 9, dims)
    est = copy_state(st)
    for k in ("mamba_fwd", "mamba_bwd"):
        e = np.zeros((edims["d_inner"], edims["d_state"]), np.float32)
        e[:dims["d_inner"], :dims["d_state"]] = st[k]
        est[k] = e
    g, s = _grad(n, 3, 0.02), np.abs(_grad(n, 4, 0.02))
    sc = f32_scalars(default_scalars(i=1, step=2, lamb_eff=2.0, wd_eff=4.5))
    ca, cb = np.zeros(dims["num_experts"], np.int32), np.zeros(dims["num_experts"], np.int32)
    a, da = _run([w.numpy() for w in Wt], st, g, s, sc, dims, precision, 256, 64, ca)
    b, db = _run([w.numpy() for w in eW], est, g, s, sc, edims, precision, 256, 64, cb)
    rel, floor = (1e-11, 1e-14) if precision == 64 else (2e-5, 1e-8)
    assert np.array_equal(da["perm"], db["perm"])
    mism = da["expert_idx"] != db["expert_idx"]
    if precision == 64:
        assert not mism.any()
        assert np.array_equal(ca, cb)
    else:
        assert (da["margin"].min(-1)[mism] < 1e-5).all()
    good = ~mism.any(-1)
    dm, di, ds = dims["d_model"], dims["d_inner"], dims["d_state"]
    ok, r = rel_close(da["ctx"], db["ctx"][:, :, :dm], rel, floor)
    assert ok, ("ctx", r)
    assert not db["ctx"][:, :, dm:].any()
    for k in ("param", "exp_avg", "exp_avg_sq", "mu"):
        ok, r = rel_close(a[k][good], b[k][good], rel, floor)
        assert ok, (k, r)
    ok, r = rel_close(a["gru"], b["gru"], rel, floor)
    assert ok, ("gru", r)
    for k in ("mamba_fwd", "mamba_bwd"):
        ok, r = rel_close(a[k], b[k][:di, :ds], rel * 10, floor)
        assert ok, (k, r)
        assert not b[k][di:].any() and not b[k][:, ds:].any()
