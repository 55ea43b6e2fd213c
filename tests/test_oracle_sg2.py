"""Pins the CPU checker of the SuperGrok v2 step (oracle/sg2_oracle.cpp).

The reference's own tests carry no numeric expectations for this path, so the
checker is pinned against things that do not share its code:
  * numpy's stable argsort and an O(N^2) rank count (sort),
  * an independently written float64 torch restatement (tests/ref_fp64.py),
  * torch.optim.AdamW when the meta-net contribution is switched off,
  * closed forms of the recurrence in special cases,
  * structural identities (reverse == forward of the flipped input, state
    carry, chunked == sequential).
"""
import numpy as np
import pytest
import torch

import workloads as wl
from helpers import (DIMS, copy_state, default_scalars, f32_scalars, fresh_state_np, random_state_np,
                     rel_close, weights_np)
from oracle import oracle as orc
import ref_fp64


def _grad(n, seed, std=1e-3):
    return (np.random.RandomState(seed).randn(n) * std).astype(np.float32)


# ----------------------------------------------------------------- sort
@pytest.mark.parametrize("n", [1, 2, 16, 255, 256, 1000, 4097])
def test_sort_matches_numpy_stable(n):
    g = _grad(n, n)
    g[::7] = g[0]                      # exact ties
    if n > 4:
        g[1], g[2], g[3] = 0.0, -0.0, np.nan
        g[4] = np.inf
    perm = orc.sort_perm(g)
    key = np.abs(np.where(np.isfinite(g), g, 0)).astype(np.float32)
    assert np.array_equal(perm, np.argsort(key, kind="stable").astype(np.int32))


def test_sort_brute_force_rank():
    g = _grad(64, 5)
    g[10] = -g[20]
    g[30] = g[20]
    key = np.abs(g)
    perm = orc.sort_perm(g)
    rank = np.empty(64, np.int64)
    for i in range(64):
        rank[i] = sum(1 for j in range(64) if key[j] < key[i] or (key[j] == key[i] and j < i))
    inv = np.empty(64, np.int64)
    inv[perm] = np.arange(64)
    assert np.array_equal(inv, rank)


# ------------------------------------------------- fp64 checker vs independent restatement
def _run_oracle(W, st, g, s, sc, precision, chunk_len=0, counts=None, window=0):
    st = copy_state(st)
    dbg = orc.sg2_step(W, st, g, s, f32_scalars(sc), precision=precision, chunk_len=chunk_len, window=window,
                       expert_counts=counts, debug=True)
    return st, dbg


@pytest.mark.parametrize("n,seed", [(1, 0), (5, 1), (64, 2), (300, 3)])
def test_f64_checker_matches_independent_restatement(n, seed):
    W = weights_np()
    st = random_state_np(n, seed)
    g = _grad(n, 100 + seed)
    s = np.abs(_grad(n, 200 + seed))
    sc = f32_scalars(default_scalars(i=2, step=3, lamb_eff=2.0, wd_eff=4.5))
    new, dbg = _run_oracle(W, st, g, s, sc, 64)
    t = lambda a: torch.from_numpy(np.asarray(a))
    ref = ref_fp64.step([t(w) for w in W], t(st["param"]), t(g), t(s), t(st["exp_avg"]), t(st["exp_avg_sq"]),
                        t(st["mu"]), t(st["gru"]), t(st["mamba_fwd"]), t(st["mamba_bwd"]), sc, DIMS)
    assert np.array_equal(dbg["perm"], ref["perm"].numpy().astype(np.int32))
    assert np.array_equal(dbg["expert_idx"], ref["expert_idx"].numpy().astype(np.int32))
    # the checker rounds its outputs to fp32: compare at fp32 resolution
    for k in ("param", "exp_avg", "exp_avg_sq", "mu", "gru", "mamba_fwd", "mamba_bwd"):
        ok, ratio = rel_close(new[k], ref[k].numpy().reshape(new[k].shape), rel=2e-7, floor=1e-12)
        assert ok, (k, ratio)
    ok, ratio = rel_close(dbg["ctx"][0], ref["ctx_f"].numpy(), rel=2e-7, floor=1e-10)
    assert ok, ratio
    ok, ratio = rel_close(dbg["ctx"][1], ref["ctx_b"].numpy(), rel=2e-7, floor=1e-10)
    assert ok, ratio


# ------------------------------------------------- fp32 policy vs fp64 policy
@pytest.mark.parametrize("n", [1, 16, 255, 256, 512, 1024])
def test_f32_policy_close_to_f64(n):
    W = weights_np()
    st = random_state_np(n, n)
    g, s = _grad(n, n + 1), np.abs(_grad(n, n + 2))
    sc = default_scalars(i=1, step=2, lamb_eff=2.0, wd_eff=4.5)
    a, da = _run_oracle(W, st, g, s, sc, 32)
    b, db = _run_oracle(W, st, g, s, sc, 64)
    assert np.array_equal(da["perm"], db["perm"])
    mism = da["expert_idx"] != db["expert_idx"]
    # a routing flip is only legitimate at a near-tie of the two best scores
    assert (db["margin"].min(-1)[mism] < 1e-5).all()
    good = ~mism.any(-1)
    for k in ("exp_avg", "exp_avg_sq", "mu", "param"):
        ok, ratio = rel_close(a[k][good], b[k][good], rel=2e-5, floor=1e-9)
        assert ok, (k, ratio)
    ok, ratio = rel_close(a["gru"], b["gru"], rel=2e-5, floor=1e-6)
    assert ok, ratio
    for k in ("mamba_fwd", "mamba_bwd"):
        ok, ratio = rel_close(a[k], b[k], rel=1e-4, floor=1e-6)
        assert ok, (k, ratio)


# ------------------------------------------------- chunked == sequential
@pytest.mark.parametrize("n,chunk", [(1000, 64), (1000, 256), (1024, 256), (257, 256), (700, 1)])
def test_chunked_scan_matches_sequential(n, chunk):
    W = weights_np()
    st = random_state_np(n, 7)
    g, s = _grad(n, 8), np.abs(_grad(n, 9))
    sc = default_scalars()
    for prec, rel in ((64, 1e-9), (32, 1e-5)):
        a, da = _run_oracle(W, st, g, s, sc, prec, 0)
        b, db = _run_oracle(W, st, g, s, sc, prec, chunk)
        ok, ratio = rel_close(da["ctx"], db["ctx"], rel=rel, floor=1e-7 if prec == 32 else 1e-12)
        assert ok, (prec, ratio)
        for k in ("mamba_fwd", "mamba_bwd"):
            ok, ratio = rel_close(a[k], b[k], rel=rel * 10, floor=1e-7)
            assert ok, (prec, k, ratio)


def test_windowed_summaries_match_full_chunks():
    """Chunk summaries built backwards in blocks of 64/128 steps, stopping once the 2x2 part is below 2^-100, give
    the sequential result to rounding -- for strongly contracting weights (the first block suffices), for poles that
    need several blocks (the reference's initialisation A = -1..-16 with a large dt: |A_bar| close to 1 again), and
    for weights that barely contract (the walk reaches the chunk start: the exact summary, re-associated)."""
    n = 1500
    W = weights_np()
    st = random_state_np(n, 11)
    g, s = _grad(n, 12), np.abs(_grad(n, 13))
    sc = default_scalars()
    Winit = [w.copy() for w in W]
    for base in (2, 11):
        Winit[base + 5][:] = np.log(np.arange(1, 17, dtype=np.float32))[None, :]     # A_log = log(1..16)
        Winit[base + 2][:] = 1.5                                                       # dt about softplus(1.5) = 1.7
    Wslow = [w.copy() for w in W]
    for base in (2, 11):
        Wslow[base + 5][:] = -12.0            # A = -6e-6, A_bar ~ 1 - 4e-6: no contraction within a chunk
    for Wx in (W, Winit, Wslow):
        for prec, rel in ((64, 1e-9), (32, 2e-5)):
            seq, dseq = _run_oracle(Wx, st, g, s, sc, prec, 0)
            for win in (64, 128):
                a, da = _run_oracle(Wx, st, g, s, sc, prec, 256, window=win)
                ok, ratio = rel_close(dseq["ctx"], da["ctx"], rel=rel, floor=1e-7 if prec == 32 else 1e-12)
                assert ok, (prec, win, ratio)
                for k in ("mamba_fwd", "mamba_bwd"):
                    # entries of a barely contracting state are sums of 1500 inputs with cancellation: the floor
                    # follows the size of the state (fp32 sequential is itself 1e-4 of it away from float64)
                    ok, ratio = rel_close(seq[k], a[k], rel=rel * 10, floor=max(1e-7, 1e-5 * float(np.abs(seq[k]).max())))
                    assert ok, (prec, win, k, ratio)
    # a window as long as the chunk, or none, is plain chunking bit for bit
    plain, dplain = _run_oracle(Wslow, st, g, s, sc, 32, 256)
    win, dwin = _run_oracle(Wslow, st, g, s, sc, 32, 256, window=256)
    assert np.array_equal(dplain["ctx"], dwin["ctx"]) and np.array_equal(plain["mamba_fwd"], win["mamba_fwd"])


def test_contracted_summary_forgets_a_finite_state_and_keeps_a_non_finite_one():
    """A chunk summary whose 2x2 part has contracted to exactly zero hands on its offset b itself: every chunk after
    the first is then independent of the (finite, however large) state the tensor carried in, bit for bit.  A carried
    state that is not finite is multiplied through instead (0 * inf = NaN) and keeps every later context of that
    direction non-finite, as the reference's chunked scan does: a diverged run stays visible."""
    n, chunk = 1500, 256
    W = weights_np()
    g, s = _grad(n, 21), np.abs(_grad(n, 22))
    sc = default_scalars()
    st_a = random_state_np(n, 23)
    st_b = copy_state(st_a)
    st_b["mamba_fwd"][:] = 3.0e30
    st_b["mamba_bwd"][:] = -3.0e30
    a, da = _run_oracle(W, st_a, g, s, sc, 32, chunk, window=64)
    b, db = _run_oracle(W, st_b, g, s, sc, 32, chunk, window=64)
    perm = da["perm"]
    assert np.array_equal(perm, db["perm"])
    later_fwd, later_bwd = perm[chunk:], perm[:n - chunk]          # scan steps >= chunk of either direction
    assert np.isfinite(db["ctx"][0][later_fwd]).all() and np.isfinite(db["ctx"][1][later_bwd]).all()
    assert np.array_equal(da["ctx"][0][later_fwd], db["ctx"][0][later_fwd])
    assert np.array_equal(da["ctx"][1][later_bwd], db["ctx"][1][later_bwd])
    assert not np.array_equal(da["ctx"][0][perm[:chunk]], db["ctx"][0][perm[:chunk]])       # the first chunk does see the carried state
    assert not np.array_equal(da["ctx"][1][perm[n - chunk:]], db["ctx"][1][perm[n - chunk:]])
    for k in ("mamba_fwd", "mamba_bwd"):                            # the new carried state comes from the last chunk
        assert np.array_equal(a[k], b[k]) and np.isfinite(b[k]).all()
    # a carried state that is not finite: every context of that direction is non-finite, and so is the new state;
    # the other direction is untouched
    st_c = copy_state(st_a)
    st_c["mamba_fwd"][:] = np.inf
    c, dc = _run_oracle(W, st_c, g, s, sc, 32, chunk, window=64)
    assert not np.isfinite(dc["ctx"][0]).any(axis=-1).all() or not np.isfinite(dc["ctx"][0]).all()
    assert (~np.isfinite(dc["ctx"][0]).all(axis=-1)).all()          # every element's forward context holds a non-finite entry
    assert not np.isfinite(c["mamba_fwd"]).all()
    assert np.array_equal(dc["ctx"][1], da["ctx"][1]) and np.array_equal(c["mamba_bwd"], a["mamba_bwd"])
    # float64 policy, sequential recurrence: the same statement from the plain formulas
    d, dd = _run_oracle(W, st_c, g, s, sc, 64, 0)
    assert (~np.isfinite(dd["ctx"][0]).all(axis=-1)).all()


# ------------------------------------------------- structural identities of the scan
def test_reverse_scan_is_forward_scan_of_flipped_sequence():
    """With identical weights for both directions, the backward context of the
    sorted sequence equals the forward context of the magnitude-reversed one."""
    n = 200
    W = weights_np()
    for k in range(9):
        W[11 + k] = W[2 + k].copy()
    mag = np.sort(np.abs(_grad(n, 3))) + 1e-6
    mag = np.unique(mag)
    n = mag.size
    g_up = mag.astype(np.float32)                       # already ascending: perm = identity
    st = fresh_state_np(np.zeros(n, np.float32))
    _, d_up = _run_oracle(W, st, g_up, np.zeros(n, np.float32), default_scalars(), 64)
    assert np.array_equal(d_up["perm"], np.arange(n))
    # forward scan over the reversed *sequence* needs the projected inputs reversed;
    # feed it through ref_fp64.scan_block directly
    t = lambda a: torch.from_numpy(np.asarray(a)).double()
    x = torch.stack([t(g_up), torch.zeros(n).double()], -1) @ t(W[0]).T + t(W[1])
    fo, _ = ref_fp64.scan_block(x.flip(0), [t(w) for w in W[2:11]], torch.zeros(16, 16))
    ok, ratio = rel_close(d_up["ctx"][1], fo.flip(0).numpy(), rel=1e-6, floor=1e-10)
    assert ok, ratio


def test_state_carry_two_halves_equal_one_call():
    n = 128
    W = weights_np()
    mag = (np.arange(1, n + 1) * 1e-5).astype(np.float32)     # strictly ascending
    s0 = np.zeros(n, np.float32)
    st = fresh_state_np(np.zeros(n, np.float32))
    full, dfull = _run_oracle(W, st, mag, s0, default_scalars(), 64)
    h = n // 2
    st1 = fresh_state_np(np.zeros(h, np.float32))
    a, da = _run_oracle(W, st1, mag[:h], s0[:h], default_scalars(), 64)
    st2 = fresh_state_np(np.zeros(h, np.float32))
    st2["mamba_fwd"] = a["mamba_fwd"].copy()
    b, db = _run_oracle(W, st2, mag[h:], s0[h:], default_scalars(), 64)
    ok, ratio = rel_close(dfull["ctx"][0][:h], da["ctx"][0], rel=1e-6, floor=1e-10)
    assert ok, ratio
    ok, ratio = rel_close(dfull["ctx"][0][h:], db["ctx"][0], rel=1e-5, floor=1e-9)   # carry went through fp32
    assert ok, ratio
    ok, ratio = rel_close(full["mamba_fwd"], b["mamba_fwd"], rel=1e-5, floor=1e-9)
    assert ok, ratio


def test_closed_form_constant_dt_no_rotation():
    """rope=0, dt_W=0 => dt=softplus(dt_b) constant, A_bar constant per state:
    h_t = A_bar h_{t-1} + dt*B_t*xb_t is a geometric sum; with B, C projections
    it must equal the explicit cumulative formula evaluated in numpy."""
    n = 50
    W = weights_np()
    for base in (2, 11):
        W[base + 1][:] = 0.0          # dt_W
        W[base + 7][:] = 0.0          # rope
    g = np.sort(np.abs(_grad(n, 4)) + 1e-6).astype(np.float32)
    st = fresh_state_np(np.zeros(n, np.float32))
    new, dbg = _run_oracle(W, st, g, np.zeros(n, np.float32), default_scalars(), 64)
    Wd = [w.astype(np.float64) for w in W]
    x = np.stack([g.astype(np.float64), np.zeros(n)], -1) @ Wd[0].T + Wd[1]
    in_proj, dt_b, Bp, Cp, A_log, D, out_proj = Wd[2], Wd[4], Wd[5], Wd[6], Wd[7], Wd[8], Wd[10]
    xb, z = (x @ in_proj.T)[:, :16], (x @ in_proj.T)[:, 16:]
    dt = np.log1p(np.exp(dt_b))                                    # [16]
    A = -np.exp(A_log)                                             # [16,16]
    Abar = (1 + dt[:, None] * A / 2) / (1 - dt[:, None] * A / 2 + 1e-8)
    B, Cm = xb @ Bp.T, xb @ Cp.T                                   # [n,16]
    u = dt[None, :, None] * B[:, None, :] * xb[:, :, None]         # [n,16(j),16(s)]
    t_idx = np.arange(n)
    # h_t = sum_{k<=t} Abar^(t-k) u_k
    pw = Abar[None, None] ** (t_idx[:, None, None, None] - t_idx[None, :, None, None]).clip(0)
    mask = (t_idx[:, None] >= t_idx[None, :])[:, :, None, None]
    h = (pw * mask * u[None]).sum(1)                               # [n,16,16]
    y = (h * Cm[:, None, :]).sum(-1) * (z / (1 + np.exp(-z))) + D * xb
    ctx = y @ out_proj.T
    ok, ratio = rel_close(dbg["ctx"][0], ctx, rel=1e-6, floor=1e-10)
    assert ok, ratio
    ok, ratio = rel_close(new["mamba_fwd"], h[-1], rel=1e-6, floor=1e-10)
    assert ok, ratio


def test_pure_rotation_preserves_pair_norm():
    """A_log -> -inf makes A_bar = 1: with B=0 the state of every RoPE pair
    only rotates, so its Euclidean norm is invariant."""
    n = 40
    W = weights_np()
    for base in (2, 11):
        W[base + 5][:] = -80.0        # A_log
        W[base + 3][:] = 0.0          # B_proj
    st = random_state_np(n, 1)
    new, _ = _run_oracle(W, st, _grad(n, 2), np.zeros(n, np.float32), default_scalars(), 64)
    for k in ("mamba_fwd", "mamba_bwd"):
        n0 = np.hypot(st[k][:, 0::2], st[k][:, 1::2])
        n1 = np.hypot(new[k][:, 0::2], new[k][:, 1::2])
        assert np.allclose(n0, n1, rtol=1e-5, atol=1e-9)


# ------------------------------------------------- update rule
@pytest.mark.parametrize("prec", [32, 64])
def test_reduces_to_adamw_when_metanet_is_off(prec):
    """rescale=0 and lamb_eff=0 leave smart_grad = g: the step must equal
    torch.optim.AdamW(lr, (beta1_i, beta2), eps, wd_eff) on that tensor."""
    n = 300
    W = weights_np()
    p0 = (np.random.RandomState(0).randn(n) * 0.02).astype(np.float32)
    st = fresh_state_np(p0)
    tp = torch.nn.Parameter(torch.from_numpy(p0.copy()).double())
    beta1 = float(np.float32(0.9 * 0.9 ** 3))
    opt = torch.optim.AdamW([tp], lr=float(np.float32(1e-3)), betas=(beta1, float(np.float32(0.999))),
                            eps=float(np.float32(1e-8)), weight_decay=2.5)
    for step in range(1, 4):
        g = _grad(n, 50 + step)
        sc = default_scalars(i=3, step=step, lamb_eff=0.0, wd_eff=2.5, rescale=0.0)
        # bias corrections from the fp32-rounded betas, as AdamW sees them
        sc["bc1"] = 1.0 - beta1 ** step
        sc["bc2"] = 1.0 - float(np.float32(0.999)) ** step
        orc.sg2_step(W, st, g, np.zeros(n, np.float32), f32_scalars(sc), precision=prec)
        tp.grad = torch.from_numpy(g).double()
        opt.step()
        ok, ratio = rel_close(st["param"], tp.detach().numpy(), rel=3e-6, floor=1e-9)
        assert ok, (step, ratio)
        ok, ratio = rel_close(st["exp_avg"], opt.state[tp]["exp_avg"].numpy(), rel=1e-6, floor=1e-10)
        assert ok, (step, ratio)
        ok, ratio = rel_close(st["exp_avg_sq"], opt.state[tp]["exp_avg_sq"].numpy(), rel=1e-6, floor=1e-14)
        assert ok, (step, ratio)


def test_expert_counts_and_index_range():
    n = 500
    W = weights_np()
    counts = np.zeros(144, np.int32)
    st = random_state_np(n, 3)
    _, dbg = _run_oracle(W, st, _grad(n, 4), np.abs(_grad(n, 5)), default_scalars(), 32, counts=counts)
    assert counts.sum() == 4 * n
    assert dbg["expert_idx"].min() >= 0 and dbg["expert_idx"].max() < 144
    assert np.array_equal(np.bincount(dbg["expert_idx"].ravel(), minlength=144), counts)


def test_nonfinite_grads_are_zeroed_and_half_dtypes():
    n = 64
    W = weights_np()
    g = _grad(n, 6)
    g[3], g[9], g[11] = np.nan, np.inf, -np.inf
    gz = g.copy()
    gz[[3, 9, 11]] = 0.0
    st = random_state_np(n, 8)
    a, da = _run_oracle(W, st, g, np.zeros(n, np.float32), default_scalars(), 32)
    b, db = _run_oracle(W, st, gz, np.zeros(n, np.float32), default_scalars(), 32)
    for k in a:
        assert np.array_equal(a[k], b[k]), k
    # bf16 parameters with fp32 state: grads are read through bf16, params rounded back
    st16 = copy_state(st)
    pb = torch.from_numpy(st["param"]).to(torch.bfloat16)
    gb = torch.from_numpy(gz).to(torch.bfloat16)
    st16["param"] = pb.view(torch.int16).numpy().view(np.uint16).copy()
    st16["dtype"] = "bfloat16"
    orc.sg2_step(W, st16, gb.view(torch.int16).numpy().view(np.uint16),
                 np.zeros(n, np.uint16), f32_scalars(default_scalars()), precision=32)
    st32 = copy_state(st)
    st32["param"] = pb.float().numpy().copy()
    orc.sg2_step(W, st32, gb.float().numpy(), np.zeros(n, np.float32), f32_scalars(default_scalars()),
                 precision=32)
    back = torch.from_numpy(st32["param"]).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)
    assert np.array_equal(st16["param"], back)
    assert np.array_equal(st16["exp_avg"], st32["exp_avg"])
