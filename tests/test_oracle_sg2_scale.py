"""The fp32 policy of the CPU checker in the configuration the benchmark runs -- chunks of 4096 steps, summary
window of 64, every polynomial shortcut of the kernels active -- against the float64 policy evaluated as the plain
sequential recurrence (csrc/supergrok2_mamba_peer_kernels.cu:138-272 of the reference), on tensors shaped like
those of the 25 M element set: a million elements, N(0, 1e-3) gradients with a Student-t (nu = 3) tail on 0.5 % of
the entries, the per-tensor clip applied, a mid-training state carried in.

The gates of the GPU tests compare the kernels with the fp32 policy; this file is the independent leg: what the
chunking, the windowed and weight-sized summaries, the Taylor / lane-polynomial / product forms and the fp32
arithmetic together cost against the mathematics.  Every float state must agree within 1e-4, every PEER routing
difference must sit at a near-tie of the float64 scores (margin < 1e-5), and the rate of such flips is printed,
for this tensor and for the 14-tensor set of the small configuration."""
from concurrent.futures import ThreadPoolExecutor

import numpy as np
import torch

import workloads as wl
from helpers import copy_state, default_scalars, f32_scalars, random_state_np, rel_close, weights_np
from oracle import oracle as orc

REL = 1e-4


def _both_policies(W, st, g, s, sc, chunk_len, window):
    """(state, debug) of the fp32 policy as the kernels chunk it, and of the float64 sequential recurrence."""
    def run(prec):
        x = copy_state(st)
        dbg = orc.sg2_step(W, x, g, s, sc, precision=prec, chunk_len=chunk_len if prec == 32 else 0,
                           window=window if prec == 32 else 0, debug=True)
        return x, dbg
    with ThreadPoolExecutor(2) as ex:       # the library releases the GIL: the two policies run side by side
        fa, fb = ex.submit(run, 32), ex.submit(run, 64)
        return fa.result(), fb.result()


def _check(a, da, b, db, label):
    assert np.array_equal(da["perm"], db["perm"])
    mism = da["expert_idx"] != db["expert_idx"]
    flips = int(mism.sum())
    margins = db["margin"].min(-1)
    worst_margin = float(margins[mism].max()) if flips else 0.0
    print("%s: %d of %d routing decisions differ between fp32 and float64 (rate %.3g), largest float64 margin among them %.3g"
          % (label, flips, mism.size, flips / mism.size, worst_margin), flush=True)
    assert (margins[mism] < 1e-5).all()
    assert flips <= 1e-3 * mism.size
    good = ~mism.any(-1)
    worst = {}
    # floors: about 1e-5 of each state's own scale (parameters 2e-2, moments 1e-4 / 1e-9, contexts and GRU of order 0.1)
    for k, floor in (("param", 1e-7), ("exp_avg", 1e-9), ("exp_avg_sq", 1e-14), ("mu", 1e-9)):
        ok, worst[k] = rel_close(a[k][good], b[k][good], rel=REL, floor=floor)
        assert ok, (label, k, worst[k])
    for k in ("gru", "mamba_fwd", "mamba_bwd"):
        ok, worst[k] = rel_close(a[k], b[k], rel=REL, floor=1e-6)
        assert ok, (label, k, worst[k])
    ok, worst["ctx"] = rel_close(da["ctx"], db["ctx"], rel=REL, floor=1e-6)
    assert ok, (label, "ctx", worst["ctx"])
    print("%s: worst tolerance ratios (1.0 = rel 1e-4) %s" % (label, {k: round(v, 4) for k, v in worst.items()}), flush=True)


def test_benchmark_chunking_against_float64_sequential_on_a_million_elements():
    n = 1 << 20
    shapes = [(1024, 1024)]
    grads = wl.clip_per_tensor(wl.make_grads(shapes, seed=5, tail_frac=0.005, tail="student3"))
    g = grads[0].reshape(-1).numpy()
    assert float(np.abs(g).max()) > 5e-3         # the tail is there: the last tiles leave the polynomial forms
    s = np.zeros(n, np.float32)
    W = weights_np()
    st = random_state_np(n, 77)
    sc = f32_scalars(default_scalars(i=3, step=4, lamb_eff=2.0, wd_eff=4.5))
    (a, da), (b, db) = _both_policies(W, st, g, s, sc, 4096, 64)
    _check(a, da, b, db, "1M-element Student-t tensor, chunk 4096, window 64")


def test_flip_rate_on_the_14_tensor_set():
    shapes = wl.shared14_shapes()
    grads = wl.make_grads(shapes, seed=1)
    sharps = [g.abs() * 0.5 for g in wl.make_grads(shapes, seed=501)]
    W = weights_np()
    flips = total = 0
    for i, (gt, stt) in enumerate(zip(grads, sharps)):
        n = gt.numel()
        st = random_state_np(n, 300 + i)
        sc = f32_scalars(default_scalars(i=i, step=2, lamb_eff=2.0))
        (a, da), (b, db) = _both_policies(W, st, gt.reshape(-1).numpy(), stt.reshape(-1).numpy(), sc, 1024, 64)
        mism = da["expert_idx"] != db["expert_idx"]
        assert (db["margin"].min(-1)[mism] < 1e-5).all(), i
        flips += int(mism.sum())
        total += mism.size
        good = ~mism.any(-1)
        for k, floor in (("param", 1e-7), ("exp_avg", 1e-9), ("mu", 1e-9)):
            ok, r = rel_close(a[k][good], b[k][good], rel=REL, floor=floor)
            assert ok, (i, k, r)
        ok, r = rel_close(da["ctx"], db["ctx"], rel=REL, floor=1e-6)
        assert ok, (i, "ctx", r)
    print("14-tensor set (420 195 elements, chunk 1024, window 64, populated sharpness): %d of %d routing decisions differ "
          "between fp32 and float64 (rate %.3g)" % (flips, total, flips / total), flush=True)
    assert flips <= 1e-3 * total


def test_flip_rate_with_routing_spread_over_most_experts():
    """The same comparison where routing decisions are close calls far more often: query rows that read the GRU state
    amplified 30 times on GRU states of unit scale, so that the elements spread over most of the 144 experts and many
    score pairs are near ties.  Every difference between the fp32 and the float64 routing must still sit at a
    float64 margin below 1e-5; the rate is printed."""
    n = 1 << 18
    g = wl.make_grads([(n,)], seed=9, tail_frac=0.005, tail="student3")[0].reshape(-1).numpy()
    s = np.abs(wl.make_grads([(n,)], seed=509)[0].reshape(-1).numpy()) * 0.5
    W = weights_np()
    W[26] = W[26].copy()
    W[26][:, :, :4] *= 30.0
    st = random_state_np(n, 78)
    st["gru"] = (st["gru"] * np.float32(1.0 / 0.3)).astype(np.float32)
    sc = f32_scalars(default_scalars(i=1, step=3, lamb_eff=2.0))
    (a, da), (b, db) = _both_policies(W, st, g, s, sc, 1024, 64)
    used = len(np.unique(db["expert_idx"]))
    print("spread routing: %d experts in use" % used, flush=True)
    assert used >= 100
    _check(a, da, b, db, "262 144 elements, routing spread over %d experts" % used)


def test_module_initialised_weights_around_the_polynomial_limits():
    """The reference's own initial meta-net (A_log = log(1..16): poles down to -16, where the lane polynomials and
    the product forms have their narrowest range of valid inputs), with gradients spread over three decades around
    1e-3 so that the sorted sequence walks through every form the kernels have -- linear products, quadratic
    products, lane polynomials with the plain update, the general recurrence -- and a populated sharpness.  The fp32
    policy as the kernels chunk it against the float64 sequential recurrence: every state within 1e-4, every routing
    difference at a float64 margin below 1e-5."""
    n = 1 << 17
    r = np.random.RandomState(31)
    g = (r.randn(n) * np.exp(r.uniform(np.log(3e-5), np.log(3e-2), size=n))).astype(np.float32)
    s = (np.abs(r.randn(n)) * 3e-4).astype(np.float32)
    W = [w.numpy().copy() for w in wl.module_weights(3)]
    st = random_state_np(n, 79)
    sc = f32_scalars(default_scalars(i=2, step=5, lamb_eff=2.0))
    (a, da), (b, db) = _both_policies(W, st, g, s, sc, 1024, 64)
    _check(a, da, b, db, "131 072 elements, module-initialised weights, gradients 3e-5 .. 3e-2")
