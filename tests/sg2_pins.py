"""Special cases of the SuperGrok v2 per-element part and of the RoPE rotation in which the mathematics fixes
the answer, written as checks over any implementation of the step ("backend").

They pin what a second restatement by the same author cannot: the GRU gate convention
(grokking_optimizers/mamba3_peer_metanet.py:186-192 of the reference: h' = (1-z) h + z h~, reset applied to h
before W_h), the column order of the GRU and PEER inputs (:320-331 there; csrc/supergrok2_mamba_peer_kernels.cu:
947-1012), the sub-key argmax with "first maximum wins" (:1030-1048 there), expert index a*pk+b with the clamp of
:1050-1051, the expert MLP of :1055-1063 and the rotation sense of :237-246.  Expected values are computed here
with explicit numpy expressions from the backend's own scan contexts (which the closed forms of
test_oracle_sg2.py pin), never with the backend's per-element code.

A backend is a callable  run(W, state, g, s, scalars, dims) -> (new_state, dbg)  with W the 33 float32 arrays
in `_ops` argument order, state a dict of numpy arrays (not modified), and dbg holding 'ctx' [2,N,d_model],
'expert_idx' [N,H] and 'smart' [N].
"""
import numpy as np

import workloads as wl
from helpers import default_scalars, f32_scalars, random_state_np

GRU_WZ, GRU_BZ, GRU_WR, GRU_BR, GRU_WH, GRU_BH, PEER_Q, KEYS_A, KEYS_B, EXP_W1, EXP_B1, EXP_W2, EXP_B2 = range(20, 33)
F_DTW, F_DTB, F_B, F_ALOG, F_ROPE = 3, 4, 5, 7, 9
B_DTW, B_DTB, B_B, B_ALOG, B_ROPE = 12, 13, 14, 16, 18


def base_case(n=48, seed=3, dims=None):
    """Random scan weights (so that the contexts are non-trivial and distinct), zero per-element weights, a state
    with non-zero GRU memory and Mamba carries, gradients and sharpness of order one."""
    dims = dict(wl.DEFAULT_DIMS if dims is None else dims)
    W = [w.numpy().copy() for w in wl.meta_weights(seed, dims, std=0.3)]
    for k in range(GRU_WZ, EXP_B2 + 1):
        W[k][...] = 0.0
    r = np.random.RandomState(seed)
    st = random_state_np(n, seed, dims)
    g = (r.randn(n) * 0.5).astype(np.float32)
    g[:2] = (0.25, -0.25)                      # both signs are always present
    s = (r.rand(n) * 0.3 + 0.01).astype(np.float32)
    sc = f32_scalars(default_scalars(i=1, step=2, lamb_eff=0.0, wd_eff=1.0, rescale=0.5))
    return dims, W, st, g, s, sc


def _close(got, want, rel, what):
    got, want = np.asarray(got, np.float64), np.asarray(want, np.float64)
    err = np.abs(got - want)
    tol = rel * np.maximum(np.abs(want), np.abs(got)) + rel * 1e-3
    assert (err <= tol).all(), "%s: worst error/tolerance %.3g" % (what, float((err / tol).max()))


def gru_inputs(dbg, g, s):
    """[g, s, fwd ctx, bwd ctx] per element, the GRU input of mamba3_peer_metanet.py:320-324."""
    return np.concatenate([g[:, None], s[:, None], dbg["ctx"][0], dbg["ctx"][1]], -1).astype(np.float64)


# ---------------------------------------------------------------------------------------------- GRU
def check_gru_update_gate_closed_keeps_state(run):
    """b_z = -40: z = sigmoid(-40) = 4e-18, so h' = (1-z) h + z h~ is h itself, bit for bit (with the two terms
    exchanged the result would be the candidate h~)."""
    dims, W, st, g, s, sc = base_case()
    r = np.random.RandomState(1)
    W[GRU_BZ][:] = -40.0
    for k in (GRU_WR, GRU_BR, GRU_WH, GRU_BH):
        W[k][...] = r.randn(*W[k].shape).astype(np.float32)
    new, _ = run(W, st, g, s, sc, dims)
    assert np.array_equal(np.asarray(new["gru"], np.float32).reshape(st["gru"].shape), st["gru"])


def check_gru_candidate_with_reset_closed(run, rel):
    """b_z = +40, b_r = -40: z = 1 and r = 0, so h' = tanh(W_h[:, :18] . [g, s, ctxF, ctxB] + b_h): the hidden
    columns of W_h see r*h = 0 (a reset gate applied after W_h, or ignored, would let them through)."""
    dims, W, st, g, s, sc = base_case()
    r = np.random.RandomState(2)
    W[GRU_BZ][:] = 40.0
    W[GRU_BR][:] = -40.0
    W[GRU_WH][...] = r.randn(*W[GRU_WH].shape).astype(np.float32)
    W[GRU_BH][...] = r.randn(*W[GRU_BH].shape).astype(np.float32) * 0.3
    new, dbg = run(W, st, g, s, sc, dims)
    x = gru_inputs(dbg, g, s)
    nx = x.shape[1]
    want = np.tanh(x @ W[GRU_WH].astype(np.float64)[:, :nx].T + W[GRU_BH].astype(np.float64))
    _close(np.asarray(new["gru"]).reshape(want.shape), want, rel, "GRU candidate")


def check_gru_gate_input_columns(run, rel):
    """One column of W_z (then of W_r) at a time: the gate must read input k of [g, s, ctxF(8), ctxB(8), h(4)].
      update gate: W_h = 0, b_h = 0 => h~ = 0 and h'_j = (1 - sigmoid(c x_k)) h_j
      reset gate:  b_z = +40 (z = 1), W_h = identity on the hidden columns => h'_j = tanh(sigmoid(c x_k) h_j)."""
    dims, W0, st, g, s, sc = base_case()
    gh = dims["gru_hidden"]
    _, dbg = run(W0, st, g, s, sc, dims)
    xh = np.concatenate([gru_inputs(dbg, g, s), st["gru"].astype(np.float64)], -1)
    h = st["gru"].astype(np.float64)
    for k in range(xh.shape[1]):
        c = np.float32(2.0 / (np.abs(xh[:, k]).max() + 1e-30))
        gate = 1.0 / (1.0 + np.exp(-np.float64(c) * xh[:, k]))[:, None]
        W = [w.copy() for w in W0]
        W[GRU_WZ][:, k] = c
        new, _ = run(W, st, g, s, sc, dims)
        _close(np.asarray(new["gru"]).reshape(h.shape), (1.0 - gate) * h, rel, "update gate, input column %d" % k)
        W = [w.copy() for w in W0]
        W[GRU_BZ][:] = 40.0
        W[GRU_WR][:, k] = c
        for j in range(gh):
            W[GRU_WH][j, xh.shape[1] - gh + j] = 1.0
        new, _ = run(W, st, g, s, sc, dims)
        _close(np.asarray(new["gru"]).reshape(h.shape), np.tanh(gate * h), rel, "reset gate, input column %d" % k)


# ---------------------------------------------------------------------------------------------- PEER routing
def _signed_unit_keys(dims):
    """12 sub-keys whose scores are exactly +-(one query component) or 0 in any precision:
    e0 e1 e2 e3 -e0 -e1 -e2 -e3, then exact duplicates of e0, e1, -e2 and a zero key."""
    pk, hd = dims["pk_dim"], dims["d_model"] // 2
    K = np.zeros((pk, hd), np.float32)
    for m in range(hd):
        K[m, m] = 1.0
        K[hd + m, m] = -1.0
    K[2 * hd, 0] = 1.0
    K[2 * hd + 1, 1] = 1.0
    K[2 * hd + 2, 2] = -1.0
    return K


def _first_argmax(scores):
    best = np.zeros(scores.shape[0], np.int64)
    for i in range(scores.shape[0]):            # strict '>' from -1e30: the first maximum wins
        b, bs = 0, -1e30
        for m in range(scores.shape[1]):
            if scores[i, m] > bs:
                b, bs = m, scores[i, m]
        best[i] = b
    return best


def check_peer_routing_by_construction(run):
    """Every query row copies ONE entry of [h'(4), ctxF(8), ctxB(8), g, s] (a different selection per head, all 22
    entries used), the sub-keys are signed unit vectors with exact duplicates: the winner follows from comparing the
    copied inputs themselves, ties between duplicate keys must go to the lower index, and a wrong concatenation
    order of the PEER input, a swapped (a, b) or '>=' in the argmax all change it."""
    dims, W, st, g, s, sc = base_case(n=96)
    H, dm, gh, pk = dims["num_heads"], dims["d_model"], dims["gru_hidden"], dims["pk_dim"]
    pin = gh + 2 * dm + 2
    r = np.random.RandomState(5)
    for k in (GRU_WZ, GRU_BZ, GRU_WR, GRU_BR, GRU_WH, GRU_BH):      # a generic GRU: h' differs from h
        W[k][...] = r.randn(*W[k].shape).astype(np.float32) * 0.5
    cols = np.array([(7 * i + 3 * (i // pin)) % pin for i in range(H * dm)]).reshape(H, dm)
    assert set(cols.ravel().tolist()) == set(range(pin))
    for hh in range(H):
        for d in range(dm):
            W[PEER_Q][hh, d, cols[hh, d]] = 1.0
        W[KEYS_A][hh] = _signed_unit_keys(dims)
        W[KEYS_B][hh] = np.roll(_signed_unit_keys(dims), 1, axis=1)       # same construction, components rotated
    new, dbg = run(W, st, g, s, sc, dims)
    hn = np.asarray(new["gru"], np.float64).reshape(-1, gh)
    x = np.concatenate([hn, dbg["ctx"][0], dbg["ctx"][1], g[:, None], s[:, None]], -1).astype(np.float64)
    want = np.zeros((g.size, H), np.int64)
    dup_wins = 0
    for hh in range(H):
        q = x[:, cols[hh]]
        sa = q[:, : dm // 2] @ W[KEYS_A][hh].astype(np.float64).T
        sb = q[:, dm // 2:] @ W[KEYS_B][hh].astype(np.float64).T
        a, b = _first_argmax(sa), _first_argmax(sb)
        dup_wins += int(((a == 0) | (a == 1)).sum())       # keys 0 and 1 have exact duplicates at 8 and 9
        want[:, hh] = a * pk + b
    assert dup_wins > 0, "no element was decided by a duplicated key"
    assert len(np.unique(want)) > 8, "the construction should spread over many experts"
    assert np.array_equal(np.asarray(dbg["expert_idx"], np.int64), want)


# ---------------------------------------------------------------------------------------------- expert MLP
def _route_by_sign_of_g(W, dims, a_pos, a_neg, b_pos=0):
    """Query component 0 (and 4) copies g; sub-key a_pos[h] = +e0, a_neg[h] = -e0: elements with g > 0 go to row
    a_pos of head h, g < 0 to a_neg.  Second half: key b_pos = +e0 (g > 0), everything else scores <= 0 -> b = 0 for
    g < 0 unless b_pos == 0."""
    H, dm, gh = dims["num_heads"], dims["d_model"], dims["gru_hidden"]
    gcol = gh + 2 * dm
    for hh in range(H):
        W[PEER_Q][hh, 0, gcol] = 1.0
        W[KEYS_A][hh][...] = 0.0
        W[KEYS_A][hh][a_pos[hh], 0] = 1.0
        W[KEYS_A][hh][a_neg[hh], 0] = -1.0
        W[KEYS_B][hh][...] = 0.0
        if b_pos:
            W[PEER_Q][hh, dm // 2, gcol] = 1.0
            W[KEYS_B][hh][b_pos, 0] = 1.0


def _expert_out(W, e, gv):
    eh = W[EXP_W1].shape[1]
    out = float(W[EXP_B2][e])
    on = 0
    for u in range(eh):
        pre = float(W[EXP_W1][e, u]) * gv + float(W[EXP_B1][e, u])
        if pre > 0.0:
            out += float(W[EXP_W2][e, u]) * pre
            on += 1
    return out, on


def check_expert_mlp_by_hand(run, rel):
    """Elements are routed by the sign of g to two known experts per head; smart = g + rescale * mean over heads of
    b2[e] + sum_u W2[e,u] relu(W1[e,u] g + b1[e,u]), evaluated unit by unit (both ReLU branches occur)."""
    dims, W, st, g, s, sc = base_case()
    H, pk = dims["num_heads"], dims["pk_dim"]
    r = np.random.RandomState(6)
    a_pos, a_neg = [2 * hh for hh in range(H)], [2 * hh + 1 for hh in range(H)]
    _route_by_sign_of_g(W, dims, a_pos, a_neg)
    for k in (EXP_W1, EXP_B1, EXP_W2, EXP_B2):
        W[k][...] = r.randn(*W[k].shape).astype(np.float32)
    _, dbg = run(W, st, g, s, sc, dims)
    want_e = np.array([[(a_pos[hh] if gv > 0 else a_neg[hh]) * pk for hh in range(H)] for gv in g])
    assert np.array_equal(np.asarray(dbg["expert_idx"], np.int64), want_e)
    want, on_total, units = np.zeros(g.size), 0, 0
    for i, gv in enumerate(g.astype(np.float64)):
        tot = 0.0
        for hh in range(H):
            o, on = _expert_out(W, int(want_e[i, hh]), gv)
            tot += o
            on_total += on
            units += W[EXP_W1].shape[1]
        want[i] = gv + float(sc["rescale"]) * tot / H
    assert 0 < on_total < units, "both ReLU branches must occur"
    _close(dbg["smart"], want, rel, "smart gradient")


def check_expert_index_clamp(run, rel):
    """pk_dim^2 > num_experts (12 x 12 sub-keys, 100 experts): (a, b) = (11, 11) gives 143, which the kernel clamps
    to the last expert, 99 (csrc/supergrok2_mamba_peer_kernels.cu:1050-1051)."""
    dims = dict(wl.DEFAULT_DIMS, num_experts=100)
    dims_, W, st, g, s, sc = base_case(dims=dims)
    H, pk, E = dims["num_heads"], dims["pk_dim"], dims["num_experts"]
    r = np.random.RandomState(7)
    _route_by_sign_of_g(W, dims, [pk - 1] * H, [0] * H, b_pos=pk - 1)
    for k in (EXP_W1, EXP_B1, EXP_W2, EXP_B2):
        W[k][...] = r.randn(*W[k].shape).astype(np.float32)
    _, dbg = run(W, st, g, s, sc, dims)
    want_e = np.where(g[:, None] > 0, E - 1, 0) * np.ones((1, H), np.int64)
    assert np.array_equal(np.asarray(dbg["expert_idx"], np.int64), want_e)
    want = np.array([gv + float(sc["rescale"]) * _expert_out(W, int(want_e[i, 0]), gv)[0]
                     for i, gv in enumerate(g.astype(np.float64))])
    _close(dbg["smart"], want, rel, "smart gradient through the clamped expert")


# ---------------------------------------------------------------------------------------------- rotation sense
def check_rotation_sense(run, rel):
    """A_log = -80 (A_bar = 1 up to the reference's 1e-8), B = 0, dt constant per column: after N steps every RoPE
    pair is its initial state rotated by +N dt f,  h_e' = h_e cos - h_o sin, h_o' = h_o cos + h_e sin
    (csrc/supergrok2_mamba_peer_kernels.cu:242-246), in both scan directions."""
    dims, W, st, g, s, sc = base_case(n=37)
    r = np.random.RandomState(8)
    for alog, bp, dtw, dtb, rope in ((F_ALOG, F_B, F_DTW, F_DTB, F_ROPE), (B_ALOG, B_B, B_DTW, B_DTB, B_ROPE)):
        W[alog][...] = -80.0
        W[bp][...] = 0.0
        W[dtw][...] = 0.0
        W[dtb][...] = r.randn(*W[dtb].shape).astype(np.float32)
        W[rope][...] = r.randn(*W[rope].shape).astype(np.float32) * 0.2
    new, _ = run(W, st, g, s, sc, dims)
    n = g.size
    for key, alog, dtb, rope in (("mamba_fwd", F_ALOG, F_DTB, F_ROPE), ("mamba_bwd", B_ALOG, B_DTB, B_ROPE)):
        dt = np.log1p(np.exp(W[dtb].astype(np.float64)))[:, None]
        A = -np.exp(W[alog].astype(np.float64))
        abar = (1.0 + dt * A / 2.0) / (1.0 - dt * A / 2.0 + 1e-8)
        th = n * dt * W[rope].astype(np.float64)
        h0 = st[key].astype(np.float64)
        he, ho = h0[:, 0::2], h0[:, 1::2]
        want = np.empty_like(h0)
        want[:, 0::2] = (he * np.cos(th) - ho * np.sin(th)) * abar[:, 0::2] ** n
        want[:, 1::2] = (ho * np.cos(th) + he * np.sin(th)) * abar[:, 1::2] ** n
        assert np.median(np.abs(np.sin(th))) > 0.1          # a reversed rotation would be far off
        _close(np.asarray(new[key]).reshape(h0.shape), want, rel, key + " after a pure rotation")
