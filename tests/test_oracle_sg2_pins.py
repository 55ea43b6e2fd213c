"""Closed-form and by-construction pins of the per-element functions of the SuperGrok v2 checker (GRU, PEER
routing, expert MLP, rotation sense, soft top-4 routing of the bilevel pass), run against all three CPU statements
used as checkers: oracle/sg2_oracle.cpp in fp32 and in fp64, and tests/ref_fp64.py.

The second half compiles deliberately broken variants of oracle/sg2_oracle.cpp (one textual change each: a gate
convention, an input order, a tie rule, a sign) and requires the matching pin to FAIL on it, so the pins are known
to be sensitive to the mistakes they are meant to exclude."""
import os
import subprocess

import numpy as np
import pytest
import torch

import ref_fp64
import sg2_pins as pins
import workloads as wl
from helpers import copy_state
from oracle import oracle as orc

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def oracle_backend(precision):
    def run(W, st, g, s, sc, dims):
        st = copy_state(st)
        dbg = orc.sg2_step(W, st, g, s, sc, dims=dims, precision=precision, debug=True)
        return st, dbg
    return run


def torch_backend(W, st, g, s, sc, dims):
    t = lambda a: torch.from_numpy(np.ascontiguousarray(a))
    ref = ref_fp64.step([t(w) for w in W], t(st["param"]), t(g), t(s), t(st["exp_avg"]), t(st["exp_avg_sq"]),
                        t(st["mu"]), t(st["gru"]), t(st["mamba_fwd"]), t(st["mamba_bwd"]), sc, dims)
    new = {k: ref[k].numpy() for k in ("param", "exp_avg", "exp_avg_sq", "mu", "gru", "mamba_fwd", "mamba_bwd")}
    dbg = dict(ctx=np.stack([ref["ctx_f"].numpy(), ref["ctx_b"].numpy()]), expert_idx=ref["expert_idx"].numpy(),
               smart=ref["smart"].numpy())
    return new, dbg


BACKENDS = [("oracle_f32", oracle_backend(32), 2e-5), ("oracle_f64", oracle_backend(64), 2e-5),
            ("torch_f64", torch_backend, 1e-12)]
IDS = [b[0] for b in BACKENDS]


@pytest.mark.parametrize("name,run,rel", BACKENDS, ids=IDS)
def test_gru_update_gate_closed_keeps_state(name, run, rel):
    pins.check_gru_update_gate_closed_keeps_state(run)


@pytest.mark.parametrize("name,run,rel", BACKENDS, ids=IDS)
def test_gru_candidate_with_reset_closed(name, run, rel):
    pins.check_gru_candidate_with_reset_closed(run, max(rel, 2e-7))        # contexts are handed over as fp32


@pytest.mark.parametrize("name,run,rel", BACKENDS, ids=IDS)
def test_gru_gate_input_columns(name, run, rel):
    pins.check_gru_gate_input_columns(run, max(rel, 2e-7))


@pytest.mark.parametrize("name,run,rel", BACKENDS, ids=IDS)
def test_peer_routing_by_construction(name, run, rel):
    pins.check_peer_routing_by_construction(run)


@pytest.mark.parametrize("name,run,rel", BACKENDS, ids=IDS)
def test_expert_mlp_by_hand(name, run, rel):
    pins.check_expert_mlp_by_hand(run, max(rel, 2e-7))


@pytest.mark.parametrize("name,run,rel", BACKENDS, ids=IDS)
def test_expert_index_clamp(name, run, rel):
    pins.check_expert_index_clamp(run, max(rel, 2e-7))


@pytest.mark.parametrize("name,run,rel", BACKENDS, ids=IDS)
def test_rotation_sense(name, run, rel):
    pins.check_rotation_sense(run, max(rel, 2e-7) * 20)      # 37 steps of fp32 state in the fp32 policy


# ------------------------------------------------------------------------------- soft top-4 routing (bilevel pass)
def test_soft_top4_routing_closed_form():
    """Two sub-keys per half carry the whole softmax: scores (1, 0.5) x s and (0.2, -0.3) x s against -100 s for
    the other ten, so softmax(10 v) over the four best is (sigmoid(5 s), 1 - sigmoid(5 s)) x (sigmoid(5 s), ...)
    up to exp(-1000 s); the smart gradient is then a 2 x 2 mixture of four known experts per head."""
    dims, W, st, g, s, sc = pins.base_case()
    s = (s + 0.3).astype(np.float32)          # s >= 0.3: the ten dead keys sit at least 300 below in the softmax argument
    H, dm, gh, pk = dims["num_heads"], dims["d_model"], dims["gru_hidden"], dims["pk_dim"]
    scol = gh + 2 * dm + 1
    r = np.random.RandomState(9)
    ka, kb = (1.0, 0.5), (float(np.float32(0.2)), float(np.float32(-0.3)))      # as stored in fp32
    rows_a = [(hh, hh + 5) for hh in range(H)]          # which sub-keys carry the two live scores, per head
    rows_b = [(11 - hh, hh + 1) for hh in range(H)]
    for hh in range(H):
        W[pins.PEER_Q][hh, 0, scol] = 1.0
        W[pins.PEER_Q][hh, dm // 2, scol] = 1.0
        W[pins.KEYS_A][hh][:, 0] = -100.0
        W[pins.KEYS_B][hh][:, 0] = -100.0
        for k in range(2):
            W[pins.KEYS_A][hh][rows_a[hh][k], 0] = ka[k]
            W[pins.KEYS_B][hh][rows_b[hh][k], 0] = kb[k]
    for k in (pins.EXP_W1, pins.EXP_B1, pins.EXP_W2, pins.EXP_B2):
        W[k][...] = r.randn(*W[k].shape).astype(np.float32)
    t = lambda a: torch.from_numpy(np.ascontiguousarray(a)).double()
    rescale = 0.37
    smart, hn, nf, nb = ref_fp64.forward_for_bilevel([t(w) for w in W], t(g), t(s), t(st["gru"]), t(st["mamba_fwd"]),
                                                     t(st["mamba_bwd"]), rescale, dims)
    want = np.zeros(g.size)
    for i, (gv, sv) in enumerate(zip(g.astype(np.float64), s.astype(np.float64))):
        pa = np.exp(10 * ka[0] * sv) / (np.exp(10 * ka[0] * sv) + np.exp(10 * ka[1] * sv))
        pb = np.exp(10 * kb[0] * sv) / (np.exp(10 * kb[0] * sv) + np.exp(10 * kb[1] * sv))
        tot = 0.0
        for hh in range(H):
            for ia, wa in zip(rows_a[hh], (pa, 1 - pa)):
                for ib, wb in zip(rows_b[hh], (pb, 1 - pb)):
                    tot += wa * wb * pins._expert_out(W, ia * pk + ib, gv)[0]
        want[i] = gv + rescale * tot / H
    assert np.abs(smart.numpy() - want).max() <= 1e-12 * np.abs(want).max()
    # the hard-routing step on the same weights picks the single best pair of the same scores
    _, dbg = torch_backend(W, st, g, s, sc, dims)
    assert np.array_equal(dbg["expert_idx"], np.array([[rows_a[hh][0] * pk + rows_b[hh][0] for hh in range(H)]] * g.size))


# ------------------------------------------------------------------------------- the pins notice injected mistakes
MUTANTS = [
    # (name, text in sg2_oracle.cpp, replacement, the pin that has to fail)
    ("gru_gates_exchanged", "hnew[j] = O::fma(zg[j], cand[j], ((R)1 - zg[j]) * hold[j]);",
     "hnew[j] = O::fma((R)1 - zg[j], cand[j], zg[j] * hold[j]);", lambda run: pins.check_gru_update_gate_closed_keeps_state(run)),
    ("gru_reset_ignored", "v = O::fma((R)wh[2 + 2 * dm + k], rg[k] * hold[k], v);",
     "v = O::fma((R)wh[2 + 2 * dm + k], hold[k], v);", lambda run: pins.check_gru_candidate_with_reset_closed(run, 2e-5)),
    ("gru_ctx_order", "vz = O::fma((R)wz[2 + k], f[k], vz); vr = O::fma((R)wr[2 + k], f[k], vr);",
     "vz = O::fma((R)wz[2 + k], b[k], vz); vr = O::fma((R)wr[2 + k], b[k], vr);",
     lambda run: pins.check_gru_gate_input_columns(run, 2e-5)),
    ("peer_g_s_exchanged", "v = O::fma((R)qr[gh + 2 * dm], gv, v);\n                v = O::fma((R)qr[gh + 2 * dm + 1], sv, v);",
     "v = O::fma((R)qr[gh + 2 * dm], sv, v);\n                v = O::fma((R)qr[gh + 2 * dm + 1], gv, v);",
     lambda run: pins.check_peer_routing_by_construction(run)),
    ("peer_input_order", "for (int k = 0; k < dm; k++) v = O::fma((R)qr[gh + k], f[k], v);\n                for (int k = 0; k < dm; k++) v = O::fma((R)qr[gh + dm + k], b[k], v);",
     "for (int k = 0; k < dm; k++) v = O::fma((R)qr[gh + k], b[k], v);\n                for (int k = 0; k < dm; k++) v = O::fma((R)qr[gh + dm + k], f[k], v);",
     lambda run: pins.check_peer_routing_by_construction(run)),
    ("argmax_last_wins", "if (dot > bs) { second = bs; bs = dot; bi = k; }", "if (dot >= bs) { second = bs; bs = dot; bi = k; }",
     lambda run: pins.check_peer_routing_by_construction(run)),
    ("expert_index_transposed", "int e = best[0] * pk + best[1];", "int e = best[1] * pk + best[0];",
     lambda run: pins.check_peer_routing_by_construction(run)),
    ("clamp_wraps", "if (e >= E) e = E - 1;", "if (e >= E) e = e % E;", lambda run: pins.check_expert_index_clamp(run, 2e-5)),
    ("relu_dropped", "zv = zv > 0 ? zv : (R)0;", "zv = zv;", lambda run: pins.check_expert_mlp_by_hand(run, 2e-5)),
    ("expert_bias_dropped", "R ho = W[W_EXP_B2][e];", "R ho = 0;", lambda run: pins.check_expert_mlp_by_hand(run, 2e-5)),
    # (both forms of the replay's update: the products of the polynomial blocks and the plain rotation)
    ("rotation_reversed",
     "ne = O::fma(ae, he, O::fma(sn, ho, be));\n                            no = O::fma(ao, ho, O::fma(cs, he, bo));\n"
     "                        } else {\n                            const R re = O::fma(he, cs, -(ho * sn));\n"
     "                            const R ro = O::fma(ho, cs, he * sn);",
     "ne = O::fma(ae, he, O::fma(-sn, ho, be));\n                            no = O::fma(ao, ho, O::fma(-cs, he, bo));\n"
     "                        } else {\n                            const R re = O::fma(he, cs, ho * sn);\n"
     "                            const R ro = O::fma(ho, cs, -(he * sn));",
     lambda run: pins.check_rotation_sense(run, 4e-4)),
]


@pytest.fixture(scope="module")
def mutant_dir(tmp_path_factory):
    return tmp_path_factory.mktemp("oracle_mutants")


@pytest.mark.parametrize("name,old,new,pin", MUTANTS, ids=[m[0] for m in MUTANTS])
def test_pins_fail_on_injected_mistake(name, old, new, pin, mutant_dir):
    src = open(os.path.join(ROOT, "oracle", "sg2_oracle.cpp")).read()
    assert src.count(old) == 1, "the text to mutate must occur exactly once: " + name
    path = os.path.join(str(mutant_dir), name + ".cpp")
    with open(path, "w") as f:
        f.write(src.replace(old, new).replace('"../include/', '"%s/include/' % ROOT))
    so = os.path.join(str(mutant_dir), name + ".so")
    subprocess.check_call(["g++", "-O1", "-std=c++17", "-fPIC", "-ffp-contract=off", "-mfma", "-shared", "-o", so, path,
                           os.path.join(ROOT, "oracle", "elem_oracle.cpp")])
    good = orc.lib()
    try:
        orc._lib = orc.load(so)
        for precision in (32, 64):
            with pytest.raises(AssertionError):
                pin(oracle_backend(precision))
    finally:
        orc._lib = good
    pin(oracle_backend(32))        # and the unmodified checker passes the same pin
