"""Pins the CPU checkers of the Grokfast, SuperGrok v1.5 and Muon steps
(oracle/elem_oracle.cpp, oracle/muon_oracle.py) against golden vectors written
by the reference's own CPU code (tests/golden/ref_*.npz, produced by
tests/golden/make_golden_ref.py from a build of the reference's csrc/ops.cpp),
against torch.optim.AdamW and against libm."""
import math
import os

import numpy as np
import pytest
import torch

from helpers import rel_close
from oracle import oracle as orc
from oracle import muon_oracle

GOLD = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
RNG = np.random.RandomState(5)


def test_erfc_and_gelu_against_libm():
    worst_c, worst_g = 0.0, 0.0
    L = orc.lib()
    for x in np.concatenate([RNG.uniform(-6, 6, 20000), [0.0, 1e-4, -1e-4, 9.0, -9.0]]):
        x = float(np.float32(x))
        r = math.erfc(x)
        worst_c = max(worst_c, abs(L.orc_erfc(x) - r) / max(r, 1e-30))
        g = 0.5 * x * (1.0 + math.erf(x / math.sqrt(2.0)))
        worst_g = max(worst_g, abs(L.orc_gelu_erf(x) - g) / max(abs(g), 1e-6))
    # erfc carries the rounding of x*x in its exponent: relative error grows like x^2 * 2^-24
    assert worst_c < 6e-6 and worst_g < 3e-6, (worst_c, worst_g)
    x = torch.linspace(-8, 8, 4001)
    mine = torch.tensor([L.orc_gelu_erf(float(v)) for v in x])
    assert torch.allclose(mine, torch.nn.functional.gelu(x.double()).float(), rtol=1e-6, atol=1e-7)
    sig = torch.tensor([L.orc_gelu_sigmoid(float(v)) for v in x])
    assert torch.allclose(sig, (x.double() * torch.sigmoid(1.702 * x.double())).float(), rtol=1e-6, atol=1e-7)


def test_grokfast_matches_reference_golden():
    z = np.load(os.path.join(GOLD, "ref_grokfast.npz"))
    n, steps = int(z["n"]), int(z["steps"])
    emas = [np.zeros(z[f"g_in_0_{i}"].size, np.float32) for i in range(n)]
    for t in range(steps):
        for i in range(n):
            g = z[f"g_in_{t}_{i}"].reshape(-1).copy()
            orc.grokfast_ema(g, emas[i], float(z["alpha"]), float(z["lamb"]))
            ok, r = rel_close(g, z[f"g_out_{t}_{i}"].reshape(-1), 1e-6, 1e-10)
            assert ok, (t, i, r)
            ok, r = rel_close(emas[i], z[f"ema_{t}_{i}"].reshape(-1), 1e-6, 1e-10)
            assert ok, (t, i, r)


def test_grokfast_closed_form_and_adamw_library():
    """EMA closed form e_t = (1-a) sum a^(t-k) g_k; the AdamW half against torch.optim.AdamW."""
    n, T, a, lam = 200, 6, 0.98, 2.0
    gs = [(RNG.randn(n) * 1e-3).astype(np.float32) for _ in range(T)]
    p0 = (RNG.randn(n) * 0.02).astype(np.float32)
    p, ema, ea, easq = p0.copy(), np.zeros(n, np.float32), np.zeros(n, np.float32), np.zeros(n, np.float32)
    tp = torch.nn.Parameter(torch.from_numpy(p0.copy()).double())
    opt = torch.optim.AdamW([tp], lr=1e-3, betas=(0.9, 0.98), eps=1e-8, weight_decay=1.0)
    for t in range(1, T + 1):
        g = gs[t - 1].copy()
        orc.grokfast_adamw(p, g, ema, ea, easq, t, a, lam, 1e-3, 0.9, 0.98, 1e-8, 1.0)
        closed = (1 - a) * sum(a ** (t - k) * gs[k - 1].astype(np.float64) for k in range(1, t + 1))
        ok, r = rel_close(ema, closed, 1e-5, 1e-10)
        assert ok, (t, r)
        amp = gs[t - 1].astype(np.float64) + lam * closed
        ok, r = rel_close(g, amp, 1e-5, 1e-10)
        assert ok, (t, r)
        tp.grad = torch.from_numpy(g.astype(np.float64))       # AdamW on the amplified gradient the checker produced
        opt.step()
        ok, r = rel_close(p, tp.detach().numpy(), 3e-6, 1e-9)
        assert ok, (t, r)


@pytest.mark.parametrize("gelu_mode", [0])
def test_sg15_matches_reference_golden(gelu_mode):
    """The reference's CPU path (exact GELU, global-norm clip that rescales the gradients in place)."""
    z = np.load(os.path.join(GOLD, "ref_sg15.npz"))
    P, steps = int(z["n"]), int(z["steps"])
    net = (z["W1"], z["b1"], z["W2"], z["b2"], float(z["rescale"]))
    params = [z[f"p_in_{i}"].copy() for i in range(P)]
    eas = [np.zeros_like(p) for p in params]
    easqs = [np.zeros_like(p) for p in params]
    mus = [np.zeros_like(p) for p in params]
    f32 = lambda v: float(np.float32(v))
    lamb_eff = f32(np.float32(z["ramp"]) * np.float32(z["gate"]) * np.float32(z["lamb"]))
    for t in range(steps):
        grads = [z[f"g_in_{t}_{i}"].copy() for i in range(P)]
        sharps = [z[f"s_in_{t}_{i}"].copy() for i in range(P)]
        step = np.float32(t + 1)
        pt = []
        for i in range(P):
            b1 = np.float32(z["beta1s"][i])
            pt.append(dict(alpha=f32(z["alphas"][i]), beta1=f32(b1), bc1=f32(np.float32(1) - np.power(b1, step)),
                           bc2=f32(np.float32(1) - np.power(np.float32(z["beta2"]), step))))
        coef, on = orc.sg15_step(params, grads, sharps, eas, easqs, mus, net, pt, lamb_eff, f32(z["beta2"]), f32(z["lr"]),
                                 f32(z["wd_eff"]), f32(z["eps"]), f32(z["clip"]), gelu_mode)
        assert on == (1 if t == 1 else 0)
        for i in range(P):
            for name, arr in (("p", params[i]), ("ea", eas[i]), ("easq", easqs[i]), ("mu", mus[i]), ("g_out", grads[i])):
                ok, r = rel_close(arr, z[f"{name}_{t}_{i}"], 2e-5, 1e-9)
                assert ok, (t, i, name, r)


def test_muon_restatement_matches_reference_golden():
    z = np.load(os.path.join(GOLD, "ref_muon.npz"))
    P, steps = int(z["n"]), int(z["steps"])
    bf16 = lambda a: torch.from_numpy(a).to(torch.bfloat16).float().numpy()
    for tag in ("f32", "bf16"):
        params = [z[f"{tag}_p_in_{i}"].copy() for i in range(P)]
        bufs = [np.zeros_like(p) for p in params]
        for t in range(steps):
            for i in range(P):
                new_p, X = muon_oracle.muon_step(params[i], z[f"{tag}_g_{t}_{i}"], bufs[i], float(z["momentum"]),
                                                 float(z["lr"]), float(z["wd"]), int(z["ns_steps"]),
                                                 round_mid=bf16 if tag == "bf16" else None,
                                                 round_decay=bf16 if tag == "bf16" else None)
                ok, r = rel_close(bufs[i], z[f"{tag}_buf_{t}_{i}"], 1e-6, 1e-10)
                assert ok, (tag, t, i, r)
                want = z[f"{tag}_p_{t}_{i}"]
                if tag == "bf16":          # CPU branch: bf16 parameter rounded after the add and after the decay
                    new_p = bf16(new_p)
                    nd = int((new_p != want).sum())     # fp32 NS differences may flip a rare rounding
                    assert nd <= max(1, new_p.size // 200), (tag, t, i, nd)
                    assert np.abs(new_p - want).max() <= np.abs(want).max() * 2.0 ** -8
                else:
                    ok, r = rel_close(new_p, want, 2e-5, 1e-8)
                    assert ok, (tag, t, i, r)
                params[i] = new_p


def test_newton_schulz_fixed_point_properties():
    """Five quintic iterations pull every singular value of X/||X||_F into roughly [0.7, 1.2];
    the tall case equals the transpose of the wide case."""
    X = RNG.randn(32, 96)
    Y = muon_oracle.newton_schulz(X / np.linalg.norm(X), 5, np.float64)
    s = np.linalg.svd(Y, compute_uv=False)
    assert s.min() > 0.6 and s.max() < 1.25
    Yt = muon_oracle.newton_schulz(X.T / np.linalg.norm(X), 5, np.float64)
    assert np.allclose(Yt.T, Y, rtol=1e-9, atol=1e-12)
    Y32 = muon_oracle.newton_schulz(X / np.linalg.norm(X), 5, np.float32)
    assert np.linalg.norm(Y32 - Y) / np.linalg.norm(Y) < 1e-5


def test_sam_helpers_golden_are_the_plain_formulas():
    z = np.load(os.path.join(GOLD, "ref_sg15.npz"))
    P = int(z["n"])
    norm = np.float32(np.sqrt(sum(float(np.sum(z[f"sam_g_{i}"].astype(np.float64) ** 2)) for i in range(P)))) + np.float32(1e-12)
    r = np.float32(0.05) / norm
    for i in range(P):
        ok, ratio = rel_close(z[f"sam_p_in_{i}"] + r * z[f"sam_g_{i}"], z[f"sam_p_out_{i}"], 1e-6, 1e-9)
        assert ok, ratio
        assert np.array_equal(z[f"sam_backup_{i}"], z[f"sam_p_in_{i}"])
        assert np.array_equal(z[f"restored_{i}"], z[f"sam_p_in_{i}"])
        # The reference's CPU branch rebinds its local copy of the list entry
        # (csrc/ops.cpp:201), so the caller's sharpness tensor is never written there;
        # only its GPU kernel stores |g_sam - g| in place (csrc/supergrok15_kernels.cu:182).
        assert not z[f"sharp_out_{i}"].any()


def test_aten_loop_matches_checker():
    """oracle/aten_loop.py (the per-timestep ATen restatement bench.py times as the CPU baseline) against the float64
    policy of the C++ checker on one small tensor: same routing, states within fp32 rounding of a 300-step recurrence."""
    import torch
    import workloads as wl
    from helpers import default_scalars, f32_scalars, random_state_np, weights_np
    from oracle import aten_loop
    from oracle import oracle as orc
    n = 300
    W = weights_np()
    st = random_state_np(n, 4)
    r = np.random.RandomState(5)
    g, s = (r.randn(n) * 1e-2).astype(np.float32), np.abs(r.randn(n) * 1e-2).astype(np.float32)
    sc = f32_scalars(default_scalars(i=1, step=3, lamb_eff=2.0, wd_eff=4.5))
    ts = {k: torch.from_numpy(v.copy()) for k, v in st.items()}
    eidx = aten_loop.step([torch.from_numpy(w) for w in W], ts, torch.from_numpy(g), torch.from_numpy(s), sc, wl.DEFAULT_DIMS)
    dbg = orc.sg2_step(W, st, g, s, sc, precision=64, chunk_len=0, debug=True)
    assert np.array_equal(eidx.numpy().astype(np.int32), dbg["expert_idx"])
    for k in ("param", "exp_avg", "exp_avg_sq", "mu", "gru", "mamba_fwd", "mamba_bwd"):
        a, b = ts[k].numpy().reshape(st[k].shape).astype(np.float64), st[k].astype(np.float64)
        assert np.all(np.abs(a - b) <= 2e-5 * np.maximum(np.abs(a), np.abs(b)) + 1e-7), k
