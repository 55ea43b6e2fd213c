"""Replays the golden cases of tests/golden/ref_family.npz through a set of
step functions (the CPU checker or the GPU entry points: same signatures) and
compares every recorded tensor.  Shared by the CPU and GPU family tests."""
import os

import numpy as np

from helpers import rel_close

GOLD = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "ref_family.npz")
P = 4


def _get(z, tag, name, t):
    return [z[f"{tag}_{name}_{t}_{i}"].astype(np.float32).copy() for i in range(P)]


def _check(z, tag, t, rel=1e-4, floor=1e-7, **named):
    for name, tensors in named.items():
        for i, x in enumerate(tensors):
            ok, worst = rel_close(np.asarray(x, dtype=np.float32), z[f"{tag}_{name}_{t}_{i}"], rel, floor)
            assert ok, (tag, name, t, i, worst)


def run_grokadamw(fn):
    z = np.load(GOLD)
    c = {k: float(z[f"gaw_{k}"]) for k in ("alpha", "lamb", "beta1", "beta2", "lr", "wd", "eps", "clip")}
    p = _get(z, "gaw", "p", "in")
    ea, easq, ema = ([np.zeros_like(x) for x in p] for _ in range(3))
    for t in range(3):
        g = _get(z, "gaw", "g_in", t)
        fn(p, g, ea, easq, ema, [t + 1] * P, c["alpha"], c["lamb"], c["beta1"], c["beta2"], c["lr"], c["wd"], c["eps"], c["clip"])
        _check(z, "gaw", t, g_out=g, p=p, ea=ea, easq=easq, ema=ema)


def run_neuralgrok(fn):
    z = np.load(GOLD)
    c = {k: float(z[f"ng_{k}"]) for k in ("alpha_amp", "beta_amp", "beta1", "beta2", "lr", "wd", "eps", "clip")}
    W = [z[f"ng_{k}"].astype(np.float32) for k in ("W1", "b1", "W2", "b2")]
    p = _get(z, "ng", "p", "in")
    ea, easq = ([np.zeros_like(x) for x in p] for _ in range(2))
    for t in range(3):
        g = _get(z, "ng", "g_in", t)
        fn(p, g, ea, easq, [t + 1] * P, *W, c["alpha_amp"], c["beta_amp"], c["beta1"], c["beta2"], c["lr"], c["wd"], c["eps"], c["clip"])
        _check(z, "ng", t, g_out=g, p=p, ea=ea, easq=easq)


def run_prodigy(fn):
    z = np.load(GOLD)
    c = {k: float(z[f"pr_{k}"]) for k in ("beta1", "beta2", "lr", "wd", "eps", "d_lr0")}
    p = _get(z, "pr", "p", "in")
    p0 = [x.copy() for x in p]
    ea, easq, s = ([np.zeros_like(x) for x in p] for _ in range(3))
    d_lr = c["d_lr0"]
    for t in range(4):
        g = _get(z, "pr", "g_in", t)
        d_lr = fn(p, g, ea, easq, s, p0, [t + 1] * P, d_lr, c["beta1"], c["beta2"], c["lr"], c["wd"], c["eps"])
        want = float(z[f"pr_d_lr_{t}"])
        assert abs(d_lr - want) <= 1e-4 * abs(want), (t, d_lr, want)
        _check(z, "pr", t, floor=1e-12, p=p, ea=ea, easq=easq, s=s)


def run_lion(fn):
    z = np.load(GOLD)
    c = {k: float(z[f"li_{k}"]) for k in ("lr", "beta1", "beta2", "wd")}
    p = _get(z, "li", "p", "in")
    ea = [np.zeros_like(x) for x in p]
    for t in range(3):
        g = _get(z, "li", "g_in", t)
        fn(p, g, ea, c["lr"], c["beta1"], c["beta2"], c["wd"])
        _check(z, "li", t, p=p, ea=ea)


def run_sg11(fn):
    z = np.load(GOLD)
    c = {k: float(z[f"s11_{k}"]) for k in ("rescale", "beta2", "lr", "wd", "eps", "lamb", "ramp", "temp", "clip")}
    W = [z[f"s11_{k}"].astype(np.float32) for k in ("W1", "b1", "W2", "b2")]
    alphas, beta1s = [float(a) for a in z["s11_alphas"]], [float(b) for b in z["s11_beta1s"]]
    p = _get(z, "s11", "p", "in")
    ea, easq, mu = ([np.zeros_like(x) for x in p] for _ in range(3))
    for t in range(3):
        g, sh = _get(z, "s11", "g_in", t), _get(z, "s11", "sharp", t)
        fn(p, g, ea, easq, mu, sh, [t] * P, alphas, beta1s, *W, c["rescale"], c["beta2"], c["lr"], c["wd"], c["eps"], c["lamb"],
           c["ramp"], c["temp"], c["clip"])
        _check(z, "s11", t, g_out=g, p=p, ea=ea, easq=easq, mu=mu)


def run_looksam(perturb, directions, adjust):
    z = np.load(GOLD)
    p, g = _get(z, "ls", "p", "in"), _get(z, "ls", "g", "in")
    perturb(p, g, float(z["ls_rho"]))
    _check(z, "ls", "pert", p=p)
    # directions: the reference's CPU code leaves its argument untouched (it rebinds a by-value copy), so
    # the recorded output equals the input; the in-place result is checked against its definition instead
    sam_g, v = _get(z, "ls", "sam_g", "dir"), _get(z, "ls", "v_in", "dir")
    _check(z, "ls", "dir", v_out=v)
    directions(v, sam_g, g)
    for i in range(P):
        d = (sam_g[i] - g[i]).astype(np.float64)
        n = np.sqrt((d * d).sum())
        want = d / n if n >= 1e-12 else np.full_like(d, 0.25)
        assert np.allclose(v[i], want, rtol=1e-5, atol=1e-7), i
    vd = _get(z, "ls", "v", "adj")
    adjust(g, vd, float(z["ls_la"]))
    _check(z, "ls", "adj", g_out=g)
