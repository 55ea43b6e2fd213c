"""Writes tests/golden/ref_*.npz: inputs and outputs of the reference's own CPU
code for the Grokfast, SuperGrok v1.5, Muon, SuperGrok v1.1, GrokAdamW,
NeuralGrok, Prodigy, Lion and LookSAM steps.

The outputs come from oracle/_ref/ref_ops*.so, which oracle/Makefile.ref
compiles from the reference's csrc/ops.cpp (CPU-only, where it lies under
/root/reference).  Only data is stored: seeds, input tensors, expected output
tensors.  Run in the build container:  python tests/golden/make_golden_ref.py
"""
import os
import sys

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
sys.path.insert(0, os.path.join(ROOT, "oracle", "_ref"))
import ref_ops  # noqa: E402

torch.set_num_threads(1)


def rnd(gen, *shape, std=1.0):
    return torch.randn(*shape, generator=gen, dtype=torch.float32) * std


def grokfast():
    gen = torch.Generator().manual_seed(11)
    shapes = [(37,), (16, 9), (1,), (300,)]
    emas = [torch.zeros(s) for s in shapes]
    out = {"alpha": 0.98, "lamb": 2.0, "n": len(shapes), "steps": 3}
    for t in range(3):
        grads = [rnd(gen, *s, std=1e-3) for s in shapes]
        for i, g in enumerate(grads):
            out[f"g_in_{t}_{i}"] = g.numpy().copy()
        ref_ops.grokfast_fused_step(grads, emas, 0.98, 2.0)
        for i, (g, e) in enumerate(zip(grads, emas)):
            out[f"g_out_{t}_{i}"] = g.numpy().copy()
            out[f"ema_{t}_{i}"] = e.numpy().copy()
    np.savez_compressed(os.path.join(HERE, "ref_grokfast.npz"), **out)


def sg15():
    gen = torch.Generator().manual_seed(12)
    sizes = [50, 257, 1, 1000]          # flat tensors: the reference's CPU path needs numel-shaped state
    H = 8
    W1, b1 = rnd(gen, H, 2, std=0.5), rnd(gen, H, std=0.1)
    W2, b2 = rnd(gen, 1, H, std=0.5), rnd(gen, 1, std=0.1)
    P = len(sizes)
    params = [rnd(gen, n, std=0.02) for n in sizes]
    eas, easqs, mus = [torch.zeros(n) for n in sizes], [torch.zeros(n) for n in sizes], [torch.zeros(n) for n in sizes]
    alphas = [0.98] * P
    beta1s = [0.9 * 0.9 ** i for i in range(P)]
    cfg = dict(rescale=0.1, beta2=0.999, lr=1e-3, wd_eff=2.5, eps=1e-8, lamb=2.0, ramp=1.0, gate=0.7, clip=1.0)
    out = dict(W1=W1.numpy(), b1=b1.numpy(), W2=W2.numpy(), b2=b2.numpy(), H=H, n=P, steps=3,
               alphas=np.array(alphas), beta1s=np.array(beta1s), **cfg)
    for i, p in enumerate(params):
        out[f"p_in_{i}"] = p.numpy().copy()
    for t in range(3):
        gstd = 0.3 if t == 1 else 1e-3         # step 1 trips the global-norm clip, steps 0 and 2 do not
        grads = [rnd(gen, n, std=gstd) for n in sizes]
        sharps = [rnd(gen, n, std=1e-3).abs() for n in sizes]
        for i in range(P):
            out[f"g_in_{t}_{i}"] = grads[i].numpy().copy()
            out[f"s_in_{t}_{i}"] = sharps[i].numpy().copy()
        steps = [t] * P                         # explicit step counts: true bias correction
        ref_ops.supergrok15_fused_step(params, grads, eas, easqs, mus, sharps, steps, alphas, beta1s, W1, b1, W2, b2,
                                       cfg["rescale"], H, cfg["beta2"], cfg["lr"], cfg["wd_eff"], cfg["eps"], cfg["lamb"],
                                       cfg["ramp"], cfg["gate"], cfg["clip"])
        for i in range(P):
            out[f"p_{t}_{i}"] = params[i].numpy().copy()
            out[f"ea_{t}_{i}"] = eas[i].numpy().copy()
            out[f"easq_{t}_{i}"] = easqs[i].numpy().copy()
            out[f"mu_{t}_{i}"] = mus[i].numpy().copy()
            out[f"g_out_{t}_{i}"] = grads[i].numpy().copy()
    # SAM helpers
    ps = [rnd(gen, n, std=0.02) for n in sizes]
    gs = [rnd(gen, n, std=1e-2) for n in sizes]
    for i in range(P):
        out[f"sam_p_in_{i}"] = ps[i].numpy().copy()
        out[f"sam_g_{i}"] = gs[i].numpy().copy()
    backups = ref_ops.supergrok15_sam_perturb_all(ps, gs, 0.05)
    for i in range(P):
        out[f"sam_p_out_{i}"] = ps[i].numpy().copy()
        out[f"sam_backup_{i}"] = backups[i].numpy().copy()
    sam_g = [rnd(gen, n, std=1e-2) for n in sizes]
    cache = [torch.zeros(n) for n in sizes]
    ref_ops.supergrok15_sharpness_restore_all(ps, cache, backups, sam_g, gs)
    for i in range(P):
        out[f"sam_g2_{i}"] = sam_g[i].numpy().copy()
        out[f"sharp_out_{i}"] = cache[i].numpy().copy()
        out[f"restored_{i}"] = ps[i].numpy().copy()
    np.savez_compressed(os.path.join(HERE, "ref_sg15.npz"), **out)


def muon():
    gen = torch.Generator().manual_seed(13)
    shapes = [(24, 40), (40, 24), (16, 16)]
    out = dict(n=len(shapes), steps=2, momentum=0.95, lr=0.02, wd=1.0, ns_steps=5)
    for tag, dt in (("f32", torch.float32), ("bf16", torch.bfloat16)):
        params = [rnd(gen, *s, std=0.02).to(dt) for s in shapes]
        bufs = [torch.zeros(s) for s in shapes]
        for i, p in enumerate(params):
            out[f"{tag}_p_in_{i}"] = p.float().numpy().copy()
        for t in range(2):
            grads = [rnd(gen, *s, std=1e-3).to(dt) for s in shapes]
            for i, g in enumerate(grads):
                out[f"{tag}_g_{t}_{i}"] = g.float().numpy().copy()
            ref_ops.muon_fused_step(params, grads, bufs, 0.95, 0.02, 1.0, 5)
            for i in range(len(shapes)):
                out[f"{tag}_p_{t}_{i}"] = params[i].float().numpy().copy()
                out[f"{tag}_buf_{t}_{i}"] = bufs[i].numpy().copy()
    np.savez_compressed(os.path.join(HERE, "ref_muon.npz"), **out)


def family():
    """The remaining fused steps (csrc/ops.cpp:209-656): SuperGrok v1.1, GrokAdamW, NeuralGrok, Prodigy, Lion, LookSAM."""
    out = {}
    sizes = [50, 257, 1, 1000]
    P = len(sizes)

    def put(tag, t, name, tensors):
        for i, x in enumerate(tensors):
            out[f"{tag}_{name}_{t}_{i}"] = x.detach().float().numpy().copy()

    # GrokAdamW: step 1 trips the global-norm clip
    gen = torch.Generator().manual_seed(21)
    params = [rnd(gen, n, std=0.02) for n in sizes]
    eas, easqs, emas = ([torch.zeros(n) for n in sizes] for _ in range(3))
    cfg = dict(alpha=0.98, lamb=5.0, beta1=0.9, beta2=0.98, lr=1e-3, wd=1.0, eps=1e-8, clip=1.0)
    out.update({f"gaw_{k}": v for k, v in cfg.items()})
    put("gaw", "in", "p", params)
    for t in range(3):
        grads = [rnd(gen, n, std=0.3 if t == 1 else 1e-3) for n in sizes]
        put("gaw", t, "g_in", grads)
        ref_ops.grokadamw_fused_step(params, grads, eas, easqs, emas, [t + 1] * P, cfg["alpha"], cfg["lamb"], cfg["beta1"],
                                     cfg["beta2"], cfg["lr"], cfg["wd"], cfg["eps"], cfg["clip"])
        for name, ts in (("g_out", grads), ("p", params), ("ea", eas), ("easq", easqs), ("ema", emas)):
            put("gaw", t, name, ts)

    # NeuralGrok
    gen = torch.Generator().manual_seed(22)
    H = 8
    W1, b1, W2, b2 = rnd(gen, H, 1, std=0.5), rnd(gen, H, std=0.1), rnd(gen, 1, H, std=0.5), rnd(gen, 1, std=0.1)
    params = [rnd(gen, n, std=0.02) for n in sizes]
    eas, easqs = ([torch.zeros(n) for n in sizes] for _ in range(2))
    cfg = dict(alpha_amp=10.0, beta_amp=4.0, beta1=0.9, beta2=0.98, lr=1e-3, wd=1.0, eps=1e-8, clip=1.0)
    out.update({f"ng_{k}": v for k, v in cfg.items()})
    out.update(ng_W1=W1.numpy(), ng_b1=b1.numpy(), ng_W2=W2.numpy(), ng_b2=b2.numpy(), ng_H=H)
    put("ng", "in", "p", params)
    for t in range(3):
        grads = [rnd(gen, n, std=0.3 if t == 1 else 1e-3) for n in sizes]
        put("ng", t, "g_in", grads)
        ref_ops.neuralgrok_fused_step(params, grads, eas, easqs, [t + 1] * P, W1, b1, W2, b2, cfg["alpha_amp"], cfg["beta_amp"], H,
                                      cfg["beta1"], cfg["beta2"], cfg["lr"], cfg["wd"], cfg["eps"], cfg["clip"])
        for name, ts in (("g_out", grads), ("p", params), ("ea", eas), ("easq", easqs)):
            put("ng", t, name, ts)

    # Prodigy: d_lr is returned and fed back
    gen = torch.Generator().manual_seed(23)
    params = [rnd(gen, n, std=0.02) for n in sizes]
    inits = [p.clone() for p in params]
    eas, easqs, ss = ([torch.zeros(n) for n in sizes] for _ in range(3))
    cfg = dict(beta1=0.9, beta2=0.999, lr=1e-3, wd=0.0, eps=1e-8, d_lr0=1e-6)
    out.update({f"pr_{k}": v for k, v in cfg.items()})
    put("pr", "in", "p", params)
    d_lr = cfg["d_lr0"]
    for t in range(4):
        grads = [rnd(gen, n, std=1e-2) for n in sizes]
        put("pr", t, "g_in", grads)
        d_lr = ref_ops.prodigy_fused_step(params, grads, eas, easqs, ss, inits, [t + 1] * P, d_lr, cfg["beta1"], cfg["beta2"],
                                          cfg["lr"], cfg["wd"], cfg["eps"])
        out[f"pr_d_lr_{t}"] = d_lr
        for name, ts in (("p", params), ("ea", eas), ("easq", easqs), ("s", ss)):
            put("pr", t, name, ts)

    # Lion (an exactly-zero gradient and momentum exercises sign(0) = 0)
    gen = torch.Generator().manual_seed(24)
    params = [rnd(gen, n, std=0.02) for n in sizes]
    eas = [torch.zeros(n) for n in sizes]
    cfg = dict(lr=1e-4, beta1=0.9, beta2=0.99, wd=3.0)
    out.update({f"li_{k}": v for k, v in cfg.items()})
    put("li", "in", "p", params)
    for t in range(3):
        grads = [rnd(gen, n, std=1e-3) for n in sizes]
        if t == 0:
            grads[1][:7] = 0.0
        put("li", t, "g_in", grads)
        ref_ops.lion_fused_step(params, grads, eas, cfg["lr"], cfg["beta1"], cfg["beta2"], cfg["wd"])
        for name, ts in (("p", params), ("ea", eas)):
            put("li", t, name, ts)

    # SuperGrok v1.1 (steps travel by value through the binding, exactly as for v1.5)
    gen = torch.Generator().manual_seed(25)
    H = 8
    W1, b1, W2, b2 = rnd(gen, H, 2, std=0.5), rnd(gen, H, std=0.1), rnd(gen, 1, H, std=0.5), rnd(gen, 1, std=0.1)
    params = [rnd(gen, n, std=0.02) for n in sizes]
    eas, easqs, mus = ([torch.zeros(n) for n in sizes] for _ in range(3))
    alphas = [0.98] * P
    beta1s = [0.9 * 0.9 ** i for i in range(P)]
    cfg = dict(rescale=0.1, beta2=0.999, lr=1e-3, wd=1.0, eps=1e-8, lamb=5.0, ramp=0.5, temp=5.0, clip=1.0)
    out.update({f"s11_{k}": v for k, v in cfg.items()})
    out.update(s11_W1=W1.numpy(), s11_b1=b1.numpy(), s11_W2=W2.numpy(), s11_b2=b2.numpy(), s11_H=H,
               s11_alphas=np.array(alphas), s11_beta1s=np.array(beta1s))
    put("s11", "in", "p", params)
    for t in range(3):
        grads = [rnd(gen, n, std=0.3 if t == 1 else 1e-3) for n in sizes]
        sharps = [rnd(gen, n, std=1e-3).abs() for n in sizes]
        put("s11", t, "g_in", grads)
        put("s11", t, "sharp", sharps)
        steps = [t] * P
        ref_ops.supergrok11_fused_step(params, grads, eas, easqs, mus, sharps, steps, alphas, beta1s, W1, b1, W2, b2, cfg["rescale"], H,
                                       cfg["beta2"], cfg["lr"], cfg["wd"], cfg["eps"], cfg["lamb"], cfg["ramp"], cfg["temp"],
                                       cfg["clip"])
        for name, ts in (("g_out", grads), ("p", params), ("ea", eas), ("easq", easqs), ("mu", mus)):
            put("s11", t, name, ts)

    # LookSAM helpers
    gen = torch.Generator().manual_seed(26)
    params = [rnd(gen, n, std=0.02) for n in sizes]
    grads = [rnd(gen, n, std=1e-3) for n in sizes]
    put("ls", "in", "p", params)
    put("ls", "in", "g", grads)
    out["ls_rho"] = 0.05
    backups = ref_ops.looksam_perturb_all(params, grads, 0.05)
    put("ls", "pert", "p", params)
    put("ls", "pert", "backup", backups)
    ref_ops.looksam_restore_all(params, backups)
    put("ls", "rest", "p", params)
    sam_grads = [rnd(gen, n, std=1e-3) for n in sizes]
    sam_grads[2] = grads[2].clone()          # zero difference: that direction is left as it was
    v_dirs = [torch.full((n,), 0.25) for n in sizes]
    put("ls", "dir", "sam_g", sam_grads)
    put("ls", "dir", "v_in", v_dirs)
    ref_ops.looksam_compute_directions(v_dirs, sam_grads, grads)
    put("ls", "dir", "v_out", v_dirs)        # unchanged: the CPU branch rebinds its by-value copy of the list
    vd = [rnd(gen, n) for n in sizes]
    vd = [v / v.norm() for v in vd]
    put("ls", "adj", "v", vd)
    out["ls_la"] = 0.7
    ref_ops.looksam_adjust_grads(grads, vd, 0.7)
    put("ls", "adj", "g_out", grads)
    np.savez_compressed(os.path.join(HERE, "ref_family.npz"), **out)


if __name__ == "__main__":
    grokfast()
    sg15()
    muon()
    family()
    for f in sorted(os.listdir(HERE)):
        if f.endswith(".npz"):
            print(f, os.path.getsize(os.path.join(HERE, f)), "bytes")
