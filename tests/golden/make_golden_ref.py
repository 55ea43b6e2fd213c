"""Writes tests/golden/ref_*.npz: inputs and outputs of the reference's own CPU
code for the Grokfast, SuperGrok v1.5 and Muon steps.

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


if __name__ == "__main__":
    grokfast()
    sg15()
    muon()
    for f in sorted(os.listdir(HERE)):
        if f.endswith(".npz"):
            print(f, os.path.getsize(os.path.join(HERE, f)), "bytes")
