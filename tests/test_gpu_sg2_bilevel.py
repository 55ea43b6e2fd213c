"""Bilevel path of SuperGrok v2, sequential part: the HIP forward (sort + bidirectional scan, through
sg2_bilevel_forward) and the HIP adjoint (sg2_bilevel_backward) against float64 autograd through the
independent torch restatement of the scan (ref_fp64.scan_block, written from
grokking_optimizers/mamba3_peer_metanet.py:90-160 of the reference).

The loss is sum(ctx * R) for a fixed random R, so every context entry of every element carries a gradient.
Gates: contexts within |a-b| <= 1e-4*max(|a|,|b|) + 1e-7; each weight gradient within 2e-4 of the largest
entry of that gradient (fp32 sums over all elements against float64)."""
import numpy as np
import pytest
import torch

import ref_fp64
import workloads as wl

pytestmark = pytest.mark.gpu

NAMES = ["input_proj.W", "input_proj.b"] + [d + n for d in ("fwd.", "bwd.") for n in
         ("in_proj", "dt_W", "dt_b", "B_proj", "C_proj", "A_log", "D", "rope_freq", "out_proj")]


def _reference(W, grads, sharps, mf, mb, R):
    Wd = [w.detach().double().cpu().requires_grad_(True) for w in W[:20]]
    loss = torch.zeros((), dtype=torch.float64)
    ctx = []
    off = 0
    for g, s, hf, hb in zip(grads, sharps, mf, mb):
        g, s = g.reshape(-1).double().cpu(), s.reshape(-1).double().cpu()
        n = g.numel()
        perm = torch.sort(g.abs().float(), stable=True).indices
        x = torch.stack([g[perm], s[perm]], -1) @ Wd[0].T + Wd[1]
        fo, _ = ref_fp64.scan_block(x, Wd[2:11], hf.double().cpu())
        bo, _ = ref_fp64.scan_block(x.flip(0), Wd[11:20], hb.double().cpu())
        unsort = torch.argsort(perm)
        cf, cb = fo[unsort], bo.flip(0)[unsort]
        loss = loss + (cf * R[0, off:off + n]).sum() + (cb * R[1, off:off + n]).sum()
        ctx.append((cf.detach(), cb.detach()))
        off += n
    loss.backward()
    return ctx, [w.grad for w in Wd]


def _case(shapes, seed, sharp, state_std, chunk_len=None):
    from grokking_optimizers import _bilevel, _cabi
    dev = torch.device("cuda:0")
    if chunk_len is not None:
        assert _cabi.lib().sg2_set_chunk_len(chunk_len) == 0
    try:
        W = [w.to(dev) for w in wl.meta_weights(seed)]
        grads = [g.to(dev) for g in wl.make_grads(shapes, seed=seed + 1, std=0.5)]
        sharps = [(g.abs() * 0.5).to(dev) if sharp else torch.zeros_like(g, device=dev)
                  for g in wl.make_grads(shapes, seed=seed + 2, std=0.5)]
        gen = torch.Generator().manual_seed(seed + 3)
        mf = [(torch.randn(16, 16, generator=gen) * state_std).to(dev) for _ in shapes]
        mb = [(torch.randn(16, 16, generator=gen) * state_std).to(dev) for _ in shapes]
        total = sum(g.numel() for g in grads)
        R = torch.randn(2, total, 8, generator=gen, dtype=torch.float64)
        params = [w.clone().requires_grad_(True) for w in W[:20]]
        print("bilevel case shapes", shapes, "seed", seed, "sharp", sharp, "chunk", chunk_len, flush=True)
        ctx = _bilevel.scan_contexts(W, params, grads, sharps, mf, mb)
        (ctx.double() * R.to(dev)).sum().backward()
        torch.cuda.synchronize()
        for m0, m1 in zip(mf + mb, [m.clone() for m in mf + mb]):
            assert torch.equal(m0, m1)
        ref_ctx, ref_grads = _reference(W, grads, sharps, mf, mb, R)
        off = 0
        for (cf, cb), g in zip(ref_ctx, grads):
            n = g.numel()
            for d, ref in ((0, cf), (1, cb)):
                got = ctx[d, off:off + n].detach().double().cpu()
                err = (got - ref).abs()
                tol = 1e-4 * torch.maximum(got.abs(), ref.abs()) + 1e-7
                assert bool((err <= tol).all()), ("ctx", d, n, float((err / tol).max()))
            off += n
        worst = {}
        for name, p, ref in zip(NAMES, params, ref_grads):
            got = p.grad.double().cpu()
            scale = float(ref.abs().max())
            ratio = float((got - ref).abs().max()) / (2e-4 * scale + 1e-12)
            worst[name] = round(ratio, 3)
            assert ratio <= 1.0, (name, ratio, scale)
        print("worst gradient tolerance ratios", worst, flush=True)
    finally:
        if chunk_len is not None:
            _cabi.lib().sg2_set_chunk_len(0)


def test_small_tensors_with_sharpness_and_carried_states():
    _case([(300,), (70,), (1,), (129,), (5, 13)], seed=11, sharp=True, state_std=0.3)


def test_zero_sharpness_and_zero_states():
    _case([(200,), (64,), (65,)], seed=12, sharp=False, state_std=0.0)


def test_several_chunks():
    """Chunk length 64: the forward pass runs summaries, chunk prefix and replay; the adjoint crosses chunk borders."""
    _case([(1000,), (257,), (640,)], seed=13, sharp=True, state_std=0.3, chunk_len=64)
