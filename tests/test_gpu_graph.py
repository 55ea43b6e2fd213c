"""The step entry points under HIP graph capture: nothing in a call blocks the host or copies from host memory (the
per-call tables travel as kernel arguments), so a call can be recorded once and replayed.  A replay repeats the
recorded scalars (step size, bias corrections); the test therefore replays the same step on restored state and
requires every replay to equal the eager result bit for bit, with eager work and synchronisations in between."""
import numpy as np
import pytest
import torch

import workloads as wl
from sg2_harness import per_tensor_scalars, shared_scalars

pytestmark = pytest.mark.gpu

KEYS = ("param", "exp_avg", "exp_avg_sq", "mu", "gru", "mamba_fwd", "mamba_bwd")


def _state(shapes, seed, dev):
    gen = torch.Generator().manual_seed(seed)
    out = []
    for p in wl.make_params(shapes, seed=seed):
        n = p.numel()
        out.append(dict(param=p.reshape(-1).clone(), exp_avg=torch.randn(n, generator=gen) * 1e-3,
                        exp_avg_sq=torch.rand(n, generator=gen) * 1e-6, mu=torch.randn(n, generator=gen) * 1e-3,
                        gru=torch.randn(n, 4, generator=gen) * 0.3, mamba_fwd=torch.randn(16, 16, generator=gen) * 0.1,
                        mamba_bwd=torch.randn(16, 16, generator=gen) * 0.1))
    return [{k: v.to(dev) for k, v in st.items()} for st in out]


def _restore(state, saved):
    for st, sv in zip(state, saved):
        for k in KEYS:
            st[k].copy_(sv[k])


def _snapshot(state):
    return [{k: st[k].clone() for k in KEYS} for st in state]


def _equal(state, want, what):
    for i, (st, w) in enumerate(zip(state, want)):
        for k in KEYS:
            assert torch.equal(st[k], w[k]), "%s: tensor %d %s differs from the eager step" % (what, i, k)


@pytest.mark.parametrize("entry", ["workspace", "static"])
def test_v2_step_replays_from_a_graph(entry):
    from grokking_optimizers import _cabi
    dev = "cuda"
    shapes = [(3000,), (64, 130), (257,), (9000,)]
    W = [w.to(dev) for w in wl.meta_weights(7)]
    state = _state(shapes, 3, dev)
    counts = torch.zeros(144, dtype=torch.int32, device=dev)
    grads = [g.reshape(-1).to(dev) for g in wl.make_grads(shapes, seed=11)]
    sharps = [(g.abs() * 0.5).contiguous() for g in grads]
    pt, sh = per_tensor_scalars(len(shapes), 3, lamb_eff=2.0), shared_scalars(wd_eff=4.5)
    if entry == "workspace":
        step = _cabi.Sg2Step(W, *[[s[k] for s in state] for k in KEYS], counts)
    else:
        from test_zz_no_alloc import _StaticStep
        step = _StaticStep(W, state, counts)
    start = _snapshot(state)
    step(grads, sharps, pt, sh)                      # eager (also the first call of the static entry on this device)
    torch.cuda.synchronize()
    want, want_counts = _snapshot(state), counts.clone()

    graph = torch.cuda.CUDAGraph()
    _restore(state, start)
    counts.zero_()
    torch.cuda.synchronize()
    print("capturing", entry, flush=True)
    with torch.cuda.graph(graph):
        step(grads, sharps, pt, sh)
    torch.cuda.synchronize()
    for rep in range(3):
        _restore(state, start)
        counts.zero_()
        scratch = torch.randn(1 << 20, device=dev).sum()     # eager work between the replays
        torch.cuda.synchronize()
        print("replay", rep, flush=True)
        graph.replay()
        torch.cuda.synchronize()
        _equal(state, want, "%s entry, replay %d" % (entry, rep))
        assert torch.equal(counts, want_counts)
        assert bool(torch.isfinite(scratch))


def test_grokfast_step_replays_from_a_graph():
    from grokking_optimizers import _ops as ops
    dev = "cuda"
    shapes = wl.small8_shapes()
    params = [p.reshape(-1).to(dev) for p in wl.make_params(shapes, seed=0)]
    grads = [g.reshape(-1).to(dev) for g in wl.make_grads(shapes, seed=1)]
    emas = [torch.zeros_like(p) for p in params]
    eas, easqs = [torch.zeros_like(p) for p in params], [torch.zeros_like(p) for p in params]
    everything = params + grads + emas + eas + easqs        # the step amplifies the gradients in place
    start = [t.clone() for t in everything]

    def run():
        ops.grokfast_adamw_fused_step(params, grads, emas, eas, easqs, [1] * len(params), 0.98, 2.0, 1e-3, 0.9, 0.999, 1e-8, 1.0)
    run()
    torch.cuda.synchronize()
    want = [t.clone() for t in everything]
    graph = torch.cuda.CUDAGraph()
    for t, s in zip(everything, start):
        t.copy_(s)
    torch.cuda.synchronize()
    with torch.cuda.graph(graph):
        run()
    for rep in range(3):
        for t, s in zip(everything, start):
            t.copy_(s)
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        for t, w in zip(everything, want):
            assert torch.equal(t, w), "replay %d differs" % rep
