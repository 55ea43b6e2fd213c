"""Full-size (50 tensors, ~25M elements) checks of the SuperGrok v2 batched
step through size-independent properties: the sort output is a sorted
permutation per tensor, expert_counts adds up, everything stays finite, and
two identically seeded runs agree bit for bit (the reference's own
reproducibility test, tests/test_supergrok2.py:513-547)."""
import pytest
import torch

import workloads as wl
from helpers import DIMS
from sg2_harness import per_tensor_scalars, shared_scalars

pytestmark = pytest.mark.gpu


def _run(steps):
    from grokking_optimizers import _cabi
    shapes = wl.scale50_shapes()
    dev = "cuda"
    gh, di, ds = DIMS["gru_hidden"], DIMS["d_inner"], DIMS["d_state"]
    params = [p.reshape(-1).to(dev) for p in wl.make_params(shapes, seed=0)]
    z = lambda *s: torch.zeros(*s, device=dev)
    eas, easqs, mus = [z(p.numel()) for p in params], [z(p.numel()) for p in params], [z(p.numel()) for p in params]
    grus = [z(p.numel(), gh) for p in params]
    mf, mb = [z(di, ds) for _ in params], [z(di, ds) for _ in params]
    counts = torch.zeros(144, dtype=torch.int32, device=dev)
    W = [w.to(dev) for w in wl.meta_weights(7)]
    step = _cabi.Sg2Step(W, params, eas, easqs, mus, grus, mf, mb, counts, debug=True)
    gl = []
    for t in range(1, steps + 1):
        grads = wl.clip_per_tensor(wl.make_grads(shapes, seed=t, tail_frac=0.005, tail="student3"))
        grads = [g.reshape(-1).to(dev) for g in grads]
        gl = grads
        step(grads, [torch.zeros_like(g) for g in grads], per_tensor_scalars(len(shapes), t), shared_scalars())
    torch.cuda.synchronize()
    return shapes, params, eas, easqs, mus, grus, mf, mb, counts, step, gl


def test_scale50_properties_and_determinism():
    print("scale50 run A", flush=True)
    shapes, params, eas, easqs, mus, grus, mf, mb, counts, step, grads = _run(2)
    total = sum(wl.numel(s) for s in shapes)
    assert int(counts.sum()) == 2 * 4 * total
    off = 0
    for g in grads:
        n = g.numel()
        perm = step.perm[off:off + n].long()
        assert torch.equal(torch.sort(perm).values, torch.arange(n, device=perm.device))
        keys = g.abs()[perm]
        assert bool((keys[1:] >= keys[:-1]).all())
        ties = keys[1:] == keys[:-1]                      # stability: equal keys keep index order
        assert bool((perm[1:][ties] > perm[:-1][ties]).all())
        off += n
    assert int(step.expert_idx.min()) >= 0 and int(step.expert_idx.max()) < 144
    for lst in (params, eas, easqs, mus, grus, mf, mb):
        for t in lst:
            assert bool(torch.isfinite(t).all())
    print("scale50 run B", flush=True)
    again = _run(2)
    for a, b in zip((params, eas, easqs, mus, grus, mf, mb), again[1:8]):
        for x, y in zip(a, b):
            assert torch.equal(x, y)
    assert torch.equal(counts, again[8])
