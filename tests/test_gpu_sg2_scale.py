"""Full-size (50 tensors, ~25M elements) checks of the SuperGrok v2 batched
step through size-independent properties: the sort output is a sorted
permutation per tensor, expert_counts adds up, everything stays finite, and
two identically seeded runs agree bit for bit (the reference's own
reproducibility test, tests/test_supergrok2.py:513-547)."""
import pytest
import torch

import workloads as wl
from helpers import DIMS
from sg2_harness import Sg2Case, per_tensor_scalars, shared_scalars

pytestmark = pytest.mark.gpu


def test_benchmark_chunking_against_the_checker():
    """The configuration the benchmark runs, compared value by value: the largest tensor of the 50-tensor set
    (2048 x 2048: 1024 chunks of 4096 steps per direction, the multi-block spine of the radix sort) and two mid-size
    ones, Student-t tailed gradients with the per-tensor clip applied (active for the large tensor), chunk length 4096
    and summary window 64 as the library chooses them for the full set, a random carried state, two chained steps.
    Sort permutation, expert indices and counts bit-exact; every float within rel 1e-4."""
    from grokking_optimizers import _cabi
    all_shapes = wl.scale50_shapes()
    shapes = [all_shapes[49], all_shapes[40], all_shapes[33]]
    assert wl.numel(shapes[0]) == 4194304
    lib = _cabi.lib()
    assert lib.sg2_set_chunk_len(4096) == 0 and lib.sg2_set_scan_window(64) == 0
    try:
        case = Sg2Case(shapes, seed=9, random_state=True)
        for t in (1, 2):
            raw = wl.make_grads(shapes, seed=40 + t, tail_frac=0.005, tail="student3")
            grads = wl.clip_per_tensor(raw)
            assert float(raw[0].norm()) > 1.0                       # the clip is active on the 4 M tensor
            sharps = [torch.zeros_like(g) for g in grads]
            pt, sh = per_tensor_scalars(len(shapes), t, lamb_eff=2.0), shared_scalars(wd_eff=4.5)
            print("benchmark chunking: step", t, "GPU", flush=True)
            case.gpu_step(grads, sharps, pt, sh)
            print("benchmark chunking: step", t, "checker", flush=True)
            dbg = case.oracle_step(grads, sharps, pt, sh, chunk_len=4096, window=64)
            worst = case.compare(dbg, 1e-4, 1e-7)
            print("benchmark chunking: step", t, "worst tolerance ratios", worst, flush=True)
    finally:
        lib.sg2_set_chunk_len(0)
        lib.sg2_set_scan_window(-1)


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


def test_bilevel_pass_at_scale_linearity_and_chunking():
    """The bilevel meta-gradient pass on the full 50-tensor set (25 M elements, up to 1024 chunks per tensor), through
    properties that do not need a CPU answer: the gradients are linear in the cotangent; a different chunk length
    (another decomposition of the same sums) gives the same result; a repeat gives every gradient bit for bit, except
    those of the expert MLPs: gradients as large as these (std 0.3) leave the intervals next to zero of their experts,
    and such elements add to their bins with LDS atomics of four waves (order of addition varies), so these repeat to
    2e-5 of their scale (fp32 sums of some 1e5 terms in another order)."""
    from grokking_optimizers import Mamba3PEERMetaNet, _bilevel, _cabi
    dev = torch.device("cuda:0")
    shapes = wl.scale50_shapes()
    torch.manual_seed(11)
    mn = Mamba3PEERMetaNet().to(dev)
    with torch.no_grad():
        for p in mn.parameters():
            if p.dim() > 0 and float(p.abs().max()) < 0.05:
                p.add_(torch.randn_like(p) * 0.2)
    grads = [g.reshape(-1).to(dev) for g in wl.make_grads(shapes, seed=3, std=0.3)]
    sharps = [g.abs() * 0.5 for g in grads]
    gen = torch.Generator().manual_seed(4)
    grus = [(torch.randn(g.numel(), 4, generator=gen) * 0.5).to(dev) for g in grads]
    mf = [(torch.randn(16, 16, generator=gen) * 0.3).to(dev) for _ in grads]
    mb = [(torch.randn(16, 16, generator=gen) * 0.3).to(dev) for _ in grads]
    c1 = [torch.randn(g.numel(), generator=gen).to(dev) for g in grads]
    c2 = [torch.randn(g.numel(), generator=gen).to(dev) for g in grads]

    def run(cots):
        mn.zero_grad()
        smart = _bilevel.accumulate_meta_gradients(mn, grads, sharps, grus, mf, mb, cots)
        torch.cuda.synchronize()
        return smart, {n: p.grad.clone() for n, p in mn.named_parameters()}

    print("bilevel at scale: cotangent 1", flush=True)
    s1, g1 = run(c1)
    print("bilevel at scale: cotangent 2", flush=True)
    s2, g2 = run(c2)
    print("bilevel at scale: sum of both", flush=True)
    s3, g3 = run([a + b for a, b in zip(c1, c2)])
    assert torch.equal(s1, s2) and torch.equal(s1, s3) and bool(torch.isfinite(s1).all())     # smart does not depend on the cotangent
    for n in g1:
        want = g1[n].double() + g2[n].double()
        scale = float(want.abs().max())
        assert bool(torch.isfinite(g3[n]).all()) and scale > 0, n
        assert float((g3[n].double() - want).abs().max()) <= 2e-4 * scale, (n, scale)
    print("bilevel at scale: repeat", flush=True)
    s1b, g1b = run(c1)
    assert torch.equal(s1, s1b)
    for n in g1:
        if n.startswith("expert_"):
            scale = float(g1[n].abs().max())
            assert float((g1[n].double() - g1b[n].double()).abs().max()) <= 2e-5 * scale, (n, scale)
        else:
            assert torch.equal(g1[n], g1b[n]), n
    print("bilevel at scale: chunk length 1024", flush=True)
    assert _cabi.lib().sg2_set_chunk_len(1024) == 0
    try:
        s1c, g1c = run(c1)
    finally:
        _cabi.lib().sg2_set_chunk_len(0)
    assert float((s1c - s1).abs().max()) <= 1e-4 * float(s1.abs().max())
    for n in g1:
        scale = float(g1[n].abs().max())
        assert float((g1c[n].double() - g1[n].double()).abs().max()) <= 2e-4 * scale, (n, scale)


def test_one_tensor_beyond_32_bit_byte_offsets():
    """One tensor of 2^27 + 12345 elements (32 769 chunks of 4096 steps per direction, 16 386 sort tiles, context and
    GRU arrays past 4 GiB, so every byte offset that could wrap a 32-bit integer is exercised), with a quarter of the
    gradients quantised so that the sort meets long runs of equal keys.  Checked through what needs no CPU answer:
    the permutation is a stable sort of |g|, expert_counts adds up, every state stays finite, a second run with a
    different chunk length (another decomposition of the same scan) agrees within the step's tolerance, and a repeat
    of the first run agrees bit for bit."""
    from grokking_optimizers import _cabi
    dev = "cuda"
    n = (1 << 27) + 12345
    gh, di, ds = DIMS["gru_hidden"], DIMS["d_inner"], DIMS["d_state"]
    gen = torch.Generator(device=dev).manual_seed(5)
    g = torch.randn(n, device=dev, generator=gen) * 1e-3
    g[::4] = torch.round(g[::4] * 4096.0) / 4096.0            # multiples of 2^-12: mostly 0 and +-2.4e-4, huge tie groups
    p0 = torch.randn(n, device=dev, generator=gen) * 0.02
    W = [w.to(dev) for w in wl.meta_weights(7)]
    lib = _cabi.lib()

    def run(chunk_len, debug):
        z = lambda *s: torch.zeros(*s, device=dev)
        st = dict(p=[p0.clone()], ea=[z(n)], easq=[z(n)], mu=[z(n)], gru=[z(n, gh)], mf=[z(di, ds)], mb=[z(di, ds)])
        counts = torch.zeros(144, dtype=torch.int32, device=dev)
        step = _cabi.Sg2Step(W, st["p"], st["ea"], st["easq"], st["mu"], st["gru"], st["mf"], st["mb"], counts, debug=debug,
                             chunk_len=chunk_len)
        print("2^27 elements: chunk_len", chunk_len, flush=True)
        step([g], [torch.zeros_like(g)], per_tensor_scalars(1, 1), shared_scalars())
        torch.cuda.synchronize()
        return st, counts, step

    assert _cabi.chunk_len_for([n]) == 4096
    st, counts, step = run(None, True)
    assert int(counts.sum()) == 4 * n
    perm = step.perm[:n].long()
    seen = torch.zeros(n, dtype=torch.bool, device=dev)
    seen[perm] = True
    assert bool(seen.all())
    keys = g.abs()[perm]
    assert bool((keys[1:] >= keys[:-1]).all())
    ties = keys[1:] == keys[:-1]
    assert int(ties.sum()) > n // 8
    assert bool((perm[1:][ties] > perm[:-1][ties]).all())
    assert int(step.expert_idx.min()) >= 0 and int(step.expert_idx.max()) < 144
    del perm, seen, keys, ties, step
    for name, lst in st.items():
        assert bool(torch.isfinite(lst[0]).all()), name
    assert float((st["p"][0] - p0).abs().max()) > 0.0
    torch.cuda.empty_cache()

    other, counts_b, _ = run(1024, False)
    worst = 0.0
    for name in ("p", "ea", "easq", "mu", "gru", "mf", "mb"):
        a, b = st[name][0], other[name][0]
        floor = 1e-5 * float(a.abs().max()) + 1e-30
        ratio = float(((a - b).abs() / (1e-4 * torch.maximum(a.abs(), b.abs()) + floor)).max())
        worst = max(worst, ratio)
        assert ratio <= 1.0, (name, ratio)
    flips = int((counts - counts_b).abs().sum()) // 2
    print("chunk 4096 against 1024: worst tolerance ratio", worst, "routing decisions that differ:", flips, flush=True)
    assert flips <= n // 100000
    del other
    torch.cuda.empty_cache()

    again, counts_c, _ = run(None, False)
    for name in st:
        assert torch.equal(st[name][0], again[name][0]), name
    assert torch.equal(counts, counts_c)
