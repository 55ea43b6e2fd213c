"""Parity of the SuperGrok v2 batched step (HIP, through the C ABI of
libsg_hip.so) with the CPU checker on identical seeded inputs.

Gates: sort permutation, PEER expert indices and expert_counts bit-exact;
param / exp_avg / exp_avg_sq / mu / gru_state / Mamba carries within
|a-b| <= 1e-4*max(|a|,|b|) + 1e-7 after every step (fp32)."""
import numpy as np
import pytest
import torch

import workloads as wl
from helpers import DIMS
from sg2_harness import Sg2Case, per_tensor_scalars, shared_scalars

pytestmark = pytest.mark.gpu

REL, FLOOR = 1e-4, 1e-7


@pytest.fixture(autouse=True)
def _default_chunk():
    from grokking_optimizers import _cabi
    _cabi.lib().sg2_set_chunk_len(0)
    _cabi.lib().sg2_set_scan_window(-1)
    yield
    _cabi.lib().sg2_set_chunk_len(0)
    _cabi.lib().sg2_set_scan_window(-1)


def _run_steps(case, steps, chunk_len, grad_seed0=1, lamb_eff=0.0, wd_eff=1.0, grad_std=1e-3, sharp=False,
               tail_frac=0.0):
    worst = {}
    for t in range(1, steps + 1):
        grads = wl.make_grads(case.shapes, seed=grad_seed0 + t, std=grad_std, tail_frac=tail_frac, tail="student3")
        sharps = ([g.abs() * 0.5 for g in wl.make_grads(case.shapes, seed=500 + t)] if sharp
                  else [torch.zeros_like(g) for g in grads])
        pt, sh = per_tensor_scalars(case.P, t, lamb_eff), shared_scalars(wd_eff)
        print("step", t, "shapes", len(case.shapes), "chunk", chunk_len, flush=True)
        case.gpu_step(grads, sharps, pt, sh)
        dbg = case.oracle_step(grads, sharps, pt, sh, chunk_len)
        w = case.compare(dbg, REL, FLOOR)
        for k, v in w.items():
            worst[k] = max(worst.get(k, 0.0), v)
    return worst


def test_small_tensors_single_chunk():
    """All tensors below 256 elements (the reference's sequential-scan regime), 3 steps."""
    case = Sg2Case(wl.small8_shapes(), seed=3)
    w = _run_steps(case, 3, chunk_len=None, sharp=True, lamb_eff=2.0, wd_eff=4.5)
    print("worst tolerance ratios", w)


def test_multi_chunk_small_chunks():
    """Chunk length 64/256 on mid-size tensors exercises summaries + chunk prefix."""
    from grokking_optimizers import _cabi
    shapes = [(1000,), (64, 65), (257,), (3, 4096), (64,), (5000,)]
    for cl in (64, 256):
        assert _cabi.lib().sg2_set_chunk_len(cl) == 0
        case = Sg2Case(shapes, seed=cl, random_state=True)
        w = _run_steps(case, 3, chunk_len=cl, sharp=True, lamb_eff=2.0, wd_eff=4.5)
        print("chunk", cl, "worst tolerance ratios", w)


def test_windowed_summaries_accept_and_fall_back():
    """Window 64 on chunks of 256: the first block is accepted with the N(0,0.1) weights; with barely contracting
    poles (A_log = -12) no block passes the 2^-100 test and the walk covers the whole chunk."""
    from grokking_optimizers import _cabi
    shapes = [(3000,), (64, 65), (700,)]
    assert _cabi.lib().sg2_set_chunk_len(256) == 0 and _cabi.lib().sg2_set_scan_window(64) == 0
    case = Sg2Case(shapes, seed=21, random_state=True)
    print("window accepted", _run_steps(case, 2, chunk_len=256, sharp=True, lamb_eff=2.0))
    W = wl.meta_weights(7)
    for base in (2, 11):
        W[base + 5].fill_(-12.0)
    case = Sg2Case(shapes, seed=22, random_state=True, weights=W)
    print("window rejected", _run_steps(case, 2, chunk_len=256, sharp=True, lamb_eff=2.0))
    assert _cabi.lib().sg2_set_scan_window(0) == 0
    case = Sg2Case(shapes, seed=23, random_state=True)
    print("window off", _run_steps(case, 1, chunk_len=256))


@pytest.mark.parametrize("seed", [0, 1, 2])
def test_module_initialised_weights_over_several_chunks(seed):
    """The optimizer's own initial meta-net (A_log = log(1..16), default Linear weights: poles with dt*|A|/2 > 1,
    i.e. negative A_bar, and columns whose 256-step window has not contracted) on tensors of several chunks, with
    gradients of order one so that dt varies along the sequence; chunk lengths 1024 (automatic) and 512."""
    from grokking_optimizers import _cabi
    shapes = [(9000,), (64, 130), (3000,), (700,)]
    W = wl.module_weights(seed)
    for cl in (None, 512):
        assert _cabi.lib().sg2_set_chunk_len(cl or 0) == 0
        case = Sg2Case(shapes, seed=30 + seed, random_state=True, weights=W)
        w = _run_steps(case, 2, chunk_len=cl, sharp=True, lamb_eff=2.0, wd_eff=4.5, grad_std=0.5 if cl else 1e-3)
        print("module weights seed", seed, "chunk", cl, "worst tolerance ratios", w)


def test_adaptive_window_needs_several_blocks():
    """A_log = log(1..16) with dt about 1.7: |A_bar| of the fast poles is close to 1 again, a 64-step block does not
    contract to 2^-100 and the summary walk has to go back several blocks (device and checker must stop at the same
    block: the results are bit-identical or the comparison of the contexts fails)."""
    from grokking_optimizers import _cabi
    shapes = [(3000,), (64, 65)]
    W = wl.meta_weights(7)
    for base in (2, 11):
        W[base + 5].copy_(torch.log(torch.arange(1, 17, dtype=torch.float32))[None, :].expand(16, 16))
        W[base + 2].fill_(1.5)
    assert _cabi.lib().sg2_set_chunk_len(512) == 0 and _cabi.lib().sg2_set_scan_window(64) == 0
    case = Sg2Case(shapes, seed=41, random_state=True, weights=W)
    print("several blocks", _run_steps(case, 2, chunk_len=512, sharp=True, lamb_eff=2.0))


def test_contracted_summaries_forget_a_finite_carried_state_only():
    """With every chunk summary contracted to (0, b) the replay takes the start state of chunk c from summary c - 1 and
    never reads what came before: the contexts of all later chunks and the new carried state are the same, bit for
    bit, whether the tensor carried in a small state or a huge finite one.  A carried state that is NOT finite switches
    that shortcut off for the call and is multiplied through: every context of that tensor and direction comes out
    non-finite, as in the reference, while the other tensors of the call keep their values bit for bit."""
    from grokking_optimizers import _cabi
    shapes, cl = [(3000,), (700,), (256,)], 256
    assert _cabi.lib().sg2_set_chunk_len(cl) == 0
    ctx, fwd, perm = [], [], None
    for poison in ("none", "huge", "inf"):
        case = Sg2Case(shapes, seed=5, random_state=True)
        if poison == "huge":
            case.gpu[0]["mamba_fwd"].fill_(3.0e30)
            case.gpu[1]["mamba_bwd"].fill_(-3.0e30)
        if poison == "inf":
            case.gpu[0]["mamba_fwd"].fill_(float("inf"))
        grads = wl.make_grads(shapes, seed=77)
        sharps = [torch.zeros_like(g) for g in grads]
        print("carried state:", poison, flush=True)
        case.gpu_step(grads, sharps, per_tensor_scalars(case.P, 1, 2.0), shared_scalars(4.5))
        ctx.append(case.step_fn.ctx.cpu().numpy().copy())
        fwd.append([case.gpu[i][k].cpu().numpy().copy() for i in range(case.P) for k in ("mamba_fwd", "mamba_bwd")])
        perm = case.step_fn.perm.cpu().numpy()
        if poison == "inf":          # the checker makes the same statement, value for value where values are finite
            for st in case.np[:1]:
                st["mamba_fwd"][:] = np.inf
            dbg = case.oracle_step(grads, sharps, per_tensor_scalars(case.P, 1, 2.0), shared_scalars(4.5), cl)
            for i in range(case.P):
                a, b = int(case.offsets[i]), int(case.offsets[i + 1])
                for d in range(2):
                    assert np.array_equal(np.isfinite(ctx[-1][d, a:b]), np.isfinite(dbg[i]["ctx"][d]))
                    ok = np.isfinite(dbg[i]["ctx"][d])
                    assert np.array_equal(ctx[-1][d, a:b][ok], dbg[i]["ctx"][d][ok])
    n0, o1, n1 = 3000, 3000, 700
    later0 = perm[:n0][cl:]                       # tensor 0, forward direction: scan steps >= one chunk
    assert np.isfinite(ctx[1][0, later0]).all() and np.array_equal(ctx[0][0, later0], ctx[1][0, later0])
    assert not np.array_equal(ctx[0][0, perm[:n0][:cl]], ctx[1][0, perm[:n0][:cl]])
    later1 = o1 + perm[o1:o1 + n1][:n1 - cl]      # tensor 1, backward direction
    assert np.array_equal(ctx[0][1, later1], ctx[1][1, later1])
    first1 = o1 + perm[o1:o1 + n1][n1 - cl:]
    assert not np.array_equal(ctx[0][1, first1], ctx[1][1, first1])
    for a, b in zip(fwd[0], fwd[1]):              # every new carried state comes from a last chunk
        assert np.isfinite(b).all() and np.array_equal(a, b)
    # the infinite state: tensor 0's forward contexts all non-finite, its new forward state too; everything else as without it
    assert (~np.isfinite(ctx[2][0, :n0]).all(axis=-1)).all() and not np.isfinite(fwd[2][0]).all()
    assert np.array_equal(ctx[0][1], ctx[2][1]) and np.array_equal(ctx[0][0, n0:], ctx[2][0, n0:])
    for k in range(1, len(fwd[0])):
        assert np.array_equal(fwd[0][k], fwd[2][k])


def test_three_hundred_tensors_in_one_call():
    """300 tensors of 0 .. 900 elements in one call (the per-call tables travel in 13 launches of 24 records each),
    chunk length 256 so that the larger ones have several chunks; two steps against the checker.  Then the same call
    with a carried state of tensor 211 made infinite: the flag that switches the contracted-summary shortcut off is
    raised by a later table launch than the first, that tensor's forward contexts come out non-finite and every other
    tensor's values stay what they were, bit for bit."""
    from grokking_optimizers import _cabi
    r = np.random.RandomState(4)
    shapes = [(int(n),) for n in r.randint(0, 900, size=300)]
    shapes[17] = (0,)
    cl = 256
    assert _cabi.lib().sg2_set_chunk_len(cl) == 0
    case = Sg2Case(shapes, seed=12, random_state=True)
    w = _run_steps(case, 2, chunk_len=cl, sharp=True, lamb_eff=2.0)
    print("300 tensors: worst tolerance ratios", w, flush=True)
    assert shapes[211][0] > cl
    ctx = []
    for poison in (False, True):
        case = Sg2Case(shapes, seed=12, random_state=True)
        if poison:
            case.gpu[211]["mamba_fwd"][3, 5] = float("inf")
        grads = wl.make_grads(shapes, seed=78)
        case.gpu_step(grads, [torch.zeros_like(g) for g in grads], per_tensor_scalars(case.P, 1, 2.0), shared_scalars(4.5))
        ctx.append(case.step_fn.ctx.cpu().numpy().copy())
    a, b = int(case.offsets[211]), int(case.offsets[212])
    assert not np.isfinite(ctx[1][0, a:b]).all(axis=-1).any()
    assert np.isfinite(ctx[0]).all() and np.isfinite(ctx[1][1]).all()
    keep = np.ones(ctx[0].shape[1], bool)
    keep[a:b] = False
    assert np.array_equal(ctx[0][:, keep], ctx[1][:, keep]) and np.array_equal(ctx[0][1], ctx[1][1])


def test_saturated_gates_take_the_plain_forms():
    """The scan's output gates, the GRU gates and the GRU candidates are formed with one shared reciprocal per group
    unless the product of the group's denominators is too large; then every value of the group takes the plain
    form.  Weights that saturate some elements' gates and not others put both forms, and lanes of one wave on
    different ones, through the device and the checker: any difference in the decision shows as a mismatch."""
    shapes = [(2500,), (64, 33), (700,)]
    W = wl.meta_weights(7)
    for base in (2, 11):
        W[base][16:, :] *= 1000.0             # z half of in_proj: gate pre-activations of order +-30
    W[20][:, 0] = 60.0                        # W_z, W_r, W_h: the gradient itself drives the GRU gates
    W[22][:, 0] = -45.0
    W[24][:, 0] = 30.0
    case = Sg2Case(shapes, seed=77, random_state=True, weights=W)
    w = _run_steps(case, 2, chunk_len=None, sharp=True, lamb_eff=2.0, wd_eff=4.5, grad_std=1.0)
    print("saturated gates: worst tolerance ratios", w)
    assert all(v == 0.0 for v in w.values()), w        # identical arithmetic on both sides: not one bit differs


def test_routing_spread_over_most_experts():
    """The query rows that read the GRU state amplified 30 times, on random GRU states (what the benchmark's
    spread-routing variant times): the lanes of a wave pick different experts, so the expert records are gathered per
    lane instead of broadcast.  Indices and counts bit for bit against the checker, with most of the 144 experts in
    use."""
    W = wl.meta_weights(7)
    W[26][:, :, :4] *= 30.0
    case = Sg2Case([(20000,), (64, 130), (3, 4096), (257,)], seed=31, weights=W, random_state=True)
    for st_cpu, st_gpu, st_np in zip(case.cpu, case.gpu, case.np):       # GRU states of unit scale
        st_cpu["gru"].mul_(1.0 / 0.3)
        st_gpu["gru"].mul_(1.0 / 0.3)
        st_np["gru"] *= np.float32(1.0 / 0.3)
        assert np.array_equal(st_np["gru"], st_gpu["gru"].cpu().numpy())
    w = _run_steps(case, 2, chunk_len=None, sharp=True, lamb_eff=2.0)
    used = int((case.counts_gpu > 0).sum())
    print("spread routing: experts in use", used, "worst tolerance ratios", w, flush=True)
    assert used >= 100


def test_shared14_one_step_default_chunk():
    """The 14-tensor, 420 195-element transformer parameter set, default chunk length."""
    case = Sg2Case(wl.shared14_shapes(), seed=0)
    w = _run_steps(case, 2, chunk_len=None)
    print("worst tolerance ratios", w)
    assert int(case.counts_gpu.sum()) == 2 * 4 * 420195


def test_edge_cases():
    """Empty tensor, N=1, all-zero grads, huge grads, NaN/Inf grads, fp16 and bf16 parameters."""
    shapes = [(0,), (1,), (300,), (300,), (300,), (1500,), (1500,)]
    dtypes = [torch.float32] * 5 + [torch.float16, torch.bfloat16]
    case = Sg2Case(shapes, dtypes=dtypes, seed=5, random_state=True)
    for t in range(1, 3):
        grads = wl.make_grads(shapes, seed=40 + t)
        grads[2].zero_()
        grads[3].fill_(1e6)
        grads[4][::17] = float("nan")
        grads[4][5::31] = float("inf")
        grads[4][7::29] = float("-inf")
        sharps = [g.abs() for g in wl.make_grads(shapes, seed=60 + t)]
        pt, sh = per_tensor_scalars(case.P, t, 2.0), shared_scalars(4.5)
        print("edge step", t, flush=True)
        case.gpu_step(grads, sharps, pt, sh)
        dbg = case.oracle_step(grads, sharps, pt, sh, None)
        case.compare(dbg, REL, FLOOR)
    for st in case.gpu:
        for k, v in st.items():
            assert torch.isfinite(v.float()).all(), k


def test_wide_dynamic_range_gradients():
    """|g| log-uniform over 1e-6 .. 1e5: the largest step sizes overflow the product of A_bar denominators of an
    8-step block, so the sorted sequence mixes blocks that share one reciprocal with blocks that fall back to
    the per-step form; device and checker have to take the same decision for every block."""
    shapes = [(3000,), (700,), (64, 130)]
    case = Sg2Case(shapes, seed=11)
    r = np.random.RandomState(5)
    for t in range(1, 3):
        grads = [torch.from_numpy((10.0 ** r.uniform(-6, 5, size=int(np.prod(s)))
                                   * r.choice([-1.0, 1.0], size=int(np.prod(s)))).astype(np.float32)).reshape(s) for s in shapes]
        sharps = [torch.zeros_like(g) for g in grads]
        pt, sh = per_tensor_scalars(case.P, t, 0.0), shared_scalars(1.0)
        print("wide range step", t, flush=True)
        case.gpu_step(grads, sharps, pt, sh)
        print("worst tolerance ratios", case.compare(case.oracle_step(grads, sharps, pt, sh, None), REL, FLOOR))


def test_heavy_ties_sort_is_stable():
    """Quantised gradients: thousands of exact ties; permutation must equal the stable argsort."""
    shapes = [(20000,), (9000,)]
    case = Sg2Case(shapes, seed=9)
    grads = [torch.round(g * 2e4) / 2e4 for g in wl.make_grads(shapes, seed=77, std=1e-3)]
    sharps = [torch.zeros_like(g) for g in grads]
    pt, sh = per_tensor_scalars(case.P, 1), shared_scalars()
    case.gpu_step(grads, sharps, pt, sh)
    perm = case.step_fn.perm.cpu().numpy()
    for i, g in enumerate(grads):
        a, b = int(case.offsets[i]), int(case.offsets[i + 1])
        want = np.argsort(np.abs(g.numpy()), kind="stable").astype(np.int32)
        assert np.array_equal(perm[a:b], want)


def test_per_call_scan_options_leave_the_process_settings_alone():
    """Two call plans with their own chunk length and summary window (sg2_batched_step_opt), stepped alternately in one
    process: each matches the checker run with ITS decomposition, and the process-wide settings stay at their defaults."""
    from grokking_optimizers import _cabi
    lib = _cabi.lib()
    shapes = [(3000,), (64, 65), (700,)]
    a = Sg2Case(shapes, seed=51, random_state=True, chunk_len=64, scan_window=0)
    b = Sg2Case(shapes, seed=52, random_state=True, chunk_len=256, scan_window=64)
    for t in (1, 2):
        for case, cl, win in ((a, 64, 0), (b, 256, 64)):
            grads = wl.make_grads(shapes, seed=60 + t)
            sharps = [g.abs() * 0.5 for g in wl.make_grads(shapes, seed=560 + t)]
            pt, sh = per_tensor_scalars(case.P, t, 2.0), shared_scalars(4.5)
            case.gpu_step(grads, sharps, pt, sh)
            dbg = case.oracle_step(grads, sharps, pt, sh, cl, window=win)
            print("options", cl, win, "step", t, case.compare(dbg, REL, FLOOR), flush=True)
    assert lib.sg2_get_chunk_len() == 0 and lib.sg2_get_scan_window() == 64
    with pytest.raises(RuntimeError, match="multiple of 64"):
        Sg2Case(shapes, seed=53, chunk_len=100)


def test_rejects_unsupported_dims_and_small_workspace():
    from grokking_optimizers import _cabi
    import ctypes as C
    d = dict(DIMS, d_state=15)
    with pytest.raises(RuntimeError, match="d_state must be even"):
        _cabi.workspace_bytes([10], d)
    d = dict(DIMS, d_model=18)
    with pytest.raises(RuntimeError, match="MAX_D_MODEL"):
        _cabi.workspace_bytes([10], d)
    assert _cabi.workspace_bytes([10], dict(DIMS, d_model=4, d_state=8, d_inner=8)) > 0      # runs embedded in (8, 16, 16)
    case = Sg2Case([(100,)], seed=1)
    case.step_fn.workspace = torch.empty(256, dtype=torch.uint8, device="cuda")
    g = [torch.zeros(100)]
    with pytest.raises(RuntimeError, match="workspace too small"):
        case.gpu_step(g, g, per_tensor_scalars(1, 1), shared_scalars())
