"""GPU parity of the remaining fused steps (SuperGrok v1.1, GrokAdamW, NeuralGrok,
Prodigy, Lion, LookSAM) through the `_ops` extension: against the golden
vectors of the reference's own CPU code (tests/golden/ref_family.npz) and, on
larger multi-tile tensors and 16-bit parameters, against oracle/family_oracle.py.
Tolerance: |a-b| <= 1e-4*max(|a|,|b|) + 1e-7 on every state tensor."""
import numpy as np
import pytest
import torch

import family_cases as fc
from helpers import rel_close
from oracle import family_oracle as fo

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _ops():
    from grokking_optimizers import _ops
    return _ops


def _up(arrs, dtype=torch.float32):
    return [torch.from_numpy(np.ascontiguousarray(a)).to(DEV).to(dtype) for a in arrs]


def _down(tensors, arrs):
    for t, a in zip(tensors, arrs):
        a[...] = t.float().cpu().numpy()


def _wrap(name, n_lists, weights_at=None):
    """numpy-in/numpy-out adapter with the checker's signature around an `_ops` function whose first
    n_lists arguments are tensor lists (updated in place)."""
    def fn(*args):
        lists = [_up(a) for a in args[:n_lists]]
        rest = list(args[n_lists:])
        if weights_at is not None:
            for k in range(weights_at, weights_at + 4):
                rest[k] = torch.from_numpy(np.ascontiguousarray(rest[k])).to(DEV)
        out = getattr(_ops(), name)(*lists, *rest)
        torch.cuda.synchronize()
        for tl, al in zip(lists, args[:n_lists]):
            _down(tl, al)
        return out
    return fn


def gpu_grokadamw(p, g, ea, easq, ema, steps, *sc):
    return _wrap("grokadamw_fused_step", 5)(p, g, ea, easq, ema, steps, *sc)


def gpu_neuralgrok(p, g, ea, easq, steps, W1, b1, W2, b2, alpha_amp, beta_amp, *sc):
    return _wrap("neuralgrok_fused_step", 4, weights_at=1)(p, g, ea, easq, steps, W1, b1, W2, b2, alpha_amp, beta_amp, int(b1.size), *sc)


def gpu_prodigy(p, g, ea, easq, s, p0, steps, d_lr, *sc):
    return _wrap("prodigy_fused_step", 6)(p, g, ea, easq, s, p0, steps, d_lr, *sc)


def gpu_lion(p, g, ea, *sc):
    return _wrap("lion_fused_step", 3)(p, g, ea, *sc)


def gpu_sg11(p, g, ea, easq, mu, sh, steps, alphas, beta1s, W1, b1, W2, b2, rescale, *sc):
    return _wrap("supergrok11_fused_step", 6, weights_at=3)(p, g, ea, easq, mu, sh, steps, alphas, beta1s, W1, b1, W2, b2, rescale,
                                                            int(b1.size), *sc)


def gpu_perturb(p, g, rho):
    tp, tg = _up(p), _up(g)
    backups = _ops().looksam_perturb_all(tp, tg, rho)
    torch.cuda.synchronize()
    for b, a in zip(backups, p):
        assert np.array_equal(b.cpu().numpy(), a)
    _down(tp, p)
    tp2 = [t.clone() for t in tp]
    _ops().looksam_restore_all(tp2, backups)
    for t, b in zip(tp2, backups):
        assert torch.equal(t, b)


def gpu_directions(v, sam_g, g):
    return _wrap("looksam_compute_directions", 3)(v, sam_g, g)


def gpu_adjust(g, v, la):
    return _wrap("looksam_adjust_grads", 2)(g, v, la)


def test_golden_grokadamw():
    fc.run_grokadamw(gpu_grokadamw)


def test_golden_neuralgrok():
    fc.run_neuralgrok(gpu_neuralgrok)


def test_golden_prodigy():
    fc.run_prodigy(gpu_prodigy)


def test_golden_lion():
    fc.run_lion(gpu_lion)


def test_golden_sg11():
    fc.run_sg11(gpu_sg11)


def test_golden_looksam():
    fc.run_looksam(gpu_perturb, gpu_directions, gpu_adjust)


SIZES = [9000, 1, 4096, 33, 70001]     # several tiles per tensor, tile-aligned and ragged


def _rand(seed, std):
    r = np.random.RandomState(seed)
    return [(r.randn(n) * std).astype(np.float32) for n in SIZES]


def _cmp(tag, got, want, rel=1e-4, floor=1e-7):
    for i, (a, b) in enumerate(zip(got, want)):
        ok, worst = rel_close(a, b, rel, floor)
        assert ok, (tag, i, worst)


def _both(run_gpu, run_cpu, state):
    """state: dict name -> list of arrays; both runners update their own copy in place"""
    a = {k: [x.copy() for x in v] for k, v in state.items()}
    b = {k: [x.copy() for x in v] for k, v in state.items()}
    ra, rb = run_gpu(a), run_cpu(b)
    for k in state:
        _cmp(k, a[k], b[k])
    return ra, rb


def test_multi_tile_against_checker():
    P = len(SIZES)
    for t in range(1, 3):
        st = dict(p=_rand(1, 0.02), g=_rand(10 + t, 0.05 if t == 2 else 1e-3), ea=_rand(2, 1e-3), easq=[np.abs(x) * 1e-3 for x in _rand(3, 1e-3)],
                  ema=_rand(4, 1e-3))
        sc = (0.98, 5.0, 0.9, 0.98, 1e-3, 1.0, 1e-8, 1.0)
        _both(lambda s: gpu_grokadamw(s["p"], s["g"], s["ea"], s["easq"], s["ema"], [t] * P, *sc),
              lambda s: fo.grokadamw_step(s["p"], s["g"], s["ea"], s["easq"], s["ema"], [t] * P, *sc), st)
    r = np.random.RandomState(7)
    H = 128
    W = [(r.randn(H, 1) * 0.5).astype(np.float32), (r.randn(H) * 0.1).astype(np.float32), (r.randn(1, H) * 0.1).astype(np.float32),
         (r.randn(1) * 0.1).astype(np.float32)]
    st = dict(p=_rand(1, 0.02), g=_rand(11, 1e-3), ea=_rand(2, 1e-3), easq=[np.abs(x) * 1e-3 for x in _rand(3, 1e-3)])
    sc = (10.0, 4.0, 0.9, 0.98, 1e-3, 1.0, 1e-8, 1.0)
    _both(lambda s: gpu_neuralgrok(s["p"], s["g"], s["ea"], s["easq"], [3] * P, *W, *sc),
          lambda s: fo.neuralgrok_step(s["p"], s["g"], s["ea"], s["easq"], [3] * P, *W, *sc), st)
    st = dict(p=_rand(1, 0.02), g=_rand(12, 1e-2), ea=_rand(2, 1e-3), easq=[np.abs(x) * 1e-3 for x in _rand(3, 1e-3)],
              s=[np.abs(x) for x in _rand(5, 1e-4)], p0=_rand(6, 0.02))
    sc = (0.9, 0.999, 1e-3, 0.01, 1e-8)
    ra, rb = _both(lambda s: gpu_prodigy(s["p"], s["g"], s["ea"], s["easq"], s["s"], s["p0"], [2] * P, 1e-3, *sc),
                   lambda s: fo.prodigy_step(s["p"], s["g"], s["ea"], s["easq"], s["s"], s["p0"], [2] * P, 1e-3, *sc), st)
    assert abs(ra - rb) <= 1e-4 * abs(rb), (ra, rb)
    st = dict(p=_rand(1, 0.02), g=_rand(13, 1e-3), ea=_rand(2, 1e-3))
    _both(lambda s: gpu_lion(s["p"], s["g"], s["ea"], 1e-4, 0.9, 0.99, 3.0), lambda s: fo.lion_step(s["p"], s["g"], s["ea"], 1e-4, 0.9, 0.99, 3.0), st)
    H = 32
    W = [(r.randn(H, 2) * 0.5).astype(np.float32), (r.randn(H) * 0.1).astype(np.float32), (r.randn(1, H) * 0.5).astype(np.float32),
         (r.randn(1) * 0.1).astype(np.float32)]
    st = dict(p=_rand(1, 0.02), g=_rand(14, 1e-3), ea=_rand(2, 1e-3), easq=[np.abs(x) * 1e-3 for x in _rand(3, 1e-3)], mu=_rand(8, 1e-3),
              sh=[np.abs(x) for x in _rand(9, 1e-3)])
    alphas, beta1s = [0.98] * P, [0.9 * 0.9 ** i for i in range(P)]
    sc = (0.1, 0.999, 1e-3, 1.0, 1e-8, 5.0, 0.7, 5.0, 1.0)
    _both(lambda s: gpu_sg11(s["p"], s["g"], s["ea"], s["easq"], s["mu"], s["sh"], [4] * P, alphas, beta1s, *W, *sc),
          lambda s: fo.sg11_step(s["p"], s["g"], s["ea"], s["easq"], s["mu"], s["sh"], [4] * P, alphas, beta1s, *W, *sc), st)
    st = dict(v=_rand(20, 1.0), sg=_rand(21, 1e-3), g=_rand(22, 1e-3))
    _both(lambda s: gpu_directions(s["v"], s["sg"], s["g"]), lambda s: fo.looksam_directions(s["v"], s["sg"], s["g"]), st)
    st = dict(g=_rand(22, 1e-3), v=_rand(20, 1.0))
    _both(lambda s: gpu_adjust(s["g"], s["v"], 0.7), lambda s: fo.looksam_adjust(s["g"], s["v"], 0.7), st)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_16bit_parameters(dtype):
    """16-bit params/grads with fp32 state: the step must equal the fp32 checker run on the widened
    inputs, up to the rounding of the stored parameter (half an ulp of the 16-bit type)."""
    ops = _ops()
    ulp = 2.0 ** -8 if dtype == torch.bfloat16 else 2.0 ** -11
    p32 = [x for x in _rand(1, 0.02)]
    g32 = [x for x in _rand(15, 1e-3)]
    tp, tg = _up(p32, dtype), _up(g32, dtype)
    pw, gw = [t.float().cpu().numpy() for t in tp], [t.float().cpu().numpy() for t in tg]
    ea, easq, ema = ([np.zeros_like(x) for x in pw] for _ in range(3))
    tea, teasq, tema = _up(ea), _up(easq), _up(ema)
    sc = (0.98, 5.0, 0.9, 0.98, 1e-3, 1.0, 1e-8, 0.0)
    ops.grokadamw_fused_step(tp, tg, tea, teasq, tema, [1] * len(SIZES), *sc)
    fo.grokadamw_step(pw, gw, ea, easq, ema, [1] * len(SIZES), *sc)
    torch.cuda.synchronize()
    _cmp("ea", [t.cpu().numpy() for t in tea], ea)
    _cmp("ema", [t.cpu().numpy() for t in tema], ema)
    for a, b in zip(tp, pw):
        assert np.all(np.abs(a.float().cpu().numpy() - b) <= ulp * np.abs(b) + 1e-7)
    tp, tea2 = _up(p32, dtype), _up([np.zeros_like(x) for x in pw])
    pw = [t.float().cpu().numpy() for t in tp]
    ea2 = [np.zeros_like(x) for x in pw]
    ops.lion_fused_step(tp, tg, tea2, 1e-4, 0.9, 0.99, 3.0)
    fo.lion_step(pw, gw, ea2, 1e-4, 0.9, 0.99, 3.0)
    torch.cuda.synchronize()
    _cmp("lion m", [t.cpu().numpy() for t in tea2], ea2)
    for a, b in zip(tp, pw):
        assert np.all(np.abs(a.float().cpu().numpy() - b) <= ulp * np.abs(b) + 1e-7)


def test_errors_and_empty_inputs():
    ops = _ops()
    ops.lion_fused_step([], [], [], 1e-4, 0.9, 0.99, 3.0)
    p = [torch.zeros(5, device=DEV)]
    ops.lion_fused_step(p, [torch.Tensor()], [torch.zeros(5, device=DEV)], 1e-4, 0.9, 0.99, 3.0)      # no gradient: skipped
    with pytest.raises(RuntimeError):
        ops.lion_fused_step([torch.zeros(5)], [torch.zeros(5)], [torch.zeros(5)], 1e-4, 0.9, 0.99, 3.0)   # CPU tensors
    with pytest.raises(RuntimeError):
        ops.grokadamw_fused_step(p, [torch.ones(5, device=DEV)], [torch.zeros(5, device=DEV)], [torch.zeros(5, device=DEV)],
                                 [torch.zeros(5, device=DEV)], [0], 0.98, 5.0, 0.9, 0.98, 1e-3, 1.0, 1e-8, 1.0)   # step 0: bc = 0
