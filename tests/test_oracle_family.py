"""Pins oracle/family_oracle.py (SuperGrok v1.1, GrokAdamW, NeuralGrok, Prodigy,
Lion, LookSAM) against golden vectors written by the reference's own CPU code
(tests/golden/ref_family.npz, produced by tests/golden/make_golden_ref.py from a
build of the reference's csrc/ops.cpp)."""
import family_cases as fc
from oracle import family_oracle as fo


def test_grokadamw_matches_reference_golden():
    fc.run_grokadamw(fo.grokadamw_step)


def test_neuralgrok_matches_reference_golden():
    fc.run_neuralgrok(fo.neuralgrok_step)


def test_prodigy_matches_reference_golden():
    fc.run_prodigy(fo.prodigy_step)


def test_lion_matches_reference_golden():
    fc.run_lion(fo.lion_step)


def test_sg11_matches_reference_golden():
    fc.run_sg11(fo.sg11_step)


def test_looksam_matches_reference_golden():
    fc.run_looksam(fo.looksam_perturb, fo.looksam_directions, fo.looksam_adjust)


def test_sg2_clip_against_torch_expressions():
    """grad*(clip/(norm+1e-12)) if norm > clip; then where(isfinite, grad, 0) - including NaN and Inf inputs,
    for which the order of the two statements matters (a NaN norm never clips, an Inf norm zeroes everything)."""
    import numpy as np
    import torch
    r = np.random.RandomState(3)
    cases = [r.randn(500).astype(np.float32), (r.randn(300) * 1e-3).astype(np.float32), r.randn(64).astype(np.float32),
             r.randn(64).astype(np.float32), np.zeros(10, np.float32)]
    cases[2][5] = np.nan
    cases[3][7] = np.inf
    got = fo.sg2_clip(cases, 0.5)
    for g, out in zip(cases, got):
        t = torch.from_numpy(g.copy())
        n = t.norm()
        if n > 0.5:
            t = t * (0.5 / (n + 1e-12))
        if not torch.isfinite(t).all():
            t = torch.where(torch.isfinite(t), t, torch.zeros_like(t))
        assert np.allclose(out, t.numpy(), rtol=1e-6, atol=0), (out[:4], t[:4])
    assert np.all(got[3] == 0) and got[2][5] == 0 and np.array_equal(got[1], cases[1])
