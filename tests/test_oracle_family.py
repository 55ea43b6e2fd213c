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
