"""Seeded sweep of the v2 batched step over the sizes where its tilings change (1, 63..65, 255..257, 1023..1025,
4095..4097, 8191..8193 elements: wave, scan tile, element tile, scan chunk, sort tile), parameter dtypes, chunk lengths,
summary windows, both geometries, and - per tensor - an all-zero or a populated sharpness (the kernels skip the
sharpness of tensors whose cache is all zero, so one call mixes both kinds).  Every case: two steps against the CPU
checker, integers bit-exact, floats within 1e-4 relative."""
import numpy as np
import pytest
import torch

import workloads as wl
from sg2_harness import Sg2Case, per_tensor_scalars, shared_scalars

pytestmark = pytest.mark.gpu

SIZES = [1, 63, 64, 65, 255, 256, 257, 1023, 1024, 1025, 4095, 4096, 4097, 8191, 8192, 8193, 12289, 0]
LARGE = dict(wl.DEFAULT_DIMS, d_model=16, d_state=32, d_inner=32)


@pytest.fixture(autouse=True)
def _default_knobs():
    from grokking_optimizers import _cabi
    yield
    _cabi.lib().sg2_set_chunk_len(0)
    _cabi.lib().sg2_set_scan_window(-1)


@pytest.mark.parametrize("seed", range(8))
def test_seeded_configuration(seed):
    from grokking_optimizers import _cabi
    r = np.random.RandomState(1000 + seed)
    P = int(r.randint(3, 9))
    shapes = [(int(SIZES[i]),) for i in r.choice(len(SIZES), size=P)]
    dtypes = [[torch.float32, torch.float32, torch.bfloat16, torch.float16][int(r.randint(4))] for _ in range(P)]
    chunk = [0, 64, 256, 1024][int(r.randint(4))]
    window = [-1, 0, 256][int(r.randint(3))]
    dims = LARGE if seed % 3 == 2 else None
    with_sharp = [bool(r.randint(2)) for _ in range(P)]
    print("sweep", seed, shapes, [str(d) for d in dtypes], "chunk", chunk, "window", window, "large" if dims else "default",
          "sharpness", with_sharp, flush=True)
    assert _cabi.lib().sg2_set_chunk_len(chunk) == 0 and _cabi.lib().sg2_set_scan_window(window) == 0
    case = Sg2Case(shapes, dtypes=dtypes, seed=seed, random_state=True, dims=dims)
    for t in range(1, 3):
        grads = wl.make_grads(shapes, seed=50 * seed + t, tail_frac=0.01, tail="student3")
        sharps = [(g.abs() * 0.5) if ws else torch.zeros_like(g) for g, ws in zip(wl.make_grads(shapes, seed=900 + 50 * seed + t), with_sharp)]
        pt, sh = per_tensor_scalars(case.P, t, 2.0), shared_scalars(4.5)
        case.gpu_step(grads, sharps, pt, sh)
        dbg = case.oracle_step(grads, sharps, pt, sh, chunk or None)
        print("  step", t, "worst tolerance ratios", case.compare(dbg, 1e-4, 1e-7), flush=True)
