"""GPU parity of the Muon step (bf16 MFMA Newton-Schulz behind `_ops.muon_fused_step`)
with the fp32 CPU restatement and the reference's golden vectors.

Gates: momentum buffer within 1e-4 relative; orthogonalised update within 2e-2
relative Frobenius norm of the fp32 iteration (bf16 operands, fp32 accumulation);
updated 16-bit parameters within one ulp of the stored value plus the deviation of
the update (fp32 parameters expose the update itself, checked in Frobenius norm)."""
import os

import numpy as np
import pytest
import torch

from helpers import rel_close
from oracle import muon_oracle

pytestmark = pytest.mark.gpu
GOLD = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


def _ops():
    from grokking_optimizers import _ops
    return _ops


def _bf16(a):
    return torch.from_numpy(np.ascontiguousarray(a)).to(torch.bfloat16).float().numpy()


def _run_case(shapes, dt, steps, seed, lr=0.02, wd=1.0, momentum=0.95, ns=5):
    ops = _ops()
    gen = torch.Generator().manual_seed(seed)
    p0 = [(torch.randn(*s, generator=gen) * 0.02).to(dt) for s in shapes]
    params = [p.clone().cuda() for p in p0]
    bufs = [torch.zeros(s, device="cuda") for s in shapes]
    rp = [p.float().numpy().copy() for p in p0]
    rb = [np.zeros(s, np.float32) for s in shapes]
    for t in range(steps):
        grads = [(torch.randn(*s, generator=gen) * 1e-3).to(dt) for s in shapes]
        print("muon step", t, shapes, dt, flush=True)
        ops.muon_fused_step(params, [g.cuda() for g in grads], bufs, momentum, lr, wd, ns)
        torch.cuda.synchronize()
        for i, s in enumerate(shapes):
            old = rp[i]
            new_p, X = muon_oracle.muon_step(old, grads[i].float().numpy(), rb[i], momentum, lr, wd, ns)
            ok, r = rel_close(bufs[i].cpu().numpy(), rb[i], 1e-4, 1e-7)
            assert ok, ("buf", t, i, r)
            got = params[i].float().cpu().numpy()
            # recover the applied update: p_new/decay - p_old = -0.2*lr*X
            decay = np.float32(1.0) - np.float32(lr) * np.float32(wd)
            if dt == torch.float32:
                X_gpu = (got / decay - old) / (-0.2 * lr)
                rel_f = np.linalg.norm(X_gpu - X) / np.linalg.norm(X)
                assert rel_f < 2e-2, ("X frobenius", t, i, rel_f)
                if ns >= 5:     # orthogonalised: singular values near 1 (rank-deficient shapes aside)
                    sv = np.linalg.svd(X_gpu.astype(np.float64), compute_uv=False)
                    assert sv.min() > 0.5 and sv.max() < 1.3, (sv.min(), sv.max())
            else:
                want = _bf16(new_p) if dt == torch.bfloat16 else new_p.astype(np.float16).astype(np.float32)
                # one spacing of the stored 16-bit parameter + what keeping X, the Gram matrix and the polynomial in bf16
                # between iterations costs against the checker's fp32 iteration: measured at most 2.2% of the largest
                # update entry over these cases, gated at 3% (Frobenius norm of the whole update: 2e-2, above)
                ulp = np.maximum(np.abs(want), np.abs(got)) * (2.0 ** -7 if dt == torch.bfloat16 else 2.0 ** -10)
                tol = ulp + 0.03 * 0.2 * lr * np.abs(X).max() + 1e-12
                nd = np.abs(got - want) / tol
                need = (np.maximum(np.abs(got - want) - ulp, 0.0) / (0.2 * lr * np.abs(X).max())).max()
                print("  bf16 NS deviation beyond one spacing, in units of the largest update entry: %.4f" % need, flush=True)
                assert nd.max() <= 1.0, ("param tolerance", t, i, nd.max())
                # keep the fp32 trajectory of the checker aligned with the 16-bit parameters of the device
                new_p = got
            rp[i] = got if dt != torch.float32 else new_p
            if dt == torch.float32:
                params[i].copy_(torch.from_numpy(new_p).cuda())      # re-sync so the next step starts identical


def test_small_shapes_all_dtypes():
    shapes = [(24, 40), (40, 24), (16, 16), (130, 70), (1, 5)]
    for dt in (torch.float32, torch.bfloat16, torch.float16):
        _run_case(shapes, dt, 2, seed=1)


def test_iteration_counts_zero_to_three():
    """ns_steps = 0 (the normalised momentum itself is the update: a tall matrix is then read back in its own
    orientation without any iteration having transposed it), 1, 2 and 3 (the final iterate sits in either of the two
    work buffers), wide, tall, square and padded shapes."""
    shapes = [(24, 40), (40, 24), (16, 16), (300, 70), (70, 300)]
    for ns in (0, 1, 2, 3):
        _run_case(shapes, torch.float32, 1, seed=10 + ns, ns=ns)
        _run_case(shapes, torch.bfloat16, 1, seed=20 + ns, ns=ns)


def test_reference_golden_f32():
    ops = _ops()
    z = np.load(os.path.join(GOLD, "ref_muon.npz"))
    P = int(z["n"])
    params = [torch.from_numpy(z[f"f32_p_in_{i}"]).cuda() for i in range(P)]
    bufs = [torch.zeros_like(p) for p in params]
    grads = [torch.from_numpy(z[f"f32_g_0_{i}"]).cuda() for i in range(P)]
    ops.muon_fused_step(params, grads, bufs, float(z["momentum"]), float(z["lr"]), float(z["wd"]), int(z["ns_steps"]))
    for i in range(P):
        ok, r = rel_close(bufs[i].cpu().numpy(), z[f"f32_buf_0_{i}"], 1e-4, 1e-7)
        assert ok, r
        p_in, want = z[f"f32_p_in_{i}"], z[f"f32_p_0_{i}"]
        upd_ref, upd_got = want / 0.98 - p_in, params[i].cpu().numpy() / 0.98 - p_in
        assert np.linalg.norm(upd_got - upd_ref) / np.linalg.norm(upd_ref) < 2e-2


def test_config5_sized_matrices():
    """One wide 1024x4096 and one tall 4096x1024 bf16 matrix, 5 Newton-Schulz iterations, two steps."""
    _run_case([(1024, 4096), (4096, 1024)], torch.bfloat16, 2, seed=5)
    # fp32 parameters expose the orthogonalised update itself
    _run_case([(1024, 4096)], torch.float32, 1, seed=6)


def test_class_and_errors():
    from grokking_optimizers import Muon
    ops = _ops()
    w = torch.nn.Parameter((torch.randn(64, 96) * 0.02).cuda())
    b = torch.nn.Parameter(torch.zeros(96).cuda())
    opt = Muon([w], [b], lr=0.02, weight_decay=0.0)
    for _ in range(2):
        w.grad, b.grad = torch.randn_like(w) * 1e-3, torch.randn_like(b) * 1e-3
        opt.step()
    assert opt.state[w]["momentum_buffer"].dtype == torch.float32 and "exp_avg" in opt.state[b]
    assert bool(torch.isfinite(w).all())
    with pytest.raises(RuntimeError, match="2-D"):
        ops.muon_fused_step([torch.zeros(4, device="cuda")], [torch.ones(4, device="cuda")], [torch.zeros(4, device="cuda")], 0.9, 0.1, 0.0, 5)
