"""TEST INFRASTRUCTURE ONLY.  numpy restatement of the Muon step of the
reference (csrc/ops.cpp:663-746): buf = momentum*buf + g; X = buf/(||buf||_F +
1e-7); ns_steps times { A = X X^T; X = a X + b A X + c A (A X) } with
(a,b,c) = (3.4445, -4.7750, 2.0315), computed in the dtype handed in (float32
reproduces the reference's fp32 iteration, float64 is the mathematical
answer); p = (p + neg_lr_scale * X.to(p.dtype)) * (1 - lr*wd) with
neg_lr_scale = -lr * (0.2*sqrt(max_dim)) / sqrt(max_dim).

Parity status: pinned in this container against the reference's own CPU code
compiled from its sources (oracle/_ref) in tests/test_oracle_elem.py, and by
the fixed-point properties of the iteration (singular values pulled into
[0.7, 1.2])."""
import numpy as np

NS_A, NS_B, NS_C = 3.4445, -4.7750, 2.0315


def newton_schulz(X, ns_steps, dtype=np.float32):
    X = X.astype(dtype)
    a, b, c = dtype(NS_A), dtype(NS_B), dtype(NS_C)
    for _ in range(ns_steps):
        A = X @ X.T
        AX = A @ X
        X = a * X + b * AX + c * (A @ AX)
    return X


def muon_step(param, grad, buf, momentum, lr, wd, ns_steps, dtype=np.float32, round_x=None, round_mid=None,
              round_decay=None):
    """param/grad: float32 arrays holding the (possibly bf16-representable) values; buf float32, updated in
    place.  round_x: optional function applied to X before the update (e.g. rounding to bf16, the
    `X.to(p.dtype)` of the reference's GPU branch, csrc/ops.cpp:738).  round_mid: optional rounding applied
    between `p += neg*X` and `p *= decay` (the reference's CPU branch, csrc/ops.cpp:741-742, rounds a
    16-bit parameter after each in-place op; its GPU kernel rounds once).  round_decay: optional rounding of
    the decay factor itself (ATen's in-place `mul_` of a bf16 tensor by a C++ float multiplies by the scalar
    rounded to bf16; observed on the reference's CPU build).  Returns (new_param float32, X)."""
    buf *= np.float32(momentum)
    buf += grad
    norm = np.float32(np.sqrt(np.sum(buf.astype(np.float64) ** 2))) + np.float32(1e-7)
    X = newton_schulz(buf * (np.float32(1.0) / norm), ns_steps, dtype)
    Xp = X.astype(np.float32)
    if round_x is not None:
        Xp = round_x(Xp)
    max_dim = np.float32(max(param.shape))
    scale = np.float32(0.2) * np.sqrt(max_dim)
    neg = -np.float32(lr) * scale / np.sqrt(max_dim)
    decay = np.float32(1.0) - np.float32(lr) * np.float32(wd)
    if round_decay is not None:
        decay = np.float32(round_decay(np.array([decay], np.float32))[0])
    mid = (param + neg * Xp).astype(np.float32)
    if round_mid is not None:
        mid = round_mid(mid)
    return (mid * decay).astype(np.float32), X
