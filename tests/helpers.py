"""Shared helpers for the test-suite: state construction and comparisons."""
import numpy as np
import torch

import workloads as wl

DIMS = dict(wl.DEFAULT_DIMS)


def default_scalars(i=0, step=1, lamb_eff=0.0, wd_eff=1.0, rescale=0.1):
    beta1 = 0.9 * (0.9 ** i)
    return dict(alpha=0.98, lamb_eff=lamb_eff, beta1=beta1, bc1=1.0 - beta1 ** step,
                bc2=1.0 - 0.999 ** step, rescale=rescale, beta2=0.999, lr=1e-3, wd_eff=wd_eff, eps=1e-8)


def f32_scalars(sc):
    """Round every scalar to fp32 (what crosses the extension boundary)."""
    return {k: float(np.float32(v)) for k, v in sc.items()}


def fresh_state_np(param, dims=DIMS):
    n = param.size
    return dict(param=np.ascontiguousarray(param.reshape(-1).astype(np.float32)).copy(),
                exp_avg=np.zeros(n, np.float32), exp_avg_sq=np.zeros(n, np.float32),
                mu=np.zeros(n, np.float32), gru=np.zeros((n, dims["gru_hidden"]), np.float32),
                mamba_fwd=np.zeros((dims["d_inner"], dims["d_state"]), np.float32),
                mamba_bwd=np.zeros((dims["d_inner"], dims["d_state"]), np.float32))


def random_state_np(n, seed, dims=DIMS):
    """A mid-training looking state: non-zero moments, GRU and Mamba carries."""
    r = np.random.RandomState(seed)
    return dict(param=(r.randn(n) * 0.02).astype(np.float32),
                exp_avg=(r.randn(n) * 1e-3).astype(np.float32),
                exp_avg_sq=(r.rand(n) * 1e-6).astype(np.float32),
                mu=(r.randn(n) * 1e-3).astype(np.float32),
                gru=(r.randn(n, dims["gru_hidden"]) * 0.3).astype(np.float32),
                mamba_fwd=(r.randn(dims["d_inner"], dims["d_state"]) * 0.1).astype(np.float32),
                mamba_bwd=(r.randn(dims["d_inner"], dims["d_state"]) * 0.1).astype(np.float32))


def copy_state(st):
    return {k: (v.copy() if isinstance(v, np.ndarray) else v) for k, v in st.items()}


def rel_close(a, b, rel=1e-4, floor=1e-7):
    """|a-b| <= rel*max(|a|,|b|) + floor, elementwise; returns (ok, worst excess ratio)."""
    a = np.asarray(a, np.float64)
    b = np.asarray(b, np.float64)
    tol = rel * np.maximum(np.abs(a), np.abs(b)) + floor
    d = np.abs(a - b)
    ratio = float((d / tol).max()) if d.size else 0.0
    return ratio <= 1.0, ratio


def weights_np(seed=7, dims=None, std=0.1):
    return [w.numpy() for w in wl.meta_weights(seed, dims, std)]
