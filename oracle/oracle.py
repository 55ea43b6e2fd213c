"""ctypes front end of the CPU checker (test infrastructure only).

Only tests/, the smoke check and bench.py's cpu_baseline leg import this.
The shipped package never does.
"""
import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB = os.path.join(_HERE, "_build", "liboracle.so")

DIM_NAMES = ("d_model", "d_state", "d_inner", "gru_hidden", "num_heads", "pk_dim",
             "expert_hidden", "num_experts")
DEFAULT_DIMS = dict(d_model=8, d_state=16, d_inner=16, gru_hidden=4, num_heads=4, pk_dim=12,
                    expert_hidden=16, num_experts=144)
SCALAR_NAMES = ("alpha", "lamb_eff", "beta1", "bc1", "bc2", "rescale", "beta2", "lr", "wd_eff", "eps")
DTYPE_CODE = {"float32": 0, "float16": 1, "bfloat16": 2}

_lib = None


def build():
    subprocess.check_call(["make", "-s", "-C", _HERE])


def load(path):
    """CDLL of a build of the checker with the return types set (tests also load deliberately broken builds)."""
    L = C.CDLL(path)
    for n in ("exp", "log", "softplus", "sigmoid", "silu", "tanh", "sin", "cos", "rcp_pos", "erfc", "gelu_erf", "sin_small", "cos_small", "sin_tiny", "cos_tiny",
              "gelu_sigmoid"):
        f = getattr(L, "orc_" + n)
        f.restype = C.c_float
        f.argtypes = [C.c_float]
    for f in (L.orc_silu_block, L.orc_sigmoid_block, L.orc_tanh_block):
        f.restype = None
        f.argtypes = [C.c_int, C.POINTER(C.c_float), C.POINTER(C.c_float)]
    L.orc_abar.restype = C.c_float
    L.orc_abar.argtypes = [C.c_float, C.c_float]
    for f in (L.orc_softplus_taylor, L.orc_silu_taylor):
        f.restype = C.c_float
        f.argtypes = [C.c_float, C.c_float]
    L.orc_abar_poly.restype = C.c_float
    L.orc_abar_poly.argtypes = [C.c_float, C.c_float, C.c_float]
    L.orc_sincos_poly.restype = C.c_float
    L.orc_sincos_poly.argtypes = [C.c_float, C.c_float, C.c_float, C.c_int]
    L.orc_pair_product.restype = C.c_float
    L.orc_pair_product.argtypes = [C.c_float] * 5 + [C.c_int]
    L.orc_contraction_steps.restype = C.c_int
    L.orc_contraction_steps.argtypes = [C.c_float, C.c_float, C.c_float]
    L.orc_f_to_f16.restype = C.c_uint16
    L.orc_f_to_f16.argtypes = [C.c_float]
    L.orc_f16_to_f.restype = C.c_float
    L.orc_f16_to_f.argtypes = [C.c_uint16]
    L.orc_f_to_bf16.restype = C.c_uint16
    L.orc_f_to_bf16.argtypes = [C.c_float]
    L.orc_bf16_to_f.restype = C.c_float
    L.orc_bf16_to_f.argtypes = [C.c_uint16]
    L.orc_sg2_step.restype = C.c_int
    return L


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB):
            build()
        _lib = load(_LIB)
    return _lib


def _ptr(a):
    return None if a is None else a.ctypes.data_as(C.c_void_p)


def sort_perm(g):
    """Stable ascending argsort of |g| (non-finite -> 0) as int32."""
    g = np.ascontiguousarray(g, dtype=np.float32)
    perm = np.empty(g.size, dtype=np.int32)
    lib().orc_sort_perm(_ptr(g), C.c_int64(g.size), _ptr(perm))
    return perm


def sg2_step(weights, state, grad, sharp, scalars, dims=None, precision=32, chunk_len=0, window=0,
             expert_counts=None, debug=False):
    """One SuperGrok v2 step on one tensor, in place on `state`.

    weights: list of 33 float32 arrays in _ops argument order.
    state: dict with 'param' (float32 array, or uint16 bit patterns for
      16-bit dtypes, see state['dtype']), 'exp_avg', 'exp_avg_sq', 'mu',
      'gru' [N,gh], 'mamba_fwd', 'mamba_bwd' [d_inner,d_state] float32.
    grad/sharp: arrays of the same storage type as param.
    scalars: dict over SCALAR_NAMES.
    Returns dict of debug arrays when debug=True.
    """
    L = lib()
    dims = dict(DEFAULT_DIMS if dims is None else dims)
    dm, H = dims["d_model"], dims["num_heads"]
    dtype = DTYPE_CODE[state.get("dtype", "float32")]
    N = int(state["exp_avg"].size)
    ws = [np.ascontiguousarray(w, dtype=np.float32) for w in weights]
    assert len(ws) == 33
    warr = (C.c_void_p * 33)(*[w.ctypes.data for w in ws])
    darr = np.array([dims[k] for k in DIM_NAMES], dtype=np.int32)
    sarr = np.array([scalars[k] for k in SCALAR_NAMES], dtype=np.float32)
    for k in ("param", "exp_avg", "exp_avg_sq", "mu", "gru", "mamba_fwd", "mamba_bwd"):
        assert state[k].flags["C_CONTIGUOUS"], k
    grad = np.ascontiguousarray(grad)
    sharp = np.ascontiguousarray(sharp)
    out = {}
    if debug:
        out["perm"] = np.empty(N, np.int32)
        out["expert_idx"] = np.empty((N, H), np.int32)
        out["ctx"] = np.empty((2, N, dm), np.float32)
        out["margin"] = np.empty((N, H, 2), np.float32)
        out["smart"] = np.empty(N, np.float32)
    rc = L.orc_sg2_step(
        C.c_int(precision), C.c_int64(chunk_len), C.c_int64(window), warr, _ptr(darr), C.c_int(dtype),
        _ptr(state["param"]), _ptr(grad), _ptr(sharp), _ptr(state["exp_avg"]),
        _ptr(state["exp_avg_sq"]), _ptr(state["mu"]), _ptr(state["gru"]),
        _ptr(state["mamba_fwd"]), _ptr(state["mamba_bwd"]), C.c_int64(N), _ptr(sarr),
        _ptr(expert_counts), _ptr(out.get("perm")), _ptr(out.get("expert_idx")),
        _ptr(out.get("ctx")), _ptr(out.get("margin")), _ptr(out.get("smart")))
    if rc != 0:
        raise RuntimeError("orc_sg2_step: unsupported dims (status %d)" % rc)
    return out


# ------------------------------------------------------------------ Grokfast / SuperGrok v1.5
def _f32(a):
    assert a.dtype == np.float32 and a.flags["C_CONTIGUOUS"]
    return a.ctypes.data_as(C.c_void_p)


def grokfast_ema(grad, ema, alpha, lamb):
    """In place on float32 arrays: ema update, grad <- grad + lamb*ema."""
    lib().orc_grokfast_ema(_f32(grad), _f32(ema), C.c_int64(grad.size), C.c_float(alpha), C.c_float(lamb))


def grokfast_adamw(param, grad, ema, ea, easq, step, alpha, lamb, lr, beta1, beta2, eps, wd):
    lib().orc_grokfast_adamw(_f32(param), _f32(grad), _f32(ema), _f32(ea), _f32(easq), C.c_int64(param.size),
                             C.c_int(step), C.c_float(alpha), C.c_float(lamb), C.c_double(lr), C.c_double(beta1),
                             C.c_double(beta2), C.c_double(eps), C.c_double(wd))


def sg15_clip_coef(grads, clip):
    """(coef, clip_on) of the global-norm clip: coef = clip/(norm+1e-6) when norm > clip."""
    tot = sum(float(np.sum(g.astype(np.float64) ** 2)) for g in grads)
    norm = np.float32(np.sqrt(tot))
    if clip > 0 and norm > np.float32(clip):
        return float(np.float32(clip) / (norm + np.float32(1e-6))), 1
    return 1.0, 0


def sg15_step(params, grads, sharps, eas, easqs, mus, net, per_tensor, lamb_eff, beta2, lr, wd_eff, eps, clip,
              gelu_mode=0):
    """All tensors, in place.  net = (W1[H,2], b1[H], W2[1,H], b2[1], rescale); per_tensor: list of dicts
    alpha, beta1, bc1, bc2."""
    coef, on = sg15_clip_coef(grads, clip)
    W1, b1, W2, b2, rescale = net
    W1, b1, W2, b2 = [np.ascontiguousarray(w, np.float32) for w in (W1, b1, W2, b2)]
    f = C.c_float
    for p, g, s, ea, easq, mu, sc in zip(params, grads, sharps, eas, easqs, mus, per_tensor):
        if p.size == 0:
            continue
        lib().orc_sg15_step(_f32(p), _f32(g), _f32(s), _f32(ea), _f32(easq), _f32(mu), C.c_int64(p.size), _f32(W1),
                            _f32(b1), _f32(W2), _f32(b2), C.c_int(b1.size), f(rescale), C.c_int(gelu_mode),
                            f(sc["alpha"]), f(sc["beta1"]), f(sc["bc1"]), f(sc["bc2"]), f(lamb_eff), f(beta2), f(lr),
                            f(wd_eff), f(eps), f(coef), C.c_int(on))
    return coef, on
