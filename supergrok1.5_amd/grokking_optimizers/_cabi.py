"""ctypes view of libsg_hip.so (the C ABI declared in include/sg_abi.h).

The torch extension `_ops` is the production caller of the library; this
module binds the same entry points directly so that the parity tests and the
benchmark can drive the C ABI with device pointers taken from torch tensors,
and read the inspection outputs (sort permutation, expert indices, contexts).
There is no fallback: if the library is missing, loading raises.
"""
import ctypes as C
import os

import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(os.path.dirname(_HERE), "lib", "libsg_hip.so")

SG_DTYPE = {torch.float32: 0, torch.float16: 1, torch.bfloat16: 2}
DIM_NAMES = ("d_model", "d_state", "d_inner", "gru_hidden", "num_heads", "pk_dim", "expert_hidden",
             "num_experts")
DEFAULT_DIMS = dict(d_model=8, d_state=16, d_inner=16, gru_hidden=4, num_heads=4, pk_dim=12,
                    expert_hidden=16, num_experts=144)


class SgDims(C.Structure):
    _fields_ = [(n, C.c_int32) for n in DIM_NAMES]


class Sg2Weights(C.Structure):
    _fields_ = [("w", C.c_void_p * 33)]


class Sg2Tensor(C.Structure):
    _fields_ = [("param", C.c_void_p), ("grad", C.c_void_p), ("sharpness", C.c_void_p),
                ("exp_avg", C.c_void_p), ("exp_avg_sq", C.c_void_p), ("mu", C.c_void_p),
                ("gru_state", C.c_void_p), ("mamba_fwd_state", C.c_void_p), ("mamba_bwd_state", C.c_void_p),
                ("numel", C.c_int64), ("dtype", C.c_int32),
                ("alpha_mu", C.c_float), ("lamb_eff", C.c_float), ("beta1", C.c_float),
                ("bc1", C.c_float), ("bc2", C.c_float)]


class Sg2Scalars(C.Structure):
    _fields_ = [("rescale", C.c_float), ("beta2", C.c_float), ("lr", C.c_float), ("wd_eff", C.c_float),
                ("eps", C.c_float)]


class Sg2Options(C.Structure):
    _fields_ = [("chunk_len", C.c_int32), ("scan_window", C.c_int32)]


class Sg2Debug(C.Structure):
    _fields_ = [("perm", C.c_void_p), ("expert_idx", C.c_void_p), ("ctx", C.c_void_p)]


EXPORTS = ("sg_last_error", "sg2_set_chunk_len", "sg2_get_chunk_len", "sg2_set_scan_window", "sg2_get_scan_window", "sg2_chunk_len_for", "sg2_workspace_bytes", "sg2_batched_step",
           "sg2_profile_enable", "sg2_profile_read")
SG2_PROF_STAGES = ("sort", "scan_summary", "chunk_prefix", "scan_output", "elementwise")

_lib = None


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError("libsg_hip.so is not built (%s); run __graft_entry__.build()" % LIB_PATH)
        L = C.CDLL(LIB_PATH)
        L.sg_last_error.restype = C.c_char_p
        L.sg2_set_chunk_len.argtypes = [C.c_int]
        L.sg2_set_scan_window.argtypes = [C.c_int]
        L.sg2_workspace_bytes.restype = C.c_size_t
        L.sg2_workspace_bytes.argtypes = [C.POINTER(SgDims), C.c_int, C.POINTER(C.c_int64)]
        L.sg2_batched_step.restype = C.c_int
        L.sg2_batched_step.argtypes = [C.POINTER(SgDims), C.POINTER(Sg2Weights), C.c_int, C.POINTER(Sg2Tensor),
                                       C.POINTER(Sg2Scalars), C.c_void_p, C.c_void_p, C.c_size_t,
                                       C.POINTER(Sg2Debug), C.c_void_p]
        L.sg2_workspace_bytes_opt.restype = C.c_size_t
        L.sg2_workspace_bytes_opt.argtypes = [C.POINTER(SgDims), C.c_int, C.POINTER(C.c_int64), C.POINTER(Sg2Options)]
        L.sg2_batched_step_opt.restype = C.c_int
        L.sg2_batched_step_opt.argtypes = [C.POINTER(SgDims), C.POINTER(Sg2Weights), C.c_int, C.POINTER(Sg2Tensor),
                                           C.POINTER(Sg2Scalars), C.c_void_p, C.c_void_p, C.c_size_t,
                                           C.POINTER(Sg2Debug), C.POINTER(Sg2Options), C.c_void_p]
        L.sg2_static_scratch_bytes.restype = C.c_size_t
        L.sg2_batched_step_static.restype = C.c_int
        L.sg2_batched_step_static.argtypes = [C.POINTER(SgDims), C.POINTER(Sg2Weights), C.c_int, C.POINTER(Sg2Tensor),
                                              C.POINTER(Sg2Scalars), C.c_void_p, C.POINTER(Sg2Debug), C.c_void_p]
        L.sg2_bilevel_workspace_bytes.restype = C.c_size_t
        L.sg2_bilevel_workspace_bytes.argtypes = [C.POINTER(SgDims), C.c_int, C.POINTER(C.c_int64)]
        L.sg2_bilevel_forward.restype = C.c_int
        L.sg2_bilevel_forward.argtypes = [C.POINTER(SgDims), C.POINTER(Sg2Weights), C.c_int, C.POINTER(Sg2Tensor), C.c_void_p,
                                          C.c_void_p, C.c_size_t, C.c_void_p]
        L.sg2_bilevel_backward.restype = C.c_int
        L.sg2_bilevel_backward.argtypes = [C.POINTER(SgDims), C.POINTER(Sg2Weights), C.c_int, C.POINTER(Sg2Tensor), C.c_void_p,
                                           C.c_void_p, C.c_void_p, C.c_size_t, C.c_void_p]
        L.sg2_bilevel_elem_workspace_bytes.restype = C.c_size_t
        L.sg2_bilevel_elem_workspace_bytes.argtypes = [C.c_int64]
        L.sg2_bilevel_elem.restype = C.c_int
        L.sg2_bilevel_elem.argtypes = [C.POINTER(SgDims), C.POINTER(Sg2Weights), C.c_int64] + [C.c_void_p] * 5 + [C.c_float] + \
                                      [C.c_void_p] * 4 + [C.c_size_t, C.c_void_p]
        L.sg2_bilevel_elem_ex.restype = C.c_int
        L.sg2_bilevel_elem_ex.argtypes = [C.POINTER(SgDims), C.POINTER(Sg2Weights), C.c_int64] + [C.c_void_p] * 5 + [C.c_float] + \
                                         [C.c_void_p] * 5 + [C.c_size_t, C.c_void_p]
        L.sg2_meta_forward.restype = C.c_int
        L.sg2_meta_forward.argtypes = [C.POINTER(SgDims), C.POINTER(Sg2Weights), C.c_int, C.POINTER(Sg2Tensor), C.c_float, C.c_void_p,
                                       C.c_void_p, C.c_void_p, C.c_void_p, C.c_size_t, C.c_void_p]
        _lib = L
    return _lib


def profile_enable(on=True):
    if lib().sg2_profile_enable(1 if on else 0) != 0:
        raise RuntimeError(last_error())


def profile_read():
    """(dict stage -> total ms, number of calls) since profile_enable(True)."""
    ms = (C.c_float * len(SG2_PROF_STAGES))()
    calls = C.c_int(0)
    if lib().sg2_profile_read(ms, C.byref(calls)) != 0:
        raise RuntimeError(last_error())
    return {n: float(ms[k]) for k, n in enumerate(SG2_PROF_STAGES)}, calls.value


def last_error():
    return lib().sg_last_error().decode()


def make_dims(dims=None):
    d = dict(DEFAULT_DIMS if dims is None else dims)
    return SgDims(*[d[n] for n in DIM_NAMES])


def chunk_len_for(numels):
    """Scan chunk length a call with these tensor sizes uses (the configured one, or the automatic choice)."""
    arr = (C.c_int64 * len(numels))(*numels)
    return lib().sg2_chunk_len_for(len(numels), arr)


def workspace_bytes(numels, dims=None, options=None):
    arr = (C.c_int64 * len(numels))(*numels)
    d = make_dims(dims)
    n = lib().sg2_workspace_bytes_opt(C.byref(d), len(numels), arr, C.byref(options) if options is not None else None)
    if n == 0 and sum(numels) > 0:
        raise RuntimeError(last_error())
    return n


class Sg2Step:
    """Reusable call plan for sg2_batched_step on a fixed list of tensors."""

    def __init__(self, weights, params, exp_avgs, exp_avg_sqs, mus, gru_states, mamba_fwd, mamba_bwd,
                 expert_counts, dims=None, debug=False, chunk_len=None, scan_window=None):
        """chunk_len / scan_window: this plan's own scan decomposition (sg2_batched_step_opt); both None = the
        process-wide settings (sg2_set_chunk_len / sg2_set_scan_window)."""
        self.dims = make_dims(dims)
        self.options = None
        if chunk_len is not None or scan_window is not None:
            self.options = Sg2Options(0 if chunk_len is None else chunk_len, -1 if scan_window is None else scan_window)
        self.weights = [w.contiguous() for w in weights]
        assert len(self.weights) == 33 and all(w.dtype == torch.float32 and w.is_cuda for w in self.weights)
        self.W = Sg2Weights()
        for k, w in enumerate(self.weights):
            self.W.w[k] = w.data_ptr()
        self.state = (params, exp_avgs, exp_avg_sqs, mus, gru_states, mamba_fwd, mamba_bwd)
        self.P = len(params)
        self.numels = [p.numel() for p in params]
        self.total = sum(self.numels)
        self.expert_counts = expert_counts
        self.ws_bytes = workspace_bytes(self.numels, dims, self.options)
        dev = params[0].device
        self.workspace = torch.empty(max(self.ws_bytes, 256), dtype=torch.uint8, device=dev)
        self.tensors = (Sg2Tensor * self.P)()
        self.debug = None
        if debug:
            H, dm = self.dims.num_heads, self.dims.d_model
            self.perm = torch.empty(self.total, dtype=torch.int32, device=dev)
            self.expert_idx = torch.empty(self.total, H, dtype=torch.int32, device=dev)
            self.ctx = torch.empty(2, self.total, dm, dtype=torch.float32, device=dev)
            self.debug = Sg2Debug(self.perm.data_ptr(), self.expert_idx.data_ptr(), self.ctx.data_ptr())

    def __call__(self, grads, sharps, per_tensor, shared):
        """per_tensor: list of dicts(alpha, lamb_eff, beta1, bc1, bc2); shared: dict(rescale, beta2, lr, wd_eff, eps)."""
        params, eas, easqs, mus, grus, mf, mb = self.state
        for i in range(self.P):
            t = self.tensors[i]
            p, g, s = params[i], grads[i], sharps[i]
            assert g.dtype == p.dtype and s.dtype == p.dtype and g.is_contiguous() and s.is_contiguous()
            t.param, t.grad, t.sharpness = p.data_ptr(), g.data_ptr(), s.data_ptr()
            t.exp_avg, t.exp_avg_sq, t.mu = eas[i].data_ptr(), easqs[i].data_ptr(), mus[i].data_ptr()
            t.gru_state, t.mamba_fwd_state, t.mamba_bwd_state = grus[i].data_ptr(), mf[i].data_ptr(), mb[i].data_ptr()
            t.numel, t.dtype = p.numel(), SG_DTYPE[p.dtype]
            sc = per_tensor[i]
            t.alpha_mu, t.lamb_eff, t.beta1, t.bc1, t.bc2 = sc["alpha"], sc["lamb_eff"], sc["beta1"], sc["bc1"], sc["bc2"]
        S = Sg2Scalars(shared["rescale"], shared["beta2"], shared["lr"], shared["wd_eff"], shared["eps"])
        stream = torch.cuda.current_stream().cuda_stream
        rc = lib().sg2_batched_step_opt(C.byref(self.dims), C.byref(self.W), self.P, self.tensors, C.byref(S),
                                        self.expert_counts.data_ptr() if self.expert_counts is not None else None,
                                        self.workspace.data_ptr(), self.workspace.numel(),
                                        C.byref(self.debug) if self.debug is not None else None,
                                        C.byref(self.options) if self.options is not None else None, stream)
        if rc != 0:
            raise RuntimeError("sg2_batched_step: " + last_error())


SG2_SCAN_GRAD_FLOATS = 3160  # gradients of the 20 scan weights, flat, in the order of Sg2Weights


class Sg2Bilevel:
    """sg2_bilevel_forward / sg2_bilevel_backward on a fixed list of tensors: the sort and the bidirectional scan of
    the meta-net, differentiable with respect to the scan's weights.  forward() returns the two contexts of every
    element ([2, sum numel, d_model], element order, tensors packed in call order); backward(d_ctx) returns the
    gradients of the 20 scan weights as one flat tensor [SG2_SCAN_GRAD_FLOATS] (layout in include/sg_abi.h).  The
    workspace is kept between the two."""

    def __init__(self, weights, grads, sharps, mamba_fwd, mamba_bwd, dims=None):
        self.dims = make_dims(dims)
        self.weights = [w.detach().float().contiguous() for w in weights]
        assert len(self.weights) == 33 and all(w.is_cuda for w in self.weights)
        self.W = Sg2Weights()
        for k, w in enumerate(self.weights):
            self.W.w[k] = w.data_ptr()
        self.P = len(grads)
        self.grads = [g.contiguous() for g in grads]
        self.sharps = [s.contiguous() for s in sharps]
        # the entry points overwrite the states with the end-of-sequence ones: work on copies
        self.mf = [m.detach().float().clone() for m in mamba_fwd]
        self.mb = [m.detach().float().clone() for m in mamba_bwd]
        self.numels = [g.numel() for g in self.grads]
        self.total = sum(self.numels)
        dev = self.grads[0].device
        arr = (C.c_int64 * self.P)(*self.numels)
        nbytes = lib().sg2_bilevel_workspace_bytes(C.byref(self.dims), self.P, arr)
        if nbytes == 0 and self.total > 0:
            raise RuntimeError(last_error())
        self.workspace = torch.empty(max(nbytes, 256), dtype=torch.uint8, device=dev)
        self.tensors = (Sg2Tensor * self.P)()
        for i in range(self.P):
            t, g, s = self.tensors[i], self.grads[i], self.sharps[i]
            assert g.dtype == s.dtype and g.is_cuda and s.is_cuda
            t.grad, t.sharpness = g.data_ptr(), s.data_ptr()
            t.mamba_fwd_state, t.mamba_bwd_state = self.mf[i].data_ptr(), self.mb[i].data_ptr()
            t.numel, t.dtype = g.numel(), SG_DTYPE[g.dtype]
        self.device = dev

    def forward(self):
        ctx = torch.empty(2, self.total, BILEVEL_SCAN_BLOCK[0], dtype=torch.float32, device=self.device)
        rc = lib().sg2_bilevel_forward(C.byref(self.dims), C.byref(self.W), self.P, self.tensors, ctx.data_ptr(),
                                       self.workspace.data_ptr(), self.workspace.numel(), torch.cuda.current_stream().cuda_stream)
        if rc != 0:
            raise RuntimeError("sg2_bilevel_forward: " + last_error())
        # a smaller scan block runs embedded: its context entries are the first d_model of the kernel's rows
        return ctx if self.dims.d_model == BILEVEL_SCAN_BLOCK[0] else ctx[..., :self.dims.d_model]

    def backward(self, d_ctx):
        d_ctx = d_ctx.detach().float()
        assert d_ctx.shape == (2, self.total, self.dims.d_model) and d_ctx.is_cuda
        d_ctx = _widen_last(d_ctx, BILEVEL_SCAN_BLOCK[0])
        out = torch.empty(SG2_SCAN_GRAD_FLOATS, dtype=torch.float32, device=self.device)
        rc = lib().sg2_bilevel_backward(C.byref(self.dims), C.byref(self.W), self.P, self.tensors, d_ctx.data_ptr(), out.data_ptr(),
                                        self.workspace.data_ptr(), self.workspace.numel(), torch.cuda.current_stream().cuda_stream)
        if rc != 0:
            raise RuntimeError("sg2_bilevel_backward: " + last_error())
        return extract_scan_grads(out, self.dims)


BILEVEL_SCAN_BLOCK = (8, 16, 16)   # (d_model, d_state, d_inner) the scan kernels of the bilevel pass are built for


def _widen_last(t, width):
    """`t` with its last dimension zero-padded to `width`, contiguous."""
    if t.shape[-1] == width:
        return t.contiguous()
    wide = torch.zeros(*t.shape[:-1], width, dtype=t.dtype, device=t.device)
    wide[..., :t.shape[-1]] = t
    return wide


def extract_scan_grads(flat, dims):
    """The gradients of a scan block smaller than BILEVEL_SCAN_BLOCK out of sg2_bilevel_backward's block, which keeps
    the kernel block's layout (include/sg_abi.h): flat again, in the caller's own shapes and the same order."""
    DM, DS, DI = BILEVEL_SCAN_BLOCK
    dm, ds, di = dims.d_model, dims.d_state, dims.d_inner
    if (dm, ds, di) == (DM, DS, DI):
        return flat
    parts, o = [], 0

    def take(*shape):
        nonlocal o
        n = 1
        for k in shape:
            n *= k
        v = flat[o:o + n].view(*shape)
        o += n
        return v
    parts += [take(DM, 2)[:dm], take(DM)[:dm]]
    for _ in range(2):
        parts += [take(2, DI, DM)[:, :di, :dm],          # in_proj: x rows, then z rows
                  take(DI, DI)[:di, :di], take(DI)[:di], take(DS, DI)[:ds, :di], take(DS, DI)[:ds, :di],
                  take(DI, DS)[:di, :ds], take(DI)[:di], take(DI, DS // 2)[:di, :ds // 2], take(DM, DI)[:dm, :di]]
    assert o == flat.numel()
    return torch.cat([v.reshape(-1) for v in parts])


SG2_ELEM_GRAD_FLOATS = 8420


BILEVEL_EXPERT_WIDTH = 16      # expert width sg2_bilevel_elem is compiled for
BILEVEL_GRU_HIDDEN = 4         # its GRU width (d_model: BILEVEL_SCAN_BLOCK[0])


def _elem_maps(dm, gh, dev):
    """Where the entries of a smaller per-element net sit in the kernel's: columns of a GRU matrix
    ([g, s, ctx_f, ctx_b, h]), columns of a query matrix ([h', ctx_f, ctx_b, g, s]) and its rows (two halves of
    d_model/2 entries)."""
    DM, GH = BILEVEL_SCAN_BLOCK[0], BILEVEL_GRU_HIDDEN
    ix = lambda v: torch.tensor(v, dtype=torch.long, device=dev)
    gru_cols = ix([0, 1] + [2 + c for c in range(dm)] + [2 + DM + c for c in range(dm)] + [2 + 2 * DM + k for k in range(gh)])
    q_cols = ix(list(range(gh)) + [GH + c for c in range(dm)] + [GH + DM + c for c in range(dm)] + [GH + 2 * DM, GH + 2 * DM + 1])
    q_rows = ix(list(range(dm // 2)) + [DM // 2 + r for r in range(dm // 2)])
    return gru_cols, q_cols, q_rows


def bilevel_elem(weights, grad, sharpness, ctx, gru_state, cotangent, rescale, dims=None, want_smart=True, want_gru=False):
    """sg2_bilevel_elem on flat fp32 GPU arrays: returns (smart [total] or None, d_ctx [2, total, d_model],
    weight-gradient block, flat in the order of include/sg_abi.h at the caller's own sizes); with want_gru a fourth
    value, the new GRU state [total, gru_hidden].

    The kernel is built for d_model 8, gru_hidden 4 and experts of width 16.  A net that is smaller in any of these
    runs embedded: the extra context entries, hidden units and expert units have zero weights (an extra hidden unit
    starts at 0 and stays there: its candidate is tanh(0); an extra expert unit is relu(0)), every chain of products
    only gains zero terms, so the real entries keep their bits, and the extra entries of the gradient block (all
    zero) are dropped.  (The reference's training harness builds experts of width 4.)"""
    d = make_dims(dims)
    DM, GH, EH = BILEVEL_SCAN_BLOCK[0], BILEVEL_GRU_HIDDEN, BILEVEL_EXPERT_WIDTH
    dm, gh, eh, E, NH, PK = d.d_model, d.gru_hidden, d.expert_hidden, d.num_experts, d.num_heads, d.pk_dim
    ws_ = [w.detach().float().contiguous() for w in weights]
    dev = ws_[20].device
    embedded = dm < DM or gh < GH or eh < EH
    if embedded:
        if dm % 2 or dm < 2 or gh < 1 or eh < 1:
            raise RuntimeError("sg2_bilevel_elem: d_model must be even and every size positive")
        gru_cols, q_cols, q_rows = _elem_maps(dm, gh, dev)
        zeros = lambda *shape: torch.zeros(*shape, dtype=torch.float32, device=dev)
        for k in (20, 22, 24):                                  # W_z, W_r, W_h [gh][2 + 2 dm + gh]
            wide = zeros(GH, 2 + 2 * DM + GH)
            wide[:gh, gru_cols] = ws_[k].reshape(gh, -1)
            ws_[k] = wide
        for k in (21, 23, 25):                                  # their biases
            ws_[k] = _widen_last(ws_[k].reshape(-1), GH)
        q = zeros(NH, DM, GH + 2 * DM + 2)                      # queries [heads][d_model][gh + 2 dm + 2]
        q[:, q_rows[:, None], q_cols[None, :]] = ws_[26].reshape(NH, dm, -1)
        ws_[26] = q
        for k in (27, 28):                                      # product keys [heads][pk][d_model / 2]
            ws_[k] = _widen_last(ws_[k].reshape(NH, PK, dm // 2), DM // 2)
        for k in (29, 30, 31):                                  # expert W1, b1, W2 [E][eh]
            ws_[k] = _widen_last(ws_[k].reshape(E, eh), EH)
        d.d_model, d.gru_hidden, d.expert_hidden = DM, GH, EH
    W = Sg2Weights()
    for k, w in enumerate(ws_):
        W.w[k] = w.data_ptr()
    arrs = [t.detach().float().contiguous() for t in (grad, sharpness, ctx, gru_state, cotangent)]
    total = arrs[0].numel()
    assert all(t.is_cuda for t in arrs) and arrs[2].shape == (2, total, dm) and arrs[3].shape == (total, gh)
    assert arrs[1].numel() == total and arrs[4].numel() == total
    arrs[2] = _widen_last(arrs[2], DM)
    arrs[3] = _widen_last(arrs[3], GH)
    smart = torch.empty(total, dtype=torch.float32, device=dev) if want_smart else None
    d_ctx = torch.empty_like(arrs[2])
    out = torch.empty(SG2_ELEM_GRAD_FLOATS, dtype=torch.float32, device=dev)
    nbytes = lib().sg2_bilevel_elem_workspace_bytes(total)
    work = torch.empty(max(nbytes, 256), dtype=torch.uint8, device=dev)
    gru_out = torch.empty_like(arrs[3]) if want_gru else None
    rc = lib().sg2_bilevel_elem_ex(C.byref(d), C.byref(W), total, *[t.data_ptr() for t in arrs], float(rescale),
                                   smart.data_ptr() if want_smart else None, gru_out.data_ptr() if want_gru else None, d_ctx.data_ptr(),
                                   out.data_ptr(), work.data_ptr(), work.numel(), torch.cuda.current_stream().cuda_stream)
    if rc != 0:
        raise RuntimeError("sg2_bilevel_elem: " + last_error())
    if embedded:
        parts, o = [], 0

        def take(*shape):
            nonlocal o
            n = 1
            for k in shape:
                n *= k
            v = out[o:o + n].view(*shape)
            o += n
            return v
        for _ in range(3):                                      # (W, b) of the three gates
            parts += [take(GH, 2 + 2 * DM + GH)[:gh][:, gru_cols], take(GH)[:gh]]
        parts.append(take(NH, DM, GH + 2 * DM + 2)[:, q_rows[:, None], q_cols[None, :]])
        parts += [take(NH, PK, DM // 2)[..., :dm // 2], take(NH, PK, DM // 2)[..., :dm // 2]]
        parts += [take(E, EH)[:, :eh], take(E, EH)[:, :eh], take(E, EH)[:, :eh], take(E)]
        assert o == out.numel()
        out = torch.cat([v.reshape(-1) for v in parts])
        d_ctx = d_ctx[..., :dm]
        gru_out = gru_out[:, :gh].contiguous() if want_gru else None
    if want_gru:
        return smart, d_ctx, out, gru_out
    return smart, d_ctx, out


def meta_forward(weights, grads, sharps, gru_states, mamba_fwd, mamba_bwd, rescale, dims=None, expert_counts=None):
    """sg2_meta_forward: the meta-net's forward (hard top-1 routing) for a list of flat tensors.  mamba_fwd / mamba_bwd
    are replaced by the new carried states.  Returns (smart [total], new GRU state [total, gru_hidden]), packed in call
    order."""
    d = make_dims(dims)
    ws_ = [w.detach().float().contiguous() for w in weights]
    W = Sg2Weights()
    for k, w in enumerate(ws_):
        W.w[k] = w.data_ptr()
    P = len(grads)
    dev = grads[0].device
    numels = [g.numel() for g in grads]
    total = sum(numels)
    keep = []
    tensors = (Sg2Tensor * P)()
    for i in range(P):
        g, s, h = grads[i].contiguous(), sharps[i].contiguous(), gru_states[i].detach().float().contiguous()
        assert s.dtype == g.dtype and s.numel() == g.numel() and h.numel() == g.numel() * d.gru_hidden
        assert mamba_fwd[i].dtype == torch.float32 and mamba_fwd[i].is_contiguous() and mamba_bwd[i].is_contiguous()
        keep += [g, s, h]
        t = tensors[i]
        t.grad, t.sharpness, t.gru_state = g.data_ptr(), s.data_ptr(), h.data_ptr()
        t.mamba_fwd_state, t.mamba_bwd_state = mamba_fwd[i].data_ptr(), mamba_bwd[i].data_ptr()
        t.numel, t.dtype = g.numel(), SG_DTYPE[g.dtype]
    smart = torch.empty(total, dtype=torch.float32, device=dev)
    gru_out = torch.empty(total, d.gru_hidden, dtype=torch.float32, device=dev)
    work = torch.empty(max(workspace_bytes(numels, dims), 256), dtype=torch.uint8, device=dev)
    rc = lib().sg2_meta_forward(C.byref(d), C.byref(W), P, tensors, float(rescale), smart.data_ptr(), gru_out.data_ptr(),
                                expert_counts.data_ptr() if expert_counts is not None else None, work.data_ptr(), work.numel(),
                                torch.cuda.current_stream().cuda_stream)
    if rc != 0:
        raise RuntimeError("sg2_meta_forward: " + last_error())
    return smart, gru_out
