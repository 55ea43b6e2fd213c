"""sg2_batched_step_static (scratch in a static device array, nothing allocated by the call) against
sg2_batched_step (caller workspace) through the C ABI: identical inputs, two calls in a row, the second on a
smaller set of tensors; every output must be bit-identical (same kernels), including the inspection outputs.
A request beyond the static buffer is rejected with an error and launches nothing."""
import ctypes as C

import numpy as np
import pytest
import torch

import workloads as wl
from sg2_harness import per_tensor_scalars, shared_scalars

pytestmark = pytest.mark.gpu

KEYS = ("param", "exp_avg", "exp_avg_sq", "mu", "gru", "mamba_fwd", "mamba_bwd")


def _state(shapes, seed, dev):
    gen = torch.Generator().manual_seed(seed)
    out = []
    for p in wl.make_params(shapes, seed=seed):
        n = p.numel()
        out.append(dict(param=p.reshape(-1).clone(), exp_avg=torch.randn(n, generator=gen) * 1e-3,
                        exp_avg_sq=torch.rand(n, generator=gen) * 1e-6, mu=torch.randn(n, generator=gen) * 1e-3,
                        gru=torch.randn(n, 4, generator=gen) * 0.3, mamba_fwd=torch.randn(16, 16, generator=gen) * 0.1,
                        mamba_bwd=torch.randn(16, 16, generator=gen) * 0.1))
    return [{k: v.to(dev) for k, v in st.items()} for st in out]


class _StaticStep:
    """ctypes call of sg2_batched_step_static on a fixed list of tensors (debug outputs on)."""

    def __init__(self, W, state, counts):
        from grokking_optimizers import _cabi
        self.cabi = _cabi
        self.L = _cabi.lib()
        self.dims = _cabi.make_dims()
        self.Wt = W
        self.W = _cabi.Sg2Weights()
        for k, w in enumerate(W):
            self.W.w[k] = w.data_ptr()
        self.state, self.counts = state, counts
        self.P = len(state)
        total = sum(s["param"].numel() for s in state)
        dev = W[0].device
        self.perm = torch.empty(total, dtype=torch.int32, device=dev)
        self.expert_idx = torch.empty(total, 4, dtype=torch.int32, device=dev)
        self.ctx = torch.empty(2, total, 8, dtype=torch.float32, device=dev)
        self.debug = _cabi.Sg2Debug(self.perm.data_ptr(), self.expert_idx.data_ptr(), self.ctx.data_ptr())
        self.tensors = (_cabi.Sg2Tensor * max(self.P, 1))()

    def __call__(self, grads, sharps, per_tensor, shared):
        for i, st in enumerate(self.state):
            t, sc = self.tensors[i], per_tensor[i]
            t.param, t.grad, t.sharpness = st["param"].data_ptr(), grads[i].data_ptr(), sharps[i].data_ptr()
            t.exp_avg, t.exp_avg_sq, t.mu = st["exp_avg"].data_ptr(), st["exp_avg_sq"].data_ptr(), st["mu"].data_ptr()
            t.gru_state, t.mamba_fwd_state, t.mamba_bwd_state = st["gru"].data_ptr(), st["mamba_fwd"].data_ptr(), st["mamba_bwd"].data_ptr()
            t.numel, t.dtype = st["param"].numel(), 0
            t.alpha_mu, t.lamb_eff, t.beta1, t.bc1, t.bc2 = sc["alpha"], sc["lamb_eff"], sc["beta1"], sc["bc1"], sc["bc2"]
        S = self.cabi.Sg2Scalars(shared["rescale"], shared["beta2"], shared["lr"], shared["wd_eff"], shared["eps"])
        return self.L.sg2_batched_step_static(C.byref(self.dims), C.byref(self.W), self.P, self.tensors, C.byref(S),
                                              self.counts.data_ptr(), C.byref(self.debug), torch.cuda.current_stream().cuda_stream)


def _run_both(shapes, seed, step, W, dev):
    from grokking_optimizers import _cabi
    sa, sb = _state(shapes, seed, dev), _state(shapes, seed, dev)
    ca = torch.zeros(144, dtype=torch.int32, device=dev)
    cb = torch.zeros(144, dtype=torch.int32, device=dev)
    grads = [g.reshape(-1).to(dev) for g in wl.make_grads(shapes, seed=seed + 1, tail_frac=0.01)]
    sharps = [g.reshape(-1).abs().to(dev) for g in wl.make_grads(shapes, seed=seed + 2)]
    pt, sh = per_tensor_scalars(len(shapes), step, lamb_eff=2.0), shared_scalars(wd_eff=4.5)
    ref = _cabi.Sg2Step(W, *[[s[k] for s in sa] for k in KEYS], ca, debug=True)
    ref(grads, sharps, pt, sh)
    new = _StaticStep(W, sb, cb)
    rc = new(grads, sharps, pt, sh)
    assert rc == 0, _cabi.last_error()
    torch.cuda.synchronize()
    for i, (a, b) in enumerate(zip(sa, sb)):
        for k in KEYS:
            assert torch.equal(a[k], b[k]), (shapes[i], k)
    assert torch.equal(ca, cb) and int(ca.sum()) == 4 * sum(wl.numel(s) for s in shapes)
    assert torch.equal(ref.perm, new.perm) and torch.equal(ref.expert_idx, new.expert_idx) and torch.equal(ref.ctx, new.ctx)


def test_static_scratch_entry_point_matches_the_workspace_one():
    from grokking_optimizers import _cabi
    dev = torch.device("cuda:0")
    W = [w.to(dev) for w in wl.meta_weights(7)]
    big = [(300,), (40, 64), (70000,), (5000,), (1,), (255,)]
    small = [(129,), (3000,)]
    assert _cabi.workspace_bytes([wl.numel(s) for s in big]) <= _cabi.lib().sg2_static_scratch_bytes()
    print("static-scratch step, first call", big, flush=True)
    _run_both(big, 31, 1, W, dev)
    print("static-scratch step, second call (smaller)", small, flush=True)
    _run_both(small, 32, 2, W, dev)
    print("static-scratch step, third call (first shapes again)", flush=True)
    _run_both(big, 33, 3, W, dev)
    # what the entry point exists for: a call allocates nothing, on the device or through torch's allocator
    st = _state(small, 40, dev)
    counts = torch.zeros(144, dtype=torch.int32, device=dev)
    step = _StaticStep(W, st, counts)
    grads = [g.reshape(-1).to(dev) for g in wl.make_grads(small, seed=41)]
    sharps = [torch.zeros_like(g) for g in grads]
    pt, sh = per_tensor_scalars(len(small), 1), shared_scalars()
    assert step(grads, sharps, pt, sh) == 0
    torch.cuda.synchronize()
    free0, alloc0, reserved0 = torch.cuda.mem_get_info()[0], torch.cuda.memory_allocated(), torch.cuda.memory_reserved()
    for _ in range(3):
        assert step(grads, sharps, pt, sh) == 0
    torch.cuda.synchronize()
    assert torch.cuda.mem_get_info()[0] == free0, "free device memory changed across static-scratch calls"
    assert torch.cuda.memory_allocated() == alloc0 and torch.cuda.memory_reserved() == reserved0


def test_static_scratch_entry_point_rejects_what_does_not_fit():
    from grokking_optimizers import _cabi
    dev = torch.device("cuda:0")
    L = _cabi.lib()
    assert L.sg2_static_scratch_bytes() == 64 << 20
    W = [w.to(dev) for w in wl.meta_weights(7)]
    shapes = [(1 << 20,)]
    assert _cabi.workspace_bytes([1 << 20]) > L.sg2_static_scratch_bytes()
    st = _state(shapes, 1, dev)
    before = [{k: v.clone() for k, v in s.items()} for s in st]
    counts = torch.zeros(144, dtype=torch.int32, device=dev)
    step = _StaticStep(W, st, counts)
    g = [torch.randn(1 << 20, device=dev) * 1e-3]
    rc = step(g, [torch.zeros_like(g[0])], per_tensor_scalars(1, 1), shared_scalars())
    torch.cuda.synchronize()
    assert rc != 0 and "static" in _cabi.last_error() and "sg2_batched_step" in _cabi.last_error()
    for a, b in zip(st, before):
        for k in KEYS:
            assert torch.equal(a[k], b[k])
    assert int(counts.sum()) == 0
