"""Drives the SuperGrok v2 batched step on the GPU through the C ABI and the
CPU checker on identical inputs, and compares them."""
from concurrent.futures import ThreadPoolExecutor

import numpy as np
import torch

import workloads as wl
from helpers import DIMS, rel_close
from oracle import oracle as orc

NP_OF = {torch.float32: np.float32, torch.float16: np.uint16, torch.bfloat16: np.uint16}
NAME_OF = {torch.float32: "float32", torch.float16: "float16", torch.bfloat16: "bfloat16"}


def to_np(t):
    t = t.detach().cpu().contiguous()
    if t.dtype in (torch.float16, torch.bfloat16):
        return t.view(torch.int16).numpy().view(np.uint16).copy()
    return t.numpy().copy()


class Sg2Case:
    """A list of parameter tensors with full optimizer state, mirrored on CPU
    (numpy, for the checker) and on the GPU (torch, for the C ABI)."""

    def __init__(self, shapes, dtypes=None, seed=0, weights=None, random_state=False, device="cuda", dims=None):
        from grokking_optimizers import _cabi
        self.shapes = shapes
        self.P = len(shapes)
        self.dtypes = dtypes or [torch.float32] * self.P
        self.dims = dict(DIMS if dims is None else dims)
        self.W = weights if weights is not None else wl.meta_weights(7, self.dims)
        params = wl.make_params(shapes, seed=seed)
        gh, di, ds = self.dims["gru_hidden"], self.dims["d_inner"], self.dims["d_state"]
        gen = torch.Generator().manual_seed(seed + 1000)
        self.cpu = []
        for p, dt in zip(params, self.dtypes):
            n = p.numel()
            if random_state:
                st = dict(exp_avg=torch.randn(n, generator=gen) * 1e-3, exp_avg_sq=torch.rand(n, generator=gen) * 1e-6,
                          mu=torch.randn(n, generator=gen) * 1e-3, gru=torch.randn(n, gh, generator=gen) * 0.3,
                          mamba_fwd=torch.randn(di, ds, generator=gen) * 0.1,
                          mamba_bwd=torch.randn(di, ds, generator=gen) * 0.1)
            else:
                st = dict(exp_avg=torch.zeros(n), exp_avg_sq=torch.zeros(n), mu=torch.zeros(n),
                          gru=torch.zeros(n, gh), mamba_fwd=torch.zeros(di, ds), mamba_bwd=torch.zeros(di, ds))
            st["param"] = p.reshape(-1).to(dt)
            self.cpu.append(st)
        keys = ("param", "exp_avg", "exp_avg_sq", "mu", "gru", "mamba_fwd", "mamba_bwd")
        self.gpu = [{k: st[k].to(device) for k in keys} for st in self.cpu]
        self.np = [dict({k: to_np(st[k]) for k in keys}, dtype=NAME_OF[dt]) for st, dt in zip(self.cpu, self.dtypes)]
        self.counts_gpu = torch.zeros(self.dims["num_experts"], dtype=torch.int32, device=device)
        self.counts_np = np.zeros(self.dims["num_experts"], np.int32)
        self.Wgpu = [w.to(device) for w in self.W]
        self.Wnp = [w.numpy() for w in self.W]
        g = self.gpu
        self.step_fn = _cabi.Sg2Step(self.Wgpu, [s["param"] for s in g], [s["exp_avg"] for s in g],
                                     [s["exp_avg_sq"] for s in g], [s["mu"] for s in g], [s["gru"] for s in g],
                                     [s["mamba_fwd"] for s in g], [s["mamba_bwd"] for s in g], self.counts_gpu,
                                     dims=self.dims, debug=True)
        self.offsets = np.concatenate([[0], np.cumsum([wl.numel(s) for s in shapes])]).astype(np.int64)

    def gpu_step(self, grads, sharps, per_tensor, shared):
        dev = self.gpu[0]["param"].device
        gg = [g.reshape(-1).to(dt).to(dev) for g, dt in zip(grads, self.dtypes)]
        ss = [s.reshape(-1).to(dt).to(dev) for s, dt in zip(sharps, self.dtypes)]
        self.step_fn(gg, ss, per_tensor, shared)
        torch.cuda.synchronize()

    def oracle_step(self, grads, sharps, per_tensor, shared, chunk_len, precision=32, threads=8, window=None):
        from grokking_optimizers import _cabi
        if window is None:
            window = _cabi.lib().sg2_get_scan_window()
        if chunk_len is None:
            chunk_len = _cabi.chunk_len_for([wl.numel(s) for s in self.shapes])
        dbg = [None] * self.P
        counts = [np.zeros_like(self.counts_np) for _ in range(self.P)]

        def one(i):
            sc = dict(per_tensor[i])
            sc.update(shared)
            g = to_np(grads[i].reshape(-1).to(self.dtypes[i]))
            s = to_np(sharps[i].reshape(-1).to(self.dtypes[i]))
            if self.np[i]["exp_avg"].size == 0:
                return
            dbg[i] = orc.sg2_step(self.Wnp, self.np[i], g, s, sc, dims=self.dims, precision=precision, chunk_len=chunk_len, window=window,
                                  expert_counts=counts[i], debug=True)
        with ThreadPoolExecutor(threads) as ex:
            list(ex.map(one, range(self.P)))
        for c in counts:
            self.counts_np += c
        return dbg

    def compare(self, dbg, rel=1e-4, floor=1e-7, check_debug=True):
        """Bit-exact integers, relative tolerance on floats.  Returns worst ratios."""
        worst = {}
        perm = self.step_fn.perm.cpu().numpy()
        eidx = self.step_fn.expert_idx.cpu().numpy()
        ctx = self.step_fn.ctx.cpu().numpy()
        for i in range(self.P):
            a, b = int(self.offsets[i]), int(self.offsets[i + 1])
            if a == b:
                continue
            if check_debug and dbg[i] is not None:
                assert np.array_equal(perm[a:b], dbg[i]["perm"]), "tensor %d: sort permutation differs" % i
                nd = int((eidx[a:b] != dbg[i]["expert_idx"]).sum())
                assert nd == 0, "tensor %d: %d expert indices differ" % (i, nd)
                for d in range(2):
                    ok, r = rel_close(ctx[d, a:b], dbg[i]["ctx"][d], rel, floor)
                    assert ok, "tensor %d: ctx[%d] ratio %.3g" % (i, d, r)
            for k in ("param", "exp_avg", "exp_avg_sq", "mu", "gru", "mamba_fwd", "mamba_bwd"):
                got = self.gpu[i][k].detach().cpu()
                want = self.np[i][k]
                if k == "param" and self.dtypes[i] != torch.float32:
                    assert np.array_equal(to_np(got), want), "tensor %d: 16-bit params differ" % i
                    continue
                ok, r = rel_close(got.float().numpy().reshape(want.shape), want, rel, floor)
                worst[k] = max(worst.get(k, 0.0), r)
                assert ok, "tensor %d: %s ratio %.3g" % (i, k, r)
        assert np.array_equal(self.counts_gpu.cpu().numpy(), self.counts_np), "expert_counts differ"
        return worst


per_tensor_scalars, shared_scalars = wl.per_tensor_scalars, wl.shared_scalars
