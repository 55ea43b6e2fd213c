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


GEOMETRIES = ((8, 16, 16), (16, 32, 32))      # (d_model, d_state, d_inner) the scan kernels are compiled for


def kernel_geometry(dims):
    """The smallest compiled scan geometry that holds these dimensions."""
    for dm, ds, di in GEOMETRIES:
        if dims["d_model"] <= dm and dims["d_state"] <= ds and dims["d_inner"] <= di:
            return dm, ds, di
    raise ValueError("no scan geometry holds %r" % (dims,))


def embed_in_geometry(W, dims):
    """The meta-net `W` (33 tensors, `_ops` order) at dimensions `dims`, embedded in the compiled scan geometry that
    holds it: a larger net that computes the same function (zero rows and columns everywhere; the extra poles copy
    real ones and the extra columns take dt_b[0], so that the never-used extra states contract like real ones).
    Written from the description of the embedding, independently of the library's device kernel; the checker runs on
    the result and the library on the original.  Returns (weights, dims) of the embedded net."""
    dm, ds, di, gh = dims["d_model"], dims["d_state"], dims["d_inner"], dims["gru_hidden"]
    H, pk = dims["num_heads"], dims["pk_dim"]
    DM, DS, DI = kernel_geometry(dims)
    if (dm, ds, di) == (DM, DS, DI):
        return [w.clone() for w in W], dict(dims)
    hd, HD = dm // 2, DM // 2
    out = [None] * 33
    z = lambda *shape: torch.zeros(*shape, dtype=torch.float32)
    out[0] = z(DM, 2); out[0][:dm] = W[0]
    out[1] = z(DM); out[1][:dm] = W[1]
    for b in (2, 11):
        in_proj, dt_W, dt_b, Bp, Cp, A_log, D, rope, out_proj = W[b:b + 9]
        e = z(2 * DI, DM); e[:di, :dm] = in_proj[:di]; e[DI:DI + di, :dm] = in_proj[di:]
        out[b] = e
        e = z(DI, DI); e[:di, :di] = dt_W
        out[b + 1] = e
        e = dt_b[0].repeat(DI).clone(); e[:di] = dt_b
        out[b + 2] = e
        for k, src in ((3, Bp), (4, Cp)):
            e = z(DS, DI); e[:ds, :di] = src
            out[b + k] = e
        e = z(DI, DS)
        e[:, :] = A_log[0, 0]
        e[di:, :ds] = A_log[0]
        e[:di, :] = A_log[:, :1]
        e[:di, :ds] = A_log
        out[b + 5] = e
        e = z(DI); e[:di] = D
        out[b + 6] = e
        e = z(DI, DS // 2); e[:di, :ds // 2] = rope
        out[b + 7] = e
        e = z(DM, DI); e[:dm, :di] = out_proj
        out[b + 8] = e
    for k in (20, 22, 24):          # GRU rows: [g, s, fwd ctx, bwd ctx, h]
        src = W[k]
        e = z(gh, 2 + 2 * DM + gh)
        e[:, :2] = src[:, :2]
        e[:, 2:2 + dm] = src[:, 2:2 + dm]
        e[:, 2 + DM:2 + DM + dm] = src[:, 2 + dm:2 + 2 * dm]
        e[:, 2 + 2 * DM:] = src[:, 2 + 2 * dm:]
        out[k] = e
        out[k + 1] = W[k + 1].clone()
    src = W[26]                     # queries [H, d_model, h | fwd ctx | bwd ctx | g | s]: the two halves of a query keep their places
    e = z(H, DM, gh + 2 * DM + 2)
    for rows_to, rows_from in ((slice(0, hd), slice(0, hd)), (slice(HD, HD + hd), slice(hd, 2 * hd))):
        e[:, rows_to, :gh] = src[:, rows_from, :gh]
        e[:, rows_to, gh:gh + dm] = src[:, rows_from, gh:gh + dm]
        e[:, rows_to, gh + DM:gh + DM + dm] = src[:, rows_from, gh + dm:gh + 2 * dm]
        e[:, rows_to, gh + 2 * DM:] = src[:, rows_from, gh + 2 * dm:]
    out[26] = e
    for k in (27, 28):
        e = z(H, pk, HD); e[:, :, :hd] = W[k]
        out[k] = e
    for k in range(29, 33):
        out[k] = W[k].clone()
    return out, dict(dims, d_model=DM, d_state=DS, d_inner=DI)


class Sg2Case:
    """A list of parameter tensors with full optimizer state, mirrored on CPU
    (numpy, for the checker) and on the GPU (torch, for the C ABI)."""

    def __init__(self, shapes, dtypes=None, seed=0, weights=None, random_state=False, device="cuda", dims=None, chunk_len=None,
                 scan_window=None):
        from grokking_optimizers import _cabi
        self.shapes = shapes
        self.P = len(shapes)
        self.dtypes = dtypes or [torch.float32] * self.P
        self.dims = dict(DIMS if dims is None else dims)
        self.W = weights if weights is not None else wl.meta_weights(7, self.dims)
        # what the checker runs on: the same net embedded in the scan geometry the library computes it with
        self.oW, self.odims = embed_in_geometry(self.W, self.dims)
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
        for st in self.np:          # the checker's carried states at the embedding geometry: zero beyond the real block
            for k in ("mamba_fwd", "mamba_bwd"):
                e = np.zeros((self.odims["d_inner"], self.odims["d_state"]), np.float32)
                e[:di, :ds] = st[k]
                st[k] = e
        self.counts_gpu = torch.zeros(self.dims["num_experts"], dtype=torch.int32, device=device)
        self.counts_np = np.zeros(self.dims["num_experts"], np.int32)
        self.Wgpu = [w.to(device) for w in self.W]
        self.Wnp = [w.numpy() for w in self.oW]
        g = self.gpu
        self.step_fn = _cabi.Sg2Step(self.Wgpu, [s["param"] for s in g], [s["exp_avg"] for s in g],
                                     [s["exp_avg_sq"] for s in g], [s["mu"] for s in g], [s["gru"] for s in g],
                                     [s["mamba_fwd"] for s in g], [s["mamba_bwd"] for s in g], self.counts_gpu,
                                     dims=self.dims, debug=True, chunk_len=chunk_len, scan_window=scan_window)
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
            dbg[i] = orc.sg2_step(self.Wnp, self.np[i], g, s, sc, dims=self.odims, precision=precision, chunk_len=chunk_len, window=window,
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
                dm = self.dims["d_model"]
                for d in range(2):
                    ok, r = rel_close(ctx[d, a:b], dbg[i]["ctx"][d][:, :dm], rel, floor)
                    assert ok, "tensor %d: ctx[%d] ratio %.3g" % (i, d, r)
                    assert not dbg[i]["ctx"][d][:, dm:].any(), "tensor %d: embedded context entries must stay zero" % i
            for k in ("param", "exp_avg", "exp_avg_sq", "mu", "gru", "mamba_fwd", "mamba_bwd"):
                got = self.gpu[i][k].detach().cpu()
                want = self.np[i][k]
                if k in ("mamba_fwd", "mamba_bwd"):
                    di, ds = self.dims["d_inner"], self.dims["d_state"]
                    assert not want[di:].any() and not want[:, ds:].any(), "tensor %d: embedded %s entries must stay zero" % (i, k)
                    want = want[:di, :ds]
                if k == "param" and self.dtypes[i] != torch.float32:
                    assert np.array_equal(to_np(got), want), "tensor %d: 16-bit params differ" % i
                    continue
                ok, r = rel_close(got.float().numpy().reshape(want.shape), want, rel, floor)
                worst[k] = max(worst.get(k, 0.0), r)
                assert ok, "tensor %d: %s ratio %.3g" % (i, k, r)
        assert np.array_equal(self.counts_gpu.cpu().numpy(), self.counts_np), "expert_counts differ"
        return worst


per_tensor_scalars, shared_scalars = wl.per_tensor_scalars, wl.shared_scalars
