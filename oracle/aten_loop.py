"""TEST INFRASTRUCTURE ONLY: the SuperGrok v2 per-tensor step the way the reference's CPU path runs it -- the
per-timestep Python loop of Mamba3ScanBlock.forward (grokking_optimizers/mamba3_peer_metanet.py:90-160 of the
reference: about twenty ATen calls per timestep and direction), then GRU, hard top-1 PEER routing and the expert MLPs
as whole-tensor ATen ops (:178-192, :319-367) and the update of grokking_optimizers/supergrok2.py:451-464 -- in fp32
torch on the host.  (The reference's own file does not run on this torch: it calls torch.softplus, which does not
exist; softplus is written out here as the reference's CUDA kernel writes it.)

Used by bench.py's cpu_baseline leg only, as a timed baseline on small tensors, and pinned against the float64
policy of the C++ checker in tests/test_oracle_elem.py::test_aten_loop_matches_checker.  Nothing shipped imports it."""
import torch


def scan_block(x, w, h0):
    in_proj, dt_W, dt_b, Bp, Cp, A_log, D, rope, out_proj = w
    di = dt_W.shape[0]
    A = -torch.exp(A_log)
    h = h0.clone()
    outs = []
    for i in range(x.shape[0]):
        xz = in_proj @ x[i]
        xb, z = xz[:di], xz[di:]
        raw = dt_W @ xb + dt_b
        dt = torch.where(raw > 20.0, raw, torch.log1p(torch.exp(torch.clamp(raw, max=20.0)))).unsqueeze(-1)
        Bv, Cv = Bp @ xb, Cp @ xb
        A_bar = (1.0 + dt * A / 2.0) / (1.0 - dt * A / 2.0 + 1e-8)
        ang = dt * rope
        c, s = torch.cos(ang), torch.sin(ang)
        he, ho = h[:, 0::2], h[:, 1::2]
        hr = torch.empty_like(h)
        hr[:, 0::2] = he * c - ho * s
        hr[:, 1::2] = ho * c + he * s
        h = A_bar * hr + (dt * Bv.unsqueeze(0)) * xb.unsqueeze(-1)
        y = (h * Cv.unsqueeze(0)).sum(-1)
        outs.append(out_proj @ (y * (z * torch.sigmoid(z)) + D * xb))
    return torch.stack(outs, 0), h


def step(W, st, grad, sharp, sc, dims):
    """One step on one tensor, in place on the dict `st` (param, exp_avg, exp_avg_sq, mu, gru [N, gh], mamba_fwd,
    mamba_bwd: fp32 torch tensors).  W: the 33 weight tensors in `_ops` order.  Returns the expert indices [N, H]."""
    dm, H, pk = dims["d_model"], dims["num_heads"], dims["pk_dim"]
    g = torch.where(torch.isfinite(grad), grad, torch.zeros_like(grad)).reshape(-1)
    s = torch.where(torch.isfinite(sharp), sharp, torch.zeros_like(sharp)).reshape(-1)
    perm = torch.sort(g.abs(), stable=True).indices
    x = torch.stack([g[perm], s[perm]], -1) @ W[0].T + W[1]
    fo, st["mamba_fwd"] = scan_block(x, W[2:11], st["mamba_fwd"])
    bo, st["mamba_bwd"] = scan_block(x.flip(0), W[11:20], st["mamba_bwd"])
    unsort = torch.argsort(perm)
    cf, cb = fo[unsort], bo.flip(0)[unsort]
    Wz, bz, Wr, br, Wh, bh = W[20:26]
    xin = torch.cat([g[:, None], s[:, None], cf, cb], -1)
    h = st["gru"]
    xh = torch.cat([xin, h], -1)
    zg, rg = torch.sigmoid(xh @ Wz.T + bz), torch.sigmoid(xh @ Wr.T + br)
    hn = (1 - zg) * h + zg * torch.tanh(torch.cat([xin, rg * h], -1) @ Wh.T + bh)
    st["gru"] = hn
    pin = torch.cat([hn, cf, cb, g[:, None], s[:, None]], -1)
    W1, b1, W2, b2 = W[29], W[30], W[31], W[32]
    total = torch.zeros_like(g)
    eidx = []
    for hh in range(H):
        q = pin @ W[26][hh].T
        e = (q[:, :dm // 2] @ W[27][hh].T).argmax(-1) * pk + (q[:, dm // 2:] @ W[28][hh].T).argmax(-1)
        e = torch.clamp(e, max=W1.shape[0] - 1)
        eidx.append(e)
        total = total + (W2[e] * torch.relu(W1[e] * g[:, None] + b1[e])).sum(-1) + b2[e]
    smart = g + sc["rescale"] * total / H
    st["mu"] = sc["alpha"] * st["mu"] + (1 - sc["alpha"]) * g
    fg = smart + sc["lamb_eff"] * st["mu"]
    st["exp_avg"] = sc["beta1"] * st["exp_avg"] + (1 - sc["beta1"]) * fg
    st["exp_avg_sq"] = sc["beta2"] * st["exp_avg_sq"] + (1 - sc["beta2"]) * fg * fg
    denom = (st["exp_avg_sq"] / sc["bc2"]).sqrt() + sc["eps"]
    st["param"] = st["param"] * (1 - sc["lr"] * sc["wd_eff"]) - (sc["lr"] / sc["bc1"]) * st["exp_avg"] / denom
    return torch.stack(eidx, -1)
