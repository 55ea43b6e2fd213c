"""Independent float64 restatement of the SuperGrok v2 per-tensor step in
vectorised torch ops, written from the reference's Python statement of the
maths (grokking_optimizers/mamba3_peer_metanet.py:90-160 scan block, :178-192
GRU, :275-370 forward; grokking_optimizers/supergrok2.py:451-464 update).
It shares no code with oracle/sg2_oracle.cpp (which follows the CUDA kernels'
loop structure); the two are compared in test_oracle_sg2.py so that an
indexing or transposition mistake in either shows up.  Small N only: the scan
is a Python loop over timesteps.
"""
import torch

F = torch.float64


def scan_block(x, w, h0):
    """x [N,dm]; w = (in_proj, dt_W, dt_b, B, C, A_log, D, rope, out_proj); h0 [di,ds]."""
    in_proj, dt_W, dt_b, Bp, Cp, A_log, D, rope, out_proj = [t.to(F) for t in w]
    di = dt_W.shape[0]
    xz = x @ in_proj.T
    xb, z = xz[:, :di], xz[:, di:]
    raw = xb @ dt_W.T + dt_b
    dt = torch.where(raw > 20.0, raw, torch.log1p(torch.exp(torch.clamp(raw, max=20.0))))
    B = xb @ Bp.T
    Cm = xb @ Cp.T
    A = -torch.exp(A_log)
    h = h0.to(F).clone()
    ys = []
    for i in range(x.shape[0]):
        dti = dt[i].unsqueeze(-1)
        A_bar = (1.0 + dti * A / 2.0) / (1.0 - dti * A / 2.0 + 1e-8)
        B_bar = dti * B[i].unsqueeze(0)
        ang = dti * rope
        c, s = torch.cos(ang), torch.sin(ang)
        he, ho = h[:, 0::2], h[:, 1::2]
        hr = torch.zeros_like(h)
        hr[:, 0::2] = he * c - ho * s
        hr[:, 1::2] = ho * c + he * s
        h = A_bar * hr + B_bar * xb[i].unsqueeze(-1)
        ys.append((h * Cm[i].unsqueeze(0)).sum(-1))
    y = torch.stack(ys, 0) if ys else torch.zeros(0, di, dtype=F)
    y = y * (z * torch.sigmoid(z)) + D.unsqueeze(0) * xb
    return y @ out_proj.T, h


def scan_block_trace(x, w, h0):
    """What the reference's forward-save kernels keep of a scan (csrc/supergrok2_mamba_peer_backward_kernels.cu:950-1008):
    x-branch, z and dt of every step [N, di] and the state after every step [N, di, ds]."""
    in_proj, dt_W, dt_b, Bp, _, A_log, _, rope, _ = [t.to(F) for t in w]
    di = dt_W.shape[0]
    xz = x @ in_proj.T
    xb, z = xz[:, :di], xz[:, di:]
    raw = xb @ dt_W.T + dt_b
    dt = torch.where(raw > 20.0, raw, torch.log1p(torch.exp(torch.clamp(raw, max=20.0))))
    B = xb @ Bp.T
    A = -torch.exp(A_log)
    h = h0.to(F).clone()
    states = []
    for i in range(x.shape[0]):
        dti = dt[i].unsqueeze(-1)
        A_bar = (1.0 + dti * A / 2.0) / (1.0 - dti * A / 2.0 + 1e-8)
        ang = dti * rope
        c, s = torch.cos(ang), torch.sin(ang)
        he, ho = h[:, 0::2], h[:, 1::2]
        hr = torch.zeros_like(h)
        hr[:, 0::2] = he * c - ho * s
        hr[:, 1::2] = ho * c + he * s
        h = A_bar * hr + dti * B[i].unsqueeze(0) * xb[i].unsqueeze(-1)
        states.append(h)
    return xb, z, dt, torch.stack(states)


def step(weights, param, grad, sharp, ea, easq, mu, gru, mfwd, mbwd, sc, dims):
    """Returns dict of new values (float64) + integer routing results."""
    W = [w.to(F) for w in weights]
    dm, gh, H, pk = dims["d_model"], dims["gru_hidden"], dims["num_heads"], dims["pk_dim"]
    g = grad.reshape(-1).to(F)
    s = sharp.reshape(-1).to(F)
    g = torch.where(torch.isfinite(g), g, torch.zeros_like(g))
    s = torch.where(torch.isfinite(s), s, torch.zeros_like(s))
    N = g.numel()
    perm = torch.sort(g.abs().float(), stable=True).indices
    x = torch.stack([g[perm], s[perm]], -1) @ W[0].T + W[1]
    fo, hf = scan_block(x, W[2:11], mfwd)
    bo, hb = scan_block(x.flip(0), W[11:20], mbwd)
    bo = bo.flip(0)
    unsort = torch.argsort(perm)
    cf, cb = fo[unsort], bo[unsort]
    Wz, bz, Wr, br, Wh, bh = W[20:26]
    xin = torch.cat([g[:, None], s[:, None], cf, cb], -1)
    h = gru.to(F)
    xh = torch.cat([xin, h], -1)
    zg = torch.sigmoid(xh @ Wz.T + bz)
    rg = torch.sigmoid(xh @ Wr.T + br)
    ht = torch.tanh(torch.cat([xin, rg * h], -1) @ Wh.T + bh)
    hn = (1 - zg) * h + zg * ht
    pin = torch.cat([hn, cf, cb, g[:, None], s[:, None]], -1)
    total = torch.zeros(N, dtype=F)
    eidx = torch.zeros(N, H, dtype=torch.int64)
    W1, b1, W2, b2 = W[29], W[30], W[31], W[32]
    for hh in range(H):
        q = pin @ W[26][hh].T
        ia = (q[:, : dm // 2] @ W[27][hh].T).argmax(-1)
        ib = (q[:, dm // 2:] @ W[28][hh].T).argmax(-1)
        e = torch.clamp(ia * pk + ib, max=W1.shape[0] - 1)     # csrc/supergrok2_mamba_peer_kernels.cu:1050-1051
        eidx[:, hh] = e
        zz = torch.relu(W1[e] * g[:, None] + b1[e])
        total = total + (W2[e] * zz).sum(-1) + b2[e]
    smart = g + sc["rescale"] * total / H
    mu_n = sc["alpha"] * mu.to(F) + (1 - sc["alpha"]) * g
    fg = smart + sc["lamb_eff"] * mu_n
    ea_n = sc["beta1"] * ea.to(F) + (1 - sc["beta1"]) * fg
    easq_n = sc["beta2"] * easq.to(F) + (1 - sc["beta2"]) * fg * fg
    denom = (easq_n / sc["bc2"]).sqrt() + sc["eps"]
    p_n = param.reshape(-1).to(F) * (1 - sc["lr"] * sc["wd_eff"]) - (sc["lr"] / sc["bc1"]) * ea_n / denom
    return dict(param=p_n, exp_avg=ea_n, exp_avg_sq=easq_n, mu=mu_n, gru=hn, mamba_fwd=hf, mamba_bwd=hb,
                perm=perm, expert_idx=eidx, ctx_f=cf, ctx_b=cb, smart=smart)


def forward_for_bilevel(W, grad, sharp, gru, mfwd, mbwd, rescale, dims, topk=4):
    """Differentiable forward with soft top-k routing (grokking_optimizers/mamba3_peer_metanet.py:372-436 of the
    reference): softmax of 10 x the k best scores of each sub-key, k*k experts per head weighted by the product.
    W: the 33 weight tensors in `_ops` argument order (float64, may require grad).
    Returns (smart_grad, new_gru, new_mamba_fwd, new_mamba_bwd)."""
    dm, H, pk = dims["d_model"], dims["num_heads"], dims["pk_dim"]
    g, s = grad.reshape(-1).to(F), sharp.reshape(-1).to(F)
    N = g.numel()
    perm = torch.sort(g.abs().float(), stable=True).indices
    x = torch.stack([g[perm], s[perm]], -1) @ W[0].T + W[1]
    fo, new_f = scan_block(x, W[2:11], mfwd)
    bo, new_b = scan_block(x.flip(0), W[11:20], mbwd)
    unsort = torch.argsort(perm)
    cf, cb = fo[unsort], bo.flip(0)[unsort]
    Wz, bz, Wr, br, Wh, bh = W[20:26]
    h = gru.to(F)
    xin = torch.cat([g[:, None], s[:, None], cf, cb], -1)
    xh = torch.cat([xin, h], -1)
    z, r = torch.sigmoid(xh @ Wz.T + bz), torch.sigmoid(xh @ Wr.T + br)
    hn = (1 - z) * h + z * torch.tanh(torch.cat([xin, r * h], -1) @ Wh.T + bh)
    pin = torch.cat([hn, cf, cb, g[:, None], s[:, None]], -1)
    W1, b1, W2, b2 = W[29], W[30], W[31], W[32]
    total = torch.zeros(N, dtype=F)
    for hh in range(H):
        q = pin @ W[26][hh].T
        va, ia = (q[:, : dm // 2] @ W[27][hh].T).topk(topk, dim=-1)
        vb, ib = (q[:, dm // 2:] @ W[28][hh].T).topk(topk, dim=-1)
        sa, sb = torch.softmax(va * 10.0, -1), torch.softmax(vb * 10.0, -1)
        idx = (ia.unsqueeze(2) * pk + ib.unsqueeze(1)).reshape(N, -1)
        rw = (sa.unsqueeze(2) * sb.unsqueeze(1)).reshape(N, -1)
        zz = torch.relu(W1[idx] * g[:, None, None] + b1[idx])
        out = (W2[idx] * zz).sum(-1) + b2[idx]
        total = total + (rw * out).sum(1)
    return g + rescale * total / H, hn, new_f, new_b
