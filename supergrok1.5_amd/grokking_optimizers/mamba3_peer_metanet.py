"""Parameter container of the SuperGrok v2 meta-network: bidirectional Mamba-3
scan blocks, per-element GRU, 4-head PEER product-key router and the expert
pool.  Same sub-module / parameter names, shapes and initialisation as the
reference (grokking_optimizers/mamba3_peer_metanet.py:44-269), so state dicts
are interchangeable; `get_weights` (:515-567 there) exports the tensors in the
layout the fused step consumes, and `_recycle_dead_experts` (:437-491 there)
is the host-side expert recycling.

The arithmetic of the network runs inside the fused HIP step
(`_ops.supergrok2_mamba_peer_batched_step`).  `forward` (:275-370 there) and
`forward_for_bilevel` (:372-436 there, soft top-4 routing) are kept for callers
that use the module outside the optimizer and run on the same kernels:
`forward` is one call of the library's forward-only entry point
(sg2_meta_forward: sort, scan, GRU, routing, experts), `forward_for_bilevel`
is differentiable through two autograd Functions over the bilevel kernels (scan
forward / adjoint, per-element forward / backward).  GPU tensors only.
The sub-modules' own forwards (Mamba3ScanBlock on an arbitrary sequence,
MiniGRU) are plain torch operations for callers that use them on their own.
"""
import math

import torch
import torch.nn as nn
import torch.nn.functional as F


class Mamba3ScanBlock(nn.Module):
    def __init__(self, d_model: int = 8, d_state: int = 16, expand: int = 2):
        super().__init__()
        assert d_state % 2 == 0, "d_state must be even for paired RoPE"
        self.d_model, self.d_state, self.d_inner = d_model, d_state, d_model * expand
        di = self.d_inner
        self.in_proj = nn.Linear(d_model, 2 * di, bias=False)
        self.dt_proj = nn.Linear(di, di, bias=True)
        self.B_proj = nn.Linear(di, d_state, bias=False)
        self.C_proj = nn.Linear(di, d_state, bias=False)
        self.A_log = nn.Parameter(torch.log(torch.linspace(1, d_state, d_state)).unsqueeze(0).repeat(di, 1))
        self.D = nn.Parameter(torch.ones(di))
        self.rope_freq = nn.Parameter(torch.randn(di, d_state // 2) * 0.01)
        self.out_proj = nn.Linear(di, d_model, bias=False)

    def export(self):
        f = lambda t: t.detach().float().contiguous()
        return [f(self.in_proj.weight), f(self.dt_proj.weight), f(self.dt_proj.bias), f(self.B_proj.weight),
                f(self.C_proj.weight), f(self.A_log), f(self.D), f(self.rope_freq), f(self.out_proj.weight)]

    def forward(self, x, initial_state=None):
        """One scan block on an arbitrary input sequence x [N, d_model] (reference: mamba3_peer_metanet.py:90-160):
        returns (output [N, d_model], final state [d_inner, d_state]).  Torch operations on x's device,
        differentiable: a utility for callers that use the block on its own, and the scan of the bilevel pass for
        blocks larger than its kernels are built for.  The optimizer's step never comes here (its scan runs in the
        fused kernels, where the input is the two-number feature (g, s) of an element).

        Every coefficient of the recurrence is formed for all steps at once; the 2 x 2 state update is then walked
        in chunks, all chunks side by side: first every chunk's affine map state-in -> state-out (three walks from
        (1, 0), (0, 1) and 0 + the drive, batched), then the chunk start states one after the other, then every
        chunk from its start state.  About 2 sqrt(N) batched steps instead of N; memory grows with
        N * d_inner * d_state."""
        n = x.shape[0]
        h0 = (torch.zeros(self.d_inner, self.d_state, device=x.device, dtype=x.dtype) if initial_state is None
              else initial_state.to(x.dtype))
        if n == 0:
            return x.new_zeros(0, self.d_model), h0
        xb, z = self.in_proj(x).chunk(2, dim=-1)
        dt = F.softplus(self.dt_proj(xb)).unsqueeze(-1)                       # [N, di, 1]
        half = 0.5 * dt * -torch.exp(self.A_log)                               # dt A / 2
        a_bar = (1.0 + half) / (1.0 - half + 1e-8)                             # [N, di, ds]
        drive = dt * self.B_proj(xb).unsqueeze(1) * xb.unsqueeze(-1)           # dt B x
        ang = dt * self.rope_freq                                              # [N, di, ds/2]
        cs, sn = torch.cos(ang), torch.sin(ang)

        length = max(1, int(math.isqrt(n)))                                    # steps per chunk
        chunks = (n + length - 1) // length
        pad = chunks * length - n

        def by_chunk(t, fill):                                                 # [N, ...] -> [length, chunks, ...]
            if pad:
                t = torch.cat([t, t.new_full((pad,) + tuple(t.shape[1:]), fill)])
            return t.reshape(chunks, length, *t.shape[1:]).transpose(0, 1)
        a_c, d_c, cs_c, sn_c = by_chunk(a_bar, 1.0), by_chunk(drive, 0.0), by_chunk(cs, 1.0), by_chunk(sn, 0.0)

        def advance(h, k, driven):                                             # one step of all chunks: h [..., chunks, di, ds]
            he, ho = h[..., 0::2], h[..., 1::2]
            rot = torch.stack([he * cs_c[k] - ho * sn_c[k], ho * cs_c[k] + he * sn_c[k]], dim=-1).flatten(-2)
            return a_c[k] * rot + driven

        shape = (chunks, self.d_inner, self.d_state)
        if chunks > 1:
            # affine map of every chunk: the responses to an even unit state, an odd unit state, and the drive alone
            basis = x.new_zeros(3, *shape)
            basis[0, ..., 0::2] = 1.0
            basis[1, ..., 1::2] = 1.0
            only_third = x.new_zeros(3, 1, 1, 1)
            only_third[2] = 1.0
            for k in range(length):
                basis = advance(basis, k, only_third * d_c[k])
            starts = [h0]
            for c in range(chunks - 1):
                he = starts[-1][:, 0::2].repeat_interleave(2, dim=-1)          # each pair's even / odd entry, at both places
                ho = starts[-1][:, 1::2].repeat_interleave(2, dim=-1)
                starts.append(basis[0, c] * he + basis[1, c] * ho + basis[2, c])
            h = torch.stack(starts)
        else:
            h = h0.unsqueeze(0)
        states = []
        for k in range(length):
            h = advance(h, k, d_c[k])
            states.append(h)
        states = torch.stack(states).transpose(0, 1).reshape(chunks * length, self.d_inner, self.d_state)[:n]
        y = (states * self.C_proj(xb).unsqueeze(1)).sum(-1)
        return self.out_proj(y * F.silu(z) + self.D * xb), states[n - 1]


class MiniGRU(nn.Module):
    def __init__(self, input_dim: int, hidden_dim: int = 4):
        super().__init__()
        self.hidden_dim = hidden_dim
        self.W_z = nn.Linear(input_dim + hidden_dim, hidden_dim)
        self.W_r = nn.Linear(input_dim + hidden_dim, hidden_dim)
        self.W_h = nn.Linear(input_dim + hidden_dim, hidden_dim)

    def forward(self, x, h):
        """New hidden state [N, hidden] from inputs x [N, input_dim] and state h (reference:
        mamba3_peer_metanet.py:178-192): update gate z, reset gate r, candidate from [x, r * h].  Torch operations,
        for callers that use the cell on its own; the fused step evaluates the same cell per element in HIP."""
        both = torch.cat([x, h], dim=-1)
        z, r = torch.sigmoid(self.W_z(both)), torch.sigmoid(self.W_r(both))
        cand = torch.tanh(self.W_h(torch.cat([x, r * h], dim=-1)))
        return (1 - z) * h + z * cand


class Mamba3PEERMetaNet(nn.Module):
    def __init__(self, d_model: int = 8, d_state: int = 16, mamba_expand: int = 2, num_peer_heads: int = 4,
                 num_experts: int = 144, expert_hidden: int = 16, gru_hidden: int = 4, rescale: float = 0.1,
                 recycle_interval: int = 100, recycle_threshold: float = 0.001):
        super().__init__()
        self.d_model, self.d_state = d_model, d_state
        self.num_peer_heads, self.num_experts = num_peer_heads, num_experts
        self.expert_hidden, self.gru_hidden = expert_hidden, gru_hidden
        self.rescale = rescale
        self.recycle_interval, self.recycle_threshold = recycle_interval, recycle_threshold
        self.pk_dim = int(math.sqrt(num_experts))
        assert self.pk_dim * self.pk_dim == num_experts, f"num_experts must be perfect square, got {num_experts}"
        self.input_proj = nn.Linear(2, d_model, bias=True)
        self.mamba_fwd = Mamba3ScanBlock(d_model, d_state, mamba_expand)
        self.mamba_bwd = Mamba3ScanBlock(d_model, d_state, mamba_expand)
        self.gru = MiniGRU(2 + 2 * d_model, gru_hidden)
        peer_in = gru_hidden + 2 * d_model + 2
        self.peer_queries = nn.ModuleList([nn.Linear(peer_in, d_model, bias=False) for _ in range(num_peer_heads)])
        mk_keys = lambda: nn.ParameterList([nn.Parameter(torch.randn(self.pk_dim, d_model // 2) * 0.02)
                                            for _ in range(num_peer_heads)])
        self.product_keys_A = mk_keys()
        self.product_keys_B = mk_keys()
        self.expert_W1 = nn.Parameter(torch.randn(num_experts, expert_hidden, 1) * 0.02)
        self.expert_b1 = nn.Parameter(torch.zeros(num_experts, expert_hidden))
        self.expert_W2 = nn.Parameter(torch.randn(num_experts, 1, expert_hidden) * 0.02)
        self.expert_b2 = nn.Parameter(torch.zeros(num_experts, 1))
        self.register_buffer("expert_counts", torch.zeros(num_experts, dtype=torch.int32))
        self.register_buffer("step_counter", torch.tensor(0, dtype=torch.long))

    def get_weights(self):
        f = lambda t: t.detach().float().contiguous()
        names = ("in_proj", "dt_proj_W", "dt_proj_b", "B_proj", "C_proj", "A_log", "D", "rope_freq", "out_proj")
        w = {"input_proj_W": f(self.input_proj.weight), "input_proj_b": f(self.input_proj.bias)}
        for tag, blk in (("fwd", self.mamba_fwd), ("bwd", self.mamba_bwd)):
            w.update({f"mamba_{tag}_{n}": t for n, t in zip(names, blk.export())})
        for g, lin in (("z", self.gru.W_z), ("r", self.gru.W_r), ("h", self.gru.W_h)):
            w[f"gru_W_{g}"], w[f"gru_b_{g}"] = f(lin.weight), f(lin.bias)
        w["peer_queries"] = [f(q.weight) for q in self.peer_queries]
        w["product_keys_A"] = [f(k) for k in self.product_keys_A]
        w["product_keys_B"] = [f(k) for k in self.product_keys_B]
        for n in ("expert_W1", "expert_b1", "expert_W2", "expert_b2"):
            w[n] = f(getattr(self, n))
        w.update(rescale=self.rescale, d_model=self.d_model, d_state=self.d_state, d_inner=self.mamba_fwd.d_inner,
                 pk_dim=self.pk_dim, expert_hidden=self.expert_hidden, gru_hidden=self.gru_hidden,
                 num_peer_heads=self.num_peer_heads, num_experts=self.num_experts)
        return w

    def forward(self, grad, sharpness, gru_state, mamba_fwd_state=None, mamba_bwd_state=None):
        """(smart_grad, new_gru_state, new_mamba_fwd_state, new_mamba_bwd_state) with the step's hard top-1 routing;
        in training mode the winners are added to expert_counts, as in the reference (:342-348 there)."""
        from grokking_optimizers import _bilevel
        return _bilevel.forward(self, grad, sharpness, gru_state, mamba_fwd_state, mamba_bwd_state)

    def forward_for_bilevel(self, grad, sharpness, gru_state, mamba_fwd_state=None, mamba_bwd_state=None):
        """(smart_grad, new_gru_state, new_mamba_fwd_state, new_mamba_bwd_state), differentiable with respect to
        every parameter of the module; GPU tensors only."""
        from grokking_optimizers import _bilevel
        return _bilevel.forward_for_bilevel(self, grad, sharpness, gru_state, mamba_fwd_state, mamba_bwd_state)

    @property
    def has_cuda_bilevel(self):
        """Whether the device kernels of the bilevel pass can serve this module (reference: :493-496): they are part
        of the library, so whenever the parameters live on the GPU."""
        return next(self.parameters()).is_cuda

    def forward_for_bilevel_cuda(self, grad, sharpness, gru_state, mamba_fwd_state=None, mamba_bwd_state=None):
        """The reference's name for the bilevel forward with device kernels behind it (:498-513 there):
        forward_for_bilevel already is that."""
        return self.forward_for_bilevel(grad, sharpness, gru_state, mamba_fwd_state, mamba_bwd_state)

    def flat_weights(self):
        """The 33 tensors in the argument order of _ops.supergrok2_mamba_peer_batched_step."""
        w = self.get_weights()
        out = [w["input_proj_W"], w["input_proj_b"]]
        for tag in ("fwd", "bwd"):
            out += [w[f"mamba_{tag}_{n}"] for n in ("in_proj", "dt_proj_W", "dt_proj_b", "B_proj", "C_proj", "A_log",
                                                    "D", "rope_freq", "out_proj")]
        out += [w["gru_W_z"], w["gru_b_z"], w["gru_W_r"], w["gru_b_r"], w["gru_W_h"], w["gru_b_h"]]
        out += [torch.stack(w["peer_queries"]), torch.stack(w["product_keys_A"]), torch.stack(w["product_keys_B"])]
        E = self.num_experts
        out += [w["expert_W1"].reshape(E, -1), w["expert_b1"], w["expert_W2"].reshape(E, -1), w["expert_b2"].reshape(-1)]
        return out

    @torch.no_grad()
    def load_flat_weights(self, weights):
        """Inverse of flat_weights: copies 33 tensors in `_ops` argument order into the module's parameters."""
        W = list(weights)
        assert len(W) == 33
        self.input_proj.weight.copy_(W[0])
        self.input_proj.bias.copy_(W[1])
        for base, blk in ((2, self.mamba_fwd), (11, self.mamba_bwd)):
            for k, prm in enumerate((blk.in_proj.weight, blk.dt_proj.weight, blk.dt_proj.bias, blk.B_proj.weight,
                                     blk.C_proj.weight, blk.A_log, blk.D, blk.rope_freq, blk.out_proj.weight)):
                prm.copy_(W[base + k].reshape(prm.shape))
        for k, lin in enumerate((self.gru.W_z, self.gru.W_r, self.gru.W_h)):
            lin.weight.copy_(W[20 + 2 * k])
            lin.bias.copy_(W[21 + 2 * k])
        for h in range(self.num_peer_heads):
            self.peer_queries[h].weight.copy_(W[26][h])
            self.product_keys_A[h].copy_(W[27][h])
            self.product_keys_B[h].copy_(W[28][h])
        for k, name in enumerate(("expert_W1", "expert_b1", "expert_W2", "expert_b2")):
            prm = getattr(self, name)
            prm.copy_(W[29 + k].reshape(prm.shape))

    @torch.no_grad()
    def _recycle_dead_experts(self):
        """Experts with fewer than recycle_threshold of the activations are replaced by a noisy clone of
        an expert sampled in proportion to its count; a product key is re-drawn only when every expert
        sharing it is dead.  Returns True if anything changed.  Random draws, in order: one multinomial,
        then per dead expert (ascending index) W1, b1, W2, b2 noise, then key A redraws per head, then
        key B redraws per head -- the sequence of the reference (mamba3_peer_metanet.py:453-488)."""
        total = self.expert_counts.sum().item()
        if total == 0:
            return False
        dead = (self.expert_counts.float() / total) < self.recycle_threshold
        if not dead.any():
            self.expert_counts.zero_()
            return False
        top = torch.multinomial(self.expert_counts.float(), 1).item()
        pk, H = self.pk_dim, self.num_peer_heads
        for i in dead.nonzero(as_tuple=True)[0].tolist():
            for name in ("expert_W1", "expert_b1", "expert_W2", "expert_b2"):
                t = getattr(self, name).data
                t[i] = t[top] + 0.01 * torch.randn_like(t[i])
            a, b = divmod(i, pk)
            if dead[a * pk:(a + 1) * pk].all():
                for h in range(H):
                    row = self.product_keys_A[h].data[a]
                    self.product_keys_A[h].data[a] = torch.randn_like(row) * 0.02
            cols = torch.arange(0, self.num_experts, pk, device=dead.device) + b
            if dead[cols[cols < self.num_experts]].all():
                for h in range(H):
                    row = self.product_keys_B[h].data[b]
                    self.product_keys_B[h].data[b] = torch.randn_like(row) * 0.02
        self.expert_counts.zero_()
        return True
