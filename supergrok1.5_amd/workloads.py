"""Synthetic parameter sets and meta-weights for the measured configurations.

Everything is drawn on the CPU from seeded torch generators so that the
device path and a CPU checker can be handed identical bits.
"""
import math

import numpy as np
import torch

DEFAULT_DIMS = dict(d_model=8, d_state=16, d_inner=16, gru_hidden=4, num_heads=4, pk_dim=12,
                    expert_hidden=16, num_experts=144)

META_WEIGHT_NAMES = (
    "input_proj_W", "input_proj_b",
    "mamba_fwd_in_proj", "mamba_fwd_dt_W", "mamba_fwd_dt_b", "mamba_fwd_B_proj", "mamba_fwd_C_proj",
    "mamba_fwd_A_log", "mamba_fwd_D", "mamba_fwd_rope", "mamba_fwd_out_proj",
    "mamba_bwd_in_proj", "mamba_bwd_dt_W", "mamba_bwd_dt_b", "mamba_bwd_B_proj", "mamba_bwd_C_proj",
    "mamba_bwd_A_log", "mamba_bwd_D", "mamba_bwd_rope", "mamba_bwd_out_proj",
    "gru_Wz", "gru_bz", "gru_Wr", "gru_br", "gru_Wh", "gru_bh",
    "peer_query_Ws", "prod_keys_A", "prod_keys_B",
    "expert_W1", "expert_b1", "expert_W2", "expert_b2",
)


def meta_weight_shapes(dims=None):
    d = dict(DEFAULT_DIMS if dims is None else dims)
    dm, ds, di, gh = d["d_model"], d["d_state"], d["d_inner"], d["gru_hidden"]
    H, pk, eh, E = d["num_heads"], d["pk_dim"], d["expert_hidden"], d["num_experts"]
    grl, pin = 2 + 2 * dm + gh, gh + 2 * dm + 2
    mamba = [(2 * di, dm), (di, di), (di,), (ds, di), (ds, di), (di, ds), (di,), (di, ds // 2), (dm, di)]
    return ([(dm, 2), (dm,)] + mamba + mamba +
            [(gh, grl), (gh,), (gh, grl), (gh,), (gh, grl), (gh,)] +
            [(H, dm, pin), (H, pk, dm // 2), (H, pk, dm // 2)] +
            [(E, eh), (E, eh), (E, eh), (E,)])


def meta_weights(seed=7, dims=None, std=0.1):
    """The 33 meta-net weight tensors, N(0, std), drawn in the argument order
    of supergrok2_mamba_peer_batched_step."""
    gen = torch.Generator().manual_seed(seed)
    return [torch.randn(*s, generator=gen, dtype=torch.float32) * std for s in meta_weight_shapes(dims)]


def shared14_shapes():
    """Parameter set of a 2-layer transformer for modular addition p=97
    (d_model 128, 4 heads, MLP 512, vocab 99): 14 tensors, 420 195 elements."""
    layer = [(384, 128), (128, 128), (512, 128), (512,), (128, 512)]
    return [(99, 128), (4, 128)] + layer + layer + [(99, 128), (99,)]


def scale50_shapes():
    """50 tensors, log-uniform sizes from 64 to 4M elements (~25M total)."""
    shapes = []
    for i in range(50):
        n = min(4194304, int(round(1.377 * 64 * 65536 ** ((i + 0.5) / 50))))
        if n < 4096:
            shapes.append((n,))
        else:
            cols = 2 ** int(math.floor(math.log2(math.sqrt(n))))
            rows = max(1, int(round(n / cols)))
            shapes.append((rows, cols))
    return shapes


def small8_shapes():
    """All tensors below 256 elements (the reference's sequential-scan regime)."""
    return [(1,), (4,), (16,), (64,), (99,), (128,), (200,), (255,)]


def numel(shape):
    n = 1
    for s in shape:
        n *= s
    return n


def make_params(shapes, seed=0, std=0.02):
    gen = torch.Generator().manual_seed(seed)
    return [torch.randn(*s, generator=gen, dtype=torch.float32) * std for s in shapes]


def make_grads(shapes, seed, std=1e-3, tail_frac=0.0, tail="normal", tail_scale=1e-1):
    """N(0,std) gradients; optionally a Bernoulli(tail_frac) mask replaces
    entries by a heavy tail: 'normal' -> N(0,tail_scale), 'student3' ->
    std * Student-t(nu=3)."""
    gen = torch.Generator().manual_seed(seed)
    out = []
    for s in shapes:
        g = torch.randn(*s, generator=gen, dtype=torch.float32) * std
        if tail_frac > 0:
            mask = torch.rand(*s, generator=gen) < tail_frac
            if tail == "normal":
                t = torch.randn(*s, generator=gen, dtype=torch.float32) * tail_scale
            else:
                z = torch.randn(*s, generator=gen, dtype=torch.float64)
                chi = torch.randn(3, *s, generator=gen, dtype=torch.float64).pow(2).sum(0)
                t = (std * z / torch.sqrt(chi / 3.0)).float()
            g = torch.where(mask, t, g)
        out.append(g)
    return out


def clip_per_tensor(grads, max_norm=1.0):
    """Per-tensor norm clip as done by the optimizer class before the step."""
    out = []
    for g in grads:
        n = g.norm()
        out.append(g * (max_norm / (n + 1e-12)) if n > max_norm else g)
    return out


def per_tensor_scalars(P, step, lamb_eff=0.0):
    """Per-tensor scalars of optimizer step `step` as the optimizer class derives them (alpha 0.98, beta1_i =
    0.9 * 0.9^i, bias corrections), rounded to fp32 as they cross the extension boundary."""
    out = []
    for i in range(P):
        b1 = float(np.float32(0.9 * 0.9 ** i))
        out.append(dict(alpha=float(np.float32(0.98)), lamb_eff=float(np.float32(lamb_eff)), beta1=b1,
                        bc1=float(np.float32(1.0 - b1 ** step)), bc2=float(np.float32(1.0 - 0.999 ** step))))
    return out


def shared_scalars(wd_eff=1.0, rescale=0.1):
    f = lambda v: float(np.float32(v))
    return dict(rescale=f(rescale), beta2=f(0.999), lr=f(1e-3), wd_eff=f(wd_eff), eps=f(1e-8))


def module_weights(seed=0):
    """The 33 meta-net weight tensors as Mamba3PEERMetaNet() initialises them (the reference's initialisation:
    A_log = log(1..16), default nn.Linear weights, keys and experts N(0, 0.02)), in `_ops` argument order."""
    from grokking_optimizers import Mamba3PEERMetaNet
    state = torch.random.get_rng_state()
    torch.manual_seed(seed)
    try:
        mn = Mamba3PEERMetaNet()
    finally:
        torch.random.set_rng_state(state)
    return [w.clone() for w in mn.flat_weights()]
