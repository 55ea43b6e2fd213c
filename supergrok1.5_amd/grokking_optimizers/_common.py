"""Argument checks and per-parameter state shared by the Adam-family optimizer classes."""
import torch


def check_hyper(lr=None, eps=None, betas=None):
    if lr is not None and lr < 0.0:
        raise ValueError(f"Invalid learning rate: {lr}")
    if eps is not None and eps < 0.0:
        raise ValueError(f"Invalid epsilon value: {eps}")
    if betas is not None:
        for k in (0, 1):
            if not 0.0 <= betas[k] < 1.0:
                raise ValueError(f"Invalid beta parameter at index {k}: {betas[k]}")


def check_ranges(checks):
    """checks: (name, value, lowest, upper bound or None); lowest <= value (< upper) or ValueError("Invalid <name>: <value>")."""
    for name, value, low, high in checks:
        if value < low or (high is not None and not value < high):
            raise ValueError(f"Invalid {name}: {value}")


def run_closure(closure):
    if closure is None:
        return None
    with torch.enable_grad():
        return closure()


def gather(optimizer, group, buffers, count_steps=True, extra_init=None):
    """Parameters of `group` that have a gradient, with their fp32 state buffers (created as zeros on
    first use) and step counters (incremented here when count_steps)."""
    out = {"params": [], "grads": [], "steps": []}
    for b in buffers:
        out[b] = []
    for p in group["params"]:
        if p.grad is None:
            continue
        st = optimizer.state[p]
        if len(st) == 0:
            st["step"] = 0
            for b in buffers:
                st[b] = torch.zeros_like(p, dtype=torch.float32)
            if extra_init is not None:
                extra_init(p, st)
        if count_steps:
            st["step"] += 1
        out["params"].append(p)
        out["grads"].append(p.grad)
        out["steps"].append(st["step"])
        for b in buffers:
            out[b].append(st[b])
    return out
