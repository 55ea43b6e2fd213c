"""TEST INFRASTRUCTURE - CPU restatement of the reference's remaining fused
optimizer steps.  Only tests/, the smoke check and bench.py's CPU baseline may
import this module; the product never does.

Each function restates, in numpy float32 arithmetic (reductions in float64),
what the corresponding host function of the reference's csrc/ops.cpp computes:

  clip_coef              clip_grad_norms_device_side          ops.cpp:23-55
  grokadamw_step         grokadamw_fused_step                 ops.cpp:311-353
  neuralgrok_step        neuralgrok_fused_step                ops.cpp:360-417
  prodigy_step           prodigy_fused_step                   ops.cpp:424-506
  lion_step              lion_fused_step                      ops.cpp:536-560
  sg11_step              supergrok11_fused_step               ops.cpp:209-288
  sg2_clip               SuperGrok2.step pre-pass             grokking_optimizers/supergrok2.py:316-321
  looksam_perturb        looksam_perturb_all                  ops.cpp:566-590
  looksam_directions     looksam_compute_directions           ops.cpp:607-630
  looksam_adjust         looksam_adjust_grads                 ops.cpp:632-652

Pinned by tests/golden/ref_family.npz, which holds inputs and outputs of the
reference's own CPU code for every ops.cpp function above
(tests/test_oracle_family.py); sg2_clip, which restates Python, is pinned there
against the same three torch expressions evaluated by torch on the CPU.
Tensors are lists of 1-D float32 arrays and are updated in place, like the
reference updates its tensor lists.
"""
import math

import numpy as np

F = np.float32


def _norm(xs):
    """sqrt of the sum of squares over a list of arrays, accumulated in float64, returned as float32."""
    return F(math.sqrt(sum(float(np.dot(x.astype(np.float64), x.astype(np.float64))) for x in xs if x.size)))


def clip_coef(grads, clip):
    """Global-norm clipping: returns the factor the gradients are multiplied by (1 when inactive)."""
    if not clip > 0:
        return F(1.0)
    n = _norm(grads)
    return F(clip) / (n + F(1e-6)) if n > F(clip) else F(1.0)


def _clip_in_place(grads, clip):
    c = clip_coef(grads, clip)
    if c != F(1.0):
        for g in grads:
            g *= c


def _adam(p, ea, easq, g, beta1, beta2, lr, wd, eps, bc1, bc2):
    beta1, beta2 = F(beta1), F(beta2)
    ea[:] = ea * beta1 + (F(1) - beta1) * g
    easq[:] = easq * beta2 + (F(1) - beta2) * g * g
    denom = np.sqrt(easq / F(bc2)) + F(eps)
    p *= F(1) - F(lr) * F(wd)
    p -= (F(lr) / F(bc1)) * ea / denom


def _bc(beta, step):
    return F(1) - F(np.power(F(beta), F(step)))


def grokadamw_step(params, grads, eas, easqs, emas, steps, alpha, lamb, beta1, beta2, lr, wd, eps, clip):
    _clip_in_place(grads, clip)
    for p, g, ea, easq, ema, st in zip(params, grads, eas, easqs, emas, steps):
        if g.size == 0:
            continue
        ema[:] = ema * F(alpha) + (F(1) - F(alpha)) * g
        amp = g + F(lamb) * ema
        _adam(p, ea, easq, amp, beta1, beta2, lr, wd, eps, _bc(beta1, st), _bc(beta2, st))


def neuralgrok_step(params, grads, eas, easqs, steps, W1, b1, W2, b2, alpha_amp, beta_amp, beta1, beta2, lr, wd, eps, clip):
    _clip_in_place(grads, clip)
    w1, w2 = W1.reshape(-1).astype(F), W2.reshape(-1).astype(F)
    for p, g, ea, easq, st in zip(params, grads, eas, easqs, steps):
        if g.size == 0:
            continue
        z = np.maximum(g[:, None] * w1[None, :] + b1[None, :].astype(F), F(0))
        scale = (z * w2[None, :]).sum(axis=1, dtype=np.float32) + F(b2.reshape(-1)[0])
        amp = g * (F(alpha_amp) * scale + F(beta_amp))
        _adam(p, ea, easq, amp.astype(F), beta1, beta2, lr, wd, eps, _bc(beta1, st), _bc(beta2, st))


def prodigy_step(params, grads, eas, easqs, ss, inits, steps, d_lr, beta1, beta2, lr, wd, eps):
    """Returns the new d_lr."""
    num = sum(float(np.dot(g.astype(np.float64), (p - p0).astype(np.float64))) for g, p, p0 in zip(grads, params, inits))
    den = sum(float(s.astype(np.float64).sum()) for s in ss)
    num, den, d_lr = F(num), F(den), F(d_lr)
    if den > F(1e-30):
        d_lr = max(d_lr, abs(num) / (den + F(1e-12)))
    for p, g, ea, easq, s, st in zip(params, grads, eas, easqs, ss, steps):
        if g.size == 0:
            continue
        dg = g * d_lr
        b1, b2 = F(beta1), F(beta2)
        s[:] = s * b2 + (F(1) - b2) * dg * dg
        ea[:] = ea * b1 + (F(1) - b1) * dg
        easq[:] = easq * b2 + (F(1) - b2) * dg * dg
        denom = np.sqrt(easq / _bc(beta2, st)) + d_lr * F(eps)
        p *= F(1) - F(lr) * d_lr * F(wd)
        p -= (F(lr) / _bc(beta1, st)) * ea / denom
    return float(d_lr)


def lion_step(params, grads, eas, lr, beta1, beta2, wd):
    for p, g, ea in zip(params, grads, eas):
        if g.size == 0:
            continue
        interp = F(beta1) * ea + (F(1) - F(beta1)) * g
        p += -F(lr) * (np.sign(interp).astype(F) + F(wd) * p)
        ea[:] = ea * F(beta2) + (F(1) - F(beta2)) * g


def _erf(x):
    from scipy.special import erf
    return erf(x.astype(np.float64))


def metanet(g, s, W1, b1, W2, b2, rescale, gelu="erf"):
    """smart gradient g + rescale * MLP([g, s]) (2 -> H -> 1)."""
    z = g[:, None] * W1[None, :, 0] + s[:, None] * W1[None, :, 1] + b1[None, :]
    z = z.astype(F)
    if gelu == "erf":
        act = (0.5 * z.astype(np.float64) * (1.0 + _erf(z / math.sqrt(2.0)))).astype(F)
    else:
        act = z / (F(1) + np.exp(F(-1.702) * z))
    out = (act * W2.reshape(-1)[None, :]).sum(axis=1, dtype=np.float32) + F(b2.reshape(-1)[0])
    return (g + F(rescale) * out).astype(F)


def sg11_gate(smart, mu, temperature):
    dot = float(np.dot(smart.astype(np.float64), mu.astype(np.float64)))
    cos = F(dot) / (_norm([smart]) * _norm([mu]) + F(1e-8))
    return F(1) / (F(1) + F(math.exp(-float(F(temperature) * cos))))


def sg11_step(params, grads, eas, easqs, mus, sharps, steps, alphas, beta1s, W1, b1, W2, b2, rescale, beta2, lr, wd, eps, lamb,
              ramp, temperature, clip, gelu="erf"):
    """steps are the values BEFORE the call; the step counts one up (ops.cpp:237)."""
    _clip_in_place(grads, clip)
    for i, (p, g, ea, easq, mu, sh) in enumerate(zip(params, grads, eas, easqs, mus, sharps)):
        if g.size == 0:
            continue
        st = steps[i] + 1
        a = F(alphas[i])
        mu[:] = mu * a + (F(1) - a) * g
        smart = metanet(g, sh, W1, b1, W2, b2, rescale, gelu)
        gate = sg11_gate(smart, mu, temperature)
        lamb_eff = F(ramp) * gate * F(lamb) if ramp > 0 else F(0)
        fg = smart + lamb_eff * mu
        _adam(p, ea, easq, fg, beta1s[i], beta2, lr, wd, eps, _bc(beta1s[i], st), _bc(beta2, st))


def sg2_clip(grads, max_norm):
    """Per-tensor pre-pass of the v2 step (grokking_optimizers/supergrok2.py:316-321): returns new arrays."""
    out = []
    for g in grads:
        n = _norm([g])
        h = g * (F(max_norm) / (n + F(1e-12))) if n > F(max_norm) else g.copy()
        out.append(np.where(np.isfinite(h), h, F(0)).astype(F))
    return out


def looksam_perturb(params, grads, rho):
    r = F(rho) / (_norm(grads) + F(1e-12))
    for p, g in zip(params, grads):
        p += r * g


def looksam_directions(v_dirs, sam_grads, grads):
    """In place, as the reference's device branch does (its CPU branch rebinds a copy and changes nothing)."""
    for v, sg, g in zip(v_dirs, sam_grads, grads):
        if g.size == 0:
            continue
        diff = (sg - g).astype(F)
        n = _norm([diff])
        if n < F(1e-12):
            continue
        v[:] = diff * (F(1) / n)


def looksam_adjust(grads, v_dirs, la):
    for g, v in zip(grads, v_dirs):
        if g.size == 0 or v.size == 0:
            continue
        g += (F(la) * _norm([g])) * v
