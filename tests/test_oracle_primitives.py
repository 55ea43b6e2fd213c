"""Pins the fixed-order fp32 primitives (include/sg_math.h, exported by the
CPU checker) against libm in double precision."""
import math

import numpy as np
import pytest

from oracle import oracle as orc

L = orc.lib()
RNG = np.random.RandomState(123)


def _maxrel(fn, ref, xs, floor=1e-30):
    worst = 0.0
    for x in xs:
        x = float(np.float32(x))
        r = ref(x)
        worst = max(worst, abs(fn(x) - r) / max(abs(r), floor))
    return worst


def test_exp():
    xs = np.concatenate([RNG.uniform(-80, 80, 20000), [0.0, -0.0, 1e-8, -86.0, 88.0, 20.0, -20.0]])
    assert _maxrel(L.orc_exp, math.exp, xs) < 2e-7
    # clamp: stays finite and monotone at the ends
    assert L.orc_exp(200.0) == L.orc_exp(88.0) and L.orc_exp(-200.0) == L.orc_exp(-86.0)
    assert L.orc_exp(0.0) == 1.0


def test_log():
    xs = np.exp(RNG.uniform(-30, 30, 20000))
    assert _maxrel(L.orc_log, math.log, xs, floor=1e-3) < 2e-7
    assert L.orc_log(1.0) == 0.0


def test_softplus_against_both_of_the_reference_s_forms():
    """sg_softplus against log1p(exp(x)) in double precision (what the reference's Python path computes,
    mamba3_peer_metanet.py:106) to 2e-7 RELATIVE over the whole range, and against the CUDA path's literal fp32
    formula logf(1 + expf(x)) with its x > 20 guard (supergrok2_mamba_peer_kernels.cu:221), which loses the digits of
    exp(x) below 1 when it rounds 1 + exp(x): the two agree to 7e-8 absolutely, which is that rounding."""
    def exact(x):
        return x + math.log1p(math.exp(-x)) if x > 0 else math.log1p(math.exp(x))
    def literal(x):
        if x > 20.0:
            return x
        return math.log(float(np.float32(1.0) + np.float32(math.exp(x))))
    xs = np.concatenate([RNG.uniform(-40, 30, 30000), RNG.uniform(-2, 2, 5000), [0.0, 20.0, -16.6, -86.0]])
    worst_rel = worst_abs = 0.0
    for x in xs:
        x = float(np.float32(x))
        got = L.orc_softplus(x)
        worst_rel = max(worst_rel, abs(got - exact(x)) / exact(x))
        worst_abs = max(worst_abs, abs(got - literal(x)) / max(1.0, abs(x)))
    assert worst_rel < 2.5e-7, worst_rel
    assert worst_abs < 1.5e-7, worst_abs
    assert L.orc_softplus(25.0) == 25.0 and L.orc_softplus(20.5) == 20.5      # the guard's pass-through, to the bit
    assert abs(L.orc_softplus(-30.0) / math.exp(-30.0) - 1.0) < 3e-7          # exp(x) itself, not 0
    assert L.orc_softplus(0.0) == np.float32(math.log(2.0))


def test_sigmoid_silu_tanh():
    xs = RNG.uniform(-30, 30, 20000)
    assert _maxrel(L.orc_sigmoid, lambda x: 1 / (1 + math.exp(-x)), xs) < 3e-7
    assert _maxrel(L.orc_silu, lambda x: x / (1 + math.exp(-x)), xs) < 3e-7
    xs = np.concatenate([RNG.uniform(-9, 9, 20000), RNG.uniform(-0.7, 0.7, 5000), [0.0, 0.625, -0.625, 1e-6]])
    assert _maxrel(L.orc_tanh, math.tanh, xs) < 4e-7
    assert L.orc_tanh(0.0) == 0.0 and L.orc_tanh(30.0) == 1.0 and L.orc_tanh(-30.0) == -1.0


def test_silu_block_shares_one_reciprocal():
    """sg_silu_block (n values, one reciprocal) against x / (1 + exp(-x)) in double precision: groups of 4 and 8,
    ordinary and mixed magnitudes, and a group whose denominators overflow the shared product (per-value fallback,
    which must then equal sg_silu bit for bit)."""
    import ctypes as C
    def block(vals):
        z = np.asarray(vals, np.float32)
        out = np.zeros_like(z)
        L.orc_silu_block(len(z), z.ctypes.data_as(C.POINTER(C.c_float)), out.ctypes.data_as(C.POINTER(C.c_float)))
        return z, out
    worst = 0.0
    for n in (4, 8):
        for scale in (0.1, 1.0, 4.0):
            for _ in range(2000):
                z, out = block(RNG.randn(n) * scale)
                ref = z.astype(np.float64) / (1.0 + np.exp(-z.astype(np.float64)))
                worst = max(worst, float(np.max(np.abs(out - ref) / np.maximum(np.abs(ref), 1e-30))))
    assert worst < 1.5e-6, worst          # a dozen roundings instead of the two of sg_silu
    z, out = block([0.0, 1.0, -1.0, 30.0])
    assert out[0] == 0.0 and abs(out[3] - 30.0) < 1e-5
    # one very negative value makes the product of denominators overflow: every value takes the plain form
    z, out = block([-80.0, -70.0, 0.5, -60.0, 2.0, -75.0, 1.0, -85.0])
    assert all(out[k] == np.float32(L.orc_silu(float(z[k]))) for k in range(8))
    # just below the limit the block form is used and agrees to rounding
    z, out = block([-8.0] * 8)
    assert np.all(np.abs(out - np.float32(-8.0 / (1 + math.exp(8.0)))) < 1e-9)


def test_sigmoid_and_tanh_blocks():
    """sg_sigmoid_block (8 values) and sg_tanh_block (4 values) against libm in double precision; saturated values
    push the shared product over its limit and must then give exactly the plain forms."""
    import ctypes as C
    def call(fn, vals):
        x = np.asarray(vals, np.float32)
        out = np.zeros_like(x)
        fn(len(x), x.ctypes.data_as(C.POINTER(C.c_float)), out.ctypes.data_as(C.POINTER(C.c_float)))
        return x, out
    ws = wt = 0.0
    for scale in (0.2, 1.0, 3.0):
        for _ in range(3000):
            x, out = call(L.orc_sigmoid_block, RNG.randn(8) * scale)
            ref = 1.0 / (1.0 + np.exp(-x.astype(np.float64)))
            ws = max(ws, float(np.max(np.abs(out - ref) / ref)))
            x, out = call(L.orc_tanh_block, RNG.randn(4) * scale)
            ref = np.tanh(x.astype(np.float64))
            wt = max(wt, float(np.max(np.abs(out - ref) / np.maximum(np.abs(ref), 1e-30))))
    assert ws < 1.5e-6 and wt < 1.5e-6, (ws, wt)
    x, out = call(L.orc_sigmoid_block, [-40.0, -41.0, 0.3, -39.0, 40.0, 1.0, -1.0, -45.0])
    assert all(out[k] == np.float32(L.orc_sigmoid(float(x[k]))) for k in range(8)) and out[4] == 1.0
    x, out = call(L.orc_tanh_block, [30.0, -25.0, 0.1, 20.0])
    assert all(out[k] == np.float32(L.orc_tanh(float(x[k]))) for k in range(4)) and out[0] == 1.0 and out[1] == -1.0
    x, out = call(L.orc_tanh_block, [0.0, 0.625, -0.625, 1e-6])
    assert out[0] == 0.0 and abs(out[1] - math.tanh(0.625)) < 1e-7 and out[2] == -out[1]


def test_sincos():
    xs = np.concatenate([RNG.uniform(-100, 100, 30000), RNG.uniform(-1, 1, 5000),
                         [0.0, math.pi / 4, -math.pi / 4, math.pi / 2, math.pi, 3 * math.pi / 2]])
    ws, wc = 0.0, 0.0
    for x in xs:
        x = float(np.float32(x))
        ws = max(ws, abs(L.orc_sin(x) - math.sin(x)))
        wc = max(wc, abs(L.orc_cos(x) - math.cos(x)))
    assert ws < 2.5e-7 and wc < 2.5e-7
    assert L.orc_sin(0.0) == 0.0 and L.orc_cos(0.0) == 1.0


def test_small_angle_sincos_is_bitwise_the_general_one():
    xs = np.concatenate([RNG.uniform(-0.78, 0.78, 50000), RNG.uniform(-1e-3, 1e-3, 5000),
                         [0.0, -0.0, 0.7799999, -0.7799999, 1e-30, -1e-30]]).astype(np.float32)
    for x in xs:
        x = float(x)
        assert abs(x) < 0.78
        assert np.float32(L.orc_sin_small(x)).tobytes() == np.float32(L.orc_sin(x)).tobytes(), x
        assert np.float32(L.orc_cos_small(x)).tobytes() == np.float32(L.orc_cos(x)).tobytes(), x


def test_tiny_angle_sincos_against_libm():
    """|theta| < 0.3 with one polynomial term less: ~1 ulp of sin (relative) and of cos (absolute), pure rotation
    (s^2 + c^2 = 1 to rounding), odd/even symmetry."""
    xs = np.concatenate([RNG.uniform(-0.3, 0.3, 50000), RNG.uniform(-1e-3, 1e-3, 5000), [0.0, 0.2999999, -0.2999999, 1e-30]])
    ws = wc = wn = 0.0
    for x in xs.astype(np.float32):
        x = float(x)
        s, c = L.orc_sin_tiny(x), L.orc_cos_tiny(x)
        ws = max(ws, abs(s - math.sin(x)) / max(abs(x), 1e-30))
        wc = max(wc, abs(c - math.cos(x)))
        wn = max(wn, abs(s * s + c * c - 1.0))
        assert L.orc_sin_tiny(-x) == -s and L.orc_cos_tiny(-x) == c
    assert ws < 1.5e-7 and wc < 1.3e-7 and wn < 3e-7, (ws, wc, wn)
    assert L.orc_sin_tiny(0.0) == 0.0 and L.orc_cos_tiny(0.0) == 1.0


def test_rcp_and_abar():
    ds = np.exp(RNG.uniform(0, 60, 20000))
    assert _maxrel(L.orc_rcp_pos, lambda d: 1.0 / d, ds) < 1.5e-7
    worst = 0.0
    for _ in range(20000):
        dt = float(np.float32(RNG.uniform(0, 25)))
        A = float(np.float32(-math.exp(RNG.uniform(-6, 4))))
        ref = (1.0 + dt * A / 2.0) / (1.0 - dt * A / 2.0 + 1e-8)
        worst = max(worst, abs(L.orc_abar(dt, A) - ref))      # |A_bar| <= 1: absolute error is what enters h
    assert worst < 4e-7
    # the dropped "+1e-8f": for every denominator >= 1 it is an fp32 no-op
    dens = np.float32(1.0) + np.abs(RNG.randn(100000).astype(np.float32)) * np.float32(10)
    dens = np.concatenate([dens, np.float32([1.0, np.nextafter(np.float32(1), np.float32(2))])])
    assert np.array_equal(dens + np.float32(1e-8), dens)
    assert L.orc_abar(0.0, -1.0) == 1.0


def test_half_conversions_match_numpy():
    xs = np.concatenate([RNG.randn(20000).astype(np.float32) * np.float32(10.0 ** RNG.randint(-9, 6)),
                         np.float32([0, -0.0, 65504, 65520, 1e-8, 6e-8, 6.1e-5, np.inf, -np.inf])])
    for x in xs:
        h = np.float32(x).astype(np.float16)
        assert L.orc_f_to_f16(float(x)) == int(h.view(np.uint16)), x
        assert L.orc_f16_to_f(int(h.view(np.uint16))) == float(h) or np.isnan(float(h))
    import torch
    t = torch.from_numpy(xs[np.isfinite(xs)])
    b = t.to(torch.bfloat16)
    bits = b.view(torch.int16).numpy().view(np.uint16)
    for x, hb, back in zip(t.numpy(), bits, b.float().numpy()):
        assert L.orc_f_to_bf16(float(x)) == int(hb)
        assert L.orc_bf16_to_f(int(hb)) == float(back)


def test_taylor_polynomials_of_step_size_and_gate():
    """softplus(c + d) and silu(c + d) from their cubic Taylor polynomials around c, for |d| below the limit a tile has
    to meet (2^-5): within an fp32 rounding or two of the functions themselves (float64), over the whole range of c.
    A wrong derivative (sign, factor) would be off by d^2 or d^3 times a derivative of order 0.1: 1e-4 .. 1e-6."""
    r = np.random.RandomState(5)
    cs = np.concatenate([r.uniform(-14, 14, 3000), r.uniform(-1, 1, 2000), [0.0, -30.0, 30.0, 88.0, -88.0]]).astype(np.float32)
    ds = np.concatenate([r.uniform(-1, 1, cs.size - 4) * 2.0 ** -5, [2.0 ** -5, -2.0 ** -5, 0.0, 1e-8]]).astype(np.float32)
    worst_sp = worst_si = 0.0
    for c, d in zip(cs, ds):
        x = float(c) + float(d)
        sp = math.log1p(math.exp(-abs(x))) + max(x, 0.0)
        si = x / (1.0 + math.exp(-x))
        e_sp = abs(L.orc_softplus_taylor(float(c), float(d)) - sp) / (3e-7 * abs(sp) + 1e-8)
        e_si = abs(L.orc_silu_taylor(float(c), float(d)) - si) / (3e-7 * abs(si) + 4e-8)
        worst_sp, worst_si = max(worst_sp, e_sp), max(worst_si, e_si)
    assert worst_sp <= 1.0 and worst_si <= 1.0, (worst_sp, worst_si)
    # at d = 0 the polynomials are the functions' own values
    for c in (-3.0, 0.25, 7.0):
        assert L.orc_softplus_taylor(c, 0.0) == L.orc_softplus(c) and L.orc_silu_taylor(c, 0.0) == np.float32(c) * np.float32(L.orc_sigmoid(c))


def test_contraction_steps_bound_the_decay():
    """sg2_contraction_steps(dt, -A_e/2, -A_o/2): the slower pole's |A_bar| to that power is below 2^-100, and one step
    fewer by more than a rounding's worth is not; poles that do not contract within a million steps give 0."""
    for dt, Ae, Ao in ((0.7, -1.0, -0.75), (0.05, -3.0, -16.0), (1.7, -16.0, -1.0), (3.0, -0.01, -0.02)):
        n = L.orc_contraction_steps(dt, -0.5 * Ae, -0.5 * Ao)
        m = max(abs((1 + dt * A / 2) / (1 - dt * A / 2)) for A in (Ae, Ao))
        assert n > 0 and m ** n < 2.0 ** -100 * 1.001 and m ** (n - 2) > 2.0 ** -100, (dt, Ae, Ao, n, m)
    assert L.orc_contraction_steps(1e-6, -0.5 * -1e-3, -0.5 * -1e-3) == 0


def test_recurrence_coefficients_as_polynomials_in_dt():
    """A_bar(dt) = (1 - a dt)/(1 + a dt) as a cubic and sin/cos(f dt) as quadratics in d = dt - dt0, inside the limits a
    block has to meet (a |d| < 2^-7, |f d| < 2^-8): within an fp32 rounding or two of the closed forms (float64).  A
    coefficient with a wrong sign or factor is off by (a d)^k of order 1e-2 .. 1e-7 relative."""
    r = np.random.RandomState(9)
    worst = 0.0
    for _ in range(4000):
        dt0 = float(np.float32(r.uniform(0.01, 3.0)))
        a = float(np.float32(np.exp(r.uniform(-4.0, 2.2))))          # -A/2 from 0.018 to 9
        f = float(np.float32(r.uniform(-1.0, 1.0)))
        lim = min(2.0 ** -7 / a, 2.0 ** -8 / max(abs(f), 1e-3), dt0)
        d = float(np.float32(r.uniform(-1.0, 1.0) * lim))
        dt = dt0 + d
        exact = (1.0 - a * dt) / (1.0 + a * dt)
        # (2 r - 1 cancels where a dt is close to 1, exactly as in sg_abar_pair: an absolute floor of one rounding of r)
        worst = max(worst, abs(L.orc_abar_poly(dt0, a, d) - exact) / (4e-7 * abs(exact) + 1.5e-7))
        worst = max(worst, abs(L.orc_sincos_poly(dt0, f, d, 0) - math.sin(f * dt)) / (4e-7 * abs(math.sin(f * dt)) + 3e-8))
        worst = max(worst, abs(L.orc_sincos_poly(dt0, f, d, 1) - math.cos(f * dt)) / (4e-7 + 3e-8))
    assert worst <= 1.0, worst


def test_update_products_as_quadratics_in_dt():
    """The four products of the replay's update, A_bar_e cos, -A_bar_e sin, A_bar_o cos, A_bar_o sin (of f dt), as
    quadratics in d = dt - dt0 inside the limit a block has to meet, (2.3 a + |f|) |d| < 2^-7.5: within an fp32 rounding
    or two of the closed forms (float64).  A sign or a dropped cross term shows at first or second order in d."""
    r = np.random.RandomState(10)
    worst = 0.0
    for _ in range(4000):
        dt0 = float(np.float32(r.uniform(0.01, 3.0)))
        ae, ao = (float(np.float32(np.exp(r.uniform(-4.0, 2.2)))) for _ in range(2))
        f = float(np.float32(r.uniform(-1.0, 1.0)))
        lim = min(2.0 ** -7.5 / (2.3 * max(ae, ao) + abs(f)), dt0)
        d = float(np.float32(r.uniform(-1.0, 1.0) * lim))
        dt = dt0 + d
        A = [(1.0 - a * dt) / (1.0 + a * dt) for a in (ae, ao)]
        want = (A[0] * math.cos(f * dt), -A[0] * math.sin(f * dt), A[1] * math.cos(f * dt), A[1] * math.sin(f * dt))
        for which in range(4):
            got = L.orc_pair_product(dt0, ae, ao, f, d, which)
            worst = max(worst, abs(got - want[which]) / (4e-7 * abs(want[which]) + 2e-7))
    assert worst <= 1.0, worst
