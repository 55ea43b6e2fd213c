/* Composed per-timestep projections of one SuperGrok v2 scan direction.
 *
 * Every linear quantity of a timestep is an affine function of the element's
 * (gradient, sharpness) pair, because the 8-vector fed to the scan is itself
 * x = W_in [g, s]^T + b_in (input_proj_sort_kernel,
 * csrc/supergrok2_mamba_peer_kernels.cu:92-117 of the reference) and in_proj,
 * dt_proj, B_proj and C_proj (:138-200 there) are applied to it without a
 * nonlinearity in between:
 *     xb_j = in_proj[j,:] x            z_j = in_proj[d_inner+j,:] x
 *     dt_raw_j = dt_W[j,:] xb + dt_b   B_s = B_proj[s,:] xb     C_s = C_proj[s,:] xb
 * This header composes those maps once per call into coefficient triples
 * (c_g, c_s, c_0) - accumulated in double, in a fixed order, rounded to float -
 * so that a timestep costs two fmas per output, v = fma(c_g, g, fma(c_s, s, c_0)),
 * instead of a chain of small matrix products.  The device kernel and the CPU
 * checker both include this file (double +,* only, no contraction), so their
 * coefficients are bit-identical.
 */
#ifndef SG2_COMPOSE_H_
#define SG2_COMPOSE_H_
#include "sg_math.h"

enum { SG2_COMP_XB = 0, SG2_COMP_Z = 1, SG2_COMP_DT = 2, SG2_COMP_B = 3, SG2_COMP_C = 4, SG2_COMP_GROUPS = 5 };
#define SG2_COMP_MAX_INNER 32
#define SG2_COMP_MAX_MODEL 16

/* Coefficient triple of output `row` of `group`.  Win [d_model,2], bin [d_model],
 * in_proj [2*d_inner, d_model], dt_W [d_inner,d_inner], dt_b [d_inner],
 * Bp / Cp [d_state, d_inner]. */
SG_HD void sg2_compose_one(int group, int row, int d_model, int d_inner, const float* Win, const float* bin,
                           const float* in_proj, const float* dt_W, const float* dt_b, const float* Bp, const float* Cp,
                           float out[3]) {
    double src[SG2_COMP_MAX_MODEL][3];
    for (int k = 0; k < d_model; k++) {
        src[k][0] = (double)Win[2 * k];
        src[k][1] = (double)Win[2 * k + 1];
        src[k][2] = (double)bin[k];
    }
    if (group == SG2_COMP_XB || group == SG2_COMP_Z) {
        const float* w = in_proj + (size_t)(group == SG2_COMP_Z ? d_inner + row : row) * d_model;
        for (int c = 0; c < 3; c++) {
            double acc = 0.0;
            for (int k = 0; k < d_model; k++) acc = acc + (double)w[k] * src[k][c];
            out[c] = (float)acc;
        }
        return;
    }
    double xb[SG2_COMP_MAX_INNER][3];
    for (int j = 0; j < d_inner; j++)
        for (int c = 0; c < 3; c++) {
            double acc = 0.0;
            for (int k = 0; k < d_model; k++) acc = acc + (double)in_proj[(size_t)j * d_model + k] * src[k][c];
            xb[j][c] = acc;
        }
    const float* w = (group == SG2_COMP_DT ? dt_W : (group == SG2_COMP_B ? Bp : Cp)) + (size_t)row * d_inner;
    for (int c = 0; c < 3; c++) {
        double acc = (group == SG2_COMP_DT && c == 2) ? (double)dt_b[row] : 0.0;
        for (int j = 0; j < d_inner; j++) acc = acc + (double)w[j] * xb[j][c];
        out[c] = (float)acc;
    }
}

/* Number of timesteps after which the 2x2 part of one RoPE pair's recurrence has shrunk below 2^-100 if every step
 * had the step size dt0: rotations preserve length, so the part's norm shrinks by at most max(|A_bar_e|, |A_bar_o|)
 * per step.  nhA = -A/2 of the pair's two poles (as sg_abar_pair takes them).  0 = not within a million steps.
 * Kernel and checker size the first block of a chunk summary with it (sg2_first_block_steps). */
SG_HD int sg2_contraction_steps(float dt0, float nhA_e, float nhA_o) {
    float ae, ao;
    sg_abar_pair(dt0, nhA_e, nhA_o, &ae, &ao);
    const float m = sg_max(sg_abs(ae), sg_abs(ao));
    if (!(m < 0.9999f)) return 0;
    if (m < 1e-30f) return 1;
    return (int)(69.3147202f / -sg_log(m)) + 1;       /* 100 ln 2 / -ln m */
}
/* The largest of those counts over all pairs of both directions (0 if one of them is 0), with an eighth and eight
 * steps of margin, rounded up to whole blocks of eight steps. */
SG_HD int sg2_first_block_steps(int largest, int any_zero) {
    if (any_zero || largest <= 0) return 0;
    return (largest + largest / 8 + 8 + 7) & ~7;
}

/* Near-constant arguments.  The step size is softplus(c_0 + d) and the gate silu(c_0' + d') with d = c_g g + c_s s: for
 * the small gradients of a trained model |d| is far below 1, and both functions are then their cubic Taylor
 * polynomials around the constant to within a fraction of an fp32 ulp (remainder <= d^4/24 times the largest fourth
 * derivative: 5e-9 for softplus, 2e-8 for silu at |d| = 2^-5).  The coefficients are formed once per call from the
 * shared fp32 primitives (so kernel and checker hold the same bits); a tile of 64 timesteps uses the polynomials when
 * cmax_g |g| + cmax_s |s| < SG2_TAYLOR_LIMIT for every timestep of the tile, cmax = the largest |c_g|, |c_s| over the dt
 * and gate rows of the direction, and the functions themselves otherwise. */
#define SG2_TAYLOR_LIMIT 0.03125f
SG_HD void sg2_softplus_taylor(float c, float t[4]) {
    const float s = sg_sigmoid(c), q = s * (1.0f - s);
    t[0] = sg_softplus(c);
    t[1] = s;
    t[2] = 0.5f * q;
    t[3] = (q * (1.0f - (s + s))) * 0.166666672f;
}
/* f = c s, f1 = s + c q, f2 = q (2 + c r), f3 = q (r (3 + c r) - 2 c q) with s = sigmoid(c), q = s (1 - s), r = 1 - 2 s */
SG_HD void sg2_silu_taylor(float c, float t[4]) {
    const float s = sg_sigmoid(c), q = s * (1.0f - s), r = 1.0f - (s + s);
    const float cr = c * r;
    t[0] = c * s;
    t[1] = sg_fma(c, q, s);
    t[2] = 0.5f * (q * (2.0f + cr));
    t[3] = (q * sg_fma(r, 3.0f + cr, -((c + c) * q))) * 0.166666672f;
}
SG_HD float sg2_taylor_delta(const float* c, float g, float s) { return sg_fma(c[0], g, c[1] * s); }
SG_HD float sg2_taylor_eval(const float* t, float d) { return sg_fma(sg_fma(sg_fma(t[3], d, t[2]), d, t[1]), d, t[0]); }
/* does this timestep qualify?  (every timestep of a tile must) */
SG_HD int sg2_taylor_ok(float cmax_g, float cmax_s, float g, float s) {
    return sg_fma(cmax_g, sg_abs(g), cmax_s * sg_abs(s)) < SG2_TAYLOR_LIMIT;
}

/* Near-constant step sizes.  Where dt stays within a small d of the zero-input step size dt0 of its column, the
 * coefficients of the recurrence are polynomials in d = dt - dt0 with per-pair constants: A_bar(dt) = 2/(1 + a dt) - 1
 * (a = -A/2) as a cubic (remainder 2 (a d)^4), sin/cos(f dt) as quadratics (remainder (f d)^3 / 6).  A block of 8
 * timesteps uses them when for each of its timesteps  kpoly_g |g| + kpoly_s |s| < 1,  with kpoly = max(128 a_max,
 * 256 f_max) times the largest |c_g|, |c_s| of the direction's dt rows (|dt - dt0| <= |c_g g + c_s s|: softplus has
 * slope <= 1): a d < 2^-7 and f d < 2^-8, remainders below 1e-8. */
SG_HD void sg2_abar_poly(float dt0, float nhA, float p[4]) {
    const float r = sg_rcp_pos(sg_fma(dt0, nhA, 1.0f));
    const float ar = nhA * r;
    p[0] = sg_fma(2.0f, r, -1.0f);
    p[1] = -((ar + ar) * r);
    p[2] = -(p[1] * ar);
    p[3] = -(p[2] * ar);
}
SG_HD void sg2_sincos_poly(float dt0, float f, float qs[3], float qc[3]) {
    float s0, c0;
    sg_sincos(dt0 * f, &s0, &c0);
    const float fs = f * s0, fc = f * c0;
    qs[0] = s0; qs[1] = fc; qs[2] = -0.5f * (f * fs);
    qc[0] = c0; qc[1] = -fs; qc[2] = -0.5f * (f * fc);
}
SG_HD float sg2_poly3(const float* p, float d) { return sg_fma(sg_fma(sg_fma(p[3], d, p[2]), d, p[1]), d, p[0]); }
SG_HD float sg2_poly2(const float* q, float d) { return sg_fma(sg_fma(q[2], d, q[1]), d, q[0]); }
SG_HD int sg2_poly_ok(float kpoly_g, float kpoly_s, float g, float s) {
    return sg_fma(kpoly_g, sg_abs(g), kpoly_s * sg_abs(s)) < 1.0f;
}
/* The factor in front of the dt rows' coefficients can be smaller than k: softplus is convex with derivative sigmoid, so
 * |dt - dt0| <= sigmoid(c_0 + m) |c_g g + c_s s| for a row with constant term c_0 while |c_g g + c_s s| <= m.  A
 * timestep that qualifies has |c_g g + c_s s| < 1 / (factor), so with m = 1/16 the largest sigmoid(c_0 + m) of the
 * direction's dt rows may multiply k as long as the product stays at least 16; otherwise k stands. */
#define SG2_SLOPE_MARGIN 0.0625f
SG_HD float sg2_dt_slope(float c0) { return sg_sigmoid(c0 + SG2_SLOPE_MARGIN); }
SG_HD float sg2_limit_factor(float k, float slope_max) {
    const float ks = k * slope_max;
    return ks >= 16.0f ? ks : k;
}

/* The output pass goes one step further: its update h' = D R h + b needs only the four products of the pair,
 * P1 = A_bar_e cos, N2 = -A_bar_e sin, P3 = A_bar_o cos, P4 = A_bar_o sin, and takes those as quadratics in d = dt - dt0
 * (products of the series above, truncated): he' = P1 he + N2 ho + b_e, ho' = P3 ho + P4 he + b_o, four fma instead of
 * two multiplications and four fma, and four quadratics instead of two cubics and two quadratics.  The truncated terms
 * are bounded by ((2.3 a + |f|) d)^3 / 6; a block uses the products when kprod_g |g| + kprod_s |s| < 1 for each of its
 * timesteps, kprod = (416 a_max + 184 f_max) times the largest |c_g|, |c_s| of the dt rows: (2.3 a + |f|) d < 2^-7.5,
 * remainder below 3e-8. */
/* Where the inputs are smaller still, kprod times 24 below 1, i.e. (2.3 a + |f|) d < 2^-12, the linear part alone is
 * within 3e-8 (remainder ((2.3 a + |f|) d)^2 / 2): SG2_PROD_LINEAR_FACTOR. */
#define SG2_PROD_LINEAR_FACTOR 24.0f
SG_HD float sg2_poly1(const float* k, float d) { return sg_fma(k[1], d, k[0]); }
SG_HD void sg2_prod_poly(const float a[3], const float c[3], float k[3]) {
    k[0] = a[0] * c[0];
    k[1] = sg_fma(a[0], c[1], a[1] * c[0]);
    k[2] = sg_fma(a[0], c[2], sg_fma(a[1], c[1], a[2] * c[0]));
}
/* k: [P1 | N2 | P3 | P4][3] of the pair with poles nhA_e, nhA_o and rotation frequency f */
SG_HD void sg2_pair_products(float dt0, float nhA_e, float nhA_o, float f, float k[12]) {
    float pe[4], po[4], qs[3], qc[3], ns[3];
    sg2_abar_poly(dt0, nhA_e, pe);
    sg2_abar_poly(dt0, nhA_o, po);
    sg2_sincos_poly(dt0, f, qs, qc);
    ns[0] = -qs[0]; ns[1] = -qs[1]; ns[2] = -qs[2];
    sg2_prod_poly(pe, qc, k);
    sg2_prod_poly(pe, ns, k + 3);
    sg2_prod_poly(po, qc, k + 6);
    sg2_prod_poly(po, qs, k + 9);
}

/* value of a composed output for one element */
SG_HD float sg2_comp_eval(const float* c, float g, float s) { return sg_fma(c[0], g, sg_fma(c[1], s, c[2])); }

#endif /* SG2_COMPOSE_H_ */
