/*
 * sg_math.h -- fp32 primitives with a FIXED operation order.
 *
 * Every function here is built only from IEEE-754 correctly rounded
 * operations (+, -, *, /, sqrt, fma, round-to-nearest-even) and integer bit
 * manipulation, so a gfx950 wavefront lane and an x86-64 host core return
 * the same bits for the same input.  That is what lets the device kernels be
 * compared bit-for-bit (sort permutations, PEER expert indices) with a CPU
 * restatement of the same algorithm.
 *
 * Build rules that the property depends on (both compilers):
 *   -ffp-contract=off      nothing is fused unless written as sg_fma()
 *   no -ffast-math         no reassociation, IEEE division and sqrt
 *   fp32 denormals kept    (the hipcc and gcc defaults)
 *
 * The transcendental approximations follow the classic Cephes single
 * precision kernels (Cody-Waite range reduction + minimax polynomial); each
 * is accurate to about 1e-7 relative on the range the optimizer uses.
 *
 * What the functions stand in for in the reference (file:line are relative
 * to the reference tree):
 *   sg_exp       expf       csrc/supergrok2_mamba_peer_kernels.cu:194,221,263,970
 *   sg_log       logf       csrc/supergrok2_mamba_peer_kernels.cu:221
 *   sg_softplus  stable softplus with the ">20 passes through" guard, :221
 *   sg_sincos    __sincosf  csrc/supergrok2_mamba_peer_kernels.cu:240,434,652
 *   sg_tanh      tanhf      csrc/supergrok2_mamba_peer_kernels.cu:989
 *   sg_sigmoid   1/(1+expf(-x))   :970-971
 *   sg_silu      z/(1+expf(-z))   :263,559,777
 *   sg_abar_pair trapezoidal A_bar for the even/odd member of a RoPE pair, :228,431-432
 *   sg_gelu_erf  exact GELU of the CPU path      csrc/ops.cpp:140 (torch::gelu)
 *   sg_gelu_sigmoid  z/(1+expf(-1.702 z))         csrc/supergrok15_kernels.cu:380
 */
#ifndef SG_MATH_H_
#define SG_MATH_H_

#include <stdint.h>

#if defined(__HIPCC__)
#define SG_HD __host__ __device__ __forceinline__
#else
#define SG_HD static inline __attribute__((always_inline))
#endif

SG_HD float sg_fma(float a, float b, float c) { return __builtin_fmaf(a, b, c); }
SG_HD float sg_rint(float x) { return __builtin_rintf(x); }

SG_HD int32_t sg_f2i(float x) {
    int32_t i;
    __builtin_memcpy(&i, &x, 4);
    return i;
}
SG_HD float sg_i2f(int32_t i) {
    float x;
    __builtin_memcpy(&x, &i, 4);
    return x;
}
SG_HD float sg_abs(float x) { return sg_i2f(sg_f2i(x) & 0x7fffffff); }
SG_HD float sg_min(float a, float b) { return a < b ? a : b; }
SG_HD float sg_max(float a, float b) { return a > b ? a : b; }

/* finite test on the bit pattern (no dependence on -ffinite-math settings) */
SG_HD int sg_isfinite(float x) { return (sg_f2i(x) & 0x7f800000) != 0x7f800000; }

/* exp(x), x clamped to [-86, 88] so the result is always a normal float. */
SG_HD float sg_exp(float x) {
    x = sg_min(sg_max(x, -86.0f), 88.0f);
    const float k = sg_rint(x * 1.44269504088896341f);
    float r = sg_fma(k, -0.693359375f, x);
    r = sg_fma(k, 2.12194440e-4f, r);
    float p = 1.9875691500e-4f;
    p = sg_fma(p, r, 1.3981999507e-3f);
    p = sg_fma(p, r, 8.3334519073e-3f);
    p = sg_fma(p, r, 4.1665795894e-2f);
    p = sg_fma(p, r, 1.6666665459e-1f);
    p = sg_fma(p, r, 5.0000001201e-1f);
    p = sg_fma(sg_fma(p, r, 1.0f), r, 1.0f);         /* 1 + r (1 + r p) */
    return sg_i2f((int32_t)((uint32_t)sg_f2i(p) + ((uint32_t)(int32_t)k << 23)));
}

/* log(u) for normal positive u. */
SG_HD float sg_log(float u) {
    const int32_t ix = sg_f2i(u);
    const int32_t e = (ix - 0x3f3504f3) >> 23;          /* mantissa -> [sqrt(.5), sqrt(2)) */
    const float f = sg_i2f((int32_t)((uint32_t)ix - ((uint32_t)e << 23))) - 1.0f;
    const float fe = (float)e;
    const float z = f * f;
    float p = 7.0376836292e-2f;
    p = sg_fma(p, f, -1.1514610310e-1f);
    p = sg_fma(p, f, 1.1676998740e-1f);
    p = sg_fma(p, f, -1.2420140846e-1f);
    p = sg_fma(p, f, 1.4249322787e-1f);
    p = sg_fma(p, f, -1.6668057665e-1f);
    p = sg_fma(p, f, 2.0000714765e-1f);
    p = sg_fma(p, f, -2.4999993993e-1f);
    p = sg_fma(p, f, 3.3333331174e-1f);
    float y = (p * f) * z;
    y = sg_fma(fe, -2.12194440e-4f, y);
    y = sg_fma(z, -0.5f, y);
    return sg_fma(fe, 0.693359375f, f + y);
}

/* softplus(x) = max(x, 0) + log1p(w), w = exp(-|x|) in (0, 1], with log1p(w) = w Q(w), Q a degree-9 fit of
 * log1p(w)/w on [0, 1] (relative error of the whole function below 2e-7 for every x).  Branch-free.  For x > 20 the
 * second term is below half an ulp of x, so x passes through as the reference's guard has it; for very negative x
 * the result is exp(x) itself, where log(1 + exp(x)) evaluated in fp32 gives 0 below -16.6. */
SG_HD float sg_softplus(float x) {
    const float w = sg_exp(-sg_abs(x));
    float q = -2.788148588e-03f;
    q = sg_fma(q, w, 1.774181798e-02f);
    q = sg_fma(q, w, -5.286746472e-02f);
    q = sg_fma(q, w, 1.017219052e-01f);
    q = sg_fma(q, w, -1.503748596e-01f);
    q = sg_fma(q, w, 1.957647055e-01f);
    q = sg_fma(q, w, -2.493286729e-01f);
    q = sg_fma(q, w, 3.332757950e-01f);
    q = sg_fma(q, w, -4.999978840e-01f);
    q = sg_fma(q, w, 1.0f);
    return sg_fma(w, q, sg_max(x, 0.0f));
}

SG_HD float sg_sigmoid(float x) { return 1.0f / (1.0f + sg_exp(-x)); }
SG_HD float sg_silu(float z) { return z / (1.0f + sg_exp(-z)); }

/* sin and cos of theta; two-constant Cody-Waite reduction by pi/2 (good to
 * ~1e-7 absolute for |theta| < ~1e3, degrading gracefully beyond). */
SG_HD void sg_sincos(float th, float* s_out, float* c_out) {
    const float k = sg_rint(th * 0.636619772367581343f);
    float r = sg_fma(k, -1.57079637050628662f, th);
    r = sg_fma(k, 4.37113900018624283e-8f, r);
    const float z = r * r;
    float sp = -1.9515295891e-4f;
    sp = sg_fma(sp, z, 8.3321608736e-3f);
    sp = sg_fma(sp, z, -1.6666654611e-1f);
    sp = sg_fma(sp * z, r, r);
    float cp = 2.443315711809948e-5f;
    cp = sg_fma(cp, z, -1.388731625493765e-3f);
    cp = sg_fma(cp, z, 4.166664568298827e-2f);
    cp = sg_fma(cp * z, z, sg_fma(z, -0.5f, 1.0f));
    const int32_t q = (int32_t)k;
    const int swap = q & 1;
    const float s0 = swap ? cp : sp;
    const float c0 = swap ? sp : cp;
    *s_out = sg_i2f((int32_t)((uint32_t)sg_f2i(s0) ^ (((uint32_t)q & 2u) << 30)));
    *c_out = sg_i2f((int32_t)((uint32_t)sg_f2i(c0) ^ ((((uint32_t)q + 1u) & 2u) << 30)));
}

/* sg_sincos for |theta| < 0.78: the reduction multiple is then 0, so the
 * general routine reduces to the two polynomials; the results are bit for
 * bit those of sg_sincos.  Lets a wavefront skip the reduction and quadrant
 * logic when all its lanes hold small angles. */
SG_HD void sg_sincos_small(float th, float* s_out, float* c_out) {
    const float z = th * th;
    float sp = -1.9515295891e-4f;
    sp = sg_fma(sp, z, 8.3321608736e-3f);
    sp = sg_fma(sp, z, -1.6666654611e-1f);
    *s_out = sg_fma(sp * z, th, th);
    float cp = 2.443315711809948e-5f;
    cp = sg_fma(cp, z, -1.388731625493765e-3f);
    cp = sg_fma(cp, z, 4.166664568298827e-2f);
    *c_out = sg_fma(cp * z, z, sg_fma(z, -0.5f, 1.0f));
}
#define SG_SINCOS_SMALL_LIMIT 0.78f

/* 1/d for normal positive d: bit-trick seed + three Newton steps (~5e-8 rel). */
SG_HD float sg_rcp_pos(float d) {
    float r = sg_i2f(0x7EF311C7 - sg_f2i(d));
    float e = sg_fma(-d, r, 1.0f);
    r = sg_fma(r, e, r);
    e = sg_fma(-d, r, 1.0f);
    r = sg_fma(r, e, r);
    e = sg_fma(-d, r, 1.0f);
    r = sg_fma(r, e, r);
    return r;
}

/* SiLU of n <= 8 values with ONE reciprocal (simultaneous inversion of the denominators 1 + exp(-z_k), all >= 1):
 * out_k = z_k * (1/P_{n-1}) * (d_{k+1} ... d_{n-1}) * P_{k-1},  P_k = d_0 ... d_k.  Used only while the product of all
 * denominators is below SG_SILU_BLOCK_LIMIT (a very negative z makes its denominator huge); sg_silu per value
 * otherwise.  Differs from sg_silu in the last bits, so both sides of a parity comparison must group the values the
 * same way. */
#define SG_SILU_BLOCK_LIMIT 1e30f
SG_HD void sg_silu_block(int n, const float* z, float* out) {
    float d[8], P[8];
    float acc = 1.0f;
    for (int k = 0; k < n; k++) {
        d[k] = 1.0f + sg_exp(-z[k]);
        acc = (k == 0) ? d[k] : acc * d[k];
        P[k] = acc;
    }
    if (acc < SG_SILU_BLOCK_LIMIT) {
        float r = sg_rcp_pos(acc);
        for (int k = n - 1; k >= 0; k--) {
            const float inv = (k > 0) ? r * P[k - 1] : r;
            if (k > 0) r = r * d[k];
            out[k] = z[k] * inv;
        }
    } else {
        for (int k = 0; k < n; k++) out[k] = z[k] / d[k];
    }
}

/* sin and cos for |theta| < 0.3 with one polynomial term less each (least-squares fit on that
 * interval; ~1 ulp).  NOT bit-identical to sg_sincos: both sides of a parity comparison must take
 * this form for the same timesteps. */
#define SG_SINCOS_TINY_LIMIT 0.3f
SG_HD void sg_sincos_tiny(float th, float* s_out, float* c_out) {
    const float z = th * th;
    const float sp = sg_fma(0.0083154970780015f, z, -0.16666646301746368f);
    *s_out = sg_fma(sp * z, th, th);
    const float cp = sg_fma(-0.0013806807110086083f, z, 0.041666239500045776f);
    *c_out = sg_fma(cp * z, z, sg_fma(z, -0.5f, 1.0f));
}

/* The same polynomials in powers of dt for a fixed frequency f, theta = dt*f: the lane's frequency is folded into six
 * coefficients once (sg_sincos_tiny_coef), after which a timestep costs seven instructions instead of nine,
 *   sin = dt (f + z (s3 f^3 + z s5 f^5)),  cos = 1 + z (-f^2/2 + z (c4 f^4 + z c6 f^6)),  z = dt^2.
 * Last-bit differences from sg_sincos_tiny: both sides of a parity comparison must take the same form. */
SG_HD void sg_sincos_tiny_coef(float f, float* c /* [6] */) {
    const float f2 = f * f;
    c[0] = f;
    c[1] = (-0.16666646301746368f * f2) * f;
    c[2] = ((0.0083154970780015f * f2) * f2) * f;
    c[3] = -0.5f * f2;
    c[4] = (0.041666239500045776f * f2) * f2;
    c[5] = ((-0.0013806807110086083f * f2) * f2) * f2;
}
SG_HD void sg_sincos_tiny_dt(float dt, const float* c, float* s_out, float* c_out) {
    const float z = dt * dt;
    *s_out = dt * sg_fma(z, sg_fma(z, c[2], c[1]), c[0]);
    *c_out = sg_fma(z, sg_fma(z, sg_fma(z, c[5], c[4]), c[3]), 1.0f);
}

/* Trapezoidal discretisation for the two states of one RoPE pair:
 *   A_bar = (1 + dt*A/2) / (1 - dt*A/2 + 1e-8)
 * With t = -dt*A/2 >= 0 (A < 0, dt >= 0) this is (1-t)/(1+t) = 2/(1+t) - 1.
 * nhA_e and nhA_o are -A/2 (exact halving and negation).  The denominator is
 * >= 1, so the "+1e-8f" of the reference is below half an ulp of it: adding it
 * never changes an fp32 value >= 1, and it is dropped.  One shared reciprocal
 * serves both members of the pair:
 *   r = 1/((1+t_e)(1+t_o));  A_bar_e = 2 r (1+t_o) - 1;  A_bar_o = 2 r (1+t_e) - 1. */
SG_HD void sg_abar_pair(float dt, float nhA_e, float nhA_o, float* ab_e, float* ab_o) {
    const float d_e = sg_fma(dt, nhA_e, 1.0f);
    const float d_o = sg_fma(dt, nhA_o, 1.0f);
    const float r = sg_rcp_pos(d_e * d_o);
    const float r2 = r + r;
    *ab_e = sg_fma(d_o, r2, -1.0f);
    *ab_o = sg_fma(d_e, r2, -1.0f);
}

/* The same A_bar values for a block of n <= 16 consecutive timesteps of one lane with ONE reciprocal
 * (simultaneous inversion): with D_k = (1+t_e,k)(1+t_o,k) and prefix products P_k = D_0 ... D_k,
 *   1/D_k = (1/P_{n-1}) * (D_{k+1} ... D_{n-1}) * P_{k-1}.
 * sg_abar_block_prefix forms d_e, d_o and P and returns P_{n-1}; the caller uses the block form only
 * while that product is below SG_ABAR_BLOCK_LIMIT (all D_k >= 1, so a finite small last product
 * means every partial product is finite too), and sg_abar_pair per timestep otherwise.  Results differ
 * from sg_abar_pair in the last bits (a few more roundings), so both sides of a parity comparison must
 * group the timesteps the same way. */
#define SG_ABAR_BLOCK_LIMIT 1e30f
SG_HD float sg_abar_block_prefix(int n, const float* dt, float nhA_e, float nhA_o, float* d_e, float* d_o, float* P) {
    float acc = 1.0f;
    for (int k = 0; k < n; k++) {
        d_e[k] = sg_fma(dt[k], nhA_e, 1.0f);
        d_o[k] = sg_fma(dt[k], nhA_o, 1.0f);
        acc = (k == 0) ? d_e[k] * d_o[k] : acc * (d_e[k] * d_o[k]);
        P[k] = acc;
    }
    return acc;
}
SG_HD void sg_abar_block_finish(int n, const float* d_e, const float* d_o, const float* P, float* ab_e, float* ab_o) {
    /* the factor 2 of A_bar = 2/(1+t) - 1 rides on the running reciprocal (doubling is exact) */
    float r = sg_rcp_pos(P[n - 1]);
    r = r + r;
    for (int k = n - 1; k >= 0; k--) {
        const float inv2 = (k > 0) ? r * P[k - 1] : r;      /* 2/D_k */
        if (k > 0) r = r * (d_e[k] * d_o[k]);
        ab_e[k] = sg_fma(d_o[k], inv2, -1.0f);
        ab_o[k] = sg_fma(d_e[k], inv2, -1.0f);
    }
}

SG_HD float sg_tanh(float x) {
    const float ax = sg_abs(x);
    float y;
    if (ax < 0.625f) {
        const float z = x * x;
        float p = -5.70498872745e-3f;
        p = sg_fma(p, z, 2.06390887954e-2f);
        p = sg_fma(p, z, -5.37397155531e-2f);
        p = sg_fma(p, z, 1.33314422036e-1f);
        p = sg_fma(p, z, -3.33332819422e-1f);
        y = sg_fma(p * z, x, x);
    } else {
        const float t = 1.0f - 2.0f / (sg_exp(ax + ax) + 1.0f);
        y = sg_i2f(sg_f2i(t) | (sg_f2i(x) & (int32_t)0x80000000));
    }
    return y;
}

/* sigmoid of n <= 8 values and tanh of n <= 4 values with ONE reciprocal each (simultaneous inversion, as in
 * sg_silu_block): the denominators 1 + exp(-x_k), resp. exp(2|x_k|) + 1, are all >= 1; the shared form is used only
 * while their product stays below SG_SILU_BLOCK_LIMIT, the plain sg_sigmoid / sg_tanh per value otherwise (so a
 * saturated gate keeps its exact value).  Last-bit differences from the plain forms: both sides of a parity
 * comparison must group the values the same way. */
SG_HD void sg_sigmoid_block(int n, const float* x, float* out) {
    float d[8], P[8];
    float acc = 1.0f;
    for (int k = 0; k < n; k++) {
        d[k] = 1.0f + sg_exp(-x[k]);
        acc = (k == 0) ? d[k] : acc * d[k];
        P[k] = acc;
    }
    if (acc < SG_SILU_BLOCK_LIMIT) {
        float r = sg_rcp_pos(acc);
        for (int k = n - 1; k >= 0; k--) {
            out[k] = (k > 0) ? r * P[k - 1] : r;
            if (k > 0) r = r * d[k];
        }
    } else {
        for (int k = 0; k < n; k++) out[k] = 1.0f / d[k];
    }
}
SG_HD void sg_tanh_block(int n, const float* x, float* out) {
    float d[4], P[4];
    float acc = 1.0f;
    for (int k = 0; k < n; k++) {
        const float ax = sg_abs(x[k]);
        d[k] = sg_exp(ax + ax) + 1.0f;
        acc = (k == 0) ? d[k] : acc * d[k];
        P[k] = acc;
    }
    if (acc < SG_SILU_BLOCK_LIMIT) {
        float r = sg_rcp_pos(acc);
        for (int k = n - 1; k >= 0; k--) {
            const float inv = (k > 0) ? r * P[k - 1] : r;
            if (k > 0) r = r * d[k];
            const float xk = x[k], ax = sg_abs(xk), z = xk * xk;
            /* the two forms of sg_tanh, selected the same way */
            float p = -5.70498872745e-3f;
            p = sg_fma(p, z, 2.06390887954e-2f);
            p = sg_fma(p, z, -5.37397155531e-2f);
            p = sg_fma(p, z, 1.33314422036e-1f);
            p = sg_fma(p, z, -3.33332819422e-1f);
            const float small = sg_fma(p * z, xk, xk);
            const float t = sg_fma(-2.0f, inv, 1.0f);
            const float large = sg_i2f(sg_f2i(t) | (sg_f2i(xk) & (int32_t)0x80000000));
            out[k] = (ax < 0.625f) ? small : large;
        }
    } else {
        for (int k = 0; k < n; k++) out[k] = sg_tanh(x[k]);
    }
}

/* erfc(x): Chebyshev fit with exponential prefactor (Numerical Recipes
 * "erfcc"), fractional error below 1.2e-7 for every x. */
SG_HD float sg_erfc(float x) {
    const float ax = sg_abs(x);
    const float t = sg_rcp_pos(sg_fma(0.5f, ax, 1.0f));      /* denominator >= 1: Newton reciprocal, no IEEE division sequence */
    float p = 0.17087277f;
    p = sg_fma(p, t, -0.82215223f);
    p = sg_fma(p, t, 1.48851587f);
    p = sg_fma(p, t, -1.13520398f);
    p = sg_fma(p, t, 0.27886807f);
    p = sg_fma(p, t, -0.18628806f);
    p = sg_fma(p, t, 0.09678418f);
    p = sg_fma(p, t, 0.37409196f);
    p = sg_fma(p, t, 1.00002368f);
    p = sg_fma(p, t, -1.26551223f);
    const float r = t * sg_exp(sg_fma(-ax, ax, p));
    return (x >= 0.0f) ? r : 2.0f - r;
}

/* exact GELU: 0.5 z (1 + erf(z/sqrt2)) = 0.5 z erfc(-z/sqrt2) */
SG_HD float sg_gelu_erf(float z) { return (0.5f * z) * sg_erfc(z * -0.707106781186547524f); }
/* the sigmoid approximation of GELU used by the reference's GPU kernel */
SG_HD float sg_gelu_sigmoid(float z) { return z / (1.0f + sg_exp(-1.702f * z)); }

#endif /* SG_MATH_H_ */
