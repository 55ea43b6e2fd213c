/*
 * TEST INFRASTRUCTURE ONLY.  CPU restatement of the SuperGrok v2 per-tensor
 * optimizer step (magnitude sort -> bidirectional Mamba-3 scan -> per-element
 * GRU -> 4-head PEER routing -> expert MLP -> mu/Adam/weight decay).
 * Nothing in the shipped package links, imports or executes this file; it is
 * the checker used by tests/, by the smoke check and by the cpu_baseline leg
 * of bench.py.
 *
 * Two arithmetic policies share one algorithm template:
 *   F32  fp32 with the fixed-order primitives of include/sg_math.h -- the
 *        device kernels use the same primitives and the same operation
 *        order, so integer results (sort permutation, expert indices,
 *        expert_counts) must match bit for bit and float results to ~1 ulp.
 *   F64  double precision, the reference's formulas written literally with
 *        libm -- the "what the mathematics says" answer the F32 result is
 *        pinned against (tests/test_oracle_*.py) and the source of the
 *        top-1/top-2 routing margins.
 *
 * Reference lines followed (paths relative to the reference tree):
 *   input projection, non-finite guard, |g| keys
 *       csrc/supergrok2_mamba_peer_kernels.cu:92-117
 *       grokking_optimizers/mamba3_peer_metanet.py:296-307
 *   ascending stable sort of |g|
 *       csrc/supergrok2_mamba_peer_kernels.cu:1538-1543,1860-1879 (radix sort => stable)
 *   per-timestep projections xb,z,dt,B,C
 *       csrc/supergrok2_mamba_peer_kernels.cu:289-346
 *       grokking_optimizers/mamba3_peer_metanet.py:100-111
 *   recurrence (trapezoidal A_bar, paired RoPE, B_bar*x, y = h.C, gate, D skip)
 *       csrc/supergrok2_mamba_peer_kernels.cu:201-268
 *       grokking_optimizers/mamba3_peer_metanet.py:122-153
 *   chunked evaluation of the same recurrence through 2x2 affine summaries
 *       csrc/supergrok2_mamba_peer_kernels.cu:59-80,444-551,662-769
 *   reverse direction walks t = N-1..0 and writes at t
 *       csrc/supergrok2_mamba_peer_kernels.cu:202,673
 *       grokking_optimizers/mamba3_peer_metanet.py:311-312
 *   out_proj, unsort, GRU, PEER argmax routing, expert MLP, skip, mu, Adam, WD
 *       csrc/supergrok2_mamba_peer_kernels.cu:917-1088
 *       grokking_optimizers/mamba3_peer_metanet.py:158,186-192,334-367
 *       grokking_optimizers/supergrok2.py:451-464
 *
 * chunk_len / window semantics: the sequence (in scan order) is cut into chunks of
 * chunk_len steps.  For every chunk but the last, the 2x2 affine summary
 * (M,b) of each (column j, RoPE pair p) is accumulated from the identity;
 * chunk start states follow by applying the summaries in order to the
 * carried state; each chunk is then replayed directly from its start state.
 * chunk_len <= 0 (or >= N) is the plain sequential recurrence of
 * csrc/supergrok2_mamba_peer_kernels.cu:138-272.  The reference's own
 * chunking (ceil(N/512) steps per thread, Blelloch tree over 512 summaries)
 * is one more member of this family: all of them differ from the sequential
 * result only by re-association of the affine products.
 * window > 0 (a multiple of 64, < chunk_len): the summary of a chunk is built
 * backwards in blocks of `window` steps.  The last block is summarised from
 * the identity; the recurrence contracts (|A_bar| < 1), so the 2x2 part M of
 * that summary is usually vanishingly small: if every |entry| of M in all
 * (j,p) is below 2^-100 the chunk summary is taken as (0, b) -- whatever state
 * entered the block is multiplied by less than 2^-100, far below fp32
 * resolution.  Otherwise the block before it is summarised from the identity
 * and the summary so far is applied on top (M, b) <- (M_late M_early,
 * M_late b_early + b_late), and the test is repeated, until it passes or the
 * chunk start is reached (then the summary is the exact one, re-associated by
 * blocks).  window <= 0 accumulates the whole chunk in one block.
 * Before that walk a windowed summary makes one cheaper attempt: a single block whose length comes from the weights
 * alone (the steps the slowest RoPE pair needs to contract below 2^-100 at the step size of a zero input, plus a
 * margin: sg2_first_block_steps in include/sg2_compose.h), walked with the state part only, while the 2x2 part is
 * bounded by the running product of max(|A_bar_e|, |A_bar_o|) (rotations preserve length).  If the bound is below
 * 2^-100 in every (j,p) the summary is (0, b) with that block's b; otherwise the walk above starts from scratch.
 * Step size and gate of a 64-step tile (fp32 policy, as the kernels): when every timestep of the tile has
 * cmax_g |g| + cmax_s |s| < 2^-5 (cmax: the largest |c_g|, |c_s| of the composed dt and gate rows of the
 * direction), softplus(c_0 + d) and silu(c_0' + d') are evaluated as their cubic Taylor polynomials in d around
 * the zero-input arguments (sg2_softplus_taylor / sg2_silu_taylor in include/sg2_compose.h: within a fraction of an
 * fp32 ulp of the functions, tests/test_oracle_primitives.py); other tiles take the functions themselves.  The
 * float64 policy always takes the functions.
 * A block of 8 steps whose timesteps all pass sg2_poly_ok takes A_bar, sin and cos of every (j,p) from polynomials in
 * dt - dt0 (dt0 = the column's step size for a zero input; sg2_abar_poly, sg2_sincos_poly), before the tiny-angle
 * and shared-reciprocal forms are considered (fp32 policy only).  The replay uses, with a tighter limit, quadratics
 * for the four products of its update instead (sg2_pair_products): he' = P1 he + N2 ho + b_e, ho' = P3 ho + P4 he + b_o.
 * A (j,p) whose M is exactly zero hands on b itself as the next start state
 * when the state before it is finite (0 * h + b is then b): the kernels read no
 * earlier state at all when every summary of a call is of that kind and every
 * carried state is finite.  A non-finite state is multiplied through and keeps
 * the rest of the tensor non-finite, as in the reference.
 *
 * Parity status: the reference's tests hold no golden vectors for this path
 * (tests/test_supergrok2.py checks finiteness and run-to-run determinism
 * only) and its CUDA kernels cannot run here, so every function below is
 * pinned by checks that do not share its code: numpy's stable argsort and a
 * brute-force rank (sort); closed forms of the recurrence, structural
 * identities and torch.optim.AdamW (tests/test_oracle_sg2.py); special cases
 * in which the mathematics fixes the per-element part -- GRU gates closed or
 * open, one input column at a time, PEER winners known by construction with
 * exact ties, hand-evaluated expert MLPs, the index clamp, the sense of the
 * RoPE rotation -- each shown to fail on a build of this file with the
 * corresponding mistake injected (tests/test_oracle_sg2_pins.py).
 */
#include <algorithm>
#include <cmath>
#include <cstdint>
#include <cstring>
#include <vector>

#include "../include/sg_math.h"
#include "../include/sg2_compose.h"

namespace {

struct Dims {
    int d_model, d_state, d_inner, gru_hidden, num_heads, pk_dim, expert_hidden, num_experts;
};

/* pointer order = argument order of supergrok2_mamba_peer_batched_step
 * (csrc/ops.h:548-581) from input_proj_W to expert_b2 */
enum {
    W_IN_W = 0, W_IN_B,
    W_F_INPROJ, W_F_DTW, W_F_DTB, W_F_B, W_F_C, W_F_ALOG, W_F_D, W_F_ROPE, W_F_OUT,
    W_B_INPROJ, W_B_DTW, W_B_DTB, W_B_B, W_B_C, W_B_ALOG, W_B_D, W_B_ROPE, W_B_OUT,
    W_GRU_WZ, W_GRU_BZ, W_GRU_WR, W_GRU_BR, W_GRU_WH, W_GRU_BH,
    W_PEER_Q, W_KEYS_A, W_KEYS_B,
    W_EXP_W1, W_EXP_B1, W_EXP_W2, W_EXP_B2,
    W_COUNT
};

enum { S_ALPHA = 0, S_LAMB, S_BETA1, S_BC1, S_BC2, S_RESCALE, S_BETA2, S_LR, S_WD, S_EPS, S_COUNT };

/* ---------------- 16-bit float conversions (round to nearest even) -------- */
inline float bf16_to_f(uint16_t h) {
    uint32_t u = (uint32_t)h << 16;
    float f;
    std::memcpy(&f, &u, 4);
    return f;
}
inline uint16_t f_to_bf16(float f) {
    uint32_t u;
    std::memcpy(&u, &f, 4);
    if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x40);
    u += 0x7fffu + ((u >> 16) & 1u);
    return (uint16_t)(u >> 16);
}
inline float f16_to_f(uint16_t h) {
    uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
    uint32_t exp = (h >> 10) & 0x1f, man = h & 0x3ffu, u;
    if (exp == 0) {
        if (man == 0) u = sign;
        else {
            int e = -1;
            do { e++; man <<= 1; } while ((man & 0x400u) == 0);
            u = sign | ((uint32_t)(127 - 15 - e) << 23) | ((man & 0x3ffu) << 13);
        }
    } else if (exp == 31) u = sign | 0x7f800000u | (man << 13);
    else u = sign | ((exp + 112) << 23) | (man << 13);
    float f;
    std::memcpy(&f, &u, 4);
    return f;
}
inline uint16_t f_to_f16(float f) {
    uint32_t x;
    std::memcpy(&x, &f, 4);
    uint32_t sign = (x >> 16) & 0x8000u;
    x &= 0x7fffffffu;
    if (x >= 0x7f800000u) return (uint16_t)(sign | 0x7c00u | (x > 0x7f800000u ? 0x200u : 0));
    if (x >= 0x477ff000u) return (uint16_t)(sign | 0x7c00u);          /* overflow -> inf */
    if (x < 0x33000001u) return (uint16_t)sign;                       /* underflow -> 0 */
    int e = (int)(x >> 23);
    uint32_t m = (x & 0x7fffffu) | 0x800000u;
    int shift;
    uint32_t base;
    if (e < 113) { shift = 126 - e; base = 0; }        /* subnormal half */
    else { shift = 13; base = (uint32_t)(e - 112) << 10; m &= 0x7fffffu; }
    uint32_t q = m >> shift, rem = m & ((1u << shift) - 1u), half = 1u << (shift - 1);
    uint32_t r = base + q;
    if (rem > half || (rem == half && (r & 1u))) r++;
    return (uint16_t)(sign | r);
}
inline float load_as_f(const void* p, int dtype, int64_t i) {
    if (dtype == 0) return ((const float*)p)[i];
    if (dtype == 1) return f16_to_f(((const uint16_t*)p)[i]);
    return bf16_to_f(((const uint16_t*)p)[i]);
}
inline void store_from_f(void* p, int dtype, int64_t i, float v) {
    if (dtype == 0) ((float*)p)[i] = v;
    else if (dtype == 1) ((uint16_t*)p)[i] = f_to_f16(v);
    else ((uint16_t*)p)[i] = f_to_bf16(v);
}

/* ---------------- arithmetic policies ------------------------------------ */
struct F32 {
    typedef float R;
    static R fma(R a, R b, R c) { return sg_fma(a, b, c); }
    static R exp(R x) { return sg_exp(x); }
    static R softplus(R x) { return sg_softplus(x); }
    static R sigmoid(R x) { return sg_sigmoid(x); }
    static R silu(R x) { return sg_silu(x); }
    /* gates of n columns in groups of `group` consecutive ones, as the kernel's waves form them (sg_silu_block) */
    static void silu_groups(const R* z, int n, int group, R* out) {
        for (int j0 = 0; j0 < n; j0 += group) sg_silu_block(group, z + j0, out + j0);
    }
    /* the per-element kernel forms the 2 x 4 GRU gates, and the 4 candidates, with one reciprocal each */
    static void sigmoid_group(int n, const R* x, R* out) {
        if (n == 8) sg_sigmoid_block(n, x, out);
        else for (int k = 0; k < n; k++) out[k] = sg_sigmoid(x[k]);
    }
    static void tanh_group(int n, const R* x, R* out) {
        if (n == 4) sg_tanh_block(n, x, out);
        else for (int k = 0; k < n; k++) out[k] = sg_tanh(x[k]);
    }
    static R tanh(R x) { return sg_tanh(x); }
    static R sqrt(R x) { return __builtin_sqrtf(x); }
    static void sincos(R t, R* s, R* c) { sg_sincos(t, s, c); }
    /* A is the (negative) continuous-time pole; the primitive wants -A/2 */
    static void abar_pair(R dt, R A_e, R A_o, R* e, R* o) { sg_abar_pair(dt, -0.5f * A_e, -0.5f * A_o, e, o); }
};
struct F64 {
    typedef double R;
    static R fma(R a, R b, R c) { return a * b + c; }
    static R exp(R x) { return std::exp(x); }
    static R softplus(R x) { return (x > 20.0) ? x : std::log(1.0 + std::exp(x)); }
    static R sigmoid(R x) { return 1.0 / (1.0 + std::exp(-x)); }
    static R silu(R x) { return x / (1.0 + std::exp(-x)); }
    static void silu_groups(const R* z, int n, int, R* out) {
        for (int j = 0; j < n; j++) out[j] = silu(z[j]);
    }
    static void sigmoid_group(int n, const R* x, R* out) { for (int k = 0; k < n; k++) out[k] = sigmoid(x[k]); }
    static void tanh_group(int n, const R* x, R* out) { for (int k = 0; k < n; k++) out[k] = tanh(x[k]); }
    static R tanh(R x) { return std::tanh(x); }
    static R sqrt(R x) { return std::sqrt(x); }
    static void sincos(R t, R* s, R* c) { *s = std::sin(t); *c = std::cos(t); }
    static void abar_pair(R dt, R A_e, R A_o, R* e, R* o) {
        *e = (1.0 + dt * A_e / 2.0) / (1.0 - dt * A_e / 2.0 + 1e-8);
        *o = (1.0 + dt * A_o / 2.0) / (1.0 - dt * A_o / 2.0 + 1e-8);
    }
};

/* ---------------- stable ascending sort of |g| ---------------------------- */
void sort_perm(const float* g, int64_t N, int32_t* perm) {
    std::vector<uint32_t> key(N);
    for (int64_t i = 0; i < N; i++) {
        float v = sg_isfinite(g[i]) ? g[i] : 0.0f;
        key[i] = (uint32_t)sg_f2i(sg_abs(v));      /* non-negative floats order like their bits */
        perm[i] = (int32_t)i;
    }
    std::stable_sort(perm, perm + N, [&](int32_t a, int32_t b) { return key[a] < key[b]; });
}

/* ---------------- one scan direction -------------------------------------- */
template <class O>
struct DirW {
    const float *in_proj, *dt_W, *dt_b, *Bp, *Cp, *A_log, *D, *rope, *out_proj;
    /* fp32 policy: composed coefficient triples [group][row][3] (include/sg2_compose.h), as the device uses them */
    std::vector<float> comp;
    int comp_rows;
    /* fp32 policy: cubic Taylor polynomials of the step size and of the gate around their zero-input arguments,
     * [dt | gate][row][4], and the largest |c_g|, |c_s| of those rows (include/sg2_compose.h) */
    std::vector<float> tay;
    float cmax[2];
    /* fp32 policy: every (column, pair) as polynomials in dt - dt0 (sg2_abar_poly, sg2_sincos_poly):
     * [lane][pe 4 | po 4 | qs 3 | qc 3], and the two factors of sg2_poly_ok */
    std::vector<float> lane_poly;
    float kpoly[2];
    /* the output pass: the four products of every (column, pair) as quadratics, [lane][P1 | N2 | P3 | P4][3]
     * (sg2_pair_products), and the factors of their limit */
    std::vector<float> lane_prod;
    float kprod[2];
};

template <class O>
struct StepProj {           /* per-timestep projections */
    typename O::R xb[32], z[32], dt[32], B[32], C[32];
    bool taylor;            /* the tile uses the Taylor polynomials: gate[] holds the gates themselves */
    typename O::R gate[32];
};

/* gs: the element's (gradient, sharpness); x: its input projection.  The fp32 policy evaluates the composed
 * affine maps from (g, s); the fp64 policy evaluates the reference's chain of projections from x literally. */
template <class O>
void project(const Dims& d, const DirW<O>& w, const typename O::R* x, const float* gs, bool need_zc, bool taylor, StepProj<O>& o) {
    typedef typename O::R R;
    const int dm = d.d_model, di = d.d_inner, ds = d.d_state;
    o.taylor = false;
    if (sizeof(R) == 4) {
        const float* c = w.comp.data();
        const int rows = w.comp_rows;
        auto eval = [&](int group, int row) { return (R)sg2_comp_eval(c + ((size_t)group * rows + row) * 3, gs[0], gs[1]); };
        auto poly = [&](int kind, int group, int row) {
            return (R)sg2_taylor_eval(&w.tay[((size_t)kind * rows + row) * 4], sg2_taylor_delta(c + ((size_t)group * rows + row) * 3, gs[0], gs[1]));
        };
        o.taylor = taylor;
        for (int j = 0; j < di; j++) {
            o.xb[j] = eval(SG2_COMP_XB, j);
            o.z[j] = need_zc ? eval(SG2_COMP_Z, j) : (R)0;
            o.dt[j] = taylor ? poly(0, SG2_COMP_DT, j) : O::softplus(eval(SG2_COMP_DT, j));
            o.gate[j] = (taylor && need_zc) ? poly(1, SG2_COMP_Z, j) : (R)0;
        }
        for (int s = 0; s < ds; s++) {
            o.B[s] = eval(SG2_COMP_B, s);
            o.C[s] = need_zc ? eval(SG2_COMP_C, s) : (R)0;
        }
        return;
    }
    for (int j = 0; j < di; j++) {
        R a = 0, b = 0;
        for (int k = 0; k < dm; k++) a = O::fma((R)w.in_proj[j * dm + k], x[k], a);
        if (need_zc)
            for (int k = 0; k < dm; k++) b = O::fma((R)w.in_proj[(j + di) * dm + k], x[k], b);
        o.xb[j] = a;
        o.z[j] = b;
    }
    for (int j = 0; j < di; j++) {
        R a = (R)w.dt_b[j];
        for (int k = 0; k < di; k++) a = O::fma((R)w.dt_W[j * di + k], o.xb[k], a);
        o.dt[j] = O::softplus(a);
    }
    for (int s = 0; s < ds; s++) {
        R a = 0, b = 0;
        for (int k = 0; k < di; k++) a = O::fma((R)w.Bp[s * di + k], o.xb[k], a);
        if (need_zc)
            for (int k = 0; k < di; k++) b = O::fma((R)w.Cp[s * di + k], o.xb[k], b);
        o.B[s] = a;
        o.C[s] = b;
    }
}

/* Coefficients of up to 64 consecutive scan steps (one tile of the device kernel): projections, A_bar and
 * sin/cos per (step, column, pair).  The fp32 policy groups the A_bar exactly like the device: blocks of 8
 * steps counted from the tile start share one reciprocal per lane (sg_abar_block_*), unless some lane of the
 * block's 64-lane wave (lanes ordered column-major, 8 pairs per column) exceeds SG_ABAR_BLOCK_LIMIT; the ragged
 * end of a tile and the fp64 policy take the per-step formula. */
template <class O>
struct TileCoef {
    std::vector<StepProj<O>> sp;
    std::vector<typename O::R> ae, ao, sn, cs;
    /* output pass: blocks of 8 steps that hold the products instead (ae = P1, sn = N2, ao = P3, cs = P4) */
    std::vector<char> prod_block;
};
enum { ORC_TILE = 64, ORC_BLOCK = 8, ORC_WAVE = 64 };

template <class O>
void tile_coefficients(const Dims& d, const DirW<O>& w, const std::vector<typename O::R>& A, const typename O::R* x,
                       const float* gs, int64_t N, bool reverse, int64_t u0, int cnt, bool need_zc, TileCoef<O>& tc) {
    typedef typename O::R R;
    const int dm = d.d_model, di = d.d_inner, ds = d.d_state, hp = ds / 2, lanes = di * hp;
    tc.sp.resize(ORC_TILE);
    tc.ae.resize((size_t)ORC_TILE * lanes);
    tc.ao.resize((size_t)ORC_TILE * lanes);
    tc.sn.resize((size_t)ORC_TILE * lanes);
    tc.cs.resize((size_t)ORC_TILE * lanes);
    /* the tile takes the Taylor polynomials if every one of its timesteps qualifies (the device decides per 64-step tile) */
    bool taylor = sizeof(R) == 4;
    for (int k = 0; k < cnt && taylor; k++) {
        const int64_t u = u0 + k, t = reverse ? (N - 1 - u) : u;
        taylor = sg2_taylor_ok(w.cmax[0], w.cmax[1], gs[2 * t], gs[2 * t + 1]) != 0;
    }
    for (int k = 0; k < cnt; k++) {
        const int64_t u = u0 + k, t = reverse ? (N - 1 - u) : u;
        project<O>(d, w, x + t * dm, gs + 2 * t, need_zc, taylor, tc.sp[k]);
        for (int j = 0; j < di; j++)
            for (int p = 0; p < hp; p++)
                O::sincos(tc.sp[k].dt[j] * (R)w.rope[j * hp + p], &tc.sn[(size_t)k * lanes + j * hp + p],
                          &tc.cs[(size_t)k * lanes + j * hp + p]);
    }
    /* blocks of 8 steps whose timesteps all pass sg2_poly_ok take A_bar, sin and cos from the lane polynomials (summary
     * pass) or, with the tighter limit of the output pass (need_zc), the four products of the update */
    std::vector<char> poly_block(ORC_TILE / ORC_BLOCK, 0);
    tc.prod_block.assign(ORC_TILE / ORC_BLOCK, 0);
    if (sizeof(R) == 4) {
        const float* lim = need_zc ? w.kprod : w.kpoly;
        /* (the device knows before its projections whether the whole 64-step tile qualifies) */
        bool whole_tile_poly = taylor && cnt == ORC_TILE;
        for (int k = 0; k < cnt && whole_tile_poly; k++) {
            const int64_t u = u0 + k, t = reverse ? (N - 1 - u) : u;
            whole_tile_poly = sg2_poly_ok(lim[0], lim[1], gs[2 * t], gs[2 * t + 1]) != 0;
        }
        for (int b0 = 0; b0 + ORC_BLOCK <= cnt; b0 += ORC_BLOCK) {
            bool ok = true;
            for (int q = 0; q < ORC_BLOCK && ok; q++) {
                const int64_t u = u0 + b0 + q, t = reverse ? (N - 1 - u) : u;
                ok = sg2_poly_ok(lim[0], lim[1], gs[2 * t], gs[2 * t + 1]) != 0;
            }
            poly_block[b0 / ORC_BLOCK] = ok;
            if (!ok) continue;
            if (need_zc) {
                tc.prod_block[b0 / ORC_BLOCK] = 1;
                /* the linear parts alone: a whole tile on Taylor step sizes and products, and this block's inputs
                 * SG2_PROD_LINEAR_FACTOR times further inside the limit */
                bool linear = whole_tile_poly;
                for (int q = 0; q < ORC_BLOCK && linear; q++) {
                    const int64_t u = u0 + b0 + q, t = reverse ? (N - 1 - u) : u;
                    linear = sg2_poly_ok(SG2_PROD_LINEAR_FACTOR * lim[0], SG2_PROD_LINEAR_FACTOR * lim[1], gs[2 * t], gs[2 * t + 1]) != 0;
                }
                for (int q = 0; q < ORC_BLOCK; q++)
                    for (int l = 0; l < lanes; l++) {
                        const float* k = &w.lane_prod[(size_t)l * 12];
                        const float dd = (float)tc.sp[b0 + q].dt[l / hp] - w.tay[((size_t)0 * w.comp_rows + l / hp) * 4];
                        tc.ae[(size_t)(b0 + q) * lanes + l] = (R)(linear ? sg2_poly1(k, dd) : sg2_poly2(k, dd));
                        tc.sn[(size_t)(b0 + q) * lanes + l] = (R)(linear ? sg2_poly1(k + 3, dd) : sg2_poly2(k + 3, dd));
                        tc.ao[(size_t)(b0 + q) * lanes + l] = (R)(linear ? sg2_poly1(k + 6, dd) : sg2_poly2(k + 6, dd));
                        tc.cs[(size_t)(b0 + q) * lanes + l] = (R)(linear ? sg2_poly1(k + 9, dd) : sg2_poly2(k + 9, dd));
                    }
                continue;
            }
            for (int q = 0; q < ORC_BLOCK; q++)
                for (int l = 0; l < lanes; l++) {
                    const float* lp = &w.lane_poly[(size_t)l * 14];
                    const float dd = (float)tc.sp[b0 + q].dt[l / hp] - w.tay[((size_t)0 * w.comp_rows + l / hp) * 4];
                    tc.ae[(size_t)(b0 + q) * lanes + l] = (R)sg2_poly3(lp, dd);
                    tc.ao[(size_t)(b0 + q) * lanes + l] = (R)sg2_poly3(lp + 4, dd);
                    tc.sn[(size_t)(b0 + q) * lanes + l] = (R)sg2_poly2(lp + 8, dd);
                    tc.cs[(size_t)(b0 + q) * lanes + l] = (R)sg2_poly2(lp + 11, dd);
                }
        }
    }
    if (sizeof(R) == 4) {
        /* blocks whose angles are all below SG_SINCOS_TINY_LIMIT, over the 8 steps and the columns of a wave, take
         * sg_sincos_tiny (the device decides with dt * max_p |rope[j,p]| per column) */
        std::vector<float> fmax(di, 0.0f);
        for (int j = 0; j < di; j++)
            for (int p = 0; p < hp; p++) fmax[j] = sg_max(fmax[j], sg_abs(w.rope[j * hp + p]));
        for (int b0 = 0; b0 + ORC_BLOCK <= cnt; b0 += ORC_BLOCK)
            for (int wave0 = 0; wave0 < lanes && !poly_block[b0 / ORC_BLOCK]; wave0 += ORC_WAVE) {
                const int wave1 = std::min(lanes, wave0 + ORC_WAVE);
                bool tiny = true;
                for (int q = 0; q < ORC_BLOCK && tiny; q++)
                    for (int j = wave0 / hp; j <= (wave1 - 1) / hp; j++)
                        if (!((float)tc.sp[b0 + q].dt[j] * fmax[j] < SG_SINCOS_TINY_LIMIT)) { tiny = false; break; }
                if (!tiny) continue;
                for (int q = 0; q < ORC_BLOCK; q++)
                    for (int l = wave0; l < wave1; l++) {
                        float sn, cs, coef[6];
                        sg_sincos_tiny_coef(w.rope[l], coef);
                        sg_sincos_tiny_dt((float)tc.sp[b0 + q].dt[l / hp], coef, &sn, &cs);
                        tc.sn[(size_t)(b0 + q) * lanes + l] = (R)sn;
                        tc.cs[(size_t)(b0 + q) * lanes + l] = (R)cs;
                    }
            }
    }
    int k0 = 0;
    if (sizeof(R) == 4) {
        std::vector<float> de((size_t)lanes * ORC_BLOCK), dod((size_t)lanes * ORC_BLOCK), P((size_t)lanes * ORC_BLOCK);
        for (; k0 + ORC_BLOCK <= cnt; k0 += ORC_BLOCK) {
            for (int wave0 = 0; wave0 < lanes && !poly_block[k0 / ORC_BLOCK]; wave0 += ORC_WAVE) {
                const int wave1 = std::min(lanes, wave0 + ORC_WAVE);
                bool block_ok = true;
                for (int l = wave0; l < wave1; l++) {
                    const int j = l / hp, p = l % hp;
                    float dts[ORC_BLOCK];
                    for (int q = 0; q < ORC_BLOCK; q++) dts[q] = (float)tc.sp[k0 + q].dt[j];
                    const float last = sg_abar_block_prefix(ORC_BLOCK, dts, -0.5f * (float)A[j * ds + 2 * p], -0.5f * (float)A[j * ds + 2 * p + 1],
                                                            &de[(size_t)l * ORC_BLOCK], &dod[(size_t)l * ORC_BLOCK], &P[(size_t)l * ORC_BLOCK]);
                    if (!(last < SG_ABAR_BLOCK_LIMIT)) block_ok = false;
                }
                for (int l = wave0; l < wave1; l++) {
                    const int j = l / hp, p = l % hp;
                    float e[ORC_BLOCK], o[ORC_BLOCK];
                    if (block_ok) {
                        sg_abar_block_finish(ORC_BLOCK, &de[(size_t)l * ORC_BLOCK], &dod[(size_t)l * ORC_BLOCK], &P[(size_t)l * ORC_BLOCK], e, o);
                    } else {
                        for (int q = 0; q < ORC_BLOCK; q++)
                            sg_abar_pair((float)tc.sp[k0 + q].dt[j], -0.5f * (float)A[j * ds + 2 * p], -0.5f * (float)A[j * ds + 2 * p + 1], &e[q], &o[q]);
                    }
                    for (int q = 0; q < ORC_BLOCK; q++) {
                        tc.ae[(size_t)(k0 + q) * lanes + l] = (R)e[q];
                        tc.ao[(size_t)(k0 + q) * lanes + l] = (R)o[q];
                    }
                }
            }
        }
    }
    for (; k0 < cnt; k0++)
        for (int j = 0; j < di; j++)
            for (int p = 0; p < hp; p++)
                O::abar_pair(tc.sp[k0].dt[j], A[j * ds + 2 * p], A[j * ds + 2 * p + 1], &tc.ae[(size_t)k0 * lanes + j * hp + p],
                             &tc.ao[(size_t)k0 * lanes + j * hp + p]);
}

/* x: [N][d_model] in sorted order.  h: [d_inner][d_state] carried state,
 * updated in place.  ctx: [N][d_model], written at sorted position t. */
template <class O>
void scan_dir(const Dims& d, const DirW<O>& w, const typename O::R* x, const float* gs, int64_t N, bool reverse,
              int64_t chunk_len, int64_t window, int64_t first_block, typename O::R* h, typename O::R* ctx) {
    typedef typename O::R R;
    const int dm = d.d_model, di = d.d_inner, ds = d.d_state, hp = ds / 2;
    if (N <= 0) return;
    if (chunk_len <= 0 || chunk_len > N) chunk_len = N;
    const int64_t nchunks = (N + chunk_len - 1) / chunk_len;

    std::vector<R> A(di * ds);
    for (int i = 0; i < di * ds; i++) A[i] = -O::exp((R)w.A_log[i]);

    std::vector<R> hstart((size_t)nchunks * di * ds);
    std::copy(h, h + di * ds, hstart.begin());
    TileCoef<O> tc;

    /* pass 1 + 2: summaries of chunks 0..nchunks-2, start states of 1..nchunks-1 */
    std::vector<R> sm(di * hp * 6);
    std::vector<R> late(di * hp * 6);
    for (int64_t c = 0; c + 1 < nchunks; c++) {
        /* the chunk is walked backwards in blocks of `window` steps: each block is summarised from the identity, the
         * summary of everything after it is applied on top, and the walk stops once the 2x2 part has contracted */
        const int64_t u0 = c * chunk_len, u1 = (c + 1) * chunk_len;
        int64_t blk_end = u1, blk_first = (window > 0 && window < chunk_len) ? std::max(u0, u1 - window) : u0;
        bool have_late = false;
        /* first attempt (windowed summaries only): ONE block of first_block steps -- what the slowest pair needs to
         * contract at the step size of a zero input, sg2_first_block_steps -- walked with the state part alone and,
         * in place of the 2x2 part, the running product of max(|A_bar_e|, |A_bar_o|), which bounds its norm.  Below
         * 2^-100 in every (j,p): the summary is (0, b).  Otherwise the general walk below starts from scratch. */
        bool lite_done = false;
        if (blk_first > u0 && first_block > 0 && u1 - first_block > u0) {
            std::vector<R> bound(di * hp, (R)1);
            for (int i = 0; i < di * hp; i++) {
                R* m = &sm[i * 6];
                m[0] = 0; m[1] = 0; m[2] = 0; m[3] = 0; m[4] = 0; m[5] = 0;
            }
            for (int64_t tile0 = u1 - first_block; tile0 < u1; tile0 += ORC_TILE) {
                const int cnt = (int)std::min<int64_t>(ORC_TILE, u1 - tile0);
                tile_coefficients<O>(d, w, A, x, gs, N, reverse, tile0, cnt, false, tc);
                for (int k = 0; k < cnt; k++) {
                    const StepProj<O>& sp = tc.sp[k];
                    for (int j = 0; j < di; j++) {
                        const R dt = sp.dt[j], xb = sp.xb[j];
                        for (int p = 0; p < hp; p++) {
                            const size_t li = (size_t)k * di * hp + j * hp + p;
                            const R ae = tc.ae[li], ao = tc.ao[li], sn = tc.sn[li], cs = tc.cs[li];
                            const R ux = dt * xb, be = ux * sp.B[2 * p], bo = ux * sp.B[2 * p + 1];
                            R* m = &sm[(j * hp + p) * 6];
                            const R abs_e = ae < 0 ? -ae : ae, abs_o = ao < 0 ? -ao : ao;
                            bound[j * hp + p] = bound[j * hp + p] * (abs_e > abs_o ? abs_e : abs_o);
                            const R ve = m[4], vo = m[5];
                            const R re = O::fma(ve, cs, -(vo * sn));
                            const R ro = O::fma(vo, cs, ve * sn);
                            m[4] = O::fma(ae, re, be);
                            m[5] = O::fma(ao, ro, bo);
                        }
                    }
                }
            }
            lite_done = true;
            for (int i = 0; i < di * hp; i++)
                if (!(bound[i] < (R)7.888609052210118e-31)) { lite_done = false; break; }
        }
        for (; !lite_done;) {
            for (int i = 0; i < di * hp; i++) {
                R* m = &sm[i * 6];
                m[0] = 1; m[1] = 0; m[2] = 0; m[3] = 1; m[4] = 0; m[5] = 0;   /* col0=(m0,m1) col1=(m2,m3) b=(m4,m5) */
            }
            for (int64_t tile0 = blk_first; tile0 < blk_end; tile0 += ORC_TILE) {
                const int cnt = (int)std::min<int64_t>(ORC_TILE, blk_end - tile0);
                tile_coefficients<O>(d, w, A, x, gs, N, reverse, tile0, cnt, false, tc);
                for (int k = 0; k < cnt; k++) {
                    const StepProj<O>& sp = tc.sp[k];
                    for (int j = 0; j < di; j++) {
                        const R dt = sp.dt[j], xb = sp.xb[j];
                        for (int p = 0; p < hp; p++) {
                            const size_t li = (size_t)k * di * hp + j * hp + p;
                            const R ae = tc.ae[li], ao = tc.ao[li], sn = tc.sn[li], cs = tc.cs[li];
                            const R ux = dt * xb, be = ux * sp.B[2 * p], bo = ux * sp.B[2 * p + 1];
                            R* m = &sm[(j * hp + p) * 6];
                            for (int v = 0; v < 3; v++) {
                                const R ve = m[2 * v], vo = m[2 * v + 1];
                                const R re = O::fma(ve, cs, -(vo * sn));
                                const R ro = O::fma(vo, cs, ve * sn);
                                if (v < 2) { m[2 * v] = ae * re; m[2 * v + 1] = ao * ro; }
                                else { m[4] = O::fma(ae, re, be); m[5] = O::fma(ao, ro, bo); }
                            }
                        }
                    }
                }
            }
            if (have_late)       /* sm covers [blk_first, blk_end), late covers [blk_end, u1): both = late o sm */
                for (int i = 0; i < di * hp; i++) {
                    const R* L = &late[i * 6];
                    R* m = &sm[i * 6];
                    const R e0 = m[0], e1 = m[1], e2 = m[2], e3 = m[3], e4 = m[4], e5 = m[5];
                    m[0] = O::fma(L[0], e0, L[2] * e1);
                    m[1] = O::fma(L[1], e0, L[3] * e1);
                    m[2] = O::fma(L[0], e2, L[2] * e3);
                    m[3] = O::fma(L[1], e2, L[3] * e3);
                    m[4] = O::fma(L[0], e4, O::fma(L[2], e5, L[4]));
                    m[5] = O::fma(L[1], e4, O::fma(L[3], e5, L[5]));
                }
            if (blk_first == u0) break;
            bool contracted = true;      /* every |M entry| < 2^-100 (a NaN counts as not contracted) */
            for (int i = 0; i < di * hp && contracted; i++)
                for (int k = 0; k < 4; k++) {
                    const R a = sm[i * 6 + k] < 0 ? -sm[i * 6 + k] : sm[i * 6 + k];
                    if (!(a < (R)7.888609052210118e-31)) { contracted = false; break; }
                }
            if (contracted) {
                for (int i = 0; i < di * hp; i++)
                    for (int k = 0; k < 4; k++) sm[i * 6 + k] = 0;
                break;
            }
            late = sm;
            have_late = true;
            blk_end = blk_first;
            blk_first = std::max(u0, blk_first - window);
        }
        const R* h0 = &hstart[(size_t)c * di * ds];
        R* h1 = &hstart[(size_t)(c + 1) * di * ds];
        for (int j = 0; j < di; j++)
            for (int p = 0; p < hp; p++) {
                const R* m = &sm[(j * hp + p) * 6];
                const R he = h0[j * ds + 2 * p], ho = h0[j * ds + 2 * p + 1];
                /* an exactly zero 2x2 part hands on the offset itself -- what 0 * h + b is for a finite h; the kernels then
                 * never read the earlier state.  A state that is not finite goes through the product (0 * inf = NaN) and
                 * stays non-finite to the end of the tensor, as in the reference (csrc/supergrok2_mamba_peer_kernels.cu:
                 * 444-551 applies every chunk's summary to the state before it). */
                const bool zero = m[0] == 0 && m[1] == 0 && m[2] == 0 && m[3] == 0 && std::isfinite((double)he) && std::isfinite((double)ho);
                h1[j * ds + 2 * p] = zero ? m[4] : O::fma(m[0], he, O::fma(m[2], ho, m[4]));
                h1[j * ds + 2 * p + 1] = zero ? m[5] : O::fma(m[1], he, O::fma(m[3], ho, m[5]));
            }
    }

    /* pass 3: replay every chunk from its start state */
    std::vector<R> hc(di * ds), yp(hp), out(di);
    R gate[32];
    /* the kernel's waves each gate d_inner / (waves per chunk) consecutive columns with one shared reciprocal */
    const int gate_group = di / std::max(1, di * hp / 64);
    for (int64_t c = 0; c < nchunks; c++) {
        std::copy(&hstart[(size_t)c * di * ds], &hstart[(size_t)c * di * ds] + di * ds, hc.begin());
        const int64_t u_end = std::min<int64_t>((c + 1) * chunk_len, N);
        for (int64_t tile0 = c * chunk_len; tile0 < u_end; tile0 += ORC_TILE) {
            const int cnt = (int)std::min<int64_t>(ORC_TILE, u_end - tile0);
            tile_coefficients<O>(d, w, A, x, gs, N, reverse, tile0, cnt, true, tc);
            for (int k = 0; k < cnt; k++) {
                const int64_t u = tile0 + k, t = reverse ? (N - 1 - u) : u;
                const StepProj<O>& sp = tc.sp[k];
                if (sp.taylor) for (int j = 0; j < di; j++) gate[j] = sp.gate[j];
                else O::silu_groups(sp.z, di, gate_group, gate);
                for (int j = 0; j < di; j++) {
                    const R dt = sp.dt[j], xb = sp.xb[j];
                    for (int p = 0; p < hp; p++) {
                        const size_t li = (size_t)k * di * hp + j * hp + p;
                        const R ae = tc.ae[li], ao = tc.ao[li], sn = tc.sn[li], cs = tc.cs[li];
                        const R ux = dt * xb, be = ux * sp.B[2 * p], bo = ux * sp.B[2 * p + 1];
                        const R he = hc[j * ds + 2 * p], ho = hc[j * ds + 2 * p + 1];
                        R ne, no;
                        if (tc.prod_block[k / ORC_BLOCK]) {      /* ae = P1, sn = N2, ao = P3, cs = P4 */
                            ne = O::fma(ae, he, O::fma(sn, ho, be));
                            no = O::fma(ao, ho, O::fma(cs, he, bo));
                        } else {
                            const R re = O::fma(he, cs, -(ho * sn));
                            const R ro = O::fma(ho, cs, he * sn);
                            ne = O::fma(ae, re, be);
                            no = O::fma(ao, ro, bo);
                        }
                        hc[j * ds + 2 * p] = ne;
                        hc[j * ds + 2 * p + 1] = no;
                        yp[p] = O::fma(no, sp.C[2 * p + 1], ne * sp.C[2 * p]);
                    }
                    /* sum over the RoPE pairs in the kernels' order: the group is folded in halves, mirrored
                     * (y_i + y_(n-1-i)), until four sums are left; those as (s0 + s1) + (s2 + s3) */
                    int n = hp;
                    for (; n > 4; n /= 2)
                        for (int p = 0; p < n / 2; p++) yp[p] = yp[p] + yp[n - 1 - p];
                    for (int st = 1; st < n; st *= 2)
                        for (int p = 0; p + st < n; p += 2 * st) yp[p] = yp[p] + yp[p + st];
                    out[j] = O::fma(yp[0], gate[j], (R)w.D[j] * xb);
                }
                for (int dd = 0; dd < dm; dd++) {
                    R a = 0;
                    for (int j = 0; j < di; j++) a = O::fma((R)w.out_proj[dd * di + j], out[j], a);
                    ctx[t * dm + dd] = a;
                }
            }
        }
    }
    std::copy(hc.begin(), hc.end(), h);
}

/* ---------------- full step for one tensor -------------------------------- */
template <class O>
int step_tensor(const Dims& d, const float* const* W, int64_t chunk_len, int64_t window, int dtype, void* param,
                const void* grad, const void* sharp, float* ea_io, float* easq_io, float* mu_io,
                float* gru_io, float* mfwd_io, float* mbwd_io, int64_t N, const float* sc,
                int32_t* expert_counts, int32_t* perm_out, int32_t* eidx_out, float* ctx_out,
                float* margin_out, float* smart_out) {
    typedef typename O::R R;
    const int dm = d.d_model, di = d.d_inner, ds = d.d_state, gh = d.gru_hidden, H = d.num_heads;
    const int pk = d.pk_dim, eh = d.expert_hidden, E = d.num_experts, hd = dm / 2;
    if (N <= 0) return 0;
    if (ds % 2 || ds > 32 || dm > 16 || gh > 8 || di > 32 || di % 4) return 1;

    std::vector<float> g(N), s(N);
    for (int64_t i = 0; i < N; i++) {
        float gv = load_as_f(grad, dtype, i), sv = load_as_f(sharp, dtype, i);
        g[i] = sg_isfinite(gv) ? gv : 0.0f;
        s[i] = sg_isfinite(sv) ? sv : 0.0f;
    }
    std::vector<int32_t> perm(N);
    sort_perm(g.data(), N, perm.data());
    if (perm_out) std::copy(perm.begin(), perm.end(), perm_out);

    /* input projection, gathered into sorted order */
    std::vector<R> x((size_t)N * dm);
    std::vector<float> gs_sorted((size_t)N * 2);
    for (int64_t t = 0; t < N; t++) {
        const R gv = g[perm[t]], sv = s[perm[t]];
        gs_sorted[2 * t] = g[perm[t]];
        gs_sorted[2 * t + 1] = s[perm[t]];
        for (int k = 0; k < dm; k++)
            x[t * dm + k] = O::fma((R)W[W_IN_W][2 * k + 1], sv, (R)W[W_IN_W][2 * k] * gv) + (R)W[W_IN_B][k];
    }

    /* length of a summary's first block, from the weights alone (the kernels' k_compose does the same) */
    int64_t first_block = 0;
    {
        int largest = 0, any_zero = 0;
        for (int dir = 0; dir < 2; dir++) {
            const int b = dir ? W_B_INPROJ : W_F_INPROJ;
            for (int j = 0; j < di; j++) {
                float c[3];
                sg2_compose_one(SG2_COMP_DT, j, dm, di, W[W_IN_W], W[W_IN_B], W[b], W[b + 1], W[b + 2], W[b + 3], W[b + 4], c);
                const float dt0 = sg_softplus(c[2]);
                const float* alog = W[b + 5] + (size_t)j * ds;
                for (int p = 0; p < ds / 2; p++) {
                    const int n = sg2_contraction_steps(dt0, -0.5f * -sg_exp(alog[2 * p]), -0.5f * -sg_exp(alog[2 * p + 1]));
                    if (n == 0) any_zero = 1;
                    if (n > largest) largest = n;
                }
            }
        }
        first_block = sg2_first_block_steps(largest, any_zero);
    }

    std::vector<R> ctx_sorted[2];
    std::vector<R> hst[2];
    for (int dir = 0; dir < 2; dir++) {
        const int b = dir ? W_B_INPROJ : W_F_INPROJ;
        DirW<O> w = {W[b], W[b + 1], W[b + 2], W[b + 3], W[b + 4], W[b + 5], W[b + 6], W[b + 7], W[b + 8], {}, 0, {}, {0.0f, 0.0f}, {}, {0.0f, 0.0f}, {}, {0.0f, 0.0f}};
        if (sizeof(R) == 4) {
            w.comp_rows = std::max(di, ds);
            w.comp.assign((size_t)SG2_COMP_GROUPS * w.comp_rows * 3, 0.0f);
            for (int grp = 0; grp < SG2_COMP_GROUPS; grp++)
                for (int row = 0; row < ((grp == SG2_COMP_B || grp == SG2_COMP_C) ? ds : di); row++)
                    sg2_compose_one(grp, row, dm, di, W[W_IN_W], W[W_IN_B], W[b], W[b + 1], W[b + 2], W[b + 3], W[b + 4],
                                    &w.comp[((size_t)grp * w.comp_rows + row) * 3]);
            w.tay.assign((size_t)2 * w.comp_rows * 4, 0.0f);
            for (int j = 0; j < di; j++) {
                const float* cd = &w.comp[((size_t)SG2_COMP_DT * w.comp_rows + j) * 3];
                const float* cz = &w.comp[((size_t)SG2_COMP_Z * w.comp_rows + j) * 3];
                sg2_softplus_taylor(cd[2], &w.tay[((size_t)0 * w.comp_rows + j) * 4]);
                sg2_silu_taylor(cz[2], &w.tay[((size_t)1 * w.comp_rows + j) * 4]);
                w.cmax[0] = sg_max(w.cmax[0], sg_max(sg_abs(cd[0]), sg_abs(cz[0])));
                w.cmax[1] = sg_max(w.cmax[1], sg_max(sg_abs(cd[1]), sg_abs(cz[1])));
            }
            /* lane polynomials and the limit of their use */
            const int hp = ds / 2;
            float amax = 0.0f, fmax = 0.0f, cdt[2] = {0.0f, 0.0f}, slope = 0.0f;
            w.lane_poly.assign((size_t)di * hp * 14, 0.0f);
            w.lane_prod.assign((size_t)di * hp * 12, 0.0f);
            for (int j = 0; j < di; j++) {
                const float* cd = &w.comp[((size_t)SG2_COMP_DT * w.comp_rows + j) * 3];
                cdt[0] = sg_max(cdt[0], sg_abs(cd[0]));
                cdt[1] = sg_max(cdt[1], sg_abs(cd[1]));
                slope = sg_max(slope, sg2_dt_slope(cd[2]));
                const float dt0 = w.tay[((size_t)0 * w.comp_rows + j) * 4];
                for (int p = 0; p < hp; p++) {
                    const float a_e = -0.5f * -sg_exp(w.A_log[j * ds + 2 * p]), a_o = -0.5f * -sg_exp(w.A_log[j * ds + 2 * p + 1]);
                    const float f = w.rope[j * hp + p];
                    amax = sg_max(amax, sg_max(a_e, a_o));
                    fmax = sg_max(fmax, sg_abs(f));
                    float* lp = &w.lane_poly[((size_t)j * hp + p) * 14];
                    sg2_abar_poly(dt0, a_e, lp);
                    sg2_abar_poly(dt0, a_o, lp + 4);
                    sg2_sincos_poly(dt0, f, lp + 8, lp + 11);
                    sg2_pair_products(dt0, a_e, a_o, f, &w.lane_prod[((size_t)j * hp + p) * 12]);
                }
            }
            const float kp = sg2_limit_factor(sg_max(128.0f * amax, 256.0f * fmax), slope);
            w.kpoly[0] = kp * cdt[0];
            w.kpoly[1] = kp * cdt[1];
            const float kq = sg2_limit_factor(sg_fma(416.0f, amax, 184.0f * fmax), slope);
            w.kprod[0] = kq * cdt[0];
            w.kprod[1] = kq * cdt[1];
        }
        float* st = dir ? mbwd_io : mfwd_io;
        hst[dir].assign(st, st + di * ds);
        ctx_sorted[dir].resize((size_t)N * dm);
        scan_dir<O>(d, w, x.data(), gs_sorted.data(), N, dir == 1, chunk_len, window, first_block, hst[dir].data(), ctx_sorted[dir].data());
        for (int i = 0; i < di * ds; i++) st[i] = (float)hst[dir][i];
    }
    /* unsort: element perm[t] takes the context computed at sorted position t */
    std::vector<R> cf((size_t)N * dm), cb((size_t)N * dm);
    for (int64_t t = 0; t < N; t++)
        for (int k = 0; k < dm; k++) {
            cf[(size_t)perm[t] * dm + k] = ctx_sorted[0][t * dm + k];
            cb[(size_t)perm[t] * dm + k] = ctx_sorted[1][t * dm + k];
        }
    if (ctx_out)
        for (int64_t i = 0; i < N * dm; i++) {
            ctx_out[i] = (float)cf[i];
            ctx_out[(size_t)N * dm + i] = (float)cb[i];
        }

    const R alpha = sc[S_ALPHA], lamb = sc[S_LAMB], beta1 = sc[S_BETA1], beta2 = sc[S_BETA2];
    const R rescale = sc[S_RESCALE], eps = sc[S_EPS];
    R step_size, decay, bc2;
    if (sizeof(R) == 4) {     /* fp32 host scalars exactly as the device entry point derives them */
        step_size = sc[S_LR] / sc[S_BC1];
        decay = 1.0f - sc[S_LR] * sc[S_WD];
        bc2 = sc[S_BC2];
    } else {
        step_size = (R)sc[S_LR] / (R)sc[S_BC1];
        decay = 1.0 - (R)sc[S_LR] * (R)sc[S_WD];
        bc2 = sc[S_BC2];
    }
    const int grl = 2 + 2 * dm + gh, pin = gh + 2 * dm + 2;
    const float *Wz = W[W_GRU_WZ], *bz = W[W_GRU_BZ], *Wr = W[W_GRU_WR], *br = W[W_GRU_BR];
    const float *Wh = W[W_GRU_WH], *bh = W[W_GRU_BH];

    for (int64_t i = 0; i < N; i++) {
        const R gv = g[i], sv = s[i];
        const R* f = &cf[(size_t)i * dm];
        const R* b = &cb[(size_t)i * dm];
        R hold[8], zg[8], rg[8], hnew[8], pre_g[16], gate[16], pre_c[8], cand[8];
        for (int k = 0; k < gh; k++) hold[k] = gru_io[i * gh + k];
        /* GRU gates: chain = bias, g, s, fwd ctx, bwd ctx, h */
        for (int j = 0; j < gh; j++) {
            const float *wz = Wz + j * grl, *wr = Wr + j * grl;
            R vz = bz[j], vr = br[j];
            vz = O::fma((R)wz[0], gv, vz); vz = O::fma((R)wz[1], sv, vz);
            vr = O::fma((R)wr[0], gv, vr); vr = O::fma((R)wr[1], sv, vr);
            for (int k = 0; k < dm; k++) { vz = O::fma((R)wz[2 + k], f[k], vz); vr = O::fma((R)wr[2 + k], f[k], vr); }
            for (int k = 0; k < dm; k++) { vz = O::fma((R)wz[2 + dm + k], b[k], vz); vr = O::fma((R)wr[2 + dm + k], b[k], vr); }
            for (int k = 0; k < gh; k++) { vz = O::fma((R)wz[2 + 2 * dm + k], hold[k], vz); vr = O::fma((R)wr[2 + 2 * dm + k], hold[k], vr); }
            pre_g[j] = vz;
            pre_g[gh + j] = vr;
        }
        O::sigmoid_group(2 * gh, pre_g, gate);
        for (int j = 0; j < gh; j++) { zg[j] = gate[j]; rg[j] = gate[gh + j]; }
        for (int j = 0; j < gh; j++) {
            const float* wh = Wh + j * grl;
            R v = bh[j];
            v = O::fma((R)wh[0], gv, v); v = O::fma((R)wh[1], sv, v);
            for (int k = 0; k < dm; k++) v = O::fma((R)wh[2 + k], f[k], v);
            for (int k = 0; k < dm; k++) v = O::fma((R)wh[2 + dm + k], b[k], v);
            for (int k = 0; k < gh; k++) v = O::fma((R)wh[2 + 2 * dm + k], rg[k] * hold[k], v);
            pre_c[j] = v;
        }
        O::tanh_group(gh, pre_c, cand);
        for (int j = 0; j < gh; j++) hnew[j] = O::fma(zg[j], cand[j], ((R)1 - zg[j]) * hold[j]);
        for (int k = 0; k < gh; k++) gru_io[i * gh + k] = (float)hnew[k];

        /* PEER: per head query -> two sub-key argmaxes -> expert MLP */
        R total = 0;
        for (int hh = 0; hh < H; hh++) {
            const float* q = W[W_PEER_Q] + (size_t)hh * dm * pin;
            R query[16];
            for (int dd = 0; dd < dm; dd++) {
                const float* qr = q + dd * pin;
                R v = 0;
                for (int k = 0; k < gh; k++) v = O::fma((R)qr[k], hnew[k], v);
                for (int k = 0; k < dm; k++) v = O::fma((R)qr[gh + k], f[k], v);
                for (int k = 0; k < dm; k++) v = O::fma((R)qr[gh + dm + k], b[k], v);
                v = O::fma((R)qr[gh + 2 * dm], gv, v);
                v = O::fma((R)qr[gh + 2 * dm + 1], sv, v);
                query[dd] = v;
            }
            int best[2];
            for (int half = 0; half < 2; half++) {
                const float* keys = W[half ? W_KEYS_B : W_KEYS_A] + (size_t)hh * pk * hd;
                int bi = 0;
                R bs = (R)-1e30f, second = (R)-1e30f;
                for (int k = 0; k < pk; k++) {
                    R dot = 0;
                    for (int dd = 0; dd < hd; dd++) dot = O::fma(query[half * hd + dd], (R)keys[k * hd + dd], dot);
                    if (dot > bs) { second = bs; bs = dot; bi = k; }
                    else if (dot > second) second = dot;
                }
                best[half] = bi;
                if (margin_out) margin_out[((size_t)i * H + hh) * 2 + half] = (float)(bs - second);
            }
            int e = best[0] * pk + best[1];
            if (e >= E) e = E - 1;
            if (expert_counts) expert_counts[e] += 1;
            if (eidx_out) eidx_out[(size_t)i * H + hh] = e;
            R ho = W[W_EXP_B2][e];
            for (int k = 0; k < eh; k++) {
                R zv = O::fma((R)W[W_EXP_W1][e * eh + k], gv, (R)W[W_EXP_B1][e * eh + k]);
                zv = zv > 0 ? zv : (R)0;
                ho = O::fma((R)W[W_EXP_W2][e * eh + k], zv, ho);
            }
            total = total + ho;
        }
        const R smart = gv + (rescale * total) / (R)H;
        if (smart_out) smart_out[i] = (float)smart;

        R mu = mu_io[i];
        mu = O::fma(alpha, mu, ((R)1 - alpha) * gv);
        mu_io[i] = (float)mu;
        const R fg = O::fma(lamb, mu, smart);
        R ea = ea_io[i], easq = easq_io[i];
        ea = O::fma(beta1, ea, ((R)1 - beta1) * fg);
        easq = O::fma(beta2, easq, (((R)1 - beta2) * fg) * fg);
        ea_io[i] = (float)ea;
        easq_io[i] = (float)easq;
        const R denom = O::sqrt(easq / bc2) + eps;
        R p = load_as_f(param, dtype, i);
        p = O::fma(p, decay, -((step_size * ea) / denom));
        store_from_f(param, dtype, i, (float)p);
    }
    return 0;
}

}  // namespace

extern "C" {

/* stable ascending argsort of |g| with non-finite entries treated as 0 */
void orc_sort_perm(const float* g, int64_t N, int32_t* perm) { sort_perm(g, N, perm); }

/* One tensor, one optimizer step.  precision: 32 or 64.  dims[8] and
 * scalars[10] in the enum orders above; W = 33 weight pointers.  Optional
 * outputs may be NULL: perm [N], expert_idx [N][H], ctx [2][N][d_model]
 * (forward then backward context in original element order), margin
 * [N][H][2] (top-1 minus top-2 score per sub-key), smart [N]. */
int orc_sg2_step(int precision, int64_t chunk_len, int64_t window, const float* const* W, const int32_t* dims,
                 int dtype, void* param, const void* grad, const void* sharp, float* ea, float* easq,
                 float* mu, float* gru, float* mfwd, float* mbwd, int64_t N, const float* scalars,
                 int32_t* expert_counts, int32_t* perm, int32_t* expert_idx, float* ctx, float* margin,
                 float* smart) {
    Dims d = {dims[0], dims[1], dims[2], dims[3], dims[4], dims[5], dims[6], dims[7]};
    if (precision == 32)
        return step_tensor<F32>(d, W, chunk_len, window, dtype, param, grad, sharp, ea, easq, mu, gru, mfwd, mbwd,
                                N, scalars, expert_counts, perm, expert_idx, ctx, margin, smart);
    return step_tensor<F64>(d, W, chunk_len, window, dtype, param, grad, sharp, ea, easq, mu, gru, mfwd, mbwd, N,
                            scalars, expert_counts, perm, expert_idx, ctx, margin, smart);
}

/* primitives exported one by one so tests can pin them against libm */
float orc_exp(float x) { return sg_exp(x); }
float orc_log(float x) { return sg_log(x); }
float orc_softplus(float x) { return sg_softplus(x); }
float orc_sin_tiny(float x) { float s, c; sg_sincos_tiny(x, &s, &c); return s; }
float orc_cos_tiny(float x) { float s, c; sg_sincos_tiny(x, &s, &c); return c; }
float orc_sigmoid(float x) { return sg_sigmoid(x); }
float orc_silu(float x) { return sg_silu(x); }
void orc_silu_block(int n, const float* z, float* out) { sg_silu_block(n, z, out); }
void orc_sigmoid_block(int n, const float* x, float* out) { sg_sigmoid_block(n, x, out); }
void orc_tanh_block(int n, const float* x, float* out) { sg_tanh_block(n, x, out); }
float orc_softplus_taylor(float c, float d) { float t[4]; sg2_softplus_taylor(c, t); return sg2_taylor_eval(t, d); }
float orc_silu_taylor(float c, float d) { float t[4]; sg2_silu_taylor(c, t); return sg2_taylor_eval(t, d); }
float orc_abar_poly(float dt0, float nhA, float d) { float p[4]; sg2_abar_poly(dt0, nhA, p); return sg2_poly3(p, d); }
float orc_sincos_poly(float dt0, float f, float d, int cosine) { float qs[3], qc[3]; sg2_sincos_poly(dt0, f, qs, qc); return sg2_poly2(cosine ? qc : qs, d); }
float orc_pair_product(float dt0, float nhA_e, float nhA_o, float f, float d, int which) {
    float k[12];
    sg2_pair_products(dt0, nhA_e, nhA_o, f, k);
    return sg2_poly2(k + 3 * which, d);
}
int orc_contraction_steps(float dt0, float nhA_e, float nhA_o) { return sg2_contraction_steps(dt0, nhA_e, nhA_o); }
float orc_tanh(float x) { return sg_tanh(x); }
float orc_sin(float x) { float s, c; sg_sincos(x, &s, &c); return s; }
float orc_cos(float x) { float s, c; sg_sincos(x, &s, &c); return c; }
float orc_rcp_pos(float x) { return sg_rcp_pos(x); }
float orc_sin_small(float x) { float s, c; sg_sincos_small(x, &s, &c); return s; }
float orc_cos_small(float x) { float s, c; sg_sincos_small(x, &s, &c); return c; }
float orc_abar(float dt, float A) { float e, o; sg_abar_pair(dt, -0.5f * A, -0.5f * A, &e, &o); return e; }
uint16_t orc_f_to_f16(float f) { return f_to_f16(f); }
float orc_f16_to_f(uint16_t h) { return f16_to_f(h); }
uint16_t orc_f_to_bf16(float f) { return f_to_bf16(f); }
float orc_bf16_to_f(uint16_t h) { return bf16_to_f(h); }

}  // extern "C"
