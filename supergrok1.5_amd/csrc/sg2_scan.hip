// Bidirectional Mamba-3 selective scan over the magnitude-sorted sequence of
// every parameter tensor, all tensors and both directions in each launch.
//
// Replaces the reference's precompute + Blelloch scan kernels
// (csrc/supergrok2_mamba_peer_kernels.cu:289-346, 577-781), the sequential
// kernels (:138-272, :1241-1390), the x_sorted gather (:1882-1906) and the
// scan-output unsort + out_proj (:2057-2060, :917-937).
//
// The sorted sequence of a tensor is cut into chunks of chunk_len timesteps
// (scan order: t ascending for the forward direction, descending for the
// backward one).  One workgroup of d_inner * d_state/2 lanes (128 for the default
// geometry, 512 for the large one) owns one chunk; lane (j,p) owns column j and
// RoPE pair p, i.e. the two states h[j][2p], h[j][2p+1].
//   k_scan<false>  every chunk but the last of a tensor: 2x2 affine summary
//                  (M,b) of the chunk, accumulated from the identity.  The
//                  recurrence contracts (|A_bar| < 1), so the chunk is walked
//                  backwards in blocks of `window` steps and the walk stops as
//                  soon as every |entry| of the running M, in all lanes, is
//                  below 2^-100: the state entering that block is multiplied
//                  by less than 2^-100, and the summary is (0, b).  A first
//                  attempt covers one block sized from the weights with the
//                  state part only and a norm bound instead of M.
//   k_chunk_prefix start state of each chunk: summaries applied in order to
//                  the carried state of the tensor.
//   k_scan<true>   every chunk replayed from its start state: y = h.C, gate,
//                  D skip, out_proj, and the 8-float context written straight
//                  to the element's original position (the "unsort").  The
//                  last chunk stores the new carried state.
//   k_compose      runs first: the input of a timestep is two numbers (g, s)
//                  and every projection of the block is linear in their 8-float
//                  input projection, so input_proj, in_proj, dt_proj, B_proj and
//                  C_proj are folded into 5 x d_inner coefficient triples per
//                  direction (include/sg2_compose.h).
// Per-timestep projections (x-branch, z, dt, B, C) are evaluated from those
// triples in both passes for tiles of 64 timesteps and staged through LDS
// instead of being materialised in HBM (the reference writes 320 B per
// element per direction).
// The inputs of a timestep come coalesced from the sort's own output: the key
// is |g|, the payload carries the sign of g and the element index, and the
// sharpness has been gathered into sorted order once.
//
// The kernels are bound by fp32 VALU issue, not by HBM: per (timestep, column,
// pair) one shared reciprocal, one sin/cos pair and the 2x2 update.  The
// recurrence loop therefore works on blocks of 8 timesteps: all LDS operands of
// the block are fetched first, the state-independent coefficients of the 8
// steps are computed as independent instruction streams, and only the short
// h-update chain is serial.  The A_bar denominators of a lane's 8 steps are
// inverted together (one division per block, sg_abar_block_*).  When every
// lane of the wave holds a small rotation angle the sin/cos range reduction is
// skipped (bit-identical results, see sg_sincos_small); when every angle of
// the block is below 0.3 a shorter polynomial pair is used (sg_sincos_tiny,
// not bit-identical to the general form: the choice depends on the angles only
// and the CPU checker makes the same one).
// Where the inputs are small (the usual case: sg2_taylor_ok, sg2_poly_ok in sg2_compose.h) the step size and the gate
// of a tile come from cubic Taylor polynomials around their zero-input arguments, and A_bar, sin and cos of a block
// from per-lane polynomials in dt - dt0; the forms above serve the remaining tiles and blocks.
// For the bilevel pass k_scan<true, true> also stores the state entering every
// 32nd step (Plan::htile), which the adjoint kernels restart from.
#include <type_traits>
#include "sg2_internal.hpp"
#include "../../include/sg2_compose.h"

namespace sg2 {
namespace {

constexpr int LDS_STRIDE = SCAN_TT + 4;   // [row][timestep] rows: 16-byte aligned (the recurrence fetches 4 timesteps per LDS read)
                                          // and padded so the 8 rows a wave reads start 4 banks apart
typedef float f32x4 __attribute__((ext_vector_type(4)));
#ifndef SG2_SCAN_UB
#define SG2_SCAN_UB 8
#endif
constexpr int UB = SG2_SCAN_UB;           // timesteps per unrolled block of the recurrence
static_assert(UB % 4 == 0 && SCAN_TT % UB == 0 && SCAN_TT == 64, "blocks are fetched 4 timesteps per LDS read; one ballot covers a tile");
static_assert(HT_STEP % UB == 0 && SCAN_TT % HT_STEP == 0 && SCAN_TT / HT_STEP <= 2, "kept states fall on block borders: tile start and at most one more");
// Three waves per SIMD (168 VGPRs) is where the default geometry's kernels stop gaining from occupancy; keep the
// register allocation from drifting just past that boundary.  The large geometry's workgroup is two waves per SIMD by itself,
// and at 128 VGPRs (two workgroups per CU) the recurrence spills: one workgroup per CU, up to 256 VGPRs.
#ifndef SG2_SCAN_WAVES
#define SG2_SCAN_WAVES 3
#endif
template <class G>
constexpr int scan_waves() { return G::PARTS == 2 ? SG2_SCAN_WAVES : 2; }
#define SG2_SCAN_ATTR __attribute__((amdgpu_waves_per_eu(scan_waves<G>(), scan_waves<G>())))

__device__ __forceinline__ float dpp_quad_swap1(float v) {   // lane ^ 1
    return sg_i2f(__builtin_amdgcn_update_dpp(0, sg_f2i(v), 0xB1, 0xF, 0xF, true));
}
__device__ __forceinline__ float dpp_quad_swap2(float v) {   // lane ^ 2
    return sg_i2f(__builtin_amdgcn_update_dpp(0, sg_f2i(v), 0x4E, 0xF, 0xF, true));
}
__device__ __forceinline__ float dpp_half_mirror(float v) {  // lane -> 7 - lane within each group of 8
    return sg_i2f(__builtin_amdgcn_update_dpp(0, sg_f2i(v), 0x141, 0xF, 0xF, true));
}
__device__ __forceinline__ float dpp_row_mirror(float v) {   // lane -> 15 - lane within each group of 16
    return sg_i2f(__builtin_amdgcn_update_dpp(0, sg_f2i(v), 0x140, 0xF, 0xF, true));
}
// sum over the HP lanes of a (column) group.  The tree folds the group in halves, mirrored, until four sums are left:
// HP = 8: s_i = y_i + y_(7-i), total = (s_0 + s_1) + (s_2 + s_3); HP = 16: r_i = y_i + y_(15-i) first, then the same on r.
// (Mirrored folds first, because a fold across DPP banks can be written to some banks only: see block_pair_sums.)
template <int HP>
__device__ __forceinline__ float pair_tree_sum(float y) {
    if (HP == 16) y = y + dpp_row_mirror(y);
    y = y + dpp_half_mirror(y);
    y = y + dpp_quad_swap1(y);
    y = y + dpp_quad_swap2(y);
    return y;
}
// The same sums for the 8 steps of a block in 16 instructions instead of 24 (32 for HP = 16).  A DPP instruction can
// be restricted to some banks (groups of four lanes) of every row of 16, leaving the destination's other lanes as
// they were.  After a mirrored fold both halves of the folded group hold the same sums, so two steps' folds are
// written into ONE register - step u into the first half's lanes, step u + 4 into the second half's - and the rest
// of the tree runs on half as many registers.  Additions commute bit for bit, so every lane that ends up holding a
// step's total holds pair_tree_sum's value.  On return, for HP = 8, y[k] (k < 4) is the total of step k + 4 (p >> 2)
// in lane (j, p); for HP = 16, y[m] (m < 2) that of step m + 2 (p >> 2).
// (Inline assembly: the compiler has no form for a bank-masked DPP addition that keeps the other lanes, and it does
// not see a hazard between instructions inside the block - a DPP operand must not be read within two instructions of the
// vector instruction that wrote it, hence the order of the instructions and the s_nop.)
template <int HP>
__device__ __forceinline__ void block_pair_sums(float (&y)[8]) {
    float z0, z1, z2, z3;
    if (HP == 8) {
        asm volatile(
            "s_nop 1\n\t"
            "v_add_f32_dpp %0, %4, %4 row_half_mirror row_mask:0xf bank_mask:0x5\n\t"
            "v_add_f32_dpp %0, %8, %8 row_half_mirror row_mask:0xf bank_mask:0xa\n\t"
            "v_add_f32_dpp %1, %5, %5 row_half_mirror row_mask:0xf bank_mask:0x5\n\t"
            "v_add_f32_dpp %1, %9, %9 row_half_mirror row_mask:0xf bank_mask:0xa\n\t"
            "v_add_f32_dpp %2, %6, %6 row_half_mirror row_mask:0xf bank_mask:0x5\n\t"
            "v_add_f32_dpp %2, %10, %10 row_half_mirror row_mask:0xf bank_mask:0xa\n\t"
            "v_add_f32_dpp %3, %7, %7 row_half_mirror row_mask:0xf bank_mask:0x5\n\t"
            "v_add_f32_dpp %3, %11, %11 row_half_mirror row_mask:0xf bank_mask:0xa\n\t"
            "v_add_f32_dpp %0, %0, %0 quad_perm:[1,0,3,2] row_mask:0xf bank_mask:0xf\n\t"
            "v_add_f32_dpp %1, %1, %1 quad_perm:[1,0,3,2] row_mask:0xf bank_mask:0xf\n\t"
            "v_add_f32_dpp %2, %2, %2 quad_perm:[1,0,3,2] row_mask:0xf bank_mask:0xf\n\t"
            "v_add_f32_dpp %3, %3, %3 quad_perm:[1,0,3,2] row_mask:0xf bank_mask:0xf\n\t"
            "v_add_f32_dpp %0, %0, %0 quad_perm:[2,3,0,1] row_mask:0xf bank_mask:0xf\n\t"
            "v_add_f32_dpp %1, %1, %1 quad_perm:[2,3,0,1] row_mask:0xf bank_mask:0xf\n\t"
            "v_add_f32_dpp %2, %2, %2 quad_perm:[2,3,0,1] row_mask:0xf bank_mask:0xf\n\t"
            "v_add_f32_dpp %3, %3, %3 quad_perm:[2,3,0,1] row_mask:0xf bank_mask:0xf\n\t"
            "s_nop 1"
            : "=&v"(z0), "=&v"(z1), "=&v"(z2), "=&v"(z3)
            : "v"(y[0]), "v"(y[1]), "v"(y[2]), "v"(y[3]), "v"(y[4]), "v"(y[5]), "v"(y[6]), "v"(y[7]));
        y[0] = z0; y[1] = z1; y[2] = z2; y[3] = z3;
    } else {
        asm volatile(
            "s_nop 1\n\t"
            "v_add_f32_dpp %0, %4, %4 row_mirror row_mask:0xf bank_mask:0x3\n\t"
            "v_add_f32_dpp %0, %8, %8 row_mirror row_mask:0xf bank_mask:0xc\n\t"
            "v_add_f32_dpp %1, %5, %5 row_mirror row_mask:0xf bank_mask:0x3\n\t"
            "v_add_f32_dpp %1, %9, %9 row_mirror row_mask:0xf bank_mask:0xc\n\t"
            "v_add_f32_dpp %2, %6, %6 row_mirror row_mask:0xf bank_mask:0x3\n\t"
            "v_add_f32_dpp %2, %10, %10 row_mirror row_mask:0xf bank_mask:0xc\n\t"
            "v_add_f32_dpp %3, %7, %7 row_mirror row_mask:0xf bank_mask:0x3\n\t"
            "v_add_f32_dpp %3, %11, %11 row_mirror row_mask:0xf bank_mask:0xc\n\t"
            "v_add_f32_dpp %0, %0, %0 row_half_mirror row_mask:0xf bank_mask:0x5\n\t"
            "v_add_f32_dpp %1, %1, %1 row_half_mirror row_mask:0xf bank_mask:0x5\n\t"
            "s_nop 0\n\t"
            "v_add_f32_dpp %0, %2, %2 row_half_mirror row_mask:0xf bank_mask:0xa\n\t"
            "v_add_f32_dpp %1, %3, %3 row_half_mirror row_mask:0xf bank_mask:0xa\n\t"
            "s_nop 1\n\t"
            "v_add_f32_dpp %0, %0, %0 quad_perm:[1,0,3,2] row_mask:0xf bank_mask:0xf\n\t"
            "v_add_f32_dpp %1, %1, %1 quad_perm:[1,0,3,2] row_mask:0xf bank_mask:0xf\n\t"
            "s_nop 1\n\t"
            "v_add_f32_dpp %0, %0, %0 quad_perm:[2,3,0,1] row_mask:0xf bank_mask:0xf\n\t"
            "v_add_f32_dpp %1, %1, %1 quad_perm:[2,3,0,1] row_mask:0xf bank_mask:0xf\n\t"
            "s_nop 1"
            : "=&v"(z0), "=&v"(z1), "=&v"(z2), "=&v"(z3)
            : "v"(y[0]), "v"(y[1]), "v"(y[2]), "v"(y[3]), "v"(y[4]), "v"(y[5]), "v"(y[6]), "v"(y[7]));
        y[0] = z0; y[1] = z1;
    }
}
template <int HP>
__device__ __forceinline__ float pair_tree_max(float f) {
    f = sg_max(f, dpp_quad_swap1(f));
    f = sg_max(f, dpp_quad_swap2(f));
    f = sg_max(f, dpp_half_mirror(f));
    if (HP == 16) f = sg_max(f, dpp_row_mirror(f));
    return f;
}

// Composed coefficient triples (see sg2_compose.h), one thread per (direction, group, row).
template <class G>
__global__ __launch_bounds__(2 * SG2_COMP_GROUPS * G::ROWS) void k_compose(Plan pl) {
    const int dir = threadIdx.x / (SG2_COMP_GROUPS * G::ROWS), r = threadIdx.x % (SG2_COMP_GROUPS * G::ROWS);
    const int group = r / G::ROWS, row = r % G::ROWS;
    const int b = dir ? W_B_INPROJ : W_F_INPROJ;
    float out[3];
    sg2_compose_one(group, row, G::DM, G::DI, pl.W.w[W_IN_W], pl.W.w[W_IN_B], pl.W.w[b], pl.W.w[b + 1], pl.W.w[b + 2], pl.W.w[b + 3],
                    pl.W.w[b + 4], out);
    float* dst = pl.comp + (size_t)threadIdx.x * 3;
    dst[0] = out[0];
    dst[1] = out[1];
    dst[2] = out[2];
    // How many steps the first block of a chunk summary should cover: what the slowest pair of either direction needs
    // to contract below 2^-100 at the step size a zero input gives (sg2_contraction_steps), plus a margin.
    __shared__ int s_largest, s_zero, s_bad, s_cmax[2][2], s_cdt[2][2], s_amax[2], s_fmax[2], s_slope[2];
    if (threadIdx.x == 0) {
        s_largest = 0; s_zero = 0; s_bad = 0;
        for (int k = 0; k < 2; k++) { s_cmax[k][0] = s_cmax[k][1] = s_cdt[k][0] = s_cdt[k][1] = s_amax[k] = s_fmax[k] = s_slope[k] = 0; }
    }
    __syncthreads();
    // Taylor polynomials of the step size and of the gate around their zero-input arguments (sg2_compose.h), and the
    // largest |c_g|, |c_s| of those rows (bit patterns of non-negative floats order like integers)
    if (group == SG2_COMP_DT || group == SG2_COMP_Z) {
        float t[4];
        if (group == SG2_COMP_DT) sg2_softplus_taylor(out[2], t);
        else sg2_silu_taylor(out[2], t);
        float* tay = pl.comp + 2 * SG2_COMP_GROUPS * G::ROWS * 3 + ((dir * 2 + (group == SG2_COMP_Z ? 1 : 0)) * G::ROWS + row) * 4;
        tay[0] = t[0]; tay[1] = t[1]; tay[2] = t[2]; tay[3] = t[3];
        atomicMax(&s_cmax[dir][0], sg_f2i(sg_abs(out[0])));
        atomicMax(&s_cmax[dir][1], sg_f2i(sg_abs(out[1])));
        if (group == SG2_COMP_DT) {
            atomicMax(&s_cdt[dir][0], sg_f2i(sg_abs(out[0])));
            atomicMax(&s_cdt[dir][1], sg_f2i(sg_abs(out[1])));
            atomicMax(&s_slope[dir], sg_f2i(sg2_dt_slope(out[2])));       // positive: its bit pattern orders like the value
        }
    }
    if (group == SG2_COMP_DT) {
        const float dt0 = sg_softplus(out[2]);
        const float* alog = pl.W.w[dir ? W_B_ALOG : W_F_ALOG] + row * G::DS;
        for (int p = 0; p < G::HP; p++) {
            const float a_e = -0.5f * -sg_exp(alog[2 * p]), a_o = -0.5f * -sg_exp(alog[2 * p + 1]);
            const int n = sg2_contraction_steps(dt0, a_e, a_o);
            if (n == 0) atomicOr(&s_zero, 1);
            atomicMax(&s_largest, n);
            // for sg2_poly_ok: the largest -A/2 and the largest |rotation frequency| of the direction
            atomicMax(&s_amax[dir], sg_f2i(sg_max(a_e, a_o)));
            atomicMax(&s_fmax[dir], sg_f2i(sg_abs(pl.W.w[dir ? W_B_ROPE : W_F_ROPE][row * G::HP + p])));
        }
    }
    for (int i = threadIdx.x; i < pl.P; i += blockDim.x)
        if (pl.state_bad[i] != 0) s_bad = 1;       // plain store: every writer stores the same value
    __syncthreads();
    if (threadIdx.x == 0) {
        pl.contracted[0] = s_bad == 0 ? 1 : 0;      // until a summary kernel finds a chunk that has not contracted; never while a carried state is not finite
        pl.contracted[2] = s_bad;
        pl.contracted[1] = sg2_first_block_steps(s_largest, s_zero);
        float* cmax = pl.comp + 2 * SG2_COMP_GROUPS * G::ROWS * 3 + 2 * 2 * G::ROWS * 4;
        cmax[0] = sg_i2f(s_cmax[0][0]); cmax[1] = sg_i2f(s_cmax[0][1]);
        cmax[2] = sg_i2f(s_cmax[1][0]); cmax[3] = sg_i2f(s_cmax[1][1]);
        for (int k = 0; k < 2; k++) {
            const float slope = sg_i2f(s_slope[k]);      // how much of a change of its argument the step size follows at most
            const float kp = sg2_limit_factor(sg_max(128.0f * sg_i2f(s_amax[k]), 256.0f * sg_i2f(s_fmax[k])), slope);
            cmax[4 + 2 * k] = kp * sg_i2f(s_cdt[k][0]);
            cmax[5 + 2 * k] = kp * sg_i2f(s_cdt[k][1]);
            // ... and for the products of the output pass (sg2_pair_products)
            const float kq = sg2_limit_factor(sg_fma(416.0f, sg_i2f(s_amax[k]), 184.0f * sg_i2f(s_fmax[k])), slope);
            cmax[8 + 2 * k] = kq * sg_i2f(s_cdt[k][0]);
            cmax[9 + 2 * k] = kq * sg_i2f(s_cdt[k][1]);
        }
    }
}

// Projections of one timestep from the element's (g, s).  Each wave of the workgroup produces its
// share (rows PART*n/PARTS ...) of dt / dt*x-branch / B (/ D*x-branch / C / gate).  PART is a template parameter so that every row
// index is a compile-time constant; a caller with many waves passes PART = 0 and array pointers moved to its wave's first row.  The coefficient triple of an output row sits in the four padding floats of the
// LDS row it produces (staged once per workgroup, see stage_coefficients): one 16-byte broadcast read per output,
// no scalar loads in the loop (a scalar load can only be waited for with lgkmcnt(0), which also drains the LDS queue).
// Returns bit 0: every rotation angle of this timestep, over this half's columns, is small enough for
// sg_sincos_small; bit 1: small enough for sg_sincos_tiny (fmax: per column, the largest |rope frequency| of its 8 pairs; dt >= 0 and
// rounding is monotone, so dt*fmax < limit is the same statement as |dt*freq| < limit for all pairs).
// TAYLOR: every timestep of the tile has passed sg2_taylor_ok: step size and gate come from their cubic Taylor
// polynomials.  Those cost no LDS of their own in the output pass (the workgroup's LDS is what limits it to six per CU):
// the step-size polynomial of column j sits in the padding of row j of s_dx, and the gate polynomial of column j
// is spread over the fourth padding floats of rows j of s_dt, s_B, s_C and s_gate, which this wave reads anyway
// (d_inner = d_state: the wave's columns and its rows of B and C carry the same indices).  The summary pass has
// no s_dx and keeps the step-size polynomials in s_tay.
// DSTORE (with TAYLOR, whole tiles whose blocks all run on the lane polynomials): the step-size row receives dt - dt0,
// which is all those blocks want to know (one subtraction per column here instead of one per pair in the recurrence),
// and nobody asks for the angle flags.
template <class G, bool OUT, int PART, bool HAS_S, bool TAYLOR, bool DSTORE = false>
__device__ __forceinline__ int project_tile(float g, float s, int tu, float* s_dt, float* s_ux, float* s_dx, float* s_B,
                                             float* s_C, float* s_gate, const float* s_fmax, const float* s_tay) {
    static_assert(G::DI == G::DS, "the gate polynomials ride on the rows of B and C");
    auto delta = [&](const f32x4 t) { return HAS_S ? sg_fma(t[0], g, t[1] * s) : t[0] * g; };
    auto poly = [&](const f32x4 t, float d) { return sg_fma(sg_fma(sg_fma(t[3], d, t[2]), d, t[1]), d, t[0]); };
    // HAS_S is false for a tensor whose sharpness is all zero: fma(c_s, 0, c_0) is c_0 itself, so the term is skipped
    auto eval = [&](const f32x4 t) { return sg_fma(t[0], g, HAS_S ? sg_fma(t[1], s, t[2]) : t[2]); };
    auto coef = [&](const float* arr, int row) { return *reinterpret_cast<const f32x4*>(arr + row * LDS_STRIDE + SCAN_TT); };
    constexpr int NR = G::DI / G::PARTS;        // this wave's columns = its rows of B and C
    float gp0[NR], gp1[NR], gp2[NR];            // first three coefficients of the gate polynomials, picked up on the way
    bool small = true, tiny = true;
#pragma unroll
    for (int q = 0; q < NR; q++) {
        const int jj = PART * NR + q;
        const f32x4 cd = coef(s_dt, jj);
        gp0[q] = cd[3];
        float dtv, dt0 = 0.0f;
        if (TAYLOR) {
            const f32x4 tp = OUT ? coef(s_dx, jj) : *reinterpret_cast<const f32x4*>(s_tay + jj * 4);
            dtv = poly(tp, delta(cd));
            dt0 = tp[0];
        } else {
            dtv = sg_softplus(eval(cd));
        }
        if (!DSTORE) {
            const float amax = dtv * s_fmax[jj];
            small = small && (amax < SG_SINCOS_SMALL_LIMIT);
            tiny = tiny && (amax < SG_SINCOS_TINY_LIMIT);
        }
        const f32x4 cx = coef(s_ux, jj);              // x-branch coefficients; [3] = D of this column
        const float xbv = eval(cx);
        s_dt[jj * LDS_STRIDE + tu] = DSTORE ? dtv - dt0 : dtv;
        s_ux[jj * LDS_STRIDE + tu] = dtv * xbv;
        if (OUT) s_dx[jj * LDS_STRIDE + tu] = cx[3] * xbv;
    }
#pragma unroll
    for (int q = 0; q < NR; q++) {
        const int ss = PART * NR + q;
        const f32x4 cb = coef(s_B, ss);
        gp1[q] = cb[3];
        s_B[ss * LDS_STRIDE + tu] = eval(cb);
        if (OUT) {
            const f32x4 cc = coef(s_C, ss);
            gp2[q] = cc[3];
            s_C[ss * LDS_STRIDE + tu] = eval(cc);
        }
    }
    if (OUT) {
        // the gates of this wave's columns share one reciprocal (sg_silu_block)
        static_assert(NR <= 8, "sg_silu_block takes at most 8 values");
        float zv[NR], gv[NR];
        if (TAYLOR) {
#pragma unroll
            for (int q = 0; q < NR; q++) {
                const f32x4 cz = coef(s_gate, PART * NR + q);
                gv[q] = poly(f32x4{gp0[q], gp1[q], gp2[q], cz[3]}, delta(cz));
            }
        } else {
#pragma unroll
            for (int q = 0; q < NR; q++) zv[q] = eval(coef(s_gate, PART * NR + q));
            sg_silu_block(NR, zv, gv);
        }
#pragma unroll
        for (int q = 0; q < NR; q++) s_gate[(PART * NR + q) * LDS_STRIDE + tu] = gv[q];
    }
    return (small ? 1 : 0) | (tiny ? 2 : 0);
}

// Once per workgroup: the composed coefficient triples of this direction (and D) into the padding of the LDS rows.
// tay: this direction's Taylor polynomials, [step size | gate][row][4] (see project_tile for where they go).
template <class G, bool OUT>
__device__ __forceinline__ void stage_coefficients(const float* __restrict__ comp, const float* __restrict__ tay, const float* __restrict__ Dw,
                                                   int tid, float* s_dt, float* s_ux, float* s_dx, float* s_B, float* s_C, float* s_gate,
                                                   float* s_tay) {
    static_assert(SG2_COMP_GROUPS * G::ROWS <= G::THREADS && G::ROWS == G::DI, "one thread per (group, row)");
    if (tid < SG2_COMP_GROUPS * G::ROWS) {
        const int group = tid / G::ROWS, row = tid % G::ROWS;
        float* arr = group == SG2_COMP_XB ? s_ux : group == SG2_COMP_DT ? s_dt : group == SG2_COMP_B ? s_B : group == SG2_COMP_C ? s_C : s_gate;
        if (OUT || (group != SG2_COMP_C && group != SG2_COMP_Z)) {
            const float* t = comp + (group * G::ROWS + row) * 3;
            // fourth float: D next to the x-branch triple; coefficient 0, 1, 2, 3 of the row's gate polynomial next to dt, B, C, z
            const float* gp = tay + (G::ROWS + row) * 4;
            const float w = group == SG2_COMP_XB ? Dw[row] : !OUT ? 0.0f : group == SG2_COMP_DT ? gp[0] : group == SG2_COMP_B ? gp[1] : group == SG2_COMP_C ? gp[2] : gp[3];
            *reinterpret_cast<f32x4*>(arr + row * LDS_STRIDE + SCAN_TT) = f32x4{t[0], t[1], t[2], w};
        }
        if (group == SG2_COMP_DT) {
            const float* dp = tay + row * 4;
            *reinterpret_cast<f32x4*>(OUT ? s_dx + row * LDS_STRIDE + SCAN_TT : s_tay + row * 4) = f32x4{dp[0], dp[1], dp[2], dp[3]};
        }
    }
}

// scan state of one lane: OUT -> (he,ho) only; summary -> also the two columns of M
struct LaneState {
    float he, ho, c0e, c0o, c1e, c1o;
};
// the lane's pair as polynomials in dt - dt0 (sg2_abar_poly, sg2_sincos_poly): dt0 = step size of its column for a zero input
// The summary pass keeps A_bar and sin/cos apart (its bound needs the A_bar); the output pass holds the four products.
template <bool OUT>
struct LanePoly {
    float dt0, pe[4], po[4], qs[3], qc[3];
};
template <>
struct LanePoly<true> {
    float dt0, k[12];
};

// LITE (summary pass only): the state part alone, and in c0e the running product of max(|A_bar_e|, |A_bar_o|), a bound
// on the norm of the 2x2 part that is not formed
template <bool OUT, bool LITE = false>
__device__ __forceinline__ void step_update(LaneState& S, float ae, float ao, float sn, float cs, float be, float bo) {
    if (!OUT && LITE) S.c0e = S.c0e * sg_max(sg_abs(ae), sg_abs(ao));
    if (!OUT && !LITE) {
        float re = sg_fma(S.c0e, cs, -(S.c0o * sn)), ro = sg_fma(S.c0o, cs, S.c0e * sn);
        S.c0e = ae * re;
        S.c0o = ao * ro;
        re = sg_fma(S.c1e, cs, -(S.c1o * sn));
        ro = sg_fma(S.c1o, cs, S.c1e * sn);
        S.c1e = ae * re;
        S.c1o = ao * ro;
    }
    const float re = sg_fma(S.he, cs, -(S.ho * sn));
    const float ro = sg_fma(S.ho, cs, S.he * sn);
    S.he = sg_fma(ae, re, be);
    S.ho = sg_fma(ao, ro, bo);
}

// UB consecutive timesteps (all valid): coefficients first, then the serial chain.  ux = dt * x-branch
// (formed once per timestep in phase A).  The A_bar of the block share one reciprocal per lane
// (sg_abar_block_*) unless some lane of the wave has a product of denominators too large for it.
// ANGLE: 0 full sin/cos, 1 sg_sincos_small (bit-identical to 0), 2 sg_sincos_tiny_dt (its own values, polynomials in dt),
// 3: every timestep of the block has passed sg2_poly_ok: A_bar, sin and cos from the lane's polynomials in dt - dt0.
// DGIVEN (ANGLE 3 only): dt[] holds dt - dt0 already (project_tile's DSTORE).  LINEAR (output pass, ANGLE 3): the
// inputs are small enough for the linear parts of the products.
template <int HP, bool OUT, int ANGLE, bool LITE = false, bool DGIVEN = false, bool LINEAR = false>
__device__ __forceinline__ void block_steps(LaneState& S, const float (&dt)[UB], const float (&ux)[UB], const float (&Be)[UB],
                                            const float (&Bo)[UB], const float (&Ce)[UB], const float (&Co)[UB], float hAe,
                                            float hAo, float freq, const LanePoly<OUT>& LP, float (&y)[UB]) {
    float ae[UB], ao[UB], sn[UB], cs[UB], be[UB], bo[UB];
    if constexpr (ANGLE == 3 && OUT) {
        // the four products of the update as quadratics: ae = P1, sn = N2, ao = P3, cs = P4 (see the update below)
#pragma unroll
        for (int u = 0; u < UB; u++) {
            const float d = DGIVEN ? dt[u] : dt[u] - LP.dt0;
            ae[u] = LINEAR ? sg2_poly1(LP.k, d) : sg2_poly2(LP.k, d);
            sn[u] = LINEAR ? sg2_poly1(LP.k + 3, d) : sg2_poly2(LP.k + 3, d);
            ao[u] = LINEAR ? sg2_poly1(LP.k + 6, d) : sg2_poly2(LP.k + 6, d);
            cs[u] = LINEAR ? sg2_poly1(LP.k + 9, d) : sg2_poly2(LP.k + 9, d);
        }
    } else if constexpr (ANGLE == 3) {
#pragma unroll
        for (int u = 0; u < UB; u++) {
            const float d = DGIVEN ? dt[u] : dt[u] - LP.dt0;
            ae[u] = sg2_poly3(LP.pe, d);
            ao[u] = sg2_poly3(LP.po, d);
            sn[u] = sg2_poly2(LP.qs, d);
            cs[u] = sg2_poly2(LP.qc, d);
        }
    } else {
        float d_e[UB], d_o[UB], P[UB];
        const float last = sg_abar_block_prefix(UB, dt, hAe, hAo, d_e, d_o, P);
        if (__builtin_amdgcn_ballot_w64(!(last < SG_ABAR_BLOCK_LIMIT)) == 0) {
            sg_abar_block_finish(UB, d_e, d_o, P, ae, ao);
        } else {
#pragma unroll
            for (int u = 0; u < UB; u++) sg_abar_pair(dt[u], hAe, hAo, &ae[u], &ao[u]);
        }
    }
    float tcoef[6];             // tiny-angle sin/cos of this lane's pair as polynomials in dt (formed here: a block that comes this way is the exception)
    if (ANGLE == 2) sg_sincos_tiny_coef(freq, tcoef);
#pragma unroll
    for (int u = 0; u < UB; u++) {
        if (ANGLE == 2) sg_sincos_tiny_dt(dt[u], tcoef, &sn[u], &cs[u]);
        else if (ANGLE == 1) sg_sincos_small(dt[u] * freq, &sn[u], &cs[u]);
        else if (ANGLE == 0) sg_sincos(dt[u] * freq, &sn[u], &cs[u]);
        be[u] = ux[u] * Be[u];
        bo[u] = ux[u] * Bo[u];
    }
#pragma unroll
    for (int u = 0; u < UB; u++) {
        if constexpr (ANGLE == 3 && OUT) {
            const float he = sg_fma(ae[u], S.he, sg_fma(sn[u], S.ho, be[u]));      // P1 he + N2 ho + b_e
            S.ho = sg_fma(ao[u], S.ho, sg_fma(cs[u], S.he, bo[u]));                // P3 ho + P4 he + b_o
            S.he = he;
        } else {
            step_update<OUT, LITE>(S, ae[u], ao[u], sn[u], cs[u], be[u], bo[u]);
        }
        if (OUT) y[u] = sg_fma(S.ho, Co[u], S.he * Ce[u]);
    }
    if (OUT) {
        static_assert(UB == 8, "block_pair_sums folds blocks of 8 steps");
        block_pair_sums<HP>(y);
    }
}

// KEEP (bilevel pass, OUT only): also store the state entering every HT_STEP-th step for the adjoint kernels.
template <class G, bool OUT, bool KEEP = false>
__global__ __launch_bounds__(G::THREADS) SG2_SCAN_ATTR void k_scan(Plan pl) {
    constexpr int DM = G::DM, DS = G::DS, DI = G::DI, HP = G::HP, SCAN_THREADS = G::THREADS, PARTS = G::PARTS;
    static_assert(!KEEP || PARTS == 2, "the bilevel pass exists for the default geometry only");
    __shared__ __attribute__((aligned(16))) float s_dt[DI * LDS_STRIDE];
    __shared__ __attribute__((aligned(16))) float s_ux[DI * LDS_STRIDE];       // dt * x-branch
    __shared__ __attribute__((aligned(16))) float s_B[DS * LDS_STRIDE];
    __shared__ __attribute__((aligned(16))) float s_C[OUT ? DS * LDS_STRIDE : 1];
    __shared__ __attribute__((aligned(16))) float s_gate[OUT ? DI * LDS_STRIDE : 1];
    __shared__ __attribute__((aligned(16))) float s_dx[OUT ? DI * LDS_STRIDE : 1];   // D * x-branch (skip term)
    // y of column j goes where dt of column j was: both are touched only by the 8 lanes of column j, in program order
    float* const s_y = s_dt;
    __shared__ float s_fmax[DI];
    __shared__ __attribute__((aligned(16))) float s_tay[OUT ? 4 : DI * 4];   // summary pass: Taylor polynomials of the step size (the output pass keeps its own in row padding)
    __shared__ __attribute__((aligned(16))) float s_wout[OUT ? DM * DI : 4];      // out_proj of this direction
    __shared__ unsigned long long s_large[PARTS];      // per wave's share of the columns: bit t set = timestep t of the tile needs the full sin/cos
    __shared__ unsigned long long s_nottiny[PARTS];    // ... bit t set = timestep t is not eligible for sg_sincos_tiny

    const int per_dir = OUT ? pl.chunks : pl.wchunks;
    const int dir = (int)blockIdx.x >= per_dir ? 1 : 0;
    const int cidx = (int)blockIdx.x - dir * per_dir;
    const sg::cint_p prefix = sg::as_const(OUT ? pl.chunk_prefix : pl.wchunk_prefix);
    const int ti = sg::upper_seg(prefix, pl.P, cidx);
    const int c = cidx - prefix[ti];                       // chunk within the tensor
    const TensorDev& T = pl.tensors[ti];
    const int N = T.numel, off = T.off;
    const int u0 = c * pl.chunk_len;                       // first scan step of the chunk
    const int u1 = min(u0 + pl.chunk_len, N);
    const uint32_t* __restrict__ skey = pl.keys[0] + off;      // sorted |g| bits
    const int32_t* __restrict__ sval = pl.vals[0] + off;       // element index | sign of g
    const float* __restrict__ ssrt = pl.ssorted + off;          // sharpness in sorted order
    const bool has_s = __builtin_amdgcn_readfirstlane(pl.sharp_nonzero[ti]) != 0;

    const int tid = threadIdx.x;
    const int tu = tid & (SCAN_TT - 1);                                   // projection role: timestep of the tile
    const int half = __builtin_amdgcn_readfirstlane(tid >> 6);           // projection role: which share of the outputs (the wave)
    const int j = tid / HP, p = tid % HP;                                 // scan role

    // -A/2 with A = -exp(A_log): the two poles of this lane's pair
    // (formed again from the weights wherever a block or a ragged end needs them: the usual blocks run on the lane
    // polynomials below, and three registers held for the exceptions would spill)
    auto pole_e = [&]() { return -0.5f * -sg_exp(pl.W.w[dir ? W_B_ALOG : W_F_ALOG][j * DS + 2 * p]); };
    auto pole_o = [&]() { return -0.5f * -sg_exp(pl.W.w[dir ? W_B_ALOG : W_F_ALOG][j * DS + 2 * p + 1]); };
    auto rope_f = [&]() { return pl.W.w[dir ? W_B_ROPE : W_F_ROPE][j * HP + p]; };
    // this lane's pair as polynomials in dt - dt0, dt0 = the step size of its column for a zero input
    LanePoly<OUT> LP;
    LP.dt0 = pl.comp[2 * SG2_COMP_GROUPS * G::ROWS * 3 + dir * 2 * G::ROWS * 4 + j * 4];
    if constexpr (OUT) {
        sg2_pair_products(LP.dt0, pole_e(), pole_o(), rope_f(), LP.k);
    } else {
        sg2_abar_poly(LP.dt0, pole_e(), LP.pe);
        sg2_abar_poly(LP.dt0, pole_o(), LP.po);
        sg2_sincos_poly(LP.dt0, rope_f(), LP.qs, LP.qc);
    }

    {   // largest |frequency| of each column's pairs
        const float f = pair_tree_max<HP>(sg_abs(rope_f()));
        if (p == 0) s_fmax[j] = f;
        stage_coefficients<G, OUT>(pl.comp + dir * (SG2_COMP_GROUPS * G::ROWS * 3), pl.comp + 2 * SG2_COMP_GROUPS * G::ROWS * 3 + dir * 2 * G::ROWS * 4,
                                   pl.W.w[dir ? W_B_D : W_F_D], tid, s_dt, s_ux, s_dx, s_B, s_C, s_gate, s_tay);
        static_assert(DM * DI == SCAN_THREADS, "one out_proj entry per thread");
        if (OUT) s_wout[tid] = pl.W.w[dir ? W_B_OUT : W_F_OUT][tid];
        __syncthreads();
    }
    // largest |c_g|, |c_s| over this direction's step-size and gate rows: what decides whether a tile may use the polynomials
    const float cmax_g = sg::as_const(pl.comp)[2 * SG2_COMP_GROUPS * G::ROWS * 3 + 2 * 2 * G::ROWS * 4 + 2 * dir];
    const float cmax_s = sg::as_const(pl.comp)[2 * SG2_COMP_GROUPS * G::ROWS * 3 + 2 * 2 * G::ROWS * 4 + 2 * dir + 1];
    // ... and whether a block of the recurrence may use the lane polynomials (sg2_poly_ok)
    // (the output pass with the tighter limit of its products)
    const float kpoly_g = sg::as_const(pl.comp)[2 * SG2_COMP_GROUPS * G::ROWS * 3 + 2 * 2 * G::ROWS * 4 + (OUT ? 8 : 4) + 2 * dir];
    const float kpoly_s = sg::as_const(pl.comp)[2 * SG2_COMP_GROUPS * G::ROWS * 3 + 2 * 2 * G::ROWS * 4 + (OUT ? 8 : 4) + 2 * dir + 1];

    LaneState S = {0.0f, 0.0f, 1.0f, 0.0f, 0.0f, 1.0f};
    bool fully_contracted = false;      // summary pass: the walk stopped because the 2x2 part had contracted
    if (OUT) {
        // When every summary of this call has an exactly zero 2x2 part, a chunk's start state is the offset of the
        // summary before it, whatever came earlier: k_chunk_prefix has then only placed the carried states (chunk 0).
        if (c > 0 && __builtin_amdgcn_readfirstlane(*pl.contracted) != 0) {
            const float* sm = pl.summaries + (size_t)(dir * pl.wchunks + pl.wchunk_prefix[ti] + c - 1) * 6 * SCAN_THREADS;
            S.he = sm[4 * SCAN_THREADS + tid];
            S.ho = sm[5 * SCAN_THREADS + tid];
        } else {
            const float* hs = pl.hstart + ((size_t)(dir * pl.chunks + cidx) * 2) * SCAN_THREADS;
            S.he = hs[tid];
            S.ho = hs[SCAN_THREADS + tid];
        }
    }

    // Summary pass: the chunk is walked backwards in blocks of `window` steps.  Each block is summarised from the
    // identity and the summary of everything after it (`late`) is applied on top; as soon as the 2x2 part of the
    // running summary has contracted below 2^-100 the steps before the block cannot matter and the walk stops.
    int blk_end = u1;
    int blk_first = u0;
    if (!OUT && pl.window > 0 && pl.window < pl.chunk_len) blk_first = max(u0, u1 - pl.window);
    // First attempt: ONE block of as many steps as k_compose expects the slowest pair to need, walked with the state
    // part only (LITE) and a bound on the 2x2 part in its place.  If the bound is below 2^-100 in every lane the summary
    // is (0, b) as below; if not, the walk starts over in its general form.
    bool lite = false;
    if (!OUT && blk_first > u0) {
        const int first_block = __builtin_amdgcn_readfirstlane(pl.contracted[1]);
        if (first_block > 0 && u1 - first_block > u0) {
            lite = true;
            blk_first = u1 - first_block;
        }
    }
    LaneState late = {0.0f, 0.0f, 1.0f, 0.0f, 0.0f, 1.0f};
    bool have_late = false;
    // inputs of one tile (sorted |g| bits, payload, sorted sharpness) for this lane's timestep; zero beyond the block
    uint32_t nx_key = 0;
    int32_t nx_val = 0;
    float nx_sh = 0.0f;
    auto load_inputs = [&](int tile0) {
        const int u = tile0 + tu;
        if (u < blk_end) {
            const int t = dir ? (N - 1 - u) : u;
            nx_key = skey[t];
            nx_val = sval[t];
            nx_sh = has_s ? ssrt[t] : 0.0f;      // an all-zero tensor has no sorted copy of its sharpness (uniform branch)
        }
    };
    for (;;) {
    load_inputs(blk_first);
    for (int tile0 = blk_first; tile0 < blk_end; tile0 += SCAN_TT) {
        const int cnt = min(SCAN_TT, blk_end - tile0);
        // ---------------- phase A: projections of SCAN_TT timesteps -> LDS
        // this tile's inputs were requested one tile ago (or just before the loop); request the next tile's now
        const uint32_t kbits = nx_key;
        const int32_t v = nx_val;
        const float shv = nx_sh;
        const bool valid = tile0 + tu < blk_end;
        if (tile0 + SCAN_TT < blk_end) load_inputs(tile0 + SCAN_TT);
        int orig = v & 0x7fffffff;
        orig = ((unsigned)orig < (unsigned)N) ? orig : 0;   // never index outside the tensor
        const float g = valid ? sg_i2f((int32_t)kbits | (v & (int32_t)0x80000000)) : 0.0f;
        const float sh = valid ? shv : 0.0f;
        int angle_t;
        bool dgiven = false;     // whole tile on the lane polynomials: phase A leaves dt - dt0 in place of dt
        // bit t set = timestep t of the tile may not use the lane polynomials (the same mask in every wave: the same 64 timesteps)
        const unsigned long long notpoly = __builtin_amdgcn_ballot_w64(!sg2_poly_ok(kpoly_g, kpoly_s, g, sh));
        // ... may not use the linear parts alone (output pass)
        const unsigned long long notlin =
            OUT ? __builtin_amdgcn_ballot_w64(!sg2_poly_ok(SG2_PROD_LINEAR_FACTOR * kpoly_g, SG2_PROD_LINEAR_FACTOR * kpoly_s, g, sh)) : ~0ull;
        {
            // the same 64 timesteps in every wave of the workgroup: the same decision without talking to one another
            const bool tay = __builtin_amdgcn_ballot_w64(!sg2_taylor_ok(cmax_g, cmax_s, g, sh)) == 0;
            dgiven = tay && notpoly == 0 && cnt == SCAN_TT;
            // PARTS == 2: the wave's share is a template parameter; more waves: one copy of the code, the arrays moved to this wave's first row
            const int rj = (PARTS == 2) ? 0 : half * (DI / PARTS) * LDS_STRIDE, rs = (PARTS == 2) ? 0 : half * (DS / PARTS) * LDS_STRIDE;
            const int rt = (PARTS == 2 || OUT) ? 0 : half * (DI / PARTS) * 4;
            auto run = [&](auto part_c, auto has_s_c, auto tay_c) {
                if (decltype(tay_c)::value && dgiven)
                    return project_tile<G, OUT, decltype(part_c)::value, decltype(has_s_c)::value, true, true>(
                        g, sh, tu, s_dt + rj, s_ux + rj, s_dx + (OUT ? rj : 0), s_B + rs, s_C + (OUT ? rs : 0), s_gate + (OUT ? rj : 0),
                        s_fmax + ((PARTS == 2) ? 0 : half * (DI / PARTS)), s_tay + rt);
                return project_tile<G, OUT, decltype(part_c)::value, decltype(has_s_c)::value, decltype(tay_c)::value>(
                    g, sh, tu, s_dt + rj, s_ux + rj, s_dx + (OUT ? rj : 0), s_B + rs, s_C + (OUT ? rs : 0), s_gate + (OUT ? rj : 0),
                    s_fmax + ((PARTS == 2) ? 0 : half * (DI / PARTS)), s_tay + rt);
            };
            auto with_part = [&](auto has_s_c, auto tay_c) {
                if (PARTS == 2 && half == 1) return run(std::integral_constant<int, (PARTS == 2) ? 1 : 0>{}, has_s_c, tay_c);
                return run(std::integral_constant<int, 0>{}, has_s_c, tay_c);
            };
            if (tay) angle_t = has_s ? with_part(std::true_type{}, std::true_type{}) : with_part(std::false_type{}, std::true_type{});
            else angle_t = has_s ? with_part(std::true_type{}, std::false_type{}) : with_part(std::false_type{}, std::false_type{});
        }
        {   // wave w projects the dt of columns w*64/HP .. (w+1)*64/HP-1, which are the columns it owns in the recurrence
            const unsigned long long large = __builtin_amdgcn_ballot_w64(!(angle_t & 1));
            const unsigned long long nottiny = __builtin_amdgcn_ballot_w64(!(angle_t & 2));
            if (tu == 0) { s_large[half] = large; s_nottiny[half] = nottiny; }
        }
        __syncthreads();
        // wave-uniform masks into scalar registers: the per-block tests below are then scalar instructions
        auto uniform64 = [](unsigned long long v) {
            const unsigned lo = (unsigned)__builtin_amdgcn_readfirstlane((int)(unsigned)v);
            const unsigned hi = (unsigned)__builtin_amdgcn_readfirstlane((int)(unsigned)(v >> 32));
            return ((unsigned long long)hi << 32) | lo;
        };
        const unsigned long long large = uniform64(s_large[half]), nottiny = uniform64(s_nottiny[half]);

        auto keep_state = [&](int u) {
            float* ht = pl.htile + ((size_t)dir * htile_count(pl.total, pl.P) + htile_index(off, ti, u)) * 2 * SCAN_THREADS;
            ht[tid] = S.he;
            ht[SCAN_THREADS + tid] = S.ho;
        };
        if (KEEP) keep_state(tile0);
        // ---------------- phase B: the recurrence over the tile, lane = (j,p)
        const float* __restrict__ r_dt = s_dt + j * LDS_STRIDE;
        const float* __restrict__ r_ux = s_ux + j * LDS_STRIDE;
        const float* __restrict__ r_Be = s_B + (2 * p) * LDS_STRIDE;
        const float* __restrict__ r_Bo = s_B + (2 * p + 1) * LDS_STRIDE;
        const float* __restrict__ r_Ce = s_C + (OUT ? (2 * p) * LDS_STRIDE : 0);
        const float* __restrict__ r_Co = s_C + (OUT ? (2 * p + 1) * LDS_STRIDE : 0);
        int k0 = 0;
        for (; k0 + UB <= cnt; k0 += UB) {
            if (KEEP && k0 == HT_STEP) keep_state(tile0 + HT_STEP);
            float dt[UB], xv[UB], Be[UB], Bo[UB], Ce[UB], Co[UB], y[UB];
#pragma unroll
            for (int q = 0; q < UB; q += 4) {
                const f32x4 a = *reinterpret_cast<const f32x4*>(r_dt + k0 + q), b = *reinterpret_cast<const f32x4*>(r_ux + k0 + q);
                const f32x4 c = *reinterpret_cast<const f32x4*>(r_Be + k0 + q), d = *reinterpret_cast<const f32x4*>(r_Bo + k0 + q);
#pragma unroll
                for (int e = 0; e < 4; e++) { dt[q + e] = a[e]; xv[q + e] = b[e]; Be[q + e] = c[e]; Bo[q + e] = d[e]; Ce[q + e] = 0.0f; Co[q + e] = 0.0f; }
                if (OUT) {
                    const f32x4 f = *reinterpret_cast<const f32x4*>(r_Ce + k0 + q), g = *reinterpret_cast<const f32x4*>(r_Co + k0 + q);
#pragma unroll
                    for (int e = 0; e < 4; e++) { Ce[q + e] = f[e]; Co[q + e] = g[e]; }
                }
            }
            const unsigned long long blk = ((1ull << UB) - 1) << k0;
            auto steps = [&](auto lite_c) {
                constexpr bool LT = decltype(lite_c)::value;
                if (OUT && dgiven && (notlin & blk) == 0)
                    block_steps<HP, OUT, 3, LT, true, true>(S, dt, xv, Be, Bo, Ce, Co, 0.0f, 0.0f, 0.0f, LP, y);
                else if (dgiven)
                    block_steps<HP, OUT, 3, LT, true>(S, dt, xv, Be, Bo, Ce, Co, 0.0f, 0.0f, 0.0f, LP, y);
                else if ((notpoly & blk) == 0)
                    block_steps<HP, OUT, 3, LT>(S, dt, xv, Be, Bo, Ce, Co, 0.0f, 0.0f, 0.0f, LP, y);
                else if ((nottiny & blk) == 0)
                    block_steps<HP, OUT, 2, LT>(S, dt, xv, Be, Bo, Ce, Co, pole_e(), pole_o(), rope_f(), LP, y);
                else if ((large & blk) == 0)
                    block_steps<HP, OUT, 1, LT>(S, dt, xv, Be, Bo, Ce, Co, pole_e(), pole_o(), rope_f(), LP, y);
                else
                    block_steps<HP, OUT, 0, LT>(S, dt, xv, Be, Bo, Ce, Co, pole_e(), pole_o(), rope_f(), LP, y);
            };
            if (!OUT && lite) steps(std::true_type{});
            else steps(std::false_type{});
            if (OUT && (p & 3) == 0) {       // the first lane of every bank holds the totals of its bank's steps (block_pair_sums)
                if constexpr (HP == 8)
                    *reinterpret_cast<f32x4*>(&s_y[j * LDS_STRIDE + k0 + 4 * (p >> 2)]) = f32x4{y[0], y[1], y[2], y[3]};
                else
                    *reinterpret_cast<float2*>(&s_y[j * LDS_STRIDE + k0 + 2 * (p >> 2)]) = make_float2(y[0], y[1]);
            }
        }
        if (KEEP && k0 == HT_STEP && cnt > HT_STEP) keep_state(tile0 + HT_STEP);      // the ragged end starts right there
        for (; k0 < cnt; k0++) {       // ragged end of the last tile of a tensor
            const float dt = r_dt[k0], ux = r_ux[k0];
            float ae, ao, sn, cs;
            sg_abar_pair(dt, pole_e(), pole_o(), &ae, &ao);
            sg_sincos(dt * rope_f(), &sn, &cs);
            if (!OUT && lite) step_update<OUT, true>(S, ae, ao, sn, cs, ux * r_Be[k0], ux * r_Bo[k0]);
            else step_update<OUT>(S, ae, ao, sn, cs, ux * r_Be[k0], ux * r_Bo[k0]);
            if (OUT) {
                const float y = pair_tree_sum<HP>(sg_fma(S.ho, r_Co[k0], S.he * r_Ce[k0]));
                if (p == 0) s_y[j * LDS_STRIDE + k0] = y;
            }
        }
        __syncthreads();

        // ---------------- phase C: gate, D skip, out_proj, scatter to element order
        if (OUT) {
            float o[DI];
#pragma unroll
            for (int jj = 0; jj < DI; jj++)
                o[jj] = sg_fma(s_y[jj * LDS_STRIDE + tu], s_gate[jj * LDS_STRIDE + tu], s_dx[jj * LDS_STRIDE + tu]);
            constexpr int CPP = DM / PARTS;     // context entries this wave produces per timestep
            float cx[CPP];
#pragma unroll
            for (int q = 0; q < CPP; q++) {
                // row CPP * half + q of out_proj: the same address for every lane of the wave (broadcast reads)
                const float* wr = s_wout + (half * CPP + q) * DI;
                float a = 0.0f;
#pragma unroll
                for (int m = 0; m < DI; m += 4) {
                    const f32x4 w4 = *reinterpret_cast<const f32x4*>(wr + m);
                    a = sg_fma(w4[0], o[m], a);
                    a = sg_fma(w4[1], o[m + 1], a);
                    a = sg_fma(w4[2], o[m + 2], a);
                    a = sg_fma(w4[3], o[m + 3], a);
                }
                cx[q] = a;
            }
            if (valid) {
                float* dst = pl.ctx + ((size_t)dir * pl.total + off + orig) * DM + half * CPP;
                static_assert(CPP == 4 || CPP == 2, "one vector store per lane");
                if constexpr (CPP == 4)
                    *reinterpret_cast<float4*>(dst) = make_float4(cx[0], cx[1], cx[2], cx[3]);
                else
                    *reinterpret_cast<float2*>(dst) = make_float2(cx[0], cx[1]);
                if constexpr (KEEP) {
                    if (pl.scan_out[dir] != nullptr) {
                        // the gated scan output itself (before out_proj), at the step's position in scan order; this half's 8 columns
                        float4* so = reinterpret_cast<float4*>(pl.scan_out[dir] + ((size_t)off + tile0 + tu) * DI) + 2 * half;
                        so[0] = half ? make_float4(o[8], o[9], o[10], o[11]) : make_float4(o[0], o[1], o[2], o[3]);
                        so[1] = half ? make_float4(o[12], o[13], o[14], o[15]) : make_float4(o[4], o[5], o[6], o[7]);
                    }
                }
            }
            __syncthreads();
        }
    }
    if (OUT) break;
    if (lite) {          // c0e holds the bound (a NaN counts as "not contracted")
        if (!__syncthreads_or(!(S.c0e < 7.888609052210118e-31f))) {
            S.c0e = S.c0o = S.c1e = S.c1o = 0.0f;
            fully_contracted = true;
            break;
        }
        lite = false;    // the general walk, from the end of the chunk
        blk_first = max(u0, u1 - pl.window);
        S = {0.0f, 0.0f, 1.0f, 0.0f, 0.0f, 1.0f};
        continue;
    }
    if (have_late) {     // S covers [blk_first, blk_end), late covers [blk_end, u1): the summary of both is late o S
        const LaneState E = S;
        S.c0e = sg_fma(late.c0e, E.c0e, late.c1e * E.c0o);
        S.c0o = sg_fma(late.c0o, E.c0e, late.c1o * E.c0o);
        S.c1e = sg_fma(late.c0e, E.c1e, late.c1e * E.c1o);
        S.c1o = sg_fma(late.c0o, E.c1e, late.c1o * E.c1o);
        S.he = sg_fma(late.c0e, E.he, sg_fma(late.c1e, E.ho, late.he));
        S.ho = sg_fma(late.c0o, E.he, sg_fma(late.c1o, E.ho, late.ho));
    }
    if (blk_first == u0) break;       // the whole chunk is covered
    {   // has the running summary contracted?  (a NaN counts as "no")
        const float mx = sg_max(sg_max(sg_abs(S.c0e), sg_abs(S.c0o)), sg_max(sg_abs(S.c1e), sg_abs(S.c1o)));
        if (!__syncthreads_or(!(mx < 7.888609052210118e-31f))) {
            S.c0e = S.c0o = S.c1e = S.c1o = 0.0f;
            fully_contracted = true;
            break;
        }
    }
    late = S;
    have_late = true;
    blk_end = blk_first;
    blk_first = max(u0, blk_first - pl.window);
    S = {0.0f, 0.0f, 1.0f, 0.0f, 0.0f, 1.0f};
    }

    if (OUT) {
        if (u1 == N) {   // last chunk in scan order: new carried state of the tensor
            float* st = dir ? T.mbwd : T.mfwd;
            if (j < pl.st_di && 2 * p < pl.st_ds) {
                st[j * pl.st_ds + 2 * p] = S.he;
                st[j * pl.st_ds + 2 * p + 1] = S.ho;
            }
        }
    } else {
        float* sm = pl.summaries + (size_t)(dir * pl.wchunks + cidx) * 6 * SCAN_THREADS;
        sm[0 * SCAN_THREADS + tid] = S.c0e;   // M = [c0e c1e; c0o c1o]
        sm[1 * SCAN_THREADS + tid] = S.c0o;
        sm[2 * SCAN_THREADS + tid] = S.c1e;
        sm[3 * SCAN_THREADS + tid] = S.c1o;
        sm[4 * SCAN_THREADS + tid] = S.he;
        sm[5 * SCAN_THREADS + tid] = S.ho;
        if (!fully_contracted && tid == 0) *pl.contracted = 0;      // plain store: every writer stores the same value
    }
}

// Projections of one timestep for the one-wave replay, for a tile that does not run on the polynomials throughout
// (project_rows covers the usual tile): the lane computes every row of every group for its timestep (what the two
// waves of k_scan each do half of through project_tile, with the same expressions in the same order).  Step size,
// dt * x-branch, B and C go to LDS for the recurrence; the skip terms D * x-branch stay in the lane's registers,
// because the lane that forms them is the one that uses them after the recurrence, and for the same reason the gates
// are not formed here at all (gates_all, after the recurrence).
// coef: [group][row] composed triple + one more float (D next to the x-branch triple); tay: [step size | gate][row][4].
// angle[h]: bit 0 / 1 = every rotation angle of columns 8 h .. 8 h + 7 at this timestep is small / tiny.
template <class G, bool HAS_S, bool TAYLOR>
__device__ __forceinline__ void project_all(float g, float s, int tu, const float* s_coef, const float* s_tay, const float* s_fmax, float* s_dt,
                                            float* s_ux, float* s_B, float* s_C, float (&dxv)[G::DI], int (&angle)[2]) {
    constexpr int DI = G::DI, DS = G::DS;
    auto delta = [&](const f32x4 t) { return HAS_S ? sg_fma(t[0], g, t[1] * s) : t[0] * g; };
    auto poly = [&](const f32x4 t, float d) { return sg_fma(sg_fma(sg_fma(t[3], d, t[2]), d, t[1]), d, t[0]); };
    auto eval = [&](const f32x4 t) { return sg_fma(t[0], g, HAS_S ? sg_fma(t[1], s, t[2]) : t[2]); };
    auto coef = [&](int group, int row) { return *reinterpret_cast<const f32x4*>(s_coef + (group * DI + row) * 4); };
    static_assert(DI == 16 && DS == 16, "two halves of eight columns");
#pragma unroll
    for (int h = 0; h < 2; h++) {
        bool small = true, tiny = true;
#pragma unroll
        for (int q = 0; q < 8; q++) {
            const int jj = 8 * h + q;
            const f32x4 cd = coef(SG2_COMP_DT, jj);
            const float dtv = TAYLOR ? poly(*reinterpret_cast<const f32x4*>(s_tay + jj * 4), delta(cd)) : sg_softplus(eval(cd));
            const float amax = dtv * s_fmax[jj];
            small = small && (amax < SG_SINCOS_SMALL_LIMIT);
            tiny = tiny && (amax < SG_SINCOS_TINY_LIMIT);
            const f32x4 cx = coef(SG2_COMP_XB, jj);       // x-branch coefficients; [3] = D of this column
            const float xbv = eval(cx);
            s_dt[jj * LDS_STRIDE + tu] = dtv;
            s_ux[jj * LDS_STRIDE + tu] = dtv * xbv;
            dxv[jj] = cx[3] * xbv;
        }
        angle[h] = (small ? 1 : 0) | (tiny ? 2 : 0);
    }
#pragma unroll
    for (int ss = 0; ss < DS; ss++) {
        s_B[ss * LDS_STRIDE + tu] = eval(coef(SG2_COMP_B, ss));
        s_C[ss * LDS_STRIDE + tu] = eval(coef(SG2_COMP_C, ss));
    }
}
// The 16 gates silu(z) of one timestep: Taylor polynomials for a tile that qualifies, else eight at a time on one shared
// reciprocal (columns 0-7, 8-15: the groups the two-wave kernel and the checker form).
template <class G, bool HAS_S, bool TAYLOR>
__device__ __forceinline__ void gates_all(float g, float s, const float* s_coef, const float* s_tay, float (&gv)[G::DI]) {
    constexpr int DI = G::DI;
    auto delta = [&](const f32x4 t) { return HAS_S ? sg_fma(t[0], g, t[1] * s) : t[0] * g; };
    auto poly = [&](const f32x4 t, float d) { return sg_fma(sg_fma(sg_fma(t[3], d, t[2]), d, t[1]), d, t[0]); };
    auto eval = [&](const f32x4 t) { return sg_fma(t[0], g, HAS_S ? sg_fma(t[1], s, t[2]) : t[2]); };
    auto coef = [&](int row) { return *reinterpret_cast<const f32x4*>(s_coef + (SG2_COMP_Z * DI + row) * 4); };
    if (TAYLOR) {
#pragma unroll
        for (int jj = 0; jj < DI; jj++) gv[jj] = poly(*reinterpret_cast<const f32x4*>(s_tay + (DI + jj) * 4), delta(coef(jj)));
    } else {
#pragma unroll
        for (int h = 0; h < 2; h++) {
            float zv[8], out[8];
#pragma unroll
            for (int q = 0; q < 8; q++) zv[q] = eval(coef(8 * h + q));
            sg_silu_block(8, zv, out);
#pragma unroll
            for (int q = 0; q < 8; q++) gv[8 * h + q] = out[q];
        }
    }
}

// Projections of a whole tile that runs on the polynomials (every step size and gate inside its Taylor range, every
// block of the recurrence on the lane polynomials), formed by lanes that own ROWS instead of timesteps: lane (column cj,
// quarter cq) forms dt - dt0, dt * x-branch and D * x-branch of column cj for timesteps 16 cq .. 16 cq + 15, and lane
// (row br, half bh) one row of B (br < 16) or C for timesteps 32 bh .. 32 bh + 31.  A row's coefficients are then four
// 16-byte LDS reads per tile and lane instead of one per (timestep, row), the 64 (g, s) of the tile travel through the
// four padding floats of the rows of s_B / s_C, and the results leave as 16-byte LDS writes: the same arithmetic as
// the timestep-per-lane form with a fifth of its LDS instructions.  Every value is formed by the expressions of
// project_all (Taylor form) on the same operands, so it is the same float; the step-size row receives dt - dt0, which
// is what the lane polynomials of the recurrence take.
// dxk: this lane's 16 skips D * x-branch of (column cj, timestep 16 cq + k), kept for gate_rows.
template <class G, bool HAS_S>
__device__ __forceinline__ void project_rows(float g, float s, int tid, const float* s_coef, const float* s_tay, float* s_dt, float* s_ux,
                                             float* s_B, float* s_C, float (&dxk)[G::DI]) {
    constexpr int DI = G::DI, DS = G::DS;
    static_assert(DI == 16 && DS == 16 && SCAN_TT == 64 && LDS_STRIDE == SCAN_TT + 4, "64 lanes: 16 columns x 4 quarters, 32 rows x 2 halves");
    auto delta = [&](const f32x4 t, float gg, float ss) { return HAS_S ? sg_fma(t[0], gg, t[1] * ss) : t[0] * gg; };
    auto poly = [&](const f32x4 t, float d) { return sg_fma(sg_fma(sg_fma(t[3], d, t[2]), d, t[1]), d, t[0]); };
    auto eval = [&](const f32x4 t, float gg, float ss) { return sg_fma(t[0], gg, HAS_S ? sg_fma(t[1], ss, t[2]) : t[2]); };
    auto coef = [&](int group, int row) { return *reinterpret_cast<const f32x4*>(s_coef + (group * DI + row) * 4); };
    s_B[(tid >> 2) * LDS_STRIDE + SCAN_TT + (tid & 3)] = g;      // timestep t: padding float t % 4 of row t / 4
    if (HAS_S) s_C[(tid >> 2) * LDS_STRIDE + SCAN_TT + (tid & 3)] = s;
    __syncthreads();
    auto inputs = [&](int t4, f32x4& g4, f32x4& s4) {            // (g, s) of timesteps 4 t4 .. 4 t4 + 3
        g4 = *reinterpret_cast<const f32x4*>(s_B + t4 * LDS_STRIDE + SCAN_TT);
        s4 = HAS_S ? *reinterpret_cast<const f32x4*>(s_C + t4 * LDS_STRIDE + SCAN_TT) : f32x4{0.0f, 0.0f, 0.0f, 0.0f};
    };
    {
        const int cj = tid & 15, cq = tid >> 4;
        const f32x4 cd = coef(SG2_COMP_DT, cj), cx = coef(SG2_COMP_XB, cj);
        const f32x4 tp = *reinterpret_cast<const f32x4*>(s_tay + cj * 4);
        float* const r_dt = s_dt + cj * LDS_STRIDE + 16 * cq;
        float* const r_ux = s_ux + cj * LDS_STRIDE + 16 * cq;
#pragma unroll
        for (int i = 0; i < 4; i++) {
            f32x4 g4, s4, d4, u4;
            inputs(4 * cq + i, g4, s4);
#pragma unroll
            for (int e = 0; e < 4; e++) {
                const float dtv = poly(tp, delta(cd, g4[e], s4[e]));
                const float xbv = eval(cx, g4[e], s4[e]);
                d4[e] = dtv - tp[0];
                u4[e] = dtv * xbv;
                dxk[4 * i + e] = cx[3] * xbv;
            }
            *reinterpret_cast<f32x4*>(r_dt + 4 * i) = d4;
            *reinterpret_cast<f32x4*>(r_ux + 4 * i) = u4;
        }
    }
    {
        const int br = tid & 31, bh = tid >> 5;
        const f32x4 cb = coef(br < DS ? SG2_COMP_B : SG2_COMP_C, br & (DS - 1));
        float* const r_bc = (br < DS ? s_B : s_C) + (br & (DS - 1)) * LDS_STRIDE + 32 * bh;
#pragma unroll
        for (int i = 0; i < 8; i++) {
            f32x4 g4, s4, v4;
            inputs(8 * bh + i, g4, s4);
#pragma unroll
            for (int e = 0; e < 4; e++) v4[e] = eval(cb, g4[e], s4[e]);
            *reinterpret_cast<f32x4*>(r_bc + 4 * i) = v4;
        }
    }
}

// The row owners' part after the recurrence: y of (column cj, timesteps 16 cq .. 16 cq + 15) becomes
// y * gate + D * x-branch in place.  The gates are formed here, from the (g, s) that project_rows left in the padding floats, so that they do
// not occupy 16 registers during the recurrence.
template <class G, bool HAS_S>
__device__ __forceinline__ void gate_rows(int tid, const float* s_coef, const float* s_tay, const float* s_B, const float* s_C, float* s_y,
                                          const float (&dxk)[G::DI]) {
    constexpr int DI = G::DI;
    auto delta = [&](const f32x4 t, float gg, float ss) { return HAS_S ? sg_fma(t[0], gg, t[1] * ss) : t[0] * gg; };
    auto poly = [&](const f32x4 t, float d) { return sg_fma(sg_fma(sg_fma(t[3], d, t[2]), d, t[1]), d, t[0]); };
    const int cj = tid & 15, cq = tid >> 4;
    const f32x4 cz = *reinterpret_cast<const f32x4*>(s_coef + (SG2_COMP_Z * DI + cj) * 4);
    const f32x4 tz = *reinterpret_cast<const f32x4*>(s_tay + (DI + cj) * 4);
    float* const r_y = s_y + cj * LDS_STRIDE + 16 * cq;
#pragma unroll
    for (int i = 0; i < 4; i++) {
        const f32x4 g4 = *reinterpret_cast<const f32x4*>(s_B + (4 * cq + i) * LDS_STRIDE + SCAN_TT);
        const f32x4 s4 = HAS_S ? *reinterpret_cast<const f32x4*>(s_C + (4 * cq + i) * LDS_STRIDE + SCAN_TT) : f32x4{0.0f, 0.0f, 0.0f, 0.0f};
        f32x4 y4 = *reinterpret_cast<const f32x4*>(r_y + 4 * i);
#pragma unroll
        for (int e = 0; e < 4; e++) y4[e] = sg_fma(y4[e], poly(tz, delta(cz, g4[e], s4[e])), dxk[4 * i + e]);
        *reinterpret_cast<f32x4*>(r_y + 4 * i) = y4;
    }
}

// UB steps of both columns of a lane on the lane polynomials, dt - dt0 given (what block_steps<HP, true, 3, false, true,
// LINEAR> does for one column), written as one straight-line block so that the two independent recurrences interleave.
template <int HP, bool LINEAR>
__device__ __forceinline__ void block_steps_pair(LaneState (&S)[2], const float (&dt)[2][UB], const float (&ux)[2][UB], const float (&Be)[UB],
                                                 const float (&Bo)[UB], const float (&Ce)[UB], const float (&Co)[UB], const LanePoly<true> (&LP)[2],
                                                 float (&y)[2][UB]) {
#pragma unroll
    for (int u = 0; u < UB; u++) {
#pragma unroll
        for (int h = 0; h < 2; h++) {
            const float d = dt[h][u];
            const float p1 = LINEAR ? sg2_poly1(LP[h].k, d) : sg2_poly2(LP[h].k, d);
            const float n2 = LINEAR ? sg2_poly1(LP[h].k + 3, d) : sg2_poly2(LP[h].k + 3, d);
            const float p3 = LINEAR ? sg2_poly1(LP[h].k + 6, d) : sg2_poly2(LP[h].k + 6, d);
            const float p4 = LINEAR ? sg2_poly1(LP[h].k + 9, d) : sg2_poly2(LP[h].k + 9, d);
            const float be = ux[h][u] * Be[u], bo = ux[h][u] * Bo[u];
            const float he = sg_fma(p1, S[h].he, sg_fma(n2, S[h].ho, be));      // P1 he + N2 ho + b_e
            S[h].ho = sg_fma(p3, S[h].ho, sg_fma(p4, S[h].he, bo));            // P3 ho + P4 he + b_o
            S[h].he = he;
            y[h][u] = sg_fma(S[h].ho, Co[u], S[h].he * Ce[u]);
        }
    }
    block_pair_sums<HP>(y[0]);
    block_pair_sums<HP>(y[1]);
}

// The replay of the default geometry (what k_scan<G, true> computes, value for value) as ONE wave per chunk: lane
// (jl, p) owns RoPE pair p of the two columns jl and jl + 8.  The 16 lanes that need the same B / C entries of a
// timestep are then 8, and each entry a lane fetches from LDS feeds two recurrences: a third less LDS traffic per
// step -- the pass was bound by the LDS queue and the vector ALU together, and the B / C fetches alone were a fifth of
// its time.  A single wave also needs no workgroup barrier between the phases of a tile (its LDS accesses execute in
// program order), forms the 16 gated outputs of a timestep once instead of once per wave, and holds all eight context
// entries of its timestep: the two 16-byte stores of an element are adjacent in one lane and leave as one 32-byte
// write.  Column jl + 8 h plays the part of wave h of the two-wave kernel throughout (its half of the projections, its
// angle masks, its ballots over the same 64 (column, pair) lanes), so every decision and every value is the one the
// checker makes for the two-wave form.
// A tile has three lane roles.  Recurrence (phase B): lane (jl, p) as above.  Timestep: lane t loads the inputs of
// timestep t, votes on the form the tile takes, and at the end multiplies its 16 gated outputs by out_proj and stores
// its element's row.  Row owner (the usual tile, on the polynomials throughout): lane (column, quarter of the tile)
// forms that column's projections before the recurrence and gates its outputs after it (project_rows, gate_rows);
// other tiles keep the timestep-per-lane projections (project_all, gates_all).
template <class G>
__global__ __launch_bounds__(64) __attribute__((amdgpu_waves_per_eu(2, 2))) void k_replay(Plan pl) {
    constexpr int DM = G::DM, DS = G::DS, DI = G::DI, HP = G::HP, LANES = G::THREADS;
    static_assert(G::PARTS == 2 && LANES == 128 && HP == 8, "two columns per lane of one wave");
    constexpr bool OUT = true;
    __shared__ __attribute__((aligned(16))) float s_dt[DI * LDS_STRIDE];
    __shared__ __attribute__((aligned(16))) float s_ux[DI * LDS_STRIDE];
    __shared__ __attribute__((aligned(16))) float s_B[DS * LDS_STRIDE];
    __shared__ __attribute__((aligned(16))) float s_C[DS * LDS_STRIDE];
    float* const s_y = s_dt;      // y of column j goes where dt of column j was: both are touched by the same lanes, in program order
    __shared__ float s_fmax[DI];
    __shared__ __attribute__((aligned(16))) float s_coef[SG2_COMP_GROUPS * DI * 4];   // [group][row]: composed triple, D beside the x-branch's
    __shared__ __attribute__((aligned(16))) float s_tay[2 * DI * 4];                  // [step size | gate][row]: cubic Taylor polynomials
    __shared__ __attribute__((aligned(16))) float s_wout[DM * DI];
    // four arrays of 16 x 68 floats and 2.4 KB of tables: 19.8 KB, eight workgroups (two waves per SIMD) share a compute unit

    const int per_dir = pl.chunks;
    const int dir = (int)blockIdx.x >= per_dir ? 1 : 0;
    const int cidx = (int)blockIdx.x - dir * per_dir;
    const sg::cint_p prefix = sg::as_const(pl.chunk_prefix);
    const int ti = sg::upper_seg(prefix, pl.P, cidx);
    const int c = cidx - prefix[ti];
    const TensorDev& T = pl.tensors[ti];
    const int N = T.numel, off = T.off;
    const int u0 = c * pl.chunk_len;
    const int u1 = min(u0 + pl.chunk_len, N);
    const uint32_t* __restrict__ skey = pl.keys[0] + off;
    const int32_t* __restrict__ sval = pl.vals[0] + off;
    const float* __restrict__ ssrt = pl.ssorted + off;
    const bool has_s = __builtin_amdgcn_readfirstlane(pl.sharp_nonzero[ti]) != 0;

    const int tid = threadIdx.x;
    const int tu = tid;                      // projection role: timestep of the tile
    const int jl = tid >> 3, p = tid & 7;    // scan role: pair p of columns jl and jl + 8
    const float* alog = pl.W.w[dir ? W_B_ALOG : W_F_ALOG];
    const float* rope = pl.W.w[dir ? W_B_ROPE : W_F_ROPE];
    auto pole_e = [&](int h) { return -0.5f * -sg_exp(alog[(jl + 8 * h) * DS + 2 * p]); };
    auto pole_o = [&](int h) { return -0.5f * -sg_exp(alog[(jl + 8 * h) * DS + 2 * p + 1]); };
    auto rope_f = [&](int h) { return rope[(jl + 8 * h) * HP + p]; };
    LanePoly<true> LP[2];
#pragma unroll
    for (int h = 0; h < 2; h++) {
        LP[h].dt0 = pl.comp[2 * SG2_COMP_GROUPS * G::ROWS * 3 + dir * 2 * G::ROWS * 4 + (jl + 8 * h) * 4];
        sg2_pair_products(LP[h].dt0, pole_e(h), pole_o(h), rope_f(h), LP[h].k);
    }
    {
#pragma unroll
        for (int h = 0; h < 2; h++) {
            const float f = pair_tree_max<HP>(sg_abs(rope_f(h)));
            if (p == 0) s_fmax[jl + 8 * h] = f;
        }
        const float* comp = pl.comp + dir * (SG2_COMP_GROUPS * G::ROWS * 3);
        const float* tay = pl.comp + 2 * SG2_COMP_GROUPS * G::ROWS * 3 + dir * 2 * G::ROWS * 4;
        const float* Dw = pl.W.w[dir ? W_B_D : W_F_D];
        for (int i = tid; i < SG2_COMP_GROUPS * DI; i += 64) {
            const float* t = comp + i * 3;
            *reinterpret_cast<f32x4*>(s_coef + i * 4) = f32x4{t[0], t[1], t[2], i / DI == SG2_COMP_XB ? Dw[i % DI] : 0.0f};
        }
        for (int i = tid; i < 2 * DI * 4; i += 64) s_tay[i] = tay[i];
        s_wout[tid] = pl.W.w[dir ? W_B_OUT : W_F_OUT][tid];
        s_wout[tid + 64] = pl.W.w[dir ? W_B_OUT : W_F_OUT][tid + 64];
        __syncthreads();
    }
    const sg::cfloat_p lim = sg::as_const(pl.comp) + 2 * SG2_COMP_GROUPS * G::ROWS * 3 + 2 * 2 * G::ROWS * 4;
    const float cmax_g = lim[2 * dir], cmax_s = lim[2 * dir + 1];
    const float kpoly_g = lim[8 + 2 * dir], kpoly_s = lim[8 + 2 * dir + 1];

    LaneState S[2];
#pragma unroll
    for (int h = 0; h < 2; h++) {
        S[h] = {0.0f, 0.0f, 1.0f, 0.0f, 0.0f, 1.0f};
        const int lane = tid + 64 * h;       // (column jl + 8 h, pair p) in the order of the summaries and start states
        if (c > 0 && __builtin_amdgcn_readfirstlane(*pl.contracted) != 0) {
            const float* sm = pl.summaries + (size_t)(dir * pl.wchunks + pl.wchunk_prefix[ti] + c - 1) * 6 * LANES;
            S[h].he = sm[4 * LANES + lane];
            S[h].ho = sm[5 * LANES + lane];
        } else {
            const float* hs = pl.hstart + ((size_t)(dir * pl.chunks + cidx) * 2) * LANES;
            S[h].he = hs[lane];
            S[h].ho = hs[LANES + lane];
        }
    }

    uint32_t nx_key = 0;
    int32_t nx_val = 0;
    float nx_sh = 0.0f;
    auto load_inputs = [&](int tile0) {
        const int u = tile0 + tu;
        if (u < u1) {
            const int t = dir ? (N - 1 - u) : u;
            nx_key = skey[t];
            nx_val = sval[t];
            nx_sh = has_s ? ssrt[t] : 0.0f;
        }
    };
    load_inputs(u0);
    // The context row of a timestep leaves one tile late, after the next tile's inputs have arrived: the counter that
    // tells a wave that its loads have landed also counts its stores, in order, so a store issued just before that
    // wait would make every tile wait for a scattered write to be acknowledged.
    static_assert(DM == 8, "two 16-byte stores per lane");
    float4 held[2];
    float4* held_dst = nullptr;
    auto flush = [&]() {
        if (held_dst != nullptr) {
            held_dst[0] = held[0];
            held_dst[1] = held[1];
        }
    };
    for (int tile0 = u0; tile0 < u1; tile0 += SCAN_TT) {
        const int cnt = min(SCAN_TT, u1 - tile0);
        // ---------------- phase A: projections of SCAN_TT timesteps -> LDS (both halves of every output group)
        const uint32_t kbits = nx_key;
        const int32_t v = nx_val;
        const float shv = nx_sh;
        const bool valid = tile0 + tu < u1;
        asm volatile("" : : "v"(kbits), "v"(v), "v"(shv) : "memory");      // the wait for this tile's inputs goes here, before the stores
        flush();
        if (tile0 + SCAN_TT < u1) load_inputs(tile0 + SCAN_TT);
        int orig = v & 0x7fffffff;
        orig = ((unsigned)orig < (unsigned)N) ? orig : 0;   // never index outside the tensor
        const float g = valid ? sg_i2f((int32_t)kbits | (v & (int32_t)0x80000000)) : 0.0f;
        const float sh = valid ? shv : 0.0f;
        const unsigned long long notpoly = __builtin_amdgcn_ballot_w64(!sg2_poly_ok(kpoly_g, kpoly_s, g, sh));
        const unsigned long long notlin =
            __builtin_amdgcn_ballot_w64(!sg2_poly_ok(SG2_PROD_LINEAR_FACTOR * kpoly_g, SG2_PROD_LINEAR_FACTOR * kpoly_s, g, sh));
        const bool tay = __builtin_amdgcn_ballot_w64(!sg2_taylor_ok(cmax_g, cmax_s, g, sh)) == 0;
        const bool dgiven = tay && notpoly == 0 && cnt == SCAN_TT;
        unsigned long long large[2] = {0, 0}, nottiny[2] = {0, 0};
        float dxv[DI];           // D * x-branch, kept for phase C: of this lane's timestep, or (dgiven) of its column's 16 timesteps
        if (dgiven) {
            if (has_s) project_rows<G, true>(g, sh, tid, s_coef, s_tay, s_dt, s_ux, s_B, s_C, dxv);
            else project_rows<G, false>(g, sh, tid, s_coef, s_tay, s_dt, s_ux, s_B, s_C, dxv);
        } else {
            int angle[2];
            auto run = [&](auto has_s_c, auto tay_c) {
                constexpr bool HS = decltype(has_s_c)::value, TY = decltype(tay_c)::value;
                project_all<G, HS, TY>(g, sh, tu, s_coef, s_tay, s_fmax, s_dt, s_ux, s_B, s_C, dxv, angle);
            };
            if (tay) { if (has_s) run(std::true_type{}, std::true_type{}); else run(std::false_type{}, std::true_type{}); }
            else { if (has_s) run(std::true_type{}, std::false_type{}); else run(std::false_type{}, std::false_type{}); }
#pragma unroll
            for (int h = 0; h < 2; h++) {
                large[h] = __builtin_amdgcn_ballot_w64(!(angle[h] & 1));
                nottiny[h] = __builtin_amdgcn_ballot_w64(!(angle[h] & 2));
            }
        }
        __syncthreads();      // one wave: no s_barrier is issued, the LDS writes above are ordered before the reads below

        // ---------------- phase B: the recurrences of this lane's two columns over the tile
        const float* __restrict__ r_Be = s_B + (2 * p) * LDS_STRIDE;
        const float* __restrict__ r_Bo = s_B + (2 * p + 1) * LDS_STRIDE;
        const float* __restrict__ r_Ce = s_C + (2 * p) * LDS_STRIDE;
        const float* __restrict__ r_Co = s_C + (2 * p + 1) * LDS_STRIDE;
        int k0 = 0;
        if (dgiven) {
            // a whole tile on the lane polynomials (the usual case): both columns in one instruction stream
            float Be[UB], Bo[UB], Ce[UB], Co[UB], dt[2][UB], xv[2][UB];
            auto fetch = [&](int kb, float (&tBe)[UB], float (&tBo)[UB], float (&tCe)[UB], float (&tCo)[UB], float (&tdt)[2][UB], float (&tux)[2][UB]) {
#pragma unroll
                for (int q = 0; q < UB; q += 4) {
                    const f32x4 c4 = *reinterpret_cast<const f32x4*>(r_Be + kb + q), d4 = *reinterpret_cast<const f32x4*>(r_Bo + kb + q);
                    const f32x4 f4 = *reinterpret_cast<const f32x4*>(r_Ce + kb + q), g4 = *reinterpret_cast<const f32x4*>(r_Co + kb + q);
#pragma unroll
                    for (int e = 0; e < 4; e++) { tBe[q + e] = c4[e]; tBo[q + e] = d4[e]; tCe[q + e] = f4[e]; tCo[q + e] = g4[e]; }
#pragma unroll
                    for (int h = 0; h < 2; h++) {
                        const f32x4 a4 = *reinterpret_cast<const f32x4*>(s_dt + (jl + 8 * h) * LDS_STRIDE + kb + q);
                        const f32x4 b4 = *reinterpret_cast<const f32x4*>(s_ux + (jl + 8 * h) * LDS_STRIDE + kb + q);
#pragma unroll
                        for (int e = 0; e < 4; e++) { tdt[h][q + e] = a4[e]; tux[h][q + e] = b4[e]; }
                    }
                }
            };
            auto compute = [&](int kb, const float (&tBe)[UB], const float (&tBo)[UB], const float (&tCe)[UB], const float (&tCo)[UB],
                               const float (&tdt)[2][UB], const float (&tux)[2][UB]) {
                float y[2][UB];
                const unsigned long long blk = ((1ull << UB) - 1) << kb;
                if ((notlin & blk) == 0) block_steps_pair<HP, true>(S, tdt, tux, tBe, tBo, tCe, tCo, LP, y);
                else block_steps_pair<HP, false>(S, tdt, tux, tBe, tBo, tCe, tCo, LP, y);
                if ((p & 3) == 0) {      // the first lane of every bank holds the totals of its bank's steps (block_pair_sums)
                    *reinterpret_cast<f32x4*>(&s_y[jl * LDS_STRIDE + kb + 4 * (p >> 2)]) = f32x4{y[0][0], y[0][1], y[0][2], y[0][3]};
                    *reinterpret_cast<f32x4*>(&s_y[(jl + 8) * LDS_STRIDE + kb + 4 * (p >> 2)]) = f32x4{y[1][0], y[1][1], y[1][2], y[1][3]};
                }
            };
#pragma unroll 1
            for (; k0 < SCAN_TT; k0 += UB) {
                fetch(k0, Be, Bo, Ce, Co, dt, xv);
                compute(k0, Be, Bo, Ce, Co, dt, xv);
            }
        }
        for (; k0 + UB <= cnt; k0 += UB) {
            float Be[UB], Bo[UB], Ce[UB], Co[UB];
#pragma unroll
            for (int q = 0; q < UB; q += 4) {
                const f32x4 c4 = *reinterpret_cast<const f32x4*>(r_Be + k0 + q), d4 = *reinterpret_cast<const f32x4*>(r_Bo + k0 + q);
                const f32x4 f4 = *reinterpret_cast<const f32x4*>(r_Ce + k0 + q), g4 = *reinterpret_cast<const f32x4*>(r_Co + k0 + q);
#pragma unroll
                for (int e = 0; e < 4; e++) { Be[q + e] = c4[e]; Bo[q + e] = d4[e]; Ce[q + e] = f4[e]; Co[q + e] = g4[e]; }
            }
            const unsigned long long blk = ((1ull << UB) - 1) << k0;
#pragma unroll
            for (int h = 0; h < 2; h++) {
                const int j = jl + 8 * h;
                float dt[UB], xv[UB], y[UB];
#pragma unroll
                for (int q = 0; q < UB; q += 4) {
                    const f32x4 a4 = *reinterpret_cast<const f32x4*>(s_dt + j * LDS_STRIDE + k0 + q), b4 = *reinterpret_cast<const f32x4*>(s_ux + j * LDS_STRIDE + k0 + q);
#pragma unroll
                    for (int e = 0; e < 4; e++) { dt[q + e] = a4[e]; xv[q + e] = b4[e]; }
                }
                if (dgiven && (notlin & blk) == 0)
                    block_steps<HP, OUT, 3, false, true, true>(S[h], dt, xv, Be, Bo, Ce, Co, 0.0f, 0.0f, 0.0f, LP[h], y);
                else if (dgiven)
                    block_steps<HP, OUT, 3, false, true>(S[h], dt, xv, Be, Bo, Ce, Co, 0.0f, 0.0f, 0.0f, LP[h], y);
                else if ((notpoly & blk) == 0)
                    block_steps<HP, OUT, 3, false>(S[h], dt, xv, Be, Bo, Ce, Co, 0.0f, 0.0f, 0.0f, LP[h], y);
                else if ((nottiny[h] & blk) == 0)
                    block_steps<HP, OUT, 2, false>(S[h], dt, xv, Be, Bo, Ce, Co, pole_e(h), pole_o(h), rope_f(h), LP[h], y);
                else if ((large[h] & blk) == 0)
                    block_steps<HP, OUT, 1, false>(S[h], dt, xv, Be, Bo, Ce, Co, pole_e(h), pole_o(h), rope_f(h), LP[h], y);
                else
                    block_steps<HP, OUT, 0, false>(S[h], dt, xv, Be, Bo, Ce, Co, pole_e(h), pole_o(h), rope_f(h), LP[h], y);
                if ((p & 3) == 0)        // the first lane of every bank holds the totals of its bank's steps (block_pair_sums)
                    *reinterpret_cast<f32x4*>(&s_y[j * LDS_STRIDE + k0 + 4 * (p >> 2)]) = f32x4{y[0], y[1], y[2], y[3]};
            }
        }
        for (; k0 < cnt; k0++) {       // ragged end of the last tile of a tensor
#pragma unroll
            for (int h = 0; h < 2; h++) {
                const int j = jl + 8 * h;
                const float dt = s_dt[j * LDS_STRIDE + k0], ux = s_ux[j * LDS_STRIDE + k0];
                float ae, ao, sn, cs;
                sg_abar_pair(dt, pole_e(h), pole_o(h), &ae, &ao);
                sg_sincos(dt * rope_f(h), &sn, &cs);
                step_update<OUT>(S[h], ae, ao, sn, cs, ux * r_Be[k0], ux * r_Bo[k0]);
                const float y = pair_tree_sum<HP>(sg_fma(S[h].ho, r_Co[k0], S[h].he * r_Ce[k0]));
                if (p == 0) s_y[j * LDS_STRIDE + k0] = y;
            }
        }
        __syncthreads();

        // ---------------- phase C: gate, D skip, out_proj, scatter to element order (one 32-byte row per lane)
        {
            float o[DI];
            if (dgiven) {        // the row owners gate their 16 outputs in place, then every timestep collects its 16 columns
                if (has_s) gate_rows<G, true>(tid, s_coef, s_tay, s_B, s_C, s_y, dxv);
                else gate_rows<G, false>(tid, s_coef, s_tay, s_B, s_C, s_y, dxv);
                __syncthreads();
#pragma unroll
                for (int jj = 0; jj < DI; jj++) o[jj] = s_y[jj * LDS_STRIDE + tu];
            } else {
                if (tay) { if (has_s) gates_all<G, true, true>(g, sh, s_coef, s_tay, o); else gates_all<G, false, true>(g, sh, s_coef, s_tay, o); }
                else { if (has_s) gates_all<G, true, false>(g, sh, s_coef, s_tay, o); else gates_all<G, false, false>(g, sh, s_coef, s_tay, o); }
#pragma unroll
                for (int jj = 0; jj < DI; jj++) o[jj] = sg_fma(s_y[jj * LDS_STRIDE + tu], o[jj], dxv[jj]);
            }
            // out_proj on the matrix pipe: v_mfma_f32_4x4x1_16b is one fused multiply-add per output and step, so 16 of them
            // in the order of the columns are the fmaf chain of the scalar form, bit for bit.  Block b of the instruction
            // is timesteps 4 b .. 4 b + 3: the lane of a timestep supplies its gated output as the B operand and receives
            // its own four outputs; the A operand of lane l is row l % 4 of out_proj (rows 4 .. 7 for the second chain).
            static_assert(DM == 8 && DI % 4 == 0, "two chains of four output rows");
            f32x4 lo = {0.0f, 0.0f, 0.0f, 0.0f}, hi = {0.0f, 0.0f, 0.0f, 0.0f};
            const float* wlo = s_wout + (tid & 3) * DI;
            const float* whi = s_wout + (4 + (tid & 3)) * DI;
#pragma unroll
            for (int m = 0; m < DI; m += 4) {
                const f32x4 wa = *reinterpret_cast<const f32x4*>(wlo + m), wb = *reinterpret_cast<const f32x4*>(whi + m);
#pragma unroll
                for (int e = 0; e < 4; e++) {
                    lo = __builtin_amdgcn_mfma_f32_4x4x1f32(wa[e], o[m + e], lo, 0, 0, 0);
                    hi = __builtin_amdgcn_mfma_f32_4x4x1f32(wb[e], o[m + e], hi, 0, 0, 0);
                }
            }
            const float cx[DM] = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
            held_dst = valid ? reinterpret_cast<float4*>(pl.ctx + ((size_t)dir * pl.total + off + orig) * DM) : nullptr;
            held[0] = make_float4(cx[0], cx[1], cx[2], cx[3]);
            held[1] = make_float4(cx[4], cx[5], cx[6], cx[7]);
        }
        __syncthreads();
    }
    flush();
    if (u1 == N) {   // last chunk in scan order: new carried state of the tensor
        float* st = dir ? T.mbwd : T.mfwd;
#pragma unroll
        for (int h = 0; h < 2; h++) {
            const int j = jl + 8 * h;
            if (j < pl.st_di && 2 * p < pl.st_ds) {
                st[j * pl.st_ds + 2 * p] = S[h].he;
                st[j * pl.st_ds + 2 * p + 1] = S[h].ho;
            }
        }
    }
}

// Start state of every chunk: h_{c+1} = M_c h_c + b_c, applied in order from
// the carried state of the tensor.  One workgroup per (tensor, direction).
// The recurrence itself is a handful of fmas per chunk; what matters is the
// latency of fetching 3 KB (12 KB for the large geometry) of summaries per chunk,
// so the 1024 lanes of the workgroup, as groups of one chunk's lanes each, stream
// batches of chunks into LDS (next batch prefetched into registers) and group 0
// applies them.
constexpr int PREFIX_PER_GROUP = 4;

template <class G>
__global__ __launch_bounds__(1024) void k_chunk_prefix(Plan pl) {
    constexpr int HP = G::HP, SCAN_THREADS = G::THREADS;
    constexpr int PREFIX_GROUPS = 1024 / SCAN_THREADS;             // 8 groups of 128 lanes, or 2 of 512
    constexpr int PREFIX_BATCH = PREFIX_PER_GROUP * PREFIX_GROUPS;
    __shared__ float lds[PREFIX_BATCH * 6 * SCAN_THREADS];     // 96 KB
    const int ti = blockIdx.x % pl.P, dir = blockIdx.x / pl.P;
    const TensorDev& T = pl.tensors[ti];
    if (T.numel == 0) return;
    const int lane = threadIdx.x % SCAN_THREADS, grp = threadIdx.x / SCAN_THREADS;
    const int j = lane / HP, p = lane % HP;
    float* __restrict__ hs = pl.hstart + ((size_t)(dir * pl.chunks + pl.chunk_prefix[ti]) * 2) * SCAN_THREADS;
    const float* __restrict__ sm = pl.summaries + (size_t)(dir * pl.wchunks + pl.wchunk_prefix[ti]) * 6 * SCAN_THREADS;
    const int ns = T.nchunks - 1;                               // summaries to apply
    float he = 0.0f, ho = 0.0f;
    if (grp == 0) {
        // the caller's state is [st_di][st_ds] (its own d_inner, d_state); the rest of the kernel geometry starts at 0
        const float* st = dir ? T.mbwd : T.mfwd;
        if (j < pl.st_di && 2 * p < pl.st_ds) {
            he = st[j * pl.st_ds + 2 * p];
            ho = st[j * pl.st_ds + 2 * p + 1];
        }
        hs[lane] = he;
        hs[SCAN_THREADS + lane] = ho;
    }
    // every summary has an exactly zero 2x2 part: the replay takes its start states from the summaries themselves
    if (__builtin_amdgcn_readfirstlane(*pl.contracted) != 0) return;
    float r[PREFIX_PER_GROUP][6];
    auto prefetch = [&](int b) {
#pragma unroll
        for (int q = 0; q < PREFIX_PER_GROUP; q++) {
            const int c = b * PREFIX_BATCH + grp + PREFIX_GROUPS * q;
#pragma unroll
            for (int k = 0; k < 6; k++) r[q][k] = (c < ns) ? sm[((size_t)c * 6 + k) * SCAN_THREADS + lane] : 0.0f;
        }
    };
    prefetch(0);
    for (int b = 0; b * PREFIX_BATCH < ns; b++) {
#pragma unroll
        for (int q = 0; q < PREFIX_PER_GROUP; q++)
#pragma unroll
            for (int k = 0; k < 6; k++) lds[((grp + PREFIX_GROUPS * q) * 6 + k) * SCAN_THREADS + lane] = r[q][k];
        __syncthreads();
        prefetch(b + 1);
        if (grp == 0) {
            const int lim = min(PREFIX_BATCH, ns - b * PREFIX_BATCH);
            for (int cc = 0; cc < lim; cc++) {
                const float* m = lds + cc * 6 * SCAN_THREADS + lane;
                // a lane whose 2x2 part is exactly zero takes the offset itself, which is what 0 * h + b is for every finite h;
                // a state that is not finite goes through the product and stays non-finite to the end of the tensor
                const bool zero = m[0] == 0.0f && m[SCAN_THREADS] == 0.0f && m[2 * SCAN_THREADS] == 0.0f && m[3 * SCAN_THREADS] == 0.0f &&
                                  sg_isfinite(he) && sg_isfinite(ho);
                const float ne = sg_fma(m[0], he, sg_fma(m[2 * SCAN_THREADS], ho, m[4 * SCAN_THREADS]));
                const float no = sg_fma(m[SCAN_THREADS], he, sg_fma(m[3 * SCAN_THREADS], ho, m[5 * SCAN_THREADS]));
                he = zero ? m[4 * SCAN_THREADS] : ne;
                ho = zero ? m[5 * SCAN_THREADS] : no;
                float* h1 = hs + (size_t)(b * PREFIX_BATCH + cc + 1) * 2 * SCAN_THREADS;
                h1[lane] = he;
                h1[SCAN_THREADS + lane] = ho;
            }
        }
        __syncthreads();
    }
}

template <class G>
int launch_scan_geo(const Plan& pl, hipStream_t st) {
    hipLaunchKernelGGL(k_compose<G>, dim3(1), dim3(2 * SG2_COMP_GROUPS * G::ROWS), 0, st, pl);
    SG_LAUNCH_CHECK("k_compose");
    if (pl.wchunks > 0) {
        hipLaunchKernelGGL((k_scan<G, false, false>), dim3(2 * pl.wchunks), dim3(G::THREADS), 0, st, pl);
        SG_LAUNCH_CHECK("k_scan<summary>");
    }
    prof_mark(2, st);
    hipLaunchKernelGGL(k_chunk_prefix<G>, dim3(2 * pl.P), dim3(1024), 0, st, pl);
    SG_LAUNCH_CHECK("k_chunk_prefix");
    prof_mark(3, st);
    if constexpr (G::PARTS == 2) {
        if (pl.htile != nullptr) {
            hipLaunchKernelGGL((k_scan<G, true, true>), dim3(2 * pl.chunks), dim3(G::THREADS), 0, st, pl);
            SG_LAUNCH_CHECK("k_scan<out, keep>");
            prof_mark(4, st);
            return 0;
        }
    }
    if (pl.htile != nullptr) return sg::fail("the bilevel pass is built for the default meta-net dimensions only");
    if constexpr (G::PARTS == 2) {          // one wave per chunk, two columns per lane
        hipLaunchKernelGGL(k_replay<G>, dim3(2 * pl.chunks), dim3(64), 0, st, pl);
        SG_LAUNCH_CHECK("k_replay");
    } else {
        hipLaunchKernelGGL((k_scan<G, true, false>), dim3(2 * pl.chunks), dim3(G::THREADS), 0, st, pl);
        SG_LAUNCH_CHECK("k_scan<out>");
    }
    prof_mark(4, st);
    return 0;
}

}  // namespace

int launch_scan(const Plan& pl, hipStream_t st) {
    if (pl.total == 0) return 0;
    return pl.geo == GEO_LARGE ? launch_scan_geo<GeoLarge>(pl, st) : launch_scan_geo<GeoDefault>(pl, st);
}

}  // namespace sg2
