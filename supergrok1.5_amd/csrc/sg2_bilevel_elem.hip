// Per-element part of the bilevel meta-net update of SuperGrok v2, forward and backward in one pass: GRU, soft
// top-4 product-key routing (softmax of 10 x the four best scores of each sub-key, 16 experts per head), expert
// MLPs and the skip connection, followed at once by the gradients of  sum_i cot_i * smart_i  with respect to the
// two scan contexts of every element and to every weight of this part.
//
// Stands in for the per-element kernels of launch_mamba3_peer_backward[_batched]
// (csrc/supergrok2_mamba_peer_backward_kernels.cu of the reference, driven from
// grokking_optimizers/supergrok2.py:516-1330); the arithmetic is that of Mamba3PEERMetaNet.forward_for_bilevel
// (grokking_optimizers/mamba3_peer_metanet.py:395-436) and its autograd derivative.
//
// One lane per element, persistent grid over tiles of 256 elements, one 256-lane workgroup per CU.  Nothing is kept
// between forward and backward: a lane holds its element's activations in registers, and the routing of a head is
// differentiated before the next head is evaluated.  Weight gradients are sums over elements:
//   * experts (16 per element and head, chosen per element).  An expert's hidden unit m is active where
//     W1[m] g + b1[m] > 0, i.e. on one side of the threshold -b1[m] / W1[m], so between two neighbouring thresholds of
//     its 16 units the expert is a straight line  out = A g + B.  Each workgroup sorts the thresholds of every expert
//     once and tabulates (A, B) for the 17 intervals; an element then finds its interval with five LDS reads and
//     evaluates the expert with one fma, instead of reading the expert's 49 weights.  The gradients of expert e need,
//     per unit, S0 = sum w [unit active] and S1 = sum w g [unit active] over the elements routed to e (w: routing
//     weight times d loss / d head), i.e. sums of (w, w g) per interval.  Small gradients lie in the interval next to
//     g = 0 on their side of it for every expert; for those the sums over elements are outer products (first sub-key
//     weights) (x) (second sub-key weights), which every wave accumulates for its 64 elements with fp32 matrix
//     instructions in registers (16 x 16 x 4: four elements a step), separately for g > 0 and g <= 0.  An element in
//     any other interval of one of its experts moves its (w, w g) there with LDS float atomics (about 3 clocks a lane,
//     which is why they are kept for the exceptions).  S0, S1 of a unit are the sums of the bins on the unit's active
//     side, formed once when the workgroup is done.
//     (An element exactly on a threshold counts the unit as inactive on both sides; forward value and gradient use
//     the same interval, so they stay consistent.)
//   * GRU and query matrices (dense outer products d (x) x): every lane leaves its x (31 values) and, per head
//     and once more for the GRU, its d (8 / 12 values) in LDS; each lane of the workgroup owns one entry of the
//     head's query matrix and up to two of the GRU matrices and sums their products over the tile's elements;
//   * product keys (rows chosen per element): the same, with d score scattered into a 12-vector per sub-key.
// Each workgroup writes its sums to its own row of a partials buffer; a second kernel adds the rows in a fixed
// order.  The dense, key and near-zero expert sums are formed in a fixed order; the other expert bins are filled by
// atomics of four waves, so where gradients reach beyond the intervals next to zero the last bits of the expert
// gradients can differ from run to run (as with the reference's atomicAdd).
#include "sg2_internal.hpp"

namespace sg2 {
namespace {

constexpr int BE_THREADS = 256;         // four waves; the LDS tables leave room for one workgroup per CU
constexpr int BE_WAVES = BE_THREADS / 64;
constexpr int TOPK = 4;
constexpr int RH = 16;                  // a staged 12-vector is padded to 16 entries (zeros): one operand row of a 16 x 16 x 4 matrix instruction
constexpr int RW = 2 * RH + 1;          // staged row of a head: first-index vector at 0, second-index vector at RH (odd stride: consecutive rows hit all banks)
static_assert(PK <= RH, "a sub-key vector fits its padded half row");
typedef float be_f32x4 __attribute__((ext_vector_type(4)));
constexpr int NBIN = EH + 1;            // intervals between an expert's sorted unit thresholds
static_assert(EH == 16, "the interval search takes steps of 8, 4, 2, 1 and one more");
constexpr int XW = 31, DW = 13;         // row strides of the staged x and d vectors (odd: lane-consecutive rows hit all banks)
// x row: g, s, fwd ctx[8], bwd ctx[8], h_old[4], r*h_old[4], h_new[4], 1
constexpr int X_G = 0, X_S = 1, X_CF = 2, X_CB = 10, X_H = 18, X_RH = 22, X_HN = 26, X_ONE = 30;
// d row, reused: d query[8] of the current head, then d pre_z[4], d pre_r[4], d pre_h[4] of the GRU
constexpr int D_Z = 0, D_R = 4, D_H = 8;
constexpr int N_GRU = 3 * (GH * GRL + GH), N_QHEAD = DM * PIN;     // 276 GRU entries, 176 query entries per head
constexpr int N_DENSE = N_GRU + NH * N_QHEAD;                      // 276 + 704
constexpr int OFF_KA = N_DENSE, OFF_KB = OFF_KA + NH * PK * (DM / 2);
constexpr int OFF_W1 = OFF_KB + NH * PK * (DM / 2), OFF_B1 = OFF_W1 + NE * EH, OFF_W2 = OFF_B1 + NE * EH, OFF_B2 = OFF_W2 + NE * EH;
constexpr int N_GRADS = OFF_B2 + NE;
static_assert(N_GRADS == SG2_ELEM_GRAD_FLOATS, "gradient layout");
constexpr int GRU_PER_LANE = (N_GRU + BE_THREADS - 1) / BE_THREADS, Q_PER_LANE = (N_QHEAD + BE_THREADS - 1) / BE_THREADS;

// (column of d, column of x) whose products make up GRU gradient entry o, in the order
// W_z[4][22] b_z[4] W_r[4][22] b_r[4] W_h[4][22] b_h[4]
__device__ __forceinline__ void gru_entry(int o, int* dcol, int* xcol) {
    const int gate = o / (GH * GRL + GH), q = o % (GH * GRL + GH);
    if (q >= GH * GRL) { *dcol = gate * GH + (q - GH * GRL); *xcol = X_ONE; return; }
    const int j = q / GRL, c = q % GRL;
    *dcol = gate * GH + j;
    *xcol = (gate == 2 && c >= 2 + 2 * DM) ? X_RH + (c - 2 - 2 * DM) : c;     // the candidate sees r*h in place of h
}
// same for entry o = r*22 + c of a head's query matrix [8][22]; query input = h_new, fwd ctx, bwd ctx, g, s
__device__ __forceinline__ void query_entry(int o, int* dcol, int* xcol) {
    const int c = o % PIN;
    *dcol = o / PIN;
    *xcol = c < GH ? X_HN + c : (c < GH + 2 * DM ? X_CF + (c - GH) : (c == GH + 2 * DM ? X_G : X_S));
}

// Is the hidden unit (w1, b1), whose threshold is the rank-th lowest of its expert, active on interval k (the k lowest
// thresholds lie below g)?  W1 > 0: above its threshold; W1 < 0: below it; W1 = 0: wherever b1 > 0.
__device__ __forceinline__ bool unit_active(float w1, float b1, int rank, int k) {
    return w1 > 0.0f ? rank < k : (w1 < 0.0f ? rank >= k : b1 > 0.0f);
}

struct ElemArgs {
    const float *g, *s, *ctx, *gru, *cot;
    float *smart, *d_ctx, *partials, *gru_out;
    int total;
    float rescale;
    Sg2Weights W;
};

__global__ __launch_bounds__(BE_THREADS) void k_bilevel_elem(ElemArgs a) {
    extern __shared__ __attribute__((aligned(16))) float lds[];
    float* s_ths = lds;                                   // [NE][EH] unit thresholds of every expert, ascending
    float* s_ab = s_ths + NE * EH;                        // [NE][NBIN][2] the expert as a line A g + B on each interval
    float* s_bin = s_ab + NE * NBIN * 2;                  // [NE][NBIN][2] sums of w and w g over the elements of each interval
    float* s_gkey = s_bin + NE * NBIN * 2;                // [2][NH][PK][DM/2]
    float* s_x = s_gkey + 2 * NH * PK * (DM / 2);         // [256][XW]
    float* s_d = s_x + BE_THREADS * XW;                   // [256][DW]
    float* s_rt = s_d + BE_THREADS * DW;                  // [256][RW]
    float* s_gq = s_rt + BE_THREADS * RW;                 // [NH][8][22] query-matrix gradients of this workgroup
    unsigned char* s_rank = reinterpret_cast<unsigned char*>(s_gq + NH * N_QHEAD);      // [NE][EH] position of a unit's threshold among its expert's
    unsigned char* s_kz = s_rank + NE * EH;               // [NE][2] the interval just below / just above g = 0: thresholds < 0, thresholds <= 0

    const int tid = threadIdx.x;
    {
        const float* __restrict__ W1 = a.W.w[W_EXP_W1];
        const float* __restrict__ B1 = a.W.w[W_EXP_B1];
        const float* __restrict__ W2 = a.W.w[W_EXP_W2];
        const float* __restrict__ B2 = a.W.w[W_EXP_B2];
        for (int i = tid; i < 2 * NH * PK * (DM / 2); i += BE_THREADS) s_gkey[i] = 0.0f;
        for (int i = tid; i < NH * N_QHEAD; i += BE_THREADS) s_gq[i] = 0.0f;
        for (int i = tid; i < NE * NBIN * 2; i += BE_THREADS) s_bin[i] = 0.0f;
        for (int i = tid; i < BE_THREADS * RW; i += BE_THREADS) s_rt[i] = 0.0f;      // the padding entries stay zero
        // one lane per expert: thresholds ranked by counting (ties by unit index), then the line of every interval.
        // A unit with W1 = 0 has no threshold (+inf, never passed): it is active or not by the sign of b1 alone.
        for (int e = tid; e < NE; e += BE_THREADS) {
            const float* w1 = W1 + e * EH;
            const float* b1 = B1 + e * EH;
            const float* w2 = W2 + e * EH;
            auto thr = [&](int m) { return w1[m] != 0.0f ? -b1[m] / w1[m] : __builtin_inff(); };
            int below = 0, upto = 0;
            for (int m = 0; m < EH; m++) {
                const float tm = thr(m);
                below += tm < 0.0f ? 1 : 0;
                upto += tm <= 0.0f ? 1 : 0;
                int r = 0;
                for (int j = 0; j < EH; j++) {
                    const float tj = thr(j);
                    r += (tj < tm || (tj == tm && j < m)) ? 1 : 0;
                }
                s_rank[e * EH + m] = (unsigned char)r;
                s_ths[e * EH + r] = tm;
            }
            s_kz[2 * e] = (unsigned char)below;
            s_kz[2 * e + 1] = (unsigned char)upto;
            for (int k = 0; k < NBIN; k++) {        // interval k: the k lowest thresholds lie below g
                float A = 0.0f, B = B2[e];
                for (int m = 0; m < EH; m++) {
                    if (!unit_active(w1[m], b1[m], (int)s_rank[e * EH + m], k)) continue;
                    A = sg_fma(w2[m], w1[m], A);
                    B = sg_fma(w2[m], b1[m], B);
                }
                s_ab[(e * NBIN + k) * 2] = A;
                s_ab[(e * NBIN + k) * 2 + 1] = B;
            }
        }
    }
    __syncthreads();

    const sg::cfloat_p Wz = sg::as_const(a.W.w[W_GRU_WZ]), bz = sg::as_const(a.W.w[W_GRU_BZ]);
    const sg::cfloat_p Wr = sg::as_const(a.W.w[W_GRU_WR]), br = sg::as_const(a.W.w[W_GRU_BR]);
    const sg::cfloat_p Wh = sg::as_const(a.W.w[W_GRU_WH]), bh = sg::as_const(a.W.w[W_GRU_BH]);
    const sg::cfloat_p Wq = sg::as_const(a.W.w[W_PEER_Q]);
    const sg::cfloat_p KA = sg::as_const(a.W.w[W_KEYS_A]), KB = sg::as_const(a.W.w[W_KEYS_B]);

    // the lane's entries of the GRU gradients (sums kept in registers) and of a head's query matrix (summed per
    // tile and head, then added to s_gq)
    int gdcol[GRU_PER_LANE], gxcol[GRU_PER_LANE], qdcol[Q_PER_LANE], qxcol[Q_PER_LANE];
    float gsum[GRU_PER_LANE];
#pragma unroll
    for (int q = 0; q < GRU_PER_LANE; q++) {
        gdcol[q] = 0; gxcol[q] = 0; gsum[q] = 0.0f;
        if (tid + q * BE_THREADS < N_GRU) gru_entry(tid + q * BE_THREADS, &gdcol[q], &gxcol[q]);
    }
#pragma unroll
    for (int q = 0; q < Q_PER_LANE; q++) {
        qdcol[q] = 0; qxcol[q] = 0;
        if (tid + q * BE_THREADS < N_QHEAD) query_entry(tid + q * BE_THREADS, &qdcol[q], &qxcol[q]);
    }

    // near-zero expert sums of this wave (the heads share the experts): sum of w for g > 0, for g <= 0, sum of w g for
    // g > 0, for g <= 0, each a 16 x 16 (first index x second index) accumulator of the matrix instruction
    be_f32x4 cen[4];
#pragma unroll
    for (int q = 0; q < 4; q++) cen[q] = be_f32x4{0.0f, 0.0f, 0.0f, 0.0f};
    const int tiles = (a.total + BE_THREADS - 1) / BE_THREADS;
    const float kscale = a.rescale / (float)NH;
    for (int tile = blockIdx.x; tile < tiles; tile += gridDim.x) {
        // every lane runs the element code (the passes over the tile need whole workgroups): lanes past the end redo
        // the last element with a zero cotangent, which zeroes everything they add, and store nothing
        const bool valid = tile * BE_THREADS + tid < a.total;
        const int i = valid ? tile * BE_THREADS + tid : a.total - 1;
        float* xrow = s_x + tid * XW;
        float* drow = s_d + tid * DW;
        float* rtrow = s_rt + tid * RW;
        {
            const float g = a.g[i], s = a.s[i], cot = valid ? a.cot[i] : 0.0f;
            float cf[DM], cb[DM], h[GH];
            {
                const float4* pf = reinterpret_cast<const float4*>(a.ctx + (size_t)i * DM);
                const float4* pb = reinterpret_cast<const float4*>(a.ctx + ((size_t)a.total + i) * DM);
                const float4 a0 = pf[0], a1 = pf[1], b0 = pb[0], b1 = pb[1];
                cf[0] = a0.x; cf[1] = a0.y; cf[2] = a0.z; cf[3] = a0.w; cf[4] = a1.x; cf[5] = a1.y; cf[6] = a1.z; cf[7] = a1.w;
                cb[0] = b0.x; cb[1] = b0.y; cb[2] = b0.z; cb[3] = b0.w; cb[4] = b1.x; cb[5] = b1.y; cb[6] = b1.z; cb[7] = b1.w;
                const float4 h4 = reinterpret_cast<const float4*>(a.gru)[i];
                h[0] = h4.x; h[1] = h4.y; h[2] = h4.z; h[3] = h4.w;
            }
            // (a zero the compiler cannot see through where the wave-uniform weights are used keeps their scalar loads there;
            //  held across the whole element they are spilled into vector-register lanes and read back, 3000 instructions)
            const int zo_gf = sg::opaque_zero();
            // ---- GRU forward
            float zg[GH], rg[GH], cand[GH], hn[GH];
#pragma unroll
            for (int j = 0; j < GH; j++) {
                const sg::cfloat_p wz = Wz + j * GRL + zo_gf, wr = Wr + j * GRL + zo_gf;
                float vz = bz[j], vr = br[j];
                vz = sg_fma(wz[0], g, vz); vz = sg_fma(wz[1], s, vz);
                vr = sg_fma(wr[0], g, vr); vr = sg_fma(wr[1], s, vr);
#pragma unroll
                for (int q = 0; q < DM; q++) { vz = sg_fma(wz[2 + q], cf[q], vz); vr = sg_fma(wr[2 + q], cf[q], vr); }
#pragma unroll
                for (int q = 0; q < DM; q++) { vz = sg_fma(wz[2 + DM + q], cb[q], vz); vr = sg_fma(wr[2 + DM + q], cb[q], vr); }
#pragma unroll
                for (int q = 0; q < GH; q++) { vz = sg_fma(wz[2 + 2 * DM + q], h[q], vz); vr = sg_fma(wr[2 + 2 * DM + q], h[q], vr); }
                zg[j] = sg_sigmoid(vz);
                rg[j] = sg_sigmoid(vr);
            }
#pragma unroll
            for (int j = 0; j < GH; j++) {
                const sg::cfloat_p wh = Wh + j * GRL + zo_gf;
                float v = bh[j];
                v = sg_fma(wh[0], g, v); v = sg_fma(wh[1], s, v);
#pragma unroll
                for (int q = 0; q < DM; q++) v = sg_fma(wh[2 + q], cf[q], v);
#pragma unroll
                for (int q = 0; q < DM; q++) v = sg_fma(wh[2 + DM + q], cb[q], v);
#pragma unroll
                for (int q = 0; q < GH; q++) v = sg_fma(wh[2 + 2 * DM + q], rg[q] * h[q], v);
                cand[j] = sg_tanh(v);
                hn[j] = sg_fma(zg[j], cand[j], (1.0f - zg[j]) * h[j]);
            }
            if (valid && a.gru_out != nullptr) reinterpret_cast<float4*>(a.gru_out)[i] = make_float4(hn[0], hn[1], hn[2], hn[3]);
            xrow[X_G] = g; xrow[X_S] = s; xrow[X_ONE] = 1.0f;
#pragma unroll
            for (int q = 0; q < DM; q++) { xrow[X_CF + q] = cf[q]; xrow[X_CB + q] = cb[q]; }
#pragma unroll
            for (int q = 0; q < GH; q++) { xrow[X_H + q] = h[q]; xrow[X_RH + q] = rg[q] * h[q]; xrow[X_HN + q] = hn[q]; }

            // ---- heads: forward, then at once the head's backward
            float total = 0.0f;
            float dhn[GH] = {0.f, 0.f, 0.f, 0.f}, dcf[DM], dcb[DM];
#pragma unroll
            for (int q = 0; q < DM; q++) { dcf[q] = 0.0f; dcb[q] = 0.0f; }
            const float kk = cot * kscale;                 // d loss / d head output
#pragma unroll 1
            for (int hh = 0; hh < NH; hh++) {
                const int zo_q = sg::opaque_zero();
                float query[DM];
#pragma unroll
                for (int dd = 0; dd < DM; dd++) {
                    const sg::cfloat_p qr = Wq + (hh * DM + dd) * PIN + zo_q;
                    float v = 0.0f;
#pragma unroll
                    for (int q = 0; q < GH; q++) v = sg_fma(qr[q], hn[q], v);
#pragma unroll
                    for (int q = 0; q < DM; q++) v = sg_fma(qr[GH + q], cf[q], v);
#pragma unroll
                    for (int q = 0; q < DM; q++) v = sg_fma(qr[GH + DM + q], cb[q], v);
                    v = sg_fma(qr[GH + 2 * DM], g, v);
                    v = sg_fma(qr[GH + 2 * DM + 1], s, v);
                    query[dd] = v;
                }
                int idx[2][TOPK];
                float wgt[2][TOPK];
#pragma unroll
                for (int hf = 0; hf < 2; hf++) {
                    const sg::cfloat_p keys = (hf ? KB : KA) + hh * PK * (DM / 2) + zo_q;
                    float sc[PK];
#pragma unroll
                    for (int q = 0; q < PK; q++) {
                        float dot = 0.0f;
#pragma unroll
                        for (int dd = 0; dd < DM / 2; dd++) dot = sg_fma(query[hf * (DM / 2) + dd], keys[q * (DM / 2) + dd], dot);
                        sc[q] = dot;
                    }
                    // four best scores, ties to the lower index; softmax of 10 x score over them
                    float val[TOPK];
                    unsigned taken = 0u;
#pragma unroll
                    for (int k = 0; k < TOPK; k++) {
                        int bi = 0;
                        float bs = -3.0e38f;
#pragma unroll
                        for (int q = 0; q < PK; q++) {
                            const bool free_ = ((taken >> q) & 1u) == 0u;
                            if (free_ && sc[q] > bs) { bs = sc[q]; bi = q; }
                        }
                        taken |= 1u << bi;
                        idx[hf][k] = bi;
                        val[k] = bs;
                    }
                    float den = 0.0f;
#pragma unroll
                    for (int k = 0; k < TOPK; k++) { wgt[hf][k] = sg_exp(10.0f * (val[k] - val[0])); den += wgt[hf][k]; }
                    const float inv = 1.0f / den;
#pragma unroll
                    for (int k = 0; k < TOPK; k++) wgt[hf][k] *= inv;
                }
                // experts: outputs per lane; each expert's bin of this element's activation pattern takes (w, w g)
                float ra[TOPK] = {0.f, 0.f, 0.f, 0.f}, rb[TOPK] = {0.f, 0.f, 0.f, 0.f};
                float head_out = 0.0f;
#pragma unroll 1
                for (int ia = 0; ia < TOPK; ia++) {
                    // the unrolled selects keep idx/wgt in registers (a dynamic index would send them to scratch); the four
                    // second indices are unrolled, so that the record reads of four experts are in flight together
                    const int ea = ia == 0 ? idx[0][0] : ia == 1 ? idx[0][1] : ia == 2 ? idx[0][2] : idx[0][3];
                    const float wa = ia == 0 ? wgt[0][0] : ia == 1 ? wgt[0][1] : ia == 2 ? wgt[0][2] : wgt[0][3];
                    float ra_sum = 0.0f;
                    int xbin[TOPK], xcen[TOPK];         // a pick outside the interval next to zero: its bin and that interval's, else -1
                    float xw[TOPK];
#pragma unroll
                    for (int ib = 0; ib < TOPK; ib++) {
                        const float wb = wgt[1][ib];
                        int e = ea * PK + idx[1][ib];
                        if (e >= NE) e = NE - 1;
                        const float* th = s_ths + e * EH;
                        int k = th[7] < g ? 8 : 0;              // how many of the expert's thresholds lie below g
                        k += th[k + 3] < g ? 4 : 0;
                        k += th[k + 1] < g ? 2 : 0;
                        k += th[k] < g ? 1 : 0;
                        k += th[k] < g ? 1 : 0;
                        const int bin = e * NBIN + k;
                        const float out = sg_fma(s_ab[2 * bin], g, s_ab[2 * bin + 1]);
                        const int kc = g > 0.0f ? s_kz[2 * e + 1] : s_kz[2 * e];
                        xbin[ib] = k != kc ? bin : -1;
                        xcen[ib] = e * NBIN + kc;
                        xw[ib] = (kk * wa) * wb;
                        head_out = sg_fma(wa * wb, out, head_out);
                        ra_sum = sg_fma(wb, out, ra_sum);
                        rb[ib] = sg_fma(wa, out, rb[ib]);
                    }
                    ra[0] += ia == 0 ? ra_sum : 0.0f; ra[1] += ia == 1 ? ra_sum : 0.0f; ra[2] += ia == 2 ? ra_sum : 0.0f; ra[3] += ia == 3 ? ra_sum : 0.0f;
                    // picks outside the interval next to zero move their share from there to their own bin; the wave skips
                    // this when none of its lanes has one (so the four interval searches above stay one straight block)
                    if (__builtin_amdgcn_ballot_w64(((xbin[0] & xbin[1]) & (xbin[2] & xbin[3])) >= 0) != 0) {
#pragma unroll
                        for (int ib = 0; ib < TOPK; ib++) {
                            if (xbin[ib] < 0) continue;
                            atomicAdd(&s_bin[2 * xbin[ib]], xw[ib]);
                            atomicAdd(&s_bin[2 * xbin[ib] + 1], xw[ib] * g);
                            atomicAdd(&s_bin[2 * xcen[ib]], -xw[ib]);
                            atomicAdd(&s_bin[2 * xcen[ib] + 1], -(xw[ib] * g));
                        }
                    }
                }
                // near-zero expert sums: this wave's 64 elements, four a step
#pragma unroll
                for (int k = 0; k < PK; k++) { rtrow[k] = 0.0f; rtrow[RH + k] = 0.0f; }
#pragma unroll
                for (int k = 0; k < TOPK; k++) {
                    rtrow[idx[0][k]] = kk * wgt[0][k];
                    rtrow[RH + idx[1][k]] = wgt[1][k];
                }
                __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
                __builtin_amdgcn_wave_barrier();
                {
                    const int li = tid & 15, el0 = (tid & ~63) + ((tid & 63) >> 4);
#pragma unroll 4
                    for (int t = 0; t < 16; t++) {
                        const int el = el0 + 4 * t;
                        const float av = s_rt[el * RW + li], bv = s_rt[el * RW + RH + li], gv = s_x[el * XW + X_G];
                        const float ap = gv > 0.0f ? av : 0.0f, an = gv > 0.0f ? 0.0f : av;
                        cen[0] = __builtin_amdgcn_mfma_f32_16x16x4f32(ap, bv, cen[0], 0, 0, 0);
                        cen[1] = __builtin_amdgcn_mfma_f32_16x16x4f32(an, bv, cen[1], 0, 0, 0);
                        cen[2] = __builtin_amdgcn_mfma_f32_16x16x4f32(ap * gv, bv, cen[2], 0, 0, 0);
                        cen[3] = __builtin_amdgcn_mfma_f32_16x16x4f32(an * gv, bv, cen[3], 0, 0, 0);
                    }
                }
                total += head_out;
                const int zo_rb = sg::opaque_zero();
                // routing backward: softmax, scores, query (the product keys' own gradients: see the end of the head)
                float dq[DM], dv[2][TOPK];
#pragma unroll
                for (int hf = 0; hf < 2; hf++) {
                    const sg::cfloat_p keys = (hf ? KB : KA) + hh * PK * (DM / 2) + zo_rb;
                    float mean = 0.0f;
#pragma unroll
                    for (int k = 0; k < TOPK; k++) mean = sg_fma(wgt[hf][k], kk * (hf ? rb[k] : ra[k]), mean);
#pragma unroll
                    for (int dd = 0; dd < DM / 2; dd++) dq[hf * (DM / 2) + dd] = 0.0f;
#pragma unroll
                    for (int k = 0; k < TOPK; k++) {
                        dv[hf][k] = 10.0f * wgt[hf][k] * (kk * (hf ? rb[k] : ra[k]) - mean);
                        const int row = idx[hf][k];
#pragma unroll
                        for (int dd = 0; dd < DM / 2; dd++)
                            dq[hf * (DM / 2) + dd] = sg_fma(dv[hf][k], keys[row * (DM / 2) + dd], dq[hf * (DM / 2) + dd]);
                    }
                }
#pragma unroll
                for (int dd = 0; dd < DM; dd++) {
                    drow[dd] = dq[dd];
                    const sg::cfloat_p qr = Wq + (hh * DM + dd) * PIN + zo_rb;
#pragma unroll
                    for (int q = 0; q < GH; q++) dhn[q] = sg_fma(qr[q], dq[dd], dhn[q]);
#pragma unroll
                    for (int q = 0; q < DM; q++) dcf[q] = sg_fma(qr[GH + q], dq[dd], dcf[q]);
#pragma unroll
                    for (int q = 0; q < DM; q++) dcb[q] = sg_fma(qr[GH + DM + q], dq[dd], dcb[q]);
                }
                __syncthreads();
                // this head's query-matrix gradients: d query (x) query input over the tile's elements
                {
                    float qs[Q_PER_LANE];
#pragma unroll
                    for (int q = 0; q < Q_PER_LANE; q++) qs[q] = 0.0f;
#pragma unroll 16
                    for (int e = 0; e < BE_THREADS; e++) {      // (unrolled: the LDS reads of 16 elements are in flight together)
#pragma unroll
                        for (int q = 0; q < Q_PER_LANE; q++) qs[q] = sg_fma(s_d[e * DW + qdcol[q]], s_x[e * XW + qxcol[q]], qs[q]);
                    }
#pragma unroll
                    for (int q = 0; q < Q_PER_LANE; q++)
                        if (tid + q * BE_THREADS < N_QHEAD) s_gq[hh * N_QHEAD + tid + q * BE_THREADS] += qs[q];      // one owner per entry
                }
                __syncthreads();
                // product-key gradients, d score (x) query half, the same way: the staged rows are free now, so each
                // lane leaves d score as two 12-vectors (four non-zeros each) and its query; 96 lanes own one entry each
#pragma unroll
                for (int k = 0; k < PK; k++) { rtrow[k] = 0.0f; rtrow[RH + k] = 0.0f; }
#pragma unroll
                for (int k = 0; k < TOPK; k++) {
                    rtrow[idx[0][k]] = dv[0][k];
                    rtrow[RH + idx[1][k]] = dv[1][k];
                }
#pragma unroll
                for (int dd = 0; dd < DM; dd++) drow[dd] = query[dd];
                __syncthreads();
                if (tid < 2 * PK * (DM / 2)) {
                    const int hf = tid / (PK * (DM / 2)), row = (tid / (DM / 2)) % PK, dd = tid % (DM / 2);
                    float acc = 0.0f;
#pragma unroll 16
                    for (int e = 0; e < BE_THREADS; e++) acc = sg_fma(s_rt[e * RW + hf * RH + row], s_d[e * DW + hf * (DM / 2) + dd], acc);
                    s_gkey[(hf * NH + hh) * PK * (DM / 2) + row * (DM / 2) + dd] += acc;
                }
                __syncthreads();
            }
            if (valid && a.smart != nullptr) a.smart[i] = sg_fma(a.rescale, total / (float)NH, g);

            const int zo_gb = sg::opaque_zero();
            // ---- GRU backward
            float dpz[GH], dpr[GH], dph[GH], drh[GH] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int j = 0; j < GH; j++) {
                dpz[j] = (dhn[j] * (cand[j] - h[j])) * (zg[j] * (1.0f - zg[j]));
                dph[j] = (dhn[j] * zg[j]) * (1.0f - cand[j] * cand[j]);
            }
#pragma unroll
            for (int j = 0; j < GH; j++) {
                const sg::cfloat_p wh = Wh + j * GRL + zo_gb;
#pragma unroll
                for (int q = 0; q < DM; q++) { dcf[q] = sg_fma(wh[2 + q], dph[j], dcf[q]); dcb[q] = sg_fma(wh[2 + DM + q], dph[j], dcb[q]); }
#pragma unroll
                for (int q = 0; q < GH; q++) drh[q] = sg_fma(wh[2 + 2 * DM + q], dph[j], drh[q]);
            }
#pragma unroll
            for (int j = 0; j < GH; j++) dpr[j] = (drh[j] * h[j]) * (rg[j] * (1.0f - rg[j]));
#pragma unroll
            for (int j = 0; j < GH; j++) {
                const sg::cfloat_p wz = Wz + j * GRL + zo_gb, wr = Wr + j * GRL + zo_gb;
#pragma unroll
                for (int q = 0; q < DM; q++) {
                    dcf[q] = sg_fma(wz[2 + q], dpz[j], dcf[q]); dcf[q] = sg_fma(wr[2 + q], dpr[j], dcf[q]);
                    dcb[q] = sg_fma(wz[2 + DM + q], dpz[j], dcb[q]); dcb[q] = sg_fma(wr[2 + DM + q], dpr[j], dcb[q]);
                }
            }
#pragma unroll
            for (int j = 0; j < GH; j++) { drow[D_Z + j] = dpz[j]; drow[D_R + j] = dpr[j]; drow[D_H + j] = dph[j]; }
            if (valid) {
                float4* of = reinterpret_cast<float4*>(a.d_ctx + (size_t)i * DM);
                float4* ob = reinterpret_cast<float4*>(a.d_ctx + ((size_t)a.total + i) * DM);
                of[0] = make_float4(dcf[0], dcf[1], dcf[2], dcf[3]); of[1] = make_float4(dcf[4], dcf[5], dcf[6], dcf[7]);
                ob[0] = make_float4(dcb[0], dcb[1], dcb[2], dcb[3]); ob[1] = make_float4(dcb[4], dcb[5], dcb[6], dcb[7]);
            }
        }
        __syncthreads();
        // ---- GRU gradients: each lane's entries, summed over the tile's elements
#pragma unroll 16
        for (int e = 0; e < BE_THREADS; e++) {
#pragma unroll
            for (int q = 0; q < GRU_PER_LANE; q++) gsum[q] = sg_fma(s_d[e * DW + gdcol[q]], s_x[e * XW + gxcol[q]], gsum[q]);
        }
        __syncthreads();
    }

    // ---- this workgroup's sums -> its row of the partials buffer
    float* out = a.partials + (size_t)blockIdx.x * N_GRADS;
#pragma unroll
    for (int q = 0; q < GRU_PER_LANE; q++) {
        const int o = tid + q * BE_THREADS;
        if (o < N_GRU) out[o] = gsum[q];
    }
    __syncthreads();
    for (int i = tid; i < NH * N_QHEAD; i += BE_THREADS) out[N_GRU + i] = s_gq[i];
    for (int i = tid; i < 2 * NH * PK * (DM / 2); i += BE_THREADS) out[OFF_KA + i] = s_gkey[i];
    // the waves' near-zero sums into the bins of those intervals, one wave after the other (a fixed order).  Register v
    // of an accumulator holds first index 4 (lane / 16) + v, second index lane % 16.
    for (int w = 0; w < BE_WAVES; w++) {
        __syncthreads();
        if ((tid >> 6) != w) continue;
#pragma unroll
        for (int v = 0; v < 4; v++) {
            const int ia = 4 * ((tid & 63) >> 4) + v, ib = tid & 15;
            if (ia >= PK || ib >= PK) continue;
            int e = ia * PK + ib;
            if (e >= NE) e = NE - 1;
            const int bp = e * NBIN + s_kz[2 * e + 1], bn = e * NBIN + s_kz[2 * e];
            s_bin[2 * bp] += cen[0][v];
            s_bin[2 * bn] += cen[1][v];
            s_bin[2 * bp + 1] += cen[2][v];
            s_bin[2 * bn + 1] += cen[3][v];
        }
    }
    __syncthreads();
    // expert gradients from the bins: d b1 = W2 * S0, d W1 = W2 * S1, d W2 = sum w relu(pre) = W1 * S1 + b1 * S0, d b2 = sum w
    for (int i = tid; i < NE * EH; i += BE_THREADS) {
        const int e = i / EH;
        const float w1 = a.W.w[W_EXP_W1][i], b1 = a.W.w[W_EXP_B1][i], w2 = a.W.w[W_EXP_W2][i];
        const int rank = s_rank[i];
        float S0 = 0.0f, S1 = 0.0f;
        for (int k = 0; k < NBIN; k++) {
            if (!unit_active(w1, b1, rank, k)) continue;
            S0 += s_bin[2 * (e * NBIN + k)];
            S1 += s_bin[2 * (e * NBIN + k) + 1];
        }
        out[OFF_W1 + i] = w2 * S1;
        out[OFF_B1 + i] = w2 * S0;
        out[OFF_W2 + i] = sg_fma(w1, S1, b1 * S0);
    }
    for (int e = tid; e < NE; e += BE_THREADS) {
        float sd = 0.0f;
        for (int k = 0; k < NBIN; k++) sd += s_bin[2 * (e * NBIN + k)];
        out[OFF_B2 + e] = sd;
    }
}

// Rows of the partials buffer added in a fixed order: 64 entries per workgroup, four lanes per entry each taking
// every fourth row, then the four partial sums in order.
__global__ __launch_bounds__(256) void k_sum_partials(const float* __restrict__ partials, int rows, float* __restrict__ out) {
    __shared__ float s_part[4][64];
    const int col = threadIdx.x & 63, slice = threadIdx.x >> 6;
    const int o = blockIdx.x * 64 + col;
    float acc = 0.0f;
    if (o < N_GRADS) {
#pragma unroll 4
        for (int r = slice; r < rows; r += 4) acc += partials[(size_t)r * N_GRADS + o];
    }
    s_part[slice][col] = acc;
    __syncthreads();
    if (slice == 0 && o < N_GRADS) out[o] = ((s_part[0][col] + s_part[1][col]) + s_part[2][col]) + s_part[3][col];
}

constexpr int BE_LDS_BYTES = 4 * (NE * EH + NE * NBIN * 4 + 2 * NH * PK * (DM / 2) + BE_THREADS * (XW + DW + RW) + NH * N_QHEAD) + NE * EH + NE * 2;
static_assert(BE_LDS_BYTES <= 160 * 1024, "one workgroup of k_bilevel_elem per CU");
constexpr int BE_MAX_GROUPS = 256;       // one resident workgroup on each of the 256 CUs: one round, every workgroup walks the same number of tiles (+-1)

int elem_groups(int64_t total) {
    const int64_t tiles = (total + BE_THREADS - 1) / BE_THREADS;
    return (int)(tiles < BE_MAX_GROUPS ? (tiles > 0 ? tiles : 1) : BE_MAX_GROUPS);
}

}  // namespace
}  // namespace sg2

extern "C" {

size_t sg2_bilevel_elem_workspace_bytes(int64_t total) {
    if (total < 0) return 0;
    return sizeof(float) * (size_t)sg2::elem_groups(total) * sg2::N_GRADS;
}

int sg2_bilevel_elem(const SgDims* dims, const Sg2Weights* weights, int64_t total, const float* grad, const float* sharpness,
                     const float* ctx, const float* gru_state, const float* cotangent, float rescale, float* smart_out,
                     float* d_ctx, float* grads_out, void* workspace, size_t workspace_bytes, void* stream) {
    return sg2_bilevel_elem_ex(dims, weights, total, grad, sharpness, ctx, gru_state, cotangent, rescale, smart_out, nullptr, d_ctx, grads_out,
                               workspace, workspace_bytes, stream);
}

int sg2_bilevel_elem_ex(const SgDims* dims, const Sg2Weights* weights, int64_t total, const float* grad, const float* sharpness,
                        const float* ctx, const float* gru_state, const float* cotangent, float rescale, float* smart_out,
                        float* gru_out, float* d_ctx, float* grads_out, void* workspace, size_t workspace_bytes, void* stream) {
    using namespace sg2;
    hipStream_t st = (hipStream_t)stream;
    if (check_dims(dims, true)) return 1;
    if (!weights || !grads_out) return sg::fail("NULL argument");
    if (total < 0 || total > 0x7fffffffLL - BE_THREADS) return sg::fail("element count %lld out of range", (long long)total);
    for (int k = W_GRU_WZ; k < SG2_NUM_WEIGHTS; k++)
        if (!weights->w[k]) return sg::fail("weight pointer %d is NULL", k);
    const int groups = elem_groups(total);
    if (!workspace || workspace_bytes < sizeof(float) * (size_t)groups * N_GRADS)
        return sg::fail("workspace too small: need %zu bytes, got %zu", sizeof(float) * (size_t)groups * N_GRADS, workspace_bytes);
    if (total > 0) {
        if (!grad || !sharpness || !ctx || !gru_state || !cotangent || !d_ctx) return sg::fail("NULL argument");
        if ((((uintptr_t)ctx | (uintptr_t)gru_state | (uintptr_t)d_ctx | (uintptr_t)gru_out) & 15u) != 0)
            return sg::fail("ctx, gru_state, gru_out and d_ctx must be 16-byte aligned");
    }
    {
        static bool raised[64] = {};
        int dev = 0;
        SG_HIP_CHECK(hipGetDevice(&dev));
        if (dev < 0 || dev >= 64) return sg::fail("device index %d out of range", dev);
        if (!raised[dev]) {
            SG_HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void*>(k_bilevel_elem), hipFuncAttributeMaxDynamicSharedMemorySize, BE_LDS_BYTES));
            raised[dev] = true;
        }
    }
    ElemArgs a;
    a.g = grad; a.s = sharpness; a.ctx = ctx; a.gru = gru_state; a.cot = cotangent;
    a.smart = smart_out; a.d_ctx = d_ctx; a.partials = static_cast<float*>(workspace); a.gru_out = gru_out;
    a.total = (int)total; a.rescale = rescale; a.W = *weights;
    hipLaunchKernelGGL(k_bilevel_elem, dim3(groups), dim3(BE_THREADS), BE_LDS_BYTES, st, a);
    SG_LAUNCH_CHECK("k_bilevel_elem");
    hipLaunchKernelGGL(k_sum_partials, dim3((N_GRADS + 63) / 64), dim3(256), 0, st, a.partials, groups, grads_out);
    SG_LAUNCH_CHECK("k_sum_partials");
    return 0;
}

}  // extern "C"
