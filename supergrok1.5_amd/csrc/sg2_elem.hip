// Per-element tail of the SuperGrok v2 step: GRU -> 4-head PEER product-key
// routing -> expert MLP -> skip connection -> mu EMA -> Adam + weight decay.
//
// Replaces fused_elem_step_kernel
// (csrc/supergrok2_mamba_peer_kernels.cu:793-1089 of the reference); the
// out_proj contraction that kernel starts with is done by the scan kernel,
// which hands over the two 8-float contexts per element in element order.
//
// One launch covers every tensor: a persistent grid walks tiles of 1024
// elements; the tile index is mapped to (tensor, offset) by a binary search
// over a P+1 entry prefix table.  The 144 expert MLPs live in LDS (records of
// 48 floats padded to 52 so that random per-lane experts spread over the
// banks); GRU and key weights are wave-uniform and come in through scalar
// loads (constant address space); the query projection is a chain of fp32
// matrix instructions.  expert_counts is accumulated in an LDS histogram and flushed
// once per workgroup (the reference issues one global atomic per element and
// head).
#include "sg2_internal.hpp"

namespace sg2 {
namespace {

constexpr int ELEM_THREADS = 256;
// floats per expert record in LDS: W1[EH] b1[EH] W2[EH] (+ pad for the 16-wide experts so that random per-lane
// experts spread over the banks)
template <int EHW>
constexpr int exp_stride() { return EHW == 16 ? 52 : 3 * EHW; }
typedef float vf4 __attribute__((ext_vector_type(4)));
typedef float vf32 __attribute__((ext_vector_type(32)));

// Four waves per SIMD for the default geometry: told so, the compiler keeps the matrix results in ordinary registers
// (115 of them, no accumulation registers to copy out of) instead of settling for three waves at 112 + 32.
template <class G>
constexpr int elem_waves() { return G::DM == 8 ? 4 : 2; }
// FWD: the net's forward alone (sg2_meta_forward) -- smart gradient and new GRU state of every element go to the packed
// arrays fwd_smart / fwd_gru, nothing of the optimizer state is read or written.
template <class G, int EH, bool DBG, bool FWD = false>
__global__ __launch_bounds__(ELEM_THREADS) __attribute__((amdgpu_waves_per_eu(elem_waves<G>(), elem_waves<G>()))) void k_elem(Plan pl, int32_t* __restrict__ expert_counts,
                                                       int32_t* __restrict__ dbg_eidx, float* __restrict__ fwd_smart,
                                                       float* __restrict__ fwd_gru) {
    constexpr int DM = G::DM, GRL = G::GRL, PIN = G::PIN, EXP_STRIDE = exp_stride<EH>();
    static_assert(EH % 4 == 0, "expert records are read 16 bytes at a time");
    __shared__ float s_exp[NE * EXP_STRIDE];
    __shared__ float s_b2[NE];
    __shared__ int s_cnt[NE];

    {
        const float* __restrict__ W1 = pl.W.w[W_EXP_W1];
        const float* __restrict__ B1 = pl.W.w[W_EXP_B1];
        const float* __restrict__ W2 = pl.W.w[W_EXP_W2];
        for (int i = threadIdx.x; i < NE * EH; i += ELEM_THREADS) {
            const int e = i / EH, k = i % EH;
            s_exp[e * EXP_STRIDE + k] = W1[i];
            s_exp[e * EXP_STRIDE + EH + k] = B1[i];
            s_exp[e * EXP_STRIDE + 2 * EH + k] = W2[i];
        }
        for (int i = threadIdx.x; i < NE; i += ELEM_THREADS) {
            s_b2[i] = pl.W.w[W_EXP_B2][i];
            s_cnt[i] = 0;
        }
    }
    __syncthreads();

    const sg::cfloat_p Wz0 = sg::as_const(pl.W.w[W_GRU_WZ]);
    const sg::cfloat_p bz0 = sg::as_const(pl.W.w[W_GRU_BZ]);
    const sg::cfloat_p Wr0 = sg::as_const(pl.W.w[W_GRU_WR]);
    const sg::cfloat_p br0 = sg::as_const(pl.W.w[W_GRU_BR]);
    const sg::cfloat_p Wh0 = sg::as_const(pl.W.w[W_GRU_WH]);
    const sg::cfloat_p bh0 = sg::as_const(pl.W.w[W_GRU_BH]);
    // The query projection runs on the matrix pipe: v_mfma_f32_32x32x1_2b is one fused multiply-add per output and
    // step, so a chain of them is the fmaf chain of the scalar form, bit for bit, in the same order.  Lane l supplies
    // row l % 32 of each 32-row slice of the query matrix (held in registers for the whole kernel) and its own
    // element's inputs; the outputs come back split over lanes l and l ^ 32 and are exchanged below.
    constexpr int NQM = NH * DM / 32;
    static_assert(NH * DM % 32 == 0 && 32 % DM == 0, "query rows are handled in slices of 32");
    float aq[NQM][PIN];
#pragma unroll
    for (int m = 0; m < NQM; m++)
#pragma unroll
        for (int q = 0; q < PIN; q++) aq[m][q] = pl.W.w[W_PEER_Q][(m * 32 + (threadIdx.x & 31)) * PIN + q];
    const sg::cfloat_p KA0 = sg::as_const(pl.W.w[W_KEYS_A]);
    const sg::cfloat_p KB0 = sg::as_const(pl.W.w[W_KEYS_B]);

    for (int tile = blockIdx.x; tile < pl.elem_tiles; tile += gridDim.x) {
        const int ti = sg::upper_seg(sg::as_const(pl.elem_tile_prefix), pl.P, tile);
        const TensorDev& T = pl.tensors[ti];
        const int start = (tile - pl.elem_tile_prefix[ti]) * ELEM_TILE;
        const int cnt = min(ELEM_TILE, T.numel - start);
        const int dtype = T.dtype;
        const bool has_s = pl.sharp_nonzero[ti] != 0;       // set by the sort's key kernel: some sharpness entry of the tensor is not 0
        const float alpha = T.alpha, lamb = T.lamb, beta1 = T.beta1, bc2 = T.bc2, step_size = T.step_size;
        const float beta2 = pl.beta2, eps = pl.eps, rescale = pl.rescale, decay = pl.decay;

        // every lane runs every iteration (the matrix instructions ignore the execution mask); lanes past the end
        // of the tile recompute its last element and store nothing
        for (int k0 = 0; k0 < cnt; k0 += ELEM_THREADS) {
            const bool live = k0 + (int)threadIdx.x < cnt;
            const int i = start + min(k0 + (int)threadIdx.x, cnt - 1);
            // the weights are re-read (scalar loads, cache hits) for every element instead of being hoisted
            const int zo = sg::opaque_zero();
            const sg::cfloat_p Wz = Wz0 + zo, bz = bz0 + zo, Wr = Wr0 + zo, br = br0 + zo, Wh = Wh0 + zo, bh = bh0 + zo;
            const sg::cfloat_p KA = KA0 + zo, KB = KB0 + zo;
            const float g = sg::finite_or_zero(sg::load_elem(T.grad, dtype, i));
            const float s = has_s ? sg::finite_or_zero(sg::load_elem(T.sharp, dtype, i)) : 0.0f;
            float cf[DM], cb[DM], hold[GH];
            {
                const SG_GLOBAL vf4* pf = (const SG_GLOBAL vf4*)(pl.ctx + ((size_t)T.off + i) * DM);
                const SG_GLOBAL vf4* pb = (const SG_GLOBAL vf4*)(pl.ctx + ((size_t)pl.total + T.off + i) * DM);
#pragma unroll
                for (int q = 0; q < DM / 4; q++) {
                    const vf4 a = pf[q], b = pb[q];
                    cf[4 * q] = a[0]; cf[4 * q + 1] = a[1]; cf[4 * q + 2] = a[2]; cf[4 * q + 3] = a[3];
                    cb[4 * q] = b[0]; cb[4 * q + 1] = b[1]; cb[4 * q + 2] = b[2]; cb[4 * q + 3] = b[3];
                }
                const vf4 h4 = ((const SG_GLOBAL vf4*)T.gru)[i];
                hold[0] = h4[0]; hold[1] = h4[1]; hold[2] = h4[2]; hold[3] = h4[3];
            }
            // the optimizer state is requested now, so that its latency passes under the meta-net's arithmetic
            float mu = 0.0f, ea = 0.0f, easq = 0.0f, pv = 0.0f;
            if (!FWD) {
                mu = sg::gptr(T.mu)[i]; ea = sg::gptr(T.ea)[i]; easq = sg::gptr(T.easq)[i];
                pv = sg::load_elem(T.param, dtype, i);
            }

            // ---- GRU: chain order = bias, g, s, fwd ctx, bwd ctx, h
            float zg[GH], rg[GH], hnew[GH];
            float pre_g[2 * GH], gate[2 * GH], pre_c[GH], cand[GH];      // gates and candidates share one reciprocal each
#pragma unroll
            for (int j = 0; j < GH; j++) {
                const sg::cfloat_p wz = Wz + j * GRL;
                const sg::cfloat_p wr = Wr + j * GRL;
                float vz = bz[j], vr = br[j];
                vz = sg_fma(wz[0], g, vz); vz = sg_fma(wz[1], s, vz);
                vr = sg_fma(wr[0], g, vr); vr = sg_fma(wr[1], s, vr);
#pragma unroll
                for (int q = 0; q < DM; q++) { vz = sg_fma(wz[2 + q], cf[q], vz); vr = sg_fma(wr[2 + q], cf[q], vr); }
#pragma unroll
                for (int q = 0; q < DM; q++) { vz = sg_fma(wz[2 + DM + q], cb[q], vz); vr = sg_fma(wr[2 + DM + q], cb[q], vr); }
#pragma unroll
                for (int q = 0; q < GH; q++) { vz = sg_fma(wz[2 + 2 * DM + q], hold[q], vz); vr = sg_fma(wr[2 + 2 * DM + q], hold[q], vr); }
                pre_g[j] = vz;
                pre_g[GH + j] = vr;
            }
            sg_sigmoid_block(2 * GH, pre_g, gate);
#pragma unroll
            for (int j = 0; j < GH; j++) { zg[j] = gate[j]; rg[j] = gate[GH + j]; }
#pragma unroll
            for (int j = 0; j < GH; j++) {
                const sg::cfloat_p wh = Wh + j * GRL;
                float v = bh[j];
                v = sg_fma(wh[0], g, v); v = sg_fma(wh[1], s, v);
#pragma unroll
                for (int q = 0; q < DM; q++) v = sg_fma(wh[2 + q], cf[q], v);
#pragma unroll
                for (int q = 0; q < DM; q++) v = sg_fma(wh[2 + DM + q], cb[q], v);
#pragma unroll
                for (int q = 0; q < GH; q++) v = sg_fma(wh[2 + 2 * DM + q], rg[q] * hold[q], v);
                pre_c[j] = v;
            }
            sg_tanh_block(GH, pre_c, cand);
#pragma unroll
            for (int j = 0; j < GH; j++) hnew[j] = sg_fma(zg[j], cand[j], (1.0f - zg[j]) * hold[j]);
            if (live) {
                if (FWD) ((SG_GLOBAL vf4*)fwd_gru)[(size_t)T.off + i] = vf4{hnew[0], hnew[1], hnew[2], hnew[3]};
                else ((SG_GLOBAL vf4*)T.gru)[i] = vf4{hnew[0], hnew[1], hnew[2], hnew[3]};
            }

            // ---- PEER queries: chain order = h, fwd ctx, bwd ctx, g, s
            float qall[NH * DM];
#pragma unroll
            for (int m = 0; m < NQM; m++) {
                vf32 acc = {};
                int c = 0;
#pragma unroll
                for (int q = 0; q < GH; q++, c++) acc = __builtin_amdgcn_mfma_f32_32x32x1f32(aq[m][c], hnew[q], acc, 0, 0, 0);
#pragma unroll
                for (int q = 0; q < DM; q++, c++) acc = __builtin_amdgcn_mfma_f32_32x32x1f32(aq[m][c], cf[q], acc, 0, 0, 0);
#pragma unroll
                for (int q = 0; q < DM; q++, c++) acc = __builtin_amdgcn_mfma_f32_32x32x1f32(aq[m][c], cb[q], acc, 0, 0, 0);
                acc = __builtin_amdgcn_mfma_f32_32x32x1f32(aq[m][c], g, acc, 0, 0, 0);
                acc = __builtin_amdgcn_mfma_f32_32x32x1f32(aq[m][c + 1], s, acc, 0, 0, 0);
                // register r of block b holds row 8 (r / 4) + 4 (lane / 32) + r % 4 of element 32 b + lane % 32:
                // exchanging the upper half of block 0 with the lower half of block 1 gives each lane its own element
#pragma unroll
                for (int r = 0; r < 16; r++) {
                    const auto pr = __builtin_amdgcn_permlane32_swap(__float_as_uint(acc[r]), __float_as_uint(acc[16 + r]), false, false);
                    qall[m * 32 + 8 * (r / 4) + r % 4] = __uint_as_float(pr[0]);
                    qall[m * 32 + 8 * (r / 4) + 4 + r % 4] = __uint_as_float(pr[1]);
                }
            }

            // ---- PEER routing + expert MLP
            float total = 0.0f;
#pragma unroll
            for (int hh = 0; hh < NH; hh++) {
                const float* query = qall + hh * DM;
                int best[2];
#pragma unroll
                for (int hf = 0; hf < 2; hf++) {
                    const sg::cfloat_p keys = (hf ? KB : KA) + hh * PK * (DM / 2);
                    int bi = 0;
                    float bs = -1e30f;
#pragma unroll
                    for (int q = 0; q < PK; q++) {
                        float dot = 0.0f;
#pragma unroll
                        for (int dd = 0; dd < DM / 2; dd++) dot = sg_fma(query[hf * (DM / 2) + dd], keys[q * (DM / 2) + dd], dot);
                        if (dot > bs) { bs = dot; bi = q; }
                    }
                    best[hf] = bi;
                }
                int e = best[0] * PK + best[1];
                if (e >= NE) e = NE - 1;
                if (live) atomicAdd(&s_cnt[e], 1);
                if (DBG && live) dbg_eidx[((size_t)T.off + i) * NH + hh] = e;

                const float4* rec = reinterpret_cast<const float4*>(s_exp + e * EXP_STRIDE);
                float ho = s_b2[e];
#pragma unroll
                for (int q4 = 0; q4 < EH / 4; q4++) {
                    const float4 w1 = rec[q4], b1 = rec[EH / 4 + q4], w2 = rec[2 * (EH / 4) + q4];
                    float z;
                    z = sg_max(sg_fma(w1.x, g, b1.x), 0.0f); ho = sg_fma(w2.x, z, ho);
                    z = sg_max(sg_fma(w1.y, g, b1.y), 0.0f); ho = sg_fma(w2.y, z, ho);
                    z = sg_max(sg_fma(w1.z, g, b1.z), 0.0f); ho = sg_fma(w2.z, z, ho);
                    z = sg_max(sg_fma(w1.w, g, b1.w), 0.0f); ho = sg_fma(w2.w, z, ho);
                }
                total = total + ho;
            }
            const float smart = g + (rescale * total) / (float)NH;
            if (FWD) {
                if (live) sg::gptr(fwd_smart)[(size_t)T.off + i] = smart;
                continue;
            }

            // ---- mu EMA, Adam moments, decoupled weight decay
            mu = sg_fma(alpha, mu, (1.0f - alpha) * g);
            if (live) sg::gptr(T.mu)[i] = mu;
            const float fg = sg_fma(lamb, mu, smart);
            ea = sg_fma(beta1, ea, (1.0f - beta1) * fg);
            easq = sg_fma(beta2, easq, ((1.0f - beta2) * fg) * fg);
            if (live) {
                sg::gptr(T.ea)[i] = ea;
                sg::gptr(T.easq)[i] = easq;
            }
            const float denom = __builtin_sqrtf(easq / bc2) + eps;
            pv = sg_fma(pv, decay, -((step_size * ea) / denom));
            if (live) sg::store_elem(T.param, dtype, i, pv);
        }
    }
    __syncthreads();
    if (expert_counts != nullptr)
        for (int i = threadIdx.x; i < NE; i += ELEM_THREADS)
            if (s_cnt[i] != 0) atomicAdd(&expert_counts[i], s_cnt[i]);
}


// The same per-element step for any dimensions the reference admits (gru_hidden <= 8, d_model <= 16, any number of
// heads, sub-keys, experts and expert width): every size is a run-time value, the loops over the bounded ones are
// unrolled to their bounds and guarded so that the small arrays stay in registers, the expert tables are read from
// global memory (per-lane gathers through the caches: 3 x E x expert_hidden floats need not fit the LDS), and the
// counts go through an LDS histogram when it fits and global atomics otherwise.  The arithmetic is the specialised
// kernel's, chain for chain (the query projection as plain fma chains: the fp32 matrix instructions compute the same
// chains); the shared reciprocals of the gates apply when gru_hidden is 4, as in the checker.  ctx rows are
// ctx_stride floats apart (d_model of the scan geometry the block was embedded in).
constexpr int MAX_DM = 16, MAX_GH = 8, MAX_HD = 8, CNT_LDS = 4096;
// fwd_smart / fwd_gru (both or neither): the net's forward alone -- smart gradient and new GRU state of every element go
// to these packed arrays, nothing of the optimizer state is read or written (sg2_meta_forward).
template <bool DBG>
__global__ __launch_bounds__(ELEM_THREADS) void k_elem_any(Plan pl, int ctx_stride, int32_t* __restrict__ expert_counts,
                                                           int32_t* __restrict__ dbg_eidx, float* __restrict__ fwd_smart,
                                                           float* __restrict__ fwd_gru) {
    __shared__ int s_cnt[CNT_LDS];
    const int dm = pl.dims.d_model, gh = pl.dims.gru_hidden, H = pl.dims.num_heads, pk = pl.dims.pk_dim;
    const int eh = pl.dims.expert_hidden, E = pl.dims.num_experts, hd = dm / 2;
    const int grl = 2 + 2 * dm + gh, pin = gh + 2 * dm + 2;
    const bool lds_counts = E <= CNT_LDS;
    if (lds_counts)
        for (int i = threadIdx.x; i < E; i += ELEM_THREADS) s_cnt[i] = 0;
    __syncthreads();
    const sg::cfloat_p Wz = sg::as_const(pl.W.w[W_GRU_WZ]), bz = sg::as_const(pl.W.w[W_GRU_BZ]);
    const sg::cfloat_p Wr = sg::as_const(pl.W.w[W_GRU_WR]), br = sg::as_const(pl.W.w[W_GRU_BR]);
    const sg::cfloat_p Wh = sg::as_const(pl.W.w[W_GRU_WH]), bh = sg::as_const(pl.W.w[W_GRU_BH]);
    const sg::cfloat_p Wq = sg::as_const(pl.W.w[W_PEER_Q]);
    const sg::cfloat_p KA = sg::as_const(pl.W.w[W_KEYS_A]), KB = sg::as_const(pl.W.w[W_KEYS_B]);
    const SG_GLOBAL float* W1 = sg::gptr(pl.W.w[W_EXP_W1]);
    const SG_GLOBAL float* B1 = sg::gptr(pl.W.w[W_EXP_B1]);
    const SG_GLOBAL float* W2 = sg::gptr(pl.W.w[W_EXP_W2]);
    const SG_GLOBAL float* B2 = sg::gptr(pl.W.w[W_EXP_B2]);

    for (int tile = blockIdx.x; tile < pl.elem_tiles; tile += gridDim.x) {
        const int ti = sg::upper_seg(sg::as_const(pl.elem_tile_prefix), pl.P, tile);
        const TensorDev& T = pl.tensors[ti];
        const int start = (tile - pl.elem_tile_prefix[ti]) * ELEM_TILE;
        const int cnt = min(ELEM_TILE, T.numel - start);
        const int dtype = T.dtype;
        const bool has_s = pl.sharp_nonzero[ti] != 0;
        const float alpha = T.alpha, lamb = T.lamb, beta1 = T.beta1, bc2 = T.bc2, step_size = T.step_size;
        const float beta2 = pl.beta2, eps = pl.eps, rescale = pl.rescale, decay = pl.decay;
        for (int k0 = (int)threadIdx.x; k0 < cnt; k0 += ELEM_THREADS) {
            const int i = start + k0;
            const float g = sg::finite_or_zero(sg::load_elem(T.grad, dtype, i));
            const float s = has_s ? sg::finite_or_zero(sg::load_elem(T.sharp, dtype, i)) : 0.0f;
            float cf[MAX_DM], cb[MAX_DM], hold[MAX_GH];
            {
                const SG_GLOBAL float* pf = sg::gptr(pl.ctx) + ((size_t)T.off + i) * ctx_stride;
                const SG_GLOBAL float* pb = sg::gptr(pl.ctx) + ((size_t)pl.total + T.off + i) * ctx_stride;
#pragma unroll
                for (int q = 0; q < MAX_DM; q++) { cf[q] = q < dm ? pf[q] : 0.0f; cb[q] = q < dm ? pb[q] : 0.0f; }
#pragma unroll
                for (int q = 0; q < MAX_GH; q++) hold[q] = q < gh ? sg::gptr(T.gru)[(size_t)i * gh + q] : 0.0f;
            }
            // ---- GRU: chain order = bias, g, s, fwd ctx, bwd ctx, h
            float pre_g[2 * MAX_GH], gate[2 * MAX_GH], pre_c[MAX_GH], cand[MAX_GH], hnew[MAX_GH];
#pragma unroll
            for (int j = 0; j < MAX_GH; j++) {
                pre_g[j] = pre_g[MAX_GH + j] = 0.0f;
                if (j < gh) {
                    const sg::cfloat_p wz = Wz + j * grl, wr = Wr + j * grl;
                    float vz = bz[j], vr = br[j];
                    vz = sg_fma(wz[0], g, vz); vz = sg_fma(wz[1], s, vz);
                    vr = sg_fma(wr[0], g, vr); vr = sg_fma(wr[1], s, vr);
#pragma unroll
                    for (int q = 0; q < MAX_DM; q++) if (q < dm) { vz = sg_fma(wz[2 + q], cf[q], vz); vr = sg_fma(wr[2 + q], cf[q], vr); }
#pragma unroll
                    for (int q = 0; q < MAX_DM; q++) if (q < dm) { vz = sg_fma(wz[2 + dm + q], cb[q], vz); vr = sg_fma(wr[2 + dm + q], cb[q], vr); }
#pragma unroll
                    for (int q = 0; q < MAX_GH; q++) if (q < gh) { vz = sg_fma(wz[2 + 2 * dm + q], hold[q], vz); vr = sg_fma(wr[2 + 2 * dm + q], hold[q], vr); }
                    pre_g[j] = vz;
                    pre_g[MAX_GH + j] = vr;
                }
            }
            if (gh == GH) {       // update and reset gates of the four units share one reciprocal
                float in8[2 * GH], out8[2 * GH];
#pragma unroll
                for (int j = 0; j < GH; j++) { in8[j] = pre_g[j]; in8[GH + j] = pre_g[MAX_GH + j]; }
                sg_sigmoid_block(2 * GH, in8, out8);
#pragma unroll
                for (int j = 0; j < MAX_GH; j++) { gate[j] = j < GH ? out8[j] : 0.0f; gate[MAX_GH + j] = j < GH ? out8[GH + j] : 0.0f; }
            } else {
#pragma unroll
                for (int j = 0; j < 2 * MAX_GH; j++) gate[j] = sg_sigmoid(pre_g[j]);
            }
#pragma unroll
            for (int j = 0; j < MAX_GH; j++) {
                pre_c[j] = 0.0f;
                if (j < gh) {
                    const sg::cfloat_p wh = Wh + j * grl;
                    float v = bh[j];
                    v = sg_fma(wh[0], g, v); v = sg_fma(wh[1], s, v);
#pragma unroll
                    for (int q = 0; q < MAX_DM; q++) if (q < dm) v = sg_fma(wh[2 + q], cf[q], v);
#pragma unroll
                    for (int q = 0; q < MAX_DM; q++) if (q < dm) v = sg_fma(wh[2 + dm + q], cb[q], v);
#pragma unroll
                    for (int q = 0; q < MAX_GH; q++) if (q < gh) v = sg_fma(wh[2 + 2 * dm + q], gate[MAX_GH + q] * hold[q], v);
                    pre_c[j] = v;
                }
            }
            if (gh == GH) {
                float in4[GH], out4[GH];
#pragma unroll
                for (int j = 0; j < GH; j++) in4[j] = pre_c[j];
                sg_tanh_block(GH, in4, out4);
#pragma unroll
                for (int j = 0; j < MAX_GH; j++) cand[j] = j < GH ? out4[j] : 0.0f;
            } else {
#pragma unroll
                for (int j = 0; j < MAX_GH; j++) cand[j] = sg_tanh(pre_c[j]);
            }
#pragma unroll
            for (int j = 0; j < MAX_GH; j++) {
                hnew[j] = sg_fma(gate[j], cand[j], (1.0f - gate[j]) * hold[j]);
                if (j < gh) {
                    if (fwd_gru != nullptr) sg::gptr(fwd_gru)[((size_t)T.off + i) * gh + j] = hnew[j];
                    else sg::gptr(T.gru)[(size_t)i * gh + j] = hnew[j];
                }
            }

            // ---- PEER: per head the query (chain order = h, fwd ctx, bwd ctx, g, s), two sub-key arg-maxes, the expert
            float total = 0.0f;
            for (int hh = 0; hh < H; hh++) {
                auto query_row = [&](int row) {
                    const sg::cfloat_p qr = Wq + ((size_t)hh * dm + row) * pin;
                    float v = 0.0f;
#pragma unroll
                    for (int q = 0; q < MAX_GH; q++) if (q < gh) v = sg_fma(qr[q], hnew[q], v);
#pragma unroll
                    for (int q = 0; q < MAX_DM; q++) if (q < dm) v = sg_fma(qr[gh + q], cf[q], v);
#pragma unroll
                    for (int q = 0; q < MAX_DM; q++) if (q < dm) v = sg_fma(qr[gh + dm + q], cb[q], v);
                    v = sg_fma(qr[gh + 2 * dm], g, v);
                    v = sg_fma(qr[gh + 2 * dm + 1], s, v);
                    return v;
                };
                float qa[MAX_HD], qb[MAX_HD];
#pragma unroll
                for (int dd = 0; dd < MAX_HD; dd++) {
                    qa[dd] = qb[dd] = 0.0f;
                    if (dd < hd) { qa[dd] = query_row(dd); qb[dd] = query_row(hd + dd); }
                }
                int best[2];
#pragma unroll
                for (int hf = 0; hf < 2; hf++) {
                    const sg::cfloat_p keys = (hf ? KB : KA) + (size_t)hh * pk * hd;
                    int bi = 0;
                    float bs = -1e30f;
                    for (int q = 0; q < pk; q++) {
                        float dot = 0.0f;
#pragma unroll
                        for (int dd = 0; dd < MAX_HD; dd++) if (dd < hd) dot = sg_fma(hf ? qb[dd] : qa[dd], keys[q * hd + dd], dot);
                        if (dot > bs) { bs = dot; bi = q; }
                    }
                    best[hf] = bi;
                }
                int e = best[0] * pk + best[1];
                if (e >= E) e = E - 1;
                if (lds_counts) atomicAdd(&s_cnt[e], 1);
                else if (expert_counts != nullptr) atomicAdd(&expert_counts[e], 1);
                if (DBG) dbg_eidx[((size_t)T.off + i) * H + hh] = e;
                float ho = B2[e];
                for (int q = 0; q < eh; q++) {
                    const float z = sg_max(sg_fma(W1[(size_t)e * eh + q], g, B1[(size_t)e * eh + q]), 0.0f);
                    ho = sg_fma(W2[(size_t)e * eh + q], z, ho);
                }
                total = total + ho;
            }
            const float smart = g + (rescale * total) / (float)H;
            if (fwd_smart != nullptr) {
                sg::gptr(fwd_smart)[(size_t)T.off + i] = smart;
                continue;
            }

            // ---- mu EMA, Adam moments, decoupled weight decay
            float mu = sg::gptr(T.mu)[i], ea = sg::gptr(T.ea)[i], easq = sg::gptr(T.easq)[i];
            float pv = sg::load_elem(T.param, dtype, i);
            mu = sg_fma(alpha, mu, (1.0f - alpha) * g);
            sg::gptr(T.mu)[i] = mu;
            const float fg = sg_fma(lamb, mu, smart);
            ea = sg_fma(beta1, ea, (1.0f - beta1) * fg);
            easq = sg_fma(beta2, easq, ((1.0f - beta2) * fg) * fg);
            sg::gptr(T.ea)[i] = ea;
            sg::gptr(T.easq)[i] = easq;
            const float denom = __builtin_sqrtf(easq / bc2) + eps;
            pv = sg_fma(pv, decay, -((step_size * ea) / denom));
            sg::store_elem(T.param, dtype, i, pv);
        }
    }
    __syncthreads();
    if (lds_counts && expert_counts != nullptr)
        for (int i = threadIdx.x; i < E; i += ELEM_THREADS)
            if (s_cnt[i] != 0) atomicAdd(&expert_counts[i], s_cnt[i]);
}

}  // namespace

int launch_elem_forward(const Plan& pl, int32_t* expert_counts, float* smart_out, float* gru_out, hipStream_t st) {
    if (pl.total == 0) return 0;
    const int grid = pl.elem_tiles < 4096 ? pl.elem_tiles : 4096;
    int32_t* const no_dbg = nullptr;
    auto go = [&](auto kernel) { hipLaunchKernelGGL(kernel, dim3(grid), dim3(ELEM_THREADS), 0, st, pl, expert_counts, no_dbg, smart_out, gru_out); };
    if (pl.elem_kind == ELEM_ANY)
        hipLaunchKernelGGL(k_elem_any<false>, dim3(grid), dim3(ELEM_THREADS), 0, st, pl, geo_info(pl.geo).dm, expert_counts, no_dbg, smart_out, gru_out);
    else if (pl.geo == GEO_LARGE) go(k_elem<GeoLarge, 16, false, true>);
    else if (pl.elem_kind == ELEM_FAST4) go(k_elem<GeoDefault, 4, false, true>);
    else go(k_elem<GeoDefault, 16, false, true>);
    SG_LAUNCH_CHECK("k_elem<forward>");
    return 0;
}

int launch_elem(const Plan& pl, int32_t* expert_counts, int32_t* dbg_expert_idx, hipStream_t st) {
    if (pl.total == 0) return 0;
    // about five workgroups per resident slot (768 at three per CU): measured 1.38 / 1.35 / 1.33 / 1.33 / 1.37 ms with 768 / 2048 / 4096 /
    // 8192 / 16384 workgroups on 24 424 tiles (fewer leave the chip unevenly loaded at the end, more pay the LDS fill too often)
    const int grid = pl.elem_tiles < 4096 ? pl.elem_tiles : 4096;
    float* const none = nullptr;
    auto go = [&](auto kernel) { hipLaunchKernelGGL(kernel, dim3(grid), dim3(ELEM_THREADS), 0, st, pl, expert_counts, dbg_expert_idx, none, none); };
    if (pl.elem_kind == ELEM_ANY) {
        const int stride = geo_info(pl.geo).dm;
        if (dbg_expert_idx) hipLaunchKernelGGL(k_elem_any<true>, dim3(grid), dim3(ELEM_THREADS), 0, st, pl, stride, expert_counts, dbg_expert_idx, none, none);
        else hipLaunchKernelGGL(k_elem_any<false>, dim3(grid), dim3(ELEM_THREADS), 0, st, pl, stride, expert_counts, dbg_expert_idx, none, none);
    } else if (pl.geo == GEO_LARGE) {
        if (dbg_expert_idx) go(k_elem<GeoLarge, 16, true>);
        else go(k_elem<GeoLarge, 16, false>);
    } else if (pl.elem_kind == ELEM_FAST4) {
        if (dbg_expert_idx) go(k_elem<GeoDefault, 4, true>);
        else go(k_elem<GeoDefault, 4, false>);
    } else if (dbg_expert_idx) {
        go(k_elem<GeoDefault, 16, true>);
    } else {
        go(k_elem<GeoDefault, 16, false>);
    }
    SG_LAUNCH_CHECK("k_elem");
    return 0;
}

}  // namespace sg2
