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
// backward one).  One 128-lane workgroup owns one chunk; lane (j,p) owns
// column j and RoPE pair p, i.e. the two states h[j][2p], h[j][2p+1].
//   k_scan<false>  every chunk but the last of a tensor: 2x2 affine summary
//                  (M,b) of the chunk, accumulated from the identity.
//   k_chunk_prefix start state of each chunk: summaries applied in order to
//                  the carried state of the tensor.
//   k_scan<true>   every chunk replayed from its start state: y = h.C, gate,
//                  D skip, out_proj, and the 8-float context written straight
//                  to the element's original position (the "unsort").  The
//                  last chunk stores the new carried state.
// Per-timestep projections (in_proj, dt, B, C) are recomputed in both passes
// for tiles of 64 timesteps and staged through LDS instead of being
// materialised in HBM (the reference writes 320 B per element per direction).
#include "sg2_internal.hpp"

namespace sg2 {
namespace {

constexpr int LDS_STRIDE = SCAN_TT + 1;   // [row][timestep] rows padded so the 8 rows a wave reads sit in 8 banks

struct DirW {
    const float *in_proj, *dt_W, *dt_b, *Bp, *Cp, *A_log, *D, *rope, *out_proj;
};
__device__ __forceinline__ DirW dir_weights(const Sg2Weights& W, int dir) {
    const int b = dir ? W_B_INPROJ : W_F_INPROJ;
    return {W.w[b], W.w[b + 1], W.w[b + 2], W.w[b + 3], W.w[b + 4], W.w[b + 5], W.w[b + 6], W.w[b + 7], W.w[b + 8]};
}

__device__ __forceinline__ float dpp_quad_swap1(float v) {   // lane ^ 1
    return sg_i2f(__builtin_amdgcn_update_dpp(0, sg_f2i(v), 0xB1, 0xF, 0xF, true));
}
__device__ __forceinline__ float dpp_quad_swap2(float v) {   // lane ^ 2
    return sg_i2f(__builtin_amdgcn_update_dpp(0, sg_f2i(v), 0x4E, 0xF, 0xF, true));
}
__device__ __forceinline__ float dpp_half_mirror(float v) {  // lane -> 7 - lane within each group of 8
    return sg_i2f(__builtin_amdgcn_update_dpp(0, sg_f2i(v), 0x141, 0xF, 0xF, true));
}


// Projections of one timestep (x = projected input, 8 floats).  Both halves of
// the workgroup compute the 16 x-branch values; each then produces its half
// of dt / B (/ C / gate) and publishes its half of the x-branch rows.  HALF is
// a template parameter so that every weight index is a compile-time constant
// (scalar loads) and the register array is never indexed dynamically.
template <bool OUT, int HALF>
__device__ __forceinline__ void project_tile(const DirW& w, const float (&x)[DM], int tu, float* s_dt, float* s_xb,
                                             float* s_B, float* s_C, float* s_gate) {
    float xb[DI];
#pragma unroll
    for (int jj = 0; jj < DI; jj++) {
        float a = 0.0f;
#pragma unroll
        for (int k = 0; k < DM; k++) a = sg_fma(w.in_proj[jj * DM + k], x[k], a);
        xb[jj] = a;
    }
#pragma unroll
    for (int q = 0; q < DI / 2; q++) {
        constexpr int base = HALF * (DI / 2);
        const int jj = base + q;
        float a = w.dt_b[jj];
#pragma unroll
        for (int k = 0; k < DI; k++) a = sg_fma(w.dt_W[jj * DI + k], xb[k], a);
        s_dt[jj * LDS_STRIDE + tu] = sg_softplus(a);
        s_xb[jj * LDS_STRIDE + tu] = xb[jj];
    }
#pragma unroll
    for (int q = 0; q < DS / 2; q++) {
        const int ss = HALF * (DS / 2) + q;
        float a = 0.0f;
#pragma unroll
        for (int k = 0; k < DI; k++) a = sg_fma(w.Bp[ss * DI + k], xb[k], a);
        s_B[ss * LDS_STRIDE + tu] = a;
        if (OUT) {
            float b = 0.0f;
#pragma unroll
            for (int k = 0; k < DI; k++) b = sg_fma(w.Cp[ss * DI + k], xb[k], b);
            s_C[ss * LDS_STRIDE + tu] = b;
        }
    }
    if (OUT) {
#pragma unroll
        for (int q = 0; q < DI / 2; q++) {
            const int jj = HALF * (DI / 2) + q;
            float z = 0.0f;
#pragma unroll
            for (int k = 0; k < DM; k++) z = sg_fma(w.in_proj[(jj + DI) * DM + k], x[k], z);
            s_gate[jj * LDS_STRIDE + tu] = sg_silu(z);
        }
    }
}

template <bool OUT>
__global__ __launch_bounds__(SCAN_THREADS) void k_scan(Plan pl) {
    __shared__ float s_dt[DI * LDS_STRIDE];
    __shared__ float s_xb[DI * LDS_STRIDE];
    __shared__ float s_B[DS * LDS_STRIDE];
    __shared__ float s_C[OUT ? DS * LDS_STRIDE : 1];
    __shared__ float s_gate[OUT ? DI * LDS_STRIDE : 1];
    __shared__ float s_y[OUT ? DI * LDS_STRIDE : 1];

    const int per_dir = OUT ? pl.chunks : pl.wchunks;
    const int dir = (int)blockIdx.x >= per_dir ? 1 : 0;
    const int cidx = (int)blockIdx.x - dir * per_dir;
    const int* __restrict__ prefix = OUT ? pl.chunk_prefix : pl.wchunk_prefix;
    const int ti = sg::upper_seg(prefix, pl.P, cidx);
    const int c = cidx - prefix[ti];                       // chunk within the tensor
    const TensorDev& T = pl.tensors[ti];
    const int N = T.numel, dtype = T.dtype, off = T.off;
    const int u0 = c * pl.chunk_len;                       // first scan step of the chunk
    const int u1 = min(u0 + pl.chunk_len, N);
    const DirW w = dir_weights(pl.W, dir);
    const int32_t* __restrict__ perm = pl.vals[0] + off;

    const int tid = threadIdx.x;
    const int tu = tid & (SCAN_TT - 1);                                   // projection role: timestep of the tile
    const int half = __builtin_amdgcn_readfirstlane(tid >> 6);           // projection role: which half of the outputs
    const int j = tid >> 3, p = tid & 7;                                  // scan role

    const float hAe = 0.5f * -sg_exp(w.A_log[j * DS + 2 * p]);
    const float hAo = 0.5f * -sg_exp(w.A_log[j * DS + 2 * p + 1]);
    const float freq = w.rope[j * HP + p];

    // scan state: OUT -> (he,ho);  summary -> columns (c0e,c0o),(c1e,c1o) and offset (be,bo)
    float he, ho, c0e = 1.0f, c0o = 0.0f, c1e = 0.0f, c1o = 1.0f;
    if (OUT) {
        const float* hs = pl.hstart + ((size_t)(dir * pl.chunks + cidx) * 2) * SCAN_THREADS;
        he = hs[tid];
        ho = hs[SCAN_THREADS + tid];
    } else {
        he = 0.0f;
        ho = 0.0f;
    }

    for (int tile0 = u0; tile0 < u1; tile0 += SCAN_TT) {
        const int cnt = min(SCAN_TT, u1 - tile0);
        // ---------------- phase A: projections of SCAN_TT timesteps -> LDS
        const int u = tile0 + tu;
        const bool valid = u < u1;
        int orig = 0;
        float x[DM];
        {
            float g = 0.0f, s = 0.0f;
            if (valid) {
                const int t = dir ? (N - 1 - u) : u;
                orig = perm[t];
                orig = ((unsigned)orig < (unsigned)N) ? orig : 0;   // never index outside the tensor
                g = sg::finite_or_zero(sg::load_elem(T.grad, dtype, orig));
                s = sg::finite_or_zero(sg::load_elem(T.sharp, dtype, orig));
            }
            const float* __restrict__ Wi = pl.W.w[W_IN_W];
            const float* __restrict__ bi = pl.W.w[W_IN_B];
#pragma unroll
            for (int k = 0; k < DM; k++) x[k] = sg_fma(Wi[2 * k + 1], s, Wi[2 * k] * g) + bi[k];
        }
        if (half == 0)
            project_tile<OUT, 0>(w, x, tu, s_dt, s_xb, s_B, s_C, s_gate);
        else
            project_tile<OUT, 1>(w, x, tu, s_dt, s_xb, s_B, s_C, s_gate);
        __syncthreads();

        // ---------------- phase B: the recurrence over the tile, lane = (j,p)
        const float* __restrict__ r_dt = s_dt + j * LDS_STRIDE;
        const float* __restrict__ r_xb = s_xb + j * LDS_STRIDE;
        const float* __restrict__ r_Be = s_B + (2 * p) * LDS_STRIDE;
        const float* __restrict__ r_Bo = s_B + (2 * p + 1) * LDS_STRIDE;
        const float* __restrict__ r_Ce = s_C + (OUT ? (2 * p) * LDS_STRIDE : 0);
        const float* __restrict__ r_Co = s_C + (OUT ? (2 * p + 1) * LDS_STRIDE : 0);
#pragma unroll 4
        for (int k = 0; k < cnt; k++) {
            const float dt = r_dt[k], xv = r_xb[k];
            float ae, ao, sn, cs;
            sg_abar_pair(dt, hAe, hAo, &ae, &ao);
            sg_sincos(dt * freq, &sn, &cs);
            const float be = (dt * r_Be[k]) * xv, bo = (dt * r_Bo[k]) * xv;
            if (OUT) {
                const float re = sg_fma(he, cs, -(ho * sn));
                const float ro = sg_fma(ho, cs, he * sn);
                he = sg_fma(ae, re, be);
                ho = sg_fma(ao, ro, bo);
                float y = sg_fma(ho, r_Co[k], he * r_Ce[k]);
                y = y + dpp_quad_swap1(y);
                y = y + dpp_quad_swap2(y);
                y = y + dpp_half_mirror(y);
                if (p == 0) s_y[j * LDS_STRIDE + k] = y;
            } else {
                float re = sg_fma(c0e, cs, -(c0o * sn)), ro = sg_fma(c0o, cs, c0e * sn);
                c0e = ae * re;
                c0o = ao * ro;
                re = sg_fma(c1e, cs, -(c1o * sn));
                ro = sg_fma(c1o, cs, c1e * sn);
                c1e = ae * re;
                c1o = ao * ro;
                re = sg_fma(he, cs, -(ho * sn));
                ro = sg_fma(ho, cs, he * sn);
                he = sg_fma(ae, re, be);
                ho = sg_fma(ao, ro, bo);
            }
        }
        __syncthreads();

        // ---------------- phase C: gate, D skip, out_proj, scatter to element order
        if (OUT) {
            float o[DI];
#pragma unroll
            for (int jj = 0; jj < DI; jj++)
                o[jj] = sg_fma(s_y[jj * LDS_STRIDE + tu], s_gate[jj * LDS_STRIDE + tu],
                               w.D[jj] * s_xb[jj * LDS_STRIDE + tu]);
            float cx[DM / 2];
#pragma unroll
            for (int q = 0; q < DM / 2; q++) {
                const int dd = half * (DM / 2) + q;
                float a = 0.0f;
#pragma unroll
                for (int jj = 0; jj < DI; jj++) a = sg_fma(w.out_proj[dd * DI + jj], o[jj], a);
                cx[q] = a;
            }
            if (valid) {
                float4* dst = reinterpret_cast<float4*>(pl.ctx + ((size_t)dir * pl.total + off + orig) * DM) + half;
                *dst = make_float4(cx[0], cx[1], cx[2], cx[3]);
            }
            __syncthreads();
        }
    }

    if (OUT) {
        if (u1 == N) {   // last chunk in scan order: new carried state of the tensor
            float* st = dir ? T.mbwd : T.mfwd;
            st[j * DS + 2 * p] = he;
            st[j * DS + 2 * p + 1] = ho;
        }
    } else {
        float* sm = pl.summaries + (size_t)(dir * pl.wchunks + cidx) * 6 * SCAN_THREADS;
        sm[0 * SCAN_THREADS + tid] = c0e;   // M = [c0e c1e; c0o c1o]
        sm[1 * SCAN_THREADS + tid] = c0o;
        sm[2 * SCAN_THREADS + tid] = c1e;
        sm[3 * SCAN_THREADS + tid] = c1o;
        sm[4 * SCAN_THREADS + tid] = he;
        sm[5 * SCAN_THREADS + tid] = ho;
    }
}

// start state of every chunk: h_{c+1} = M_c h_c + b_c, from the carried state
__global__ __launch_bounds__(SCAN_THREADS) void k_chunk_prefix(Plan pl) {
    const int ti = blockIdx.x % pl.P, dir = blockIdx.x / pl.P;
    const TensorDev& T = pl.tensors[ti];
    if (T.numel == 0) return;
    const int tid = threadIdx.x, j = tid >> 3, p = tid & 7;
    const float* st = dir ? T.mbwd : T.mfwd;
    float he = st[j * DS + 2 * p], ho = st[j * DS + 2 * p + 1];
    float* hs = pl.hstart + ((size_t)(dir * pl.chunks + pl.chunk_prefix[ti]) * 2) * SCAN_THREADS;
    const float* sm = pl.summaries + (size_t)(dir * pl.wchunks + pl.wchunk_prefix[ti]) * 6 * SCAN_THREADS;
    hs[tid] = he;
    hs[SCAN_THREADS + tid] = ho;
    const int nc = T.nchunks;
#pragma unroll 4
    for (int c = 0; c + 1 < nc; c++) {
        const float* m = sm + (size_t)c * 6 * SCAN_THREADS;
        const float m0 = m[tid], m1 = m[SCAN_THREADS + tid], m2 = m[2 * SCAN_THREADS + tid];
        const float m3 = m[3 * SCAN_THREADS + tid], m4 = m[4 * SCAN_THREADS + tid], m5 = m[5 * SCAN_THREADS + tid];
        const float ne = sg_fma(m0, he, sg_fma(m2, ho, m4));
        const float no = sg_fma(m1, he, sg_fma(m3, ho, m5));
        he = ne;
        ho = no;
        float* h1 = hs + (size_t)(c + 1) * 2 * SCAN_THREADS;
        h1[tid] = he;
        h1[SCAN_THREADS + tid] = ho;
    }
}

}  // namespace

int launch_scan(const Plan& pl, hipStream_t st) {
    if (pl.total == 0) return 0;
    if (pl.wchunks > 0) {
        hipLaunchKernelGGL(k_scan<false>, dim3(2 * pl.wchunks), dim3(SCAN_THREADS), 0, st, pl);
        SG_LAUNCH_CHECK("k_scan<summary>");
    }
    prof_mark(2, st);
    hipLaunchKernelGGL(k_chunk_prefix, dim3(2 * pl.P), dim3(SCAN_THREADS), 0, st, pl);
    SG_LAUNCH_CHECK("k_chunk_prefix");
    prof_mark(3, st);
    hipLaunchKernelGGL(k_scan<true>, dim3(2 * pl.chunks), dim3(SCAN_THREADS), 0, st, pl);
    SG_LAUNCH_CHECK("k_scan<out>");
    prof_mark(4, st);
    return 0;
}

}  // namespace sg2
