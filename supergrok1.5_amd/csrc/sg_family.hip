// The reference's remaining fused optimizer steps: GrokAdamW, NeuralGrok,
// Prodigy, Lion, SuperGrok v1.1 and the LookSAM helpers.  Replaces the bodies of
// grokadamw_fused_step, neuralgrok_fused_step, prodigy_fused_step,
// lion_fused_step, supergrok11_fused_step and looksam_* of the reference's
// csrc/ops.cpp:209-656 with their per-optimizer kernels.
//
// Same batching as the other elementwise steps: one launch per stage covers
// every tensor (tile of 4096 elements -> tensor by binary search in a prefix
// table).  Everything the reference reads back to the host between stages -
// the global gradient norm, Prodigy's numerator/denominator, v1.1's cosine
// gate per tensor, LookSAM's per-tensor norms - is reduced on the device
// (per-tile partial sums in double, one block per result) and consumed from
// device memory by the next kernel, so a step enqueues without a host sync.
#include "sg_elemwise.hpp"

namespace sgew {
namespace {

struct FamRec {
    void* param;
    void* grad;
    float* ea;
    float* easq;
    float* aux;
    const void* aux2;
    float* smart;          // v1.1: this tensor's slice of the smart-gradient scratch
    int64_t numel;
    int32_t dtype;
    float bc1, bc2, alpha, beta1;
    int32_t vec4;          // fp32 tensor and every pointer 16-byte aligned: four elements per lane and access
};

typedef float f32x4 __attribute__((ext_vector_type(4)));
__device__ __forceinline__ f32x4 ld4(const void* p, int i) { return *(const SG_GLOBAL f32x4*)(static_cast<const float*>(p) + i); }
__device__ __forceinline__ void st4(void* p, int i, f32x4 v) { *(SG_GLOBAL f32x4*)(static_cast<float*>(p) + i) = v; }

// Runs body(i) for every element of the tile; when the tensor allows 16-byte accesses, body4(i) handles four
// consecutive elements per lane and body(i) only the ragged end.
template <class B1, class B4>
__device__ __forceinline__ void for_tile(const FamRec& R, int start, int cnt, B1 body, B4 body4) {
    int done = 0;
    if (R.vec4) {
        done = cnt & ~3;
        for (int k = threadIdx.x * 4; k < done; k += THREADS * 4) body4(start + k);
    }
    for (int k = done + threadIdx.x; k < cnt; k += THREADS) body(start + k);
}

// clipped gradient, written back in place when clipping is active (clip_grad_norms_device_side, csrc/ops.cpp:23-55)
__device__ __forceinline__ float clipped_grad(const FamRec& R, int i, bool clip_on, float coef) {
    float g = sg::load_elem(R.grad, R.dtype, i);
    if (clip_on) {
        sg::store_elem(R.grad, R.dtype, i, g * coef);
        g = (R.dtype == SG_F32) ? g * coef : sg::load_elem(R.grad, R.dtype, i);
    }
    return g;
}
__device__ __forceinline__ f32x4 clipped_grad4(const FamRec& R, int i, bool clip_on, float coef) {
    f32x4 g = ld4(R.grad, i);
    if (clip_on) {
        g = g * coef;
        st4(R.grad, i, g);
    }
    return g;
}

// decoupled decay, then the Adam step: p*(1 - lr*wd) - (lr/bc1) * ea / (sqrt(easq/bc2) + eps)
__device__ __forceinline__ float adam_core(float fg, float p, float& ea, float& easq, float beta1, float beta2, float bc2,
                                           float eps_eff, float decay, float step_size) {
    ea = sg_fma(beta1, ea, (1.0f - beta1) * fg);
    easq = sg_fma(beta2, easq, ((1.0f - beta2) * fg) * fg);
    const float denom = __builtin_sqrtf(easq / bc2) + eps_eff;
    return sg_fma(p, decay, -((step_size * ea) / denom));
}
__device__ __forceinline__ void adam_update(const FamRec& R, int i, float fg, float beta1, float beta2, float eps_eff, float decay,
                                            float step_size) {
    float ea = R.ea[i], easq = R.easq[i];
    const float p = adam_core(fg, sg::load_elem(R.param, R.dtype, i), ea, easq, beta1, beta2, R.bc2, eps_eff, decay, step_size);
    R.ea[i] = ea;
    R.easq[i] = easq;
    sg::store_elem(R.param, R.dtype, i, p);
}
__device__ __forceinline__ void adam_update4(const FamRec& R, int i, f32x4 fg, float beta1, float beta2, float eps_eff, float decay,
                                             float step_size) {
    f32x4 ea = ld4(R.ea, i), easq = ld4(R.easq, i), p = ld4(R.param, i);
#pragma unroll
    for (int c = 0; c < 4; c++) {
        float a = ea[c], q = easq[c];
        p[c] = adam_core(fg[c], p[c], a, q, beta1, beta2, R.bc2, eps_eff, decay, step_size);
        ea[c] = a;
        easq[c] = q;
    }
    st4(R.ea, i, ea);
    st4(R.easq, i, easq);
    st4(R.param, i, p);
}

__global__ __launch_bounds__(THREADS) void k_grokadamw(Batch<FamRec> B, float alpha, float lamb, float beta1, float beta2, float lr,
                                                        float eps, float decay) {
    int start, cnt;
    const FamRec& R = tile_rec(B, blockIdx.x, &start, &cnt);
    const float coef = B.red->coef;
    const bool clip_on = B.red->clip_on != 0;
    const float step_size = lr / R.bc1;
    for_tile(R, start, cnt,
        [&](int i) {
            const float g = clipped_grad(R, i, clip_on, coef);
            float fg = g;
            if (R.aux) {        // no EMA buffer: plain AdamW
                const float e = sg_fma(alpha, R.aux[i], (1.0f - alpha) * g);
                R.aux[i] = e;
                fg = sg_fma(lamb, e, g);
            }
            adam_update(R, i, fg, beta1, beta2, eps, decay, step_size);
        },
        [&](int i) {
            const f32x4 g = clipped_grad4(R, i, clip_on, coef);
            f32x4 fg = g;
            if (R.aux) {
                f32x4 e = ld4(R.aux, i);
#pragma unroll
                for (int c = 0; c < 4; c++) {
                    e[c] = sg_fma(alpha, e[c], (1.0f - alpha) * g[c]);
                    fg[c] = sg_fma(lamb, e[c], g[c]);
                }
                st4(R.aux, i, e);
            }
            adam_update4(R, i, fg, beta1, beta2, eps, decay, step_size);
        });
}

__global__ __launch_bounds__(THREADS) void k_neuralgrok(Batch<FamRec> B, const float* __restrict__ W1, const float* __restrict__ b1,
                                                         const float* __restrict__ W2, const float* __restrict__ b2, int H,
                                                         float alpha_amp, float beta_amp, float beta1, float beta2, float lr,
                                                         float eps, float decay) {
    __shared__ float sW1[MAX_HIDDEN], sb1[MAX_HIDDEN], sW2[MAX_HIDDEN];
    for (int k = threadIdx.x; k < H; k += THREADS) { sW1[k] = W1[k]; sb1[k] = b1[k]; sW2[k] = W2[k]; }
    __syncthreads();
    const float bias2 = b2[0];
    int start, cnt;
    const FamRec& R = tile_rec(B, blockIdx.x, &start, &cnt);
    const float coef = B.red->coef;
    const bool clip_on = B.red->clip_on != 0;
    const float step_size = lr / R.bc1;
    for (int k = threadIdx.x; k < cnt; k += THREADS) {
        const int i = start + k;
        const float g = clipped_grad(R, i, clip_on, coef);
        float acc = 0.0f;
        for (int h = 0; h < H; h++) acc = sg_fma(sW2[h], sg_max(sg_fma(sW1[h], g, sb1[h]), 0.0f), acc);
        const float ag = g * sg_fma(alpha_amp, acc + bias2, beta_amp);
        adam_update(R, i, ag, beta1, beta2, eps, decay, step_size);
    }
}

__device__ __forceinline__ void lion_core(float g, float& m, float& p, float lr, float beta1, float beta2, float wd) {
    const float interp = sg_fma(beta1, m, (1.0f - beta1) * g);
    const float s = interp > 0.0f ? 1.0f : (interp < 0.0f ? -1.0f : 0.0f);
    p = sg_fma(-lr, sg_fma(wd, p, s), p);
    m = sg_fma(beta2, m, (1.0f - beta2) * g);
}
__global__ __launch_bounds__(THREADS) void k_lion(Batch<FamRec> B, float lr, float beta1, float beta2, float wd) {
    int start, cnt;
    const FamRec& R = tile_rec(B, blockIdx.x, &start, &cnt);
    for_tile(R, start, cnt,
        [&](int i) {
            float m = R.ea[i], p = sg::load_elem(R.param, R.dtype, i);
            lion_core(sg::load_elem(R.grad, R.dtype, i), m, p, lr, beta1, beta2, wd);
            sg::store_elem(R.param, R.dtype, i, p);
            R.ea[i] = m;
        },
        [&](int i) {
            const f32x4 g = ld4(R.grad, i);
            f32x4 m = ld4(R.ea, i), p = ld4(R.param, i);
#pragma unroll
            for (int c = 0; c < 4; c++) {
                float mc = m[c], pc = p[c];
                lion_core(g[c], mc, pc, lr, beta1, beta2, wd);
                m[c] = mc;
                p[c] = pc;
            }
            st4(R.param, i, p);
            st4(R.ea, i, m);
        });
}

// ---- reductions: up to three sums per tile, then one block per tensor (or one for the call) -------------
__device__ __forceinline__ void tile_sums(const Batch<FamRec>& B, double a, double b, double c) {
    __shared__ double sm[4];
    const double ta = block_sum(a, sm), tb = block_sum(b, sm), tc = block_sum(c, sm);
    if (threadIdx.x == 0) {
        B.partials[3 * (size_t)blockIdx.x + 0] = ta;
        B.partials[3 * (size_t)blockIdx.x + 1] = tb;
        B.partials[3 * (size_t)blockIdx.x + 2] = tc;
    }
}

// per_tensor != 0: block t sums the tiles of tensor t into tred[t]; else one block sums every tile into tred[0]
__global__ __launch_bounds__(THREADS) void k_sum_tiles(Batch<FamRec> B, int per_tensor) {
    __shared__ double sm[4];
    const int t = blockIdx.x;
    const int lo = per_tensor ? B.prefix[t] : 0, hi = per_tensor ? B.prefix[t + 1] : B.tiles;
    double a = 0.0, b = 0.0, c = 0.0;
    for (int k = lo + (int)threadIdx.x; k < hi; k += THREADS) {
        a += B.partials[3 * (size_t)k];
        b += B.partials[3 * (size_t)k + 1];
        c += B.partials[3 * (size_t)k + 2];
    }
    const double ta = block_sum(a, sm), tb = block_sum(b, sm), tc = block_sum(c, sm);
    if (threadIdx.x == 0) {
        B.tred[t].s[0] = ta;
        B.tred[t].s[1] = tb;
        B.tred[t].s[2] = tc;
    }
}

// ---- Prodigy ------------------------------------------------------------------------------------------
__global__ __launch_bounds__(THREADS) void k_prodigy_partial(Batch<FamRec> B) {
    int start, cnt;
    const FamRec& R = tile_rec(B, blockIdx.x, &start, &cnt);
    const float* p0 = static_cast<const float*>(R.aux2);
    float num = 0.0f, den = 0.0f;
    for_tile(R, start, cnt,
        [&](int i) {
            num = sg_fma(sg::load_elem(R.grad, R.dtype, i), sg::load_elem(R.param, R.dtype, i) - p0[i], num);
            den += R.aux[i];
        },
        [&](int i) {
            const f32x4 g = ld4(R.grad, i), p = ld4(R.param, i), q = ld4(p0, i), sv = ld4(R.aux, i);
#pragma unroll
            for (int c = 0; c < 4; c++) {
                num = sg_fma(g[c], p[c] - q[c], num);
                den += sv[c];
            }
        });
    tile_sums(B, (double)num, (double)den, 0.0);
}

__global__ void k_prodigy_dlr(Batch<FamRec> B, float d_lr) {
    if (threadIdx.x != 0 || blockIdx.x != 0) return;
    const float num = (float)B.tred[0].s[0], den = (float)B.tred[0].s[1];
    if (den > 1e-30f) d_lr = sg_max(d_lr, sg_abs(num) / (den + 1e-12f));
    B.tred[0].d_lr = d_lr;
}

__global__ __launch_bounds__(THREADS) void k_prodigy(Batch<FamRec> B, float beta1, float beta2, float lr, float wd, float eps) {
    int start, cnt;
    const FamRec& R = tile_rec(B, blockIdx.x, &start, &cnt);
    const float d_lr = B.tred[0].d_lr;
    const float decay = 1.0f - (lr * d_lr) * wd, step_size = lr / R.bc1, eps_eff = d_lr * eps;
    for_tile(R, start, cnt,
        [&](int i) {
            const float dg = d_lr * sg::load_elem(R.grad, R.dtype, i);
            R.aux[i] = sg_fma(beta2, R.aux[i], ((1.0f - beta2) * dg) * dg);
            adam_update(R, i, dg, beta1, beta2, eps_eff, decay, step_size);
        },
        [&](int i) {
            f32x4 dg = ld4(R.grad, i), sv = ld4(R.aux, i);
#pragma unroll
            for (int c = 0; c < 4; c++) {
                dg[c] = d_lr * dg[c];
                sv[c] = sg_fma(beta2, sv[c], ((1.0f - beta2) * dg[c]) * dg[c]);
            }
            st4(R.aux, i, sv);
            adam_update4(R, i, dg, beta1, beta2, eps_eff, decay, step_size);
        });
}

// ---- SuperGrok v1.1 -------------------------------------------------------------------------------------
template <int GELU>
__global__ __launch_bounds__(THREADS) void k_sg11_smart(Batch<FamRec> B, const float* __restrict__ W1, const float* __restrict__ b1,
                                                         const float* __restrict__ W2, const float* __restrict__ b2, int H,
                                                         float rescale) {
    __shared__ float sW1[2 * MAX_HIDDEN], sb1[MAX_HIDDEN], sW2[MAX_HIDDEN];
    for (int k = threadIdx.x; k < 2 * H; k += THREADS) sW1[k] = W1[k];
    for (int k = threadIdx.x; k < H; k += THREADS) { sb1[k] = b1[k]; sW2[k] = W2[k]; }
    __syncthreads();
    const float bias2 = b2[0];
    int start, cnt;
    const FamRec& R = tile_rec(B, blockIdx.x, &start, &cnt);
    const float coef = B.red->coef;
    const bool clip_on = B.red->clip_on != 0;
    const float alpha = R.alpha;
    float dot = 0.0f, ss = 0.0f, mm = 0.0f;
    for (int k = threadIdx.x; k < cnt; k += THREADS) {
        const int i = start + k;
        const float g = clipped_grad(R, i, clip_on, coef);
        const float s = sg::load_elem(R.aux2, R.dtype, i);
        const float mu = sg_fma(alpha, R.aux[i], (1.0f - alpha) * g);
        R.aux[i] = mu;
        float acc = 0.0f;
        for (int h = 0; h < H; h++) {
            const float z = sg_fma(sW1[2 * h + 1], s, sW1[2 * h] * g) + sb1[h];
            acc = sg_fma(sW2[h], (GELU == 0) ? sg_gelu_erf(z) : sg_gelu_sigmoid(z), acc);
        }
        const float smart = sg_fma(rescale, acc + bias2, g);
        R.smart[i] = smart;
        dot = sg_fma(smart, mu, dot);
        ss = sg_fma(smart, smart, ss);
        mm = sg_fma(mu, mu, mm);
    }
    tile_sums(B, (double)dot, (double)ss, (double)mm);
}

__global__ __launch_bounds__(THREADS) void k_sg11_adam(Batch<FamRec> B, float beta2, float lr, float eps, float decay, float lamb,
                                                        float ramp, float temperature) {
    int start, cnt;
    const int ti = sg::upper_seg(B.prefix, B.n, (int)blockIdx.x);
    const FamRec& R = tile_rec(B, blockIdx.x, &start, &cnt);
    // cosine gate of this tensor (compute_cosine_gate_fused; csrc/ops.cpp:272-278)
    const TRed& T = B.tred[ti];
    const float cosv = (float)T.s[0] / ((float)sqrt(T.s[1]) * (float)sqrt(T.s[2]) + 1e-8f);
    const float gate = 1.0f / (1.0f + sg_exp(-temperature * cosv));
    const float lamb_eff = ramp > 0.0f ? (ramp * gate) * lamb : 0.0f;
    const float step_size = lr / R.bc1;
    for (int k = threadIdx.x; k < cnt; k += THREADS) {
        const int i = start + k;
        adam_update(R, i, sg_fma(lamb_eff, R.aux[i], R.smart[i]), R.beta1, beta2, eps, decay, step_size);
    }
}

// ---- LookSAM ----------------------------------------------------------------------------------------------
// FamRec roles: restore  param=param, aux2=backup;  directions  aux=v (fp32), grad=sam_grad, aux2=normal_grad;
//               adjust   grad=grad, aux=v (fp32)
__global__ __launch_bounds__(THREADS) void k_ls_restore(Batch<FamRec> B) {
    int start, cnt;
    const FamRec& R = tile_rec(B, blockIdx.x, &start, &cnt);
    for (int k = threadIdx.x; k < cnt; k += THREADS) sg::store_elem(R.param, R.dtype, start + k, sg::load_elem(R.aux2, R.dtype, start + k));
}

// difference as the reference forms it: subtracted in the gradients' own type, then widened
__device__ __forceinline__ float ls_diff(const FamRec& R, int i) {
    const float d = sg::load_elem(R.grad, R.dtype, i) - sg::load_elem(R.aux2, R.dtype, i);
    if (R.dtype == SG_F16) return __half2float(__float2half_rn(d));
    if (R.dtype == SG_BF16) return sg::bf16_bits_to_f(sg::f_to_bf16_bits(d));
    return d;
}

__global__ __launch_bounds__(THREADS) void k_ls_diff_sumsq(Batch<FamRec> B) {
    int start, cnt;
    const FamRec& R = tile_rec(B, blockIdx.x, &start, &cnt);
    float acc = 0.0f;
    for (int k = threadIdx.x; k < cnt; k += THREADS) {
        const float d = ls_diff(R, start + k);
        acc = sg_fma(d, d, acc);
    }
    tile_sums(B, (double)acc, 0.0, 0.0);
}

__global__ __launch_bounds__(THREADS) void k_ls_direction(Batch<FamRec> B) {
    int start, cnt;
    const int ti = sg::upper_seg(B.prefix, B.n, (int)blockIdx.x);
    const FamRec& R = tile_rec(B, blockIdx.x, &start, &cnt);
    const float norm = (float)sqrt(B.tred[ti].s[0]);
    if (!(norm >= 1e-12f)) return;          // that tensor's direction stays as it was
    const float inv = 1.0f / norm;
    for (int k = threadIdx.x; k < cnt; k += THREADS) {
        const int i = start + k;
        // the device branch widens both gradients before subtracting (csrc/ops.cpp:621-623)
        R.aux[i] = (sg::load_elem(R.grad, R.dtype, i) - sg::load_elem(R.aux2, R.dtype, i)) * inv;
    }
}

__global__ __launch_bounds__(THREADS) void k_ls_grad_sumsq(Batch<FamRec> B) {
    int start, cnt;
    const FamRec& R = tile_rec(B, blockIdx.x, &start, &cnt);
    float acc = 0.0f;
    for (int k = threadIdx.x; k < cnt; k += THREADS) {
        const float g = sg::load_elem(R.grad, R.dtype, start + k);
        acc = sg_fma(g, g, acc);
    }
    tile_sums(B, (double)acc, 0.0, 0.0);
}

__global__ __launch_bounds__(THREADS) void k_ls_adjust(Batch<FamRec> B, float la) {
    int start, cnt;
    const int ti = sg::upper_seg(B.prefix, B.n, (int)blockIdx.x);
    const FamRec& R = tile_rec(B, blockIdx.x, &start, &cnt);
    const float scale = la * (float)sqrt(B.tred[ti].s[0]);
    for (int k = threadIdx.x; k < cnt; k += THREADS) {
        const int i = start + k;
        float v = R.aux[i];                  // the direction is converted to the gradient's type first (csrc/ops.cpp:646)
        if (R.dtype == SG_F16) v = __half2float(__float2half_rn(v));
        if (R.dtype == SG_BF16) v = sg::bf16_bits_to_f(sg::f_to_bf16_bits(v));
        sg::store_elem(R.grad, R.dtype, i, sg_fma(scale, v, sg::load_elem(R.grad, R.dtype, i)));
    }
}

// ---- SuperGrok v2 pre-pass: per-tensor norm clip + non-finite guard ------------------------------------------
// FamRec roles: grad = input gradient, param = output (a new tensor, as the reference makes one)
__global__ __launch_bounds__(THREADS) void k_sg2_clip(Batch<FamRec> B, float max_norm) {
    int start, cnt;
    const int ti = sg::upper_seg(B.prefix, B.n, (int)blockIdx.x);
    const FamRec& R = tile_rec(B, blockIdx.x, &start, &cnt);
    // a NaN norm compares false (no clip); an infinite one gives scale 0 and the guard below zeroes what 0*inf leaves
    const float norm = (float)sqrt(B.tred[ti].s[0]);
    const float scale = (norm > max_norm) ? max_norm / (norm + 1e-12f) : 1.0f;
    for (int k = threadIdx.x; k < cnt; k += THREADS) {
        const int i = start + k;
        float g = sg::load_elem(R.grad, R.dtype, i);
        if (scale != 1.0f) {
            g = g * scale;
            if (R.dtype == SG_F16) g = __half2float(__float2half_rn(g));        // the product is a tensor of the gradient's type
            if (R.dtype == SG_BF16) g = sg::bf16_bits_to_f(sg::f_to_bf16_bits(g));
        }
        sg::store_elem(R.param, R.dtype, i, sg::finite_or_zero(g));
    }
}

// ---- host side ---------------------------------------------------------------------------------------------
enum Need { N_PARAM = 1, N_GRAD = 2, N_EA = 4, N_EASQ = 8, N_AUX = 16, N_AUX2 = 32 };

int collect(int n, const SgFamilyTensor* ts, int need, std::vector<FamRec>* recs) {
    if (!ts) return sg::fail("NULL argument");
    for (int i = 0; i < n; i++) {
        const SgFamilyTensor& t = ts[i];
        if (t.numel == 0) continue;
        if (((need & N_PARAM) && !t.param) || ((need & N_GRAD) && !t.grad) || ((need & N_EA) && !t.exp_avg) ||
            ((need & N_EASQ) && !t.exp_avg_sq) || ((need & N_AUX) && !t.aux) || ((need & N_AUX2) && !t.aux2))
            return sg::fail("tensor %d: NULL pointer", i);
        if (check_dtype(i, t.dtype)) return 1;
        const uintptr_t all = (uintptr_t)t.param | (uintptr_t)t.grad | (uintptr_t)t.exp_avg | (uintptr_t)t.exp_avg_sq | (uintptr_t)t.aux |
                              (uintptr_t)t.aux2;
        recs->push_back({t.param, t.grad, t.exp_avg, t.exp_avg_sq, t.aux, t.aux2, nullptr, t.numel, t.dtype, t.bc1, t.bc2, t.alpha, t.beta1,
                         (t.dtype == SG_F32 && (all & 15u) == 0) ? 1 : 0});
    }
    return 0;
}

int check_bc(const std::vector<FamRec>& recs) {
    for (size_t i = 0; i < recs.size(); i++)
        if (!(recs[i].bc1 > 0.0f) || !(recs[i].bc2 > 0.0f)) return sg::fail("bias corrections must be positive (step >= 1)");
    return 0;
}

int looksam_collect(int n, const SgLookSamTensor* ts, int mode, std::vector<FamRec>* recs) {
    if (!ts) return sg::fail("NULL argument");
    for (int i = 0; i < n; i++) {
        const SgLookSamTensor& t = ts[i];
        if (t.numel == 0) continue;
        if (!t.a || !t.b || (mode == 1 && !t.c)) return sg::fail("tensor %d: NULL pointer", i);
        if (check_dtype(i, t.dtype)) return 1;
        FamRec r = {};
        r.numel = t.numel;
        r.dtype = t.dtype;
        if (mode == 0) { r.param = t.a; r.aux2 = t.b; }
        if (mode == 1) { r.aux = static_cast<float*>(t.a); r.grad = const_cast<void*>(t.b); r.aux2 = t.c; }
        if (mode == 2) { r.grad = t.a; r.aux = const_cast<float*>(static_cast<const float*>(t.b)); }
        recs->push_back(r);
    }
    return 0;
}

}  // namespace
}  // namespace sgew

extern "C" {

size_t sg_family_workspace_bytes(int num_tensors, const int64_t* numels) {
    if (num_tensors < 0 || (num_tensors > 0 && !numels)) return 0;
    sgew::Layout L;
    if (sgew::make_layout(num_tensors, numels, &L)) return 0;
    return L.bytes + sizeof(float) * (size_t)L.total + 256;
}

int sg_grokadamw_step(int num_tensors, const SgFamilyTensor* tensors, float alpha, float lamb, float beta1, float beta2, float lr,
                      float wd, float eps, float grad_clip_norm, void* workspace, size_t workspace_bytes, void* stream) {
    using namespace sgew;
    if (num_tensors <= 0) return 0;
    std::vector<FamRec> recs;
    // the EMA buffer may be NULL for every tensor when lamb == 0: the step is then plain AdamW
    if (collect(num_tensors, tensors, N_PARAM | N_GRAD | N_EA | N_EASQ | (lamb != 0.0f ? N_AUX : 0), &recs) || check_bc(recs)) return 1;
    if (recs.empty()) return 0;
    hipStream_t st = (hipStream_t)stream;
    Batch<FamRec> B;
    if (upload(recs, workspace, workspace_bytes, st, &B)) return 1;
    if (reduce_sumsq(recs, B, grad_clip_norm, st)) return 1;
    hipLaunchKernelGGL(k_grokadamw, dim3(B.tiles), dim3(THREADS), 0, st, B, alpha, lamb, beta1, beta2, lr, eps, 1.0f - lr * wd);
    SG_LAUNCH_CHECK("k_grokadamw");
    return 0;
}

int sg_neuralgrok_step(int num_tensors, const SgFamilyTensor* tensors, const SgAmplifier* amp, float alpha_amp, float beta_amp,
                       float beta1, float beta2, float lr, float wd, float eps, float grad_clip_norm, void* workspace,
                       size_t workspace_bytes, void* stream) {
    using namespace sgew;
    if (num_tensors <= 0) return 0;
    if (!amp || !amp->W1 || !amp->b1 || !amp->W2 || !amp->b2) return sg::fail("NULL argument");
    if (amp->hidden < 1 || amp->hidden > MAX_HIDDEN) return sg::fail("hidden_dim %d outside [1,%d]", amp->hidden, MAX_HIDDEN);
    std::vector<FamRec> recs;
    if (collect(num_tensors, tensors, N_PARAM | N_GRAD | N_EA | N_EASQ, &recs) || check_bc(recs)) return 1;
    if (recs.empty()) return 0;
    hipStream_t st = (hipStream_t)stream;
    Batch<FamRec> B;
    if (upload(recs, workspace, workspace_bytes, st, &B)) return 1;
    if (reduce_sumsq(recs, B, grad_clip_norm, st)) return 1;
    hipLaunchKernelGGL(k_neuralgrok, dim3(B.tiles), dim3(THREADS), 0, st, B, amp->W1, amp->b1, amp->W2, amp->b2, amp->hidden, alpha_amp,
                       beta_amp, beta1, beta2, lr, eps, 1.0f - lr * wd);
    SG_LAUNCH_CHECK("k_neuralgrok");
    return 0;
}

int sg_prodigy_step(int num_tensors, const SgFamilyTensor* tensors, float d_lr, float beta1, float beta2, float lr, float wd, float eps,
                    float* d_lr_out, void* workspace, size_t workspace_bytes, void* stream) {
    using namespace sgew;
    if (d_lr_out) *d_lr_out = d_lr;
    if (num_tensors <= 0) return 0;
    std::vector<FamRec> recs;
    if (collect(num_tensors, tensors, N_PARAM | N_GRAD | N_EA | N_EASQ | N_AUX | N_AUX2, &recs) || check_bc(recs)) return 1;
    if (recs.empty()) return 0;
    hipStream_t st = (hipStream_t)stream;
    Batch<FamRec> B;
    if (upload(recs, workspace, workspace_bytes, st, &B)) return 1;
    hipLaunchKernelGGL(k_prodigy_partial, dim3(B.tiles), dim3(THREADS), 0, st, B);
    hipLaunchKernelGGL(k_sum_tiles, dim3(1), dim3(THREADS), 0, st, B, 0);
    hipLaunchKernelGGL(k_prodigy_dlr, dim3(1), dim3(64), 0, st, B, d_lr);
    hipLaunchKernelGGL(k_prodigy, dim3(B.tiles), dim3(THREADS), 0, st, B, beta1, beta2, lr, wd, eps);
    SG_LAUNCH_CHECK("k_prodigy");
    if (d_lr_out) {
        SG_HIP_CHECK(hipMemcpyAsync(d_lr_out, &B.tred[0].d_lr, sizeof(float), hipMemcpyDeviceToHost, st));
        SG_HIP_CHECK(hipStreamSynchronize(st));
    }
    return 0;
}

int sg_lion_step(int num_tensors, const SgFamilyTensor* tensors, float lr, float beta1, float beta2, float wd, void* workspace,
                 size_t workspace_bytes, void* stream) {
    using namespace sgew;
    if (num_tensors <= 0) return 0;
    std::vector<FamRec> recs;
    if (collect(num_tensors, tensors, N_PARAM | N_GRAD | N_EA, &recs)) return 1;
    if (recs.empty()) return 0;
    hipStream_t st = (hipStream_t)stream;
    Batch<FamRec> B;
    if (upload(recs, workspace, workspace_bytes, st, &B)) return 1;
    hipLaunchKernelGGL(k_lion, dim3(B.tiles), dim3(THREADS), 0, st, B, lr, beta1, beta2, wd);
    SG_LAUNCH_CHECK("k_lion");
    return 0;
}

int sg11_fused_step(int num_tensors, const SgFamilyTensor* tensors, const Sg15Net* net, float beta2, float lr, float wd, float eps,
                    float lamb, float ramp, float gate_temperature, float grad_clip_norm, void* workspace, size_t workspace_bytes,
                    void* stream) {
    using namespace sgew;
    if (num_tensors <= 0) return 0;
    if (!net || !net->W1 || !net->b1 || !net->W2 || !net->b2) return sg::fail("NULL argument");
    if (net->hidden < 1 || net->hidden > MAX_HIDDEN) return sg::fail("hidden_dim %d outside [1,%d]", net->hidden, MAX_HIDDEN);
    if (net->gelu_mode != 0 && net->gelu_mode != 1) return sg::fail("bad gelu_mode %d", net->gelu_mode);
    std::vector<FamRec> recs;
    if (collect(num_tensors, tensors, N_PARAM | N_GRAD | N_EA | N_EASQ | N_AUX | N_AUX2, &recs) || check_bc(recs)) return 1;
    if (recs.empty()) return 0;
    // the smart-gradient scratch follows the bookkeeping region
    std::vector<int64_t> numels(recs.size());
    for (size_t i = 0; i < recs.size(); i++) numels[i] = recs[i].numel;
    Layout L;
    if (make_layout((int)recs.size(), numels.data(), &L)) return 1;
    const size_t need = L.bytes + sizeof(float) * (size_t)L.total;
    if (!workspace || workspace_bytes < need) return sg::fail("workspace too small: need %zu bytes, got %zu", need, workspace_bytes);
    float* smart = reinterpret_cast<float*>(static_cast<unsigned char*>(workspace) + L.bytes);
    for (size_t i = 0; i < recs.size(); i++) { recs[i].smart = smart; smart += recs[i].numel; }
    hipStream_t st = (hipStream_t)stream;
    Batch<FamRec> B;
    if (upload(recs, workspace, workspace_bytes, st, &B)) return 1;
    if (reduce_sumsq(recs, B, grad_clip_norm, st)) return 1;
    if (net->gelu_mode == 0)
        hipLaunchKernelGGL(k_sg11_smart<0>, dim3(B.tiles), dim3(THREADS), 0, st, B, net->W1, net->b1, net->W2, net->b2, net->hidden, net->rescale);
    else
        hipLaunchKernelGGL(k_sg11_smart<1>, dim3(B.tiles), dim3(THREADS), 0, st, B, net->W1, net->b1, net->W2, net->b2, net->hidden, net->rescale);
    hipLaunchKernelGGL(k_sum_tiles, dim3(B.n), dim3(THREADS), 0, st, B, 1);
    hipLaunchKernelGGL(k_sg11_adam, dim3(B.tiles), dim3(THREADS), 0, st, B, beta2, lr, eps, 1.0f - lr * wd, lamb, ramp, gate_temperature);
    SG_LAUNCH_CHECK("k_sg11");
    return 0;
}

int sg2_clip_grads(int num_tensors, const Sg2ClipTensor* tensors, float max_norm, void* workspace, size_t workspace_bytes, void* stream) {
    using namespace sgew;
    if (num_tensors <= 0) return 0;
    if (!tensors) return sg::fail("NULL argument");
    std::vector<FamRec> recs;
    for (int i = 0; i < num_tensors; i++) {
        const Sg2ClipTensor& t = tensors[i];
        if (t.numel == 0) continue;
        if (!t.grad || !t.out) return sg::fail("tensor %d: NULL pointer", i);
        if (check_dtype(i, t.dtype)) return 1;
        FamRec r = {};
        r.grad = const_cast<void*>(t.grad);
        r.param = t.out;
        r.numel = t.numel;
        r.dtype = t.dtype;
        recs.push_back(r);
    }
    if (recs.empty()) return 0;
    hipStream_t st = (hipStream_t)stream;
    Batch<FamRec> B;
    if (upload(recs, workspace, workspace_bytes, st, &B)) return 1;
    hipLaunchKernelGGL(k_ls_grad_sumsq, dim3(B.tiles), dim3(THREADS), 0, st, B);
    hipLaunchKernelGGL(k_sum_tiles, dim3(B.n), dim3(THREADS), 0, st, B, 1);
    hipLaunchKernelGGL(k_sg2_clip, dim3(B.tiles), dim3(THREADS), 0, st, B, max_norm);
    SG_LAUNCH_CHECK("k_sg2_clip");
    return 0;
}

int sg_looksam_restore(int num_tensors, const SgLookSamTensor* tensors, void* workspace, size_t workspace_bytes, void* stream) {
    using namespace sgew;
    if (num_tensors <= 0) return 0;
    std::vector<FamRec> recs;
    if (looksam_collect(num_tensors, tensors, 0, &recs)) return 1;
    if (recs.empty()) return 0;
    hipStream_t st = (hipStream_t)stream;
    Batch<FamRec> B;
    if (upload(recs, workspace, workspace_bytes, st, &B)) return 1;
    hipLaunchKernelGGL(k_ls_restore, dim3(B.tiles), dim3(THREADS), 0, st, B);
    SG_LAUNCH_CHECK("k_ls_restore");
    return 0;
}

int sg_looksam_directions(int num_tensors, const SgLookSamTensor* tensors, void* workspace, size_t workspace_bytes, void* stream) {
    using namespace sgew;
    if (num_tensors <= 0) return 0;
    std::vector<FamRec> recs;
    if (looksam_collect(num_tensors, tensors, 1, &recs)) return 1;
    if (recs.empty()) return 0;
    hipStream_t st = (hipStream_t)stream;
    Batch<FamRec> B;
    if (upload(recs, workspace, workspace_bytes, st, &B)) return 1;
    hipLaunchKernelGGL(k_ls_diff_sumsq, dim3(B.tiles), dim3(THREADS), 0, st, B);
    hipLaunchKernelGGL(k_sum_tiles, dim3(B.n), dim3(THREADS), 0, st, B, 1);
    hipLaunchKernelGGL(k_ls_direction, dim3(B.tiles), dim3(THREADS), 0, st, B);
    SG_LAUNCH_CHECK("k_ls_direction");
    return 0;
}

int sg_looksam_adjust(int num_tensors, const SgLookSamTensor* tensors, float la, void* workspace, size_t workspace_bytes, void* stream) {
    using namespace sgew;
    if (num_tensors <= 0) return 0;
    std::vector<FamRec> recs;
    if (looksam_collect(num_tensors, tensors, 2, &recs)) return 1;
    if (recs.empty()) return 0;
    hipStream_t st = (hipStream_t)stream;
    Batch<FamRec> B;
    if (upload(recs, workspace, workspace_bytes, st, &B)) return 1;
    hipLaunchKernelGGL(k_ls_grad_sumsq, dim3(B.tiles), dim3(THREADS), 0, st, B);
    hipLaunchKernelGGL(k_sum_tiles, dim3(B.n), dim3(THREADS), 0, st, B, 1);
    hipLaunchKernelGGL(k_ls_adjust, dim3(B.tiles), dim3(THREADS), 0, st, B, la);
    SG_LAUNCH_CHECK("k_ls_adjust");
    return 0;
}

}  // extern "C"
