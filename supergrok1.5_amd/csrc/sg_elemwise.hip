// Batched elementwise optimizer steps: Grokfast (EMA filter + amplification,
// optionally fused with its AdamW update) and SuperGrok v1.5 (device-side
// global-norm clip, mu EMA, 2->H->1 sharpness meta-net, Adam, progressive
// weight decay; SAM perturb / sharpness restore helpers).
//
// Every entry point covers all tensors with one launch per stage: a tile of
// 4096 elements is mapped to (tensor, offset) by binary search in a P+1 entry
// prefix table, so small parameter sets cost a handful of launches instead of
// several per tensor (the reference launches per tensor and syncs the host for
// the gradient norm).
#include <cmath>
#include <vector>

#include "sg_common.hpp"

#include "sg_elemwise.hpp"

namespace sgew {
namespace {

// ---- Grokfast ------------------------------------------------------------------
struct GfRec {
    void* param;
    void* grad;
    float* ema;
    float* ea;
    float* easq;
    int64_t numel;
    int32_t dtype;
    float step_size, bc2;
};

template <bool ADAM>
__global__ __launch_bounds__(THREADS) void k_grokfast(Batch<GfRec> B, float alpha, float lamb, float beta1, float om_beta1,
                                                       float beta2, float om_beta2, float eps, float decay) {
    int start, cnt;
    const GfRec& R = tile_rec(B, blockIdx.x, &start, &cnt);
    const int dtype = R.dtype;
    const float om_alpha = 1.0f - alpha;
    for (int k = threadIdx.x; k < cnt; k += THREADS) {
        const int i = start + k;
        const float g = sg::load_elem(R.grad, dtype, i);
        const float e = sg_fma(alpha, R.ema[i], om_alpha * g);
        R.ema[i] = e;
        const float amp = sg_fma(lamb, e, g);
        sg::store_elem(R.grad, dtype, i, amp);
        if (ADAM) {
            // AdamW consumes the gradient as stored, i.e. rounded to the tensor's element type
            const float ga = (dtype == SG_F32) ? amp : sg::load_elem(R.grad, dtype, i);
            const float ea = sg_fma(beta1, R.ea[i], om_beta1 * ga);
            const float easq = sg_fma(beta2, R.easq[i], (om_beta2 * ga) * ga);
            R.ea[i] = ea;
            R.easq[i] = easq;
            const float denom = __builtin_sqrtf(easq / R.bc2) + eps;
            const float p = sg::load_elem(R.param, dtype, i);
            sg::store_elem(R.param, dtype, i, sg_fma(p, decay, -((R.step_size * ea) / denom)));
        }
    }
}

// ---- SuperGrok v1.5 --------------------------------------------------------------
struct S15Rec {
    void* param;
    void* grad;
    const void* sharp;
    float* ea;
    float* easq;
    float* mu;
    int64_t numel;
    int32_t dtype;
    float alpha, beta1, bc2, step_size;
};

template <int GELU>
__global__ __launch_bounds__(THREADS) void k_sg15(Batch<S15Rec> B, const float* __restrict__ W1, const float* __restrict__ b1,
                                                   const float* __restrict__ W2, const float* __restrict__ b2, int H,
                                                   float rescale, float lamb_eff, float beta2, float eps, float decay) {
    __shared__ float sW1[2 * MAX_HIDDEN], sb1[MAX_HIDDEN], sW2[MAX_HIDDEN];
    for (int k = threadIdx.x; k < 2 * H; k += THREADS) sW1[k] = W1[k];
    for (int k = threadIdx.x; k < H; k += THREADS) { sb1[k] = b1[k]; sW2[k] = W2[k]; }
    __syncthreads();
    const float bias2 = b2[0];
    const float coef = B.red->coef;
    const bool clip_on = B.red->clip_on != 0;

    int start, cnt;
    const S15Rec& R = tile_rec(B, blockIdx.x, &start, &cnt);
    const int dtype = R.dtype;
    const float alpha = R.alpha, beta1 = R.beta1;
    for (int k = threadIdx.x; k < cnt; k += THREADS) {
        const int i = start + k;
        float g = sg::load_elem(R.grad, dtype, i);
        if (clip_on) {                       // gradients are rescaled in place, as the reference does
            sg::store_elem(R.grad, dtype, i, g * coef);
            g = (dtype == SG_F32) ? g * coef : sg::load_elem(R.grad, dtype, i);
        }
        const float s = sg::load_elem(R.sharp, dtype, i);
        const float mu = sg_fma(alpha, R.mu[i], (1.0f - alpha) * g);
        R.mu[i] = mu;
        float acc = 0.0f;
        for (int h = 0; h < H; h++) {
            const float z = sg_fma(sW1[2 * h + 1], s, sW1[2 * h] * g) + sb1[h];
            const float a = (GELU == 0) ? sg_gelu_erf(z) : sg_gelu_sigmoid(z);
            acc = sg_fma(sW2[h], a, acc);
        }
        const float smart = sg_fma(rescale, acc + bias2, g);
        const float fg = sg_fma(lamb_eff, mu, smart);
        const float ea = sg_fma(beta1, R.ea[i], (1.0f - beta1) * fg);
        const float easq = sg_fma(beta2, R.easq[i], ((1.0f - beta2) * fg) * fg);
        R.ea[i] = ea;
        R.easq[i] = easq;
        const float denom = __builtin_sqrtf(easq / R.bc2) + eps;
        const float p = sg::load_elem(R.param, dtype, i);
        sg::store_elem(R.param, dtype, i, sg_fma(p, decay, -((R.step_size * ea) / denom)));
    }
}

struct SamRec {
    void* param;
    const void* grad;
    int64_t numel;
    int32_t dtype;
};
__global__ __launch_bounds__(THREADS) void k_sam_perturb(Batch<SamRec> B, float rho) {
    int start, cnt;
    const SamRec& R = tile_rec(B, blockIdx.x, &start, &cnt);
    const float r = rho / (B.red->norm + 1e-12f);
    for (int k = threadIdx.x; k < cnt; k += THREADS) {
        const int i = start + k;
        const float p = sg::load_elem(R.param, R.dtype, i), g = sg::load_elem(R.grad, R.dtype, i);
        sg::store_elem(R.param, R.dtype, i, sg_fma(r, g, p));
    }
}

struct RestoreRec {
    void* param;
    void* sharp;
    const void* backup;
    const void* sam_grad;
    const void* grad;      // the normal gradient
    int64_t numel;
    int32_t dtype;
};
__global__ __launch_bounds__(THREADS) void k_restore(Batch<RestoreRec> B) {
    int start, cnt;
    const RestoreRec& R = tile_rec(B, blockIdx.x, &start, &cnt);
    for (int k = threadIdx.x; k < cnt; k += THREADS) {
        const int i = start + k;
        const float sgv = sg::load_elem(R.sam_grad, R.dtype, i), ng = sg::load_elem(R.grad, R.dtype, i);
        sg::store_elem(R.sharp, R.dtype, i, sg_abs(sgv - ng));
        sg::store_elem(R.param, R.dtype, i, sg::load_elem(R.backup, R.dtype, i));
    }
}

}  // namespace
}  // namespace sgew

extern "C" {

size_t sg_elemwise_workspace_bytes(int num_tensors, const int64_t* numels) {
    if (num_tensors < 0 || (num_tensors > 0 && !numels)) return 0;
    sgew::Layout L;
    if (sgew::make_layout(num_tensors, numels, &L)) return 0;
    return L.bytes;
}

int sg_grokfast_ema(int num_tensors, const SgGrokfastTensor* tensors, float alpha, float lamb, void* workspace,
                    size_t workspace_bytes, void* stream) {
    using namespace sgew;
    if (num_tensors <= 0) return 0;
    if (!tensors) return sg::fail("NULL argument");
    std::vector<GfRec> recs;
    for (int i = 0; i < num_tensors; i++) {
        const SgGrokfastTensor& t = tensors[i];
        if (t.numel == 0) continue;
        if (!t.grad || !t.ema) return sg::fail("tensor %d: NULL pointer", i);
        if (check_dtype(i, t.dtype)) return 1;
        recs.push_back({nullptr, t.grad, t.ema, nullptr, nullptr, t.numel, t.dtype, 0.0f, 1.0f});
    }
    if (recs.empty()) return 0;
    hipStream_t st = (hipStream_t)stream;
    Batch<GfRec> B;
    if (upload(recs, workspace, workspace_bytes, st, &B)) return 1;
    hipLaunchKernelGGL(k_grokfast<false>, dim3(B.tiles), dim3(THREADS), 0, st, B, alpha, lamb, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f);
    SG_LAUNCH_CHECK("k_grokfast<ema>");
    return 0;
}

int sg_grokfast_adamw_step(int num_tensors, const SgGrokfastAdamTensor* tensors, float alpha, float lamb, double lr,
                           double beta1, double beta2, double eps, double weight_decay, void* workspace,
                           size_t workspace_bytes, void* stream) {
    using namespace sgew;
    if (num_tensors <= 0) return 0;
    if (!tensors) return sg::fail("NULL argument");
    std::vector<GfRec> recs;
    for (int i = 0; i < num_tensors; i++) {
        const SgGrokfastAdamTensor& t = tensors[i];
        if (t.numel == 0) continue;
        if (!t.param || !t.grad || !t.ema || !t.exp_avg || !t.exp_avg_sq) return sg::fail("tensor %d: NULL pointer", i);
        if (check_dtype(i, t.dtype)) return 1;
        if (t.step < 1) return sg::fail("tensor %d: step must be >= 1", i);
        // bias corrections in double, as the Python helper computes them
        const double bc1 = 1.0 - std::pow(beta1, (double)t.step), bc2 = 1.0 - std::pow(beta2, (double)t.step);
        recs.push_back({t.param, t.grad, t.ema, t.exp_avg, t.exp_avg_sq, t.numel, t.dtype, (float)(lr / bc1), (float)bc2});
    }
    if (recs.empty()) return 0;
    hipStream_t st = (hipStream_t)stream;
    Batch<GfRec> B;
    if (upload(recs, workspace, workspace_bytes, st, &B)) return 1;
    hipLaunchKernelGGL(k_grokfast<true>, dim3(B.tiles), dim3(THREADS), 0, st, B, alpha, lamb, (float)beta1,
                       (float)(1.0 - beta1), (float)beta2, (float)(1.0 - beta2), (float)eps, (float)(1.0 - lr * weight_decay));
    SG_LAUNCH_CHECK("k_grokfast<adamw>");
    return 0;
}

int sg15_fused_step(int num_tensors, const Sg15Tensor* tensors, const Sg15Net* net, float lamb_eff, float beta2, float lr,
                    float wd_eff, float eps, float grad_clip_norm, void* workspace, size_t workspace_bytes, void* stream) {
    using namespace sgew;
    if (num_tensors <= 0) return 0;
    if (!tensors || !net || !net->W1 || !net->b1 || !net->W2 || !net->b2) return sg::fail("NULL argument");
    if (net->hidden < 1 || net->hidden > MAX_HIDDEN) return sg::fail("hidden_dim %d outside [1,%d]", net->hidden, MAX_HIDDEN);
    if (net->gelu_mode != 0 && net->gelu_mode != 1) return sg::fail("bad gelu_mode %d", net->gelu_mode);
    std::vector<S15Rec> recs;
    for (int i = 0; i < num_tensors; i++) {
        const Sg15Tensor& t = tensors[i];
        if (t.numel == 0) continue;
        if (!t.param || !t.grad || !t.sharpness || !t.exp_avg || !t.exp_avg_sq || !t.mu) return sg::fail("tensor %d: NULL pointer", i);
        if (check_dtype(i, t.dtype)) return 1;
        recs.push_back({t.param, t.grad, t.sharpness, t.exp_avg, t.exp_avg_sq, t.mu, t.numel, t.dtype, t.alpha, t.beta1, t.bc2,
                        lr / t.bc1});
    }
    if (recs.empty()) return 0;
    hipStream_t st = (hipStream_t)stream;
    Batch<S15Rec> B;
    if (upload(recs, workspace, workspace_bytes, st, &B)) return 1;
    if (reduce_sumsq(recs, B, grad_clip_norm, st)) return 1;
    const float decay = 1.0f - lr * wd_eff;
    if (net->gelu_mode == 0)
        hipLaunchKernelGGL(k_sg15<0>, dim3(B.tiles), dim3(THREADS), 0, st, B, net->W1, net->b1, net->W2, net->b2, net->hidden,
                           net->rescale, lamb_eff, beta2, eps, decay);
    else
        hipLaunchKernelGGL(k_sg15<1>, dim3(B.tiles), dim3(THREADS), 0, st, B, net->W1, net->b1, net->W2, net->b2, net->hidden,
                           net->rescale, lamb_eff, beta2, eps, decay);
    SG_LAUNCH_CHECK("k_sg15");
    return 0;
}

int sg15_sam_perturb(int num_tensors, const Sg15SamTensor* tensors, float rho, void* workspace, size_t workspace_bytes,
                     void* stream) {
    using namespace sgew;
    if (num_tensors <= 0) return 0;
    if (!tensors) return sg::fail("NULL argument");
    std::vector<SamRec> recs;
    for (int i = 0; i < num_tensors; i++) {
        const Sg15SamTensor& t = tensors[i];
        if (t.numel == 0) continue;
        if (!t.param || !t.grad) return sg::fail("tensor %d: NULL pointer", i);
        if (check_dtype(i, t.dtype)) return 1;
        recs.push_back({t.param, t.grad, t.numel, t.dtype});
    }
    if (recs.empty()) return 0;
    hipStream_t st = (hipStream_t)stream;
    Batch<SamRec> B;
    if (upload(recs, workspace, workspace_bytes, st, &B)) return 1;
    if (reduce_sumsq(recs, B, 0.0f, st)) return 1;
    hipLaunchKernelGGL(k_sam_perturb, dim3(B.tiles), dim3(THREADS), 0, st, B, rho);
    SG_LAUNCH_CHECK("k_sam_perturb");
    return 0;
}

int sg15_sharpness_restore(int num_tensors, const Sg15RestoreTensor* tensors, void* workspace, size_t workspace_bytes,
                           void* stream) {
    using namespace sgew;
    if (num_tensors <= 0) return 0;
    if (!tensors) return sg::fail("NULL argument");
    std::vector<RestoreRec> recs;
    for (int i = 0; i < num_tensors; i++) {
        const Sg15RestoreTensor& t = tensors[i];
        if (t.numel == 0) continue;
        if (!t.param || !t.sharpness || !t.backup || !t.sam_grad || !t.normal_grad) return sg::fail("tensor %d: NULL pointer", i);
        if (check_dtype(i, t.dtype)) return 1;
        recs.push_back({t.param, t.sharpness, t.backup, t.sam_grad, t.normal_grad, t.numel, t.dtype});
    }
    if (recs.empty()) return 0;
    hipStream_t st = (hipStream_t)stream;
    Batch<RestoreRec> B;
    if (upload(recs, workspace, workspace_bytes, st, &B)) return 1;
    hipLaunchKernelGGL(k_restore, dim3(B.tiles), dim3(THREADS), 0, st, B);
    SG_LAUNCH_CHECK("k_restore");
    return 0;
}

}  // extern "C"
