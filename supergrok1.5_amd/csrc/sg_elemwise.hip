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

namespace sgew {
namespace {

constexpr int TILE = 4096;
constexpr int THREADS = 256;
constexpr int MAX_HIDDEN = 256;

struct Red {            // result of the device-side norm reduction
    double norm_sq;
    float norm;         // sqrt(norm_sq)
    float coef;         // clip coefficient (1 when clipping is inactive)
    int clip_on;
    int pad_;
};

struct Layout {
    int n, tiles;
    size_t off_recs, off_nrecs, off_prefix, off_partials, off_red, bytes;
};
constexpr size_t REC_BYTES = 96;   // upper bound of any per-tensor record below
constexpr size_t NREC_BYTES = 24;  // view of a record used by the norm reduction

int make_layout(int n, const int64_t* numels, Layout* L) {
    int64_t tiles = 0, total = 0;
    for (int i = 0; i < n; i++) {
        if (numels[i] < 0 || numels[i] > 0x7fffffff) return sg::fail("tensor %d: bad numel %lld", i, (long long)numels[i]);
        tiles += (numels[i] + TILE - 1) / TILE;
        total += numels[i];
    }
    if (tiles > 0x7fffffff) return sg::fail("too many elements");
    L->n = n;
    L->tiles = (int)tiles;
    size_t o = 0;
    auto take = [&](size_t b) { size_t r = o; o = sg::align_up(o + b, 256); return r; };
    L->off_recs = take(REC_BYTES * (size_t)n);
    L->off_nrecs = take(NREC_BYTES * (size_t)n);
    L->off_prefix = take(sizeof(int) * (size_t)(n + 1));
    L->off_partials = take(sizeof(double) * (size_t)(tiles + 1));
    L->off_red = take(sizeof(Red));
    L->bytes = o;
    return 0;
}

template <class Rec>
struct Batch {
    const Rec* recs;
    const int* prefix;
    int n, tiles;
    double* partials;
    Red* red;
    void* nrecs;      // device room for n norm-reduction views
};

// Upload records + tile prefix; fills the Batch.  Rec must have .numel.
template <class Rec>
int upload(const std::vector<Rec>& recs, void* workspace, size_t ws_bytes, hipStream_t st, Batch<Rec>* B) {
    static_assert(sizeof(Rec) <= REC_BYTES, "record too large");
    const int n = (int)recs.size();
    std::vector<int64_t> numels(n);
    for (int i = 0; i < n; i++) numels[i] = recs[i].numel;
    Layout L;
    if (make_layout(n, numels.data(), &L)) return 1;
    if (!workspace || ws_bytes < L.bytes) return sg::fail("workspace too small: need %zu bytes, got %zu", L.bytes, ws_bytes);
    if (((uintptr_t)workspace & 255u) != 0) return sg::fail("workspace must be 256-byte aligned");
    std::vector<int> prefix(n + 1, 0);
    for (int i = 0; i < n; i++) prefix[i + 1] = prefix[i] + (int)((numels[i] + TILE - 1) / TILE);
    unsigned char* ws = static_cast<unsigned char*>(workspace);
    SG_HIP_CHECK(hipMemcpyAsync(ws + L.off_recs, recs.data(), sizeof(Rec) * (size_t)n, hipMemcpyHostToDevice, st));
    SG_HIP_CHECK(hipMemcpyAsync(ws + L.off_prefix, prefix.data(), sizeof(int) * (size_t)(n + 1), hipMemcpyHostToDevice, st));
    B->recs = reinterpret_cast<const Rec*>(ws + L.off_recs);
    B->prefix = reinterpret_cast<const int*>(ws + L.off_prefix);
    B->n = n;
    B->tiles = L.tiles;
    B->partials = reinterpret_cast<double*>(ws + L.off_partials);
    B->red = reinterpret_cast<Red*>(ws + L.off_red);
    B->nrecs = ws + L.off_nrecs;
    return 0;
}

template <class Rec>
__device__ __forceinline__ const Rec& tile_rec(const Batch<Rec>& B, int tile, int* start, int* cnt) {
    const int ti = sg::upper_seg(B.prefix, B.n, tile);
    const Rec& R = B.recs[ti];
    *start = (tile - B.prefix[ti]) * TILE;
    *cnt = min(TILE, (int)R.numel - *start);
    return R;
}

// ---- deterministic sum of squares -------------------------------------------
__device__ __forceinline__ double block_sum(double v, double* sm /*[4]*/) {
#pragma unroll
    for (int d = 32; d >= 1; d >>= 1) v += __shfl_down(v, d, 64);
    if ((threadIdx.x & 63) == 0) sm[threadIdx.x >> 6] = v;
    __syncthreads();
    const double r = (sm[0] + sm[1]) + (sm[2] + sm[3]);
    __syncthreads();
    return r;
}

struct NormRec {
    const void* grad;
    int64_t numel;
    int32_t dtype;
};

__global__ __launch_bounds__(THREADS) void k_sumsq_partial(Batch<NormRec> B) {
    __shared__ double sm[4];
    int start, cnt;
    const NormRec& R = tile_rec(B, blockIdx.x, &start, &cnt);
    float acc = 0.0f;
    for (int k = threadIdx.x; k < cnt; k += THREADS) {
        const float g = sg::load_elem(R.grad, R.dtype, start + k);
        acc = sg_fma(g, g, acc);
    }
    const double tot = block_sum((double)acc, sm);
    if (threadIdx.x == 0) B.partials[blockIdx.x] = tot;
}

// clip_norm > 0: clipping semantics of clip_grad_norms_device_side; rho_mode: nothing extra (norm is read by the consumer)
__global__ __launch_bounds__(THREADS) void k_sumsq_final(const double* __restrict__ partials, int tiles, float clip_norm, Red* red) {
    __shared__ double sm[4];
    double acc = 0.0;
    for (int k = threadIdx.x; k < tiles; k += THREADS) acc += partials[k];
    const double tot = block_sum(acc, sm);
    if (threadIdx.x == 0) {
        const float norm = (float)sqrt(tot);
        red->norm_sq = tot;
        red->norm = norm;
        const bool on = clip_norm > 0.0f && norm > clip_norm;
        red->clip_on = on ? 1 : 0;
        red->coef = on ? clip_norm / (norm + 1e-6f) : 1.0f;
    }
}

template <class Rec>
int reduce_sumsq(const std::vector<Rec>& recs, const Batch<Rec>& B, float clip_norm, hipStream_t st) {
    static_assert(sizeof(NormRec) == NREC_BYTES, "NormRec layout");
    std::vector<NormRec> nr(recs.size());
    for (size_t i = 0; i < recs.size(); i++) nr[i] = {recs[i].grad, recs[i].numel, recs[i].dtype};
    SG_HIP_CHECK(hipMemcpyAsync(B.nrecs, nr.data(), sizeof(NormRec) * nr.size(), hipMemcpyHostToDevice, st));
    Batch<NormRec> NB;
    NB.recs = reinterpret_cast<const NormRec*>(B.nrecs);
    NB.prefix = B.prefix;
    NB.n = B.n;
    NB.tiles = B.tiles;
    NB.partials = B.partials;
    NB.red = B.red;
    NB.nrecs = nullptr;
    hipLaunchKernelGGL(k_sumsq_partial, dim3(B.tiles), dim3(THREADS), 0, st, NB);
    hipLaunchKernelGGL(k_sumsq_final, dim3(1), dim3(THREADS), 0, st, B.partials, B.tiles, clip_norm, B.red);
    SG_LAUNCH_CHECK("sumsq");
    return 0;
}

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

int check_dtype(int i, int dtype) {
    if (dtype != SG_F32 && dtype != SG_F16 && dtype != SG_BF16) return sg::fail("tensor %d: bad dtype %d", i, dtype);
    return 0;
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
