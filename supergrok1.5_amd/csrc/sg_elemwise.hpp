// Shared plumbing of the elementwise fused steps: per-call records and tile
// prefix uploaded into the caller's workspace, tile -> tensor lookup, and the
// deterministic device-side reductions (per-tile partial sums in double, then
// one block per result).
#ifndef SG_ELEMWISE_HPP_
#define SG_ELEMWISE_HPP_
#include <cmath>
#include <vector>

#include "sg_common.hpp"

namespace sgew {
namespace {

// Elements per workgroup.  Large calls use 4096 (16 per lane: few, long workgroups stream best); small calls use
// shorter tiles so that there are several workgroups per CU and few elements in series per lane (the v1.5 / v1.1
// steps spend ~1500 instructions per element).  A function of the call's total size only, so the workspace
// layout, the upload and the kernels agree.
inline int tile_for(int64_t total) { return total >= (8 << 20) ? 4096 : (total >= (1 << 20) ? 1024 : 256); }
constexpr int THREADS = 256;
constexpr int MAX_HIDDEN = 256;

struct Red {            // result of the device-side norm reduction
    double norm_sq;
    float norm;         // sqrt(norm_sq)
    float coef;         // clip coefficient (1 when clipping is inactive)
    int clip_on;
    int pad_;
};

struct TRed {           // up to three sums of one tensor (or of the whole call, in slot 0)
    double s[3];
    float d_lr;         // Prodigy: the step size estimate after this call's update
    int pad_;
};

struct Layout {
    int n, tiles, tile;
    size_t off_recs, off_nrecs, off_prefix, off_partials, off_red, off_tred, bytes;
    int64_t total;
};
constexpr size_t REC_BYTES = 96;   // upper bound of any per-tensor record below
constexpr size_t NREC_BYTES = 24;  // view of a record used by the norm reduction

inline int make_layout(int n, const int64_t* numels, Layout* L) {
    int64_t tiles = 0, total = 0;
    for (int i = 0; i < n; i++) {
        if (numels[i] < 0 || numels[i] > 0x7fffffff) return sg::fail("tensor %d: bad numel %lld", i, (long long)numels[i]);
        total += numels[i];
    }
    const int TILE = tile_for(total);
    for (int i = 0; i < n; i++) tiles += (numels[i] + TILE - 1) / TILE;
    L->tile = TILE;
    if (tiles > 0x7fffffff) return sg::fail("too many elements");
    L->n = n;
    L->tiles = (int)tiles;
    size_t o = 0;
    auto take = [&](size_t b) { size_t r = o; o = sg::align_up(o + b, 256); return r; };
    // records and tile prefix table back to back: one upload
    L->off_recs = take(REC_BYTES * (size_t)n + sizeof(int) * (size_t)(n + 1));
    L->off_prefix = L->off_recs + REC_BYTES * (size_t)n;
    L->off_nrecs = take(NREC_BYTES * (size_t)n);
    L->off_partials = take(sizeof(double) * 3 * (size_t)(tiles + 1));     // up to three sums per tile
    L->off_red = take(sizeof(Red));
    L->off_tred = take(sizeof(TRed) * (size_t)(n + 1));                   // per-tensor sums
    L->total = total;
    L->bytes = o;
    return 0;
}

template <class Rec>
struct Batch {
    const Rec* recs;
    const int* prefix;
    int n, tiles, tile;
    double* partials;
    Red* red;
    TRed* tred;
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
    // host image of [records (REC_BYTES apart is the layout's bound; they lie sizeof(Rec) apart) | prefix table]
    std::vector<uint32_t> blob((REC_BYTES * (size_t)n + sizeof(int) * (size_t)(n + 1)) / 4, 0u);
    static_assert(sizeof(Rec) % 4 == 0 && REC_BYTES % 4 == 0, "records are whole words");
    const uint32_t* rw = reinterpret_cast<const uint32_t*>(recs.data());
    for (size_t i = 0; i < sizeof(Rec) * (size_t)n / 4; i++) blob[i] = rw[i];
    int* prefix = reinterpret_cast<int*>(blob.data() + REC_BYTES * (size_t)n / 4);
    for (int i = 0; i < n; i++) prefix[i + 1] = prefix[i] + (int)((numels[i] + L.tile - 1) / L.tile);
    unsigned char* ws = static_cast<unsigned char*>(workspace);
    if (sg::upload_words(ws + L.off_recs, blob.data(), blob.size() * 4, st)) return 1;
    B->recs = reinterpret_cast<const Rec*>(ws + L.off_recs);
    B->prefix = reinterpret_cast<const int*>(ws + L.off_prefix);
    B->n = n;
    B->tiles = L.tiles;
    B->tile = L.tile;
    B->partials = reinterpret_cast<double*>(ws + L.off_partials);
    B->red = reinterpret_cast<Red*>(ws + L.off_red);
    B->tred = reinterpret_cast<TRed*>(ws + L.off_tred);
    B->nrecs = ws + L.off_nrecs;
    return 0;
}

template <class Rec>
__device__ __forceinline__ const Rec& tile_rec(const Batch<Rec>& B, int tile, int* start, int* cnt) {
    const int ti = sg::upper_seg(B.prefix, B.n, tile);
    const Rec& R = B.recs[ti];
    *start = (tile - B.prefix[ti]) * B.tile;
    *cnt = min(B.tile, (int)R.numel - *start);
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
    int done = 0;
    if (R.dtype == SG_F32 && ((uintptr_t)R.grad & 15u) == 0) {     // four elements per lane and access
        typedef float f32x4 __attribute__((ext_vector_type(4)));
        done = cnt & ~3;
        for (int k = threadIdx.x * 4; k < done; k += THREADS * 4) {
            const f32x4 g = *(const SG_GLOBAL f32x4*)(static_cast<const float*>(R.grad) + start + k);
            acc = sg_fma(g[0], g[0], acc);
            acc = sg_fma(g[1], g[1], acc);
            acc = sg_fma(g[2], g[2], acc);
            acc = sg_fma(g[3], g[3], acc);
        }
    }
    for (int k = done + threadIdx.x; k < cnt; k += THREADS) {
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
    if (sg::upload_words(B.nrecs, nr.data(), sizeof(NormRec) * nr.size(), st)) return 1;
    Batch<NormRec> NB;
    NB.recs = reinterpret_cast<const NormRec*>(B.nrecs);
    NB.prefix = B.prefix;
    NB.n = B.n;
    NB.tiles = B.tiles;
    NB.tile = B.tile;
    NB.partials = B.partials;
    NB.red = B.red;
    NB.tred = B.tred;
    NB.nrecs = nullptr;
    hipLaunchKernelGGL(k_sumsq_partial, dim3(B.tiles), dim3(THREADS), 0, st, NB);
    hipLaunchKernelGGL(k_sumsq_final, dim3(1), dim3(THREADS), 0, st, B.partials, B.tiles, clip_norm, B.red);
    SG_LAUNCH_CHECK("sumsq");
    return 0;
}

inline int check_dtype(int i, int dtype) {
    if (dtype != SG_F32 && dtype != SG_F16 && dtype != SG_BF16) return sg::fail("tensor %d: bad dtype %d", i, dtype);
    return 0;
}

}  // namespace
}  // namespace sgew
#endif
