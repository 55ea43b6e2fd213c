// Segmented, stable, ascending LSD radix sort of (|grad| bits, element index)
// for all parameter tensors at once.  One segment per tensor.
//
// Stands in for the reference's input_proj_sort_kernel key generation
// (csrc/supergrok2_mamba_peer_kernels.cu:92-117) and its
// cub::DeviceSegmentedRadixSort::SortPairs call (:1860-1879).  Non-negative
// floats order like their bit patterns, so the keys are sorted as uint32.
//
// Four passes of 8 bits over tiles of 8192 keys (512 lanes x 16).  Per pass:
//   hist     per-tile digit counts -> spine[segment][digit][tile]  (first pass: counted while the keys are made)
//   scan     exclusive prefix over the whole spine (2 small kernels; one for small models).  Because
//            the spine is laid out segment-major, the global prefix of entry
//            (seg, d, tile) is exactly: keys in earlier segments + keys of this
//            segment with a smaller digit + keys with digit d in earlier tiles
//            = destination of the first such key of this tile.
//   scatter  stable rank inside the tile (each wave owns a contiguous quarter
//            of the tile; match-any ballots give the rank among equal digits)
//            and write to destination.
#include <type_traits>

#include "sg2_internal.hpp"

namespace sg2 {
namespace {

#ifndef SG2_SORT_THREADS
#define SG2_SORT_THREADS 512
#endif
constexpr int SORT_THREADS = SG2_SORT_THREADS;
constexpr int ITEMS = SORT_TILE / SORT_THREADS;      // rounds per wave
constexpr int WAVES = SORT_THREADS / 64;
constexpr int WAVE_ITEMS = SORT_TILE / WAVES;        // contiguous keys per wave
static_assert(SORT_THREADS >= 256 && SORT_THREADS % 64 == 0 && SORT_TILE % SORT_THREADS == 0, "one thread per digit at least");

struct TileRef {
    int base;        // index of the tile's first key in the packed arrays
    int cnt;         // keys in the tile
    int spine0;      // index of spine entry (digit 0) for this tile
    int stride;      // spine stride between digits (= tiles of the segment)
};
__device__ __forceinline__ TileRef tile_ref(const Plan& pl, int tile) {
    const int seg = sg::upper_seg(pl.sort_tile_prefix, pl.P, tile);
    const int t0 = pl.sort_tile_prefix[seg];
    const int nt = pl.sort_tile_prefix[seg + 1] - t0;
    const TensorDev& T = pl.tensors[seg];
    TileRef r;
    r.base = T.off + (tile - t0) * SORT_TILE;
    r.cnt = min(SORT_TILE, T.numel - (tile - t0) * SORT_TILE);
    r.spine0 = 256 * t0 + (tile - t0);
    r.stride = nt;
    return r;
}


// ---- digit counts of the first pass, straight from the gradients ----------------------
// One sort tile per workgroup.  The keys themselves are never written in element order: the first scatter pass
// forms them again from the gradients (key_of / payload_of) while it moves them.
// key = |g| bits; the sign rides in bit 31 of the payload so that the sorted (key, payload) pair gives back g
// exactly and the scan never has to gather gradients from element order
__device__ __forceinline__ uint32_t key_of(float g) { return (uint32_t)sg_f2i(sg_abs(sg::finite_or_zero(g))); }
__device__ __forceinline__ int32_t payload_of(float g, int index) { return index | (sg_f2i(sg::finite_or_zero(g)) & (int32_t)0x80000000); }

__global__ __launch_bounds__(SORT_THREADS) void k_keys(Plan pl) {
    // lane-selected copies of the counters, as in k_hist: gradients that came from a 16-bit format have one value of digit 0
    constexpr int HCOPY = 8, HSTRIDE = 256 + 8;
    __shared__ uint32_t hc[HCOPY * HSTRIDE];
    const int seg = sg::upper_seg(pl.sort_tile_prefix, pl.P, (int)blockIdx.x);
    const TileRef tr = tile_ref(pl, blockIdx.x);
    const TensorDev& T = pl.tensors[seg];
    const int start = tr.base - T.off;
    for (int k = threadIdx.x; k < HCOPY * HSTRIDE; k += SORT_THREADS) hc[k] = 0;
    uint32_t* const h = hc + (threadIdx.x & (HCOPY - 1)) * HSTRIDE;
    __syncthreads();
    bool nz = false;
    const float* gp = static_cast<const float*>(T.grad) + start;
    const float* sp = static_cast<const float*>(T.sharp) + start;
    if (T.dtype == SG_F32 && tr.cnt == SORT_TILE && ((((uintptr_t)gp) | ((uintptr_t)sp)) & 15u) == 0) {
        // whole fp32 tile on a 16-byte boundary: 16 bytes per lane and load, everything requested before the first use
        constexpr int VR = SORT_TILE / (4 * SORT_THREADS);
        typedef float vf4 __attribute__((ext_vector_type(4)));
        vf4 g[VR], sh[VR];
#pragma unroll
        for (int r = 0; r < VR; r++) g[r] = ((const SG_GLOBAL vf4*)gp)[r * SORT_THREADS + (int)threadIdx.x];
#pragma unroll
        for (int r = 0; r < VR; r++) sh[r] = ((const SG_GLOBAL vf4*)sp)[r * SORT_THREADS + (int)threadIdx.x];
#pragma unroll
        for (int r = 0; r < VR; r++)
#pragma unroll
            for (int e = 0; e < 4; e++) {
                atomicAdd(&h[key_of(g[r][e]) & 255u], 1u);
                nz = nz || (sg::finite_or_zero(sh[r][e]) != 0.0f);
            }
    } else {
        float g[ITEMS];
#pragma unroll
        for (int r = 0; r < ITEMS; r++) {
            const int k = r * SORT_THREADS + (int)threadIdx.x;
            g[r] = (k < tr.cnt) ? sg::load_elem(T.grad, T.dtype, start + k) : 0.0f;
        }
#pragma unroll
        for (int r = 0; r < ITEMS; r++) {
            const int k = r * SORT_THREADS + (int)threadIdx.x;
            if (k < tr.cnt) nz = nz || (sg::finite_or_zero(sg::load_elem(T.sharp, T.dtype, start + k)) != 0.0f);
        }
#pragma unroll
        for (int r = 0; r < ITEMS; r++) {
            const int k = r * SORT_THREADS + (int)threadIdx.x;
            if (k < tr.cnt) atomicAdd(&h[key_of(g[r]) & 255u], 1u);
        }
    }
    // Without SAM the sharpness of every element is 0 (the optimizer's initial state): remember per tensor
    // whether anything else was seen, so that the gather into sorted order can be skipped for such tensors.
    // (plain store, and only while the flag still reads 0: every writer stores the same value)
    if (__syncthreads_or(nz) && threadIdx.x == 0) {
        volatile int* flag = pl.sharp_nonzero + seg;
        if (*flag == 0) *flag = 1;
    }
    if (threadIdx.x < 256) {
        uint32_t tot = 0;
#pragma unroll
        for (int c = 0; c < HCOPY; c++) tot += hc[c * HSTRIDE + threadIdx.x];
        pl.spine[tr.spine0 + (int)threadIdx.x * tr.stride] = tot;
    }
}

// ---- per-tile histogram ---------------------------------------------------------
__global__ __launch_bounds__(SORT_THREADS) void k_hist(Plan pl, int src, int shift) {
    // HCOPY copies of the counters, chosen by lane: a pass whose digit takes few values (the exponent byte of the
    // magnitudes) would otherwise queue most of a wave's lanes on a dozen counters.  Copies start 8 banks apart.
    constexpr int HCOPY = 8, HSTRIDE = 256 + 8;
    __shared__ uint32_t hc[HCOPY * HSTRIDE];
    const TileRef tr = tile_ref(pl, blockIdx.x);
    for (int k = threadIdx.x; k < HCOPY * HSTRIDE; k += SORT_THREADS) hc[k] = 0;
    uint32_t* const h = hc + (threadIdx.x & (HCOPY - 1)) * HSTRIDE;
    __syncthreads();
    const uint32_t* __restrict__ keys = pl.keys[src] + tr.base;
    // 16 bytes per lane where the tile starts on a 16-byte boundary (tensor offsets are arbitrary); the ragged end by single keys
    const int vec = ((tr.base & 3) == 0) ? (tr.cnt & ~3) : 0;
    for (int k = threadIdx.x * 4; k < vec; k += SORT_THREADS * 4) {
        const uint4 q = *reinterpret_cast<const uint4*>(keys + k);
        atomicAdd(&h[(q.x >> shift) & 255u], 1u);
        atomicAdd(&h[(q.y >> shift) & 255u], 1u);
        atomicAdd(&h[(q.z >> shift) & 255u], 1u);
        atomicAdd(&h[(q.w >> shift) & 255u], 1u);
    }
    for (int k = vec + threadIdx.x; k < tr.cnt; k += SORT_THREADS) atomicAdd(&h[(keys[k] >> shift) & 255u], 1u);
    __syncthreads();
    if (threadIdx.x < 256) {
        uint32_t tot = 0;
#pragma unroll
        for (int c = 0; c < HCOPY; c++) tot += hc[c * HSTRIDE + threadIdx.x];
        pl.spine[tr.spine0 + (int)threadIdx.x * tr.stride] = tot;
    }
}

// ---- exclusive scan of the spine -------------------------------------------------
__device__ __forceinline__ uint32_t wave_incl_scan(uint32_t v) {
    const int lane = threadIdx.x & 63;
#pragma unroll
    for (int d = 1; d < 64; d <<= 1) {
        const uint32_t o = __shfl_up(v, d, 64);
        if (lane >= d) v += o;
    }
    return v;
}
// exclusive scan over the 256 threads of a block; *total receives the block sum
__device__ __forceinline__ uint32_t block_excl_scan(uint32_t v, uint32_t* smem /*[4]*/, uint32_t* total) {
    const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
    const uint32_t inc = wave_incl_scan(v);
    if (lane == 63) smem[w] = inc;
    __syncthreads();
    uint32_t base = 0, tot = 0;
#pragma unroll
    for (int k = 0; k < 4; k++) {
        const uint32_t s = smem[k];
        if (k < w) base += s;
        tot += s;
    }
    __syncthreads();
    *total = tot;
    return base + inc - v;
}

__global__ __launch_bounds__(256) void k_spine_reduce(const uint32_t* __restrict__ spine, uint32_t* blocksums, int n) {
    __shared__ uint32_t sm[4];
    const int base = blockIdx.x * SCAN_BLOCK_ITEMS;
    uint32_t s = 0;
    for (int k = threadIdx.x; k < SCAN_BLOCK_ITEMS; k += 256)
        if (base + k < n) s += spine[base + k];
    uint32_t tot;
    block_excl_scan(s, sm, &tot);
    if (threadIdx.x == 0) blocksums[blockIdx.x] = tot;
}
// Every workgroup adds up the block sums before its own by itself (a few hundred values for tens of millions of
// elements; 16 K on average at the 2^31-element limit, still small beside that step): no launch for a scan of them.
__global__ __launch_bounds__(256) void k_spine_down(uint32_t* spine, const uint32_t* __restrict__ blocksums, int n) {
    __shared__ uint32_t sm[4];
    constexpr int PER = SCAN_BLOCK_ITEMS / 256;
    uint32_t before;
    {
        uint32_t part = 0;
        for (int k = threadIdx.x; k < (int)blockIdx.x; k += 256) part += blocksums[k];
        block_excl_scan(part, sm, &before);
    }
    const int base = blockIdx.x * SCAN_BLOCK_ITEMS + threadIdx.x * PER;
    uint32_t v[PER], s = 0;
#pragma unroll
    for (int k = 0; k < PER; k++) {
        v[k] = (base + k < n) ? spine[base + k] : 0u;
        s += v[k];
    }
    uint32_t tot;
    uint32_t run = before + block_excl_scan(s, sm, &tot);
#pragma unroll
    for (int k = 0; k < PER; k++) {
        if (base + k < n) spine[base + k] = run;
        run += v[k];
    }
}

// The whole scan in one workgroup, for spines of at most SPINE_SINGLE_MAX entries (a model of up to a million
// elements): dependent launches of a few microseconds each cost more than the scan itself there.
constexpr int SPINE_SINGLE_MAX = 32768;
__global__ __launch_bounds__(1024) void k_spine_single(uint32_t* spine, int n /* a multiple of 256 */) {
    __shared__ uint32_t sm[16];
    const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
    uint32_t carry = 0;
    for (int base = 0; base < n; base += 4096) {
        const int i = base + (int)threadIdx.x * 4;
        uint4 v = make_uint4(0u, 0u, 0u, 0u);
        if (i < n) v = *reinterpret_cast<const uint4*>(spine + i);
        const uint32_t s = (v.x + v.y) + (v.z + v.w);
        const uint32_t inc = wave_incl_scan(s);
        if (lane == 63) sm[w] = inc;
        __syncthreads();
        uint32_t before = 0, tot = 0;
#pragma unroll
        for (int k = 0; k < 16; k++) {
            const uint32_t t = sm[k];
            if (k < w) before += t;
            tot += t;
        }
        __syncthreads();
        const uint32_t run = carry + before + inc - s;
        if (i < n) *reinterpret_cast<uint4*>(spine + i) = make_uint4(run, run + v.x, run + v.x + v.y, run + v.x + v.y + v.z);
        carry += tot;
    }
}

// ---- stable scatter ---------------------------------------------------------------
// FIRST: the pass over digit 0 takes its keys and payloads from the tensor's gradients (element order) instead of
// the key / payload arrays, which nothing has written yet.
template <bool FIRST>
__global__ __launch_bounds__(SORT_THREADS) void k_scatter(Plan pl, int src, int shift) {
    __shared__ uint32_t cnt[WAVES][256];     // running digit counts of each wave; later: destinations
    __shared__ uint32_t lbase[256], gdelta[256], wsum[4];
    __shared__ uint32_t skey[SORT_TILE];
    __shared__ int32_t sval[SORT_TILE];
    const TileRef tr = tile_ref(pl, blockIdx.x);
    const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
    for (int k = threadIdx.x; k < WAVES * 256; k += SORT_THREADS) (&cnt[0][0])[k] = 0;
    __syncthreads();

    // a whole tile (all but the last tile of a tensor) needs no bounds tests: the body exists in both forms
    auto body = [&](auto full_c) {
    constexpr bool FULL = decltype(full_c)::value;
    const uint32_t* __restrict__ keys = pl.keys[src] + tr.base;
    const int32_t* __restrict__ vals = pl.vals[src] + tr.base;
    const uint64_t lt = (lane == 0) ? 0ull : (~0ull >> (64 - lane));

    uint32_t key[ITEMS], rank[ITEMS];
    int32_t val[ITEMS];
    if (FIRST) {
        const TensorDev& T = pl.tensors[sg::upper_seg(pl.sort_tile_prefix, pl.P, (int)blockIdx.x)];
        const int start = tr.base - T.off, dtype = T.dtype;
        float g[ITEMS];
#pragma unroll
        for (int r = 0; r < ITEMS; r++) {
            const int i = w * WAVE_ITEMS + r * 64 + lane;
            g[r] = (FULL || i < tr.cnt) ? sg::load_elem(T.grad, dtype, start + i) : 0.0f;
        }
#pragma unroll
        for (int r = 0; r < ITEMS; r++) {
            const int i = w * WAVE_ITEMS + r * 64 + lane;
            const bool ok = FULL || i < tr.cnt;
            key[r] = ok ? key_of(g[r]) : 0u;
            val[r] = ok ? payload_of(g[r], start + i) : 0;
        }
    } else {
#pragma unroll
        for (int r = 0; r < ITEMS; r++) {
            const int i = w * WAVE_ITEMS + r * 64 + lane;
            const bool ok = FULL || i < tr.cnt;
            key[r] = ok ? keys[i] : 0u;
            val[r] = ok ? vals[i] : 0;
        }
    }
#pragma unroll
    for (int r = 0; r < ITEMS; r++) {
        const int i = w * WAVE_ITEMS + r * 64 + lane;
        const bool ok = FULL || i < tr.cnt;
        const uint32_t d = (key[r] >> shift) & 255u;       // 0 for a lane past the end (its key reads as 0)
        // lanes of the wave with the same digit: for every bit, keep the lanes whose bit equals this lane's.  With
        // rep = the lane's bit spread over a word, that is m & ~(ballot ^ rep): one three-input bit operation per
        // half (truth table 0x90 = a & ~(b ^ c)).  Lanes past the end hold no set bit and are outside the initial mask.
        const uint64_t m0 = __ballot(ok);
        uint32_t mlo = (uint32_t)m0, mhi = (uint32_t)(m0 >> 32);
#pragma unroll
        for (int b = 0; b < 8; b++) {
            const int32_t rep_b = __builtin_amdgcn_sbfe((int32_t)d, b, 1);
            const uint64_t bal = __ballot(rep_b != 0);
            mlo = __builtin_amdgcn_bitop3_b32(mlo, (uint32_t)bal, (uint32_t)rep_b, 0x90);
            mhi = __builtin_amdgcn_bitop3_b32(mhi, (uint32_t)(bal >> 32), (uint32_t)rep_b, 0x90);
        }
        const uint64_t m = ((uint64_t)mhi << 32) | mlo;
        if (ok) {
            const uint32_t before = __popcll(m & lt);
            const uint32_t prev = cnt[w][d];
            rank[r] = prev + before;
            if (before == 0) cnt[w][d] = prev + (uint32_t)__popcll(m);
        }
    }
    __syncthreads();
    // digit d = threadIdx.x: position of each wave's first key of digit d inside the tile's digit-sorted order
    // (cnt[k][d]), start of digit d in that order (lbase[d]) and its distance to the global destination (gdelta[d])
    {
        const int d = threadIdx.x & 255;       // (threads beyond the 256 digits repeat the first ones' work and store nothing)
        const bool own = threadIdx.x < 256;
        uint32_t tot = 0;
#pragma unroll
        for (int k = 0; k < WAVES; k++) tot += cnt[k][d];
        uint32_t inc = tot;     // inclusive scan over the 64 digits of this wave, then across the 4 waves
#pragma unroll
        for (int o = 1; o < 64; o <<= 1) {
            const uint32_t up = __shfl_up(inc, o, 64);
            if (lane >= o) inc += up;
        }
        if (lane == 63 && own) wsum[w] = inc;
        __syncthreads();
        uint32_t before = 0;
#pragma unroll
        for (int k = 0; k < 4; k++) before += (k < (d >> 6)) ? wsum[k] : 0u;
        const uint32_t lb = before + inc - tot;
        if (own) {
            lbase[d] = lb;
            gdelta[d] = pl.spine[tr.spine0 + d * tr.stride] - lb;     // global destination = gdelta[d] + local position (mod 2^32)
            uint32_t run = lb;
#pragma unroll
            for (int k = 0; k < WAVES; k++) {
                const uint32_t c = cnt[k][d];
                cnt[k][d] = run;
                run += c;
            }
        }
    }
    __syncthreads();
    // reorder through LDS so that global stores go out in digit-sorted order: consecutive lanes then write
    // consecutive addresses within each digit's run instead of 4-byte pieces all over the tile's 256 runs
#pragma unroll
    for (int r = 0; r < ITEMS; r++) {
        const int i = w * WAVE_ITEMS + r * 64 + lane;
        if (FULL || i < tr.cnt) {
            const uint32_t lp = cnt[w][(key[r] >> shift) & 255u] + rank[r];
            skey[lp] = key[r];
            sval[lp] = val[r];
        }
    }
    __syncthreads();
    uint32_t* __restrict__ kout = pl.keys[src ^ 1];
    int32_t* __restrict__ vout = pl.vals[src ^ 1];
#pragma unroll
    for (int r = 0; r < ITEMS; r++) {
        const int lp = r * SORT_THREADS + threadIdx.x;
        if (FULL || lp < tr.cnt) {
            const uint32_t kk = skey[lp];
            const uint32_t dst = gdelta[(kk >> shift) & 255u] + (uint32_t)lp;
            kout[dst] = kk;
            vout[dst] = sval[lp];
        }
    }
    };
    if (tr.cnt == SORT_TILE) body(std::true_type{});
    else body(std::false_type{});
}

// After the sort: sharpness gathered into sorted order (one random read per element, once, instead of
// one per scan pass and direction), and optionally the plain permutation for inspection.
__global__ __launch_bounds__(256) void k_gather_sorted(Plan pl, int32_t* __restrict__ dbg_perm) {
    const int tile = blockIdx.x;
    const int ti = sg::upper_seg(sg::as_const(pl.elem_tile_prefix), pl.P, tile);
    const TensorDev& T = pl.tensors[ti];
    const int start = (tile - pl.elem_tile_prefix[ti]) * ELEM_TILE;
    const int cnt = min(ELEM_TILE, T.numel - start);
    const bool gather = pl.sharp_nonzero[ti] != 0;      // all-zero sharpness: nothing to gather, no sorted copy is made
    if (!gather && !dbg_perm) return;                   // every reader tests the same flag before it touches ssorted
    for (int k = threadIdx.x; k < cnt; k += 256) {
        const int t = T.off + start + k;
        int idx = pl.vals[0][t] & 0x7fffffff;
        idx = ((unsigned)idx < (unsigned)T.numel) ? idx : 0;       // never index outside the tensor
        if (gather) pl.ssorted[t] = sg::finite_or_zero(sg::load_elem(T.sharp, T.dtype, idx));
        if (dbg_perm) dbg_perm[t] = idx;
    }
}

}  // namespace

int launch_sort(const Plan& pl, int32_t* dbg_perm, hipStream_t st) {
    if (pl.total == 0) return 0;
    hipLaunchKernelGGL(k_keys, dim3(pl.sort_tiles), dim3(SORT_THREADS), 0, st, pl);
    SG_LAUNCH_CHECK("k_keys");
    const int n = 256 * pl.sort_tiles;
    const int nb = (n + SCAN_BLOCK_ITEMS - 1) / SCAN_BLOCK_ITEMS;
    for (int pass = 0; pass < 4; pass++) {
        const int src = pass & 1, shift = 8 * pass;
        if (pass > 0) hipLaunchKernelGGL(k_hist, dim3(pl.sort_tiles), dim3(SORT_THREADS), 0, st, pl, src, shift);     // the first pass's counts come from k_keys
        if (n <= SPINE_SINGLE_MAX) {
            hipLaunchKernelGGL(k_spine_single, dim3(1), dim3(1024), 0, st, pl.spine, n);
        } else {
            hipLaunchKernelGGL(k_spine_reduce, dim3(nb), dim3(256), 0, st, pl.spine, pl.blocksums, n);
            hipLaunchKernelGGL(k_spine_down, dim3(nb), dim3(256), 0, st, pl.spine, pl.blocksums, n);
        }
        if (pass == 0) hipLaunchKernelGGL(k_scatter<true>, dim3(pl.sort_tiles), dim3(SORT_THREADS), 0, st, pl, src, shift);
        else hipLaunchKernelGGL(k_scatter<false>, dim3(pl.sort_tiles), dim3(SORT_THREADS), 0, st, pl, src, shift);
        SG_LAUNCH_CHECK("radix pass");
    }
    // result is back in keys[0] / vals[0]
    hipLaunchKernelGGL(k_gather_sorted, dim3(pl.elem_tiles), dim3(256), 0, st, pl, dbg_perm);
    SG_LAUNCH_CHECK("k_gather_sorted");
    return 0;
}

}  // namespace sg2
