// Muon step: momentum (which also leaves the bf16 work copy), Frobenius norm (folded into the first iteration), quintic Newton-Schulz
// orthogonalisation as bf16 MFMA GEMMs with fp32 accumulation, parameter
// update.  Replaces the body of muon_fused_step (csrc/ops.cpp:663-746 of the
// reference: ATen norm + one host sync, three torch::mm per iteration,
// muon_ns_combine_kernel / muon_update_kernel of csrc/muon_kernels.cu:37-72).
//
// Every matrix is worked on in its "wide" orientation Y [m x n] (m = min dim)
// so the Gram matrix is always the small m x m one:
//     G = Y Y^T            H = a I + b G + c G G            Y <- H Y
// (the a Y term rides on H's diagonal, so the apply step is one product with no third operand; the diagonal entry
// is rounded to bf16 like every other entry of H: against the fp32 iteration this is no less accurate than adding
// a Y in the epilogue, the error of either form is set by the rounding of G)
// (for a tall parameter X this is X^T X and X (bG + cG^2): the reference's
// X X^T form re-associated, 6 m^2 n instead of 6 n^2 m flops per iteration).
// The Gram and polynomial products are "NT" GEMMs (both operands K-contiguous).
// The apply step is an "NN" one: its B operand is Y itself, whose K axis is
// the slow one.  Its tiles are staged in LDS as they lie in memory
// ([k][n], n contiguous) and the MFMA operand (8 consecutive k per lane) is
// fetched with gfx950's transposing LDS read (ds_read_b64_tr_b16), so no
// transposed copy of Y is kept: an iteration reads Y as an operand of two products and writes it once,
// into the other of two buffers (the current one is still being read as the B
// operand by other workgroups).  A tall parameter enters and leaves the wide
// orientation in the momentum and update kernels, which transpose 64x64 tiles
// through LDS.
// Work buffers are zero-padded to multiples of 256 so the GEMM needs no edge
// handling (zero rows/columns stay zero through the iteration).
//
// GEMM: 256x256 output tile per 512-thread workgroup, 8 waves as 2x4, each
// wave 128x64 = 4x2 MFMA 32x32x16 bf16 tiles (128 fp32 accumulators per
// lane, two waves per SIMD), K tiles of 32 in four LDS stages, filled by loads that go from global
// memory straight into LDS (global_load_lds_dwordx4) three tiles ahead of their
// use; no padding is possible in such a copy, so the tiles are swizzled by the
// choice of the chunk each lane fetches (conflict-free operand fetches); memory
// instructions are dealt between the MFMAs.  A 256x256 tile takes 128 flop per
// byte fetched, which keeps the MFMA pipe ahead of the ~64 B/clk a CU can pull
// from L2; the symmetric products (G and G*G) compute only the tiles on or above
// the diagonal.  Tile index -> XCD-contiguous order so that the workgroups
// sharing operand panels share an L2.
#include <cmath>
#include <vector>

#include "sg_common.hpp"
#include <type_traits>

namespace sgmu {
namespace {

typedef uint16_t bf16_t;
typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(16))) float f32x16;

constexpr int BT = 256;            // GEMM tile (M and N)
// Waves of a workgroup along N (2 along M).  Eight waves of 128 x 64 (two per SIMD, 128 accumulators each) measured
// 3.5 % faster per step than four waves of 128 x 128: they fetch 1.5 x the operand bytes from LDS, but a second wave per
// SIMD covers the fetch latencies that one wave cannot.
constexpr int GWN = 4;
constexpr int GWAVES = 2 * GWN, GTHREADS = 64 * GWAVES;
constexpr int WCOLS = BT / GWN;      // columns of a wave's block
constexpr int GEMM_LDS_BYTES = 4 * 2 * BT * 32 * 2;          // four stages of {A tile, B tile} of 32 k: 131,072 bytes of the CU's 160 KB
constexpr float NS_A = 3.4445f, NS_B = -4.7750f, NS_C = 2.0315f;

struct Mat {
    void* param;
    const void* grad;
    float* buf;
    bf16_t *Y, *Y2, *G, *H;       // [mp x np] twice (an iteration reads one and writes the other), [mp x mp], [mp x mp]
    int rows, cols, dtype;
    int m, n, mp, np;              // min / max dim and their padded sizes
    int wide;                      // rows <= cols
    int vec8;                      // cols % 8 == 0 and param/grad/buf 16-byte aligned: elementwise kernels move 8 elements per lane
};

struct Batch {
    const Mat* mats;
    const int* gtile_prefix[3];    // [P+1] GEMM output tiles for the three products
    const int* ttile_prefix;       // [P+1] 64x64 tiles of Y (the elementwise kernels work on these)
    int P, gtiles[3], ttiles;
    double* partials;              // [ttiles] sums of squares of the 64x64 tiles
    float* inv_norm;               // [P]
};

// ---- momentum + sum of squares ------------------------------------------------
__device__ __forceinline__ double block_sum(double v, double* sm) {
#pragma unroll
    for (int d = 32; d >= 1; d >>= 1) v += __shfl_down(v, d, 64);
    if ((threadIdx.x & 63) == 0) sm[threadIdx.x >> 6] = v;
    __syncthreads();
    const double r = (sm[0] + sm[1]) + (sm[2] + sm[3]);
    __syncthreads();
    return r;
}

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef float f32x4 __attribute__((ext_vector_type(4)));

// eight consecutive elements in the tensor's storage type; i a multiple of 8, base 16-byte aligned
__device__ __forceinline__ void load8(const void* p, int dtype, size_t i, float v[8]) {
    if (dtype == SG_F32) {
        const SG_GLOBAL f32x4* q = (const SG_GLOBAL f32x4*)(static_cast<const float*>(p) + i);
        const f32x4 a = q[0], b = q[1];
#pragma unroll
        for (int k = 0; k < 4; k++) { v[k] = a[k]; v[4 + k] = b[k]; }
    } else {
        const u32x4 w = *(const SG_GLOBAL u32x4*)(static_cast<const uint16_t*>(p) + i);
#pragma unroll
        for (int k = 0; k < 8; k++) {
            const uint16_t h = (uint16_t)((k & 1) ? (w[k >> 1] >> 16) : (w[k >> 1] & 0xffffu));
            v[k] = (dtype == SG_F16) ? __half2float(__ushort_as_half(h)) : sg::bf16_bits_to_f(h);
        }
    }
}
__device__ __forceinline__ void store8(void* p, int dtype, size_t i, const float v[8]) {
    if (dtype == SG_F32) {
        SG_GLOBAL f32x4* q = (SG_GLOBAL f32x4*)(static_cast<float*>(p) + i);
        q[0] = f32x4{v[0], v[1], v[2], v[3]};
        q[1] = f32x4{v[4], v[5], v[6], v[7]};
    } else {
        u32x4 w;
#pragma unroll
        for (int k = 0; k < 4; k++) {
            const uint32_t lo = (dtype == SG_F16) ? __half_as_ushort(__float2half_rn(v[2 * k])) : sg::f_to_bf16_bits(v[2 * k]);
            const uint32_t hi = (dtype == SG_F16) ? __half_as_ushort(__float2half_rn(v[2 * k + 1])) : sg::f_to_bf16_bits(v[2 * k + 1]);
            w[k] = lo | (hi << 16);
        }
        *(SG_GLOBAL u32x4*)(static_cast<uint16_t*>(p) + i) = w;
    }
}

// buf = momentum * buf + grad, the sum of squares of the new buf, and the new buf as bf16 into Y ([mp x np], the wide
// orientation) - NOT yet divided by its norm, which is only known once every tile of the matrix has been summed: the
// first iteration's Gram and apply epilogues carry the factors 1/norm^2 and 1/norm instead (bf16 rounding is relative,
// so rounding before or after the scaling costs the same), and no separate normalisation pass reads buf again.
// One 64x64 tile of the parameter's own orientation per workgroup: rows are read and written along the fast axis, a
// tall parameter's tile is transposed through LDS.
__global__ __launch_bounds__(256) void k_momentum(Batch B, float momentum) {
    __shared__ bf16_t t[64][66];
    __shared__ double sm[4];
    const int mi = sg::upper_seg(B.ttile_prefix, B.P, blockIdx.x);
    const Mat& M = B.mats[mi];
    bf16_t* own = M.Y;                            // wide: [R x C] in the parameter's orientation, padded
    bf16_t* other = M.Y;                          // tall: [C x R]
    const int R = M.wide ? M.mp : M.np, C = M.wide ? M.np : M.mp;
    const int tile = (int)blockIdx.x - B.ttile_prefix[mi];
    const int tc = C / 64, tr0 = (tile / tc) * 64, tc0 = (tile % tc) * 64;
    const bool w_own = M.wide, w_other = !M.wide;               // uniform over the workgroup
    const bool full = tr0 + 64 <= M.rows && tc0 + 64 <= M.cols && M.vec8;
    double acc = 0.0;
    if (full) {
        // interior tile: a lane moves 16 consecutive elements of a row
        const int lr = threadIdx.x >> 2, c0 = (threadIdx.x & 3) * 16;
        const size_t at = (size_t)(tr0 + lr) * M.cols + tc0 + c0;
        float g[16], b[16], part = 0.0f;
        load8(M.grad, M.dtype, at, g);
        load8(M.grad, M.dtype, at + 8, g + 8);
        load8(M.buf, SG_F32, at, b);
        load8(M.buf, SG_F32, at + 8, b + 8);
#pragma unroll
        for (int e = 0; e < 16; e++) { b[e] = sg_fma(momentum, b[e], g[e]); part = sg_fma(b[e], b[e], part); }
        store8(M.buf, SG_F32, at, b);
        store8(M.buf, SG_F32, at + 8, b + 8);
        acc = (double)part;
        uint32_t pk[8];
#pragma unroll
        for (int q = 0; q < 8; q++) {
            const uint32_t b0 = sg::f_to_bf16_bits(b[2 * q]), b1 = sg::f_to_bf16_bits(b[2 * q + 1]);
            pk[q] = b0 | (b1 << 16);
            t[lr][c0 + 2 * q] = (bf16_t)b0;
            t[lr][c0 + 2 * q + 1] = (bf16_t)b1;
        }
        if (w_own) {
            SG_GLOBAL u32x4* dst = (SG_GLOBAL u32x4*)(own + (size_t)(tr0 + lr) * C + tc0 + c0);
            dst[0] = u32x4{pk[0], pk[1], pk[2], pk[3]};
            dst[1] = u32x4{pk[4], pk[5], pk[6], pk[7]};
        }
        if (w_other) {
            __syncthreads();
            // transposed copy: output row lr (= own column), 16 consecutive output columns (= own rows)
#pragma unroll
            for (int q = 0; q < 8; q++) pk[q] = (uint32_t)t[c0 + 2 * q][lr] | ((uint32_t)t[c0 + 2 * q + 1][lr] << 16);
            SG_GLOBAL u32x4* dt = (SG_GLOBAL u32x4*)(other + (size_t)(tc0 + lr) * R + tr0 + c0);
            dt[0] = u32x4{pk[0], pk[1], pk[2], pk[3]};
            dt[1] = u32x4{pk[4], pk[5], pk[6], pk[7]};
        }
    } else {
        float part = 0.0f;
        for (int k = threadIdx.x; k < 64 * 64; k += 256) {
            const int r = tr0 + (k >> 6), c = tc0 + (k & 63);
            bf16_t v = 0;
            if (r < M.rows && c < M.cols) {
                const size_t i = (size_t)r * M.cols + c;
                const float bv = sg_fma(momentum, M.buf[i], sg::load_elem(M.grad, M.dtype, (int64_t)i));
                M.buf[i] = bv;
                part = sg_fma(bv, bv, part);
                v = sg::f_to_bf16_bits(bv);
            }
            if (w_own) own[(size_t)r * C + c] = v;
            t[k >> 6][k & 63] = v;
        }
        acc = (double)part;
        if (w_other) {
            __syncthreads();
            for (int k = threadIdx.x; k < 64 * 64; k += 256) {
                const int r = k >> 6, c = k & 63;     // output row r (= own column), column c (= own row)
                other[(size_t)(tc0 + r) * R + tr0 + c] = t[c][r];
            }
        }
    }
    const double tot = block_sum(acc, sm);
    if (threadIdx.x == 0) B.partials[blockIdx.x] = tot;
}

__global__ __launch_bounds__(256) void k_norm(Batch B) {
    __shared__ double sm[4];
    const int mi = blockIdx.x;
    double acc = 0.0;
    for (int k = B.ttile_prefix[mi] + (int)threadIdx.x; k < B.ttile_prefix[mi + 1]; k += 256) acc += B.partials[k];
    const double tot = block_sum(acc, sm);
    if (threadIdx.x == 0) B.inv_norm[mi] = 1.0f / ((float)sqrt(tot) + 1e-7f);
}

// ---- GEMM  C[M x N] = A[M x K] * B  with fused epilogues; B given as [N x K] (Gram, polynomial) or as [K x N] (apply)
// 256x256 output tile per workgroup of 2 x GWN waves, each wave 128 x (256/GWN) as MFMA 32x32x16 tiles.
// Per 16-wide k step a wave fetches 4+4 16-byte operands from LDS for 16 MFMAs.
// The Gram and polynomial products are symmetric: only tiles on or above the diagonal are
// computed, each off-diagonal tile is also stored transposed.
enum { EPI_GRAM = 0, EPI_POLY = 1, EPI_APPLY = 2 };
// explicit global address space: a generic (flat) load would count against the LDS wait counter as well
typedef const __attribute__((address_space(1))) u32x4* gvec_p;
typedef __attribute__((address_space(1))) u32x4* gvec_w;

// two floats rounded to bf16 (nearest even, NaN stays NaN), packed lo | hi << 16: one v_cvt_pk_bf16_f32 on gfx950
__device__ __forceinline__ uint32_t bf16r2(float lo, float hi) {
    typedef __attribute__((ext_vector_type(2))) float f32x2;
    typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2;
    return __builtin_bit_cast(uint32_t, __builtin_convertvector((f32x2){lo, hi}, bf16x2));
}

// The R operand reads of the next k step are dealt over the first eight of a phase's M MFMAs (R/8 after each, one more
// after the first R%8), the other MFMAs follow on their own
#define SG_MUON_SCHED_READS(R, M)                                                       \
    do {                                                                               \
        _Pragma("unroll") for (int g_ = 0; g_ < 8; g_++) {                              \
            __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);                          \
            if ((R) / 8 + (g_ < (R) % 8 ? 1 : 0) == 2) __builtin_amdgcn_sched_group_barrier(0x100, 2, 0); \
            else if ((R) / 8 + (g_ < (R) % 8 ? 1 : 0) == 1) __builtin_amdgcn_sched_group_barrier(0x100, 1, 0); \
        }                                                                              \
        if ((M) > 8) __builtin_amdgcn_sched_group_barrier(0x008, (M) - 8, 0);           \
    } while (0)

typedef short i16x4 __attribute__((ext_vector_type(4)));
typedef __attribute__((address_space(3))) i16x4* lds_i16x4_p;

// y_sel: which of the two Y buffers holds the current iterate
// iter_flags: bit 1 = first iteration (Y still carries the factor norm: see k_momentum)
template <int EPI>
__global__ __launch_bounds__(GTHREADS) void k_gemm_nt(Batch Bt, int y_sel, int iter_flags) {
    constexpr bool BKN = EPI == EPI_APPLY;             // B operand stored [K x N]
    constexpr int TM = BT / 64, TN = WCOLS / 32;       // MFMA tiles per wave in each direction (4 x 4 or 4 x 2)
    constexpr int LPT = 16 / GWAVES;                  // loads per wave, tile and operand (a tile is 16 blocks of 1 KB)
    extern __shared__ __attribute__((aligned(16))) bf16_t smem[];

    // XCD-contiguous tile order: hardware deals consecutive workgroups round-robin over the 8 XCDs,
    // so that tiles that run together on an XCD share operand panels in its L2
    const int nblk = gridDim.x;
    int lb = blockIdx.x;
    if (nblk % 8 == 0) lb = (blockIdx.x % 8) * (nblk / 8) + blockIdx.x / 8;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm = wave / GWN, wn = wave % GWN;
    const sg::cint_p prefix = sg::as_const(Bt.gtile_prefix[EPI]);
    const int mi = sg::upper_seg(prefix, Bt.P, lb);
    const Mat& Mt = Bt.mats[mi];
    int tile = lb - prefix[mi];

    const bf16_t *A, *B;
    bf16_t *C, *CT;         // CT: where the transposed tile goes (the symmetric products mirror into C itself)
    int K, lda, ldb, ldc, ldct, tm, tn;
    if (EPI == EPI_APPLY) {
        A = Mt.H; B = y_sel ? Mt.Y2 : Mt.Y; C = y_sel ? Mt.Y : Mt.Y2; K = Mt.mp; lda = Mt.mp; ldb = ldc = Mt.np;
        CT = C; ldct = ldc;      // unused: the apply step never mirrors
        // bands of 8 tile columns: 32 tiles that run together span 4 x 8 tiles instead of 2 x 16,
        // which halves the panel bytes they pull into L2
        const int ntm = Mt.mp / BT, ntn = Mt.np / BT;
        if (ntn % 8 == 0) {
            const int band = tile / (ntm * 8), w = tile % (ntm * 8);
            tm = w / 8;
            tn = band * 8 + w % 8;
        } else {
            tm = tile / ntn;
            tn = tile % ntn;
        }
    } else {
        if (EPI == EPI_GRAM) { A = y_sel ? Mt.Y2 : Mt.Y; B = A; C = Mt.G; K = Mt.np; lda = ldb = Mt.np; ldc = Mt.mp; }
        else { A = Mt.G; B = Mt.G; C = Mt.H; K = Mt.mp; lda = ldb = ldc = Mt.mp; }
        CT = C; ldct = ldc;
        const int nt = Mt.mp / BT;      // upper-triangular enumeration: row tm holds nt - tm tiles
        tm = 0;
        while (tile >= nt - tm) { tile -= nt - tm; tm++; }
        tn = tm + tile;
    }
    A += (size_t)tm * BT * lda;
    B += BKN ? (size_t)tn * BT : (size_t)tn * BT * ldb;

    f32x16 acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; i++)
#pragma unroll
        for (int j = 0; j < TN; j++)
#pragma unroll
            for (int e = 0; e < 16; e++) acc[i][j][e] = 0.0f;

    // Global memory -> LDS without passing through registers (global_load_lds_dwordx4: the 64 lanes' 16-byte chunks land
    // contiguously, 1 KB per instruction, at the wave-uniform LDS address in M0).  K tiles of 32, four stages of
    // {A tile, B tile} (16 KB each): the loads of a tile are issued three tiles ahead of its use and nothing of the
    // copy occupies the wave's registers or its LDS-write slots.  A 1 KB block cannot carry padding, so the tiles are
    // swizzled instead, by the choice of the chunk each lane fetches:
    //   [256 rows x 32 k] tile (K-contiguous operand): block = 16 rows x 4 chunks, chunk c of row r at position
    //                          c ^ ((r >> 2) & 3) of its row: 16 consecutive rows read one k chunk without a bank conflict
    //   [32 k x 256 n] tile (the apply step's B): block = 2 k rows x 32 chunks, the 64-byte group g of row k at
    //                          g ^ sw(k), sw(k) = (k & 3) | ((k >> 1) & 4): the 8 rows one transposing read touches
    //                          (k0..k0+3 and k0+8..k0+11) fall on 8 different groups
    constexpr int BKD = 32, STAGES = 4;
    constexpr int OP_BYTES = BT * BKD * 2, STAGE_BYTES = 2 * OP_BYTES;
    static_assert(STAGES * STAGE_BYTES <= GEMM_LDS_BYTES, "four stages fit the GEMM's LDS");
    const unsigned char* const lds = reinterpret_cast<const unsigned char*>(smem);
    const uint32_t lds0 = (uint32_t)(size_t)(__attribute__((address_space(3))) unsigned char*)smem;     // LDS byte address of smem
    const int wv = __builtin_amdgcn_readfirstlane(wave);
    // address = wave-uniform 64-bit base (scalar registers, advanced by scalar adds) + this lane's constant 32-bit offset
    auto dma16 = [](uint32_t lane_off, const void* base, uint32_t lds_addr) {
        asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1\n" : : "v"(lane_off), "s"(base), "s"(lds_addr) : "memory");
    };
    // this lane's share of a block: row lane/4 of the block's 16 (block 4i + w of the tile), chunk (lane%4) ^ ((lane/16)%4)
    // (block GWAVES*i + w of the tile for this wave's i-th load)
    const uint32_t lo_a = (uint32_t)((((lane >> 2) + 16 * wv) * lda + (((lane & 3) ^ ((lane >> 4) & 3)) * 8)) * 2);
    const uint32_t lo_b = (uint32_t)((((lane >> 2) + 16 * wv) * ldb + (((lane & 3) ^ ((lane >> 4) & 3)) * 8)) * 2);
    // [k][n] tile: wave w's i-th load fetches k rows 2(GWAVES*i + w) + lane/32; sw of a row k is (k & 3) | ((k >> 1) & 4)
    const int kn_row = 2 * wv + (lane >> 5);
    const int kn_c0 = (lane & 31) ^ ((((kn_row & 3) | ((kn_row >> 1) & 4)) & 7) << 2);
    const uint32_t lo_kn0 = (uint32_t)((kn_row * ldb + kn_c0 * 8) * 2);            // rows whose bit 3 is that of 2w + lane/32
    const uint32_t lo_kn1 = (uint32_t)((kn_row * ldb + (kn_c0 ^ 16) * 8) * 2);     // ... the other value (four waves: odd i)
    // the q-th of a tile's 2*LPT loads (first the A tile's, then the B tile's)
    auto dma_one = [&](int kt, int q) {
        const uint32_t st = lds0 + (uint32_t)(kt & (STAGES - 1)) * STAGE_BYTES;
        const int i = q % LPT, blk = GWAVES * i + wv;
        if (q < LPT) dma16(lo_a, reinterpret_cast<const char*>(A) + ((size_t)i * 16 * GWAVES * lda + (size_t)kt * BKD) * 2, st + blk * 1024);
        else if (BKN) dma16(((2 * GWAVES * i) & 8) ? lo_kn1 : lo_kn0, reinterpret_cast<const char*>(B) + (size_t)(kt * BKD + 2 * GWAVES * i) * ldb * 2, st + OP_BYTES + blk * 1024);
        else dma16(lo_b, reinterpret_cast<const char*>(B) + ((size_t)i * 16 * GWAVES * ldb + (size_t)kt * BKD) * 2, st + OP_BYTES + blk * 1024);
    };
    auto dma_tile = [&](int kt) {
#pragma unroll
        for (int q = 0; q < 2 * LPT; q++) dma_one(kt, q);
    };
    // operand fetches.  K-contiguous tile: lane = row lane%32 of a 32-row MFMA block, k chunk 2kk + lane/32
    const int ra0 = wm * (BT / 2) + (lane & 31), rb0 = wn * WCOLS + (lane & 31);
    const int a_rd0 = (ra0 >> 4) * 1024 + (ra0 & 15) * 64 + (((lane >> 5) ^ ((ra0 >> 2) & 3)) * 16);                 // kk = 0; kk = 1 is this ^ 32
    const int b_rd0 = OP_BYTES + (rb0 >> 4) * 1024 + (rb0 & 15) * 64 + (((lane >> 5) ^ ((rb0 >> 2) & 3)) * 16);
    // [k][n] tile, transposing read (ds_read_b64_tr_b16: within a 16-lane group, lane i receives as element e element i%4 of
    // the 8 bytes that lane 4e + i/4 addressed; groups 0/1 cover columns 0-15 / 16-31 of a 32-column MFMA block, groups 2/3
    // the same columns of the next 8 k): lane -> k row 8(lane/32) + (lane%16)/4,
    // columns 16((lane/16)%2) + 4(lane%4) of the 32-column MFMA block j of this wave; the block's 64-byte group is wn*4 + j
    const int kn_q2 = (lane & 15) >> 2, kn_h = lane >> 5;
    const int kn_rd0 = OP_BYTES + (8 * kn_h + kn_q2) * 512 + 32 * ((lane >> 4) & 1) + 8 * (lane & 3);
    const int kn_sw = kn_q2 | (kn_h << 2);
    constexpr int NREADS = TM + TN * (BKN ? 2 : 1);     // LDS reads of a k step's operands
    bf16x8 av[2][TM], bv[2][TN];
    auto lds_load = [&](int stage, int kk, int s) {
        const unsigned char* base = lds + stage * STAGE_BYTES;
#pragma unroll
        for (int i = 0; i < TM; i++) av[s][i] = *reinterpret_cast<const bf16x8*>(base + ((a_rd0 ^ (kk * 32)) + i * 2048));
#pragma unroll
        for (int j = 0; j < TN; j++) {
            if (BKN) {
                const unsigned char* q = base + kn_rd0 + (((wn * TN + j) ^ kn_sw) << 6) + kk * 16 * 512;
                const i16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_i16x4_p)(q));
                const i16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_i16x4_p)(q + 4 * 512));
                typedef short i16x8 __attribute__((ext_vector_type(8)));
                const i16x8 both = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
                bv[s][j] = __builtin_bit_cast(bf16x8, both);
            } else {
                bv[s][j] = *reinterpret_cast<const bf16x8*>(base + ((b_rd0 ^ (kk * 32)) + j * 2048));
            }
        }
    };
    auto mma = [&](int s) {
#pragma unroll
        for (int i = 0; i < TM; i++)
#pragma unroll
            for (int j = 0; j < TN; j++) acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(av[s][i], bv[s][j], acc[i][j], 0, 0, 0);
    };

    const int nk = K / BKD;      // a multiple of 8: K is a multiple of 256
    const bf16_t* aux = Mt.G;
    const int gcol0 = tn * BT + wn * WCOLS;
    // the auxiliary operand of the polynomial's epilogue (G):
    // 16 bytes per lane and 8-column chunk of a 32-row block of this wave's tile.  The first two blocks are requested during
    // the last K tile, each later one while the block two before it is
    // being written, so that the epilogue does not wait for memory
    u32x4 ax[2][WCOLS / 16];
    auto aux_load = [&](int i) {
#pragma unroll
        for (int c = 0; c < WCOLS / 16; c++) {
            const int id = lane + 64 * c, row = id / (WCOLS / 8), c8 = id % (WCOLS / 8);
            ax[i & 1][c] = *(gvec_p)(aux + (size_t)(tm * BT + wm * (BT / 2) + i * 32 + row) * ldc + gcol0 + c8 * 8);
        }
    };
    // wait until at most n of this wave's loads are outstanding (vmcnt only; the other counters unconstrained)
#define SG_WAIT_VM(n) __builtin_amdgcn_s_waitcnt(0x0F70 | ((n) & 15) | (((n) >> 4) << 14))
    dma_tile(0); dma_tile(1); dma_tile(2); dma_tile(3);
    SG_WAIT_VM(6 * LPT);
    __syncthreads();
    lds_load(0, 0, 0);
    // A K tile is two phases of 16 MFMAs.  Phase 0 multiplies k step 0 while the operands of k step 1 are read; then
    // the wave makes sure the next tile has landed (its loads were issued three tiles ago: only the two tiles after it
    // may still be in flight) and that its own reads of this stage are done, the workgroup meets, and the stage is
    // handed to the loads of the tile four ahead; phase 1 multiplies k step 1 while the first operands of the next
    // tile are read.
    // Phase 1 is written out as eight pairs of MFMAs, each followed by one load of the tile four ahead and one operand
    // read of the next tile: a burst of memory instructions would leave the matrix pipe idle while it issues.
    auto ktile = [&](int kt, auto dma_c, auto wait_c, auto next_c) {
        constexpr bool DMA = decltype(dma_c)::value != 0, NEXT = decltype(next_c)::value != 0;
        constexpr int WAIT = decltype(wait_c)::value;      // loads that may stay in flight once the next tile has landed
        const int stage = kt & (STAGES - 1), nstage = (kt + 1) & (STAGES - 1);
        __builtin_amdgcn_sched_barrier(0);
        lds_load(stage, 1, 1);
        mma(0);
        SG_MUON_SCHED_READS(NREADS, TM * TN);
        __builtin_amdgcn_sched_barrier(0);
        if (NEXT) SG_WAIT_VM(WAIT);
        __builtin_amdgcn_s_waitcnt(0xC07F);     // lgkmcnt(0): this wave's reads of the stage have returned
        __syncthreads();
        if (!NEXT && EPI == EPI_POLY) { aux_load(0); aux_load(1); }
        const unsigned char* nbase = lds + nstage * STAGE_BYTES;
        constexpr int MPG = TM * TN / 8;        // MFMAs per group
#pragma unroll
        for (int g = 0; g < 8; g++) {
            // operand reads of the next tile's k step 0: one fragment per group
            if (NEXT) {
                if (g < TM) av[0][g] = *reinterpret_cast<const bf16x8*>(nbase + a_rd0 + g * 2048);
                else if (g - TM >= TN) {}
                else if (!BKN) bv[0][g - TM] = *reinterpret_cast<const bf16x8*>(nbase + b_rd0 + (g - TM) * 2048);
                else {
                    const unsigned char* q = nbase + kn_rd0 + (((wn * TN + (g - TM)) ^ kn_sw) << 6);
                    const i16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_i16x4_p)(q));
                    const i16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_i16x4_p)(q + 4 * 512));
                    bv[0][g - TM] = __builtin_bit_cast(bf16x8, __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7));
                }
            }
#pragma unroll
            for (int m = MPG * g; m < MPG * (g + 1); m++)
                acc[m / TN][m % TN] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(av[1][m / TN], bv[1][m % TN], acc[m / TN][m % TN], 0, 0, 0);
            __builtin_amdgcn_sched_barrier(0);
            if (DMA && g < 2 * LPT) dma_one(kt + 4, g);
            __builtin_amdgcn_sched_barrier(0);
        }
    };
    using c0 = std::integral_constant<int, 0>;
    using c1 = std::integral_constant<int, 1>;
    int kt = 0;
    for (; kt + 4 < nk; kt++) ktile(kt, c1{}, std::integral_constant<int, 4 * LPT>{}, c1{});     // steady state
    ktile(kt, c0{}, std::integral_constant<int, 4 * LPT>{}, c1{});      // tiles nk-2 and nk-1 may still be in flight
    ktile(kt + 1, c0{}, std::integral_constant<int, 2 * LPT>{}, c1{});
    ktile(kt + 2, c0{}, std::integral_constant<int, 0>{}, c1{});
    ktile(kt + 3, c0{}, std::integral_constant<int, 0>{}, c0{});
#undef SG_WAIT_VM
    __syncthreads();        // the epilogue reuses the LDS stages: every wave is done reading them

    // ---- epilogue, staged through LDS (free after the last barrier) so that global memory sees
    // 16-byte accesses along rows.  Accumulator element e of MFMA tile (i,j) is
    // row 8*(e/4) + 4*(lane/32) + e%4, column lane%32.  One 32-row block of the wave's
    // tile at a time: fp32 block -> LDS, read back as 8-column chunks, combine with the auxiliary
    // operand, round to bf16 and store.  Off-diagonal tiles of the symmetric products also store
    // the transposed block: the rounded values go back into the staged block and are read down
    // its columns.  Every wave stages in its own LDS region and LDS executes a wave's
    // instructions in order, so no workgroup barrier is needed, only the compiler kept from
    // reordering (wave_barrier).
    constexpr int EP_ROW = WCOLS + 4;     // floats per staged row
    constexpr int RCH = WCOLS / 8;        // 8-column chunks per row
    constexpr int NC = 32 * RCH / 64;     // chunks per lane and 32-row block
    static_assert(GWAVES * 32 * EP_ROW * 4 <= GEMM_LDS_BYTES, "epilogue staging exceeds the GEMM's LDS");
    float* ep = reinterpret_cast<float*>(smem) + wave * (32 * EP_ROW);
    // uniform over the workgroup
    const bool mirror = EPI != EPI_APPLY && tm != tn;
    // first iteration: Y is the unnormalised momentum, so its Gram matrix carries 1/norm^2 and the applied Y 1/norm
    const float inv = Bt.inv_norm[mi];
    const bool diag_wave = EPI == EPI_POLY && tm == tn && wn / (GWN / 2) == wm;     // this wave's block meets the diagonal
    const bool first = (iter_flags & 2) != 0;
    const float first_scale = first ? (EPI == EPI_GRAM ? inv * inv : (EPI == EPI_APPLY ? inv : 1.0f)) : 1.0f;
#pragma unroll
    for (int i = 0; i < TM; i++) {
        const int grow0 = tm * BT + wm * (BT / 2) + i * 32;
#pragma unroll
        for (int j = 0; j < TN; j++)
#pragma unroll
            for (int e = 0; e < 16; e++)
                ep[(8 * (e >> 2) + 4 * (lane >> 5) + (e & 3)) * EP_ROW + 32 * j + (lane & 31)] = acc[i][j][e];
        __builtin_amdgcn_wave_barrier();
#pragma unroll
        for (int c = 0; c < NC; c++) {
            const int id = lane + 64 * c, row = id / RCH, c8 = id % RCH;
            f32x4* src = reinterpret_cast<f32x4*>(&ep[row * EP_ROW + c8 * 8]);
            const f32x4 lo = src[0], hi = src[1];
            float v[8] = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
            if (EPI == EPI_POLY) {
#pragma unroll
                for (int k = 0; k < 8; k++) {
                    const uint32_t w = ax[i & 1][c][k >> 1];
                    const float x = sg_i2f((int32_t)((k & 1) ? (w & 0xffff0000u) : (w << 16)));
                    v[k] = sg_fma(NS_C, v[k], NS_B * x);
                }
                if (diag_wave) {        // H + a I: the apply step is then the single product (H + a I) Y
                    const int dk = (wm * (BT / 2) + i * 32 + row) - (wn * WCOLS + c8 * 8);
#pragma unroll
                    for (int k = 0; k < 8; k++) v[k] += (dk == k) ? NS_A : 0.0f;
                }
            }
            if (EPI != EPI_POLY && first) {      // uniform over the grid
#pragma unroll
                for (int k = 0; k < 8; k++) v[k] *= first_scale;
            }
            u32x4 out;
#pragma unroll
            for (int k = 0; k < 4; k++) out[k] = bf16r2(v[2 * k], v[2 * k + 1]);
            *(gvec_w)(C + (size_t)(grow0 + row) * ldc + gcol0 + c8 * 8) = out;
            if (mirror) {   // rounded values (as bf16 bit patterns) back into the staged block
                u32x4 b0 = {out[0] & 0xffffu, out[0] >> 16, out[1] & 0xffffu, out[1] >> 16};
                u32x4 b1 = {out[2] & 0xffffu, out[2] >> 16, out[3] & 0xffffu, out[3] >> 16};
                reinterpret_cast<u32x4*>(src)[0] = b0;
                reinterpret_cast<u32x4*>(src)[1] = b1;
            }
        }
        if (EPI == EPI_POLY && i + 2 < TM) aux_load(i + 2);
        __builtin_amdgcn_wave_barrier();
        if (mirror) {
            const uint32_t* epb = reinterpret_cast<const uint32_t*>(ep);
#pragma unroll
            for (int c = 0; c < NC; c++) {
                const int id = lane + 64 * c, col = id >> 2, r8 = id & 3;
                u32x4 t;
#pragma unroll
                for (int k = 0; k < 4; k++)
                    t[k] = epb[(r8 * 8 + 2 * k) * EP_ROW + col] | (epb[(r8 * 8 + 2 * k + 1) * EP_ROW + col] << 16);
                *(gvec_w)(CT + (size_t)(gcol0 + col) * ldct + grow0 + r8 * 8) = t;
            }
            __builtin_amdgcn_wave_barrier();
        }
    }
}

// p = (p - 0.2*lr*X) * (1 - lr*wd).  X lies in the wide orientation; one 64x64 tile of the parameter's own
// orientation per workgroup (the grid of k_momentum), a tall parameter's tile of X is transposed through LDS.
// scale_inv: no iteration ran, X is still the unnormalised momentum
__global__ __launch_bounds__(256) void k_update(Batch B, float lr, float decay, int y_sel, int scale_inv) {
    __shared__ bf16_t t[64][66];
    const int mi = sg::upper_seg(B.ttile_prefix, B.P, blockIdx.x);
    const Mat& M = B.mats[mi];
    const bf16_t* X = y_sel ? M.Y2 : M.Y;         // [mp x np]
    const int C = M.wide ? M.np : M.mp;           // padded columns of the parameter's orientation
    const int tile = (int)blockIdx.x - B.ttile_prefix[mi];
    const int tc = C / 64, tr0 = (tile / tc) * 64, tc0 = (tile % tc) * 64;
    if (tr0 >= M.rows || tc0 >= M.cols) return;   // padding only (uniform over the workgroup)
    // the reference's scalar arithmetic (csrc/ops.cpp:729-734)
    const float max_dim = (float)max(M.rows, M.cols);
    const float scale_factor = 0.2f * sqrtf(max_dim);
    const float neg_lr_scale = -lr * scale_factor / sqrtf(max_dim);
    const float xs = scale_inv ? B.inv_norm[mi] : 1.0f;
    const bool full = tr0 + 64 <= M.rows && tc0 + 64 <= M.cols && M.vec8;
    const int lr_ = threadIdx.x >> 2, c0 = (threadIdx.x & 3) * 16;
    if (!M.wide) {
        // X tile: rows = the parameter's columns tc0.., columns = its rows tr0.. (the padded buffer covers all of it)
        const SG_GLOBAL u32x4* src = (const SG_GLOBAL u32x4*)(X + (size_t)(tc0 + lr_) * M.np + tr0 + c0);
        const u32x4 w0 = src[0], w1 = src[1];
#pragma unroll
        for (int q = 0; q < 4; q++) {
            t[lr_][c0 + 2 * q] = (bf16_t)(w0[q] & 0xffffu);
            t[lr_][c0 + 2 * q + 1] = (bf16_t)(w0[q] >> 16);
            t[lr_][c0 + 8 + 2 * q] = (bf16_t)(w1[q] & 0xffffu);
            t[lr_][c0 + 8 + 2 * q + 1] = (bf16_t)(w1[q] >> 16);
        }
        __syncthreads();
    }
    if (full) {
        // interior tile: a lane moves 16 consecutive elements of a row
        const size_t at = (size_t)(tr0 + lr_) * M.cols + tc0 + c0;
        float o[16], p[16];
        if (M.wide) {
            load8(X, SG_BF16, (size_t)(tr0 + lr_) * M.np + tc0 + c0, o);
            load8(X, SG_BF16, (size_t)(tr0 + lr_) * M.np + tc0 + c0 + 8, o + 8);
        } else {
#pragma unroll
            for (int e = 0; e < 16; e++) o[e] = sg::bf16_bits_to_f(t[c0 + e][lr_]);
        }
        load8(M.param, M.dtype, at, p);
        load8(M.param, M.dtype, at + 8, p + 8);
#pragma unroll
        for (int e = 0; e < 16; e++) {
            o[e] *= xs;
            if (M.dtype == SG_F16) o[e] = __half2float(__float2half_rn(o[e]));     // X.to(p.dtype)
            p[e] = sg_fma(neg_lr_scale, o[e], p[e]) * decay;
        }
        store8(M.param, M.dtype, at, p);
        store8(M.param, M.dtype, at + 8, p + 8);
        return;
    }
    for (int k = threadIdx.x; k < 64 * 64; k += 256) {
        const int r = tr0 + (k >> 6), c = tc0 + (k & 63);
        if (r >= M.rows || c >= M.cols) continue;
        float o = sg::bf16_bits_to_f(M.wide ? X[(size_t)r * M.np + c] : t[k & 63][k >> 6]) * xs;
        if (M.dtype == SG_F16) o = __half2float(__float2half_rn(o));
        const int64_t i = (int64_t)r * M.cols + c;
        const float p = sg::load_elem(M.param, M.dtype, i);
        sg::store_elem(M.param, M.dtype, i, sg_fma(neg_lr_scale, o, p) * decay);
    }
}

__global__ __launch_bounds__(256) void k_zero(uint4* p, size_t n16) {
    for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < n16; i += (size_t)gridDim.x * 256) p[i] = make_uint4(0, 0, 0, 0);
}

inline int round_up(int x, int a) { return (x + a - 1) / a * a; }

struct Layout {
    int P;
    std::vector<Mat> mats;
    std::vector<int> pre_g[3], pre_t;
    size_t off_mats, off_pre_g[3], off_pre_t, off_partials, off_inv, off_buffers, bytes;
};

int make_layout(int P, const SgMuonMatrix* in, Layout* L) {
    L->P = P;
    L->mats.resize(P);
    for (int k = 0; k < 3; k++) L->pre_g[k].assign(P + 1, 0);
    L->pre_t.assign(P + 1, 0);
    size_t o = 0;
    auto take = [&](size_t b) { size_t r = o; o = sg::align_up(o + b, 256); return r; };
    L->off_mats = take(sizeof(Mat) * (size_t)P);
    for (int k = 0; k < 3; k++) L->off_pre_g[k] = take(sizeof(int) * (size_t)(P + 1));
    L->off_pre_t = take(sizeof(int) * (size_t)(P + 1));
    for (int i = 0; i < P; i++) {
        const SgMuonMatrix& s = in[i];
        if (s.rows <= 0 || s.cols <= 0 || s.rows * s.cols > 0x7fffffff) return sg::fail("matrix %d: bad shape %lld x %lld", i, (long long)s.rows, (long long)s.cols);
        if (s.dtype != SG_F32 && s.dtype != SG_F16 && s.dtype != SG_BF16) return sg::fail("matrix %d: bad dtype %d", i, s.dtype);
        Mat& M = L->mats[i];
        M.param = s.param; M.grad = s.grad; M.buf = s.buf;
        M.rows = (int)s.rows; M.cols = (int)s.cols; M.dtype = s.dtype;
        M.wide = s.rows <= s.cols;
        M.vec8 = (s.cols % 8 == 0) && ((((uintptr_t)s.param | (uintptr_t)s.grad | (uintptr_t)s.buf) & 15u) == 0);
        M.m = (int)std::min(s.rows, s.cols); M.n = (int)std::max(s.rows, s.cols);
        M.mp = round_up(M.m, BT); M.np = round_up(M.n, BT);
        const int nt = M.mp / BT, tri = nt * (nt + 1) / 2;      // symmetric products: tiles on or above the diagonal
        L->pre_g[EPI_GRAM][i + 1] = L->pre_g[EPI_GRAM][i] + tri;
        L->pre_g[EPI_POLY][i + 1] = L->pre_g[EPI_POLY][i] + tri;
        L->pre_g[EPI_APPLY][i + 1] = L->pre_g[EPI_APPLY][i] + (M.mp / BT) * (M.np / BT);
        L->pre_t[i + 1] = L->pre_t[i] + (M.mp / 64) * (M.np / 64);
    }
    int64_t ttiles = 0;
    for (int i = 0; i < P; i++) ttiles += (int64_t)(L->mats[i].mp / 64) * (L->mats[i].np / 64);
    L->off_partials = take(sizeof(double) * (size_t)(ttiles + 1));
    L->off_inv = take(sizeof(float) * (size_t)P);
    L->off_buffers = o;
    for (int i = 0; i < P; i++) {
        Mat& M = L->mats[i];
        // offsets for now; turned into pointers once the workspace base is known
        M.Y = (bf16_t*)take(2 * (size_t)M.mp * M.np);
        M.Y2 = (bf16_t*)take(2 * (size_t)M.mp * M.np);
        M.G = (bf16_t*)take(2 * (size_t)M.mp * M.mp);
        M.H = (bf16_t*)take(2 * (size_t)M.mp * M.mp);
    }
    L->bytes = o;
    return 0;
}

}  // namespace
}  // namespace sgmu

extern "C" {

size_t sg_muon_workspace_bytes(int num_matrices, const SgMuonMatrix* mats) {
    if (num_matrices <= 0 || !mats) return 0;
    sgmu::Layout L;
    if (sgmu::make_layout(num_matrices, mats, &L)) return 0;
    return L.bytes;
}

int sg_muon_step(int num_matrices, const SgMuonMatrix* mats, float momentum, float lr, float wd, int ns_steps, void* workspace,
                 size_t workspace_bytes, void* stream) {
    using namespace sgmu;
    if (num_matrices <= 0) return 0;
    if (!mats) return sg::fail("NULL argument");
    if (ns_steps < 0) return sg::fail("ns_steps must be >= 0");
    for (int i = 0; i < num_matrices; i++)
        if (!mats[i].param || !mats[i].grad || !mats[i].buf) return sg::fail("matrix %d: NULL pointer", i);
    Layout L;
    if (make_layout(num_matrices, mats, &L)) return 1;
    if (!workspace || workspace_bytes < L.bytes) return sg::fail("workspace too small: need %zu bytes, got %zu", L.bytes, workspace_bytes);
    if (((uintptr_t)workspace & 255u) != 0) return sg::fail("workspace must be 256-byte aligned");
    hipStream_t st = (hipStream_t)stream;
    unsigned char* ws = static_cast<unsigned char*>(workspace);
    const int P = L.P;
    for (auto& M : L.mats) {
        M.Y = (bf16_t*)(ws + (size_t)M.Y); M.Y2 = (bf16_t*)(ws + (size_t)M.Y2);
        M.G = (bf16_t*)(ws + (size_t)M.G); M.H = (bf16_t*)(ws + (size_t)M.H);
    }
    // per-call tables: through kernel arguments (no host-to-device copy, nothing blocks the host)
    if (sg::upload_words(ws + L.off_mats, L.mats.data(), sizeof(Mat) * (size_t)P, st)) return 1;
    for (int k = 0; k < 3; k++)
        if (sg::upload_words(ws + L.off_pre_g[k], L.pre_g[k].data(), sizeof(int) * (size_t)(P + 1), st)) return 1;
    if (sg::upload_words(ws + L.off_pre_t, L.pre_t.data(), sizeof(int) * (size_t)(P + 1), st)) return 1;
    Batch B;
    B.mats = reinterpret_cast<const Mat*>(ws + L.off_mats);
    for (int k = 0; k < 3; k++) B.gtile_prefix[k] = reinterpret_cast<const int*>(ws + L.off_pre_g[k]);
    B.ttile_prefix = reinterpret_cast<const int*>(ws + L.off_pre_t);
    B.P = P;
    for (int k = 0; k < 3; k++) B.gtiles[k] = L.pre_g[k][P];
    B.ttiles = L.pre_t[P];
    B.partials = reinterpret_cast<double*>(ws + L.off_partials);
    B.inv_norm = reinterpret_cast<float*>(ws + L.off_inv);

    {   // the GEMM needs more LDS than the default per-kernel limit: raise it once per device
        static bool raised[64] = {};
        int dev = 0;
        SG_HIP_CHECK(hipGetDevice(&dev));
        if (dev < 0 || dev >= 64) return sg::fail("device index %d out of range", dev);
        if (!raised[dev]) {

            SG_HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void*>(k_gemm_nt<EPI_GRAM>), hipFuncAttributeMaxDynamicSharedMemorySize, GEMM_LDS_BYTES));
            SG_HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void*>(k_gemm_nt<EPI_POLY>), hipFuncAttributeMaxDynamicSharedMemorySize, GEMM_LDS_BYTES));
            SG_HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void*>(k_gemm_nt<EPI_APPLY>), hipFuncAttributeMaxDynamicSharedMemorySize, GEMM_LDS_BYTES));
            raised[dev] = true;
        }
    }

    // padded work buffers start from zero (a fill kernel, not a memset node, so the call stays capturable)
    bool any_pad = false;
    for (const auto& M : L.mats) any_pad = any_pad || M.mp != M.m || M.np != M.n;
    if (any_pad) {
        const size_t n16 = (L.bytes - L.off_buffers) / 16;
        hipLaunchKernelGGL(k_zero, dim3((unsigned)std::min<size_t>((n16 + 255) / 256, 65535)), dim3(256), 0, st,
                           reinterpret_cast<uint4*>(ws + L.off_buffers), n16);
    }

    hipLaunchKernelGGL(k_momentum, dim3(B.ttiles), dim3(256), 0, st, B, momentum);
    hipLaunchKernelGGL(k_norm, dim3(P), dim3(256), 0, st, B);
    SG_LAUNCH_CHECK("muon prologue");
    for (int it = 0; it < ns_steps; it++) {
        const int sel = it & 1, last = it == 0 ? 2 : 0;     // iter_flags
        hipLaunchKernelGGL(k_gemm_nt<EPI_GRAM>, dim3(B.gtiles[EPI_GRAM]), dim3(GTHREADS), GEMM_LDS_BYTES, st, B, sel, last);
        hipLaunchKernelGGL(k_gemm_nt<EPI_POLY>, dim3(B.gtiles[EPI_POLY]), dim3(GTHREADS), GEMM_LDS_BYTES, st, B, sel, last);
        hipLaunchKernelGGL(k_gemm_nt<EPI_APPLY>, dim3(B.gtiles[EPI_APPLY]), dim3(GTHREADS), GEMM_LDS_BYTES, st, B, sel, last);
        SG_LAUNCH_CHECK("muon newton-schulz");
    }
    hipLaunchKernelGGL(k_update, dim3(B.ttiles), dim3(256), 0, st, B, lr, 1.0f - lr * wd, ns_steps & 1, ns_steps == 0 ? 1 : 0);
    SG_LAUNCH_CHECK("k_update");
    return 0;
}

}  // extern "C"
