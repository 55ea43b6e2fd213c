// Internal layout shared by the SuperGrok v2 translation units.
#pragma once

#include "sg_common.hpp"

namespace sg2 {

// Compile-time meta-net geometries the step kernels are instantiated for: the
// defaults of the optimizer class and the largest scan block the reference
// admits (csrc/supergrok2_mamba_peer_kernels.cu:36-42 caps d_model at 16 and
// d_state / d_inner at 32).  Any smaller scan block runs on the smallest of the
// two that holds it, with its weights embedded in that geometry (zero rows and
// columns, see k_pad_weights in sg2_step.hip).  The specialised per-element
// kernel is built for the GRU, routing and expert sizes below (expert width 16,
// the class default, or 4, what the reference's training harness passes); every
// other combination takes the run-time-dimension kernel (k_elem_any).
constexpr int GH = 4;      // gru_hidden
constexpr int NH = 4;      // PEER heads
constexpr int PK = 12;     // sub-keys per half
constexpr int EH = 16;     // expert hidden (class default)
constexpr int NE = 144;    // experts
enum { ELEM_FAST16 = 0, ELEM_FAST4 = 1, ELEM_ANY = 2 };    // Plan::elem_kind
template <int DM_, int DS_, int DI_>
struct Geo {
    static constexpr int DM = DM_;               // d_model
    static constexpr int DS = DS_;               // d_state
    static constexpr int DI = DI_;               // d_inner
    static constexpr int HP = DS_ / 2;           // RoPE pairs
    static constexpr int THREADS = DI_ * HP;     // scan workgroup: one lane per (column, RoPE pair)
    static constexpr int PARTS = THREADS / 64;   // waves of that workgroup; each projects 1/PARTS of every output group
    static constexpr int ROWS = DI_;             // rows per group of composed coefficients
    static constexpr int GRL = 2 + 2 * DM_ + GH; // GRU row length
    static constexpr int PIN = GH + 2 * DM_ + 2; // PEER query input length
    static_assert(DI_ == DS_, "coefficient groups of equal height");
    static_assert(HP == 8 || HP == 16, "a column's pairs are one half or one whole DPP row");
    static_assert(THREADS % 64 == 0 && THREADS <= 1024 && DI_ % PARTS == 0 && DS_ % PARTS == 0 && DM_ % PARTS == 0 && DM_ % 4 == 0,
                  "whole waves; every output group splits evenly over them");
    static_assert(DM_ * DI_ == THREADS, "one out_proj entry per lane when it is staged");
};
using GeoDefault = Geo<8, 16, 16>;
using GeoLarge = Geo<16, 32, 32>;
enum { GEO_DEFAULT = 0, GEO_LARGE = 1, GEO_COUNT = 2 };
// run-time view of a geometry for the host code that sizes the work arrays
struct GeoInfo {
    int dm, ds, di, threads, rows;
};
inline GeoInfo geo_info(int geo) {
    return geo == GEO_LARGE ? GeoInfo{GeoLarge::DM, GeoLarge::DS, GeoLarge::DI, GeoLarge::THREADS, GeoLarge::ROWS}
                            : GeoInfo{GeoDefault::DM, GeoDefault::DS, GeoDefault::DI, GeoDefault::THREADS, GeoDefault::ROWS};
}
// the bilevel kernels exist for the default geometry only and use its constants directly
constexpr int DM = GeoDefault::DM;
constexpr int DS = GeoDefault::DS;
constexpr int DI = GeoDefault::DI;
constexpr int HP = GeoDefault::HP;
constexpr int GRL = GeoDefault::GRL;
constexpr int PIN = GeoDefault::PIN;

constexpr int ELEM_TILE = 1024;        // elements per tile of the elementwise kernels
#ifndef SG2_SORT_TILE
#define SG2_SORT_TILE 8192
#endif
constexpr int SORT_TILE = SG2_SORT_TILE;   // keys per radix-sort tile (16 per thread)
constexpr int SCAN_TT = 64;            // timesteps projected per LDS tile
constexpr int SCAN_THREADS = GeoDefault::THREADS;
constexpr int SCAN_BLOCK_ITEMS = 2048; // entries per block of the spine scan

// weight slots (argument order of supergrok2_mamba_peer_batched_step)
enum {
    W_IN_W = 0, W_IN_B,
    W_F_INPROJ, W_F_DTW, W_F_DTB, W_F_B, W_F_C, W_F_ALOG, W_F_D, W_F_ROPE, W_F_OUT,
    W_B_INPROJ, W_B_DTW, W_B_DTB, W_B_B, W_B_C, W_B_ALOG, W_B_D, W_B_ROPE, W_B_OUT,
    W_GRU_WZ, W_GRU_BZ, W_GRU_WR, W_GRU_BR, W_GRU_WH, W_GRU_BH,
    W_PEER_Q, W_KEYS_A, W_KEYS_B,
    W_EXP_W1, W_EXP_B1, W_EXP_W2, W_EXP_B2
};

// Per-tensor record as the kernels see it.
struct TensorDev {
    void* param;
    const void* grad;
    const void* sharp;
    float* ea;
    float* easq;
    float* mu;
    float* gru;
    float* mfwd;
    float* mbwd;
    int off;        // element offset of this tensor in the packed work arrays
    int numel;
    int dtype;
    int nchunks;    // scan chunks of this tensor
    float alpha, lamb, beta1, bc2, step_size;
    int pad_[5];
};
static_assert(sizeof(TensorDev) == 128, "TensorDev layout");

// Everything a kernel needs, passed by value.
struct Plan {
    const TensorDev* tensors;
    const int* elem_tile_prefix;   // [P+1] tiles of ELEM_TILE elements
    const int* sort_tile_prefix;   // [P+1] tiles of SORT_TILE keys
    const int* chunk_prefix;       // [P+1] scan chunks
    const int* wchunk_prefix;      // [P+1] scan chunks that need a summary (all but the last of a tensor)
    int P;
    int total;                     // sum of numel
    int elem_tiles, sort_tiles, chunks, wchunks;
    int geo;                       // GEO_*: which instantiation of the scan / elementwise kernels runs
    int elem_kind;                 // ELEM_*: which per-element kernel runs
    int st_di, st_ds;              // the caller's carried Mamba states are [st_di][st_ds] (the true d_inner, d_state;
                                   // entries of the kernel geometry beyond them read as 0 and are not stored)
    SgDims dims;                   // the caller's dimensions (what k_elem_any indexes the per-element weights with)
    int chunk_len;
    int window;                    // summary window (0: whole chunk), see k_scan<false>
    uint32_t* keys[2];
    int32_t* vals[2];              // element index within the tensor | sign bit of the gradient in bit 31
    float* ssorted;                // [total] sharpness gathered into sorted order
    uint32_t* spine;               // [256 * sort_tiles] per-tile digit counts, layout [segment][digit][tile]
    uint32_t* blocksums;
    float* summaries;              // [2][wchunks][6][THREADS]
    float* hstart;                 // [2][chunks][2][THREADS]
    float* comp;                   // [2][SG2_COMP_GROUPS][ROWS][3] composed projection coefficients per direction
    float* htile;                  // bilevel: [2][htile_count][2][128] state entering every HT_STEP-th step, or NULL
    float* scan_out[2];            // bilevel, optional (NULL): per direction [total][DI] gated scan output of every step, in scan order
    float* adj_summ;               // bilevel: [2][chunks][128][6] adjoint transfer map of every chunk
    float* adj_lam;                // bilevel: [2][chunks][128][2] adjoint state arriving at the end of every chunk
    float* adj_blk;                // bilevel: [2][SG2_BWD_STRIDE] sums of adj_part's rows
    float* adj_part;               // bilevel: [2][ADJ_GROUPS][SG2_BWD_STRIDE] per-workgroup gradient sums
    int* contracted;               // [0] set by k_compose (1 while every carried state of the call is finite), cleared by any summary whose 2x2 part is not exactly zero; [1] steps of a summary's first block (k_compose); [2] k_compose: some carried state is not finite
    int* state_bad;                // [P] set by k_tables: a carried Mamba state of the tensor holds a non-finite entry
    int* sharp_nonzero;            // [P] uploaded as 0; set by k_keys when some (finite) sharpness entry of the tensor is not 0
    float* ctx;                    // [2][total][d_model]
    float decay, beta2, eps, rescale;
    Sg2Weights W;
};

// records a profiling event (no-op unless profiling is enabled)
void prof_mark(int idx, hipStream_t st);

int launch_sort(const Plan& pl, int32_t* dbg_perm, hipStream_t st);
int launch_scan(const Plan& pl, hipStream_t st);
// bilevel path: the forward scan keeps the state entering every HT_STEP-th step of a tensor; index of scan step u
// (a multiple of HT_STEP) of tensor ti (element offset off) in that array, and the array's length
constexpr int HT_STEP = 32;
__host__ __device__ inline int htile_index(int off, int ti, int u) { return off / HT_STEP + ti + u / HT_STEP; }
__host__ __device__ inline int htile_count(int total, int P) { return total / HT_STEP + P + 1; }
// floats per direction of the adjoint kernels' sums: composed coefficients [5][16][3], A_log [16][16], rope_freq [16][8], D [16], out_proj [8][16]
constexpr int SG2_BWD_STRIDE = 768;
constexpr int ADJ_GROUPS = 512;    // workgroups per direction of the adjoint replay (upper bound)
// GEO_* of the smallest compiled geometry that holds these dimensions, or -1 with the error set
int geo_of(const SgDims* d);
// whether (d_model, d_state, d_inner) are exactly that geometry's (else the scan weights are embedded in it)
bool scan_exact(const SgDims* d, int geo);
// ELEM_* for these dimensions
int elem_kind_of(const SgDims* d, int geo);
// 0 if the dimensions are the default geometry (what the bilevel kernels are built for), else 1 with the error set
// per_element: also the GRU / routing / expert sizes the bilevel per-element kernel is built for
int check_dims(const SgDims* d, bool per_element = false);
// exactly one of d_ctx (element order, after out_proj) / d_scan (scan order, before out_proj) is given; dx (with rx) is optional
int launch_bilevel_backward(const Plan& pl, const float* d_ctx, const float* const d_scan[2], const float* rx, float* dx, float* grads_out,
                            hipStream_t st);
int launch_saved_intermediates(const Plan& pl, const Sg2BilevelExtra& ex, hipStream_t st);
int launch_x_sorted(const Plan& pl, float* x_out, hipStream_t st);
int launch_elem(const Plan& pl, int32_t* expert_counts, int32_t* dbg_expert_idx, hipStream_t st);
// the net's forward alone (run-time-dimension kernel): smart gradients [total] and new GRU states [total][gru_hidden], packed
int launch_elem_forward(const Plan& pl, int32_t* expert_counts, float* smart_out, float* gru_out, hipStream_t st);

}  // namespace sg2
