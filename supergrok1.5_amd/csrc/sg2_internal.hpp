// Internal layout shared by the SuperGrok v2 translation units.
#pragma once

#include "sg_common.hpp"

namespace sg2 {

// Compile-time meta-net dimensions the kernels are specialised for (the
// defaults of the optimizer class; csrc/supergrok2_mamba_peer_kernels.cu:36-42
// of the reference only caps them).
constexpr int DM = 8;      // d_model
constexpr int DS = 16;     // d_state
constexpr int DI = 16;     // d_inner
constexpr int HP = DS / 2; // RoPE pairs
constexpr int GH = 4;      // gru_hidden
constexpr int NH = 4;      // PEER heads
constexpr int PK = 12;     // sub-keys per half
constexpr int EH = 16;     // expert hidden
constexpr int NE = 144;    // experts
constexpr int GRL = 2 + 2 * DM + GH;   // GRU row length (22)
constexpr int PIN = GH + 2 * DM + 2;   // PEER query input length (22)

constexpr int ELEM_TILE = 1024;        // elements per tile of the elementwise kernels
constexpr int SORT_TILE = 4096;        // keys per radix-sort tile (256 threads x 16)
constexpr int SCAN_TT = 64;            // timesteps projected per LDS tile
constexpr int SCAN_THREADS = DI * HP;  // one lane per (column, RoPE pair)
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
    int chunk_len;
    int window;                    // summary window (0: whole chunk), see k_scan<false>
    uint32_t* keys[2];
    int32_t* vals[2];              // element index within the tensor | sign bit of the gradient in bit 31
    float* ssorted;                // [total] sharpness gathered into sorted order
    uint32_t* spine;               // [256 * sort_tiles] per-tile digit counts, layout [segment][digit][tile]
    uint32_t* blocksums;
    float* summaries;              // [2][wchunks][6][128]
    float* hstart;                 // [2][chunks][2][128]
    float* comp;                   // [2][SG2_COMP_GROUPS][16][3] composed projection coefficients per direction
    float* htile;                  // bilevel: [2][htile_count][2][128] state entering every HT_STEP-th step, or NULL
    float* scan_out[2];            // bilevel, optional (NULL): per direction [total][DI] gated scan output of every step, in scan order
    float* adj_summ;               // bilevel: [2][chunks][128][6] adjoint transfer map of every chunk
    float* adj_lam;                // bilevel: [2][chunks][128][2] adjoint state arriving at the end of every chunk
    float* adj_blk;                // bilevel: [2][SG2_BWD_STRIDE] sums of adj_part's rows
    float* adj_part;               // bilevel: [2][ADJ_GROUPS][SG2_BWD_STRIDE] per-workgroup gradient sums
    int* sharp_nonzero;            // [P] uploaded as 0; set by k_keys when some (finite) sharpness entry of the tensor is not 0
    float* ctx;                    // [2][total][DM]
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
int check_dims(const SgDims* d);
// exactly one of d_ctx (element order, after out_proj) / d_scan (scan order, before out_proj) is given; dx (with rx) is optional
int launch_bilevel_backward(const Plan& pl, const float* d_ctx, const float* const d_scan[2], const float* rx, float* dx, float* grads_out,
                            hipStream_t st);
int launch_x_sorted(const Plan& pl, float* x_out, hipStream_t st);
int launch_elem(const Plan& pl, int32_t* expert_counts, int32_t* dbg_expert_idx, hipStream_t st);

}  // namespace sg2
