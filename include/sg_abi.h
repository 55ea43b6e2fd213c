/*
 * sg_abi.h -- C ABI of libsg_hip.so: hand-written gfx950 kernels for the
 * fused per-parameter optimizer steps.  Plain pointers and sizes only; no
 * torch types.  Every entry point
 *   - returns 0 on success, non-zero on error (sg_last_error() has the text;
 *     no exception crosses the boundary),
 *   - enqueues its work on the hipStream_t passed as `stream` (void* so the
 *     header needs no HIP include) and returns without synchronising,
 *   - performs no device allocation: scratch memory comes in as `workspace`.
 *
 * The torch extension `_ops` (csrc/ops_shim.cpp in the package) keeps the
 * reference's pybind signatures and forwards here.  Each declaration names
 * the reference interface it stands behind (paths relative to the reference
 * tree).
 */
#ifndef SG_ABI_H_
#define SG_ABI_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* element type of param / grad / sharpness tensors */
enum { SG_F32 = 0, SG_F16 = 1, SG_BF16 = 2 };

/* meta-net dimensions, the trailing ints of
 * launch_mamba3_peer_batched_step (csrc/ops.h:196-229).  The step takes every
 * set that the reference's kernels admit
 * (supergrok2_mamba_peer_kernels.cu:1796-1801: d_state even and <= 32,
 * d_model <= 16, d_inner a multiple of 4 and <= 32, gru_hidden <= 8) with
 * d_model even and num_experts <= pk_dim * pk_dim; anything else is refused
 * with an error that names the limit.  Scan blocks other than the two
 * compiled ones, (d_model, d_state, d_inner) = (8, 16, 16) and (16, 32, 32),
 * run embedded in the smallest compiled block that holds them.  The bilevel
 * entry points take (8, 16, 16) with gru_hidden 4, num_heads 4, pk_dim 12 and
 * expert_hidden <= 16 (sg2_bilevel_elem: exactly 16; narrower experts are
 * passed zero-padded). */
typedef struct SgDims {
    int32_t d_model, d_state, d_inner, gru_hidden, num_heads, pk_dim, expert_hidden, num_experts;
} SgDims;

/* The 33 fp32 meta-net weight tensors (device pointers) in the argument
 * order of supergrok2_mamba_peer_batched_step (csrc/ops.h:548-581):
 * input_proj_W, input_proj_b, 9 forward-Mamba, 9 backward-Mamba
 * (in_proj, dt_W, dt_b, B_proj, C_proj, A_log, D, rope, out_proj),
 * gru_Wz,bz,Wr,br,Wh,bh, peer_query_Ws, prod_keys_A, prod_keys_B,
 * expert_W1, expert_b1, expert_W2, expert_b2.
 * Shapes: csrc/supergrok2_mamba_peer_kernels.cu:1453-1487. */
#define SG2_NUM_WEIGHTS 33
typedef struct Sg2Weights {
    const float* w[SG2_NUM_WEIGHTS];
} Sg2Weights;

/* One parameter tensor of the batched step: the i-th entries of the
 * std::vector arguments of supergrok2_mamba_peer_batched_step
 * (csrc/ops.h:548-556,575-576).  All pointers are device pointers to
 * contiguous storage; the tensor is treated as flat (numel elements).
 * param, grad and sharpness share `dtype`; every state tensor is fp32. */
typedef struct Sg2Tensor {
    void* param;              /* [numel]            updated in place        */
    const void* grad;         /* [numel]            read only               */
    const void* sharpness;    /* [numel]            read only               */
    float* exp_avg;           /* [numel]            updated                 */
    float* exp_avg_sq;        /* [numel]            updated                 */
    float* mu;                /* [numel]            updated                 */
    float* gru_state;         /* [numel,gru_hidden] updated                 */
    float* mamba_fwd_state;   /* [d_inner,d_state]  updated (scan carry)    */
    float* mamba_bwd_state;   /* [d_inner,d_state]  updated (scan carry)    */
    int64_t numel;
    int32_t dtype;            /* SG_F32 / SG_F16 / SG_BF16                  */
    float alpha_mu, lamb_eff, beta1, bc1, bc2;
} Sg2Tensor;

/* shared scalars of the batched step (csrc/ops.h:577) */
typedef struct Sg2Scalars {
    float rescale, beta2, lr, wd_eff, eps;
} Sg2Scalars;

/* Optional inspection outputs for parity tests (device pointers, any may be
 * NULL).  Element order is the concatenation of the tensors in call order. */
typedef struct Sg2Debug {
    int32_t* perm;          /* [total]     sorted position -> element index within its tensor */
    int32_t* expert_idx;    /* [total][num_heads]                                             */
    float* ctx;             /* [2][total][d_model] forward / backward context, element order  */
} Sg2Debug;

/* text of the last error raised on the calling thread */
const char* sg_last_error(void);

/* Length (timesteps) of the scan chunks a tensor's sorted sequence is cut
 * into; a multiple of 64.  0 (the default) lets each call choose 4096, 2048,
 * 1024 or 512 from the amount of work; sg2_chunk_len_for tells what a call with
 * these tensor sizes will use.  Affects results only by re-association of the
 * chunk products. */
int sg2_set_chunk_len(int chunk_len);
int sg2_get_chunk_len(void);
int sg2_chunk_len_for(int num_tensors, const int64_t* numels);

/* Summary window of the scan (timesteps, a multiple of 64; 0 disables, a
 * negative value restores the default, SG2_DEFAULT_SCAN_WINDOW).  The recurrence contracts, so a
 * chunk summary is built backwards in blocks of `window` steps and the walk
 * stops as soon as every entry of the 2x2 part of the running summary is below
 * 2^-100 (the chunk summary is then (0, b)); a chunk that never contracts is
 * covered completely.  Before that walk one block whose length follows from
 * the weights (the steps the slowest RoPE pair needs to contract at the step
 * size of a zero input) is tried with a bound in place of the 2x2 part; the
 * walk is the fallback.  Takes effect when window < chunk_len. */
#define SG2_DEFAULT_SCAN_WINDOW 64
int sg2_set_scan_window(int window);
int sg2_get_scan_window(void);

/* Bytes of scratch the batched step needs for these tensor sizes. */
size_t sg2_workspace_bytes(const SgDims* dims, int num_tensors, const int64_t* numels);

/* SuperGrok v2 full step over all tensors: replaces
 * launch_mamba3_peer_batched_step (csrc/ops.h:196-229,
 * csrc/supergrok2_mamba_peer_kernels.cu:1754-2117) behind
 * supergrok2_mamba_peer_batched_step (csrc/ops.cpp:815-877).
 * `tensors` is a host array; tensors with numel == 0 are skipped.
 * expert_counts: device int32[num_experts], incremented. */
int sg2_batched_step(const SgDims* dims, const Sg2Weights* weights, int num_tensors,
                     const Sg2Tensor* tensors, const Sg2Scalars* scalars, int32_t* expert_counts,
                     void* workspace, size_t workspace_bytes, const Sg2Debug* debug, void* stream);

/* The same step with the scan's decomposition chosen by the caller for this
 * call instead of by the process-wide settings above (no counterpart in the
 * reference).  chunk_len: 0 = the automatic choice, else a positive multiple
 * of 64; scan_window: negative = SG2_DEFAULT_SCAN_WINDOW, 0 = off, else a
 * multiple of 64.  options == NULL means the process-wide settings, i.e.
 * exactly sg2_workspace_bytes / sg2_batched_step.  The workspace must be sized
 * with the same options. */
typedef struct Sg2Options {
    int32_t chunk_len;
    int32_t scan_window;
} Sg2Options;
size_t sg2_workspace_bytes_opt(const SgDims* dims, int num_tensors, const int64_t* numels, const Sg2Options* options);
int sg2_batched_step_opt(const SgDims* dims, const Sg2Weights* weights, int num_tensors,
                         const Sg2Tensor* tensors, const Sg2Scalars* scalars, int32_t* expert_counts,
                         void* workspace, size_t workspace_bytes, const Sg2Debug* debug,
                         const Sg2Options* options, void* stream);

/* sg2_batched_step without a workspace argument, for callers that cannot
 * allocate device memory (code under HIP graph capture, tight serving loops,
 * harnesses that forbid hipMalloc).  It has no counterpart in the reference.
 * The scratch lives in a static device array of SG2_STATIC_SCRATCH_BYTES inside
 * the library (one copy per GPU the library runs on, held until the process
 * ends); the call allocates and frees nothing, on the device or through any
 * library.  Calls whose tensors need more scratch than that (about 700 000
 * elements in total; sg2_workspace_bytes tells) are rejected with an error.
 * Every call on a GPU uses that GPU's one array: calls that overlap on one
 * GPU (different streams or threads) race; calls on one stream are ordered.
 * Same kernels and results as sg2_batched_step.
 * The first call on a device looks the array's device address up
 * (hipGetDevice + hipGetSymbolAddress, no stream work): make one plain call per
 * device before a stream capture starts, so that the captured calls only
 * launch kernels.  The array is part of the library's device image: every
 * process that loads libsg_hip.so holds SG2_STATIC_SCRATCH_BYTES (64 MiB) on each
 * GPU it initialises, whether or not this entry point is ever called. */
#define SG2_STATIC_SCRATCH_BYTES (64u << 20)
size_t sg2_static_scratch_bytes(void);
int sg2_batched_step_static(const SgDims* dims, const Sg2Weights* weights, int num_tensors,
                            const Sg2Tensor* tensors, const Sg2Scalars* scalars, int32_t* expert_counts,
                            const Sg2Debug* debug, void* stream);

/* Per-stage device timing of sg2_batched_step with HIP events recorded on the
 * step's own stream (no counterpart in the reference, which has no profiling
 * hooks).  Stages: 0 key generation + radix sort, 1 scan chunk summaries,
 * 2 chunk prefix, 3 scan output, 4 per-element kernel.
 * sg2_profile_enable(1) starts collecting (at most SG2_PROF_MAX_CALLS calls are
 * kept), sg2_profile_read waits for the recorded events, adds each stage's
 * elapsed milliseconds over the collected calls into ms[SG2_PROF_STAGES],
 * stores the number of calls and clears the collection.  A measurement aid
 * for one caller: while collecting, step calls must come from one thread. */
#define SG2_PROF_STAGES 5
#define SG2_PROF_MAX_CALLS 256
int sg2_profile_enable(int on);
int sg2_profile_read(float* ms, int* calls);

/* ======================= Grokfast / SuperGrok v1.5 ======================== */

/* Scratch for the elementwise entry points below (tables + reduction
 * partials) for n tensors with these sizes. */
size_t sg_elemwise_workspace_bytes(int num_tensors, const int64_t* numels);

/* Grokfast EMA filter + amplification over all tensors in one launch:
 *   ema = alpha*ema + (1-alpha)*g ;  grad <- g + lamb*ema   (grad overwritten)
 * Replaces launch_fused_grokfast_ema (csrc/grokfast_kernels.cu:20-60) called
 * per tensor by grokfast_fused_step (csrc/ops.cpp:514-532). */
typedef struct SgGrokfastTensor {
    void* grad;        /* [numel] dtype, overwritten with the amplified gradient */
    float* ema;        /* [numel] fp32 */
    int64_t numel;
    int32_t dtype;
} SgGrokfastTensor;
int sg_grokfast_ema(int num_tensors, const SgGrokfastTensor* tensors, float alpha, float lamb,
                    void* workspace, size_t workspace_bytes, void* stream);

/* The whole Grokfast.step body in one pass: the EMA/amplify above followed by
 * the AdamW update of adamw_step (grokking_optimizers/_adamw_helper.py:12-22,
 * called from grokking_optimizers/grokfast.py:124-143): p *= 1-lr*wd first,
 * bias corrections from the per-tensor step computed in double as Python
 * does.  grad is still overwritten with the amplified gradient. */
typedef struct SgGrokfastAdamTensor {
    void* param;       /* [numel] dtype */
    void* grad;        /* [numel] dtype */
    float* ema;        /* [numel] fp32 */
    float* exp_avg;    /* [numel] fp32 */
    float* exp_avg_sq; /* [numel] fp32 */
    int64_t numel;
    int32_t dtype;
    int32_t step;      /* already incremented, >= 1 */
} SgGrokfastAdamTensor;
int sg_grokfast_adamw_step(int num_tensors, const SgGrokfastAdamTensor* tensors, float alpha, float lamb,
                           double lr, double beta1, double beta2, double eps, double weight_decay,
                           void* workspace, size_t workspace_bytes, void* stream);

/* SuperGrok v1.5 full step over all tensors: global-norm gradient clip
 * (coef = c/(norm+1e-6) when norm > c, gradients rescaled in place) with the
 * norm reduced on the device, then mu EMA, the 2->H->1 sharpness meta-net,
 * Adam and progressive weight decay in one pass.  Replaces
 * clip_grad_norms_device_side (csrc/ops.cpp:23-55) and
 * launch_fused_supergrok15_full_step (csrc/supergrok15_kernels.cu:323-459)
 * behind supergrok15_fused_step (csrc/ops.cpp:83-152).
 * gelu_mode 0: exact erf GELU (the reference's CPU path, csrc/ops.cpp:140);
 * gelu_mode 1: z/(1+exp(-1.702 z)) (its GPU kernel, supergrok15_kernels.cu:380). */
typedef struct Sg15Tensor {
    void* param;            /* [numel] dtype */
    void* grad;             /* [numel] dtype, rescaled in place when clipping is active */
    const void* sharpness;  /* [numel] dtype */
    float* exp_avg;         /* [numel] fp32 */
    float* exp_avg_sq;      /* [numel] fp32 */
    float* mu;              /* [numel] fp32 */
    int64_t numel;
    int32_t dtype;
    float alpha, beta1, bc1, bc2;
} Sg15Tensor;
typedef struct Sg15Net {
    const float* W1;        /* [hidden,2] */
    const float* b1;        /* [hidden]   */
    const float* W2;        /* [1,hidden] */
    const float* b2;        /* [1]        */
    int32_t hidden;         /* <= 256 */
    float rescale;
    int32_t gelu_mode;
} Sg15Net;
int sg15_fused_step(int num_tensors, const Sg15Tensor* tensors, const Sg15Net* net, float lamb_eff, float beta2,
                    float lr, float wd_eff, float eps, float grad_clip_norm, void* workspace,
                    size_t workspace_bytes, void* stream);

/* SAM ascent step p += rho/(||g||+1e-12) * g with the global norm reduced on
 * the device: replaces compute_sam_grad_norm_device_side + launch_sam_perturb
 * (csrc/ops.cpp:58-75,154-177; csrc/supergrok15_kernels.cu:151-162).  The
 * caller clones the parameters beforehand. */
typedef struct Sg15SamTensor {
    void* param;
    const void* grad;
    int64_t numel;
    int32_t dtype;
} Sg15SamTensor;
int sg15_sam_perturb(int num_tensors, const Sg15SamTensor* tensors, float rho, void* workspace,
                     size_t workspace_bytes, void* stream);

/* sharpness = |g_sam - g| ; param <- backup.  Replaces launch_sharpness_restore
 * (csrc/supergrok15_kernels.cu:170-184, csrc/ops.cpp:179-204). */
typedef struct Sg15RestoreTensor {
    void* param;
    void* sharpness;
    const void* backup;
    const void* sam_grad;
    const void* normal_grad;
    int64_t numel;
    int32_t dtype;
} Sg15RestoreTensor;
int sg15_sharpness_restore(int num_tensors, const Sg15RestoreTensor* tensors, void* workspace,
                           size_t workspace_bytes, void* stream);

/* ---- bilevel meta-net training: the scan, forward and backward ------------
 *
 * The reference trains the meta-net by differentiating smart_grad with respect
 * to its weights (grokking_optimizers/supergrok2.py:516-1330 over
 * supergrok2_bilevel_fwd_save / supergrok2_bilevel_backward, csrc/ops.h:232-371).
 * Here the sequential part - sort and bidirectional scan - runs forward and
 * backward in HIP (sg2_bilevel_forward / sg2_bilevel_backward), and so does
 * the per-element part - GRU, soft top-4 PEER routing, experts -
 * (sg2_bilevel_elem, forward and backward in one pass).
 *
 * sg2_bilevel_forward: sort + scan exactly as in sg2_batched_step, writing the
 * two contexts of every element to ctx_out ([2][sum numel][d_model] floats,
 * element order, tensors packed in call order) and keeping what the backward
 * pass needs in the workspace.  Of Sg2Tensor only grad, sharpness,
 * mamba_fwd_state, mamba_bwd_state, numel and dtype are read; the two states
 * are OVERWRITTEN with the end-of-sequence states, so pass copies.
 *
 * sg2_bilevel_backward: same tensors and the SAME, untouched workspace; d_ctx
 * has ctx_out's layout.  grads_out receives SG2_SCAN_GRAD_FLOATS floats, the
 * gradients of the 20 scan weights in the order of Sg2Weights:
 *   input_proj W [8][2], b [8]; then for the forward and the backward block
 *   in_proj [32][8], dt_proj W [16][16], b [16], B_proj [16][16], C_proj
 *   [16][16], A_log [16][16], D [16], rope_freq [16][8], out_proj [8][16].
 * The adjoint is exact (no truncation window); sums over elements are formed in
 * a fixed order, so the result is reproducible run to run.
 *
 * Scan blocks smaller than (d_model, d_state, d_inner) = (8, 16, 16) run
 * embedded in that block (zero rows and columns, as in the step): ctx_out and
 * d_ctx rows stay 8 floats wide (entries from d_model on are +0 / ignored),
 * grads_out keeps the layout above with the block's gradients at the embedded
 * positions (row r, column c of a smaller matrix at row r, column c of the
 * listed one) and zeros elsewhere, and the two Mamba states keep the caller's
 * own [d_inner][d_state] shape.  Larger blocks are refused. */
#define SG2_SCAN_GRAD_FLOATS 3160
size_t sg2_bilevel_workspace_bytes(const SgDims* dims, int num_tensors, const int64_t* numels);

/* The same pair with the quantities the reference's own bilevel entry points
 * exchange with their Python caller (supergrok2_bilevel_fwd_save[_batched] /
 * supergrok2_bilevel_backward[_batched], csrc/ops.h:232-371; caller
 * grokking_optimizers/supergrok2.py:646-1040).
 * sg2_bilevel_forward_ex: ctx_out may be NULL; `extra` (may be NULL, and any of
 * its members) receives
 *   scan_out_fwd / scan_out_bwd [sum numel][d_inner]  the gated scan output
 *            y*silu(z) + D*x of every step, before out_proj, in scan order
 *            (forward: sorted position t; backward: step u = N-1-t), tensors
 *            packed in call order -- the reference's fwd/bwd_scan_out_packed;
 *   x_sorted [sum numel][d_model]     W_in [g, s] + b_in in sorted order;
 *   perm     [sum numel]              sorted position -> element index.
 * sg2_bilevel_backward_ex: exactly one of d_ctx (as above) and the pair
 * d_scan_out_fwd / d_scan_out_bwd (scan_out's layout; out_proj then stays with
 * the caller and its gradient is returned as zeros) is given.  dx_out (optional, with row_dx) receives
 * [2][sum numel][d_model]: each direction's gradient with respect to x_sorted,
 * in sorted order; row_dx is [2][80][d_model], the derivative of the 80
 * pre-activation rows of each direction (x-branch, z, dt, B, C: 16 each) with
 * respect to x, i.e. in_proj[:16], in_proj[16:], dt_W in_proj[:16],
 * B_proj in_proj[:16], C_proj in_proj[:16].
 * The backward call uses the chunk length and window of the forward call on the
 * same workspace, whatever the settings are by then. */
typedef struct Sg2BilevelExtra {
    float* scan_out_fwd;
    float* scan_out_bwd;
    float* x_sorted;
    int32_t* perm;
    /* What launch_mamba3_peer_bilevel_fwd_save[_batched] leaves for its backward pass
     * (csrc/supergrok2_mamba_peer_backward_kernels.cu:950-1008), per direction (0 forward, 1 backward), each may be
     * NULL: the x-branch, the gate pre-activation z and the step size dt of every scan step
     * ([sum numel][d_inner], rows in the order of the direction's own scan, like scan_out), and the scan state after
     * a step ([rows][d_inner][d_state]).  checkpoint_interval <= 1: after every step, row = the tensor's offset +
     * the step; otherwise after every checkpoint_interval-th step of the scan and after the last one, row = (sum
     * over the earlier tensors of ceil(numel / checkpoint_interval)) + step / checkpoint_interval.  This library's
     * own backward pass reads none of them. */
    float* saved_x_branch[2];
    float* saved_z[2];
    float* saved_dt[2];
    float* saved_states[2];
    int32_t checkpoint_interval;
} Sg2BilevelExtra;
int sg2_bilevel_forward_ex(const SgDims* dims, const Sg2Weights* weights, int num_tensors, const Sg2Tensor* tensors,
                           float* ctx_out, const Sg2BilevelExtra* extra, void* workspace, size_t workspace_bytes, void* stream);
int sg2_bilevel_backward_ex(const SgDims* dims, const Sg2Weights* weights, int num_tensors, const Sg2Tensor* tensors,
                            const float* d_ctx, const float* d_scan_out_fwd, const float* d_scan_out_bwd, const float* row_dx,
                            float* dx_out, float* grads_out, void* workspace, size_t workspace_bytes, void* stream);
int sg2_bilevel_forward(const SgDims* dims, const Sg2Weights* weights, int num_tensors, const Sg2Tensor* tensors,
                        float* ctx_out, void* workspace, size_t workspace_bytes, void* stream);
int sg2_bilevel_backward(const SgDims* dims, const Sg2Weights* weights, int num_tensors, const Sg2Tensor* tensors,
                         const float* d_ctx, float* grads_out, void* workspace, size_t workspace_bytes, void* stream);

/* sg2_bilevel_elem: the per-element part of Mamba3PEERMetaNet.forward_for_bilevel
 * (grokking_optimizers/mamba3_peer_metanet.py:395-436 of the reference) and its
 * derivative, for `total` elements given as flat fp32 arrays (all tensors of
 * the call packed in the order of sg2_bilevel_forward's ctx_out):
 *   grad, sharpness, cotangent [total]; ctx [2][total][d_model];
 *   gru_state [total][gru_hidden] (read only).
 * With smart_i = grad_i + rescale/heads * sum over heads of the softly routed
 * expert outputs, it writes
 *   smart_out [total]            (may be NULL)
 *   d_ctx     [2][total][d_model]   d/d ctx of  sum_i cotangent_i * smart_i
 *   grads_out [SG2_ELEM_GRAD_FLOATS], the same derivative for the weights:
 *     gru W_z[4][22] b_z[4] W_r[4][22] b_r[4] W_h[4][22] b_h[4], peer queries
 *     [4][8][22], product keys A [4][12][4], B [4][12][4], expert W1 [144][16],
 *     b1 [144][16], W2 [144][16], b2 [144].
 * Of `weights` only the GRU, query, key and expert entries are read.  ctx,
 * gru_state and d_ctx must be 16-byte aligned; the workspace holds one row of
 * partial sums per workgroup. */
#define SG2_ELEM_GRAD_FLOATS 8420
size_t sg2_bilevel_elem_workspace_bytes(int64_t total);
int sg2_bilevel_elem(const SgDims* dims, const Sg2Weights* weights, int64_t total, const float* grad, const float* sharpness,
                     const float* ctx, const float* gru_state, const float* cotangent, float rescale, float* smart_out,
                     float* d_ctx, float* grads_out, void* workspace, size_t workspace_bytes, void* stream);
/* ... and additionally the new GRU state of every element, gru_out [total][gru_hidden] (may be NULL): the second
 * return value of forward_for_bilevel (mamba3_peer_metanet.py:436). */
int sg2_bilevel_elem_ex(const SgDims* dims, const Sg2Weights* weights, int64_t total, const float* grad, const float* sharpness,
                        const float* ctx, const float* gru_state, const float* cotangent, float rescale, float* smart_out,
                        float* gru_out, float* d_ctx, float* grads_out, void* workspace, size_t workspace_bytes, void* stream);

/* The meta-net's own forward with the step's hard top-1 routing, for callers that use the net outside the fused
 * step: Mamba3PEERMetaNet.forward (grokking_optimizers/mamba3_peer_metanet.py:275-370 of the reference).  Sort,
 * scan and the per-element GRU / routing / experts as in sg2_batched_step, without the optimizer update: of every
 * tensor record only grad, sharpness, gru_state (read), the two Mamba states (replaced by the new carried states),
 * numel and dtype are used.  rescale: the net's output scale (smart = g + rescale * mean of the heads' expert
 * outputs).  smart_out [total] and gru_out [total][gru_hidden] are packed in call order;
 * expert_counts may be NULL.  Workspace as for sg2_batched_step (sg2_workspace_bytes). */
int sg2_meta_forward(const SgDims* dims, const Sg2Weights* weights, int num_tensors, const Sg2Tensor* tensors,
                     float rescale, float* smart_out, float* gru_out, int32_t* expert_counts, void* workspace,
                     size_t workspace_bytes, void* stream);

/* ================== the other fused steps of the reference ================== */

/* One tensor of an Adam-family fused step: the i-th entries of the tensor
 * vectors of the reference's *_fused_step functions.  Fields an entry point
 * does not use are ignored (may be NULL / 0). */
typedef struct SgFamilyTensor {
    void* param;        /* [numel] dtype, updated in place */
    void* grad;         /* [numel] dtype; rescaled in place when global-norm clipping is active */
    float* exp_avg;     /* [numel] fp32 */
    float* exp_avg_sq;  /* [numel] fp32 (not Lion) */
    float* aux;         /* [numel] fp32: GrokAdamW ema, Prodigy s, SuperGrok v1.1 mu */
    const void* aux2;   /* Prodigy: param_init [numel] fp32; SuperGrok v1.1: sharpness [numel] dtype */
    int64_t numel;
    int32_t dtype;
    float bc1, bc2;     /* 1 - beta1^step, 1 - beta2^step as the caller computed them */
    float alpha, beta1; /* SuperGrok v1.1 per-layer values */
} SgFamilyTensor;

/* 1 -> H -> 1 ReLU amplifier of NeuralGrok (first and last Linear of its _Amplifier). */
typedef struct SgAmplifier {
    const float* W1;    /* [hidden,1] */
    const float* b1;    /* [hidden]   */
    const float* W2;    /* [1,hidden] */
    const float* b2;    /* [1]        */
    int32_t hidden;     /* <= 256 */
} SgAmplifier;

/* Workspace for every entry point of this section: the elementwise bookkeeping
 * plus one float per element (SuperGrok v1.1 keeps the smart gradient there
 * between its two passes). */
size_t sg_family_workspace_bytes(int num_tensors, const int64_t* numels);

/* GrokAdamW: global-norm clip, ema = alpha*ema + (1-alpha)*g, g' = g + lamb*ema,
 * AdamW on g'.  Replaces grokadamw_fused_step (csrc/ops.cpp:311-353;
 * launch_fused_grokadamw_step, csrc/grokadamw_kernels.cu).  With lamb == 0 the
 * aux (ema) pointers may be NULL and the step is plain AdamW: the update of
 * grokking_optimizers/_adamw_helper.py:12-22 as one launch. */
int sg_grokadamw_step(int num_tensors, const SgFamilyTensor* tensors, float alpha, float lamb, float beta1, float beta2,
                      float lr, float wd, float eps, float grad_clip_norm, void* workspace, size_t workspace_bytes,
                      void* stream);

/* NeuralGrok: global-norm clip, g' = g * (alpha_amp * MLP(g) + beta_amp), AdamW
 * on g' in one pass.  Replaces neuralgrok_fused_step (csrc/ops.cpp:360-417;
 * fused_neuralgrok_full_step_kernel, csrc/neuralgrok_kernels.cu). */
int sg_neuralgrok_step(int num_tensors, const SgFamilyTensor* tensors, const SgAmplifier* amp, float alpha_amp,
                       float beta_amp, float beta1, float beta2, float lr, float wd, float eps, float grad_clip_norm,
                       void* workspace, size_t workspace_bytes, void* stream);

/* Prodigy: num = sum g.(p - p0), den = sum s reduced on the device;
 * d_lr <- max(d_lr, |num|/(den+1e-12)) when den > 1e-30; then the d_lr-scaled
 * Adam step.  The new d_lr is computed on the device, consumed by the step
 * kernel from device memory, and copied to *d_lr_out (the call synchronises
 * the stream for that copy, as the reference's own single sync does).
 * Replaces prodigy_fused_step (csrc/ops.cpp:424-506; csrc/prodigy_kernels.cu:50-170). */
int sg_prodigy_step(int num_tensors, const SgFamilyTensor* tensors, float d_lr, float beta1, float beta2, float lr,
                    float wd, float eps, float* d_lr_out, void* workspace, size_t workspace_bytes, void* stream);

/* Lion: p -= lr*(sign(beta1*m + (1-beta1)*g) + wd*p); m = beta2*m + (1-beta2)*g.
 * Replaces lion_fused_step (csrc/ops.cpp:536-560; csrc/lion_kernels.cu:20-56). */
int sg_lion_step(int num_tensors, const SgFamilyTensor* tensors, float lr, float beta1, float beta2, float wd,
                 void* workspace, size_t workspace_bytes, void* stream);

/* SuperGrok v1.1: global-norm clip; mu EMA and the 2->H->1 meta-net (pass 1,
 * smart gradient kept in the workspace); per tensor the cosine gate
 * sigmoid(T * <smart,mu> / (|smart||mu| + 1e-8)) from sums reduced on the
 * device, lamb_eff = ramp*gate*lamb (0 when ramp <= 0); Adam with decoupled
 * decay (pass 2).  No host synchronisation: the reference reads the gate back
 * once per tensor.  Replaces supergrok11_fused_step (csrc/ops.cpp:209-288;
 * csrc/supergrok11_kernels.cu).  net->gelu_mode as for sg15_fused_step. */
int sg11_fused_step(int num_tensors, const SgFamilyTensor* tensors, const Sg15Net* net, float beta2, float lr, float wd,
                    float eps, float lamb, float ramp, float gate_temperature, float grad_clip_norm, void* workspace,
                    size_t workspace_bytes, void* stream);

/* LookSAM.  The ascent step is sg15_sam_perturb (looksam_perturb_all is the same
 * computation, csrc/ops.cpp:566-590). */
typedef struct SgLookSamTensor {
    void* a;            /* restore: param;  directions: v_dir (fp32);      adjust: grad (dtype)  */
    const void* b;      /* restore: backup; directions: sam_grad (dtype);  adjust: v_dir (fp32)  */
    const void* c;      /*                  directions: normal_grad (dtype)                      */
    int64_t numel;
    int32_t dtype;
} SgLookSamTensor;
/* param <- backup (looksam_restore_all, csrc/ops.cpp:592-605). */
int sg_looksam_restore(int num_tensors, const SgLookSamTensor* tensors, void* workspace, size_t workspace_bytes,
                       void* stream);
/* v = (g_sam - g)/|g_sam - g| per tensor, left untouched when the norm is below
 * 1e-12; norms reduced on the device (looksam_compute_directions,
 * csrc/ops.cpp:607-630; launch_looksam_direction). */
int sg_looksam_directions(int num_tensors, const SgLookSamTensor* tensors, void* workspace, size_t workspace_bytes,
                          void* stream);
/* g += la*|g| * v per tensor (looksam_adjust_grads, csrc/ops.cpp:632-652). */
int sg_looksam_adjust(int num_tensors, const SgLookSamTensor* tensors, float la, void* workspace,
                      size_t workspace_bytes, void* stream);

/* Pre-pass of the SuperGrok v2 step, per tensor: out = g * c/(|g|+1e-12) when
 * |g| > c, else g; non-finite entries of the result become 0.  Norms are
 * reduced on the device.  Replaces the two host syncs per tensor of
 * grokking_optimizers/supergrok2.py:316-321 (grad.norm() > clip, then
 * isfinite(grad).all()).  out is a separate tensor, as the reference makes one;
 * workspace: sg_family_workspace_bytes. */
typedef struct Sg2ClipTensor {
    const void* grad;   /* [numel] dtype */
    void* out;          /* [numel] dtype */
    int64_t numel;
    int32_t dtype;
} Sg2ClipTensor;
int sg2_clip_grads(int num_tensors, const Sg2ClipTensor* tensors, float max_norm, void* workspace,
                   size_t workspace_bytes, void* stream);

/* ================================ Muon ==================================== */

/* One 2-D parameter of the Muon step: the i-th entries of the vectors of
 * muon_fused_step (csrc/ops.h:510-514).  buf is the fp32 momentum buffer
 * (grokking_optimizers/muon.py:145-147). */
typedef struct SgMuonMatrix {
    void* param;        /* [rows,cols] dtype, updated in place */
    const void* grad;   /* [rows,cols] dtype                   */
    float* buf;         /* [rows,cols] fp32, updated           */
    int64_t rows, cols;
    int32_t dtype;
} SgMuonMatrix;

size_t sg_muon_workspace_bytes(int num_matrices, const SgMuonMatrix* mats);

/* Muon step for all matrices: buf = momentum*buf + g; X = buf/(||buf||_F+1e-7)
 * with the norm reduced on the device; ns_steps quintic Newton-Schulz
 * iterations X <- aX + b(XX^T)X + c(XX^T)^2 X with (a,b,c) = (3.4445, -4.7750,
 * 2.0315); p = (p - 0.2*lr*X) * (1 - lr*wd).  The iterations run as bf16 MFMA
 * GEMMs with fp32 accumulation, on the Gram matrix of the smaller dimension
 * (X^T X for tall matrices; the same product re-associated).  Replaces the
 * body of muon_fused_step (csrc/ops.cpp:663-746: ATen norm + host sync,
 * three torch::mm per iteration, muon_ns_combine_kernel and
 * muon_update_kernel, csrc/muon_kernels.cu:37-72). */
int sg_muon_step(int num_matrices, const SgMuonMatrix* mats, float momentum, float lr, float wd, int ns_steps,
                 void* workspace, size_t workspace_bytes, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* SG_ABI_H_ */
