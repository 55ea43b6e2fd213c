// The reference's four bilevel entry points of the SuperGrok v2 meta-net
//   supergrok2_bilevel_fwd_save[_batched], supergrok2_bilevel_backward[_batched]
// (csrc/ops.h:232-371, bound at csrc/ops.cpp:1072-1085 of the reference), with the reference's argument lists,
// over sg2_bilevel_forward_ex / sg2_bilevel_backward_ex of libsg_hip.so.
//
// What is honoured: everything the reference's caller (grokking_optimizers/supergrok2.py:646-1040) reads between the
// two calls and after them -- the gated scan outputs before out_proj in scan order, x_sorted, sort_indices, offsets,
// the gradients of the 16 Mamba weight tensors (accumulated into the d_* arguments) and d_x_sorted.
// What is not: the per-step `*_saved_*` buffers stay untouched.  The HIP adjoint recomputes the states of a 32-step
// tile from the state entering it, which the forward call keeps in a workspace of its own; fwd_save_batched parks that
// workspace under the address of `x_sorted_packed`, where backward_batched (which receives the same tensor) finds it.
// checkpoint_interval is accepted and ignored.
#include <torch/extension.h>

#include <c10/hip/HIPStream.h>

#include <map>
#include <mutex>
#include <vector>

#include "../../include/sg_abi.h"

namespace {

void require_f32_gpu(const torch::Tensor& t, const char* fn, const char* what) {
    TORCH_CHECK(t.defined() && t.is_cuda(), fn, ": ", what, " must be a GPU tensor");
    TORCH_CHECK(t.scalar_type() == torch::kFloat32 && t.is_contiguous(), fn, ": ", what, " must be contiguous float32");
}
void* stream_of(const torch::Tensor& t) { return (void*)c10::hip::getCurrentHIPStream(t.device().index()).stream(); }
int dtype_of(const torch::Tensor& t, const char* fn) {
    if (t.scalar_type() == torch::kFloat32) return SG_F32;
    if (t.scalar_type() == torch::kFloat16) return SG_F16;
    TORCH_CHECK(t.scalar_type() == torch::kBFloat16, fn, ": gradients must be float32, float16 or bfloat16");
    return SG_BF16;
}

// the meta-net dimensions the HIP kernels are built for; the scan part only depends on the first three
SgDims default_dims(int d_model, int d_state, int d_inner) { return SgDims{d_model, d_state, d_inner, 4, 4, 12, 16, 144}; }

struct ScanWeights {
    torch::Tensor t[20];          // input_proj W, b; forward block (9); backward block (9)
    Sg2Weights W;
    void fill(const char* fn, const SgDims& d) {
        // element counts in argument order: input_proj W [d_model, 2], b [d_model]; per direction in_proj [2 d_inner, d_model],
        // dt_W [d_inner, d_inner], dt_b [d_inner], B_proj / C_proj [d_state, d_inner], A_log [d_inner, d_state], D [d_inner],
        // rope [d_inner, d_state/2], out_proj [d_model, d_inner]
        const int64_t dm = d.d_model, ds = d.d_state, di = d.d_inner;
        const int64_t block[9] = {2 * di * dm, di * di, di, ds * di, ds * di, di * ds, di, di * (ds / 2), dm * di};
        for (int k = 0; k < 20; k++) {
            require_f32_gpu(t[k], fn, "meta-net weight");
            const int64_t want = k == 0 ? 2 * dm : (k == 1 ? dm : block[(k - 2) % 9]);
            TORCH_CHECK(t[k].numel() == want, fn, ": meta-net weight ", k, " has ", t[k].numel(), " elements, expected ", want);
            W.w[k] = t[k].data_ptr<float>();
        }
        for (int k = 20; k < SG2_NUM_WEIGHTS; k++) W.w[k] = W.w[0];      // per-element weights: never read by sort and scan
    }
};

// everything the backward call needs again, kept alive between the two calls
struct Saved {
    ScanWeights w;
    std::vector<torch::Tensor> grads, sharps;
    torch::Tensor mf, mb, workspace;
    std::vector<Sg2Tensor> tensors;
    int64_t total = 0;
};
std::mutex g_mutex;
std::map<const void*, Saved> g_saved;          // keyed by x_sorted_packed.data_ptr()

void run_forward(const char* fn, Saved& S, const SgDims& dims, torch::Tensor fwd_scan_out, torch::Tensor bwd_scan_out, torch::Tensor x_sorted,
                 torch::Tensor sort_indices) {
    const size_t P = S.grads.size();
    std::vector<int64_t> numels(P);
    S.tensors.assign(P, Sg2Tensor{});
    S.total = 0;
    for (size_t i = 0; i < P; i++) {
        const auto& g = S.grads[i];
        const auto& s = S.sharps[i];
        TORCH_CHECK(g.is_cuda() && s.is_cuda() && g.is_contiguous() && s.is_contiguous(), fn, ": gradients and sharpness must be contiguous GPU tensors");
        TORCH_CHECK(g.scalar_type() == s.scalar_type() && g.numel() == s.numel(), fn, ": gradient and sharpness of a parameter must match");
        Sg2Tensor& t = S.tensors[i];
        t.grad = g.data_ptr();
        t.sharpness = s.data_ptr();
        t.mamba_fwd_state = S.mf.data_ptr<float>() + (int64_t)i * dims.d_inner * dims.d_state;
        t.mamba_bwd_state = S.mb.data_ptr<float>() + (int64_t)i * dims.d_inner * dims.d_state;
        t.numel = g.numel();
        t.dtype = dtype_of(g, fn);
        numels[i] = g.numel();
        S.total += g.numel();
    }
    for (const torch::Tensor* out : {&fwd_scan_out, &bwd_scan_out}) {
        require_f32_gpu(*out, fn, "scan_out");
        TORCH_CHECK(out->numel() == S.total * dims.d_inner, fn, ": scan_out must hold [sum N, d_inner] floats");
    }
    require_f32_gpu(x_sorted, fn, "x_sorted");
    TORCH_CHECK(x_sorted.numel() == S.total * dims.d_model, fn, ": x_sorted must hold [sum N, d_model] floats");
    TORCH_CHECK(sort_indices.is_cuda() && sort_indices.scalar_type() == torch::kInt32 && sort_indices.is_contiguous() &&
                    sort_indices.numel() == S.total, fn, ": sort_indices must be a contiguous int32 GPU tensor of sum N entries");
    const size_t bytes = sg2_bilevel_workspace_bytes(&dims, (int)P, numels.data());
    TORCH_CHECK(bytes > 0 || S.total == 0, fn, ": ", sg_last_error());
    S.workspace = torch::empty({(int64_t)std::max<size_t>(bytes, 256)}, torch::TensorOptions().device(S.w.t[0].device()).dtype(torch::kUInt8));
    Sg2BilevelExtra extra = {fwd_scan_out.data_ptr<float>(), bwd_scan_out.data_ptr<float>(), x_sorted.data_ptr<float>(),
                             sort_indices.data_ptr<int32_t>()};
    const int rc = sg2_bilevel_forward_ex(&dims, &S.w.W, (int)P, S.tensors.data(), nullptr, &extra, S.workspace.data_ptr(),
                                          (size_t)S.workspace.numel(), stream_of(S.w.t[0]));
    TORCH_CHECK(rc == 0, fn, ": ", sg_last_error());
}

torch::Tensor initial_states(const char* fn, const torch::Tensor& given, int64_t P, const SgDims& dims, const torch::Tensor& like) {
    const int64_t per = (int64_t)dims.d_inner * dims.d_state;
    if (!given.defined() || given.numel() == 0) return torch::zeros({P, dims.d_inner, dims.d_state}, like.options().dtype(torch::kFloat32));
    TORCH_CHECK(given.is_cuda() && given.numel() == P * per, fn, ": initial Mamba states must hold [num_params, d_inner, d_state] floats");
    return given.to(torch::kFloat32).contiguous().clone();       // the forward overwrites its state argument with the final state
}

}  // namespace

void supergrok2_bilevel_fwd_save_batched(
    std::vector<torch::Tensor> grads, std::vector<torch::Tensor> sharpness_list, torch::Tensor input_proj_W, torch::Tensor input_proj_b,
    torch::Tensor mamba_fwd_in_proj, torch::Tensor mamba_fwd_dt_W, torch::Tensor mamba_fwd_dt_b, torch::Tensor mamba_fwd_B_proj,
    torch::Tensor mamba_fwd_C_proj, torch::Tensor mamba_fwd_A_log, torch::Tensor mamba_fwd_D, torch::Tensor mamba_fwd_rope,
    torch::Tensor mamba_fwd_out_proj, torch::Tensor mamba_bwd_in_proj, torch::Tensor mamba_bwd_dt_W, torch::Tensor mamba_bwd_dt_b,
    torch::Tensor mamba_bwd_B_proj, torch::Tensor mamba_bwd_C_proj, torch::Tensor mamba_bwd_A_log, torch::Tensor mamba_bwd_D,
    torch::Tensor mamba_bwd_rope, torch::Tensor mamba_bwd_out_proj, int d_model, int d_state, int d_inner,
    torch::Tensor fwd_scan_out_packed, torch::Tensor bwd_scan_out_packed, torch::Tensor fwd_saved_states_packed,
    torch::Tensor fwd_saved_xb_packed, torch::Tensor fwd_saved_z_packed, torch::Tensor fwd_saved_dt_packed,
    torch::Tensor bwd_saved_states_packed, torch::Tensor bwd_saved_xb_packed, torch::Tensor bwd_saved_z_packed,
    torch::Tensor bwd_saved_dt_packed, torch::Tensor x_sorted_packed, torch::Tensor offsets_t, torch::Tensor sort_indices_packed,
    torch::Tensor fwd_initial_states, torch::Tensor bwd_initial_states, int checkpoint_interval) {
    const char* fn = "supergrok2_bilevel_fwd_save_batched";
    (void)checkpoint_interval;
    if (grads.empty()) return;
    TORCH_CHECK(sharpness_list.size() == grads.size(), fn, ": one sharpness tensor per gradient");
    if (!grads[0].is_cuda()) throw std::runtime_error("supergrok2_bilevel_fwd_save_batched requires CUDA tensors.");
    const SgDims dims = default_dims(d_model, d_state, d_inner);
    Saved S;
    const torch::Tensor w[20] = {input_proj_W, input_proj_b, mamba_fwd_in_proj, mamba_fwd_dt_W, mamba_fwd_dt_b, mamba_fwd_B_proj,
                                 mamba_fwd_C_proj, mamba_fwd_A_log, mamba_fwd_D, mamba_fwd_rope, mamba_fwd_out_proj, mamba_bwd_in_proj,
                                 mamba_bwd_dt_W, mamba_bwd_dt_b, mamba_bwd_B_proj, mamba_bwd_C_proj, mamba_bwd_A_log, mamba_bwd_D,
                                 mamba_bwd_rope, mamba_bwd_out_proj};
    for (int k = 0; k < 20; k++) S.w.t[k] = w[k];
    S.w.fill(fn, dims);
    S.grads = grads;
    S.sharps = sharpness_list;
    const int64_t P = (int64_t)grads.size();
    S.mf = initial_states(fn, fwd_initial_states, P, dims, input_proj_W);
    S.mb = initial_states(fn, bwd_initial_states, P, dims, input_proj_W);
    run_forward(fn, S, dims, fwd_scan_out_packed, bwd_scan_out_packed, x_sorted_packed, sort_indices_packed);
    // element offsets of the tensors in the packed arrays
    TORCH_CHECK(offsets_t.scalar_type() == torch::kInt32 && offsets_t.numel() == P + 1, fn, ": offsets_t must be int32[num_params + 1]");
    std::vector<int32_t> off(P + 1, 0);
    for (int64_t i = 0; i < P; i++) off[i + 1] = off[i] + (int32_t)grads[i].numel();
    offsets_t.copy_(torch::from_blob(off.data(), {P + 1}, torch::kInt32).clone());
    std::lock_guard<std::mutex> lock(g_mutex);
    if (g_saved.size() >= 4) g_saved.clear();          // forward calls that were never followed by a backward call
    g_saved[x_sorted_packed.data_ptr()] = std::move(S);
}

void supergrok2_bilevel_backward_batched(
    torch::Tensor d_fwd_scan_out_packed, torch::Tensor d_bwd_scan_out_packed, torch::Tensor x_sorted_packed,
    torch::Tensor fwd_saved_states_packed, torch::Tensor fwd_saved_xb_packed, torch::Tensor fwd_saved_z_packed,
    torch::Tensor fwd_saved_dt_packed, torch::Tensor bwd_saved_states_packed, torch::Tensor bwd_saved_xb_packed,
    torch::Tensor bwd_saved_z_packed, torch::Tensor bwd_saved_dt_packed, torch::Tensor offsets_t, torch::Tensor mamba_fwd_in_proj,
    torch::Tensor mamba_fwd_dt_W, torch::Tensor mamba_fwd_dt_b, torch::Tensor mamba_fwd_B_proj, torch::Tensor mamba_fwd_C_proj,
    torch::Tensor mamba_fwd_A_log, torch::Tensor mamba_fwd_D, torch::Tensor mamba_fwd_rope, torch::Tensor mamba_bwd_in_proj,
    torch::Tensor mamba_bwd_dt_W, torch::Tensor mamba_bwd_dt_b, torch::Tensor mamba_bwd_B_proj, torch::Tensor mamba_bwd_C_proj,
    torch::Tensor mamba_bwd_A_log, torch::Tensor mamba_bwd_D, torch::Tensor mamba_bwd_rope, torch::Tensor d_mamba_fwd_in_proj,
    torch::Tensor d_mamba_fwd_dt_W, torch::Tensor d_mamba_fwd_dt_b, torch::Tensor d_mamba_fwd_B_proj, torch::Tensor d_mamba_fwd_C_proj,
    torch::Tensor d_mamba_fwd_A_log, torch::Tensor d_mamba_fwd_D, torch::Tensor d_mamba_fwd_rope, torch::Tensor d_mamba_bwd_in_proj,
    torch::Tensor d_mamba_bwd_dt_W, torch::Tensor d_mamba_bwd_dt_b, torch::Tensor d_mamba_bwd_B_proj, torch::Tensor d_mamba_bwd_C_proj,
    torch::Tensor d_mamba_bwd_A_log, torch::Tensor d_mamba_bwd_D, torch::Tensor d_mamba_bwd_rope, torch::Tensor d_x_sorted_packed,
    torch::Tensor fwd_initial_states, torch::Tensor bwd_initial_states, int d_model, int d_state, int d_inner, int num_params,
    int checkpoint_interval) {
    const char* fn = "supergrok2_bilevel_backward_batched";
    (void)checkpoint_interval;
    if (num_params == 0) return;
    Saved S;
    {
        std::lock_guard<std::mutex> lock(g_mutex);
        const auto it = g_saved.find(x_sorted_packed.data_ptr());
        TORCH_CHECK(it != g_saved.end(), fn, ": no supergrok2_bilevel_fwd_save_batched call has filled this x_sorted_packed tensor "
                    "(the backward pass restarts from what that call kept)");
        S = std::move(it->second);
        g_saved.erase(it);
    }
    TORCH_CHECK((int)S.grads.size() == num_params, fn, ": num_params differs from the forward call");
    const torch::Tensor given[16] = {mamba_fwd_in_proj, mamba_fwd_dt_W, mamba_fwd_dt_b, mamba_fwd_B_proj, mamba_fwd_C_proj, mamba_fwd_A_log,
                                     mamba_fwd_D, mamba_fwd_rope, mamba_bwd_in_proj, mamba_bwd_dt_W, mamba_bwd_dt_b, mamba_bwd_B_proj,
                                     mamba_bwd_C_proj, mamba_bwd_A_log, mamba_bwd_D, mamba_bwd_rope};
    for (int dir = 0; dir < 2; dir++)
        for (int k = 0; k < 8; k++)
            TORCH_CHECK(given[dir * 8 + k].data_ptr() == S.w.t[2 + dir * 9 + k].data_ptr(), fn,
                        ": the Mamba weights must be the tensors the forward call received");
    const SgDims dims = default_dims(d_model, d_state, d_inner);
    require_f32_gpu(d_fwd_scan_out_packed, fn, "d_fwd_scan_out_packed");
    require_f32_gpu(d_bwd_scan_out_packed, fn, "d_bwd_scan_out_packed");
    require_f32_gpu(d_x_sorted_packed, fn, "d_x_sorted_packed");
    TORCH_CHECK(d_fwd_scan_out_packed.numel() == S.total * d_inner && d_bwd_scan_out_packed.numel() == S.total * d_inner &&
                    d_x_sorted_packed.numel() == S.total * d_model, fn, ": packed gradient tensors do not match the forward call");
    // derivative of the 80 pre-activation rows of each direction with respect to x: [x-branch, z, dt, B, C] x d_model
    std::vector<torch::Tensor> rows;
    for (int dir = 0; dir < 2; dir++) {
        const torch::Tensor& in_proj = S.w.t[2 + dir * 9];
        const torch::Tensor X = in_proj.view({2 * d_inner, d_model}).narrow(0, 0, d_inner), Z = in_proj.view({2 * d_inner, d_model}).narrow(0, d_inner, d_inner);
        rows.push_back(torch::cat({X, Z, torch::mm(S.w.t[3 + dir * 9].view({d_inner, d_inner}), X), torch::mm(S.w.t[5 + dir * 9].view({d_state, d_inner}), X),
                                   torch::mm(S.w.t[6 + dir * 9].view({d_state, d_inner}), X)}, 0));
    }
    const torch::Tensor row_dx = torch::stack(rows, 0).contiguous();
    auto opts = d_x_sorted_packed.options();
    torch::Tensor dx = torch::empty({2, S.total, (int64_t)d_model}, opts), block = torch::empty({SG2_SCAN_GRAD_FLOATS}, opts);
    const int rc = sg2_bilevel_backward_ex(&dims, &S.w.W, num_params, S.tensors.data(), nullptr, d_fwd_scan_out_packed.data_ptr<float>(),
                                           d_bwd_scan_out_packed.data_ptr<float>(), row_dx.data_ptr<float>(), dx.data_ptr<float>(),
                                           block.data_ptr<float>(), S.workspace.data_ptr(), (size_t)S.workspace.numel(), stream_of(block));
    TORCH_CHECK(rc == 0, fn, ": ", sg_last_error());
    d_x_sorted_packed.view({S.total, (int64_t)d_model}).add_(dx[0]).add_(dx[1]);
    // block layout: input_proj W [8][2], b [8]; per direction in_proj, dt_W, dt_b, B_proj, C_proj, A_log, D, rope, out_proj
    torch::Tensor d_out[16] = {d_mamba_fwd_in_proj, d_mamba_fwd_dt_W, d_mamba_fwd_dt_b, d_mamba_fwd_B_proj, d_mamba_fwd_C_proj, d_mamba_fwd_A_log,
                               d_mamba_fwd_D, d_mamba_fwd_rope, d_mamba_bwd_in_proj, d_mamba_bwd_dt_W, d_mamba_bwd_dt_b, d_mamba_bwd_B_proj,
                               d_mamba_bwd_C_proj, d_mamba_bwd_A_log, d_mamba_bwd_D, d_mamba_bwd_rope};
    int64_t at = 3 * d_model;
    for (int dir = 0; dir < 2; dir++) {
        for (int k = 0; k < 8; k++) {
            torch::Tensor& d = d_out[dir * 8 + k];
            require_f32_gpu(d, fn, "gradient accumulator");
            TORCH_CHECK(d.numel() == S.w.t[2 + dir * 9 + k].numel(), fn, ": gradient accumulator ", dir * 8 + k, " has the wrong size");
            d.view({-1}).add_(block.narrow(0, at, d.numel()));
            at += d.numel();
        }
        at += (int64_t)d_model * d_inner;       // out_proj: stays with the caller in this interface
    }
}

void supergrok2_bilevel_fwd_save(
    torch::Tensor grad, torch::Tensor sharpness, torch::Tensor input_proj_W, torch::Tensor input_proj_b, torch::Tensor mamba_fwd_in_proj,
    torch::Tensor mamba_fwd_dt_W, torch::Tensor mamba_fwd_dt_b, torch::Tensor mamba_fwd_B_proj, torch::Tensor mamba_fwd_C_proj,
    torch::Tensor mamba_fwd_A_log, torch::Tensor mamba_fwd_D, torch::Tensor mamba_fwd_rope, torch::Tensor mamba_fwd_out_proj,
    torch::Tensor mamba_bwd_in_proj, torch::Tensor mamba_bwd_dt_W, torch::Tensor mamba_bwd_dt_b, torch::Tensor mamba_bwd_B_proj,
    torch::Tensor mamba_bwd_C_proj, torch::Tensor mamba_bwd_A_log, torch::Tensor mamba_bwd_D, torch::Tensor mamba_bwd_rope,
    torch::Tensor mamba_bwd_out_proj, int d_model, int d_state, int d_inner, torch::Tensor fwd_scan_out, torch::Tensor bwd_scan_out,
    torch::Tensor fwd_final_state, torch::Tensor bwd_final_state, torch::Tensor fwd_saved_states, torch::Tensor fwd_saved_x_branch,
    torch::Tensor fwd_saved_z, torch::Tensor fwd_saved_dt, torch::Tensor bwd_saved_states, torch::Tensor bwd_saved_x_branch,
    torch::Tensor bwd_saved_z, torch::Tensor bwd_saved_dt, torch::Tensor x_sorted, torch::Tensor sort_indices,
    torch::Tensor fwd_initial_state, torch::Tensor bwd_initial_state, int checkpoint_interval) {
    const char* fn = "supergrok2_bilevel_fwd_save";
    (void)checkpoint_interval;
    if (!grad.defined() || grad.numel() == 0) return;
    if (!grad.is_cuda()) throw std::runtime_error("supergrok2_bilevel_fwd_save requires CUDA tensors.");
    const SgDims dims = default_dims(d_model, d_state, d_inner);
    Saved S;
    const torch::Tensor w[20] = {input_proj_W, input_proj_b, mamba_fwd_in_proj, mamba_fwd_dt_W, mamba_fwd_dt_b, mamba_fwd_B_proj,
                                 mamba_fwd_C_proj, mamba_fwd_A_log, mamba_fwd_D, mamba_fwd_rope, mamba_fwd_out_proj, mamba_bwd_in_proj,
                                 mamba_bwd_dt_W, mamba_bwd_dt_b, mamba_bwd_B_proj, mamba_bwd_C_proj, mamba_bwd_A_log, mamba_bwd_D,
                                 mamba_bwd_rope, mamba_bwd_out_proj};
    for (int k = 0; k < 20; k++) S.w.t[k] = w[k];
    S.w.fill(fn, dims);
    S.grads = {grad.contiguous()};
    S.sharps = {sharpness.contiguous()};
    S.mf = initial_states(fn, fwd_initial_state, 1, dims, input_proj_W);
    S.mb = initial_states(fn, bwd_initial_state, 1, dims, input_proj_W);
    run_forward(fn, S, dims, fwd_scan_out, bwd_scan_out, x_sorted, sort_indices);
    require_f32_gpu(fwd_final_state, fn, "fwd_final_state");
    require_f32_gpu(bwd_final_state, fn, "bwd_final_state");
    fwd_final_state.view({-1}).copy_(S.mf.view({-1}));
    bwd_final_state.view({-1}).copy_(S.mb.view({-1}));
}
