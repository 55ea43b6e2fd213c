// The reference's four bilevel entry points of the SuperGrok v2 meta-net
//   supergrok2_bilevel_fwd_save[_batched], supergrok2_bilevel_backward[_batched]
// (csrc/ops.h:232-371, bound at csrc/ops.cpp:1072-1085 of the reference), with the reference's argument lists,
// over sg2_bilevel_forward_ex / sg2_bilevel_backward_ex of libsg_hip.so.
//
// What is honoured: everything the reference's caller (grokking_optimizers/supergrok2.py:646-1330) reads between the
// two calls and after them -- the gated scan outputs before out_proj in scan order, x_sorted, sort_indices, offsets,
// the gradients of the Mamba weight tensors (accumulated into the d_* arguments) and d_x_sorted; for the one-tensor
// pair also the gradients of every other weight of the meta-net.
// The per-step buffers of the interface are filled too, with the reference's layout (`*_saved_x_branch / z / dt` per
// sorted position; `*_saved_states` after every step, or after every checkpoint_interval-th step of a scan and its
// last one), although this library's backward pass reads none of them: its adjoint recomputes the states of a
// 32-step tile from the state entering it, which the forward call keeps in a workspace of its own.  That workspace
// (with the tensors it refers to) is parked in this process under a fresh 64-bit ticket, and the ticket is written
// into the first four floats of the caller's `fwd_saved_states` tensor (which therefore do not hold state entries)
// -- the tensor the backward call receives again: it reads the ticket back (one 16-byte device-to-host copy) and
// claims exactly the forward call that filled its buffers.  Two optimizers, or interleaved forward / backward pairs,
// therefore never see each other's state; a buffer no forward call has filled, or one whose ticket was already
// claimed, is refused.  At most MAX_PARKED forward calls are kept; the oldest is dropped first.
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
    const void* x_sorted_ptr = nullptr;
};
std::mutex g_mutex;
std::map<uint64_t, Saved> g_saved;             // keyed by ticket; std::map iterates in ticket order = age
uint64_t g_next_ticket = 1;
constexpr size_t MAX_PARKED = 16;
constexpr uint32_t TICKET_MAGIC = 0x5347324Bu;  // "SG2K"

// Parks a forward call and writes its ticket into the caller's fwd_saved_states tensor: [magic, low, high, ~magic].
void park(const char* fn, Saved&& S, torch::Tensor& tag) {
    TORCH_CHECK(tag.defined() && tag.is_cuda() && tag.scalar_type() == torch::kFloat32 && tag.is_contiguous() && tag.numel() >= 4, fn,
                ": fwd_saved_states must be a contiguous float32 GPU tensor of at least 4 elements (it carries the ticket of this call)");
    uint64_t ticket;
    {
        std::lock_guard<std::mutex> lock(g_mutex);
        ticket = g_next_ticket++;
        while (g_saved.size() >= MAX_PARKED) g_saved.erase(g_saved.begin());     // forward calls never followed by a backward call: oldest first
        g_saved.emplace(ticket, std::move(S));
    }
    torch::Tensor words = torch::empty({4}, torch::kInt32);
    int32_t* w = words.data_ptr<int32_t>();
    w[0] = (int32_t)TICKET_MAGIC; w[1] = (int32_t)(uint32_t)ticket; w[2] = (int32_t)(uint32_t)(ticket >> 32); w[3] = (int32_t)~TICKET_MAGIC;
    tag.view({-1}).narrow(0, 0, 4).view(torch::kInt32).copy_(words);
}

// Reads the ticket back and takes the parked call out of the table.
Saved claim(const char* fn, const char* fwd_name, const torch::Tensor& tag) {
    TORCH_CHECK(tag.defined() && tag.is_cuda() && tag.scalar_type() == torch::kFloat32 && tag.is_contiguous() && tag.numel() >= 4, fn,
                ": fwd_saved_states must be the tensor the forward call received");
    const torch::Tensor words = tag.view({-1}).narrow(0, 0, 4).view(torch::kInt32).cpu();
    const int32_t* w = words.data_ptr<int32_t>();
    const bool tagged = (uint32_t)w[0] == TICKET_MAGIC && (uint32_t)w[3] == ~TICKET_MAGIC;
    const uint64_t ticket = (uint64_t)(uint32_t)w[1] | ((uint64_t)(uint32_t)w[2] << 32);
    std::lock_guard<std::mutex> lock(g_mutex);
    const auto it = tagged ? g_saved.find(ticket) : g_saved.end();
    TORCH_CHECK(it != g_saved.end(), fn, ": no ", fwd_name, " call has filled these buffers, or its backward pass has already run "
                "(the backward pass restarts from what that call kept; one forward call, then one backward call)");
    Saved S = std::move(it->second);
    g_saved.erase(it);
    return S;
}

// The per-step buffers of the reference's interface (saved x-branch, z, dt: [sum N, d_inner]; saved states:
// [rows, d_inner, d_state], rows = sum N for checkpoint_interval <= 1, else sum of ceil(N_i / checkpoint_interval)).
// A tensor of exactly that size is filled; a smaller one is taken as "not wanted" (fwd_saved_states still carries the
// ticket of the call in its first four floats, which therefore do not hold state entries).
struct SavedBuffers {
    torch::Tensor states[2], xb[2], z[2], dt[2];
    int checkpoint_interval = 1;
};
float* wanted(const char* fn, const torch::Tensor& t, int64_t numel, const char* what) {
    if (!t.defined() || t.numel() < numel) return nullptr;
    TORCH_CHECK(t.numel() == numel, fn, ": ", what, " holds ", t.numel(), " floats, more than the ", numel, " this call fills");
    require_f32_gpu(t, fn, what);
    return t.data_ptr<float>();
}

void run_forward(const char* fn, Saved& S, const SgDims& dims, torch::Tensor fwd_scan_out, torch::Tensor bwd_scan_out, torch::Tensor x_sorted,
                 torch::Tensor sort_indices, const SavedBuffers& sv) {
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
    S.x_sorted_ptr = x_sorted.data_ptr();
    TORCH_CHECK(sort_indices.is_cuda() && sort_indices.scalar_type() == torch::kInt32 && sort_indices.is_contiguous() &&
                    sort_indices.numel() == S.total, fn, ": sort_indices must be a contiguous int32 GPU tensor of sum N entries");
    const size_t bytes = sg2_bilevel_workspace_bytes(&dims, (int)P, numels.data());
    TORCH_CHECK(bytes > 0 || S.total == 0, fn, ": ", sg_last_error());
    S.workspace = torch::empty({(int64_t)std::max<size_t>(bytes, 256)}, torch::TensorOptions().device(S.w.t[0].device()).dtype(torch::kUInt8));
    Sg2BilevelExtra extra = {};
    extra.scan_out_fwd = fwd_scan_out.data_ptr<float>();
    extra.scan_out_bwd = bwd_scan_out.data_ptr<float>();
    extra.x_sorted = x_sorted.data_ptr<float>();
    extra.perm = sort_indices.data_ptr<int32_t>();
    extra.checkpoint_interval = sv.checkpoint_interval;
    int64_t rows = 0;
    for (size_t i = 0; i < P; i++) rows += sv.checkpoint_interval <= 1 ? numels[i] : (numels[i] + sv.checkpoint_interval - 1) / sv.checkpoint_interval;
    for (int d = 0; d < 2; d++) {
        extra.saved_x_branch[d] = wanted(fn, sv.xb[d], S.total * dims.d_inner, "saved_x_branch");
        extra.saved_z[d] = wanted(fn, sv.z[d], S.total * dims.d_inner, "saved_z");
        extra.saved_dt[d] = wanted(fn, sv.dt[d], S.total * dims.d_inner, "saved_dt");
        extra.saved_states[d] = wanted(fn, sv.states[d], rows * dims.d_inner * dims.d_state, "saved_states");
    }
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
    SavedBuffers sv;
    sv.states[0] = fwd_saved_states_packed; sv.xb[0] = fwd_saved_xb_packed; sv.z[0] = fwd_saved_z_packed; sv.dt[0] = fwd_saved_dt_packed;
    sv.states[1] = bwd_saved_states_packed; sv.xb[1] = bwd_saved_xb_packed; sv.z[1] = bwd_saved_z_packed; sv.dt[1] = bwd_saved_dt_packed;
    sv.checkpoint_interval = checkpoint_interval;
    run_forward(fn, S, dims, fwd_scan_out_packed, bwd_scan_out_packed, x_sorted_packed, sort_indices_packed, sv);
    // element offsets of the tensors in the packed arrays
    TORCH_CHECK(offsets_t.scalar_type() == torch::kInt32 && offsets_t.numel() == P + 1, fn, ": offsets_t must be int32[num_params + 1]");
    std::vector<int32_t> off(P + 1, 0);
    for (int64_t i = 0; i < P; i++) off[i + 1] = off[i] + (int32_t)grads[i].numel();
    offsets_t.copy_(torch::from_blob(off.data(), {P + 1}, torch::kInt32).clone());
    park(fn, std::move(S), fwd_saved_states_packed);
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
    (void)checkpoint_interval;      // the adjoint restarts from the tile states of the forward call's workspace
    if (num_params == 0) return;
    Saved S = claim(fn, "supergrok2_bilevel_fwd_save_batched", fwd_saved_states_packed);
    TORCH_CHECK((int)S.grads.size() == num_params, fn, ": num_params differs from the forward call");
    TORCH_CHECK(S.x_sorted_ptr == x_sorted_packed.data_ptr(), fn, ": x_sorted_packed is not the tensor the forward call filled");
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
    SavedBuffers sv;
    sv.states[0] = fwd_saved_states; sv.xb[0] = fwd_saved_x_branch; sv.z[0] = fwd_saved_z; sv.dt[0] = fwd_saved_dt;
    sv.states[1] = bwd_saved_states; sv.xb[1] = bwd_saved_x_branch; sv.z[1] = bwd_saved_z; sv.dt[1] = bwd_saved_dt;
    sv.checkpoint_interval = checkpoint_interval;
    run_forward(fn, S, dims, fwd_scan_out, bwd_scan_out, x_sorted, sort_indices, sv);
    require_f32_gpu(fwd_final_state, fn, "fwd_final_state");
    require_f32_gpu(bwd_final_state, fn, "bwd_final_state");
    fwd_final_state.view({-1}).copy_(S.mf.view({-1}));
    bwd_final_state.view({-1}).copy_(S.mb.view({-1}));
    park(fn, std::move(S), fwd_saved_states);
}


// One tensor, the whole meta-net (csrc/ops.h:256-299, launch_mamba3_peer_backward in
// csrc/supergrok2_mamba_peer_backward_kernels.cu:2745-3098 of the reference).  The caller has run the per-element
// part of the forward pass itself, in torch, and hands over what it saw there (gates, candidates, routing weights,
// hidden activations of the picked experts ...), so the per-element backward is a chain of small dense products over
// those saved values and is written with ATen calls here, step for step as the reference's launcher orders it
// (experts and routing, GRU, context gradients, sort, out_proj); the scan's adjoint -- the expensive part -- is the
// HIP pass of sg2_bilevel_backward_ex on the workspace the forward call parked, and the input projection is one
// more product.  Every d_* argument is accumulated into.  (The reference overwrites d_B_proj / d_C_proj with the
// current tensor's term, `torch::mm_out` at :2999-3000 and :3045-3046 there, so that after its loop over parameters
// only the last one's contribution is left; this function adds like it does everywhere else.)
void supergrok2_bilevel_backward(
    torch::Tensor d_smart_grad, torch::Tensor grad, torch::Tensor sharpness, float rescale, torch::Tensor sort_indices, torch::Tensor x_sorted,
    torch::Tensor fwd_scan_out, torch::Tensor bwd_scan_out, torch::Tensor fwd_saved_states, torch::Tensor fwd_saved_x_branch,
    torch::Tensor fwd_saved_z, torch::Tensor fwd_saved_dt, torch::Tensor bwd_saved_states, torch::Tensor bwd_saved_x_branch,
    torch::Tensor bwd_saved_z, torch::Tensor bwd_saved_dt, torch::Tensor gru_input, torch::Tensor gru_h_old, torch::Tensor gru_z_gate,
    torch::Tensor gru_r_gate, torch::Tensor gru_h_tilde, torch::Tensor peer_input, torch::Tensor expert_indices, torch::Tensor routing_weights,
    torch::Tensor saved_z_hidden, torch::Tensor saved_scores_a, torch::Tensor saved_scores_b, torch::Tensor saved_top_a_idx,
    torch::Tensor saved_top_b_idx, torch::Tensor saved_soft_a, torch::Tensor saved_soft_b, torch::Tensor mamba_fwd_in_proj,
    torch::Tensor mamba_fwd_dt_W, torch::Tensor mamba_fwd_dt_b, torch::Tensor mamba_fwd_B_proj, torch::Tensor mamba_fwd_C_proj,
    torch::Tensor mamba_fwd_A_log, torch::Tensor mamba_fwd_D, torch::Tensor mamba_fwd_rope, torch::Tensor mamba_fwd_out_proj,
    torch::Tensor mamba_bwd_in_proj, torch::Tensor mamba_bwd_dt_W, torch::Tensor mamba_bwd_dt_b, torch::Tensor mamba_bwd_B_proj,
    torch::Tensor mamba_bwd_C_proj, torch::Tensor mamba_bwd_A_log, torch::Tensor mamba_bwd_D, torch::Tensor mamba_bwd_rope,
    torch::Tensor mamba_bwd_out_proj, torch::Tensor gru_Wz, torch::Tensor gru_Wr, torch::Tensor gru_Wh, torch::Tensor peer_query_Ws,
    torch::Tensor prod_keys_A, torch::Tensor prod_keys_B, torch::Tensor expert_W1, torch::Tensor expert_W2, torch::Tensor expert_b1_in,
    torch::Tensor expert_b2_in, torch::Tensor input_proj_W, torch::Tensor mamba_fwd_init_state, torch::Tensor mamba_bwd_init_state,
    torch::Tensor d_mamba_fwd_in_proj, torch::Tensor d_mamba_fwd_dt_W, torch::Tensor d_mamba_fwd_dt_b, torch::Tensor d_mamba_fwd_B_proj,
    torch::Tensor d_mamba_fwd_C_proj, torch::Tensor d_mamba_fwd_A_log, torch::Tensor d_mamba_fwd_D, torch::Tensor d_mamba_fwd_rope,
    torch::Tensor d_mamba_fwd_out_proj, torch::Tensor d_mamba_bwd_in_proj, torch::Tensor d_mamba_bwd_dt_W, torch::Tensor d_mamba_bwd_dt_b,
    torch::Tensor d_mamba_bwd_B_proj, torch::Tensor d_mamba_bwd_C_proj, torch::Tensor d_mamba_bwd_A_log, torch::Tensor d_mamba_bwd_D,
    torch::Tensor d_mamba_bwd_rope, torch::Tensor d_mamba_bwd_out_proj, torch::Tensor d_gru_Wz, torch::Tensor d_gru_bz, torch::Tensor d_gru_Wr,
    torch::Tensor d_gru_br, torch::Tensor d_gru_Wh, torch::Tensor d_gru_bh, torch::Tensor d_peer_query_Ws, torch::Tensor d_prod_keys_A,
    torch::Tensor d_prod_keys_B, torch::Tensor d_expert_W1, torch::Tensor d_expert_b1, torch::Tensor d_expert_W2, torch::Tensor d_expert_b2,
    torch::Tensor d_input_proj_W, torch::Tensor d_input_proj_b, int d_model, int d_state, int d_inner, int gru_hidden, int gru_input_dim,
    int num_heads, int topk, int pk_dim, int expert_hidden, int peer_input_dim, int num_experts, int checkpoint_interval) {
    const char* fn = "supergrok2_bilevel_backward";
    (void)checkpoint_interval; (void)fwd_saved_x_branch; (void)fwd_saved_z; (void)fwd_saved_dt; (void)bwd_saved_states;
    (void)bwd_saved_x_branch; (void)bwd_saved_z; (void)bwd_saved_dt; (void)mamba_fwd_init_state; (void)mamba_bwd_init_state;
    (void)input_proj_W; (void)expert_b1_in; (void)saved_scores_a; (void)saved_scores_b;
    const int64_t N = d_smart_grad.numel();
    if (N == 0) return;
    if (!d_smart_grad.is_cuda()) throw std::runtime_error("supergrok2_bilevel_backward requires CUDA tensors.");
    torch::NoGradGuard no_grad;
    const SgDims dims = default_dims(d_model, d_state, d_inner);
    Saved S = claim(fn, "supergrok2_bilevel_fwd_save", fwd_saved_states);
    TORCH_CHECK(S.grads.size() == 1 && S.total == N, fn, ": the forward call on these buffers had ", S.total, " elements, this call has ", N);
    TORCH_CHECK(S.x_sorted_ptr == x_sorted.data_ptr(), fn, ": x_sorted is not the tensor the forward call filled");
    const int64_t H = num_heads, A = (int64_t)topk * topk, eh = expert_hidden, E = num_experts, hd = d_model / 2, gh = gru_hidden;
    TORCH_CHECK(gru_input_dim == 2 + 2 * d_model && peer_input_dim == gh + 2 * d_model + 2, fn, ": gru_input_dim / peer_input_dim do not match d_model and gru_hidden");
    auto f32 = [](const torch::Tensor& t) { return t.to(torch::kFloat32).contiguous(); };
    const torch::Tensor g = f32(grad).reshape({N});
    const torch::Tensor s = f32(sharpness).reshape({N});
    const torch::Tensor pin = f32(peer_input).reshape({N, peer_input_dim});
    // ---- 1: d(total expert output) = rescale * d_smart_grad; every head contributes 1/H of it
    const torch::Tensor d_head = (f32(d_smart_grad).reshape({N}) * rescale / (double)H).unsqueeze(1);                  // [N,1]
    // ---- 2: experts and soft top-k routing, head by head
    const torch::Tensor eidx = expert_indices.reshape({N, H, A}).to(torch::kLong);
    const torch::Tensor rw = f32(routing_weights).reshape({N, H, A});
    const torch::Tensor zh = f32(saved_z_hidden).reshape({N, H, A, eh});
    const torch::Tensor top_a = saved_top_a_idx.reshape({N, H, topk}).to(torch::kLong), top_b = saved_top_b_idx.reshape({N, H, topk}).to(torch::kLong);
    const torch::Tensor soft_a = f32(saved_soft_a).reshape({N, H, topk}), soft_b = f32(saved_soft_b).reshape({N, H, topk});
    const torch::Tensor W2 = f32(expert_W2).reshape({E, eh}), b2 = f32(expert_b2_in).reshape({E});
    torch::Tensor d_pin = torch::zeros({N, peer_input_dim}, pin.options());
    torch::Tensor dW1 = torch::zeros({E, eh}, pin.options()), db1 = torch::zeros({E, eh}, pin.options()), dW2 = torch::zeros({E, eh}, pin.options());
    torch::Tensor db2 = torch::zeros({E}, pin.options());
    const torch::Tensor Wq = f32(peer_query_Ws).reshape({H, d_model, peer_input_dim});
    const torch::Tensor KA = f32(prod_keys_A).reshape({H, pk_dim, hd}), KB = f32(prod_keys_B).reshape({H, pk_dim, hd});
    for (int64_t h = 0; h < H; h++) {
        const torch::Tensor idx = eidx.select(1, h);                                   // [N,A]
        const torch::Tensor z = zh.select(1, h);                                       // [N,A,eh]  relu(W1 g + b1) of the picked experts
        const torch::Tensor w2 = W2.index_select(0, idx.reshape({-1})).reshape({N, A, eh});
        const torch::Tensor out_k = (w2 * z).sum(-1) + b2.index_select(0, idx.reshape({-1})).reshape({N, A});
        const torch::Tensor d_out = rw.select(1, h) * d_head;                          // [N,A]
        const torch::Tensor d_rw = out_k * d_head;                                     // [N,A]
        const torch::Tensor dz = d_out.unsqueeze(-1) * w2 * (z > 0).to(torch::kFloat32);    // through the ReLU
        const torch::Tensor flat = idx.reshape({-1});
        dW2.index_add_(0, flat, (d_out.unsqueeze(-1) * z).reshape({N * A, eh}));
        db2.index_add_(0, flat, d_out.reshape({-1}));
        dW1.index_add_(0, flat, (dz * g.reshape({N, 1, 1})).reshape({N * A, eh}));
        db1.index_add_(0, flat, dz.reshape({N * A, eh}));
        // routing weight of expert (i, j) is soft_a[i] * soft_b[j]
        const torch::Tensor d_rw2 = d_rw.reshape({N, topk, topk});
        const torch::Tensor sa = soft_a.select(1, h), sb = soft_b.select(1, h);
        const torch::Tensor d_sa = (d_rw2 * sb.unsqueeze(1)).sum(2), d_sb = (d_rw2 * sa.unsqueeze(2)).sum(1);
        // softmax of 10 x the k best scores
        const torch::Tensor d_va = 10.0 * sa * (d_sa - (sa * d_sa).sum(-1, true)), d_vb = 10.0 * sb * (d_sb - (sb * d_sb).sum(-1, true));
        torch::Tensor d_score_a = torch::zeros({N, pk_dim}, pin.options()), d_score_b = torch::zeros({N, pk_dim}, pin.options());
        d_score_a.scatter_add_(1, top_a.select(1, h), d_va);
        d_score_b.scatter_add_(1, top_b.select(1, h), d_vb);
        const torch::Tensor q = torch::mm(pin, Wq[h].t());                             // [N,d_model]
        d_prod_keys_A.view({H, pk_dim, hd})[h].addmm_(d_score_a.t(), q.narrow(1, 0, hd));
        d_prod_keys_B.view({H, pk_dim, hd})[h].addmm_(d_score_b.t(), q.narrow(1, hd, hd));
        const torch::Tensor d_q = torch::cat({torch::mm(d_score_a, KA[h]), torch::mm(d_score_b, KB[h])}, 1);      // [N,2 hd]
        d_peer_query_Ws.view({H, d_model, peer_input_dim})[h].narrow(0, 0, 2 * hd).addmm_(d_q.t(), pin);
        d_pin.addmm_(d_q, Wq[h].narrow(0, 0, 2 * hd));
    }
    d_expert_W1.view({E, eh}).add_(dW1);
    d_expert_b1.view({E, eh}).add_(db1);
    d_expert_W2.view({E, eh}).add_(dW2);
    d_expert_b2.view({E}).add_(db2);
    // ---- 3, 4: GRU.  h' = (1 - z) h + z h~, gates over [input, h], candidate over [input, r * h]
    const torch::Tensor d_hn = d_pin.narrow(1, 0, gh);
    const torch::Tensor inp = f32(gru_input).reshape({N, gru_input_dim}), h_old = f32(gru_h_old).reshape({N, gh});
    const torch::Tensor zg = f32(gru_z_gate).reshape({N, gh}), rg = f32(gru_r_gate).reshape({N, gh}), ht = f32(gru_h_tilde).reshape({N, gh});
    const torch::Tensor Wz = f32(gru_Wz).reshape({gh, gru_input_dim + gh}), Wr = f32(gru_Wr).reshape({gh, gru_input_dim + gh}), Wh = f32(gru_Wh).reshape({gh, gru_input_dim + gh});
    const torch::Tensor d_pre_h = d_hn * zg * (1.0 - ht * ht);
    const torch::Tensor d_pre_z = d_hn * (ht - h_old) * zg * (1.0 - zg);
    const torch::Tensor xh = torch::cat({inp, h_old}, 1), xrh = torch::cat({inp, rg * h_old}, 1);
    const torch::Tensor d_xrh = torch::mm(d_pre_h, Wh);
    const torch::Tensor d_pre_r = d_xrh.narrow(1, gru_input_dim, gh) * h_old * rg * (1.0 - rg);
    d_gru_Wh.view({gh, gru_input_dim + gh}).addmm_(d_pre_h.t(), xrh);
    d_gru_bh.view({gh}).add_(d_pre_h.sum(0));
    d_gru_Wz.view({gh, gru_input_dim + gh}).addmm_(d_pre_z.t(), xh);
    d_gru_bz.view({gh}).add_(d_pre_z.sum(0));
    d_gru_Wr.view({gh, gru_input_dim + gh}).addmm_(d_pre_r.t(), xh);
    d_gru_br.view({gh}).add_(d_pre_r.sum(0));
    const torch::Tensor d_inp = d_xrh.narrow(1, 0, gru_input_dim) + torch::mm(d_pre_z, Wz).narrow(1, 0, gru_input_dim) +
                                torch::mm(d_pre_r, Wr).narrow(1, 0, gru_input_dim);
    // ---- 5, 6: context gradients (GRU input [g, s, fwd, bwd]; query input [h', fwd, bwd, g, s]), into scan order
    const torch::Tensor d_ctx_f = d_inp.narrow(1, 2, d_model) + d_pin.narrow(1, gh, d_model);
    const torch::Tensor d_ctx_b = d_inp.narrow(1, 2 + d_model, d_model) + d_pin.narrow(1, gh + d_model, d_model);
    const torch::Tensor order = sort_indices.reshape({N}).to(torch::kLong);
    const torch::Tensor d_f_sorted = d_ctx_f.index_select(0, order), d_b_sorted = d_ctx_b.index_select(0, order).flip(0).contiguous();
    // ---- 7: out_proj of both directions
    const torch::Tensor fso = f32(fwd_scan_out).reshape({N, d_inner}), bso = f32(bwd_scan_out).reshape({N, d_inner});
    d_mamba_fwd_out_proj.view({d_model, d_inner}).addmm_(d_f_sorted.t(), fso);
    d_mamba_bwd_out_proj.view({d_model, d_inner}).addmm_(d_b_sorted.t(), bso);
    const torch::Tensor d_fso = torch::mm(d_f_sorted, f32(mamba_fwd_out_proj).reshape({d_model, d_inner})).contiguous();
    const torch::Tensor d_bso = torch::mm(d_b_sorted, f32(mamba_bwd_out_proj).reshape({d_model, d_inner})).contiguous();
    // ---- 8: the scan's adjoint in HIP, on what the forward call kept
    const torch::Tensor given[16] = {mamba_fwd_in_proj, mamba_fwd_dt_W, mamba_fwd_dt_b, mamba_fwd_B_proj, mamba_fwd_C_proj, mamba_fwd_A_log,
                                     mamba_fwd_D, mamba_fwd_rope, mamba_bwd_in_proj, mamba_bwd_dt_W, mamba_bwd_dt_b, mamba_bwd_B_proj,
                                     mamba_bwd_C_proj, mamba_bwd_A_log, mamba_bwd_D, mamba_bwd_rope};
    for (int dir = 0; dir < 2; dir++)
        for (int k = 0; k < 8; k++)
            TORCH_CHECK(given[dir * 8 + k].data_ptr() == S.w.t[2 + dir * 9 + k].data_ptr(), fn, ": the Mamba weights must be the tensors the forward call received");
    std::vector<torch::Tensor> rows;
    for (int dir = 0; dir < 2; dir++) {
        const torch::Tensor& in_proj = S.w.t[2 + dir * 9];
        const torch::Tensor X = in_proj.view({2 * d_inner, d_model}).narrow(0, 0, d_inner), Z = in_proj.view({2 * d_inner, d_model}).narrow(0, d_inner, d_inner);
        rows.push_back(torch::cat({X, Z, torch::mm(S.w.t[3 + dir * 9].view({d_inner, d_inner}), X), torch::mm(S.w.t[5 + dir * 9].view({d_state, d_inner}), X),
                                   torch::mm(S.w.t[6 + dir * 9].view({d_state, d_inner}), X)}, 0));
    }
    const torch::Tensor row_dx = torch::stack(rows, 0).contiguous();
    torch::Tensor dx = torch::empty({2, N, (int64_t)d_model}, pin.options()), block = torch::empty({SG2_SCAN_GRAD_FLOATS}, pin.options());
    const int rc = sg2_bilevel_backward_ex(&dims, &S.w.W, 1, S.tensors.data(), nullptr, d_fso.data_ptr<float>(), d_bso.data_ptr<float>(),
                                           row_dx.data_ptr<float>(), dx.data_ptr<float>(), block.data_ptr<float>(), S.workspace.data_ptr(),
                                           (size_t)S.workspace.numel(), stream_of(block));
    TORCH_CHECK(rc == 0, fn, ": ", sg_last_error());
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
        at += (int64_t)d_model * d_inner;       // out_proj: formed above from the scan outputs
    }
    // ---- 9: input projection, x = W [g, s] + b in element order
    const torch::Tensor d_x_sorted = dx[0] + dx[1];
    const torch::Tensor unsort = torch::empty_like(order).scatter_(0, order, torch::arange(N, order.options()));
    const torch::Tensor d_x = d_x_sorted.index_select(0, unsort);
    d_input_proj_W.view({d_model, 2}).addmm_(d_x.t(), torch::stack({g, s}, 1));
    d_input_proj_b.view({d_model}).add_(d_x.sum(0));
}
