// Torch extension `grokking_optimizers._ops`: the reference's pybind surface
// (csrc/ops.h:378-581, bindings csrc/ops.cpp:897-1068 of the reference) for the
// Grokfast, SuperGrok v1.5, Muon and SuperGrok v2 steps, kept name for name and
// argument for argument so the Python optimizer classes are drop-in.  Every
// function validates its tensors and forwards to the C ABI of libsg_hip.so
// (include/sg_abi.h) on PyTorch's current HIP stream; scratch memory comes from
// the caching allocator.  There is no CPU path: non-GPU tensors raise.
#include <torch/extension.h>
#include <c10/hip/HIPStream.h>

#include <cmath>
#include <stdexcept>
#include <string>
#include <vector>

#include "../../include/sg_abi.h"

namespace {

void* current_stream(const torch::Tensor& t) {
    return (void*)c10::hip::getCurrentHIPStream(t.device().index()).stream();
}

int dtype_code(const torch::Tensor& t, const char* what) {
    switch (t.scalar_type()) {
        case torch::kFloat32: return SG_F32;
        case torch::kFloat16: return SG_F16;
        case torch::kBFloat16: return SG_BF16;
        default: TORCH_CHECK(false, what, ": unsupported dtype ", t.scalar_type());
    }
    return -1;
}

void check_gpu(const torch::Tensor& t, const char* fn, const char* what) {
    if (!t.is_cuda()) throw std::runtime_error(std::string(fn) + " requires CUDA tensors (" + what + " is on the CPU).");
    TORCH_CHECK(t.is_contiguous(), fn, ": ", what, " must be contiguous");
}
void check_f32(const torch::Tensor& t, const char* fn, const char* what) {
    check_gpu(t, fn, what);
    TORCH_CHECK(t.scalar_type() == torch::kFloat32, fn, ": ", what, " must be float32");
}

torch::Tensor make_workspace(size_t bytes, const torch::Tensor& like) {
    return torch::empty({(int64_t)std::max<size_t>(bytes, 256)},
                        torch::TensorOptions().device(like.device()).dtype(torch::kUInt8));
}

void check_status(int rc, const char* fn) { TORCH_CHECK(rc == 0, fn, ": ", sg_last_error()); }

int g_sg15_gelu_mode = 0;   // 0 exact erf GELU, 1 sigmoid approximation

}  // namespace

// ───────────────────────── Grokfast ─────────────────────────
void grokfast_fused_step(std::vector<torch::Tensor>& grads, std::vector<torch::Tensor>& ema_bufs, float alpha, float lamb) {
    std::vector<SgGrokfastTensor> ts;
    std::vector<int64_t> numels;
    const torch::Tensor* first = nullptr;
    for (size_t i = 0; i < grads.size(); i++) {
        if (!grads[i].defined() || grads[i].numel() == 0) continue;
        check_gpu(grads[i], "grokfast_fused_step", "grad");
        check_f32(ema_bufs[i], "grokfast_fused_step", "ema_buf");
        TORCH_CHECK(ema_bufs[i].numel() == grads[i].numel(), "grokfast_fused_step: ema/grad size mismatch");
        ts.push_back({grads[i].data_ptr(), ema_bufs[i].data_ptr<float>(), grads[i].numel(), dtype_code(grads[i], "grad")});
        numels.push_back(grads[i].numel());
        if (!first) first = &grads[i];
    }
    if (ts.empty()) return;
    const size_t bytes = sg_elemwise_workspace_bytes((int)ts.size(), numels.data());
    auto ws = make_workspace(bytes, *first);
    check_status(sg_grokfast_ema((int)ts.size(), ts.data(), alpha, lamb, ws.data_ptr(), (size_t)ws.numel(), current_stream(*first)),
                 "grokfast_fused_step");
}

// Grokfast.step in one pass (EMA + amplify + AdamW); not part of the reference surface.
void grokfast_adamw_fused_step(std::vector<torch::Tensor>& params, std::vector<torch::Tensor>& grads,
                               std::vector<torch::Tensor>& ema_bufs, std::vector<torch::Tensor>& exp_avgs,
                               std::vector<torch::Tensor>& exp_avg_sqs, std::vector<int64_t> steps, float alpha, float lamb,
                               double lr, double beta1, double beta2, double eps, double weight_decay) {
    std::vector<SgGrokfastAdamTensor> ts;
    std::vector<int64_t> numels;
    const torch::Tensor* first = nullptr;
    for (size_t i = 0; i < grads.size(); i++) {
        if (!grads[i].defined() || grads[i].numel() == 0) continue;
        const char* fn = "grokfast_adamw_fused_step";
        check_gpu(params[i], fn, "param");
        check_gpu(grads[i], fn, "grad");
        check_f32(ema_bufs[i], fn, "ema_buf");
        check_f32(exp_avgs[i], fn, "exp_avg");
        check_f32(exp_avg_sqs[i], fn, "exp_avg_sq");
        TORCH_CHECK(params[i].scalar_type() == grads[i].scalar_type(), fn, ": param/grad dtype mismatch");
        ts.push_back({params[i].data_ptr(), grads[i].data_ptr(), ema_bufs[i].data_ptr<float>(), exp_avgs[i].data_ptr<float>(),
                      exp_avg_sqs[i].data_ptr<float>(), grads[i].numel(), dtype_code(grads[i], "grad"), (int32_t)steps[i]});
        numels.push_back(grads[i].numel());
        if (!first) first = &grads[i];
    }
    if (ts.empty()) return;
    auto ws = make_workspace(sg_elemwise_workspace_bytes((int)ts.size(), numels.data()), *first);
    check_status(sg_grokfast_adamw_step((int)ts.size(), ts.data(), alpha, lamb, lr, beta1, beta2, eps, weight_decay, ws.data_ptr(),
                                        (size_t)ws.numel(), current_stream(*first)),
                 "grokfast_adamw_fused_step");
}

// ───────────────────────── SuperGrok v1.5 ─────────────────────────
void supergrok15_fused_step(std::vector<torch::Tensor>& params, std::vector<torch::Tensor>& grads,
                            std::vector<torch::Tensor>& exp_avgs, std::vector<torch::Tensor>& exp_avg_sqs,
                            std::vector<torch::Tensor>& mus, std::vector<torch::Tensor>& sharpness_cache,
                            std::vector<int64_t>& steps, std::vector<float>& layer_alphas, std::vector<float>& layer_beta1s,
                            torch::Tensor W1, torch::Tensor b1, torch::Tensor W2, torch::Tensor b2, float rescale, int hidden_dim,
                            float beta2, float lr, float wd_eff, float eps, float lamb, float ramp, float gate_signal,
                            float grad_clip_norm) {
    const char* fn = "supergrok15_fused_step";
    float lamb_eff = 0.0f;
    if (ramp > 0.0f) lamb_eff = ramp * gate_signal * lamb;
    std::vector<Sg15Tensor> ts;
    std::vector<int64_t> numels;
    const torch::Tensor* first = nullptr;
    for (size_t i = 0; i < params.size(); i++) {
        if (!grads[i].defined() || grads[i].numel() == 0) continue;
        steps[i] += 1;   // `steps` is pybind's copy of the Python list, exactly as in the reference
        const float step = static_cast<float>(steps[i]);
        const float beta1 = layer_beta1s[i];
        const float bc1 = 1.0f - std::pow(beta1, step);
        const float bc2 = 1.0f - std::pow(beta2, step);
        check_gpu(params[i], fn, "param");
        check_gpu(grads[i], fn, "grad");
        check_gpu(sharpness_cache[i], fn, "sharpness");
        check_f32(exp_avgs[i], fn, "exp_avg");
        check_f32(exp_avg_sqs[i], fn, "exp_avg_sq");
        check_f32(mus[i], fn, "mu");
        TORCH_CHECK(params[i].scalar_type() == grads[i].scalar_type() && sharpness_cache[i].scalar_type() == grads[i].scalar_type(),
                    fn, ": param, grad and sharpness must share one dtype");
        ts.push_back({params[i].data_ptr(), grads[i].data_ptr(), sharpness_cache[i].data_ptr(), exp_avgs[i].data_ptr<float>(),
                      exp_avg_sqs[i].data_ptr<float>(), mus[i].data_ptr<float>(), grads[i].numel(), dtype_code(grads[i], "grad"),
                      layer_alphas[i], beta1, bc1, bc2});
        numels.push_back(grads[i].numel());
        if (!first) first = &grads[i];
    }
    if (ts.empty()) return;
    auto W1f = W1.to(torch::kFloat32).contiguous(), b1f = b1.to(torch::kFloat32).contiguous();
    auto W2f = W2.to(torch::kFloat32).contiguous(), b2f = b2.to(torch::kFloat32).contiguous();
    check_f32(W1f, fn, "W1");
    check_f32(b1f, fn, "b1");
    check_f32(W2f, fn, "W2");
    check_f32(b2f, fn, "b2");
    TORCH_CHECK(W1f.numel() == 2 * hidden_dim && b1f.numel() == hidden_dim && W2f.numel() == hidden_dim && b2f.numel() == 1, fn,
                ": meta-net weight shapes do not match hidden_dim");
    Sg15Net net = {W1f.data_ptr<float>(), b1f.data_ptr<float>(), W2f.data_ptr<float>(), b2f.data_ptr<float>(), hidden_dim, rescale,
                   g_sg15_gelu_mode};
    auto ws = make_workspace(sg_elemwise_workspace_bytes((int)ts.size(), numels.data()), *first);
    check_status(sg15_fused_step((int)ts.size(), ts.data(), &net, lamb_eff, beta2, lr, wd_eff, eps, grad_clip_norm, ws.data_ptr(),
                                 (size_t)ws.numel(), current_stream(*first)),
                 fn);
}

std::vector<torch::Tensor> supergrok15_sam_perturb_all(std::vector<torch::Tensor>& params, std::vector<torch::Tensor>& grads, float rho) {
    const char* fn = "supergrok15_sam_perturb_all";
    std::vector<torch::Tensor> backups;
    backups.reserve(params.size());
    std::vector<Sg15SamTensor> ts;
    std::vector<int64_t> numels;
    const torch::Tensor* first = nullptr;
    for (size_t i = 0; i < params.size(); i++) {
        backups.push_back(params[i].clone());
        if (!grads[i].defined() || grads[i].numel() == 0) continue;
        check_gpu(params[i], fn, "param");
        check_gpu(grads[i], fn, "grad");
        TORCH_CHECK(params[i].scalar_type() == grads[i].scalar_type(), fn, ": param/grad dtype mismatch");
        ts.push_back({params[i].data_ptr(), grads[i].data_ptr(), grads[i].numel(), dtype_code(grads[i], "grad")});
        numels.push_back(grads[i].numel());
        if (!first) first = &grads[i];
    }
    if (ts.empty()) return backups;
    auto ws = make_workspace(sg_elemwise_workspace_bytes((int)ts.size(), numels.data()), *first);
    check_status(sg15_sam_perturb((int)ts.size(), ts.data(), rho, ws.data_ptr(), (size_t)ws.numel(), current_stream(*first)), fn);
    return backups;
}

void supergrok15_sharpness_restore_all(std::vector<torch::Tensor>& params, std::vector<torch::Tensor>& sharpness_cache,
                                       std::vector<torch::Tensor>& backups, std::vector<torch::Tensor>& sam_grads,
                                       std::vector<torch::Tensor>& normal_grads) {
    const char* fn = "supergrok15_sharpness_restore_all";
    std::vector<Sg15RestoreTensor> ts;
    std::vector<int64_t> numels;
    const torch::Tensor* first = nullptr;
    for (size_t i = 0; i < params.size(); i++) {
        if (!sam_grads[i].defined() || !normal_grads[i].defined() || sam_grads[i].numel() == 0) {
            params[i].copy_(backups[i]);
            continue;
        }
        check_gpu(params[i], fn, "param");
        check_gpu(sharpness_cache[i], fn, "sharpness");
        check_gpu(backups[i], fn, "backup");
        check_gpu(sam_grads[i], fn, "sam_grad");
        check_gpu(normal_grads[i], fn, "normal_grad");
        const auto dt = params[i].scalar_type();
        TORCH_CHECK(sharpness_cache[i].scalar_type() == dt && backups[i].scalar_type() == dt && sam_grads[i].scalar_type() == dt &&
                        normal_grads[i].scalar_type() == dt,
                    fn, ": all tensors of one parameter must share one dtype");
        ts.push_back({params[i].data_ptr(), sharpness_cache[i].data_ptr(), backups[i].data_ptr(), sam_grads[i].data_ptr(),
                      normal_grads[i].data_ptr(), params[i].numel(), dtype_code(params[i], "param")});
        numels.push_back(params[i].numel());
        if (!first) first = &params[i];
    }
    if (ts.empty()) return;
    auto ws = make_workspace(sg_elemwise_workspace_bytes((int)ts.size(), numels.data()), *first);
    check_status(sg15_sharpness_restore((int)ts.size(), ts.data(), ws.data_ptr(), (size_t)ws.numel(), current_stream(*first)), fn);
}

void supergrok15_set_gelu_mode(const std::string& mode) {
    if (mode == "erf") g_sg15_gelu_mode = 0;
    else if (mode == "sigmoid") g_sg15_gelu_mode = 1;
    else TORCH_CHECK(false, "supergrok15_set_gelu_mode: expected 'erf' or 'sigmoid', got '", mode, "'");
}

// ───────────────────────── Muon ─────────────────────────
void muon_fused_step(std::vector<torch::Tensor>& params, std::vector<torch::Tensor>& grads, std::vector<torch::Tensor>& bufs,
                     float momentum, float lr, float wd, int ns_steps) {
    const char* fn = "muon_fused_step";
    std::vector<SgMuonMatrix> ms;
    const torch::Tensor* first = nullptr;
    for (size_t i = 0; i < params.size(); i++) {
        if (!grads[i].defined() || grads[i].numel() == 0) continue;
        check_gpu(params[i], fn, "param");
        check_gpu(grads[i], fn, "grad");
        check_f32(bufs[i], fn, "momentum buffer");
        TORCH_CHECK(params[i].dim() == 2, fn, ": parameters must be 2-D");
        TORCH_CHECK(params[i].scalar_type() == grads[i].scalar_type(), fn, ": param/grad dtype mismatch");
        TORCH_CHECK(bufs[i].numel() == params[i].numel(), fn, ": buffer size mismatch");
        ms.push_back({params[i].data_ptr(), grads[i].data_ptr(), bufs[i].data_ptr<float>(), params[i].size(0), params[i].size(1),
                      dtype_code(params[i], "param")});
        if (!first) first = &params[i];
    }
    if (ms.empty()) return;
    auto ws = make_workspace(sg_muon_workspace_bytes((int)ms.size(), ms.data()), *first);
    check_status(sg_muon_step((int)ms.size(), ms.data(), momentum, lr, wd, ns_steps, ws.data_ptr(), (size_t)ws.numel(),
                              current_stream(*first)),
                 fn);
}

// ───────────────────────── SuperGrok v2 ─────────────────────────
void supergrok2_mamba_peer_batched_step(
    std::vector<torch::Tensor> params, std::vector<torch::Tensor> grads, std::vector<torch::Tensor> sharpness_list,
    std::vector<torch::Tensor> exp_avgs, std::vector<torch::Tensor> exp_avg_sqs, std::vector<torch::Tensor> mus,
    std::vector<torch::Tensor> gru_states, std::vector<torch::Tensor> mamba_fwd_states,
    std::vector<torch::Tensor> mamba_bwd_states, torch::Tensor input_proj_W, torch::Tensor input_proj_b,
    torch::Tensor mamba_fwd_in_proj, torch::Tensor mamba_fwd_dt_W, torch::Tensor mamba_fwd_dt_b, torch::Tensor mamba_fwd_B_proj,
    torch::Tensor mamba_fwd_C_proj, torch::Tensor mamba_fwd_A_log, torch::Tensor mamba_fwd_D, torch::Tensor mamba_fwd_rope,
    torch::Tensor mamba_fwd_out_proj, torch::Tensor mamba_bwd_in_proj, torch::Tensor mamba_bwd_dt_W, torch::Tensor mamba_bwd_dt_b,
    torch::Tensor mamba_bwd_B_proj, torch::Tensor mamba_bwd_C_proj, torch::Tensor mamba_bwd_A_log, torch::Tensor mamba_bwd_D,
    torch::Tensor mamba_bwd_rope, torch::Tensor mamba_bwd_out_proj, torch::Tensor gru_Wz, torch::Tensor gru_bz,
    torch::Tensor gru_Wr, torch::Tensor gru_br, torch::Tensor gru_Wh, torch::Tensor gru_bh, torch::Tensor peer_query_Ws,
    torch::Tensor prod_keys_A, torch::Tensor prod_keys_B, torch::Tensor expert_W1, torch::Tensor expert_b1,
    torch::Tensor expert_W2, torch::Tensor expert_b2, std::vector<float> alpha_mus, std::vector<float> lamb_effs,
    std::vector<float> beta1s, std::vector<float> bc1s, std::vector<float> bc2s, float rescale, float beta2, float lr,
    float wd_eff, float eps, int d_model, int d_state, int d_inner, int gru_hidden, int num_heads, int pk_dim,
    int expert_hidden, int num_experts, torch::Tensor expert_counts) {
    const char* fn = "supergrok2_mamba_peer_batched_step";
    if (params.empty()) return;
    if (!params[0].is_cuda()) throw std::runtime_error("supergrok2_mamba_peer_batched_step requires CUDA tensors.");
    const size_t P = params.size();
    TORCH_CHECK(grads.size() == P && sharpness_list.size() == P && exp_avgs.size() == P && exp_avg_sqs.size() == P &&
                    mus.size() == P && gru_states.size() == P && mamba_fwd_states.size() == P && mamba_bwd_states.size() == P &&
                    alpha_mus.size() == P && lamb_effs.size() == P && beta1s.size() == P && bc1s.size() == P && bc2s.size() == P,
                fn, ": per-parameter lists must all have ", P, " entries");
    SgDims dims = {d_model, d_state, d_inner, gru_hidden, num_heads, pk_dim, expert_hidden, num_experts};
    const int gru_row = 2 + 2 * d_model + gru_hidden, peer_in = gru_hidden + 2 * d_model + 2;
    torch::Tensor w[SG2_NUM_WEIGHTS] = {
        input_proj_W, input_proj_b, mamba_fwd_in_proj, mamba_fwd_dt_W, mamba_fwd_dt_b, mamba_fwd_B_proj, mamba_fwd_C_proj,
        mamba_fwd_A_log, mamba_fwd_D, mamba_fwd_rope, mamba_fwd_out_proj, mamba_bwd_in_proj, mamba_bwd_dt_W, mamba_bwd_dt_b,
        mamba_bwd_B_proj, mamba_bwd_C_proj, mamba_bwd_A_log, mamba_bwd_D, mamba_bwd_rope, mamba_bwd_out_proj, gru_Wz, gru_bz,
        gru_Wr, gru_br, gru_Wh, gru_bh, peer_query_Ws, prod_keys_A, prod_keys_B, expert_W1, expert_b1, expert_W2, expert_b2};
    const int64_t mamba_numel[9] = {2LL * d_inner * d_model, (int64_t)d_inner * d_inner, d_inner, (int64_t)d_state * d_inner,
                                    (int64_t)d_state * d_inner, (int64_t)d_inner * d_state, d_inner,
                                    (int64_t)d_inner * (d_state / 2), (int64_t)d_model * d_inner};
    const int64_t gmat = (int64_t)gru_hidden * gru_row;
    int64_t want[SG2_NUM_WEIGHTS] = {2LL * d_model, d_model};
    for (int k = 0; k < 9; k++) want[2 + k] = want[11 + k] = mamba_numel[k];
    const int64_t tail[13] = {gmat, gru_hidden, gmat, gru_hidden, gmat, gru_hidden, (int64_t)num_heads * d_model * peer_in,
                              (int64_t)num_heads * pk_dim * (d_model / 2), (int64_t)num_heads * pk_dim * (d_model / 2),
                              (int64_t)num_experts * expert_hidden, (int64_t)num_experts * expert_hidden,
                              (int64_t)num_experts * expert_hidden, num_experts};
    for (int k = 0; k < 13; k++) want[20 + k] = tail[k];
    Sg2Weights W;
    for (int k = 0; k < SG2_NUM_WEIGHTS; k++) {
        check_f32(w[k], fn, "meta-net weight");
        TORCH_CHECK(w[k].numel() == want[k], fn, ": meta-net weight ", k, " has ", w[k].numel(), " elements, expected ", want[k]);
        W.w[k] = w[k].data_ptr<float>();
    }
    check_gpu(expert_counts, fn, "expert_counts");
    TORCH_CHECK(expert_counts.scalar_type() == torch::kInt32 && expert_counts.numel() == num_experts, fn,
                ": expert_counts must be int32[num_experts]");

    std::vector<Sg2Tensor> ts(P);
    std::vector<int64_t> numels(P);
    for (size_t i = 0; i < P; i++) {
        Sg2Tensor& t = ts[i];
        const int64_t n = grads[i].defined() ? grads[i].numel() : 0;
        numels[i] = n;
        t = Sg2Tensor{};
        t.numel = n;
        if (n == 0) continue;
        check_gpu(params[i], fn, "param");
        check_gpu(grads[i], fn, "grad");
        check_gpu(sharpness_list[i], fn, "sharpness");
        check_f32(exp_avgs[i], fn, "exp_avg");
        check_f32(exp_avg_sqs[i], fn, "exp_avg_sq");
        check_f32(mus[i], fn, "mu");
        check_f32(gru_states[i], fn, "gru_state");
        check_f32(mamba_fwd_states[i], fn, "mamba_fwd_state");
        check_f32(mamba_bwd_states[i], fn, "mamba_bwd_state");
        const auto dt = params[i].scalar_type();
        TORCH_CHECK(grads[i].scalar_type() == dt && sharpness_list[i].scalar_type() == dt, fn,
                    ": param, grad and sharpness of a parameter must share one dtype");
        TORCH_CHECK(params[i].numel() == n && sharpness_list[i].numel() == n && exp_avgs[i].numel() == n &&
                        exp_avg_sqs[i].numel() == n && mus[i].numel() == n && gru_states[i].numel() == n * gru_hidden,
                    fn, ": state sizes of parameter ", i, " do not match its gradient");
        TORCH_CHECK(mamba_fwd_states[i].numel() == (int64_t)d_inner * d_state && mamba_bwd_states[i].numel() == (int64_t)d_inner * d_state,
                    fn, ": Mamba state of parameter ", i, " must be [d_inner, d_state]");
        t.param = params[i].data_ptr();
        t.grad = grads[i].data_ptr();
        t.sharpness = sharpness_list[i].data_ptr();
        t.exp_avg = exp_avgs[i].data_ptr<float>();
        t.exp_avg_sq = exp_avg_sqs[i].data_ptr<float>();
        t.mu = mus[i].data_ptr<float>();
        t.gru_state = gru_states[i].data_ptr<float>();
        t.mamba_fwd_state = mamba_fwd_states[i].data_ptr<float>();
        t.mamba_bwd_state = mamba_bwd_states[i].data_ptr<float>();
        t.dtype = dtype_code(params[i], "param");
        t.alpha_mu = alpha_mus[i];
        t.lamb_eff = lamb_effs[i];
        t.beta1 = beta1s[i];
        t.bc1 = bc1s[i];
        t.bc2 = bc2s[i];
    }
    int64_t total = 0;
    for (size_t i = 0; i < P; i++) total += numels[i];
    const size_t bytes = sg2_workspace_bytes(&dims, (int)P, numels.data());
    // 0 bytes with elements to process means the library refused the call (its message is fresh); with no elements
    // at all there is no message to report: the call below validates the dimensions and returns
    TORCH_CHECK(bytes > 0 || total == 0, fn, ": ", sg_last_error());
    auto ws = make_workspace(bytes, params[0]);
    Sg2Scalars sc = {rescale, beta2, lr, wd_eff, eps};
    check_status(sg2_batched_step(&dims, &W, (int)P, ts.data(), &sc, expert_counts.data_ptr<int32_t>(), ws.data_ptr(),
                                  (size_t)ws.numel(), nullptr, current_stream(params[0])),
                 fn);
}

void supergrok2_mamba_peer_step(
    torch::Tensor param, torch::Tensor grad, torch::Tensor sharpness, torch::Tensor exp_avg, torch::Tensor exp_avg_sq,
    torch::Tensor mu, torch::Tensor gru_state, torch::Tensor mamba_fwd_state, torch::Tensor mamba_bwd_state,
    torch::Tensor input_proj_W, torch::Tensor input_proj_b, torch::Tensor mamba_fwd_in_proj, torch::Tensor mamba_fwd_dt_W,
    torch::Tensor mamba_fwd_dt_b, torch::Tensor mamba_fwd_B_proj, torch::Tensor mamba_fwd_C_proj, torch::Tensor mamba_fwd_A_log,
    torch::Tensor mamba_fwd_D, torch::Tensor mamba_fwd_rope, torch::Tensor mamba_fwd_out_proj, torch::Tensor mamba_bwd_in_proj,
    torch::Tensor mamba_bwd_dt_W, torch::Tensor mamba_bwd_dt_b, torch::Tensor mamba_bwd_B_proj, torch::Tensor mamba_bwd_C_proj,
    torch::Tensor mamba_bwd_A_log, torch::Tensor mamba_bwd_D, torch::Tensor mamba_bwd_rope, torch::Tensor mamba_bwd_out_proj,
    torch::Tensor gru_Wz, torch::Tensor gru_bz, torch::Tensor gru_Wr, torch::Tensor gru_br, torch::Tensor gru_Wh,
    torch::Tensor gru_bh, torch::Tensor peer_query_Ws, torch::Tensor prod_keys_A, torch::Tensor prod_keys_B,
    torch::Tensor expert_W1, torch::Tensor expert_b1, torch::Tensor expert_W2, torch::Tensor expert_b2, float rescale,
    float alpha_mu, float lamb_eff, float beta1, float beta2, float lr, float wd_eff, float eps, float bc1, float bc2, int d_model,
    int d_state, int d_inner, int gru_hidden, int num_heads, int pk_dim, int expert_hidden, int num_experts,
    torch::Tensor expert_counts) {
    if (grad.numel() == 0) return;
    if (!param.is_cuda())
        throw std::runtime_error("supergrok2_mamba_peer_step requires CUDA tensors. Use the Python meta-net fallback for CPU.");
    // an empty Mamba state means "start from zero and do not carry", as in the reference's single-tensor launcher
    auto opts = torch::TensorOptions().device(param.device()).dtype(torch::kFloat32);
    auto fwd = mamba_fwd_state.numel() > 0 ? mamba_fwd_state : torch::zeros({d_inner, d_state}, opts);
    auto bwd = mamba_bwd_state.numel() > 0 ? mamba_bwd_state : torch::zeros({d_inner, d_state}, opts);
    supergrok2_mamba_peer_batched_step(
        {param}, {grad}, {sharpness}, {exp_avg}, {exp_avg_sq}, {mu}, {gru_state}, {fwd}, {bwd}, input_proj_W, input_proj_b,
        mamba_fwd_in_proj, mamba_fwd_dt_W, mamba_fwd_dt_b, mamba_fwd_B_proj, mamba_fwd_C_proj, mamba_fwd_A_log, mamba_fwd_D,
        mamba_fwd_rope, mamba_fwd_out_proj, mamba_bwd_in_proj, mamba_bwd_dt_W, mamba_bwd_dt_b, mamba_bwd_B_proj, mamba_bwd_C_proj,
        mamba_bwd_A_log, mamba_bwd_D, mamba_bwd_rope, mamba_bwd_out_proj, gru_Wz, gru_bz, gru_Wr, gru_br, gru_Wh, gru_bh,
        peer_query_Ws, prod_keys_A, prod_keys_B, expert_W1, expert_b1, expert_W2, expert_b2, {alpha_mu}, {lamb_eff}, {beta1},
        {bc1}, {bc2}, rescale, beta2, lr, wd_eff, eps, d_model, d_state, d_inner, gru_hidden, num_heads, pk_dim, expert_hidden,
        num_experts, expert_counts);
}


// ---- the other fused steps (csrc/ops.h:408-508 of the reference: same names, same argument order) ----------

namespace {
struct FamilyArgs {
    std::vector<SgFamilyTensor> ts;
    std::vector<int64_t> numels;
    const torch::Tensor* first = nullptr;
    torch::Tensor ws;
    void make_ws() { ws = make_workspace(sg_family_workspace_bytes((int)ts.size(), numels.data()), *first); }
};

// fills one SgFamilyTensor per tensor with a gradient; aux/aux2 may be NULL lists
void gather_family(const char* fn, FamilyArgs* A, std::vector<torch::Tensor>& params, std::vector<torch::Tensor>& grads,
                   std::vector<torch::Tensor>* eas, std::vector<torch::Tensor>* easqs, std::vector<torch::Tensor>* aux,
                   std::vector<torch::Tensor>* aux2, bool aux2_f32, const std::vector<float>* bc1, const std::vector<float>* bc2,
                   const std::vector<float>* alphas, const std::vector<float>* beta1s) {
    for (size_t i = 0; i < params.size(); i++) {
        if (!grads[i].defined() || grads[i].numel() == 0) continue;
        check_gpu(params[i], fn, "param");
        check_gpu(grads[i], fn, "grad");
        TORCH_CHECK(params[i].scalar_type() == grads[i].scalar_type(), fn, ": param/grad dtype mismatch");
        TORCH_CHECK(params[i].numel() == grads[i].numel(), fn, ": param/grad size mismatch");
        SgFamilyTensor t = {};
        t.param = params[i].data_ptr();
        t.grad = grads[i].data_ptr();
        if (eas) { check_f32((*eas)[i], fn, "exp_avg"); t.exp_avg = (*eas)[i].data_ptr<float>(); }
        if (easqs) { check_f32((*easqs)[i], fn, "exp_avg_sq"); t.exp_avg_sq = (*easqs)[i].data_ptr<float>(); }
        if (aux) { check_f32((*aux)[i], fn, "state"); t.aux = (*aux)[i].data_ptr<float>(); }
        if (aux2) {
            if (aux2_f32) check_f32((*aux2)[i], fn, "param_init");
            else {
                check_gpu((*aux2)[i], fn, "sharpness");
                TORCH_CHECK((*aux2)[i].scalar_type() == grads[i].scalar_type(), fn, ": sharpness must have the gradient's dtype");
            }
            TORCH_CHECK((*aux2)[i].numel() == grads[i].numel(), fn, ": size mismatch");
            t.aux2 = (*aux2)[i].data_ptr();
        }
        t.numel = grads[i].numel();
        t.dtype = dtype_code(grads[i], "grad");
        t.bc1 = bc1 ? (*bc1)[i] : 1.0f;
        t.bc2 = bc2 ? (*bc2)[i] : 1.0f;
        t.alpha = alphas ? (*alphas)[i] : 0.0f;
        t.beta1 = beta1s ? (*beta1s)[i] : 0.0f;
        A->ts.push_back(t);
        A->numels.push_back(t.numel);
        if (!A->first) A->first = &grads[i];
    }
}

void bias_corrections(const std::vector<int64_t>& steps, float beta1, float beta2, std::vector<float>* bc1, std::vector<float>* bc2) {
    for (int64_t st : steps) {      // float pow, as the reference computes them (csrc/ops.cpp:333-334)
        bc1->push_back(1.0f - std::pow(beta1, static_cast<float>(st)));
        bc2->push_back(1.0f - std::pow(beta2, static_cast<float>(st)));
    }
}
}  // namespace

void grokadamw_fused_step(std::vector<torch::Tensor>& params, std::vector<torch::Tensor>& grads, std::vector<torch::Tensor>& exp_avgs,
                          std::vector<torch::Tensor>& exp_avg_sqs, std::vector<torch::Tensor>& emas, std::vector<int64_t>& steps,
                          float alpha, float lamb, float beta1, float beta2, float lr, float wd, float eps, float grad_clip_norm) {
    const char* fn = "grokadamw_fused_step";
    std::vector<float> bc1, bc2;
    bias_corrections(steps, beta1, beta2, &bc1, &bc2);
    FamilyArgs A;
    gather_family(fn, &A, params, grads, &exp_avgs, &exp_avg_sqs, &emas, nullptr, false, &bc1, &bc2, nullptr, nullptr);
    if (A.ts.empty()) return;
    A.make_ws();
    check_status(sg_grokadamw_step((int)A.ts.size(), A.ts.data(), alpha, lamb, beta1, beta2, lr, wd, eps, grad_clip_norm, A.ws.data_ptr(),
                                   (size_t)A.ws.numel(), current_stream(*A.first)), fn);
}

// AdamW over a list of tensors as one launch: what adamw_step of the reference's
// grokking_optimizers/_adamw_helper.py:12-22 does with six ATen calls per tensor (bias corrections in double).
void adamw_fused_step(std::vector<torch::Tensor>& params, std::vector<torch::Tensor>& grads, std::vector<torch::Tensor>& exp_avgs,
                      std::vector<torch::Tensor>& exp_avg_sqs, std::vector<int64_t>& steps, double lr, double beta1, double beta2,
                      double eps, double wd) {
    const char* fn = "adamw_fused_step";
    std::vector<float> bc1, bc2;
    for (int64_t st : steps) {
        bc1.push_back((float)(1.0 - std::pow(beta1, (double)st)));
        bc2.push_back((float)(1.0 - std::pow(beta2, (double)st)));
    }
    FamilyArgs A;
    gather_family(fn, &A, params, grads, &exp_avgs, &exp_avg_sqs, nullptr, nullptr, false, &bc1, &bc2, nullptr, nullptr);
    if (A.ts.empty()) return;
    A.make_ws();
    check_status(sg_grokadamw_step((int)A.ts.size(), A.ts.data(), 0.0f, 0.0f, (float)beta1, (float)beta2, (float)lr, (float)wd, (float)eps,
                                   0.0f, A.ws.data_ptr(), (size_t)A.ws.numel(), current_stream(*A.first)), fn);
}

void neuralgrok_fused_step(std::vector<torch::Tensor>& params, std::vector<torch::Tensor>& grads, std::vector<torch::Tensor>& exp_avgs,
                           std::vector<torch::Tensor>& exp_avg_sqs, std::vector<int64_t>& steps, torch::Tensor W1, torch::Tensor b1,
                           torch::Tensor W2, torch::Tensor b2, float alpha_amp, float beta_amp, int hidden_dim, float beta1, float beta2,
                           float lr, float wd, float eps, float grad_clip_norm) {
    const char* fn = "neuralgrok_fused_step";
    std::vector<float> bc1, bc2;
    bias_corrections(steps, beta1, beta2, &bc1, &bc2);
    FamilyArgs A;
    gather_family(fn, &A, params, grads, &exp_avgs, &exp_avg_sqs, nullptr, nullptr, false, &bc1, &bc2, nullptr, nullptr);
    if (A.ts.empty()) return;
    auto W1f = W1.to(torch::kFloat32).contiguous(), b1f = b1.to(torch::kFloat32).contiguous();
    auto W2f = W2.to(torch::kFloat32).contiguous(), b2f = b2.to(torch::kFloat32).contiguous();
    check_f32(W1f, fn, "W1"); check_f32(b1f, fn, "b1"); check_f32(W2f, fn, "W2"); check_f32(b2f, fn, "b2");
    TORCH_CHECK(W1f.numel() == hidden_dim && b1f.numel() == hidden_dim && W2f.numel() == hidden_dim && b2f.numel() == 1, fn,
                ": amplifier weight shapes do not match hidden_dim");
    SgAmplifier amp = {W1f.data_ptr<float>(), b1f.data_ptr<float>(), W2f.data_ptr<float>(), b2f.data_ptr<float>(), hidden_dim};
    A.make_ws();
    check_status(sg_neuralgrok_step((int)A.ts.size(), A.ts.data(), &amp, alpha_amp, beta_amp, beta1, beta2, lr, wd, eps, grad_clip_norm,
                                    A.ws.data_ptr(), (size_t)A.ws.numel(), current_stream(*A.first)), fn);
}

float prodigy_fused_step(std::vector<torch::Tensor>& params, std::vector<torch::Tensor>& grads, std::vector<torch::Tensor>& exp_avgs,
                         std::vector<torch::Tensor>& exp_avg_sqs, std::vector<torch::Tensor>& s_bufs,
                         std::vector<torch::Tensor>& param_inits, std::vector<int64_t>& steps, float d_lr, float beta1, float beta2,
                         float lr, float wd, float eps) {
    const char* fn = "prodigy_fused_step";
    std::vector<float> bc1, bc2;
    bias_corrections(steps, beta1, beta2, &bc1, &bc2);
    FamilyArgs A;
    gather_family(fn, &A, params, grads, &exp_avgs, &exp_avg_sqs, &s_bufs, &param_inits, true, &bc1, &bc2, nullptr, nullptr);
    if (A.ts.empty()) return d_lr;
    A.make_ws();
    float out = d_lr;
    check_status(sg_prodigy_step((int)A.ts.size(), A.ts.data(), d_lr, beta1, beta2, lr, wd, eps, &out, A.ws.data_ptr(), (size_t)A.ws.numel(),
                                 current_stream(*A.first)), fn);
    return out;
}

void lion_fused_step(std::vector<torch::Tensor>& params, std::vector<torch::Tensor>& grads, std::vector<torch::Tensor>& exp_avgs, float lr,
                     float beta1, float beta2, float wd) {
    const char* fn = "lion_fused_step";
    FamilyArgs A;
    gather_family(fn, &A, params, grads, &exp_avgs, nullptr, nullptr, nullptr, false, nullptr, nullptr, nullptr, nullptr);
    if (A.ts.empty()) return;
    A.make_ws();
    check_status(sg_lion_step((int)A.ts.size(), A.ts.data(), lr, beta1, beta2, wd, A.ws.data_ptr(), (size_t)A.ws.numel(),
                              current_stream(*A.first)), fn);
}

void supergrok11_fused_step(std::vector<torch::Tensor>& params, std::vector<torch::Tensor>& grads, std::vector<torch::Tensor>& exp_avgs,
                            std::vector<torch::Tensor>& exp_avg_sqs, std::vector<torch::Tensor>& mus,
                            std::vector<torch::Tensor>& sharpness_cache, std::vector<int64_t>& steps, std::vector<float>& layer_alphas,
                            std::vector<float>& layer_beta1s, torch::Tensor W1, torch::Tensor b1, torch::Tensor W2, torch::Tensor b2,
                            float rescale, int hidden_dim, float beta2, float lr, float wd_eff, float eps, float lamb, float ramp,
                            float gate_temperature, float grad_clip_norm) {
    const char* fn = "supergrok11_fused_step";
    std::vector<float> bc1(params.size(), 1.0f), bc2(params.size(), 1.0f);
    for (size_t i = 0; i < params.size(); i++) {
        if (!grads[i].defined() || grads[i].numel() == 0) continue;
        steps[i] += 1;   // pybind's copy of the Python list, exactly as in the reference (csrc/ops.cpp:237)
        const float step = static_cast<float>(steps[i]);
        bc1[i] = 1.0f - std::pow(layer_beta1s[i], step);
        bc2[i] = 1.0f - std::pow(beta2, step);
    }
    FamilyArgs A;
    gather_family(fn, &A, params, grads, &exp_avgs, &exp_avg_sqs, &mus, &sharpness_cache, false, &bc1, &bc2, &layer_alphas, &layer_beta1s);
    if (A.ts.empty()) return;
    auto W1f = W1.to(torch::kFloat32).contiguous(), b1f = b1.to(torch::kFloat32).contiguous();
    auto W2f = W2.to(torch::kFloat32).contiguous(), b2f = b2.to(torch::kFloat32).contiguous();
    check_f32(W1f, fn, "W1"); check_f32(b1f, fn, "b1"); check_f32(W2f, fn, "W2"); check_f32(b2f, fn, "b2");
    TORCH_CHECK(W1f.numel() == 2 * hidden_dim && b1f.numel() == hidden_dim && W2f.numel() == hidden_dim && b2f.numel() == 1, fn,
                ": meta-net weight shapes do not match hidden_dim");
    Sg15Net net = {W1f.data_ptr<float>(), b1f.data_ptr<float>(), W2f.data_ptr<float>(), b2f.data_ptr<float>(), hidden_dim, rescale,
                   g_sg15_gelu_mode};
    A.make_ws();
    check_status(sg11_fused_step((int)A.ts.size(), A.ts.data(), &net, beta2, lr, wd_eff, eps, lamb, ramp, gate_temperature, grad_clip_norm,
                                 A.ws.data_ptr(), (size_t)A.ws.numel(), current_stream(*A.first)), fn);
}

std::vector<torch::Tensor> supergrok11_sam_perturb_all(std::vector<torch::Tensor>& params, std::vector<torch::Tensor>& grads, float rho) {
    return supergrok15_sam_perturb_all(params, grads, rho);
}
void supergrok11_sharpness_restore_all(std::vector<torch::Tensor>& params, std::vector<torch::Tensor>& sharpness_cache,
                                       std::vector<torch::Tensor>& backups, std::vector<torch::Tensor>& sam_grads,
                                       std::vector<torch::Tensor>& normal_grads) {
    supergrok15_sharpness_restore_all(params, sharpness_cache, backups, sam_grads, normal_grads);
}

std::vector<torch::Tensor> looksam_perturb_all(std::vector<torch::Tensor>& params, std::vector<torch::Tensor>& grads, float rho) {
    return supergrok15_sam_perturb_all(params, grads, rho);
}

namespace {
void looksam_call(const char* fn, int mode, std::vector<torch::Tensor>& a, std::vector<torch::Tensor>& b, std::vector<torch::Tensor>* c, float la) {
    std::vector<SgLookSamTensor> ts;
    std::vector<int64_t> numels;
    const torch::Tensor* first = nullptr;
    for (size_t i = 0; i < a.size(); i++) {
        // mode 0: a=param, b=backup; mode 1: a=v_dir, b=sam_grad, c=normal_grad; mode 2: a=grad, b=v_dir
        const torch::Tensor& typed = (mode == 1) ? b[i] : a[i];
        if (!a[i].defined() || !b[i].defined() || a[i].numel() == 0 || b[i].numel() == 0) continue;
        if (mode == 1 && (!(*c)[i].defined() || (*c)[i].numel() == 0)) continue;
        check_gpu(a[i], fn, "tensor");
        check_gpu(b[i], fn, "tensor");
        if (mode == 0) TORCH_CHECK(a[i].scalar_type() == b[i].scalar_type(), fn, ": param/backup dtype mismatch");
        if (mode == 1) {
            check_f32(a[i], fn, "v_dir");
            check_gpu((*c)[i], fn, "normal_grad");
            TORCH_CHECK(b[i].scalar_type() == (*c)[i].scalar_type(), fn, ": gradient dtype mismatch");
        }
        if (mode == 2) check_f32(b[i], fn, "v_dir");
        TORCH_CHECK(a[i].numel() == b[i].numel(), fn, ": size mismatch");
        ts.push_back({a[i].data_ptr(), b[i].data_ptr(), mode == 1 ? (*c)[i].data_ptr() : nullptr, typed.numel(), dtype_code(typed, "tensor")});
        numels.push_back(typed.numel());
        if (!first) first = &a[i];
    }
    if (ts.empty()) return;
    auto ws = make_workspace(sg_family_workspace_bytes((int)ts.size(), numels.data()), *first);
    int rc = 0;
    if (mode == 0) rc = sg_looksam_restore((int)ts.size(), ts.data(), ws.data_ptr(), (size_t)ws.numel(), current_stream(*first));
    if (mode == 1) rc = sg_looksam_directions((int)ts.size(), ts.data(), ws.data_ptr(), (size_t)ws.numel(), current_stream(*first));
    if (mode == 2) rc = sg_looksam_adjust((int)ts.size(), ts.data(), la, ws.data_ptr(), (size_t)ws.numel(), current_stream(*first));
    check_status(rc, fn);
}
}  // namespace

void looksam_restore_all(std::vector<torch::Tensor>& params, std::vector<torch::Tensor>& backups) {
    looksam_call("looksam_restore_all", 0, params, backups, nullptr, 0.0f);
}
void looksam_compute_directions(std::vector<torch::Tensor>& v_dirs, std::vector<torch::Tensor>& sam_grads,
                                std::vector<torch::Tensor>& normal_grads) {
    looksam_call("looksam_compute_directions", 1, v_dirs, sam_grads, &normal_grads, 0.0f);
}
void looksam_adjust_grads(std::vector<torch::Tensor>& grads, std::vector<torch::Tensor>& v_dirs, float la) {
    looksam_call("looksam_adjust_grads", 2, grads, v_dirs, nullptr, la);
}

// Per-tensor clip + non-finite guard of the v2 pre-pass (grokking_optimizers/supergrok2.py:316-321 of the
// reference), for all tensors in three launches and without host syncs.  Returns new tensors.
std::vector<torch::Tensor> supergrok2_clip_grads(std::vector<torch::Tensor>& grads, float max_norm) {
    const char* fn = "supergrok2_clip_grads";
    std::vector<torch::Tensor> out;
    std::vector<Sg2ClipTensor> ts;
    std::vector<int64_t> numels;
    const torch::Tensor* first = nullptr;
    for (size_t i = 0; i < grads.size(); i++) {
        if (!grads[i].defined()) { out.push_back(grads[i]); continue; }
        check_gpu(grads[i], fn, "grad");
        out.push_back(torch::empty_like(grads[i]));
        if (grads[i].numel() == 0) continue;
        ts.push_back({grads[i].data_ptr(), out.back().data_ptr(), grads[i].numel(), dtype_code(grads[i], "grad")});
        numels.push_back(grads[i].numel());
        if (!first) first = &grads[i];
    }
    if (ts.empty()) return out;
    auto ws = make_workspace(sg_family_workspace_bytes((int)ts.size(), numels.data()), *first);
    check_status(sg2_clip_grads((int)ts.size(), ts.data(), max_norm, ws.data_ptr(), (size_t)ws.numel(), current_stream(*first)), fn);
    return out;
}

// ---- the reference's bilevel entry points (ops_bilevel.cpp)
void supergrok2_bilevel_fwd_save_batched(
    std::vector<torch::Tensor>, std::vector<torch::Tensor>, torch::Tensor, torch::Tensor, torch::Tensor, torch::Tensor, torch::Tensor,
    torch::Tensor, torch::Tensor, torch::Tensor, torch::Tensor, torch::Tensor, torch::Tensor, torch::Tensor, torch::Tensor, torch::Tensor,
    torch::Tensor, torch::Tensor, torch::Tensor, torch::Tensor, torch::Tensor, torch::Tensor, int, int, int, torch::Tensor, torch::Tensor,
    torch::Tensor, torch::Tensor, torch::Tensor, torch::Tensor, torch::Tensor, torch::Tensor, torch::Tensor, torch::Tensor, torch::Tensor,
    torch::Tensor, torch::Tensor, torch::Tensor, torch::Tensor, int);
void supergrok2_bilevel_backward_batched(
    torch::Tensor, torch::Tensor, torch::Tensor, torch::Tensor, torch::Tensor, torch::Tensor, torch::Tensor, torch::Tensor, torch::Tensor,
    torch::Tensor, torch::Tensor, torch::Tensor, torch::Tensor, torch::Tensor, torch::Tensor, torch::Tensor, torch::Tensor, torch::Tensor,
    torch::Tensor, torch::Tensor, torch::Tensor, torch::Tensor, torch::Tensor, torch::Tensor, torch::Tensor, torch::Tensor, torch::Tensor,
    torch::Tensor, torch::Tensor, torch::Tensor, torch::Tensor, torch::Tensor, torch::Tensor, torch::Tensor, torch::Tensor, torch::Tensor,
    torch::Tensor, torch::Tensor, torch::Tensor, torch::Tensor, torch::Tensor, torch::Tensor, torch::Tensor, torch::Tensor, torch::Tensor,
    torch::Tensor, torch::Tensor, int, int, int, int, int);
void supergrok2_bilevel_fwd_save(
    torch::Tensor, torch::Tensor, torch::Tensor, torch::Tensor, torch::Tensor, torch::Tensor, torch::Tensor, torch::Tensor, torch::Tensor,
    torch::Tensor, torch::Tensor, torch::Tensor, torch::Tensor, torch::Tensor, torch::Tensor, torch::Tensor, torch::Tensor, torch::Tensor,
    torch::Tensor, torch::Tensor, torch::Tensor, torch::Tensor, int, int, int, torch::Tensor, torch::Tensor, torch::Tensor, torch::Tensor,
    torch::Tensor, torch::Tensor, torch::Tensor, torch::Tensor, torch::Tensor, torch::Tensor, torch::Tensor, torch::Tensor, torch::Tensor,
    torch::Tensor, torch::Tensor, torch::Tensor, int);
void supergrok2_bilevel_backward(
    torch::Tensor, torch::Tensor, torch::Tensor, float, torch::Tensor, torch::Tensor, torch::Tensor, torch::Tensor, torch::Tensor,
    torch::Tensor, torch::Tensor, torch::Tensor, torch::Tensor, torch::Tensor, torch::Tensor, torch::Tensor, torch::Tensor, torch::Tensor,
    torch::Tensor, torch::Tensor, torch::Tensor, torch::Tensor, torch::Tensor, torch::Tensor, torch::Tensor, torch::Tensor, torch::Tensor,
    torch::Tensor, torch::Tensor, torch::Tensor, torch::Tensor, torch::Tensor, torch::Tensor, torch::Tensor, torch::Tensor, torch::Tensor,
    torch::Tensor, torch::Tensor, torch::Tensor, torch::Tensor, torch::Tensor, torch::Tensor, torch::Tensor, torch::Tensor, torch::Tensor,
    torch::Tensor, torch::Tensor, torch::Tensor, torch::Tensor, torch::Tensor, torch::Tensor, torch::Tensor, torch::Tensor, torch::Tensor,
    torch::Tensor, torch::Tensor, torch::Tensor, torch::Tensor, torch::Tensor, torch::Tensor, torch::Tensor, torch::Tensor, torch::Tensor,
    torch::Tensor, torch::Tensor, torch::Tensor, torch::Tensor, torch::Tensor, torch::Tensor, torch::Tensor, torch::Tensor, torch::Tensor,
    torch::Tensor, torch::Tensor, torch::Tensor, torch::Tensor, torch::Tensor, torch::Tensor, torch::Tensor, torch::Tensor, torch::Tensor,
    torch::Tensor, torch::Tensor, torch::Tensor, torch::Tensor, torch::Tensor, torch::Tensor, torch::Tensor, torch::Tensor, torch::Tensor,
    torch::Tensor, torch::Tensor, torch::Tensor, torch::Tensor, torch::Tensor, int, int, int, int, int, int, int, int, int, int, int, int);

PYBIND11_MODULE(TORCH_EXTENSION_NAME, m) {
    m.doc() = "Grokking optimizers: fused steps on MI355X (hand-written HIP behind the reference's _ops surface)";
    m.def("supergrok15_fused_step", &supergrok15_fused_step, "SuperGrok1.5: fused clip + mu + meta-net + gating + adam + progressive wd",
          py::arg("params"), py::arg("grads"), py::arg("exp_avgs"), py::arg("exp_avg_sqs"), py::arg("mus"),
          py::arg("sharpness_cache"), py::arg("steps"), py::arg("layer_alphas"), py::arg("layer_beta1s"), py::arg("W1"),
          py::arg("b1"), py::arg("W2"), py::arg("b2"), py::arg("rescale"), py::arg("hidden_dim"), py::arg("beta2"), py::arg("lr"),
          py::arg("wd_eff"), py::arg("eps"), py::arg("lamb"), py::arg("ramp"), py::arg("gate_signal"), py::arg("grad_clip_norm"));
    m.def("supergrok15_sam_perturb_all", &supergrok15_sam_perturb_all, py::arg("params"), py::arg("grads"), py::arg("rho"));
    m.def("supergrok15_sharpness_restore_all", &supergrok15_sharpness_restore_all, py::arg("params"), py::arg("sharpness_cache"),
          py::arg("backups"), py::arg("sam_grads"), py::arg("normal_grads"));
    m.def("supergrok11_fused_step", &supergrok11_fused_step, "SuperGrok1.1: fused clip + mu + meta-net + cosine gate + adam",
          py::arg("params"), py::arg("grads"), py::arg("exp_avgs"), py::arg("exp_avg_sqs"), py::arg("mus"), py::arg("sharpness_cache"),
          py::arg("steps"), py::arg("layer_alphas"), py::arg("layer_beta1s"), py::arg("W1"), py::arg("b1"), py::arg("W2"), py::arg("b2"),
          py::arg("rescale"), py::arg("hidden_dim"), py::arg("beta2"), py::arg("lr"), py::arg("wd_eff"), py::arg("eps"), py::arg("lamb"),
          py::arg("ramp"), py::arg("gate_temperature"), py::arg("grad_clip_norm"));
    m.def("supergrok11_sam_perturb_all", &supergrok11_sam_perturb_all, py::arg("params"), py::arg("grads"), py::arg("rho"));
    m.def("supergrok11_sharpness_restore_all", &supergrok11_sharpness_restore_all, py::arg("params"), py::arg("sharpness_cache"),
          py::arg("backups"), py::arg("sam_grads"), py::arg("normal_grads"));
    m.def("grokadamw_fused_step", &grokadamw_fused_step, "GrokAdamW: fused EMA filter + amplification + Adam", py::arg("params"),
          py::arg("grads"), py::arg("exp_avgs"), py::arg("exp_avg_sqs"), py::arg("emas"), py::arg("steps"), py::arg("alpha"),
          py::arg("lamb"), py::arg("beta1"), py::arg("beta2"), py::arg("lr"), py::arg("wd"), py::arg("eps"), py::arg("grad_clip_norm"));
    m.def("neuralgrok_fused_step", &neuralgrok_fused_step, "NeuralGrok: fused MLP amplifier + Adam", py::arg("params"), py::arg("grads"),
          py::arg("exp_avgs"), py::arg("exp_avg_sqs"), py::arg("steps"), py::arg("W1"), py::arg("b1"), py::arg("W2"), py::arg("b2"),
          py::arg("alpha_amp"), py::arg("beta_amp"), py::arg("hidden_dim"), py::arg("beta1"), py::arg("beta2"), py::arg("lr"),
          py::arg("wd"), py::arg("eps"), py::arg("grad_clip_norm"));
    m.def("prodigy_fused_step", &prodigy_fused_step, "Prodigy: distance-aware self-tuning Adam; returns the new d_lr", py::arg("params"),
          py::arg("grads"), py::arg("exp_avgs"), py::arg("exp_avg_sqs"), py::arg("s_bufs"), py::arg("param_inits"), py::arg("steps"),
          py::arg("d_lr"), py::arg("beta1"), py::arg("beta2"), py::arg("lr"), py::arg("wd"), py::arg("eps"));
    m.def("adamw_fused_step", &adamw_fused_step, "AdamW over a tensor list in one launch", py::arg("params"), py::arg("grads"),
          py::arg("exp_avgs"), py::arg("exp_avg_sqs"), py::arg("steps"), py::arg("lr"), py::arg("beta1"), py::arg("beta2"), py::arg("eps"),
          py::arg("wd"));
    m.def("supergrok2_clip_grads", &supergrok2_clip_grads, "SuperGrok2 pre-pass: per-tensor norm clip + non-finite guard, device-side",
          py::arg("grads"), py::arg("max_norm"));
    m.def("lion_fused_step", &lion_fused_step, "Lion: fused sign-momentum step", py::arg("params"), py::arg("grads"), py::arg("exp_avgs"),
          py::arg("lr"), py::arg("beta1"), py::arg("beta2"), py::arg("wd"));
    m.def("looksam_perturb_all", &looksam_perturb_all, py::arg("params"), py::arg("grads"), py::arg("rho"));
    m.def("looksam_restore_all", &looksam_restore_all, py::arg("params"), py::arg("backups"));
    m.def("looksam_compute_directions", &looksam_compute_directions, py::arg("v_dirs"), py::arg("sam_grads"), py::arg("normal_grads"));
    m.def("looksam_adjust_grads", &looksam_adjust_grads, py::arg("grads"), py::arg("v_dirs"), py::arg("la"));
    m.def("supergrok15_set_gelu_mode", &supergrok15_set_gelu_mode, py::arg("mode"));
    m.def("grokfast_fused_step", &grokfast_fused_step, "Grokfast: fused EMA update + gradient amplification", py::arg("grads"),
          py::arg("ema_bufs"), py::arg("alpha"), py::arg("lamb"));
    m.def("grokfast_adamw_fused_step", &grokfast_adamw_fused_step, "Grokfast: EMA + amplification + AdamW in one pass",
          py::arg("params"), py::arg("grads"), py::arg("ema_bufs"), py::arg("exp_avgs"), py::arg("exp_avg_sqs"), py::arg("steps"),
          py::arg("alpha"), py::arg("lamb"), py::arg("lr"), py::arg("beta1"), py::arg("beta2"), py::arg("eps"),
          py::arg("weight_decay"));
    m.def("muon_fused_step", &muon_fused_step, "Muon: momentum + Newton-Schulz ortho + update + WD", py::arg("params"),
          py::arg("grads"), py::arg("bufs"), py::arg("momentum"), py::arg("lr"), py::arg("wd"), py::arg("ns_steps"));
    m.def("supergrok2_mamba_peer_step", &supergrok2_mamba_peer_step, "SuperGrok2: per-param Mamba-3+PEER meta-net + mu + Adam + WD",
          py::arg("param"), py::arg("grad"), py::arg("sharpness"), py::arg("exp_avg"), py::arg("exp_avg_sq"), py::arg("mu"),
          py::arg("gru_state"), py::arg("mamba_fwd_state"), py::arg("mamba_bwd_state"), py::arg("input_proj_W"),
          py::arg("input_proj_b"), py::arg("mamba_fwd_in_proj"), py::arg("mamba_fwd_dt_W"), py::arg("mamba_fwd_dt_b"),
          py::arg("mamba_fwd_B_proj"), py::arg("mamba_fwd_C_proj"), py::arg("mamba_fwd_A_log"), py::arg("mamba_fwd_D"),
          py::arg("mamba_fwd_rope"), py::arg("mamba_fwd_out_proj"), py::arg("mamba_bwd_in_proj"), py::arg("mamba_bwd_dt_W"),
          py::arg("mamba_bwd_dt_b"), py::arg("mamba_bwd_B_proj"), py::arg("mamba_bwd_C_proj"), py::arg("mamba_bwd_A_log"),
          py::arg("mamba_bwd_D"), py::arg("mamba_bwd_rope"), py::arg("mamba_bwd_out_proj"), py::arg("gru_Wz"), py::arg("gru_bz"),
          py::arg("gru_Wr"), py::arg("gru_br"), py::arg("gru_Wh"), py::arg("gru_bh"), py::arg("peer_query_Ws"),
          py::arg("prod_keys_A"), py::arg("prod_keys_B"), py::arg("expert_W1"), py::arg("expert_b1"), py::arg("expert_W2"),
          py::arg("expert_b2"), py::arg("rescale"), py::arg("alpha_mu"), py::arg("lamb_eff"), py::arg("beta1"), py::arg("beta2"),
          py::arg("lr"), py::arg("wd_eff"), py::arg("eps"), py::arg("bc1"), py::arg("bc2"), py::arg("d_model"), py::arg("d_state"),
          py::arg("d_inner"), py::arg("gru_hidden"), py::arg("num_heads"), py::arg("pk_dim"), py::arg("expert_hidden"),
          py::arg("num_experts"), py::arg("expert_counts"));
    m.def("supergrok2_mamba_peer_batched_step", &supergrok2_mamba_peer_batched_step,
          "SuperGrok2: batched Mamba-3+PEER step for all params at once", py::arg("params"), py::arg("grads"),
          py::arg("sharpness_list"), py::arg("exp_avgs"), py::arg("exp_avg_sqs"), py::arg("mus"), py::arg("gru_states"),
          py::arg("mamba_fwd_states"), py::arg("mamba_bwd_states"), py::arg("input_proj_W"), py::arg("input_proj_b"),
          py::arg("mamba_fwd_in_proj"), py::arg("mamba_fwd_dt_W"), py::arg("mamba_fwd_dt_b"), py::arg("mamba_fwd_B_proj"),
          py::arg("mamba_fwd_C_proj"), py::arg("mamba_fwd_A_log"), py::arg("mamba_fwd_D"), py::arg("mamba_fwd_rope"),
          py::arg("mamba_fwd_out_proj"), py::arg("mamba_bwd_in_proj"), py::arg("mamba_bwd_dt_W"), py::arg("mamba_bwd_dt_b"),
          py::arg("mamba_bwd_B_proj"), py::arg("mamba_bwd_C_proj"), py::arg("mamba_bwd_A_log"), py::arg("mamba_bwd_D"),
          py::arg("mamba_bwd_rope"), py::arg("mamba_bwd_out_proj"), py::arg("gru_Wz"), py::arg("gru_bz"), py::arg("gru_Wr"),
          py::arg("gru_br"), py::arg("gru_Wh"), py::arg("gru_bh"), py::arg("peer_query_Ws"), py::arg("prod_keys_A"),
          py::arg("prod_keys_B"), py::arg("expert_W1"), py::arg("expert_b1"), py::arg("expert_W2"), py::arg("expert_b2"),
          py::arg("alpha_mus"), py::arg("lamb_effs"), py::arg("beta1s"), py::arg("bc1s"), py::arg("bc2s"), py::arg("rescale"),
          py::arg("beta2"), py::arg("lr"), py::arg("wd_eff"), py::arg("eps"), py::arg("d_model"), py::arg("d_state"),
          py::arg("d_inner"), py::arg("gru_hidden"), py::arg("num_heads"), py::arg("pk_dim"), py::arg("expert_hidden"),
          py::arg("num_experts"), py::arg("expert_counts"));
    // bilevel meta-training: the reference's names and argument lists (csrc/ops.cpp:1072-1085 there)
    m.def("supergrok2_bilevel_fwd_save", &supergrok2_bilevel_fwd_save, "SuperGrok2 bilevel: forward scan with state saving for backward");
    m.def("supergrok2_bilevel_fwd_save_batched", &supergrok2_bilevel_fwd_save_batched,
          "SuperGrok2 bilevel: batched forward scan with state saving");
    m.def("supergrok2_bilevel_backward_batched", &supergrok2_bilevel_backward_batched, "SuperGrok2 bilevel: batched backward through scan");
    m.def("supergrok2_bilevel_backward", &supergrok2_bilevel_backward, "SuperGrok2 bilevel: full backward through meta-net");
}
