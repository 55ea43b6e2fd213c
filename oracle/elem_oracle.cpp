/*
 * TEST INFRASTRUCTURE ONLY.  CPU restatement of the Grokfast and SuperGrok
 * v1.5 fused steps, fp32 with the fixed-order primitives of
 * include/sg_math.h (the device kernels use the same expressions).  Nothing
 * in the shipped package links or calls this file.
 *
 * Reference lines followed (paths relative to the reference tree):
 *   Grokfast EMA + amplification        csrc/grokfast_kernels.cu:20-39, csrc/ops.cpp:528-530
 *   AdamW (decay first, double scalars) grokking_optimizers/_adamw_helper.py:12-22
 *   v1.5 clip coefficient               csrc/ops.cpp:46-52
 *   v1.5 mu / meta-net / Adam / WD      csrc/supergrok15_kernels.cu:363-403, csrc/ops.cpp:132-150
 *   GELU: exact erf (CPU path, csrc/ops.cpp:140) or sigmoid form (csrc/supergrok15_kernels.cu:380)
 *   SAM perturb / sharpness restore     csrc/supergrok15_kernels.cu:151-184, csrc/ops.cpp:154-204
 *
 * Parity status: pinned in this container against the reference's own CPU
 * code compiled from its sources (oracle/_ref, tests/test_oracle_elem.py),
 * against torch.optim.AdamW and against libm-based float64 restatements.
 */
#include <cmath>
#include <cstdint>

#include "../include/sg_math.h"

extern "C" {

void orc_grokfast_ema(float* grad, float* ema, int64_t n, float alpha, float lamb) {
    const float om = 1.0f - alpha;
    for (int64_t i = 0; i < n; i++) {
        const float g = grad[i];
        const float e = sg_fma(alpha, ema[i], om * g);
        ema[i] = e;
        grad[i] = sg_fma(lamb, e, g);
    }
}

void orc_grokfast_adamw(float* param, float* grad, float* ema, float* ea, float* easq, int64_t n, int step, float alpha,
                        float lamb, double lr, double beta1, double beta2, double eps, double wd) {
    orc_grokfast_ema(grad, ema, n, alpha, lamb);
    const double bc1 = 1.0 - std::pow(beta1, (double)step), bc2d = 1.0 - std::pow(beta2, (double)step);
    const float step_size = (float)(lr / bc1), bc2 = (float)bc2d, b1 = (float)beta1, ob1 = (float)(1.0 - beta1);
    const float b2 = (float)beta2, ob2 = (float)(1.0 - beta2), epsf = (float)eps, decay = (float)(1.0 - lr * wd);
    for (int64_t i = 0; i < n; i++) {
        const float g = grad[i];
        const float m = sg_fma(b1, ea[i], ob1 * g);
        const float v = sg_fma(b2, easq[i], (ob2 * g) * g);
        ea[i] = m;
        easq[i] = v;
        const float denom = __builtin_sqrtf(v / bc2) + epsf;
        param[i] = sg_fma(param[i], decay, -((step_size * m) / denom));
    }
}

/* one tensor; coef/clip_on come from the global norm over all tensors */
void orc_sg15_step(float* param, float* grad, const float* sharp, float* ea, float* easq, float* mu, int64_t n,
                   const float* W1, const float* b1, const float* W2, const float* b2, int H, float rescale, int gelu_mode,
                   float alpha, float beta1, float bc1, float bc2, float lamb_eff, float beta2, float lr, float wd_eff,
                   float eps, float coef, int clip_on) {
    const float step_size = lr / bc1, decay = 1.0f - lr * wd_eff;
    for (int64_t i = 0; i < n; i++) {
        float g = grad[i];
        if (clip_on) {
            g = g * coef;
            grad[i] = g;
        }
        const float s = sharp[i];
        const float m = sg_fma(alpha, mu[i], (1.0f - alpha) * g);
        mu[i] = m;
        float acc = 0.0f;
        for (int h = 0; h < H; h++) {
            const float z = sg_fma(W1[2 * h + 1], s, W1[2 * h] * g) + b1[h];
            const float a = gelu_mode == 0 ? sg_gelu_erf(z) : sg_gelu_sigmoid(z);
            acc = sg_fma(W2[h], a, acc);
        }
        const float smart = sg_fma(rescale, acc + b2[0], g);
        const float fg = sg_fma(lamb_eff, m, smart);
        const float e1 = sg_fma(beta1, ea[i], (1.0f - beta1) * fg);
        const float e2 = sg_fma(beta2, easq[i], ((1.0f - beta2) * fg) * fg);
        ea[i] = e1;
        easq[i] = e2;
        const float denom = __builtin_sqrtf(e2 / bc2) + eps;
        param[i] = sg_fma(param[i], decay, -((step_size * e1) / denom));
    }
}

float orc_erfc(float x) { return sg_erfc(x); }
float orc_gelu_erf(float x) { return sg_gelu_erf(x); }
float orc_gelu_sigmoid(float x) { return sg_gelu_sigmoid(x); }

}  // extern "C"
