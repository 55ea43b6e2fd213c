// Issue-rate probe of the fp32 vector ALU: what one MI355X sustains in wave64 instructions per nanosecond and
// SIMD for plain (non-packed) fma / mul / add / DPP-add streams, as a function of the waves resident per SIMD and
// of the share of the chip that is busy.  It is the yardstick the arithmetic-bound kernels of this library
// (the v2 scan and per-element kernels) are priced against; the reference has nothing comparable.
// Op 4 is the same for the matrix cores: a stream of independent v_mfma_f32_32x32x16_bf16 on register operands
// (no memory traffic at all), the ceiling the Muon GEMM's main loop is priced against.
#include "../../supergrok1.5_amd/csrc/sg_common.hpp"

namespace {

constexpr int PROBE_ILP = 8;       // independent accumulators per lane: no instruction waits for its predecessor
constexpr int PROBE_UNROLL = 16;

template <int OP>
__global__ __launch_bounds__(256) void k_probe(float* sink, long long* ticks, int iters, float a, float b) {
    float acc[PROBE_ILP];
#pragma unroll
    for (int k = 0; k < PROBE_ILP; k++) acc[k] = threadIdx.x * 1e-3f + k + 1.0f;
    float xs[4], ys[4];        // per-lane factors of the accumulate form, of both signs so that the sums stay bounded
#pragma unroll
    for (int k = 0; k < 4; k++) {
        xs[k] = ((k & 1) ? -1.0f : 1.0f) * (a + 1e-3f * (threadIdx.x & 15) + 0.01f * k);
        ys[k] = ((k & 2) ? -1.0f : 1.0f) * (b + 1e-3f * (threadIdx.x & 7));
    }
    const long long t0 = clock64();
    for (int i = 0; i < iters; i++) {
#pragma unroll
        for (int r = 0; r < PROBE_UNROLL; r++) {
#pragma unroll
            for (int k = 0; k < PROBE_ILP; k++) {
                if (OP == 0) acc[k] = __builtin_fmaf(acc[k], a, b);
                else if (OP == 4) acc[k] = __builtin_fmaf(xs[(k + r) & 3], ys[k & 3], acc[k]);      // accumulate form: v_fmac_f32
                else if (OP == 5) acc[k] = __builtin_fmaf(acc[k], xs[(k + r) & 3], ys[k & 3]);      // op 0 with per-lane register operands
                else if (OP == 6) acc[k] = __builtin_fmaf(acc[k], a, acc[(k + 1) % PROBE_ILP]);     // three vector registers, one scalar
                else if (OP == 1) acc[k] = acc[k] * a;
                else if (OP == 2) acc[k] = acc[k] + a;
                else acc[k] = acc[k] + sg_i2f(__builtin_amdgcn_update_dpp(0, sg_f2i(acc[k]), 0xB1, 0xF, 0xF, true));
            }
        }
    }
    const long long t1 = clock64();
    float s = 0.0f;
#pragma unroll
    for (int k = 0; k < PROBE_ILP; k++) s += acc[k];
    if (s == 12345.678f) sink[0] = s;       // keeps the arithmetic alive
    if (threadIdx.x == 0) ticks[blockIdx.x] = t1 - t0;
}

typedef __attribute__((ext_vector_type(8))) __bf16 probe_bf16x8;
typedef __attribute__((ext_vector_type(16))) float probe_f32x16;
constexpr int PROBE_MFMA_ACC = 4;  // independent accumulator tiles per wave

// RANDOM: operands are pseudo-random bf16 values in (-1, 1), different in every lane and element, and four operand
// pairs alternate: what the data of a real product costs in power (and therefore clock) against constant operands
template <bool RANDOM>
__global__ __launch_bounds__(256) void k_probe_mfma(float* sink, long long* ticks, int iters) {
    probe_f32x16 acc[PROBE_MFMA_ACC];
    probe_bf16x8 av[PROBE_MFMA_ACC], bv[PROBE_MFMA_ACC];
#pragma unroll
    for (int k = 0; k < PROBE_MFMA_ACC; k++)
#pragma unroll
        for (int e = 0; e < 8; e++) {
            if (RANDOM) {
                uint32_t h = (threadIdx.x * 8u + e + 2048u * k + 8192u * blockIdx.x) * 2654435761u;
                h ^= h >> 15; h *= 2246822519u; h ^= h >> 13;
                av[k][e] = (__bf16)(((int)(h & 0xffffu) - 32768) * (1.0f / 32768.0f));
                bv[k][e] = (__bf16)(((int)(h >> 16) - 32768) * (1.0f / 32768.0f));
            } else {
                av[k][e] = (__bf16)(1.0f + 0.001f * (threadIdx.x & 7));
                bv[k][e] = (__bf16)(0.5f);
            }
        }
#pragma unroll
    for (int k = 0; k < PROBE_MFMA_ACC; k++)
#pragma unroll
        for (int e = 0; e < 16; e++) acc[k][e] = 0.0f;
    const long long t0 = clock64();
    for (int i = 0; i < iters; i++) {
#pragma unroll
        for (int r = 0; r < PROBE_UNROLL * PROBE_ILP / PROBE_MFMA_ACC; r++) {
#pragma unroll
            for (int k = 0; k < PROBE_MFMA_ACC; k++) acc[k] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(av[(k + r) % PROBE_MFMA_ACC], bv[k], acc[k], 0, 0, 0);
        }
    }
    const long long t1 = clock64();
    float s = 0.0f;
#pragma unroll
    for (int k = 0; k < PROBE_MFMA_ACC; k++)
#pragma unroll
        for (int e = 0; e < 16; e++) s += acc[k][e];
    if (s == 12345.678f) sink[0] = s;
    if (threadIdx.x == 0) ticks[blockIdx.x] = t1 - t0;
}

typedef __attribute__((ext_vector_type(32))) float probe_f32x32;
typedef __attribute__((ext_vector_type(4))) float probe_f32x4;
// fp32 matrix instructions with one fused multiply-add per output (k = 1), the forms whose chains equal fmaf chains
// bit for bit.  KIND 0: v_mfma_f32_32x32x1_2b (2048 multiply-adds); 1: the same with 8 independent vector fma after
// every matrix instruction, in the same wave (do the two pipes overlap?); 2: v_mfma_f32_4x4x1_16b (256 multiply-adds).
template <int KIND>
__global__ __launch_bounds__(256) void k_probe_mfma_f32(float* sink, long long* ticks, int iters, float a, float b) {
    probe_f32x32 big[2];
    probe_f32x4 small[PROBE_ILP];
    float acc[PROBE_ILP];
#pragma unroll
    for (int k = 0; k < 2; k++)
#pragma unroll
        for (int e = 0; e < 32; e++) big[k][e] = 0.0f;
#pragma unroll
    for (int k = 0; k < PROBE_ILP; k++) {
        acc[k] = threadIdx.x * 1e-3f + k + 1.0f;
        small[k] = probe_f32x4{0.0f, 0.0f, 0.0f, 0.0f};
    }
    const float av = a + 1e-3f * (threadIdx.x & 31), bv = b + 1e-3f * (threadIdx.x & 15);
    const long long t0 = clock64();
    for (int i = 0; i < iters; i++) {
#pragma unroll
        for (int r = 0; r < PROBE_UNROLL * PROBE_ILP; r++) {
            if (KIND == 2) {
                small[r % PROBE_ILP] = __builtin_amdgcn_mfma_f32_4x4x1f32(av, bv, small[r % PROBE_ILP], 0, 0, 0);
            } else {
                big[r & 1] = __builtin_amdgcn_mfma_f32_32x32x1f32(av, bv, big[r & 1], 0, 0, 0);
                if (KIND == 1) {
#pragma unroll
                    for (int k = 0; k < PROBE_ILP; k++) acc[k] = __builtin_fmaf(acc[k], a, b);
                }
            }
        }
    }
    const long long t1 = clock64();
    float s = 0.0f;
#pragma unroll
    for (int k = 0; k < PROBE_ILP; k++) s += acc[k] + small[k][0] + small[k][3];
    s += big[0][0] + big[0][31] + big[1][7];
    if (s == 12345.678f) sink[0] = s;
    if (threadIdx.x == 0) ticks[blockIdx.x] = t1 - t0;
}

}  // namespace

extern "C" {

const char* sg_probe_last_error(void) { return sg::last_error().c_str(); }

size_t sg_probe_workspace_bytes(int num_cus, int waves_per_simd) {
    if (num_cus <= 0 || waves_per_simd <= 0) return 0;
    return 256 + sizeof(long long) * (size_t)num_cus * (size_t)waves_per_simd;
}

int sg_probe_valu(int op, int num_cus, int waves_per_simd, int iters, float* ms_out, double* ticks_per_wave_out,
                  double* instr_per_wave_out, void* workspace, size_t workspace_bytes, void* stream) {
    hipStream_t st = (hipStream_t)stream;
    if (op < 0 || op > 11)
        return sg::fail("op must be 0 (fma), 1 (mul), 2 (add), 3 (add with a DPP operand), 4 (32x32x16 bf16 MFMA, constant operands), 5 (the same, random "
                        "operands), 6 (32x32x1 fp32 MFMA), 7 (the same with 8 vector fma after each), 8 (4x4x1 fp32 MFMA), 9 (fma in its accumulate "
                        "form, per-lane factors), 10 (fma, vector-register operands only) or 11 (fma with one scalar-register operand)");
    if (num_cus <= 0 || num_cus > 1024 || waves_per_simd <= 0 || waves_per_simd > 8 || iters <= 0 || iters > 100000)
        return sg::fail("probe size out of range");
    if (!ms_out || !ticks_per_wave_out || !instr_per_wave_out) return sg::fail("NULL argument");
    const int blocks = num_cus * waves_per_simd;         // 256 threads = one wave on each of the four SIMDs of a CU
    if (!workspace || workspace_bytes < sg_probe_workspace_bytes(num_cus, waves_per_simd)) return sg::fail("workspace too small");
    float* sink = static_cast<float*>(workspace);
    long long* ticks = reinterpret_cast<long long*>(static_cast<unsigned char*>(workspace) + 256);
    hipEvent_t e0, e1;
    SG_HIP_CHECK(hipEventCreate(&e0));
    SG_HIP_CHECK(hipEventCreate(&e1));
    auto launch = [&](int n) {
        switch (op) {
            case 0: hipLaunchKernelGGL(k_probe<0>, dim3(blocks), dim3(256), 0, st, sink, ticks, n, 1.0001f, 0.5f); break;
            case 1: hipLaunchKernelGGL(k_probe<1>, dim3(blocks), dim3(256), 0, st, sink, ticks, n, 1.0001f, 0.5f); break;
            case 2: hipLaunchKernelGGL(k_probe<2>, dim3(blocks), dim3(256), 0, st, sink, ticks, n, 1.0001f, 0.5f); break;
            case 4: hipLaunchKernelGGL(k_probe_mfma<false>, dim3(blocks), dim3(256), 0, st, sink, ticks, n); break;
            case 5: hipLaunchKernelGGL(k_probe_mfma<true>, dim3(blocks), dim3(256), 0, st, sink, ticks, n); break;
            case 6: hipLaunchKernelGGL(k_probe_mfma_f32<0>, dim3(blocks), dim3(256), 0, st, sink, ticks, n, 1.0001f, 0.5f); break;
            case 7: hipLaunchKernelGGL(k_probe_mfma_f32<1>, dim3(blocks), dim3(256), 0, st, sink, ticks, n, 1.0001f, 0.5f); break;
            case 8: hipLaunchKernelGGL(k_probe_mfma_f32<2>, dim3(blocks), dim3(256), 0, st, sink, ticks, n, 1.0001f, 0.5f); break;
            case 9: hipLaunchKernelGGL(k_probe<4>, dim3(blocks), dim3(256), 0, st, sink, ticks, n, 1.0001f, 0.5f); break;
            case 10: hipLaunchKernelGGL(k_probe<5>, dim3(blocks), dim3(256), 0, st, sink, ticks, n, 0.9f, 0.5f); break;
            case 11: hipLaunchKernelGGL(k_probe<6>, dim3(blocks), dim3(256), 0, st, sink, ticks, n, 0.4f, 0.5f); break;
            default: hipLaunchKernelGGL(k_probe<3>, dim3(blocks), dim3(256), 0, st, sink, ticks, n, 1.0001f, 0.5f); break;
        }
    };
    launch(8);                                            // warm-up: code object load, clocks
    SG_HIP_CHECK(hipEventRecord(e0, st));
    launch(iters);
    SG_HIP_CHECK(hipEventRecord(e1, st));
    SG_LAUNCH_CHECK("k_probe");
    SG_HIP_CHECK(hipEventSynchronize(e1));
    SG_HIP_CHECK(hipEventElapsedTime(ms_out, e0, e1));
    double sum = 0.0;
    for (int b0 = 0; b0 < blocks; b0 += 256) {
        long long h[256];
        const int n = blocks - b0 < 256 ? blocks - b0 : 256;
        SG_HIP_CHECK(hipMemcpy(h, ticks + b0, sizeof(long long) * n, hipMemcpyDeviceToHost));
        for (int k = 0; k < n; k++) sum += (double)h[k];
    }
    *ticks_per_wave_out = sum / blocks;
    *instr_per_wave_out = (double)iters * PROBE_UNROLL * PROBE_ILP;
    (void)hipEventDestroy(e0);
    (void)hipEventDestroy(e1);
    return 0;
}

}  // extern "C"
