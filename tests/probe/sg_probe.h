/* C interface of libsg_probe.so: an issue-rate probe of the gfx950 vector ALU and matrix cores.  A measurement aid
 * that prices the rooflines quoted for the optimizer-step kernels; it is built beside the tests, is not part of
 * libsg_hip.so and has no counterpart in the reference. */
#ifndef SG_PROBE_H_
#define SG_PROBE_H_
#include <stddef.h>
#ifdef __cplusplus
extern "C" {
#endif
/* Issue-rate probe of the fp32 vector ALU (measurement aid, no counterpart in
 * the reference): `iters` x 128 independent wave64 instructions of one kind
 * per wave (op 0 v_fma_f32, 1 v_mul_f32, 2 v_add_f32, 3 v_add_f32 with a DPP
 * operand; plain, not packed; 4 v_mfma_f32_32x32x16_bf16 on constant register
 * operands, 5 the same on pseudo-random operands: the matrix cores' own
 * ceiling and what real data makes of it through the power limit; 6
 * v_mfma_f32_32x32x1_2b_f32, 7 the same with 8 v_fma_f32 after each in the
 * same wave (the vector instructions are not counted), 8
 * v_mfma_f32_4x4x1_16b_f32: the fp32 matrix forms that are one fused
 * multiply-add per output; 9 v_fmac_f32, the accumulate form of the fma, on
 * per-lane factors; 10 op 0 with its two other operands in per-lane vector
 * registers; 11 v_fma_f32 with one scalar-register operand and three vector
 * registers: an instruction that reads a scalar register issues more slowly
 * once several waves share a SIMD) on num_cus x waves_per_simd workgroups of four
 * waves, i.e. waves_per_simd waves on every SIMD of num_cus compute units
 * when the dispatcher spreads them evenly.  Synchronises the stream.  Returns
 * the elapsed milliseconds of the launch, the shader-clock ticks a wave took
 * on average and the instructions each wave issued. */
size_t sg_probe_workspace_bytes(int num_cus, int waves_per_simd);
int sg_probe_valu(int op, int num_cus, int waves_per_simd, int iters, float* ms_out, double* ticks_per_wave_out,
                  double* instr_per_wave_out, void* workspace, size_t workspace_bytes, void* stream);

/* text of the last error raised on the calling thread */
const char* sg_probe_last_error(void);
#ifdef __cplusplus
}
#endif
#endif
