// Shared host/device helpers for the gfx950 kernels of libsg_hip.so.
#pragma once

#include <hip/hip_runtime.h>
#include <hip/hip_fp16.h>
#include <stdint.h>

#include <cstdarg>
#include <cstdio>
#include <string>

#include "../../include/sg_abi.h"
#include "../../include/sg_math.h"

namespace sg {

// ---- error text of the calling thread -------------------------------------
inline std::string& last_error() {
    static thread_local std::string e;
    return e;
}
inline int fail(const char* fmt, ...) {
    char buf[512];
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(buf, sizeof(buf), fmt, ap);
    va_end(ap);
    last_error() = buf;
    return 1;
}
#define SG_HIP_CHECK(expr)                                                              \
    do {                                                                                \
        hipError_t e_ = (expr);                                                         \
        if (e_ != hipSuccess) return sg::fail("%s: %s", #expr, hipGetErrorString(e_));  \
    } while (0)
#define SG_LAUNCH_CHECK(name)                                                           \
    do {                                                                                \
        hipError_t e_ = hipGetLastError();                                              \
        if (e_ != hipSuccess) return sg::fail("launch %s: %s", name, hipGetErrorString(e_)); \
    } while (0)

// ---- element load/store with the tensor's storage type ---------------------
__device__ __forceinline__ float bf16_bits_to_f(uint16_t h) { return sg_i2f((int32_t)((uint32_t)h << 16)); }
__device__ __forceinline__ uint16_t f_to_bf16_bits(float f) {
    uint32_t u = (uint32_t)sg_f2i(f);
    if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x40);
    u += 0x7fffu + ((u >> 16) & 1u);
    return (uint16_t)(u >> 16);
}
// Device buffers handed in by the caller are addressed in the global address space: a generic (flat) access also
// counts against the wait counter of LDS, so a kernel that uses both would wait for memory whenever it waits for LDS.
#define SG_GLOBAL __attribute__((address_space(1)))
template <class T>
__device__ __forceinline__ SG_GLOBAL T* gptr(T* p) { return (SG_GLOBAL T*)p; }
__device__ __forceinline__ float load_elem(const void* p, int dtype, int64_t i) {
    if (dtype == SG_F32) return ((const SG_GLOBAL float*)p)[i];
    if (dtype == SG_F16) return __half2float(__ushort_as_half(((const SG_GLOBAL uint16_t*)p)[i]));
    return bf16_bits_to_f(((const SG_GLOBAL uint16_t*)p)[i]);
}
__device__ __forceinline__ void store_elem(void* p, int dtype, int64_t i, float v) {
    if (dtype == SG_F32) ((SG_GLOBAL float*)p)[i] = v;
    else if (dtype == SG_F16) ((SG_GLOBAL uint16_t*)p)[i] = __half_as_ushort(__float2half_rn(v));
    else ((SG_GLOBAL uint16_t*)p)[i] = f_to_bf16_bits(v);
}
__device__ __forceinline__ float finite_or_zero(float v) { return sg_isfinite(v) ? v : 0.0f; }

// Read-only tables and weights are read through the constant address space: a
// wave-uniform index then becomes a scalar load (s_load_dword*), which the
// compiler will not emit for plain global pointers in a kernel that also
// stores to global memory.  Only for memory no kernel of the same launch writes.
typedef const __attribute__((address_space(4))) float* cfloat_p;
typedef const __attribute__((address_space(4))) int* cint_p;
__device__ __forceinline__ cfloat_p as_const(const float* p) { return (cfloat_p)p; }
__device__ __forceinline__ cint_p as_const(const int* p) { return (cint_p)p; }

// A zero the optimiser cannot see through, held in a scalar register.  Adding it to a weight pointer
// inside a loop keeps the loop-invariant scalar loads where they are used: hoisted out of the loop,
// a thousand of them would be spilled from SGPRs into VGPR lanes and read back with v_readlane.
__device__ __forceinline__ int opaque_zero() {
    int z = 0;
    asm volatile("" : "+s"(z));
    return z;
}

// largest i in [0, n) with prefix[i] <= x   (prefix is non-decreasing, prefix[0] == 0)
template <class P>
__device__ __forceinline__ int upper_seg(P prefix, int n, int x) {
    int lo = 0, hi = n;
    while (hi - lo > 1) {
        const int mid = (lo + hi) >> 1;
        if (prefix[mid] <= x) lo = mid; else hi = mid;
    }
    return lo;
}

inline size_t align_up(size_t x, size_t a) { return (x + a - 1) / a * a; }

// ---- small host tables into device memory through kernel arguments -----------
// A copy from pageable host memory blocks the calling thread until the stream has drained to it and cannot be
// recorded into a graph; a few KB of per-call tables travel as kernel arguments instead, UPLOAD_WORDS 32-bit words
// per launch.  dst 4-byte aligned, bytes a multiple of 4; the source is read before the call returns.
constexpr int UPLOAD_WORDS = 896;            // 3584 bytes of payload: the argument block stays below 4 KB
struct UploadChunk {
    uint32_t w[UPLOAD_WORDS];
    uint32_t* dst;
    int n;
};
static __global__ __launch_bounds__(256) void k_upload(UploadChunk c) {
    for (int i = threadIdx.x; i < c.n; i += 256) c.dst[i] = c.w[i];
}
inline int upload_words(void* dst, const void* src, size_t bytes, hipStream_t st) {
    if ((bytes & 3u) != 0 || (reinterpret_cast<uintptr_t>(dst) & 3u) != 0) return fail("upload: size and destination must be multiples of 4");
    const uint32_t* s = static_cast<const uint32_t*>(src);
    uint32_t* d = static_cast<uint32_t*>(dst);
    size_t left = bytes / 4;
    while (left > 0) {
        UploadChunk c;
        c.n = (int)(left < (size_t)UPLOAD_WORDS ? left : (size_t)UPLOAD_WORDS);
        for (int i = 0; i < c.n; i++) c.w[i] = s[i];
        c.dst = d;
        hipLaunchKernelGGL(k_upload, dim3(1), dim3(256), 0, st, c);
        SG_LAUNCH_CHECK("k_upload");
        s += c.n; d += c.n; left -= (size_t)c.n;
    }
    return 0;
}

}  // namespace sg
