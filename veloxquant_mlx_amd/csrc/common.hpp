// Shared helpers for the gfx950 kernels: error reporting, element loads/stores.
#pragma once

#include <hip/hip_runtime.h>
#include <hip/hip_fp16.h>
#include <hip/hip_bf16.h>
#include <stdint.h>
#include <stdio.h>

#include "../../include/veloxquant_hip.h"

namespace vq {

void set_error(const char *fmt, ...);
int fail(int code, const char *fmt, ...);

#define VQ_REQUIRE(cond, code, ...)                 \
    do {                                            \
        if (!(cond)) return vq::fail(code, __VA_ARGS__); \
    } while (0)

#define VQ_HIP_CHECK_LAUNCH(name)                                                    \
    do {                                                                             \
        hipError_t e__ = hipGetLastError();                                          \
        if (e__ != hipSuccess)                                                       \
            return vq::fail(VQ_ERR_HIP, "%s: launch failed: %s", name, hipGetErrorString(e__)); \
    } while (0)

typedef _Float16 f16;
typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));
typedef _Float16 f16x4 __attribute__((ext_vector_type(4)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef unsigned short u16;

struct bf16_t { u16 bits; };

// Barrier for data that the block exchanges through LDS.  __syncthreads() is a fence as well: it also
// waits for every outstanding global access of the wave, so a loop that requests the next step's data
// and then meets a __syncthreads() waits for that data once per step.  This one waits for the wave's LDS
// accesses only; global stores that other waves of the block are to read still need __syncthreads().
__device__ __forceinline__ void lds_barrier() { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); }
// Waits until every global access of the wave has completed.  Before a loop that uses lds_barrier():
// what was requested before the loop would otherwise be waited for at the loop head in every iteration,
// and with it whatever the iteration before requested.
__device__ __forceinline__ void wait_global_accesses() { __builtin_amdgcn_s_waitcnt(0x0F70); }   // vmcnt(0)

__device__ __forceinline__ float bf16_to_f32(u16 b) { return __uint_as_float(((uint32_t)b) << 16); }
__device__ __forceinline__ u16 f32_to_bf16(float f) {
    uint32_t u = __float_as_uint(f);
    if ((u & 0x7fffffffu) > 0x7f800000u) return (u16)((u >> 16) | 0x40);  // quiet NaN
    u += 0x7fffu + ((u >> 16) & 1u);                                        // round to nearest even
    return (u16)(u >> 16);
}

template <typename T> struct Elem;
template <> struct Elem<f16> {
    static __device__ __forceinline__ float ld(const f16 *p) { return (float)*p; }
    static __device__ __forceinline__ void st(f16 *p, float v) { *p = (f16)v; }
};
template <> struct Elem<bf16_t> {
    static __device__ __forceinline__ float ld(const bf16_t *p) { return bf16_to_f32(p->bits); }
    static __device__ __forceinline__ void st(bf16_t *p, float v) { p->bits = f32_to_bf16(v); }
};
template <> struct Elem<float> {
    static __device__ __forceinline__ float ld(const float *p) { return *p; }
    static __device__ __forceinline__ void st(float *p, float v) { *p = v; }
};

// Dispatch a float element type tag (VQ_F16/VQ_BF16/VQ_F32) to a template.
#define VQ_DISPATCH_FLOAT(tag, T, ...)                                   \
    switch (tag) {                                                      \
        case VQ_F16: { using T = vq::f16; __VA_ARGS__; } break;         \
        case VQ_BF16: { using T = vq::bf16_t; __VA_ARGS__; } break;     \
        case VQ_F32: { using T = float; __VA_ARGS__; } break;           \
        default: return vq::fail(VQ_ERR_INVALID, "unsupported float dtype tag %d", (int)(tag)); \
    }

static inline bool is_float_tag(int t) { return t == VQ_F16 || t == VQ_BF16 || t == VQ_F32; }
static inline int64_t cdiv(int64_t a, int64_t b) { return (a + b - 1) / b; }

}  // namespace vq
