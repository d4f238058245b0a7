/* Shared device-side types and host-side helpers of the gfx950 backend. */
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>

typedef __bf16 bf16;
typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) __bf16 bf16x4;
typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2;
typedef __attribute__((ext_vector_type(16))) float f32x16;
typedef __attribute__((ext_vector_type(4))) float f32x4;
typedef __attribute__((ext_vector_type(2))) float f32x2;
typedef __attribute__((ext_vector_type(4))) unsigned u32x4;

extern "C" {
/* Records a message for flux_hip_last_error() and returns 0. */
int flux_hip_fail(const char *fmt, ...);
/* The backend's stream (created by flux_hip_init). */
hipStream_t flux_hip_stream_handle(void);
}

#define HIP_OK(call)                                                                   \
    do {                                                                               \
        hipError_t e_ = (call);                                                        \
        if (e_ != hipSuccess)                                                          \
            return flux_hip_fail("%s failed: %s (%s:%d)", #call, hipGetErrorString(e_), \
                                 __FILE__, __LINE__);                                  \
    } while (0)

__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }
__device__ __forceinline__ float fast_rcp(float x) { return __builtin_amdgcn_rcpf(x); }
/* x * sigmoid(x) */
__device__ __forceinline__ float silu_f(float x) {
    return x * fast_rcp(1.0f + fast_exp2(-1.44269504088896341f * x));
}
