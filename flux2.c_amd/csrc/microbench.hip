/*
 * microbench.hip - what the matrix pipes of this GPU sustain with nothing else in the way: a
 * register-resident loop of independent bf16 MFMAs (no memory traffic inside the loop), for the two
 * instruction shapes and for operand data of different entropy. It is the yardstick the GEMM and
 * attention kernels are judged against besides the datasheet figure, because with operands that
 * toggle the chip reaches its power limit well below that figure. No counterpart in the reference.
 *
 * Each wave keeps a grid of accumulator blocks (4 x 4 blocks for 16x16x32, 2 x 2 for 32x32x16; 64
 * accumulator registers either way) and walks it in serpentine order, so that one operand changes
 * from one MFMA to the next, as in the GEMM kernel. The MFMAs are written as inline assembly: left
 * to the compiler's builtin, a loop with one wave per SIMD moves accumulators between the two
 * register files between the MFMAs and measures that instead.
 */
#include "common.h"
#include "../../include/flux_hip.h"
#include "../../include/flux_hip_debug.h"

#define MFMA16(acc, a, b) asm volatile("v_mfma_f32_16x16x32_bf16 %0, %1, %2, %0" : "+v"(acc) : "v"(a), "v"(b))
#define MFMA32(acc, a, b) asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, %0" : "+v"(acc) : "v"(a), "v"(b))

__device__ __forceinline__ unsigned mix(unsigned x) {
    x ^= x >> 16; x *= 0x7feb352du; x ^= x >> 15; x *= 0x846ca68bu; x ^= x >> 16;
    return x;
}

/* pattern 0: all zeros; 1: 1.0 <= x < 2.0 with a random low byte (sign and exponent fixed); 2: random bit patterns
 * with the exponent kept away from inf / nan (top exponent bit cleared) */
__device__ __forceinline__ bf16x8 operand(int pattern, unsigned seed) {
    union { bf16x8 v; unsigned u[4]; } r;
#pragma unroll
    for (int i = 0; i < 4; i++) {
        const unsigned h = mix(seed * 4u + i + 1u);
        r.u[i] = pattern == 0 ? 0u : pattern == 1 ? (0x3f803f80u | (h & 0x007f007fu)) : (h & 0xbfffbfffu);
    }
    return r.v;
}

template <int SHAPE>
__global__ __launch_bounds__(512) void mfma_peak_kernel(float *out, int iters, int pattern) {
    constexpr int G = SHAPE == 0 ? 4 : 2; /* G x G accumulator blocks */
    const unsigned id = blockIdx.x * blockDim.x + threadIdx.x;
    bf16x8 a[G], b[G];
#pragma unroll
    for (int i = 0; i < G; i++) {
        a[i] = operand(pattern, id * 16u + i);
        b[i] = operand(pattern, id * 16u + 8u + i);
    }
    float sum = 0.0f;
    if constexpr (SHAPE == 0) {
        f32x4 acc[G][G];
#pragma unroll
        for (int i = 0; i < G; i++)
#pragma unroll
            for (int j = 0; j < G; j++) acc[i][j] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
        asm volatile("s_nop 7" ::: "memory"); /* the zeroes are in place before the first MFMA reads them */
        for (int it = 0; it < iters; it++) {
#pragma unroll
            for (int k = 0; k < G * G; k++) {
                const int i = k / G, j = (i & 1) ? G - 1 - k % G : k % G;
                MFMA16(acc[i][j], a[i], b[j]);
            }
        }
        asm volatile("s_nop 15\n\ts_nop 15" ::: "memory"); /* the last results retire before they are read */
#pragma unroll
        for (int i = 0; i < G; i++)
#pragma unroll
            for (int j = 0; j < G; j++) sum += acc[i][j][0] + acc[i][j][3];
    } else {
        f32x16 acc[G][G];
#pragma unroll
        for (int i = 0; i < G; i++)
#pragma unroll
            for (int j = 0; j < G; j++)
#pragma unroll
                for (int e = 0; e < 16; e++) acc[i][j][e] = 0.0f;
        asm volatile("s_nop 7" ::: "memory");
        for (int it = 0; it < iters; it++) {
#pragma unroll
            for (int r = 0; r < 4; r++) /* 16 MFMAs per iteration, like the other shape */
#pragma unroll
                for (int k = 0; k < G * G; k++) {
                    const int i = k / G, j = (i & 1) ? G - 1 - k % G : k % G;
                    MFMA32(acc[i][j], a[i], b[j]);
                }
        }
        asm volatile("s_nop 15\n\ts_nop 15\n\ts_nop 15\n\ts_nop 15" ::: "memory");
#pragma unroll
        for (int i = 0; i < G; i++)
#pragma unroll
            for (int j = 0; j < G; j++) sum += acc[i][j][0] + acc[i][j][15];
    }
    if (sum == 12345.678f) out[id] = sum; /* keeps the accumulators alive; practically never taken */
}

/*
 * Runs the loop on every compute unit (one workgroup each, waves_per_simd = 1 or 2 waves on each of its four
 * SIMDs), `launches` times, and returns the best launch's rate in TFLOP/s in *tflops.
 * shape 0 = v_mfma_f32_16x16x32_bf16, 1 = v_mfma_f32_32x32x16_bf16; pattern 0 zeros, 1 fixed exponent with a
 * random low byte, 2 random bits.
 */
extern "C" int flux_hip_mfma_peak(int shape, int pattern, int waves_per_simd, int iters, int launches, float *tflops) {
    if (!flux_hip_available()) return 0;
    if (shape < 0 || shape > 1 || pattern < 0 || pattern > 2 || waves_per_simd < 1 || waves_per_simd > 2 || iters < 1 || iters > (1 << 22) ||
        launches < 1 || launches > 100 || !tflops)
        return flux_hip_fail("flux_hip_mfma_peak: bad argument");
    int dev = 0, cus = 0;
    HIP_OK(hipGetDevice(&dev));
    HIP_OK(hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev));
    const int threads = 256 * waves_per_simd;
    float *out = nullptr;
    HIP_OK(hipMalloc((void **)&out, (size_t)cus * threads * sizeof(float)));
    hipEvent_t e0, e1;
    HIP_OK(hipEventCreate(&e0));
    HIP_OK(hipEventCreate(&e1));
    hipStream_t st = flux_hip_stream_handle();
    float best = 1e30f;
    int ok = 1;
    for (int l = 0; l < launches + 1 && ok; l++) { /* the first launch is a warm-up */
        ok = hipEventRecord(e0, st) == hipSuccess;
        if (shape == 0) hipLaunchKernelGGL(mfma_peak_kernel<0>, dim3(cus), dim3(threads), 0, st, out, iters, pattern);
        else hipLaunchKernelGGL(mfma_peak_kernel<1>, dim3(cus), dim3(threads), 0, st, out, iters, pattern);
        ok = ok && hipGetLastError() == hipSuccess && hipEventRecord(e1, st) == hipSuccess && hipEventSynchronize(e1) == hipSuccess;
        float ms = 0.0f;
        ok = ok && hipEventElapsedTime(&ms, e0, e1) == hipSuccess;
        if (ok && l > 0 && ms < best) best = ms;
    }
    (void)hipEventDestroy(e0);
    (void)hipEventDestroy(e1);
    (void)hipFree(out);
    if (!ok) return flux_hip_fail("flux_hip_mfma_peak: launch or timing failed: %s", hipGetErrorString(hipGetLastError()));
    const double flops = (double)cus * (threads / 64) * (double)iters * 16.0 * (shape == 0 ? 16384.0 : 32768.0);
    *tflops = (float)(flops / (best * 1e-3) / 1e12);
    return 1;
}
