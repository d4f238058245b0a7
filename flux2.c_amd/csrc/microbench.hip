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
 *
 * A second loop (mfma_issue_kernel) measures what another instruction costs a lone wave when it sits between
 * that wave's MFMAs: the GEMM and attention kernels run one wave per SIMD, so whatever such an instruction keeps
 * the wave's issue slot for beyond the 16 cycles of the MFMA before it is time the matrix pipe idles.
 */
#include <stdlib.h>
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

/* ---------------------------------------------------------------------------------------
 * Cost of an instruction between a lone wave's MFMAs. Every wave runs `iters` x 16 independent MFMAs
 * (16 accumulator blocks) and behind every EVERY-th MFMA one instruction of kind MODE:
 *   0 nothing, 1 global_load_lds_dwordx4 (1 KB per wave from the workgroup's own 64 KB of a buffer, into its own LDS
 *   region), 2 ds_read_b128, 3 v_exp_f32, 4 three v_fma_f32, 5 global_load_dwordx4 followed a round later by ds_write_b128
 * and reports its cycle count (clock64 around the loop). One workgroup of four waves per compute unit.
 * --------------------------------------------------------------------------------------- */
#define MB_GLOBAL_PTR(p) ((const __attribute__((address_space(1))) void *)(p))
#define MB_LDS_PTR(p) ((__attribute__((address_space(3))) void *)(p))
template <int MODE, int EVERY>
__global__ __launch_bounds__(256) void mfma_issue_kernel(const char *buf, int iters, long long *cyc, float *sink) {
    extern __shared__ __attribute__((aligned(16))) char smem[];
    const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    f32x4 acc[16];
#pragma unroll
    for (int i = 0; i < 16; i++) acc[i] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
    bf16x8 a = operand(1, threadIdx.x), b = operand(1, threadIdx.x + 4096u);
    const char *src = buf + (size_t)blockIdx.x * 65536 + wave * 1024; /* this wave's KB of each 4 KB step */
    const unsigned voff = lane * 16;
    const char *base = src + voff;
    const unsigned lds = wave * 16384 + lane * 16;
    u32x4 r[4] = {};
    u32x4 rd = {};
    float x[4] = {0.5f, 0.25f, 0.125f, 0.75f}, y[3] = {1.0f, 2.0f, 3.0f};
    unsigned pos = 0;
    asm volatile("s_nop 7" ::: "memory");
    const long long t0 = clock64();
    for (int it = 0; it < iters; it++) {
#pragma unroll
        for (int m = 0; m < 16; m++) {
            asm volatile("v_mfma_f32_16x16x32_bf16 %0, %1, %2, %0" : "+a"(acc[m]) : "v"(a), "v"(b));
            if (m % EVERY == 0) {
                const int n = m / EVERY;
                if (MODE == 1) __builtin_amdgcn_global_load_lds(MB_GLOBAL_PTR(base + pos), MB_LDS_PTR(smem + wave * 16384 + (n & 7) * 1024), 16, 0, 0);
                if (MODE == 2) asm volatile("ds_read_b128 %0, %1" : "=v"(rd) : "v"(lds + (n & 7) * 1024) : "memory");
                if (MODE == 3) asm volatile("v_exp_f32_e32 %0, %0" : "+v"(x[n & 3]));
                if (MODE == 4) {
#pragma unroll
                    for (int e = 0; e < 3; e++) asm volatile("v_fma_f32 %0, %0, %1, %1" : "+v"(y[e]) : "v"(x[0]));
                }
                if (MODE == 5) {
                    asm volatile("s_waitcnt vmcnt(3)\n\tds_write_b128 %0, %1" ::"v"(lds + (n & 7) * 1024), "v"(r[n & 3]) : "memory");
                    /* the load as assembly as well: the wait for it is the one written above, a round later */
                    asm volatile("global_load_dwordx4 %0, %1, %2" : "=v"(r[n & 3]) : "v"(voff), "s"(src + pos) : "memory");
                }
                pos = (pos + 4096u) & 0xFFFFu;
            }
        }
        if (MODE == 2) asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    }
    asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)\n\ts_nop 15\n\ts_nop 15" ::: "memory");
    const long long t1 = clock64();
    float s = x[0] + x[1] + x[2] + x[3] + y[0] + y[1] + y[2] + (float)rd[0];
#pragma unroll
    for (int i = 0; i < 16; i++) {
        asm volatile("" : "+a"(acc[i]));
        s += acc[i][0];
    }
#pragma unroll
    for (int j = 0; j < 4; j++) s += (float)r[j][0];
    if (lane == 0) cyc[blockIdx.x * 4 + wave] = t1 - t0;
    if (s == 12345.678f) sink[0] = s;
}

template <int MODE>
static int issue_launch(int every, int cus, hipStream_t st, const char *buf, int iters, long long *cyc, float *sink) {
#define MB_CASE(E) \
    case E: { \
        auto kern = mfma_issue_kernel<MODE, E>; \
        if (hipFuncSetAttribute((const void *)kern, hipFuncAttributeMaxDynamicSharedMemorySize, 65536) != hipSuccess) return 0; \
        hipLaunchKernelGGL(kern, dim3(cus), dim3(256), 65536, st, buf, iters, cyc, sink); \
        return hipGetLastError() == hipSuccess; \
    }
    switch (every) {
        MB_CASE(1) MB_CASE(2) MB_CASE(4) MB_CASE(8) MB_CASE(16)
        default: return 0;
    }
#undef MB_CASE
}

/*
 * mode as above (0..5), every = 1, 2, 4, 8 or 16 MFMAs per interleaved instruction. Returns the average number of
 * clock cycles per MFMA over all waves in *cycles_per_mfma (16 = the matrix pipe never waits) and the core clock
 * during the run in *ghz (cycle counter against the launch's duration).
 */
extern "C" int flux_hip_mfma_issue_cost(int mode, int every, int iters, float *cycles_per_mfma, float *ghz) {
    if (!flux_hip_available()) return 0;
    if (mode < 0 || mode > 5 || iters < 1 || iters > (1 << 20) || !cycles_per_mfma || !ghz) return flux_hip_fail("flux_hip_mfma_issue_cost: bad argument");
    int dev = 0, cus = 0;
    HIP_OK(hipGetDevice(&dev));
    HIP_OK(hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev));
    char *buf = nullptr;
    long long *cyc = nullptr;
    float *sink = nullptr;
    const size_t bytes = (size_t)(cus + 1) * 65536;
    HIP_OK(hipMalloc((void **)&buf, bytes));
    HIP_OK(hipMalloc((void **)&cyc, (size_t)cus * 4 * sizeof(long long)));
    HIP_OK(hipMalloc((void **)&sink, sizeof(float)));
    hipStream_t st = flux_hip_stream_handle();
    hipEvent_t e0, e1;
    HIP_OK(hipEventCreate(&e0));
    HIP_OK(hipEventCreate(&e1));
    int ok = hipMemsetAsync(buf, 1, bytes, st) == hipSuccess;
    float best = 1e30f;
    for (int l = 0; l < 3 && ok; l++) { /* the first launch is a warm-up */
        ok = hipEventRecord(e0, st) == hipSuccess;
        switch (mode) {
            case 0: ok = ok && issue_launch<0>(every, cus, st, buf, iters, cyc, sink); break;
            case 1: ok = ok && issue_launch<1>(every, cus, st, buf, iters, cyc, sink); break;
            case 2: ok = ok && issue_launch<2>(every, cus, st, buf, iters, cyc, sink); break;
            case 3: ok = ok && issue_launch<3>(every, cus, st, buf, iters, cyc, sink); break;
            case 4: ok = ok && issue_launch<4>(every, cus, st, buf, iters, cyc, sink); break;
            default: ok = ok && issue_launch<5>(every, cus, st, buf, iters, cyc, sink); break;
        }
        ok = ok && hipEventRecord(e1, st) == hipSuccess && hipEventSynchronize(e1) == hipSuccess;
        float ms = 0.0f;
        ok = ok && hipEventElapsedTime(&ms, e0, e1) == hipSuccess;
        if (ok && l > 0 && ms < best) best = ms;
    }
    double avg = 0.0;
    if (ok) {
        long long *h = (long long *)malloc((size_t)cus * 4 * sizeof(long long));
        ok = h && hipMemcpy(h, cyc, (size_t)cus * 4 * sizeof(long long), hipMemcpyDeviceToHost) == hipSuccess;
        for (int i = 0; ok && i < cus * 4; i++) avg += (double)h[i];
        free(h);
        avg /= (double)cus * 4;
    }
    (void)hipEventDestroy(e0);
    (void)hipEventDestroy(e1);
    (void)hipFree(buf);
    (void)hipFree(cyc);
    (void)hipFree(sink);
    if (!ok) return flux_hip_fail("flux_hip_mfma_issue_cost: launch or timing failed (every must be 1, 2, 4, 8 or 16): %s", hipGetErrorString(hipGetLastError()));
    *cycles_per_mfma = (float)(avg / ((double)iters * 16.0));
    *ghz = (float)(avg / (best * 1e-3) / 1e9);
    return 1;
}
