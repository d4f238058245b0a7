/*
 * elementwise.hip - bandwidth-bound kernels of the denoising step for gfx950:
 * LayerNorm + AdaLN modulation, small-M projections (time embedding, modulation vectors),
 * layout/precision edges and the Euler / CFG latent updates.
 * All reductions are wavefront reductions (64 lanes); all global accesses are 16-byte where
 * the data allows.
 */
#include "common.h"
#include "../../include/flux_hip.h"

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
    return v;
}

/* ---------------------------------------------------------------------------------------
 * out = (1 + scale) * (x - mean) / sqrt(var + eps) + shift, biased two-pass variance
 * (reference: apply_adaln, flux_transformer.c:1021-1046). One wave per row; the row lives in
 * registers between the passes, so HBM sees one read of x and one write of out.
 * --------------------------------------------------------------------------------------- */
#define ADALN_MAX_V4 16 /* float4 per lane: rows up to 64*4*16 = 4096 columns */

/* A wave takes R rows and requests all of them before it reduces the first: with one row per wave a launch over
 * 4608 rows needs more workgroups than the GPU holds at a time, and its last few run alone. NV = float4 per lane
 * the registers are laid out for (hidden <= 256 NV; EXACT: hidden = 256 NV, no guards around the loads). */
template <int R, int NV, bool EXACT>
__global__ __launch_bounds__(256) void adaln_kernel(bf16 *__restrict__ out, int ldo, const float *__restrict__ x,
                                                    int rows, int hidden, int split,
                                                    const float *__restrict__ shift0, const float *__restrict__ scale0,
                                                    const float *__restrict__ shift1, const float *__restrict__ scale1,
                                                    float eps) {
    const int row0 = (blockIdx.x * 4 + (threadIdx.x >> 6)) * R;
    if (row0 >= rows) return;
    const int lane = threadIdx.x & 63;
    const int nv = EXACT ? NV : hidden >> 8; /* float4 per lane */
    f32x4 v[R][NV];
#pragma unroll
    for (int r = 0; r < R; r++) {
        const float *xr = x + (size_t)min(row0 + r, rows - 1) * hidden;
#pragma unroll
        for (int i = 0; i < NV; i++)
            if (i < nv) v[r][i] = *(const f32x4 *)(xr + (i * 64 + lane) * 4);
    }
#pragma unroll
    for (int r = 0; r < R; r++) {
        const int row = row0 + r;
        if (row >= rows) break;
        float s = 0.0f;
#pragma unroll
        for (int i = 0; i < NV; i++)
            if (i < nv) s += (v[r][i][0] + v[r][i][1]) + (v[r][i][2] + v[r][i][3]);
        const float mean = wave_sum(s) / (float)hidden;
        float q = 0.0f;
#pragma unroll
        for (int i = 0; i < NV; i++)
            if (i < nv) {
#pragma unroll
                for (int e = 0; e < 4; e++) { float d = v[r][i][e] - mean; q += d * d; }
            }
        const float inv = 1.0f / sqrtf(wave_sum(q) / (float)hidden + eps);
        const float *shift = row < split ? shift0 : shift1;
        const float *scale = row < split ? scale0 : scale1;
        bf16 *o = out + (size_t)row * ldo;
#pragma unroll
        for (int i = 0; i < NV; i++)
            if (i < nv) {
                const int c = (i * 64 + lane) * 4;
                f32x4 sh = *(const f32x4 *)(shift + c), sc = *(const f32x4 *)(scale + c);
                bf16x4 rr;
#pragma unroll
                for (int e = 0; e < 4; e++) rr[e] = (bf16)((1.0f + sc[e]) * ((v[r][i][e] - mean) * inv) + sh[e]);
                *(bf16x4 *)(o + c) = rr;
            }
    }
}

extern "C" int flux_hip_adaln_norm(void *out_bf16, int ldo, const float *x, int rows, int hidden, int split,
                                   const float *shift0, const float *scale0,
                                   const float *shift1, const float *scale1, float eps) {
    if (rows <= 0) return 1;
    if (hidden <= 0 || (hidden & 255) || hidden > 256 * ADALN_MAX_V4)
        return flux_hip_fail("flux_hip_adaln_norm: hidden=%d must be a multiple of 256 up to %d", hidden, 256 * ADALN_MAX_V4);
    if (!out_bf16 || !x || !shift0 || !scale0) return flux_hip_fail("flux_hip_adaln_norm: NULL argument");
    if (split < rows && (!shift1 || !scale1)) return flux_hip_fail("flux_hip_adaln_norm: second modulation missing");
    if (ldo < hidden || (ldo & 3)) return flux_hip_fail("flux_hip_adaln_norm: bad ldo=%d", ldo);
    hipStream_t st = flux_hip_stream_handle();
    if (hidden == 256 * 12)
        hipLaunchKernelGGL((adaln_kernel<2, 12, true>), dim3((rows + 7) / 8), dim3(256), 0, st, (bf16 *)out_bf16, ldo, x, rows, hidden, split, shift0,
                           scale0, shift1, scale1, eps);
    else
        hipLaunchKernelGGL((adaln_kernel<1, ADALN_MAX_V4, false>), dim3((rows + 3) / 4), dim3(256), 0, st, (bf16 *)out_bf16, ldo, x, rows, hidden, split,
                           shift0, scale0, shift1, scale1, eps);
    HIP_OK(hipGetLastError());
    return 1;
}

/* ---------------------------------------------------------------------------------------
 * Small-M projection with fp32 activations and bf16 weights:
 *   y[m, n] = sum_k f(x[m, k]) * W[n, k]
 * One wave per output feature n; the weight row is streamed once (16-byte loads) and used for
 * up to 8 rows of x at a time. Reference: the M=1 calls of flux_linear_nobias at
 * flux_transformer.c:962-968, 3024, 3231-3234, 3530.
 * --------------------------------------------------------------------------------------- */
#define GEMV_MT 8

template <int SILU>
__global__ __launch_bounds__(256) void gemv_kernel(float *__restrict__ y, const float *__restrict__ x,
                                                   const bf16 *__restrict__ W, int M, int N, int K) {
    const int n = blockIdx.x * 4 + (threadIdx.x >> 6);
    if (n >= N) return;
    const int lane = threadIdx.x & 63;
    const bf16 *w = W + (size_t)n * K;
    for (int m0 = 0; m0 < M; m0 += GEMV_MT) {
        float acc[GEMV_MT];
#pragma unroll
        for (int i = 0; i < GEMV_MT; i++) acc[i] = 0.0f;
        for (int k = lane * 8; k < K; k += 512) {
            bf16x8 wv = *(const bf16x8 *)(w + k);
            float wf[8];
#pragma unroll
            for (int e = 0; e < 8; e++) wf[e] = (float)wv[e];
#pragma unroll
            for (int i = 0; i < GEMV_MT; i++)
                if (m0 + i < M) {
                    const float *xr = x + (size_t)(m0 + i) * K + k;
                    f32x4 a = *(const f32x4 *)xr, b = *(const f32x4 *)(xr + 4);
#pragma unroll
                    for (int e = 0; e < 4; e++) {
                        float xa = a[e], xb = b[e];
                        if (SILU) { xa = silu_f(xa); xb = silu_f(xb); }
                        acc[i] += xa * wf[e] + xb * wf[4 + e];
                    }
                }
        }
#pragma unroll
        for (int i = 0; i < GEMV_MT; i++)
            if (m0 + i < M) {
                float r = wave_sum(acc[i]);
                if (lane == 0) y[(size_t)(m0 + i) * N + n] = r;
            }
    }
}

extern "C" int flux_hip_gemv(float *y, const float *x, const void *W_bf16, int M, int N, int K, int silu_input) {
    if (M <= 0 || N <= 0) return 1;
    if (K <= 0 || (K & 7)) return flux_hip_fail("flux_hip_gemv: K=%d must be a positive multiple of 8", K);
    if (!y || !x || !W_bf16) return flux_hip_fail("flux_hip_gemv: NULL argument");
    dim3 grid((N + 3) / 4), block(256);
    if (silu_input)
        hipLaunchKernelGGL(gemv_kernel<1>, grid, block, 0, flux_hip_stream_handle(), y, x, (const bf16 *)W_bf16, M, N, K);
    else
        hipLaunchKernelGGL(gemv_kernel<0>, grid, block, 0, flux_hip_stream_handle(), y, x, (const bf16 *)W_bf16, M, N, K);
    HIP_OK(hipGetLastError());
    return 1;
}

/* ---------------------------------------------------------------------------------------
 * latent [C, n] f32 (channel-major, what the sampler holds) -> tokens [n, C] bf16
 * (reference: the NCHW -> NLC loops at flux_transformer.c:3156-3161). 32x32 tiles through LDS
 * so that both the read and the write are contiguous.
 * --------------------------------------------------------------------------------------- */
__global__ __launch_bounds__(256) void latent_to_tokens_kernel(bf16 *__restrict__ tok, const float *__restrict__ lat,
                                                               int C, int n) {
    __shared__ float tile[32][33];
    const int p0 = blockIdx.x * 32, c0 = blockIdx.y * 32;
    const int tx = threadIdx.x & 31, ty = threadIdx.x >> 5;
    for (int r = ty; r < 32; r += 8) {
        int c = c0 + r, p = p0 + tx;
        tile[r][tx] = (c < C && p < n) ? lat[(size_t)c * n + p] : 0.0f;
    }
    __syncthreads();
    for (int r = ty; r < 32; r += 8) {
        int p = p0 + r, c = c0 + tx;
        if (p < n && c < C) tok[(size_t)p * C + c] = (bf16)tile[tx][r];
    }
}

extern "C" int flux_hip_latent_to_tokens(void *tok_bf16, const float *latent, int channels, int n) {
    if (n <= 0 || channels <= 0) return 1;
    if (!tok_bf16 || !latent) return flux_hip_fail("flux_hip_latent_to_tokens: NULL argument");
    hipLaunchKernelGGL(latent_to_tokens_kernel, dim3((n + 31) / 32, (channels + 31) / 32), dim3(256), 0,
                       flux_hip_stream_handle(), (bf16 *)tok_bf16, latent, channels, n);
    HIP_OK(hipGetLastError());
    return 1;
}

__global__ __launch_bounds__(256) void f32_to_bf16_kernel(bf16 *__restrict__ out, const float *__restrict__ in, size_t n) {
    size_t i = ((size_t)blockIdx.x * 256 + threadIdx.x) * 4;
    if (i + 3 < n) {
        f32x4 v = *(const f32x4 *)(in + i);
        bf16x4 r;
#pragma unroll
        for (int e = 0; e < 4; e++) r[e] = (bf16)v[e];
        *(bf16x4 *)(out + i) = r;
    } else {
        for (; i < n; i++) out[i] = (bf16)in[i];
    }
}

extern "C" int flux_hip_f32_to_bf16(void *out_bf16, const float *in, size_t n) {
    if (!n) return 1;
    if (!out_bf16 || !in) return flux_hip_fail("flux_hip_f32_to_bf16: NULL argument");
    size_t blocks = (n + 1023) / 1024;
    hipLaunchKernelGGL(f32_to_bf16_kernel, dim3((unsigned)blocks), dim3(256), 0, flux_hip_stream_handle(),
                       (bf16 *)out_bf16, in, n);
    HIP_OK(hipGetLastError());
    return 1;
}

/* ---------------------------------------------------------------------------------------
 * Latent updates on the fp32 latent (reference: flux_axpy at flux_sample.c:248 and the CFG
 * combine at flux_sample.c:496-499).
 * --------------------------------------------------------------------------------------- */
__global__ __launch_bounds__(256) void euler_kernel(float *__restrict__ z, const float *__restrict__ v, float dt, size_t n) {
    size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (i < n) z[i] += dt * v[i];
}

__global__ __launch_bounds__(256) void cfg_euler_kernel(float *__restrict__ z, const float *__restrict__ vu,
                                                        const float *__restrict__ vc, float g, float dt, size_t n) {
    size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (i < n) {
        float v = vu[i] + g * (vc[i] - vu[i]);
        z[i] += dt * v;
    }
}

/* Heun (flux_sample.c:780-796): predictor out = z + dt v1 into a second buffer, corrector
 * z += dt/2 (v1 + v2). */
__global__ __launch_bounds__(256) void axpy_out_kernel(float *__restrict__ out, const float *__restrict__ z,
                                                       const float *__restrict__ v, float dt, size_t n) {
    size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (i < n) out[i] = z[i] + dt * v[i];
}

__global__ __launch_bounds__(256) void heun_kernel(float *__restrict__ z, const float *__restrict__ v1,
                                                   const float *__restrict__ v2, float dt, size_t n) {
    size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (i < n) z[i] += 0.5f * dt * (v1[i] + v2[i]);
}

extern "C" int flux_hip_euler_predict(float *out, const float *z, const float *v, float dt, size_t n) {
    if (!n) return 1;
    if (!out || !z || !v) return flux_hip_fail("flux_hip_euler_predict: NULL argument");
    hipLaunchKernelGGL(axpy_out_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, flux_hip_stream_handle(), out, z, v, dt, n);
    HIP_OK(hipGetLastError());
    return 1;
}

extern "C" int flux_hip_heun_update(float *z, const float *v1, const float *v2, float dt, size_t n) {
    if (!n) return 1;
    if (!z || !v1 || !v2) return flux_hip_fail("flux_hip_heun_update: NULL argument");
    hipLaunchKernelGGL(heun_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, flux_hip_stream_handle(), z, v1, v2, dt, n);
    HIP_OK(hipGetLastError());
    return 1;
}

extern "C" int flux_hip_euler_update(float *z, const float *v, float dt, size_t n) {
    if (!n) return 1;
    if (!z || !v) return flux_hip_fail("flux_hip_euler_update: NULL argument");
    hipLaunchKernelGGL(euler_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, flux_hip_stream_handle(), z, v, dt, n);
    HIP_OK(hipGetLastError());
    return 1;
}

extern "C" int flux_hip_cfg_euler_update(float *z, const float *v_uncond, const float *v_cond, float guidance,
                                         float dt, size_t n) {
    if (!n) return 1;
    if (!z || !v_uncond || !v_cond) return flux_hip_fail("flux_hip_cfg_euler_update: NULL argument");
    hipLaunchKernelGGL(cfg_euler_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, flux_hip_stream_handle(),
                       z, v_uncond, v_cond, guidance, dt, n);
    HIP_OK(hipGetLastError());
    return 1;
}
