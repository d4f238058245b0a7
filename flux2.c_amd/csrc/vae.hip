/*
 * vae.hip - the memory-bound kernels of the VAE decoder and encoder (reference: flux_vae_decode,
 * flux_vae.c:690-837; flux_vae_encode, flux_vae.c:320-443); their convolutions and attention
 * products run as MFMA GEMMs (gemm.hip).
 *
 * Images are channels-last with a one-pixel zero border: position p = y * Wp + x over the
 * (H+2) x (W+2) grid, channels contiguous. That makes a 3x3 convolution one GEMM whose K steps
 * read the same rows shifted by a constant (flux_hip_conv), and every kernel here keeps the
 * border at zero so that the next convolution sees its padding. The residual stream is fp32;
 * what feeds an MFMA is bf16.
 */
#include "common.h"
#include "../../include/flux_hip.h"
#include <math.h>

#define LAUNCH_OK(what)                                                                         \
    do {                                                                                        \
        hipError_t e_ = hipGetLastError();                                                      \
        if (e_ != hipSuccess) return flux_hip_fail("%s launch failed: %s", what, hipGetErrorString(e_)); \
    } while (0)

__device__ __forceinline__ bool interior(int p, int hp, int wp) {
    const int y = p / wp, x = p - y * wp;
    return y >= 1 && y < hp - 1 && x >= 1 && x < wp - 1;
}

/* latent [128, h, w] fp32 -> x * sqrt(var + eps) + mean per latent channel (flux_vae.c:718-728),
 * 2x2 unpatchify to 32 channels at (2h, 2w) (flux_kernels.c:1067-1097), 1x1 post-quant
 * convolution 32 -> 32 (flux_vae.c:739-741); written as bf16 [Hp*Wp, 64] with channels 32..63
 * zero (the first 3x3 convolution wants a multiple of 64 input channels). One workgroup of 64
 * threads per position. */
__global__ __launch_bounds__(64) void vae_latent_kernel(bf16 *__restrict__ out, const float *__restrict__ latent,
                                                        const float *__restrict__ bn_mean, const float *__restrict__ bn_var,
                                                        const float *__restrict__ pq_w, const float *__restrict__ pq_b,
                                                        int h, int w, float eps) {
    const int hp = 2 * h + 2, wp = 2 * w + 2;
    const int p = blockIdx.x, c = threadIdx.x;
    const int y = p / wp, x = p - y * wp;
    float v = 0.0f;
    if (c < 32 && y >= 1 && y < hp - 1 && x >= 1 && x < wp - 1) {
        const int ph = (y - 1) >> 1, pi = (y - 1) & 1, pw = (x - 1) >> 1, pj = (x - 1) & 1;
        v = pq_b[c];
        for (int ci = 0; ci < 32; ci++) {
            const int lc = ci * 4 + pi * 2 + pj;
            const float z = latent[((size_t)lc * h + ph) * w + pw] * sqrtf(bn_var[lc] + eps) + bn_mean[lc];
            v += pq_w[c * 32 + ci] * z;
        }
    }
    out[(size_t)p * 64 + c] = (bf16)v;
}

/* ---- group norm (flux_group_norm, flux_kernels.c:511-553): 32 groups of C/32 adjacent channels,
 * statistics over the whole image. Three kernels: per-block partial sums, their combination in
 * double precision, and the normalisation itself. Border positions hold zeros and add nothing
 * to the sums; the element count is the interior's. ---- */
#define GN_ROWS 256 /* positions per workgroup */

/* p / wp for p < 2^22, wp < 2^12 through a multiplication: magic = ceil(2^40 / wp) */
__device__ __forceinline__ int div_wp(int p, unsigned long long magic) { return (int)(((unsigned long long)p * magic) >> 40); }

__device__ __forceinline__ f32x4 load_quad(const float *p) { return *(const f32x4 *)p; }
__device__ __forceinline__ f32x4 load_quad(const bf16 *p) {
    const bf16x4 v = *(const bf16x4 *)p;
    f32x4 o;
#pragma unroll
    for (int e = 0; e < 4; e++) o[e] = (float)v[e];
    return o;
}

/* A workgroup covers GN_ROWS positions: thread (r0, q) walks rows r0, r0 + rpi, ... of quad q
 * (4 adjacent channels, always inside one group), four rows per trip so that four loads are in
 * flight. */
template <typename T>
__global__ __launch_bounds__(256) void gn_partial_kernel(float *__restrict__ partial, const T *__restrict__ x, int rows, int C) {
    __shared__ float sh[256][2];
    const int quads = C >> 2, rpi = 256 / quads; /* C is 128, 256 or 512: 32, 64 or 128 quads */
    const int q = threadIdx.x % quads, r0 = threadIdx.x / quads;
    const int row_begin = blockIdx.x * GN_ROWS, row_end = min(rows, row_begin + GN_ROWS);
    float s = 0.0f, ss = 0.0f;
    const T *src = x + q * 4;
    int r = row_begin + r0;
    for (; r + 3 * rpi < row_end; r += 4 * rpi) {
        f32x4 v[4];
#pragma unroll
        for (int k = 0; k < 4; k++) v[k] = load_quad(src + (size_t)(r + k * rpi) * C);
#pragma unroll
        for (int k = 0; k < 4; k++)
#pragma unroll
            for (int e = 0; e < 4; e++) { s += v[k][e]; ss += v[k][e] * v[k][e]; }
    }
    for (; r < row_end; r += rpi) {
        const f32x4 v = load_quad(src + (size_t)r * C);
#pragma unroll
        for (int e = 0; e < 4; e++) { s += v[e]; ss += v[e] * v[e]; }
    }
    sh[threadIdx.x][0] = s;
    sh[threadIdx.x][1] = ss;
    __syncthreads();
    if (threadIdx.x < 32) {
        /* group g owns quads [g * qpg, (g+1) * qpg) of every thread row; fixed summation order */
        const int g = threadIdx.x, qpg = quads >> 5;
        float a = 0.0f, b = 0.0f;
        for (int rr = 0; rr < rpi; rr++)
            for (int k = 0; k < qpg; k++) {
                a += sh[rr * quads + g * qpg + k][0];
                b += sh[rr * quads + g * qpg + k][1];
            }
        partial[((size_t)blockIdx.x * 32 + g) * 2 + 0] = a;
        partial[((size_t)blockIdx.x * 32 + g) * 2 + 1] = b;
    }
}

/* one workgroup per group: mean and 1/sqrt(var + eps) with the biased variance */
__global__ __launch_bounds__(256) void gn_finalize_kernel(float *__restrict__ stats, const float *__restrict__ partial, int nblocks,
                                                          double count, float eps) {
    __shared__ double sh[256][2];
    const int g = blockIdx.x;
    double a = 0.0, b = 0.0;
    for (int i = threadIdx.x; i < nblocks; i += 256) {
        a += (double)partial[((size_t)i * 32 + g) * 2 + 0];
        b += (double)partial[((size_t)i * 32 + g) * 2 + 1];
    }
    sh[threadIdx.x][0] = a;
    sh[threadIdx.x][1] = b;
    __syncthreads();
    for (int s = 128; s > 0; s >>= 1) {
        if (threadIdx.x < s) {
            sh[threadIdx.x][0] += sh[threadIdx.x + s][0];
            sh[threadIdx.x][1] += sh[threadIdx.x + s][1];
        }
        __syncthreads();
    }
    if (threadIdx.x == 0) {
        const double mean = sh[0][0] / count;
        double var = sh[0][1] / count - mean * mean;
        if (var < 0.0) var = 0.0;
        stats[g * 2 + 0] = (float)mean;
        stats[g * 2 + 1] = (float)(1.0 / sqrt(var + (double)eps));
    }
}

/* First stage when the sums come from convolution epilogues (flux_hip_conv_stats): conv
 * [prows][C/4][2] holds one (sum, sum of squares) per row-tile half and 4-channel quad. Each
 * workgroup folds a contiguous range of those rows into per-group sums, in the layout the
 * finalize kernel reads. Same thread-to-quad map as the partial-sum pass: coalesced reads. */
__global__ __launch_bounds__(256) void gn_fold_quads_kernel(float *__restrict__ partial, const float *__restrict__ conv, int prows, int C) {
    __shared__ float sh[256][2];
    const int quads = C >> 2, rpi = 256 / quads;
    const int q = threadIdx.x % quads, r0 = threadIdx.x / quads;
    const int per = (prows + gridDim.x - 1) / gridDim.x;
    const int row_begin = blockIdx.x * per, row_end = min(prows, row_begin + per);
    float s = 0.0f, ss = 0.0f;
    for (int r = row_begin + r0; r < row_end; r += rpi) {
        const f32x2 v = *(const f32x2 *)(conv + ((size_t)r * quads + q) * 2);
        s += v[0];
        ss += v[1];
    }
    sh[threadIdx.x][0] = s;
    sh[threadIdx.x][1] = ss;
    __syncthreads();
    if (threadIdx.x < 32) {
        const int g = threadIdx.x, qpg = quads >> 5;
        float a = 0.0f, b = 0.0f;
        for (int rr = 0; rr < rpi; rr++)
            for (int k = 0; k < qpg; k++) {
                a += sh[rr * quads + g * qpg + k][0];
                b += sh[rr * quads + g * qpg + k][1];
            }
        partial[((size_t)blockIdx.x * 32 + g) * 2 + 0] = a;
        partial[((size_t)blockIdx.x * 32 + g) * 2 + 1] = b;
    }
}

/* out bf16 = [swish](gamma * (x - mean) * rstd + beta), zeros on the border; raw (optional)
 * receives x itself as bf16, the input of a residual block's 1x1 shortcut convolution. Same
 * thread-to-data map as the partial-sum pass. */
template <typename T>
__global__ __launch_bounds__(256) void gn_apply_kernel(bf16 *__restrict__ out, bf16 *__restrict__ raw, const T *__restrict__ x,
                                                       const float *__restrict__ stats, const float *__restrict__ gamma,
                                                       const float *__restrict__ beta, int rows, int C, int hp, int wp,
                                                       unsigned long long magic, int swish) {
    const int quads = C >> 2, rpi = 256 / quads;
    const int q = threadIdx.x % quads, r0 = threadIdx.x / quads;
    const int row_begin = blockIdx.x * GN_ROWS, row_end = min(rows, row_begin + GN_ROWS);
    const int g = (q * 4) / (C >> 5);
    const float mean = stats[g * 2], rstd = stats[g * 2 + 1];
    const f32x4 gm = *(const f32x4 *)(gamma + q * 4), bt = *(const f32x4 *)(beta + q * 4);
    f32x4 sc, sh;
#pragma unroll
    for (int e = 0; e < 4; e++) { sc[e] = gm[e] * rstd; sh[e] = bt[e] - mean * sc[e]; }
    auto one = [&](int r, const f32x4 &v) {
        const int y = div_wp(r, magic), xx = r - y * wp;
        const bool in = y >= 1 && y < hp - 1 && xx >= 1 && xx < wp - 1;
        bf16x4 o;
#pragma unroll
        for (int e = 0; e < 4; e++) {
            float t = v[e] * sc[e] + sh[e];
            if (swish) t = silu_f(t);
            o[e] = (bf16)(in ? t : 0.0f);
        }
        *(bf16x4 *)(out + (size_t)r * C + q * 4) = o;
        if (raw) {
            bf16x4 rw;
#pragma unroll
            for (int e = 0; e < 4; e++) rw[e] = (bf16)v[e];
            *(bf16x4 *)(raw + (size_t)r * C + q * 4) = rw;
        }
    };
    const T *src = x + q * 4;
    int r = row_begin + r0;
    for (; r + 3 * rpi < row_end; r += 4 * rpi) {
        f32x4 v[4];
#pragma unroll
        for (int k = 0; k < 4; k++) v[k] = load_quad(src + (size_t)(r + k * rpi) * C);
#pragma unroll
        for (int k = 0; k < 4; k++) one(r + k * rpi, v[k]);
    }
    for (; r < row_end; r += rpi) one(r, load_quad(src + (size_t)r * C));
}

/* nearest-neighbour 2x upsample (flux_upsample_nearest, flux_kernels.c:1017-1036): fp32
 * [hp*wp, C] -> bf16 [(2H+2)*(2W+2), C] with a fresh zero border */
__global__ __launch_bounds__(256) void vae_upsample_kernel(bf16 *__restrict__ out, const float *__restrict__ x, int hp, int wp, int C) {
    const int quads = C >> 2;
    const int H2 = 2 * (hp - 2), W2 = 2 * (wp - 2), hp2 = H2 + 2, wp2 = W2 + 2;
    const size_t idx = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (idx >= (size_t)hp2 * wp2 * quads) return;
    const int p = (int)(idx / quads), q = (int)(idx - (size_t)p * quads);
    const int y = p / wp2, xx = p - y * wp2;
    bf16x4 o = {(bf16)0.0f, (bf16)0.0f, (bf16)0.0f, (bf16)0.0f};
    if (y >= 1 && y <= H2 && xx >= 1 && xx <= W2) {
        const int sy = 1 + ((y - 1) >> 1), sx = 1 + ((xx - 1) >> 1);
        const f32x4 v = *(const f32x4 *)(x + ((size_t)sy * wp + sx) * C + q * 4);
#pragma unroll
        for (int e = 0; e < 4; e++) o[e] = (bf16)v[e];
    }
    *(bf16x4 *)(out + (size_t)p * C + q * 4) = o;
}

/* ---- encoder side (flux_vae_encode, flux_vae.c:320-443) ---- */

/* image [3, H, W] fp32 -> the 3x3 neighbourhood of every position as one row of 64 bf16:
 * element (ky*3 + kx)*3 + c = img[c, y-1+ky, x-1+kx] (zero outside the image), elements 27..63
 * zero. The first convolution (3 -> 128 channels, flux_vae.c:336-338) is then a GEMM with K = 64
 * over these rows. 32 positions per workgroup of 256 threads. */
__global__ __launch_bounds__(256) void vae_image_in_kernel(bf16 *__restrict__ out, const float *__restrict__ img, int H, int W) {
    const int wp = W + 2, rows = (H + 2) * wp;
    const int p = blockIdx.x * 32 + (threadIdx.x >> 3), k0 = (threadIdx.x & 7) * 8; /* eight elements (16 bytes) per thread */
    if (p >= rows) return;
    const int py = p / wp, px = p - py * wp;
    bf16x8 o;
#pragma unroll
    for (int e = 0; e < 8; e++) {
        const int k = k0 + e;
        float v = 0.0f;
        if (k < 27) {
            const int tap = k / 3, c = k - tap * 3, ky = tap / 3, kx = tap - ky * 3;
            const int y = py - 2 + ky, x = px - 2 + kx; /* image coordinates: bordered position minus 1, tap offset minus 1 */
            if (y >= 0 && y < H && x >= 0 && x < W) v = img[((size_t)c * H + y) * W + x];
        }
        o[e] = (bf16)v;
    }
    *(bf16x8 *)(out + (size_t)p * 64 + k0) = o;
}

/* The downsampling step (flux_vae.c:363-377: one row of zeros below and one column on the right,
 * then a 3x3 convolution with stride 2): fp32 [hp*wp, C] -> bf16 [hp2*wp2, 9*C] over the bordered
 * half-size grid, row (y', x') holding in[2(y'-1)+ky, 2(x'-1)+kx] for the nine taps, in the K order
 * of flux_hip_conv's weights ([C/64 chunks][9 taps][64 channels]), so that the convolution is a
 * plain GEMM with K = 9*C over these rows. The input's own zero border
 * supplies the padding: the furthest row read is its bottom border. Border rows of the output
 * are zero. One thread per (position, tap, 4 channels). */
__global__ __launch_bounds__(256) void vae_downsample_gather_kernel(bf16 *__restrict__ out, const float *__restrict__ x, int hp, int wp, int C) {
    const int quads = C >> 2;
    const int H2 = (hp - 2) >> 1, W2 = (wp - 2) >> 1, hp2 = H2 + 2, wp2 = W2 + 2;
    const size_t idx = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (idx >= (size_t)hp2 * wp2 * 9 * quads) return;
    const int q = (int)(idx % quads);
    const size_t pt = idx / quads;
    const int tap = (int)(pt % 9), p = (int)(pt / 9);
    const int y = p / wp2, xx = p - y * wp2;
    bf16x4 o = {(bf16)0.0f, (bf16)0.0f, (bf16)0.0f, (bf16)0.0f};
    if (y >= 1 && y <= H2 && xx >= 1 && xx <= W2) {
        const int ky = tap / 3, kx = tap - ky * 3;
        const int sy = 2 * (y - 1) + ky + 1, sx = 2 * (xx - 1) + kx + 1; /* bordered input coordinates, at most hp-1 / wp-1 */
        const f32x4 v = *(const f32x4 *)(x + ((size_t)sy * wp + sx) * C + q * 4);
#pragma unroll
        for (int e = 0; e < 4; e++) o[e] = (bf16)v[e];
    }
    const int c = q * 4;
    *(bf16x4 *)(out + (size_t)p * 9 * C + ((c >> 6) * 9 + tap) * 64 + (c & 63)) = o;
}

/* Output of the quant convolution, fp32 [(2h+2)*(2w+2), ldx] (channels 0..31 = the posterior's
 * mean, flux_vae.c:411-424) -> 2x2 patchify to 128 channels (flux_kernels.c:1038-1065) ->
 * (v - running_mean) / sqrt(running_var + eps) (flux_kernels.c:555-575) -> latent [128, h, w]. */
__global__ __launch_bounds__(256) void vae_latent_out_kernel(float *__restrict__ latent, const float *__restrict__ x, int ldx,
                                                             const float *__restrict__ bn_mean, const float *__restrict__ bn_var, int h, int w,
                                                             float eps) {
    const int idx = blockIdx.x * 256 + threadIdx.x;
    if (idx >= 128 * h * w) return;
    const int lc = idx / (h * w), r = idx - lc * (h * w), ph = r / w, pw = r - ph * w;
    const int c = lc >> 2, pi = (lc >> 1) & 1, pj = lc & 1, wp = 2 * w + 2;
    const float v = x[((size_t)(2 * ph + pi + 1) * wp + (2 * pw + pj + 1)) * ldx + c];
    latent[idx] = (v - bn_mean[lc]) / sqrtf(bn_var[lc] + eps);
}

/* ---- attention over all positions with one head (attnblock_forward, flux_vae.c:223-313).
 * Scores are materialised, as in the reference: S = q k^T (GEMM), P = softmax(S * scale + bias)
 * (below), O = P v (GEMM against v^T). Keys run over the bordered grid plus padding up to a
 * multiple of 128; key_bias is 0 for real pixels and -inf for border and padding columns. ---- */
__global__ __launch_bounds__(256) void vae_key_bias_kernel(float *__restrict__ bias, int n, int rows, int hp, int wp) {
    const int i = blockIdx.x * 256 + threadIdx.x;
    if (i >= n) return;
    bias[i] = (i < rows && interior(i, hp, wp)) ? 0.0f : -INFINITY;
}

__global__ __launch_bounds__(256) void vae_softmax_kernel(bf16 *__restrict__ P, const float *__restrict__ S, const float *__restrict__ key_bias,
                                                          int ld, float scale) {
    __shared__ float red[4];
    const float *s = S + (size_t)blockIdx.x * ld;
    bf16 *p = P + (size_t)blockIdx.x * ld;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    float mx = -INFINITY;
    for (int i = threadIdx.x * 4; i < ld; i += 1024) {
        const f32x4 v = *(const f32x4 *)(s + i), kb = *(const f32x4 *)(key_bias + i);
#pragma unroll
        for (int e = 0; e < 4; e++) mx = fmaxf(mx, v[e] * scale + kb[e]);
    }
    for (int o = 32; o > 0; o >>= 1) mx = fmaxf(mx, __shfl_xor(mx, o));
    if (lane == 0) red[wave] = mx;
    __syncthreads();
    mx = fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3]));
    __syncthreads();
    float sum = 0.0f;
    for (int i = threadIdx.x * 4; i < ld; i += 1024) {
        const f32x4 v = *(const f32x4 *)(s + i), kb = *(const f32x4 *)(key_bias + i);
#pragma unroll
        for (int e = 0; e < 4; e++) sum += __expf(v[e] * scale + kb[e] - mx);
    }
    for (int o = 32; o > 0; o >>= 1) sum += __shfl_xor(sum, o);
    if (lane == 0) red[wave] = sum;
    __syncthreads();
    const float inv = 1.0f / (red[0] + red[1] + red[2] + red[3]);
    for (int i = threadIdx.x * 4; i < ld; i += 1024) {
        const f32x4 v = *(const f32x4 *)(s + i), kb = *(const f32x4 *)(key_bias + i);
        bf16x4 o;
#pragma unroll
        for (int e = 0; e < 4; e++) o[e] = (bf16)(__expf(v[e] * scale + kb[e] - mx) * inv);
        *(bf16x4 *)(p + i) = o;
    }
}

/* The same for rows of up to 1024 * SOFTMAX_REG_V4 * 4 columns (1024x1024 images have 17024), with
 * the row held in registers between the three steps: S is read once. */
#define SOFTMAX_REG_V4 20
__global__ __launch_bounds__(256) void vae_softmax_reg_kernel(bf16 *__restrict__ P, const float *__restrict__ S, const float *__restrict__ key_bias,
                                                              int ld, float scale) {
    __shared__ float red[4];
    const float *s = S + (size_t)blockIdx.x * ld;
    bf16 *p = P + (size_t)blockIdx.x * ld;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    f32x4 v[SOFTMAX_REG_V4];
    float mx = -INFINITY;
#pragma unroll
    for (int i = 0; i < SOFTMAX_REG_V4; i++) {
        const int c = (i * 256 + threadIdx.x) * 4;
        if (c < ld) {
            const f32x4 t = *(const f32x4 *)(s + c), kb = *(const f32x4 *)(key_bias + c);
#pragma unroll
            for (int e = 0; e < 4; e++) { v[i][e] = t[e] * scale + kb[e]; mx = fmaxf(mx, v[i][e]); }
        }
    }
    for (int o = 32; o > 0; o >>= 1) mx = fmaxf(mx, __shfl_xor(mx, o));
    if (lane == 0) red[wave] = mx;
    __syncthreads();
    mx = fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3]));
    __syncthreads();
    float sum = 0.0f;
#pragma unroll
    for (int i = 0; i < SOFTMAX_REG_V4; i++)
        if ((i * 256 + threadIdx.x) * 4 < ld) {
#pragma unroll
            for (int e = 0; e < 4; e++) { v[i][e] = __expf(v[i][e] - mx); sum += v[i][e]; }
        }
    for (int o = 32; o > 0; o >>= 1) sum += __shfl_xor(sum, o);
    if (lane == 0) red[wave] = sum;
    __syncthreads();
    const float inv = 1.0f / (red[0] + red[1] + red[2] + red[3]);
#pragma unroll
    for (int i = 0; i < SOFTMAX_REG_V4; i++) {
        const int c = (i * 256 + threadIdx.x) * 4;
        if (c < ld) {
            bf16x4 o;
#pragma unroll
            for (int e = 0; e < 4; e++) o[e] = (bf16)(v[i][e] * inv);
            *(bf16x4 *)(p + c) = o;
        }
    }
}

/* vt[c][j] = v[j][c] for j < rows, 0 for rows <= j < ld: the value matrix as the "weight" operand
 * of the second attention GEMM. 64 x 64 tiles through LDS. */
__global__ __launch_bounds__(256) void vae_transpose_kernel(bf16 *__restrict__ vt, int ld, const bf16 *__restrict__ v, int ldv, int rows) {
    __shared__ bf16 tile[64][66];
    const int j0 = blockIdx.x * 64, c0 = blockIdx.y * 64;
    for (int i = threadIdx.x; i < 64 * 64; i += 256) {
        const int jj = i >> 6, cc = i & 63;
        tile[jj][cc] = (j0 + jj < rows) ? v[(size_t)(j0 + jj) * ldv + c0 + cc] : (bf16)0.0f;
    }
    __syncthreads();
    for (int i = threadIdx.x; i < 64 * 64; i += 256) {
        const int cc = i >> 6, jj = i & 63;
        if (j0 + jj < ld) vt[(size_t)(c0 + cc) * ld + j0 + jj] = tile[jj][cc];
    }
}

/* decoder output fp32 [hp*wp, ldx] (channels 0..2 used) -> image: 8-bit [H, W, 3] with the
 * reference's conversion (v + 1) * 0.5 * 255, clamped, truncated (flux_vae.c:820-833), and
 * optionally the unquantised values as [3, H, W] */
__global__ __launch_bounds__(256) void vae_image_kernel(uint8_t *__restrict__ rgb, float *__restrict__ rgb_f32, const float *__restrict__ x,
                                                        int ldx, int H, int W) {
    const int i = blockIdx.x * 256 + threadIdx.x;
    if (i >= H * W) return;
    const int y = i / W, xx = i - y * W;
    const float *src = x + ((size_t)(y + 1) * (W + 2) + xx + 1) * ldx;
#pragma unroll
    for (int c = 0; c < 3; c++) {
        const float v = src[c];
        float val = (v + 1.0f) * 0.5f * 255.0f;
        val = val < 0.0f ? 0.0f : val > 255.0f ? 255.0f : val;
        if (rgb) rgb[(size_t)i * 3 + c] = (uint8_t)val;
        if (rgb_f32) rgb_f32[(size_t)c * H * W + i] = v;
    }
}

/* ------------------------------------------------------------------ host entry points */

extern "C" int flux_hip_vae_latent_in(void *out_bf16, const float *latent, const float *bn_mean, const float *bn_var,
                                      const float *pq_w, const float *pq_b, int h, int w, float eps) {
    if (h <= 0 || w <= 0) return flux_hip_fail("flux_hip_vae_latent_in: bad size %d x %d", h, w);
    const int positions = (2 * h + 2) * (2 * w + 2);
    hipLaunchKernelGGL(vae_latent_kernel, dim3(positions), dim3(64), 0, flux_hip_stream_handle(), (bf16 *)out_bf16, latent, bn_mean, bn_var,
                       pq_w, pq_b, h, w, eps);
    LAUNCH_OK("vae_latent_kernel");
    return 1;
}

template <typename T>
static int group_norm_run(void *out_bf16, void *raw_bf16, const T *x, const float *gamma, const float *beta, float *scratch, int hp, int wp,
                          int C, float eps, int swish, const float *conv_stats, int conv_stats_rows) {
    const int rows = hp * wp, nblocks = (rows + GN_ROWS - 1) / GN_ROWS;
    float *partial = scratch + 64, *stats = scratch;
    hipStream_t st = flux_hip_stream_handle();
    const double count = (double)(hp - 2) * (wp - 2) * (C / 32);
    if (conv_stats) {
        const int rpi = 256 / (C / 4);
        int nb = (conv_stats_rows + 8 * rpi - 1) / (8 * rpi); /* about eight trips per thread, at most as many workgroups as the scratch has rows */
        nb = nb < 1 ? 1 : nb > nblocks ? nblocks : nb > 256 ? 256 : nb;
        hipLaunchKernelGGL(gn_fold_quads_kernel, dim3(nb), dim3(256), 0, st, partial, conv_stats, conv_stats_rows, C);
        LAUNCH_OK("gn_fold_quads_kernel");
        hipLaunchKernelGGL(gn_finalize_kernel, dim3(32), dim3(256), 0, st, stats, partial, nb, count, eps);
        LAUNCH_OK("gn_finalize_kernel");
    } else {
        hipLaunchKernelGGL(gn_partial_kernel<T>, dim3(nblocks), dim3(256), 0, st, partial, x, rows, C);
        LAUNCH_OK("gn_partial_kernel");
        hipLaunchKernelGGL(gn_finalize_kernel, dim3(32), dim3(256), 0, st, stats, partial, nblocks, count, eps);
        LAUNCH_OK("gn_finalize_kernel");
    }
    const unsigned long long magic = ((1ull << 40) + (unsigned)wp - 1) / (unsigned)wp;
    hipLaunchKernelGGL(gn_apply_kernel<T>, dim3(nblocks), dim3(256), 0, st, (bf16 *)out_bf16, (bf16 *)raw_bf16, x, stats, gamma, beta, rows, C, hp,
                       wp, magic, swish);
    LAUNCH_OK("gn_apply_kernel");
    return 1;
}

extern "C" int flux_hip_group_norm_stats(void *out_bf16, void *raw_bf16, const void *x, int x_is_bf16, const float *gamma, const float *beta,
                                         float *scratch, int hp, int wp, int C, float eps, int swish, const float *conv_stats,
                                         int conv_stats_rows) {
    if (C != 128 && C != 256 && C != 512) return flux_hip_fail("flux_hip_group_norm: C=%d (128, 256 or 512)", C);
    if (hp < 3 || wp < 3 || wp >= 4096 || (long long)hp * wp >= (1 << 22)) return flux_hip_fail("flux_hip_group_norm: bad image %d x %d", hp, wp);
    if (conv_stats && conv_stats_rows <= 0) return flux_hip_fail("flux_hip_group_norm_stats: conv_stats_rows=%d", conv_stats_rows);
    return x_is_bf16 ? group_norm_run(out_bf16, raw_bf16, (const bf16 *)x, gamma, beta, scratch, hp, wp, C, eps, swish, conv_stats, conv_stats_rows)
                     : group_norm_run(out_bf16, raw_bf16, (const float *)x, gamma, beta, scratch, hp, wp, C, eps, swish, conv_stats, conv_stats_rows);
}

extern "C" int flux_hip_group_norm(void *out_bf16, void *raw_bf16, const void *x, int x_is_bf16, const float *gamma, const float *beta,
                                   float *scratch, int hp, int wp, int C, float eps, int swish) {
    return flux_hip_group_norm_stats(out_bf16, raw_bf16, x, x_is_bf16, gamma, beta, scratch, hp, wp, C, eps, swish, nullptr, 0);
}

extern "C" size_t flux_hip_group_norm_scratch_floats(int hp, int wp) {
    return 64 + (size_t)((hp * wp + GN_ROWS - 1) / GN_ROWS) * 64;
}

extern "C" int flux_hip_upsample2x(void *out_bf16, const float *x, int hp, int wp, int C) {
    if (C <= 0 || (C & 3) || hp < 3 || wp < 3) return flux_hip_fail("flux_hip_upsample2x: bad shape");
    const size_t total = (size_t)(2 * (hp - 2) + 2) * (2 * (wp - 2) + 2) * (C / 4);
    hipLaunchKernelGGL(vae_upsample_kernel, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, flux_hip_stream_handle(), (bf16 *)out_bf16, x, hp,
                       wp, C);
    LAUNCH_OK("vae_upsample_kernel");
    return 1;
}

extern "C" int flux_hip_vae_image_in(void *out_bf16, const float *img, int H, int W) {
    if (H <= 0 || W <= 0) return flux_hip_fail("flux_hip_vae_image_in: bad shape");
    const int rows = (H + 2) * (W + 2);
    hipLaunchKernelGGL(vae_image_in_kernel, dim3((rows + 31) / 32), dim3(256), 0, flux_hip_stream_handle(), (bf16 *)out_bf16, img, H, W);
    LAUNCH_OK("vae_image_in_kernel");
    return 1;
}

extern "C" int flux_hip_downsample_gather(void *out_bf16, const float *x, int hp, int wp, int C) {
    if (C <= 0 || (C & 3) || hp < 4 || wp < 4 || ((hp | wp) & 1)) return flux_hip_fail("flux_hip_downsample_gather: bad shape (the image must have even sides)");
    const size_t total = (size_t)((hp - 2) / 2 + 2) * ((wp - 2) / 2 + 2) * 9 * (C / 4);
    hipLaunchKernelGGL(vae_downsample_gather_kernel, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, flux_hip_stream_handle(), (bf16 *)out_bf16,
                       x, hp, wp, C);
    LAUNCH_OK("vae_downsample_gather_kernel");
    return 1;
}

extern "C" int flux_hip_vae_latent_out(float *latent, const float *x, int ldx, const float *bn_mean, const float *bn_var, int h, int w, float eps) {
    if (h <= 0 || w <= 0 || ldx < 32) return flux_hip_fail("flux_hip_vae_latent_out: bad shape");
    hipLaunchKernelGGL(vae_latent_out_kernel, dim3((128 * h * w + 255) / 256), dim3(256), 0, flux_hip_stream_handle(), latent, x, ldx, bn_mean,
                       bn_var, h, w, eps);
    LAUNCH_OK("vae_latent_out_kernel");
    return 1;
}

extern "C" int flux_hip_vae_key_bias(float *bias, int n, int hp, int wp) {
    hipLaunchKernelGGL(vae_key_bias_kernel, dim3((n + 255) / 256), dim3(256), 0, flux_hip_stream_handle(), bias, n, hp * wp, hp, wp);
    LAUNCH_OK("vae_key_bias_kernel");
    return 1;
}

extern "C" int flux_hip_softmax_rows(void *p_bf16, const float *s, const float *key_bias, int rows, int ld, float scale) {
    if (rows <= 0 || ld <= 0 || (ld & 3)) return flux_hip_fail("flux_hip_softmax_rows: bad shape %d x %d", rows, ld);
    if (ld <= 1024 * SOFTMAX_REG_V4)
        hipLaunchKernelGGL(vae_softmax_reg_kernel, dim3(rows), dim3(256), 0, flux_hip_stream_handle(), (bf16 *)p_bf16, s, key_bias, ld, scale);
    else
        hipLaunchKernelGGL(vae_softmax_kernel, dim3(rows), dim3(256), 0, flux_hip_stream_handle(), (bf16 *)p_bf16, s, key_bias, ld, scale);
    LAUNCH_OK("vae_softmax_kernel");
    return 1;
}

extern "C" int flux_hip_transpose_bf16(void *vt, int ld, const void *v, int ldv, int rows, int cols) {
    if (cols <= 0 || (cols & 63) || ld < rows) return flux_hip_fail("flux_hip_transpose_bf16: bad shape");
    hipLaunchKernelGGL(vae_transpose_kernel, dim3((ld + 63) / 64, cols / 64), dim3(256), 0, flux_hip_stream_handle(), (bf16 *)vt, ld, (const bf16 *)v,
                       ldv, rows);
    LAUNCH_OK("vae_transpose_kernel");
    return 1;
}

extern "C" int flux_hip_vae_image_out(uint8_t *rgb, float *rgb_f32, const float *x, int ldx, int H, int W) {
    hipLaunchKernelGGL(vae_image_kernel, dim3((H * W + 255) / 256), dim3(256), 0, flux_hip_stream_handle(), rgb, rgb_f32, x, ldx, H, W);
    LAUNCH_OK("vae_image_kernel");
    return 1;
}
