/*
 * qwen3.hip - the kernels of the Qwen3 text encoder that are not GEMMs (reference: CPU arms of
 * flux_qwen3.c): embedding lookup, RMS norm, per-head RMS norm + rotate-half RoPE, causal
 * grouped-query attention with a padding mask, and the copy that collects three layers' hidden
 * states side by side. The projections and the MLP run through flux_hip_linear (gemm.hip).
 */
#include "common.h"
#include "../../include/flux_hip.h"
#include <math.h>

#define LAUNCH_OK(what)                                                                         \
    do {                                                                                        \
        hipError_t e_ = hipGetLastError();                                                      \
        if (e_ != hipSuccess) return flux_hip_fail("%s launch failed: %s", what, hipGetErrorString(e_)); \
    } while (0)

/* x[s] = embed[ids[s]], or zeros for an id outside the vocabulary (qwen3_forward,
 * flux_qwen3.c:1046-1056). One workgroup per token. */
__global__ __launch_bounds__(256) void qwen3_embed_kernel(float *__restrict__ x, const bf16 *__restrict__ embed, const int *__restrict__ ids,
                                                          int hidden, int vocab) {
    const int s = blockIdx.x, id = ids[s];
    const bool ok = id >= 0 && id < vocab;
    for (int i = threadIdx.x; i < hidden; i += 256) x[(size_t)s * hidden + i] = ok ? (float)embed[(size_t)id * hidden + i] : 0.0f;
}

/* out bf16 = x / sqrt(mean(x^2) + eps) * w per row (qwen3_rms_norm, flux_qwen3.c:177-197) */
__global__ __launch_bounds__(256) void qwen3_rms_norm_kernel(bf16 *__restrict__ out, const float *__restrict__ x, const float *__restrict__ w,
                                                             int hidden, float eps) {
    __shared__ float red[4];
    const float *xr = x + (size_t)blockIdx.x * hidden;
    float ss = 0.0f;
    for (int i = threadIdx.x * 4; i < hidden; i += 1024) {
        const f32x4 v = *(const f32x4 *)(xr + i);
        ss += v[0] * v[0] + v[1] * v[1] + v[2] * v[2] + v[3] * v[3];
    }
    for (int o = 32; o > 0; o >>= 1) ss += __shfl_xor(ss, o);
    if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = ss;
    __syncthreads();
    const float inv = 1.0f / sqrtf((red[0] + red[1] + red[2] + red[3]) / hidden + eps);
    for (int i = threadIdx.x * 4; i < hidden; i += 1024) {
        const f32x4 v = *(const f32x4 *)(xr + i), g = *(const f32x4 *)(w + i);
        bf16x4 o;
#pragma unroll
        for (int e = 0; e < 4; e++) o[e] = (bf16)(v[e] * inv * g[e]);
        *(bf16x4 *)(out + (size_t)blockIdx.x * hidden + i) = o;
    }
}

/* In place on the fused projection output qkv bf16 [seq, (heads + 2 kv_heads) * 128]: every q and k
 * head gets RMS norm * weight over its 128 values (qwen3_head_rms_norm, flux_qwen3.c:199-220)
 * and rotate-half RoPE, pairs (i, i + 64) with the table's angle for (position, i)
 * (apply_rope, flux_qwen3.c:264-307). One wave per (token, head): lane i holds the pair.
 * The v heads are written transposed to vt [kv_heads * 128, ldv] (keys contiguous), the layout the
 * attention kernel's second product reads. */
__global__ __launch_bounds__(64) void qwen3_qk_rope_kernel(bf16 *__restrict__ qkv, bf16 *__restrict__ vt, int ldv, const float *__restrict__ q_w,
                                                           const float *__restrict__ k_w, const float *__restrict__ rope_cos,
                                                           const float *__restrict__ rope_sin, int heads, int kv_heads, float eps) {
    const int s = blockIdx.x, h = blockIdx.y, lane = threadIdx.x;
    const int width = (heads + 2 * kv_heads) * 128;
    bf16 *p = qkv + (size_t)s * width + h * 128;
    if (h >= heads + kv_heads) { /* a v head: transpose */
        const int vh = h - heads - kv_heads;
        vt[(size_t)(vh * 128 + lane) * ldv + s] = p[lane];
        vt[(size_t)(vh * 128 + lane + 64) * ldv + s] = p[lane + 64];
        return;
    }
    const float *w = h < heads ? q_w : k_w;
    const float x0 = (float)p[lane], x1 = (float)p[lane + 64];
    float ss = x0 * x0 + x1 * x1;
    for (int o = 32; o > 0; o >>= 1) ss += __shfl_xor(ss, o);
    const float inv = 1.0f / sqrtf(ss / 128.0f + eps);
    const float a = x0 * inv * w[lane], b = x1 * inv * w[lane + 64];
    const float cs = rope_cos[s * 64 + lane], sn = rope_sin[s * 64 + lane];
    p[lane] = (bf16)(a * cs - b * sn);
    p[lane + 64] = (bf16)(a * sn + b * cs);
}

/*
 * Causal grouped-query attention, head_dim 128, up to 512 keys (qwen3_attention_forward,
 * flux_qwen3.c:352-437): scores = q.k / sqrt(128); a key after the query, or one whose mask entry
 * is 0, gets the score -1e9 (not -inf: a row with no admissible key then comes out uniform over all
 * seq columns, exactly as in the reference); softmax over all seq columns; out = P v.
 *
 * One workgroup per (16 queries, kv head): its waves are the query heads that share that kv head,
 * so each 32-key tile of K and of V^T is fetched once and shared through LDS (two slots; the next
 * tile travels global -> registers while the current one is multiplied, then registers -> LDS,
 * one barrier per tile). A wave keeps all scores of its 16 queries against all keys in registers
 * (S^T = K Q^T as 16 x 16 blocks, keys x queries: 32 blocks of 4 registers), so the softmax is
 * the plain three-step one. Inside each group of 32 keys the K rows are assigned to MFMA rows so
 * that a lane ends up with 8 consecutive keys of one query: that is the B-operand layout of the
 * second product O^T = V^T P^T. LDS rows are chunk-swizzled so that the 16 rows a fragment read
 * touches fall into different banks.
 */
#define QW_MAXT 16 /* 32-key steps: 512 keys */
__device__ __forceinline__ int qw_kswz(int j) { return (j & 15) ^ ((j >> 4) << 2); } /* K tile: 32 rows of 16 chunks */
__device__ __forceinline__ int qw_vswz(int d) { return (d >> 2) & 3; }               /* V^T tile: 128 rows of 4 chunks */

/* The body for NT 32-key steps, NT a compile-time constant (straight-line code). Steps beyond the
 * sequence read clamped rows and are masked like the padding of the last step. */
template <int NT, int G>
__device__ __forceinline__ void qwen3_attend(bf16 *__restrict__ out, const bf16 *__restrict__ qkv, const bf16 *__restrict__ vt, int ldv,
                                             const int *__restrict__ mask, int seq, int heads, int kv_heads, char *smem) {
    const int tid = threadIdx.x, lane = tid & 63, l15 = lane & 15, lq = lane >> 4;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    constexpr int nthreads = 64 * G;
    const int q0 = blockIdx.x * 16, kh = blockIdx.y, h = kh * (heads / kv_heads) + wave;
    const int width = (heads + 2 * kv_heads) * 128;
    const float scale = 0.08838834764831845f; /* 1 / sqrt(128) */
    constexpr int per_lane = 512 / nthreads;  /* 16-byte chunks of a tile per lane: 8, 4, 2 or 1 */

    /* Q^T fragments (MFMA B operand): lane (query l15, lq) holds dims [32 ks + 8 lq, +8) */
    const int qrow = min(q0 + l15, seq - 1);
    bf16x8 qf[4];
#pragma unroll
    for (int ks = 0; ks < 4; ks++) qf[ks] = *(const bf16x8 *)(qkv + (size_t)qrow * width + h * 128 + ks * 32 + lq * 8);

    bf16x8 stage[per_lane];
    /* K tile t: LDS row j = key 32 t + j, 16 chunks of 8 dims, chunk c stored at c ^ kswz(j) */
    auto fetch_k = [&](int t) {
#pragma unroll
        for (int u = 0; u < per_lane; u++)
            {
                const int idx = tid + u * nthreads, j = idx >> 4, c = idx & 15;
                stage[u] = *(const bf16x8 *)(qkv + (size_t)min(32 * t + j, seq - 1) * width + (heads + kh) * 128 + c * 8);
            }
    };
    auto put_k = [&](int slot) {
#pragma unroll
        for (int u = 0; u < per_lane; u++)
            {
                const int idx = tid + u * nthreads, j = idx >> 4, c = idx & 15;
                *(bf16x8 *)(smem + slot * 8192 + j * 256 + ((c ^ qw_kswz(j)) << 4)) = stage[u];
            }
    };
    /* V^T tile t: LDS row d = head dim, 4 chunks of 8 keys, chunk c stored at c ^ vswz(d) */
    auto fetch_v = [&](int t) {
#pragma unroll
        for (int u = 0; u < per_lane; u++)
            {
                const int idx = tid + u * nthreads, d = idx >> 2, c = idx & 3;
                stage[u] = *(const bf16x8 *)(vt + (size_t)(kh * 128 + d) * ldv + min(32 * t, ldv - 32) + c * 8);
            }
    };
    auto put_v = [&](int slot) {
#pragma unroll
        for (int u = 0; u < per_lane; u++)
            {
                const int idx = tid + u * nthreads, d = idx >> 2, c = idx & 3;
                *(bf16x8 *)(smem + 16384 + slot * 8192 + d * 64 + ((c ^ qw_vswz(d)) << 4)) = stage[u];
            }
    };

    f32x4 sc[2 * NT];
    fetch_k(0);
    put_k(0);
    __syncthreads();
#pragma unroll
    for (int t = 0; t < NT; t++) {
        if (t + 1 < NT) fetch_k(t + 1);
        const char *kt = smem + (t & 1) * 8192;
#pragma unroll
        for (int half = 0; half < 2; half++) {
            /* MFMA row m = l15 of this block is key 32 t + j with j = 8 (m / 4) + 4 half + (m % 4) */
            const int j = 8 * (l15 >> 2) + 4 * half + (l15 & 3);
            f32x4 acc = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
            for (int ks = 0; ks < 4; ks++) {
                const bf16x8 kf = *(const bf16x8 *)(kt + j * 256 + (((ks * 4 + lq) ^ qw_kswz(j)) << 4));
                acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kf, qf[ks], acc, 0, 0, 0);
            }
            sc[2 * t + half] = acc;
        }
        if (t + 1 < NT) {
            put_k((t + 1) & 1);
            __syncthreads();
        }
    }
    fetch_v(0); /* in flight during the softmax */

    /* padding mask as bits: word w covers keys [64 w, 64 w + 64), one ballot per word */
    unsigned long long keep[(NT + 1) / 2];
#pragma unroll
    for (int w = 0; w < (NT + 1) / 2; w++) {
        const int key = 64 * w + lane;
        keep[w] = __ballot(key < seq && (!mask || mask[key] != 0));
    }
    /* accumulator element e of block (t, half): query l15, key 32 t + 8 lq + 4 half + e */
    const int qi = q0 + l15;
    float mx = -3.0e38f;
#pragma unroll
    for (int t = 0; t < NT; t++) {
        const unsigned bits = (unsigned)(keep[t >> 1] >> (32 * (t & 1))) >> (8 * lq); /* this lane's 8 keys of step t */
#pragma unroll
        for (int half = 0; half < 2; half++)
#pragma unroll
            for (int e = 0; e < 4; e++) {
                const int key = 32 * t + 8 * lq + 4 * half + e;
                float v = sc[2 * t + half][e] * scale;
                if (key > qi || !((bits >> (4 * half + e)) & 1)) v = -1e9f;
                if (key >= seq) v = -INFINITY; /* padding of the last 32-key step: no column of the reference's matrix */
                sc[2 * t + half][e] = v;
                mx = fmaxf(mx, v);
            }
    }
    mx = fmaxf(mx, __shfl_xor(mx, 16));
    mx = fmaxf(mx, __shfl_xor(mx, 32));
    float sum = 0.0f;
#pragma unroll
    for (int t = 0; t < NT; t++)
#pragma unroll
        for (int half = 0; half < 2; half++)
#pragma unroll
            for (int e = 0; e < 4; e++) {
                const float p = __expf(sc[2 * t + half][e] - mx);
                sc[2 * t + half][e] = p;
                sum += p;
            }
    sum += __shfl_xor(sum, 16);
    sum += __shfl_xor(sum, 32);
    const float inv = 1.0f / sum;

    /* O^T[d][q] = sum_key V^T[d][key] P^T[key][q]: A operand = V^T rows (lane: dim l15, keys
     * [32 t + 8 lq, +8)), B operand = this lane's 8 probabilities of step t */
    f32x4 o[8];
#pragma unroll
    for (int d = 0; d < 8; d++) o[d] = (f32x4){0.0f, 0.0f, 0.0f, 0.0f};
    put_v(0);
    __syncthreads();
#pragma unroll
    for (int t = 0; t < NT; t++) {
        if (t + 1 < NT) fetch_v(t + 1);
        const char *vtile = smem + 16384 + (t & 1) * 8192;
        bf16x8 pf;
#pragma unroll
        for (int e = 0; e < 4; e++) {
            pf[e] = (bf16)(sc[2 * t][e] * inv);
            pf[4 + e] = (bf16)(sc[2 * t + 1][e] * inv);
        }
#pragma unroll
        for (int d = 0; d < 8; d++) {
            const int row = d * 16 + l15;
            const bf16x8 vf = *(const bf16x8 *)(vtile + row * 64 + ((lq ^ qw_vswz(row)) << 4));
            o[d] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vf, pf, o[d], 0, 0, 0);
        }
        if (t + 1 < NT) {
            put_v((t + 1) & 1);
            __syncthreads();
        }
    }
    /* accumulator element e of block d: query l15, dim 16 d + 4 lq + e */
    if (qi < seq) {
        bf16 *op = out + (size_t)qi * heads * 128 + h * 128 + 4 * lq;
#pragma unroll
        for (int d = 0; d < 8; d++) {
            bf16x4 ov;
#pragma unroll
            for (int e = 0; e < 4; e++) ov[e] = (bf16)o[d][e];
            *(bf16x4 *)(op + d * 16) = ov;
        }
    }
}

/* Steps whose 32 keys all lie after the block's last query hold no admissible key and are left
 * out - unless the first key is masked: only then can a row have no admissible key at all, and such
 * a row is uniform over every column (see above), so every step is computed. The step count is
 * rounded up to one of five compiled bodies. Workgroup = heads / kv_heads waves. */
template <int G>
__global__ __launch_bounds__(64 * G) void qwen3_attention_kernel(bf16 *__restrict__ out, const bf16 *__restrict__ qkv, const bf16 *__restrict__ vt,
                                                              int ldv, const int *__restrict__ mask, int seq, int heads, int kv_heads) {
    __shared__ __attribute__((aligned(16))) char smem[32768]; /* K tiles: 2 x 8 KB, V^T tiles: 2 x 8 KB */
    const int all = (seq + 31) >> 5;
    const bool first_masked = mask && mask[0] == 0;
    const int need = first_masked ? all : min(all, ((blockIdx.x * 16 + 15) >> 5) + 1);
    if (need <= 2) qwen3_attend<2, G>(out, qkv, vt, ldv, mask, seq, heads, kv_heads, smem);
    else if (need <= 4) qwen3_attend<4, G>(out, qkv, vt, ldv, mask, seq, heads, kv_heads, smem);
    else if (need <= 8) qwen3_attend<8, G>(out, qkv, vt, ldv, mask, seq, heads, kv_heads, smem);
    else if (need <= 12) qwen3_attend<12, G>(out, qkv, vt, ldv, mask, seq, heads, kv_heads, smem);
    else qwen3_attend<16, G>(out, qkv, vt, ldv, mask, seq, heads, kv_heads, smem);
}

/* dst[s, col0 + i] = src[s, i]: one layer's hidden state into its third of the output rows */
__global__ __launch_bounds__(256) void qwen3_collect_kernel(float *__restrict__ dst, int ldd, int col0, const float *__restrict__ src, int hidden) {
    for (int i = threadIdx.x; i < hidden; i += 256) dst[(size_t)blockIdx.x * ldd + col0 + i] = src[(size_t)blockIdx.x * hidden + i];
}

/* ------------------------------------------------------------------ host entry points */

extern "C" int flux_hip_qwen3_embed(float *x, const void *embed_bf16, const int *ids_dev, int seq, int hidden, int vocab) {
    if (seq <= 0 || hidden <= 0) return flux_hip_fail("flux_hip_qwen3_embed: bad shape");
    hipLaunchKernelGGL(qwen3_embed_kernel, dim3(seq), dim3(256), 0, flux_hip_stream_handle(), x, (const bf16 *)embed_bf16, ids_dev, hidden, vocab);
    LAUNCH_OK("qwen3_embed_kernel");
    return 1;
}

extern "C" int flux_hip_rms_norm(void *out_bf16, const float *x, const float *w, int rows, int hidden, float eps) {
    if (rows <= 0 || hidden <= 0 || (hidden & 3)) return flux_hip_fail("flux_hip_rms_norm: bad shape %d x %d", rows, hidden);
    hipLaunchKernelGGL(qwen3_rms_norm_kernel, dim3(rows), dim3(256), 0, flux_hip_stream_handle(), (bf16 *)out_bf16, x, w, hidden, eps);
    LAUNCH_OK("qwen3_rms_norm_kernel");
    return 1;
}

extern "C" int flux_hip_qwen3_qk_rope(void *qkv_bf16, void *vt_bf16, int ldv, const float *q_w, const float *k_w, const float *rope_cos,
                                      const float *rope_sin, int seq, int heads, int kv_heads, float eps) {
    if (seq <= 0 || heads <= 0 || kv_heads <= 0 || ldv < seq) return flux_hip_fail("flux_hip_qwen3_qk_rope: bad shape");
    hipLaunchKernelGGL(qwen3_qk_rope_kernel, dim3(seq, heads + 2 * kv_heads), dim3(64), 0, flux_hip_stream_handle(), (bf16 *)qkv_bf16,
                       (bf16 *)vt_bf16, ldv, q_w, k_w, rope_cos, rope_sin, heads, kv_heads, eps);
    LAUNCH_OK("qwen3_qk_rope_kernel");
    return 1;
}

extern "C" int flux_hip_causal_attention(void *out_bf16, const void *qkv_bf16, const void *vt_bf16, int ldv, const int *mask_dev, int seq,
                                         int heads, int kv_heads) {
    if (seq <= 0 || seq > 32 * QW_MAXT) return flux_hip_fail("flux_hip_causal_attention: seq=%d (1..%d)", seq, 32 * QW_MAXT);
    if (heads <= 0 || kv_heads <= 0 || heads % kv_heads) return flux_hip_fail("flux_hip_causal_attention: heads=%d kv_heads=%d", heads, kv_heads);
    const int group = heads / kv_heads; /* waves per workgroup */
    if (group != 1 && group != 2 && group != 4 && group != 8)
        return flux_hip_fail("flux_hip_causal_attention: %d query heads per kv head (1, 2, 4 or 8)", group);
    if (ldv < ((seq + 31) & ~31) || (ldv & 7)) return flux_hip_fail("flux_hip_causal_attention: ldv=%d too small or not a multiple of 8", ldv);
    const dim3 grid((seq + 15) / 16, kv_heads);
#define QW_LAUNCH(G)                                                                                                                   \
    hipLaunchKernelGGL(qwen3_attention_kernel<G>, grid, dim3(64 * G), 0, flux_hip_stream_handle(), (bf16 *)out_bf16, (const bf16 *)qkv_bf16, \
                       (const bf16 *)vt_bf16, ldv, mask_dev, seq, heads, kv_heads)
    if (group == 1) QW_LAUNCH(1);
    else if (group == 2) QW_LAUNCH(2);
    else if (group == 4) QW_LAUNCH(4);
    else QW_LAUNCH(8);
#undef QW_LAUNCH
    LAUNCH_OK("qwen3_attention_kernel");
    return 1;
}

extern "C" int flux_hip_qwen3_collect(float *dst, int ldd, int col0, const float *src, int seq, int hidden) {
    hipLaunchKernelGGL(qwen3_collect_kernel, dim3(seq), dim3(256), 0, flux_hip_stream_handle(), dst, ldd, col0, src, hidden);
    LAUNCH_OK("qwen3_collect_kernel");
    return 1;
}
