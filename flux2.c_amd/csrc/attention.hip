/*
 * attention.hip - joint text+image attention for gfx950: a K/V preparation pass and a
 * flash-style MFMA kernel with online softmax that never stores the score matrix.
 *
 * Reference semantics: joint_attention / mha_forward (flux_transformer.c:1249-1460):
 * softmax(q k^T / sqrt(128)) v per head, no mask, every query sees every key; before that
 * apply_qk_norm (flux_transformer.c:1052-1106) and apply_rope_2d (flux_transformer.c:719-741)
 * on q and k. Text and image tokens live in one [text ; image] buffer, so the reference's K/V
 * concatenation (flux_transformer.c:1351-1354) is the buffer itself.
 *
 * Orientation. The kernel computes S^T = K Q^T and O^T = V^T P^T with 32x32x16 bf16 MFMA.
 * In an MFMA accumulator a lane owns one column, so here a lane owns one *query*: the row
 * maximum and row sum of the softmax are reductions over the lane's own registers plus one
 * exchange with lane^32, and the rescale of O is a per-lane scalar. The accumulator of S^T
 * also already has the register layout the "B" operand of the second product needs, up to a
 * permutation of keys inside each group of 16, which is applied to the V^T operand instead
 * (two 8-byte LDS reads per fragment).
 */
#include "common.h"
#include "../../include/flux_hip.h"

#define HD 128

__device__ __forceinline__ float wave16_sum(float v) {
#pragma unroll
    for (int o = 8; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
    return v;
}

/* ---------------------------------------------------------------------------------------
 * K/V preparation. One workgroup handles 64 tokens of one head.
 *   K: RMSNorm over the 128 dims * weight, then rotation of pairs (d, d+1) by the token's
 *      cos/sin row; written token-major.
 *   V: written transposed, vt[head*128 + d][token], columns beyond `rows` zero-filled up to
 *      the next multiple of 64 so that the attention kernel can read whole key tiles.
 * --------------------------------------------------------------------------------------- */
__global__ __launch_bounds__(256) void kv_prepare_kernel(bf16 *__restrict__ k_out, bf16 *__restrict__ vt_out, int ld_vt,
                                                         const bf16 *__restrict__ qkv, int ld, int k_col, int v_col,
                                                         int rows, int heads, int split,
                                                         const float *__restrict__ k_w0, const float *__restrict__ k_w1,
                                                         const float *__restrict__ rope_cos,
                                                         const float *__restrict__ rope_sin, float eps) {
    __shared__ __attribute__((aligned(16))) bf16 vt_tile[64][HD + 8];
    const int r0 = blockIdx.x * 64, h = blockIdx.y;
    const int tid = threadIdx.x;
    const int c = tid & 15; /* 16-byte chunk of the 128-dim head row */
    const int H = heads * HD;

#pragma unroll
    for (int i = 0; i < 4; i++) {
        const int r = (tid >> 4) + i * 16;
        const int row = r0 + r;
        const int rowc = min(row, rows - 1);
        /* V chunk into the LDS tile */
        bf16x8 vv = *(const bf16x8 *)(qkv + (size_t)rowc * ld + v_col + h * HD + c * 8);
        if (row >= rows)
#pragma unroll
            for (int e = 0; e < 8; e++) vv[e] = (bf16)0.0f;
        *(bf16x8 *)(&vt_tile[r][c * 8]) = vv;

        /* K chunk: norm + rope */
        bf16x8 kv = *(const bf16x8 *)(qkv + (size_t)rowc * ld + k_col + h * HD + c * 8);
        float x[8];
        float ss = 0.0f;
#pragma unroll
        for (int e = 0; e < 8; e++) { x[e] = (float)kv[e]; ss += x[e] * x[e]; }
        ss = wave16_sum(ss);
        const float inv = 1.0f / sqrtf(ss * (1.0f / HD) + eps);
        const float *w = (rowc < split ? k_w0 : k_w1) + c * 8;
        const float *cs = rope_cos + (size_t)rowc * HD + c * 8;
        const float *sn = rope_sin + (size_t)rowc * HD + c * 8;
        f32x4 w0 = *(const f32x4 *)w, w1 = *(const f32x4 *)(w + 4);
        f32x4 c0 = *(const f32x4 *)cs, c1 = *(const f32x4 *)(cs + 4);
        f32x4 s0 = *(const f32x4 *)sn, s1 = *(const f32x4 *)(sn + 4);
        float wv[8] = {w0[0], w0[1], w0[2], w0[3], w1[0], w1[1], w1[2], w1[3]};
        float cv[8] = {c0[0], c0[1], c0[2], c0[3], c1[0], c1[1], c1[2], c1[3]};
        float sv[8] = {s0[0], s0[1], s0[2], s0[3], s1[0], s1[1], s1[2], s1[3]};
        bf16x8 o;
#pragma unroll
        for (int e = 0; e < 8; e += 2) {
            float a = x[e] * inv * wv[e], b = x[e + 1] * inv * wv[e + 1];
            o[e] = (bf16)(a * cv[e] - b * sv[e]);
            o[e + 1] = (bf16)(b * cv[e] + a * sv[e]);
        }
        if (row < rows) *(bf16x8 *)(k_out + (size_t)row * H + h * HD + c * 8) = o;
    }
    __syncthreads();
    /* transposed write: thread -> (d, group of 8 tokens) */
#pragma unroll
    for (int i = 0; i < 4; i++) {
        const int tg = tid & 7, d = (tid >> 3) + i * 32;
        bf16x8 o;
#pragma unroll
        for (int e = 0; e < 8; e++) o[e] = vt_tile[tg * 8 + e][d];
        *(bf16x8 *)(vt_out + (size_t)(h * HD + d) * ld_vt + r0 + tg * 8) = o;
    }
}

extern "C" int flux_hip_kv_prepare(void *k_out, void *vt_out, int ld_vt, const void *qkv, int ld, int k_col, int v_col,
                                   int rows, int heads, int split, const float *k_w0, const float *k_w1,
                                   const float *rope_cos, const float *rope_sin, float eps) {
    if (rows <= 0) return 1;
    if (!k_out || !vt_out || !qkv || !k_w0 || !rope_cos || !rope_sin) return flux_hip_fail("flux_hip_kv_prepare: NULL argument");
    if (split < rows && !k_w1) return flux_hip_fail("flux_hip_kv_prepare: second weight missing");
    const int padded = (rows + 63) / 64 * 64;
    if (ld_vt < padded || (ld_vt & 7)) return flux_hip_fail("flux_hip_kv_prepare: ld_vt=%d must be >= %d and a multiple of 8", ld_vt, padded);
    if ((ld & 7) || (k_col & 7) || (v_col & 7)) return flux_hip_fail("flux_hip_kv_prepare: ld/k_col/v_col must be multiples of 8");
    hipLaunchKernelGGL(kv_prepare_kernel, dim3(padded / 64, heads), dim3(256), 0, flux_hip_stream_handle(),
                       (bf16 *)k_out, (bf16 *)vt_out, ld_vt, (const bf16 *)qkv, ld, k_col, v_col, rows, heads, split,
                       k_w0, k_w1 ? k_w1 : k_w0, rope_cos, rope_sin, eps);
    HIP_OK(hipGetLastError());
    return 1;
}

/* ---------------------------------------------------------------------------------------
 * Flash attention. Workgroup = 4 waves = 128 queries of one head; a wave owns 32 queries and
 * the full head dimension. Keys are walked in tiles of 64 through two LDS stages.
 *   LDS stage: K tile [64 keys][128 d] (256-byte rows, 16-byte chunks XOR-swizzled by key%16)
 *              V^T tile [128 d][64 keys] (128-byte rows, 16-byte chunks swizzled by (d/2)%8)
 * --------------------------------------------------------------------------------------- */
#define ATT_STAGE (64 * 256 + 128 * 128)

__global__ __launch_bounds__(256, 2) void attention_kernel(bf16 *__restrict__ out, int ldo,
                                                           const bf16 *__restrict__ q, int ldq,
                                                           const bf16 *__restrict__ k, const bf16 *__restrict__ vt, int ld_vt,
                                                           int seq_q, int seq_k, int heads, int split,
                                                           const float *__restrict__ q_w0, const float *__restrict__ q_w1,
                                                           const float *__restrict__ rope_cos,
                                                           const float *__restrict__ rope_sin, float eps) {
    extern __shared__ __attribute__((aligned(16))) char smem[];
    const int h = blockIdx.y;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int l31 = lane & 31, lhi = lane >> 5;
    const int H = heads * HD;
    const int qrow = blockIdx.x * 128 + wave * 32 + l31;
    const int qrc = min(qrow, seq_q - 1);

    /* ---- Q fragments: B operand, lane = query, 8 consecutive dims per K-step ---- */
    bf16x8 qf[8];
    {
        const bf16 *qp = q + (size_t)qrc * ldq + h * HD + lhi * 8;
        float x[8][8];
        float ss = 0.0f;
#pragma unroll
        for (int kk = 0; kk < 8; kk++) {
            bf16x8 v = *(const bf16x8 *)(qp + kk * 16);
#pragma unroll
            for (int e = 0; e < 8; e++) { x[kk][e] = (float)v[e]; ss += x[kk][e] * x[kk][e]; }
        }
        ss += __shfl_xor(ss, 32, 64);
        /* fold 1/sqrt(128) and log2(e) into q so that scores are base-2 logits */
        const float inv = 1.0f / sqrtf(ss * (1.0f / HD) + eps);
        const float fold = 0.08838834764831845f * 1.44269504088896341f;
        const float *w = (qrc < split ? q_w0 : q_w1) + lhi * 8;
        const float *cs = rope_cos + (size_t)qrc * HD + lhi * 8;
        const float *sn = rope_sin + (size_t)qrc * HD + lhi * 8;
#pragma unroll
        for (int kk = 0; kk < 8; kk++) {
            f32x4 w0 = *(const f32x4 *)(w + kk * 16), w1 = *(const f32x4 *)(w + kk * 16 + 4);
            f32x4 c0 = *(const f32x4 *)(cs + kk * 16), c1 = *(const f32x4 *)(cs + kk * 16 + 4);
            f32x4 s0 = *(const f32x4 *)(sn + kk * 16), s1 = *(const f32x4 *)(sn + kk * 16 + 4);
            float wv[8] = {w0[0], w0[1], w0[2], w0[3], w1[0], w1[1], w1[2], w1[3]};
            float cv[8] = {c0[0], c0[1], c0[2], c0[3], c1[0], c1[1], c1[2], c1[3]};
            float sv[8] = {s0[0], s0[1], s0[2], s0[3], s1[0], s1[1], s1[2], s1[3]};
#pragma unroll
            for (int e = 0; e < 8; e += 2) {
                float a = x[kk][e] * inv * wv[e], b = x[kk][e + 1] * inv * wv[e + 1];
                /* round to bf16 first (what the key side does), then apply the folded scale */
                float ra = a * cv[e] - b * sv[e], rb = b * cv[e] + a * sv[e];
                qf[kk][e] = (bf16)(ra * fold);
                qf[kk][e + 1] = (bf16)(rb * fold);
            }
        }
    }

    /* ---- tile loader mapping ---- */
    const int kc = tid & 15, kr = tid >> 4;  /* K: 16 chunks per row, rows kr + 16 i */
    const int vc = tid & 7, vr = tid >> 3;   /* V^T: 8 chunks per row, rows vr + 32 i */
    const bf16 *kbase = k + h * HD + kc * 8;
    const bf16 *vbase = vt + (size_t)(h * HD) * ld_vt + vc * 8;
    int k_lds[4], v_lds[4];
#pragma unroll
    for (int i = 0; i < 4; i++) {
        int r = kr + i * 16;
        k_lds[i] = r * 256 + ((kc ^ (r & 15)) << 4);
        int d = vr + i * 32;
        v_lds[i] = 64 * 256 + d * 128 + ((vc ^ ((d >> 1) & 7)) << 4);
    }
    const int ntiles = (seq_k + 63) >> 6;
    bf16x8 rk[4], rv[4];
    auto load_tile = [&](int t) {
        const int key0 = t * 64;
#pragma unroll
        for (int i = 0; i < 4; i++) {
            int r = min(key0 + kr + i * 16, seq_k - 1);
            rk[i] = *(const bf16x8 *)(kbase + (size_t)r * H);
            rv[i] = *(const bf16x8 *)(vbase + (size_t)(vr + i * 32) * ld_vt + key0);
        }
    };
    auto store_tile = [&](int stage) {
        char *s = smem + stage * ATT_STAGE;
#pragma unroll
        for (int i = 0; i < 4; i++) {
            *(bf16x8 *)(s + k_lds[i]) = rk[i];
            *(bf16x8 *)(s + v_lds[i]) = rv[i];
        }
    };
    load_tile(0);
    store_tile(0);
    __syncthreads();

    f32x16 o_acc[4];
#pragma unroll
    for (int i = 0; i < 4; i++)
#pragma unroll
        for (int e = 0; e < 16; e++) o_acc[i][e] = 0.0f;
    float m_run = -1e30f, l_run = 0.0f;

    const int kswz = l31 & 15;
    for (int t = 0; t < ntiles; t++) {
        const int cur = t & 1;
        if (t + 1 < ntiles) load_tile(t + 1);
        const char *st = smem + cur * ATT_STAGE;

        /* S^T[keys][queries] for 64 keys */
        f32x16 s_acc[2];
#pragma unroll
        for (int i = 0; i < 2; i++)
#pragma unroll
            for (int e = 0; e < 16; e++) s_acc[i][e] = 0.0f;
#pragma unroll
        for (int kk = 0; kk < 8; kk++) {
#pragma unroll
            for (int i = 0; i < 2; i++) {
                bf16x8 kf = *(const bf16x8 *)(st + (i * 32 + l31) * 256 + (((kk * 2 + lhi) ^ kswz) << 4));
                s_acc[i] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(kf, qf[kk], s_acc[i], 0, 0, 0);
            }
        }
        if (t == ntiles - 1 && (seq_k & 63)) {
            const int key0 = t * 64;
#pragma unroll
            for (int i = 0; i < 2; i++)
#pragma unroll
                for (int e = 0; e < 16; e++) {
                    int key = key0 + i * 32 + (e >> 2) * 8 + lhi * 4 + (e & 3);
                    if (key >= seq_k) s_acc[i][e] = -1e30f;
                }
        }
        /* online softmax, one query per lane (shared with lane ^ 32) */
        float mx = s_acc[0][0];
#pragma unroll
        for (int i = 0; i < 2; i++)
#pragma unroll
            for (int e = 0; e < 16; e++) mx = fmaxf(mx, s_acc[i][e]);
        mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
        const float m_new = fmaxf(m_run, mx);
        const float alpha = fast_exp2(m_run - m_new);
        m_run = m_new;
        float psum = 0.0f;
#pragma unroll
        for (int i = 0; i < 2; i++)
#pragma unroll
            for (int e = 0; e < 16; e++) {
                float p = fast_exp2(s_acc[i][e] - m_new);
                s_acc[i][e] = p;
                psum += p;
            }
        l_run = l_run * alpha + psum;
#pragma unroll
        for (int i = 0; i < 4; i++)
#pragma unroll
            for (int e = 0; e < 16; e++) o_acc[i][e] *= alpha;

        /* O^T += V^T P^T. Key slot s of lane group j in 16-key chunk c is key
         * 16c + 8(s/4) + 4j + s%4, on both operands. */
        bf16x8 pf[4];
#pragma unroll
        for (int c = 0; c < 4; c++)
#pragma unroll
            for (int s = 0; s < 8; s++) pf[c][s] = (bf16)s_acc[c >> 1][(c & 1) * 8 + s];
#pragma unroll
        for (int dt = 0; dt < 4; dt++) {
            const int d = dt * 32 + l31;
            const char *vrow = st + 64 * 256 + d * 128 + lhi * 8;
            const int vs = (d >> 1) & 7;
#pragma unroll
            for (int c = 0; c < 4; c++) {
                bf16x4 lo = *(const bf16x4 *)(vrow + (((c * 2) ^ vs) << 4));
                bf16x4 hi = *(const bf16x4 *)(vrow + (((c * 2 + 1) ^ vs) << 4));
                bf16x8 vf = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
                o_acc[dt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(vf, pf[c], o_acc[dt], 0, 0, 0);
            }
        }
        if (t + 1 < ntiles) store_tile(cur ^ 1);
        __syncthreads();
    }

    l_run += __shfl_xor(l_run, 32, 64);
    const float inv_l = 1.0f / l_run;
    if (qrow < seq_q) {
        bf16 *op = out + (size_t)qrow * ldo + h * HD + lhi * 4;
#pragma unroll
        for (int dt = 0; dt < 4; dt++)
#pragma unroll
            for (int g = 0; g < 4; g++) {
                bf16x4 r;
#pragma unroll
                for (int e = 0; e < 4; e++) r[e] = (bf16)(o_acc[dt][g * 4 + e] * inv_l);
                *(bf16x4 *)(op + dt * 32 + g * 8) = r;
            }
    }
}

extern "C" int flux_hip_attention(void *out_bf16, int ldo, const void *q, int ldq, const void *k, const void *vt,
                                  int ld_vt, int seq_q, int seq_k, int heads, int split, const float *q_w0,
                                  const float *q_w1, const float *rope_cos, const float *rope_sin, float eps) {
    if (seq_q <= 0) return 1;
    if (seq_k <= 0) return flux_hip_fail("flux_hip_attention: seq_k=%d", seq_k);
    if (!out_bf16 || !q || !k || !vt || !q_w0 || !rope_cos || !rope_sin) return flux_hip_fail("flux_hip_attention: NULL argument");
    if (split < seq_q && !q_w1) return flux_hip_fail("flux_hip_attention: second weight missing");
    if ((ldo & 3) || (ldq & 7) || (ld_vt & 7) || ld_vt < (seq_k + 63) / 64 * 64)
        return flux_hip_fail("flux_hip_attention: bad leading dimensions (ldo=%d ldq=%d ld_vt=%d)", ldo, ldq, ld_vt);
    static bool attr_done = false;
    if (!attr_done) {
        HIP_OK(hipFuncSetAttribute((const void *)attention_kernel, hipFuncAttributeMaxDynamicSharedMemorySize, 2 * ATT_STAGE));
        attr_done = true;
    }
    hipLaunchKernelGGL(attention_kernel, dim3((seq_q + 127) / 128, heads), dim3(256), 2 * ATT_STAGE, flux_hip_stream_handle(),
                       (bf16 *)out_bf16, ldo, (const bf16 *)q, ldq, (const bf16 *)k, (const bf16 *)vt, ld_vt, seq_q, seq_k,
                       heads, split, q_w0, q_w1 ? q_w1 : q_w0, rope_cos, rope_sin, eps);
    HIP_OK(hipGetLastError());
    return 1;
}
