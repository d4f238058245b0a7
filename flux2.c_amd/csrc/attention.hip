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
 * Orientation. The kernel computes S^T = K Q^T and O^T = V^T P^T with bf16 MFMA.
 * In an MFMA accumulator a lane owns one column, so here a lane owns one *query*: the row
 * maximum and row sum of the softmax are reductions over the lane's own registers plus two
 * lane exchanges, and the rescale of O is a per-lane scalar. The accumulator of S^T
 * also already has the register layout the "B" operand of the second product needs, up to a
 * permutation of keys inside each group of 32, which is applied for free when the K tile is
 * loaded (the loader picks which key goes to which LDS row).
 */
#include "common.h"
#include "../../include/flux_hip.h"
#include "../../include/flux_hip_debug.h"

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
    if (((uintptr_t)k_out | (uintptr_t)vt_out | (uintptr_t)qkv | (uintptr_t)k_w0 | (uintptr_t)k_w1 | (uintptr_t)rope_cos | (uintptr_t)rope_sin) & 15)
        return flux_hip_fail("flux_hip_kv_prepare: operands must be 16-byte aligned");
    hipLaunchKernelGGL(kv_prepare_kernel, dim3(padded / 64, heads), dim3(256), 0, flux_hip_stream_handle(),
                       (bf16 *)k_out, (bf16 *)vt_out, ld_vt, (const bf16 *)qkv, ld, k_col, v_col, rows, heads, split,
                       k_w0, k_w1 ? k_w1 : k_w0, rope_cos, rope_sin, eps);
    HIP_OK(hipGetLastError());
    return 1;
}

/* ---------------------------------------------------------------------------------------
 * Flash attention. Workgroup = 4 or 8 waves = 128 or 256 queries of one head; a wave owns 32
 * queries (two 16-query MFMA columns) and the full head dimension. Keys are walked in tiles of 64
 * through two LDS stages filled by direct global->LDS loads (no register staging).
 *   LDS stage: K tile [64 keys][128 d] (256-byte rows, 16-byte chunks XOR-swizzled by key%16)
 *              V^T tile [128 d][64 keys] (128-byte rows, 16-byte chunks swizzled by (d/2)%8)
 * MFMA: v_mfma_f32_16x16x32_bf16 (the form that sustains the most under the power limit).
 *   S^T[key][q]: A = K fragment (lane: key l%16, dims 8(l/16)..+8 of a 32-dim chunk),
 *                B = Q fragment (lane: query l%16, same dims); accumulator lane: query l%16,
 *                keys 4(l/16)..+4 of the 16-key block.
 *   O^T[d][q]:   B = P^T fragment for 32 keys = the accumulators of two 16-row score blocks;
 *                the K rows are permuted when the tile is loaded so that these are 8
 *                consecutive keys per lane, and A = V^T fragment is one 16-byte LDS read.
 * --------------------------------------------------------------------------------------- */
#define ATT_STAGE (64 * 256 + 128 * 128)
__device__ __forceinline__ int vt_swz(int d) { return ((d >> 1) & 7) ^ ((d & 1) << 2); }
#define GLOBAL_PTR(p) ((const __attribute__((address_space(1))) void *)(p))
#define LDS_PTR(p) ((__attribute__((address_space(3))) void *)(p))

template <bool V> struct AttFlag { static constexpr bool value = V; };

template <int NW>
__global__ __launch_bounds__(NW * 64, NW == 4 ? 2 : 1) void attention_kernel(bf16 *__restrict__ out, int ldo,
                                                           const bf16 *__restrict__ q, int ldq,
                                                           const bf16 *__restrict__ k, const bf16 *__restrict__ vt, int ld_vt,
                                                           int seq_q, int seq_k, int heads, int split,
                                                           const float *__restrict__ q_w0, const float *__restrict__ q_w1,
                                                           const float *__restrict__ rope_cos,
                                                           const float *__restrict__ rope_sin, float eps) {
    extern __shared__ __attribute__((aligned(16))) char smem[];
    /* Workgroups are dealt round-robin to the 8 XCDs, each with its own L2. Give every XCD a
     * contiguous run of (head, query block) pairs, so that all query blocks of a head run on one
     * XCD and its K / V^T (2.4 MB at 4608 tokens) are fetched from HBM once and then served from
     * that L2, instead of by all eight. */
    constexpr int BQ = NW * 32;  /* queries per workgroup */
    constexpr int LP = 16 / NW;  /* wave-wide load instructions per wave and tile, for K and for V^T */
    const int nqb = (seq_q + BQ - 1) / BQ;
    const int logical = (blockIdx.x & 7) * (gridDim.x >> 3) + (blockIdx.x >> 3);
    if (logical >= nqb * heads) return;
    const int h = logical / nqb, qb = logical - h * nqb;
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int l15 = lane & 15, lq = lane >> 4;
    const int H = heads * HD;

    /* ---- tile loader: per-lane global sources (un-swizzled) and per-wave LDS destinations ---- */
    const int ntiles = (seq_k + 63) >> 6;
    const bf16 *k_src[LP];
    const bf16 *v_src[LP];
    int k_dst[LP], v_dst[LP], k_row[LP];
#pragma unroll
    for (int i = 0; i < LP; i++) {
        /* K: one wave instruction covers 4 rows of 256 bytes */
        int r = wave * 4 + i * (NW * 4) + (lane >> 4); /* LDS row */
        /* LDS row 16 i' + 4 j + e (i' = 2c + b) holds key 32c + 8j + 4b + e of the tile: the
         * score accumulators of two 16-row blocks then cover 8 consecutive keys per lane */
        {
            int ib = r >> 4, jj = (r >> 2) & 3, ee = r & 3;
            k_row[i] = 32 * (ib >> 1) + 8 * jj + 4 * (ib & 1) + ee;
        }
        k_src[i] = k + h * HD + (((lane & 15) ^ (r & 15)) << 3);
        k_dst[i] = (wave * 4 + i * (NW * 4)) * 256;
        /* V^T: one wave instruction covers 8 rows of 128 bytes */
        int d = wave * 8 + i * (NW * 8) + (lane >> 3);
        v_src[i] = vt + (size_t)(h * HD + d) * ld_vt + (((lane & 7) ^ vt_swz(d)) << 3);
        v_dst[i] = (wave * 8 + i * (NW * 8)) * 128;
    }
    /* LDS: K ring = 2 slots of 16 KB at 0 and 16 KB; V^T ring = 2 slots of 16 KB at 32 and 48 KB */
    auto issue_k = [&](int t) {
        char *base = smem + (t & 1) * (64 * 256);
        const int key0 = t * 64;
#pragma unroll
        for (int i = 0; i < LP; i++) {
            int r = min(key0 + k_row[i], seq_k - 1);
            __builtin_amdgcn_global_load_lds(GLOBAL_PTR(k_src[i] + (size_t)r * H), LDS_PTR(base + k_dst[i]), 16, 0, 0);
        }
    };
    auto issue_v = [&](int t) {
        char *base = smem + 2 * (64 * 256) + (t & 1) * (128 * 128);
        const int key0 = t * 64;
#pragma unroll
        for (int i = 0; i < LP; i++)
            __builtin_amdgcn_global_load_lds(GLOBAL_PTR(v_src[i] + key0), LDS_PTR(base + v_dst[i]), 16, 0, 0);
    };
    issue_k(0);
    issue_v(0);

    /* ---- Q fragments (B operand), with RMSNorm * weight, RoPE and the softmax scale ---- */
    bf16x8 qf[2][4];
    int qrow[2];
#pragma unroll
    for (int t = 0; t < 2; t++) {
        qrow[t] = qb * BQ + wave * 32 + t * 16 + l15;
        const int qrc = min(qrow[t], seq_q - 1);
        const bf16 *qp = q + (size_t)qrc * ldq + h * HD + lq * 8;
        float x[4][8];
        float ss = 0.0f;
#pragma unroll
        for (int kk = 0; kk < 4; kk++) {
            bf16x8 v = *(const bf16x8 *)(qp + kk * 32);
#pragma unroll
            for (int e = 0; e < 8; e++) { x[kk][e] = (float)v[e]; ss += x[kk][e] * x[kk][e]; }
        }
        ss += __shfl_xor(ss, 16, 64);
        ss += __shfl_xor(ss, 32, 64);
        const float inv = 1.0f / sqrtf(ss * (1.0f / HD) + eps);
        /* 1/sqrt(128) and log2(e) folded into q: scores come out as base-2 logits */
        const float fold = 0.08838834764831845f * 1.44269504088896341f;
        const float *w = (qrc < split ? q_w0 : q_w1) + lq * 8;
        const float *cs = rope_cos + (size_t)qrc * HD + lq * 8;
        const float *sn = rope_sin + (size_t)qrc * HD + lq * 8;
#pragma unroll
        for (int kk = 0; kk < 4; kk++) {
            f32x4 w0 = *(const f32x4 *)(w + kk * 32), w1 = *(const f32x4 *)(w + kk * 32 + 4);
            f32x4 c0 = *(const f32x4 *)(cs + kk * 32), c1 = *(const f32x4 *)(cs + kk * 32 + 4);
            f32x4 s0 = *(const f32x4 *)(sn + kk * 32), s1 = *(const f32x4 *)(sn + kk * 32 + 4);
            float wv[8] = {w0[0], w0[1], w0[2], w0[3], w1[0], w1[1], w1[2], w1[3]};
            float cv[8] = {c0[0], c0[1], c0[2], c0[3], c1[0], c1[1], c1[2], c1[3]};
            float sv[8] = {s0[0], s0[1], s0[2], s0[3], s1[0], s1[1], s1[2], s1[3]};
#pragma unroll
            for (int e = 0; e < 8; e += 2) {
                float a = x[kk][e] * inv * wv[e], b = x[kk][e + 1] * inv * wv[e + 1];
                qf[t][kk][e] = (bf16)((a * cv[e] - b * sv[e]) * fold);
                qf[t][kk][e + 1] = (bf16)((b * cv[e] + a * sv[e]) * fold);
            }
        }
    }

    f32x4 o_acc[8][2];
#pragma unroll
    for (int i = 0; i < 8; i++)
#pragma unroll
        for (int t = 0; t < 2; t++)
#pragma unroll
            for (int e = 0; e < 4; e++) o_acc[i][t][e] = 0.0f;
    /* m_run: reference maximum of the online softmax (base-2 logits). The score accumulators of
     * a tile are *initialised* with -m_run, so the MFMAs deliver s - m_run and the exponent needs
     * no subtraction; the first tile starts from 0 and is re-based when it is processed. */
    float m_run[2] = {0.0f, 0.0f};
    f32x4 s_acc[4][2];
    /* Row sums of P come from the matrix pipe too: one more 16-row block of "V^T" that is all
     * ones, so that every accumulator element of a lane is the sum, over the keys seen so far, of
     * the bf16 probabilities that also multiply V (4 MFMAs per tile instead of 32 additions). */
    f32x4 l_acc[2];
    bf16x8 ones;
#pragma unroll
    for (int e = 0; e < 8; e++) ones[e] = (bf16)1.0f;
#pragma unroll
    for (int u = 0; u < 2; u++)
#pragma unroll
        for (int e = 0; e < 4; e++) l_acc[u][e] = 0.0f;

    /* One key tile: S^T = K Q^T - m_run (32 MFMAs), online softmax, O^T += V^T P^T (32 MFMAs).
     * K(t) and V^T(t) sit in slot t%2 of their rings; the loads of tile t+1 are issued at the
     * top of the step and awaited at the top of the next one. Fragments are read from LDS one
     * block of four (8 MFMAs) ahead of their use; the first V^T block is requested before the
     * softmax so that its latency hides behind the exponentials. */
    auto step = [&](int t, auto edge_c) {
        constexpr bool EDGE = decltype(edge_c)::value; /* first or last tile: re-base the maximum, mask the ragged end */
        __builtin_amdgcn_s_waitcnt(0x0F70); /* vmcnt(0): this wave's parts of K(t), V(t) are in LDS */
        __syncthreads();
        if (t + 1 < ntiles) {
            issue_k(t + 1);
            issue_v(t + 1);
        }
        const char *kt = smem + (t & 1) * (64 * 256);
        const char *vtile = smem + 2 * (64 * 256) + (t & 1) * (128 * 128);
        auto kread = [&](int kk, bf16x8 (&dst)[4]) { /* 32 head dims, key blocks 0..3 */
#pragma unroll
            for (int i = 0; i < 4; i++) dst[i] = *(const bf16x8 *)(kt + (i * 16 + l15) * 256 + (((kk * 4 + lq) ^ l15) << 4));
        };
        auto vread = [&](int b, bf16x8 (&dst)[4]) { /* 32-key chunk b/2, head-dim blocks 4(b%2) .. +3 */
#pragma unroll
            for (int f = 0; f < 4; f++) {
                const int d = ((b & 1) * 4 + f) * 16 + l15;
                dst[f] = *(const bf16x8 *)(vtile + d * 128 + (((4 * (b >> 1) + lq) ^ vt_swz(d)) << 4));
            }
        };
        bf16x8 fa[4], fb[4];
        {
            f32x4 init[2];
#pragma unroll
            for (int u = 0; u < 2; u++)
#pragma unroll
                for (int e = 0; e < 4; e++) init[u][e] = -m_run[u];
            kread(0, fa);
            kread(1, fb);
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int kk = 0; kk < 4; kk++) {
                bf16x8 (&cur)[4] = (kk & 1) ? fb : fa;
#pragma unroll
                for (int i = 0; i < 4; i++)
#pragma unroll
                    for (int u = 0; u < 2; u++)
                        s_acc[i][u] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(cur[i], qf[u][kk], kk == 0 ? init[u] : s_acc[i][u], 0, 0, 0);
                __builtin_amdgcn_sched_barrier(0); /* keep the read distance: nothing moves across */
                if (kk + 2 < 4) kread(kk + 2, cur);
                __builtin_amdgcn_sched_barrier(0);
            }
        }
        vread(0, fa); /* in flight during the softmax */
        __builtin_amdgcn_sched_barrier(0);

        if (EDGE && t == ntiles - 1 && (seq_k & 63)) {
            const int key0 = t * 64;
#pragma unroll
            for (int i = 0; i < 4; i++)
#pragma unroll
                for (int e = 0; e < 4; e++)
                    if (key0 + 32 * (i >> 1) + 8 * lq + 4 * (i & 1) + e >= seq_k) { s_acc[i][0][e] = -1e30f; s_acc[i][1][e] = -1e30f; }
        }
        /* Online softmax; a query's scores sit in lanes l, l^16, l^32, l^48. The reference
         * maximum is only moved when a tile's maximum exceeds it by more than 2^8 (scores are
         * base-2 logits): until then p = 2^(s - m_run) <= 256 is exact enough in fp32/bf16, the
         * final division by the row sum cancels the choice of m_run, and the rescale of O -
         * 64 multiplies per lane - is skipped for almost every tile. The first tile takes its
         * own maximum as the reference. */
        bool grow = EDGE && t == 0;
        float m_new[2];
#pragma unroll
        for (int u = 0; u < 2; u++) {
            float mx = fmaxf(fmaxf(s_acc[0][u][0], s_acc[0][u][1]), fmaxf(s_acc[0][u][2], s_acc[0][u][3]));
#pragma unroll
            for (int i = 1; i < 4; i++) mx = fmaxf(fmaxf(mx, fmaxf(s_acc[i][u][0], s_acc[i][u][1])), fmaxf(s_acc[i][u][2], s_acc[i][u][3]));
            mx = fmaxf(mx, __shfl_xor(mx, 16, 64));
            mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
            m_new[u] = mx; /* relative to m_run */
            grow = grow || (mx > 8.0f);
        }
        if (__any(grow)) {
#pragma unroll
            for (int u = 0; u < 2; u++) {
                /* on the first tile the accumulators are still zero and stay so: the tile's maximum may lie
                 * far below zero, and 2^-d would then be infinite (0 * inf) */
                const bool first = EDGE && t == 0;
                const float d = first ? m_new[u] : fmaxf(m_new[u], 0.0f);
                const float alpha = first ? 1.0f : fast_exp2(-d);
                m_run[u] += d;
#pragma unroll
                for (int e = 0; e < 4; e++) l_acc[u][e] *= alpha;
#pragma unroll
                for (int i = 0; i < 4; i++)
#pragma unroll
                    for (int e = 0; e < 4; e++) s_acc[i][u][e] -= d;
#pragma unroll
                for (int i = 0; i < 8; i++)
#pragma unroll
                    for (int e = 0; e < 4; e++) o_acc[i][u][e] *= alpha;
            }
        }
        bf16x8 pf[2][2]; /* P^T as MFMA B fragments: [32-key chunk][query block] */
#pragma unroll
        for (int u = 0; u < 2; u++) {
#pragma unroll
            for (int i = 0; i < 4; i++)
#pragma unroll
                for (int e = 0; e < 4; e++) s_acc[i][u][e] = fast_exp2(s_acc[i][u][e]);
#pragma unroll
            for (int c = 0; c < 2; c++)
#pragma unroll
                for (int e = 0; e < 4; e++) {
                    pf[c][u][e] = (bf16)s_acc[2 * c][u][e];
                    pf[c][u][4 + e] = (bf16)s_acc[2 * c + 1][u][e];
                }
        }
        /* O^T += V^T P^T over two 32-key chunks, four blocks of 8 MFMAs; row sums first */
#pragma unroll
        for (int c = 0; c < 2; c++)
#pragma unroll
            for (int u = 0; u < 2; u++) l_acc[u] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ones, pf[c][u], l_acc[u], 0, 0, 0);
        __builtin_amdgcn_sched_barrier(0);
        vread(1, fb);
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int b = 0; b < 4; b++) {
            bf16x8 (&cur)[4] = (b & 1) ? fb : fa;
#pragma unroll
            for (int f = 0; f < 4; f++)
#pragma unroll
                for (int u = 0; u < 2; u++)
                    o_acc[(b & 1) * 4 + f][u] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(cur[f], pf[b >> 1][u], o_acc[(b & 1) * 4 + f][u], 0, 0, 0);
            __builtin_amdgcn_sched_barrier(0);
            if (b + 2 < 4) vread(b + 2, cur);
            __builtin_amdgcn_sched_barrier(0);
        }
    };

    step(0, AttFlag<true>{});
    for (int t = 1; t < ntiles - 1; t++) step(t, AttFlag<false>{});
    if (ntiles > 1) step(ntiles - 1, AttFlag<true>{});

#pragma unroll
    for (int u = 0; u < 2; u++) {
        const float inv_l = 1.0f / l_acc[u][0];
        if (qrow[u] < seq_q) {
            bf16 *op = out + (size_t)qrow[u] * ldo + h * HD + lq * 4;
#pragma unroll
            for (int dt = 0; dt < 8; dt++) {
                bf16x4 r;
#pragma unroll
                for (int e = 0; e < 4; e++) r[e] = (bf16)(o_acc[dt][u][e] * inv_l);
                *(bf16x4 *)(op + dt * 16) = r;
            }
        }
    }
}


/* ---------------------------------------------------------------------------------------
 * The same attention with 16 NQ queries per wave (NQ = 1 .. 4) and four waves, one per SIMD, per
 * workgroup: 64 NQ queries per workgroup. A K or V^T fragment read from LDS now feeds NQ MFMAs instead
 * of two, so a 64-query wave needs half the LDS bytes and fragment reads per FLOP of the 32-query
 * waves above. The price is registers - 32 NQ for the output accumulators, 16 NQ each for the scores
 * and the Q fragments - which is why there is one wave per SIMD and why the MFMAs are written as inline
 * assembly: the output accumulators and the Q fragments are pinned to AGPRs, the scores to VGPRs, and
 * nothing migrates between the register files (left to the register allocator, a kernel of this
 * shape moves some two hundred registers per key tile between them).
 * Hazards the compiler cannot see in inline assembly are kept apart by construction: the same
 * accumulator is written again only after at least four other MFMAs, and vector code reads MFMA
 * results only behind an explicit run of idle cycles (mfma_results_fence).
 * --------------------------------------------------------------------------------------- */
#define MFMA_ACC_A(acc, a, b) asm volatile("v_mfma_f32_16x16x32_bf16 %0, %1, %2, %0" : "+a"(acc) : "v"(a), "v"(b))
#define MFMA_ACC_V(acc, a, b) asm volatile("v_mfma_f32_16x16x32_bf16 %0, %1, %2, %0" : "+v"(acc) : "v"(a), "v"(b))
#define MFMA_ACC_VQ(acc, a, q) asm volatile("v_mfma_f32_16x16x32_bf16 %0, %1, %2, %0" : "+v"(acc) : "v"(a), "a"(q))
#define MFMA_NEW_VQ(acc, a, q, c) asm volatile("v_mfma_f32_16x16x32_bf16 %0, %1, %2, %3" : "=&v"(acc) : "v"(a), "a"(q), "v"(c))
/* Guarded forms, for MFMAs whose operands a vector instruction may have written just before (the bf16
 * probabilities, a start value the compiler re-creates, a register copy it slips in): two idle issue slots travel
 * inside the statement, so nothing can come between them and the MFMA. */
#define MFMA_NEW_VQ_GUARDED(acc, a, q, c) \
    asm volatile("s_nop 1\n\tv_mfma_f32_16x16x32_bf16 %0, %1, %2, %3" : "=&v"(acc) : "v"(a), "a"(q), "v"(c))
#define MFMA_ACC_V_ONES_GUARDED(acc, ones, b) asm volatile("s_nop 1\n\tv_mfma_f32_16x16x32_bf16 %0, %1, %2, %0" : "+v"(acc) : "a"(ones), "v"(b))

/* Idle cycles until the last MFMAs have written their results, then every listed accumulator passes
 * through an empty asm statement ordered with the MFMAs, so that reads of them stay behind it. */
template <int N>
__device__ __forceinline__ void mfma_results_fence_v(f32x4 (&acc)[4][N]) {
    asm volatile("s_nop 7\n\ts_nop 7" ::: "memory");
#pragma unroll
    for (int i = 0; i < 4; i++)
#pragma unroll
        for (int j = 0; j < N; j++) asm volatile("" : "+v"(acc[i][j]));
}
template <int N>
__device__ __forceinline__ void mfma_results_fence_a(f32x4 (&acc)[8][N]) {
    asm volatile("s_nop 7\n\ts_nop 7" ::: "memory");
#pragma unroll
    for (int i = 0; i < 8; i++)
#pragma unroll
        for (int j = 0; j < N; j++) asm volatile("" : "+a"(acc[i][j]));
}

template <int NQ>
__global__ __launch_bounds__(256, 1) void attention_wide_kernel(bf16 *__restrict__ out, int ldo, const bf16 *__restrict__ q, int ldq,
                                                                const bf16 *__restrict__ k, const bf16 *__restrict__ vt, int ld_vt,
                                                                int seq_q, int seq_k, int heads, int split,
                                                                const float *__restrict__ q_w0, const float *__restrict__ q_w1,
                                                                const float *__restrict__ rope_cos, const float *__restrict__ rope_sin,
                                                                float eps) {
    extern __shared__ __attribute__((aligned(16))) char smem[];
    constexpr int NW = 4, WQ = 16 * NQ, BQ = NW * WQ, LP = 16 / NW;
    /* every XCD gets a contiguous run of (head, query block) pairs, as above */
    const int nqb = (seq_q + BQ - 1) / BQ;
    const int logical = (blockIdx.x & 7) * (gridDim.x >> 3) + (blockIdx.x >> 3);
    if (logical >= nqb * heads) return;
    const int h = logical / nqb, qb = logical - h * nqb;
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int l15 = lane & 15, lq = lane >> 4;
    const int H = heads * HD;

    /* ---- tile loader: as in attention_kernel<4> ---- */
    const int ntiles = (seq_k + 63) >> 6;
    const bf16 *k_src[LP];
    const bf16 *v_src[LP];
    int k_dst[LP], v_dst[LP], k_row[LP];
#pragma unroll
    for (int i = 0; i < LP; i++) {
        int r = wave * 4 + i * (NW * 4) + (lane >> 4);
        {
            int ib = r >> 4, jj = (r >> 2) & 3, ee = r & 3;
            k_row[i] = 32 * (ib >> 1) + 8 * jj + 4 * (ib & 1) + ee;
        }
        k_src[i] = k + h * HD + (((lane & 15) ^ (r & 15)) << 3);
        k_dst[i] = (wave * 4 + i * (NW * 4)) * 256;
        int d = wave * 8 + i * (NW * 8) + (lane >> 3);
        v_src[i] = vt + (size_t)(h * HD + d) * ld_vt + (((lane & 7) ^ vt_swz(d)) << 3);
        v_dst[i] = (wave * 8 + i * (NW * 8)) * 128;
    }
    auto issue_k = [&](int t) {
        char *base = smem + (t & 1) * (64 * 256);
        const int key0 = t * 64;
#pragma unroll
        for (int i = 0; i < LP; i++) {
            int r = min(key0 + k_row[i], seq_k - 1);
            __builtin_amdgcn_global_load_lds(GLOBAL_PTR(k_src[i] + (size_t)r * H), LDS_PTR(base + k_dst[i]), 16, 0, 0);
        }
    };
    auto issue_v = [&](int t) {
        char *base = smem + 2 * (64 * 256) + (t & 1) * (128 * 128);
        const int key0 = t * 64;
#pragma unroll
        for (int i = 0; i < LP; i++)
            __builtin_amdgcn_global_load_lds(GLOBAL_PTR(v_src[i] + key0), LDS_PTR(base + v_dst[i]), 16, 0, 0);
    };
    issue_k(0);
    issue_v(0);

    /* ---- Q fragments (B operand) with RMSNorm * weight, RoPE and the softmax scale; they live in AGPRs ---- */
    bf16x8 qf[NQ][4];
    int qrow[NQ];
#pragma unroll
    for (int t = 0; t < NQ; t++) {
        qrow[t] = qb * BQ + wave * WQ + t * 16 + l15;
        const int qrc = min(qrow[t], seq_q - 1);
        const bf16 *qp = q + (size_t)qrc * ldq + h * HD + lq * 8;
        float x[4][8];
        float ss = 0.0f;
#pragma unroll
        for (int kk = 0; kk < 4; kk++) {
            bf16x8 v = *(const bf16x8 *)(qp + kk * 32);
#pragma unroll
            for (int e = 0; e < 8; e++) { x[kk][e] = (float)v[e]; ss += x[kk][e] * x[kk][e]; }
        }
        ss += __shfl_xor(ss, 16, 64);
        ss += __shfl_xor(ss, 32, 64);
        const float inv = 1.0f / sqrtf(ss * (1.0f / HD) + eps);
        const float fold = 0.08838834764831845f * 1.44269504088896341f; /* 1/sqrt(128) and log2(e): scores are base-2 logits */
        const float *w = (qrc < split ? q_w0 : q_w1) + lq * 8;
        const float *cs = rope_cos + (size_t)qrc * HD + lq * 8;
        const float *sn = rope_sin + (size_t)qrc * HD + lq * 8;
#pragma unroll
        for (int kk = 0; kk < 4; kk++) {
            f32x4 w0 = *(const f32x4 *)(w + kk * 32), w1 = *(const f32x4 *)(w + kk * 32 + 4);
            f32x4 c0 = *(const f32x4 *)(cs + kk * 32), c1 = *(const f32x4 *)(cs + kk * 32 + 4);
            f32x4 s0 = *(const f32x4 *)(sn + kk * 32), s1 = *(const f32x4 *)(sn + kk * 32 + 4);
            float wv[8] = {w0[0], w0[1], w0[2], w0[3], w1[0], w1[1], w1[2], w1[3]};
            float cv[8] = {c0[0], c0[1], c0[2], c0[3], c1[0], c1[1], c1[2], c1[3]};
            float sv[8] = {s0[0], s0[1], s0[2], s0[3], s1[0], s1[1], s1[2], s1[3]};
#pragma unroll
            for (int e = 0; e < 8; e += 2) {
                float a = x[kk][e] * inv * wv[e], b = x[kk][e + 1] * inv * wv[e + 1];
                qf[t][kk][e] = (bf16)((a * cv[e] - b * sv[e]) * fold);
                qf[t][kk][e + 1] = (bf16)((b * cv[e] + a * sv[e]) * fold);
            }
            asm volatile("" : "+a"(qf[t][kk])); /* one aligned AGPR quad per fragment from here on */
        }
    }

    f32x4 o_acc[8][NQ]; /* AGPRs */
#pragma unroll
    for (int i = 0; i < 8; i++)
#pragma unroll
        for (int j = 0; j < NQ; j++)
#pragma unroll
            for (int e = 0; e < 4; e++) o_acc[i][j][e] = 0.0f;
    /* neg_m: minus the reference maximum of the online softmax, four copies per query block: the start value
     * of the score accumulators (see attention_kernel) */
    f32x4 neg_m[NQ];
    f32x4 l_acc[NQ];
#pragma unroll
    for (int j = 0; j < NQ; j++) {
#pragma unroll
        for (int e = 0; e < 4; e++) { neg_m[j][e] = 0.0f; l_acc[j][e] = 0.0f; }
    }
    bf16x8 ones;
#pragma unroll
    for (int e = 0; e < 8; e++) ones[e] = (bf16)1.0f;
    /* from here on a value the compiler cannot re-create: it stays in four AGPRs instead of being written anew
     * right in front of the MFMA that reads it (the compiler does not know that its inline assembly is an MFMA,
     * which must not read a register in the two issue slots after a vector instruction wrote it) */
    asm volatile("" : "+a"(ones));
    f32x4 s_acc[4][NQ];

    /* One key tile, as in attention_kernel: S^T = K Q^T - m_run (16 NQ MFMAs), online softmax with the lazily
     * moved maximum, O^T += V^T P^T (16 NQ MFMAs) and the row sums (2 NQ). */
    auto step = [&](int t, auto edge_c) {
        constexpr bool EDGE = decltype(edge_c)::value;
        __builtin_amdgcn_s_waitcnt(0x0F70);
        __syncthreads();
        if (t + 1 < ntiles) {
            issue_k(t + 1);
            issue_v(t + 1);
        }
        const char *kt = smem + (t & 1) * (64 * 256);
        const char *vtile = smem + 2 * (64 * 256) + (t & 1) * (128 * 128);
        auto kread = [&](int kk, bf16x8 (&dst)[4]) {
#pragma unroll
            for (int i = 0; i < 4; i++) dst[i] = *(const bf16x8 *)(kt + (i * 16 + l15) * 256 + (((kk * 4 + lq) ^ l15) << 4));
        };
        auto vread = [&](int b, bf16x8 (&dst)[4]) {
#pragma unroll
            for (int f = 0; f < 4; f++) {
                const int d = ((b & 1) * 4 + f) * 16 + l15;
                dst[f] = *(const bf16x8 *)(vtile + d * 128 + (((4 * (b >> 1) + lq) ^ vt_swz(d)) << 4));
            }
        };
        bf16x8 fa[4], fb[4];
        {
            kread(0, fa);
            kread(1, fb);
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int kk = 0; kk < 4; kk++) {
                bf16x8 (&cur)[4] = (kk & 1) ? fb : fa;
#pragma unroll
                for (int i = 0; i < 4; i++)
#pragma unroll
                    for (int j = 0; j < NQ; j++) {
                        if (kk == 0 && i == 0) MFMA_NEW_VQ_GUARDED(s_acc[i][j], cur[i], qf[j][0], neg_m[j]); /* first reader of neg_m[j] */
                        else if (kk == 0) MFMA_NEW_VQ(s_acc[i][j], cur[i], qf[j][0], neg_m[j]);
                        else MFMA_ACC_VQ(s_acc[i][j], cur[i], qf[j][kk]);
                    }
                __builtin_amdgcn_sched_barrier(0);
                if (kk + 2 < 4) kread(kk + 2, cur);
                __builtin_amdgcn_sched_barrier(0);
            }
        }
        vread(0, fa); /* in flight during the softmax */
        __builtin_amdgcn_sched_barrier(0);
        mfma_results_fence_v<NQ>(s_acc);

        if (EDGE && t == ntiles - 1 && (seq_k & 63)) {
            const int key0 = t * 64;
#pragma unroll
            for (int i = 0; i < 4; i++)
#pragma unroll
                for (int e = 0; e < 4; e++)
                    if (key0 + 32 * (i >> 1) + 8 * lq + 4 * (i & 1) + e >= seq_k) {
#pragma unroll
                        for (int j = 0; j < NQ; j++) s_acc[i][j][e] = -1e30f;
                    }
        }
        bool grow = EDGE && t == 0;
        float m_new[NQ];
#pragma unroll
        for (int j = 0; j < NQ; j++) {
            float mx = fmaxf(fmaxf(s_acc[0][j][0], s_acc[0][j][1]), fmaxf(s_acc[0][j][2], s_acc[0][j][3]));
#pragma unroll
            for (int i = 1; i < 4; i++) mx = fmaxf(fmaxf(mx, fmaxf(s_acc[i][j][0], s_acc[i][j][1])), fmaxf(s_acc[i][j][2], s_acc[i][j][3]));
            m_new[j] = mx; /* this lane's keys only; relative to m_run */
            grow = grow || (mx > 8.0f);
        }
        if (__any(grow)) {
            /* rare: some score lies more than 2^8 above the reference (or this is the first tile). The exact row
             * maxima (a query's scores sit in lanes l, l^16, l^32, l^48) move the references; see attention_kernel. */
            if (t > 0) mfma_results_fence_a<NQ>(o_acc);
#pragma unroll
            for (int j = 0; j < NQ; j++) {
                float mx = m_new[j];
                mx = fmaxf(mx, __shfl_xor(mx, 16, 64));
                mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
                const bool first = EDGE && t == 0;
                const float d = first ? mx : fmaxf(mx, 0.0f);
                const float alpha = first ? 1.0f : fast_exp2(-d);
#pragma unroll
                for (int e = 0; e < 4; e++) { neg_m[j][e] -= d; l_acc[j][e] *= alpha; }
#pragma unroll
                for (int i = 0; i < 4; i++)
#pragma unroll
                    for (int e = 0; e < 4; e++) s_acc[i][j][e] -= d;
#pragma unroll
                for (int i = 0; i < 8; i++)
#pragma unroll
                    for (int e = 0; e < 4; e++) o_acc[i][j][e] *= alpha;
            }
        }
        bf16x8 pf[2][NQ];
#pragma unroll
        for (int j = 0; j < NQ; j++) {
#pragma unroll
            for (int i = 0; i < 4; i++)
#pragma unroll
                for (int e = 0; e < 4; e++) s_acc[i][j][e] = fast_exp2(s_acc[i][j][e]);
#pragma unroll
            for (int c = 0; c < 2; c++)
#pragma unroll
                for (int e = 0; e < 4; e++) {
                    pf[c][j][e] = (bf16)s_acc[2 * c][j][e];
                    pf[c][j][4 + e] = (bf16)s_acc[2 * c + 1][j][e];
                }
        }
        __builtin_amdgcn_sched_barrier(0);
        /* the row sums are the first readers of each probability fragment */
#pragma unroll
        for (int j = 0; j < NQ; j++) MFMA_ACC_V_ONES_GUARDED(l_acc[j], ones, pf[0][j]);
        __builtin_amdgcn_sched_barrier(0);
        vread(1, fb);
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int b = 0; b < 4; b++) {
            bf16x8 (&cur)[4] = (b & 1) ? fb : fa;
            if (b == 2) {
#pragma unroll
                for (int j = 0; j < NQ; j++) MFMA_ACC_V_ONES_GUARDED(l_acc[j], ones, pf[1][j]);
            }
#pragma unroll
            for (int f = 0; f < 4; f++)
#pragma unroll
                for (int j = 0; j < NQ; j++) MFMA_ACC_A(o_acc[(b & 1) * 4 + f][j], cur[f], pf[b >> 1][j]);
            __builtin_amdgcn_sched_barrier(0);
            if (b + 2 < 4) vread(b + 2, cur);
            __builtin_amdgcn_sched_barrier(0);
        }
    };

    step(0, AttFlag<true>{});
    for (int t = 1; t < ntiles - 1; t++) step(t, AttFlag<false>{});
    if (ntiles > 1) step(ntiles - 1, AttFlag<true>{});

    mfma_results_fence_a<NQ>(o_acc);
    asm volatile("s_nop 7\n\ts_nop 7" ::: "memory");
#pragma unroll
    for (int j = 0; j < NQ; j++) asm volatile("" : "+v"(l_acc[j]));
#pragma unroll
    for (int j = 0; j < NQ; j++) {
        const float inv_l = 1.0f / l_acc[j][0];
        if (qrow[j] < seq_q) {
            bf16 *op = out + (size_t)qrow[j] * ldo + h * HD + lq * 4;
#pragma unroll
            for (int dt = 0; dt < 8; dt++) {
                bf16x4 r;
#pragma unroll
                for (int e = 0; e < 4; e++) r[e] = (bf16)(o_acc[dt][j][e] * inv_l);
                *(bf16x4 *)(op + dt * 16) = r;
            }
        }
    }
}

static int g_att_force = -1;
extern "C" void flux_hip_attention_force_variant(int v) { g_att_force = v; }

extern "C" int flux_hip_attention(void *out_bf16, int ldo, const void *q, int ldq, const void *k, const void *vt,
                                  int ld_vt, int seq_q, int seq_k, int heads, int split, const float *q_w0,
                                  const float *q_w1, const float *rope_cos, const float *rope_sin, float eps) {
    if (seq_q <= 0) return 1;
    if (seq_k <= 0) return flux_hip_fail("flux_hip_attention: seq_k=%d", seq_k);
    if (!out_bf16 || !q || !k || !vt || !q_w0 || !rope_cos || !rope_sin) return flux_hip_fail("flux_hip_attention: NULL argument");
    if (split < seq_q && !q_w1) return flux_hip_fail("flux_hip_attention: second weight missing");
    if ((((uintptr_t)q | (uintptr_t)k | (uintptr_t)vt | (uintptr_t)q_w0 | (uintptr_t)q_w1 | (uintptr_t)rope_cos | (uintptr_t)rope_sin) & 15) ||
        ((uintptr_t)out_bf16 & 7))
        return flux_hip_fail("flux_hip_attention: operands must be 16-byte aligned (output 8-byte)");
    if ((ldo & 3) || (ldq & 7) || (ld_vt & 7) || ld_vt < (seq_k + 63) / 64 * 64)
        return flux_hip_fail("flux_hip_attention: bad leading dimensions (ldo=%d ldq=%d ld_vt=%d)", ldo, ldq, ld_vt);
    /* 256-query workgroups (8 waves) share each K / V^T tile among twice as many queries;
     * 128-query workgroups (two per CU) balance better when there are few of them. */
    const int big = g_att_force >= 0 ? g_att_force : (((seq_q + 255) / 256) * heads >= 256);
    static bool attr_done = false;
    if (!attr_done) {
        HIP_OK(hipFuncSetAttribute((const void *)attention_wide_kernel<1>, hipFuncAttributeMaxDynamicSharedMemorySize, 2 * ATT_STAGE));
        HIP_OK(hipFuncSetAttribute((const void *)attention_wide_kernel<2>, hipFuncAttributeMaxDynamicSharedMemorySize, 2 * ATT_STAGE));
        HIP_OK(hipFuncSetAttribute((const void *)attention_wide_kernel<3>, hipFuncAttributeMaxDynamicSharedMemorySize, 2 * ATT_STAGE));
        HIP_OK(hipFuncSetAttribute((const void *)attention_wide_kernel<4>, hipFuncAttributeMaxDynamicSharedMemorySize, 2 * ATT_STAGE));
        HIP_OK(hipFuncSetAttribute((const void *)attention_kernel<4>, hipFuncAttributeMaxDynamicSharedMemorySize, 2 * ATT_STAGE));
        HIP_OK(hipFuncSetAttribute((const void *)attention_kernel<8>, hipFuncAttributeMaxDynamicSharedMemorySize, 2 * ATT_STAGE));
        attr_done = true;
    }
    if (big >= 11 && big <= 14) {
        /* 16 NQ queries per wave, four waves per workgroup (variants 11 .. 14 = NQ 1 .. 4) */
        const int nq = big - 10, bq = 64 * nq;
        const int blocks = ((seq_q + bq - 1) / bq) * heads;
        auto kern = nq == 1 ? attention_wide_kernel<1> : nq == 2 ? attention_wide_kernel<2> : nq == 3 ? attention_wide_kernel<3> : attention_wide_kernel<4>;
        hipLaunchKernelGGL(kern, dim3((blocks + 7) & ~7), dim3(256), 2 * ATT_STAGE, flux_hip_stream_handle(),
                           (bf16 *)out_bf16, ldo, (const bf16 *)q, ldq, (const bf16 *)k, (const bf16 *)vt, ld_vt, seq_q, seq_k,
                           heads, split, q_w0, q_w1 ? q_w1 : q_w0, rope_cos, rope_sin, eps);
    } else if (big) {
        const int blocks = ((seq_q + 255) / 256) * heads;
        hipLaunchKernelGGL(attention_kernel<8>, dim3((blocks + 7) & ~7), dim3(512), 2 * ATT_STAGE, flux_hip_stream_handle(),
                           (bf16 *)out_bf16, ldo, (const bf16 *)q, ldq, (const bf16 *)k, (const bf16 *)vt, ld_vt, seq_q, seq_k,
                           heads, split, q_w0, q_w1 ? q_w1 : q_w0, rope_cos, rope_sin, eps);
    } else {
        const int blocks = ((seq_q + 127) / 128) * heads;
        hipLaunchKernelGGL(attention_kernel<4>, dim3((blocks + 7) & ~7), dim3(256), 2 * ATT_STAGE, flux_hip_stream_handle(),
                           (bf16 *)out_bf16, ldo, (const bf16 *)q, ldq, (const bf16 *)k, (const bf16 *)vt, ld_vt, seq_q, seq_k,
                           heads, split, q_w0, q_w1 ? q_w1 : q_w0, rope_cos, rope_sin, eps);
    }
    HIP_OK(hipGetLastError());
    return 1;
}
