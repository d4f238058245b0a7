/*
 * attention.hip - joint text+image attention for gfx950: a K preparation pass and a
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
 * loaded (the loader picks which key goes to which LDS row). V is taken row-major, straight from
 * the projection's output: the "A" operand V^T of the second product is read from the LDS tile with
 * transposing reads (ds_read_b64_tr_b16), so no transposed copy of V is ever written.
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
 * Q/K preparation. One workgroup handles 16 tokens of 1 to 12 heads, Q and K: RMSNorm over the 128 dims *
 * weight, then rotation of pairs (d, d+1) by the token's cos/sin row.
 * K is written token-major to k_out. Q is written back in place, already multiplied by
 * 1/sqrt(128) and log2(e), so that the attention kernel's scores are base-2 logits and its Q
 * fragments are plain loads. (The same arithmetic inside the attention kernel, where a lane owns a
 * query row, read the cos/sin rows 16 bytes per lane and row: a fifth of a workgroup's time at 4608
 * tokens went into those loads. Here 16 lanes share a row.) V needs no preparation: the attention
 * kernel reads it where the projection wrote it.
 * --------------------------------------------------------------------------------------- */
#define Q_FOLD (0.08838834764831845f * 1.44269504088896341f)
/* norm * weight, RoPE and scale of one 8-dim chunk whose squared sum over the row's 16 lanes is already in ss */
__device__ __forceinline__ bf16x8 qk_prepare_chunk(const float (&x)[8], float ss, float eps, const float (&wv)[8], const float (&cv)[8],
                                                   const float (&sv)[8], float scale) {
    const float inv = 1.0f / sqrtf(ss * (1.0f / HD) + eps);
    bf16x8 o;
#pragma unroll
    for (int e = 0; e < 8; e += 2) {
        float a = x[e] * inv * wv[e], b = x[e + 1] * inv * wv[e + 1];
        o[e] = (bf16)((a * cv[e] - b * sv[e]) * scale);
        o[e + 1] = (bf16)((b * cv[e] + a * sv[e]) * scale);
    }
    return o;
}
/* A thread owns one 8-dim chunk of one token (16 lanes share the token's row of a head) and walks HG heads with it:
 * the token's cos/sin chunk and the two norm weights' chunks are read once and serve every head's Q and K (read per head,
 * as an earlier version did, the tables were 113 MB of L2 traffic per call at 4608 tokens, as much as Q and K
 * themselves). UN heads are requested before the first of them is used. With few tokens fewer heads per thread, so
 * that the launch still has a few hundred workgroups. */
template <int HG, int UN>
__global__ __launch_bounds__(256) void qk_prepare_kernel(bf16 *__restrict__ k_out, bf16 *qkv, int ld, int q_col, int k_col,
                                                         int rows, int heads, int split,
                                                         const float *__restrict__ q_w0, const float *__restrict__ q_w1,
                                                         const float *__restrict__ k_w0, const float *__restrict__ k_w1,
                                                         const float *__restrict__ rope_cos,
                                                         const float *__restrict__ rope_sin, float eps) {
    const int tid = threadIdx.x;
    const int c = tid & 15; /* 16-byte chunk of the 128-dim head row */
    const int row = blockIdx.x * 16 + (tid >> 4), rowc = min(row, rows - 1);
    const int h0 = blockIdx.y * HG, h1 = min(h0 + HG, heads);
    const int H = heads * HD;
    bf16 *qp = qkv + (size_t)rowc * ld + q_col + c * 8;
    const bf16 *kp = qkv + (size_t)rowc * ld + k_col + c * 8;
    bf16 *ko = k_out + (size_t)rowc * H + c * 8;
    float cv[8], sv[8], wq[8], wk[8];
    {
        const float *cs = rope_cos + (size_t)rowc * HD + c * 8, *sn = rope_sin + (size_t)rowc * HD + c * 8;
        const bool first = rowc < split;
        const float *a = (first ? q_w0 : q_w1) + c * 8, *b = (first ? k_w0 : k_w1) + c * 8;
        const f32x4 c0 = *(const f32x4 *)cs, c1 = *(const f32x4 *)(cs + 4), s0 = *(const f32x4 *)sn, s1 = *(const f32x4 *)(sn + 4);
        const f32x4 a0 = *(const f32x4 *)a, a1 = *(const f32x4 *)(a + 4), b0 = *(const f32x4 *)b, b1 = *(const f32x4 *)(b + 4);
#pragma unroll
        for (int e = 0; e < 4; e++) {
            cv[e] = c0[e]; cv[4 + e] = c1[e]; sv[e] = s0[e]; sv[4 + e] = s1[e];
            wq[e] = a0[e]; wq[4 + e] = a1[e]; wk[e] = b0[e]; wk[4 + e] = b1[e];
        }
    }
    for (int hb = h0; hb < h1; hb += UN) {
        bf16x8 qv[UN], kv[UN];
#pragma unroll
        for (int u = 0; u < UN; u++) {
            const int h = min(hb + u, h1 - 1);
            qv[u] = *(const bf16x8 *)(qp + h * HD);
            kv[u] = *(const bf16x8 *)(kp + h * HD);
        }
#pragma unroll
        for (int u = 0; u < UN; u++) {
            float xq[8], xk[8];
            float sq = 0.0f, sk = 0.0f;
#pragma unroll
            for (int e = 0; e < 8; e++) {
                xq[e] = (float)qv[u][e]; sq += xq[e] * xq[e];
                xk[e] = (float)kv[u][e]; sk += xk[e] * xk[e];
            }
            sq = wave16_sum(sq);
            sk = wave16_sum(sk);
            const bf16x8 oq = qk_prepare_chunk(xq, sq, eps, wq, cv, sv, Q_FOLD);
            const bf16x8 ok = qk_prepare_chunk(xk, sk, eps, wk, cv, sv, 1.0f);
            if (row < rows && hb + u < h1) {
                *(bf16x8 *)(qp + (hb + u) * HD) = oq;
                *(bf16x8 *)(ko + (hb + u) * HD) = ok;
            }
        }
    }
}

extern "C" int flux_hip_qk_prepare(void *k_out, void *qkv, int ld, int q_col, int k_col, int rows, int heads, int split,
                                   const float *q_w0, const float *q_w1, const float *k_w0, const float *k_w1,
                                   const float *rope_cos, const float *rope_sin, float eps) {
    if (rows <= 0) return 1;
    if (!k_out || !qkv || !q_w0 || !k_w0 || !rope_cos || !rope_sin) return flux_hip_fail("flux_hip_qk_prepare: NULL argument");
    if (split < rows && (!q_w1 || !k_w1)) return flux_hip_fail("flux_hip_qk_prepare: second weight missing");
    if ((ld & 7) || (q_col & 7) || (k_col & 7)) return flux_hip_fail("flux_hip_qk_prepare: ld, q_col and k_col must be multiples of 8");
    if (q_col + heads * HD > ld || k_col + heads * HD > ld || (q_col < k_col + heads * HD && k_col < q_col + heads * HD))
        return flux_hip_fail("flux_hip_qk_prepare: Q and K columns (%d, %d; %d wide) do not fit ld=%d or overlap", q_col, k_col, heads * HD, ld);
    if (((uintptr_t)k_out | (uintptr_t)qkv | (uintptr_t)q_w0 | (uintptr_t)q_w1 | (uintptr_t)k_w0 | (uintptr_t)k_w1 | (uintptr_t)rope_cos |
         (uintptr_t)rope_sin) & 15)
        return flux_hip_fail("flux_hip_qk_prepare: operands must be 16-byte aligned");
    {
        /* K goes to k_out while the same launch still reads and rewrites qkv: the two must not overlap */
        const uintptr_t a0 = (uintptr_t)qkv, a1 = a0 + (size_t)rows * ld * 2, b0 = (uintptr_t)k_out, b1 = b0 + (size_t)rows * heads * HD * 2;
        if (a0 < b1 && b0 < a1) return flux_hip_fail("flux_hip_qk_prepare: k_out overlaps the qkv buffer");
    }
    /* as many heads per thread as leave the launch some five hundred workgroups */
    const int rb = (rows + 15) / 16;
    const int hg = rb * ((heads + 11) / 12) >= 512 ? 12 : rb * ((heads + 3) / 4) >= 512 ? 4 : rb * ((heads + 1) / 2) >= 512 ? 2 : 1;
    auto kern = hg == 12 ? qk_prepare_kernel<12, 6> : hg == 4 ? qk_prepare_kernel<4, 4> : hg == 2 ? qk_prepare_kernel<2, 2> : qk_prepare_kernel<1, 1>;
    hipLaunchKernelGGL(kern, dim3(rb, (heads + hg - 1) / hg), dim3(256), 0, flux_hip_stream_handle(),
                       (bf16 *)k_out, (bf16 *)qkv, ld, q_col, k_col, rows, heads, split, q_w0, q_w1 ? q_w1 : q_w0, k_w0, k_w1 ? k_w1 : k_w0,
                       rope_cos, rope_sin, eps);
    HIP_OK(hipGetLastError());
    return 1;
}

/* ---------------------------------------------------------------------------------------
 * Flash attention. Workgroup = 4 or 8 waves = 128 or 256 queries of one head; a wave owns 32
 * queries (two 16-query MFMA columns) and the full head dimension. Keys are walked in tiles of 64
 * through two LDS stages filled by direct global->LDS loads (no register staging).
 *   LDS stage: K tile [64 keys][128 d] (256-byte rows, 16-byte chunks XOR-swizzled by key%16)
 *              V tile [64 keys][128 d] (256-byte rows, 16-byte chunk c of key r at position c ^ 2 (r%4) ^ (r&8))
 * MFMA: v_mfma_f32_16x16x32_bf16 (the form that sustains the most under the power limit).
 *   S^T[key][q]: A = K fragment (lane: key l%16, dims 8(l/16)..+8 of a 32-dim chunk),
 *                B = Q fragment (lane: query l%16, same dims); accumulator lane: query l%16,
 *                keys 4(l/16)..+4 of the 16-key block.
 *   O^T[d][q]:   B = P^T fragment for 32 keys = the accumulators of two 16-row score blocks;
 *                the K rows are permuted when the tile is loaded so that these are 8
 *                consecutive keys per lane, and A = V^T fragment (lane: dim l%16 of a 16-dim block,
 *                keys 8(l/16)..+8 of the chunk) is two transposing LDS reads of four keys each.
 * A transposing read works in groups of 16 lanes: lane 4 e + t of the group points at four
 * consecutive dims (quad t of a 16-dim block) of key e of four keys, and lane j of the group receives
 * dim j of the block for those four keys. The four keys' rows lie 256 bytes apart, i.e. on the same
 * banks; the swizzle moves each row's 32-byte piece of a block to a different bank group, and the
 * pieces of the rows eight further on (the next group of 16 lanes, served in the same cycle) to
 * the other half of the 256 bytes.
 * --------------------------------------------------------------------------------------- */
#define ATT_STAGE (64 * 256 + 64 * 256)
#define ATT_WIDE_LDS (8 * 16384) /* attention_wide_kernel: four K and four V slots */
#define GLOBAL_PTR(p) ((const __attribute__((address_space(1))) void *)(p))
#define LDS_PTR(p) ((__attribute__((address_space(3))) void *)(p))
typedef short s16x4 __attribute__((ext_vector_type(4)));
typedef short s16x8 __attribute__((ext_vector_type(8)));
/* Half a V^T fragment: one transposing read, four keys of this lane's dim. */
__device__ __forceinline__ s16x4 v_half_fragment(const char *p) {
    return __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) s16x4 *)LDS_PTR(p));
}
/* The same from an LDS byte address (what a pointer into LDS is, as a number). */
__device__ __forceinline__ s16x4 v_half_fragment_at(unsigned lds_addr) {
    return __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) s16x4 *)(uintptr_t)lds_addr);
}
__device__ __forceinline__ bf16x8 lds_read_bf16x8(unsigned lds_addr) {
    return *(const __attribute__((address_space(3))) bf16x8 *)(uintptr_t)lds_addr;
}
__device__ __forceinline__ bf16x8 v_join(s16x4 lo, s16x4 hi) {
    const s16x8 both = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
    return __builtin_bit_cast(bf16x8, both);
}
/* The V^T fragment of eight keys from two transposing reads 1024 bytes (four key rows) apart. */
__device__ __forceinline__ bf16x8 v_fragment(const char *p) { return v_join(v_half_fragment(p), v_half_fragment(p + 1024)); }

template <bool V> struct AttFlag { static constexpr bool value = V; };
template <int V> struct AttInt { static constexpr int value = V; };

/* One workgroup's work: the queries [q_begin, q_end) of head h, at most 32 NW of them. All NW waves must call it. */
template <int NW>
__device__ __forceinline__ void attention_block(char *smem, const int h, const int q_begin, const int q_end, bf16 *__restrict__ out, int ldo,
                                const bf16 *__restrict__ q, int ldq, const bf16 *__restrict__ k, const bf16 *__restrict__ v, int ldv,
                                int seq_k, int heads) {
    constexpr int LP = 16 / NW;  /* wave-wide load instructions per wave and tile, for K and for V */
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int l15 = lane & 15, lq = lane >> 4;
    const int H = heads * HD;

    /* ---- tile loader: per-lane global sources (un-swizzled) and per-wave LDS destinations ---- */
    const int ntiles = (seq_k + 63) >> 6;
    const bf16 *k_src[LP];
    const bf16 *v_src[LP];
    int k_dst[LP], k_row[LP];
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
        /* V: the same four rows, keys in their natural order (LDS row r = key r of the tile) */
        v_src[i] = v + h * HD + (((lane & 15) ^ (2 * (r & 3)) ^ (r & 8)) << 3);
    }
    /* LDS: K ring = 2 slots of 16 KB at 0 and 16 KB; V ring = 2 slots of 16 KB at 32 and 48 KB */
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
        char *base = smem + 2 * (64 * 256) + (t & 1) * (64 * 256);
        const int key0 = t * 64;
#pragma unroll
        for (int i = 0; i < LP; i++) {
            int r = min(key0 + wave * 4 + i * (NW * 4) + (lane >> 4), seq_k - 1); /* beyond the end: any finite row (its probabilities are 0) */
            __builtin_amdgcn_global_load_lds(GLOBAL_PTR(v_src[i] + (size_t)r * ldv), LDS_PTR(base + k_dst[i]), 16, 0, 0);
        }
    };
    issue_k(0);
    issue_v(0);

    /* ---- Q fragments (B operand): prepared by qk_prepare_kernel (norm, RoPE, softmax scale), loaded as they are ---- */
    bf16x8 qf[2][4];
    int qrow[2];
#pragma unroll
    for (int t = 0; t < 2; t++) {
        qrow[t] = q_begin + wave * 32 + t * 16 + l15;
        const bf16 *qp = q + (size_t)min(qrow[t], q_end - 1) * ldq + h * HD + lq * 8;
#pragma unroll
        for (int kk = 0; kk < 4; kk++) qf[t][kk] = *(const bf16x8 *)(qp + kk * 32);
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
     * K(t) and V(t) sit in slot t%2 of their rings; the loads of tile t+1 are issued at the
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
        const char *vtile = smem + 2 * (64 * 256) + (t & 1) * (64 * 256);
        auto kread = [&](int kk, bf16x8 (&dst)[4]) { /* 32 head dims, key blocks 0..3 */
#pragma unroll
            for (int i = 0; i < 4; i++) dst[i] = *(const bf16x8 *)(kt + (i * 16 + l15) * 256 + (((kk * 4 + lq) ^ l15) << 4));
        };
        auto vread = [&](int b, bf16x8 (&dst)[4]) { /* 32-key chunk b/2, head-dim blocks 4(b%2) .. +3 */
#pragma unroll
            for (int f = 0; f < 4; f++) /* this lane points at key 32 (b/2) + 8 lq + l15/4 (+4), dims 4 (l15%4) .. +3 of block f */
                dst[f] = v_fragment(vtile + (32 * (b >> 1) + 8 * lq + (l15 >> 2)) * 256 + ((f ^ (l15 >> 2)) << 5) + (l15 & 3) * 8 + (((b ^ lq) & 1) << 7));
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
        if (qrow[u] < q_end) {
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


template <int NW>
__global__ __launch_bounds__(NW * 64, NW == 4 ? 2 : 1) void attention_kernel(bf16 *__restrict__ out, int ldo,
                                                           const bf16 *__restrict__ q, int ldq,
                                                           const bf16 *__restrict__ k, const bf16 *__restrict__ v, int ldv,
                                                           int seq_q, int seq_k, int heads) {
    extern __shared__ __attribute__((aligned(16))) char smem[];
    /* Workgroups are dealt round-robin to the 8 XCDs, each with its own L2. Give every XCD a
     * contiguous run of (head, query block) pairs, so that all query blocks of a head run on one
     * XCD and its K / V (2.4 MB at 4608 tokens) are fetched from HBM once and then served from
     * that L2, instead of by all eight. */
    constexpr int BQ = NW * 32;  /* queries per workgroup */
    const int nqb = (seq_q + BQ - 1) / BQ;
    const int logical = (blockIdx.x & 7) * (gridDim.x >> 3) + (blockIdx.x >> 3);
    if (logical >= nqb * heads) return;
    const int h = logical / nqb, qb = logical - h * nqb;
    attention_block<NW>(smem, h, qb * BQ, min(qb * BQ + BQ, seq_q), out, ldo, q, ldq, k, v, ldv, seq_k, heads);
}

/* The wide kernel's way out for a workgroup whose softmax references did not hold (see first_reference): the same
 * queries once more with moving references, 128 at a time. Inlined into every instance of the wide kernel: as an
 * out-of-line function it gave each of them a call frame in scratch memory (1072 bytes per lane that every launch
 * had to have backed, though only this path touched it). */
__device__ __forceinline__ void attention_redo(char *smem, int h, int q_begin, int q_end, bf16 *out, int ldo, const bf16 *q, int ldq,
                                                         const bf16 *k, const bf16 *v, int ldv, int seq_k, int heads) {
    for (int qs = q_begin; qs < q_end; qs += 128) {
        attention_block<4>(smem, h, qs, min(qs + 128, q_end), out, ldo, q, ldq, k, v, ldv, seq_k, heads);
        __syncthreads(); /* the next block's first loads go to LDS slots this one may still be reading */
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
#define MFMA_ACC_VQ_GUARDED(acc, a, q) asm volatile("s_nop 1\n\tv_mfma_f32_16x16x32_bf16 %0, %1, %2, %0" : "+v"(acc) : "v"(a), "a"(q))
#define MFMA_ACC_A_GUARDED(acc, a, b) asm volatile("s_nop 1\n\tv_mfma_f32_16x16x32_bf16 %0, %1, %2, %0" : "+a"(acc) : "v"(a), "v"(b))
#define MFMA_ACC_A_ONES_GUARDED(acc, ones, b) asm volatile("s_nop 1\n\tv_mfma_f32_16x16x32_bf16 %0, %1, %2, %0" : "+a"(acc) : "a"(ones), "v"(b))

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

#define WIDE_BIAS 32.0f
/* One workgroup's work: the 64 NQ queries from q0 on of head h. */
template <int NQ>
__device__ __forceinline__ void attention_wide_body(char *smem, const int h, const int q0, bf16 *__restrict__ out, int ldo,
                                                    const bf16 *__restrict__ q, int ldq, const bf16 *__restrict__ k,
                                                    const bf16 *__restrict__ v, int ldv, int seq_q, int seq_k, int heads) {
    constexpr int NW = 4, WQ = 16 * NQ, LP = 16 / NW;
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int l15 = lane & 15, lq = lane >> 4;
    const int H = heads * HD;

    /* ---- Q fragments (B operand): prepared by qk_prepare_kernel (norm, RoPE, softmax scale). Requested before the
     * tile loads: loads return in order, and behind 28 tile loads these would arrive last ---- */
    bf16x8 qf[NQ][4];
#pragma unroll
    for (int t = 0; t < NQ; t++) {
        const bf16 *qp = q + (size_t)min(q0 + wave * WQ + t * 16 + l15, seq_q - 1) * ldq + h * HD + lq * 8;
#pragma unroll
        for (int kk = 0; kk < 4; kk++) qf[t][kk] = *(const bf16x8 *)(qp + kk * 32);
    }
    __builtin_amdgcn_sched_barrier(0);

    /* ---- tile loader: LDS layout and key permutation as in attention_kernel<4>; the global sources are a
     * uniform base plus one running 32-bit byte offset per lane and load ---- */
    const int ntiles = (seq_k + 63) >> 6;
    const char *k_base = (const char *)(k + h * HD);
    const char *v_base = (const char *)(v + h * HD);
    int k_row[LP];       /* key of the tile that this lane fetches with load i */
    const unsigned k_chunk = (unsigned)(((lane & 15) ^ ((wave * 4 + (lane >> 4)) & 15)) << 4);
    /* V: LDS row = key of the tile, 16-byte chunk c of row r at position c ^ 2 (r % 4) ^ (r & 8) */
    const unsigned v_chunk = (unsigned)(((lane & 15) ^ (2 * (lane >> 4)) ^ ((wave & 2) << 2)) << 4);
#pragma unroll
    for (int i = 0; i < LP; i++) {
        const int r = wave * 4 + i * (NW * 4) + (lane >> 4); /* LDS row; (r & 15) is the same for every i */
        const int ib = r >> 4, jj = (r >> 2) & 3, ee = r & 3;
        k_row[i] = 32 * (ib >> 1) + 8 * jj + 4 * (ib & 1) + ee;
    }
    /* LDS: four K slots of 16 KB, then four V slots of 16 KB; tile x lives in slot x % 4 of its ring.
     * Each load of a lane moves its offset on by 64 rows and stops at the last row (a multiply per load in the loop
     * costs as much as four other vector instructions), so the tile is implied by the order of the calls: one per
     * tile and load. Beyond the last tile the last row is fetched again, into a slot nobody reads any more: no
     * branches in the loop. */
    unsigned k_cur[LP], v_cur[LP];
    const unsigned k_last = (unsigned)(seq_k - 1) * (unsigned)(H * 2) + k_chunk, k_step = 64u * (unsigned)(H * 2);
    const unsigned v_last = (unsigned)(seq_k - 1) * (unsigned)(ldv * 2) + v_chunk, v_step = 64u * (unsigned)(ldv * 2);
#pragma unroll
    for (int i = 0; i < LP; i++) {
        k_cur[i] = min((unsigned)k_row[i] * (unsigned)(H * 2) + k_chunk, k_last);
        v_cur[i] = min((unsigned)(wave * 4 + i * (NW * 4) + (lane >> 4)) * (unsigned)(ldv * 2) + v_chunk, v_last);
    }
    auto load_k1 = [&](int slot, int i) {
        __builtin_amdgcn_global_load_lds(GLOBAL_PTR(k_base + k_cur[i]), LDS_PTR(smem + slot * 16384 + (wave * 4 + i * (NW * 4)) * 256), 16, 0, 0);
    };
    /* (assembly, so that the two instructions stay behind the MFMA they are written behind) */
    auto next_k1 = [&](int i) { asm volatile("v_add_u32 %0, %1, %0\n\tv_min_u32 %0, %0, %2" : "+v"(k_cur[i]) : "s"(k_step), "v"(k_last)); };
    auto load_v1 = [&](int slot, int i) {
        __builtin_amdgcn_global_load_lds(GLOBAL_PTR(v_base + v_cur[i]), LDS_PTR(smem + 4 * 16384 + slot * 16384 + (wave * 4 + i * (NW * 4)) * 256), 16, 0, 0);
    };
    auto next_v1 = [&](int i) { asm volatile("v_add_u32 %0, %1, %0\n\tv_min_u32 %0, %0, %2" : "+v"(v_cur[i]) : "s"(v_step), "v"(v_last)); };
    auto issue_k1 = [&](int slot, int i) { load_k1(slot, i); next_k1(i); };
    auto issue_v1 = [&](int slot, int i) { load_v1(slot, i); next_v1(i); };
    /* before the loop, in this order: K(0), V(0), K(1), V(1), K(2), V(2), K(3) */
#pragma unroll
    for (int x = 0; x < 4; x++) {
#pragma unroll
        for (int i = 0; i < LP; i++) issue_k1(x, i);
        if (x < 3) {
#pragma unroll
            for (int i = 0; i < LP; i++) issue_v1(x, i);
        }
    }

    /* the Q fragments arrive first (requested before the tile loads) and live in AGPRs */
#pragma unroll
    for (int t = 0; t < NQ; t++)
#pragma unroll
        for (int kk = 0; kk < 4; kk++) asm volatile("" : "+a"(qf[t][kk])); /* one aligned AGPR quad per fragment from here on */

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

    /* The loop is software-pipelined inside each wave, because with one wave per SIMD nothing else overlaps the
     * softmax with the matrix pipe. The unit is a chunk of 32 keys (half a tile): while chunk u is exponentiated
     * and multiplied into O, the scores of chunk u + 1 are already being computed:
     *   phase 1: S(u+1) = K Q^T - m   (8 NQ MFMAs)  with  the conversion of 2^S(u) to bf16 P(u) (4 NQ vector instructions),
     *            the requests for chunk u's V^T fragments and, in its last eight gaps, four tile loads
     *   phase 2: row sums and O += V^T P(u)^T (9 NQ MFMAs)  with  2^S(u+1) (8 NQ exponentials) and the requests for
     *            chunk u+2's K fragments
     * (The row sums as an MFMA against a fragment of ones cost a seventeenth of the loop's matrix time. Taken by the lanes
     * themselves from their own eight probabilities per query, in gaps of phase 1 that carry one other instruction or
     * none, they cost more: v_dot2c_f32_bf16 against (1, 1), four per query block and chunk, +3 % on the kernel, and even
     * a plain addition in its place, which is not enough instructions for the sums, only -1.4 %.)
     * Vector instructions sit one or two behind each MFMA; sched_barrier keeps them there. Two score buffers
     * alternate, so one trip of the loop is one tile: an "even" step (second chunk's scores, first chunk's
     * product) and an "odd" step (next tile's first chunk's scores, second chunk's product). One barrier per
     * tile, at the start of the odd step: behind it K(t)'s and V(t-1)'s slots are free and take K(t+4) and
     * V(t+3), whose eight loads go behind MFMAs of the two score phases up to the next barrier that carry little else
     * (in a run of eight behind MFMAs that also carry an exponential a direct global->LDS load cost the matrix pipe 30
     * cycles; alone behind its MFMA nothing that can be measured). With four slots per
     * ring those loads are not needed before the barrier after the next, so a barrier waits for all but the newest
     * eight loads (a count, not "all": the compiler's own barrier would wait for every load in flight).
     * Everything read before the next barrier landed before this one, so fragments are requested from LDS a phase
     * ahead of their MFMAs, across the barrier too.
     * The reference maxima are fixed on the first chunk, see first_reference. */
    constexpr int EXP0 = NQ < 2 ? 4 : 0; /* with 16 queries per wave the score phase is so short that the first exponentials wait four MFMAs */
    constexpr int CVT0 = NQ; /* the conversions start NQ MFMAs into the score phase: the product phase's last readers of P have long issued */
    f32x4 s_a[2][NQ], s_b[2][NQ];
    bf16x8 kf[4][2];  /* K fragments of a chunk: [32-dim step of the head dim][key block of the chunk] */
    s16x4 vh[8][2];   /* V^T fragments: [16-row block of the head dim][first / second four keys of the lane's eight] */
    u32x4 pf[NQ];     /* P^T of the chunk as MFMA B fragments (8 bf16), per query block */

    /* Fragments are requested from LDS a whole phase before the MFMAs that read them (the chunk's eight K
     * fragments during the product phase before, its sixteen V^T half fragments during the score phase before),
     * spread over the phase in the order of their use (reads in a run cost the matrix pipe 4-5 cycles each, a read
     * every few MFMAs next to nothing): no MFMA waits for LDS. */
    /* Per-lane LDS addresses of the fragments in slot 0 of each ring, kept in registers: the K fragments of head-dim
     * step kk, key block 0 of chunk 0 (the others lie 4096 (2 cp + i) further), and the V^T fragments of chunk 0 for
     * head-dim block x, as this lane of a transposing read sees them (the swizzle moves a block by the lane's key;
     * chunk 1 lies 8192 further). The slot is part of each read's immediate offset: the loop is written out for four
     * tiles, one per slot (moving these twelve registers on by a slot per tile cost twelve vector additions a tile, and
     * recomputing them from a slot number one addition per read). Only the last two tiles, whose slots depend on the
     * number of tiles, move the registers instead (move_slots) and read with the offsets of slot 0 (K: slot 1). */
    const unsigned lds0 = (unsigned)(uintptr_t)LDS_PTR(smem); /* folded into the addresses once, not added at every read */
    unsigned ka[4], va[8];
#pragma unroll
    for (int kk = 0; kk < 4; kk++) ka[kk] = lds0 + l15 * 256 + (((kk * 4 + lq) ^ l15) << 4);
#pragma unroll
    for (int x = 0; x < 8; x++) va[x] = lds0 + 4 * 16384 + (8 * lq + (l15 >> 2)) * 256 + ((x ^ (l15 >> 2) ^ ((lq & 1) << 2)) << 5) + (l15 & 3) * 8;
    auto kfrag1 = [&](int slot, int cp, int x) { /* x = 0..7: key block 2cp + x%2 of the tile, head dims 32 (x/2) .. +31 */
        const int kk = x >> 1, i = x & 1;
        kf[kk][i] = lds_read_bf16x8(ka[kk] + slot * 16384 + (2 * cp + i) * 4096);
    };
    auto vhalf1 = [&](int slot, int cp, int y) { /* y = 0..15: head-dim block y / 2, keys 8 lq + 4 (y % 2) .. +3 of 32-key chunk cp */
        const int x = y >> 1;
        vh[x][y & 1] = v_half_fragment_at(va[x] + slot * 16384 + cp * 8192 + (y & 1) * 1024);
    };
    /* what a phase of 8 NQ MFMAs requests behind MFMA m: K fragment x behind MFMA x NQ, V^T half fragment y behind
     * MFMA y NQ / 2 */
    auto k_reads_at = [&](int slot, int cp, int m) {
#pragma unroll
        for (int x = 0; x < 8; x++)
            if (x * NQ == m) kfrag1(slot, cp, x);
    };
    auto v_reads_at = [&](int slot, int cp, int m) {
#pragma unroll
        for (int y = 0; y < 16; y++)
            if (y * NQ / 2 == m) vhalf1(slot, cp, y);
    };
    auto move_slots = [&](int dk, int dv) { /* byte distances by which the K and the V^T addresses move */
#pragma unroll
        for (int kk = 0; kk < 4; kk++) ka[kk] += dk;
#pragma unroll
        for (int x = 0; x < 8; x++) va[x] += dv;
    };
    /* The vector instructions of the loop are inline assembly as well: an ordinary expression the compiler may
     * sink to its use in the next phase, and then nothing overlaps.
     * The exponentiation of a chunk is 8 NQ exponentials (16 cycles of the transcendental unit each) and 4 NQ
     * conversions of pairs. The exponentials run behind the MFMAs of the product phase BEFORE (the chunk's scores are
     * complete by then: the MFMA that finishes query block j, key block i is the (2 NQ - i NQ - j)-th from the end
     * of the score phase, and its eight exponentials come 8 j + 4 i MFMAs into the product phase, behind the NQ
     * row-sum MFMAs), the conversions behind the first MFMAs of the chunk's own score phase: that way both phases
     * carry about as much vector work as matrix work, instead of all of it sitting in the score phase. */
    auto exp1 = [&](f32x4 (&sc)[2][NQ], int n) { /* n = 0 .. 8 NQ - 1: query block n / 8, its eight scores in turn */
        const int j = n >> 3, r = n & 7;
        float x = sc[r >> 2][j][r & 3];
        asm volatile("v_exp_f32_e32 %0, %0" : "+v"(x));
        sc[r >> 2][j][r & 3] = x;
    };
    auto cvt1 = [&](f32x4 (&sc)[2][NQ], int n) { /* n = 0 .. 4 NQ - 1: query block n / 4, its four pairs in turn */
        const int j = n >> 2, hh = n & 3, i = hh >> 1, e = 2 * (hh & 1);
        unsigned w;
        asm volatile("v_cvt_pk_bf16_f32 %0, %1, %2" : "=v"(w) : "v"(sc[i][j][e]), "v"(sc[i][j][e + 1]));
        pf[j][hh] = w;
    };
    /* lane-wise maximum of a chunk's scores, one instruction at a time: 4 per query block (three-operand maxima
     * over the block's 8 values), the query blocks taking turns so that dependent instructions lie NQ apart */
    float lmax[NQ];
    auto max_op = [&](f32x4 (&sc)[2][NQ], int k) {
        const int q4 = k / NQ, j = k % NQ;
        auto v = [&](int idx) { return sc[idx >> 2][j][idx & 3]; };
        if (q4 == 0) asm volatile("v_max3_f32 %0, %1, %2, %3" : "=v"(lmax[j]) : "v"(v(0)), "v"(v(1)), "v"(v(2)));
        else if (q4 < 3) asm volatile("v_max3_f32 %0, %0, %1, %2" : "+v"(lmax[j]) : "v"(v(2 * q4 + 1)), "v"(v(2 * q4 + 2)));
        else asm volatile("v_max_f32_e32 %0, %0, %1" : "+v"(lmax[j]) : "v"(v(7)));
    };
    /* S = K Q^T - m for one chunk; kf must already hold (or be receiving) the chunk's fragments.
     * between(m) runs behind MFMA m (m = 0 .. 8 NQ - 1). */
    /* guard_c: outside the loop, where the register allocator may reconcile its assignments with copies right in
     * front of an MFMA, every MFMA carries its two idle slots with it */
    auto s_phase = [&](f32x4 (&sc)[2][NQ], auto &&between, auto guard_c) {
        constexpr bool GUARD = decltype(guard_c)::value;
#pragma unroll
        for (int kk = 0; kk < 4; kk++) {
#pragma unroll
            for (int i = 0; i < 2; i++)
#pragma unroll
                for (int j = 0; j < NQ; j++) {
                    if (kk == 0 && (i == 0 || GUARD)) MFMA_NEW_VQ_GUARDED(sc[i][j], kf[0][i], qf[j][0], neg_m[j]); /* first reader of neg_m[j] */
                    else if (kk == 0) MFMA_NEW_VQ(sc[i][j], kf[0][i], qf[j][0], neg_m[j]);
                    else if (GUARD) MFMA_ACC_VQ_GUARDED(sc[i][j], kf[kk][i], qf[j][kk]);
                    else MFMA_ACC_VQ(sc[i][j], kf[kk][i], qf[j][kk]);
                    between((kk * 2 + i) * NQ + j);
                    __builtin_amdgcn_sched_barrier(0);
                }
        }
    };
    /* row sums and O^T += V^T P^T for one chunk; vh must already hold (or be receiving) the chunk's fragments.
     * between(m) runs behind PV MFMA m (m = 0 .. 8 NQ - 1); the row-sum MFMAs carry nothing (starting the exponentials
     * behind them, so that the last NQ product MFMAs carry none, changed nothing). */
    auto pv_phase = [&](auto &&between, auto guard_c) {
        constexpr bool GUARD = decltype(guard_c)::value;
        /* the row sums are the first readers of each probability fragment */
#pragma unroll
        for (int j = 0; j < NQ; j++) {
            MFMA_ACC_A_ONES_GUARDED(l_acc[j], ones, pf[j]);
            __builtin_amdgcn_sched_barrier(0);
        }
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int g = 0; g < 2; g++)
#pragma unroll
            for (int f = 0; f < 4; f++)
#pragma unroll
                for (int j = 0; j < NQ; j++) {
                    const bf16x8 vf = v_join(vh[g * 4 + f][0], vh[g * 4 + f][1]);
                    if (GUARD) MFMA_ACC_A_GUARDED(o_acc[g * 4 + f][j], vf, pf[j]);
                    else MFMA_ACC_A(o_acc[g * 4 + f][j], vf, pf[j]);
                    between((g * 4 + f) * NQ + j);
                    __builtin_amdgcn_sched_barrier(0);
                }
    };
    auto fence_scores = [&](f32x4 (&sc)[2][NQ]) {
        asm volatile("s_nop 7\n\ts_nop 7" ::: "memory");
#pragma unroll
        for (int i = 0; i < 2; i++)
#pragma unroll
            for (int j = 0; j < NQ; j++) asm volatile("" : "+v"(sc[i][j]));
    };
    auto mask_chunk = [&](f32x4 (&sc)[2][NQ], int u) { /* keys of chunk u beyond seq_k (chunks of the last tile only) */
        if ((u + 1) * 32 <= seq_k) return;
        fence_scores(sc);
#pragma unroll
        for (int i = 0; i < 2; i++)
#pragma unroll
            for (int e = 0; e < 4; e++)
                if (u * 32 + 8 * lq + 4 * i + e >= seq_k) {
#pragma unroll
                    for (int j = 0; j < NQ; j++) sc[i][j][e] = -1e30f;
                }
    };
    /* The references of the online softmax are set once, from the first chunk: its exact row maxima (a query's
     * scores sit in lanes l, l^16, l^32, l^48) plus WIDE_BIAS. Probabilities then start near 2^-WIDE_BIAS, and a
     * later score may exceed the first chunk's maximum by more than 100 base-2 logits (a factor of 2^100 between
     * probabilities of one row) before anything leaves the range of fp32. The loop never looks at the scores'
     * size again and never moves the references: maxima cost a vector instruction per two scores, and rescaling
     * O with vector instructions inside the loop makes the register allocator carry O through VGPRs on every
     * trip. Should a row overflow all the same, its sums show it at the end: the workgroup then writes no output
     * and computes its queries once more with moving references (attention_redo). */
    auto first_reference = [&](f32x4 (&sc)[2][NQ]) {
#pragma unroll
        for (int j = 0; j < NQ; j++) {
            float mx = lmax[j];
            mx = fmaxf(mx, __shfl_xor(mx, 16, 64));
            mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
            const float d = mx + WIDE_BIAS;
#pragma unroll
            for (int e = 0; e < 4; e++) neg_m[j][e] = -d;
#pragma unroll
            for (int i = 0; i < 2; i++)
#pragma unroll
                for (int e = 0; e < 4; e++) sc[i][j][e] -= d;
        }
    };
    auto nothing = [](int) {};
    /* ---- first chunk, not pipelined: S(0) and its exact maxima ---- */
    asm volatile("s_waitcnt vmcnt(%0)\n\ts_barrier" ::"n"(6 * LP) : "memory"); /* K(0) is in LDS, the other six tiles on their way */
#pragma unroll
    for (int x = 0; x < 8; x++) kfrag1(0, 0, x);
    s_phase(s_a, nothing, AttFlag<true>{});
    fence_scores(s_a);
    mask_chunk(s_a, 0);
#pragma unroll
    for (int k = 0; k < 4 * NQ; k++) max_op(s_a, k);
    first_reference(s_a);
#pragma unroll
    for (int n = 0; n < 8 * NQ; n++) exp1(s_a, n);
#pragma unroll
    for (int x = 0; x < 8; x++) kfrag1(0, 1, x);
    asm volatile("s_waitcnt vmcnt(%0)\n\ts_barrier" ::"n"(4 * LP) : "memory"); /* V(0), K(1) are in LDS; V(1), K(2), V(2), K(3) on their way */

    /* The tile's eight loads, K(t+4) and V(t+3): the four of K in the last eight gaps of the odd step's score phase, the
     * four of V in those of the next even step's (gaps that carry little else): a load behind an even MFMA, the step of
     * its offset behind the next. */
    auto k_loads_at = [&](int slot, int m) {
#pragma unroll
        for (int i = 0; i < LP; i++) {
            if (m == 8 * NQ - 8 + 2 * i) load_k1(slot, i);
            if (m == 8 * NQ - 7 + 2 * i) next_k1(i);
        }
    };
    auto v_loads_at = [&](int slot, int m) {
#pragma unroll
        for (int i = 0; i < LP; i++) {
            if (m == 8 * NQ - 8 + 2 * i) load_v1(slot, i);
            if (m == 8 * NQ - 7 + 2 * i) next_v1(i);
        }
    };
    /* Even step of tile t, whose slot is sv: scores of its second chunk into s_b, product of its first chunk. The K
     * fragments of the odd step's chunk (first chunk of tile t + 1, slot sk) are requested meanwhile, and V(t+2) into
     * slot sl. Only the last tile can be ragged: the check for keys beyond the end (a branch: 30 cycles with nothing to
     * hide it) is compiled into the copies of the steps that can meet it, not into the loop. */
    auto even_step = [&](int t, int sv, int sk, int sl, auto loads_c, auto last_c, auto guard_c) {
        constexpr bool LOADS = decltype(loads_c)::value, LAST = decltype(last_c)::value;
        s_phase(s_b, [&](int m) {
            v_reads_at(sv, 0, m);
            if (m >= CVT0 && m < CVT0 + 4 * NQ) cvt1(s_a, m - CVT0);
            if (LOADS) v_loads_at(sl, m);
        }, guard_c);
        if (LAST) mask_chunk(s_b, 2 * t + 1);
        pv_phase([&](int m) {
            if (!LAST) k_reads_at(sk, 0, m);
            if (m >= EXP0) exp1(s_b, m - EXP0);
        }, guard_c);
#pragma unroll
        for (int n = 8 * NQ - EXP0; n < 8 * NQ; n++) exp1(s_b, n);
    };
    /* Odd step of tile t (slot sv): the barrier, scores of tile t+1's first chunk into s_a, product of tile t's second
     * chunk; tile t+1's second chunk of K fragments (slot sk) requested meanwhile, and K(t+4) into slot sl (tile t's). */
    auto odd_step = [&](int t, int sv, int sk, int sl, auto ragged_c, auto guard_c) {
        /* this wave's parts of K(t+2) and V(t+1) are in LDS: everything but the eight loads issued since the last barrier */
        asm volatile("s_waitcnt vmcnt(%0)\n\ts_barrier" ::"n"(2 * LP) : "memory");
        s_phase(s_a, [&](int m) {
            v_reads_at(sv, 1, m);
            if (m >= CVT0 && m < CVT0 + 4 * NQ) cvt1(s_b, m - CVT0);
            k_loads_at(sl, m);
        }, guard_c);
        if (decltype(ragged_c)::value) mask_chunk(s_a, 2 * t + 2);
        pv_phase([&](int m) {
            k_reads_at(sk, 1, m);
            if (m >= EXP0) exp1(s_a, m - EXP0);
        }, guard_c);
#pragma unroll
        for (int n = 8 * NQ - EXP0; n < 8 * NQ; n++) exp1(s_a, n);
    };
    /* the last chunk (second chunk of the tile whose V^T fragments va points at): nothing left to overlap */
    auto last_step = [&]() {
#pragma unroll
        for (int y = 0; y < 16; y++) vhalf1(0, 1, y);
#pragma unroll
        for (int n = 0; n < 4 * NQ; n++) cvt1(s_b, n);
        __builtin_amdgcn_sched_barrier(0);
        pv_phase(nothing, AttFlag<true>{});
    };
    /* a pair of steps in the loop: tile t (slot S) finishes, tile t + 1 starts */
    auto pair = [&](int t, auto slot_c) {
        constexpr int S = decltype(slot_c)::value;
        odd_step(t, S, (S + 1) & 3, S, AttFlag<false>{}, AttFlag<false>{});
        even_step(t + 1, (S + 1) & 3, (S + 2) & 3, (S + 3) & 3, AttFlag<true>{}, AttFlag<false>{}, AttFlag<false>{});
    };
    /* (outside the loop every MFMA carries its guard, see s_phase) */
    if (ntiles == 1) {
        even_step(0, 0, 1, 2, AttFlag<false>{}, AttFlag<true>{}, AttFlag<true>{});
    } else {
        even_step(0, 0, 1, 2, AttFlag<false>{}, AttFlag<false>{}, AttFlag<true>{});
        int t = 0;
        for (; t + 4 <= ntiles - 2; t += 4) {
            pair(t, AttInt<0>{});
            pair(t + 1, AttInt<1>{});
            pair(t + 2, AttInt<2>{});
            pair(t + 3, AttInt<3>{});
        }
        /* t is a multiple of four; up to three pairs are left before the last one */
        if (t < ntiles - 2) pair(t, AttInt<0>{});
        if (t + 1 < ntiles - 2) pair(t + 1, AttInt<1>{});
        if (t + 2 < ntiles - 2) pair(t + 2, AttInt<2>{});
        /* The last two tiles: their slots depend on the number of tiles, so the address registers move instead: V^T
         * fragments of tile ntiles - 2 at slot offset 0, K fragments of tile ntiles - 1 at slot offset 1. The odd step's
         * loads go where nobody reads any more (beyond the last tile the loaders fetch its last row again). */
        const int sv = (ntiles - 2) & 3, sk = (ntiles - 1) & 3;
        move_slots((sk - 1) * 16384, sv * 16384);
        odd_step(ntiles - 2, 0, 1, sv, AttFlag<true>{}, AttFlag<true>{});
        move_slots(0, (sk - sv) * 16384);
        even_step(ntiles - 1, 0, 1, 2, AttFlag<false>{}, AttFlag<true>{}, AttFlag<true>{});
    }
    last_step();
    __builtin_amdgcn_s_waitcnt(0x0F70); /* no load into LDS is left in flight */

    mfma_results_fence_a<NQ>(o_acc);
    asm volatile("s_nop 7\n\ts_nop 7" ::: "memory");
#pragma unroll
    for (int j = 0; j < NQ; j++) asm volatile("" : "+a"(l_acc[j]));
    /* Did a score come within reach of fp32 overflow (see first_reference)? Then a row sum or an accumulator is
     * infinite, not a number, or beyond 2^100: tested on the exponent bits (this file is compiled to assume that
     * there are no NaNs, so a floating-point comparison would not do). */
    unsigned worst = 0;
#pragma unroll
    for (int j = 0; j < NQ; j++) {
        worst = max(worst, __float_as_uint(l_acc[j][0]) & 0x7fffffffu);
#pragma unroll
        for (int i = 0; i < 8; i++)
#pragma unroll
            for (int e = 0; e < 4; e++) worst = max(worst, __float_as_uint(o_acc[i][j][e]) & 0x7fffffffu);
    }
    /* the workgroup decides as one: the way out needs all four waves */
    if (__syncthreads_or(worst >= 0x71800000u)) {
        attention_redo(smem, h, q0, min(q0 + NW * WQ, seq_q), out, ldo, q, ldq, k, v, ldv, seq_k, heads);
        return;
    }
#pragma unroll
    for (int j = 0; j < NQ; j++) {
        const float inv_l = 1.0f / l_acc[j][0];
        const int qr = q0 + wave * WQ + j * 16 + l15;
        if (qr < seq_q) {
            bf16 *op = out + (size_t)qr * ldo + h * HD + lq * 4;
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

/* The launch: every head's queries are cut into na blocks of 64 NQA queries followed by nb blocks of 64 NQB
 * (NQB = NQA - 1): a launch whose workgroups are all alike leaves compute units idle in its last round (18 blocks
 * of 256 queries per head, 24 heads: 432 workgroups, 1.69 rounds over 256 units, paid as 2), and with shorter
 * blocks at the end the last round is a short one. Each XCD takes a contiguous run of heads, so that a head's K and
 * V are fetched into one L2 only, and within its run the long blocks of all its heads come first (workgroups are
 * dealt to the XCDs round-robin and started in order). */
/* One or two sequences per launch (the two forwards of a classifier-free-guidance step attend separately but can
 * share a launch: more workgroups per round, one launch less per layer). */
struct AttSeq { bf16 *out; const bf16 *q, *k, *v; int seq_q, seq_k, na, nb; };
struct AttSeqs { AttSeq s[2]; int nseq; };

template <int NQA, int NQB>
__global__ __launch_bounds__(256, 1) void attention_wide_kernel(AttSeqs p, int ldo, int ldq, int ldv, int heads) {
    extern __shared__ __attribute__((aligned(16))) char smem[];
    const int xcd = blockIdx.x & 7, hx0 = xcd * heads / 8, nh = (xcd + 1) * heads / 8 - hx0;
    int item = blockIdx.x >> 3;
    /* within an XCD's run: the long blocks of the first sequence, of the second, then the short blocks likewise */
    const int la0 = nh * p.s[0].na, la1 = p.nseq > 1 ? nh * p.s[1].na : 0;
    const int lb0 = nh * p.s[0].nb, lb1 = p.nseq > 1 ? nh * p.s[1].nb : 0;
    const bool is_long = item < la0 + la1;
    bool second;
    if (is_long) {
        second = item >= la0;
        if (second) item -= la0;
    } else {
        item -= la0 + la1;
        if (item >= lb0 + lb1) return;
        second = item >= lb0;
        if (second) item -= lb0;
    }
    /* (fields picked one by one: an index into the argument structure would send it through scratch memory) */
    bf16 *out = second ? p.s[1].out : p.s[0].out;
    const bf16 *q = second ? p.s[1].q : p.s[0].q, *k = second ? p.s[1].k : p.s[0].k, *v = second ? p.s[1].v : p.s[0].v;
    const int seq_q = second ? p.s[1].seq_q : p.s[0].seq_q, seq_k = second ? p.s[1].seq_k : p.s[0].seq_k;
    const int na = second ? p.s[1].na : p.s[0].na, nb = second ? p.s[1].nb : p.s[0].nb;
    if (is_long) {
        attention_wide_body<NQA>(smem, hx0 + item / na, (item % na) * 64 * NQA, out, ldo, q, ldq, k, v, ldv, seq_q, seq_k, heads);
    } else {
        attention_wide_body<NQB>(smem, hx0 + item / nb, na * 64 * NQA + (item % nb) * 64 * NQB, out, ldo, q, ldq, k, v, ldv, seq_q,
                                 seq_k, heads);
    }
}

/* How a head's queries are cut into blocks: na blocks of 64 nqa queries, then nb blocks of 64 (nqa - 1). The choice
 * minimises the time of the slowest XCD under a simple model: an XCD's compute units (one workgroup each at a
 * time) take its blocks in order, and a block of 64 NQ queries costs cost[NQ] (relative times of one workgroup
 * measured at 4608 keys: the per-tile work that does not depend on NQ - loads, barrier, fragment reads - makes short
 * blocks dearer per query). */
struct WidePlan { int nqa, na, nb; };
static WidePlan wide_plan(int seq_q, int heads) {
    /* the search below is some 1e5 operations at 4608 queries: its last results are kept, keyed by everything it
     * depends on (two alternating query lengths, or two devices, would otherwise repeat it on every call) */
    struct Entry { int seq, heads, cus; WidePlan plan; };
    static Entry cache[8];
    static int n_cached = 0, next = 0;
    static const double cost[5] = {0.0, 0.44, 0.62, 0.81, 1.0};
    int cus = 256, dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus < 8) cus = 256;
    for (int i = 0; i < n_cached; i++)
        if (cache[i].seq == seq_q && cache[i].heads == heads && cache[i].cus == cus) return cache[i].plan;
    const int per_xcd = cus / 8, nh = (heads + 7) / 8;
    WidePlan best = {2, 0, (seq_q + 63) / 64};
    double best_t = 1e30;
    for (int nqa = 4; nqa >= 2; nqa--) {
        const int la = 64 * nqa, lb = 64 * (nqa - 1);
        for (int na = (seq_q + la - 1) / la; na >= 0; na--) {
            const int rest = seq_q - na * la, nb = rest > 0 ? (rest + lb - 1) / lb : 0;
            /* list scheduling of nh * na long blocks, then nh * nb short ones, on per_xcd units */
            double busy[64];
            const int units = per_xcd < 64 ? per_xcd : 64;
            for (int u = 0; u < units; u++) busy[u] = 0.0;
            for (int i = 0; i < nh * (na + nb); i++) {
                int u0 = 0;
                for (int u = 1; u < units; u++)
                    if (busy[u] < busy[u0]) u0 = u;
                busy[u0] += i < nh * na ? cost[nqa] : cost[nqa - 1];
            }
            double t = 0.0;
            for (int u = 0; u < units; u++) t = busy[u] > t ? busy[u] : t;
            t += 1e-4 * nh * (na + nb); /* ties: fewer workgroups */
            if (t < best_t) { best_t = t; best = {nqa, na, nb}; }
        }
    }
    cache[next] = {seq_q, heads, cus, best};
    next = (next + 1) % 8;
    if (n_cached < 8) n_cached++;
    return best;
}

static int g_att_force = -1;
extern "C" void flux_hip_attention_force_variant(int v) { g_att_force = v; }

static int attention_check(const void *out_bf16, int ldo, const void *q, int ldq, const void *k, const void *v, int ldv, int seq_k, int heads) {
    if (seq_k <= 0) return flux_hip_fail("flux_hip_attention: seq_k=%d", seq_k);
    if (heads <= 0) return flux_hip_fail("flux_hip_attention: heads=%d", heads);
    if (!out_bf16 || !q || !k || !v) return flux_hip_fail("flux_hip_attention: NULL argument");
    if ((((uintptr_t)q | (uintptr_t)k | (uintptr_t)v) & 15) || ((uintptr_t)out_bf16 & 7))
        return flux_hip_fail("flux_hip_attention: operands must be 16-byte aligned (output 8-byte)");
    if ((ldo & 3) || (ldq & 7) || (ldv & 7) || ldv < heads * HD || ldq < heads * HD || ldo < heads * HD)
        return flux_hip_fail("flux_hip_attention: bad leading dimensions (ldo=%d ldq=%d ldv=%d; each at least heads * %d = %d)", ldo, ldq, ldv, HD,
                             heads * HD);
    /* the tile loaders address K and V rows with 32-bit byte offsets that run up to 64 rows past the end */
    if ((double)(seq_k + 64) * ldv * 2.0 >= 4294967296.0 || (double)(seq_k + 64) * heads * HD * 2.0 >= 4294967296.0)
        return flux_hip_fail("flux_hip_attention: %d keys of %d-element rows exceed 32-bit offsets", seq_k, ldv);
    return 1;
}

static WidePlan attention_plan(int variant, int seq_q, int heads) {
    WidePlan plan;
    if (variant >= 11 && variant <= 14) {
        const int nq = variant - 10;
        plan.nqa = nq > 1 ? nq : 2;
        plan.na = nq > 1 ? (seq_q + 64 * nq - 1) / (64 * nq) : 0;
        plan.nb = nq > 1 ? 0 : (seq_q + 63) / 64;
    } else {
        plan = wide_plan(seq_q, heads);
    }
    return plan;
}

extern "C" int flux_hip_attention_batch(int nseq, void *const *out_bf16, int ldo, const void *const *q, int ldq, const void *const *k,
                                        const void *const *v, int ldv, const int *seq_q, const int *seq_k, int heads) {
    if (nseq <= 0) return 1;
    if (!out_bf16 || !q || !k || !v || !seq_q || !seq_k) return flux_hip_fail("flux_hip_attention_batch: NULL argument");
    for (int i = 0; i < nseq; i++)
        if (seq_q[i] > 0 && !attention_check(out_bf16[i], ldo, q[i], ldq, k[i], v[i], ldv, seq_k[i], heads)) return 0;
    /* Variants: 0 / 1 = attention_kernel with 128 / 256 queries per workgroup; 11 .. 14 = attention_wide_kernel with
     * 16 NQ queries per wave throughout (NQ = 1 .. 4); -1 (default) and 15 = attention_wide_kernel with the mix of
     * block lengths that wide_plan() finds. */
    static bool attr_done = false;
    if (!attr_done) {
        HIP_OK(hipFuncSetAttribute((const void *)attention_kernel<4>, hipFuncAttributeMaxDynamicSharedMemorySize, 2 * ATT_STAGE));
        HIP_OK(hipFuncSetAttribute((const void *)attention_kernel<8>, hipFuncAttributeMaxDynamicSharedMemorySize, 2 * ATT_STAGE));
        HIP_OK(hipFuncSetAttribute((const void *)attention_wide_kernel<4, 3>, hipFuncAttributeMaxDynamicSharedMemorySize, ATT_WIDE_LDS));
        HIP_OK(hipFuncSetAttribute((const void *)attention_wide_kernel<3, 2>, hipFuncAttributeMaxDynamicSharedMemorySize, ATT_WIDE_LDS));
        HIP_OK(hipFuncSetAttribute((const void *)attention_wide_kernel<2, 1>, hipFuncAttributeMaxDynamicSharedMemorySize, ATT_WIDE_LDS));
        attr_done = true;
    }
    const int variant = g_att_force;
    const int max_nh = (heads + 7) / 8; /* the most heads one XCD takes */
    for (int i = 0; i < nseq;) {
        if (seq_q[i] <= 0) { i++; continue; }
        if (variant == 0 || variant == 1) {
            const int bq = variant ? 256 : 128, blocks = ((seq_q[i] + bq - 1) / bq) * heads;
            hipLaunchKernelGGL(variant ? attention_kernel<8> : attention_kernel<4>, dim3((blocks + 7) & ~7), dim3(variant ? 512 : 256), 2 * ATT_STAGE,
                               flux_hip_stream_handle(), (bf16 *)out_bf16[i], ldo, (const bf16 *)q[i], ldq, (const bf16 *)k[i], (const bf16 *)v[i],
                               ldv, seq_q[i], seq_k[i], heads);
            i++;
            continue;
        }
        /* two sequences share a launch when their blocks have the same lengths */
        AttSeqs p = {};
        const WidePlan plan = attention_plan(variant, seq_q[i], heads);
        p.s[0] = {(bf16 *)out_bf16[i], (const bf16 *)q[i], (const bf16 *)k[i], (const bf16 *)v[i], seq_q[i], seq_k[i], plan.na, plan.nb};
        p.nseq = 1;
        int blocks = plan.na + plan.nb;
        if (i + 1 < nseq && seq_q[i + 1] > 0) {
            const WidePlan plan1 = attention_plan(variant, seq_q[i + 1], heads);
            if (plan1.nqa == plan.nqa) {
                p.s[1] = {(bf16 *)out_bf16[i + 1], (const bf16 *)q[i + 1], (const bf16 *)k[i + 1], (const bf16 *)v[i + 1], seq_q[i + 1], seq_k[i + 1],
                          plan1.na, plan1.nb};
                p.nseq = 2;
                blocks += plan1.na + plan1.nb;
            }
        }
        auto kern = plan.nqa == 4 ? attention_wide_kernel<4, 3> : plan.nqa == 3 ? attention_wide_kernel<3, 2> : attention_wide_kernel<2, 1>;
        hipLaunchKernelGGL(kern, dim3(8 * max_nh * blocks), dim3(256), ATT_WIDE_LDS, flux_hip_stream_handle(), p, ldo, ldq, ldv, heads);
        i += p.nseq;
    }
    HIP_OK(hipGetLastError());
    return 1;
}

extern "C" int flux_hip_attention(void *out_bf16, int ldo, const void *q, int ldq, const void *k, const void *v,
                                  int ldv, int seq_q, int seq_k, int heads) {
    return flux_hip_attention_batch(1, &out_bf16, ldo, &q, ldq, &k, &v, ldv, &seq_q, &seq_k, heads);
}
