/*
 * gemm.hip - bf16 MFMA GEMM  C[M,N] = A[M,K] * W[N,K]^T  with fused epilogues, for gfx950.
 *
 * This is the linear layer of the denoising transformer (reference: flux_linear,
 * flux_kernels.c:210-282, cblas_sgemm NoTrans x Trans). Both operands have K contiguous, so
 * an MFMA operand fragment (8 consecutive bf16 of one row) is one 16-byte LDS read.
 *
 * Tiling: a workgroup owns a BM x BN tile; K is walked in steps of 64 through two LDS stages.
 * Tiles go from global memory straight into LDS (global_load_lds_dwordx4, no register
 * staging, no ds_write): the next stage is in flight while the current one is multiplied, with
 * one barrier per step. Each 64-lane wave owns a WM x WN sub-tile made of 16x16 blocks of
 * v_mfma_f32_16x16x32_bf16. On this part the matrix pipes are power limited with real data;
 * the 16x16x32 form sustains about 15 % more than 32x32x16 at the same tile, and skipping the
 * register/ds_write hop saves both time and energy (measured: 800 -> 1000 TFLOP/s on the
 * 4608 x 18432 x 3072 projection).
 *
 * The weight fragment is the MFMA "A" operand and the activation fragment the "B" operand,
 * so that in the accumulator a lane holds one token (m) and four consecutive output features
 * (n): epilogues use 8/16-byte accesses and pair gate/up columns inside a lane.
 *
 * Two kernels share the tile decode and the epilogues. gemm_kernel<BM,BN,WGM,WGN> (8 or 4
 * waves, two waves per SIMD) serves the small tiles. gemm4w_kernel<TM,TN> is for the
 * large projections, as a 256 x 256 or a 288 x 192 tile (the second divides 4608-token problems
 * into a whole number of rounds over 256 CUs): 4 waves, one per SIMD, each owning 128 x 128
 * (144 x 96) of the tile with its 256 (216) accumulator registers pinned to AGPRs. A 128 x 128 wave tile needs 16 fragment reads per 64
 * MFMAs instead of 12 per 32, i.e. a third less LDS traffic per FLOP, which under the power
 * limit is what buys throughput (1020 -> 1145 TFLOP/s sustained back to back on the
 * 4608 x 18432 x 3072 projection). With a single wave per SIMD nothing hides latency for free,
 * so the loop is software-pipelined by hand: fragments are double-buffered in registers, every
 * third or fourth MFMA is followed by one LDS read for the next half-step and (in the second half) one
 * global->LDS load for the stage after next, and there is one barrier per 64-wide K step. The
 * reads come after their MFMA, not before it, so that the half-step opens with an MFMA whose
 * operands arrived long ago: the compiler puts an lgkmcnt(0) wait in front of the first MFMA after
 * the loop's back edge, and with a read issued just before it that wait exposed a full LDS latency
 * per K step. Global sources are a scalar base plus a 32-bit offset per lane, so stepping along K
 * is scalar work. Blocks are walked in serpentine order (one MFMA operand changes at a time).
 * A workgroup goes on to further tiles (one workgroup per compute unit is launched) and requests the
 * next tile's first stage before it stores the finished one.
 * One wave per SIMD does keep the matrix pipe full when its MFMAs are written by hand: a register-
 * resident loop of independent v_mfma_f32_16x16x32_bf16 reaches 2.4 PFLOP/s on zero operands and
 * 1.86 on random bits with 256 threads per compute unit, accumulators in VGPRs or AGPRs alike (the
 * same loop left to the compiler's builtin gets 1.46: it shuffles accumulators between the two
 * register files). Cycle stamps in this kernel on zero operands (4608 x 18432 x 3072, clocks near
 * their maximum) put 91 % of a wave's life in the K loop, 7 % in the epilogue and next-tile
 * set-up, 4 % in the mid-step wait and barrier; the K loop ran at 75 % of the MFMA issue rate
 * before the reads moved behind their MFMAs. On real operands the chip is at its power limit, in a
 * denoising step as well as back to back: removing those stalls made the kernel 5 % faster back to
 * back and the step 1 % faster.
 * The same loop also exists over a WGM x WGN grid of waves; with 8 waves (2 x 4, 128 x 64 each, two
 * per SIMD) on the 256 x 256 tile it runs at the speed of the 4-wave form and is kept for comparison
 * runs (tile id 4).
 *
 * Three kernels, then: gemm_kernel (small tiles; with NS > 2 a ring of NS LDS stages for row ranges of few
 * rows, where a launch only streams weights), gemm4w_kernel (large tiles, two LDS stages; convolutions, and the
 * comparison form of the next one) and gemm4d_kernel (large tiles with an LDS ring per operand, the form the
 * transformer's projections run). What separates the last two is the barrier: __syncthreads() carries a fence
 * that waits for every global->LDS load in flight, so a two-stage loop can never have more than the next stage
 * on its way, requested one to two half-steps earlier; operands that come from HBM arrive later than that now and
 * then, and a wave that waits holds its three neighbours up at the barrier (measured: the same launch takes
 * 232-241 us when its operands are reused from the memory-side cache and 272-277 us when they rotate through
 * six buffer sets; a copy without the barrier does not care). gemm4d_kernel waits with a count instead
 * (s_waitcnt vmcnt(n) + s_barrier in one asm statement): everything but the last n loads, which belong to the
 * operand whose ring has a third slot and are needed a whole K step later.
 *
 * LDS rows are 128 bytes (64 bf16); the 16-byte chunk index is XOR-swizzled with a function of
 * the row so that the 16 rows a fragment read touches spread over all banks. A direct-to-LDS
 * load writes lane i's 16 bytes at (wave base + 16 i), so the swizzle is applied on the global
 * side: each lane fetches the chunk that belongs at its LDS position.
 */
#include "common.h"
#include "../../include/flux_hip.h"
#include "../../include/flux_hip_debug.h"

#define GEMM_MAX_PARTS 4
struct GemmArgs {
    const bf16 *A[GEMM_MAX_PARTS];
    const bf16 *W[GEMM_MAX_PARTS];
    void *C[GEMM_MAX_PARTS];
    const float *gate[GEMM_MAX_PARTS];
    int M[GEMM_MAX_PARTS];
    int mt_end[GEMM_MAX_PARTS]; /* row tiles of parts 0..i together; unused parts repeat the total */
    int mtiles, ntiles, total_tiles;
    int vgrid; /* workgroups' worth of tiles (a multiple of 8); a launch with fewer workgroups walks them in strides of its size */
    int N, K, lda, ldw, ldc, w_row0, w_row1;
    /* fused [Q | K | V | gate | up] projection (EPI_QKV_SWIGLU): the first nq_cols columns (weight rows from w_row0)
     * are stored as bf16 to C, the other N - nq_cols are gate / up pairs (gate rows from w_row1, up rows from
     * w_row2) whose silu(gate) * up goes to C2; nq_tiles = nq_cols / tile width */
    int w_row2, nq_cols, nq_tiles, ldc2;
    void *C2;
    /* split-K: workgroup (tile, s) multiplies K-steps [s*kt_per, (s+1)*kt_per) and stores its
     * fp32 partial tile into ws[s][moff[part] + m][n]; a second kernel sums the slices */
    int ksplit, kt_per;
    float *ws;
    int moff[GEMM_MAX_PARTS], ws_rows;
    /* convolution epilogues (see flux_hip_conv): rows are the positions of a zero-bordered
     * conv_hp x conv_wp image with channels contiguous. With 9 taps K runs over
     * [cin / 64 channel chunks][9 taps][64 channels]: K step kt = 9 * chunk + tap reads the
     * activation rows shifted by its tap's (dy, dx). The nine taps of a chunk follow each other so
     * that what one tap fetched is still in L2 when the next asks for the neighbouring rows
     * (tap-major order re-fetched wide images 3 to 10 times from HBM). */
    int conv_taps, conv_wp, conv_hp;
    const float *bias, *res;
    /* optional: per (row-tile half, 4-channel group) sums and sums of squares of what a convolution
     * epilogue writes, [prow][N/4][2], for the group norm that follows */
    float *stats;
};

template <int EPI> struct IsConv { static constexpr bool value = EPI == FLUX_HIP_EPI_CONV_BF16 || EPI == FLUX_HIP_EPI_CONV_F32; };

/* Element offset of K step kt within an activation row. Plain GEMM: kt * 64. 3x3 convolution:
 * kt = 9 * chunk + tap; the tap selects a neighbour dy*Wp + dx rows away (uniform for the whole
 * launch, because border positions are rows of the matrix too), the chunk a 64-channel slice. */
template <int EPI>
__device__ __forceinline__ int a_step_offset(const GemmArgs &g, int kt) {
    if (IsConv<EPI>::value && g.conv_taps == 9) {
        const int chunk = (kt * 7282) >> 16, tap = kt - 9 * chunk; /* kt / 9, kt % 9 for kt < 2048 */
        const int dy = (tap * 11) >> 5, dx = tap - dy * 3;         /* tap / 3, tap % 3 for tap < 9 */
        return ((dy - 1) * g.conv_wp + (dx - 1)) * g.lda + chunk * 64;
    }
    return kt * 64;
}

/* internal epilogue: fp32 partial sums of one K slice (see split-K above) */
#define EPI_PARTIAL 5
/* internal epilogue of flux_hip_linear_qkv_swiglu: bf16 store for the leading column tiles, SiLU(gate) * up beyond */
#define EPI_QKV_SWIGLU 8

__device__ __forceinline__ int lds_swz(int r) { return ((r >> 1) & 7) ^ ((r & 1) << 2); }

#define GROUP_M 4
#define GLOBAL_PTR(p) ((const __attribute__((address_space(1))) void *)(p))
#define LDS_PTR(p) ((__attribute__((address_space(3))) void *)(p))
/* s_waitcnt vmcnt(0) only (expcnt and lgkmcnt fields left at their maxima) */
#define WAIT_VMCNT0() __builtin_amdgcn_s_waitcnt(0x0F70)

/* Which tile (and K slice) a workgroup owns. Workgroups are dealt round-robin to the 8 XCDs;
 * each XCD gets a contiguous run of tiles so that its L2 sees the reuse, and tiles are walked in
 * groups of GROUP_M rows. */
struct TileId {
    int ks, tm, tn, prob, tml;
};
__device__ __forceinline__ bool decode_tile(const GemmArgs &g, int vb, TileId &t) {
    int per_xcd = g.vgrid >> 3;
    int logical = (vb & 7) * per_xcd + (vb >> 3);
    if (logical >= g.total_tiles * g.ksplit) return false;
    t.ks = logical / g.total_tiles;
    logical -= t.ks * g.total_tiles;
    int per_group = GROUP_M * g.ntiles;
    int grp = logical / per_group;
    int first_m = grp * GROUP_M;
    int gsz = min(g.mtiles - first_m, GROUP_M);
    int in_grp = logical - grp * per_group;
    t.tm = first_m + in_grp % gsz;
    t.tn = in_grp / gsz;
    t.prob = (t.tm >= g.mt_end[0]) + (t.tm >= g.mt_end[1]) + (t.tm >= g.mt_end[2]);
    t.tml = t.prob ? t.tm - g.mt_end[t.prob - 1] : t.tm;
    return true;
}

/* Which feature of its wave's slice of the output row r of MFMA block blk computes, for the two epilogues that
 * store bf16. In the accumulator a lane holds four consecutive MFMA rows of a block (rows 4 (lane / 16) .. + 3): with
 * rows numbered plainly that is four consecutive features, an 8-byte store, and a wave's store instruction writes
 * 32 bytes to each of 16 output rows. Here two neighbouring blocks interleave instead: block 2p takes features
 * 32 p + 8 q + 0 .. 3 on its rows 4 q .. 4 q + 3 and block 2p + 1 features 32 p + 8 q + 4 .. 7, so that a lane's
 * results of the two blocks are eight consecutive features: one 16-byte store, 64 bytes per output row and
 * instruction, half as many store instructions and write requests. Only the weight rows a block reads change. */
__device__ __forceinline__ int bf16_pair_feature(int blk, int r) { return 32 * (blk >> 1) + 8 * (r >> 2) + 4 * (blk & 1) + (r & 3); }
/* the same for a wave that owns TN blocks: with TN odd the last block has no neighbour and keeps the plain numbering */
template <int TN>
__device__ __forceinline__ int bf16_feature(int blk, int r) { return blk < (TN & ~1) ? bf16_pair_feature(blk, r) : 16 * blk + r; }
/* Tile widths that divide none of the model's matrix widths (224: 3072 = 13 x 224 + 160, 9216 = 41 x 224 + 32): the
 * last column tile is cut off. Its missing weight rows are read from the matrix's last row and its missing columns are
 * not stored (whole 16-column blocks for fp32 outputs, whole pairs of blocks for bf16: N is a multiple of 32). */
template <int BN> struct CutTile { static constexpr bool value = BN % 64 != 0; };
/* SiLU(gate) * up: blocks alternate gate, up, so that a lane holds matching pairs; the (gate, up) pairs interleave
 * two by two in the same way, and a last odd pair keeps the plain numbering (features 16 k + r). */
template <int TN>
__device__ __forceinline__ int swiglu_feature(int blk, int r) {
    const int k = blk >> 1;
    return k < 2 * (TN / 4) ? bf16_pair_feature(k, r) : 16 * k + r;
}

/* Weight row that feeds column v of the tile. */
template <int BN, int WN, int EPI>
__device__ __forceinline__ int weight_row(const GemmArgs &g, int tn, int v) {
    constexpr int TN = WN / 16;
    const int wv = v / WN, blk = (v % WN) >> 4, r = v & 15;
    if (EPI == FLUX_HIP_EPI_SWIGLU || (EPI == EPI_QKV_SWIGLU && tn >= g.nq_tiles)) {
        const int idx = wv * (WN / 2) + swiglu_feature<TN>(blk, r);
        if (EPI == EPI_QKV_SWIGLU) return ((blk & 1) ? g.w_row2 : g.w_row1) + (tn - g.nq_tiles) * (BN / 2) + idx;
        return ((blk & 1) ? g.w_row1 : g.w_row0) + tn * (BN / 2) + idx;
    }
    int col;
    if (EPI == FLUX_HIP_EPI_BF16 || EPI == EPI_QKV_SWIGLU) col = tn * BN + wv * WN + bf16_feature<TN>(blk, r);
    else col = tn * BN + v;
    if (CutTile<BN>::value) col = min(col, g.N - 1);
    return g.w_row0 + col;
}

/* eight bf16 to consecutive addresses: one 16-byte store where the address allows it, else two of 8 bytes */
__device__ __forceinline__ void store_bf16x8(bf16 *p, bf16x4 lo, bf16x4 hi, bool aligned16) {
    if (aligned16) {
        bf16x8 o;
#pragma unroll
        for (int e = 0; e < 4; e++) { o[e] = lo[e]; o[4 + e] = hi[e]; }
        *(bf16x8 *)p = o;
    } else {
        *(bf16x4 *)p = lo;
        *(bf16x4 *)(p + 4) = hi;
    }
}

template <bool V> struct BoolC { static constexpr bool value = V; };
template <int V> struct IntC { static constexpr int value = V; };

/* Accumulator element e of block (i, j): feature n = 4*(lane/16) + e of the 16-column block,
 * token m = lane%16 of the 16-row block. */
template <int BN, int WM, int WN, int EPI, bool HERE = false>
__device__ __forceinline__ void store_tile_to(const GemmArgs &g, const TileId &t, f32x4 (&acc_in)[WN / 16][WM / 16], int m0, int M,
                                              int wm, int wn, int l15, int lq, int prow, void *Cp, const int ldc, const int tn) {
    constexpr int TM = WM / 16, TN = WN / 16;
    const int prob = t.prob, n0 = tn * BN, ks = t.ks;
    const bool aligned16 = (((uintptr_t)Cp | ((uintptr_t)ldc << 1)) & 15) == 0; /* every 8-feature group of the output starts on 16 bytes */
    f32x4 acc_here[HERE ? TN : 1][HERE ? TM : 1];
    auto &acc = [&]() -> auto & { if constexpr (HERE) return acc_here; else return acc_in; }();
    if constexpr (EPI == FLUX_HIP_EPI_RESID && HERE) {
        /* x += gate * acc on the fp32 residual: a read, and a write that depends on it. Row block by row block in
         * program order that is a chain of round trips to memory (request a row's values, wait, store; the wait
         * counter also holds the stores of the row before, so every wait is for those as well): nine such chains made
         * up most of the 57 us that this epilogue cost a 288 x 192 x 12288 tile's launch of 261 us. Here the values of
         * row block j + 1 are requested before row block j is touched: the wait for block j's values leaves the block
         * before's stores and the next block's loads in flight. Rows beyond M read the last row (no branch around the
         * loads) and store nothing; a wave whose rows are all valid runs a copy without that test, i.e. without
         * branches (behind a skipped store the compiler must assume that the loads in front of it are still under
         * way, and it waits for them before it reuses their registers: one row block in flight instead of two). */
        const auto cut = [&](int i) { return CutTile<BN>::value && n0 + wn * WN + i * 16 >= g.N; }; /* the same for the whole wave */
        /* the unit that is requested ahead: a row block's TN column blocks, or half of them where the accumulators fill the
         * AGPRs and the fragments most of the VGPRs (256 x 256) */
        constexpr int UN = TM * TN * 4 > 224 && TN % 2 == 0 ? TN / 2 : TN, UPR = TN / UN, NU = TM * UPR;
        constexpr int NB = 2; /* units in flight, the one being stored included (a third one measured no different: what is left is the burst itself) */
        f32x4 gt[TN], xb[NB][UN];
#pragma unroll
        for (int i = 0; i < TN; i++)
            if (!cut(i)) gt[i] = *(const f32x4 *)(g.gate[prob] + n0 + wn * WN + i * 16 + lq * 4);
        const auto fetch = [&](int u) {
            const int j = u / UPR, i0 = u % UPR * UN;
            const float *p = (const float *)Cp + (size_t)min(m0 + wm * WM + j * 16 + l15, M - 1) * ldc + n0 + wn * WN + lq * 4;
#pragma unroll
            for (int i = 0; i < UN; i++)
                if (!cut(i0 + i)) xb[u % NB][i] = *(const f32x4 *)(p + (i0 + i) * 16);
        };
        const auto rows = [&](auto full_c) {
#pragma unroll
            for (int u = 0; u < NB - 1 && u < NU; u++) fetch(u);
#pragma unroll
            for (int u = 0; u < NU; u++) {
                const int j = u / UPR, i0 = u % UPR * UN;
                if (u + NB - 1 < NU) fetch(u + NB - 1);
                const int m = m0 + wm * WM + j * 16 + l15;
                float *p = (float *)Cp + (size_t)m * ldc + n0 + wn * WN + lq * 4;
#pragma unroll
                for (int i = 0; i < UN; i++) {
                    if (cut(i0 + i)) continue;
                    f32x4 a = acc_in[i0 + i][j]; /* out of its AGPRs here, one block at a time */
                    asm volatile("" : "+v"(a));
                    f32x4 x = xb[u % NB][i];
#pragma unroll
                    for (int e = 0; e < 4; e++) x[e] += gt[i0 + i][e] * a[e];
                    if (decltype(full_c)::value || m < M) *(f32x4 *)(p + (i0 + i) * 16) = x;
                }
            }
        };
        if (m0 + wm * WM + WM <= M) rows(BoolC<true>{});
        else rows(BoolC<false>{});
        return;
    }
    float st_s[TN], st_q[TN]; /* convolutions with statistics: this lane's sums per 16-column block */
#pragma unroll
    for (int i = 0; i < TN; i++) st_s[i] = st_q[i] = 0.0f;
#pragma unroll
    for (int j = 0; j < TM; j++) {
        const int m = m0 + wm * WM + j * 16 + l15;
        if (m >= M) continue;
        if constexpr (HERE) {
#pragma unroll
            for (int i = 0; i < TN; i++) {
                acc[i][j] = acc_in[i][j];
                asm volatile("" : "+v"(acc[i][j]));
            }
        }
        bool inside = true; /* convolutions: border positions of the image are written as zeros */
        if (IsConv<EPI>::value && g.conv_wp > 0) {
            const int y = m / g.conv_wp, x = m - y * g.conv_wp;
            inside = y >= 1 && y < g.conv_hp - 1 && x >= 1 && x < g.conv_wp - 1;
        }
        if (EPI == FLUX_HIP_EPI_SWIGLU) {
            /* see swiglu_feature: two (gate, up) pairs give eight consecutive features, a last odd pair four */
            bf16 *C = (bf16 *)Cp + (size_t)m * ldc + tn * (BN / 2) + wn * (WN / 2);
            bf16x4 o[TN / 2];
#pragma unroll
            for (int k = 0; k < TN / 2; k++)
#pragma unroll
                for (int e = 0; e < 4; e++) o[k][e] = (bf16)(silu_f(acc[2 * k][j][e]) * acc[2 * k + 1][j][e]);
#pragma unroll
            for (int p = 0; p < TN / 4; p++) store_bf16x8(C + 32 * p + 8 * lq, o[2 * p], o[2 * p + 1], aligned16);
            if (TN / 2 % 2) *(bf16x4 *)(C + 16 * (TN / 2 - 1) + 4 * lq) = o[TN / 2 - 1];
        } else if (EPI == FLUX_HIP_EPI_BF16) {
            /* see bf16_pair_feature: blocks 2p and 2p + 1 give eight consecutive features */
            bf16 *C = (bf16 *)Cp + (size_t)m * ldc + n0 + wn * WN + 8 * lq;
#pragma unroll
            for (int p = 0; p < TN / 2; p++) {
                if (CutTile<BN>::value && n0 + wn * WN + 32 * p >= g.N) continue; /* the same for the whole wave */
                bf16x4 lo, hi;
#pragma unroll
                for (int e = 0; e < 4; e++) { lo[e] = (bf16)acc[2 * p][j][e]; hi[e] = (bf16)acc[2 * p + 1][j][e]; }
                store_bf16x8(C + 32 * p, lo, hi, aligned16);
            }
            if (TN % 2 && !(CutTile<BN>::value && n0 + wn * WN + 16 * (TN - 1) >= g.N)) { /* a last block without a neighbour */
                bf16x4 o;
#pragma unroll
                for (int e = 0; e < 4; e++) o[e] = (bf16)acc[TN - 1][j][e];
                *(bf16x4 *)((bf16 *)Cp + (size_t)m * ldc + n0 + wn * WN + 16 * (TN - 1) + 4 * lq) = o;
            }
        } else {
#pragma unroll
            for (int i = 0; i < TN; i++) {
                if (CutTile<BN>::value && n0 + wn * WN + i * 16 >= g.N) continue; /* the same for the whole wave */
                const int n = n0 + wn * WN + i * 16 + lq * 4;
                if (EPI == EPI_PARTIAL) {
                    *(f32x4 *)(g.ws + ((size_t)ks * g.ws_rows + g.moff[prob] + m) * g.N + n) = acc[i][j];
                } else if (EPI == FLUX_HIP_EPI_F32) {
                    *(f32x4 *)((float *)Cp + (size_t)m * ldc + n) = acc[i][j];
                } else if (EPI == FLUX_HIP_EPI_F32_T) {
#pragma unroll
                    for (int e = 0; e < 4; e++) ((float *)Cp)[(size_t)(n + e) * ldc + m] = acc[i][j][e];
                } else if (EPI == FLUX_HIP_EPI_RESID) {
                    float *p = (float *)Cp + (size_t)m * ldc + n;
                    f32x4 x = *(f32x4 *)p;
                    f32x4 gt = *(const f32x4 *)(g.gate[prob] + n);
#pragma unroll
                    for (int e = 0; e < 4; e++) x[e] += gt[e] * acc[i][j][e];
                    *(f32x4 *)p = x;
                } else if (EPI == FLUX_HIP_EPI_CONV_BF16) {
                    const f32x4 bv = *(const f32x4 *)(g.bias + n);
                    bf16x4 o;
#pragma unroll
                    for (int e = 0; e < 4; e++) {
                        const float v = inside ? acc[i][j][e] + bv[e] : 0.0f;
                        o[e] = (bf16)v;
                        st_s[i] += v;
                        st_q[i] += v * v;
                    }
                    *(bf16x4 *)((bf16 *)Cp + (size_t)m * ldc + n) = o;
                } else if (EPI == FLUX_HIP_EPI_CONV_F32) {
                    const f32x4 bv = *(const f32x4 *)(g.bias + n);
                    f32x4 r = {0.0f, 0.0f, 0.0f, 0.0f};
                    if (g.res) r = *(const f32x4 *)(g.res + (size_t)m * ldc + n);
#pragma unroll
                    for (int e = 0; e < 4; e++) {
                        r[e] = inside ? r[e] + acc[i][j][e] + bv[e] : 0.0f;
                        st_s[i] += r[e];
                        st_q[i] += r[e] * r[e];
                    }
                    *(f32x4 *)((float *)Cp + (size_t)m * ldc + n) = r;
                }
            }
        }
    }
    if (IsConv<EPI>::value && g.stats) {
        /* sum over the 16 rows held by lanes of equal lane/16, then one lane per column quad stores */
#pragma unroll
        for (int i = 0; i < TN; i++) {
#pragma unroll
            for (int o = 1; o < 16; o <<= 1) {
                st_s[i] += __shfl_xor(st_s[i], o);
                st_q[i] += __shfl_xor(st_q[i], o);
            }
            if (l15 == 0) {
                const int n = n0 + wn * WN + i * 16 + lq * 4;
                f32x2 v = {st_s[i], st_q[i]};
                *(f32x2 *)(g.stats + ((size_t)prow * (g.N >> 2) + (n >> 2)) * 2) = v;
            }
        }
    }
}

/* Cp, ldc, tn: where the tile goes - the part's output, or for the fused [Q|K|V|gate|up] projection the output of the
 * side of the boundary the tile lies on (the tile width divides nq_cols, so a tile is wholly on one side) */
template <int BN, int WM, int WN, int EPI, bool PINNED = false>
__device__ __forceinline__ void store_tile(const GemmArgs &g, const TileId &t, f32x4 (&acc)[WN / 16][WM / 16], int m0, int M,
                                           int wm, int wn, int l15, int lq, int prow) {
    if constexpr (EPI == EPI_QKV_SWIGLU) {
        /* HERE = true: each side reads the accumulators through an empty asm statement, row by row. The conversions
         * are then work of that side; left to itself the compiler converted the whole tile to bf16 in front of the
         * branch, for both sides, and kept the hundred results in registers next to the other side's work, past
         * what the register file holds beside the fragments. */
        if (t.tn < g.nq_tiles) store_tile_to<BN, WM, WN, FLUX_HIP_EPI_BF16, true>(g, t, acc, m0, M, wm, wn, l15, lq, prow, g.C[0], g.ldc, t.tn);
        else store_tile_to<BN, WM, WN, FLUX_HIP_EPI_SWIGLU, true>(g, t, acc, m0, M, wm, wn, l15, lq, prow, g.C2, g.ldc2, t.tn - g.nq_tiles);
    } else {
        /* PINNED: the kernels whose accumulators live in AGPRs take them out row by row as well (the 16-byte / 8-byte
         * choice of the bf16 stores is a branch with the same conversions on both sides) */
        store_tile_to<BN, WM, WN, EPI, PINNED>(g, t, acc, m0, M, wm, wn, l15, lq, prow, g.C[t.prob], g.ldc, t.tn);
    }
}

template <int BM, int BN, int WGM, int WGN, int EPI, int NS = 2>
__global__ __launch_bounds__(WGM *WGN * 64) void gemm_kernel(GemmArgs g) {
    constexpr int T = WGM * WGN * 64;
    constexpr int WM = BM / WGM, WN = BN / WGN, TM = WM / 16, TN = WN / 16;
    constexpr int RPP = T / 8; /* tile rows fetched per pass: one wave instruction covers 8 rows */
    constexpr int PA = BM / RPP, PB = BN / RPP;
    constexpr int STAGE = (BM + BN) * 128;
    static_assert(BM % RPP == 0 && BN % RPP == 0, "tile rows must divide evenly over threads");
    static_assert((EPI != FLUX_HIP_EPI_SWIGLU && EPI != EPI_QKV_SWIGLU) || (TN % 2 == 0), "swiglu pairs 16-column blocks");
    extern __shared__ __attribute__((aligned(16))) char smem[];

    TileId t;
    if (!decode_tile(g, blockIdx.x, t)) return;
    const int ks = t.ks, tn = t.tn, prob = t.prob;
    const bf16 *__restrict__ A = g.A[prob];
    const bf16 *__restrict__ W = g.W[prob];
    const int M = g.M[prob];
    const int m0 = t.tml * BM;

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave / WGN, wn = wave % WGN;
    const int lrow = tid >> 3, lchunk = tid & 7;

    /* Per-lane global sources (already un-swizzled) and per-wave LDS destinations. */
    const bf16 *a_ptr[PA];
    const bf16 *b_ptr[PB];
    int a_lds[PA], b_lds[PB];
#pragma unroll
    for (int i = 0; i < PA; i++) {
        int r = lrow + i * RPP;
        int gm = min(m0 + r, M - 1);
        a_ptr[i] = A + (size_t)gm * g.lda + ((lchunk ^ lds_swz(r)) << 3);
        a_lds[i] = (wave * 8 + i * RPP) * 128;
    }
#pragma unroll
    for (int i = 0; i < PB; i++) {
        int v = lrow + i * RPP; /* column of the tile */
        int wrow = weight_row<BN, WN, EPI>(g, tn, v);
        b_ptr[i] = W + (size_t)wrow * g.ldw + ((lchunk ^ lds_swz(v)) << 3);
        b_lds[i] = BM * 128 + (wave * 8 + i * RPP) * 128;
    }
    auto issue = [&](int kt, int stage) {
        char *base = smem + stage * STAGE;
        const int aoff = a_step_offset<EPI>(g, kt);
#pragma unroll
        for (int i = 0; i < PA; i++)
            __builtin_amdgcn_global_load_lds(GLOBAL_PTR(a_ptr[i] + aoff), LDS_PTR(base + a_lds[i]), 16, 0, 0);
#pragma unroll
        for (int i = 0; i < PB; i++)
            __builtin_amdgcn_global_load_lds(GLOBAL_PTR(b_ptr[i] + kt * 64), LDS_PTR(base + b_lds[i]), 16, 0, 0);
    };
    const int kt_begin = ks * g.kt_per;
    const int KT = min(g.K >> 6, kt_begin + g.kt_per) - kt_begin;
    /* NS - 1 stages are requested ahead: with few rows (M <= BM, weights streamed once, hardly any arithmetic) a
     * workgroup is only as fast as the bytes it keeps in flight, and the ring then takes the whole LDS */
#pragma unroll
    for (int s = 0; s < NS - 1; s++)
        if (s < KT) issue(kt_begin + s, s);

    f32x4 acc[TN][TM];
#pragma unroll
    for (int i = 0; i < TN; i++)
#pragma unroll
        for (int j = 0; j < TM; j++)
#pragma unroll
            for (int e = 0; e < 4; e++) acc[i][j][e] = 0.0f;

    const int l15 = lane & 15, lq = lane >> 4;
    const int swzl = lds_swz(l15);
    const int a_frag = (wm * WM + l15) * 128;
    const int b_frag = BM * 128 + (wn * WN + l15) * 128;

    int cur = 0;
    for (int kt = 0; kt < KT; kt++) {
        /* stage `cur` has landed for this wave (the NS - 2 stages requested after it may still be on their way);
         * after the barrier it has for all, and everyone is done reading the stage before it, which is refilled */
        if constexpr (NS > 2) {
            /* __syncthreads() would wait for every load in flight (its fence counts the global->LDS loads); here the
             * wait names what must have landed, and this wave's own LDS reads of the stage that is refilled next */
            if (kt + NS - 2 < KT) asm volatile("s_waitcnt vmcnt(%0) lgkmcnt(0)\n\ts_barrier" ::"n"((NS - 2) * (PA + PB)) : "memory");
            else asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)\n\ts_barrier" ::: "memory");
        } else {
            WAIT_VMCNT0();
            __syncthreads();
        }
        const int refill = cur == 0 ? NS - 1 : cur - 1;
        if (kt + NS - 1 < KT) issue(kt_begin + kt + NS - 1, refill);
        const char *st = smem + cur * STAGE;
#pragma unroll
        for (int kk = 0; kk < 2; kk++) {
            const int coff = ((kk * 4 + lq) ^ swzl) << 4;
            bf16x8 fa[TM], fb[TN];
#pragma unroll
            for (int t = 0; t < TM; t++) fa[t] = *(const bf16x8 *)(st + a_frag + t * 16 * 128 + coff);
#pragma unroll
            for (int t = 0; t < TN; t++) fb[t] = *(const bf16x8 *)(st + b_frag + t * 16 * 128 + coff);
#pragma unroll
            for (int i = 0; i < TN; i++)
#pragma unroll
                for (int j = 0; j < TM; j++)
                    acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(fb[i], fa[j], acc[i][j], 0, 0, 0);
        }
        cur = cur == NS - 1 ? 0 : cur + 1;
    }

    store_tile<BN, WM, WN, EPI>(g, t, acc, m0, M, wm, wn, l15, lq, t.tm * WGM + wm);
}

/* The large tiles: 4 waves (2 x 2), one per SIMD, each owning a (16 TM) x (16 TN) part of a
 * (32 TM) x (32 TN) tile, see the file comment. The MFMA is issued through inline asm so that the
 * accumulator stays in one AGPR quad for the whole loop (left to the register allocator,
 * accumulators migrate between VGPRs and AGPRs with hundreds of copies per K step). Statements with
 * side effects keep their program order, which is what places the LDS reads and global->LDS
 * loads between the MFMAs. */
#define MFMA_AGPR(acc, a, b) asm volatile("v_mfma_f32_16x16x32_bf16 %0, %1, %2, %0" : "+a"(acc) : "v"(a), "v"(b))
/* the first MFMA of an accumulator block: adds to zero instead of to the register's old contents */
#define MFMA_AGPR_NEW(acc, a, b) asm volatile("v_mfma_f32_16x16x32_bf16 %0, %1, %2, 0" : "=a"(acc) : "v"(a), "v"(b))

/* The compiler neither sees those MFMAs' register hazards nor keeps plain register moves in order
 * around them. acc_fence passes every accumulator through an empty asm statement that is ordered
 * with the MFMAs: accumulator writes before it stay before it, reads after it stay after it.
 * Idle cycles for the hazards are placed explicitly next to it. */
template <int TM, int TN>
__device__ __forceinline__ void acc_fence(f32x4 (&acc)[TN][TM]) {
    static_assert(TN == 8 || TN == 7 || TN == 6 || TN == 4, "one asm statement per accumulator column");
#pragma unroll
    for (int j = 0; j < TM; j++) {
        if constexpr (TN == 7)
            asm volatile("" : "+a"(acc[0][j]), "+a"(acc[1][j]), "+a"(acc[2][j]), "+a"(acc[3][j]),
                              "+a"(acc[4][j]), "+a"(acc[5][j]), "+a"(acc[6][j]));
        else if constexpr (TN == 8)
            asm volatile("" : "+a"(acc[0][j]), "+a"(acc[1][j]), "+a"(acc[2][j]), "+a"(acc[3][j]),
                              "+a"(acc[4][j]), "+a"(acc[5][j]), "+a"(acc[6][j]), "+a"(acc[7][j]));
        else if constexpr (TN == 6)
            asm volatile("" : "+a"(acc[0][j]), "+a"(acc[1][j]), "+a"(acc[2][j]), "+a"(acc[3][j]),
                              "+a"(acc[4][j]), "+a"(acc[5][j]));
        else
            asm volatile("" : "+a"(acc[0][j]), "+a"(acc[1][j]), "+a"(acc[2][j]), "+a"(acc[3][j]));
    }
}

/* whether a workgroup of gemm4w_kernel goes on to further tiles (the 4-wave form of the transformer's epilogues;
 * with the convolution epilogues the values kept across tiles would spill) */
template <int EPI, int WAVES> struct Walks4w { static constexpr bool value = !IsConv<EPI>::value && WAVES == 4; };

template <int TM, int TN, int EPI, int WGM = 2, int WGN = 2>
__global__ __launch_bounds__(64 * WGM * WGN) void gemm4w_kernel(GemmArgs g) {
    constexpr int WM = 16 * TM, WN = 16 * TN, BM = WGM * WM, BN = WGN * WN;
    constexpr int RPP = 8 * WGM * WGN; /* tile rows one pass of the workgroup's loads covers: 8 per wave instruction */
    static_assert(BM % RPP == 0 && BN % RPP == 0, "tile rows must divide evenly over the waves' loads");
    constexpr int LA = BM / RPP, LB = BN / RPP;
    constexpr int NL = LA + LB;     /* global->LDS loads per wave and stage: 8 tile rows each */
    constexpr int NF = TM + TN;     /* fragments per K half-step: TN weight side, TM activation side */
    constexpr int NM = TM * TN;     /* MFMAs per K half-step */
    constexpr int RD = NM / NF;     /* one LDS read (and one load) every RD MFMAs */
    constexpr int STAGE = (BM + BN) * 128;
    static_assert((EPI != FLUX_HIP_EPI_SWIGLU && EPI != EPI_QKV_SWIGLU) || (TN % 2 == 0), "swiglu pairs 16-column blocks");
    static_assert(RD >= 2 && RD * (NF - 1) + 1 < NM, "reads and loads must fit between the MFMAs");
    extern __shared__ __attribute__((aligned(16))) char smem[];

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave / WGN, wn = wave % WGN;
    const int lrow = tid >> 3, lchunk = tid & 7;
    const int l15 = lane & 15, lq = lane >> 4;
    const int swzl = lds_swz(l15);
    const int a_frag = (wm * WM + l15) * 128;
    const int b_frag = BM * 128 + (wn * WN + l15) * 128;
    const int coff0 = (lq ^ swzl) << 4, coff1 = ((4 + lq) ^ swzl) << 4;
    /* fragment q of a half-step: 0..TN-1 weight side (MFMA A operand), then activation side */
    auto frag = [&](const char *st, int coff, int q) -> bf16x8 {
        return q < TN ? *(const bf16x8 *)(st + b_frag + q * 2048 + coff) : *(const bf16x8 *)(st + a_frag + (q - TN) * 2048 + coff);
    };

    /* A launch has at most one workgroup per compute unit; each walks the tiles vb, vb + gridDim.x, ...
     * of the virtual grid, so that a tile's stores drain, and the next tile's first stage arrives,
     * while the matrix pipes already work again (with one workgroup per tile, the end of one and the
     * start of the next on a compute unit cost 5-14 us of a 60 us tile). */
    int vb = blockIdx.x;
    TileId t;
    if (!decode_tile(g, vb, t)) return;

    /* Load i of a stage by this wave covers tile rows lrow + RPP i (8 rows of 128 bytes per wave
     * instruction): activation rows for i < LA, weight rows after. Rows RPP apart share a swizzle.
     * The K offset of this workgroup's slice is folded into the per-lane sources. */
    /* Sources are a uniform base per operand (tile's matrix + this workgroup's K slice + the K step, all scalar
     * arithmetic) plus a 32-bit byte offset per lane and load, so that stepping along K costs no vector work. */
    unsigned voff[NL];
    const char *baseA, *baseW;
    auto set_sources = [&](const TileId &tt) {
        const int M = g.M[tt.prob], m0 = tt.tml * BM;
        const int chunk = (lchunk ^ lds_swz(lrow)) << 3;
        baseA = (const char *)(g.A[tt.prob] + tt.ks * g.kt_per * 64);
        baseW = (const char *)(g.W[tt.prob] + tt.ks * g.kt_per * 64);
#pragma unroll
        for (int i = 0; i < LA; i++) voff[i] = ((unsigned)min(m0 + lrow + i * RPP, M - 1) * (unsigned)g.lda + chunk) * 2u;
#pragma unroll
        for (int i = 0; i < LB; i++) voff[LA + i] = ((unsigned)weight_row<BN, WN, EPI>(g, tt.tn, lrow + i * RPP) * (unsigned)g.ldw + chunk) * 2u;
    };
    /* (convolutions never split K, so for them kt below is the absolute K step) */
    auto issue1 = [&](int kt, int stage, int i) {
        const char *base = i < LA ? baseA + (ptrdiff_t)a_step_offset<EPI>(g, kt) * 2 : baseW + kt * 128;
        asm volatile("" : "+v"(voff[i])); /* keeps the load in its scalar base + 32-bit lane offset form, see gemm4d_kernel */
        __builtin_amdgcn_global_load_lds(GLOBAL_PTR(base + voff[i]), LDS_PTR(smem + stage * STAGE + (wave * 8 + i * RPP) * 128), 16, 0, 0);
    };
    set_sources(t);
#pragma unroll
    for (int i = 0; i < NL; i++) issue1(0, 0, i);

    for (;;) {
        const int kt_begin = t.ks * g.kt_per;
        const int KT = min(g.K >> 6, kt_begin + g.kt_per) - kt_begin;

        f32x4 acc[TN][TM];
#pragma unroll
        for (int i = 0; i < TN; i++)
#pragma unroll
            for (int j = 0; j < TM; j++)
#pragma unroll
                for (int e = 0; e < 4; e++) acc[i][j][e] = 0.0f;
        acc_fence<TM, TN>(acc); /* the zeroes are written, and a few cycles pass, before the first MFMA reads them */
        asm volatile("s_nop 7" ::: "memory");

        bf16x8 f0[NF], f1[NF];

        WAIT_VMCNT0();
        __syncthreads();
        if (KT > 1) {
#pragma unroll
            for (int i = 0; i < NL; i++) issue1(1, 1, i);
        }
#pragma unroll
        for (int q = 0; q < NF; q++) f0[q] = frag(smem, coff0, q);

        /* The blocks of a half-step are walked in serpentine order: exactly one MFMA operand changes from one
         * instruction to the next (the matrix pipes draw less power that way than when the weight fragment
         * wraps around together with a new activation fragment). */
        auto serp = [](int b) { return ((b / TN) & 1) ? TN - 1 - b % TN : b % TN; };
        auto step = [&](int kt, auto more_c, auto more2_c) {
            constexpr bool more = decltype(more_c)::value, more2 = decltype(more2_c)::value;
            auto &accr = acc;
            const int cur = kt & 1;
            const char *st = smem + cur * STAGE;
            const char *nx = smem + (cur ^ 1) * STAGE;
            /* first K half of the stage from f0, while the second half's fragments arrive in f1 */
#pragma unroll
            for (int b = 0; b < NM; b++) {
                MFMA_AGPR(accr[serp(b)][b / TN], f0[serp(b)], f0[TN + b / TN]);
                if (b % RD == 0 && b / RD < NF) f1[b / RD] = frag(st, coff1, b / RD);
            }
            if (more) {
                /* the next stage has landed for this wave; past the barrier it has for all, and
                 * everyone has finished reading this stage, which is refilled below */
                WAIT_VMCNT0();
                __syncthreads();
            }
            /* second half from f1, while the next stage's first fragments arrive in f0 and the stage
             * after next is requested; at most one other instruction between two MFMAs */
#pragma unroll
            for (int b = 0; b < NM; b++) {
                MFMA_AGPR(accr[serp(b)][b / TN], f1[serp(b)], f1[TN + b / TN]);
                if (more && b % RD == 0 && b / RD < NF) f0[b / RD] = frag(nx, coff0, b / RD);
                if (more2 && b % RD == 1 && b / RD < NL) issue1(kt + 2, cur, b / RD);
            }
        };
        int kt = 0;
        for (; kt < KT - 2; kt++) step(kt, BoolC<true>{}, BoolC<true>{});
        if (kt < KT - 1) {
            step(kt, BoolC<true>{}, BoolC<false>{});
            kt++;
        }
        step(kt, BoolC<false>{}, BoolC<false>{});

        /* The next tile's first stage is requested before this tile is stored: every wave has taken
         * its last fragments out of LDS once it is past this barrier. */
        const TileId done = t;
        vb += gridDim.x;
        const bool again = Walks4w<EPI, WGM * WGN>::value && vb < g.vgrid && decode_tile(g, vb, t);
        if (again) {
            __syncthreads();
            set_sources(t);
#pragma unroll
            for (int i = 0; i < NL; i++) issue1(0, 0, i);
        }
        asm volatile("s_nop 15\n\ts_nop 15" ::: "memory"); /* the last MFMA results retire before they are read */
        acc_fence<TM, TN>(acc);

        /* The lane's position enters the epilogue through an empty asm statement: what the epilogue derives from it
         * (row and column offsets of every store, for the fused projection those of both store bodies) is then computed
         * per tile. Left visible, the compiler computes all of it once before the first tile and keeps it in registers
         * across the K loops, beyond what the register file holds beside the accumulators and fragments. */
        int l15e = l15, lqe = lq;
        asm volatile("" : "+v"(l15e), "+v"(lqe));
        store_tile<BN, WM, WN, EPI, true>(g, done, acc, done.tml * BM, g.M[done.prob], wm, wn, l15e, lqe, done.tm * WGM + wm);
        if (!again) break;
    }
}

/* The same tiles with deeper operand rings, for the transformer's epilogues. gemm4w_kernel holds two stages and
 * waits at its barrier for every load it has in flight (requested one to two half-steps earlier); operands that
 * come from HBM rather than from a cache arrive later than that now and then, and a wave that waits holds the
 * other three up at the barrier. Here the activation tile and the weight tile have rings of their own, NSA and NSW
 * slots of one K step (128-byte rows, the layout of gemm4w_kernel) each, as many as the 160 KB of LDS hold, and
 * the barrier waits with a count instead of a fence. The MFMA order is that of gemm4w_kernel: bit-identical results.
 *
 * Loads of a K step kt are spread over both of its halves (one load costs a lone wave 12 cycles of matrix-pipe
 * time at one load per eight MFMAs and 19 at one per four). The "first" operand - the one with three slots,
 * activations if both have three - is requested in the first half for step kt + 2, into the slot that step kt - 1
 * left at the last barrier; the "second" operand in the second half for step kt + NS2 (its ring's depth), into
 * the slot whose last reads completed at this step's barrier. The barrier in the middle of step kt needs step
 * kt + 1 in LDS: everything but the loads issued after it, which is a count (vector memory operations of a wave
 * complete in the order of their issue).
 *
 * Tiles follow each other without a gap in that pipeline: the last steps of a tile request the first steps of the
 * workgroup's next tile where they would request steps beyond their own K range, the last step reads the next
 * tile's first fragments, and the ring positions carry over. The finished tile is stored between the two K
 * loops, and nothing waits for those stores there: the first barrier of the next tile allows them (and the
 * loads behind them) to be in flight, the second one needs loads that were issued after them. Before that, a
 * tile began by waiting for every store of its predecessor to be acknowledged and for its own first steps,
 * requested only then, with the matrix pipes idle: 12 % of a 288 x 192 x 3072 tile's time. */
template <int EPI, int TM, int TN>
struct EpilogueOps { /* vector memory instructions a wave issues in the epilogue of a tile whose rows are all valid */
    static constexpr int value = EPI == FLUX_HIP_EPI_SWIGLU || EPI == EPI_QKV_SWIGLU ? TM * (TN / 4 + TN / 2 % 2) /* 16-byte stores + a last 8-byte one */
                                 : EPI == FLUX_HIP_EPI_BF16 ? TM * (TN / 2 + TN % 2) : EPI == FLUX_HIP_EPI_F32_T ? 4 * TM * TN : TM * TN;
};

template <int TM, int TN, int EPI, int NSA, int NSW>
__global__ __launch_bounds__(256) void gemm4d_kernel(GemmArgs g) {
    constexpr int WGM = 2, WGN = 2;
    constexpr int WM = 16 * TM, WN = 16 * TN, BM = WGM * WM, BN = WGN * WN;
    constexpr int RPP = 32; /* tile rows one pass of the workgroup's loads covers: 8 per wave instruction */
    static_assert(BM % RPP == 0 && BN % RPP == 0, "tile rows must divide evenly over the waves' loads");
    constexpr int LA = BM / RPP, LB = BN / RPP, NL = LA + LB;
    constexpr int NF = TM + TN, NM = TM * TN, RD = NM / NF;
    constexpr int ASZ = BM * 128, WSZ = BN * 128;
    static_assert((NSA == 2 || NSA == 3) && (NSW == 2 || NSW == 3) && (NSA == 3 || NSW == 3) && NSA * ASZ + NSW * WSZ <= 160 * 1024,
                  "rings of two or three slots within the LDS, one of them with three");
    static_assert((EPI != FLUX_HIP_EPI_SWIGLU && EPI != EPI_QKV_SWIGLU) || (TN % 2 == 0), "swiglu pairs 16-column blocks");
    static_assert(RD >= 2 && RD * (NF - 1) + 1 < NM, "reads must fit between the MFMAs");
    constexpr bool FIRST_A = NSA == 3;
    constexpr int LF = FIRST_A ? LA : LB, LS = FIRST_A ? LB : LA, NS2 = FIRST_A ? NSW : NSA;
    constexpr int SF = (NM / LF) / RD * RD, SS = (NM / LS) / RD * RD; /* MFMAs between two loads of a half: a multiple of RD */
    static_assert(SF >= RD && SS >= RD && 1 + SF * (LF - 1) < NM && 1 + SS * (LS - 1) < NM, "the loads of a half fit between its MFMAs");
    constexpr int AHEAD = LF + (NS2 == 3 ? LS : 0); /* loads that may be in flight past the barrier */
    /* first barrier of a tile that follows another: also the stored tile's memory operations may be in flight (the wait
     * counter holds 63) */
    constexpr int AHEAD_STORES = AHEAD + EpilogueOps<EPI, TM, TN>::value < 63 ? AHEAD + EpilogueOps<EPI, TM, TN>::value : 63;
    extern __shared__ __attribute__((aligned(16))) char smem[];

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6) & 3;
    const int wm = wave / WGN, wn = wave % WGN;
    const int lrow = tid >> 3, lchunk = tid & 7;
    const int l15 = lane & 15, lq = lane >> 4;
    const int swzl = lds_swz(l15);
    const int coff0 = (lq ^ swzl) << 4, coff1 = ((4 + lq) ^ swzl) << 4;
    const unsigned a_frag = (wm * WM + l15) * 128, w_frag = NSA * ASZ + (wn * WN + l15) * 128;

    int vb = blockIdx.x;
    TileId t;
    if (!decode_tile(g, vb, t)) return;

    /* Sources of a tile's loads: a uniform base per operand (the tile's matrix + this workgroup's K slice) and a 32-bit
     * byte offset per lane and load, so that stepping along K is scalar work. Two sets: the tile being multiplied and
     * the workgroup's next one. */
    struct Src {
        unsigned voff[NL];
        const char *baseA, *baseW;
    };
    Src cur, nxt;
    auto set_sources = [&](Src &sc, const TileId &tt) {
        const int M = g.M[tt.prob], m0 = tt.tml * BM;
        /* the lane's row enters through an empty asm statement, so that the per-load row numbers derived from it (two
         * sets of weight rows for the fused projection) are computed here, per tile, and not once before the first
         * tile, from where they would have to be kept in registers across every K loop */
        int lr = lrow;
        asm volatile("" : "+v"(lr));
        const int chunk = (lchunk ^ lds_swz(lr)) << 3;
        sc.baseA = (const char *)(g.A[tt.prob] + tt.ks * g.kt_per * 64);
        sc.baseW = (const char *)(g.W[tt.prob] + tt.ks * g.kt_per * 64);
#pragma unroll
        for (int i = 0; i < LA; i++) sc.voff[i] = ((unsigned)min(m0 + lr + i * RPP, M - 1) * (unsigned)g.lda + chunk) * 2u;
#pragma unroll
        for (int i = 0; i < LB; i++) sc.voff[LA + i] = ((unsigned)weight_row<BN, WN, EPI>(g, tt.tn, lr + i * RPP) * (unsigned)g.ldw + chunk) * 2u;
    };
    /* load i of K step kt of the tile whose sources are (baseA, baseW, vo): activation rows for i < LA (into slot sa
     * of their ring), weight rows after (slot sw). The offset passes through an empty asm statement where it is used: the
     * load is then selected in its "scalar base + 32-bit lane offset" form. Without it the compiler widens every offset
     * to 64 bits once, outside the K loop, keeps NL register pairs instead of NL registers, and adds the base with a
     * 64-bit vector addition in front of every load. */
    auto issue1 = [&](const char *baseA, const char *baseW, unsigned &vo, int kt, int sa, int sw, int i) {
        const char *base = (i < LA ? baseA : baseW) + (ptrdiff_t)kt * 128;
        const int dst = i < LA ? sa * ASZ + (wave * 8 + i * RPP) * 128 : NSA * ASZ + sw * WSZ + (wave * 8 + (i - LA) * RPP) * 128;
        asm volatile("" : "+v"(vo));
        __builtin_amdgcn_global_load_lds(GLOBAL_PTR(base + vo), LDS_PTR(smem + dst), 16, 0, 0);
    };
    auto k_steps = [&](const TileId &tt) { return min(g.K >> 6, tt.ks * g.kt_per + g.kt_per) - tt.ks * g.kt_per; };
    /* The first K steps of a tile that no predecessor requested, into slots 0, 1 (and 2): what the pipeline below has
     * in flight when it enters a tile's step 0, oldest first */
    auto prime = [&](Src &sc, int KTn) {
#pragma unroll
        for (int s = 0; s < 2; s++) {
            if (s < KTn) {
#pragma unroll
                for (int i = 0; i < NL; i++) issue1(sc.baseA, sc.baseW, sc.voff[i], s, s, s, i);
            }
        }
        if (NS2 == 3 && KTn > 2) {
#pragma unroll
            for (int n = 0; n < LS; n++) issue1(sc.baseA, sc.baseW, sc.voff[(FIRST_A ? LA : 0) + n], 2, 2, 2, (FIRST_A ? LA : 0) + n);
        }
    };

    bf16x8 f0[NF], f1[NF];
    int ca = 0, cw = 0;                   /* ring slots of the step being multiplied */
    unsigned va = a_frag, vw = w_frag;    /* this lane's fragment rows in those slots */
    auto frag = [&](unsigned xa, unsigned xw, int coff, int q) -> bf16x8 {
        return q < TN ? *(const bf16x8 *)(smem + xw + coff + q * 2048) : *(const bf16x8 *)(smem + xa + coff + (q - TN) * 2048);
    };
    /* the first tile: its first steps are requested here, and everything has landed before its step 0 */
    set_sources(cur, t);
    prime(cur, k_steps(t));
    asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)\n\ts_barrier" ::: "memory");
#pragma unroll
    for (int q = 0; q < NF; q++) f0[q] = frag(va, vw, coff0, q);
    bool strict = false; /* the first barrier of the tile must not count on the stored tile's operations */

    for (;;) {
        const int KT = k_steps(t); /* at least 4: the host sends shorter K ranges to gemm4w_kernel */

        f32x4 acc[TN][TM]; /* started by the MFMAs of step 0's first half (no pass over 4 TM TN registers to clear them) */

        auto serp = [](int b) { return ((b / TN) & 1) ? TN - 1 - b % TN : b % TN; };
        /* TAIL = false: steps kt + 1 .. kt + 3 belong to this tile. TAIL = true: one of the last three steps of a tile;
         * loads for steps beyond its K range request the first steps of the tile in nxt instead (every load is issued,
         * so the wait counts stay exact). WAIT: what may be in flight at the barrier. */
        auto step = [&](int kt, auto tail_c, auto wait_c, auto first_c) {
            constexpr bool TAIL = decltype(tail_c)::value;
            constexpr int WAIT = decltype(wait_c)::value;
            constexpr bool FIRST = decltype(first_c)::value; /* step 0: its first half starts the accumulators */
            auto &accr = acc;
            const int na = ca == NSA - 1 ? 0 : ca + 1, nw = cw == NSW - 1 ? 0 : cw + 1;
            const unsigned van = a_frag + na * ASZ, vwn = w_frag + nw * WSZ;
            auto load = [&](int ks, int sa, int sw, int i) {
                if (!TAIL) {
                    issue1(cur.baseA, cur.baseW, cur.voff[i], ks, sa, sw, i);
                } else {
                    const bool over = ks >= KT;
                    unsigned vo = over ? nxt.voff[i] : cur.voff[i];
                    issue1(over ? nxt.baseA : cur.baseA, over ? nxt.baseW : cur.baseW, vo, over ? ks - KT : ks, sa, sw, i);
                }
            };
#pragma unroll
            for (int b = 0; b < NM; b++) {
                if (FIRST) MFMA_AGPR_NEW(accr[serp(b)][b / TN], f0[serp(b)], f0[TN + b / TN]);
                else MFMA_AGPR(accr[serp(b)][b / TN], f0[serp(b)], f0[TN + b / TN]);
                if (b % RD == 0 && b / RD < NF) f1[b / RD] = frag(va, vw, coff1, b / RD);
                /* step kt + 2 of the first operand, into the slot that step kt - 1 left */
                if (b % SF == 1 && b / SF < LF) load(kt + 2, ca == 0 ? 2 : ca - 1, cw == 0 ? 2 : cw - 1, (FIRST_A ? 0 : LA) + b / SF);
            }
            /* step kt + 1 has landed for this wave and its reads of step kt are complete; past the barrier both hold
             * for all */
            if (FIRST && strict) asm volatile("s_waitcnt vmcnt(%0)" ::"n"(AHEAD) : "memory");
            asm volatile("s_waitcnt vmcnt(%0) lgkmcnt(0)\n\ts_barrier" ::"n"(WAIT) : "memory");
#pragma unroll
            for (int b = 0; b < NM; b++) {
                MFMA_AGPR(accr[serp(b)][b / TN], f1[serp(b)], f1[TN + b / TN]);
                if (b % RD == 0 && b / RD < NF) f0[b / RD] = frag(van, vwn, coff0, b / RD);
                /* step kt + NS2 of the second operand, into the slot of step kt */
                if (b % SS == 1 && b / SS < LS) load(kt + NS2, ca, cw, (FIRST_A ? LA : 0) + b / SS);
            }
            ca = na;
            cw = nw;
            va = van;
            vw = vwn;
        };
        /* step 0: the stored tile's memory operations are older than anything its barrier needs (for the first tile
         * everything has landed already) */
        step(0, BoolC<false>{}, IntC<AHEAD_STORES>{}, BoolC<true>{});
        int kt = 1;
        for (; kt < KT - 3; kt++) step(kt, BoolC<false>{}, IntC<AHEAD>{}, BoolC<false>{});

        /* the workgroup's next tile: its first steps are requested by this tile's last ones. After the last tile they
         * request this tile's first steps once more, into slots that nobody reads again. */
        const TileId done = t;
        vb += gridDim.x;
        const bool again = vb < g.vgrid && decode_tile(g, vb, t);
        if (again) set_sources(nxt, t);
        else nxt = cur;
        for (; kt < KT; kt++) step(kt, BoolC<true>{}, IntC<AHEAD>{}, BoolC<false>{});

        asm volatile("s_nop 15\n\ts_nop 15" ::: "memory"); /* the last MFMA results retire before they are read */
        acc_fence<TM, TN>(acc);

        /* The lane's position enters the epilogue through an empty asm statement: what the epilogue derives from it
         * (row and column offsets of every store, for the fused projection those of both store bodies) is then computed
         * per tile. Left visible, the compiler computes all of it once before the first tile and keeps it in registers
         * across the K loops, beyond what the register file holds beside the accumulators and fragments. */
        int l15e = l15, lqe = lq;
        asm volatile("" : "+v"(l15e), "+v"(lqe));
        store_tile<BN, WM, WN, EPI, true>(g, done, acc, done.tml * BM, g.M[done.prob], wm, wn, l15e, lqe, done.tm * WGM + wm);
        if (!again) break;
        /* not every row of this wave's part of the stored tile was valid, or not every column: it issued fewer than
         * EpilogueOps operations */
        strict = done.tml * BM + wm * WM + WM > g.M[done.prob] || (CutTile<BN>::value && done.tn == g.ntiles - 1);
        cur = nxt;
    }
    /* the requests made in place of a next tile's land in this workgroup's LDS: not after it has gone */
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
}

/* ------------------------------------------------------------------ host side */

static int g_persistent = 1;
extern "C" void flux_hip_linear_persistent(int on) { g_persistent = on; }
static int compute_units() {
    static int n = 0;
    if (!n) {
        int dev = 0;
        if (hipGetDevice(&dev) != hipSuccess || hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n < 8) n = 256;
    }
    return n;
}

static void set_row_tiles(GemmArgs &g, int BM) {
    int end = 0;
    for (int i = 0; i < GEMM_MAX_PARTS; i++) {
        end += (g.M[i] + BM - 1) / BM; /* empty parts (M = 0) add nothing */
        g.mt_end[i] = end;
    }
    g.mtiles = end;
}

template <int BM, int BN, int WGM, int WGN, int EPI, int NS = 2>
static int launch_cfg(GemmArgs &g) {
    constexpr int T = WGM * WGN * 64;
    constexpr int LDS = NS * (BM + BN) * 128;
    static_assert(LDS <= 160 * 1024 && (NS - 2) * ((BM + BN) * 8 / T) < 64, "the ring fits the LDS, the loads in flight the wait counter");
    static bool attr_done = false;
    auto kern = gemm_kernel<BM, BN, WGM, WGN, EPI, NS>;
    if (!attr_done) {
        HIP_OK(hipFuncSetAttribute((const void *)kern, hipFuncAttributeMaxDynamicSharedMemorySize, LDS));
        attr_done = true;
    }
    set_row_tiles(g, BM);
    g.ntiles = g.N / BN;
    g.nq_tiles = g.nq_cols / BN;
    g.total_tiles = g.mtiles * g.ntiles;
    int grid = (g.total_tiles * g.ksplit + 7) & ~7;
    g.vgrid = grid;
    hipLaunchKernelGGL(kern, dim3(grid), dim3(T), LDS, flux_hip_stream_handle(), g);
    HIP_OK(hipGetLastError());
    return 1;
}

template <int TM, int TN, int EPI, int WGM = 2, int WGN = 2>
static int launch_4w(GemmArgs &g) {
    constexpr int BM = 16 * TM * WGM, BN = 16 * TN * WGN, LDS = 2 * (BM + BN) * 128;
    static bool attr_done = false;
    auto kern = gemm4w_kernel<TM, TN, EPI, WGM, WGN>;
    if (!attr_done) {
        HIP_OK(hipFuncSetAttribute((const void *)kern, hipFuncAttributeMaxDynamicSharedMemorySize, LDS));
        attr_done = true;
    }
    set_row_tiles(g, BM);
    g.ntiles = g.N / BN;
    g.nq_tiles = g.nq_cols / BN;
    g.total_tiles = g.mtiles * g.ntiles;
    /* the kernel addresses operand rows with 32-bit byte offsets from the matrix base */
    size_t span = ((size_t)max(max(g.w_row0, g.w_row1), g.w_row2) + g.N) * g.ldw * 2;
    for (int i = 0; i < GEMM_MAX_PARTS; i++) span = max(span, (size_t)g.M[i] * g.lda * 2);
    if (span >= ((size_t)1 << 32)) return g.N % 128 == 0 ? launch_cfg<128, 128, 2, 2, EPI>(g) : launch_cfg<64, 64, 2, 2, EPI>(g);
    /* one workgroup fits on a compute unit (registers, LDS): launch at most that many, each walks its share of the tiles */
    g.vgrid = (g.total_tiles * g.ksplit + 7) & ~7;
    const int grid = g_persistent && Walks4w<EPI, WGM * WGN>::value ? min(g.vgrid, compute_units() & ~7) : g.vgrid;
    hipLaunchKernelGGL(kern, dim3(grid), dim3(64 * WGM * WGN), LDS, flux_hip_stream_handle(), g);
    HIP_OK(hipGetLastError());
    return 1;
}

static int g_ring = 1;
extern "C" void flux_hip_linear_ring(int on) { g_ring = on; }

/* The deep-ring form of the 4-wave tiles: one workgroup per compute unit at most, each walks its share of the tiles. */
template <int TM, int TN, int EPI, int NSA, int NSW>
static int launch_4d(GemmArgs &g) {
    constexpr int BM = 32 * TM, BN = 32 * TN, LDS = (NSA * BM + NSW * BN) * 128;
    static bool attr_done = false;
    auto kern = gemm4d_kernel<TM, TN, EPI, NSA, NSW>;
    if (!attr_done) {
        HIP_OK(hipFuncSetAttribute((const void *)kern, hipFuncAttributeMaxDynamicSharedMemorySize, LDS));
        attr_done = true;
    }
    set_row_tiles(g, BM);
    g.ntiles = (g.N + BN - 1) / BN; /* (a last tile that is cut off: CutTile) */
    g.nq_tiles = g.nq_cols / BN;
    g.total_tiles = g.mtiles * g.ntiles;
    size_t span = ((size_t)max(max(g.w_row0, g.w_row1), g.w_row2) + g.N) * g.ldw * 2;
    for (int i = 0; i < GEMM_MAX_PARTS; i++) span = max(span, (size_t)g.M[i] * g.lda * 2);
    if (span >= ((size_t)1 << 32)) return g.N % 128 == 0 ? launch_cfg<128, 128, 2, 2, EPI>(g) : launch_cfg<64, 64, 2, 2, EPI>(g);
    g.vgrid = (g.total_tiles * g.ksplit + 7) & ~7;
    const int grid = min(g.vgrid, compute_units() & ~7);
    hipLaunchKernelGGL(kern, dim3(grid), dim3(256), LDS, flux_hip_stream_handle(), g);
    HIP_OK(hipGetLastError());
    return 1;
}

template <int EPI>
static int launch_epi(GemmArgs &g, int tile) {
    /* the ring kernel runs its tiles as one pipeline and wants at least four K steps in every K slice (the last slice
     * may be shorter than the others); shorter ones go to the two-stage kernel */
    const int kt_total = g.K >> 6, kt_last = kt_total - (g.ksplit - 1) * g.kt_per;
    if (g_ring && g_persistent && g.kt_per >= 4 && kt_last >= 4) {
        /* three weight slots, two activation slots: in a denoising step the weights always come from HBM, the
         * activations mostly from the memory-side cache (measured per kernel in a step, this split beat the other
         * one by 0 - 10 %); the 192 x 192 tile has room for three of each */
        switch (tile) {
            case 2: return launch_4d<8, 8, EPI, 2, 3>(g);
            case 5: return launch_4d<9, 6, EPI, 2, 3>(g);
            case 6: return launch_4d<6, 6, EPI, 3, 3>(g);
            case 7: return launch_4d<8, 6, EPI, 2, 3>(g);
            case 11:
                if constexpr (EPI == FLUX_HIP_EPI_RESID || EPI == FLUX_HIP_EPI_BF16) return launch_4d<8, 7, EPI, 2, 3>(g);
                break;
            default: break;
        }
    }
    if (tile == 11) tile = g.N % 256 == 0 ? 2 : 1; /* (the dispatch offers 256 x 224 only where the ring kernel takes it) */
    switch (tile) {
        case 2: return launch_4w<8, 8, EPI>(g);
        case 5: return launch_4w<9, 6, EPI>(g);
        case 6: return launch_4w<6, 6, EPI>(g);
        case 7: return launch_4w<8, 6, EPI>(g);
        case 4: return launch_4w<8, 4, EPI, 2, 4>(g); /* 8 waves, two per SIMD, on the 256x256 tile */
        case 1: return launch_cfg<128, 128, 2, 2, EPI>(g);
        case 3: return launch_cfg<64, 64, 2, 2, EPI>(g);
        case 8: return launch_cfg<64, 128, 2, 2, EPI, 6>(g);  /* few rows: the same tiles with a ring that fills the LDS */
        case 9: return launch_cfg<128, 128, 2, 2, EPI, 5>(g);
        case 10: return launch_cfg<96, 128, 2, 2, EPI, 5>(g);
        default: return launch_cfg<64, 128, 2, 2, EPI>(g);
    }
}

/* The convolution epilogues exist for the tiles whose width divides 64, 128, 256 or 512 output
 * channels. */
template <int EPI>
static int launch_conv(GemmArgs &g, int tile) {
    switch (tile) {
        case 2: return launch_4w<8, 8, EPI>(g);
        case 1: return launch_cfg<128, 128, 2, 2, EPI>(g);
        case 3: return launch_cfg<64, 64, 2, 2, EPI>(g);
        default: return launch_cfg<64, 128, 2, 2, EPI>(g);
    }
}

/* Second pass of a split-K GEMM: sums the K slices ws[s][moff + m][n] in a fixed order and
 * applies the epilogue to the sum (for the residual form the same arithmetic as gated_add,
 * flux_transformer.c:90-97). For SwiGLU the workspace holds plain columns - gate features in
 * [0, N/2), up features in [N/2, N) - and thread n4 combines column n with column N/2 + n. */
template <int EPI>
__global__ __launch_bounds__(256) void splitk_finish_kernel(GemmArgs g) {
    const int ncols = EPI == FLUX_HIP_EPI_SWIGLU ? g.N >> 1 : g.N;
    const int n4 = ncols >> 2;
    const size_t total = (size_t)g.ws_rows * n4;
    size_t idx = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (idx >= total) return;
    int row = (int)(idx / n4), n = (int)(idx - (size_t)row * n4) << 2;
    /* moff[i] = first workspace row of part i; unused parts start at ws_rows */
    int prob = (row >= g.moff[1]) + (row >= g.moff[2]) + (row >= g.moff[3]);
    int m = row - g.moff[prob];
    f32x4 sum = {0.0f, 0.0f, 0.0f, 0.0f}, sum2 = {0.0f, 0.0f, 0.0f, 0.0f};
    for (int s = 0; s < g.ksplit; s++) {
        const float *w = g.ws + ((size_t)s * g.ws_rows + g.moff[prob] + m) * g.N + n;
        f32x4 v = *(const f32x4 *)w;
#pragma unroll
        for (int e = 0; e < 4; e++) sum[e] += v[e];
        if (EPI == FLUX_HIP_EPI_SWIGLU) {
            f32x4 u = *(const f32x4 *)(w + ncols);
#pragma unroll
            for (int e = 0; e < 4; e++) sum2[e] += u[e];
        }
    }
    if (EPI == FLUX_HIP_EPI_RESID) {
        float *p = (float *)g.C[prob] + (size_t)m * g.ldc + n;
        f32x4 x = *(f32x4 *)p;
        f32x4 gt = *(const f32x4 *)(g.gate[prob] + n);
#pragma unroll
        for (int e = 0; e < 4; e++) x[e] += gt[e] * sum[e];
        *(f32x4 *)p = x;
    } else if (EPI == FLUX_HIP_EPI_F32) {
        *(f32x4 *)((float *)g.C[prob] + (size_t)m * g.ldc + n) = sum;
    } else {
        bf16x4 o;
#pragma unroll
        for (int e = 0; e < 4; e++) o[e] = (bf16)(EPI == FLUX_HIP_EPI_SWIGLU ? silu_f(sum[e]) * sum2[e] : sum[e]);
        *(bf16x4 *)((bf16 *)g.C[prob] + (size_t)m * g.ldc + n) = o;
    }
}

/* What follows a residual projection in every block is the AdaLN of the updated rows
 * (apply_adaln, flux_transformer.c:979-1048). When the projection ran as K slices, this kernel is
 * its second pass and that normalisation in one: a workgroup owns one row, sums the slices in
 * the fixed order, updates x (as splitk_finish_kernel<RESID> does), and while the row is still in
 * registers computes mean and biased variance (two passes) and writes
 * (1 + scale) * (x - mean) / sqrt(var + eps) + shift as bf16. One read of the partial sums, one
 * read and write of x, one write of the normalised row. N <= 4096. */
struct AdalnArgs {
    bf16 *out[GEMM_MAX_PARTS];
    const float *shift[GEMM_MAX_PARTS], *scale[GEMM_MAX_PARTS]; /* RMS form: scale = the norm's weight, shift unused */
    int ldo;
    float eps;
};

__device__ __forceinline__ float block_sum_256(float v, float *red) {
    for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o);
    __syncthreads(); /* red is free again */
    if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = v;
    __syncthreads();
    return (red[0] + red[1]) + (red[2] + red[3]);
}

/* RMS = true: the norm that follows is x / sqrt(mean(x^2) + eps) * weight instead (qwen3_rms_norm,
 * flux_qwen3.c:177-197) */
template <bool RMS>
__global__ __launch_bounds__(256) void splitk_finish_adaln_kernel(GemmArgs g, AdalnArgs a) {
    __shared__ float red[4];
    const int row = blockIdx.x;
    const int prob = (row >= g.moff[1]) + (row >= g.moff[2]) + (row >= g.moff[3]);
    const int m = row - g.moff[prob];
    const int N = g.N;
    f32x4 v[4];
#pragma unroll
    for (int i = 0; i < 4; i++) v[i] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
    /* What the row needs besides the partial sums is requested ahead of its use - the residual and its gate in front of
     * the slices, scale and shift in front of the sums over the row - so that the row costs two round trips to memory
     * rather than four in a row (with 80 to 768 rows the kernel is a few waves per compute unit that wait for memory
     * most of their time). */
    float *xr = (float *)g.C[prob] + (size_t)m * g.ldc;
    f32x4 x0[4], gt0[4], sc0[4], sh0[4];
#pragma unroll
    for (int i = 0; i < 4; i++) {
        const int c = (i * 256 + threadIdx.x) * 4;
        if (c < N) {
            x0[i] = *(const f32x4 *)(xr + c);
            gt0[i] = *(const f32x4 *)(g.gate[prob] + c);
        }
    }
    /* slices four at a time, so that a row with many short slices keeps enough loads in flight;
     * the additions stay in slice order */
    const size_t slice = (size_t)g.ws_rows * N;
    const float *w0 = g.ws + (size_t)row * N;
    int s = 0;
    for (; s + 4 <= g.ksplit; s += 4) {
        f32x4 t[4][4];
#pragma unroll
        for (int u = 0; u < 4; u++)
#pragma unroll
            for (int i = 0; i < 4; i++) {
                const int c = (i * 256 + threadIdx.x) * 4;
                if (c < N) t[u][i] = *(const f32x4 *)(w0 + (size_t)(s + u) * slice + c);
            }
#pragma unroll
        for (int u = 0; u < 4; u++)
#pragma unroll
            for (int i = 0; i < 4; i++) {
                const int c = (i * 256 + threadIdx.x) * 4;
                if (c < N) {
#pragma unroll
                    for (int e = 0; e < 4; e++) v[i][e] += t[u][i][e];
                }
            }
    }
    for (; s < g.ksplit; s++) {
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const int c = (i * 256 + threadIdx.x) * 4;
            if (c < N) {
                const f32x4 t = *(const f32x4 *)(w0 + (size_t)s * slice + c);
#pragma unroll
                for (int e = 0; e < 4; e++) v[i][e] += t[e];
            }
        }
    }
#pragma unroll
    for (int i = 0; i < 4; i++) {
        const int c = (i * 256 + threadIdx.x) * 4;
        if (c < N) {
            sc0[i] = *(const f32x4 *)(a.scale[prob] + c);
            if (!RMS) sh0[i] = *(const f32x4 *)(a.shift[prob] + c);
        }
    }
    float s1 = 0.0f;
#pragma unroll
    for (int i = 0; i < 4; i++) {
        const int c = (i * 256 + threadIdx.x) * 4;
        if (c < N) {
            f32x4 x = x0[i];
            const f32x4 gt = gt0[i];
#pragma unroll
            for (int e = 0; e < 4; e++) x[e] += gt[e] * v[i][e];
            *(f32x4 *)(xr + c) = x;
            v[i] = x;
            s1 += (x[0] + x[1]) + (x[2] + x[3]);
        }
    }
    const float mean = RMS ? 0.0f : block_sum_256(s1, red) / (float)N;
    float q = 0.0f;
#pragma unroll
    for (int i = 0; i < 4; i++) {
        const int c = (i * 256 + threadIdx.x) * 4;
        if (c < N) {
#pragma unroll
            for (int e = 0; e < 4; e++) { const float d = v[i][e] - mean; q += d * d; }
        }
    }
    const float inv = 1.0f / sqrtf(block_sum_256(q, red) / (float)N + a.eps);
    bf16 *o = a.out[prob] + (size_t)m * a.ldo;
#pragma unroll
    for (int i = 0; i < 4; i++) {
        const int c = (i * 256 + threadIdx.x) * 4;
        if (c < N) {
            const f32x4 sc = sc0[i];
            bf16x4 r;
            if (RMS) {
#pragma unroll
                for (int e = 0; e < 4; e++) r[e] = (bf16)(v[i][e] * inv * sc[e]);
            } else {
                const f32x4 sh = sh0[i];
#pragma unroll
                for (int e = 0; e < 4; e++) r[e] = (bf16)((1.0f + sc[e]) * ((v[i][e] - mean) * inv) + sh[e]);
            }
            *(bf16x4 *)(o + c) = r;
        }
    }
}

template <int EPI>
static int launch_split(GemmArgs &g, int tile) {
    if (!launch_epi<EPI_PARTIAL>(g, tile)) return 0;
    const size_t total = (size_t)g.ws_rows * ((EPI == FLUX_HIP_EPI_SWIGLU ? g.N >> 1 : g.N) >> 2);
    hipLaunchKernelGGL(splitk_finish_kernel<EPI>, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, flux_hip_stream_handle(), g);
    return hipGetLastError() == hipSuccess ? 1 : flux_hip_fail("split-K reduction launch failed");
}

static int launch_split_adaln(GemmArgs &g, int tile, const AdalnArgs &a) {
    if (!launch_epi<EPI_PARTIAL>(g, tile)) return 0;
    if (a.shift[0])
        hipLaunchKernelGGL(splitk_finish_adaln_kernel<false>, dim3((unsigned)g.ws_rows), dim3(256), 0, flux_hip_stream_handle(), g, a);
    else
        hipLaunchKernelGGL(splitk_finish_adaln_kernel<true>, dim3((unsigned)g.ws_rows), dim3(256), 0, flux_hip_stream_handle(), g, a);
    return hipGetLastError() == hipSuccess ? 1 : flux_hip_fail("split-K reduction + AdaLN launch failed");
}

/* Workspace of flux_hip_linear_static: the K slices' partial sums live in this array instead of in
 * memory from hipMalloc. Each GPU that loads the library holds its own copy until the process ends.
 * In host code the array's name is only a handle for hipGetSymbolAddress; the address a kernel can
 * use is asked for once per device (static_ws_for_current_device) and kept. */
#define STATIC_WS_BYTES ((size_t)FLUX_HIP_LINEAR_STATIC_BYTES)
static __device__ __align__(256) float g_static_ws[STATIC_WS_BYTES / sizeof(float)];
#define STATIC_WS_MAX_DEVICES 64
static float *g_static_ws_ptr[STATIC_WS_MAX_DEVICES];

static float *static_ws_for_current_device() {
    int dev = -1;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= STATIC_WS_MAX_DEVICES) {
        flux_hip_fail("flux_hip_linear_static: no current device (or a device number beyond %d)", STATIC_WS_MAX_DEVICES - 1);
        return nullptr;
    }
    if (!g_static_ws_ptr[dev]) {
        float *p = nullptr;
        const hipError_t e = hipGetSymbolAddress((void **)&p, HIP_SYMBOL(g_static_ws));
        if (e != hipSuccess || !p) {
            flux_hip_fail("flux_hip_linear_static: hipGetSymbolAddress failed: %s", hipGetErrorString(e));
            return nullptr;
        }
        g_static_ws_ptr[dev] = p;
    }
    return g_static_ws_ptr[dev];
}

/* called by flux_hip_init with its device current */
extern "C" int flux_hip_linear_static_init(void) { return static_ws_for_current_device() != nullptr; }

extern "C" void flux_hip_linear_release(void);
static float *g_ws = nullptr;
static size_t g_ws_bytes = 0;
static int ensure_ws(size_t bytes) {
    if (bytes <= g_ws_bytes) return 1;
    HIP_OK(hipStreamSynchronize(flux_hip_stream_handle()));
    if (g_ws) (void)hipFree(g_ws);
    g_ws = nullptr;
    g_ws_bytes = 0;
    HIP_OK(hipMalloc((void **)&g_ws, bytes));
    g_ws_bytes = bytes;
    return 1;
}

extern "C" void flux_hip_linear_release(void) {
    if (g_ws) (void)hipFree(g_ws);
    g_ws = nullptr;
    g_ws_bytes = 0;
}

static int g_force_tile = -1;
static unsigned g_tile_mask = 0xFEF; /* tiles the automatic choice may use: all but the 8-wave form of 256 x 256 */
static int g_splitk_enabled = 1;
extern "C" void flux_hip_linear_force_tile(int tile) { g_force_tile = tile; }
extern "C" void flux_hip_linear_tile_mask(unsigned mask) { g_tile_mask = mask ? mask : 0xFEF; }
extern "C" void flux_hip_linear_enable_splitk(int on) { g_splitk_enabled = on; }
static int g_force_split = 0; /* > 1: every projection that can run as K slices runs as this many (comparison runs and tests) */
extern "C" void flux_hip_linear_force_split(int slices) { g_force_split = slices > 1 ? slices : 0; }

/* Launch probe: HIP events around every launch with one chosen epilogue, so a benchmark can
 * read that kernel's average duration inside its timed region. */
#define PROBE_MAX 4096
static int g_probe_epi = -1, g_probe_n = 0;
static hipEvent_t g_probe_ev[PROBE_MAX][2];
static unsigned char g_probe_tile[PROBE_MAX];
static int g_probe_created = 0;

extern "C" int flux_hip_linear_probe(int epilogue) {
    g_probe_epi = epilogue;
    g_probe_n = 0;
    return 1;
}

/* Count and summed duration of the recorded launches that used `tile` (-1: all of them). The
 * record is kept until the next flux_hip_linear_probe call. */
extern "C" int flux_hip_linear_probe_read_tile(int tile, int *launches, float *total_ms) {
    float sum = 0.0f;
    int n = 0;
    for (int i = 0; i < g_probe_n; i++) {
        if (tile >= 0 && g_probe_tile[i] != tile) continue;
        float ms = 0.0f;
        HIP_OK(hipEventSynchronize(g_probe_ev[i][1]));
        HIP_OK(hipEventElapsedTime(&ms, g_probe_ev[i][0], g_probe_ev[i][1]));
        sum += ms;
        n++;
    }
    if (launches) *launches = n;
    if (total_ms) *total_ms = sum;
    return 1;
}

extern "C" int flux_hip_linear_probe_read(int *launches, float *total_ms) {
    return flux_hip_linear_probe_read_tile(-1, launches, total_ms);
}

/* Duration and tile id of each recorded launch, in launch order; returns how many were written. */
extern "C" int flux_hip_linear_probe_read_launches(int max, int *tiles, float *ms) {
    int n = 0;
    for (int i = 0; i < g_probe_n && n < max; i++, n++) {
        float t = 0.0f;
        if (hipEventSynchronize(g_probe_ev[i][1]) != hipSuccess || hipEventElapsedTime(&t, g_probe_ev[i][0], g_probe_ev[i][1]) != hipSuccess) return -1;
        if (tiles) tiles[n] = g_probe_tile[i];
        if (ms) ms[n] = t;
    }
    return n;
}

static int probe_slot(int epilogue) {
    const bool conv = epilogue == FLUX_HIP_EPI_CONV_BF16 || epilogue == FLUX_HIP_EPI_CONV_F32;
    if ((g_probe_epi == -2 ? !conv : epilogue != g_probe_epi) || g_probe_n >= PROBE_MAX) return -1;
    while (g_probe_created <= g_probe_n) {
        if (hipEventCreate(&g_probe_ev[g_probe_created][0]) != hipSuccess) return -1;
        if (hipEventCreate(&g_probe_ev[g_probe_created][1]) != hipSuccess) return -1;
        g_probe_created++;
    }
    return g_probe_n++;
}

/* Tile and K-split choice, then the launch; `allowed` has bit t set for every tile id that may be used. */
static int gemm_dispatch(GemmArgs &g, int np, int epilogue, unsigned allowed, int *tile_out = nullptr, const AdalnArgs *adaln = nullptr,
                         int *adaln_done = nullptr, float *fixed_ws = nullptr, size_t fixed_ws_bytes = 0) {
    /* Choose tile and K split with a small cost model: workgroups run in rounds over
     * 256 CUs x occupancy; a workgroup's time is its FLOPs at the tile's measured rate plus a
     * fixed prologue/epilogue cost; the launch cannot beat the time to stream its operands,
     * which depends on how many bytes the resident workgroups keep in flight. */
    /* tile ids: 0..3 the small tiles and 256 x 256, 4 = the 8-wave form of 256 x 256 (only when
     * forced, for comparison runs), 5 = 288 x 192, 6 = 192 x 192, 7 = 256 x 192, 8, 9 and 10 = 64 x 128, 128 x 128 and
     * 96 x 128 with a ring of 6, 5 and 5 stages instead of 2 (one workgroup per compute unit; for parts of at most that
     * many rows), 11 = 256 x 224 (4096 + 512 rows x 3072 columns are 252 such tiles, one round of workgroups on 256
     * compute units of which each does 7/8 of a 256 x 256 tile's work; 216 tiles of 256 x 256 are one round as well) */
    constexpr int NT = 12;
    static const int bm[NT] = {64, 128, 256, 64, 256, 288, 192, 256, 64, 128, 96, 256}, bn[NT] = {128, 128, 256, 64, 256, 192, 192, 192, 128, 128, 128, 224};
    static const int occ[NT] = {3, 2, 1, 4, 1, 1, 1, 1, 1, 1, 1, 1}, ahead[NT] = {1, 1, 1, 1, 1, 1, 1, 1, 5, 4, 4, 1}; /* stages a workgroup keeps in flight */
    static const double rate[NT] = {2.0e12, 2.9e12, 6.05e12, 1.5e12, 4.6e12, 6.0e12, 5.7e12, 5.75e12, 1.6e12, 3.0e12, 2.4e12, 5.9e12}; /* FLOP/s of one CU running this tile */
    const int kt_total = g.K >> 6;
    int tile = -1, best_split = 1;
    {
        double best = 1e30;
        static const int splits[] = {1, 2, 3, 4, 6, 8, 12, 16, 24, 32};
        /* every epilogue but the transposed store can run as K slices + a finishing pass; for
         * SwiGLU the gate and up rows must be one contiguous block of the weight matrix */
        const int N = g.N, K = g.K, w_row0 = g.w_row0, w_row1 = g.w_row1;
        const bool can_split = g_splitk_enabled &&
                               (epilogue == FLUX_HIP_EPI_RESID || epilogue == FLUX_HIP_EPI_BF16 || epilogue == FLUX_HIP_EPI_F32 ||
                                (epilogue == FLUX_HIP_EPI_SWIGLU && w_row1 == w_row0 + N / 2));
        double rows = 0.0;
        for (int i = 0; i < np; i++) rows += g.M[i];
        for (int t = 0; t < NT; t++) {
            /* 256 x 224 (tile 11) divides no width and cuts its last column tile off: for the outputs whose stores can do
             * that, through the ring kernel only, never in K slices */
            const bool cut = t == 11;
            if (cut && !((epilogue == FLUX_HIP_EPI_RESID || epilogue == FLUX_HIP_EPI_BF16) && g_ring && g_persistent && kt_total >= 4)) continue;
            /* bf16 outputs leave in pairs of 16-column blocks: the cut must fall between two pairs of a wave's 112 columns */
            if (cut && epilogue == FLUX_HIP_EPI_BF16 && (N % 224) % 112 % 32 != 0) continue;
            if (!cut && (N % bn[t] || g.nq_cols % bn[t])) continue;
            if (!((allowed >> t) & 1)) continue;
            if (ahead[t] > 1) { /* the deep rings stream the weights once: every part in one row tile */
                bool fits = true;
                for (int i = 0; i < np; i++) fits = fits && g.M[i] <= bm[t];
                if (!fits) continue;
            }
            long tiles = 0;
            for (int i = 0; i < np; i++) tiles += (g.M[i] + bm[t] - 1) / bm[t];
            tiles *= (N + bn[t] - 1) / bn[t];
            for (int si = 0; si < 10; si++) {
                const int sp = splits[si];
                if (sp > 1 && (cut || !can_split || kt_total / sp < 4)) break;
                if (g_force_split && can_split && sp != g_force_split && kt_total / g_force_split >= 4) continue;
                if (sp > 1 && fixed_ws && (double)sp * rows * N * sizeof(float) > (double)fixed_ws_bytes) {
                    /* the slices must fit the given workspace: fewer slices then, down to none - unless this number
                     * of slices was demanded, which is the one request the fixed workspace refuses */
                    if (sp == g_force_split)
                        return flux_hip_fail("flux_hip_linear_static: %d K slices of %.0f rows x %d columns need %.1f MiB of partial sums, beyond the maximum "
                                             "of %zu MiB of the static workspace", sp, rows, N, sp * rows * N * 4.0 / 1048576.0, fixed_ws_bytes >> 20);
                    break;
                }
                const int per = (kt_total + sp - 1) / sp;
                const long blocks = tiles * ((kt_total + per - 1) / per);
                const long slots = 256L * occ[t];
                const long rounds = (blocks + slots - 1) / slots;
                const long resident = blocks < slots ? blocks : slots;
                const long per_cu = (resident + 255) / 256;          /* workgroups sharing one CU */
                const double t_block = 2.0 * bm[t] * bn[t] * 64.0 * per / (rate[t] / per_cu) + 2.5e-6;
                double t_compute = rounds * t_block;
                const double bytes = (rows + N) * (double)K * 2.0;
                /* what a launch that only streams its operands has been seen to reach: 3.2-3.5 TB/s with two LDS stages
                 * (every step waits for the loads it has just requested), 4.3-5.2 TB/s with a deep ring */
                const double bw_cap = ahead[t] > 1 ? 4.6e12 : 3.4e12;
                double bw = 5.5e12 * (double)(resident * ahead[t] * (bm[t] + bn[t]) * 128) / 12.0e6;
                if (bw > bw_cap) bw = bw_cap;
                double est = t_compute > bytes / bw ? t_compute : bytes / bw;
                if (sp > 1) est += 3.0e-6 + (sp + 2.0) * rows * N * 4.0 / 4.0e12;
                if (est < best) { best = est; tile = t; best_split = sp; }
            }
        }
    }
    if (tile < 0) tile = g.N % 128 == 0 ? 1 : 3; /* no permitted tile divides N (a forced tile that does not fit): 128 x 128, else 64 x 64 */
    g.ksplit = 1;
    g.kt_per = kt_total;
    if (best_split > 1) {
        g.kt_per = (kt_total + best_split - 1) / best_split;
        g.ksplit = (kt_total + g.kt_per - 1) / g.kt_per;
        g.ws_rows = 0;
        for (int i = 0; i < GEMM_MAX_PARTS; i++) {
            g.moff[i] = g.ws_rows;
            g.ws_rows += g.M[i];
        }
        if (fixed_ws) {
            g.ws = fixed_ws;
        } else {
            if (!ensure_ws((size_t)g.ksplit * g.ws_rows * g.N * sizeof(float))) return 0;
            g.ws = g_ws;
        }
    }

    if (tile_out) *tile_out = tile;
    /* the launch probe creates events: never on the path that promises to allocate nothing */
    const int slot = fixed_ws ? -1 : probe_slot(epilogue);
    if (slot >= 0) g_probe_tile[slot] = (unsigned char)tile;
    if (slot >= 0) (void)hipEventRecord(g_probe_ev[slot][0], flux_hip_stream_handle());
    int ok;
    const bool split = g.ksplit > 1;
    switch (epilogue) {
        case FLUX_HIP_EPI_BF16: ok = split ? launch_split<FLUX_HIP_EPI_BF16>(g, tile) : launch_epi<FLUX_HIP_EPI_BF16>(g, tile); break;
        case FLUX_HIP_EPI_F32: ok = split ? launch_split<FLUX_HIP_EPI_F32>(g, tile) : launch_epi<FLUX_HIP_EPI_F32>(g, tile); break;
        case FLUX_HIP_EPI_F32_T: ok = launch_epi<FLUX_HIP_EPI_F32_T>(g, tile); break;
        case FLUX_HIP_EPI_RESID:
            if (split && adaln) {
                ok = launch_split_adaln(g, tile, *adaln);
                if (adaln_done) *adaln_done = ok;
            } else {
                ok = split ? launch_split<FLUX_HIP_EPI_RESID>(g, tile) : launch_epi<FLUX_HIP_EPI_RESID>(g, tile);
            }
            break;
        case FLUX_HIP_EPI_SWIGLU: ok = split ? launch_split<FLUX_HIP_EPI_SWIGLU>(g, tile) : launch_epi<FLUX_HIP_EPI_SWIGLU>(g, tile); break;
        case EPI_QKV_SWIGLU: ok = launch_epi<EPI_QKV_SWIGLU>(g, tile); break;
        case FLUX_HIP_EPI_CONV_BF16: ok = launch_conv<FLUX_HIP_EPI_CONV_BF16>(g, tile); break;
        case FLUX_HIP_EPI_CONV_F32: ok = launch_conv<FLUX_HIP_EPI_CONV_F32>(g, tile); break;
        default: return flux_hip_fail("flux_hip_linear: unknown epilogue %d", epilogue);
    }
    if (slot >= 0) (void)hipEventRecord(g_probe_ev[slot][1], flux_hip_stream_handle());
    return ok;
}

static int linear_impl(int epilogue, int nparts, const flux_hip_linear_part *parts, int N, int K, int lda, int ldw, int ldc, int w_row0,
                       int w_row1, const flux_hip_adaln_part *norm, float eps, int *fused, float *fixed_ws = nullptr, size_t fixed_ws_bytes = 0,
                       const char *who = "flux_hip_linear") {
    if (epilogue < FLUX_HIP_EPI_BF16 || epilogue > FLUX_HIP_EPI_SWIGLU) return flux_hip_fail("%s: unknown epilogue %d", who, epilogue);
    if (nparts < 1 || nparts > GEMM_MAX_PARTS) return flux_hip_fail("%s: nparts=%d (1 to %d)", who, nparts, GEMM_MAX_PARTS);
    if (K <= 0 || (K & 63)) return flux_hip_fail("%s: K=%d must be a positive multiple of 64", who, K);
    if (N <= 0 || (N & 127)) return flux_hip_fail("%s: N=%d must be a positive multiple of 128", who, N);
    if (lda < K || ldw < K || (lda & 7) || (ldw & 7))
        return flux_hip_fail("%s: lda=%d ldw=%d must be >= K and multiples of 8", who, lda, ldw);
    if (epilogue != FLUX_HIP_EPI_F32_T && (ldc & 3)) return flux_hip_fail("%s: ldc=%d must be a multiple of 4", who, ldc);
    GemmArgs g = {};
    AdalnArgs a = {};
    int maxm = 0;
    for (int i = 0; i < nparts; i++) {
        if (parts[i].M < 0) return flux_hip_fail("flux_hip_linear: negative row count");
        if (parts[i].M > 0 && (!parts[i].A || !parts[i].W || !parts[i].C))
            return flux_hip_fail("flux_hip_linear: NULL operand");
        if (epilogue == FLUX_HIP_EPI_RESID && parts[i].M > 0 && !parts[i].gate)
            return flux_hip_fail("flux_hip_linear: residual epilogue needs a gate vector");
        if (parts[i].M > 0 && ((((uintptr_t)parts[i].A | (uintptr_t)parts[i].W | (uintptr_t)parts[i].gate) & 15) ||
                               ((uintptr_t)parts[i].C & (epilogue == FLUX_HIP_EPI_F32_T ? 3 : epilogue == FLUX_HIP_EPI_BF16 || epilogue == FLUX_HIP_EPI_SWIGLU ? 7 : 15))))
            return flux_hip_fail("flux_hip_linear: operands must be 16-byte aligned (bf16 outputs 8-byte)");
    }
    /* drop empty parts */
    int np = 0;
    for (int i = 0; i < nparts; i++) {
        if (parts[i].M == 0) continue;
        g.A[np] = (const bf16 *)parts[i].A;
        g.W[np] = (const bf16 *)parts[i].W;
        g.C[np] = parts[i].C;
        g.gate[np] = parts[i].gate;
        g.M[np] = parts[i].M;
        if (norm) {
            a.out[np] = (bf16 *)norm[i].out_bf16;
            a.shift[np] = norm[i].shift;
            a.scale[np] = norm[i].scale;
        }
        if (parts[i].M > maxm) maxm = parts[i].M;
        np++;
    }
    if (np == 0) return 1;
    g.N = N; g.K = K; g.lda = lda; g.ldw = ldw; g.ldc = ldc; g.w_row0 = w_row0; g.w_row1 = w_row1;
    a.ldo = N;
    a.eps = eps;
    return gemm_dispatch(g, np, epilogue, (g_force_tile >= 0 ? 1u << g_force_tile : g_tile_mask) & 0xFFFu, nullptr, norm ? &a : nullptr, fused,
                         fixed_ws, fixed_ws_bytes);
}

extern "C" int flux_hip_linear(int epilogue, int nparts, const flux_hip_linear_part *parts,
                               int N, int K, int lda, int ldw, int ldc, int w_row0, int w_row1) {
    return linear_impl(epilogue, nparts, parts, N, K, lda, ldw, ldc, w_row0, w_row1, nullptr, 0.0f, nullptr);
}

/* One launch for the fused projection of a single-stream block, see the header. Never split along K. */
extern "C" int flux_hip_linear_qkv_swiglu(const void *A, const void *W, void *qkv_out, void *mlp_out, int M, int qkv_cols, int mlp, int K,
                                          int lda, int ldw, int ld_qkv, int ld_mlp) {
    if (M <= 0) return 1;
    if (K <= 0 || (K & 63)) return flux_hip_fail("flux_hip_linear_qkv_swiglu: K=%d must be a positive multiple of 64", K);
    if (qkv_cols <= 0 || (qkv_cols & 127) || mlp <= 0 || (mlp & 63))
        return flux_hip_fail("flux_hip_linear_qkv_swiglu: qkv_cols=%d must be a multiple of 128, mlp=%d of 64", qkv_cols, mlp);
    if (lda < K || ldw < K || (lda & 7) || (ldw & 7) || (ld_qkv & 3) || (ld_mlp & 3))
        return flux_hip_fail("flux_hip_linear_qkv_swiglu: bad leading dimensions");
    if (!A || !W || !qkv_out || !mlp_out) return flux_hip_fail("flux_hip_linear_qkv_swiglu: NULL operand");
    if ((((uintptr_t)A | (uintptr_t)W) & 15) || (((uintptr_t)qkv_out | (uintptr_t)mlp_out) & 7))
        return flux_hip_fail("flux_hip_linear_qkv_swiglu: operands must be 16-byte aligned (outputs 8-byte)");
    GemmArgs g = {};
    g.A[0] = (const bf16 *)A; g.W[0] = (const bf16 *)W; g.C[0] = qkv_out; g.C2 = mlp_out; g.M[0] = M;
    g.N = qkv_cols + 2 * mlp; g.K = K; g.lda = lda; g.ldw = ldw; g.ldc = ld_qkv; g.ldc2 = ld_mlp;
    g.w_row0 = 0; g.w_row1 = qkv_cols; g.w_row2 = qkv_cols + mlp; g.nq_cols = qkv_cols;
    int tile = -1;
    const int saved = g_splitk_enabled;
    g_splitk_enabled = 0;
    const int ok = gemm_dispatch(g, 1, EPI_QKV_SWIGLU, (g_force_tile >= 0 ? 1u << g_force_tile : g_tile_mask) & 0xFFFu, &tile);
    g_splitk_enabled = saved;
    return ok;
}

/* flux_hip_linear for callers that must not allocate: the partial sums of the K slices go to the
 * static device array above. Nothing here or below it calls hipMalloc, hipFree or an allocating
 * library routine. Every partial sum the second pass reads has been written by the first pass of the
 * same call, so the array needs no clearing between calls; calls that overlap on one GPU (two
 * streams, two host threads) would share it and race. */
extern "C" int flux_hip_linear_static(int epilogue, int nparts, const flux_hip_linear_part *parts,
                                      int N, int K, int lda, int ldw, int ldc, int w_row0, int w_row1) {
    float *ws = static_ws_for_current_device();
    if (!ws) return 0;
    return linear_impl(epilogue, nparts, parts, N, K, lda, ldw, ldc, w_row0, w_row1, nullptr, 0.0f, nullptr, ws, STATIC_WS_BYTES,
                       "flux_hip_linear_static");
}

/* The residual projection, and - when it runs as K slices - the AdaLN of the updated rows in its
 * second pass, see the header. */
extern "C" int flux_hip_linear_resid_adaln(int nparts, const flux_hip_linear_part *parts, int N, int K, int lda, int ldw, int ldc,
                                           const flux_hip_adaln_part *norm, float eps, int *fused) {
    if (!fused) return flux_hip_fail("flux_hip_linear_resid_adaln: fused must not be NULL");
    *fused = 0;
    if (norm) {
        if (N > 4096) return flux_hip_fail("flux_hip_linear_resid_adaln: N=%d (at most 4096 columns per row)", N);
        for (int i = 0; i < nparts && i < GEMM_MAX_PARTS; i++)
            if (parts[i].M > 0 && (!norm[i].out_bf16 || !norm[i].scale || (!norm[i].shift) != (!norm[0].shift) ||
                                   (((uintptr_t)norm[i].out_bf16 | (uintptr_t)norm[i].shift | (uintptr_t)norm[i].scale) & 15)))
                return flux_hip_fail("flux_hip_linear_resid_adaln: NULL or unaligned norm operand (shift must be given for all parts or for none)");
    }
    return linear_impl(FLUX_HIP_EPI_RESID, nparts, parts, N, K, lda, ldw, ldc, 0, 0, norm, eps, fused);
}



/* Convolution over a zero-bordered channels-last image as one GEMM, see the header. */
extern "C" int flux_hip_conv_stats(int epilogue, const void *in, const void *w, const float *bias, const float *res, void *out, int rows,
                                   int wp, int cin, int cout, int taps, float *stats, int *stats_rows);

extern "C" int flux_hip_conv(int epilogue, const void *in, const void *w, const float *bias, const float *res,
                             void *out, int rows, int wp, int cin, int cout, int taps) {
    return flux_hip_conv_stats(epilogue, in, w, bias, res, out, rows, wp, cin, cout, taps, nullptr, nullptr);
}

/* The same, and (stats != NULL) the sums for the group norm that follows, see the header. */
extern "C" int flux_hip_conv_stats(int epilogue, const void *in, const void *w, const float *bias, const float *res, void *out, int rows,
                                   int wp, int cin, int cout, int taps, float *stats, int *stats_rows) {
    if (epilogue != FLUX_HIP_EPI_CONV_BF16 && epilogue != FLUX_HIP_EPI_CONV_F32)
        return flux_hip_fail("flux_hip_conv: epilogue %d is not a convolution epilogue", epilogue);
    if (taps != 1 && taps != 9) return flux_hip_fail("flux_hip_conv: taps=%d (1 or 9)", taps);
    if (rows <= 0 || cin <= 0 || (cin & 63) || cout <= 0 || (cout & 63))
        return flux_hip_fail("flux_hip_conv: rows=%d cin=%d cout=%d (channels must be multiples of 64)", rows, cin, cout);
    if (taps == 9 && (wp < 3 || rows % wp || rows / wp < 3 || cin > 64 * 227))
        return flux_hip_fail("flux_hip_conv: a 3x3 convolution needs a bordered image (rows=%d wp=%d cin=%d)", rows, wp, cin);
    if (wp > 0 && rows % wp) return flux_hip_fail("flux_hip_conv: rows=%d is not a multiple of the image width %d", rows, wp);
    if (!in || !w || !bias || !out) return flux_hip_fail("flux_hip_conv: NULL operand");
    if ((((uintptr_t)in | (uintptr_t)w | (uintptr_t)bias | (uintptr_t)res | (uintptr_t)out) & 15))
        return flux_hip_fail("flux_hip_conv: operands must be 16-byte aligned");
    if (res && epilogue != FLUX_HIP_EPI_CONV_F32) return flux_hip_fail("flux_hip_conv: only the fp32 epilogue adds a residual");
    GemmArgs g = {};
    g.A[0] = (const bf16 *)in;
    g.W[0] = (const bf16 *)w;
    g.C[0] = out;
    g.M[0] = rows;
    g.N = cout; g.K = taps * cin; g.lda = cin; g.ldw = taps * cin; g.ldc = cout;
    g.conv_taps = taps; g.conv_wp = wp; g.conv_hp = wp > 0 ? rows / wp : 0;
    g.bias = bias; g.res = res; g.stats = stats;
    if (stats && (!stats_rows || ((uintptr_t)stats & 7))) return flux_hip_fail("flux_hip_conv_stats: stats needs stats_rows and 8-byte alignment");
    const unsigned conv_tiles = 0x0F; /* 64x128, 128x128, 256x256 (4 waves), 64x64 */
    static const int width[4] = {128, 128, 256, 64};
    unsigned allowed;
    if (g_force_tile >= 0 && g_force_tile < 4 && cout % width[g_force_tile] == 0) {
        allowed = 1u << g_force_tile; /* a forced tile that this layer cannot use is ignored */
    } else {
        /* These layers move many bytes per FLOP (fp32 image in and out of the epilogue), which a
         * second resident workgroup hides and the one-workgroup-per-CU 256 x 256 tile does not:
         * measured over the decoder's layers, 128 x 128 wins (3-15 %) until the launch is at least
         * eight full rounds of 256 x 256 tiles, where the big tile's higher MFMA rate takes over. */
        const long big_tiles = cout % 256 ? 0 : (long)((rows + 255) / 256) * (cout / 256);
        allowed = big_tiles >= 2048 ? 1u << 2 : cout % 128 == 0 ? 1u << 1 : 1u << 3;
    }
    int tile = -1;
    if (!gemm_dispatch(g, 1, epilogue, allowed & conv_tiles, &tile)) return 0;
    static const int tile_rows[4] = {64, 128, 256, 64}; /* every convolution tile is two waves high */
    if (stats_rows) *stats_rows = 2 * ((rows + tile_rows[tile & 3] - 1) / tile_rows[tile & 3]);
    return 1;
}
