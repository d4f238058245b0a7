/*
 * flux_hip_debug.h - test and measurement switches of libflux_hip.so.
 *
 * None of these has a counterpart in the reference and none is needed to use the library; an
 * application includes flux_hip.h only. They are process-wide mutable state (like the reference's
 * own globals, flux_kernels.c:32-45): set one, run, and restore the default. tests/conftest.py
 * restores all of them before every test module.
 */
#ifndef FLUX_HIP_DEBUG_H
#define FLUX_HIP_DEBUG_H

#include "flux_hip.h"

#ifdef __cplusplus
extern "C" {
#endif

/* force_tile: 0/1/2/3/5/6/7 pins the GEMM tile of flux_hip_linear (64x128, 128x128, 256x256, 64x64,
 * 288x192, 192x192, 256x192; 4 = 256x256 in its 8-wave form, never chosen automatically; 8 / 9 / 10 = 64x128 / 128x128 / 96x128
 * with a ring of 6 / 5 / 5 LDS stages, only for row ranges of at most 64 / 128 / 96 rows; 11 = 256x224, whose last column
 * tile is cut off at N: for the residual and bf16 epilogues with at least four 64-wide K steps and no K slices), -1
 * restores the automatic choice (a tile whose width does not divide N is skipped, tile 11 apart; if none is left the
 * 128x128 tile runs). */
void flux_hip_linear_force_tile(int tile);
/* bit t set = the automatic choice may use tile t (default 0xFEF: all but tile 4; 0 restores it) */
void flux_hip_linear_tile_mask(unsigned mask);
/* 0 turns the split-K path off (default 1) */
void flux_hip_linear_enable_splitk(int on);
/* slices > 1: projections whose epilogue and K length allow it run as exactly that many K slices (one of 2, 3, 4, 6,
 * 8, 12, 16, 24, 32; at least four 64-wide K steps per slice), whatever the cost model would choose; 0 (default):
 * the cost model chooses. With flux_hip_linear_static a demanded number of slices whose partial sums do not fit the
 * static workspace is refused. */
void flux_hip_linear_force_split(int slices);
/* 1 (default): the 4-wave GEMM launches at most one workgroup per compute unit and each walks several
 * tiles; 0: one workgroup per tile */
void flux_hip_linear_persistent(int on);
/* 1 (default): the 4-wave tiles run as gemm4d_kernel (operand rings of two or three LDS slots, count-based waits at
 * the barrier); 0: as gemm4w_kernel (two stages, everything in flight awaited at the barrier). Bit-identical results. */
void flux_hip_linear_ring(int on);
/* attention kernel: -1 and 15 = automatic (default: 64-query waves, block lengths chosen per sequence length);
 * 0 / 1 = the 32-query-per-wave kernel with 128 / 256 queries per workgroup; 11..14 = 16, 32, 48, 64 queries per wave
 * throughout */
void flux_hip_attention_force_variant(int v);
/* 1 (default): a CFG step runs its two forwards as one batch of two sequences; 0: one after the other.
 * Takes effect at the next flux_hip_session_begin. */
void flux_hip_set_batched_cfg(int on);
/* The fused projection of a single-stream block: 1 (default) = one launch (flux_hip_linear_qkv_swiglu), 0 = two
 * (QKV, then gate/up). */
void flux_hip_set_fused_qkv_mlp(int on);
/* VAE attention: at most `rows` query rows per chunk (0 = default: 1 GB of fp32 scores per chunk). */
void flux_hip_vae_set_attention_chunk(int rows);

/* Launch probe: probe(epilogue) records HIP events around every later flux_hip_linear launch with
 * that epilogue (-2: every flux_hip_conv launch; -1 stops); probe_read waits for them and returns
 * their count and summed duration, probe_read_tile the same for the launches that used one tile id,
 * probe_read_launches copies out, in launch order, the tile id and duration (ms) of up to `max`
 * recorded launches and returns their number (-1 on error). */
int flux_hip_linear_probe(int epilogue);
int flux_hip_linear_probe_read(int *launches, float *total_ms);
int flux_hip_linear_probe_read_tile(int tile, int *launches, float *total_ms);
int flux_hip_linear_probe_read_launches(int max, int *tiles, float *ms);

/* What the matrix pipes sustain on their own: a register-resident loop of independent bf16 MFMAs on every
 * compute unit (one workgroup each, waves_per_simd = 1 or 2 waves per SIMD; `iters` x 16 MFMAs per wave),
 * run launches + 1 times; the best launch's rate in TFLOP/s goes to *tflops. shape 0 =
 * v_mfma_f32_16x16x32_bf16, 1 = v_mfma_f32_32x32x16_bf16; pattern 0 = all-zero operands, 1 = values in
 * [1, 2) with a random low byte, 2 = random bit patterns. `bench.py --workload mfma_peak` prints the table. */
int flux_hip_mfma_peak(int shape, int pattern, int waves_per_simd, int iters, int launches, float *tflops);
/* What an instruction between a lone wave's MFMAs costs the matrix pipe (csrc/microbench.hip): mode 0 nothing,
 * 1 global_load_lds_dwordx4, 2 ds_read_b128, 3 v_exp_f32, 4 three v_fma_f32, 5 global_load_dwordx4 + ds_write_b128; one
 * such instruction behind every `every`-th MFMA (1, 2, 4, 8, 16). Returns clock cycles per MFMA (16 = no loss) and
 * the core clock of the run. */
int flux_hip_mfma_issue_cost(int mode, int every, int iters, float *cycles_per_mfma, float *ghz);

#ifdef __cplusplus
}
#endif
#endif /* FLUX_HIP_DEBUG_H */
