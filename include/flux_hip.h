/*
 * flux_hip.h - C ABI of the MI355X (gfx950) backend for the FLUX.2-klein
 * denoising transformer.
 *
 * Three layers, all plain C (pointers and sizes only):
 *   1. runtime:   device lifetime, buffers, errors       (role of flux_metal.h:23-129, 140-198)
 *   2. operators: one entry point per hot operator, on device pointers
 *                 (role of flux_kernels.h:22-226 and the flux_gpu_* list in flux_metal.h:214-529)
 *   3. model:     loader, forward passes and samplers with the reference's own
 *                 names and signatures (flux.c:45-110), so the reference's
 *                 flux.c links against this library unchanged.
 *
 * Conventions: functions returning int give 1 on success and 0 on failure
 * (as the reference's GPU operators do, flux_metal.h:232-234); functions
 * returning pointers give NULL on failure. flux_hip_last_error() then holds a
 * message. Nothing here falls back to a CPU path: without a usable GPU every
 * call fails. Not thread-safe (neither is the reference: see the globals at
 * flux_kernels.c:32-45): one forward at a time per process.
 *
 * Switches that pin a tile, a kernel variant or a code path for tests and measurements, and the
 * launch probe the benchmark reads, are process-wide state and no part of this interface: they are
 * declared in flux_hip_debug.h.
 */
#ifndef FLUX_HIP_H
#define FLUX_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* ------------------------------------------------------------------ runtime */

/* Selects device 0 and creates the compute stream. Idempotent.
 * Replaces flux_metal_init (flux_metal.h:23). */
int flux_hip_init(void);
/* 1 when a gfx950 device is usable. Replaces flux_metal_available (flux_metal.h:28). */
int flux_hip_available(void);
/* Releases the stream. Replaces flux_metal_cleanup (flux_metal.h:33). */
void flux_hip_cleanup(void);
/* Waits for all queued work. Replaces flux_metal_sync / flux_gpu_sync (flux_metal.h:106,277). */
int flux_hip_sync(void);
/* Last failure message (static storage), "" if none. Role of flux_get_error (flux.c:155-169). */
const char *flux_hip_last_error(void);
/* The backend's stream as an opaque hipStream_t, for callers that time or profile. */
void *flux_hip_stream(void);

/* Device buffers: role of flux_gpu_tensor_alloc/create/read/free (flux_metal.h:147-188). */
void *flux_hip_malloc(size_t bytes);
void flux_hip_free(void *dptr);
int flux_hip_upload(void *dst, const void *src, size_t bytes);
int flux_hip_download(void *dst, const void *src, size_t bytes);
int flux_hip_memset(void *dst, int value, size_t bytes);

/* Timing helper on the backend's stream: returns elapsed milliseconds between
 * flux_hip_timer_start() and flux_hip_timer_stop() measured with HIP events. */
int flux_hip_timer_start(void);
float flux_hip_timer_stop(void);

/* ---------------------------------------------------------------- operators */

/* Output handling of flux_hip_linear. */
enum {
    FLUX_HIP_EPI_BF16 = 0,    /* C bf16 [M, ldc] = A W^T */
    FLUX_HIP_EPI_F32 = 1,     /* C f32  [M, ldc] = A W^T */
    FLUX_HIP_EPI_F32_T = 2,   /* C f32  [N, ldc] = (A W^T)^T  (token-major -> channel-major) */
    FLUX_HIP_EPI_RESID = 3,   /* C f32  [M, ldc] += gate[n] * (A W^T)      gated_add, flux_transformer.c:90 */
    FLUX_HIP_EPI_SWIGLU = 4,  /* C bf16 [M, ldc] = silu(A Wg^T) * (A Wu^T) swiglu, flux_transformer.c:1749-1757 */
    /* 5 is used inside the library */
    FLUX_HIP_EPI_CONV_BF16 = 6, /* flux_hip_conv: out bf16 = conv + bias, zeros on the image border */
    FLUX_HIP_EPI_CONV_F32 = 7   /* flux_hip_conv: out f32 = [res +] conv + bias, zeros on the image border */
};

/* One row range of a linear layer. */
typedef struct {
    const void *A;      /* bf16 [M, lda] activations */
    const void *W;      /* bf16 [rows, ldw] weight, row-major [out, in] */
    void *C;            /* output, type per epilogue */
    const float *gate;  /* f32 [N], FLUX_HIP_EPI_RESID only */
    int M;              /* rows */
} flux_hip_linear_part;

/*
 * y = x W^T on MFMA, bf16 inputs, fp32 accumulation. Replaces flux_linear_nobias /
 * flux_linear_nobias_bf16 (flux_kernels.h:59,66; flux_kernels.c:210-320) and, through the
 * epilogues, gated_add (flux_transformer.c:90), flux_silu + flux_mul_inplace
 * (flux_kernels.c:120,581) and the output transposes (flux_transformer.c:3547-3552).
 * Up to four row ranges with their own weights run in one launch (the image and text streams
 * of a double block, for one sequence or for the two sequences of a batched CFG step). K % 64 == 0 and N % 128 == 0 are required.
 * For FLUX_HIP_EPI_SWIGLU, N counts gate+up columns (2*mlp); gate rows start at W row w_row0,
 * up rows at w_row1; the output has N/2 columns. Otherwise W rows [w_row0, w_row0+N) are used.
 */
int flux_hip_linear(int epilogue, int nparts, const flux_hip_linear_part *parts,
                    int N, int K, int lda, int ldw, int ldc, int w_row0, int w_row1);

/*
 * The fused projection of a single-stream block in one launch: the reference runs one linear
 * hidden -> 3*hidden + 2*mlp whose output rows are [Q, K, V, gate, up] (flux_transformer.c:3034-3058).
 * Here A bf16 [M, lda] is multiplied by W bf16 [qkv_cols + 2*mlp, ldw] once; output columns
 * [0, qkv_cols) are stored as bf16 to qkv_out [M, ld_qkv], and for the rest silu(gate) * up
 * (weight rows qkv_cols.. are the gate, qkv_cols + mlp.. the up features) goes as bf16 to
 * mlp_out [M, ld_mlp] (mlp columns). Bit for bit what flux_hip_linear gives in two launches with
 * FLUX_HIP_EPI_BF16 and FLUX_HIP_EPI_SWIGLU on the same tile; the activations are read once and
 * one launch has all the column tiles. qkv_cols % 128 == 0, mlp % 64 == 0, K % 64 == 0.
 */
int flux_hip_linear_qkv_swiglu(const void *A, const void *W, void *qkv_out, void *mlp_out, int M, int qkv_cols, int mlp, int K,
                               int lda, int ldw, int ld_qkv, int ld_mlp);

/*
 * flux_hip_linear that allocates nothing. No counterpart in the reference: it is for callers that
 * cannot call hipMalloc - code under HIP graph capture, tight serving loops, harnesses that forbid
 * allocation. flux_hip_linear takes a workspace from hipMalloc (kept and grown on demand) when it
 * runs a projection with few rows and a long K as K slices; this entry point keeps the slices'
 * fp32 partial sums in a static device array of FLUX_HIP_LINEAR_STATIC_BYTES instead, which every GPU
 * the library runs on holds until the process ends, and considers only as many slices as fit there.
 * Same arguments, epilogues and results (to fp32 summation order when the number of slices differs)
 * as flux_hip_linear, at every size: a call whose outputs (row counts of all parts together times N)
 * exceed FLUX_HIP_LINEAR_STATIC_MAX_OUTPUTS cannot keep even two slices in the array and runs as one
 * launch without slices, which needs no workspace at all (the large projections of the model never
 * split anyway). The one thing it refuses, with an error that says so and before anything is
 * launched, is a number of slices demanded through flux_hip_linear_force_split (flux_hip_debug.h)
 * whose partial sums exceed the array. It creates no events either: the launch probe of
 * flux_hip_debug.h does not see these calls. All calls on one GPU share the array: calls that overlap
 * there (two streams, two host threads) race. The array's contents need no clearing between calls.
 */
#define FLUX_HIP_LINEAR_STATIC_BYTES (64u << 20)
#define FLUX_HIP_LINEAR_STATIC_MAX_OUTPUTS (FLUX_HIP_LINEAR_STATIC_BYTES / 8u) /* rows * N up to which K slices are considered */
int flux_hip_linear_static(int epilogue, int nparts, const flux_hip_linear_part *parts,
                           int N, int K, int lda, int ldw, int ldc, int w_row0, int w_row1);

/*
 * flux_hip_linear with FLUX_HIP_EPI_RESID, with the AdaLN that follows every residual projection
 * (apply_adaln, flux_transformer.c:979-1048, called at :1845, :1919, :3030) folded into it when the
 * projection runs as K slices (few rows, long K): the pass that sums the slices and updates x then
 * also writes (1 + scale) * LayerNorm(x) + shift as bf16 [M, N] (row stride N) per part, and
 * *fused = 1. Otherwise (*fused = 0) only the projection has run and the caller normalises with
 * flux_hip_adaln_norm. norm = NULL: plain projection. N <= 4096.
 * With shift = NULL in every part the norm is the text encoder's RMS norm instead (qwen3_rms_norm,
 * flux_qwen3.c:177-197, which follows both residual projections of a layer): x / sqrt(mean(x^2) +
 * eps) * scale, scale being that norm's weight; *fused = 0 then leaves it to flux_hip_rms_norm.
 */
typedef struct {
    void *out_bf16;       /* bf16 [M, N] */
    const float *shift;   /* f32 [N], or NULL for the RMS form */
    const float *scale;   /* f32 [N] */
} flux_hip_adaln_part;
int flux_hip_linear_resid_adaln(int nparts, const flux_hip_linear_part *parts, int N, int K, int lda, int ldw, int ldc,
                                const flux_hip_adaln_part *norm, float eps, int *fused);

/*
 * 3x3 (taps = 9, padding 1, stride 1) or 1x1 (taps = 1) convolution with bias as one MFMA GEMM
 * over a channels-last image. Replaces flux_conv2d (flux_kernels.c:342-470; im2col + sgemm
 * there) for the VAE decoder's layers, with the residual add of resblock_forward /
 * attnblock_forward (flux_vae.c:218, 311) in the fp32 epilogue.
 *   in   bf16 [rows, cin]: the image including a one-pixel zero border, rows = (H+2) * (W+2)
 *        positions in row-major order, wp = W+2. With 9 taps the kernel reads up to wp+1 rows
 *        before `in` and after its end: the allocation must extend that far (contents there
 *        only reach border outputs, which are written as zeros).
 *   w    bf16 [cout, taps * cin]; with 9 taps K runs over [cin/64 chunks][9 taps][64 channels]:
 *        w[o][((c / 64) * 9 + ky*3+kx) * 64 + c % 64] (the nine taps of a channel chunk are
 *        consecutive K steps, so that neighbouring rows are fetched while they are still cached)
 *   bias f32 [cout]; res f32 [rows, cout] or NULL (may be `out` itself); out [rows, cout]
 * Border positions of `out` are written as zeros, so it can feed the next convolution. wp = 0
 * (1x1 only) treats every row as interior. cin, cout: multiples of 64.
 */
int flux_hip_conv(int epilogue, const void *in, const void *w, const float *bias, const float *res,
                  void *out, int rows, int wp, int cin, int cout, int taps);
/* The same; when stats is given, the epilogue also leaves there the sums the following group norm
 * needs (sum and sum of squares of what it writes, per half row-tile and 4-channel quad:
 * [*stats_rows][cout/4][2] floats, at most rows/32 + 2 rows), which saves that norm its pass over
 * the image (flux_hip_group_norm_stats). */
int flux_hip_conv_stats(int epilogue, const void *in, const void *w, const float *bias, const float *res, void *out, int rows,
                        int wp, int cin, int cout, int taps, float *stats, int *stats_rows);

/*
 * out = (1 + scale) * LayerNorm(x) + shift per row, x f32 [rows, hidden], out bf16.
 * Rows [0, split) use mod0, the rest mod1; each mod points at shift[hidden] and scale[hidden]
 * through explicit pointers. Replaces apply_adaln (flux_transformer.c:979-1048) /
 * flux_gpu_adaln_norm_bf16 (flux_metal.h:384).
 */
int flux_hip_adaln_norm(void *out_bf16, int ldo, const float *x, int rows, int hidden, int split,
                        const float *shift0, const float *scale0,
                        const float *shift1, const float *scale1, float eps);

/*
 * Prepares Q and K of one attention call in the fused qkv buffer (bf16 [rows, ld] with Q at column
 * q_col and K at column k_col): per-head RMSNorm * weight, then RoPE. K is written to k_out
 * [rows, heads*128]; Q is written back in place, already multiplied by 1/sqrt(128) and log2(e) (the
 * attention kernel works on base-2 logits). Rows [0, split) use q_w0 / k_w0, the rest q_w1 / k_w1.
 * Replaces apply_qk_norm (flux_transformer.c:1052-1106) and apply_rope_2d
 * (flux_transformer.c:719-741). The reference's head transposes (flux_transformer.c:1117-1138)
 * have no counterpart: the attention kernel reads V where the projection wrote it and transposes
 * tiles of it on the way into the matrix unit.
 */
int flux_hip_qk_prepare(void *k_out, void *qkv, int ld, int q_col, int k_col, int rows, int heads, int split,
                        const float *q_w0, const float *q_w1, const float *k_w0, const float *k_w1,
                        const float *rope_cos, const float *rope_sin, float eps);

/*
 * Multi-head attention, no mask: out = softmax(q k^T) v per head with base-2 exponentials, online
 * softmax, scores never stored. q (prepared in place by flux_hip_qk_prepare) and v are read from
 * the qkv buffer (row strides ldq and ldv, the pointers already at their first column); k
 * [seq_k, heads*128] comes from flux_hip_qk_prepare. head_dim is 128. The queries may be a row
 * range of the sequence (q and out at its first row). (seq_k + 64) * ldv * 2 must stay below 2^32.
 * Replaces joint_attention / mha_forward (flux_transformer.c:1249-1460), flux_flash_attention
 * (flux_kernels.c:877) and flux_softmax (flux_kernels.c:596).
 */
int flux_hip_attention(void *out_bf16, int ldo, const void *q, int ldq, const void *k, const void *v, int ldv,
                       int seq_q, int seq_k, int heads);
/* The same for nseq independent sequences (arrays of nseq pointers and lengths; leading dimensions and heads in
 * common): sequences whose query blocks have the same lengths share a launch, two at a time. For the two forwards of
 * a classifier-free-guidance step (flux_sample.c:485-493), which attend separately. */
int flux_hip_attention_batch(int nseq, void *const *out_bf16, int ldo, const void *const *q, int ldq, const void *const *k,
                             const void *const *v, int ldv, const int *seq_q, const int *seq_k, int heads);

/* y[m, n] = sum_k f(x[m, k]) * W[n, k], x f32 [M, K] (M small), W bf16, y f32; f = SiLU when
 * silu_input. The modulation and time-embedding projections (flux_transformer.c:956-969,
 * 3226-3234, 3016-3024, 3523-3530). */
int flux_hip_gemv(float *y, const float *x, const void *W_bf16, int M, int N, int K, int silu_input);

/* Layout/precision edges: NCHW f32 latent [C, n] -> token-major bf16 [n, C]
 * (flux_transformer.c:3156-3161), and f32 -> bf16 (flux_shaders.metal:1430). */
int flux_hip_latent_to_tokens(void *tok_bf16, const float *latent, int channels, int n);
int flux_hip_f32_to_bf16(void *out_bf16, const float *in, size_t n);

/* z += dt * v   (flux_axpy, flux_kernels.c:126; flux_sample.c:248) */
int flux_hip_euler_update(float *z, const float *v, float dt, size_t n);
/* z += dt * (vu + g * (vc - vu))   (flux_sample.c:496-499) */
int flux_hip_cfg_euler_update(float *z, const float *v_uncond, const float *v_cond, float guidance, float dt, size_t n);
/* Heun: out = z + dt * v (predictor, flux_sample.c:780-782); z += dt/2 * (v1 + v2) (corrector, :789-792) */
int flux_hip_euler_predict(float *out, const float *z, const float *v, float dt, size_t n);
int flux_hip_heun_update(float *z, const float *v1, const float *v2, float dt, size_t n);

/* -------------------------------------------------------------------- model */

typedef struct flux_transformer flux_transformer_t;

typedef struct {
    int hidden, heads, head_dim, mlp, n_double, n_single, text_dim, channels;
    int axis_dim, sincos_dim;
    float rope_theta;
} flux_hip_config;

/* FLUX.2-klein-4B sizes (flux.h:33-41, flux_transformer.c:4418-4434). */
void flux_hip_default_config(flux_hip_config *cfg);

/* Builds a model from bf16 tensors handed over by name (the safetensors keys read at
 * flux_transformer.c:4452-4602). All tensors must be set before the first forward. */
flux_transformer_t *flux_hip_transformer_new(const flux_hip_config *cfg);
int flux_hip_transformer_set_tensor(flux_transformer_t *tf, const char *name, const uint16_t *bf16, int64_t numel);
/* Opens a .safetensors file (bf16 tensors) and uploads it; 4B sizes unless cfg is given. */
flux_transformer_t *flux_hip_transformer_load_file(const char *path, const flux_hip_config *cfg);

/* Reference loader entry points (flux_transformer.c:4411, 4659; called at flux.c:300-326).
 * `sf` is the reference's safetensors_file_t (flux_safetensors.h:41-49). Both upload the bf16
 * tensors once; the mmap variant takes ownership of sf and closes it in flux_transformer_free,
 * as the reference does (flux_transformer.c:4305-4309). */
struct safetensors_file;
flux_transformer_t *flux_transformer_load_safetensors(void *sf);
flux_transformer_t *flux_transformer_load_safetensors_mmap(void *sf);
/* The reference's loader for its own binary weight format (flux_transformer.c:4059, declared at flux.c:45 and
 * called from nowhere in its pipeline). Exported so that every flux_transformer_load* name of the reference
 * resolves; the format is not read here: returns NULL and sets the error text. `f` is a FILE*. */
flux_transformer_t *flux_transformer_load(void *f);
void flux_transformer_free(flux_transformer_t *tf);

typedef struct {
    const float *latent; /* [channels, h, w] */
    int h, w;
    int t_offset;        /* RoPE T coordinate: 10, 20, ... */
} flux_ref_t;

/* One velocity prediction; inputs on the host, result malloc'd [channels, h*w], caller frees.
 * Same contracts as flux_transformer.c:3115, 3605, 3815. */
float *flux_transformer_forward(flux_transformer_t *tf, const float *img_latent, int img_h, int img_w,
                                const float *txt_emb, int txt_seq, float timestep);
float *flux_transformer_forward_with_refs(flux_transformer_t *tf, const float *img_latent, int img_h, int img_w,
                                          const float *ref_latent, int ref_h, int ref_w, int t_offset,
                                          const float *txt_emb, int txt_seq, float timestep);
float *flux_transformer_forward_with_multi_refs(flux_transformer_t *tf, const float *img_latent, int img_h, int img_w,
                                                const flux_ref_t *refs, int num_refs,
                                                const float *txt_emb, int txt_seq, float timestep);

/* Samplers with the reference's signatures (flux_sample.c:212, 303, 381, 457, 534, 615). The
 * whole loop runs on the device: inputs are uploaded once, the latent is read back once. */
float *flux_sample_euler(void *transformer, void *text_encoder, float *z, int batch, int channels, int h, int w,
                         const float *text_emb, int text_seq, const float *schedule, int num_steps,
                         void (*progress_callback)(int step, int total));
float *flux_sample_euler_with_refs(void *transformer, void *text_encoder, float *z, int batch, int channels, int h, int w,
                                   const float *ref_latent, int ref_h, int ref_w, int t_offset,
                                   const float *text_emb, int text_seq, const float *schedule, int num_steps,
                                   void (*progress_callback)(int step, int total));
float *flux_sample_euler_with_multi_refs(void *transformer, void *text_encoder, float *z, int batch, int channels, int h, int w,
                                         const flux_ref_t *refs, int num_refs,
                                         const float *text_emb, int text_seq, const float *schedule, int num_steps,
                                         void (*progress_callback)(int step, int total));
float *flux_sample_euler_cfg(void *transformer, void *text_encoder, float *z, int batch, int channels, int h, int w,
                             const float *text_emb_cond, int text_seq_cond,
                             const float *text_emb_uncond, int text_seq_uncond, float guidance_scale,
                             const float *schedule, int num_steps, void (*progress_callback)(int step, int total));
float *flux_sample_euler_cfg_with_refs(void *transformer, void *text_encoder, float *z, int batch, int channels, int h, int w,
                                       const float *ref_latent, int ref_h, int ref_w, int t_offset,
                                       const float *text_emb_cond, int text_seq_cond,
                                       const float *text_emb_uncond, int text_seq_uncond, float guidance_scale,
                                       const float *schedule, int num_steps, void (*progress_callback)(int step, int total));
float *flux_sample_euler_cfg_with_multi_refs(void *transformer, void *text_encoder, float *z, int batch, int channels, int h, int w,
                                             const flux_ref_t *refs, int num_refs,
                                             const float *text_emb_cond, int text_seq_cond,
                                             const float *text_emb_uncond, int text_seq_uncond, float guidance_scale,
                                             const float *schedule, int num_steps,
                                             void (*progress_callback)(int step, int total));

/* Second-order and noise-injecting samplers (flux_sample.c:760, 697): text-only conditioning,
 * no reference images, as in the reference. Heun runs 2 * num_steps - 1 forwards. The noise of
 * the ancestral sampler comes from flux_randn in its current state. */
float *flux_sample_heun(void *transformer, float *z, int batch, int channels, int h, int w,
                        const float *text_emb, int text_seq, const float *schedule, int num_steps,
                        void (*progress_callback)(int step, int total));
float *flux_sample_euler_ancestral(void *transformer, float *z, int batch, int channels, int h, int w,
                                   const float *text_emb, int text_seq, const float *schedule, int num_steps,
                                   float eta, void (*progress_callback)(int step, int total));

/* Schedules (flux_sample.c:49, 62, 75, 96, 145); malloc'd [num_steps + 1], caller frees. */
float *flux_linear_schedule(int num_steps);
float *flux_power_schedule(int num_steps, float alpha);
float *flux_sigmoid_schedule(int num_steps, float shift);
float *flux_resolution_schedule(int num_steps, int height, int width);
float *flux_official_schedule(int num_steps, int image_seq_len);

/* Host generator of the reference (flux_kernels.c:45-102: xoshiro256** seeded through
 * SplitMix64, Box-Muller), and the initial latent noise drawn from it (flux_sample.c:837-877):
 * malloc'd [batch, channels, h, w], caller frees; seed < 0 continues the current stream. */
void flux_rng_seed(uint64_t seed);
void flux_randn(float *out, int n);
float *flux_init_noise(int batch, int channels, int h, int w, int64_t seed);

/* Noise + linear schedule + Euler sampler for a height x width image (flux_sample.c:891-919);
 * the first argument is the transformer. */
float *flux_generate_latent(void *ctx_ptr, const float *text_emb, int text_seq, int height, int width, int num_steps,
                            int64_t seed, void (*progress_callback)(int step, int total));
extern void (*flux_progress_callback)(int, int);
void flux_set_progress_callback(void (*callback)(int, int));

/* Same sampling loops, additionally copying every forward's velocity (in call order,
 * [forwards, channels*h*w] f32) to v_trace when it is not NULL. For parity tests. */
float *flux_hip_sample_traced(void *transformer, const float *z, int channels, int h, int w,
                              const flux_ref_t *refs, int num_refs,
                              const float *text_emb_cond, int text_seq_cond,
                              const float *text_emb_uncond, int text_seq_uncond, float guidance_scale,
                              const float *schedule, int num_steps, float *v_trace);
/* Heun: v_trace holds v1, v2 of every step in call order (2 * num_steps - 1 velocities). */
float *flux_hip_sample_heun_traced(void *transformer, const float *z, int channels, int h, int w,
                                   const float *text_emb, int text_seq, const float *schedule, int num_steps,
                                   float *v_trace, void (*progress)(int, int));
float *flux_hip_sample_ancestral_traced(void *transformer, const float *z, int channels, int h, int w,
                                        const float *text_emb, int text_seq, const float *schedule, int num_steps,
                                        float eta, float *v_trace, void (*progress)(int, int));

/* ---------------------------------------------------------------- VAE decoder
 * The step after the sampling loop: final latent -> RGB image (flux_vae_decode,
 * flux_vae.c:690-837; the reference's device path is vae_decode_gpu, flux_vae.c:505). Images on
 * the device are channels-last with a one-pixel zero border, positions in row-major order over
 * the (H+2) x (W+2) grid: hp = H+2, wp = W+2 below. */

/*
 * GroupNorm(32 groups, statistics over the whole image) with optional swish, x f32 or bf16
 * [hp*wp, C] -> out bf16, zeros on the border. raw (optional) receives x itself as bf16.
 * scratch: flux_hip_group_norm_scratch_floats(hp, wp) floats. C is 128, 256 or 512;
 * hp * wp < 2^22.
 * Replaces flux_group_norm (flux_kernels.c:511-553) + flux_silu (flux_kernels.c:581).
 */
int flux_hip_group_norm(void *out_bf16, void *raw_bf16, const void *x, int x_is_bf16, const float *gamma, const float *beta,
                        float *scratch, int hp, int wp, int C, float eps, int swish);
/* conv_stats / conv_stats_rows: what flux_hip_conv_stats left behind for this x (NULL: sums are computed here) */
int flux_hip_group_norm_stats(void *out_bf16, void *raw_bf16, const void *x, int x_is_bf16, const float *gamma, const float *beta,
                              float *scratch, int hp, int wp, int C, float eps, int swish, const float *conv_stats, int conv_stats_rows);
size_t flux_hip_group_norm_scratch_floats(int hp, int wp);
/* nearest-neighbour 2x: x f32 [hp*wp, C] -> out bf16 [(2H+2)*(2W+2), C] (flux_upsample_nearest, flux_kernels.c:1017) */
int flux_hip_upsample2x(void *out_bf16, const float *x, int hp, int wp, int C);
/* P bf16 [rows, ld] = softmax over each row of (S * scale + key_bias), S f32 [rows, ld], key_bias f32 [ld]
 * (0 or -inf); flux_softmax, flux_kernels.c:596, with the scale of flux_vae.c:247 */
int flux_hip_softmax_rows(void *p_bf16, const float *s, const float *key_bias, int rows, int ld, float scale);
/* vt bf16 [cols, ld] = v^T for v bf16 [rows, ldv] (first `cols` columns), zero-filled for columns rows..ld-1 */
int flux_hip_transpose_bf16(void *vt, int ld, const void *v, int ldv, int rows, int cols);

typedef struct flux_hip_vae flux_hip_vae;
/* VAE weights from a .safetensors file (tensor names as flux_vae_load_safetensors reads them,
 * flux_vae.c:1232-1330), or from the reference's parsed-file handle (safetensors_file_t *). The
 * decoder's tensors must all be there; a file without the encoder's loads, and encoding with it
 * fails. NULL on failure. */
flux_hip_vae *flux_hip_vae_load_file(const char *path);
flux_hip_vae *flux_hip_vae_load_safetensors(void *safetensors_file);
/* Piecewise construction: new, then one set_tensor per tensor (dtype 0 = f32, 1 = f16, 2 = bf16). */
flux_hip_vae *flux_hip_vae_new(void);
int flux_hip_vae_set_tensor(flux_hip_vae *v, const char *name, int dtype, const void *data, int64_t numel);
void flux_hip_vae_free(flux_hip_vae *v);
/* latent f32 [128, h, w] (host) -> rgb u8 [16h, 16w, 3] and/or rgb_f32 [3, 16h, 16w] (decoder output
 * before the conversion to 8 bits); either may be NULL. h, w <= 112. 1 = ok, 0 = failed. */
int flux_hip_vae_decode(flux_hip_vae *v, const float *latent, int h, int w, uint8_t *rgb, float *rgb_f32);
/* image f32 [3, H, W] in [-1, 1] (host; H, W multiples of 16, at most 1792) -> normalised latent f32
 * [128, H/16, W/16] (host): flux_vae_encode, flux_vae.c:320-443, for one image. A residual block
 * that widens computes skip + conv2(...) as written; the reference's plain-C build overwrites part
 * of that convolution's input while it runs (flux_vae.c:203 with flux_kernels.c:441-470), its
 * BLAS path in one tile does not. 1 = ok, 0 = failed. */
int flux_hip_vae_encode(flux_hip_vae *v, const float *img, int H, int W, float *latent);
/* Encoder pieces: img f32 [3, H, W] (device) -> bf16 [(H+2)*(W+2), 64], the 27 values under every
 * 3x3 window first (conv_in as a GEMM with K = 64, flux_vae.c:336); x f32 [hp*wp, C] -> bf16
 * [(H/2+2)*(W/2+2), 9*C], the nine taps of the stride-2 convolution side by side in flux_hip_conv's
 * K order (flux_vae.c:363-377); quant-convolution output f32 [(2h+2)*(2w+2), ldx] -> latent f32 [128, h, w]
 * (mean channels, patchify, latent normalisation, flux_vae.c:411-437). */
int flux_hip_vae_image_in(void *out_bf16, const float *img, int H, int W);
int flux_hip_downsample_gather(void *out_bf16, const float *x, int hp, int wp, int C);
int flux_hip_vae_latent_out(float *latent, const float *x, int ldx, const float *bn_mean, const float *bn_var, int h, int w, float eps);
/* When set, called after each of the decoder's 15 / the encoder's 11 blocks has been queued (role of
 * flux_vae_progress_callback, flux_kernels.h:292-293). */
extern void (*flux_hip_vae_progress)(int block, int total);

/* The reference's own VAE entry points (flux.c:36-43) over the device VAE; see flux_vae_dropin.c
 * for how an application links them (and how it keeps its CPU encoder if it wants to). The
 * handles are flux_vae_t * / flux_image * / safetensors_file_t * in the reference's headers. */
void *flux_vae_load_safetensors(void *safetensors_file);
void *flux_vae_decode(void *vae, const float *latent, int batch, int latent_h, int latent_w);
float *flux_vae_encode(void *vae, const float *img, int batch, int H, int W, int *out_h, int *out_w);
void flux_vae_free(void *vae);

/* ---------------------------------------------------------------- Qwen3 text encoder
 * The step before the sampling loop: token ids -> the transformer's text input
 * (qwen3_forward, flux_qwen3.c:1041-1156). */

/* out bf16 [rows, hidden] = x / sqrt(mean(x^2) + eps) * w per row, x f32 (qwen3_rms_norm, flux_qwen3.c:177-197) */
int flux_hip_rms_norm(void *out_bf16, const float *x, const float *w, int rows, int hidden, float eps);
/*
 * Causal grouped-query attention with a padding mask, head_dim 128, seq <= 512
 * (qwen3_attention_forward, flux_qwen3.c:352-437, and flux_metal_causal_attention there).
 * qkv bf16 [seq, (heads + 2 kv_heads) * 128]: q heads, then k heads (both already normed and
 * rotated); vt bf16 [kv_heads * 128, ldv]: v transposed, ldv >= seq rounded up to 32, columns
 * beyond seq finite; mask int [seq] on the device or NULL. out bf16 [seq, heads * 128].
 * A masked or future key scores -1e9 before the softmax over all seq columns, as in the reference.
 */
int flux_hip_causal_attention(void *out_bf16, const void *qkv_bf16, const void *vt_bf16, int ldv, const int *mask_dev, int seq,
                              int heads, int kv_heads);

typedef struct {
    int hidden, intermediate, heads, kv_heads, head_dim, layers, vocab;
    int out_layer[3];          /* hidden states after these layers (0-based) form the output, side by side */
    float rope_theta, eps;
} flux_hip_qwen3_config;
void flux_hip_qwen3_default_config(flux_hip_qwen3_config *c);   /* flux_qwen3.h:22-39 */

typedef struct flux_hip_qwen3 flux_hip_qwen3;
/* From a directory with model-00001-of-00002.safetensors + model-00002-of-00002.safetensors
 * (flux_qwen3.c:1341-1343) or one model.safetensors; sizes are read from the tensors. */
flux_hip_qwen3 *flux_hip_qwen3_load_dir(const char *model_dir);
/* Piecewise: new (NULL = the reference's sizes), one set_tensor per tensor (dtype 0 f32, 1 f16, 2 bf16). */
flux_hip_qwen3 *flux_hip_qwen3_new(const flux_hip_qwen3_config *cfg);
int flux_hip_qwen3_set_tensor(flux_hip_qwen3 *q, const char *name, int dtype, const void *data, int64_t numel);
void flux_hip_qwen3_free(flux_hip_qwen3 *q);
/* ids / mask: host int [seq_len], mask may be NULL; returns a malloc'd host array [seq_len, 3 * hidden]
 * (caller frees) or NULL. seq_len <= 512. */
float *flux_hip_qwen3_forward(flux_hip_qwen3 *q, const int *input_ids, const int *attention_mask, int seq_len);
/* When set, called after each layer has been queued (role of flux_text_progress_callback). */
extern void (*flux_hip_qwen3_progress)(int layer, int total);

/* qwen3_encoder_free keeps the encoder's weights on the device and the next qwen3_encoder_load of the
 * same directory takes them over instead of uploading 6 GB again (the reference frees its encoder
 * after every prompt, flux.c:285-295; its weights are a memory map). keep_resident(0) switches that
 * off and frees what is kept, drop_resident() frees it once; resident_hits counts the loads served
 * from the kept weights. The files are not checked for changes in between. */
void flux_hip_qwen3_keep_resident(int on);
void flux_hip_qwen3_drop_resident(void);
extern int flux_hip_qwen3_resident_hits;

/* The reference's own entry points (flux_qwen3.h:93-141) over the device encoder: an application
 * keeps flux_qwen3_tokenizer.c and leaves flux_qwen3.c out of its link. Declared here only when the
 * reference's header has not been included (its declarations use its own opaque types). */
#ifndef FLUX_QWEN3_H
void *qwen3_model_load(const char *model_dir);
void *qwen3_model_load_mmap(const char *model_dir);
void qwen3_model_free(void *model);
float *qwen3_forward(void *model, const int *input_ids, const int *attention_mask, int seq_len);
void *qwen3_encoder_load(const char *model_dir, int use_mmap);
void qwen3_encoder_free(void *enc);
float *qwen3_encode_text(void *enc, const char *prompt);
#endif

/*
 * The sampling loop in pieces, for callers that drive or time the steps themselves. begin()
 * uploads latent, text and reference tokens and computes every step's modulation vectors;
 * step() only queues kernels (no host round trip unless v_trace is given, which receives that
 * step's velocity or, under CFG, the unconditional then the conditional one); read_latent()
 * waits and copies the current latent out. The samplers above are built from these.
 */
/* A CFG step's unconditional and conditional forwards run as one batch of two sequences (each weight
 * matrix streamed once, twice the rows per GEMM); flux_hip_set_batched_cfg(0) in flux_hip_debug.h
 * switches back to two separate forwards, the reference's order (flux_sample.c:485-493). */
typedef struct flux_hip_session flux_hip_session;
flux_hip_session *flux_hip_session_begin(void *transformer, const float *z, int channels, int h, int w,
                                         const flux_ref_t *refs, int num_refs,
                                         const float *text_emb_cond, int text_seq_cond,
                                         const float *text_emb_uncond, int text_seq_uncond, float guidance_scale,
                                         const float *schedule, int num_steps);
int flux_hip_session_step(flux_hip_session *s, int step, float *v_trace);
int flux_hip_session_read_latent(flux_hip_session *s, float *z_out);
void flux_hip_session_free(flux_hip_session *s);

/* Per-stage device time of the last sampling call in milliseconds (role of the
 * flux_timing_transformer_* counters, flux_sample.c:29-39). */
extern double flux_timing_transformer_total;
extern double flux_timing_transformer_double;
extern double flux_timing_transformer_single;
extern double flux_timing_transformer_final;
void flux_reset_timing(void);

/* Progress hooks with the reference's names (flux_kernels.h:245-256). They fire on the host
 * thread when the corresponding work has been queued, not when it has finished. */
typedef enum { FLUX_SUBSTEP_DOUBLE_BLOCK, FLUX_SUBSTEP_SINGLE_BLOCK, FLUX_SUBSTEP_FINAL_LAYER } flux_substep_type_t;
typedef void (*flux_substep_callback_t)(flux_substep_type_t type, int index, int total);
typedef void (*flux_step_callback_t)(int step, int total);
extern flux_substep_callback_t flux_substep_callback;
extern flux_step_callback_t flux_step_callback;
extern int flux_verbose;

#ifdef __cplusplus
}
#endif
#endif /* FLUX_HIP_H */
