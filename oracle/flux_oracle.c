/*
 * flux_oracle.c - CPU restatement (fp32) of the FLUX.2-klein denoising
 * transformer and its Euler samplers.
 *
 * THIS FILE IS TEST INFRASTRUCTURE. It is the checker that the HIP backend is
 * compared against; it is never part of the shipped code path. Only tests,
 * the smoke entry and the cpu_baseline leg of the benchmark may load it.
 *
 * Every function cites the file:line of antirez/flux2.c it restates. All
 * arithmetic is IEEE fp32; weights arrive as bf16 and are widened exactly
 * (bits << 16), as the reference loader does (flux_safetensors.c:303-308).
 * Unlike the reference, the architecture is a run-time parameter so that the
 * same code can be exercised on tiny models in seconds.
 *
 * Pinning status of each function (see tests/test_oracle_*.py):
 *   fo_timestep_embedding, fo_time_mlp, fo_rope_image, fo_rope_text,
 *   fo_apply_rope, fo_adaln, fo_qk_norm, fo_linear, fo_attention,
 *   fo_double_block, fo_single_block, fo_forward (0/1/2 references),
 *   fo_sample_euler, fo_sample_euler_cfg, fo_sample_heun, fo_sample_euler_ancestral,
 *   schedules (linear, power, sigmoid, resolution, official), fo_init_noise:
 *   pinned against golden vectors produced by the reference's own C code
 *   compiled from its sources (oracle/ref_probe.c -> oracle/_ref/), and
 *   against closed forms / brute force in tests/test_oracle_math.py.
 *
 * Build: see oracle/Makefile (gcc -O3 -march=native -fopenmp).
 */
#include <stdint.h>
#include <stdlib.h>
#include <string.h>
#include <stdio.h>
#include <math.h>
#include <dlfcn.h>
#ifdef _OPENMP
#include <omp.h>
#endif

/* ------------------------------------------------------------------------
 * Optional BLAS (resolved at run time with dlopen; the reference's fast CPU
 * build calls cblas_sgemm at flux_kernels.c:249 and flux_transformer.c:1308).
 * ------------------------------------------------------------------------ */
typedef void (*sgemm_fn)(int order, int ta, int tb, int M, int N, int K,
                         float alpha, const float *A, int lda,
                         const float *B, int ldb, float beta, float *C, int ldc);
static sgemm_fn g_sgemm = NULL;
static void *g_blas_handle = NULL;
static int g_blas_threads = 0;

/* Returns 1 if `symbol` was found in `path`. */
int fo_set_blas(const char *path, const char *symbol) {
    void *h = dlopen(path, RTLD_NOW | RTLD_LOCAL);
    if (!h) return 0;
    void *f = dlsym(h, symbol);
    if (!f) { dlclose(h); return 0; }
    g_blas_handle = h;
    g_sgemm = (sgemm_fn)f;
    int (*getn)(void) = (int (*)(void))dlsym(h, "scipy_openblas_get_num_threads");
    if (!getn) getn = (int (*)(void))dlsym(h, "openblas_get_num_threads");
    g_blas_threads = getn ? getn() : 0;
    return 1;
}

void fo_set_blas_threads(int n) {
    if (!g_blas_handle) return;
    void (*setn)(int) = (void (*)(int))dlsym(g_blas_handle, "scipy_openblas_set_num_threads");
    if (!setn) setn = (void (*)(int))dlsym(g_blas_handle, "openblas_set_num_threads");
    if (setn) { setn(n); g_blas_threads = n; }
}

int fo_has_blas(void) { return g_sgemm != NULL; }

/* Threads the GEMMs actually use (BLAS pool or OpenMP team). */
int fo_num_threads(void) {
    if (g_sgemm && g_blas_threads > 0) return g_blas_threads;
#ifdef _OPENMP
    return omp_get_max_threads();
#else
    return 1;
#endif
}

/* ------------------------------------------------------------------------
 * y[s,o] = sum_i x[s,i] * W[o,i]   (flux_kernels.c:210-282, no bias in model)
 * Strided variant so attention can address one head inside [seq, hidden].
 * ------------------------------------------------------------------------ */
static void gemm_nt(float *C, int ldc, const float *A, int lda,
                    const float *B, int ldb, int M, int N, int K, float alpha) {
    if (g_sgemm) {
        /* CblasRowMajor=101, NoTrans=111, Trans=112 */
        g_sgemm(101, 111, 112, M, N, K, alpha, A, lda, B, ldb, 0.0f, C, ldc);
        return;
    }
    /* Register-blocked dot products: 4 rows of A against 4 rows of B. */
    #pragma omp parallel for schedule(static) collapse(2)
    for (int n0 = 0; n0 < N; n0 += 4) {
        for (int m0 = 0; m0 < M; m0 += 4) {
            int nn = N - n0 < 4 ? N - n0 : 4;
            int mm = M - m0 < 4 ? M - m0 : 4;
            if (nn == 4 && mm == 4) {
                float acc[4][4] = {{0}};
                const float *a0 = A + (size_t)m0 * lda, *b0 = B + (size_t)n0 * ldb;
                for (int k = 0; k < K; k++) {
                    float av[4], bv[4];
                    for (int i = 0; i < 4; i++) av[i] = a0[(size_t)i * lda + k];
                    for (int j = 0; j < 4; j++) bv[j] = b0[(size_t)j * ldb + k];
                    for (int i = 0; i < 4; i++)
                        for (int j = 0; j < 4; j++) acc[i][j] += av[i] * bv[j];
                }
                for (int i = 0; i < 4; i++)
                    for (int j = 0; j < 4; j++)
                        C[(size_t)(m0 + i) * ldc + n0 + j] = alpha * acc[i][j];
            } else {
                for (int i = 0; i < mm; i++)
                    for (int j = 0; j < nn; j++) {
                        const float *a = A + (size_t)(m0 + i) * lda;
                        const float *b = B + (size_t)(n0 + j) * ldb;
                        float s = 0.0f;
                        for (int k = 0; k < K; k++) s += a[k] * b[k];
                        C[(size_t)(m0 + i) * ldc + n0 + j] = alpha * s;
                    }
            }
        }
    }
}

/* C[M,N] = A[M,K] * B[K,N]  (second attention product, flux_transformer.c:1317) */
static void gemm_nn(float *C, int ldc, const float *A, int lda,
                    const float *B, int ldb, int M, int N, int K) {
    if (g_sgemm) {
        g_sgemm(101, 111, 111, M, N, K, 1.0f, A, lda, B, ldb, 0.0f, C, ldc);
        return;
    }
    #pragma omp parallel for schedule(static)
    for (int m = 0; m < M; m++) {
        float *c = C + (size_t)m * ldc;
        for (int n = 0; n < N; n++) c[n] = 0.0f;
        for (int k = 0; k < K; k++) {
            float a = A[(size_t)m * lda + k];
            const float *b = B + (size_t)k * ldb;
            for (int n = 0; n < N; n++) c[n] += a * b[n];
        }
    }
}

void fo_linear(float *y, const float *x, const float *W, int seq, int in_dim, int out_dim) {
    gemm_nt(y, out_dim, x, in_dim, W, in_dim, seq, out_dim, in_dim, 1.0f);
}

/* x * sigmoid(x)   (flux_kernels.c:581-594) */
void fo_silu(float *x, int64_t n) {
    #pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < n; i++) { float v = x[i]; x[i] = v / (1.0f + expf(-v)); }
}

/* Row softmax with max subtraction   (flux_kernels.c:596-628) */
void fo_softmax(float *x, int rows, int cols) {
    #pragma omp parallel for schedule(static)
    for (int r = 0; r < rows; r++) {
        float *row = x + (size_t)r * cols;
        float mx = row[0];
        for (int c = 1; c < cols; c++) if (row[c] > mx) mx = row[c];
        float sum = 0.0f;
        for (int c = 0; c < cols; c++) { row[c] = expf(row[c] - mx); sum += row[c]; }
        float inv = 1.0f / sum;
        for (int c = 0; c < cols; c++) row[c] *= inv;
    }
}

/* ------------------------------------------------------------------------
 * Timestep embedding   (flux_transformer.c:940-951): [cos | sin] halves,
 * freq_i = exp(-ln(max_period) * i / half). Caller passes t already * 1000.
 * ------------------------------------------------------------------------ */
void fo_timestep_embedding(float *out, float t, int dim, float max_period) {
    int half = dim / 2;
    float lm = logf(max_period);
    for (int i = 0; i < half; i++) {
        float f = expf(-lm * (float)i / (float)half);
        float a = t * f;
        out[i] = cosf(a);
        out[i + half] = sinf(a);
    }
}

/* fc2(silu(fc1(e)))   (flux_transformer.c:956-969) */
void fo_time_mlp(float *out, const float *e, const float *fc1, const float *fc2,
                 int sincos_dim, int hidden) {
    float *tmp = (float *)malloc(sizeof(float) * hidden);
    fo_linear(tmp, e, fc1, 1, sincos_dim, hidden);
    fo_silu(tmp, hidden);
    fo_linear(out, tmp, fc2, 1, hidden, hidden);
    free(tmp);
}

/* ------------------------------------------------------------------------
 * RoPE tables, 4 axes (T,H,W,L) of axis_dim each; each frequency's cos/sin is
 * stored twice, on dims (2d, 2d+1).
 * Image tokens: T = t_offset, H = row, W = col, L = 0
 *   (flux_transformer.c:591-649 for t_offset = 0, 655-712 otherwise).
 * Text tokens: T = H = W = 0, L = token index (flux_transformer.c:747-779).
 * ------------------------------------------------------------------------ */
static void rope_axis(float *c, float *s, int pos, const float *freqs, int half_axis) {
    for (int d = 0; d < half_axis; d++) {
        float a = (float)pos * freqs[d];
        float cv = cosf(a), sv = sinf(a);
        c[2 * d] = cv; c[2 * d + 1] = cv;
        s[2 * d] = sv; s[2 * d + 1] = sv;
    }
}

static void rope_base_freqs(float *freqs, int axis_dim, float theta) {
    for (int d = 0; d < axis_dim / 2; d++)
        freqs[d] = 1.0f / powf(theta, (float)(2 * d) / (float)axis_dim);
}

void fo_rope_image(float *cos_out, float *sin_out, int ph, int pw, int axis_dim,
                   float theta, int t_offset) {
    float freqs[64];
    int half = axis_dim / 2;
    rope_base_freqs(freqs, axis_dim, theta);
    for (int y = 0; y < ph; y++)
        for (int x = 0; x < pw; x++) {
            size_t o = (size_t)(y * pw + x) * axis_dim * 4;
            rope_axis(cos_out + o, sin_out + o, t_offset, freqs, half);
            rope_axis(cos_out + o + axis_dim, sin_out + o + axis_dim, y, freqs, half);
            rope_axis(cos_out + o + 2 * axis_dim, sin_out + o + 2 * axis_dim, x, freqs, half);
            rope_axis(cos_out + o + 3 * axis_dim, sin_out + o + 3 * axis_dim, 0, freqs, half);
        }
}

void fo_rope_text(float *cos_out, float *sin_out, int seq, int axis_dim, float theta) {
    float freqs[64];
    int half = axis_dim / 2;
    rope_base_freqs(freqs, axis_dim, theta);
    for (int s = 0; s < seq; s++) {
        size_t o = (size_t)s * axis_dim * 4;
        for (int a = 0; a < 3; a++)
            rope_axis(cos_out + o + a * axis_dim, sin_out + o + a * axis_dim, 0, freqs, half);
        rope_axis(cos_out + o + 3 * axis_dim, sin_out + o + 3 * axis_dim, s, freqs, half);
    }
}

/* Rotate consecutive pairs (d, d+1); one table row per token, shared by all
 * heads   (flux_transformer.c:719-741). */
void fo_apply_rope(float *x, const float *cos_t, const float *sin_t,
                   int seq, int heads, int head_dim) {
    #pragma omp parallel for schedule(static)
    for (int s = 0; s < seq; s++) {
        const float *c = cos_t + (size_t)s * head_dim, *sn = sin_t + (size_t)s * head_dim;
        for (int h = 0; h < heads; h++) {
            float *v = x + ((size_t)s * heads + h) * head_dim;
            for (int d = 0; d < head_dim; d += 2) {
                float x0 = v[d], x1 = v[d + 1];
                v[d] = x0 * c[d] - x1 * sn[d];
                v[d + 1] = x1 * c[d] + x0 * sn[d];
            }
        }
    }
}

/* LayerNorm without affine, biased two-pass variance, then
 * (1 + scale) * xhat + shift   (flux_transformer.c:1021-1046). */
void fo_adaln(float *out, const float *x, const float *shift, const float *scale,
              int seq, int hidden, float eps) {
    #pragma omp parallel for schedule(static)
    for (int s = 0; s < seq; s++) {
        const float *xr = x + (size_t)s * hidden;
        float *o = out + (size_t)s * hidden;
        float sum = 0.0f;
        for (int i = 0; i < hidden; i++) sum += xr[i];
        float mean = sum / hidden;
        float vs = 0.0f;
        for (int i = 0; i < hidden; i++) { float d = xr[i] - mean; vs += d * d; }
        float inv = 1.0f / sqrtf(vs / hidden + eps);
        for (int i = 0; i < hidden; i++)
            o[i] = (1.0f + scale[i]) * ((xr[i] - mean) * inv) + shift[i];
    }
}

/* Per (token, head) RMSNorm times a [head_dim] weight, separately for q and k
 * (flux_transformer.c:1080-1104). */
static void rms_heads(float *x, const float *w, int seq, int heads, int head_dim, float eps) {
    #pragma omp parallel for schedule(static)
    for (int s = 0; s < seq; s++)
        for (int h = 0; h < heads; h++) {
            float *v = x + ((size_t)s * heads + h) * head_dim;
            float ss = 0.0f;
            for (int d = 0; d < head_dim; d++) ss += v[d] * v[d];
            float inv = 1.0f / sqrtf(ss / head_dim + eps);
            for (int d = 0; d < head_dim; d++) v[d] = v[d] * inv * w[d];
        }
}

void fo_qk_norm(float *q, float *k, const float *qw, const float *kw,
                int seq, int heads, int head_dim, float eps) {
    rms_heads(q, qw, seq, heads, head_dim, eps);
    rms_heads(k, kw, seq, heads, head_dim, eps);
}

/* out[s,i] += gate[i] * proj[s,i]   (flux_transformer.c:90-97) */
void fo_gated_add(float *out, const float *gate, const float *proj, int seq, int hidden) {
    #pragma omp parallel for schedule(static)
    for (int s = 0; s < seq; s++)
        for (int i = 0; i < hidden; i++)
            out[(size_t)s * hidden + i] += gate[i] * proj[(size_t)s * hidden + i];
}

/* ------------------------------------------------------------------------
 * Multi-head attention on [seq, heads*head_dim] tensors, no mask,
 * softmax(scale * q k^T) v per head. seq_q may differ from seq_k.
 * Restates the materialised-score path (flux_transformer.c:1300-1321 and
 * 1416-1447); the strides replace the reference's head transposes.
 * ------------------------------------------------------------------------ */
void fo_attention(float *out, const float *q, const float *k, const float *v,
                  int seq_q, int seq_k, int heads, int head_dim) {
    int hidden = heads * head_dim;
    float scale = 1.0f / sqrtf((float)head_dim);
    float *scores = (float *)malloc(sizeof(float) * (size_t)seq_q * seq_k);
    for (int h = 0; h < heads; h++) {
        gemm_nt(scores, seq_k, q + h * head_dim, hidden, k + h * head_dim, hidden,
                seq_q, seq_k, head_dim, scale);
        fo_softmax(scores, seq_q, seq_k);
        gemm_nn(out + h * head_dim, hidden, scores, seq_k, v + h * head_dim, hidden,
                seq_q, head_dim, seq_k);
    }
    free(scores);
}

/* ------------------------------------------------------------------------
 * Model container
 * ------------------------------------------------------------------------ */
typedef struct {
    int hidden, heads, head_dim, mlp, n_double, n_single, text_dim, channels;
    int axis_dim, sincos_dim;
    float rope_theta;
} fo_config;

typedef struct {
    float *q, *k, *v, *norm_q, *norm_k, *proj, *ff_in, *ff_out;
} fo_stream;

typedef struct { fo_stream img, txt; } fo_double;
typedef struct { float *norm_q, *norm_k, *qkv_mlp, *out; } fo_single;

typedef struct {
    fo_config c;
    float *img_in, *txt_in, *t_fc1, *t_fc2;
    float *mod_img, *mod_txt, *mod_single, *norm_out, *proj_out;
    fo_double *dbl;
    fo_single *sgl;
} fo_model;

void fo_default_config(fo_config *c) {
    /* flux.h:33-41 and flux_transformer.c:4418-4434 */
    c->hidden = 3072; c->heads = 24; c->head_dim = 128; c->mlp = 9216;
    c->n_double = 5; c->n_single = 20; c->text_dim = 7680; c->channels = 128;
    c->axis_dim = 32; c->sincos_dim = 256; c->rope_theta = 2000.0f;
}

fo_model *fo_model_new(const fo_config *c) {
    fo_model *m = (fo_model *)calloc(1, sizeof(fo_model));
    m->c = *c;
    m->dbl = (fo_double *)calloc(c->n_double > 0 ? c->n_double : 1, sizeof(fo_double));
    m->sgl = (fo_single *)calloc(c->n_single > 0 ? c->n_single : 1, sizeof(fo_single));
    return m;
}

static void free_stream(fo_stream *s) {
    free(s->q); free(s->k); free(s->v); free(s->norm_q); free(s->norm_k);
    free(s->proj); free(s->ff_in); free(s->ff_out);
}

void fo_model_free(fo_model *m) {
    if (!m) return;
    free(m->img_in); free(m->txt_in); free(m->t_fc1); free(m->t_fc2);
    free(m->mod_img); free(m->mod_txt); free(m->mod_single);
    free(m->norm_out); free(m->proj_out);
    for (int i = 0; i < m->c.n_double; i++) { free_stream(&m->dbl[i].img); free_stream(&m->dbl[i].txt); }
    for (int i = 0; i < m->c.n_single; i++) {
        free(m->sgl[i].norm_q); free(m->sgl[i].norm_k); free(m->sgl[i].qkv_mlp); free(m->sgl[i].out);
    }
    free(m->dbl); free(m->sgl); free(m);
}

/* Tensor names are the safetensors keys the reference loader asks for
 * (flux_transformer.c:4452-4602). Returns the slot and expected element count. */
static float **slot_for(fo_model *m, const char *name, int64_t *expect) {
    const fo_config *c = &m->c;
    int64_t H = c->hidden, M = c->mlp;
    int i; char rest[200];
    if (!strcmp(name, "x_embedder.weight")) { *expect = H * c->channels; return &m->img_in; }
    if (!strcmp(name, "context_embedder.weight")) { *expect = H * c->text_dim; return &m->txt_in; }
    if (!strcmp(name, "time_guidance_embed.timestep_embedder.linear_1.weight")) { *expect = H * c->sincos_dim; return &m->t_fc1; }
    if (!strcmp(name, "time_guidance_embed.timestep_embedder.linear_2.weight")) { *expect = H * H; return &m->t_fc2; }
    if (!strcmp(name, "double_stream_modulation_img.linear.weight")) { *expect = 6 * H * H; return &m->mod_img; }
    if (!strcmp(name, "double_stream_modulation_txt.linear.weight")) { *expect = 6 * H * H; return &m->mod_txt; }
    if (!strcmp(name, "single_stream_modulation.linear.weight")) { *expect = 3 * H * H; return &m->mod_single; }
    if (!strcmp(name, "norm_out.linear.weight")) { *expect = 2 * H * H; return &m->norm_out; }
    if (!strcmp(name, "proj_out.weight")) { *expect = c->channels * H; return &m->proj_out; }
    if (sscanf(name, "transformer_blocks.%d.%199s", &i, rest) == 2 && i >= 0 && i < c->n_double) {
        fo_double *b = &m->dbl[i];
        if (!strcmp(rest, "attn.norm_q.weight")) { *expect = c->head_dim; return &b->img.norm_q; }
        if (!strcmp(rest, "attn.norm_k.weight")) { *expect = c->head_dim; return &b->img.norm_k; }
        if (!strcmp(rest, "attn.norm_added_q.weight")) { *expect = c->head_dim; return &b->txt.norm_q; }
        if (!strcmp(rest, "attn.norm_added_k.weight")) { *expect = c->head_dim; return &b->txt.norm_k; }
        if (!strcmp(rest, "attn.to_q.weight")) { *expect = H * H; return &b->img.q; }
        if (!strcmp(rest, "attn.to_k.weight")) { *expect = H * H; return &b->img.k; }
        if (!strcmp(rest, "attn.to_v.weight")) { *expect = H * H; return &b->img.v; }
        if (!strcmp(rest, "attn.add_q_proj.weight")) { *expect = H * H; return &b->txt.q; }
        if (!strcmp(rest, "attn.add_k_proj.weight")) { *expect = H * H; return &b->txt.k; }
        if (!strcmp(rest, "attn.add_v_proj.weight")) { *expect = H * H; return &b->txt.v; }
        if (!strcmp(rest, "attn.to_out.0.weight")) { *expect = H * H; return &b->img.proj; }
        if (!strcmp(rest, "attn.to_add_out.weight")) { *expect = H * H; return &b->txt.proj; }
        if (!strcmp(rest, "ff.linear_in.weight")) { *expect = 2 * M * H; return &b->img.ff_in; }
        if (!strcmp(rest, "ff_context.linear_in.weight")) { *expect = 2 * M * H; return &b->txt.ff_in; }
        if (!strcmp(rest, "ff.linear_out.weight")) { *expect = H * M; return &b->img.ff_out; }
        if (!strcmp(rest, "ff_context.linear_out.weight")) { *expect = H * M; return &b->txt.ff_out; }
        return NULL;
    }
    if (sscanf(name, "single_transformer_blocks.%d.%199s", &i, rest) == 2 && i >= 0 && i < c->n_single) {
        fo_single *b = &m->sgl[i];
        if (!strcmp(rest, "attn.norm_q.weight")) { *expect = c->head_dim; return &b->norm_q; }
        if (!strcmp(rest, "attn.norm_k.weight")) { *expect = c->head_dim; return &b->norm_k; }
        if (!strcmp(rest, "attn.to_qkv_mlp_proj.weight")) { *expect = (3 * H + 2 * M) * H; return &b->qkv_mlp; }
        if (!strcmp(rest, "attn.to_out.weight")) { *expect = H * (H + M); return &b->out; }
        return NULL;
    }
    return NULL;
}

/* Widen a bf16 tensor into the model (exact). 0 = ok, -1 unknown name,
 * -2 wrong element count. */
int fo_model_set_bf16(fo_model *m, const char *name, const uint16_t *data, int64_t n) {
    int64_t expect = 0;
    float **slot = slot_for(m, name, &expect);
    if (!slot) return -1;
    if (expect != n) return -2;
    free(*slot);
    float *dst = (float *)malloc(sizeof(float) * (size_t)n);
    #pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < n; i++) {
        uint32_t b = ((uint32_t)data[i]) << 16;
        memcpy(&dst[i], &b, 4);
    }
    *slot = dst;
    return 0;
}

/* ------------------------------------------------------------------------
 * Blocks
 * ------------------------------------------------------------------------ */

/* down(silu(gate(x)) * up(x)); linear_in rows are [gate ; up]
 * (flux_transformer.c:1737-1763 and the split at 4503-4523). */
static void swiglu(float *out, const float *x, const float *ff_in, const float *ff_out,
                   int seq, int hidden, int mlp) {
    float *gu = (float *)malloc(sizeof(float) * (size_t)seq * 2 * mlp);
    fo_linear(gu, x, ff_in, seq, hidden, 2 * mlp);
    float *act = (float *)malloc(sizeof(float) * (size_t)seq * mlp);
    #pragma omp parallel for schedule(static)
    for (int s = 0; s < seq; s++)
        for (int j = 0; j < mlp; j++) {
            float g = gu[(size_t)s * 2 * mlp + j], u = gu[(size_t)s * 2 * mlp + mlp + j];
            act[(size_t)s * mlp + j] = (g / (1.0f + expf(-g))) * u;
        }
    fo_linear(out, act, ff_out, seq, mlp, hidden);
    free(gu); free(act);
}

/* One double-stream block, in place on img_h [img_seq,H] and txt_h [txt_seq,H]
 * (flux_transformer.c:1774-1986). mod = [shift1,scale1,gate1,shift2,scale2,gate2]. */
void fo_double_block(const fo_model *m, int idx, float *img_h, float *txt_h,
                     const float *img_mod, const float *txt_mod,
                     const float *img_cos, const float *img_sin,
                     const float *txt_cos, const float *txt_sin,
                     int img_seq, int txt_seq) {
    const fo_config *c = &m->c;
    const fo_double *b = &m->dbl[idx];
    int H = c->hidden, heads = c->heads, hd = c->head_dim, tot = img_seq + txt_seq;
    float eps = 1e-6f;
    size_t nt = (size_t)tot * H;
    float *norm = (float *)malloc(sizeof(float) * nt);
    float *q = (float *)malloc(sizeof(float) * nt);
    float *k = (float *)malloc(sizeof(float) * nt);
    float *v = (float *)malloc(sizeof(float) * nt);
    float *att = (float *)malloc(sizeof(float) * nt);
    float *proj = (float *)malloc(sizeof(float) * nt);

    /* Rows [0,txt_seq) hold text, [txt_seq,tot) hold image: the K/V order the
     * reference concatenates in (flux_transformer.c:1351-1354). */
    float *tq = q, *tk = k, *tv = v, *iq = q + (size_t)txt_seq * H,
          *ik = k + (size_t)txt_seq * H, *iv = v + (size_t)txt_seq * H;
    float *tnorm = norm, *inorm = norm + (size_t)txt_seq * H;

    fo_adaln(inorm, img_h, img_mod, img_mod + H, img_seq, H, eps);
    fo_linear(iq, inorm, b->img.q, img_seq, H, H);
    fo_linear(ik, inorm, b->img.k, img_seq, H, H);
    fo_linear(iv, inorm, b->img.v, img_seq, H, H);
    fo_qk_norm(iq, ik, b->img.norm_q, b->img.norm_k, img_seq, heads, hd, eps);
    fo_apply_rope(iq, img_cos, img_sin, img_seq, heads, hd);
    fo_apply_rope(ik, img_cos, img_sin, img_seq, heads, hd);

    fo_adaln(tnorm, txt_h, txt_mod, txt_mod + H, txt_seq, H, eps);
    fo_linear(tq, tnorm, b->txt.q, txt_seq, H, H);
    fo_linear(tk, tnorm, b->txt.k, txt_seq, H, H);
    fo_linear(tv, tnorm, b->txt.v, txt_seq, H, H);
    fo_qk_norm(tq, tk, b->txt.norm_q, b->txt.norm_k, txt_seq, heads, hd, eps);
    fo_apply_rope(tq, txt_cos, txt_sin, txt_seq, heads, hd);
    fo_apply_rope(tk, txt_cos, txt_sin, txt_seq, heads, hd);

    /* Joint attention: both query sets see all keys (flux_transformer.c:1335-1460). */
    fo_attention(att, q, k, v, tot, tot, heads, hd);

    float *tatt = att, *iatt = att + (size_t)txt_seq * H;
    float *tproj = proj, *iproj = proj + (size_t)txt_seq * H;
    fo_linear(iproj, iatt, b->img.proj, img_seq, H, H);
    fo_linear(tproj, tatt, b->txt.proj, txt_seq, H, H);
    fo_gated_add(img_h, img_mod + 2 * H, iproj, img_seq, H);
    fo_gated_add(txt_h, txt_mod + 2 * H, tproj, txt_seq, H);

    fo_adaln(inorm, img_h, img_mod + 3 * H, img_mod + 4 * H, img_seq, H, eps);
    swiglu(iproj, inorm, b->img.ff_in, b->img.ff_out, img_seq, H, c->mlp);
    fo_gated_add(img_h, img_mod + 5 * H, iproj, img_seq, H);

    fo_adaln(tnorm, txt_h, txt_mod + 3 * H, txt_mod + 4 * H, txt_seq, H, eps);
    swiglu(tproj, tnorm, b->txt.ff_in, b->txt.ff_out, txt_seq, H, c->mlp);
    fo_gated_add(txt_h, txt_mod + 5 * H, tproj, txt_seq, H);

    free(norm); free(q); free(k); free(v); free(att); free(proj);
}

/* One single-stream block, in place on x [seq,H] laid out [text ; image]
 * (flux_transformer.c:2992-3109). mod = [shift, scale, gate] (3026-3028). */
void fo_single_block(const fo_model *m, int idx, float *x, const float *mod,
                     const float *img_cos, const float *img_sin,
                     const float *txt_cos, const float *txt_sin,
                     int seq, int txt_seq) {
    const fo_config *c = &m->c;
    const fo_single *b = &m->sgl[idx];
    int H = c->hidden, heads = c->heads, hd = c->head_dim, M = c->mlp;
    int fused = 3 * H + 2 * M, img_seq = seq - txt_seq;
    float eps = 1e-6f;
    float *norm = (float *)malloc(sizeof(float) * (size_t)seq * H);
    float *f = (float *)malloc(sizeof(float) * (size_t)seq * fused);
    float *q = (float *)malloc(sizeof(float) * (size_t)seq * H);
    float *k = (float *)malloc(sizeof(float) * (size_t)seq * H);
    float *v = (float *)malloc(sizeof(float) * (size_t)seq * H);
    float *cat = (float *)malloc(sizeof(float) * (size_t)seq * (H + M));
    float *att = (float *)malloc(sizeof(float) * (size_t)seq * H);
    float *proj = (float *)malloc(sizeof(float) * (size_t)seq * H);

    fo_adaln(norm, x, mod, mod + H, seq, H, eps);
    /* Row layout of the fused projection: [Q | K | V | gate | up] (3034-3058). */
    fo_linear(f, norm, b->qkv_mlp, seq, H, fused);
    #pragma omp parallel for schedule(static)
    for (int s = 0; s < seq; s++) {
        const float *r = f + (size_t)s * fused;
        memcpy(q + (size_t)s * H, r, sizeof(float) * H);
        memcpy(k + (size_t)s * H, r + H, sizeof(float) * H);
        memcpy(v + (size_t)s * H, r + 2 * H, sizeof(float) * H);
        float *cm = cat + (size_t)s * (H + M) + H;
        for (int j = 0; j < M; j++) {
            float g = r[3 * H + j], u = r[3 * H + M + j];
            cm[j] = (g / (1.0f + expf(-g))) * u;
        }
    }
    fo_qk_norm(q, k, b->norm_q, b->norm_k, seq, heads, hd, eps);
    fo_apply_rope(q, txt_cos, txt_sin, txt_seq, heads, hd);
    fo_apply_rope(k, txt_cos, txt_sin, txt_seq, heads, hd);
    fo_apply_rope(q + (size_t)txt_seq * H, img_cos, img_sin, img_seq, heads, hd);
    fo_apply_rope(k + (size_t)txt_seq * H, img_cos, img_sin, img_seq, heads, hd);
    fo_attention(att, q, k, v, seq, seq, heads, hd);
    /* concat [attention | mlp] then one projection (3093-3103) */
    #pragma omp parallel for schedule(static)
    for (int s = 0; s < seq; s++)
        memcpy(cat + (size_t)s * (H + M), att + (size_t)s * H, sizeof(float) * H);
    fo_linear(proj, cat, b->out, seq, H + M, H);
    fo_gated_add(x, mod + 2 * H, proj, seq, H);

    free(norm); free(f); free(q); free(k); free(v); free(cat); free(att); free(proj);
}

typedef struct { const float *latent; int h, w, t_offset; } fo_ref;

static void silu_vec(float *out, const float *in, int n) {
    for (int i = 0; i < n; i++) { float x = in[i]; out[i] = x / (1.0f + expf(-x)); }
}

/* Full forward. Image stream = [target ; ref_1 ; ...]; only target rows are
 * projected out. Returns malloc'd [channels, img_h*img_w] (NCHW), caller frees.
 * (flux_transformer.c:3115-3577 without references, 3605-3799 with one,
 * 3815-4043 with several.) */
float *fo_forward(const fo_model *m, const float *img_latent, int img_h, int img_w,
                  const fo_ref *refs, int num_refs,
                  const float *txt_emb, int txt_seq, float timestep) {
    const fo_config *c = &m->c;
    int H = c->hidden, C = c->channels, hd = c->head_dim;
    int img_seq = img_h * img_w, comb = img_seq;
    for (int r = 0; r < num_refs; r++) comb += refs[r].h * refs[r].w;
    int tot = comb + txt_seq;

    /* timestep embedding: t is scaled by 1000 first (3140) */
    float *e = (float *)malloc(sizeof(float) * c->sincos_dim);
    float *t_emb = (float *)malloc(sizeof(float) * H);
    float *t_silu = (float *)malloc(sizeof(float) * H);
    fo_timestep_embedding(e, timestep * 1000.0f, c->sincos_dim, 10000.0f);
    fo_time_mlp(t_emb, e, m->t_fc1, m->t_fc2, c->sincos_dim, H);
    silu_vec(t_silu, t_emb, H);

    /* RoPE tables: target at T=0, each reference at its own T offset */
    float *icos = (float *)malloc(sizeof(float) * (size_t)comb * hd);
    float *isin = (float *)malloc(sizeof(float) * (size_t)comb * hd);
    float *tcos = (float *)malloc(sizeof(float) * (size_t)txt_seq * hd);
    float *tsin = (float *)malloc(sizeof(float) * (size_t)txt_seq * hd);
    fo_rope_image(icos, isin, img_h, img_w, c->axis_dim, c->rope_theta, 0);
    {
        size_t off = (size_t)img_seq * hd;
        for (int r = 0; r < num_refs; r++) {
            fo_rope_image(icos + off, isin + off, refs[r].h, refs[r].w, c->axis_dim,
                          c->rope_theta, refs[r].t_offset);
            off += (size_t)refs[r].h * refs[r].w * hd;
        }
    }
    fo_rope_text(tcos, tsin, txt_seq, c->axis_dim, c->rope_theta);

    /* NCHW -> [seq, channels] for target and references (3156-3161, 3654-3664) */
    float *tok = (float *)malloc(sizeof(float) * (size_t)comb * C);
    for (int p = 0; p < img_seq; p++)
        for (int ch = 0; ch < C; ch++) tok[(size_t)p * C + ch] = img_latent[(size_t)ch * img_seq + p];
    {
        int off = img_seq;
        for (int r = 0; r < num_refs; r++) {
            int rs = refs[r].h * refs[r].w;
            for (int p = 0; p < rs; p++)
                for (int ch = 0; ch < C; ch++)
                    tok[(size_t)(off + p) * C + ch] = refs[r].latent[(size_t)ch * rs + p];
            off += rs;
        }
    }

    /* x = [text ; image] hidden states; the reference keeps two buffers until
     * the single-stream stage and then concatenates in this order (3278-3281). */
    float *x = (float *)malloc(sizeof(float) * (size_t)tot * H);
    float *txt_h = x, *img_hid = x + (size_t)txt_seq * H;
    fo_linear(img_hid, tok, m->img_in, comb, C, H);
    fo_linear(txt_h, txt_emb, m->txt_in, txt_seq, c->text_dim, H);
    free(tok);

    /* Double-stream modulation, computed once per forward (3226-3234) */
    float *mod_i = (float *)malloc(sizeof(float) * 6 * H);
    float *mod_t = (float *)malloc(sizeof(float) * 6 * H);
    fo_linear(mod_i, t_silu, m->mod_img, 1, H, 6 * H);
    fo_linear(mod_t, t_silu, m->mod_txt, 1, H, 6 * H);
    for (int i = 0; i < c->n_double; i++)
        fo_double_block(m, i, img_hid, txt_h, mod_i, mod_t, icos, isin, tcos, tsin, comb, txt_seq);

    /* Single-stream modulation: same vector for every block (3024) */
    float *mod_s = (float *)malloc(sizeof(float) * 3 * H);
    fo_linear(mod_s, t_silu, m->mod_single, 1, H, 3 * H);
    for (int i = 0; i < c->n_single; i++)
        fo_single_block(m, i, x, mod_s, icos, isin, tcos, tsin, tot, txt_seq);

    /* Final layer on target rows only; chunk order is (scale, shift) (3532-3534) */
    float *fm = (float *)malloc(sizeof(float) * 2 * H);
    fo_linear(fm, t_silu, m->norm_out, 1, H, 2 * H);
    float *fn = (float *)malloc(sizeof(float) * (size_t)img_seq * H);
    fo_adaln(fn, img_hid, fm + H, fm, img_seq, H, 1e-6f);
    float *nlc = (float *)malloc(sizeof(float) * (size_t)img_seq * C);
    fo_linear(nlc, fn, m->proj_out, img_seq, H, C);
    float *out = (float *)malloc(sizeof(float) * (size_t)img_seq * C);
    for (int p = 0; p < img_seq; p++)
        for (int ch = 0; ch < C; ch++) out[(size_t)ch * img_seq + p] = nlc[(size_t)p * C + ch];

    free(e); free(t_emb); free(t_silu); free(icos); free(isin); free(tcos); free(tsin);
    free(x); free(mod_i); free(mod_t); free(mod_s); free(fm); free(fn); free(nlc);
    return out;
}

void fo_free(void *p) { free(p); }

/* ------------------------------------------------------------------------
 * Schedules   (flux_sample.c:49-155)
 * ------------------------------------------------------------------------ */
void fo_linear_schedule(float *s, int n) {
    for (int i = 0; i <= n; i++) s[i] = 1.0f - (float)i / (float)n;
}

void fo_power_schedule(float *s, int n, float alpha) {
    for (int i = 0; i <= n; i++) s[i] = 1.0f - powf((float)i / (float)n, alpha);
}

/* Shifted sigmoid, endpoints forced to 1 and 0 (flux_sample.c:75-91). */
void fo_sigmoid_schedule(float *s, int n, float shift) {
    for (int i = 0; i <= n; i++) {
        float x = ((float)i / (float)n - 0.5f) * 10.0f + shift;
        s[i] = 1.0f - 1.0f / (1.0f + expf(-x));
    }
    s[0] = 1.0f;
    s[n] = 0.0f;
}

/* 1 - (i/n)^(1 + shift/2), shift 1 from 1024x1024 pixels, 0.5 from 512x512, else 0
 * (flux_sample.c:96-116). */
void fo_resolution_schedule(float *s, int n, int height, int width) {
    int pixels = height * width;
    float shift = pixels >= 1024 * 1024 ? 1.0f : pixels >= 512 * 512 ? 0.5f : 0.0f;
    for (int i = 0; i <= n; i++) s[i] = 1.0f - powf((float)i / (float)n, 1.0f + shift * 0.5f);
}

static float empirical_mu(int seq_len, int steps) {
    const float a1 = 8.73809524e-05f, b1 = 1.89833333f;
    const float a2 = 0.00016927f, b2 = 0.45666666f;
    if (seq_len > 4300) return a2 * seq_len + b2;
    float m200 = a2 * seq_len + b2, m10 = a1 * seq_len + b1;
    float a = (m200 - m10) / 190.0f;
    float b = m200 - 200.0f * a;
    return a * steps + b;
}

void fo_official_schedule(float *s, int n, int image_seq_len) {
    float mu = empirical_mu(image_seq_len, n);
    for (int i = 0; i <= n; i++) {
        float t = 1.0f - (float)i / (float)n;
        if (t <= 0.0f) s[i] = 0.0f;
        else if (t >= 1.0f) s[i] = 1.0f;
        else s[i] = expf(mu) / (expf(mu) + powf(1.0f / t - 1.0f, 1.0f));
    }
}

/* ------------------------------------------------------------------------
 * Samplers. z is [channels,h,w]; returns malloc'd final latent. When v_trace
 * is non-NULL it receives every forward's velocity, in call order
 * ([num_steps * forwards_per_step, channels*h*w]).
 * Euler: flux_sample.c:212-290 (no refs), 303-375 / 381-444 (refs).
 * CFG:   flux_sample.c:457-529, 534-610, 615-691 (uncond first, then cond;
 *        v = vu + g*(vc - vu); z += dt*v).
 * ------------------------------------------------------------------------ */
float *fo_sample_euler(const fo_model *m, const float *z, int h, int w,
                       const fo_ref *refs, int num_refs,
                       const float *txt, int txt_seq,
                       const float *schedule, int num_steps, float *v_trace) {
    int n = m->c.channels * h * w;
    float *zc = (float *)malloc(sizeof(float) * n);
    memcpy(zc, z, sizeof(float) * n);
    for (int s = 0; s < num_steps; s++) {
        float dt = schedule[s + 1] - schedule[s];
        float *v = fo_forward(m, zc, h, w, refs, num_refs, txt, txt_seq, schedule[s]);
        if (v_trace) memcpy(v_trace + (size_t)s * n, v, sizeof(float) * n);
        for (int i = 0; i < n; i++) zc[i] += dt * v[i];
        free(v);
    }
    return zc;
}

float *fo_sample_euler_cfg(const fo_model *m, const float *z, int h, int w,
                           const fo_ref *refs, int num_refs,
                           const float *txt_cond, int seq_cond,
                           const float *txt_uncond, int seq_uncond,
                           float guidance, const float *schedule, int num_steps,
                           float *v_trace) {
    int n = m->c.channels * h * w;
    float *zc = (float *)malloc(sizeof(float) * n);
    memcpy(zc, z, sizeof(float) * n);
    for (int s = 0; s < num_steps; s++) {
        float dt = schedule[s + 1] - schedule[s];
        float *vu = fo_forward(m, zc, h, w, refs, num_refs, txt_uncond, seq_uncond, schedule[s]);
        float *vc = fo_forward(m, zc, h, w, refs, num_refs, txt_cond, seq_cond, schedule[s]);
        if (v_trace) {
            memcpy(v_trace + (size_t)(2 * s) * n, vu, sizeof(float) * n);
            memcpy(v_trace + (size_t)(2 * s + 1) * n, vc, sizeof(float) * n);
        }
        for (int i = 0; i < n; i++) {
            float v = vu[i] + guidance * (vc[i] - vu[i]);
            zc[i] += dt * v;
        }
        free(vu); free(vc);
    }
    return zc;
}

/* Heun (flux_sample.c:760-826): v1 at (z, t_s); predictor zp = z + dt v1; v2 at (zp, t_{s+1});
 * z += dt/2 (v1 + v2); the last step is a plain Euler step. v_trace gets v1, v2 of every step
 * in call order (2*num_steps - 1 velocities). */
float *fo_sample_heun(const fo_model *m, const float *z, int h, int w,
                      const float *txt, int txt_seq,
                      const float *schedule, int num_steps, float *v_trace) {
    int n = m->c.channels * h * w;
    float *zc = (float *)malloc(sizeof(float) * n);
    float *zp = (float *)malloc(sizeof(float) * n);
    memcpy(zc, z, sizeof(float) * n);
    size_t k = 0;
    for (int s = 0; s < num_steps; s++) {
        float dt = schedule[s + 1] - schedule[s];
        float *v1 = fo_forward(m, zc, h, w, NULL, 0, txt, txt_seq, schedule[s]);
        if (v_trace) memcpy(v_trace + (k++) * n, v1, sizeof(float) * n);
        if (s < num_steps - 1) {
            for (int i = 0; i < n; i++) zp[i] = zc[i] + dt * v1[i];
            float *v2 = fo_forward(m, zp, h, w, NULL, 0, txt, txt_seq, schedule[s + 1]);
            if (v_trace) memcpy(v_trace + (k++) * n, v2, sizeof(float) * n);
            for (int i = 0; i < n; i++) zc[i] += 0.5f * dt * (v1[i] + v2[i]);
            free(v2);
        } else {
            for (int i = 0; i < n; i++) zc[i] += dt * v1[i];
        }
        free(v1);
    }
    free(zp);
    return zc;
}

void fo_randn(float *out, int64_t n);

/* Euler with noise injection (flux_sample.c:697-748): after every step but the last,
 * z += eta sqrt(|dt|) * N(0,1) drawn from the global generator in its current state. */
float *fo_sample_euler_ancestral(const fo_model *m, const float *z, int h, int w,
                                 const float *txt, int txt_seq,
                                 const float *schedule, int num_steps, float eta, float *v_trace) {
    int n = m->c.channels * h * w;
    float *zc = (float *)malloc(sizeof(float) * n);
    float *noise = (float *)malloc(sizeof(float) * n);
    memcpy(zc, z, sizeof(float) * n);
    for (int s = 0; s < num_steps; s++) {
        float dt = schedule[s + 1] - schedule[s];
        float *v = fo_forward(m, zc, h, w, NULL, 0, txt, txt_seq, schedule[s]);
        if (v_trace) memcpy(v_trace + (size_t)s * n, v, sizeof(float) * n);
        for (int i = 0; i < n; i++) zc[i] += dt * v[i];
        if (eta > 0 && s < num_steps - 1) {
            float sigma = eta * sqrtf(fabsf(dt));
            fo_randn(noise, n);
            for (int i = 0; i < n; i++) zc[i] += sigma * noise[i];
        }
        free(v);
    }
    free(noise);
    return zc;
}

/* ------------------------------------------------------------------------
 * Reference RNG: SplitMix64-seeded xoshiro256** + Box-Muller
 * (flux_kernels.c:45-102), and the size-independent noise initialiser
 * (flux_sample.c:837-877).
 * ------------------------------------------------------------------------ */
static uint64_t g_rng[4] = {0x853c49e6748fea9bULL, 0xda3e39cb94b95bdbULL,
                            0x647c4677a2884327ULL, 0xc6e7918d2e2969f5ULL};
static inline uint64_t rotl64(uint64_t x, int k) { return (x << k) | (x >> (64 - k)); }

static uint64_t rng_next(void) {
    uint64_t r = rotl64(g_rng[1] * 5, 7) * 9, t = g_rng[1] << 17;
    g_rng[2] ^= g_rng[0]; g_rng[3] ^= g_rng[1]; g_rng[1] ^= g_rng[2]; g_rng[0] ^= g_rng[3];
    g_rng[2] ^= t; g_rng[3] = rotl64(g_rng[3], 45);
    return r;
}

void fo_rng_seed(uint64_t seed) {
    for (int i = 0; i < 4; i++) {
        seed += 0x9e3779b97f4a7c15ULL;
        uint64_t z = seed;
        z = (z ^ (z >> 30)) * 0xbf58476d1ce4e5b9ULL;
        z = (z ^ (z >> 27)) * 0x94d049bb133111ebULL;
        g_rng[i] = z ^ (z >> 31);
    }
}

static float rng_uniform(void) { return (rng_next() >> 11) * (1.0 / 9007199254740992.0); }

static float rng_normal(void) {
    float u1 = rng_uniform(), u2 = rng_uniform();
    while (u1 == 0.0f) u1 = rng_uniform();
    return sqrtf(-2.0f * logf(u1)) * cosf(2.0f * 3.14159265358979323846f * u2);
}

void fo_randn(float *out, int64_t n) { for (int64_t i = 0; i < n; i++) out[i] = rng_normal(); }

void fo_init_noise(float *noise, int channels, int h, int w, int64_t seed) {
    const int MAXD = 112;
    if (seed >= 0) fo_rng_seed((uint64_t)seed);
    if (h >= MAXD && w >= MAXD) { fo_randn(noise, (int64_t)channels * h * w); return; }
    float *big = (float *)malloc(sizeof(float) * (size_t)channels * MAXD * MAXD);
    fo_randn(big, (int64_t)channels * MAXD * MAXD);
    for (int c = 0; c < channels; c++)
        for (int y = 0; y < h; y++)
            for (int x = 0; x < w; x++)
                noise[((size_t)c * h + y) * w + x] =
                    big[((size_t)c * MAXD + y * MAXD / h) * MAXD + x * MAXD / w];
    free(big);
}
