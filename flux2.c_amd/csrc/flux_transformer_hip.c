/*
 * flux_transformer_hip.c - host side of the FLUX.2-klein denoising transformer on MI355X.
 *
 * Plain C over the operator ABI of flux_hip.h. It exports the reference's transformer entry
 * points (flux_transformer.c:3115, 3605, 3815, 4189, 4411, 4659) and keeps their contracts:
 * host fp32 in, malloc'd host fp32 out. What differs is where the work happens:
 *
 *  - weights stay in bf16 and are uploaded once; Q/K/V of a double block are stored as one
 *    [3H, H] matrix per stream so the three projections are one GEMM;
 *  - text and image tokens share one [text ; image(target ; refs)] activation buffer, which is
 *    the order the reference concatenates in (flux_transformer.c:1351-1354, 3278-3281), so the
 *    double blocks run two row ranges with different weights in one launch and no concat or
 *    split copies exist;
 *  - the residual stream is fp32, everything that feeds a GEMM is bf16;
 *  - all modulation vectors depend only on the timestep: they are computed for every step of
 *    a schedule in one batch before the loop (the reference recomputes the single-stream
 *    modulation in each of the 20 blocks, flux_transformer.c:3024).
 */
#include "../../include/flux_hip.h"
#include "../../include/flux_hip_debug.h"
#include "host_internal.h"
#include <math.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

flux_substep_callback_t flux_substep_callback = NULL;
flux_step_callback_t flux_step_callback = NULL;
int flux_verbose = 0;

void flux_hip_default_config(flux_hip_config *c) {
    c->hidden = 3072; c->heads = 24; c->head_dim = 128; c->mlp = 9216;
    c->n_double = 5; c->n_single = 20; c->text_dim = 7680; c->channels = 128;
    c->axis_dim = 32; c->sincos_dim = 256; c->rope_theta = 2000.0f;
}

/* ------------------------------------------------------------------ construction */

static int config_ok(const flux_hip_config *c) {
    if (c->head_dim != 128 || c->axis_dim != 32)
        return flux_hip_fail("config: head_dim must be 128 and axis_dim 32 (got %d, %d)", c->head_dim, c->axis_dim);
    if (c->hidden != c->heads * c->head_dim) return flux_hip_fail("config: hidden != heads * head_dim");
    if (c->hidden % 256 || c->hidden > 4096) return flux_hip_fail("config: hidden=%d must be a multiple of 256, at most 4096", c->hidden);
    if (c->mlp % 64 || c->text_dim % 64 || c->channels % 128 || c->sincos_dim % 8)
        return flux_hip_fail("config: mlp/text_dim must be multiples of 64, channels of 128, sincos_dim of 8");
    if (c->n_double < 0 || c->n_single < 0) return flux_hip_fail("config: negative layer count");
    return 1;
}

flux_transformer_t *flux_hip_transformer_new(const flux_hip_config *cfg) {
    if (!flux_hip_available()) return NULL;
    if (!config_ok(cfg)) return NULL;
    flux_transformer_t *tf = (flux_transformer_t *)calloc(1, sizeof(*tf));
    if (!tf) { flux_hip_fail("out of host memory"); return NULL; }
    tf->c = *cfg;
    tf->dbl = (fh_double *)calloc(cfg->n_double ? cfg->n_double : 1, sizeof(fh_double));
    tf->sgl = (fh_single *)calloc(cfg->n_single ? cfg->n_single : 1, sizeof(fh_single));
    return tf;
}

/* Uploads `numel` bf16 values into *slot at element offset `at` of a buffer of `total`. */
static int put_bf16(void **slot, size_t total, size_t at, const uint16_t *src, size_t numel) {
    if (!*slot) {
        *slot = flux_hip_malloc(total * 2);
        if (!*slot) return 0;
    }
    return flux_hip_upload((char *)*slot + at * 2, src, numel * 2);
}

/* QK-norm weights are kept in fp32 on the device (the reference keeps them fp32 too,
 * flux_transformer.c:117-118). */
static int put_norm(float **slot, const uint16_t *src, size_t numel) {
    float tmp[128];
    if (numel != 128) return flux_hip_fail("norm weight must have 128 elements");
    for (int i = 0; i < 128; i++) {
        uint32_t b = ((uint32_t)src[i]) << 16;
        memcpy(&tmp[i], &b, 4);
    }
    if (!*slot) {
        *slot = (float *)flux_hip_malloc(sizeof(tmp));
        if (!*slot) return 0;
    }
    return flux_hip_upload(*slot, tmp, sizeof(tmp));
}

#define EXPECT(n)                                                                          \
    do {                                                                                   \
        if ((int64_t)(n) != numel)                                                         \
            return flux_hip_fail("tensor %s: %lld elements, expected %lld", name,          \
                                 (long long)numel, (long long)(n));                        \
    } while (0)

int flux_hip_transformer_set_tensor(flux_transformer_t *tf, const char *name, const uint16_t *d, int64_t numel) {
    if (!tf || !name || !d) return flux_hip_fail("flux_hip_transformer_set_tensor: NULL argument");
    const flux_hip_config *c = &tf->c;
    const size_t H = c->hidden, M = c->mlp;
    int i;
    char rest[200];
    if (!strcmp(name, "x_embedder.weight")) { EXPECT(H * c->channels); return put_bf16(&tf->img_in, numel, 0, d, numel); }
    if (!strcmp(name, "context_embedder.weight")) { EXPECT(H * c->text_dim); return put_bf16(&tf->txt_in, numel, 0, d, numel); }
    if (!strcmp(name, "time_guidance_embed.timestep_embedder.linear_1.weight")) { EXPECT(H * c->sincos_dim); return put_bf16(&tf->t_fc1, numel, 0, d, numel); }
    if (!strcmp(name, "time_guidance_embed.timestep_embedder.linear_2.weight")) { EXPECT(H * H); return put_bf16(&tf->t_fc2, numel, 0, d, numel); }
    if (!strcmp(name, "double_stream_modulation_img.linear.weight")) { EXPECT(6 * H * H); return put_bf16(&tf->mod_w[1], numel, 0, d, numel); }
    if (!strcmp(name, "double_stream_modulation_txt.linear.weight")) { EXPECT(6 * H * H); return put_bf16(&tf->mod_w[0], numel, 0, d, numel); }
    if (!strcmp(name, "single_stream_modulation.linear.weight")) { EXPECT(3 * H * H); return put_bf16(&tf->mod_w[2], numel, 0, d, numel); }
    if (!strcmp(name, "norm_out.linear.weight")) { EXPECT(2 * H * H); return put_bf16(&tf->mod_w[3], numel, 0, d, numel); }
    if (!strcmp(name, "proj_out.weight")) { EXPECT(c->channels * H); return put_bf16(&tf->proj_out, numel, 0, d, numel); }
    if (sscanf(name, "transformer_blocks.%d.%199s", &i, rest) == 2) {
        if (i < 0 || i >= c->n_double) return flux_hip_fail("tensor %s: block index out of range", name);
        fh_double *b = &tf->dbl[i];
        /* stream 0 = text ("added"/"context" names), stream 1 = image */
        if (!strcmp(rest, "attn.norm_q.weight")) return put_norm(&b->norm_q[1], d, numel);
        if (!strcmp(rest, "attn.norm_k.weight")) return put_norm(&b->norm_k[1], d, numel);
        if (!strcmp(rest, "attn.norm_added_q.weight")) return put_norm(&b->norm_q[0], d, numel);
        if (!strcmp(rest, "attn.norm_added_k.weight")) return put_norm(&b->norm_k[0], d, numel);
        if (!strcmp(rest, "attn.to_q.weight")) { EXPECT(H * H); return put_bf16(&b->qkv[1], 3 * H * H, 0, d, numel); }
        if (!strcmp(rest, "attn.to_k.weight")) { EXPECT(H * H); return put_bf16(&b->qkv[1], 3 * H * H, H * H, d, numel); }
        if (!strcmp(rest, "attn.to_v.weight")) { EXPECT(H * H); return put_bf16(&b->qkv[1], 3 * H * H, 2 * H * H, d, numel); }
        if (!strcmp(rest, "attn.add_q_proj.weight")) { EXPECT(H * H); return put_bf16(&b->qkv[0], 3 * H * H, 0, d, numel); }
        if (!strcmp(rest, "attn.add_k_proj.weight")) { EXPECT(H * H); return put_bf16(&b->qkv[0], 3 * H * H, H * H, d, numel); }
        if (!strcmp(rest, "attn.add_v_proj.weight")) { EXPECT(H * H); return put_bf16(&b->qkv[0], 3 * H * H, 2 * H * H, d, numel); }
        if (!strcmp(rest, "attn.to_out.0.weight")) { EXPECT(H * H); return put_bf16(&b->proj[1], numel, 0, d, numel); }
        if (!strcmp(rest, "attn.to_add_out.weight")) { EXPECT(H * H); return put_bf16(&b->proj[0], numel, 0, d, numel); }
        if (!strcmp(rest, "ff.linear_in.weight")) { EXPECT(2 * M * H); return put_bf16(&b->ff_in[1], numel, 0, d, numel); }
        if (!strcmp(rest, "ff_context.linear_in.weight")) { EXPECT(2 * M * H); return put_bf16(&b->ff_in[0], numel, 0, d, numel); }
        if (!strcmp(rest, "ff.linear_out.weight")) { EXPECT(H * M); return put_bf16(&b->ff_out[1], numel, 0, d, numel); }
        if (!strcmp(rest, "ff_context.linear_out.weight")) { EXPECT(H * M); return put_bf16(&b->ff_out[0], numel, 0, d, numel); }
    } else if (sscanf(name, "single_transformer_blocks.%d.%199s", &i, rest) == 2) {
        if (i < 0 || i >= c->n_single) return flux_hip_fail("tensor %s: block index out of range", name);
        fh_single *b = &tf->sgl[i];
        if (!strcmp(rest, "attn.norm_q.weight")) return put_norm(&b->norm_q, d, numel);
        if (!strcmp(rest, "attn.norm_k.weight")) return put_norm(&b->norm_k, d, numel);
        if (!strcmp(rest, "attn.to_qkv_mlp_proj.weight")) { EXPECT((3 * H + 2 * M) * H); return put_bf16(&b->qkv_mlp, numel, 0, d, numel); }
        if (!strcmp(rest, "attn.to_out.weight")) { EXPECT(H * (H + M)); return put_bf16(&b->out, numel, 0, d, numel); }
    }
    return flux_hip_fail("tensor %s is not part of the transformer", name);
}

/* Every weight must be present before a forward (the reference exits on a missing weight,
 * flux_transformer.c:81-83; here the call fails instead). */
int fh_model_complete(flux_transformer_t *tf) {
    if (tf->complete) return 1;
    int ok = tf->img_in && tf->txt_in && tf->t_fc1 && tf->t_fc2 && tf->proj_out;
    for (int i = 0; i < 4; i++) ok = ok && tf->mod_w[i];
    for (int i = 0; ok && i < tf->c.n_double; i++)
        for (int s = 0; s < 2; s++) {
            fh_double *b = &tf->dbl[i];
            ok = ok && b->qkv[s] && b->norm_q[s] && b->norm_k[s] && b->proj[s] && b->ff_in[s] && b->ff_out[s];
        }
    for (int i = 0; ok && i < tf->c.n_single; i++) {
        fh_single *b = &tf->sgl[i];
        ok = ok && b->norm_q && b->norm_k && b->qkv_mlp && b->out;
    }
    if (!ok) return flux_hip_fail("transformer weights are incomplete");
    tf->complete = 1;
    return 1;
}

static void free_ws(flux_transformer_t *tf) {
    flux_hip_free(tf->x); flux_hip_free(tf->xn); flux_hip_free(tf->qkv); flux_hip_free(tf->kn);
    flux_hip_free(tf->cat); flux_hip_free(tf->tok);
    tf->x = NULL; tf->xn = tf->qkv = tf->kn = tf->cat = tf->tok = NULL;
    tf->cap_tokens = 0;
}

extern void fh_safetensors_close_compat(void *sf);

void flux_transformer_free(flux_transformer_t *tf) {
    if (!tf) return;
    flux_hip_sync();
    flux_hip_free(tf->img_in); flux_hip_free(tf->txt_in); flux_hip_free(tf->t_fc1); flux_hip_free(tf->t_fc2);
    flux_hip_free(tf->proj_out);
    for (int i = 0; i < 4; i++) flux_hip_free(tf->mod_w[i]);
    for (int i = 0; i < tf->c.n_double; i++)
        for (int s = 0; s < 2; s++) {
            fh_double *b = &tf->dbl[i];
            flux_hip_free(b->qkv[s]); flux_hip_free(b->norm_q[s]); flux_hip_free(b->norm_k[s]);
            flux_hip_free(b->proj[s]); flux_hip_free(b->ff_in[s]); flux_hip_free(b->ff_out[s]);
        }
    for (int i = 0; i < tf->c.n_single; i++) {
        fh_single *b = &tf->sgl[i];
        flux_hip_free(b->norm_q); flux_hip_free(b->norm_k); flux_hip_free(b->qkv_mlp); flux_hip_free(b->out);
    }
    free(tf->dbl); free(tf->sgl);
    free_ws(tf);
    for (int i = 0; i < FH_ROPE_SLOTS; i++) { flux_hip_free(tf->rope[i].cos); flux_hip_free(tf->rope[i].sin); }
    flux_hip_free(tf->mod); flux_hip_free(tf->temb); flux_hip_free(tf->sincos);
    if (tf->owned_sf) fh_safetensors_close_compat(tf->owned_sf);
    free(tf);
}

/* ------------------------------------------------------------------ per-shape state */

/* Work buffers grow on demand, like ensure_work_buffers (flux_transformer.c:1172-1244). */
int fh_ensure_workspace(flux_transformer_t *tf, int tokens) {
    if (tokens <= tf->cap_tokens) return 1;
    flux_hip_sync();
    free_ws(tf);
    const size_t H = tf->c.hidden, M = tf->c.mlp, n = tokens;
    tf->x = (float *)flux_hip_malloc(n * H * 4);
    tf->xn = flux_hip_malloc(n * H * 2);
    tf->qkv = flux_hip_malloc(n * 3 * H * 2);
    tf->kn = flux_hip_malloc(n * H * 2);
    tf->cat = flux_hip_malloc(n * (H + M) * 2);
    tf->tok = flux_hip_malloc(n * tf->c.channels * 2);
    if (!tf->x || !tf->xn || !tf->qkv || !tf->kn || !tf->cat || !tf->tok) {
        free_ws(tf);
        return flux_hip_fail("cannot allocate work buffers for %d tokens", tokens);
    }
    tf->cap_tokens = tokens;
    return 1;
}

/* cos/sin rows of one RoPE axis: each frequency on dims (2d, 2d+1)
 * (flux_transformer.c:620-629). */
static void rope_axis(float *c, float *s, int pos, const float *freqs, int half) {
    for (int d = 0; d < half; d++) {
        float a = (float)pos * freqs[d];
        float cv = cosf(a), sv = sinf(a);
        c[2 * d] = c[2 * d + 1] = cv;
        s[2 * d] = s[2 * d + 1] = sv;
    }
}

/* Table for rows [text ; target ; refs]: text has L = index (flux_transformer.c:747-779),
 * image tokens H = row, W = col and T = 0 or the reference's offset (591-712). */
fh_rope *fh_get_rope(flux_transformer_t *tf, int txt_seq, int img_h, int img_w, const flux_ref_t *refs, int num_refs) {
    if (num_refs > FH_MAX_REFS) { flux_hip_fail("at most %d reference images", FH_MAX_REFS); return NULL; }
    for (int i = 0; i < FH_ROPE_SLOTS; i++) {
        fh_rope *r = &tf->rope[i];
        if (!r->cos || r->txt_seq != txt_seq || r->h != img_h || r->w != img_w || r->num_refs != num_refs) continue;
        int same = 1;
        for (int j = 0; j < num_refs; j++)
            same = same && r->ref_h[j] == refs[j].h && r->ref_w[j] == refs[j].w && r->ref_t[j] == refs[j].t_offset;
        if (same) return r;
    }
    fh_rope *r = &tf->rope[tf->rope_next];
    tf->rope_next = (tf->rope_next + 1) % FH_ROPE_SLOTS;
    flux_hip_sync();
    flux_hip_free(r->cos); flux_hip_free(r->sin);
    r->cos = r->sin = NULL;

    const int ad = tf->c.axis_dim, half = ad / 2, hd = 4 * ad;
    int n_img = img_h * img_w;
    for (int j = 0; j < num_refs; j++) n_img += refs[j].h * refs[j].w;
    const int n = txt_seq + n_img;
    float freqs[64];
    for (int d = 0; d < half; d++) freqs[d] = 1.0f / powf(tf->c.rope_theta, (float)(2 * d) / (float)ad);
    float *c = (float *)malloc((size_t)n * hd * 4), *s = (float *)malloc((size_t)n * hd * 4);
    if (!c || !s) { free(c); free(s); flux_hip_fail("out of host memory"); return NULL; }
    size_t row = 0;
    for (int t = 0; t < txt_seq; t++, row++) {
        for (int a = 0; a < 3; a++) rope_axis(c + row * hd + a * ad, s + row * hd + a * ad, 0, freqs, half);
        rope_axis(c + row * hd + 3 * ad, s + row * hd + 3 * ad, t, freqs, half);
    }
    for (int g = -1; g < num_refs; g++) {
        int gh = g < 0 ? img_h : refs[g].h, gw = g < 0 ? img_w : refs[g].w, gt = g < 0 ? 0 : refs[g].t_offset;
        for (int y = 0; y < gh; y++)
            for (int x = 0; x < gw; x++, row++) {
                rope_axis(c + row * hd, s + row * hd, gt, freqs, half);
                rope_axis(c + row * hd + ad, s + row * hd + ad, y, freqs, half);
                rope_axis(c + row * hd + 2 * ad, s + row * hd + 2 * ad, x, freqs, half);
                rope_axis(c + row * hd + 3 * ad, s + row * hd + 3 * ad, 0, freqs, half);
            }
    }
    r->cos = (float *)flux_hip_malloc((size_t)n * hd * 4);
    r->sin = (float *)flux_hip_malloc((size_t)n * hd * 4);
    int ok = r->cos && r->sin && flux_hip_upload(r->cos, c, (size_t)n * hd * 4) && flux_hip_upload(r->sin, s, (size_t)n * hd * 4);
    free(c); free(s);
    if (!ok) { flux_hip_free(r->cos); flux_hip_free(r->sin); r->cos = r->sin = NULL; return NULL; }
    r->txt_seq = txt_seq; r->h = img_h; r->w = img_w; r->num_refs = num_refs;
    for (int j = 0; j < num_refs; j++) { r->ref_h[j] = refs[j].h; r->ref_w[j] = refs[j].w; r->ref_t[j] = refs[j].t_offset; }
    r->n_img = n_img; r->n = n;
    return r;
}

/* ------------------------------------------------------------------ modulation */

/* Sizes of the four modulation vectors per step: text 6H, image 6H, single 3H, final 2H. */
static const int MOD_MULT[4] = {6, 6, 3, 2};

/* Computes, for each of `steps` timesteps, t_emb and the four modulation vectors
 * (flux_transformer.c:940-969, 3226-3234, 3024, 3530). Result: tf->mod, [steps][17 H]. */
int fh_compute_modulation(flux_transformer_t *tf, const float *timesteps, int steps) {
    const int H = tf->c.hidden, sd = tf->c.sincos_dim, half = sd / 2;
    if (steps > tf->mod_cap) {
        flux_hip_sync();
        flux_hip_free(tf->mod); flux_hip_free(tf->temb); flux_hip_free(tf->sincos);
        tf->mod = (float *)flux_hip_malloc((size_t)steps * 17 * H * 4);
        tf->temb = (float *)flux_hip_malloc((size_t)steps * 2 * H * 4);
        tf->sincos = (float *)flux_hip_malloc((size_t)steps * sd * 4);
        tf->mod_cap = (tf->mod && tf->temb && tf->sincos) ? steps : 0;
        if (!tf->mod_cap) return flux_hip_fail("cannot allocate modulation buffers");
    }
    float *e = (float *)malloc((size_t)steps * sd * 4);
    if (!e) return flux_hip_fail("out of host memory");
    const float lm = logf(10000.0f);
    for (int s = 0; s < steps; s++) {
        float t = timesteps[s] * 1000.0f; /* flux_transformer.c:3140 */
        for (int i = 0; i < half; i++) {
            float a = t * expf(-lm * (float)i / (float)half);
            e[s * sd + i] = cosf(a);
            e[s * sd + half + i] = sinf(a);
        }
    }
    int ok = flux_hip_upload(tf->sincos, e, (size_t)steps * sd * 4);
    free(e);
    if (!ok) return 0;
    float *t1 = tf->temb, *t2 = tf->temb + (size_t)steps * H;
    if (!flux_hip_gemv(t1, tf->sincos, tf->t_fc1, steps, H, sd, 0)) return 0;
    if (!flux_hip_gemv(t2, t1, tf->t_fc2, steps, H, H, 1)) return 0;
    /* mod layout: region v holds [steps][MOD_MULT[v] * H] */
    size_t off = 0;
    for (int v = 0; v < 4; v++) {
        if (!flux_hip_gemv(tf->mod + off, t2, tf->mod_w[v], steps, MOD_MULT[v] * H, H, 1)) return 0;
        off += (size_t)steps * MOD_MULT[v] * H;
    }
    tf->mod_steps = steps;
    return 1;
}

static const float *mod_ptr(const flux_transformer_t *tf, int which, int step) {
    size_t off = 0;
    const size_t H = tf->c.hidden;
    for (int v = 0; v < which; v++) off += (size_t)tf->mod_steps * MOD_MULT[v] * H;
    return tf->mod + off + (size_t)step * MOD_MULT[which] * H;
}

/* ------------------------------------------------------------------ forward on the device */

/* The fused projection of a single-stream block as one launch (flux_hip_linear_qkv_swiglu; the default) or, for
 * comparison runs, as two (QKV, then gate/up with the SwiGLU epilogue). Measured per denoising step, one launch
 * against two: 80 tokens 3.10 / 3.35 ms, 768 tokens 6.24 / 6.48, 1536 tokens 10.86 / 10.73, 4608 tokens 30.31 / 30.40. */
static int g_fused_qkv_mlp = 1;
void flux_hip_set_fused_qkv_mlp(int on) { g_fused_qkv_mlp = on != 0; }

static int linear1(int epi, const void *A, const void *W, void *C, const float *gate, int M,
                   int N, int K, int lda, int ldw, int ldc, int r0, int r1) {
    flux_hip_linear_part p = {A, W, C, gate, M};
    return flux_hip_linear(epi, 1, &p, N, K, lda, ldw, ldc, r0, r1);
}

/* Attention of every sequence of the batch (rows R[b] .. R[b] + N[b] of the qkv, K and output buffers): one call, so that
 * two sequences can share a launch. */
static int attention_of_all(int nb, char *cat, int ldcat, char *qkv, char *kn, const int *R, const int *N, int H, int heads) {
    void *out[2];
    const void *q[2], *k[2], *v[2];
    for (int b = 0; b < nb; b++) {
        out[b] = cat + (size_t)R[b] * ldcat * 2;
        q[b] = qkv + (size_t)R[b] * 3 * H * 2;
        k[b] = kn + (size_t)R[b] * H * 2;
        v[b] = qkv + (size_t)R[b] * 3 * H * 2 + (size_t)2 * H * 2;
    }
    return flux_hip_attention_batch(nb, out, ldcat, q, 3 * H, k, v, 3 * H, N, N, heads);
}

/*
 * One velocity prediction per sequence, entirely on the device, for nb = 1 or 2 sequences that
 * share the target latent, the reference tokens and the timestep (the unconditional and the
 * conditional pass of a CFG step; the reference runs them one after the other,
 * flux_sample.c:485-493). Rows are laid out sequence after sequence, each as
 * [text ; target ; refs], so every GEMM of the single-stream blocks sees all rows of both
 * sequences as one matrix (each weight matrix is streamed once per step instead of twice, and the
 * launch has twice the tiles), the double-stream GEMMs run as 2 nb row ranges; attention attends per
 * sequence (in one launch for both when their block lengths agree), its Q/K preparation runs per sequence.
 *   z_dev      fp32 [channels, img_h*img_w] target latent
 *   txt_dev[b] bf16 [txt_seq_b, text_dim]
 *   tf->tok rows [n_target, n_img) must already hold the reference tokens (bf16)
 *   v_dev[b]   fp32 [channels, img_h*img_w] outputs
 * Mirrors flux_transformer_forward (flux_transformer.c:3115-3577) and the refs variants.
 */
int fh_forward_device_n(flux_transformer_t *tf, int nb, const fh_rope *const *rp, const float *z_dev, int n_target,
                        const void *const *txt_dev, int step, float *const *v_dev, fh_events *ev) {
    const flux_hip_config *c = &tf->c;
    const int H = c->hidden, M = c->mlp, C = c->channels, heads = c->heads;
    const int ldcat = H + M;
    const float eps = 1e-6f;
    if (nb < 1 || nb > 2) return flux_hip_fail("forward: %d sequences (1 or 2)", nb);
    int R[2] = {0, 0}, Nt[2] = {0, 0}, N[2] = {0, 0}, Ntot = 0;
    const int Ni = rp[0]->n_img;
    for (int b = 0; b < nb; b++) {
        if (rp[b]->n_img != Ni) return flux_hip_fail("forward: sequences differ in image tokens");
        R[b] = Ntot; Nt[b] = rp[b]->txt_seq; N[b] = rp[b]->n;
        Ntot += N[b];
    }
    if (Ntot > tf->cap_tokens) return flux_hip_fail("forward: work buffers hold %d tokens, %d needed", tf->cap_tokens, Ntot);
    char *xn = (char *)tf->xn, *qkv = (char *)tf->qkv, *cat = (char *)tf->cat, *kn = (char *)tf->kn;
    float *x = tf->x;
    const float *mt = mod_ptr(tf, 0, step), *mi = mod_ptr(tf, 1, step), *ms = mod_ptr(tf, 2, step), *mf = mod_ptr(tf, 3, step);
    flux_hip_linear_part p[4];
    flux_hip_adaln_part an[4];
    /* normed: xn already holds the AdaLN output that the next projection reads, written by the
     * second pass of the residual projection before it (flux_hip_linear_resid_adaln) */
    int normed = 0;

    if (ev) fh_event_record(ev, 0);
    /* inputs -> hidden (flux_transformer.c:3156-3196) */
    if (!flux_hip_latent_to_tokens(tf->tok, z_dev, C, n_target)) return 0;
    for (int b = 0; b < nb; b++) p[b] = (flux_hip_linear_part){tf->tok, tf->img_in, x + (size_t)(R[b] + Nt[b]) * H, NULL, Ni};
    if (!flux_hip_linear(FLUX_HIP_EPI_F32, nb, p, H, C, C, C, H, 0, 0)) return 0;
    for (int b = 0; b < nb; b++) p[b] = (flux_hip_linear_part){txt_dev[b], tf->txt_in, x + (size_t)R[b] * H, NULL, Nt[b]};
    if (!flux_hip_linear(FLUX_HIP_EPI_F32, nb, p, H, c->text_dim, c->text_dim, c->text_dim, H, 0, 0)) return 0;

    /* double-stream blocks (flux_transformer.c:1774-1986); per sequence: text rows, then image rows */
    for (int i = 0; i < c->n_double; i++) {
        const fh_double *blk = &tf->dbl[i];
        for (int b = 0; b < nb && !normed; b++)
            if (!flux_hip_adaln_norm(xn + (size_t)R[b] * H * 2, H, x + (size_t)R[b] * H, N[b], H, Nt[b], mt, mt + H, mi, mi + H, eps)) return 0;
        for (int b = 0; b < nb; b++) {
            p[2 * b] = (flux_hip_linear_part){xn + (size_t)R[b] * H * 2, blk->qkv[0], qkv + (size_t)R[b] * 3 * H * 2, NULL, Nt[b]};
            p[2 * b + 1] = (flux_hip_linear_part){xn + (size_t)(R[b] + Nt[b]) * H * 2, blk->qkv[1], qkv + (size_t)(R[b] + Nt[b]) * 3 * H * 2, NULL, Ni};
        }
        if (!flux_hip_linear(FLUX_HIP_EPI_BF16, 2 * nb, p, 3 * H, H, H, H, 3 * H, 0, 0)) return 0;
        for (int b = 0; b < nb; b++) {
            char *q_b = qkv + (size_t)R[b] * 3 * H * 2;
            if (!flux_hip_qk_prepare(kn + (size_t)R[b] * H * 2, q_b, 3 * H, 0, H, N[b], heads, Nt[b], blk->norm_q[0], blk->norm_q[1],
                                     blk->norm_k[0], blk->norm_k[1], rp[b]->cos, rp[b]->sin, eps)) return 0;
        }
        if (!attention_of_all(nb, cat, ldcat, qkv, kn, R, N, H, heads)) return 0;
        for (int b = 0; b < nb; b++) {
            p[2 * b] = (flux_hip_linear_part){cat + (size_t)R[b] * ldcat * 2, blk->proj[0], x + (size_t)R[b] * H, mt + 2 * H, Nt[b]};
            p[2 * b + 1] = (flux_hip_linear_part){cat + (size_t)(R[b] + Nt[b]) * ldcat * 2, blk->proj[1], x + (size_t)(R[b] + Nt[b]) * H, mi + 2 * H, Ni};
        }
        for (int b = 0; b < nb; b++) {
            an[2 * b] = (flux_hip_adaln_part){xn + (size_t)R[b] * H * 2, mt + 3 * H, mt + 4 * H};
            an[2 * b + 1] = (flux_hip_adaln_part){xn + (size_t)(R[b] + Nt[b]) * H * 2, mi + 3 * H, mi + 4 * H};
        }
        if (!flux_hip_linear_resid_adaln(2 * nb, p, H, H, ldcat, H, H, an, eps, &normed)) return 0;
        for (int b = 0; b < nb && !normed; b++)
            if (!flux_hip_adaln_norm(xn + (size_t)R[b] * H * 2, H, x + (size_t)R[b] * H, N[b], H, Nt[b], mt + 3 * H, mt + 4 * H, mi + 3 * H, mi + 4 * H, eps)) return 0;
        /* linear_in rows are [gate ; up] (flux_transformer.c:4503-4523) */
        for (int b = 0; b < nb; b++) {
            p[2 * b] = (flux_hip_linear_part){xn + (size_t)R[b] * H * 2, blk->ff_in[0], cat + ((size_t)R[b] * ldcat + H) * 2, NULL, Nt[b]};
            p[2 * b + 1] = (flux_hip_linear_part){xn + (size_t)(R[b] + Nt[b]) * H * 2, blk->ff_in[1], cat + ((size_t)(R[b] + Nt[b]) * ldcat + H) * 2, NULL, Ni};
        }
        if (!flux_hip_linear(FLUX_HIP_EPI_SWIGLU, 2 * nb, p, 2 * M, H, H, H, ldcat, 0, M)) return 0;
        for (int b = 0; b < nb; b++) {
            p[2 * b] = (flux_hip_linear_part){cat + ((size_t)R[b] * ldcat + H) * 2, blk->ff_out[0], x + (size_t)R[b] * H, mt + 5 * H, Nt[b]};
            p[2 * b + 1] = (flux_hip_linear_part){cat + ((size_t)(R[b] + Nt[b]) * ldcat + H) * 2, blk->ff_out[1], x + (size_t)(R[b] + Nt[b]) * H, mi + 5 * H, Ni};
        }
        /* what reads x next: the next double block's first AdaLN, or the first single block's */
        const int more = i + 1 < c->n_double;
        for (int b = 0; b < nb; b++) {
            an[2 * b] = (flux_hip_adaln_part){xn + (size_t)R[b] * H * 2, more ? mt : ms, more ? mt + H : ms + H};
            an[2 * b + 1] = (flux_hip_adaln_part){xn + (size_t)(R[b] + Nt[b]) * H * 2, more ? mi : ms, more ? mi + H : ms + H};
        }
        if (!flux_hip_linear_resid_adaln(2 * nb, p, H, M, ldcat, M, H, more || c->n_single > 0 ? an : NULL, eps, &normed)) return 0;
        if (flux_substep_callback) flux_substep_callback(FLUX_SUBSTEP_DOUBLE_BLOCK, i, c->n_double);
    }
    if (ev) fh_event_record(ev, 1);

    /* single-stream blocks (flux_transformer.c:2992-3109): fused rows [Q | K | V | gate | up]; all rows of all sequences at once */
    for (int i = 0; i < c->n_single; i++) {
        const fh_single *blk = &tf->sgl[i];
        if (!normed && !flux_hip_adaln_norm(xn, H, x, Ntot, H, Ntot, ms, ms + H, NULL, NULL, eps)) return 0;
        if (g_fused_qkv_mlp) {
            if (!flux_hip_linear_qkv_swiglu(xn, blk->qkv_mlp, qkv, cat + (size_t)H * 2, Ntot, 3 * H, M, H, H, H, 3 * H, ldcat)) return 0;
        } else {
            if (!linear1(FLUX_HIP_EPI_BF16, xn, blk->qkv_mlp, qkv, NULL, Ntot, 3 * H, H, H, H, 3 * H, 0, 0)) return 0;
            if (!linear1(FLUX_HIP_EPI_SWIGLU, xn, blk->qkv_mlp, cat + (size_t)H * 2, NULL, Ntot, 2 * M, H, H, H, ldcat, 3 * H, 3 * H + M)) return 0;
        }
        for (int b = 0; b < nb; b++) {
            char *q_b = qkv + (size_t)R[b] * 3 * H * 2;
            if (!flux_hip_qk_prepare(kn + (size_t)R[b] * H * 2, q_b, 3 * H, 0, H, N[b], heads, N[b], blk->norm_q, NULL, blk->norm_k, NULL,
                                     rp[b]->cos, rp[b]->sin, eps)) return 0;
        }
        if (!attention_of_all(nb, cat, ldcat, qkv, kn, R, N, H, heads)) return 0;
        p[0] = (flux_hip_linear_part){cat, blk->out, x, ms + 2 * H, Ntot};
        an[0] = (flux_hip_adaln_part){xn, ms, ms + H};
        if (!flux_hip_linear_resid_adaln(1, p, H, H + M, ldcat, H + M, H, i + 1 < c->n_single ? an : NULL, eps, &normed)) return 0;
        if (flux_substep_callback) flux_substep_callback(FLUX_SUBSTEP_SINGLE_BLOCK, i, c->n_single);
    }
    if (ev) fh_event_record(ev, 2);

    /* final layer on the target rows; modulation chunks are (scale, shift) (flux_transformer.c:3532-3534) */
    for (int b = 0; b < nb; b++) {
        if (!flux_hip_adaln_norm(xn + (size_t)R[b] * H * 2, H, x + (size_t)(R[b] + Nt[b]) * H, n_target, H, n_target, mf + H, mf, NULL, NULL, eps)) return 0;
        p[b] = (flux_hip_linear_part){xn + (size_t)R[b] * H * 2, tf->proj_out, v_dev[b], NULL, n_target};
    }
    if (!flux_hip_linear(FLUX_HIP_EPI_F32_T, nb, p, C, H, H, H, n_target, 0, 0)) return 0;
    if (flux_substep_callback) flux_substep_callback(FLUX_SUBSTEP_FINAL_LAYER, 0, 1);
    if (ev) fh_event_record(ev, 3);
    return 1;
}

int fh_forward_device(flux_transformer_t *tf, const fh_rope *rp, const float *z_dev, int n_target,
                      const void *txt_dev, int step, float *v_dev, fh_events *ev) {
    return fh_forward_device_n(tf, 1, &rp, z_dev, n_target, &txt_dev, step, &v_dev, ev);
}
