/*
 * qwen3_oracle.c - CPU restatement (fp32) of the Qwen3 text encoder forward that produces the
 * denoising transformer's text input (the step before the sampling loop).
 *
 * THIS FILE IS TEST INFRASTRUCTURE, like flux_oracle.c next to it: the checker that the HIP
 * encoder is compared against. It is never part of the shipped code path.
 *
 * Every function cites the file:line of antirez/flux2.c it restates (CPU arms of flux_qwen3.c).
 * The architecture is a run-time parameter (the reference fixes it in flux_qwen3.h:22-31) so
 * that tiny models run in milliseconds.
 *
 * Pinning status (tests/test_oracle_golden.py, tests/test_oracle_math.py):
 *   fo_qwen3_forward (with its rms norm, per-head norm, rotate-half RoPE, causal + padding-masked
 *   grouped-query attention and SwiGLU MLP): against the reference's own qwen3_forward compiled
 *   from its sources, on a synthetic full-size model (golden vectors), and against properties the
 *   mathematics fixes (causality, padding invariance, a numpy evaluation of one layer).
 */
#include <math.h>
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

typedef struct {
    int hidden, intermediate, heads, kv_heads, head_dim, layers, vocab;
    int out_layer[3];
    float rope_theta, eps;
} fo_qwen3_config;

typedef struct {
    float *in_norm, *post_norm, *q, *k, *v, *o, *q_norm, *k_norm, *gate, *up, *down;
} fo_qwen3_layer;

typedef struct fo_qwen3 {
    fo_qwen3_config c;
    float *embed;
    fo_qwen3_layer *layer;
} fo_qwen3;

void fo_qwen3_default_config(fo_qwen3_config *c) {
    /* flux_qwen3.h:22-39 */
    c->hidden = 2560; c->intermediate = 9728; c->heads = 32; c->kv_heads = 8; c->head_dim = 128;
    c->layers = 36; c->vocab = 151936;
    c->out_layer[0] = 8; c->out_layer[1] = 17; c->out_layer[2] = 26;
    c->rope_theta = 1000000.0f; c->eps = 1e-6f;
}

fo_qwen3 *fo_qwen3_new(const fo_qwen3_config *c) {
    fo_qwen3 *m = (fo_qwen3 *)calloc(1, sizeof *m);
    m->c = *c;
    m->layer = (fo_qwen3_layer *)calloc((size_t)c->layers, sizeof(fo_qwen3_layer));
    return m;
}

void fo_qwen3_free(fo_qwen3 *m) {
    if (!m) return;
    free(m->embed);
    for (int i = 0; i < m->c.layers; i++) {
        fo_qwen3_layer *l = &m->layer[i];
        free(l->in_norm); free(l->post_norm); free(l->q); free(l->k); free(l->v); free(l->o);
        free(l->q_norm); free(l->k_norm); free(l->gate); free(l->up); free(l->down);
    }
    free(m->layer);
    free(m);
}

/* Tensor names are the safetensors keys the reference loader asks for (flux_qwen3.c:1211-1253,
 * 1361, 1376). 0 = stored, 1 = a tensor this forward does not use, -1 unknown, -2 wrong size. */
int fo_qwen3_set_bf16(fo_qwen3 *m, const char *name, const uint16_t *data, int64_t n) {
    const fo_qwen3_config *c = &m->c;
    const int64_t H = c->hidden, I = c->intermediate, QD = (int64_t)c->heads * c->head_dim, KD = (int64_t)c->kv_heads * c->head_dim;
    float **slot = NULL;
    int64_t expect = 0;
    int li;
    char rest[128];
    if (!strcmp(name, "model.embed_tokens.weight")) { slot = &m->embed; expect = (int64_t)c->vocab * H; }
    else if (!strcmp(name, "model.norm.weight")) return 1;
    else if (sscanf(name, "model.layers.%d.%127s", &li, rest) == 2) {
        if (li < 0) return -1;
        if (li >= c->layers) return 1;
        fo_qwen3_layer *l = &m->layer[li];
        if (!strcmp(rest, "input_layernorm.weight")) { slot = &l->in_norm; expect = H; }
        else if (!strcmp(rest, "post_attention_layernorm.weight")) { slot = &l->post_norm; expect = H; }
        else if (!strcmp(rest, "self_attn.q_proj.weight")) { slot = &l->q; expect = QD * H; }
        else if (!strcmp(rest, "self_attn.k_proj.weight")) { slot = &l->k; expect = KD * H; }
        else if (!strcmp(rest, "self_attn.v_proj.weight")) { slot = &l->v; expect = KD * H; }
        else if (!strcmp(rest, "self_attn.o_proj.weight")) { slot = &l->o; expect = H * QD; }
        else if (!strcmp(rest, "self_attn.q_norm.weight")) { slot = &l->q_norm; expect = c->head_dim; }
        else if (!strcmp(rest, "self_attn.k_norm.weight")) { slot = &l->k_norm; expect = c->head_dim; }
        else if (!strcmp(rest, "mlp.gate_proj.weight")) { slot = &l->gate; expect = I * H; }
        else if (!strcmp(rest, "mlp.up_proj.weight")) { slot = &l->up; expect = I * H; }
        else if (!strcmp(rest, "mlp.down_proj.weight")) { slot = &l->down; expect = H * I; }
    }
    if (!slot) return -1;
    if (n != expect) return -2;
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

/* y[s,o] = sum_i x[s,i] W[o,i] (qwen3_linear, flux_qwen3.c:141-175) */
static void linear(float *y, const float *x, const float *W, int seq, int in_dim, int out_dim) {
    #pragma omp parallel for schedule(static)
    for (int o = 0; o < out_dim; o++) {
        const float *w = W + (size_t)o * in_dim;
        for (int s = 0; s < seq; s++) {
            const float *xr = x + (size_t)s * in_dim;
            float acc = 0.0f;
            for (int i = 0; i < in_dim; i++) acc += xr[i] * w[i];
            y[(size_t)s * out_dim + o] = acc;
        }
    }
}

/* x / sqrt(mean(x^2) + eps) * w over rows of `width` (qwen3_rms_norm :177-197; with width =
 * head_dim and rows = seq*heads it is qwen3_head_rms_norm :199-220) */
void fo_qwen3_rms_norm(float *out, const float *x, const float *w, int rows, int width, float eps) {
    for (int r = 0; r < rows; r++) {
        const float *xr = x + (size_t)r * width;
        float ss = 0.0f;
        for (int i = 0; i < width; i++) ss += xr[i] * xr[i];
        float inv = 1.0f / sqrtf(ss / width + eps);
        for (int i = 0; i < width; i++) out[(size_t)r * width + i] = xr[i] * inv * w[i];
    }
}

/* Rotate-half RoPE: pairs (i, i + head_dim/2), angle pos / theta^(2i/head_dim)
 * (compute_rope_freqs :250-262, apply_rope :264-307) */
void fo_qwen3_rope(float *x, int seq, int heads, int head_dim, float theta) {
    const int half = head_dim / 2;
    for (int s = 0; s < seq; s++)
        for (int i = 0; i < half; i++) {
            float freq = 1.0f / powf(theta, (float)(2 * i) / head_dim);
            float ang = s * freq, cs = cosf(ang), sn = sinf(ang);
            for (int h = 0; h < heads; h++) {
                float *p = x + ((size_t)s * heads + h) * head_dim;
                float x0 = p[i], x1 = p[i + half];
                p[i] = x0 * cs - x1 * sn;
                p[i + half] = x0 * sn + x1 * cs;
            }
        }
}

/* Grouped-query attention with the causal and the padding mask applied as -1e9 before a softmax
 * over all seq columns (flux_qwen3.c:352-437) */
void fo_qwen3_attention(float *out, const float *q, const float *k, const float *v, const int *mask,
                        int seq, int heads, int kv_heads, int head_dim) {
    const int qd = heads * head_dim, kd = kv_heads * head_dim, per = heads / kv_heads;
    const float scale = 1.0f / sqrtf((float)head_dim);
    #pragma omp parallel
    {
        float *sc = (float *)malloc(sizeof(float) * (size_t)seq);
        #pragma omp for collapse(2) schedule(static)
        for (int h = 0; h < heads; h++)
            for (int i = 0; i < seq; i++) {
                const int kh = h / per;
                const float *qi = q + (size_t)i * qd + h * head_dim;
                float mx = -3.0e38f;
                for (int j = 0; j < seq; j++) {
                    const float *kj = k + (size_t)j * kd + kh * head_dim;
                    float d = 0.0f;
                    for (int e = 0; e < head_dim; e++) d += qi[e] * kj[e];
                    d *= scale;
                    if (j > i) d = -1e9f;
                    if (mask && mask[j] == 0) d = -1e9f;
                    sc[j] = d;
                    if (d > mx) mx = d;
                }
                float sum = 0.0f;
                for (int j = 0; j < seq; j++) { sc[j] = expf(sc[j] - mx); sum += sc[j]; }
                float inv = 1.0f / sum;
                float *o = out + (size_t)i * qd + h * head_dim;
                for (int e = 0; e < head_dim; e++) o[e] = 0.0f;
                for (int j = 0; j < seq; j++) {
                    const float p = sc[j] * inv;
                    const float *vj = v + (size_t)j * kd + kh * head_dim;
                    for (int e = 0; e < head_dim; e++) o[e] += p * vj[e];
                }
            }
        free(sc);
    }
}

/* One layer in place on h [seq, hidden] (qwen3_layer_forward :484-520, qwen3_attention_forward
 * :313-448, qwen3_mlp_forward :458-478). */
void fo_qwen3_layer_forward(const fo_qwen3 *m, int idx, float *h, const int *mask, int seq) {
    const fo_qwen3_config *c = &m->c;
    const fo_qwen3_layer *l = &m->layer[idx];
    const int H = c->hidden, I = c->intermediate, QD = c->heads * c->head_dim, KD = c->kv_heads * c->head_dim;
    float *n = (float *)malloc(sizeof(float) * (size_t)seq * H);
    float *q = (float *)malloc(sizeof(float) * (size_t)seq * QD), *k = (float *)malloc(sizeof(float) * (size_t)seq * KD);
    float *v = (float *)malloc(sizeof(float) * (size_t)seq * KD), *a = (float *)malloc(sizeof(float) * (size_t)seq * QD);
    float *t = (float *)malloc(sizeof(float) * (size_t)seq * H);
    float *g = (float *)malloc(sizeof(float) * (size_t)seq * I), *u = (float *)malloc(sizeof(float) * (size_t)seq * I);
    fo_qwen3_rms_norm(n, h, l->in_norm, seq, H, c->eps);
    linear(q, n, l->q, seq, H, QD);
    linear(k, n, l->k, seq, H, KD);
    linear(v, n, l->v, seq, H, KD);
    fo_qwen3_rms_norm(q, q, l->q_norm, seq * c->heads, c->head_dim, c->eps);
    fo_qwen3_rms_norm(k, k, l->k_norm, seq * c->kv_heads, c->head_dim, c->eps);
    fo_qwen3_rope(q, seq, c->heads, c->head_dim, c->rope_theta);
    fo_qwen3_rope(k, seq, c->kv_heads, c->head_dim, c->rope_theta);
    fo_qwen3_attention(a, q, k, v, mask, seq, c->heads, c->kv_heads, c->head_dim);
    linear(t, a, l->o, seq, QD, H);
    for (size_t i = 0; i < (size_t)seq * H; i++) h[i] += t[i];
    fo_qwen3_rms_norm(n, h, l->post_norm, seq, H, c->eps);
    linear(g, n, l->gate, seq, H, I);
    linear(u, n, l->up, seq, H, I);
    for (size_t i = 0; i < (size_t)seq * I; i++) g[i] = g[i] / (1.0f + expf(-g[i])) * u[i];
    linear(t, g, l->down, seq, I, H);
    for (size_t i = 0; i < (size_t)seq * H; i++) h[i] += t[i];
    free(n); free(q); free(k); free(v); free(a); free(t); free(g); free(u);
}

/* ids [seq], mask [seq] (1 = real token, 0 = padding; may be NULL) -> malloc'd [seq, 3*hidden]:
 * the hidden states after layers out_layer[0..2] side by side (qwen3_forward :1041-1156; ids
 * outside the vocabulary give a zero row :1047-1056). Layers after the last captured one do not
 * influence the result and are not run. */
float *fo_qwen3_forward(const fo_qwen3 *m, const int *ids, const int *mask, int seq) {
    const fo_qwen3_config *c = &m->c;
    const int H = c->hidden;
    float *h = (float *)calloc((size_t)seq * H, sizeof(float));
    float *out = (float *)malloc(sizeof(float) * (size_t)seq * 3 * H);
    for (int s = 0; s < seq; s++)
        if (ids[s] >= 0 && ids[s] < c->vocab) memcpy(h + (size_t)s * H, m->embed + (size_t)ids[s] * H, sizeof(float) * H);
    int last = c->out_layer[0];
    for (int j = 1; j < 3; j++) if (c->out_layer[j] > last) last = c->out_layer[j];
    for (int li = 0; li <= last && li < c->layers; li++) {
        fo_qwen3_layer_forward(m, li, h, mask, seq);
        for (int j = 0; j < 3; j++)
            if (c->out_layer[j] == li)
                for (int s = 0; s < seq; s++) memcpy(out + ((size_t)s * 3 + j) * H, h + (size_t)s * H, sizeof(float) * H);
    }
    free(h);
    return out;
}
