/*
 * flux_qwen3_hip.c - the Qwen3 text encoder on the device: weights, work buffers, the forward
 * pass, and the reference's own entry points (flux_qwen3.h:93-141) over it.
 *
 * Follows the CPU arm of qwen3_forward (flux_qwen3.c:1041-1156): embedding lookup, then per layer
 * RMS norm -> q/k/v projections -> per-head RMS norm + rotate-half RoPE -> causal grouped-query
 * attention with the padding mask -> output projection + residual -> RMS norm -> SwiGLU MLP +
 * residual; the hidden states after three layers (8, 17, 26 in the reference's model) side by side
 * are the result. Layers after the last captured one cannot influence it and are neither stored
 * nor run (the reference's device path skips them too, flux_qwen3.c:902).
 *
 * q, k and v share one [QD + 2 KD, H] matrix and gate/up one [2 I, H] matrix so that each is one
 * GEMM; both residual adds and SiLU(gate)*up are GEMM epilogues (gemm.hip). The residual stream is
 * fp32, GEMM operands bf16.
 */
#include "../../include/flux_hip.h"
#include "host_internal.h"
#include <math.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

/* qwen3.hip */
int flux_hip_qwen3_embed(float *x, const void *embed_bf16, const int *ids_dev, int seq, int hidden, int vocab);
int flux_hip_qwen3_qk_rope(void *qkv_bf16, void *vt_bf16, int ldv, const float *q_w, const float *k_w, const float *rope_cos,
                           const float *rope_sin, int seq, int heads, int kv_heads, float eps);
int flux_hip_qwen3_collect(float *dst, int ldd, int col0, const float *src, int seq, int hidden);

#define QW_MAX_SEQ 512 /* QWEN3_MAX_SEQ_LEN, flux_qwen3.h:29 */

enum { T_IN_NORM, T_POST_NORM, T_Q, T_K, T_V, T_O, T_QN, T_KN, T_GATE, T_UP, T_DOWN, T_COUNT };

typedef struct {
    float *in_norm, *post_norm, *q_norm, *k_norm;
    void *qkv, *o, *gate_up, *down;
    unsigned loaded; /* bit per T_* */
} qlayer;

struct flux_hip_qwen3 {
    flux_hip_qwen3_config c;
    int n_run;        /* layers that are stored and run: up to the last captured one */
    int embed_loaded;
    void *embed;
    qlayer *layer;
    float *ones, *rope_cos, *rope_sin;
    /* work buffers for QW_MAX_SEQ tokens */
    float *x, *out;
    void *xn, *qkv, *vt, *att, *act;
    int *ids, *mask;
};

void flux_hip_qwen3_default_config(flux_hip_qwen3_config *c) {
    /* flux_qwen3.h:22-39 */
    c->hidden = 2560; c->intermediate = 9728; c->heads = 32; c->kv_heads = 8; c->head_dim = 128;
    c->layers = 36; c->vocab = 151936;
    c->out_layer[0] = 8; c->out_layer[1] = 17; c->out_layer[2] = 26;
    c->rope_theta = 1000000.0f; c->eps = 1e-6f;
}

static float *dev_f32_zero(size_t n) {
    float *p = (float *)flux_hip_malloc(n * 4);
    if (p && !flux_hip_memset(p, 0, n * 4)) { flux_hip_free(p); return NULL; }
    return p;
}

flux_hip_qwen3 *flux_hip_qwen3_new(const flux_hip_qwen3_config *cfg) {
    if (!flux_hip_available()) return NULL;
    flux_hip_qwen3_config c;
    if (cfg) c = *cfg; else flux_hip_qwen3_default_config(&c);
    const int H = c.hidden, I = c.intermediate, QD = c.heads * c.head_dim, KD = c.kv_heads * c.head_dim;
    if (c.head_dim != 128) { flux_hip_fail("qwen3: head_dim=%d (the attention kernel is built for 128)", c.head_dim); return NULL; }
    if (H <= 0 || (H & 127) || I <= 0 || (I & 63) || c.heads <= 0 || c.kv_heads <= 0 || c.heads % c.kv_heads || ((QD + 2 * KD) & 127) ||
        c.vocab <= 0 || c.layers <= 0) {
        flux_hip_fail("qwen3: unsupported sizes (hidden %d, intermediate %d, heads %d/%d): hidden and q+k+v widths must be multiples of 128, "
                      "intermediate of 64", H, I, c.heads, c.kv_heads);
        return NULL;
    }
    int last = -1;
    for (int j = 0; j < 3; j++) {
        if (c.out_layer[j] < 0 || c.out_layer[j] >= c.layers) { flux_hip_fail("qwen3: output layer %d outside 0..%d", c.out_layer[j], c.layers - 1); return NULL; }
        if (c.out_layer[j] > last) last = c.out_layer[j];
    }
    flux_hip_qwen3 *q = (flux_hip_qwen3 *)calloc(1, sizeof *q);
    if (!q) { flux_hip_fail("out of host memory"); return NULL; }
    q->c = c;
    q->n_run = last + 1;
    q->layer = (qlayer *)calloc((size_t)q->n_run, sizeof(qlayer));
    int ok = q->layer != NULL;
    ok = ok && (q->embed = flux_hip_malloc((size_t)c.vocab * H * 2));
    for (int i = 0; ok && i < q->n_run; i++) {
        qlayer *l = &q->layer[i];
        ok = (l->in_norm = dev_f32_zero(H)) && (l->post_norm = dev_f32_zero(H)) && (l->q_norm = dev_f32_zero(128)) &&
             (l->k_norm = dev_f32_zero(128)) && (l->qkv = flux_hip_malloc((size_t)(QD + 2 * KD) * H * 2)) &&
             (l->o = flux_hip_malloc((size_t)H * QD * 2)) && (l->gate_up = flux_hip_malloc((size_t)2 * I * H * 2)) &&
             (l->down = flux_hip_malloc((size_t)H * I * 2));
    }
    /* the angle table of compute_rope_freqs (flux_qwen3.c:250-262), same fp32 expressions */
    float *cs = (float *)malloc(sizeof(float) * QW_MAX_SEQ * 64), *sn = (float *)malloc(sizeof(float) * QW_MAX_SEQ * 64);
    float *one = (float *)malloc(sizeof(float) * (size_t)H);
    ok = ok && cs && sn && one;
    if (ok) {
        for (int pos = 0; pos < QW_MAX_SEQ; pos++)
            for (int i = 0; i < 64; i++) {
                float freq = 1.0f / powf(c.rope_theta, (float)(2 * i) / 128.0f);
                float angle = pos * freq;
                cs[pos * 64 + i] = cosf(angle);
                sn[pos * 64 + i] = sinf(angle);
            }
        for (int i = 0; i < H; i++) one[i] = 1.0f;
        ok = (q->rope_cos = (float *)flux_hip_malloc(sizeof(float) * QW_MAX_SEQ * 64)) && (q->rope_sin = (float *)flux_hip_malloc(sizeof(float) * QW_MAX_SEQ * 64)) &&
             (q->ones = (float *)flux_hip_malloc(sizeof(float) * (size_t)H)) && flux_hip_upload(q->rope_cos, cs, sizeof(float) * QW_MAX_SEQ * 64) &&
             flux_hip_upload(q->rope_sin, sn, sizeof(float) * QW_MAX_SEQ * 64) && flux_hip_upload(q->ones, one, sizeof(float) * (size_t)H);
    }
    free(cs); free(sn); free(one);
    const size_t S = QW_MAX_SEQ;
    ok = ok && (q->x = (float *)flux_hip_malloc(S * H * 4)) && (q->out = (float *)flux_hip_malloc(S * 3 * H * 4)) &&
         (q->xn = flux_hip_malloc(S * H * 2)) && (q->qkv = flux_hip_malloc(S * (QD + 2 * KD) * 2)) && (q->vt = flux_hip_malloc((size_t)KD * S * 2)) &&
         (q->att = flux_hip_malloc(S * QD * 2)) && (q->act = flux_hip_malloc(S * I * 2)) && (q->ids = (int *)flux_hip_malloc(S * 4)) &&
         (q->mask = (int *)flux_hip_malloc(S * 4));
    /* columns of vt beyond the current sequence are multiplied by zero probabilities: keep them finite */
    ok = ok && flux_hip_memset(q->vt, 0, (size_t)KD * S * 2);
    if (!ok) { flux_hip_qwen3_free(q); return NULL; }
    return q;
}

void flux_hip_qwen3_free(flux_hip_qwen3 *q) {
    if (!q) return;
    flux_hip_sync();
    flux_hip_free(q->embed);
    for (int i = 0; q->layer && i < q->n_run; i++) {
        qlayer *l = &q->layer[i];
        flux_hip_free(l->in_norm); flux_hip_free(l->post_norm); flux_hip_free(l->q_norm); flux_hip_free(l->k_norm);
        flux_hip_free(l->qkv); flux_hip_free(l->o); flux_hip_free(l->gate_up); flux_hip_free(l->down);
    }
    free(q->layer);
    flux_hip_free(q->ones); flux_hip_free(q->rope_cos); flux_hip_free(q->rope_sin);
    flux_hip_free(q->x); flux_hip_free(q->out); flux_hip_free(q->xn); flux_hip_free(q->qkv); flux_hip_free(q->vt);
    flux_hip_free(q->att); flux_hip_free(q->act); flux_hip_free(q->ids); flux_hip_free(q->mask);
    free(q);
}

static uint16_t to_bf16(float f) {
    uint32_t u;
    memcpy(&u, &f, 4);
    u += 0x7fffu + ((u >> 16) & 1u);
    return (uint16_t)(u >> 16);
}

static int upload_bf16(void *dst, int dtype, const void *data, int64_t n) {
    if (dtype == FH_DT_BF16) return flux_hip_upload(dst, data, (size_t)n * 2);
    uint16_t *tmp = (uint16_t *)malloc((size_t)n * 2);
    if (!tmp) return flux_hip_fail("out of host memory");
    for (int64_t i = 0; i < n; i++) tmp[i] = to_bf16(fh_tensor_value(dtype, data, i));
    int ok = flux_hip_upload(dst, tmp, (size_t)n * 2);
    free(tmp);
    return ok;
}

static int upload_f32(float *dst, int dtype, const void *data, int64_t n) {
    if (dtype == FH_DT_F32) return flux_hip_upload(dst, data, (size_t)n * 4);
    float *tmp = (float *)malloc((size_t)n * 4);
    if (!tmp) return flux_hip_fail("out of host memory");
    for (int64_t i = 0; i < n; i++) tmp[i] = fh_tensor_value(dtype, data, i);
    int ok = flux_hip_upload(dst, tmp, (size_t)n * 4);
    free(tmp);
    return ok;
}

/* Stores one tensor (names as the reference loader asks for them, flux_qwen3.c:1211-1253, 1361).
 * Tensors of layers that are not run, and the final norm, are accepted and ignored. */
int flux_hip_qwen3_set_tensor(flux_hip_qwen3 *q, const char *name, int dtype, const void *data, int64_t numel) {
    if (!q || !name || !data) return flux_hip_fail("flux_hip_qwen3_set_tensor: NULL argument");
    if (dtype != FH_DT_F32 && dtype != FH_DT_F16 && dtype != FH_DT_BF16) return flux_hip_fail("tensor %s: unsupported dtype %d", name, dtype);
    const flux_hip_qwen3_config *c = &q->c;
    const int64_t H = c->hidden, I = c->intermediate, QD = (int64_t)c->heads * 128, KD = (int64_t)c->kv_heads * 128;
    if (!strcmp(name, "model.embed_tokens.weight")) {
        if (numel != (int64_t)c->vocab * H) return flux_hip_fail("tensor %s has %lld elements, expected %lld", name, (long long)numel, (long long)c->vocab * H);
        if (!upload_bf16(q->embed, dtype, data, numel)) return 0;
        q->embed_loaded = 1;
        return 1;
    }
    if (!strcmp(name, "model.norm.weight") || !strcmp(name, "lm_head.weight")) return 1;
    int li;
    char rest[128];
    if (sscanf(name, "model.layers.%d.%127s", &li, rest) != 2 || li < 0) return flux_hip_fail("tensor %s is not part of the text encoder", name);
    if (li >= q->n_run) return 1;
    qlayer *l = &q->layer[li];
    static const char *names[T_COUNT] = {"input_layernorm.weight", "post_attention_layernorm.weight", "self_attn.q_proj.weight",
                                         "self_attn.k_proj.weight", "self_attn.v_proj.weight", "self_attn.o_proj.weight",
                                         "self_attn.q_norm.weight", "self_attn.k_norm.weight", "mlp.gate_proj.weight",
                                         "mlp.up_proj.weight", "mlp.down_proj.weight"};
    int t = -1;
    for (int i = 0; i < T_COUNT; i++)
        if (!strcmp(rest, names[i])) t = i;
    if (t < 0) return flux_hip_fail("tensor %s is not part of the text encoder", name);
    const int64_t expect[T_COUNT] = {H, H, QD * H, KD * H, KD * H, H * QD, 128, 128, I * H, I * H, H * I};
    if (numel != expect[t]) return flux_hip_fail("tensor %s has %lld elements, expected %lld", name, (long long)numel, (long long)expect[t]);
    int ok;
    switch (t) {
        case T_IN_NORM: ok = upload_f32(l->in_norm, dtype, data, numel); break;
        case T_POST_NORM: ok = upload_f32(l->post_norm, dtype, data, numel); break;
        case T_QN: ok = upload_f32(l->q_norm, dtype, data, numel); break;
        case T_KN: ok = upload_f32(l->k_norm, dtype, data, numel); break;
        case T_Q: ok = upload_bf16(l->qkv, dtype, data, numel); break;
        case T_K: ok = upload_bf16((char *)l->qkv + (size_t)QD * H * 2, dtype, data, numel); break;
        case T_V: ok = upload_bf16((char *)l->qkv + (size_t)(QD + KD) * H * 2, dtype, data, numel); break;
        case T_O: ok = upload_bf16(l->o, dtype, data, numel); break;
        case T_GATE: ok = upload_bf16(l->gate_up, dtype, data, numel); break;
        case T_UP: ok = upload_bf16((char *)l->gate_up + (size_t)I * H * 2, dtype, data, numel); break;
        default: ok = upload_bf16(l->down, dtype, data, numel); break;
    }
    if (ok) l->loaded |= 1u << t;
    return ok;
}

static int qwen3_complete(const flux_hip_qwen3 *q) {
    if (!q->embed_loaded) return flux_hip_fail("text encoder: model.embed_tokens.weight was not loaded");
    for (int i = 0; i < q->n_run; i++)
        if (q->layer[i].loaded != (1u << T_COUNT) - 1) return flux_hip_fail("text encoder: layer %d is missing tensors (mask %x)", i, q->layer[i].loaded);
    return 1;
}

/* ---- loading a model directory: sizes are read from the tensors themselves ---- */
typedef struct { int64_t h, hd, qd, kd, inter, embed; int layers; } qprobe;

static int probe_cb(void *ctx, const char *name, int dtype, const void *data, int64_t numel) {
    qprobe *p = (qprobe *)ctx;
    (void)dtype; (void)data;
    int li;
    char rest[128];
    if (!strcmp(name, "model.embed_tokens.weight")) p->embed = numel;
    else if (sscanf(name, "model.layers.%d.%127s", &li, rest) == 2) {
        if (li + 1 > p->layers) p->layers = li + 1;
        if (li == 0) {
            if (!strcmp(rest, "input_layernorm.weight")) p->h = numel;
            else if (!strcmp(rest, "self_attn.q_norm.weight")) p->hd = numel;
            else if (!strcmp(rest, "self_attn.q_proj.weight")) p->qd = numel;
            else if (!strcmp(rest, "self_attn.k_proj.weight")) p->kd = numel;
            else if (!strcmp(rest, "mlp.gate_proj.weight")) p->inter = numel;
        }
    }
    return 1;
}

static int set_cb(void *ctx, const char *name, int dtype, const void *data, int64_t numel) {
    return flux_hip_qwen3_set_tensor((flux_hip_qwen3 *)ctx, name, dtype, data, numel);
}

/* model_dir holds model-00001-of-00002.safetensors and model-00002-of-00002.safetensors, as
 * qwen3_model_load expects (flux_qwen3.c:1341-1343), or a single model.safetensors. */
flux_hip_qwen3 *flux_hip_qwen3_load_dir(const char *model_dir) {
    char path[3][600];
    int nfiles = 2;
    snprintf(path[0], sizeof path[0], "%s/model-00001-of-00002.safetensors", model_dir);
    snprintf(path[1], sizeof path[1], "%s/model-00002-of-00002.safetensors", model_dir);
    FILE *f = fopen(path[0], "rb");
    if (f) fclose(f);
    else {
        snprintf(path[0], sizeof path[0], "%s/model.safetensors", model_dir);
        nfiles = 1;
    }
    qprobe p;
    memset(&p, 0, sizeof p);
    for (int i = 0; i < nfiles; i++)
        if (!fh_safetensors_walk(path[i], probe_cb, &p)) return NULL;
    if (p.h <= 0 || p.hd <= 0 || p.qd <= 0 || p.kd <= 0 || p.inter <= 0 || p.embed <= 0 || p.layers <= 0) {
        flux_hip_fail("%s: not a Qwen3 text encoder (tensors of layer 0 or the embedding are missing)", model_dir);
        return NULL;
    }
    flux_hip_qwen3_config c;
    flux_hip_qwen3_default_config(&c);
    c.hidden = (int)p.h; c.head_dim = (int)p.hd;
    c.heads = (int)(p.qd / p.h / p.hd); c.kv_heads = (int)(p.kd / p.h / p.hd);
    c.intermediate = (int)(p.inter / p.h); c.vocab = (int)(p.embed / p.h); c.layers = p.layers;
    if (c.layers <= c.out_layer[2]) { flux_hip_fail("%s: %d layers, the output needs layers %d, %d and %d", model_dir, c.layers, c.out_layer[0], c.out_layer[1], c.out_layer[2]); return NULL; }
    flux_hip_qwen3 *q = flux_hip_qwen3_new(&c);
    if (!q) return NULL;
    for (int i = 0; i < nfiles; i++)
        if (!fh_safetensors_walk(path[i], set_cb, q)) { flux_hip_qwen3_free(q); return NULL; }
    if (!qwen3_complete(q)) { flux_hip_qwen3_free(q); return NULL; }
    return q;
}

/* Called (when set) after each layer has been queued: (layer, layers run). */
void (*flux_hip_qwen3_progress)(int layer, int total) = NULL;

static int linear1(int epi, const void *A, const void *W, void *C, const float *gate, int M, int N, int K, int lda, int ldc, int r0, int r1) {
    flux_hip_linear_part p = {A, W, C, gate, M};
    return flux_hip_linear(epi, 1, &p, N, K, lda, K, ldc, r0, r1);
}

/* ids, mask: host int [seq] (mask 1 = token, 0 = padding; NULL = no padding). Returns a malloc'd
 * host array [seq, 3 * hidden] (qwen3_forward, flux_qwen3.c:1041), or NULL. */
float *flux_hip_qwen3_forward(flux_hip_qwen3 *q, const int *input_ids, const int *attention_mask, int seq_len) {
    if (!q || !input_ids) { flux_hip_fail("flux_hip_qwen3_forward: NULL argument"); return NULL; }
    if (seq_len <= 0 || seq_len > QW_MAX_SEQ) { flux_hip_fail("flux_hip_qwen3_forward: seq_len=%d (1..%d)", seq_len, QW_MAX_SEQ); return NULL; }
    if (!qwen3_complete(q)) return NULL;
    const flux_hip_qwen3_config *c = &q->c;
    const int H = c->hidden, I = c->intermediate, QD = c->heads * 128, KD = c->kv_heads * 128, W = QD + 2 * KD, S = seq_len;
    if (!flux_hip_upload(q->ids, input_ids, (size_t)S * 4)) return NULL;
    if (attention_mask && !flux_hip_upload(q->mask, attention_mask, (size_t)S * 4)) return NULL;
    const int *mask = attention_mask ? q->mask : NULL;
    if (!flux_hip_qwen3_embed(q->x, q->embed, q->ids, S, H, c->vocab)) return NULL;
    /* normed: xn already holds the RMS norm that the next projection reads, written by the second pass
     * of the residual projection before it (flux_hip_linear_resid_adaln in its RMS form) */
    int normed = 0;
    int parts = 1;   /* 1: parts travel as they are produced; 0: no staging buffer, one download at the end */
    const size_t part_bytes = (size_t)S * H * 4;
    for (int li = 0; li < q->n_run; li++) {
        const qlayer *l = &q->layer[li];
        if (!normed && !flux_hip_rms_norm(q->xn, q->x, l->in_norm, S, H, c->eps)) return NULL;
        if (!linear1(FLUX_HIP_EPI_BF16, q->xn, l->qkv, q->qkv, NULL, S, W, H, H, W, 0, 0)) return NULL;
        if (!flux_hip_qwen3_qk_rope(q->qkv, q->vt, QW_MAX_SEQ, l->q_norm, l->k_norm, q->rope_cos, q->rope_sin, S, c->heads, c->kv_heads, c->eps)) return NULL;
        if (!flux_hip_causal_attention(q->att, q->qkv, q->vt, QW_MAX_SEQ, mask, S, c->heads, c->kv_heads)) return NULL;
        flux_hip_linear_part po = {q->att, l->o, q->x, q->ones, S};
        flux_hip_adaln_part no = {q->xn, NULL, l->post_norm};
        if (!flux_hip_linear_resid_adaln(1, &po, H, QD, QD, QD, H, &no, c->eps, &normed)) return NULL;
        if (!normed && !flux_hip_rms_norm(q->xn, q->x, l->post_norm, S, H, c->eps)) return NULL;
        if (!linear1(FLUX_HIP_EPI_SWIGLU, q->xn, l->gate_up, q->act, NULL, S, 2 * I, H, H, I, 0, I)) return NULL;
        flux_hip_linear_part pd = {q->act, l->down, q->x, q->ones, S};
        flux_hip_adaln_part nd = {q->xn, NULL, li + 1 < q->n_run ? q->layer[li + 1].in_norm : NULL};
        if (!flux_hip_linear_resid_adaln(1, &pd, H, I, I, I, H, nd.scale ? &nd : NULL, c->eps, &normed)) return NULL;
        /* a captured layer goes to its third of q->out ([3][S][H], layer-major) and from there to the
         * host at once, on the copy stream, while the layers after it run */
        for (int j = 0; j < 3; j++) {
            if (c->out_layer[j] != li) continue;
            if (!flux_hip_qwen3_collect(q->out + (size_t)j * S * H, H, 0, q->x, S, H)) return NULL;
            if (parts > 0) parts = flux_hip_download_part_begin(j, j * part_bytes, 3 * part_bytes, q->out + (size_t)j * S * H, part_bytes);
            if (parts < 0) return NULL;
        }
        if (flux_hip_qwen3_progress) flux_hip_qwen3_progress(li, q->n_run);
    }
    float *out = (float *)malloc((size_t)S * 3 * H * sizeof(float));
    if (!out) { flux_hip_fail("out of host memory"); return NULL; }
    float *whole = NULL;    /* without a staging buffer (results under 1 MB): one download at the end */
    if (!parts) {
        whole = (float *)malloc(3 * part_bytes);
        if (!whole || !flux_hip_download(whole, q->out, 3 * part_bytes)) {
            if (!whole) flux_hip_fail("out of host memory");
            free(whole); free(out);
            return NULL;
        }
    }
    /* [3][S][H] -> [S][3H]: the first two parts are interleaved while the device still computes */
    for (int j = 0; j < 3; j++) {
        const float *part = whole ? whole + (size_t)j * S * H : (const float *)flux_hip_download_part_wait(j);
        if (!part) { free(out); return NULL; }
        for (int r = 0; r < S; r++) memcpy(out + ((size_t)r * 3 + j) * H, part + (size_t)r * H, (size_t)H * 4);
    }
    free(whole);
    return out;
}

/* ------------------------------------------------------------------ the reference's names
 * (flux_qwen3.h:93-141). An application links flux_qwen3_tokenizer.c as before and leaves
 * flux_qwen3.c out. The tokenizer's functions and the progress callback are the application's;
 * they are weak here so that the library also loads without them. */
typedef struct qwen3_tokenizer qwen3_tokenizer_t;
extern qwen3_tokenizer_t *qwen3_tokenizer_load(const char *path) __attribute__((weak));
extern void qwen3_tokenizer_free(qwen3_tokenizer_t *tok) __attribute__((weak));
extern int *qwen3_tokenize_chat(qwen3_tokenizer_t *tok, const char *prompt, int *num_tokens, int max_len) __attribute__((weak));
extern int *qwen3_pad_tokens(int *tokens, int num_tokens, int max_len, int *attention_mask) __attribute__((weak));
typedef void (*text_progress_fn)(int layer, int total);
extern text_progress_fn flux_text_progress_callback __attribute__((weak)); /* flux_kernels.h */

typedef struct { qwen3_tokenizer_t *tokenizer; flux_hip_qwen3 *model; char dir[600]; } dropin_encoder; /* qwen3_encoder_t, flux_qwen3.h:117-120 */

/* The reference frees the text encoder after every prompt to make room for the transformer
 * (flux_release_text_encoder, flux.c:285-295) and loads it again for the next one; its weights are
 * a memory map, so that is cheap there. Here a load is a 6 GB upload, and 288 GB of HBM hold encoder
 * and transformer side by side: the weights of the encoder freed last stay on the device and the
 * next qwen3_encoder_load of the same directory takes them over. */
static struct { char dir[600]; flux_hip_qwen3 *model; } g_kept;
static int g_keep_resident = 1;
int flux_hip_qwen3_resident_hits = 0;

void flux_hip_qwen3_drop_resident(void) {
    flux_hip_qwen3_free(g_kept.model);
    g_kept.model = NULL;
    g_kept.dir[0] = 0;
}

void flux_hip_qwen3_keep_resident(int on) {
    g_keep_resident = on != 0;
    if (!on) flux_hip_qwen3_drop_resident();
}

void *qwen3_model_load(const char *model_dir) { return flux_hip_qwen3_load_dir(model_dir); }
/* weights live on the device either way */
void *qwen3_model_load_mmap(const char *model_dir) { return flux_hip_qwen3_load_dir(model_dir); }
void qwen3_model_free(void *model) { flux_hip_qwen3_free((flux_hip_qwen3 *)model); }

float *qwen3_forward(void *model, const int *input_ids, const int *attention_mask, int seq_len) {
    flux_hip_qwen3_progress = &flux_text_progress_callback ? flux_text_progress_callback : NULL;
    float *out = flux_hip_qwen3_forward((flux_hip_qwen3 *)model, input_ids, attention_mask, seq_len);
    flux_hip_qwen3_progress = NULL;
    return out;
}

void *qwen3_encoder_load(const char *model_dir, int use_mmap) {
    (void)use_mmap;
    if (!qwen3_tokenizer_load || !qwen3_tokenizer_free) { flux_hip_fail("qwen3_encoder_load: the tokenizer (flux_qwen3_tokenizer.c) is not linked"); return NULL; }
    dropin_encoder *enc = (dropin_encoder *)calloc(1, sizeof *enc);
    if (!enc) return NULL;
    char path[600];
    snprintf(path, sizeof path, "%s/tokenizer/tokenizer.json", model_dir);
    enc->tokenizer = qwen3_tokenizer_load(path);
    if (!enc->tokenizer) { flux_hip_fail("qwen3_encoder_load: failed to load %s", path); free(enc); return NULL; }
    snprintf(enc->dir, sizeof enc->dir, "%s/text_encoder", model_dir);
    if (g_kept.model && !strcmp(g_kept.dir, enc->dir)) {
        enc->model = g_kept.model;
        g_kept.model = NULL;
        flux_hip_qwen3_resident_hits++;
    } else {
        enc->model = flux_hip_qwen3_load_dir(enc->dir);
    }
    if (!enc->model) { qwen3_tokenizer_free(enc->tokenizer); free(enc); return NULL; }
    return enc;
}

void qwen3_encoder_free(void *p) {
    dropin_encoder *enc = (dropin_encoder *)p;
    if (!enc) return;
    if (qwen3_tokenizer_free) qwen3_tokenizer_free(enc->tokenizer);
    if (g_keep_resident && enc->model) {
        flux_hip_qwen3_drop_resident();
        g_kept.model = enc->model;
        snprintf(g_kept.dir, sizeof g_kept.dir, "%s", enc->dir);
    } else {
        flux_hip_qwen3_free(enc->model);
    }
    free(enc);
}

/* chat template, padding to 512 tokens, forward (qwen3_encode_text, flux_qwen3.c:1627-1652) */
float *qwen3_encode_text(void *p, const char *prompt) {
    dropin_encoder *enc = (dropin_encoder *)p;
    if (!enc || !enc->tokenizer || !enc->model || !prompt || !qwen3_tokenize_chat || !qwen3_pad_tokens) return NULL;
    int num_tokens = 0;
    int *tokens = qwen3_tokenize_chat(enc->tokenizer, prompt, &num_tokens, QW_MAX_SEQ);
    if (!tokens) return NULL;
    int *mask = (int *)malloc(QW_MAX_SEQ * sizeof(int));
    int *padded = mask ? qwen3_pad_tokens(tokens, num_tokens, QW_MAX_SEQ, mask) : NULL;
    free(tokens);
    if (!padded) { free(mask); return NULL; }
    float *emb = qwen3_forward(enc->model, padded, mask, QW_MAX_SEQ);
    free(padded);
    free(mask);
    return emb;
}
