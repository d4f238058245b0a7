/*
 * ref_probe.c - thin exports around the reference's own C code.
 *
 * TEST INFRASTRUCTURE. This translation unit textually includes
 * flux_transformer.c from the read-only reference checkout (path given with
 * -DREF_TRANSFORMER_C=...), so that its file-static functions and its model
 * struct are reachable, and re-exports them under ref_* names. Nothing of the
 * reference is copied into this repository: the build reads the sources where
 * they lie and writes only oracle/_ref/libfluxref.so. It is built with the
 * reference's "generic" flags (no BLAS: no cblas.h exists in this image).
 *
 * The only thing added here is a model constructor that fills the reference's
 * flux_transformer_t for an arbitrary (small) architecture, because the
 * reference loader hard-codes the 4B sizes (flux_transformer.c:4418-4434).
 */
#include REF_TRANSFORMER_C

/* flux_sample.c entry points (compiled as its own object) */
extern float *flux_sample_euler(void *transformer, void *text_encoder,
                                float *z, int batch, int channels, int h, int w,
                                const float *text_emb, int text_seq,
                                const float *schedule, int num_steps,
                                void (*progress_callback)(int step, int total));

typedef struct {
    int hidden, heads, head_dim, mlp, n_double, n_single, text_dim, channels;
    int axis_dim, sincos_dim;
    float rope_theta;
} probe_config;

flux_transformer_t *ref_model_new(const probe_config *c) {
    flux_transformer_t *tf = calloc(1, sizeof(flux_transformer_t));
    tf->hidden_size = c->hidden;
    tf->num_heads = c->heads;
    tf->head_dim = c->head_dim;
    tf->mlp_hidden = c->mlp;
    tf->num_double_layers = c->n_double;
    tf->num_single_layers = c->n_single;
    tf->text_dim = c->text_dim;
    tf->latent_channels = c->channels;
    tf->max_seq_len = 0;
    tf->rope_dim = c->head_dim;
    tf->rope_theta = c->rope_theta;
    tf->axis_dim = c->axis_dim;
    tf->use_bf16 = 0;
    tf->time_embed.sincos_dim = c->sincos_dim;
    tf->double_blocks = calloc(c->n_double ? c->n_double : 1, sizeof(double_block_t));
    tf->single_blocks = calloc(c->n_single ? c->n_single : 1, sizeof(single_block_t));
    tf->t_emb_silu = malloc(c->hidden * sizeof(float));
    tf->double_mod_img = malloc(c->hidden * 6 * sizeof(float));
    tf->double_mod_txt = malloc(c->hidden * 6 * sizeof(float));
    return tf;
}

static float *widen(const uint16_t *src, int64_t n) {
    float *dst = malloc((size_t)n * sizeof(float));
    for (int64_t i = 0; i < n; i++) {
        uint32_t b = ((uint32_t)src[i]) << 16;
        memcpy(&dst[i], &b, 4);
    }
    return dst;
}

/* Store a tensor under its safetensors key, doing what the reference loader
 * does with it (ff linear_in is split into gate and up halves). */
int ref_model_set_bf16(flux_transformer_t *tf, const char *name, const uint16_t *data, int64_t n) {
    int i; char rest[200];
    int64_t h = tf->hidden_size, mlp = tf->mlp_hidden;
    float **slot = NULL;
    if (!strcmp(name, "x_embedder.weight")) slot = &tf->img_in_weight;
    else if (!strcmp(name, "context_embedder.weight")) slot = &tf->txt_in_weight;
    else if (!strcmp(name, "time_guidance_embed.timestep_embedder.linear_1.weight")) slot = &tf->time_embed.fc1_weight;
    else if (!strcmp(name, "time_guidance_embed.timestep_embedder.linear_2.weight")) slot = &tf->time_embed.fc2_weight;
    else if (!strcmp(name, "double_stream_modulation_img.linear.weight")) slot = &tf->adaln_double_img_weight;
    else if (!strcmp(name, "double_stream_modulation_txt.linear.weight")) slot = &tf->adaln_double_txt_weight;
    else if (!strcmp(name, "single_stream_modulation.linear.weight")) slot = &tf->adaln_single_weight;
    else if (!strcmp(name, "norm_out.linear.weight")) slot = &tf->final_norm_weight;
    else if (!strcmp(name, "proj_out.weight")) slot = &tf->final_proj_weight;
    else if (sscanf(name, "transformer_blocks.%d.%199s", &i, rest) == 2 && i < tf->num_double_layers) {
        double_block_t *b = &tf->double_blocks[i];
        if (!strcmp(rest, "attn.norm_q.weight")) slot = &b->img_norm_q_weight;
        else if (!strcmp(rest, "attn.norm_k.weight")) slot = &b->img_norm_k_weight;
        else if (!strcmp(rest, "attn.norm_added_q.weight")) slot = &b->txt_norm_q_weight;
        else if (!strcmp(rest, "attn.norm_added_k.weight")) slot = &b->txt_norm_k_weight;
        else if (!strcmp(rest, "attn.to_q.weight")) slot = &b->img_q_weight;
        else if (!strcmp(rest, "attn.to_k.weight")) slot = &b->img_k_weight;
        else if (!strcmp(rest, "attn.to_v.weight")) slot = &b->img_v_weight;
        else if (!strcmp(rest, "attn.add_q_proj.weight")) slot = &b->txt_q_weight;
        else if (!strcmp(rest, "attn.add_k_proj.weight")) slot = &b->txt_k_weight;
        else if (!strcmp(rest, "attn.add_v_proj.weight")) slot = &b->txt_v_weight;
        else if (!strcmp(rest, "attn.to_out.0.weight")) slot = &b->img_proj_weight;
        else if (!strcmp(rest, "attn.to_add_out.weight")) slot = &b->txt_proj_weight;
        else if (!strcmp(rest, "ff.linear_out.weight")) slot = &b->img_mlp_down_weight;
        else if (!strcmp(rest, "ff_context.linear_out.weight")) slot = &b->txt_mlp_down_weight;
        else if (!strcmp(rest, "ff.linear_in.weight") || !strcmp(rest, "ff_context.linear_in.weight")) {
            if (n != 2 * mlp * h) return -2;
            float *all = widen(data, n);
            float *g = malloc(mlp * h * sizeof(float)), *u = malloc(mlp * h * sizeof(float));
            memcpy(g, all, mlp * h * sizeof(float));
            memcpy(u, all + mlp * h, mlp * h * sizeof(float));
            free(all);
            if (rest[2] == '.') { b->img_mlp_gate_weight = g; b->img_mlp_up_weight = u; }
            else { b->txt_mlp_gate_weight = g; b->txt_mlp_up_weight = u; }
            return 0;
        } else return -1;
    } else if (sscanf(name, "single_transformer_blocks.%d.%199s", &i, rest) == 2 && i < tf->num_single_layers) {
        single_block_t *b = &tf->single_blocks[i];
        if (!strcmp(rest, "attn.norm_q.weight")) slot = &b->norm_q_weight;
        else if (!strcmp(rest, "attn.norm_k.weight")) slot = &b->norm_k_weight;
        else if (!strcmp(rest, "attn.to_qkv_mlp_proj.weight")) slot = &b->qkv_mlp_weight;
        else if (!strcmp(rest, "attn.to_out.weight")) slot = &b->proj_mlp_weight;
        else return -1;
    } else return -1;
    *slot = widen(data, n);
    return 0;
}

void ref_model_free(flux_transformer_t *tf) { flux_transformer_free(tf); }

/* ---- file-static functions of flux_transformer.c ---- */
void ref_timestep_embedding(float *out, float t, int dim, float max_period) {
    get_timestep_embedding(out, t, dim, max_period);
}
void ref_time_mlp(float *out, const float *e, const float *fc1, const float *fc2, int sincos, int hidden) {
    time_embed_t te = {(float *)fc1, (float *)fc2, sincos};
    float *work = malloc(hidden * sizeof(float));
    time_embed_forward(out, e, &te, hidden, work);
    free(work);
}
void ref_rope_image(float *c, float *s, int ph, int pw, int axis_dim, float theta, int t_offset) {
    if (t_offset == 0) compute_rope_2d(c, s, ph, pw, axis_dim, theta);
    else compute_rope_2d_with_t_offset(c, s, ph, pw, axis_dim, theta, t_offset);
}
void ref_rope_text(float *c, float *s, int seq, int axis_dim, float theta) {
    compute_rope_text(c, s, seq, axis_dim, theta);
}
void ref_apply_rope(float *x, const float *c, const float *s, int seq, int heads, int head_dim) {
    apply_rope_2d(x, c, s, seq, heads, head_dim, head_dim / 4);
}
void ref_adaln(float *out, const float *x, const float *shift, const float *scale, int seq, int hidden, float eps) {
    apply_adaln(out, x, shift, scale, seq, hidden, eps);
}
void ref_qk_norm(float *q, float *k, const float *qw, const float *kw, int seq, int heads, int head_dim, float eps) {
    apply_qk_norm(q, k, qw, kw, seq, heads, head_dim, eps);
}
void ref_gated_add(float *out, const float *gate, const float *proj, int seq, int hidden) {
    gated_add(out, gate, proj, seq, hidden);
}
/* joint attention over separate image/text streams (needs tf work buffers) */
int ref_joint_attention(flux_transformer_t *tf, float *img_out, float *txt_out,
                        const float *iq, const float *ik, const float *iv,
                        const float *tq, const float *tk, const float *tv,
                        int img_seq, int txt_seq) {
    if (ensure_work_buffers(tf, img_seq + txt_seq) < 0) return -1;
    joint_attention(img_out, txt_out, iq, ik, iv, tq, tk, tv, img_seq, txt_seq,
                    tf->num_heads, tf->head_dim, tf);
    return 0;
}
int ref_mha(flux_transformer_t *tf, float *out, const float *q, const float *k, const float *v, int seq) {
    if (ensure_work_buffers(tf, seq) < 0) return -1;
    mha_forward(out, q, k, v, seq, tf->num_heads, tf->head_dim, tf);
    return 0;
}
int ref_double_block(flux_transformer_t *tf, int idx, float *img_h, float *txt_h,
                     const float *img_mod, const float *txt_mod,
                     const float *ic, const float *is, const float *tc, const float *ts,
                     int img_seq, int txt_seq) {
    if (ensure_work_buffers(tf, img_seq + txt_seq) < 0) return -1;
    double_block_forward(img_h, txt_h, &tf->double_blocks[idx], img_mod, txt_mod,
                         ic, is, tc, ts, img_seq, txt_seq, tf);
    return 0;
}
/* The reference derives the modulation inside the block from t_emb. */
int ref_single_block(flux_transformer_t *tf, int idx, float *x, const float *t_emb,
                     const float *ic, const float *is, const float *tc, const float *ts,
                     int seq, int txt_seq) {
    if (ensure_work_buffers(tf, seq) < 0) return -1;
    single_block_forward(x, &tf->single_blocks[idx], t_emb, tf->adaln_single_weight,
                         ic, is, tc, ts, seq, txt_seq, tf);
    return 0;
}
void ref_free(void *p) { free(p); }
