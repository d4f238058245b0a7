/*
 * flux_vae_hip.c - the VAE on the device: weights, work buffers and the sequence of launches.
 *
 * Decoder: follows flux_vae_decode (flux_vae.c:690-837): latent de-normalisation, unpatchify,
 * post-quant 1x1 convolution, conv_in, mid block (residual, attention, residual), four levels of
 * three residual blocks with a nearest-2x upsample + convolution between them, group norm, swish,
 * conv_out, conversion to 8 bits. The architecture is the reference's (flux_vae.c:1243-1252):
 * 32 latent channels after unpatchify, base width 128, multipliers {1,2,4,4}, 32 groups,
 * eps 1e-4 for both the latent statistics and the group norms.
 *
 * Encoder: follows flux_vae_encode (flux_vae.c:320-443): conv_in, four levels of two residual
 * blocks with a stride-2 convolution after each of the first three, the same mid block, group
 * norm, swish, conv_out to 64 channels, 1x1 quant convolution, the 32 mean channels, 2x2 patchify,
 * latent normalisation. A residual block that widens computes what it is written to compute; the
 * reference's plain-C build overwrites part of that block's second convolution's input while it
 * runs (buffer offsets at flux_vae.c:203, loop order at flux_kernels.c:441-470), its BLAS path in
 * one tile does not.
 *
 * Convolutions run as MFMA GEMMs over bordered channels-last images (flux_hip_conv), the
 * attention as two GEMMs around a row softmax; everything else is in vae.hip.
 */
#include "../../include/flux_hip.h"
#include "../../include/flux_hip_debug.h"
#include "host_internal.h"
#include <hip/hip_runtime_api.h>
#include <math.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

/* vae.hip */
int flux_hip_vae_latent_in(void *out_bf16, const float *latent, const float *bn_mean, const float *bn_var,
                           const float *pq_w, const float *pq_b, int h, int w, float eps);
int flux_hip_vae_key_bias(float *bias, int n, int hp, int wp);
int flux_hip_vae_image_out(uint8_t *rgb, float *rgb_f32, const float *x, int ldx, int H, int W);
int flux_hip_vae_image_in(void *out_bf16, const float *img, int H, int W);
int flux_hip_downsample_gather(void *out_bf16, const float *x, int hp, int wp, int C);
int flux_hip_vae_latent_out(float *latent, const float *x, int ldx, const float *bn_mean, const float *bn_var, int h, int w, float eps);

enum { K_VEC, K_CONV3, K_CONV1, K_RAW, K_CONV3_PACKED };
enum { SIDE_BOTH, SIDE_DECODER, SIDE_ENCODER };

typedef struct {
    void *w;     /* bf16 [cout_pad, taps * cin_pad] */
    float *b;    /* f32 [cout_pad] */
    int cin, cout, taps, cin_pad, cout_pad;
} vconv;

typedef struct {
    float *n1g, *n1b, *n2g, *n2b;
    vconv c1, c2, skip;
    int cin, cout;
} vres;

typedef struct {
    float *g, *b; /* group norm */
    vconv qkv;    /* q, k, v share one [3 C, C] matrix so that one GEMM makes all three */
    vconv out;
} vattn;

typedef struct {
    char name[96];
    int kind, side;
    void *dst;       /* device destination */
    int rows, cols;  /* K_CONV*: cout, cin of the source tensor; K_VEC/K_RAW: rows = element count */
    int cin_pad;     /* row stride / taps of the destination, K_CONV* */
    int loaded;
} vslot;

struct flux_hip_vae {
    float eps;
    float *bn_mean, *bn_var, *pq_w, *pq_b;
    vconv conv_in, conv_out, up_conv[3];
    vres mid[2], up[12];
    vattn attn;
    float *out_g, *out_b;
    /* encoder */
    vconv enc_conv_in; /* K = 27 in one row of 64, see vae_image_in_kernel */
    vconv enc_down_conv[3], enc_conv_out, quant;
    vres enc_down[8], enc_mid[2];
    vattn enc_attn;
    float *enc_out_g, *enc_out_b;
    vslot *slots;
    int nslots, cap_slots, adding_side;
    /* work buffers, grown on demand */
    size_t f32_elems, bf16_elems, guard, att_ld, att_chunk, gn_floats, lat_elems, img_pixels, st_floats;
    float *X, *Y, *Hb, *S, *kbias, *gn, *lat, *img_f32, *st_x, *st_h;
    void *A_base, *R, *P, *VT;
    uint8_t *img_u8;
};

static uint16_t to_bf16(float f) {
    uint32_t u;
    memcpy(&u, &f, 4);
    u += 0x7fffu + ((u >> 16) & 1u);
    return (uint16_t)(u >> 16);
}

static vslot *add_slot(flux_hip_vae *v, const char *name, int kind, void *dst, int rows, int cols, int cin_pad) {
    if (v->nslots == v->cap_slots) {
        v->cap_slots = v->cap_slots ? v->cap_slots * 2 : 128;
        v->slots = (vslot *)realloc(v->slots, sizeof(vslot) * (size_t)v->cap_slots);
    }
    vslot *s = &v->slots[v->nslots++];
    memset(s, 0, sizeof *s);
    snprintf(s->name, sizeof s->name, "%s", name);
    s->kind = kind; s->side = v->adding_side; s->dst = dst; s->rows = rows; s->cols = cols; s->cin_pad = cin_pad;
    return s;
}

static float *dev_f32(size_t n) {
    float *p = (float *)flux_hip_malloc(n * sizeof(float));
    if (p) flux_hip_memset(p, 0, n * sizeof(float));
    return p;
}

/* vector of n floats under `name` */
static int add_vec(flux_hip_vae *v, const char *prefix, const char *suffix, float **dst, int n) {
    char name[128];
    snprintf(name, sizeof name, "%s%s", prefix, suffix);
    if (!*dst && !(*dst = dev_f32((size_t)n))) return 0;
    add_slot(v, name, K_VEC, *dst, n, 1, 0);
    return 1;
}

/* convolution `prefix`.weight / .bias; the device copies are padded to multiples of 64 channels */
static int add_conv(flux_hip_vae *v, const char *prefix, vconv *c, int cout, int cin, int taps) {
    c->cin = cin; c->cout = cout; c->taps = taps;
    c->cin_pad = (cin + 63) & ~63;
    c->cout_pad = (cout + 63) & ~63;
    size_t wbytes = (size_t)c->cout_pad * taps * c->cin_pad * 2;
    c->w = flux_hip_malloc(wbytes);
    c->b = dev_f32((size_t)c->cout_pad);
    if (!c->w || !c->b || !flux_hip_memset(c->w, 0, wbytes)) return 0;
    char name[128];
    snprintf(name, sizeof name, "%s.weight", prefix);
    add_slot(v, name, taps == 9 ? K_CONV3 : K_CONV1, c->w, cout, cin, c->cin_pad);
    snprintf(name, sizeof name, "%s.bias", prefix);
    add_slot(v, name, K_VEC, c->b, cout, 1, 0);
    return 1;
}

static int add_res(flux_hip_vae *v, const char *prefix, vres *r, int cin, int cout) {
    char name[128];
    r->cin = cin; r->cout = cout;
    if (!add_vec(v, prefix, ".norm1.weight", &r->n1g, cin) || !add_vec(v, prefix, ".norm1.bias", &r->n1b, cin) ||
        !add_vec(v, prefix, ".norm2.weight", &r->n2g, cout) || !add_vec(v, prefix, ".norm2.bias", &r->n2b, cout))
        return 0;
    snprintf(name, sizeof name, "%s.conv1", prefix);
    if (!add_conv(v, name, &r->c1, cout, cin, 9)) return 0;
    snprintf(name, sizeof name, "%s.conv2", prefix);
    if (!add_conv(v, name, &r->c2, cout, cout, 9)) return 0;
    if (cin != cout) {
        snprintf(name, sizeof name, "%s.conv_shortcut", prefix);
        if (!add_conv(v, name, &r->skip, cout, cin, 1)) return 0;
    }
    return 1;
}

/* attention block `prefix`: group norm, to_q / to_k / to_v into one matrix, to_out.0 */
static int add_attn(flux_hip_vae *v, const char *prefix, vattn *a, int C) {
    char name[160];
    snprintf(name, sizeof name, "%s.group_norm", prefix);
    if (!add_vec(v, name, ".weight", &a->g, C) || !add_vec(v, name, ".bias", &a->b, C)) return 0;
    a->qkv.cin = a->qkv.cin_pad = C; a->qkv.cout = a->qkv.cout_pad = 3 * C; a->qkv.taps = 1;
    a->qkv.w = flux_hip_malloc((size_t)3 * C * C * 2);
    a->qkv.b = dev_f32((size_t)3 * C);
    if (!a->qkv.w || !a->qkv.b) return 0;
    static const char *part[3] = {"to_q", "to_k", "to_v"};
    for (int i = 0; i < 3; i++) {
        snprintf(name, sizeof name, "%s.%s.weight", prefix, part[i]);
        add_slot(v, name, K_CONV1, (char *)a->qkv.w + (size_t)i * C * C * 2, C, C, C);
        snprintf(name, sizeof name, "%s.%s.bias", prefix, part[i]);
        add_slot(v, name, K_VEC, a->qkv.b + (size_t)i * C, C, 1, 0);
    }
    snprintf(name, sizeof name, "%s.to_out.0", prefix);
    return add_conv(v, name, &a->out, C, C, 1);
}

flux_hip_vae *flux_hip_vae_new(void) {
    if (!flux_hip_available()) return NULL;
    static const int mult[4] = {1, 2, 4, 4};
    const int base = 128, zc = 32, lc = 128, mid = base * mult[3];
    flux_hip_vae *v = (flux_hip_vae *)calloc(1, sizeof *v);
    if (!v) { flux_hip_fail("out of host memory"); return NULL; }
    v->eps = 1e-4f; /* flux_vae.c:1249 */
    v->adding_side = SIDE_BOTH;
    int ok = add_vec(v, "bn.running_mean", "", &v->bn_mean, lc) && add_vec(v, "bn.running_var", "", &v->bn_var, lc);
    v->adding_side = SIDE_DECODER;
    ok = ok && (v->pq_w = dev_f32((size_t)zc * zc)) && (v->pq_b = dev_f32(zc));
    if (ok) {
        add_slot(v, "post_quant_conv.weight", K_RAW, v->pq_w, zc * zc, 1, 0);
        add_slot(v, "post_quant_conv.bias", K_VEC, v->pq_b, zc, 1, 0);
    }
    ok = ok && add_conv(v, "decoder.conv_in", &v->conv_in, mid, zc, 9);
    ok = ok && add_res(v, "decoder.mid_block.resnets.0", &v->mid[0], mid, mid) && add_res(v, "decoder.mid_block.resnets.1", &v->mid[1], mid, mid);
    ok = ok && add_attn(v, "decoder.mid_block.attentions.0", &v->attn, mid);
    int prev = mid, bi = 0;
    for (int level = 3; ok && level >= 0; level--) {
        const int ch = base * mult[level], up = 3 - level;
        char name[128];
        for (int r = 0; ok && r < 3; r++) {
            snprintf(name, sizeof name, "decoder.up_blocks.%d.resnets.%d", up, r);
            ok = add_res(v, name, &v->up[bi++], r == 0 ? prev : ch, ch);
        }
        if (ok && level > 0) {
            snprintf(name, sizeof name, "decoder.up_blocks.%d.upsamplers.0.conv", up);
            ok = add_conv(v, name, &v->up_conv[up], ch, ch, 9);
        }
        prev = ch;
    }
    ok = ok && add_vec(v, "decoder.conv_norm_out", ".weight", &v->out_g, base) && add_vec(v, "decoder.conv_norm_out", ".bias", &v->out_b, base);
    ok = ok && add_conv(v, "decoder.conv_out", &v->conv_out, 3, base, 9);

    /* encoder (names: flux_vae.c:1254-1296) */
    v->adding_side = SIDE_ENCODER;
    if (ok) {
        vconv *c = &v->enc_conv_in;
        c->cin = 3; c->cout = c->cout_pad = base; c->taps = 1; c->cin_pad = 64;
        c->w = flux_hip_malloc((size_t)base * 64 * 2);
        c->b = dev_f32((size_t)base);
        ok = c->w && c->b && flux_hip_memset(c->w, 0, (size_t)base * 64 * 2);
        if (ok) {
            add_slot(v, "encoder.conv_in.weight", K_CONV3_PACKED, c->w, base, 3, 64);
            add_slot(v, "encoder.conv_in.bias", K_VEC, c->b, base, 1, 0);
        }
    }
    prev = base; bi = 0;
    for (int level = 0; ok && level < 4; level++) {
        const int ch = base * mult[level];
        char name[128];
        for (int r = 0; ok && r < 2; r++) {
            snprintf(name, sizeof name, "encoder.down_blocks.%d.resnets.%d", level, r);
            ok = add_res(v, name, &v->enc_down[bi++], r == 0 ? prev : ch, ch);
        }
        if (ok && level < 3) {
            snprintf(name, sizeof name, "encoder.down_blocks.%d.downsamplers.0.conv", level);
            ok = add_conv(v, name, &v->enc_down_conv[level], ch, ch, 9);
        }
        prev = ch;
    }
    ok = ok && add_res(v, "encoder.mid_block.resnets.0", &v->enc_mid[0], mid, mid) && add_res(v, "encoder.mid_block.resnets.1", &v->enc_mid[1], mid, mid);
    ok = ok && add_attn(v, "encoder.mid_block.attentions.0", &v->enc_attn, mid);
    ok = ok && add_vec(v, "encoder.conv_norm_out", ".weight", &v->enc_out_g, mid) && add_vec(v, "encoder.conv_norm_out", ".bias", &v->enc_out_b, mid);
    ok = ok && add_conv(v, "encoder.conv_out", &v->enc_conv_out, 2 * zc, mid, 9) && add_conv(v, "quant_conv", &v->quant, 2 * zc, 2 * zc, 1);
    if (!ok) { flux_hip_vae_free(v); return NULL; }
    return v;
}

/* Stores one tensor of the VAE file (names as flux_vae_load_safetensors asks for them,
 * flux_vae.c:1150-1330). */
int flux_hip_vae_set_tensor(flux_hip_vae *v, const char *name, int dtype, const void *data, int64_t numel) {
    if (!v || !name || !data) return flux_hip_fail("flux_hip_vae_set_tensor: NULL argument");
    if (dtype != FH_DT_F32 && dtype != FH_DT_F16 && dtype != FH_DT_BF16) return flux_hip_fail("tensor %s: unsupported dtype %d", name, dtype);
    vslot *s = NULL;
    for (int i = 0; i < v->nslots; i++)
        if (!strcmp(v->slots[i].name, name)) { s = &v->slots[i]; break; }
    if (!s) return flux_hip_fail("tensor %s is not part of the VAE", name);
    const int taps = s->kind == K_CONV3 || s->kind == K_CONV3_PACKED ? 9 : 1;
    const int64_t expect = s->kind == K_VEC || s->kind == K_RAW ? s->rows : (int64_t)s->rows * s->cols * taps;
    if (numel != expect) return flux_hip_fail("tensor %s has %lld elements, expected %lld", name, (long long)numel, (long long)expect);
    int ok;
    if (s->kind == K_VEC || s->kind == K_RAW) {
        float *tmp = (float *)malloc(sizeof(float) * (size_t)numel);
        if (!tmp) return flux_hip_fail("out of host memory");
        for (int64_t i = 0; i < numel; i++) tmp[i] = fh_tensor_value(dtype, data, i);
        ok = flux_hip_upload(s->dst, tmp, sizeof(float) * (size_t)numel);
        free(tmp);
    } else {
        /* [cout][cin][ky][kx] -> bf16 [cout][cin_pad / 64][ky*3+kx][64]: the nine taps of a 64-channel
         * chunk side by side (flux_hip_conv's K order); for a 1x1 convolution that is [cout][cin_pad] */
        const int cout = s->rows, cin = s->cols, cp = s->cin_pad;
        uint16_t *tmp = (uint16_t *)calloc((size_t)cout * taps * cp, 2);
        if (!tmp) return flux_hip_fail("out of host memory");
        /* K_CONV3_PACKED: the nine taps of all cin channels in one row of cin_pad, [cout][(ky*3+kx) * cin + cin] */
        const int packed = s->kind == K_CONV3_PACKED;
        for (int o = 0; o < cout; o++)
            for (int c = 0; c < cin; c++)
                for (int t = 0; t < taps; t++)
                    tmp[packed ? (size_t)o * cp + t * cin + c : (size_t)o * taps * cp + ((size_t)(c >> 6) * taps + t) * 64 + (c & 63)] =
                        to_bf16(fh_tensor_value(dtype, data, ((int64_t)o * cin + c) * taps + t));
        ok = flux_hip_upload(s->dst, tmp, packed ? (size_t)cout * cp * 2 : (size_t)cout * taps * cp * 2);
        free(tmp);
    }
    if (ok) s->loaded = 1;
    return ok;
}

/* every tensor that `side` needs has been stored */
static int vae_complete(const flux_hip_vae *v, int side) {
    for (int i = 0; i < v->nslots; i++)
        if (!v->slots[i].loaded && (v->slots[i].side == SIDE_BOTH || v->slots[i].side == side))
            return flux_hip_fail("VAE tensor %s was not loaded", v->slots[i].name);
    return 1;
}

static int vae_tensor_cb(void *ctx, const char *name, int dtype, const void *data, int64_t numel) {
    return flux_hip_vae_set_tensor((flux_hip_vae *)ctx, name, dtype, data, numel);
}

flux_hip_vae *flux_hip_vae_load_file(const char *path) {
    flux_hip_vae *v = flux_hip_vae_new();
    if (!v) return NULL;
    if (!fh_safetensors_walk(path, vae_tensor_cb, v) || !vae_complete(v, SIDE_DECODER)) { flux_hip_vae_free(v); return NULL; }
    return v;
}

/* From the reference's parsed-file handle (safetensors_file_t *), as flux_vae_load_safetensors
 * receives it (flux_vae.c:1232). */
flux_hip_vae *flux_hip_vae_load_safetensors(void *sf) {
    flux_hip_vae *v = flux_hip_vae_new();
    if (!v) return NULL;
    if (!fh_safetensors_walk_handle(sf, vae_tensor_cb, v) || !vae_complete(v, SIDE_DECODER)) { flux_hip_vae_free(v); return NULL; }
    return v;
}

static void free_conv(vconv *c) { flux_hip_free(c->w); flux_hip_free(c->b); }
static void free_attn(vattn *a) { flux_hip_free(a->g); flux_hip_free(a->b); free_conv(&a->qkv); free_conv(&a->out); }
static void free_res(vres *r) {
    flux_hip_free(r->n1g); flux_hip_free(r->n1b); flux_hip_free(r->n2g); flux_hip_free(r->n2b);
    free_conv(&r->c1); free_conv(&r->c2); free_conv(&r->skip);
}

static void free_work(flux_hip_vae *v) {
    flux_hip_free(v->X); flux_hip_free(v->Y); flux_hip_free(v->Hb); flux_hip_free(v->S); flux_hip_free(v->kbias);
    flux_hip_free(v->gn); flux_hip_free(v->lat); flux_hip_free(v->img_f32); flux_hip_free(v->A_base); flux_hip_free(v->R);
    flux_hip_free(v->P); flux_hip_free(v->VT); flux_hip_free(v->img_u8); flux_hip_free(v->st_x); flux_hip_free(v->st_h);
    v->X = v->Y = v->Hb = v->S = v->kbias = v->gn = v->lat = v->img_f32 = v->st_x = v->st_h = NULL;
    v->A_base = v->R = v->P = v->VT = NULL;
    v->img_u8 = NULL;
    v->f32_elems = v->bf16_elems = v->guard = v->att_ld = v->att_chunk = v->gn_floats = v->lat_elems = v->img_pixels = v->st_floats = 0;
}

void flux_hip_vae_free(flux_hip_vae *v) {
    if (!v) return;
    flux_hip_sync();
    flux_hip_free(v->bn_mean); flux_hip_free(v->bn_var); flux_hip_free(v->pq_w); flux_hip_free(v->pq_b);
    free_conv(&v->conv_in); free_conv(&v->conv_out); free_attn(&v->attn);
    for (int i = 0; i < 3; i++) free_conv(&v->up_conv[i]);
    for (int i = 0; i < 2; i++) free_res(&v->mid[i]);
    for (int i = 0; i < 12; i++) free_res(&v->up[i]);
    flux_hip_free(v->out_g); flux_hip_free(v->out_b);
    free_conv(&v->enc_conv_in); free_conv(&v->enc_conv_out); free_conv(&v->quant); free_attn(&v->enc_attn);
    for (int i = 0; i < 3; i++) free_conv(&v->enc_down_conv[i]);
    for (int i = 0; i < 2; i++) free_res(&v->enc_mid[i]);
    for (int i = 0; i < 8; i++) free_res(&v->enc_down[i]);
    flux_hip_free(v->enc_out_g); flux_hip_free(v->enc_out_b);
    free_work(v);
    free(v->slots);
    free(v);
}

/* Test hook: upper bound on the query rows per attention chunk (0 = the buffer's own bound,
 * 1 GB of fp32 scores). */
static int g_att_chunk_limit = 0;
void flux_hip_vae_set_attention_chunk(int rows) { g_att_chunk_limit = rows > 0 ? rows : 0; }

/* Work buffers for a latent of h x w. The largest image is the full-resolution one with 256
 * channels (output of the last upsample convolution). bf16 convolution inputs carry a guard of
 * one image row + 2 positions on both sides (flux_hip_conv reads that far beyond the image). */
static int ensure_work(flux_hip_vae *v, int h, int w) {
    const size_t hp0 = 16 * (size_t)h + 2, wp0 = 16 * (size_t)w + 2, mp0 = hp0 * wp0;
    const size_t hpm = 2 * (size_t)h + 2, wpm = 2 * (size_t)w + 2, mpm = hpm * wpm;
    const size_t ld = (mpm + 127) & ~(size_t)127;
    size_t f32_elems = mp0 * 256, guard = (wp0 + 2) * 512;
    size_t bf16_elems = mp0 * 256;
    if (bf16_elems < ld * 1536) bf16_elems = ld * 1536; /* R also holds q, k, v of the attention */
    const size_t mp_half = (8 * (size_t)h + 2) * (8 * (size_t)w + 2);
    if (bf16_elems < mp_half * 9 * 128) bf16_elems = mp_half * 9 * 128; /* the encoder's first downsampling step: nine taps of 128 channels per half-size position */
    size_t chunk = ((size_t)1 << 28) / ld;               /* at most 1 GB of fp32 scores at a time */
    if (chunk < 128) chunk = 128;
    if (chunk > mpm) chunk = mpm;
    const size_t gn_floats = flux_hip_group_norm_scratch_floats((int)hp0, (int)wp0);
    const size_t st_floats = (mp0 / 32 + 2) * (256 / 4) * 2; /* convolution statistics: at most rows/32 + 2 partial rows of cout/4 quads */
    if (f32_elems <= v->f32_elems && bf16_elems <= v->bf16_elems && guard <= v->guard && ld <= v->att_ld && chunk <= v->att_chunk &&
        gn_floats <= v->gn_floats && st_floats <= v->st_floats && (size_t)128 * h * w <= v->lat_elems && (size_t)256 * h * w <= v->img_pixels)
        return 1;
    flux_hip_sync();
    free_work(v);
    v->X = (float *)flux_hip_malloc(f32_elems * 4);
    v->Y = (float *)flux_hip_malloc(f32_elems * 4);
    v->Hb = (float *)flux_hip_malloc(f32_elems * 4);
    v->A_base = flux_hip_malloc((bf16_elems + 2 * guard) * 2);
    v->R = flux_hip_malloc(bf16_elems * 2);
    v->S = (float *)flux_hip_malloc(chunk * ld * 4);
    v->P = flux_hip_malloc(chunk * ld * 2);
    v->VT = flux_hip_malloc(512 * ld * 2);
    v->kbias = (float *)flux_hip_malloc(ld * 4);
    v->gn = (float *)flux_hip_malloc(gn_floats * 4);
    v->st_x = (float *)flux_hip_malloc(st_floats * 4);
    v->st_h = (float *)flux_hip_malloc(st_floats * 4);
    v->lat = (float *)flux_hip_malloc((size_t)128 * h * w * 4);
    v->img_f32 = (float *)flux_hip_malloc((size_t)256 * h * w * 3 * 4);
    v->img_u8 = (uint8_t *)flux_hip_malloc((size_t)256 * h * w * 3);
    if (!v->X || !v->Y || !v->Hb || !v->A_base || !v->R || !v->S || !v->P || !v->VT || !v->kbias || !v->gn || !v->lat || !v->img_f32 ||
        !v->img_u8 || !v->st_x || !v->st_h) {
        free_work(v);
        return flux_hip_fail("VAE work buffers for a %d x %d latent could not be allocated", h, w);
    }
    /* guards are read (their contents never reach an output that is kept), so give them defined values */
    if (!flux_hip_memset(v->A_base, 0, (bf16_elems + 2 * guard) * 2)) return 0;
    v->f32_elems = f32_elems; v->bf16_elems = bf16_elems; v->guard = guard; v->att_ld = ld; v->att_chunk = chunk;
    v->gn_floats = gn_floats; v->st_floats = st_floats; v->lat_elems = (size_t)128 * h * w; v->img_pixels = (size_t)256 * h * w;
    return 1;
}

/* Called (when set) after each of the 15 blocks has been queued: 3 mid + 12 up, the reference's
 * count (flux_vae.c:757-758). */
void (*flux_hip_vae_progress)(int block, int total) = NULL;

typedef struct {
    flux_hip_vae *v;
    float *x, *y; /* residual stream and the spare fp32 image */
    void *A;      /* bf16 convolution input (inside its guards) */
    int hp, wp;
    int x_rows, h_rows; /* partial rows of the statistics the last convolution into x / into Hb left in st_x / st_h */
} vstate;

/* stats: NULL, or the buffer that receives the sums for the next group norm over `out` (its row count goes to *stats_rows) */
static int run_conv(vstate *s, const vconv *c, int epi, const void *in, const float *res, void *out, int masked, float *stats, int *stats_rows) {
    return flux_hip_conv_stats(epi, in, c->w, c->b, res, out, s->hp * s->wp, masked ? s->wp : 0, c->cin_pad, c->cout_pad, c->taps, stats,
                               stats_rows);
}

/* resblock_forward, flux_vae.c:179-219. Every group norm takes its statistics from the epilogue of
 * the convolution that produced its input. */
static int run_res(vstate *s, const vres *r) {
    flux_hip_vae *v = s->v;
    const int differ = r->cin != r->cout;
    if (!flux_hip_group_norm_stats(s->A, differ ? v->R : NULL, s->x, 0, r->n1g, r->n1b, v->gn, s->hp, s->wp, r->cin, v->eps, 1, v->st_x, s->x_rows)) return 0;
    if (!run_conv(s, &r->c1, FLUX_HIP_EPI_CONV_BF16, s->A, NULL, v->Hb, 1, v->st_h, &s->h_rows)) return 0; /* only the next norm reads it */
    if (!flux_hip_group_norm_stats(s->A, NULL, v->Hb, 1, r->n2g, r->n2b, v->gn, s->hp, s->wp, r->cout, v->eps, 1, v->st_h, s->h_rows)) return 0;
    if (differ) {
        if (!run_conv(s, &r->skip, FLUX_HIP_EPI_CONV_F32, v->R, NULL, s->y, 1, NULL, NULL)) return 0;
        if (!run_conv(s, &r->c2, FLUX_HIP_EPI_CONV_F32, s->A, s->y, s->y, 1, v->st_x, &s->x_rows)) return 0;
        float *t = s->x; s->x = s->y; s->y = t;
        return 1;
    }
    return run_conv(s, &r->c2, FLUX_HIP_EPI_CONV_F32, s->A, s->x, s->x, 1, v->st_x, &s->x_rows);
}

/* attnblock_forward, flux_vae.c:223-313 */
static int run_attn(vstate *s, const vattn *a) {
    flux_hip_vae *v = s->v;
    const int C = 512, rows = s->hp * s->wp, ld = (rows + 127) & ~127;
    if (!flux_hip_group_norm_stats(s->A, NULL, s->x, 0, a->g, a->b, v->gn, s->hp, s->wp, C, v->eps, 0, v->st_x, s->x_rows)) return 0;
    /* key rows between the image and the padded width are read by the score GEMM: zero them */
    if (ld > rows && !flux_hip_memset((char *)v->R + (size_t)rows * 3 * C * 2, 0, (size_t)(ld - rows) * 3 * C * 2)) return 0;
    if (!run_conv(s, &a->qkv, FLUX_HIP_EPI_CONV_BF16, s->A, NULL, v->R, 0, NULL, NULL)) return 0;
    if (!flux_hip_vae_key_bias(v->kbias, ld, s->hp, s->wp)) return 0;
    if (!flux_hip_transpose_bf16(v->VT, ld, (char *)v->R + 2 * C * 2, 3 * C, rows, C)) return 0;
    const float scale = 1.0f / sqrtf((float)C);
    int chunk = (int)v->att_chunk;
    if (g_att_chunk_limit && g_att_chunk_limit < chunk) chunk = g_att_chunk_limit;
    for (int r0 = 0; r0 < rows; r0 += chunk) {
        const int n = rows - r0 < chunk ? rows - r0 : chunk;
        flux_hip_linear_part sp = {(char *)v->R + (size_t)r0 * 3 * C * 2, (char *)v->R + C * 2, v->S, NULL, n};
        if (!flux_hip_linear(FLUX_HIP_EPI_F32, 1, &sp, ld, C, 3 * C, 3 * C, ld, 0, 0)) return 0;
        if (!flux_hip_softmax_rows(v->P, v->S, v->kbias, n, ld, scale)) return 0;
        flux_hip_linear_part pv = {v->P, v->VT, (char *)s->A + (size_t)r0 * C * 2, NULL, n};
        if (!flux_hip_linear(FLUX_HIP_EPI_BF16, 1, &pv, C, ld, ld, ld, C, 0, 0)) return 0;
    }
    return run_conv(s, &a->out, FLUX_HIP_EPI_CONV_F32, s->A, s->x, s->x, 1, v->st_x, &s->x_rows);
}

/* latent [128, h, w] on the host -> 8-bit image [16h, 16w, 3] and/or the unquantised decoder
 * output [3, 16h, 16w], both optional, on the host. */
int flux_hip_vae_decode(flux_hip_vae *v, const float *latent, int h, int w, uint8_t *rgb, float *rgb_f32) {
    if (!v || !latent) return flux_hip_fail("flux_hip_vae_decode: NULL argument");
    if (h <= 0 || w <= 0 || h > 112 || w > 112) /* the reference's limit: 1792 pixels, flux.h:52 */
        return flux_hip_fail("flux_hip_vae_decode: latent %d x %d out of range (1..112)", h, w);
    if (!vae_complete(v, SIDE_DECODER) || !ensure_work(v, h, w)) return 0;
    vstate s = {v, v->X, v->Y, (char *)v->A_base + v->guard * 2, 2 * h + 2, 2 * w + 2, 0, 0};
    if (!flux_hip_upload(v->lat, latent, (size_t)128 * h * w * 4)) return 0;
    if (!flux_hip_vae_latent_in(s.A, v->lat, v->bn_mean, v->bn_var, v->pq_w, v->pq_b, h, w, v->eps)) return 0;
    if (!run_conv(&s, &v->conv_in, FLUX_HIP_EPI_CONV_F32, s.A, NULL, s.x, 1, v->st_x, &s.x_rows)) return 0;
    int done = 0;
    const int total = 15;
    if (!run_res(&s, &v->mid[0])) return 0;
    if (flux_hip_vae_progress) flux_hip_vae_progress(done++, total);
    if (!run_attn(&s, &v->attn)) return 0;
    if (flux_hip_vae_progress) flux_hip_vae_progress(done++, total);
    if (!run_res(&s, &v->mid[1])) return 0;
    if (flux_hip_vae_progress) flux_hip_vae_progress(done++, total);
    int bi = 0;
    for (int level = 3; level >= 0; level--) {
        for (int r = 0; r < 3; r++) {
            if (!run_res(&s, &v->up[bi++])) return 0;
            if (flux_hip_vae_progress) flux_hip_vae_progress(done++, total);
        }
        if (level > 0) {
            const vconv *c = &v->up_conv[3 - level];
            if (!flux_hip_upsample2x(s.A, s.x, s.hp, s.wp, c->cin)) return 0;
            s.hp = 2 * (s.hp - 2) + 2;
            s.wp = 2 * (s.wp - 2) + 2;
            if (!run_conv(&s, c, FLUX_HIP_EPI_CONV_F32, s.A, NULL, s.x, 1, v->st_x, &s.x_rows)) return 0;
        }
    }
    if (!flux_hip_group_norm_stats(s.A, NULL, s.x, 0, v->out_g, v->out_b, v->gn, s.hp, s.wp, 128, v->eps, 1, v->st_x, s.x_rows)) return 0;
    if (!run_conv(&s, &v->conv_out, FLUX_HIP_EPI_CONV_F32, s.A, NULL, v->Hb, 1, NULL, NULL)) return 0;
    const int H = 16 * h, W = 16 * w;
    if (!flux_hip_vae_image_out(rgb ? v->img_u8 : NULL, rgb_f32 ? v->img_f32 : NULL, v->Hb, v->conv_out.cout_pad, H, W)) return 0;
    if (rgb && !flux_hip_download(rgb, v->img_u8, (size_t)H * W * 3)) return 0;
    if (rgb_f32 && !flux_hip_download(rgb_f32, v->img_f32, (size_t)H * W * 3 * 4)) return 0;
    return flux_hip_sync();
}

/* image [3, H, W] fp32 in [-1, 1] on the host (H, W multiples of 16, at most 1792) -> normalised
 * latent [128, H/16, W/16] on the host (flux_vae_encode, flux_vae.c:320-443, batch 1). */
int flux_hip_vae_encode(flux_hip_vae *v, const float *img, int H, int W, float *latent) {
    if (!v || !img || !latent) return flux_hip_fail("flux_hip_vae_encode: NULL argument");
    if (H <= 0 || W <= 0 || (H & 15) || (W & 15) || H > 1792 || W > 1792) /* the reference's limit, flux.h:52 */
        return flux_hip_fail("flux_hip_vae_encode: image %d x %d (sides must be multiples of 16, at most 1792)", H, W);
    const int h = H / 16, w = W / 16;
    if (!vae_complete(v, SIDE_ENCODER) || !ensure_work(v, h, w)) return 0;
    vstate s = {v, v->X, v->Y, (char *)v->A_base + v->guard * 2, H + 2, W + 2, 0, 0};
    if (!flux_hip_upload(v->img_f32, img, (size_t)3 * H * W * 4)) return 0;
    if (!flux_hip_vae_image_in(s.A, v->img_f32, H, W)) return 0;
    if (!run_conv(&s, &v->enc_conv_in, FLUX_HIP_EPI_CONV_F32, s.A, NULL, s.x, 1, v->st_x, &s.x_rows)) return 0;
    int done = 0, bi = 0;
    const int total = 11; /* 8 down + 3 mid, the reference's count (flux_vae.c:343) */
    for (int level = 0; level < 4; level++) {
        for (int r = 0; r < 2; r++) {
            if (!run_res(&s, &v->enc_down[bi++])) return 0;
            if (flux_hip_vae_progress) flux_hip_vae_progress(done++, total);
        }
        if (level < 3) {
            const vconv *c = &v->enc_down_conv[level];
            if (!flux_hip_downsample_gather(s.A, s.x, s.hp, s.wp, c->cin)) return 0;
            s.hp = (s.hp - 2) / 2 + 2;
            s.wp = (s.wp - 2) / 2 + 2;
            /* the nine taps sit side by side in every row of A, in the weights' K order: a 1x1 convolution over 9 * cin channels */
            if (!flux_hip_conv_stats(FLUX_HIP_EPI_CONV_F32, s.A, c->w, c->b, NULL, s.x, s.hp * s.wp, s.wp, 9 * c->cin_pad, c->cout_pad, 1, v->st_x,
                                     &s.x_rows))
                return 0;
        }
    }
    if (!run_res(&s, &v->enc_mid[0])) return 0;
    if (flux_hip_vae_progress) flux_hip_vae_progress(done++, total);
    if (!run_attn(&s, &v->enc_attn)) return 0;
    if (flux_hip_vae_progress) flux_hip_vae_progress(done++, total);
    if (!run_res(&s, &v->enc_mid[1])) return 0;
    if (flux_hip_vae_progress) flux_hip_vae_progress(done++, total);
    if (!flux_hip_group_norm_stats(s.A, NULL, s.x, 0, v->enc_out_g, v->enc_out_b, v->gn, s.hp, s.wp, 512, v->eps, 1, v->st_x, s.x_rows)) return 0;
    if (!run_conv(&s, &v->enc_conv_out, FLUX_HIP_EPI_CONV_BF16, s.A, NULL, v->R, 1, NULL, NULL)) return 0;
    if (!run_conv(&s, &v->quant, FLUX_HIP_EPI_CONV_F32, v->R, NULL, v->Hb, 1, NULL, NULL)) return 0;
    if (!flux_hip_vae_latent_out(v->lat, v->Hb, v->quant.cout_pad, v->bn_mean, v->bn_var, h, w, v->eps)) return 0;
    if (!flux_hip_download(latent, v->lat, (size_t)128 * h * w * 4)) return 0;
    return flux_hip_sync();
}
