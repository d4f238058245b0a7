/*
 * vae_oracle.c - CPU restatement (fp32) of the FLUX.2 VAE: the decoder, which turns the sampler's
 * final latent into an RGB image, and the encoder, which turns a reference image into the latent
 * that image-to-image and multi-reference generation feed to the transformer.
 *
 * THIS FILE IS TEST INFRASTRUCTURE, like flux_oracle.c next to it: the checker that the HIP
 * decoder is compared against. It is never part of the shipped code path.
 *
 * Every function cites the file:line of antirez/flux2.c it restates. Tensors are NCHW fp32 as
 * in the reference. The channel width is a parameter (the reference fixes base_channels = 128,
 * flux_vae.c:1243-1247); everything else - channel multipliers {1,2,4,4}, 2+1 residual blocks
 * per level, 32 groups, 32 latent channels, 2x2 patches - is the reference's.
 *
 * Pinning status (tests/test_oracle_golden.py, tests/test_oracle_math.py):
 *   fo_conv2d, fo_group_norm, fo_upsample_nearest, fo_unpatchify: against the reference's own
 *   flux_conv2d / flux_group_norm / flux_upsample_nearest / flux_unpatchify compiled from its
 *   sources (golden vectors), and against closed forms (identity kernel, constant image,
 *   zero-mean/unit-variance groups);
 *   fo_vae_decode: against images produced by the reference's flux_vae_decode on the same
 *   synthetic weights (golden vectors), which also covers the residual and attention blocks;
 *   fo_conv2d_down, fo_patchify: against the reference's flux_conv2d (stride 2 over an image
 *   padded on the right and below) and flux_patchify (golden vectors), and against fo_conv2d
 *   sampled at every other pixel / fo_unpatchify's inverse;
 *   fo_vae_encode: against latents produced by the reference's flux_vae_encode (generic build) on
 *   the same synthetic weights (golden vectors), with fo_vae_set_reference_aliasing(1): that build
 *   overwrites the input of one convolution in each widening residual block while it runs, see
 *   resblock(). The default path differs from the pinned one in that convolution only, where it
 *   calls fo_conv2d like every other block.
 */
#include <math.h>
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

/* out[oc, y, x] = bias[oc] + sum_{ic, ky, kx} in[ic, y+ky-pad, x+kx-pad] * w[oc, ic, ky, kx]
 * with zeros outside the image; stride 1 (flux_kernels.c:342-350 and the plain loops at
 * :441-470; the decoder only uses 3x3/pad 1 and 1x1/pad 0). */
void fo_conv2d(float *out, const float *in, const float *w, const float *bias,
               int in_ch, int out_ch, int H, int W, int k, int pad) {
    #pragma omp parallel for schedule(static)
    for (int oc = 0; oc < out_ch; oc++) {
        float *o = out + (size_t)oc * H * W;
        float b = bias ? bias[oc] : 0.0f;
        for (int i = 0; i < H * W; i++) o[i] = b;
        for (int ic = 0; ic < in_ch; ic++) {
            const float *src = in + (size_t)ic * H * W;
            for (int ky = 0; ky < k; ky++)
                for (int kx = 0; kx < k; kx++) {
                    float wv = w[(((size_t)oc * in_ch + ic) * k + ky) * k + kx];
                    int dy = ky - pad, dx = kx - pad;
                    int y0 = dy < 0 ? -dy : 0, y1 = dy > 0 ? H - dy : H;
                    int x0 = dx < 0 ? -dx : 0, x1 = dx > 0 ? W - dx : W;
                    for (int y = y0; y < y1; y++) {
                        float *orow = o + (size_t)y * W;
                        const float *irow = src + (size_t)(y + dy) * W + dx;
                        for (int x = x0; x < x1; x++) orow[x] += wv * irow[x];
                    }
                }
        }
    }
}

/* The encoder's downsampling step: the image gets one row of zeros below and one column on the
 * right, then a 3x3 convolution with stride 2 and no further padding runs over it
 * (vae_pad_right_bottom + vae_conv2d, flux_vae.c:151-172, 363-377; sizes flux_kernels.c:345-346):
 * out[oc, y, x] = bias[oc] + sum_{ic, ky, kx} in[ic, 2y+ky, 2x+kx] * w[oc, ic, ky, kx], zeros at
 * row H and column W; the output is ((H+1-3)/2+1) x ((W+1-3)/2+1). */
void fo_conv2d_down(float *out, const float *in, const float *w, const float *bias, int in_ch, int out_ch, int H, int W) {
    const int oH = (H + 1 - 3) / 2 + 1, oW = (W + 1 - 3) / 2 + 1;
    #pragma omp parallel for schedule(static)
    for (int oc = 0; oc < out_ch; oc++) {
        float *o = out + (size_t)oc * oH * oW;
        float b = bias ? bias[oc] : 0.0f;
        for (int i = 0; i < oH * oW; i++) o[i] = b;
        for (int ic = 0; ic < in_ch; ic++) {
            const float *src = in + (size_t)ic * H * W;
            for (int ky = 0; ky < 3; ky++)
                for (int kx = 0; kx < 3; kx++) {
                    const float wv = w[(((size_t)oc * in_ch + ic) * 3 + ky) * 3 + kx];
                    for (int y = 0; y < oH; y++) {
                        const int iy = 2 * y + ky;
                        if (iy >= H) continue;
                        const float *irow = src + (size_t)iy * W;
                        float *orow = o + (size_t)y * oW;
                        for (int x = 0; x < oW; x++) {
                            const int ix = 2 * x + kx;
                            if (ix < W) orow[x] += wv * irow[ix];
                        }
                    }
                }
        }
    }
}

/* Per group of channels/num_groups channels: mean, biased variance around that mean (two
 * passes), (x - mean) / sqrt(var + eps) * gamma[c] + beta[c] (flux_kernels.c:511-553). */
void fo_group_norm(float *out, const float *x, const float *gamma, const float *beta,
                   int channels, int H, int W, int num_groups, float eps) {
    int cpg = channels / num_groups;
    size_t n = (size_t)cpg * H * W;
    #pragma omp parallel for schedule(static)
    for (int g = 0; g < num_groups; g++) {
        const float *xs = x + (size_t)g * n;
        double s = 0.0;
        for (size_t i = 0; i < n; i++) s += xs[i];
        float mean = (float)(s / (double)n);
        double v = 0.0;
        for (size_t i = 0; i < n; i++) { double d = xs[i] - mean; v += d * d; }
        float inv = 1.0f / sqrtf((float)(v / (double)n) + eps);
        for (int c = 0; c < cpg; c++) {
            int ch = g * cpg + c;
            for (int i = 0; i < H * W; i++) {
                size_t idx = (size_t)ch * H * W + i;
                out[idx] = gamma[ch] * ((x[idx] - mean) * inv) + beta[ch];
            }
        }
    }
}

/* out[c, y, x] = in[c, y/2, x/2] (flux_kernels.c:1017-1036 with both scales 2) */
void fo_upsample_nearest(float *out, const float *in, int channels, int H, int W) {
    for (int c = 0; c < channels; c++)
        for (int y = 0; y < 2 * H; y++)
            for (int x = 0; x < 2 * W; x++)
                out[((size_t)c * 2 * H + y) * 2 * W + x] = in[((size_t)c * H + y / 2) * W + x / 2];
}

/* [C*p*p, H, W] -> [C, H*p, W*p], input channel c*p*p + pi*p + pj lands at pixel
 * (ph*p + pi, pw*p + pj) of output channel c (flux_kernels.c:1067-1097) */
void fo_unpatchify(float *out, const float *in, int channels, int H, int W, int p) {
    for (int c = 0; c < channels; c++)
        for (int ph = 0; ph < H; ph++)
            for (int pw = 0; pw < W; pw++)
                for (int pi = 0; pi < p; pi++)
                    for (int pj = 0; pj < p; pj++)
                        out[((size_t)c * H * p + ph * p + pi) * W * p + pw * p + pj] =
                            in[((size_t)(c * p * p + pi * p + pj) * H + ph) * W + pw];
}

/* [C, H, W] -> [C*p*p, H/p, W/p], the inverse of fo_unpatchify: pixel (ph*p + pi, pw*p + pj) of
 * channel c lands at (ph, pw) of output channel c*p*p + pi*p + pj (flux_kernels.c:1038-1065) */
void fo_patchify(float *out, const float *in, int channels, int H, int W, int p) {
    const int oH = H / p, oW = W / p;
    for (int c = 0; c < channels; c++)
        for (int ph = 0; ph < oH; ph++)
            for (int pw = 0; pw < oW; pw++)
                for (int pi = 0; pi < p; pi++)
                    for (int pj = 0; pj < p; pj++)
                        out[((size_t)(c * p * p + pi * p + pj) * oH + ph) * oW + pw] =
                            in[((size_t)c * H + ph * p + pi) * W + pw * p + pj];
}

static void swish(float *x, size_t n) { /* flux_vae.c:174-176 -> flux_silu, flux_kernels.c:581-585 */
    #pragma omp parallel for schedule(static)
    for (size_t i = 0; i < n; i++) x[i] = x[i] / (1.0f + expf(-x[i]));
}

/* ---- weights: a flat table keyed by the safetensors names the reference loader asks for
 * (flux_vae.c:1150-1330) ---- */
typedef struct { char name[128]; float *data; int64_t n; } fo_vae_tensor;
typedef struct fo_vae {
    int base;           /* base_channels: 128 in the reference */
    float eps;          /* 1e-4 for both the latent de-normalisation and the group norms (flux_vae.c:1249) */
    int ref_aliasing;   /* reproduce the overlap of the reference's residual-block buffers, see resblock() */
    int count, cap;
    fo_vae_tensor *t;
} fo_vae;

fo_vae *fo_vae_new(int base_channels) {
    fo_vae *v = (fo_vae *)calloc(1, sizeof(fo_vae));
    v->base = base_channels;
    v->eps = 1e-4f;
    return v;
}

/* See resblock(): on = restate what the reference's plain-C build computes, off (default) = the
 * arithmetic the block is written to compute. */
void fo_vae_set_reference_aliasing(fo_vae *v, int on) { v->ref_aliasing = on != 0; }

void fo_vae_free(fo_vae *v) {
    if (!v) return;
    for (int i = 0; i < v->count; i++) free(v->t[i].data);
    free(v->t);
    free(v);
}

int fo_vae_set(fo_vae *v, const char *name, const float *data, int64_t n) {
    if (strlen(name) >= sizeof(v->t[0].name)) return -1;
    if (v->count == v->cap) {
        v->cap = v->cap ? v->cap * 2 : 64;
        v->t = (fo_vae_tensor *)realloc(v->t, sizeof(fo_vae_tensor) * (size_t)v->cap);
    }
    fo_vae_tensor *t = &v->t[v->count++];
    strcpy(t->name, name);
    t->n = n;
    t->data = (float *)malloc(sizeof(float) * (size_t)n);
    memcpy(t->data, data, sizeof(float) * (size_t)n);
    return 0;
}

static const float *find(const fo_vae *v, const char *prefix, const char *suffix, int64_t expect, int *err) {
    char name[256];
    snprintf(name, sizeof name, "%s%s", prefix, suffix);
    for (int i = 0; i < v->count; i++)
        if (!strcmp(v->t[i].name, name)) {
            if (v->t[i].n != expect) { fprintf(stderr, "vae oracle: %s has %lld elements, expected %lld\n", name, (long long)v->t[i].n, (long long)expect); *err = 1; return NULL; }
            return v->t[i].data;
        }
    fprintf(stderr, "vae oracle: tensor %s missing\n", name);
    *err = 1;
    return NULL;
}

/* skip (1x1 conv when the widths differ) + conv2(swish(norm2(conv1(swish(norm1(x))))))
 * (flux_vae.c:179-219).
 *
 * The reference keeps norm outputs at the start of one work buffer and convolution outputs
 * in_ch planes further on (flux_vae.c:203). When a block widens (in_ch < out_ch: the first block
 * of encoder levels 1 and 2) the second convolution therefore reads planes [0, out_ch) and writes
 * planes [in_ch, in_ch + out_ch) of the same buffer. Its im2col path copies the input out before
 * it writes (flux_kernels.c:380-425) and is unaffected as long as it runs in one tile (up to 2^28
 * im2col floats: images to about 680 pixels a side); the plain loops of the generic build
 * (flux_kernels.c:441-470) go output channel by output channel, so channel oc is computed from an
 * input whose planes in_ch .. in_ch+oc-1 already hold output channels 0 .. oc-1. With
 * v->ref_aliasing the same happens here, which is what lets the whole encoder be checked against
 * the generic build of the reference; without it (the default, and what the device is compared
 * with) the block computes what it is written to compute. */
static int resblock(const fo_vae *v, const char *prefix, float *out, const float *x, int in_ch, int out_ch, int H, int W) {
    int err = 0;
    size_t sp = (size_t)H * W;
    const float *n1w = find(v, prefix, ".norm1.weight", in_ch, &err), *n1b = find(v, prefix, ".norm1.bias", in_ch, &err);
    const float *c1w = find(v, prefix, ".conv1.weight", (int64_t)out_ch * in_ch * 9, &err), *c1b = find(v, prefix, ".conv1.bias", out_ch, &err);
    const float *n2w = find(v, prefix, ".norm2.weight", out_ch, &err), *n2b = find(v, prefix, ".norm2.bias", out_ch, &err);
    const float *c2w = find(v, prefix, ".conv2.weight", (int64_t)out_ch * out_ch * 9, &err), *c2b = find(v, prefix, ".conv2.bias", out_ch, &err);
    const float *sw = NULL, *sb = NULL;
    if (in_ch != out_ch) {
        sw = find(v, prefix, ".conv_shortcut.weight", (int64_t)out_ch * in_ch, &err);
        sb = find(v, prefix, ".conv_shortcut.bias", out_ch, &err);
    }
    if (err) return -1;
    float *a = (float *)malloc(sizeof(float) * sp * (size_t)(in_ch > out_ch ? in_ch : out_ch));
    float *b = (float *)malloc(sizeof(float) * sp * (size_t)out_ch);
    if (sw) fo_conv2d(out, x, sw, sb, in_ch, out_ch, H, W, 1, 0);
    else memcpy(out, x, sizeof(float) * sp * (size_t)in_ch);
    fo_group_norm(a, x, n1w, n1b, in_ch, H, W, 32, v->eps);
    swish(a, sp * (size_t)in_ch);
    fo_conv2d(b, a, c1w, c1b, in_ch, out_ch, H, W, 3, 1);
    fo_group_norm(a, b, n2w, n2b, out_ch, H, W, 32, v->eps);
    swish(a, sp * (size_t)out_ch);
    if (v->ref_aliasing && in_ch < out_ch) {
        float *work = (float *)malloc(sizeof(float) * sp * (size_t)(in_ch + out_ch));
        memcpy(work, a, sizeof(float) * sp * (size_t)out_ch);
        /* pixel by pixel in the reference's loop order (output channel, row, column), each result
         * stored at once: plane in_ch+oc is read while it is being replaced */
        float *dst = work + (size_t)in_ch * sp;
        for (int oc = 0; oc < out_ch; oc++)
            for (int oy = 0; oy < H; oy++)
                for (int ox = 0; ox < W; ox++) {
                    float sum = c2b[oc];
                    for (int ic = 0; ic < out_ch; ic++)
                        for (int ky = 0; ky < 3; ky++)
                            for (int kx = 0; kx < 3; kx++) {
                                const int iy = oy - 1 + ky, ix = ox - 1 + kx;
                                if (iy >= 0 && iy < H && ix >= 0 && ix < W)
                                    sum += work[(size_t)ic * sp + (size_t)iy * W + ix] * c2w[(((size_t)oc * out_ch + ic) * 3 + ky) * 3 + kx];
                            }
                    dst[(size_t)oc * sp + (size_t)oy * W + ox] = sum;
                }
        memcpy(b, dst, sizeof(float) * sp * (size_t)out_ch);
        free(work);
    } else {
        fo_conv2d(b, a, c2w, c2b, out_ch, out_ch, H, W, 3, 1);
    }
    for (size_t i = 0; i < sp * (size_t)out_ch; i++) out[i] += b[i];
    free(a); free(b);
    return 0;
}

/* x + out_proj(softmax(q k^T / sqrt(ch)) v) over all H*W positions with one head, q/k/v/out
 * being 1x1 convolutions of the group-normalised input (flux_vae.c:223-313) */
static int attnblock(const fo_vae *v, const char *prefix, float *out, const float *x, int ch, int H, int W) {
    int err = 0;
    int sp = H * W;
    const float *nw = find(v, prefix, ".group_norm.weight", ch, &err), *nb = find(v, prefix, ".group_norm.bias", ch, &err);
    const float *qw = find(v, prefix, ".to_q.weight", (int64_t)ch * ch, &err), *qb = find(v, prefix, ".to_q.bias", ch, &err);
    const float *kw = find(v, prefix, ".to_k.weight", (int64_t)ch * ch, &err), *kb = find(v, prefix, ".to_k.bias", ch, &err);
    const float *vw = find(v, prefix, ".to_v.weight", (int64_t)ch * ch, &err), *vb = find(v, prefix, ".to_v.bias", ch, &err);
    const float *ow = find(v, prefix, ".to_out.0.weight", (int64_t)ch * ch, &err), *ob = find(v, prefix, ".to_out.0.bias", ch, &err);
    if (err) return -1;
    size_t n = (size_t)ch * sp;
    float *xn = (float *)malloc(sizeof(float) * n), *q = (float *)malloc(sizeof(float) * n);
    float *k = (float *)malloc(sizeof(float) * n), *vv = (float *)malloc(sizeof(float) * n);
    float *o = (float *)malloc(sizeof(float) * n);
    fo_group_norm(xn, x, nw, nb, ch, H, W, 32, v->eps);
    fo_conv2d(q, xn, qw, qb, ch, ch, H, W, 1, 0);
    fo_conv2d(k, xn, kw, kb, ch, ch, H, W, 1, 0);
    fo_conv2d(vv, xn, vw, vb, ch, ch, H, W, 1, 0);
    float scale = 1.0f / sqrtf((float)ch);
    /* token-major copies, as the reference makes them (flux_vae.c:267-275), so that the inner
     * loops run over contiguous memory */
    float *qt = (float *)malloc(sizeof(float) * n), *kt = (float *)malloc(sizeof(float) * n), *vt = (float *)malloc(sizeof(float) * n);
    #pragma omp parallel for schedule(static)
    for (int i = 0; i < sp; i++)
        for (int c = 0; c < ch; c++) {
            qt[(size_t)i * ch + c] = q[(size_t)c * sp + i] * scale;
            kt[(size_t)i * ch + c] = k[(size_t)c * sp + i];
            vt[(size_t)i * ch + c] = vv[(size_t)c * sp + i];
        }
    #pragma omp parallel
    {
        float *row = (float *)malloc(sizeof(float) * (size_t)sp);
        float *acc = (float *)malloc(sizeof(float) * (size_t)ch);
        #pragma omp for schedule(static)
        for (int i = 0; i < sp; i++) {
            const float *qi = qt + (size_t)i * ch;
            float mx = -3.0e38f;
            for (int j = 0; j < sp; j++) {
                const float *kj = kt + (size_t)j * ch;
                float s = 0.0f;
                for (int c = 0; c < ch; c++) s += qi[c] * kj[c];
                row[j] = s;
                if (s > mx) mx = s;
            }
            float sum = 0.0f;
            for (int j = 0; j < sp; j++) { row[j] = expf(row[j] - mx); sum += row[j]; }
            float inv = 1.0f / sum;
            for (int c = 0; c < ch; c++) acc[c] = 0.0f;
            for (int j = 0; j < sp; j++) {
                const float p = row[j];
                const float *vj = vt + (size_t)j * ch;
                for (int c = 0; c < ch; c++) acc[c] += p * vj[c];
            }
            for (int c = 0; c < ch; c++) o[(size_t)c * sp + i] = acc[c] * inv;
        }
        free(row); free(acc);
    }
    free(qt); free(kt); free(vt);
    fo_conv2d(xn, o, ow, ob, ch, ch, H, W, 1, 0);
    for (size_t i = 0; i < n; i++) out[i] = x[i] + xn[i];
    free(xn); free(q); free(k); free(vv); free(o);
    return 0;
}

/* latent [128, h, w] -> RGB. rgb_f32 (optional) receives the decoder output [3, 16h, 16w] before
 * quantisation, rgb_u8 (optional) the image [16h, 16w, 3] with the reference's conversion
 * (v + 1) * 0.5 * 255, clamped, truncated (flux_vae.c:690-837). Returns 0, or -1 when a
 * tensor is missing. */
int fo_vae_decode(const fo_vae *v, const float *latent, int h, int w, float *rgb_f32, uint8_t *rgb_u8) {
    static const int mult[4] = {1, 2, 4, 4};
    const int zc = 32, lc = 128, base = v->base, mid = base * mult[3];
    int err = 0;
    const float *bn_mean = find(v, "bn.running_mean", "", lc, &err), *bn_var = find(v, "bn.running_var", "", lc, &err);
    const float *pqw = find(v, "post_quant_conv.weight", "", zc * zc, &err), *pqb = find(v, "post_quant_conv.bias", "", zc, &err);
    const float *ciw = find(v, "decoder.conv_in.weight", "", (int64_t)mid * zc * 9, &err), *cib = find(v, "decoder.conv_in.bias", "", mid, &err);
    const float *now_ = find(v, "decoder.conv_norm_out.weight", "", base, &err), *nob = find(v, "decoder.conv_norm_out.bias", "", base, &err);
    const float *cow = find(v, "decoder.conv_out.weight", "", (int64_t)3 * base * 9, &err), *cob = find(v, "decoder.conv_out.bias", "", 3, &err);
    if (err) return -1;

    int H = 2 * h, W = 2 * w;
    size_t cap = (size_t)base * (16 * h) * (16 * w);          /* largest tensor: base channels at full size */
    if (cap < (size_t)mid * (4 * h) * (4 * w)) cap = (size_t)mid * (4 * h) * (4 * w); /* after the first upsample */
    cap *= 2;                                                  /* levels 1 and 2 enter an upsample with 2x the channels */
    float *x = (float *)malloc(sizeof(float) * cap), *y = (float *)malloc(sizeof(float) * cap);

    /* x * sqrt(var + eps) + mean per latent channel, then 2x2 unpatchify, then the 1x1 post-quant conv */
    for (int c = 0; c < lc; c++) {
        float sd = sqrtf(bn_var[c] + v->eps);
        for (int i = 0; i < h * w; i++) y[(size_t)c * h * w + i] = latent[(size_t)c * h * w + i] * sd + bn_mean[c];
    }
    fo_unpatchify(x, y, zc, h, w, 2);
    fo_conv2d(y, x, pqw, pqb, zc, zc, H, W, 1, 0);
    fo_conv2d(x, y, ciw, cib, zc, mid, H, W, 3, 1);

    int rc = 0;
    rc |= resblock(v, "decoder.mid_block.resnets.0", y, x, mid, mid, H, W);
    rc |= attnblock(v, "decoder.mid_block.attentions.0", x, y, mid, H, W);
    rc |= resblock(v, "decoder.mid_block.resnets.1", y, x, mid, mid, H, W);
    { float *t = x; x = y; y = t; }

    int prev = mid;
    for (int level = 3; level >= 0 && !rc; level--) {
        int ch = base * mult[level];
        char name[128];
        for (int r = 0; r < 3; r++) {
            snprintf(name, sizeof name, "decoder.up_blocks.%d.resnets.%d", 3 - level, r);
            rc |= resblock(v, name, y, x, r == 0 ? prev : ch, ch, H, W);
            { float *t = x; x = y; y = t; }
        }
        if (level > 0) {
            snprintf(name, sizeof name, "decoder.up_blocks.%d.upsamplers.0.conv", 3 - level);
            const float *uw = find(v, name, ".weight", (int64_t)ch * ch * 9, &err), *ub = find(v, name, ".bias", ch, &err);
            if (err) { rc = -1; break; }
            fo_upsample_nearest(y, x, ch, H, W);
            H *= 2; W *= 2;
            fo_conv2d(x, y, uw, ub, ch, ch, H, W, 3, 1);
        }
        prev = ch;
    }
    if (!rc) {
        fo_group_norm(y, x, now_, nob, base, H, W, 32, v->eps);
        swish(y, (size_t)base * H * W);
        fo_conv2d(x, y, cow, cob, base, 3, H, W, 3, 1);
        if (rgb_f32) memcpy(rgb_f32, x, sizeof(float) * 3 * (size_t)H * W);
        if (rgb_u8)
            for (int i = 0; i < H * W; i++)
                for (int c = 0; c < 3; c++) {
                    float val = (x[(size_t)c * H * W + i] + 1.0f) * 0.5f * 255.0f;
                    if (val < 0) val = 0;
                    if (val > 255) val = 255;
                    rgb_u8[(size_t)i * 3 + c] = (uint8_t)val;
                }
    }
    free(x); free(y);
    return rc ? -1 : 0;
}

/* image [3, H, W] in [-1, 1] -> normalised latent [128, H/16, W/16] (flux_vae_encode,
 * flux_vae.c:320-443): conv_in, four levels of two residual blocks with a stride-2 convolution
 * after each of the first three, mid block (residual, attention, residual), group norm, swish,
 * conv_out to 64 channels, 1x1 quant conv, the first 32 channels (the mean of the posterior), 2x2
 * patchify, (x - running_mean) / sqrt(running_var + eps) per latent channel
 * (flux_kernels.c:555-575 without affine). H and W must be multiples of 16. Returns 0, or -1 when
 * a tensor is missing or the size does not fit. */
int fo_vae_encode(const fo_vae *v, const float *img, int H, int W, float *latent) {
    static const int mult[4] = {1, 2, 4, 4};
    const int zc = 32, lc = 128, base = v->base, mid = base * mult[3];
    if (H <= 0 || W <= 0 || H % 16 || W % 16) return -1;
    int err = 0;
    const float *bn_mean = find(v, "bn.running_mean", "", lc, &err), *bn_var = find(v, "bn.running_var", "", lc, &err);
    const float *ciw = find(v, "encoder.conv_in.weight", "", (int64_t)base * 3 * 9, &err), *cib = find(v, "encoder.conv_in.bias", "", base, &err);
    const float *now_ = find(v, "encoder.conv_norm_out.weight", "", mid, &err), *nob = find(v, "encoder.conv_norm_out.bias", "", mid, &err);
    const float *cow = find(v, "encoder.conv_out.weight", "", (int64_t)2 * zc * mid * 9, &err), *cob = find(v, "encoder.conv_out.bias", "", 2 * zc, &err);
    const float *qw = find(v, "quant_conv.weight", "", (int64_t)4 * zc * zc, &err), *qb = find(v, "quant_conv.bias", "", 2 * zc, &err);
    if (err) return -1;

    size_t cap = (size_t)base * H * W;                          /* level 0 is the largest: base channels at full size */
    if (cap < (size_t)2 * zc * (H / 8) * (W / 8)) cap = (size_t)2 * zc * (H / 8) * (W / 8);
    float *x = (float *)malloc(sizeof(float) * cap), *y = (float *)malloc(sizeof(float) * cap);
    fo_conv2d(x, img, ciw, cib, 3, base, H, W, 3, 1);

    int rc = 0, prev = base;
    char name[128];
    for (int level = 0; level < 4 && !rc; level++) {
        const int ch = base * mult[level];
        for (int r = 0; r < 2; r++) {
            snprintf(name, sizeof name, "encoder.down_blocks.%d.resnets.%d", level, r);
            rc |= resblock(v, name, y, x, r == 0 ? prev : ch, ch, H, W);
            { float *t = x; x = y; y = t; }
        }
        if (level < 3) {
            snprintf(name, sizeof name, "encoder.down_blocks.%d.downsamplers.0.conv", level);
            const float *dw = find(v, name, ".weight", (int64_t)ch * ch * 9, &err), *db = find(v, name, ".bias", ch, &err);
            if (err) { rc = -1; break; }
            fo_conv2d_down(y, x, dw, db, ch, ch, H, W);
            H = (H + 1 - 3) / 2 + 1; W = (W + 1 - 3) / 2 + 1;
            { float *t = x; x = y; y = t; }
        }
        prev = ch;
    }
    if (!rc) rc |= resblock(v, "encoder.mid_block.resnets.0", y, x, mid, mid, H, W);
    if (!rc) rc |= attnblock(v, "encoder.mid_block.attentions.0", x, y, mid, H, W);
    if (!rc) rc |= resblock(v, "encoder.mid_block.resnets.1", y, x, mid, mid, H, W);
    if (!rc) {
        fo_group_norm(x, y, now_, nob, mid, H, W, 32, v->eps);
        swish(x, (size_t)mid * H * W);
        fo_conv2d(y, x, cow, cob, mid, 2 * zc, H, W, 3, 1);
        fo_conv2d(x, y, qw, qb, 2 * zc, 2 * zc, H, W, 1, 0);
        /* the first zc channels are the posterior's mean: they are the first zc planes of x */
        fo_patchify(y, x, zc, H, W, 2);
        const int h = H / 2, w = W / 2;
        for (int c = 0; c < lc; c++) {
            const float inv = 1.0f / sqrtf(bn_var[c] + v->eps);
            for (int i = 0; i < h * w; i++) latent[(size_t)c * h * w + i] = (y[(size_t)c * h * w + i] - bn_mean[c]) * inv;
        }
    }
    free(x); free(y);
    return rc ? -1 : 0;
}
