/*
 * flux_sample_hip.c - samplers and the single-forward entry points on MI355X.
 *
 * Exports everything the reference's flux_sample.c exports, with the same signatures: the
 * Euler / CFG samplers (flux_sample.c:212, 303, 381, 457, 534, 615), the noise-injecting and
 * Heun samplers (:697, :760), the schedules (:49, 62, 75, 96, 145), flux_init_noise (:837),
 * flux_generate_latent (:891) and the timing and progress globals. The loop itself is device
 * resident: latent, text and reference tokens are uploaded once, every step's latent update
 * runs as a kernel (z += dt v, or the CFG combine), and the latent comes back once at the end.
 * The host thread only queues work; step callbacks therefore fire at queue time.
 */
#include "../../include/flux_hip.h"
#include "../../include/flux_hip_debug.h"
#include "host_internal.h"
#include <hip/hip_runtime_api.h>
#include <math.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

double flux_timing_transformer_total = 0.0;
double flux_timing_transformer_double = 0.0;
double flux_timing_transformer_single = 0.0;
double flux_timing_transformer_final = 0.0;

void flux_reset_timing(void) {
    flux_timing_transformer_total = flux_timing_transformer_double = 0.0;
    flux_timing_transformer_single = flux_timing_transformer_final = 0.0;
}

/* ------------------------------------------------------------------ schedules */

float *flux_linear_schedule(int num_steps) {
    float *s = (float *)malloc((num_steps + 1) * sizeof(float));
    for (int i = 0; i <= num_steps; i++) s[i] = 1.0f - (float)i / (float)num_steps;
    return s;
}

float *flux_power_schedule(int num_steps, float alpha) {
    float *s = (float *)malloc((num_steps + 1) * sizeof(float));
    for (int i = 0; i <= num_steps; i++) s[i] = 1.0f - powf((float)i / (float)num_steps, alpha);
    return s;
}

/* mu from two line fits in the image sequence length, then t -> e^mu / (e^mu + (1/t - 1))
 * (flux_sample.c:122-155). */
float *flux_official_schedule(int num_steps, int image_seq_len) {
    const float a1 = 8.73809524e-05f, b1 = 1.89833333f, a2 = 0.00016927f, b2 = 0.45666666f;
    float mu;
    if (image_seq_len > 4300) {
        mu = a2 * image_seq_len + b2;
    } else {
        float m200 = a2 * image_seq_len + b2, m10 = a1 * image_seq_len + b1;
        float a = (m200 - m10) / 190.0f;
        mu = a * num_steps + (m200 - 200.0f * a);
    }
    float *s = (float *)malloc((num_steps + 1) * sizeof(float));
    for (int i = 0; i <= num_steps; i++) {
        float t = 1.0f - (float)i / (float)num_steps;
        if (t <= 0.0f) s[i] = 0.0f;
        else if (t >= 1.0f) s[i] = 1.0f;
        else s[i] = expf(mu) / (expf(mu) + (1.0f / t - 1.0f));
    }
    return s;
}

/* 1 - sigmoid(10 (i/n - 1/2) + shift), endpoints forced to 1 and 0 (flux_sample.c:75-91). */
float *flux_sigmoid_schedule(int num_steps, float shift) {
    float *s = (float *)malloc((num_steps + 1) * sizeof(float));
    for (int i = 0; i <= num_steps; i++) {
        float x = ((float)i / (float)num_steps - 0.5f) * 10.0f + shift;
        s[i] = 1.0f - 1.0f / (1.0f + expf(-x));
    }
    s[0] = 1.0f;
    s[num_steps] = 0.0f;
    return s;
}

/* 1 - (i/n)^(1 + shift/2) with shift 1 from 1024x1024 pixels up, 0.5 from 512x512 up, else 0
 * (flux_sample.c:96-116). */
float *flux_resolution_schedule(int num_steps, int height, int width) {
    const int pixels = height * width;
    const float shift = pixels >= 1024 * 1024 ? 1.0f : pixels >= 512 * 512 ? 0.5f : 0.0f;
    float *s = (float *)malloc((num_steps + 1) * sizeof(float));
    for (int i = 0; i <= num_steps; i++) s[i] = 1.0f - powf((float)i / (float)num_steps, 1.0f + shift * 0.5f);
    return s;
}

/* ------------------------------------------------------------------ initial noise */

/* Host RNG of the reference: SplitMix64-seeded xoshiro256** and Box-Muller (flux_kernels.c:45-102),
 * exported under the reference's names. In a process that also links the reference's
 * flux_kernels.c the executable's definitions take precedence at load time, here too, so an
 * unseeded call continues the stream the application seeded (main.c:254). */
static uint64_t rng_s[4] = {0x853c49e6748fea9bULL, 0xda3e39cb94b95bdbULL, 0x647c4677a2884327ULL, 0xc6e7918d2e2969f5ULL};
static uint64_t rotl64(uint64_t x, int k) { return (x << k) | (x >> (64 - k)); }
static uint64_t rng_next(void) {
    const uint64_t r = rotl64(rng_s[1] * 5, 7) * 9, t = rng_s[1] << 17;
    rng_s[2] ^= rng_s[0]; rng_s[3] ^= rng_s[1]; rng_s[1] ^= rng_s[2]; rng_s[0] ^= rng_s[3];
    rng_s[2] ^= t; rng_s[3] = rotl64(rng_s[3], 45);
    return r;
}
void flux_rng_seed(uint64_t seed) {
    for (int i = 0; i < 4; i++) {
        seed += 0x9e3779b97f4a7c15ULL;
        uint64_t z = seed;
        z = (z ^ (z >> 30)) * 0xbf58476d1ce4e5b9ULL;
        z = (z ^ (z >> 27)) * 0x94d049bb133111ebULL;
        rng_s[i] = z ^ (z >> 31);
    }
}
static float rng_uniform(void) { return (rng_next() >> 11) * (1.0 / 9007199254740992.0); }
void flux_randn(float *out, int n) {
    for (int i = 0; i < n; i++) {
        float u1 = rng_uniform(), u2 = rng_uniform();
        while (u1 == 0.0f) u1 = rng_uniform();
        out[i] = sqrtf(-2.0f * logf(u1)) * cosf(2.0f * 3.14159265358979323846f * u2);
    }
}

/* Noise is drawn at 112 x 112 and subsampled (nearest) so that a seed gives similar compositions
 * at every resolution (flux_sample.c:837-877). Returns malloc'd [batch, channels, h, w]. */
float *flux_init_noise(int batch, int channels, int h, int w, int64_t seed) {
    const int MAXD = 112;
    const int n = batch * channels * h * w;
    float *noise = (float *)malloc((size_t)n * sizeof(float));
    if (!noise) return NULL;
    if (seed >= 0) flux_rng_seed((uint64_t)seed);
    if (h >= MAXD && w >= MAXD) { flux_randn(noise, n); return noise; }
    const int big_n = batch * channels * MAXD * MAXD;
    float *big = (float *)malloc((size_t)big_n * sizeof(float));
    if (!big) { free(noise); return NULL; }
    flux_randn(big, big_n);
    for (int bc = 0; bc < batch * channels; bc++)
        for (int y = 0; y < h; y++)
            for (int x = 0; x < w; x++)
                noise[((size_t)bc * h + y) * w + x] = big[((size_t)bc * MAXD + y * MAXD / h) * MAXD + x * MAXD / w];
    free(big);
    return noise;
}

/* ------------------------------------------------------------------ stage timing */

#define EV_MAX_FORWARDS 512
struct fh_events {
    hipEvent_t e[EV_MAX_FORWARDS][4];
    int created, used;
};
static struct fh_events g_events;

void fh_event_record(fh_events *ev, int which) {
    if (ev->used >= EV_MAX_FORWARDS) return;
    hipEventRecord(ev->e[ev->used][which], (hipStream_t)flux_hip_stream());
}

static fh_events *events_begin(int forwards) {
    if (forwards > EV_MAX_FORWARDS) return NULL;
    while (g_events.created < forwards) {
        for (int k = 0; k < 4; k++)
            if (hipEventCreate(&g_events.e[g_events.created][k]) != hipSuccess) return NULL;
        g_events.created++;
    }
    g_events.used = 0;
    return &g_events;
}

static void events_collect(fh_events *ev) {
    if (!ev) return;
    for (int i = 0; i < ev->used; i++) {
        float d = 0, s = 0, f = 0;
        hipEventElapsedTime(&d, ev->e[i][0], ev->e[i][1]);
        hipEventElapsedTime(&s, ev->e[i][1], ev->e[i][2]);
        hipEventElapsedTime(&f, ev->e[i][2], ev->e[i][3]);
        flux_timing_transformer_double += d;
        flux_timing_transformer_single += s;
        flux_timing_transformer_final += f;
        flux_timing_transformer_total += d + s + f;
    }
}

/* ------------------------------------------------------------------ the loop */

/* Uploads fp32 host data and leaves it on the device as bf16. */
static void *upload_as_bf16(const float *src, size_t n) {
    float *tmp = (float *)flux_hip_malloc(n * 4);
    void *dst = flux_hip_malloc(n * 2);
    int ok = tmp && dst && flux_hip_upload(tmp, src, n * 4) && flux_hip_f32_to_bf16(dst, tmp, n) && flux_hip_sync();
    flux_hip_free(tmp);
    if (!ok) { flux_hip_free(dst); return NULL; }
    return dst;
}

/* Puts the reference images' tokens behind the target's in tf->tok. */
static int upload_ref_tokens(flux_transformer_t *tf, int n_target, const flux_ref_t *refs, int num_refs) {
    const int C = tf->c.channels;
    int row = n_target;
    for (int r = 0; r < num_refs; r++) {
        int n = refs[r].h * refs[r].w;
        if (!refs[r].latent || n <= 0) return flux_hip_fail("reference image %d is empty", r);
        float *tmp = (float *)flux_hip_malloc((size_t)n * C * 4);
        int ok = tmp && flux_hip_upload(tmp, refs[r].latent, (size_t)n * C * 4) &&
                 flux_hip_latent_to_tokens((char *)tf->tok + (size_t)row * C * 2, tmp, C, n) && flux_hip_sync();
        flux_hip_free(tmp);
        if (!ok) return 0;
        row += n;
    }
    return 1;
}

/* CFG steps run their two forwards as one batch of two sequences unless this is switched off
 * (comparison runs). */
static int g_batched_cfg = 1;
void flux_hip_set_batched_cfg(int on) { g_batched_cfg = on != 0; }

/* Device-resident state of one sampling run. */
struct flux_hip_session {
    flux_transformer_t *tf;
    fh_rope *rp_c, *rp_u;
    int cfg, batched, n_target, num_steps, next_forward, h, w;
    size_t n_lat;
    float guidance;
    float *schedule;
    float *z_dev, *v_c, *v_u;
    void *txt_c, *txt_u;
    fh_events *ev;
    int owns_tf;
};

void flux_hip_session_free(flux_hip_session *s) {
    if (!s) return;
    flux_hip_sync();
    flux_hip_free(s->z_dev); flux_hip_free(s->v_c); flux_hip_free(s->v_u);
    flux_hip_free(s->txt_c); flux_hip_free(s->txt_u);
    free(s->schedule);
    if (s->tf && s->owns_tf) s->tf->session_active = 0;
    free(s);
}

static flux_hip_session *session_begin_impl(void *transformer, const float *z, int channels, int h, int w,
                                            const flux_ref_t *refs, int num_refs,
                                            const float *text_emb_cond, int text_seq_cond,
                                            const float *text_emb_uncond, int text_seq_uncond, float guidance_scale,
                                            const float *schedule, int num_steps, int reset_timing) {
    flux_transformer_t *tf = (flux_transformer_t *)transformer;
    if (!tf || !z || !text_emb_cond || !schedule) { flux_hip_fail("sampler: NULL argument"); return NULL; }
    if (!fh_model_complete(tf)) return NULL;
    if (channels != tf->c.channels) { flux_hip_fail("sampler: %d channels, model has %d", channels, tf->c.channels); return NULL; }
    if (h <= 0 || w <= 0 || text_seq_cond <= 0 || num_steps < 0 || num_refs < 0) { flux_hip_fail("sampler: bad sizes"); return NULL; }
    if (num_refs > 0 && !refs) { flux_hip_fail("sampler: refs is NULL"); return NULL; }
    const int cfg = text_emb_uncond != NULL;
    if (cfg && text_seq_uncond <= 0) { flux_hip_fail("sampler: empty unconditional text"); return NULL; }

    if (tf->session_active) { flux_hip_fail("sampler: another run is active on this transformer"); return NULL; }
    flux_hip_session *s = (flux_hip_session *)calloc(1, sizeof(*s));
    if (!s) { flux_hip_fail("out of host memory"); return NULL; }
    tf->session_active = 1;
    s->owns_tf = 1;
    s->tf = tf; s->cfg = cfg; s->batched = cfg && g_batched_cfg; s->n_target = h * w; s->num_steps = num_steps; s->guidance = guidance_scale;
    s->h = h; s->w = w;
    s->n_lat = (size_t)channels * s->n_target;
    s->schedule = (float *)malloc((num_steps + 1) * sizeof(float));
    if (!s->schedule) { flux_hip_fail("out of host memory"); goto fail; }
    memcpy(s->schedule, schedule, (num_steps + 1) * sizeof(float));

    s->rp_c = fh_get_rope(tf, text_seq_cond, h, w, refs, num_refs);
    if (!s->rp_c) goto fail;
    int max_tokens = s->rp_c->n;
    if (cfg) {
        s->rp_u = fh_get_rope(tf, text_seq_uncond, h, w, refs, num_refs);
        if (!s->rp_u) goto fail;
        /* the table cache may have recycled the first slot */
        s->rp_c = fh_get_rope(tf, text_seq_cond, h, w, refs, num_refs);
        if (!s->rp_c) goto fail;
        max_tokens = s->batched ? max_tokens + s->rp_u->n : (s->rp_u->n > max_tokens ? s->rp_u->n : max_tokens);
    }
    if (!fh_ensure_workspace(tf, max_tokens)) goto fail;
    if (num_steps > 0 && !fh_compute_modulation(tf, schedule, num_steps)) goto fail;

    s->z_dev = (float *)flux_hip_malloc(s->n_lat * 4);
    s->v_c = (float *)flux_hip_malloc(s->n_lat * 4);
    s->v_u = cfg ? (float *)flux_hip_malloc(s->n_lat * 4) : NULL;
    s->txt_c = upload_as_bf16(text_emb_cond, (size_t)text_seq_cond * tf->c.text_dim);
    s->txt_u = cfg ? upload_as_bf16(text_emb_uncond, (size_t)text_seq_uncond * tf->c.text_dim) : NULL;
    if (!s->z_dev || !s->v_c || !s->txt_c || (cfg && (!s->v_u || !s->txt_u))) goto fail;
    if (!flux_hip_upload(s->z_dev, z, s->n_lat * 4)) goto fail;
    if (!upload_ref_tokens(tf, s->n_target, refs, num_refs)) goto fail;
    s->ev = events_begin(num_steps * (cfg ? 2 : 1));
    if (reset_timing) flux_reset_timing();
    return s;
fail:
    flux_hip_session_free(s);
    return NULL;
}

flux_hip_session *flux_hip_session_begin(void *transformer, const float *z, int channels, int h, int w,
                                         const flux_ref_t *refs, int num_refs,
                                         const float *text_emb_cond, int text_seq_cond,
                                         const float *text_emb_uncond, int text_seq_uncond, float guidance_scale,
                                         const float *schedule, int num_steps) {
    return session_begin_impl(transformer, z, channels, h, w, refs, num_refs, text_emb_cond, text_seq_cond, text_emb_uncond,
                              text_seq_uncond, guidance_scale, schedule, num_steps, 1);
}

int flux_hip_session_step(flux_hip_session *s, int step, float *v_trace) {
    if (!s || step < 0 || step >= s->num_steps) return flux_hip_fail("session step %d out of range", step);
    flux_transformer_t *tf = s->tf;
    const float dt = s->schedule[step + 1] - s->schedule[step];
    const size_t n = s->n_lat;
    if (flux_step_callback) flux_step_callback(step + 1, s->num_steps);
    if (s->batched) {
        /* the unconditional and the conditional pass (flux_sample.c:485-493) as one batch of two sequences */
        const fh_rope *rp[2] = {s->rp_u, s->rp_c};
        const void *txt[2] = {s->txt_u, s->txt_c};
        float *v[2] = {s->v_u, s->v_c};
        if (!fh_forward_device_n(tf, 2, rp, s->z_dev, s->n_target, txt, step, v, s->ev)) return 0;
        if (s->ev) s->ev->used++;
    } else if (s->cfg) {
        /* unconditional first, then conditional (flux_sample.c:485-493) */
        if (!fh_forward_device(tf, s->rp_u, s->z_dev, s->n_target, s->txt_u, step, s->v_u, s->ev)) return 0;
        if (s->ev) s->ev->used++;
        if (!fh_forward_device(tf, s->rp_c, s->z_dev, s->n_target, s->txt_c, step, s->v_c, s->ev)) return 0;
        if (s->ev) s->ev->used++;
    }
    if (s->cfg) {
        if (v_trace) {
            if (!flux_hip_download(v_trace, s->v_u, n * 4)) return 0;
            if (!flux_hip_download(v_trace + n, s->v_c, n * 4)) return 0;
        }
        return flux_hip_cfg_euler_update(s->z_dev, s->v_u, s->v_c, s->guidance, dt, n);
    }
    if (!fh_forward_device(tf, s->rp_c, s->z_dev, s->n_target, s->txt_c, step, s->v_c, s->ev)) return 0;
    if (s->ev) s->ev->used++;
    if (v_trace && !flux_hip_download(v_trace, s->v_c, n * 4)) return 0;
    return flux_hip_euler_update(s->z_dev, s->v_c, dt, n);
}

int flux_hip_session_read_latent(flux_hip_session *s, float *z_out) {
    if (!s || !z_out) return flux_hip_fail("session: NULL argument");
    if (!flux_hip_download(z_out, s->z_dev, s->n_lat * 4)) return 0;
    events_collect(s->ev);
    if (s->ev) s->ev->used = 0;
    return 1;
}

/* Intermediate-image hook of the reference (flux_sample.c:258-266): when the application has set
 * flux_step_image_callback and flux_step_image_vae (flux.c:161-164), every step but the last
 * hands the current latent to the application's own VAE decoder and the image to the callback.
 * The two globals and flux_image_free belong to the application (flux_kernels.c:35-36,
 * flux_image.c); they are weak here, and without them the hook does nothing. flux_vae_decode is
 * the application's own when it links one, else the device decoder's entry point of that name.
 * Each use waits for the device. */
struct flux_image;
typedef void (*fh_step_image_cb)(int step, int total, const struct flux_image *img);
extern fh_step_image_cb flux_step_image_callback __attribute__((weak));
extern void *flux_step_image_vae __attribute__((weak));
extern void flux_image_free(struct flux_image *img) __attribute__((weak));

static void step_image_hook(flux_hip_session *s, int step) {
    if (!&flux_step_image_callback || !&flux_step_image_vae || !flux_image_free) return;
    if (!flux_step_image_callback || !flux_step_image_vae || step + 1 >= s->num_steps) return;
    float *z = (float *)malloc(s->n_lat * 4);
    if (!z) return;
    if (flux_hip_download(z, s->z_dev, s->n_lat * 4)) {
        struct flux_image *img = (struct flux_image *)flux_vae_decode(flux_step_image_vae, z, 1, s->h, s->w);
        if (img) {
            flux_step_image_callback(step + 1, s->num_steps, img);
            flux_image_free(img);
        }
    }
    free(z);
}

static void print_stage_times(void) {
    if (flux_verbose)
        fprintf(stderr, "denoising on device: double %.2f ms, single %.2f ms, final %.2f ms, total %.2f ms\n",
                flux_timing_transformer_double, flux_timing_transformer_single, flux_timing_transformer_final,
                flux_timing_transformer_total);
}

static float *sample_impl(void *transformer, const float *z, int channels, int h, int w,
                          const flux_ref_t *refs, int num_refs,
                          const float *text_emb_cond, int text_seq_cond,
                          const float *text_emb_uncond, int text_seq_uncond, float guidance_scale,
                          const float *schedule, int num_steps, float *v_trace, void (*progress)(int, int)) {
    flux_hip_session *s = flux_hip_session_begin(transformer, z, channels, h, w, refs, num_refs, text_emb_cond,
                                                 text_seq_cond, text_emb_uncond, text_seq_uncond, guidance_scale,
                                                 schedule, num_steps);
    if (!s) return NULL;
    const size_t per_step = s->n_lat * (s->cfg ? 2 : 1);
    float *out = NULL;
    for (int i = 0; i < num_steps; i++) {
        if (!flux_hip_session_step(s, i, v_trace ? v_trace + (size_t)i * per_step : NULL)) goto done;
        if (progress) progress(i + 1, num_steps); /* the step has been queued (flux_sample.c:254) */
        step_image_hook(s, i);
    }
    out = (float *)malloc(s->n_lat * 4);
    if (!out) { flux_hip_fail("out of host memory"); goto done; }
    if (!flux_hip_session_read_latent(s, out)) { free(out); out = NULL; goto done; }
    print_stage_times();
done:
    flux_hip_session_free(s);
    return out;
}

/* Heun (flux_sample.c:760-826): v1 = f(z, t_i); z' = z + dt v1; v2 = f(z', t_{i+1});
 * z += dt/2 (v1 + v2); the last step is a plain Euler step. The modulation vectors of t_{i+1}
 * are those the next step uses, so they exist already. v_trace (optional) receives v1, v2 of
 * every step in call order: 2 * num_steps - 1 velocities. */
float *flux_hip_sample_heun_traced(void *transformer, const float *z, int channels, int h, int w,
                                   const float *text_emb, int text_seq, const float *schedule, int num_steps,
                                   float *v_trace, void (*progress)(int, int)) {
    flux_hip_session *s = flux_hip_session_begin(transformer, z, channels, h, w, NULL, 0, text_emb, text_seq, NULL, 0,
                                                 0.0f, schedule, num_steps);
    if (!s) return NULL;
    const size_t n = s->n_lat;
    float *out = NULL, *z_pred = NULL;
    size_t k = 0;
    s->ev = events_begin(2 * num_steps);
    z_pred = (float *)flux_hip_malloc(n * 4);
    s->v_u = (float *)flux_hip_malloc(n * 4); /* second velocity; released with the session */
    if (!z_pred || !s->v_u) goto done;
    for (int i = 0; i < num_steps; i++) {
        const float dt = schedule[i + 1] - schedule[i];
        if (!fh_forward_device(s->tf, s->rp_c, s->z_dev, s->n_target, s->txt_c, i, s->v_c, s->ev)) goto done;
        if (s->ev) s->ev->used++;
        if (v_trace && !flux_hip_download(v_trace + (k++) * n, s->v_c, n * 4)) goto done;
        if (i < num_steps - 1) {
            if (!flux_hip_euler_predict(z_pred, s->z_dev, s->v_c, dt, n)) goto done;
            if (!fh_forward_device(s->tf, s->rp_c, z_pred, s->n_target, s->txt_c, i + 1, s->v_u, s->ev)) goto done;
            if (s->ev) s->ev->used++;
            if (v_trace && !flux_hip_download(v_trace + (k++) * n, s->v_u, n * 4)) goto done;
            if (!flux_hip_heun_update(s->z_dev, s->v_c, s->v_u, dt, n)) goto done;
        } else if (!flux_hip_euler_update(s->z_dev, s->v_c, dt, n)) {
            goto done;
        }
        if (progress) progress(i + 1, num_steps);
        step_image_hook(s, i);
    }
    out = (float *)malloc(n * 4);
    if (!out) { flux_hip_fail("out of host memory"); goto done; }
    if (!flux_hip_session_read_latent(s, out)) { free(out); out = NULL; goto done; }
    print_stage_times();
done:
    flux_hip_free(z_pred);
    flux_hip_session_free(s);
    return out;
}

/* Euler with noise injection (flux_sample.c:697-748): after every step but the last,
 * z += eta sqrt(|dt|) N(0,1). The normals come from the host generator flux_randn, in the
 * order the reference draws them (nothing else draws during a run), but all at once before the
 * loop so that the loop itself never waits for the host. */
float *flux_hip_sample_ancestral_traced(void *transformer, const float *z, int channels, int h, int w,
                                        const float *text_emb, int text_seq, const float *schedule, int num_steps,
                                        float eta, float *v_trace, void (*progress)(int, int)) {
    flux_hip_session *s = flux_hip_session_begin(transformer, z, channels, h, w, NULL, 0, text_emb, text_seq, NULL, 0,
                                                 0.0f, schedule, num_steps);
    if (!s) return NULL;
    const size_t n = s->n_lat;
    const int draws = (eta > 0 && num_steps > 1) ? num_steps - 1 : 0;
    float *out = NULL, *noise_dev = NULL;
    if (draws) {
        if (n > 0x7fffffff) { flux_hip_fail("ancestral sampler: latent too large"); goto done; }
        float *noise = (float *)malloc((size_t)draws * n * 4);
        noise_dev = (float *)flux_hip_malloc((size_t)draws * n * 4);
        if (!noise || !noise_dev) { free(noise); flux_hip_fail("ancestral sampler: out of memory"); goto done; }
        for (int i = 0; i < draws; i++) flux_randn(noise + (size_t)i * n, (int)n);
        int ok = flux_hip_upload(noise_dev, noise, (size_t)draws * n * 4);
        free(noise);
        if (!ok) goto done;
    }
    for (int i = 0; i < num_steps; i++) {
        const float dt = schedule[i + 1] - schedule[i];
        if (!fh_forward_device(s->tf, s->rp_c, s->z_dev, s->n_target, s->txt_c, i, s->v_c, s->ev)) goto done;
        if (s->ev) s->ev->used++;
        if (v_trace && !flux_hip_download(v_trace + (size_t)i * n, s->v_c, n * 4)) goto done;
        if (!flux_hip_euler_update(s->z_dev, s->v_c, dt, n)) goto done;
        if (i < draws && !flux_hip_euler_update(s->z_dev, noise_dev + (size_t)i * n, eta * sqrtf(fabsf(dt)), n)) goto done;
        if (progress) progress(i + 1, num_steps);
        step_image_hook(s, i);
    }
    out = (float *)malloc(n * 4);
    if (!out) { flux_hip_fail("out of host memory"); goto done; }
    if (!flux_hip_session_read_latent(s, out)) { free(out); out = NULL; goto done; }
    print_stage_times();
done:
    flux_hip_free(noise_dev);
    flux_hip_session_free(s);
    return out;
}

float *flux_hip_sample_traced(void *transformer, const float *z, int channels, int h, int w,
                              const flux_ref_t *refs, int num_refs,
                              const float *text_emb_cond, int text_seq_cond,
                              const float *text_emb_uncond, int text_seq_uncond, float guidance_scale,
                              const float *schedule, int num_steps, float *v_trace) {
    return sample_impl(transformer, z, channels, h, w, refs, num_refs, text_emb_cond, text_seq_cond, text_emb_uncond,
                       text_seq_uncond, guidance_scale, schedule, num_steps, v_trace, NULL);
}

/* ------------------------------------------------------------------ reference-named entry points */

static float *run(void *tf, float *z, int batch, int channels, int h, int w, const flux_ref_t *refs, int num_refs,
                  const float *tc, int sc, const float *tu, int su, float g, const float *schedule, int steps,
                  void (*progress)(int, int)) {
    if (batch != 1) { flux_hip_fail("sampler: batch=%d (the pipeline always passes 1)", batch); return NULL; }
    return sample_impl(tf, z, channels, h, w, refs, num_refs, tc, sc, tu, su, g, schedule, steps, NULL, progress);
}

float *flux_sample_euler(void *transformer, void *text_encoder, float *z, int batch, int channels, int h, int w,
                         const float *text_emb, int text_seq, const float *schedule, int num_steps,
                         void (*progress_callback)(int step, int total)) {
    (void)text_encoder;
    return run(transformer, z, batch, channels, h, w, NULL, 0, text_emb, text_seq, NULL, 0, 0.0f, schedule, num_steps, progress_callback);
}

float *flux_sample_euler_with_refs(void *transformer, void *text_encoder, float *z, int batch, int channels, int h, int w,
                                   const float *ref_latent, int ref_h, int ref_w, int t_offset,
                                   const float *text_emb, int text_seq, const float *schedule, int num_steps,
                                   void (*progress_callback)(int step, int total)) {
    (void)text_encoder;
    flux_ref_t r = {ref_latent, ref_h, ref_w, t_offset};
    return run(transformer, z, batch, channels, h, w, &r, ref_latent ? 1 : 0, text_emb, text_seq, NULL, 0, 0.0f, schedule, num_steps, progress_callback);
}

float *flux_sample_euler_with_multi_refs(void *transformer, void *text_encoder, float *z, int batch, int channels, int h, int w,
                                         const flux_ref_t *refs, int num_refs,
                                         const float *text_emb, int text_seq, const float *schedule, int num_steps,
                                         void (*progress_callback)(int step, int total)) {
    (void)text_encoder;
    return run(transformer, z, batch, channels, h, w, refs, refs ? num_refs : 0, text_emb, text_seq, NULL, 0, 0.0f, schedule, num_steps, progress_callback);
}

float *flux_sample_euler_cfg(void *transformer, void *text_encoder, float *z, int batch, int channels, int h, int w,
                             const float *text_emb_cond, int text_seq_cond,
                             const float *text_emb_uncond, int text_seq_uncond, float guidance_scale,
                             const float *schedule, int num_steps, void (*progress_callback)(int step, int total)) {
    (void)text_encoder;
    if (!text_emb_uncond) { flux_hip_fail("cfg sampler: unconditional text is NULL"); return NULL; }
    return run(transformer, z, batch, channels, h, w, NULL, 0, text_emb_cond, text_seq_cond, text_emb_uncond, text_seq_uncond,
               guidance_scale, schedule, num_steps, progress_callback);
}

float *flux_sample_euler_cfg_with_refs(void *transformer, void *text_encoder, float *z, int batch, int channels, int h, int w,
                                       const float *ref_latent, int ref_h, int ref_w, int t_offset,
                                       const float *text_emb_cond, int text_seq_cond,
                                       const float *text_emb_uncond, int text_seq_uncond, float guidance_scale,
                                       const float *schedule, int num_steps, void (*progress_callback)(int step, int total)) {
    (void)text_encoder;
    if (!text_emb_uncond) { flux_hip_fail("cfg sampler: unconditional text is NULL"); return NULL; }
    flux_ref_t r = {ref_latent, ref_h, ref_w, t_offset};
    return run(transformer, z, batch, channels, h, w, &r, ref_latent ? 1 : 0, text_emb_cond, text_seq_cond, text_emb_uncond,
               text_seq_uncond, guidance_scale, schedule, num_steps, progress_callback);
}

float *flux_sample_euler_cfg_with_multi_refs(void *transformer, void *text_encoder, float *z, int batch, int channels, int h, int w,
                                             const flux_ref_t *refs, int num_refs,
                                             const float *text_emb_cond, int text_seq_cond,
                                             const float *text_emb_uncond, int text_seq_uncond, float guidance_scale,
                                             const float *schedule, int num_steps,
                                             void (*progress_callback)(int step, int total)) {
    (void)text_encoder;
    if (!text_emb_uncond) { flux_hip_fail("cfg sampler: unconditional text is NULL"); return NULL; }
    return run(transformer, z, batch, channels, h, w, refs, refs ? num_refs : 0, text_emb_cond, text_seq_cond, text_emb_uncond,
               text_seq_uncond, guidance_scale, schedule, num_steps, progress_callback);
}

float *flux_sample_heun(void *transformer, float *z, int batch, int channels, int h, int w,
                        const float *text_emb, int text_seq, const float *schedule, int num_steps,
                        void (*progress_callback)(int step, int total)) {
    if (batch != 1) { flux_hip_fail("sampler: batch=%d (the pipeline always passes 1)", batch); return NULL; }
    return flux_hip_sample_heun_traced(transformer, z, channels, h, w, text_emb, text_seq, schedule, num_steps, NULL,
                                       progress_callback);
}

float *flux_sample_euler_ancestral(void *transformer, float *z, int batch, int channels, int h, int w,
                                   const float *text_emb, int text_seq, const float *schedule, int num_steps,
                                   float eta, void (*progress_callback)(int step, int total)) {
    if (batch != 1) { flux_hip_fail("sampler: batch=%d (the pipeline always passes 1)", batch); return NULL; }
    return flux_hip_sample_ancestral_traced(transformer, z, channels, h, w, text_emb, text_seq, schedule, num_steps, eta,
                                            NULL, progress_callback);
}

/* Noise, linear schedule and the Euler sampler in one call (flux_sample.c:891-919). As in the
 * reference, the first argument is handed to the sampler as the transformer. */
float *flux_generate_latent(void *ctx_ptr, const float *text_emb, int text_seq, int height, int width, int num_steps,
                            int64_t seed, void (*progress_callback)(int step, int total)) {
    const int lh = height / 16, lw = width / 16, channels = 128;
    if (lh <= 0 || lw <= 0 || num_steps <= 0) { flux_hip_fail("flux_generate_latent: bad sizes"); return NULL; }
    float *z = flux_init_noise(1, channels, lh, lw, seed);
    float *schedule = flux_linear_schedule(num_steps);
    float *latent = (z && schedule) ? flux_sample_euler(ctx_ptr, NULL, z, 1, channels, lh, lw, text_emb, text_seq, schedule,
                                                        num_steps, progress_callback)
                                    : NULL;
    free(z);
    free(schedule);
    return latent;
}

/* Legacy step-progress global kept for source compatibility (flux_sample.c:926-930); the
 * reference never calls it either. */
void (*flux_progress_callback)(int, int) = NULL;
void flux_set_progress_callback(void (*callback)(int, int)) { flux_progress_callback = callback; }

/* One forward (flux_transformer.c:3115, 3605, 3815; used by flux_denoise_step, flux.c:1109): the
 * device state of a one-step run is set up, the forward is queued and its velocity read back. As in
 * the reference, a forward fires no step callback, moves no latent and adds its stage times to the
 * flux_timing_transformer_* counters instead of starting them afresh (flux_transformer.c:3561-3564);
 * the block-level flux_substep_callback fires as it does there. */
float *flux_transformer_forward_with_multi_refs(flux_transformer_t *tf, const float *img_latent, int img_h, int img_w,
                                                const flux_ref_t *refs, int num_refs,
                                                const float *txt_emb, int txt_seq, float timestep) {
    if (!tf || !img_latent || !txt_emb) { flux_hip_fail("forward: NULL argument"); return NULL; }
    if (img_h <= 0 || img_w <= 0 || txt_seq <= 0) { flux_hip_fail("forward: bad sizes"); return NULL; }
    const size_t n = (size_t)tf->c.channels * img_h * img_w;
    const float sched[2] = {timestep, timestep};
    flux_hip_session *s = session_begin_impl(tf, img_latent, tf->c.channels, img_h, img_w, refs, refs ? num_refs : 0, txt_emb,
                                             txt_seq, NULL, 0, 0.0f, sched, 1, 0);
    if (!s) return NULL;
    float *v = (float *)malloc(n * 4);
    if (!v) flux_hip_fail("out of host memory");
    if (v && fh_forward_device(tf, s->rp_c, s->z_dev, s->n_target, s->txt_c, 0, s->v_c, s->ev)) {
        if (s->ev) s->ev->used++;
        if (flux_hip_download(v, s->v_c, n * 4)) {
            events_collect(s->ev);
            flux_hip_session_free(s);
            return v;
        }
    }
    free(v);
    flux_hip_session_free(s);
    return NULL;
}

float *flux_transformer_forward(flux_transformer_t *tf, const float *img_latent, int img_h, int img_w,
                                const float *txt_emb, int txt_seq, float timestep) {
    return flux_transformer_forward_with_multi_refs(tf, img_latent, img_h, img_w, NULL, 0, txt_emb, txt_seq, timestep);
}

float *flux_transformer_forward_with_refs(flux_transformer_t *tf, const float *img_latent, int img_h, int img_w,
                                          const float *ref_latent, int ref_h, int ref_w, int t_offset,
                                          const float *txt_emb, int txt_seq, float timestep) {
    flux_ref_t r = {ref_latent, ref_h, ref_w, t_offset};
    return flux_transformer_forward_with_multi_refs(tf, img_latent, img_h, img_w, &r, ref_latent ? 1 : 0, txt_emb, txt_seq, timestep);
}
