/*
 * Stand-in for the application side of the reference's intermediate-image hook, for
 * tests/test_hip_samplers.py: defines the four symbols the sampler library looks up weakly
 * (flux_step_image_callback, flux_step_image_vae: flux_kernels.c:35-36; flux_vae_decode,
 * flux_image_free: used at flux_sample.c:258-266) and records what the library hands over.
 * Loaded with RTLD_GLOBAL before the library so that the weak references bind to it.
 */
#include <stdlib.h>
#include <string.h>

struct flux_image { int width, height; };
typedef void (*step_image_cb)(int step, int total, const struct flux_image *img);

step_image_cb flux_step_image_callback = 0;
void *flux_step_image_vae = 0;

#define SHIM_MAX 16
static float *g_latent[SHIM_MAX];
static int g_decodes = 0, g_frees = 0, g_calls = 0, g_step[SHIM_MAX], g_total[SHIM_MAX];
static struct flux_image g_img;
static int g_vae_token;

struct flux_image *flux_vae_decode(void *vae, const float *latent, int batch, int latent_h, int latent_w) {
    if (vae != &g_vae_token || g_decodes >= SHIM_MAX) return 0;
    size_t n = (size_t)batch * 128 * latent_h * latent_w;
    g_latent[g_decodes] = (float *)malloc(n * sizeof(float));
    memcpy(g_latent[g_decodes], latent, n * sizeof(float));
    g_decodes++;
    g_img.width = latent_w * 16;
    g_img.height = latent_h * 16;
    return &g_img;
}

void flux_image_free(struct flux_image *img) { if (img == &g_img) g_frees++; }

static void on_image(int step, int total, const struct flux_image *img) {
    if (g_calls < SHIM_MAX && img == &g_img) { g_step[g_calls] = step; g_total[g_calls] = total; g_calls++; }
}

void shim_enable(int on) {
    flux_step_image_callback = on ? on_image : 0;
    flux_step_image_vae = on ? (void *)&g_vae_token : 0;
}
int shim_decodes(void) { return g_decodes; }
int shim_frees(void) { return g_frees; }
int shim_calls(void) { return g_calls; }
int shim_step(int i) { return g_step[i]; }
int shim_total(int i) { return g_total[i]; }
const float *shim_latent(int i) { return g_latent[i]; }
