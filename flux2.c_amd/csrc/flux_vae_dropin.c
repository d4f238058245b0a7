/*
 * flux_vae_dropin.c - the reference's VAE entry points as flux.c binds them (flux.c:36-43) over
 * the device VAE: flux_vae_load_safetensors, flux_vae_decode, flux_vae_encode, flux_vae_free.
 *
 * An application keeps its flux_vae.c (flux_image_to_tensor lives there) and compiles that one
 * file with
 *     -Dflux_vae_load_safetensors=flux_vae_load_safetensors_cpu
 *     -Dflux_vae_decode=flux_vae_decode_cpu -Dflux_vae_free=flux_vae_free_cpu
 *     -Dflux_vae_encode=flux_vae_encode_cpu
 * so that the four names resolve here. Leaving the last one out keeps the reference's CPU encoder:
 * the handle handed back to flux.c is then the reference's own flux_vae_t, which that encoder
 * needs, and the device VAE is kept beside it. Otherwise the handle is the device VAE itself.
 * There is no fallback: when the device fails, flux_vae_decode and flux_vae_encode return NULL.
 */
#include "../../include/flux_hip.h"
#include "host_internal.h"
#include <stdlib.h>
#include <string.h>

typedef struct { int width, height, channels; uint8_t *data; } dropin_image; /* flux_image, flux.h:73-78 */

extern void *flux_vae_load_safetensors_cpu(void *sf) __attribute__((weak));
extern void flux_vae_free_cpu(void *vae) __attribute__((weak));
extern float *flux_vae_encode_cpu(void *vae, const float *img, int batch, int H, int W, int *out_h, int *out_w) __attribute__((weak));
typedef void (*vae_progress_fn)(int block, int total);
extern vae_progress_fn flux_vae_progress_callback __attribute__((weak)); /* flux_kernels.h:292-293 */

#define MAX_VAES 16
static struct { void *handle; flux_hip_vae *dev; } g_vaes[MAX_VAES];

void *flux_vae_load_safetensors(void *sf) {
    int slot = -1;
    for (int i = 0; i < MAX_VAES; i++)
        if (!g_vaes[i].handle) { slot = i; break; }
    if (slot < 0) { flux_hip_fail("flux_vae_load_safetensors: too many VAEs are loaded"); return NULL; }
    flux_hip_vae *dev = flux_hip_vae_load_safetensors(sf);
    if (!dev) return NULL;
    void *handle = dev;
    if (flux_vae_load_safetensors_cpu && !flux_vae_encode_cpu) { /* the application's CPU encoder is in use */
        handle = flux_vae_load_safetensors_cpu(sf);
        if (!handle) { flux_hip_vae_free(dev); return NULL; }
    }
    g_vaes[slot].handle = handle;
    g_vaes[slot].dev = dev;
    return handle;
}

static int find_vae(void *vae) {
    for (int i = 0; i < MAX_VAES; i++)
        if (vae && g_vaes[i].handle == vae) return i;
    return -1;
}

/* flux_vae_decode, flux_vae.c:690: the first image of the batch as 8-bit RGB, caller frees with
 * flux_image_free (free of the pixel block and of the struct, flux_image.c:39-44). */
void *flux_vae_decode(void *vae, const float *latent, int batch, int latent_h, int latent_w) {
    const int slot = find_vae(vae);
    if (slot < 0) { flux_hip_fail("flux_vae_decode: unknown VAE handle"); return NULL; }
    if (batch < 1 || !latent) { flux_hip_fail("flux_vae_decode: bad arguments"); return NULL; }
    dropin_image *img = (dropin_image *)malloc(sizeof *img);
    if (!img) return NULL;
    img->width = 16 * latent_w;
    img->height = 16 * latent_h;
    img->channels = 3;
    img->data = (uint8_t *)malloc((size_t)img->width * img->height * 3);
    if (!img->data) { free(img); return NULL; }
    flux_hip_vae_progress = &flux_vae_progress_callback ? flux_vae_progress_callback : NULL;
    const int ok = flux_hip_vae_decode(g_vaes[slot].dev, latent, latent_h, latent_w, img->data, NULL);
    flux_hip_vae_progress = NULL;
    if (!ok) { free(img->data); free(img); return NULL; }
    return img;
}

/* flux_vae_encode, flux_vae.c:320: image [1, 3, H, W] in [-1, 1] -> normalised latent
 * [128, H/16, W/16], caller frees. */
float *flux_vae_encode(void *vae, const float *img, int batch, int H, int W, int *out_h, int *out_w) {
    const int slot = find_vae(vae);
    if (slot < 0) { flux_hip_fail("flux_vae_encode: unknown VAE handle"); return NULL; }
    if (batch != 1 || !img || !out_h || !out_w) { flux_hip_fail("flux_vae_encode: bad arguments (one image at a time)"); return NULL; }
    if (H <= 0 || W <= 0 || (H & 15) || (W & 15)) { flux_hip_fail("flux_vae_encode: image %d x %d, sides must be multiples of 16", H, W); return NULL; }
    float *latent = (float *)malloc(sizeof(float) * 128 * (size_t)(H / 16) * (W / 16));
    if (!latent) return NULL;
    flux_hip_vae_progress = &flux_vae_progress_callback ? flux_vae_progress_callback : NULL;
    const int ok = flux_hip_vae_encode(g_vaes[slot].dev, img, H, W, latent);
    flux_hip_vae_progress = NULL;
    if (!ok) { free(latent); return NULL; }
    *out_h = H / 16;
    *out_w = W / 16;
    return latent;
}

void flux_vae_free(void *vae) {
    const int slot = find_vae(vae);
    if (slot < 0) return;
    flux_hip_vae_free(g_vaes[slot].dev);
    if (flux_vae_free_cpu && vae != (void *)g_vaes[slot].dev) flux_vae_free_cpu(vae);
    g_vaes[slot].handle = NULL;
    g_vaes[slot].dev = NULL;
}
