/*
 * flux_vae_dropin.c - the reference's VAE entry points as flux.c binds them (flux.c:36-43)
 * with the decoder on the device: flux_vae_load_safetensors, flux_vae_decode, flux_vae_free.
 *
 * The encoder (image-to-image input) stays the reference's CPU code. An application keeps its
 * flux_vae.c and compiles that one file with
 *     -Dflux_vae_load_safetensors=flux_vae_load_safetensors_cpu
 *     -Dflux_vae_decode=flux_vae_decode_cpu -Dflux_vae_free=flux_vae_free_cpu
 * so that the three names resolve here. The handle handed back to flux.c is still the reference's
 * own flux_vae_t (flux_vae_encode needs it); the device decoder is kept beside it. Without a CPU
 * VAE in the link the handle is the device decoder itself.
 * There is no fallback: when the device decoder fails, flux_vae_decode returns NULL.
 */
#include "../../include/flux_hip.h"
#include "host_internal.h"
#include <stdlib.h>
#include <string.h>

typedef struct { int width, height, channels; uint8_t *data; } dropin_image; /* flux_image, flux.h:73-78 */

extern void *flux_vae_load_safetensors_cpu(void *sf) __attribute__((weak));
extern void flux_vae_free_cpu(void *vae) __attribute__((weak));
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
    if (flux_vae_load_safetensors_cpu) {
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

void flux_vae_free(void *vae) {
    const int slot = find_vae(vae);
    if (slot < 0) return;
    flux_hip_vae_free(g_vaes[slot].dev);
    if (flux_vae_free_cpu && vae != (void *)g_vaes[slot].dev) flux_vae_free_cpu(vae);
    g_vaes[slot].handle = NULL;
    g_vaes[slot].dev = NULL;
}
