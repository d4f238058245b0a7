/* Private host-side structures shared by the transformer, sampler and loader files. */
#ifndef FLUX_HIP_HOST_INTERNAL_H
#define FLUX_HIP_HOST_INTERNAL_H

#include "../../include/flux_hip.h"

#ifdef __cplusplus
extern "C" {
#endif

#define FH_MAX_REFS 8
#define FH_ROPE_SLOTS 4

/* Double-stream block: index 0 = text stream, 1 = image stream. */
typedef struct {
    void *qkv[2];      /* bf16 [3H, H]: rows Q, K, V */
    float *norm_q[2];  /* f32 [128] */
    float *norm_k[2];
    void *proj[2];     /* bf16 [H, H] */
    void *ff_in[2];    /* bf16 [2M, H]: rows gate, up */
    void *ff_out[2];   /* bf16 [H, M] */
} fh_double;

typedef struct {
    float *norm_q, *norm_k;
    void *qkv_mlp;     /* bf16 [3H + 2M, H]: rows Q, K, V, gate, up */
    void *out;         /* bf16 [H, H + M] */
} fh_single;

/* RoPE table of one token layout [text ; target ; refs], f32 [n, 128] on the device. */
typedef struct {
    float *cos, *sin;
    int txt_seq, h, w, num_refs;
    int ref_h[FH_MAX_REFS], ref_w[FH_MAX_REFS], ref_t[FH_MAX_REFS];
    int n_img, n;
} fh_rope;

struct flux_transformer {
    flux_hip_config c;
    int complete;
    void *img_in, *txt_in, *t_fc1, *t_fc2, *proj_out;
    void *mod_w[4]; /* text 6H, image 6H, single 3H, final 2H rows, each [., H] bf16 */
    fh_double *dbl;
    fh_single *sgl;
    /* work buffers for cap_tokens tokens */
    int cap_tokens;
    float *x;                      /* f32 [n, H] residual stream */
    void *xn, *qkv, *kn, *cat, *tok;
    fh_rope rope[FH_ROPE_SLOTS];
    int rope_next;
    /* per-schedule modulation */
    float *mod, *temb, *sincos;
    int mod_cap, mod_steps;
    void *owned_sf; /* reference safetensors handle owned in mmap mode */
    int session_active; /* work buffers, RoPE tables and modulation belong to one run at a time */
};

/* Four HIP events per forward: start, after double blocks, after single blocks, end. */
typedef struct fh_events fh_events;
void fh_event_record(fh_events *ev, int which);

int fh_model_complete(flux_transformer_t *tf);
int fh_ensure_workspace(flux_transformer_t *tf, int tokens);
fh_rope *fh_get_rope(flux_transformer_t *tf, int txt_seq, int img_h, int img_w, const flux_ref_t *refs, int num_refs);
int fh_compute_modulation(flux_transformer_t *tf, const float *timesteps, int steps);
int fh_forward_device(flux_transformer_t *tf, const fh_rope *rp, const float *z_dev, int n_target,
                      const void *txt_dev, int step, float *v_dev, fh_events *ev);
int fh_forward_device_n(flux_transformer_t *tf, int nb, const fh_rope *const *rp, const float *z_dev, int n_target,
                        const void *const *txt_dev, int step, float *const *v_dev, fh_events *ev);
int flux_hip_fail(const char *fmt, ...);

/* safetensors access shared by the transformer and VAE loaders (flux_loader_hip.c) */
enum { FH_DT_F32 = 0, FH_DT_F16 = 1, FH_DT_BF16 = 2 }; /* the reference's numbering, flux_safetensors.h:20-28 */
typedef int (*fh_tensor_cb)(void *ctx, const char *name, int dtype, const void *data, int64_t numel);
int fh_safetensors_walk(const char *path, fh_tensor_cb cb, void *ctx);
/* the same over the reference's parsed-file handle (safetensors_file_t, flux_safetensors.h:31-49) */
int fh_safetensors_walk_handle(void *sf, fh_tensor_cb cb, void *ctx);
/* element i of a tensor of the given dtype as fp32 */
float fh_tensor_value(int dtype, const void *data, int64_t i);

#ifdef __cplusplus
}
#endif
/* runtime.hip: a result copied to the host part by part while later work runs (see there) */
int flux_hip_download_part_begin(int part, size_t stage_offset, size_t stage_total, const void *src, size_t bytes);
const void *flux_hip_download_part_wait(int part);

#endif
