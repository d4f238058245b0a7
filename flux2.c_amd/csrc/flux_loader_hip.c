/*
 * flux_loader_hip.c - getting transformer weights onto the device.
 *
 * Two ways in:
 *  - flux_hip_transformer_load_file(): a self-contained reader for .safetensors files
 *    (8-byte little-endian header length, JSON header, raw data; flux_safetensors.h:4-8),
 *    mmap'd and uploaded tensor by tensor, bf16 staying bf16 (the zero-copy idea of
 *    safetensors_get_bf16_direct, flux_safetensors.c:407);
 *  - flux_transformer_load_safetensors[_mmap](): the reference's loader entry points
 *    (flux_transformer.c:4411, 4659), which receive the reference's own parsed file handle.
 *    Its layout (flux_safetensors.h:31-49) is mirrored below because that struct is the ABI.
 */
#include "../../include/flux_hip.h"
#include "host_internal.h"
#include <ctype.h>
#include <fcntl.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>
#include <sys/mman.h>
#include <sys/stat.h>
#include <unistd.h>

/* Converts fp32/fp16 host data to bf16 (round to nearest even) for tensors not stored as bf16. */
static uint16_t f32_to_bf16(float f) {
    uint32_t u;
    memcpy(&u, &f, 4);
    u += 0x7fffu + ((u >> 16) & 1u);
    return (uint16_t)(u >> 16);
}

static float f16_to_f32(uint16_t h) {
    uint32_t sign = (uint32_t)(h & 0x8000u) << 16, exp = (h >> 10) & 0x1f, man = h & 0x3ff, u;
    if (exp == 0) {
        if (man == 0) u = sign;
        else {
            int e = -1;
            do { man <<= 1; e++; } while (!(man & 0x400));
            u = sign | ((uint32_t)(112 - e) << 23) | ((man & 0x3ff) << 13);
        }
    } else if (exp == 31) u = sign | 0x7f800000u | (man << 13);
    else u = sign | ((exp + 112) << 23) | (man << 13);
    float f;
    memcpy(&f, &u, 4);
    return f;
}

enum { DT_F32 = FH_DT_F32, DT_F16 = FH_DT_F16, DT_BF16 = FH_DT_BF16 };

static int set_from(flux_transformer_t *tf, const char *name, int dtype, const void *data, int64_t numel) {
    if (dtype == DT_BF16) return flux_hip_transformer_set_tensor(tf, name, (const uint16_t *)data, numel);
    if (dtype != DT_F32 && dtype != DT_F16) return flux_hip_fail("tensor %s: unsupported dtype", name);
    uint16_t *tmp = (uint16_t *)malloc((size_t)numel * 2);
    if (!tmp) return flux_hip_fail("out of host memory");
    if (dtype == DT_F32)
        for (int64_t i = 0; i < numel; i++) tmp[i] = f32_to_bf16(((const float *)data)[i]);
    else
        for (int64_t i = 0; i < numel; i++) tmp[i] = f32_to_bf16(f16_to_f32(((const uint16_t *)data)[i]));
    int ok = flux_hip_transformer_set_tensor(tf, name, tmp, numel);
    free(tmp);
    return ok;
}

/* ---- minimal JSON walk over the safetensors header ---- */
static const char *skip_ws(const char *p, const char *e) { while (p < e && isspace((unsigned char)*p)) p++; return p; }

static const char *parse_string(const char *p, const char *e, char *out, size_t cap) {
    if (p >= e || *p != '"') return NULL;
    p++;
    size_t n = 0;
    while (p < e && *p != '"') {
        if (*p == '\\' && p + 1 < e) p++;
        if (n + 1 < cap) out[n++] = *p;
        p++;
    }
    if (p >= e) return NULL;
    out[n] = 0;
    return p + 1;
}

/* Skips one JSON value of any kind. */
static const char *skip_value(const char *p, const char *e) {
    p = skip_ws(p, e);
    if (p >= e) return NULL;
    if (*p == '"') { char tmp[8]; return parse_string(p, e, tmp, sizeof tmp); }
    if (*p == '{' || *p == '[') {
        int depth = 0;
        while (p < e) {
            if (*p == '"') { char tmp[8]; p = parse_string(p, e, tmp, sizeof tmp); if (!p) return NULL; continue; }
            if (*p == '{' || *p == '[') depth++;
            if (*p == '}' || *p == ']') { depth--; if (depth == 0) return p + 1; }
            p++;
        }
        return NULL;
    }
    while (p < e && *p != ',' && *p != '}' && *p != ']') p++;
    return p;
}

/* Walks a .safetensors file: calls cb(ctx, name, dtype, data, numel) for every tensor, in file
 * order. cb returns 0 to abort (after recording an error). Returns 1 when every call did. */
int fh_safetensors_walk(const char *path, fh_tensor_cb cb, void *ctx) {
    int fd = open(path, O_RDONLY);
    if (fd < 0) return flux_hip_fail("cannot open %s", path);
    struct stat sb;
    if (fstat(fd, &sb) != 0 || sb.st_size < 8) { close(fd); return flux_hip_fail("%s: not a safetensors file", path); }
    size_t fsize = (size_t)sb.st_size;
    char *map = (char *)mmap(NULL, fsize, PROT_READ, MAP_PRIVATE, fd, 0);
    close(fd);
    if (map == MAP_FAILED) return flux_hip_fail("%s: mmap failed", path);
    uint64_t hlen = 0;
    memcpy(&hlen, map, 8);
    if (hlen == 0 || hlen > fsize - 8) { flux_hip_fail("%s: bad header length", path); goto fail; }
    {
        const char *p = map + 8, *e = map + 8 + hlen, *data = e;
        size_t dsize = fsize - 8 - hlen;
        p = skip_ws(p, e);
        if (p >= e || *p != '{') { flux_hip_fail("%s: header is not a JSON object", path); goto fail; }
        p++;
        for (;;) {
            char name[256];
            p = skip_ws(p, e);
            if (p < e && *p == '}') break;
            p = parse_string(p, e, name, sizeof name);
            if (!p) { flux_hip_fail("%s: malformed header", path); goto fail; }
            p = skip_ws(p, e);
            if (p >= e || *p != ':') { flux_hip_fail("%s: malformed header", path); goto fail; }
            p++;
            p = skip_ws(p, e);
            if (!strcmp(name, "__metadata__") || p >= e || *p != '{') {
                p = skip_value(p, e);
                if (!p) { flux_hip_fail("%s: malformed header", path); goto fail; }
            } else {
                p++;
                char dtype[16] = "";
                int64_t numel = 1;
                uint64_t off0 = 0, off1 = 0;
                int have_off = 0;
                for (;;) {
                    char key[32];
                    p = skip_ws(p, e);
                    if (p < e && *p == '}') { p++; break; }
                    p = parse_string(p, e, key, sizeof key);
                    if (!p) { flux_hip_fail("%s: malformed entry %s", path, name); goto fail; }
                    p = skip_ws(p, e);
                    if (p >= e || *p != ':') { flux_hip_fail("%s: malformed entry %s", path, name); goto fail; }
                    p = skip_ws(p + 1, e);
                    if (!strcmp(key, "dtype")) {
                        p = parse_string(p, e, dtype, sizeof dtype);
                    } else if (!strcmp(key, "shape") || !strcmp(key, "data_offsets")) {
                        int is_shape = key[0] == 's';
                        if (p >= e || *p != '[') { flux_hip_fail("%s: malformed entry %s", path, name); goto fail; }
                        p++;
                        int idx = 0;
                        for (;;) {
                            p = skip_ws(p, e);
                            if (p < e && *p == ']') { p++; break; }
                            char *end;
                            unsigned long long v = strtoull(p, &end, 10);
                            if (end == p) { flux_hip_fail("%s: malformed entry %s", path, name); goto fail; }
                            p = end;
                            if (is_shape) {
                                /* no product of sizes in a file that fits an address space comes near 2^62 */
                                if (v > ((uint64_t)1 << 40) || (v && numel > (((int64_t)1 << 62) / (int64_t)v))) {
                                    flux_hip_fail("%s: tensor %s has an impossible shape", path, name);
                                    goto fail;
                                }
                                numel *= (int64_t)v;
                            } else if (idx == 0) { off0 = v; have_off = 1; }
                            else if (idx == 1) off1 = v;
                            else { flux_hip_fail("%s: tensor %s has more than two data offsets", path, name); goto fail; }
                            idx++;
                            p = skip_ws(p, e);
                            if (p < e && *p == ',') p++;
                        }
                    } else {
                        p = skip_value(p, e);
                    }
                    if (!p) { flux_hip_fail("%s: malformed entry %s", path, name); goto fail; }
                    p = skip_ws(p, e);
                    if (p < e && *p == ',') p++;
                }
                int dt = !strcmp(dtype, "BF16") ? DT_BF16 : !strcmp(dtype, "F32") ? DT_F32 : !strcmp(dtype, "F16") ? DT_F16 : -1;
                size_t esz = dt == DT_F32 ? 4 : 2;
                if (dt < 0) {   /* a type this library has no use for (integers, fp64, fp8): not handed on */
                    p = skip_ws(p, e);
                    if (p < e && *p == ',') p++;
                    continue;
                }
                if (!have_off || off1 < off0 || off1 > dsize || (off1 - off0) != (uint64_t)numel * esz) {
                    flux_hip_fail("%s: tensor %s has inconsistent offsets", path, name);
                    goto fail;
                }
                if (!cb(ctx, name, dt, data + off0, numel)) goto fail;
            }
            p = skip_ws(p, e);
            if (p < e && *p == ',') p++;
        }
    }
    munmap(map, fsize);
    return 1;
fail:
    munmap(map, fsize);
    return 0;
}

static int transformer_tensor_cb(void *ctx, const char *name, int dtype, const void *data, int64_t numel) {
    if (set_from((flux_transformer_t *)ctx, name, dtype, data, numel)) return 1;
    /* files may carry tensors this path does not use; only real failures abort */
    return strstr(flux_hip_last_error(), "is not part of the transformer") != NULL;
}

flux_transformer_t *flux_hip_transformer_load_file(const char *path, const flux_hip_config *cfg) {
    flux_hip_config c;
    if (cfg) c = *cfg; else flux_hip_default_config(&c);
    flux_transformer_t *tf = flux_hip_transformer_new(&c);
    if (!tf) return NULL;
    if (!fh_safetensors_walk(path, transformer_tensor_cb, tf) || !fh_model_complete(tf)) {
        flux_transformer_free(tf);
        return NULL;
    }
    return tf;
}

/* ---- the reference's parsed-file handle (flux_safetensors.h:31-49) ---- */
typedef struct {
    char name[256];
    int dtype; /* 0 F32, 1 F16, 2 BF16 (flux_safetensors.h:20-28) */
    int ndim;
    int64_t shape[8];
    size_t data_offset;
    size_t data_size;
} ref_safetensor;

typedef struct {
    char *path;
    void *data;
    size_t file_size;
    size_t header_size;
    char *header_json;
    int num_tensors;
    ref_safetensor tensors[512];
} ref_safetensors_file;

void fh_safetensors_close_compat(void *p) {
    /* what safetensors_close does (flux_safetensors.c:272-278) */
    ref_safetensors_file *sf = (ref_safetensors_file *)p;
    if (!sf) return;
    if (sf->data) munmap(sf->data, sf->file_size);
    free(sf->path);
    free(sf->header_json);
    free(sf);
}

/* Tensors of other types (integers, fp64, fp8, booleans: the reference's numbering goes on past 2,
 * flux_safetensors.h:20-28) are passed over, as the file walker above does; their element size is
 * not known here, so they are not sized either. */
static int usable_dtype(int dtype) { return dtype == DT_F32 || dtype == DT_F16 || dtype == DT_BF16; }

/* Entry i of a parsed handle: where its data lies and how many elements it has. The handle comes
 * from the reference's parser; what is checked here is that reading the entry stays inside the
 * mapping it describes. */
static int handle_entry(const ref_safetensors_file *sf, int i, const char **data, int64_t *numel) {
    const ref_safetensor *t = &sf->tensors[i];
    if (t->ndim < 0 || t->ndim > 8) return flux_hip_fail("safetensors handle: tensor %d has %d dimensions", i, t->ndim);
    int64_t n = 1;
    for (int d = 0; d < t->ndim; d++) {
        if (t->shape[d] < 0 || (t->shape[d] && n > (((int64_t)1 << 62) / t->shape[d]))) return flux_hip_fail("safetensors handle: tensor %.200s has an impossible shape", t->name);
        n *= t->shape[d];
    }
    const size_t esz = t->dtype == DT_F32 ? 4 : 2, head = 8 + sf->header_size;
    if (head > sf->file_size || t->data_offset > sf->file_size - head || (uint64_t)n * esz > sf->file_size - head - t->data_offset)
        return flux_hip_fail("safetensors handle: tensor %.200s lies outside its file", t->name);
    *data = (const char *)sf->data + head + t->data_offset;
    *numel = n;
    return 1;
}

int fh_safetensors_walk_handle(void *p, fh_tensor_cb cb, void *ctx) {
    ref_safetensors_file *sf = (ref_safetensors_file *)p;
    if (!sf || !sf->data) return flux_hip_fail("safetensors handle is NULL");
    if (sf->num_tensors < 0 || sf->num_tensors > 512) return flux_hip_fail("safetensors handle: bad tensor count");
    for (int i = 0; i < sf->num_tensors; i++) {
        const char *data;
        int64_t numel;
        if (!usable_dtype(sf->tensors[i].dtype)) continue;
        if (!handle_entry(sf, i, &data, &numel)) return 0;
        if (!cb(ctx, sf->tensors[i].name, sf->tensors[i].dtype, data, numel)) return 0;
    }
    return 1;
}

float fh_tensor_value(int dtype, const void *data, int64_t i) {
    if (dtype == DT_F32) return ((const float *)data)[i];
    if (dtype == DT_F16) return f16_to_f32(((const uint16_t *)data)[i]);
    uint32_t u = (uint32_t)((const uint16_t *)data)[i] << 16;
    float f;
    memcpy(&f, &u, 4);
    return f;
}

/* The reference fixes the architecture in its loader (flux_transformer.c:4418-4434). The file
 * itself says what it holds, so the sizes are read from the tensor shapes; a FLUX.2-klein-4B
 * file gives exactly the reference's constants, and a smaller model of the same family loads too. */
static const ref_safetensor *find_tensor(const ref_safetensors_file *sf, const char *name) {
    for (int i = 0; i < sf->num_tensors; i++)
        if (!strcmp(sf->tensors[i].name, name)) return &sf->tensors[i];
    return NULL;
}

static void infer_config(const ref_safetensors_file *sf, flux_hip_config *c) {
    const ref_safetensor *t;
    if ((t = find_tensor(sf, "x_embedder.weight")) && t->ndim == 2) { c->hidden = (int)t->shape[0]; c->channels = (int)t->shape[1]; }
    if ((t = find_tensor(sf, "context_embedder.weight")) && t->ndim == 2) c->text_dim = (int)t->shape[1];
    if ((t = find_tensor(sf, "transformer_blocks.0.ff.linear_in.weight")) && t->ndim == 2) c->mlp = (int)(t->shape[0] / 2);
    if ((t = find_tensor(sf, "transformer_blocks.0.attn.norm_q.weight")) && t->ndim == 1) c->head_dim = (int)t->shape[0];
    if (c->head_dim > 0) c->heads = c->hidden / c->head_dim;
    int nd = 0, ns = 0;
    for (int i = 0; i < sf->num_tensors; i++) {
        int idx;
        if (sscanf(sf->tensors[i].name, "transformer_blocks.%d.", &idx) == 1 && idx + 1 > nd) nd = idx + 1;
        if (sscanf(sf->tensors[i].name, "single_transformer_blocks.%d.", &idx) == 1 && idx + 1 > ns) ns = idx + 1;
    }
    if (nd > 0) c->n_double = nd;
    if (ns > 0) c->n_single = ns;
}

static flux_transformer_t *load_from_handle(void *p) {
    ref_safetensors_file *sf = (ref_safetensors_file *)p;
    if (!sf || !sf->data) { flux_hip_fail("flux_transformer_load_safetensors: NULL file"); return NULL; }
    if (sf->num_tensors < 0 || sf->num_tensors > 512) { flux_hip_fail("flux_transformer_load_safetensors: bad tensor count"); return NULL; }
    flux_hip_config c;
    flux_hip_default_config(&c);
    infer_config(sf, &c);
    flux_transformer_t *tf = flux_hip_transformer_new(&c);
    if (!tf) return NULL;
    for (int i = 0; i < sf->num_tensors; i++) {
        const ref_safetensor *t = &sf->tensors[i];
        const char *data;
        int64_t numel;
        if (!usable_dtype(t->dtype)) continue;
        if (!handle_entry(sf, i, &data, &numel)) { flux_transformer_free(tf); return NULL; }
        if (!set_from(tf, t->name, t->dtype, data, numel)) {
            /* files may carry tensors this path does not use; only real failures abort */
            if (strstr(flux_hip_last_error(), "is not part of the transformer")) continue;
            flux_transformer_free(tf);
            return NULL;
        }
    }
    if (!fh_model_complete(tf)) { flux_transformer_free(tf); return NULL; }
    return tf;
}

flux_transformer_t *flux_transformer_load_safetensors(void *sf) { return load_from_handle(sf); }

flux_transformer_t *flux_transformer_load(void *f) {
    (void)f;
    flux_hip_fail("flux_transformer_load: the binary weight format is not read by this backend; load the safetensors file "
                  "(flux_transformer_load_safetensors)");
    return NULL;
}

flux_transformer_t *flux_transformer_load_safetensors_mmap(void *sf) {
    /* Weights are device resident after loading, so the mapping is not needed afterwards; the
     * handle is still owned and closed on free, as callers of the reference expect
     * (flux.c:311-313, flux_transformer.c:4305-4309). */
    flux_transformer_t *tf = load_from_handle(sf);
    if (tf) tf->owned_sf = sf;
    return tf;
}
