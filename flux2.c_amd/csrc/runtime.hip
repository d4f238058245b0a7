/*
 * runtime.hip - device lifetime, buffers, error text and event timing of the gfx950 backend.
 * Plays the part flux_metal_init/available/sync and the flux_gpu_tensor_* calls play for the
 * reference's Apple backend (flux_metal.h:23-198).
 */
#include "common.h"
#include "../../include/flux_hip.h"
#include <stdarg.h>
#include <string.h>
#include <stdlib.h>

static char g_err[512] = "";
static hipStream_t g_stream = nullptr;
static int g_ready = 0;
static hipEvent_t g_ev0 = nullptr, g_ev1 = nullptr;
static void *g_stage = nullptr; /* pinned staging buffer of flux_hip_download */
static size_t g_stage_bytes = 0;
#define DOWNLOAD_PARTS 4
static hipStream_t g_copy_stream = nullptr; /* carries flux_hip_download_part_begin's copies beside the main stream */
static hipEvent_t g_part_ready[DOWNLOAD_PARTS], g_part_done[DOWNLOAD_PARTS];
static const void *g_part_at[DOWNLOAD_PARTS];

extern "C" int flux_hip_fail(const char *fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof(g_err), fmt, ap);
    va_end(ap);
    if (flux_verbose) fprintf(stderr, "flux_hip: %s\n", g_err);
    return 0;
}

extern "C" const char *flux_hip_last_error(void) { return g_err; }

extern "C" hipStream_t flux_hip_stream_handle(void) { return g_stream; }
extern "C" void *flux_hip_stream(void) { return (void *)g_stream; }

extern "C" int flux_hip_linear_static_init(void);

extern "C" int flux_hip_init(void) {
    if (g_ready) return 1;
    int n = 0;
    if (hipGetDeviceCount(&n) != hipSuccess || n < 1) return flux_hip_fail("no HIP device is visible");
    HIP_OK(hipSetDevice(0));
    hipDeviceProp_t prop;
    HIP_OK(hipGetDeviceProperties(&prop, 0));
    if (strncmp(prop.gcnArchName, "gfx950", 6) != 0)
        return flux_hip_fail("device 0 is %s; this library holds gfx950 code only", prop.gcnArchName);
    HIP_OK(hipStreamCreate(&g_stream));
    HIP_OK(hipEventCreate(&g_ev0));
    HIP_OK(hipEventCreate(&g_ev1));
    HIP_OK(hipStreamCreateWithFlags(&g_copy_stream, hipStreamNonBlocking));
    for (int i = 0; i < DOWNLOAD_PARTS; i++) {
        HIP_OK(hipEventCreateWithFlags(&g_part_ready[i], hipEventDisableTiming));
        HIP_OK(hipEventCreateWithFlags(&g_part_done[i], hipEventDisableTiming));
    }
    if (!flux_hip_linear_static_init()) return 0; /* device address of the static workspace, with device 0 current */
    g_ready = 1;
    return 1;
}

extern "C" int flux_hip_available(void) { return g_ready || flux_hip_init(); }

extern "C" void flux_hip_linear_release(void);

extern "C" void flux_hip_cleanup(void) {
    if (!g_ready) return;
    (void)hipStreamSynchronize(g_stream);
    flux_hip_linear_release();
    if (g_stage) (void)hipHostFree(g_stage);
    g_stage = nullptr;
    g_stage_bytes = 0;
    (void)hipEventDestroy(g_ev0);
    (void)hipEventDestroy(g_ev1);
    (void)hipStreamSynchronize(g_copy_stream);
    for (int i = 0; i < DOWNLOAD_PARTS; i++) {
        (void)hipEventDestroy(g_part_ready[i]);
        (void)hipEventDestroy(g_part_done[i]);
    }
    (void)hipStreamDestroy(g_copy_stream);
    g_copy_stream = nullptr;
    (void)hipStreamDestroy(g_stream);
    g_stream = nullptr;
    g_ready = 0;
}

extern "C" int flux_hip_sync(void) {
    if (!g_ready) return flux_hip_fail("flux_hip_sync: backend not initialised");
    HIP_OK(hipStreamSynchronize(g_stream));
    return 1;
}

extern "C" void *flux_hip_malloc(size_t bytes) {
    if (!flux_hip_available()) return nullptr;
    void *p = nullptr;
    hipError_t e = hipMalloc(&p, bytes ? bytes : 1);
    if (e != hipSuccess) {
        flux_hip_fail("hipMalloc(%zu) failed: %s", bytes, hipGetErrorString(e));
        return nullptr;
    }
    return p;
}

extern "C" void flux_hip_free(void *p) {
    if (p) (void)hipFree(p);
}

#define STAGE_MIN ((size_t)1 << 20)
#define STAGE_MAX ((size_t)256 << 20)
/* Pinned staging buffer (kept, grown on demand) for results of 1 to 256 MB: a copy from the device
 * into pageable memory runs at a fraction of the link's rate (measured: 0.2 ms less per 15.7 MB
 * result with the extra host copy included). NULL when it cannot be had. */
static void *stage_buffer(size_t bytes) {
    if (bytes < STAGE_MIN || bytes > STAGE_MAX) return nullptr;
    if (bytes > g_stage_bytes) {
        if (g_stage) (void)hipHostFree(g_stage);
        g_stage = nullptr;
        g_stage_bytes = 0;
        if (hipHostMalloc(&g_stage, bytes, hipHostMallocDefault) == hipSuccess) g_stage_bytes = bytes;
        else { g_stage = nullptr; (void)hipGetLastError(); }
    }
    return g_stage;
}

extern "C" int flux_hip_upload(void *dst, const void *src, size_t bytes) {
    if (!flux_hip_available()) return 0;
    if (!bytes) return 1;
    HIP_OK(hipMemcpyAsync(dst, src, bytes, hipMemcpyHostToDevice, g_stream));
    HIP_OK(hipStreamSynchronize(g_stream)); /* the host buffer may be reused at once */
    return 1;
}

extern "C" int flux_hip_download(void *dst, const void *src, size_t bytes) {
    if (!flux_hip_available()) return 0;
    if (!bytes) return 1;
    void *stage = stage_buffer(bytes);
    HIP_OK(hipMemcpyAsync(stage ? stage : dst, src, bytes, hipMemcpyDeviceToHost, g_stream));
    HIP_OK(hipStreamSynchronize(g_stream));
    if (stage) memcpy(dst, stage, bytes);
    return 1;
}

/* A result whose parts become final one after the other (the captured layers of the text encoder):
 * part_begin queues, on a second stream, the copy of one part into the pinned staging buffer at
 * stage_offset, to start when the work queued so far on the main stream has run; the main stream goes
 * on meanwhile. part_wait returns the part's host address once it has arrived. All parts of one
 * result name the same stage_total. part_begin returns 1, 0 when there is no staging buffer of that
 * size (the caller then downloads the whole result at the end), -1 on an error. */
extern "C" int flux_hip_download_part_begin(int part, size_t stage_offset, size_t stage_total, const void *src, size_t bytes) {
    if (!flux_hip_available()) return -1;
    if (part < 0 || part >= DOWNLOAD_PARTS || stage_offset + bytes > stage_total) {
        flux_hip_fail("flux_hip_download_part_begin: bad part");
        return -1;
    }
    char *stage = (char *)stage_buffer(stage_total);
    if (!stage) return 0;
    if (hipEventRecord(g_part_ready[part], g_stream) != hipSuccess ||
        hipStreamWaitEvent(g_copy_stream, g_part_ready[part], 0) != hipSuccess ||
        hipMemcpyAsync(stage + stage_offset, src, bytes, hipMemcpyDeviceToHost, g_copy_stream) != hipSuccess ||
        hipEventRecord(g_part_done[part], g_copy_stream) != hipSuccess) {
        flux_hip_fail("flux_hip_download_part_begin: %s", hipGetErrorString(hipGetLastError()));
        return -1;
    }
    g_part_at[part] = stage + stage_offset;
    return 1;
}

extern "C" const void *flux_hip_download_part_wait(int part) {
    if (!g_ready || part < 0 || part >= DOWNLOAD_PARTS || !g_part_at[part]) {
        flux_hip_fail("flux_hip_download_part_wait: no such part");
        return nullptr;
    }
    if (hipEventSynchronize(g_part_done[part]) != hipSuccess) {
        flux_hip_fail("flux_hip_download_part_wait: %s", hipGetErrorString(hipGetLastError()));
        return nullptr;
    }
    const void *at = g_part_at[part];
    g_part_at[part] = nullptr;
    return at;
}

extern "C" int flux_hip_memset(void *dst, int value, size_t bytes) {
    if (!flux_hip_available()) return 0;
    HIP_OK(hipMemsetAsync(dst, value, bytes, g_stream));
    return 1;
}

extern "C" int flux_hip_timer_start(void) {
    if (!flux_hip_available()) return 0;
    HIP_OK(hipEventRecord(g_ev0, g_stream));
    return 1;
}

extern "C" float flux_hip_timer_stop(void) {
    if (!g_ready) return -1.0f;
    float ms = -1.0f;
    if (hipEventRecord(g_ev1, g_stream) != hipSuccess) return -1.0f;
    if (hipEventSynchronize(g_ev1) != hipSuccess) return -1.0f;
    if (hipEventElapsedTime(&ms, g_ev0, g_ev1) != hipSuccess) return -1.0f;
    return ms;
}
