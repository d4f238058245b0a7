/*
 * flux_synth.c - deterministic synthetic tensors for tests and benchmarks.
 *
 * Counter-based normal generator: element i of stream (seed, stream_id) is a
 * pure function of (seed, stream_id, i), so tensors of any size can be filled
 * in parallel and regenerated identically on any machine. Used to make
 * random-init bf16 weights ~N(0, std) and N(0,1) inputs of the shapes the
 * denoising transformer consumes; there are no model files in this repo.
 */
#include <stdint.h>
#include <math.h>
#include <string.h>

static inline uint64_t mix64(uint64_t z) {
    z = (z ^ (z >> 30)) * 0xbf58476d1ce4e5b9ULL;
    z = (z ^ (z >> 27)) * 0x94d049bb133111ebULL;
    return z ^ (z >> 31);
}

/* Two independent normals from one 64-bit hash (Box-Muller, both branches). */
static inline void normal_pair(uint64_t key, uint64_t pair, float *a, float *b) {
    uint64_t h = mix64(key + 0x9e3779b97f4a7c15ULL * (pair + 1));
    float u1 = ((float)((h >> 40) + 1)) * (1.0f / 16777216.0f);      /* (0,1] */
    float u2 = ((float)((h >> 8) & 0xffffff)) * (1.0f / 16777216.0f); /* [0,1) */
    float r = sqrtf(-2.0f * logf(u1));
    float ang = 6.28318530717958647692f * u2;
    *a = r * cosf(ang);
    *b = r * sinf(ang);
}

static inline uint64_t stream_key(uint64_t seed, uint64_t stream_id) {
    return mix64(seed * 0xd1342543de82ef95ULL + mix64(stream_id + 0x632be59bd9b4e019ULL));
}

static inline uint16_t f32_to_bf16_rne(float f) {
    uint32_t u;
    memcpy(&u, &f, 4);
    u += 0x7fffu + ((u >> 16) & 1u);
    return (uint16_t)(u >> 16);
}

void flux_synth_normal_f32(float *out, int64_t n, uint64_t seed, uint64_t stream_id,
                           float mean, float std) {
    uint64_t key = stream_key(seed, stream_id);
    int64_t pairs = (n + 1) / 2;
    #pragma omp parallel for schedule(static)
    for (int64_t p = 0; p < pairs; p++) {
        float a, b;
        normal_pair(key, (uint64_t)p, &a, &b);
        out[2 * p] = mean + std * a;
        if (2 * p + 1 < n) out[2 * p + 1] = mean + std * b;
    }
}

void flux_synth_normal_bf16(uint16_t *out, int64_t n, uint64_t seed, uint64_t stream_id,
                            float mean, float std) {
    uint64_t key = stream_key(seed, stream_id);
    int64_t pairs = (n + 1) / 2;
    #pragma omp parallel for schedule(static)
    for (int64_t p = 0; p < pairs; p++) {
        float a, b;
        normal_pair(key, (uint64_t)p, &a, &b);
        out[2 * p] = f32_to_bf16_rne(mean + std * a);
        if (2 * p + 1 < n) out[2 * p + 1] = f32_to_bf16_rne(mean + std * b);
    }
}

void flux_synth_fill_bf16(uint16_t *out, int64_t n, float value) {
    uint16_t v = f32_to_bf16_rne(value);
    #pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < n; i++) out[i] = v;
}

/* Round fp32 -> bf16 (nearest even) and widen bf16 -> fp32, for host checks. */
void flux_synth_f32_to_bf16(uint16_t *out, const float *in, int64_t n) {
    #pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < n; i++) out[i] = f32_to_bf16_rne(in[i]);
}

void flux_synth_bf16_to_f32(float *out, const uint16_t *in, int64_t n) {
    #pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < n; i++) {
        uint32_t u = ((uint32_t)in[i]) << 16;
        memcpy(&out[i], &u, 4);
    }
}
