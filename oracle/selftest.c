/*
 * Exercises every entry point of the CPU oracle on awkward sizes.  TEST INFRASTRUCTURE: built with
 * -fsanitize=address,undefined (and once with -fsanitize=thread for the threaded step) so that an
 * out-of-bounds index, a signed overflow or a data race in the checker itself does not go unnoticed.
 */
#include <math.h>
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

float orc_h2f(uint16_t);
uint16_t orc_f2h(float);
void orc_adamw_fp16_clip(float*, uint16_t*, const uint16_t*, float*, float*, int64_t, float, float, float, float,
                         float, float, float, float, int);
void orc_adamw_fp32_clip(float*, const float*, float*, float*, int64_t, float, float, float, float, float, float,
                         float, float, int);
void orc_optimizer_step(float*, uint16_t*, const uint16_t*, float*, float*, int64_t, int64_t, float*, const float*,
                        float*, float*, int64_t, float, float, float, float, float, int*);
float orc_clip_grad_norm(uint16_t*, int64_t, float*, int64_t, float, float*);
int64_t orc_sumsq_mirror_partials(const void*, int, int64_t, int, double*);
double orc_sumsq_mirror_final(const double*, int64_t);
void orc_fill_f16(uint16_t*, int64_t, uint64_t, int64_t, float, float, uint32_t, int64_t, uint32_t);
void orc_fill_f32(float*, int64_t, uint64_t, int64_t, float, float, uint32_t, int64_t, uint32_t);
float orc_step_fp16_threaded(float*, uint16_t*, const uint16_t*, float*, float*, int64_t, float, float, float,
                             float, float, float, float, float, int);

int main(void)
{
    const int64_t sizes[] = {1, 7, 8, 9, 255, 2047, 2049, 8191, 8193, 100003};
    for (unsigned s = 0; s < sizeof(sizes) / sizeof(sizes[0]); s++) {
        const int64_t n = sizes[s];
        uint16_t* p = malloc(n * 2); uint16_t* g = malloc(n * 2);
        float* m = calloc(n, 4); float* v = calloc(n, 4); float* w = malloc(n * 4); float* g32 = malloc(n * 4);
        double* parts = malloc(2 * ((n + 2047) / 2048 + 1) * sizeof(double));
        orc_fill_f16(p, n, 1, 0, 0.0f, 0.02f, 0, 0, 0);
        orc_fill_f16(g, n, 2, 5, 0.0f, 5e-3f, 0, 64, 0x80000000u);
        orc_fill_f32(w, n, 3, 0, 1.0f, 0.1f, 1, 0, 0);
        orc_fill_f32(g32, n, 4, 0, 0.0f, 1e-2f, 0, 0, 0);
        for (int64_t i = 0; i < n; i++) w[i] = orc_h2f(orc_f2h(w[i]));
        float scale = 1.0f;
        float norm = orc_clip_grad_norm(g, n, g32, n, 0.01f, &scale);
        if (!(norm >= 0.0f) || !(scale > 0.0f && scale <= 1.0f)) { printf("bad norm\n"); return 1; }
        orc_adamw_fp16_clip(NULL, p, g, m, v, n, 1e-3f, 0.9f, 0.999f, 1e-8f, 0.01f, 0.1f, 0.001f, scale, 1);
        orc_adamw_fp16_clip(w, p, g, m, v, n, 1e-3f, 0.9f, 0.999f, 1e-8f, 0.01f, 0.19f, 0.002f, 1.0f, 0);
        orc_adamw_fp32_clip(w, g32, m, v, n, 1e-3f, 0.9f, 0.999f, 1e-8f, 0.0f, 0.27f, 0.003f, scale, 1);
        int step = 0;
        orc_optimizer_step(w, p, g, m, v, n, n / 2, w, g32, m, v, n, 1e-3f, 0.9f, 0.999f, 1e-8f, 0.01f, &step);
        int64_t k = orc_sumsq_mirror_partials(g, 0, n, 2048, parts);
        k += orc_sumsq_mirror_partials(g32, 1, n, 2048, parts + k);
        if (!(orc_sumsq_mirror_final(parts, k) >= 0.0)) { printf("bad mirror\n"); return 1; }
        for (int threads = 1; threads <= 9; threads += 4)
            orc_step_fp16_threaded(NULL, p, g, m, v, n, 1e-3f, 0.9f, 0.999f, 1e-8f, 0.01f, 0.1f, 0.001f, 0.01f, threads);
        free(p); free(g); free(m); free(v); free(w); free(g32); free(parts);
    }
    for (uint32_t h = 0; h < 65536; h++) {
        float f = orc_h2f((uint16_t)h);
        if (f == f && orc_f2h(f) != h) { printf("round trip %u\n", h); return 1; }
    }
    printf("selftest ok\n");
    return 0;
}
