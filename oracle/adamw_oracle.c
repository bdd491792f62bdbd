/*
 * CPU oracle for the AdamW + grad-norm/clip path.  TEST INFRASTRUCTURE ONLY.
 *
 * This file restates, in plain C, the arithmetic of the reference's optimizer
 * step so that the HIP path can be checked against it.  Only tests, the smoke
 * check and the bench's cpu_baseline leg may call it; the product library
 * never links or loads it.
 *
 * Reference lines restated (paths are inside the reference tree):
 *   orc_adamw_fp16        src/kernels/adamw.cu:7-58   (kernel body 25-39, host reciprocals 52-53, n<=0 at 49)
 *   orc_adamw_fp32        src/kernels/adamw.cu:63-108 (kernel body 80-90, n<=0 at 99)
 *   orc_bias_correction   include/training/optimizer.h:121-122
 *   orc_optimizer_step    include/training/optimizer.h:119-147 (three groups, wd only on projections)
 *   orc_fp16_to_fp32      include/training/optimizer.h:46-57
 *   orc_sum_sq_half/float include/training/trainer.h:103-133 (sum of squares; accumulated here in FP64,
 *                         the reference accumulates in FP32 with unordered atomics)
 *   orc_scale_half/float  include/training/trainer.h:136-145 (orc_scale_float is also the arithmetic of
 *                         scale_grad_kernel, trainer.h:96-99: one FP32 multiply per element)
 *   orc_clip_grad_norm    include/training/trainer.h:323-352
 *
 * Parity pins (tests/test_oracle_*.py): orc_h2f is checked on all 65,536 inputs and
 * orc_f2h on ties, subnormals, overflow and random floats against numpy's float16;
 * the update is checked against the step-1 loop of the reference's own test
 * (tests/test_adamw.cu:194-206,276-293), against torch.optim.AdamW, and against
 * closed forms (g=0 decay, sign step); the norm against numpy float64 and known vectors;
 * the clip rule against its published definition (strict '>' and the +1e-6f).
 * orc_sumsq_mirror_* and orc_fill_* have no counterpart in the reference: the first
 * restates the HIP reduction order so that the device norm can be compared bit for
 * bit, the second is the seeded input generator shared with the device.
 *
 * Build: gcc -O3 -fno-math-errno -ffp-contract=off (no fast-math, no FMA contraction,
 * so that every operation rounds once, as in the HIP kernels built with the same policy).
 */
#include <math.h>
#include <pthread.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#if defined(__GNUC__) && defined(__x86_64__)
#define ORC_CLONES __attribute__((target_clones("avx2", "default")))
#else
#define ORC_CLONES
#endif

/* ------------------------------------------------------------------ */
/* IEEE binary16 <-> binary32, bit exact, round to nearest even        */
/* ------------------------------------------------------------------ */

static inline float bits2f(uint32_t u) { float f; memcpy(&f, &u, 4); return f; }
static inline uint32_t f2bits(float f) { uint32_t u; memcpy(&u, &f, 4); return u; }

static inline float h2f_inl(uint16_t h)
{
    uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
    uint32_t exp  = (h >> 10) & 0x1Fu;
    uint32_t man  = h & 0x3FFu;
    if (exp == 0x1F) return bits2f(sign | 0x7F800000u | (man << 13));   /* inf / nan */
    if (exp != 0)    return bits2f(sign | ((exp + 112u) << 23) | (man << 13));
    /* zero or subnormal: value = man * 2^-24, exact in binary32 */
    float mag = (float)man * 5.9604644775390625e-08f;
    return bits2f(sign | f2bits(mag));
}

static inline uint16_t f2h_inl(float f)
{
    uint32_t x    = f2bits(f);
    uint16_t sign = (uint16_t)((x >> 16) & 0x8000u);
    uint32_t ax   = x & 0x7FFFFFFFu;
    if (ax >= 0x7F800000u)                       /* inf or nan */
        return (uint16_t)(sign | 0x7C00u | (ax > 0x7F800000u ? (0x0200u | ((ax >> 13) & 0x3FFu)) : 0u));
    if (ax >= 0x477FF000u)                       /* >= 65520 rounds to inf */
        return (uint16_t)(sign | 0x7C00u);
    if (ax >= 0x38800000u) {                     /* normal half range (>= 2^-14) */
        uint32_t r   = ax - 0x38000000u;         /* rebias exponent 127 -> 15 */
        uint32_t out = r >> 13;
        uint32_t rem = r & 0x1FFFu;
        if (rem > 0x1000u || (rem == 0x1000u && (out & 1u))) out++;   /* may carry into exponent: correct */
        return (uint16_t)(sign | out);
    }
    if (ax < 0x33000000u)                        /* < 2^-25 rounds to zero (2^-25 itself ties to even = 0) */
        return sign;
    {
        /* subnormal half: result = round(|f| / 2^-24) as an integer in [0, 1024] */
        uint32_t e     = ax >> 23;               /* biased exponent, 102..112 */
        uint32_t man   = (ax & 0x7FFFFFu) | 0x800000u;
        uint32_t shift = 126u - e;               /* 14..24 */
        uint32_t out   = man >> shift;
        uint32_t rem   = man & ((1u << shift) - 1u);
        uint32_t half  = 1u << (shift - 1u);
        if (rem > half || (rem == half && (out & 1u))) out++;
        return (uint16_t)(sign | out);
    }
}

float    orc_h2f(uint16_t h) { return h2f_inl(h); }
uint16_t orc_f2h(float f)    { return f2h_inl(f); }

ORC_CLONES void orc_h2f_array(float* dst, const uint16_t* src, int64_t n)
{
    for (int64_t i = 0; i < n; i++) dst[i] = h2f_inl(src[i]);
}

ORC_CLONES void orc_f2h_array(uint16_t* dst, const float* src, int64_t n)
{
    for (int64_t i = 0; i < n; i++) dst[i] = f2h_inl(src[i]);
}

/* master init: dst[i] = h2f(src[i])   (optimizer.h:46-57) */
void orc_fp16_to_fp32(float* dst, const uint16_t* src, int64_t n) { orc_h2f_array(dst, src, n); }

/* ------------------------------------------------------------------ */
/* AdamW                                                               */
/* ------------------------------------------------------------------ */

/* bias_correction = 1 - powf(beta, (float)step)   (optimizer.h:121-122) */
float orc_bias_correction(float beta, int step) { return 1.0f - powf(beta, (float)step); }

/*
 * FP16-weight update (adamw.cu:25-39).  master may be NULL: then the FP16 weight
 * itself is the source of truth (w = h2f(model_w[i])), which is the 22-byte-per-
 * parameter mode; the reference always has a master copy.
 * clip_scale != 1 applies the clip in the same pass exactly as a preceding
 * scale_half_kernel would have (trainer.h:136-139): g = h2f(f2h(h2f(g) * scale)).
 */
ORC_CLONES static void adamw_fp16_range(
    float* master_w, uint16_t* model_w, const uint16_t* grad, float* m, float* v,
    int64_t lo, int64_t hi,
    float lr, float beta1, float beta2, float eps, float weight_decay,
    float bc1_inv, float bc2_inv, float clip_scale, int apply_clip)
{
    for (int64_t i = lo; i < hi; i++) {
        float g = h2f_inl(grad[i]);
        if (apply_clip) g = h2f_inl(f2h_inl(g * clip_scale));
        float mi = beta1 * m[i] + (1.0f - beta1) * g;
        float vi = beta2 * v[i] + (1.0f - beta2) * g * g;
        m[i] = mi;
        v[i] = vi;
        float m_hat = mi * bc1_inv;
        float v_hat = vi * bc2_inv;
        float w = master_w ? master_w[i] : h2f_inl(model_w[i]);
        w = w * (1.0f - lr * weight_decay) - lr * m_hat / (sqrtf(v_hat) + eps);
        if (master_w) master_w[i] = w;
        model_w[i] = f2h_inl(w);
    }
}

void orc_adamw_fp16_clip(
    float* master_w, uint16_t* model_w, const uint16_t* grad, float* m, float* v, int64_t n,
    float lr, float beta1, float beta2, float eps, float weight_decay,
    float bias_correction1, float bias_correction2, float clip_scale, int apply_clip)
{
    if (n <= 0) return;                                   /* adamw.cu:49 */
    float bc1_inv = 1.0f / bias_correction1;              /* adamw.cu:52-53 */
    float bc2_inv = 1.0f / bias_correction2;
    adamw_fp16_range(master_w, model_w, grad, m, v, 0, n, lr, beta1, beta2, eps,
                     weight_decay, bc1_inv, bc2_inv, clip_scale, apply_clip);
}

void orc_adamw_fp16(
    float* master_w, uint16_t* model_w, const uint16_t* grad, float* m, float* v, int64_t n,
    float lr, float beta1, float beta2, float eps, float weight_decay,
    float bias_correction1, float bias_correction2)
{
    orc_adamw_fp16_clip(master_w, model_w, grad, m, v, n, lr, beta1, beta2, eps, weight_decay,
                        bias_correction1, bias_correction2, 1.0f, 0);
}

/* FP32-weight update, in place (adamw.cu:80-90); clip as scale_float_kernel (trainer.h:142-145). */
ORC_CLONES static void adamw_fp32_range(
    float* w, const float* grad, float* m, float* v, int64_t lo, int64_t hi,
    float lr, float beta1, float beta2, float eps, float weight_decay,
    float bc1_inv, float bc2_inv, float clip_scale, int apply_clip)
{
    for (int64_t i = lo; i < hi; i++) {
        float g = grad[i];
        if (apply_clip) g = g * clip_scale;
        float mi = beta1 * m[i] + (1.0f - beta1) * g;
        float vi = beta2 * v[i] + (1.0f - beta2) * g * g;
        m[i] = mi;
        v[i] = vi;
        float m_hat = mi * bc1_inv;
        float v_hat = vi * bc2_inv;
        w[i] = w[i] * (1.0f - lr * weight_decay) - lr * m_hat / (sqrtf(v_hat) + eps);
    }
}

void orc_adamw_fp32_clip(
    float* w, const float* grad, float* m, float* v, int64_t n,
    float lr, float beta1, float beta2, float eps, float weight_decay,
    float bias_correction1, float bias_correction2, float clip_scale, int apply_clip)
{
    if (n <= 0) return;                                   /* adamw.cu:99 */
    float bc1_inv = 1.0f / bias_correction1;
    float bc2_inv = 1.0f / bias_correction2;
    adamw_fp32_range(w, grad, m, v, 0, n, lr, beta1, beta2, eps, weight_decay,
                     bc1_inv, bc2_inv, clip_scale, apply_clip);
}

void orc_adamw_fp32(
    float* w, const float* grad, float* m, float* v, int64_t n,
    float lr, float beta1, float beta2, float eps, float weight_decay,
    float bias_correction1, float bias_correction2)
{
    orc_adamw_fp32_clip(w, grad, m, v, n, lr, beta1, beta2, eps, weight_decay,
                        bias_correction1, bias_correction2, 1.0f, 0);
}

/*
 * One optimizer step over the reference's flat pools (optimizer.h:119-147):
 * the step counter is incremented first, bias corrections use powf on the host,
 * projections get weight_decay, the embedding tail of the FP16 pool and the whole
 * FP32 pool get 0.  *step is in/out.
 */
void orc_optimizer_step(
    float* fp16_master, uint16_t* fp16_pool, const uint16_t* half_grads, float* fp16_m, float* fp16_v,
    int64_t n16, int64_t proj_n,
    float* fp32_pool, const float* float_grads, float* fp32_m, float* fp32_v, int64_t n32,
    float lr, float beta1, float beta2, float eps, float weight_decay, int* step)
{
    *step += 1;
    float bc1 = orc_bias_correction(beta1, *step);
    float bc2 = orc_bias_correction(beta2, *step);
    orc_adamw_fp16(fp16_master, fp16_pool, half_grads, fp16_m, fp16_v, proj_n,
                   lr, beta1, beta2, eps, weight_decay, bc1, bc2);
    orc_adamw_fp16(fp16_master + proj_n, fp16_pool + proj_n, half_grads + proj_n,
                   fp16_m + proj_n, fp16_v + proj_n, n16 - proj_n,
                   lr, beta1, beta2, eps, 0.0f, bc1, bc2);
    orc_adamw_fp32(fp32_pool, float_grads, fp32_m, fp32_v, n32,
                   lr, beta1, beta2, eps, 0.0f, bc1, bc2);
}

/* ------------------------------------------------------------------ */
/* Gradient norm and clip                                              */
/* ------------------------------------------------------------------ */

ORC_CLONES double orc_sum_sq_half(const uint16_t* g, int64_t n)
{
    double acc = 0.0;
    for (int64_t i = 0; i < n; i++) { double x = (double)h2f_inl(g[i]); acc += x * x; }
    return acc;
}

ORC_CLONES double orc_sum_sq_float(const float* g, int64_t n)
{
    double acc = 0.0;
    for (int64_t i = 0; i < n; i++) { double x = (double)g[i]; acc += x * x; }
    return acc;
}

/* g[i] = f2h(h2f(g[i]) * scale)   (trainer.h:136-139) */
ORC_CLONES void orc_scale_half(uint16_t* g, float scale, int64_t n)
{
    for (int64_t i = 0; i < n; i++) g[i] = f2h_inl(h2f_inl(g[i]) * scale);
}

/* g[i] *= scale   (trainer.h:142-145) */
ORC_CLONES void orc_scale_float(float* g, float scale, int64_t n)
{
    for (int64_t i = 0; i < n; i++) g[i] *= scale;
}

/*
 * The clip rule alone (trainer.h:341-345): total_norm = sqrtf(sum_sq);
 * scale = max_norm / (total_norm + 1e-6f) iff total_norm > max_norm, else no scaling.
 * A NaN norm compares false and leaves the gradients alone, as in the reference.
 * Returns the scale (1.0f when no scaling happens); *norm_out gets the pre-clip norm.
 */
float orc_clip_scale(float sum_sq, float max_norm, float* norm_out)
{
    float total_norm = sqrtf(sum_sq);
    if (norm_out) *norm_out = total_norm;
    if (total_norm > max_norm) return max_norm / (total_norm + 1e-6f);
    return 1.0f;
}

/*
 * clip_grad_norm_ over the two gradient pools, in place (trainer.h:323-352).
 * Returns the pre-clip norm.  *scale_out gets the applied scale (1.0f if none).
 */
float orc_clip_grad_norm(uint16_t* half_pool, int64_t n16, float* float_pool, int64_t n32,
                         float max_norm, float* scale_out)
{
    double s = 0.0;
    if (n16 > 0) s += orc_sum_sq_half(half_pool, n16);
    if (n32 > 0) s += orc_sum_sq_float(float_pool, n32);
    float norm;
    float scale = orc_clip_scale((float)s, max_norm, &norm);
    if (norm > max_norm) {
        if (n16 > 0) orc_scale_half(half_pool, scale, n16);
        if (n32 > 0) orc_scale_float(float_pool, scale, n32);
    }
    if (scale_out) *scale_out = scale;
    return norm;
}

/* ------------------------------------------------------------------ */
/* Mirror of the device reduction order (no counterpart in the         */
/* reference).  A chunk is `chunk` consecutive elements of one tensor; */
/* with L = min(512, chunk/8) lanes, lane t owns the 8-element groups  */
/* t, t+L, ... of the chunk and adds x*x into one FP32 accumulator in  */
/* element order; the 64 lanes of a wave combine by xor-butterfly      */
/* (32,16,8,4,2,1); the L/64 wave sums are added in FP64 in wave order.*/
/* ------------------------------------------------------------------ */

static double mirror_chunk(const void* g, int is_f32, int64_t count, int chunk)
{
    float lane[512];
    int groups = chunk / 8;
    int lanes = groups < 512 ? groups : 512;
    if (lanes < 64) lanes = 64;
    for (int t = 0; t < lanes; t++) {
        float acc = 0.0f;
        for (int grp = t; grp < groups; grp += lanes) {
            for (int e = 0; e < 8; e++) {
                int64_t i = (int64_t)grp * 8 + e;
                if (i < count) {
                    float x = is_f32 ? ((const float*)g)[i] : h2f_inl(((const uint16_t*)g)[i]);
                    acc = acc + x * x;
                }
            }
        }
        lane[t] = acc;
    }
    double total = 0.0;
    for (int w = 0; w < lanes / 64; w++) {
        float* l = lane + 64 * w;
        for (int mask = 32; mask >= 1; mask >>= 1) {
            float nxt[64];
            for (int t = 0; t < 64; t++) nxt[t] = l[t] + l[t ^ mask];
            memcpy(l, nxt, sizeof(nxt));
        }
        total += (double)l[0];
    }
    return total;
}

/* Per-chunk partials of one tensor, appended at partials[0..]; returns how many were written. */
int64_t orc_sumsq_mirror_partials(const void* g, int is_f32, int64_t n, int chunk, double* partials)
{
    int64_t k = 0;
    for (int64_t start = 0; start < n; start += chunk) {
        int64_t count = n - start < chunk ? n - start : chunk;
        const void* base = is_f32 ? (const void*)((const float*)g + start)
                                  : (const void*)((const uint16_t*)g + start);
        partials[k++] = mirror_chunk(base, is_f32, count, chunk);
    }
    return k;
}

/*
 * Group partials (plans with 512-element chunks only): 16 consecutive chunk partials are
 * added in FP64, in index order, starting from 0.0.  Returns the number of groups written.
 */
int64_t orc_sumsq_mirror_groups(const double* partials, int64_t n_partials, double* groups)
{
    int64_t k = 0;
    for (int64_t first = 0; first < n_partials; first += 16) {
        double total = 0.0;
        for (int64_t i = first; i < first + 16 && i < n_partials; i++) total += partials[i];
        groups[k++] = total;
    }
    return k;
}

/*
 * Final pass: 1024 threads, thread t adds its values t, t+1024, ... in order (FP64),
 * then a halving tree (512, 256, ..., 1) in FP64.  The values are the chunk partials, or
 * the group partials for 512-element chunks (orc_sumsq_mirror_total picks).
 */
double orc_sumsq_mirror_final(const double* partials, int64_t n_partials)
{
    double acc[1024];
    for (int t = 0; t < 1024; t++) {
        double a = 0.0;
        for (int64_t i = t; i < n_partials; i += 1024) a += partials[i];
        acc[t] = a;
    }
    for (int s = 512; s >= 1; s >>= 1)
        for (int t = 0; t < s; t++) acc[t] = acc[t] + acc[t + s];
    return acc[0];
}

/* The device's sum of squares from the per-chunk partials of a plan with chunks of `chunk` elements. */
double orc_sumsq_mirror_total(const double* partials, int64_t n_partials, int chunk)
{
    if (chunk != 512) return orc_sumsq_mirror_final(partials, n_partials);
    int64_t n_groups = (n_partials + 15) / 16;
    double* groups = (double*)malloc(sizeof(double) * (size_t)(n_groups > 0 ? n_groups : 1));
    orc_sumsq_mirror_groups(partials, n_partials, groups);
    double total = orc_sumsq_mirror_final(groups, n_groups);
    free(groups);
    return total;
}

/* ------------------------------------------------------------------ */
/* Seeded input generator shared with the device (no counterpart in    */
/* the reference).  Integer hash -> sum of eight 16-bit uniforms ->    */
/* one FP32 multiply and one FP32 add, so host and device agree bit    */
/* for bit without libm.                                               */
/* ------------------------------------------------------------------ */

static inline uint64_t hash64(uint64_t seed, uint64_t idx)
{
    uint64_t z = seed + idx * 0x9E3779B97F4A7C15ULL;
    z ^= z >> 30; z *= 0xBF58476D1CE4E5B9ULL;
    z ^= z >> 27; z *= 0x94D049BB133111EBULL;
    z ^= z >> 31;
    return z;
}

static inline float unit_normal(uint64_t seed, uint64_t idx)
{
    uint64_t a = hash64(seed, 2 * idx), b = hash64(seed, 2 * idx + 1);
    uint32_t s = 0;
    for (int k = 0; k < 4; k++) { s += (uint32_t)((a >> (16 * k)) & 0xFFFFu); s += (uint32_t)((b >> (16 * k)) & 0xFFFFu); }
    return ((float)(int32_t)s - 262140.0f) * 0x1.3988e2p-16f;      /* 1/sqrt(8*(65536^2-1)/12) */
}

#define ORC_FILL_ABS 1u      /* use |z| instead of z */

/*
 * value(i) = mean + std * z(seed, first + i); rows of row_len elements whose
 * hash(seed ^ ROW_SALT, row) >> 32 is below zero_rows_below are all zero.
 */
static inline float fill_value(uint64_t seed, uint64_t i, float mean, float std, uint32_t flags,
                               int64_t row_len, uint32_t zero_rows_below)
{
    if (row_len > 0 && zero_rows_below) {
        uint64_t row = i / (uint64_t)row_len;
        if ((uint32_t)(hash64(seed ^ 0xA5A5A5A55A5A5A5AULL, row) >> 32) < zero_rows_below) return 0.0f;
    }
    float z = unit_normal(seed, i);
    if (flags & ORC_FILL_ABS) z = fabsf(z);
    return mean + std * z;
}

void orc_fill_f16(uint16_t* dst, int64_t n, uint64_t seed, int64_t first, float mean, float std,
                  uint32_t flags, int64_t row_len, uint32_t zero_rows_below)
{
    for (int64_t i = 0; i < n; i++)
        dst[i] = f2h_inl(fill_value(seed, (uint64_t)(first + i), mean, std, flags, row_len, zero_rows_below));
}

void orc_fill_f32(float* dst, int64_t n, uint64_t seed, int64_t first, float mean, float std,
                  uint32_t flags, int64_t row_len, uint32_t zero_rows_below)
{
    for (int64_t i = 0; i < n; i++)
        dst[i] = fill_value(seed, (uint64_t)(first + i), mean, std, flags, row_len, zero_rows_below);
}

/* ------------------------------------------------------------------ */
/* Threaded FP16 step for the CPU baseline: static contiguous split.   */
/* ------------------------------------------------------------------ */

typedef struct {
    float* master; uint16_t* model; const uint16_t* grad; float* m; float* v;
    int64_t lo, hi;
    float lr, beta1, beta2, eps, wd, bc1_inv, bc2_inv, clip_scale; int apply_clip;
    double sumsq;
} mt_job;

static void* mt_update(void* arg)
{
    mt_job* j = (mt_job*)arg;
    adamw_fp16_range(j->master, j->model, j->grad, j->m, j->v, j->lo, j->hi, j->lr, j->beta1, j->beta2,
                     j->eps, j->wd, j->bc1_inv, j->bc2_inv, j->clip_scale, j->apply_clip);
    return NULL;
}

static void* mt_sumsq(void* arg)
{
    mt_job* j = (mt_job*)arg;
    j->sumsq = orc_sum_sq_half(j->grad + j->lo, j->hi - j->lo);
    return NULL;
}

static void run_jobs(mt_job* jobs, int threads, void* (*fn)(void*))
{
    pthread_t* tid = (pthread_t*)malloc(sizeof(pthread_t) * (size_t)threads);
    for (int t = 1; t < threads; t++) pthread_create(&tid[t], NULL, fn, &jobs[t]);
    fn(&jobs[0]);
    for (int t = 1; t < threads; t++) pthread_join(tid[t], NULL);
    free(tid);
}

/*
 * Norm (optional, max_norm > 0) + clip + update of one FP16 tensor on `threads` host
 * threads.  Same arithmetic per element as orc_adamw_fp16_clip; the norm is the FP64
 * sum of per-thread FP64 sums in thread order.  Returns the pre-clip norm (0 if off).
 */
float orc_step_fp16_threaded(
    float* master_w, uint16_t* model_w, const uint16_t* grad, float* m, float* v, int64_t n,
    float lr, float beta1, float beta2, float eps, float weight_decay,
    float bias_correction1, float bias_correction2, float max_norm, int threads)
{
    if (n <= 0) return 0.0f;
    if (threads < 1) threads = 1;
    mt_job* jobs = (mt_job*)calloc((size_t)threads, sizeof(mt_job));
    int64_t per = (n + threads - 1) / threads;
    for (int t = 0; t < threads; t++) {
        mt_job* j = &jobs[t];
        j->master = master_w; j->model = model_w; j->grad = grad; j->m = m; j->v = v;
        j->lo = per * t < n ? per * t : n;
        j->hi = per * (t + 1) < n ? per * (t + 1) : n;
        j->lr = lr; j->beta1 = beta1; j->beta2 = beta2; j->eps = eps; j->wd = weight_decay;
        j->bc1_inv = 1.0f / bias_correction1; j->bc2_inv = 1.0f / bias_correction2;
        j->clip_scale = 1.0f; j->apply_clip = 0;
    }
    float norm = 0.0f;
    if (max_norm > 0.0f) {
        run_jobs(jobs, threads, mt_sumsq);
        double s = 0.0;
        for (int t = 0; t < threads; t++) s += jobs[t].sumsq;
        float scale = orc_clip_scale((float)s, max_norm, &norm);
        if (norm > max_norm)
            for (int t = 0; t < threads; t++) { jobs[t].clip_scale = scale; jobs[t].apply_clip = 1; }
    }
    run_jobs(jobs, threads, mt_update);
    free(jobs);
    return norm;
}

/* ------------------------------------------------------------------ */
/* Threaded FP16 step over a LIST of tensors for the CPU baseline: the  */
/* concatenated index space of all tensors is split into `threads`      */
/* contiguous ranges, so small tensors cost no thread start of their    */
/* own.  Same arithmetic per element as orc_adamw_fp16_clip.            */
/* ------------------------------------------------------------------ */

typedef struct {
    int64_t n_tensors;
    uint16_t* const* model; const uint16_t* const* grad; float* const* m; float* const* v;
    const int64_t* start;            /* start[i] = elements before tensor i; start[n_tensors] = total */
    int64_t lo, hi;                  /* this thread's range of the concatenated index space */
    float lr, beta1, beta2, eps, wd, bc1_inv, bc2_inv, clip_scale; int apply_clip;
    double sumsq;
} list_job;

static int64_t list_first_tensor(const list_job* j)
{
    int64_t a = 0, b = j->n_tensors;             /* last i with start[i] <= lo */
    while (b - a > 1) { int64_t mid = (a + b) / 2; if (j->start[mid] <= j->lo) a = mid; else b = mid; }
    return a;
}

static void* list_update(void* arg)
{
    list_job* j = (list_job*)arg;
    for (int64_t i = list_first_tensor(j); i < j->n_tensors && j->start[i] < j->hi; i++) {
        int64_t lo = j->lo > j->start[i] ? j->lo - j->start[i] : 0;
        int64_t n = j->start[i + 1] - j->start[i];
        int64_t hi = j->hi - j->start[i] < n ? j->hi - j->start[i] : n;
        if (hi > lo)
            adamw_fp16_range(NULL, j->model[i], j->grad[i], j->m[i], j->v[i], lo, hi, j->lr, j->beta1, j->beta2, j->eps,
                             j->wd, j->bc1_inv, j->bc2_inv, j->clip_scale, j->apply_clip);
    }
    return NULL;
}

static void* list_sumsq(void* arg)
{
    list_job* j = (list_job*)arg;
    double s = 0.0;
    for (int64_t i = list_first_tensor(j); i < j->n_tensors && j->start[i] < j->hi; i++) {
        int64_t lo = j->lo > j->start[i] ? j->lo - j->start[i] : 0;
        int64_t n = j->start[i + 1] - j->start[i];
        int64_t hi = j->hi - j->start[i] < n ? j->hi - j->start[i] : n;
        if (hi > lo) s += orc_sum_sq_half(j->grad[i] + lo, hi - lo);
    }
    j->sumsq = s;
    return NULL;
}

static void run_list_jobs(list_job* jobs, int threads, void* (*fn)(void*))
{
    pthread_t* tid = (pthread_t*)malloc(sizeof(pthread_t) * (size_t)threads);
    for (int t = 1; t < threads; t++) pthread_create(&tid[t], NULL, fn, &jobs[t]);
    fn(&jobs[0]);
    for (int t = 1; t < threads; t++) pthread_join(tid[t], NULL);
    free(tid);
}

/*
 * Norm (optional, max_norm > 0: FP64 sum of per-thread FP64 sums in thread order, then the clip rule of
 * trainer.h:341-345) + update of n_tensors FP16 tensors (no master copy) on `threads` host threads.
 * counts[i] elements each; every tensor takes the same weight decay.  Returns the pre-clip norm (0 if off).
 */
float orc_step_list_fp16_threaded(
    int64_t n_tensors, uint16_t* const* model_w, const uint16_t* const* grad, float* const* m, float* const* v,
    const int64_t* counts, float lr, float beta1, float beta2, float eps, float weight_decay,
    float bias_correction1, float bias_correction2, float max_norm, int threads)
{
    if (n_tensors <= 0) return 0.0f;
    if (threads < 1) threads = 1;
    int64_t* start = (int64_t*)malloc(sizeof(int64_t) * (size_t)(n_tensors + 1));
    start[0] = 0;
    for (int64_t i = 0; i < n_tensors; i++) start[i + 1] = start[i] + (counts[i] > 0 ? counts[i] : 0);
    const int64_t total = start[n_tensors];
    list_job* jobs = (list_job*)calloc((size_t)threads, sizeof(list_job));
    const int64_t per = (total + threads - 1) / threads;
    for (int t = 0; t < threads; t++) {
        list_job* j = &jobs[t];
        j->n_tensors = n_tensors; j->model = model_w; j->grad = grad; j->m = m; j->v = v; j->start = start;
        j->lo = per * t < total ? per * t : total;
        j->hi = per * (t + 1) < total ? per * (t + 1) : total;
        j->lr = lr; j->beta1 = beta1; j->beta2 = beta2; j->eps = eps; j->wd = weight_decay;
        j->bc1_inv = 1.0f / bias_correction1; j->bc2_inv = 1.0f / bias_correction2;
        j->clip_scale = 1.0f; j->apply_clip = 0;
    }
    float norm = 0.0f;
    if (max_norm > 0.0f) {
        run_list_jobs(jobs, threads, list_sumsq);
        double s = 0.0;
        for (int t = 0; t < threads; t++) s += jobs[t].sumsq;
        float scale = orc_clip_scale((float)s, max_norm, &norm);
        if (norm > max_norm)
            for (int t = 0; t < threads; t++) { jobs[t].clip_scale = scale; jobs[t].apply_clip = 1; }
    }
    run_list_jobs(jobs, threads, list_update);
    free(jobs);
    free(start);
    return norm;
}

/*
 * The update of the same list as a loop over the tensors, each tensor split over the threads by itself
 * (orc_step_fp16_threaded without clipping): what one call per tensor costs on the host, for comparison
 * with the single split above.  Same results.
 */
void orc_update_per_tensor_fp16_threaded(
    int64_t n_tensors, uint16_t* const* model_w, const uint16_t* const* grad, float* const* m, float* const* v,
    const int64_t* counts, float lr, float beta1, float beta2, float eps, float weight_decay,
    float bias_correction1, float bias_correction2, int threads)
{
    for (int64_t i = 0; i < n_tensors; i++)
        orc_step_fp16_threaded(NULL, model_w[i], grad[i], m[i], v[i], counts[i], lr, beta1, beta2, eps, weight_decay,
                               bias_correction1, bias_correction2, 0.0f, threads);
}
