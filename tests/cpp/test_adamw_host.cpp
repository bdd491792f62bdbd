// test_adamw_host.cpp
//
// C++ host-side test of the optimizer path on a GPU, shaped like the reference's
// tests/test_adamw.cu (standalone executable, PASS/FAIL lines, exit code = failures), but on
// seeded synthetic weights and gradients instead of a loaded model:
//   1. FP32 AdamW vs an inline CPU loop (step 1, no decay)            max err < 1e-6
//   2. FP16 AdamW vs an inline CPU loop and vs the C oracle           master err < 1e-6; oracle: identical bits
//   3. moments finite and non-zero after a step
//   4. get_step() counts 0 -> 3
//   5. clip_grad_norm_ returns the pre-clip norm; clipped gradients have norm <= max; fused == unfused
//   6. operator API (launch_adamw_fp16 / launch_adamw_fp32) on raw pointers
//   7. frozen embedding flagged in the plan, gradients cleared inside the update
//   8. optimizer state save / load   9. train loop with LR schedule and JSON-lines log
//   10. gradient pools   11. training_step with accumulation   12. steps from an uploaded table of hyper-parameters
//   13. one recorded clip + scheduled step replayed through three uploaded windows, against the oracle
// The oracle (liborc_adamw.so) is used as the checker only.
#include <cmath>
#include <cstdint>
#include <cstdio>
#include <filesystem>
#include <string>
#include <vector>

#include "training/optim_step.h"

extern "C" {
float orc_h2f(uint16_t h);
uint16_t orc_f2h(float f);
void orc_adamw_fp16(float*, uint16_t*, const uint16_t*, float*, float*, int64_t, float, float, float, float, float,
                    float, float);
void orc_adamw_fp16_clip(float*, uint16_t*, const uint16_t*, float*, float*, int64_t, float, float, float, float,
                         float, float, float, float, int);
void orc_adamw_fp32(float*, const float*, float*, float*, int64_t, float, float, float, float, float, float, float);
float orc_clip_grad_norm(uint16_t*, int64_t, float*, int64_t, float, float*);
double orc_sum_sq_half(const uint16_t*, int64_t);
double orc_sum_sq_float(const float*, int64_t);
int64_t orc_sumsq_mirror_partials(const void* g, int is_f32, int64_t n, int chunk, double* partials);
double orc_sumsq_mirror_total(const double* partials, int64_t n_partials, int chunk);
float orc_clip_scale(float sum_sq, float max_norm, float* norm);
void orc_scale_half(uint16_t*, float, int64_t);
void orc_scale_float(float*, float, int64_t);
void orc_optimizer_step(float* master, uint16_t* pool16, const uint16_t* g16, float* m16, float* v16, int64_t n16,
                        int64_t proj_n, float* pool32, const float* g32, float* m32, float* v32, int64_t n32, float lr,
                        float beta1, float beta2, float eps, float wd, int* step);
}

static int g_fails = 0;
#define PASS(name) printf("[PASS] %s\n", (name))
#define FAIL(name, ...) do { printf("[FAIL] %s: ", (name)); printf(__VA_ARGS__); printf("\n"); g_fails++; } while (0)

// A small model-shaped pool set: projections, embedding, norm weights, and a workspace tail
// behind the norm gradients.
struct Fixture {
    size_t proj_n = 3 * 8192 + 1024, embed_n = 500 * 64, n32 = 2304 + 64, tail = 777;
    size_t n16 = proj_n + embed_n;
    half *w16 = nullptr, *g16 = nullptr;
    float *w32 = nullptr, *g32 = nullptr;
    ParamPools pools;
    GradPools grads;
    std::vector<uint16_t> h_w16, h_g16;
    std::vector<float> h_w32, h_g32;

    explicit Fixture(float grad_std) {
        HIP_CHECK(hipMalloc((void**)&w16, n16 * 2));
        HIP_CHECK(hipMalloc((void**)&g16, n16 * 2));
        HIP_CHECK(hipMalloc((void**)&w32, n32 * 4));
        HIP_CHECK(hipMalloc((void**)&g32, (n32 + tail) * 4));
        RLX_CHECK(rlx_fill_f16((uint16_t*)w16, n16, 1, 0, 0.0f, 0.02f, 0, 0, 0, nullptr));
        RLX_CHECK(rlx_fill_f16((uint16_t*)g16, n16, 2, 0, 0.0f, grad_std, 0, 0, 0, nullptr));
        RLX_CHECK(rlx_fill_f32(w32, n32, 3, 0, 1.0f, 0.05f, 0, 0, 0, nullptr));
        RLX_CHECK(rlx_fill_f32(g32, n32 + tail, 4, 0, 0.0f, grad_std, 0, 0, 0, nullptr));
        HIP_CHECK(hipDeviceSynchronize());
        pools.fp16_pool = w16; pools.fp16_pool_elems = n16; pools.proj_elems = proj_n;
        pools.fp32_pool = w32; pools.fp32_pool_elems = n32;
        grads.half_pool = g16; grads.half_pool_bytes = n16 * 2;
        grads.float_pool = g32; grads.float_pool_bytes = (n32 + tail) * 4;
        h_w16.resize(n16); h_g16.resize(n16); h_w32.resize(n32); h_g32.resize(n32 + tail);
        download();
    }
    void download() {
        HIP_CHECK(hipMemcpy(h_w16.data(), w16, n16 * 2, hipMemcpyDeviceToHost));
        HIP_CHECK(hipMemcpy(h_g16.data(), g16, n16 * 2, hipMemcpyDeviceToHost));
        HIP_CHECK(hipMemcpy(h_w32.data(), w32, n32 * 4, hipMemcpyDeviceToHost));
        HIP_CHECK(hipMemcpy(h_g32.data(), g32, (n32 + tail) * 4, hipMemcpyDeviceToHost));
    }
    ~Fixture() { (void)hipFree(w16); (void)hipFree(g16); (void)hipFree(w32); (void)hipFree(g32); }
};

template <typename T> static std::vector<T> d2h(const T* d, size_t n) {
    std::vector<T> h(n);
    HIP_CHECK(hipMemcpy(h.data(), d, n * sizeof(T), hipMemcpyDeviceToHost));
    return h;
}

// The oracle's copy of a Fixture's training state, advanced on the host in the reference's order
// (trainer.h:279-286): norm of all gradients, added up in the device's fixed order so that it can be compared
// bit for bit, clip rule, scale pass if norm > max, optimizer step with the three decay groups.
struct OracleReplay {
    Fixture& f;
    std::vector<float> master, m16, v16, w32, m32, v32;
    std::vector<uint16_t> w16;
    int step = 0;
    float beta1 = 0.9f, beta2 = 0.999f, eps = 1e-8f, wd = 0.01f;

    explicit OracleReplay(Fixture& fx) : f(fx), master(fx.n16), m16(fx.n16, 0.0f), v16(fx.n16, 0.0f), w32(fx.h_w32),
                                         m32(fx.n32, 0.0f), v32(fx.n32, 0.0f), w16(fx.h_w16) {
        for (size_t i = 0; i < fx.n16; i++) master[i] = orc_h2f(fx.h_w16[i]);
    }
    // One step on the gradients that the device holds now.  Returns the pre-clip norm.
    float advance(float lr, float max_norm, int64_t chunk) {
        std::vector<uint16_t> g16 = d2h((const uint16_t*)f.g16, f.n16);
        std::vector<float> g32 = d2h((const float*)f.g32, f.n32 + f.tail);
        float norm = 0.0f;
        if (max_norm > 0.0f) {
            std::vector<double> partials((f.n16 + f.n32 + f.tail) / 512 + 16);
            int64_t k = 0;      // plan order: projections, embedding, norm gradients, workspace tail
            k += orc_sumsq_mirror_partials(g16.data(), 0, (int64_t)f.proj_n, (int)chunk, partials.data() + k);
            k += orc_sumsq_mirror_partials(g16.data() + f.proj_n, 0, (int64_t)f.embed_n, (int)chunk, partials.data() + k);
            k += orc_sumsq_mirror_partials(g32.data(), 1, (int64_t)f.n32, (int)chunk, partials.data() + k);
            k += orc_sumsq_mirror_partials(g32.data() + f.n32, 1, (int64_t)f.tail, (int)chunk, partials.data() + k);
            const float scale = orc_clip_scale((float)orc_sumsq_mirror_total(partials.data(), k, (int)chunk), max_norm, &norm);
            if (norm > max_norm) {
                orc_scale_half(g16.data(), scale, (int64_t)f.n16);
                orc_scale_float(g32.data(), scale, (int64_t)(f.n32 + f.tail));
            }
        }
        orc_optimizer_step(master.data(), w16.data(), g16.data(), m16.data(), v16.data(), (int64_t)f.n16,
                           (int64_t)f.proj_n, w32.data(), g32.data(), m32.data(), v32.data(), (int64_t)f.n32, lr, beta1,
                           beta2, eps, wd, &step);
        return norm;
    }
    // Values of the device state (weights, master copy, moments) that differ from the oracle's in any bit.
    size_t differences(AdamWOptimizer& opt) const {
        size_t diff = 0;
        const auto dw16 = d2h((const uint16_t*)f.w16, f.n16);
        const auto dw32 = d2h((const float*)f.w32, f.n32);
        const auto dmaster = d2h((const float*)opt.fp16_master(), f.n16);
        const auto dm16 = d2h((const float*)opt.fp16_m(), f.n16), dv16 = d2h((const float*)opt.fp16_v(), f.n16);
        const auto dm32 = d2h((const float*)opt.fp32_m(), f.n32), dv32 = d2h((const float*)opt.fp32_v(), f.n32);
        for (size_t i = 0; i < f.n16; i++)
            diff += dw16[i] != w16[i] || memcmp(&dmaster[i], &master[i], 4) || memcmp(&dm16[i], &m16[i], 4) ||
                    memcmp(&dv16[i], &v16[i], 4);
        for (size_t i = 0; i < f.n32; i++)
            diff += memcmp(&dw32[i], &w32[i], 4) || memcmp(&dm32[i], &m32[i], 4) || memcmp(&dv32[i], &v32[i], 4);
        return diff;
    }
};

// 1. FP32 path vs the CPU loop of the reference's test (step 1, division by the bias corrections)
static void test_cpu_reference_fp32() {
    const char* name = "CPU reference: FP32 AdamW (norm weights)";
    Fixture f(1e-2f);
    AdamWOptimizer opt(f.pools, /*lr=*/1e-3f);
    float bc1 = 1.0f - opt.beta1, bc2 = 1.0f - opt.beta2;
    std::vector<float> cpu_w(f.n32);
    for (size_t i = 0; i < f.n32; i++) {
        float g = f.h_g32[i];
        float mi = (1.0f - opt.beta1) * g, vi = (1.0f - opt.beta2) * g * g;
        float m_hat = mi / bc1, v_hat = vi / bc2;
        cpu_w[i] = f.h_w32[i] - opt.lr * m_hat / (sqrtf(v_hat) + opt.eps);
    }
    opt.step(&f.grads);
    HIP_CHECK(hipDeviceSynchronize());
    auto gpu_w = d2h(f.w32, f.n32);
    float max_err = 0.0f;
    for (size_t i = 0; i < f.n32; i++) max_err = fmaxf(max_err, fabsf(gpu_w[i] - cpu_w[i]));
    printf("  max_err(GPU vs CPU) = %.8e\n", max_err);
    if (max_err < 1e-6f) PASS(name); else FAIL(name, "max_err=%.8e", max_err);
}

// 2. FP16 path (projections: decay 0.01) vs the inline loop and vs the oracle
static void test_cpu_reference_fp16() {
    const char* name = "CPU reference: FP16 AdamW (projections)";
    Fixture f(1e-3f);
    AdamWOptimizer opt(f.pools, 1e-3f, 0.9f, 0.999f, 1e-8f, 0.01f);
    const size_t n = f.proj_n;
    float bc1 = 1.0f - opt.beta1, bc2 = 1.0f - opt.beta2;
    std::vector<float> cpu_master(n);
    for (size_t i = 0; i < n; i++) {
        float g = orc_h2f(f.h_g16[i]);
        float mi = (1.0f - opt.beta1) * g, vi = (1.0f - opt.beta2) * g * g;
        float m_hat = mi / bc1, v_hat = vi / bc2;
        cpu_master[i] = orc_h2f(f.h_w16[i]) * (1.0f - opt.lr * opt.weight_decay) - opt.lr * m_hat / (sqrtf(v_hat) + opt.eps);
    }
    // oracle: whole FP16 pool, embedding without decay (optimizer.h:131-140)
    std::vector<float> o_master(f.n16), o_m(f.n16, 0.0f), o_v(f.n16, 0.0f);
    for (size_t i = 0; i < f.n16; i++) o_master[i] = orc_h2f(f.h_w16[i]);
    std::vector<uint16_t> o_w = f.h_w16;
    orc_adamw_fp16(o_master.data(), o_w.data(), f.h_g16.data(), o_m.data(), o_v.data(), n, opt.lr, opt.beta1,
                   opt.beta2, opt.eps, opt.weight_decay, bc1, bc2);
    orc_adamw_fp16(o_master.data() + n, o_w.data() + n, f.h_g16.data() + n, o_m.data() + n, o_v.data() + n,
                   f.n16 - n, opt.lr, opt.beta1, opt.beta2, opt.eps, 0.0f, bc1, bc2);
    opt.step(&f.grads);
    HIP_CHECK(hipDeviceSynchronize());
    auto gpu_w = d2h((const uint16_t*)f.w16, f.n16);
    auto gpu_master = d2h(opt.fp16_master(), f.n16);
    auto gpu_m = d2h(opt.fp16_m(), f.n16);
    auto gpu_v = d2h(opt.fp16_v(), f.n16);
    float max_err_master = 0.0f;
    for (size_t i = 0; i < n; i++) max_err_master = fmaxf(max_err_master, fabsf(gpu_master[i] - cpu_master[i]));
    size_t vs_oracle = 0, not_f2h = 0;
    for (size_t i = 0; i < f.n16; i++) {
        if (gpu_w[i] != o_w[i] || memcmp(&gpu_master[i], &o_master[i], 4) || memcmp(&gpu_m[i], &o_m[i], 4) ||
            memcmp(&gpu_v[i], &o_v[i], 4))
            vs_oracle++;
        if (gpu_w[i] != orc_f2h(gpu_master[i])) not_f2h++;
    }
    printf("  master max_err=%.8e  mismatches vs oracle=%zu/%zu  model!=f2h(master): %zu\n", max_err_master,
           vs_oracle, f.n16, not_f2h);
    if (max_err_master < 1e-6f && vs_oracle == 0 && not_f2h == 0) PASS(name);
    else FAIL(name, "master_err=%.8e oracle_mismatch=%zu", max_err_master, vs_oracle);
}

// 3. moments are finite and non-zero after a step
static void test_moments_nonzero() {
    const char* name = "Moments non-zero after step";
    Fixture f(1e-3f);
    AdamWOptimizer opt(f.pools, 1e-4f);
    opt.step(&f.grads);
    HIP_CHECK(hipDeviceSynchronize());
    auto m = d2h(opt.fp16_m(), f.n16);
    auto v = d2h(opt.fp32_v(), f.n32);
    size_t nz_m = 0, nz_v = 0, bad = 0;
    for (float x : m) { nz_m += x != 0.0f; bad += !std::isfinite(x); }
    for (float x : v) { nz_v += x != 0.0f; bad += !std::isfinite(x); }
    if (bad == 0 && nz_m > f.n16 / 2 && nz_v > f.n32 / 2) PASS(name); else FAIL(name, "nz_m=%zu nz_v=%zu bad=%zu", nz_m, nz_v, bad);
}

// 4. step counter
static void test_step_counter() {
    const char* name = "get_step() counts steps";
    Fixture f(1e-3f);
    AdamWOptimizer opt(f.pools, 1e-4f);
    bool ok = opt.get_step() == 0;
    for (int i = 0; i < 3; i++) opt.step(&f.grads);
    HIP_CHECK(hipDeviceSynchronize());
    ok = ok && opt.get_step() == 3;
    // (layer, tensor) accessors follow the pool order of the reference
    ParamPools q = ParamPools::for_qwen3(28, 1024, 2048, 1024, 3072, 128, 151936);
    ok = ok && q.fp16_pool_elems == 595984384u && q.fp32_pool_elems == 65536u && q.proj_elems == 440401920u;
    ParamPools small = ParamPools::for_qwen3(2, 32, 64, 16, 80, 16, 1000);
    ok = ok && small.fp16_pool_elems == f.n16 && small.proj_elems == f.proj_n && small.fp32_pool_elems == 224u;
    small.fp16_pool = f.w16; small.fp32_pool = f.w32;
    {
        AdamWOptimizer lay(small, 1e-4f);
        const size_t per16 = 12800, q = 64 * 32, kv = 16 * 32;
        ok = ok && lay.get_fp16_m(0, 0) == lay.fp16_m() && lay.get_fp16_m(1, 0) == lay.fp16_m() + per16 &&
             lay.get_fp16_v(0, 3) == lay.fp16_v() + q + 2 * kv &&
             lay.get_fp16_master(1, 6) == lay.fp16_master() + 2 * per16 - 32 * 80 &&
             lay.get_fp32_m_norm(1, 2) == lay.fp32_m() + 96 + 32 + 16 &&
             lay.get_final_norm_v() == lay.fp32_v() + 192;
    }
    AdamWOptimizer moved(std::move(opt));
    ok = ok && moved.get_step() == 3 && opt.fp16_m() == nullptr;
    moved.set_lr(5e-5f);
    ok = ok && moved.lr == 5e-5f;
    if (ok) PASS(name); else FAIL(name, "step=%d", moved.get_step());
}

// 5. clip: pre-clip norm returned, workspace tail included and scaled, fused == unfused
static void test_clip() {
    const char* name = "clip_grad_norm_ and fused clip";
    const float max_norm = 0.25f;
    Fixture a(5e-3f), b(5e-3f);
    AdamWOptimizer oa(a.pools, 1e-3f, 0.9f, 0.999f, 1e-8f, 0.01f, /*use_master=*/false);
    AdamWOptimizer ob(b.pools, 1e-3f, 0.9f, 0.999f, 1e-8f, 0.01f, /*use_master=*/false);
    OptimStepConfig ca; ca.max_grad_norm = max_norm;
    OptimStepConfig cb = ca; cb.fused_clip = true;
    OptimStep sa(&oa, ca), sb(&ob, cb);
    std::vector<uint16_t> og16 = a.h_g16;
    std::vector<float> og32 = a.h_g32;
    float o_scale = 0.0f;
    float o_norm = orc_clip_grad_norm(og16.data(), a.n16, og32.data(), a.n32 + a.tail, max_norm, &o_scale);
    float na = sa.apply(&a.grads), nb = sb.apply(&b.grads);
    HIP_CHECK(hipDeviceSynchronize());
    bool ok = na == nb && fabsf(na - o_norm) <= 1e-5f * o_norm && na > max_norm;
    a.download(); b.download();
    size_t bad_g = 0, untouched = 0, diff = 0;
    for (size_t i = 0; i < a.n16; i++) { bad_g += a.h_g16[i] != og16[i]; diff += a.h_w16[i] != b.h_w16[i]; }
    for (size_t i = 0; i < a.n32 + a.tail; i++) bad_g += memcmp(&a.h_g32[i], &og32[i], 4) != 0;
    Fixture fresh(5e-3f);
    for (size_t i = 0; i < b.n16; i++) untouched += b.h_g16[i] == fresh.h_g16[i];
    for (size_t i = 0; i < a.n32; i++) diff += memcmp(&a.h_w32[i], &b.h_w32[i], 4) != 0;
    double post = sqrt(orc_sum_sq_half(a.h_g16.data(), a.n16) + orc_sum_sq_float(a.h_g32.data(), a.n32 + a.tail));
    printf("  norm=%.6f (oracle %.6f)  scaled-grad mismatches=%zu  fused-vs-unfused diffs=%zu  post-clip norm=%.6f\n",
           na, o_norm, bad_g, diff, post);
    ok = ok && bad_g == 0 && diff == 0 && untouched == b.n16 && post <= max_norm * 1.002;
    if (ok) PASS(name); else FAIL(name, "na=%f nb=%f", na, nb);
}

// 6. operator API on raw pointers, n <= 0 no-op
static void test_launch_api() {
    const char* name = "launch_adamw_fp16 / launch_adamw_fp32";
    Fixture f(1e-3f);
    float *m, *v;
    const int n = 10007;
    HIP_CHECK(hipMalloc((void**)&m, n * 4)); HIP_CHECK(hipMalloc((void**)&v, n * 4));
    HIP_CHECK(hipMemset(m, 0, n * 4)); HIP_CHECK(hipMemset(v, 0, n * 4));
    launch_adamw_fp16(nullptr, f.w16, f.g16, m, v, 0, 1e-3f, 0.9f, 0.999f, 1e-8f, 0.01f, 0.1f, 0.001f);   // no-op
    launch_adamw_fp16(nullptr, f.w16, f.g16, m, v, n, 1e-3f, 0.9f, 0.999f, 1e-8f, 0.01f, 0.1f, 0.001f);
    HIP_CHECK(hipDeviceSynchronize());
    std::vector<uint16_t> w = f.h_w16;
    std::vector<float> om(n, 0.0f), ov(n, 0.0f);
    orc_adamw_fp16(nullptr, w.data(), f.h_g16.data(), om.data(), ov.data(), n, 1e-3f, 0.9f, 0.999f, 1e-8f, 0.01f, 0.1f, 0.001f);
    auto gw = d2h((const uint16_t*)f.w16, f.n16);
    auto gm = d2h(m, n);
    size_t bad = 0;
    for (size_t i = 0; i < f.n16; i++) bad += gw[i] != w[i];
    for (int i = 0; i < n; i++) bad += memcmp(&gm[i], &om[i], 4) != 0;
    HIP_CHECK(hipMemset(m, 0, n * 4)); HIP_CHECK(hipMemset(v, 0, n * 4));
    launch_adamw_fp32(f.w32, f.g32, m, v, (int)f.n32, 1e-3f, 0.9f, 0.999f, 1e-8f, 0.0f, 0.1f, 0.001f);
    HIP_CHECK(hipDeviceSynchronize());
    std::vector<float> w32 = f.h_w32, m32(f.n32, 0.0f), v32(f.n32, 0.0f);
    orc_adamw_fp32(w32.data(), f.h_g32.data(), m32.data(), v32.data(), f.n32, 1e-3f, 0.9f, 0.999f, 1e-8f, 0.0f, 0.1f, 0.001f);
    auto gw32 = d2h(f.w32, f.n32);
    for (size_t i = 0; i < f.n32; i++) bad += memcmp(&gw32[i], &w32[i], 4) != 0;
    (void)hipFree(m); (void)hipFree(v);
    if (bad == 0) PASS(name); else FAIL(name, "%zu mismatches", bad);
}

// 7. frozen embedding in the plan + gradient clearing inside the update == memset + identity update
static void test_frozen_and_zeroing() {
    const char* name = "frozen embedding and zeroing in the update";
    Fixture a(5e-3f), b(5e-3f);
    AdamWOptimizer oa(a.pools, 1e-3f), ob(b.pools, 1e-3f);
    OptimStepConfig ca; ca.max_grad_norm = 0.25f; ca.freeze_embed = true; ca.fused_clip = true;
    OptimStepConfig cb = ca; cb.freeze_in_plan = true; cb.zero_grads = true;
    OptimStep sa(&oa, ca), sb(&ob, cb);
    float na = sa.apply(&a.grads, a.embed_n), nb = sb.apply(&b.grads, b.embed_n);
    HIP_CHECK(hipDeviceSynchronize());
    std::vector<uint16_t> w0 = a.h_w16;
    a.download(); b.download();
    size_t diff = 0, nonzero = 0, moved = 0;
    for (size_t i = 0; i < a.n16; i++) diff += a.h_w16[i] != b.h_w16[i];
    for (size_t i = 0; i < a.n32; i++) diff += memcmp(&a.h_w32[i], &b.h_w32[i], 4) != 0;
    for (size_t i = a.proj_n; i < a.n16; i++) moved += a.h_w16[i] != w0[i];
    for (uint16_t x : b.h_g16) nonzero += x != 0;
    for (float x : b.h_g32) nonzero += x != 0.0f;
    auto ma = d2h(oa.fp16_m(), a.n16), mb = d2h(ob.fp16_m(), b.n16);
    for (size_t i = 0; i < a.n16; i++) diff += memcmp(&ma[i], &mb[i], 4) != 0;
    printf("  norm %.6f / %.6f  diffs=%zu  embedding weights moved=%zu  gradients left=%zu\n", na, nb, diff, moved, nonzero);
    if (na == nb && diff == 0 && moved == 0 && nonzero == 0) PASS(name); else FAIL(name, "diff=%zu", diff);
}

// 8. optimizer state: save, continue, reload into a fresh optimizer, continue: identical bits
static void test_checkpoint() {
    const char* name = "optimizer state save / load";
    const std::string path = "/tmp/rlx_test_opt.state";
    Fixture a(5e-3f), b(5e-3f);
    AdamWOptimizer oa(a.pools, 1e-3f), ob(b.pools, 1e-3f);
    OptimStepConfig c; c.max_grad_norm = 0.25f; c.fused_clip = true;
    OptimStep sa(&oa, c), sb(&ob, c);
    oa.set_state_staging(10000);      // sections of 57,600 and 2,368 floats pass through a 10,000-float buffer
    ob.set_state_staging(777);
    for (int i = 0; i < 3; i++) sa.apply(&a.grads);
    bool ok = oa.save_state(path);
    HIP_CHECK(hipMemcpy(b.w16, a.w16, a.n16 * 2, hipMemcpyDeviceToDevice));   // weights are the model's to save
    HIP_CHECK(hipMemcpy(b.w32, a.w32, a.n32 * 4, hipMemcpyDeviceToDevice));
    ok = ok && ob.load_state(path) && ob.get_step() == 3;
    for (int i = 0; i < 2; i++) { sa.apply(&a.grads); sb.apply(&b.grads); }
    HIP_CHECK(hipDeviceSynchronize());
    a.download(); b.download();
    size_t diff = 0;
    for (size_t i = 0; i < a.n16; i++) diff += a.h_w16[i] != b.h_w16[i];
    auto ma = d2h(oa.fp16_master(), a.n16), mb = d2h(ob.fp16_master(), b.n16);
    auto va = d2h(oa.fp32_v(), a.n32), vb = d2h(ob.fp32_v(), b.n32);
    for (size_t i = 0; i < a.n16; i++) diff += memcmp(&ma[i], &mb[i], 4) != 0;
    for (size_t i = 0; i < a.n32; i++) diff += memcmp(&va[i], &vb[i], 4) != 0;
    // a damaged file is refused and changes nothing
    FILE* f = fopen(path.c_str(), "r+b");
    fseek(f, -9, SEEK_END); fputc(0x5A, f); fclose(f);
    AdamWOptimizer oc(a.pools, 1e-3f);
    bool refused = !oc.load_state(path) && oc.get_step() == 0 && !oc.load_state("/tmp/rlx_no_such_file");
    remove(path.c_str());
    if (ok && diff == 0 && refused && ob.get_step() == 5) PASS(name); else FAIL(name, "ok=%d diff=%zu refused=%d", ok, diff, refused);
}

// 9. scheduled learning rate, train loop, JSON-lines log: the loop's logged pre-clip norm (trainer.h:208-216,
//    288, 351) and the state it leaves are those of the oracle replaying set_lr -> clip -> step on the host;
//    the state file written at save_steps holds the oracle's state of that step
static void test_train_loop() {
    const char* name = "train loop with LR schedule and JSONL log == oracle replay";
    const std::string dir = "/tmp/rlx_test_run";
    std::filesystem::remove_all(dir);
    std::filesystem::create_directories(dir);
    Fixture f(5e-3f);
    AdamWOptimizer opt(f.pools, 1e-3f);
    OracleReplay oracle(f);
    LRScheduler sched;
    sched.init_cosine(1e-3f, 1e-4f, 2, 8);
    OptimStepConfig c; c.max_grad_norm = 0.25f; c.fused_clip = true;
    OptimStep tail(&opt, c);
    TrainLoopConfig lc; lc.total_steps = 8; lc.logging_steps = 2; lc.tokens_per_step = 4096.0f;
    lc.save_steps = 4; lc.save_path = dir + "/opt_state.bin";
    const int64_t chunk = rlx_plan_chunk_elems(opt.plan_for(&f.grads));
    std::vector<float> norms;                       // the oracle's pre-clip norm of every step
    size_t saved_diff = 0;
    int steps;
    {
        Logger logger(dir);
        steps = run_train_loop(opt, sched, logger, tail, &f.grads, [&](int s) {
            if (s == 4) {     // the loop has just written the state of step 4: load it into a second optimizer
                Fixture g(5e-3f);
                AdamWOptimizer reloaded(g.pools, 1e-3f);
                OracleReplay then = oracle;
                const bool ok = reloaded.load_state(lc.save_path) && reloaded.get_step() == 4;
                // weights are not part of the state file: compare master copy and moments
                const auto dmaster = d2h((const float*)reloaded.fp16_master(), g.n16);
                const auto dm = d2h((const float*)reloaded.fp16_m(), g.n16), dv = d2h((const float*)reloaded.fp16_v(), g.n16);
                const auto dm32 = d2h((const float*)reloaded.fp32_m(), g.n32), dv32 = d2h((const float*)reloaded.fp32_v(), g.n32);
                saved_diff += ok ? 0 : 1;
                for (size_t i = 0; i < g.n16; i++)
                    saved_diff += memcmp(&dmaster[i], &then.master[i], 4) || memcmp(&dm[i], &then.m16[i], 4) ||
                                  memcmp(&dv[i], &then.v16[i], 4);
                for (size_t i = 0; i < g.n32; i++) saved_diff += memcmp(&dm32[i], &then.m32[i], 4) || memcmp(&dv32[i], &then.v32[i], 4);
            }
            RLX_CHECK(rlx_fill_f16((uint16_t*)f.g16, f.n16, 100 + s, 0, 0.0f, 5e-3f, 0, 0, 0, nullptr));
            HIP_CHECK(hipDeviceSynchronize());
            norms.push_back(oracle.advance(sched.get_lr(s), c.max_grad_norm, chunk));
            return 3.0f / (1 + s);
        }, lc);
        bool ok = steps == 8 && opt.get_step() == 8 && logger.history().size() == 4 && opt.lr == sched.get_lr(7) &&
                  logger.history()[0].step == 2 && fabsf(logger.last("loss") - (3.0f / 7 + 3.0f / 8) / 2) < 1e-6f &&
                  std::isnan(logger.last("nope"));
        // every logged window mean of grad_norm is the FP32 mean of the oracle's norms of its two steps
        size_t norm_diff = 0;
        for (size_t w = 0; ok && w < 4; w++) {
            const float want = (0.0f + norms[2 * w] + norms[2 * w + 1]) / 2.0f;
            const float got = logger.history()[w].values.at("grad_norm");
            norm_diff += memcmp(&want, &got, 4) != 0;
            ok = ok && norms[2 * w] > 0.25f && fabsf(got - want) <= 1e-7f * want;
        }
        const size_t state_diff = oracle.differences(opt);
        printf("  logged grad_norm windows differing from the oracle's: %zu; state values differing after 8 steps: %zu; "
               "in the state file of step 4: %zu\n", norm_diff, state_diff, saved_diff);
        if (!ok || norm_diff || state_diff || saved_diff || oracle.step != 8) {
            FAIL(name, "ok=%d norm_diff=%zu state_diff=%zu saved_diff=%zu", ok, norm_diff, state_diff, saved_diff);
            return;
        }
    }
    FILE* fp = fopen((dir + "/train_log.jsonl").c_str(), "r");
    int lines = 0; char buf[1024]; bool shape = fp != nullptr;
    while (fp && fgets(buf, sizeof(buf), fp)) {
        lines++;
        std::string l(buf);
        shape = shape && l.rfind("{\"grad_norm\":", 0) == 0 && l.find("\"loss\":") != std::string::npos &&
                l.find("\"lr\":") != std::string::npos && l.find("\"step\":" + std::to_string(2 * lines)) != std::string::npos &&
                l.find("\"step_ms\":") != std::string::npos && l.find("\"tok_per_sec\":") != std::string::npos;
    }
    if (fp) fclose(fp);
    std::filesystem::remove_all(dir);
    if (shape && lines == 4 && Logger::number(1e-5) == "1e-05" && Logger::number(2.0) == "2.0") PASS(name);
    else FAIL(name, "lines=%d shape=%d", lines, shape);
}

// 10. Gradient pools: sizes and pointer partition of qwen3_gradients_alloc (src/model/qwen3.cu:1016-1085),
//     cleared on allocation and by grad_pools_zero; rlx_clear at odd addresses leaves its neighbours alone
static void test_grad_pools() {
    const char* name = "gradient pools: alloc, partition, zero";
    // Qwen3-0.6B dimensions with 2 layers and a small vocabulary
    const int L = 2, H = 1024, QD = 2048, KVD = 1024, I = 3072, HD = 128, V = 1000, max_T = 64, heads = 16;
    ParamPools pools = ParamPools::for_qwen3(L, H, QD, KVD, I, HD, V);
    GradPools g = grad_pools_alloc(pools, (size_t)max_T * heads);
    const size_t per16 = (size_t)QD * H + 2 * (size_t)KVD * H + (size_t)H * QD + 3 * (size_t)I * H;
    const size_t per32 = 2 * (size_t)H + 2 * HD;
    bool ok = g.half_pool_bytes == (per16 * L + (size_t)V * H) * 2 &&
              g.float_pool_bytes == (per32 * L + H + (size_t)max_T * heads) * 4;
    ok = ok && grad_proj(g, pools, 0, 0) == g.half_pool && grad_proj(g, pools, 0, 1) == g.half_pool + (size_t)QD * H &&
         grad_proj(g, pools, 1, 0) == g.half_pool + per16 &&
         grad_proj(g, pools, 1, 6) == g.half_pool + 2 * per16 - (size_t)H * I &&
         grad_embed(g, pools) == g.half_pool + per16 * L &&
         grad_norm_weight(g, pools, 0, 1) == g.float_pool + H && grad_norm_weight(g, pools, 1, 3) == g.float_pool + per32 + H + 2 * HD &&
         grad_final_norm(g, pools) == g.float_pool + per32 * L && grad_workspace(g, pools) == g.float_pool + per32 * L + H;
    std::vector<uint16_t> h16 = d2h((const uint16_t*)g.half_pool, g.half_pool_bytes / 2);
    std::vector<float> h32 = d2h((const float*)g.float_pool, g.float_pool_bytes / 4);
    size_t nonzero = 0;
    for (uint16_t x : h16) nonzero += x != 0;
    for (float x : h32) nonzero += x != 0.0f;
    // dirty both pools, clear them again
    RLX_CHECK(rlx_fill_f16((uint16_t*)g.half_pool, g.half_pool_bytes / 2, 9, 0, 1.0f, 0.1f, 0, 0, 0, nullptr));
    RLX_CHECK(rlx_fill_f32(g.float_pool, g.float_pool_bytes / 4, 9, 0, 1.0f, 0.1f, 0, 0, 0, nullptr));
    grad_pools_zero(&g);
    HIP_CHECK(hipDeviceSynchronize());
    h16 = d2h((const uint16_t*)g.half_pool, g.half_pool_bytes / 2);
    h32 = d2h((const float*)g.float_pool, g.float_pool_bytes / 4);
    for (uint16_t x : h16) nonzero += x != 0;
    for (float x : h32) nonzero += x != 0.0f;
    // rlx_clear on ranges that start and end at odd byte addresses
    size_t wrong = 0;
    const size_t span = 1000;
    unsigned char* buf = nullptr;
    HIP_CHECK(hipMalloc((void**)&buf, span));
    const int cases[][2] = {{0, 1000}, {1, 1}, {3, 13}, {15, 17}, {16, 16}, {7, 990}, {33, 0}, {5, 40}};
    for (const auto& c : cases) {
        HIP_CHECK(hipMemset(buf, 0xAB, span));
        RLX_CHECK(rlx_clear(buf + c[0], c[1], nullptr));
        HIP_CHECK(hipDeviceSynchronize());
        std::vector<unsigned char> h = d2h((const unsigned char*)buf, span);
        for (size_t i = 0; i < span; i++) {
            const bool inside = i >= (size_t)c[0] && i < (size_t)(c[0] + c[1]);
            wrong += h[i] != (inside ? 0x00 : 0xAB);
        }
    }
    (void)hipFree(buf);
    grad_pools_free(&g);
    ok = ok && g.half_pool == nullptr && g.float_pool_bytes == 0;
    if (ok && nonzero == 0 && wrong == 0) PASS(name); else FAIL(name, "ok=%d nonzero=%zu wrong=%zu", ok, nonzero, wrong);
}

// 11. training_step with gradient accumulation: pools cleared first, loss gradient scaled by 1/acc_steps,
//     then clip + step; equals doing the same by hand
static void test_accumulation() {
    const char* name = "training_step: clear, scaled micro-batches, clip, step";
    Fixture fa(5e-3f), fb(5e-3f);
    AdamWOptimizer oa(fa.pools, 1e-3f), ob(fb.pools, 1e-3f);
    OptimStepConfig cfg;
    cfg.max_grad_norm = 0.5f;
    cfg.fused_clip = true;
    OptimStep sa(&oa, cfg), sb(&ob, cfg);
    const int acc = 4;
    const size_t T = 50;
    float* lg = nullptr;
    HIP_CHECK(hipMalloc((void**)&lg, T * 4));
    std::vector<float> seen;      // loss_grad[0] after scaling, per micro-batch
    // stand-in backward: the last micro-batch writes seeded gradients (so the pools' final content is known)
    auto micro = [&](int k, const OptimStep::ScaleLossGrad& scale_loss_grad) {
        RLX_CHECK(rlx_fill_f32(lg, T, 40 + k, 0, 3.0f, 0.0f, 0, 0, 0, nullptr));
        scale_loss_grad(lg, T);
        seen.push_back(d2h((const float*)lg, 1)[0]);
        if (k == 0) {             // the pools must have been cleared before the first micro-batch
            std::vector<uint16_t> h = d2h((const uint16_t*)fa.g16, fa.n16);
            size_t nz = 0;
            for (uint16_t x : h) nz += x != 0;
            if (nz) seen.push_back(-1.0f);
        }
        if (k == acc - 1) {
            RLX_CHECK(rlx_fill_f16((uint16_t*)fa.g16, fa.n16, 2, 0, 0.0f, 5e-3f, 0, 0, 0, nullptr));
            RLX_CHECK(rlx_fill_f32(fa.g32, fa.n32 + fa.tail, 4, 0, 0.0f, 5e-3f, 0, 0, 0, nullptr));
        }
        return (float)(k + 1);
    };
    const float loss = sa.training_step(&fa.grads, acc, micro);
    const float nb = sb.apply(&fb.grads);           // fb still holds the same seeded gradients
    HIP_CHECK(hipDeviceSynchronize());
    bool scaled = seen.size() == (size_t)acc;
    for (float x : seen) scaled = scaled && x == 3.0f * (1.0f / (float)acc);
    std::vector<uint16_t> wa = d2h((const uint16_t*)fa.w16, fa.n16), wb = d2h((const uint16_t*)fb.w16, fb.n16);
    size_t diff = 0;
    for (size_t i = 0; i < fa.n16; i++) diff += wa[i] != wb[i];
    (void)hipFree(lg);
    if (scaled && loss == 2.5f && sa.last_grad_norm() == nb && nb > 0.5f && diff == 0) PASS(name);
    else FAIL(name, "scaled=%d loss=%f na=%f nb=%f diff=%zu", scaled, loss, sa.last_grad_norm(), nb, diff);
}

// 12. Steps from an uploaded table of hyper-parameters (no host values at launch time) equal ordinary steps
//     with set_lr: rates from the LR scheduler, bias corrections formed by the same powf
static void test_scheduled_steps() {
    const char* name = "scheduled steps == set_lr + step";
    Fixture a(5e-3f), b(5e-3f);
    AdamWOptimizer oa(a.pools, 1e-3f), ob(b.pools, 1e-3f);
    oa.set_fused_clip(true); ob.set_fused_clip(true);
    LRScheduler sched;
    sched.init_cosine(1e-3f, 1e-4f, 1, 6);
    float lrs[4];
    for (int k = 0; k < 4; k++) lrs[k] = sched.get_lr(k);
    ob.upload_schedule(&b.grads, lrs, 4);
    bool ok = true;
    for (int k = 0; k < 4; k++) {
        oa.set_lr(lrs[k]);
        const float na = oa.clip_grad_norm_(&a.grads, 0.25f);
        oa.step(&a.grads);
        const float nb = ob.clip_grad_norm_(&b.grads, 0.25f);
        ob.step_scheduled(&b.grads);
        ok = ok && na == nb;
    }
    HIP_CHECK(hipDeviceSynchronize());
    int64_t taken = -1, total = -1;
    RLX_CHECK(rlx_plan_schedule_position(ob.plan_for(&b.grads), &taken, &total, nullptr));
    a.download(); b.download();
    size_t diff = 0;
    for (size_t i = 0; i < a.n16; i++) diff += a.h_w16[i] != b.h_w16[i];
    for (size_t i = 0; i < a.n32; i++) diff += memcmp(&a.h_w32[i], &b.h_w32[i], 4) != 0;
    auto ma = d2h(oa.fp16_master(), a.n16), mb = d2h(ob.fp16_master(), b.n16);
    auto va = d2h(oa.fp16_v(), a.n16), vb = d2h(ob.fp16_v(), b.n16);
    for (size_t i = 0; i < a.n16; i++) diff += memcmp(&ma[i], &mb[i], 4) != 0 || memcmp(&va[i], &vb[i], 4) != 0;
    // a table with a zero bias correction is refused
    rlx_step_params bad = {1e-3f, 0.9f, 0.999f, 1e-8f, 0.0f, 0.0f, 0.1f};
    const bool refused = rlx_plan_schedule_upload(ob.plan_for(&b.grads), &bad, 1, nullptr) == RLX_ERR_BAD_HYPER;
    if (ok && diff == 0 && taken == 4 && total == 4 && refused && ob.get_step() == 4) PASS(name);
    else FAIL(name, "ok=%d diff=%zu taken=%lld total=%lld refused=%d", ok, diff, (long long)taken, (long long)total, refused);
}

// 13. The recorded step of the header's recipe: clip_grad_norm_async + step_scheduled captured once into a HIP
//     graph after the first upload, replayed through window 1 (3 steps), a longer window 2 (6 steps) and a shorter
//     window 3 (2 steps).  The reference sets the scheduler's rate before every step of the whole run
//     (trainer.h:193-194) and forms the bias corrections from the step number (optimizer.h:120-122): the oracle
//     replays exactly that on the host, and weights, master copy and moments must agree bit for bit after every
//     window; get_step() counts the replays and not the capture; no step overruns its table.
static void test_recorded_step_across_windows() {
    const char* name = "one recorded clip + scheduled step through three uploaded windows == oracle";
    Fixture f(5e-3f);
    AdamWOptimizer opt(f.pools, 1e-3f);
    OracleReplay oracle(f);
    LRScheduler sched;
    sched.init_cosine(1e-3f, 1e-5f, 2, 11);
    const float max_norm = 0.25f;
    opt.set_fused_clip(true);
    hipStream_t s;
    HIP_CHECK(hipStreamCreate(&s));
    const int64_t chunk = rlx_plan_chunk_elems(opt.plan_for(&f.grads));
    const int windows[3] = {3, 6, 2};
    hipGraph_t graph = nullptr;
    hipGraphExec_t exec = nullptr;
    bool ok = true;
    size_t diff = 0;
    int global = 0;
    for (int w = 0; w < 3; w++) {
        const int n = windows[w];
        std::vector<float> lrs((size_t)n);
        for (int k = 0; k < n; k++) lrs[(size_t)k] = sched.get_lr(global + k);
        ok = ok && opt.get_step() == global;
        opt.upload_schedule(&f.grads, lrs.data(), n, s);
        if (!exec) {
            HIP_CHECK(hipStreamBeginCapture(s, hipStreamCaptureModeThreadLocal));
            opt.clip_grad_norm_async(&f.grads, max_norm, s);
            opt.step_scheduled(&f.grads, s);
            HIP_CHECK(hipStreamEndCapture(s, &graph));
            HIP_CHECK(hipGraphInstantiate(&exec, graph, nullptr, nullptr, 0));
            ok = ok && opt.get_step() == 0;               // recording is not a step
        }
        for (int k = 0; k < n; k++) {
            RLX_CHECK(rlx_fill_f16((uint16_t*)f.g16, f.n16, 300 + global + k, 0, 0.0f, 2e-3f * (float)(global + k + 1), 0, 0, 0, s));
            RLX_CHECK(rlx_fill_f32(f.g32, f.n32 + f.tail, 400 + global + k, 0, 0.0f, 3e-3f, 0, 0, 0, s));
            HIP_CHECK(hipStreamSynchronize(s));
            const float want = oracle.advance(lrs[(size_t)k], max_norm, chunk);
            HIP_CHECK(hipGraphLaunch(exec, s));
            HIP_CHECK(hipStreamSynchronize(s));
            float got = 0.0f;
            RLX_CHECK(rlx_plan_norm_read(opt.plan_for(&f.grads), &got, nullptr, nullptr, s));
            int64_t taken = -1, total = -1, overrun = -1;
            RLX_CHECK(rlx_plan_schedule_position(opt.plan_for(&f.grads), &taken, &total, s));
            RLX_CHECK(rlx_plan_schedule_overrun(opt.plan_for(&f.grads), &overrun, s));
            ok = ok && memcmp(&got, &want, 4) == 0 && want > max_norm && taken == k + 1 && total == n && overrun == 0;
        }
        ok = ok && opt.note_replayed_steps(n);
        global += n;
        diff += oracle.differences(opt);
    }
    ok = ok && opt.get_step() == 11 && oracle.step == 11;
    HIP_CHECK(hipGraphExecDestroy(exec));
    HIP_CHECK(hipGraphDestroy(graph));
    HIP_CHECK(hipStreamDestroy(s));
    if (ok && diff == 0) PASS(name); else FAIL(name, "ok=%d diff=%zu step=%d", ok, diff, opt.get_step());
}

int main() {
    int ndev = 0;
    if (hipGetDeviceCount(&ndev) != hipSuccess || ndev == 0) {
        printf("no GPU: this test needs one\n");
        return 2;
    }
    printf("=== AdamW host-side tests ===\n");
    test_cpu_reference_fp32();
    test_cpu_reference_fp16();
    test_moments_nonzero();
    test_step_counter();
    test_clip();
    test_launch_api();
    test_frozen_and_zeroing();
    test_checkpoint();
    test_train_loop();
    test_grad_pools();
    test_accumulation();
    test_scheduled_steps();
    test_recorded_step_across_windows();
    printf("=== %s (%d failure%s) ===\n", g_fails ? "FAILED" : "ALL PASSED", g_fails, g_fails == 1 ? "" : "s");
    return g_fails;
}
