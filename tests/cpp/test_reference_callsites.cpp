// test_reference_callsites.cpp
//
// The reference's own call sites of the optimizer path, compiled as they stand against
// rl.cu_amd/host and run on a GPU.  The types below are named as in the reference (Qwen3Config,
// Qwen3Weights, Qwen3Model, Qwen3Gradients, TrainingConfig) and carry only the members that this path
// reads; the `Trainer` below holds, between the marker comments, lines copied unchanged from
//   include/training/trainer.h:162-163   optimizer_(model, config.base_lr, ...)      (constructor)
//   include/training/trainer.h:194       optimizer_.set_lr(cur_lr);
//   include/training/trainer.h:280-286   clip_grad_norm_(grads_, ...) ; optimizer_.step(grads_);
//   include/training/GRPO_trainer.h:508-514   the same tail in the GRPO trainer
// and the accessor calls of tests/test_adamw.cu (get_fp16_master(layer, proj), get_final_norm_m(), ...).
// Trainer::clip_grad_norm_ keeps the reference's signature (trainer.h:323); its body is the one line a
// maintainer writes.  Every result is compared bit for bit with the CPU oracle replaying the reference's
// order of operations (clip in place, then the three-group step).  The oracle is the checker only.
#include <cmath>
#include <cstdint>
#include <cstdio>
#include <cstring>
#include <string>
#include <vector>

#include "training/optimizer.h"

extern "C" {
float orc_h2f(uint16_t h);
void orc_adamw_fp16(float*, uint16_t*, const uint16_t*, float*, float*, int64_t, float, float, float, float, float,
                    float, float);
void orc_adamw_fp32(float*, const float*, float*, float*, int64_t, float, float, float, float, float, float, float);
void orc_scale_half(uint16_t*, float, int64_t);
void orc_scale_float(float*, float, int64_t);
float orc_clip_scale(float sum_sq, float max_norm, float* norm_out);
double orc_sum_sq_half(const uint16_t*, int64_t);
double orc_sum_sq_float(const float*, int64_t);
int64_t orc_sumsq_mirror_partials(const void* g, int is_f32, int64_t n, int chunk, double* partials);
double orc_sumsq_mirror_total(const double* partials, int64_t n_partials, int chunk);
void orc_optimizer_step(float* fp16_master, uint16_t* fp16_pool, const uint16_t* half_grads, float* fp16_m, float* fp16_v,
                        int64_t n16, int64_t proj_n, float* fp32_pool, const float* float_grads, float* fp32_m,
                        float* fp32_v, int64_t n32, float lr, float beta1, float beta2, float eps, float weight_decay,
                        int* step);
}

static int g_fails = 0;
#define PASS(name) printf("[PASS] %s\n", (name))
#define FAIL(name, ...) do { printf("[FAIL] %s: ", (name)); printf(__VA_ARGS__); printf("\n"); g_fails++; } while (0)

// ---------------------------------------------------------------------------------------------------
// The reference's types, reduced to what the optimizer path reads (include/model/config.h:5-30,
// include/model/weights.h:43-61, include/model/qwen3.h:35-37,190-197, include/training/trainer.h:28-43)
// ---------------------------------------------------------------------------------------------------
struct Qwen3Config {
    int vocab_size = 1000;
    int hidden_size = 64;
    int intermediate_size = 192;
    int num_hidden_layers = 2;
    int num_attention_heads = 4;
    int num_key_value_heads = 2;
    int head_dim = 16;
    int n_rep, q_dim, kv_dim;
    void compute_derived() {
        n_rep = num_attention_heads / num_key_value_heads;
        q_dim = num_attention_heads * head_dim;
        kv_dim = num_key_value_heads * head_dim;
    }
};

struct Qwen3Weights {
    half* fp16_pool = nullptr;
    float* fp32_pool = nullptr;
    size_t fp16_pool_elems = 0;
    size_t fp32_pool_elems = 0;
};

struct Qwen3Model {
    Qwen3Config config;
    Qwen3Weights weights;
};

struct Qwen3Gradients {
    half* half_pool = nullptr;
    float* float_pool = nullptr;
    size_t half_pool_bytes = 0;
    size_t float_pool_bytes = 0;
};

struct TrainingConfig {
    float base_lr = 1e-5f;
    float beta1 = 0.9f;
    float beta2 = 0.999f;
    float opt_eps = 1e-8f;
    float weight_decay = 0.01f;
    float max_grad_norm = 1.0f;
    bool freeze_embed = false;
};

// ---------------------------------------------------------------------------------------------------
// A trainer with the reference's member names around the copied lines
// ---------------------------------------------------------------------------------------------------
class Trainer {
public:
    Trainer(const TrainingConfig& config, Qwen3Model* model, Qwen3Gradients* grads)
        : model_(model),
          // >>> include/training/trainer.h:162-163, unchanged
          optimizer_(model, config.base_lr, config.beta1, config.beta2,
                     config.opt_eps, config.weight_decay),
          // <<<
          grads_(grads),
          config_(config) {}

    void set_learning_rate(float cur_lr) {
        // >>> include/training/trainer.h:194, unchanged
                optimizer_.set_lr(cur_lr);
        // <<<
    }

    // The end of Trainer::training_step (include/training/trainer.h:269-289)
    float training_step_tail(float accum_loss, int acc_steps) {
        // trainer.h:271-277 with the memset spelled for HIP (rlx_clear; a kernel, safe under graph capture)
        if (config_.freeze_embed) {
            const Qwen3Config& c = model_->config;
            const size_t embed_elems = (size_t)c.vocab_size * c.hidden_size;
            const size_t half_elems  = grads_->half_pool_bytes / sizeof(half);
            half* embed_grad = grads_->half_pool + (half_elems - embed_elems);
            RLX_CHECK(rlx_clear(embed_grad, (int64_t)(embed_elems * sizeof(half)), nullptr));
        }

        // >>> include/training/trainer.h:279-286, unchanged
        // Gradient clipping: scale all gradients so global L2 norm <= max_grad_norm.
        float grad_norm = 0.0f;
        if (config_.max_grad_norm > 0.0f) {
            grad_norm = clip_grad_norm_(grads_, config_.max_grad_norm);
        }

        // One optimizer step after all micro-batches
        optimizer_.step(grads_);
        // <<<

        last_grad_norm_ = grad_norm;
        return accum_loss / acc_steps;
    }

    // The end of GRPOTrainer::training_step (include/training/GRPO_trainer.h:507-516)
    float grpo_step_tail(float total_loss, int N_active) {
        // >>> include/training/GRPO_trainer.h:507-514, unchanged
        // Gradient clipping
        float grad_norm = 0.0f;
        if (config_.max_grad_norm > 0.0f)
            grad_norm = clip_grad_norm_(grads_, config_.max_grad_norm);
        last_grad_norm_ = grad_norm;

        // Optimizer step
        optimizer_.step(grads_);
        // <<<

        return (N_active > 0) ? total_loss / N_active : 0.0f;
    }

    AdamWOptimizer& optimizer() { return optimizer_; }
    float last_grad_norm() const { return last_grad_norm_; }

protected:
    Qwen3Model*      model_;
    AdamWOptimizer   optimizer_;
    Qwen3Gradients*  grads_        = nullptr;
    TrainingConfig   config_;
    float            last_grad_norm_ = 0.0f;

    // The reference's signature (include/training/trainer.h:323); the body is the maintainer's one line.
    float clip_grad_norm_(Qwen3Gradients* grads, float max_norm) {
        return ::clip_grad_norm_(optimizer_, grads, max_norm);
    }
};

// ---------------------------------------------------------------------------------------------------
// Device pools of a small model and their host mirror, which the oracle advances
// ---------------------------------------------------------------------------------------------------
template <typename T> static std::vector<T> d2h(const void* d, size_t n) {
    std::vector<T> h(n);
    HIP_CHECK(hipMemcpy(h.data(), d, n * sizeof(T), hipMemcpyDeviceToHost));
    return h;
}

struct World {
    Qwen3Model model;
    Qwen3Gradients grads;
    size_t n16 = 0, n32 = 0, proj_n = 0, embed_n = 0, tail = 37 * 4;     // tail: D_buf, max_T * heads floats
    // host mirror
    std::vector<uint16_t> w16;
    std::vector<float> w32, master, m16, v16, m32, v32;
    int step = 0;

    explicit World(const Qwen3Config& config = Qwen3Config()) {
        model.config = config;
        Qwen3Config& c = model.config;
        c.compute_derived();
        const size_t H = c.hidden_size;
        const size_t per16 = 2 * (size_t)c.q_dim * H + 2 * (size_t)c.kv_dim * H + 3 * (size_t)c.intermediate_size * H;
        proj_n = per16 * c.num_hidden_layers;
        embed_n = (size_t)c.vocab_size * H;
        n16 = proj_n + embed_n;
        n32 = (2 * H + 2 * c.head_dim) * c.num_hidden_layers + H;
        model.weights.fp16_pool_elems = n16;
        model.weights.fp32_pool_elems = n32;
        HIP_CHECK(hipMalloc((void**)&model.weights.fp16_pool, n16 * 2));
        HIP_CHECK(hipMalloc((void**)&model.weights.fp32_pool, n32 * 4));
        grads.half_pool_bytes = n16 * 2;
        grads.float_pool_bytes = (n32 + tail) * 4;
        HIP_CHECK(hipMalloc((void**)&grads.half_pool, grads.half_pool_bytes));
        HIP_CHECK(hipMalloc((void**)&grads.float_pool, grads.float_pool_bytes));
        RLX_CHECK(rlx_fill_f16((uint16_t*)model.weights.fp16_pool, n16, 71, 0, 0.0f, 0.02f, 0, 0, 0, nullptr));
        RLX_CHECK(rlx_fill_f32(model.weights.fp32_pool, n32, 72, 0, 1.0f, 0.05f, 0, 0, 0, nullptr));
        HIP_CHECK(hipDeviceSynchronize());
        w16 = d2h<uint16_t>(model.weights.fp16_pool, n16);
        w32 = d2h<float>(model.weights.fp32_pool, n32);
        master.resize(n16);
        for (size_t i = 0; i < n16; i++) master[i] = orc_h2f(w16[i]);      // optimizer.h:242
        m16.assign(n16, 0.0f); v16.assign(n16, 0.0f); m32.assign(n32, 0.0f); v32.assign(n32, 0.0f);
    }
    ~World() {
        (void)hipFree(model.weights.fp16_pool); (void)hipFree(model.weights.fp32_pool);
        (void)hipFree(grads.half_pool); (void)hipFree(grads.float_pool);
    }
    void new_gradients(uint64_t seed, float std) {
        RLX_CHECK(rlx_fill_f16((uint16_t*)grads.half_pool, n16, seed, 0, 0.0f, std, 0, 0, 0, nullptr));
        RLX_CHECK(rlx_fill_f32(grads.float_pool, n32 + tail, seed + 1, 0, 0.0f, std, 0, 0, 0, nullptr));
        HIP_CHECK(hipDeviceSynchronize());
    }
};

// The reference's order on the host mirror: [clear embedding gradients] -> norm -> scale in place if
// norm > max -> three-group step.  The norm is added up in the device's fixed order (restated by the
// oracle), so the returned norm, the scale and everything after it can be compared bit for bit; the same
// norm is also held against the plain FP64 sum (1e-5 relative).
struct Expected { float norm; std::vector<uint16_t> g16; std::vector<float> g32; };
static Expected oracle_tail(World& w, const TrainingConfig& cfg, float lr, int64_t chunk, bool& norm_close) {
    Expected e;
    e.g16 = d2h<uint16_t>(w.grads.half_pool, w.n16);
    e.g32 = d2h<float>(w.grads.float_pool, w.n32 + w.tail);
    if (cfg.freeze_embed) std::fill(e.g16.begin() + w.proj_n, e.g16.end(), (uint16_t)0);
    e.norm = 0.0f;
    norm_close = true;
    if (cfg.max_grad_norm > 0.0f) {
        // plan order: projections, embedding, norm gradients, workspace tail
        std::vector<double> partials((w.n16 + w.n32 + w.tail) / 512 + 16);
        int64_t k = 0;
        k += orc_sumsq_mirror_partials(e.g16.data(), 0, (int64_t)w.proj_n, (int)chunk, partials.data() + k);
        k += orc_sumsq_mirror_partials(e.g16.data() + w.proj_n, 0, (int64_t)w.embed_n, (int)chunk, partials.data() + k);
        k += orc_sumsq_mirror_partials(e.g32.data(), 1, (int64_t)w.n32, (int)chunk, partials.data() + k);
        k += orc_sumsq_mirror_partials(e.g32.data() + w.n32, 1, (int64_t)w.tail, (int)chunk, partials.data() + k);
        const double sum_sq = orc_sumsq_mirror_total(partials.data(), k, (int)chunk);
        const float scale = orc_clip_scale((float)sum_sq, cfg.max_grad_norm, &e.norm);
        const double exact = sqrt(orc_sum_sq_half(e.g16.data(), (int64_t)w.n16) +
                                  orc_sum_sq_float(e.g32.data(), (int64_t)(w.n32 + w.tail)));
        norm_close = fabs((double)e.norm - exact) <= 1e-5 * exact;
        if (e.norm > cfg.max_grad_norm) {                       // trainer.h:343-349
            orc_scale_half(e.g16.data(), scale, (int64_t)w.n16);
            orc_scale_float(e.g32.data(), scale, (int64_t)(w.n32 + w.tail));
        }
    }
    orc_optimizer_step(w.master.data(), w.w16.data(), e.g16.data(), w.m16.data(), w.v16.data(), (int64_t)w.n16,
                       (int64_t)w.proj_n, w.w32.data(), e.g32.data(), w.m32.data(), w.v32.data(), (int64_t)w.n32, lr,
                       cfg.beta1, cfg.beta2, cfg.opt_eps, cfg.weight_decay, &w.step);
    return e;
}

template <typename T> static size_t count_diff(const std::vector<T>& a, const std::vector<T>& b) {
    size_t d = a.size() != b.size();
    for (size_t i = 0; i < a.size() && i < b.size(); i++) d += memcmp(&a[i], &b[i], sizeof(T)) != 0;
    return d;
}

// device state against the host mirror; grads_expected == nullptr: gradients must be all zero
static size_t compare_all(World& w, AdamWOptimizer& opt, const Expected* grads_expected, bool grads_cleared) {
    size_t d = 0;
    d += count_diff(d2h<uint16_t>(w.model.weights.fp16_pool, w.n16), w.w16);
    d += count_diff(d2h<float>(w.model.weights.fp32_pool, w.n32), w.w32);
    d += count_diff(d2h<float>(opt.fp16_master(), w.n16), w.master);
    d += count_diff(d2h<float>(opt.fp16_m(), w.n16), w.m16);
    d += count_diff(d2h<float>(opt.fp16_v(), w.n16), w.v16);
    d += count_diff(d2h<float>(opt.fp32_m(), w.n32), w.m32);
    d += count_diff(d2h<float>(opt.fp32_v(), w.n32), w.v32);
    std::vector<uint16_t> g16 = d2h<uint16_t>(w.grads.half_pool, w.n16);
    std::vector<float> g32 = d2h<float>(w.grads.float_pool, w.n32 + w.tail);
    if (grads_cleared) {
        for (uint16_t x : g16) d += x != 0;
        for (float x : g32) { uint32_t u; memcpy(&u, &x, 4); d += u != 0; }
    } else if (grads_expected) {
        d += count_diff(g16, grads_expected->g16);
        d += count_diff(g32, grads_expected->g32);
    }
    return d;
}

// 1. The SFT trainer's tail, reference behaviour (master copy, clip scales the gradients in place): four
//    steps with fresh gradients and a scheduled rate; step 3 has small gradients (norm below the limit:
//    nothing is scaled); everything including the clipped gradients equals the oracle.
static void test_sft_tail() {
    const char* name = "trainer.h:280-286 unchanged, reference behaviour, vs oracle";
    World w;
    TrainingConfig cfg;
    cfg.base_lr = 1e-3f;
    Trainer t(cfg, &w.model, &w.grads);
    const int64_t chunk = rlx_plan_chunk_elems(t.optimizer().plan_for(&w.grads));
    size_t diffs = 0;
    bool norms = true, close = true, ret = true;
    for (int s = 0; s < 4; s++) {
        const float lr = 1e-3f / (float)(s + 1);
        t.set_learning_rate(lr);
        w.new_gradients(500 + 10 * s, s == 2 ? 1e-4f : 5e-3f);
        bool c;
        const Expected e = oracle_tail(w, cfg, lr, chunk, c);
        const float loss = t.training_step_tail(6.0f, 4);
        HIP_CHECK(hipDeviceSynchronize());
        ret = ret && loss == 1.5f;
        close = close && c;
        const float got = t.last_grad_norm();
        norms = norms && memcmp(&e.norm, &got, 4) == 0 &&
                (s == 2 ? e.norm < cfg.max_grad_norm : e.norm > cfg.max_grad_norm);
        diffs += compare_all(w, t.optimizer(), &e, false);
    }
    printf("  chunk=%lld  last norm=%.6f  mismatching values over 4 steps=%zu\n", (long long)chunk, t.last_grad_norm(), diffs);
    if (diffs == 0 && norms && close && ret && t.optimizer().get_step() == 4) PASS(name);
    else FAIL(name, "diffs=%zu norms=%d close=%d ret=%d", diffs, norms, close, ret);
}

// 2. The same tail with freeze_embed (the embedding's gradients are cleared before the clip)
static void test_sft_tail_frozen_embedding() {
    const char* name = "trainer.h:269-286 with freeze_embed, vs oracle";
    World w;
    TrainingConfig cfg;
    cfg.base_lr = 1e-3f;
    cfg.freeze_embed = true;
    cfg.max_grad_norm = 0.5f;
    Trainer t(cfg, &w.model, &w.grads);
    const int64_t chunk = rlx_plan_chunk_elems(t.optimizer().plan_for(&w.grads));
    const std::vector<uint16_t> embed_before(w.w16.begin() + w.proj_n, w.w16.end());
    size_t diffs = 0;
    bool norms = true;
    for (int s = 0; s < 2; s++) {
        w.new_gradients(900 + 10 * s, 5e-3f);
        bool c;
        const Expected e = oracle_tail(w, cfg, cfg.base_lr, chunk, c);
        t.training_step_tail(1.0f, 1);
        HIP_CHECK(hipDeviceSynchronize());
        const float got = t.last_grad_norm();
        norms = norms && c && memcmp(&e.norm, &got, 4) == 0;
        diffs += compare_all(w, t.optimizer(), &e, false);
    }
    const std::vector<uint16_t> embed_after(w.w16.begin() + w.proj_n, w.w16.end());
    const bool identity = embed_before == embed_after;           // zero gradients, zero moments, no decay
    if (diffs == 0 && norms && identity) PASS(name); else FAIL(name, "diffs=%zu norms=%d identity=%d", diffs, norms, identity);
}

// 3. The GRPO trainer's tail, unchanged, once as the reference behaves and once with the two options of this
//    library switched on (clip applied inside the update, gradients cleared by the update): weights and
//    optimizer state are the same bits either way; the gradients end up scaled in the first and zero in the second.
static void test_grpo_tail(bool fast) {
    const std::string label = std::string("GRPO_trainer.h:507-514 unchanged, ") +
                              (fast ? "fused clip + gradient clearing" : "reference behaviour") + ", vs oracle";
    const char* name = label.c_str();
    World w;
    TrainingConfig cfg;
    cfg.base_lr = 2e-4f;
    cfg.max_grad_norm = 0.3f;
    Trainer t(cfg, &w.model, &w.grads);
    if (fast) { t.optimizer().set_fused_clip(true); t.optimizer().set_zero_grads(true); }
    const int64_t chunk = rlx_plan_chunk_elems(t.optimizer().plan_for(&w.grads));
    size_t diffs = 0;
    bool norms = true, ret = true;
    for (int s = 0; s < 3; s++) {
        w.new_gradients(1300 + 10 * s, 5e-3f);
        bool c;
        const Expected e = oracle_tail(w, cfg, cfg.base_lr, chunk, c);
        ret = ret && t.grpo_step_tail(9.0f, 3) == 3.0f;
        HIP_CHECK(hipDeviceSynchronize());
        const float got = t.last_grad_norm();
        norms = norms && c && memcmp(&e.norm, &got, 4) == 0;
        diffs += compare_all(w, t.optimizer(), &e, fast);
    }
    if (diffs == 0 && norms && ret) PASS(name); else FAIL(name, "diffs=%zu norms=%d ret=%d", diffs, norms, ret);
}

// 4. max_grad_norm = 0 disables the clip (trainer.h:281): the norm stays 0 and the gradients are used as they are
static void test_clip_disabled() {
    const char* name = "max_grad_norm = 0: no clip, step only";
    World w;
    TrainingConfig cfg;
    cfg.base_lr = 1e-3f;
    cfg.max_grad_norm = 0.0f;
    Trainer t(cfg, &w.model, &w.grads);
    w.new_gradients(77, 5e-3f);
    bool c;
    const Expected e = oracle_tail(w, cfg, cfg.base_lr, 8192, c);
    t.training_step_tail(1.0f, 1);
    HIP_CHECK(hipDeviceSynchronize());
    const size_t diffs = compare_all(w, t.optimizer(), &e, false);
    if (diffs == 0 && t.last_grad_norm() == 0.0f) PASS(name); else FAIL(name, "diffs=%zu norm=%f", diffs, t.last_grad_norm());
}

// 5. The calls of the reference's own optimizer test (tests/test_adamw.cu): construction from the model,
//    step(grads), get_step(), and the (layer, tensor) accessors, which must point into the flat buffers at the
//    reference's offsets (optimizer.h:107-116,165-184)
static void test_reference_test_calls() {
    const char* name = "tests/test_adamw.cu calls: AdamWOptimizer opt(model, lr, ...); opt.step(grads); accessors";
    World w;
    Qwen3Model* model = &w.model;
    Qwen3Gradients* grads = &w.grads;
    w.new_gradients(5, 1e-3f);
    const float lr = 1e-3f;
    AdamWOptimizer opt(model, lr, 0.9f, 0.999f, 1e-8f, 0.0f);
    bool ok = opt.get_step() == 0 && opt.num_fp16_params() == w.n16 && opt.num_fp32_params() == w.n32;
    opt.step(grads);
    HIP_CHECK(hipDeviceSynchronize());
    ok = ok && opt.get_step() == 1;
    const Qwen3Config& c = model->config;
    const size_t H = c.hidden_size, q = (size_t)c.q_dim * H, kv = (size_t)c.kv_dim * H, in = (size_t)c.intermediate_size * H;
    const size_t per16 = 2 * q + 2 * kv + 3 * in, per32 = 2 * H + 2 * c.head_dim;
    ok = ok && opt.get_fp16_master(0, 0) == opt.fp16_master() && opt.get_fp16_m(0, 1) == opt.fp16_m() + q &&
         opt.get_fp16_v(1, 3) == opt.fp16_v() + per16 + q + 2 * kv &&
         opt.get_fp16_m(1, 6) == opt.fp16_m() + 2 * per16 - in &&
         opt.get_fp32_m_norm(0, 1) == opt.fp32_m() + H && opt.get_fp32_v_norm(1, 3) == opt.fp32_v() + per32 + H + 2 * c.head_dim &&
         opt.get_final_norm_m() == opt.fp32_m() + per32 * c.num_hidden_layers &&
         opt.get_final_norm_v() == opt.fp32_v() + per32 * c.num_hidden_layers;
    // step 1 from zero moments: m = (1-beta1) g, as the reference's test checks through these accessors
    const std::vector<float> m_k = d2h<float>(opt.get_fp16_m(0, 1), 64);
    const std::vector<uint16_t> g_k = d2h<uint16_t>(grads->half_pool + q, 64);
    for (int i = 0; i < 64; i++) ok = ok && m_k[i] == (1.0f - 0.9f) * orc_h2f(g_k[i]);
    if (ok) PASS(name); else FAIL(name, "accessor or step mismatch");
}

// 7. The reference's own dimensions (Qwen3-0.6B, include/model/config.h:6-12: 595,984,384 FP16 and 65,536 FP32
//    parameters, 7.15 GB of optimizer state): the trainer tail unchanged, two steps; the norm against the FP64 sum
//    over all gradients, and windows of every pool (its start, both sides of the boundary between the projections,
//    which decay, and the embedding, which does not, its end, and the whole FP32 pool) against the oracle.
static void test_full_size_model() {
    const char* name = "Qwen3-0.6B dimensions through the reference's call sites, windows vs oracle";
    Qwen3Config q;
    q.vocab_size = 151936; q.hidden_size = 1024; q.intermediate_size = 3072; q.num_hidden_layers = 28;
    q.num_attention_heads = 16; q.num_key_value_heads = 8; q.head_dim = 128;
    World w(q);
    TrainingConfig cfg;
    cfg.base_lr = 1e-4f;
    Trainer t(cfg, &w.model, &w.grads);
    bool ok = w.n16 == 595984384u && w.n32 == 65536u && w.proj_n == 440401920u &&
              t.optimizer().num_fp16_params() == w.n16;
    struct Win { size_t lo, n; };
    const Win wins[] = {{0, 40000}, {w.proj_n - 30000, 60000}, {w.n16 - 50000, 50000}, {123456789, 33333}};
    size_t diffs = 0;
    bool norms = true;
    for (int s = 0; s < 2; s++) {
        w.new_gradients(4000 + 10 * s, 5e-3f);
        const std::vector<uint16_t> g16 = d2h<uint16_t>(w.grads.half_pool, w.n16);
        std::vector<float> g32 = d2h<float>(w.grads.float_pool, w.n32 + w.tail);
        const double exact = sqrt(orc_sum_sq_half(g16.data(), (int64_t)w.n16) +
                                  orc_sum_sq_float(g32.data(), (int64_t)(w.n32 + w.tail)));
        t.training_step_tail(1.0f, 1);
        HIP_CHECK(hipDeviceSynchronize());
        const float norm = t.last_grad_norm();
        norms = norms && fabs((double)norm - exact) <= 1e-5 * exact && norm > cfg.max_grad_norm;
        const float scale = cfg.max_grad_norm / (norm + 1e-6f);                   // trainer.h:344
        w.step++;
        const float bc1 = 1.0f - powf(cfg.beta1, (float)w.step), bc2 = 1.0f - powf(cfg.beta2, (float)w.step);
        for (const Win& win : wins) {
            // the window's state on the host mirror (weights, master, moments), advanced by the oracle
            std::vector<uint16_t> gw(g16.begin() + win.lo, g16.begin() + win.lo + win.n);
            orc_scale_half(gw.data(), scale, (int64_t)win.n);
            // elements below proj_n decay, the others do not (optimizer.h:124-140)
            const size_t split = win.lo >= w.proj_n ? 0 : (win.lo + win.n <= w.proj_n ? win.n : w.proj_n - win.lo);
            orc_adamw_fp16(w.master.data() + win.lo, w.w16.data() + win.lo, gw.data(), w.m16.data() + win.lo,
                           w.v16.data() + win.lo, (int64_t)split, cfg.base_lr, cfg.beta1, cfg.beta2, cfg.opt_eps,
                           cfg.weight_decay, bc1, bc2);
            orc_adamw_fp16(w.master.data() + win.lo + split, w.w16.data() + win.lo + split, gw.data() + split,
                           w.m16.data() + win.lo + split, w.v16.data() + win.lo + split, (int64_t)(win.n - split),
                           cfg.base_lr, cfg.beta1, cfg.beta2, cfg.opt_eps, 0.0f, bc1, bc2);
            const std::vector<uint16_t> dw = d2h<uint16_t>((const uint16_t*)w.model.weights.fp16_pool + win.lo, win.n);
            const std::vector<float> dm = d2h<float>(t.optimizer().fp16_m() + win.lo, win.n);
            const std::vector<float> dv = d2h<float>(t.optimizer().fp16_v() + win.lo, win.n);
            const std::vector<float> dmas = d2h<float>(t.optimizer().fp16_master() + win.lo, win.n);
            const std::vector<uint16_t> dg = d2h<uint16_t>((const uint16_t*)w.grads.half_pool + win.lo, win.n);
            for (size_t i = 0; i < win.n; i++)
                diffs += dw[i] != w.w16[win.lo + i] || memcmp(&dm[i], &w.m16[win.lo + i], 4) ||
                         memcmp(&dv[i], &w.v16[win.lo + i], 4) || memcmp(&dmas[i], &w.master[win.lo + i], 4) ||
                         dg[i] != gw[i];
        }
        orc_scale_float(g32.data(), scale, (int64_t)(w.n32 + w.tail));
        orc_adamw_fp32(w.w32.data(), g32.data(), w.m32.data(), w.v32.data(), (int64_t)w.n32, cfg.base_lr, cfg.beta1,
                       cfg.beta2, cfg.opt_eps, 0.0f, bc1, bc2);
        diffs += count_diff(d2h<float>(w.model.weights.fp32_pool, w.n32), w.w32);
        diffs += count_diff(d2h<float>(t.optimizer().fp32_v(), w.n32), w.v32);
        diffs += count_diff(d2h<float>(w.grads.float_pool, w.n32 + w.tail), g32);
    }
    printf("  norm=%.6f  mismatching values in the windows over 2 steps=%zu\n", t.last_grad_norm(), diffs);
    if (ok && norms && diffs == 0 && t.optimizer().get_step() == 2) PASS(name);
    else FAIL(name, "ok=%d norms=%d diffs=%zu", ok, norms, diffs);
}

int main() {
    int ndev = 0;
    if (hipGetDeviceCount(&ndev) != hipSuccess || ndev == 0) {
        printf("no GPU: this test needs one\n");
        return 2;
    }
    printf("=== reference call sites on the MI355X optimizer path ===\n");
    test_sft_tail();
    test_sft_tail_frozen_embedding();
    test_grpo_tail(false);
    test_grpo_tail(true);
    test_clip_disabled();
    test_reference_test_calls();
    test_full_size_model();
    printf("=== %s (%d failure%s) ===\n", g_fails ? "FAILED" : "ALL PASSED", g_fails, g_fails == 1 ? "" : "s");
    return g_fails;
}
