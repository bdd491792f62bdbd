// AdamWOptimizer for C++ callers: the reference's class (include/training/optimizer.h:59-274)
// with the same public members and methods.  It is built either from flat pools (ParamPools) or, with the
// reference's own constructor signature, from a pointer to any model type that has the members the
// reference's constructor reads (model->config.* and model->weights.fp16_pool / fp32_pool / *_elems);
// step() and clip_grad_norm_() take a pointer to any gradient type with half_pool / float_pool /
// half_pool_bytes / float_pool_bytes, so the reference's call sites (optimizer_(model, ...),
// clip_grad_norm_(grads_, max), optimizer_.step(grads_)) compile as they stand.
//
// Like the reference it owns the FP32 state as flat buffers co-indexed with the weight pools:
// [master | m | v] for the FP16 pool and [m | v] for the FP32 pool, zero-filled, master
// initialised from the FP16 weights.  step() increments the step counter, forms the bias
// corrections with powf on the host and updates every parameter; where the reference issues
// three launches (projections with decay, embedding and norm weights without), this issues
// one multi-tensor launch with the same three groups.
#pragma once
#include <sys/types.h>

#include <cassert>
#include <cmath>
#include <cstdint>
#include <cstring>
#include <string>
#include <type_traits>
#include <utility>
#include <vector>

#include "../kernels/adamw.h"

#ifndef HIP_CHECK
#define HIP_CHECK(x)                                                                                        \
    do {                                                                                                    \
        hipError_t err_ = (x);                                                                              \
        if (err_ != hipSuccess) {                                                                           \
            fprintf(stderr, "HIP error %s at %s:%d\n", hipGetErrorString(err_), __FILE__, __LINE__);        \
            exit(1);                                                                                        \
        }                                                                                                   \
    } while (0)
#endif

// The weight pools of the model (Qwen3Weights::fp16_pool / fp32_pool, include/model/weights.h:43-61).
// The FP16 pool is [projections of all layers | embedding]; proj_elems is the size of the first part.
struct ParamPools {
    half* fp16_pool = nullptr;
    size_t fp16_pool_elems = 0;
    size_t proj_elems = 0;
    float* fp32_pool = nullptr;
    size_t fp32_pool_elems = 0;
    // Optional per-layer structure, only used by the (layer, tensor) accessors below:
    // sizes of q, k, v, o, gate, up, down and of input_norm, q_norm, k_norm, post_attn_norm.
    int num_layers = 0;
    size_t proj_sizes[7] = {};
    size_t norm_sizes[4] = {};

    // Fills sizes and structure from the model dimensions (include/model/config.h:5-30; pool order
    // of include/training/optimizer.h:30-32).  The pool pointers stay for the caller to set.
    static ParamPools for_qwen3(int num_layers, int hidden, int q_dim, int kv_dim, int intermediate, int head_dim,
                                int vocab) {
        ParamPools p;
        const size_t H = (size_t)hidden;
        const size_t ps[7] = {(size_t)q_dim * H, (size_t)kv_dim * H, (size_t)kv_dim * H, H * (size_t)q_dim,
                              (size_t)intermediate * H, (size_t)intermediate * H, H * (size_t)intermediate};
        const size_t ns[4] = {H, (size_t)head_dim, (size_t)head_dim, H};
        size_t per16 = 0, per32 = 0;
        for (int i = 0; i < 7; i++) { p.proj_sizes[i] = ps[i]; per16 += ps[i]; }
        for (int i = 0; i < 4; i++) { p.norm_sizes[i] = ns[i]; per32 += ns[i]; }
        p.num_layers = num_layers;
        p.proj_elems = per16 * (size_t)num_layers;
        p.fp16_pool_elems = p.proj_elems + (size_t)vocab * H;
        p.fp32_pool_elems = per32 * (size_t)num_layers + H;
        return p;
    }
};

// The gradient pools (Qwen3Gradients, include/model/qwen3.h:190-218).  float_pool may be longer
// than the FP32 weight pool: the reference keeps an attention-backward workspace behind the norm
// gradients, and its clip includes that tail in the norm and scales it.
struct GradPools {
    half* half_pool = nullptr;
    float* float_pool = nullptr;
    size_t half_pool_bytes = 0;
    size_t float_pool_bytes = 0;
};

// Allocation, clearing and release of the gradient pools: the roles of qwen3_gradients_alloc, _zero and
// _free (src/model/qwen3.cu:1016-1112).  workspace_floats is the tail behind the norm gradients
// (max_T * num_attention_heads floats in the reference).  The pools come back cleared.
inline void grad_pools_zero(GradPools* g, hipStream_t stream = 0) {
    RLX_CHECK(rlx_clear(g->half_pool, (int64_t)g->half_pool_bytes, (void*)stream));
    RLX_CHECK(rlx_clear(g->float_pool, (int64_t)g->float_pool_bytes, (void*)stream));
}

inline GradPools grad_pools_alloc(const ParamPools& pools, size_t workspace_floats) {
    GradPools g;
    g.half_pool_bytes = pools.fp16_pool_elems * sizeof(half);
    g.float_pool_bytes = (pools.fp32_pool_elems + workspace_floats) * sizeof(float);
    if (g.half_pool_bytes) HIP_CHECK(hipMalloc((void**)&g.half_pool, g.half_pool_bytes));
    if (g.float_pool_bytes) HIP_CHECK(hipMalloc((void**)&g.float_pool, g.float_pool_bytes));
    grad_pools_zero(&g);
    HIP_CHECK(hipDeviceSynchronize());
    return g;
}

inline void grad_pools_free(GradPools* g) {
    if (g->half_pool) (void)hipFree(g->half_pool);
    if (g->float_pool) (void)hipFree(g->float_pool);
    *g = GradPools();
}

// Where one tensor's gradient lies in the pools: what the dW_* pointer arrays of Qwen3Gradients hold
// (include/model/qwen3.h:190-218).  proj: 0=q 1=k 2=v 3=o 4=gate 5=up 6=down; norm: 0=input 1=q 2=k
// 3=post_attn.  They need the per-layer structure in ParamPools.
inline size_t pool_offset(const size_t* sizes, int count, int layer, int which) {
    size_t per = 0, off = 0;
    for (int i = 0; i < count; i++) { per += sizes[i]; if (i < which) off += sizes[i]; }
    return (size_t)layer * per + off;
}
inline half* grad_proj(const GradPools& g, const ParamPools& p, int layer, int proj) {
    assert(layer >= 0 && layer < p.num_layers && proj >= 0 && proj < 7);
    return g.half_pool + pool_offset(p.proj_sizes, 7, layer, proj);
}
inline half* grad_embed(const GradPools& g, const ParamPools& p) { return g.half_pool + p.proj_elems; }
inline float* grad_norm_weight(const GradPools& g, const ParamPools& p, int layer, int norm) {
    assert(layer >= 0 && layer < p.num_layers && norm >= 0 && norm < 4);
    return g.float_pool + pool_offset(p.norm_sizes, 4, layer, norm);
}
inline float* grad_final_norm(const GradPools& g, const ParamPools& p) {
    return g.float_pool + pool_offset(p.norm_sizes, 4, p.num_layers, 0);
}
inline float* grad_workspace(const GradPools& g, const ParamPools& p) { return g.float_pool + p.fp32_pool_elems; }

class AdamWOptimizer {
public:
    // Hyper-parameters (public, as in the reference)
    float lr;
    float beta1;
    float beta2;
    float eps;
    float weight_decay;

    AdamWOptimizer() : lr(1e-5f), beta1(0.9f), beta2(0.999f), eps(1e-8f), weight_decay(0.01f) {}

    // use_master = true keeps the reference's FP32 master copy (28 bytes per parameter and step);
    // false reads the FP16 weight as the source of truth (22 bytes).
    explicit AdamWOptimizer(const ParamPools& pools, float lr = 1e-4f, float beta1 = 0.9f, float beta2 = 0.999f,
                            float eps = 1e-8f, float weight_decay = 0.01f, bool use_master = true)
        : lr(lr), beta1(beta1), beta2(beta2), eps(eps), weight_decay(weight_decay) {
        init(pools, use_master);
    }

    // The reference's constructor (optimizer.h:70-80) for any model type with the members it reads:
    // model->config.{num_hidden_layers, hidden_size, q_dim, kv_dim, intermediate_size, head_dim, vocab_size}
    // and model->weights.{fp16_pool, fp16_pool_elems, fp32_pool, fp32_pool_elems}.  The sizes derived from the
    // configuration must equal the pool sizes (the reference asserts the same, optimizer.h:221-222).
    template <class Model, class = decltype(std::declval<Model&>().weights.fp16_pool_elems)>
    explicit AdamWOptimizer(Model* model, float lr = 1e-4f, float beta1 = 0.9f, float beta2 = 0.999f,
                            float eps = 1e-8f, float weight_decay = 0.01f, bool use_master = true)
        : lr(lr), beta1(beta1), beta2(beta2), eps(eps), weight_decay(weight_decay) {
        const auto& c = model->config;
        ParamPools pools = ParamPools::for_qwen3(c.num_hidden_layers, c.hidden_size, c.q_dim, c.kv_dim,
                                                 c.intermediate_size, c.head_dim, c.vocab_size);
        if (pools.fp16_pool_elems != (size_t)model->weights.fp16_pool_elems ||
            pools.fp32_pool_elems != (size_t)model->weights.fp32_pool_elems) {
            fprintf(stderr, "[AdamW] the model's weight pools (%zu FP16, %zu FP32 elements) do not have the sizes that "
                            "its configuration gives (%zu, %zu)\n", (size_t)model->weights.fp16_pool_elems,
                    (size_t)model->weights.fp32_pool_elems, pools.fp16_pool_elems, pools.fp32_pool_elems);
            exit(1);
        }
        pools.fp16_pool = model->weights.fp16_pool;
        pools.fp32_pool = model->weights.fp32_pool;
        init(pools, use_master);
    }

    ~AdamWOptimizer() { free(); }

    AdamWOptimizer(const AdamWOptimizer&) = delete;
    AdamWOptimizer& operator=(const AdamWOptimizer&) = delete;
    AdamWOptimizer(AdamWOptimizer&& o) noexcept { move_from(o); }
    AdamWOptimizer& operator=(AdamWOptimizer&& o) noexcept {
        if (this != &o) { free(); move_from(o); }
        return *this;
    }

    void set_lr(float new_lr) { lr = new_lr; }
    int get_step() const { return step_; }

    float* fp16_master() { return fp16_master_; }
    float* fp16_m() { return fp16_m_; }
    float* fp16_v() { return fp16_v_; }
    float* fp32_m() { return fp32_m_; }
    float* fp32_v() { return fp32_v_; }
    size_t num_fp16_params() const { return n16_; }
    size_t num_fp32_params() const { return n32_; }

    // Test accessors by (layer, tensor), as in the reference (optimizer.h:107-116); they need the
    // per-layer structure in ParamPools.  proj: 0=q 1=k 2=v 3=o 4=gate 5=up 6=down;
    // norm: 0=input 1=q 2=k 3=post_attn.
    float* get_fp16_master(int layer, int proj) const { return fp16_master_ ? fp16_master_ + fp16_offset(layer, proj) : nullptr; }
    float* get_fp16_m(int layer, int proj) const { return fp16_m_ + fp16_offset(layer, proj); }
    float* get_fp16_v(int layer, int proj) const { return fp16_v_ + fp16_offset(layer, proj); }
    float* get_fp32_m_norm(int layer, int norm) const { return fp32_m_ + fp32_offset(layer, norm); }
    float* get_fp32_v_norm(int layer, int norm) const { return fp32_v_ + fp32_offset(layer, norm); }
    float* get_final_norm_m() const { return fp32_m_ + fp32_offset(pools_.num_layers, 0); }
    float* get_final_norm_v() const { return fp32_v_ + fp32_offset(pools_.num_layers, 0); }

    // Treat the embedding (the tail of the FP16 pool) as frozen: its gradients count as zero in the
    // norm and the update leaves it alone, instead of clearing the gradients and streaming an
    // identity update over it (trainer.h:269-277).  Exact while its moments are zero.
    void set_embed_frozen(bool frozen) {
        if (frozen != embed_frozen_) {
            embed_frozen_ = frozen;
            if (plan_) { RLX_CHECK(rlx_plan_destroy(plan_)); plan_ = nullptr; }
            sched_len_ = 0;
        }
    }

    // How the reference's two calls behave here (both off by default, which is the reference's behaviour):
    // fused clip: clip_grad_norm_() leaves the gradients unscaled and the following step() applies the scale
    // inside the update (one pass over the gradients less); zero grads: step() clears both gradient pools after
    // reading them (then the caller drops its qwen3_gradients_zero at the start of the next step).
    void set_fused_clip(bool on) { fused_clip_ = on; if (!on) clip_pending_ = false; }
    void set_zero_grads(bool on) { zero_grads_ = on; }
    bool fused_clip() const { return fused_clip_; }

    // One optimizer step with the reference's signature (optimizer.h:119): step(grads, stream = 0).
    // `grads` is any type with half_pool, float_pool, half_pool_bytes, float_pool_bytes
    // (Qwen3Gradients, include/model/qwen3.h:190-218; GradPools above).
    template <class Grads>
    void step(Grads* grads, hipStream_t stream = 0) {
        const bool fused = clip_pending_;
        clip_pending_ = false;
        step(grads, stream, fused, zero_grads_);
    }

    // The same with the two options given per call.  fused_clip: apply the clip scale that the last norm
    // pass of plan_for(grads) left on the device, inside the update.  zero_grads: clear both gradient
    // pools after they have been read (the job of qwen3_gradients_zero at the next step).
    template <class Grads>
    void step(Grads* grads, hipStream_t stream, bool fused_clip, bool zero_grads) {
        step_++;
        rlx_step_params sp;
        sp.lr = lr; sp.beta1 = beta1; sp.beta2 = beta2; sp.eps = eps; sp.weight_decay = weight_decay;
        sp.bias_correction1 = 1.0f - powf(beta1, (float)step_);
        sp.bias_correction2 = 1.0f - powf(beta2, (float)step_);
        const int flags = (fused_clip ? RLX_CLIP_FUSED : 0) | (zero_grads ? RLX_STEP_ZERO_GRADS : 0);
        RLX_CHECK(rlx_plan_adamw(plan_for(grads), &sp, flags, (void*)stream));
    }

    // Steps without the host (a recorded norm + update replayed step after step).  upload_schedule puts the
    // hyper-parameters of the next n steps (steps get_step()+1, ...) on the device: the given learning rates and
    // the bias corrections formed here with powf, as in step().  step_scheduled launches the update with the
    // current entry; the device then moves on to the next entry by itself, so a recorded step_scheduled can be
    // replayed with nothing written by the host in between, through this window and every later one (the
    // recorded launch does not depend on the table's address or length).
    //
    //     optimizer.set_fused_clip(true);
    //     optimizer.upload_schedule(grads, lrs, n);              // window 1
    //     hipStreamBeginCapture(s, ...);
    //     optimizer.clip_grad_norm_async(grads, max_norm, s);    // norm and clip scale, nothing read by the host
    //     optimizer.step_scheduled(grads, s);                    // recorded, not run: get_step() does not move
    //     hipStreamEndCapture(s, &graph); ...
    //     for (k = 0; k < n; k++) hipGraphLaunch(exec, s);       // new gradients before each replay
    //     optimizer.note_replayed_steps(n);                      // get_step() += n
    //     optimizer.upload_schedule(grads, next_lrs, n2);        // window 2: same graph, replay on
    //
    // A call while `stream` is being captured does not count as a step; every eager call does.  Running more
    // scheduled steps than the table holds would reuse the last entry's learning rate and bias corrections: an
    // eager step_scheduled refuses (exits with a message), note_replayed_steps reports it.
    // The table belongs to the plan: if the gradient pools move or set_embed_frozen changes, the plan is rebuilt
    // and the schedule has to be uploaded again.
    template <class Grads>
    void upload_schedule(Grads* grads, const float* lrs, int n, hipStream_t stream = 0) {
        std::vector<rlx_step_params> steps((size_t)n);
        for (int k = 0; k < n; k++) {
            rlx_step_params& sp = steps[(size_t)k];
            sp.lr = lrs[k]; sp.beta1 = beta1; sp.beta2 = beta2; sp.eps = eps; sp.weight_decay = weight_decay;
            sp.bias_correction1 = 1.0f - powf(beta1, (float)(step_ + 1 + k));
            sp.bias_correction2 = 1.0f - powf(beta2, (float)(step_ + 1 + k));
        }
        RLX_CHECK(rlx_plan_schedule_upload(plan_for(grads), steps.data(), n, (void*)stream));
        sched_from_ = step_;
        sched_len_ = n;
    }

    // fused_clip: apply, inside the update, the clip scale that the last norm of plan_for(grads) left on the
    // device.  The two-argument form takes it from clip_grad_norm_ / clip_grad_norm_async having run with
    // set_fused_clip(true) since the last step.
    template <class Grads>
    void step_scheduled(Grads* grads, hipStream_t stream, bool fused_clip) {
        rlx_plan* plan = plan_for(grads);
        hipStreamCaptureStatus capturing = hipStreamCaptureStatusNone;
        if (stream) HIP_CHECK(hipStreamIsCapturing(stream, &capturing));
        if (capturing == hipStreamCaptureStatusNone) {
            if (step_ - sched_from_ >= sched_len_) {
                fprintf(stderr, "[AdamW] step_scheduled: the uploaded table of %d steps is used up (or none was uploaded "
                                "for these gradient pools); call upload_schedule for the next window first\n", sched_len_);
                exit(1);
            }
            step_++;
        }
        const int flags = (fused_clip ? RLX_CLIP_FUSED : 0) | (zero_grads_ ? RLX_STEP_ZERO_GRADS : 0);
        RLX_CHECK(rlx_plan_adamw_scheduled(plan, flags, (void*)stream));
    }
    template <class Grads>
    void step_scheduled(Grads* grads, hipStream_t stream = 0) {
        const bool fused = clip_pending_;
        clip_pending_ = false;
        step_scheduled(grads, stream, fused);
    }
    // After n replays of a recorded step_scheduled.  Returns false (and says so) if that was more than the table held.
    bool note_replayed_steps(int n) {
        step_ += n;
        if (step_ - sched_from_ <= sched_len_) return true;
        fprintf(stderr, "[AdamW] %d scheduled steps have run since a table of %d was uploaded: the last %d reused the "
                        "table's last learning rate and bias corrections\n", step_ - sched_from_, sched_len_,
                step_ - sched_from_ - sched_len_);
        return false;
    }

    // The half of clip_grad_norm_ that needs no host (so that it can be recorded): norm and clip scale stay on
    // the device.  With set_fused_clip(true) the next step / step_scheduled applies the scale; otherwise the
    // scale pass is launched here (it reads the scale on the device and touches nothing when it is 1).
    template <class Grads>
    void clip_grad_norm_async(Grads* grads, float max_norm, hipStream_t stream = 0) {
        rlx_plan* plan = plan_for(grads);
        RLX_CHECK(rlx_plan_grad_norm(plan, max_norm, (void*)stream));
        if (fused_clip_) clip_pending_ = true;
        else RLX_CHECK(rlx_plan_scale_grads(plan, (void*)stream));
    }

    // Trainer::clip_grad_norm_ (trainer.h:323-352) over the same gradient type: clips all gradients
    // (half_pool + float_pool) so that the global L2 norm is <= max_norm and returns the pre-clip norm
    // (host scalar, synchronous), like the reference.  With set_fused_clip(true) the gradients stay as they
    // are and the next step() applies the scale.  It lives here because the optimizer owns the plan.
    template <class Grads>
    float clip_grad_norm_(Grads* grads, float max_norm, hipStream_t stream = 0) {
        rlx_plan* plan = plan_for(grads);
        RLX_CHECK(rlx_plan_grad_norm(plan, max_norm, (void*)stream));
        float total_norm = 0.0f;
        RLX_CHECK(rlx_plan_norm_read(plan, &total_norm, nullptr, nullptr, (void*)stream));
        if (fused_clip_) clip_pending_ = true;
        else if (total_norm > max_norm) RLX_CHECK(rlx_plan_scale_grads(plan, (void*)stream));
        return total_norm;
    }

    // Optimizer state on disk (the reference's save_checkpoint is a stub, trainer.h:317-319, so the format is
    // this library's; rl.cu_amd/host.py reads and writes the same files).
    // File: "RLXOPT02", int32 step, 5 floats (lr, beta1, beta2, eps, weight_decay), int32 sections;
    // per section: uint16 name length, name, uint8 dtype (1 = FP32), int64 count, uint64 sum of the
    // data's 32-bit words, data.  Sections, in this order, each over a whole pool (all FP16 tensors in pool
    // order, then all FP32 tensors) and left out when empty: fp16.master (if kept), fp16.m, fp16.v, fp32.m,
    // fp32.v.  Data moves through a 64 MB staging buffer, so the host never holds a whole pool.
    // Both return false (and print why) on failure; load_state checks the whole file before it touches the
    // state and leaves it alone if anything is wrong.
    // Size of the staging buffer of save_state / load_state in floats (default 16 Mi = 64 MB).
    void set_state_staging(size_t floats) { stage_limit_ = floats ? floats : 1; }

    bool save_state(const std::string& path) const {
        HIP_CHECK(hipDeviceSynchronize());
        const std::string tmp = path + ".tmp";
        FILE* f = fopen(tmp.c_str(), "wb");
        if (!f) { fprintf(stderr, "[AdamW] cannot write %s\n", tmp.c_str()); return false; }
        const std::vector<Section> secs = sections();
        const int32_t step = step_, nsec = (int32_t)secs.size();
        const float hyper[5] = {lr, beta1, beta2, eps, weight_decay};
        bool ok = fwrite(kStateMagic, 1, 8, f) == 8 && fwrite(&step, 4, 1, f) == 1 && fwrite(hyper, 4, 5, f) == 5 &&
                  fwrite(&nsec, 4, 1, f) == 1;
        std::vector<float> stage(stage_floats(secs));
        for (const Section& s : secs) {
            if (!ok) break;
            const uint16_t len = (uint16_t)s.name.size();
            const uint8_t dtype = 1;
            const int64_t count = (int64_t)s.n;
            uint64_t sum = 0;
            ok = fwrite(&len, 2, 1, f) == 1 && fwrite(s.name.data(), 1, len, f) == len &&
                 fwrite(&dtype, 1, 1, f) == 1 && fwrite(&count, 8, 1, f) == 1;
            const off_t sum_at = ftello(f);
            ok = ok && sum_at >= 0 && fwrite(&sum, 8, 1, f) == 1;      // patched below, once the data has passed
            for (size_t done = 0; ok && done < s.n; done += stage.size()) {
                const size_t k = s.n - done < stage.size() ? s.n - done : stage.size();
                HIP_CHECK(hipMemcpy(stage.data(), s.dev + done, k * sizeof(float), hipMemcpyDeviceToHost));
                sum += word_sum(stage.data(), k);
                ok = fwrite(stage.data(), sizeof(float), k, f) == k;
            }
            ok = ok && fseeko(f, sum_at, SEEK_SET) == 0 && fwrite(&sum, 8, 1, f) == 1 && fseeko(f, 0, SEEK_END) == 0;
        }
        ok = (fclose(f) == 0) && ok;
        if (ok) ok = rename(tmp.c_str(), path.c_str()) == 0;
        if (!ok) { fprintf(stderr, "[AdamW] writing %s failed\n", path.c_str()); remove(tmp.c_str()); }
        return ok;
    }

    bool load_state(const std::string& path) {
        FILE* f = fopen(path.c_str(), "rb");
        if (!f) { fprintf(stderr, "[AdamW] cannot read %s\n", path.c_str()); return false; }
        const std::vector<Section> secs = sections();
        std::string why;
        char magic[8];
        int32_t step = 0, nsec = 0;
        float hyper[5] = {};
        if (fread(magic, 1, 8, f) != 8) why = "shorter than a header";
        else if (memcmp(magic, "RLXOPT01", 8) == 0) why = "written in the older RLXOPT01 layout, which is no longer read";
        else if (memcmp(magic, kStateMagic, 8) != 0) why = "not an optimizer state file";
        else if (fread(&step, 4, 1, f) != 1 || fread(hyper, 4, 5, f) != 5 || fread(&nsec, 4, 1, f) != 1) why = "truncated header";
        else if (step < 0) why = "negative step counter";
        else if (nsec != (int32_t)secs.size())
            why = "holds " + std::to_string(nsec) + " sections, this optimizer has " + std::to_string(secs.size()) +
                  " (different layout: master copy or FP32 pool present on one side only)";
        for (int k = 0; why.empty() && k < 5; k++)
            if (!std::isfinite(hyper[k])) why = "hyper-parameter that is not finite";
        // pass 1: every section header must match and every checksum must hold, before anything is changed
        std::vector<float> stage(why.empty() ? stage_floats(secs) : 0);
        std::vector<off_t> data_at(secs.size(), 0);
        for (size_t i = 0; why.empty() && i < secs.size(); i++) {
            uint16_t len = 0;
            uint8_t dtype = 0;
            int64_t count = 0;
            uint64_t want = 0, sum = 0;
            char name[256];
            if (fread(&len, 2, 1, f) != 1 || len >= sizeof(name) || fread(name, 1, len, f) != len ||
                fread(&dtype, 1, 1, f) != 1 || fread(&count, 8, 1, f) != 1 || fread(&want, 8, 1, f) != 1) {
                why = "truncated in the header of section " + std::to_string(i);
            } else if (std::string(name, len) != secs[i].name || dtype != 1 || count != (int64_t)secs[i].n) {
                why = "section " + std::to_string(i) + " is '" + std::string(name, len) + "' with " + std::to_string(count) +
                      " values, this optimizer needs '" + secs[i].name + "' with " + std::to_string(secs[i].n) +
                      " (different model or layout)";
            } else {
                data_at[i] = ftello(f);
                for (size_t done = 0; why.empty() && done < secs[i].n; done += stage.size()) {
                    const size_t k = secs[i].n - done < stage.size() ? secs[i].n - done : stage.size();
                    if (fread(stage.data(), sizeof(float), k, f) != k) why = "truncated in the data of section '" + secs[i].name + "'";
                    else sum += word_sum(stage.data(), k);
                }
                if (why.empty() && sum != want) why = "damaged: checksum of section '" + secs[i].name + "' does not match";
            }
        }
        if (why.empty() && fgetc(f) != EOF) why = "longer than its sections";
        if (!why.empty()) {
            fclose(f);
            fprintf(stderr, "[AdamW] %s: %s\n", path.c_str(), why.c_str());
            return false;
        }
        // pass 2: copy to the device
        bool ok = true;
        for (size_t i = 0; ok && i < secs.size(); i++) {
            ok = fseeko(f, data_at[i], SEEK_SET) == 0;
            for (size_t done = 0; ok && done < secs[i].n; done += stage.size()) {
                const size_t k = secs[i].n - done < stage.size() ? secs[i].n - done : stage.size();
                ok = fread(stage.data(), sizeof(float), k, f) == k;
                if (ok) HIP_CHECK(hipMemcpy(secs[i].dev + done, stage.data(), k * sizeof(float), hipMemcpyHostToDevice));
            }
        }
        fclose(f);
        if (!ok) {      // the file changed under us between the passes: the state is now partly overwritten
            fprintf(stderr, "[AdamW] %s: read error while loading; the optimizer state is incomplete\n", path.c_str());
            exit(1);
        }
        step_ = step;
        lr = hyper[0]; beta1 = hyper[1]; beta2 = hyper[2]; eps = hyper[3]; weight_decay = hyper[4];
        return true;
    }

    // The multi-tensor plan over {projections, embedding, norm weights, workspace tail} for these
    // gradient pools; built on first use and rebuilt if the pools move.
    template <class Grads>
    rlx_plan* plan_for(Grads* grads) {
        if (plan_ && grads->half_pool == plan_half_ && grads->float_pool == plan_float_ &&
            grads->float_pool_bytes == plan_float_bytes_)
            return plan_;
        if (plan_) { RLX_CHECK(rlx_plan_destroy(plan_)); plan_ = nullptr; }
        sched_len_ = 0;                 // an uploaded step table went with the old plan
        assert(grads->half_pool_bytes / sizeof(half) == n16_);
        assert(grads->float_pool_bytes / sizeof(float) >= n32_);
        rlx_tensor_desc d[4];
        int k = 0;
        const size_t embed_n = n16_ - proj_n_;
        if (proj_n_) {
            d[k++] = {pools_.fp16_pool, grads->half_pool, fp16_m_, fp16_v_, fp16_master_, (int64_t)proj_n_,
                      RLX_DTYPE_F16, 0};
        }
        if (embed_n) {   // no decay on the embedding (optimizer.h:131-140)
            d[k++] = {pools_.fp16_pool + proj_n_, grads->half_pool + proj_n_, fp16_m_ + proj_n_, fp16_v_ + proj_n_,
                      fp16_master_ ? fp16_master_ + proj_n_ : nullptr, (int64_t)embed_n, RLX_DTYPE_F16,
                      (uint32_t)(RLX_TENSOR_NO_DECAY | (embed_frozen_ ? RLX_TENSOR_FROZEN : 0))};
        }
        if (n32_) {      // no decay on the norm weights (optimizer.h:142-146)
            d[k++] = {pools_.fp32_pool, grads->float_pool, fp32_m_, fp32_v_, nullptr, (int64_t)n32_, RLX_DTYPE_F32,
                      RLX_TENSOR_NO_DECAY};
        }
        const size_t tail = grads->float_pool_bytes / sizeof(float) - n32_;
        if (tail) {
            d[k++] = {nullptr, (float*)grads->float_pool + n32_, nullptr, nullptr, nullptr, (int64_t)tail, RLX_DTYPE_F32,
                      RLX_TENSOR_GRAD_ONLY};
        }
        RLX_CHECK(rlx_plan_create(d, k, 0, &plan_));
        plan_half_ = grads->half_pool; plan_float_ = grads->float_pool; plan_float_bytes_ = grads->float_pool_bytes;
        return plan_;
    }

private:
    ParamPools pools_;
    int step_ = 0;
    float* fp16_master_ = nullptr;
    float* fp16_m_ = nullptr;
    float* fp16_v_ = nullptr;
    float* fp32_m_ = nullptr;
    float* fp32_v_ = nullptr;
    float* fp16_state_ = nullptr;   // single allocation: [master | m | v] or [m | v]
    float* fp32_state_ = nullptr;   // single allocation: [m | v]
    size_t n16_ = 0, n32_ = 0, proj_n_ = 0;
    rlx_plan* plan_ = nullptr;
    half* plan_half_ = nullptr;
    float* plan_float_ = nullptr;
    size_t plan_float_bytes_ = 0;
    bool embed_frozen_ = false;
    bool fused_clip_ = false, zero_grads_ = false;
    bool clip_pending_ = false;     // a fused clip_grad_norm_() has run since the last step()
    int sched_from_ = 0, sched_len_ = 0;   // get_step() at the last upload_schedule and that table's length

    size_t fp16_offset(int layer, int proj) const {
        assert(pools_.num_layers > 0 && layer >= 0 && layer < pools_.num_layers && proj >= 0 && proj < 7);
        return pool_offset(pools_.proj_sizes, 7, layer, proj);
    }
    size_t fp32_offset(int layer, int norm) const {
        assert(pools_.num_layers > 0 && layer >= 0 && layer <= pools_.num_layers && norm >= 0 && norm < 4);
        return pool_offset(pools_.norm_sizes, 4, layer, norm);
    }

    struct Section { std::string name; float* dev; size_t n; };
    std::vector<Section> sections() const {
        std::vector<Section> s;
        if (fp16_master_) s.push_back({"fp16.master", fp16_master_, n16_});
        if (n16_) { s.push_back({"fp16.m", fp16_m_, n16_}); s.push_back({"fp16.v", fp16_v_, n16_}); }
        if (n32_) { s.push_back({"fp32.m", fp32_m_, n32_}); s.push_back({"fp32.v", fp32_v_, n32_}); }
        return s;
    }
    static constexpr const char* kStateMagic = "RLXOPT02";
    size_t stage_limit_ = (size_t)16 << 20;         // floats: 64 MB between the device and the file
    size_t stage_floats(const std::vector<Section>& secs) const {
        size_t most = 1;
        for (const Section& s : secs) most = s.n > most ? s.n : most;
        return most < stage_limit_ ? most : stage_limit_;
    }
    static uint64_t word_sum(const float* p, size_t n) {
        uint64_t acc = 0;
        for (size_t i = 0; i < n; i++) { uint32_t w; memcpy(&w, p + i, 4); acc += w; }
        return acc;
    }

    void init(const ParamPools& pools, bool use_master) {
        pools_ = pools;
        n16_ = pools.fp16_pool_elems;
        n32_ = pools.fp32_pool_elems;
        proj_n_ = pools.proj_elems;
        assert(proj_n_ <= n16_);
        const size_t parts = use_master ? 3 : 2;
        if (n16_) {
            HIP_CHECK(hipMalloc((void**)&fp16_state_, n16_ * parts * sizeof(float)));
            HIP_CHECK(hipMemset(fp16_state_, 0, n16_ * parts * sizeof(float)));
        }
        if (n32_) {
            HIP_CHECK(hipMalloc((void**)&fp32_state_, n32_ * 2 * sizeof(float)));
            HIP_CHECK(hipMemset(fp32_state_, 0, n32_ * 2 * sizeof(float)));
        }
        float* q = fp16_state_;
        if (use_master) { fp16_master_ = q; q += n16_; }
        fp16_m_ = q;
        fp16_v_ = q + n16_;
        fp32_m_ = fp32_state_;
        fp32_v_ = fp32_state_ + n32_;
        if (use_master && n16_) {
            RLX_CHECK(rlx_fp16_to_fp32(fp16_master_, reinterpret_cast<const uint16_t*>(pools.fp16_pool),
                                       (int64_t)n16_, nullptr));
        }
        HIP_CHECK(hipDeviceSynchronize());
        printf("[AdamW] state on device: %zu FP16 params -> %.1f MB (%s), %zu FP32 params -> %.2f MB; lr=%.1e wd=%.2f\n",
               n16_, n16_ * parts * sizeof(float) / (1024.0 * 1024.0), use_master ? "master, m, v" : "m, v", n32_,
               n32_ * 2 * sizeof(float) / (1024.0 * 1024.0), lr, weight_decay);
    }

    void free() {
        if (plan_) { rlx_plan_destroy(plan_); plan_ = nullptr; }
        if (fp16_state_) { (void)hipFree(fp16_state_); fp16_state_ = nullptr; }
        if (fp32_state_) { (void)hipFree(fp32_state_); fp32_state_ = nullptr; }
        fp16_master_ = fp16_m_ = fp16_v_ = fp32_m_ = fp32_v_ = nullptr;
    }

    void move_from(AdamWOptimizer& o) {
        lr = o.lr; beta1 = o.beta1; beta2 = o.beta2; eps = o.eps; weight_decay = o.weight_decay;
        pools_ = o.pools_; step_ = o.step_;
        fp16_master_ = o.fp16_master_; fp16_m_ = o.fp16_m_; fp16_v_ = o.fp16_v_;
        fp32_m_ = o.fp32_m_; fp32_v_ = o.fp32_v_;
        fp16_state_ = o.fp16_state_; fp32_state_ = o.fp32_state_;
        n16_ = o.n16_; n32_ = o.n32_; proj_n_ = o.proj_n_;
        plan_ = o.plan_; plan_half_ = o.plan_half_; plan_float_ = o.plan_float_; plan_float_bytes_ = o.plan_float_bytes_;
        embed_frozen_ = o.embed_frozen_; stage_limit_ = o.stage_limit_;
        fused_clip_ = o.fused_clip_; zero_grads_ = o.zero_grads_; clip_pending_ = o.clip_pending_;
        sched_from_ = o.sched_from_; sched_len_ = o.sched_len_;
        o.plan_ = nullptr; o.fp16_state_ = nullptr; o.fp32_state_ = nullptr;
        o.fp16_master_ = o.fp16_m_ = o.fp16_v_ = o.fp32_m_ = o.fp32_v_ = nullptr;
    }
};

// Body for the reference's Trainer::clip_grad_norm_(Qwen3Gradients* grads, float max_norm) (trainer.h:323-352),
// whose call sites (trainer.h:282, GRPO_trainer.h:511) then stay as they are:
//     float clip_grad_norm_(Qwen3Gradients* grads, float max_norm) { return ::clip_grad_norm_(optimizer_, grads, max_norm); }
template <class Grads>
inline float clip_grad_norm_(AdamWOptimizer& optimizer, Grads* grads, float max_norm) {
    return optimizer.clip_grad_norm_(grads, max_norm);
}
