// The optimizer end of Trainer::training_step for C++ callers (include/training/trainer.h:269-288
// and :323-352; GRPO_trainer.h:508-514 calls the same two functions): optional zeroing of the
// embedding gradients, gradient clipping by global L2 norm, one optimizer step.
#pragma once
#include "optimizer.h"

struct OptimStepConfig {          // the fields of TrainingConfig that this path reads (trainer.h:36-43)
    float max_grad_norm = 1.0f;   // <= 0 disables clipping
    bool freeze_embed = false;
    bool fused_clip = false;      // apply the clip scale inside the update instead of a scale pass
    bool zero_grads = false;      // clear the gradient pools inside the update (then the caller drops its
                                  // qwen3_gradients_zero at the start of the next step)
    bool freeze_in_plan = false;  // with freeze_embed: flag the embedding as frozen in the plan instead
                                  // of clearing its gradients and updating it with zeros
};

class OptimStep {
public:
    OptimStep(AdamWOptimizer* optimizer, OptimStepConfig config) : optimizer_(optimizer), config_(config) {}

    // Clip all gradients (half_pool + float_pool) so that the global L2 norm is <= max_norm.
    // Returns the pre-clip norm (host scalar, synchronous), like the reference.
    float clip_grad_norm_(GradPools* grads, float max_norm, hipStream_t stream = 0) {
        rlx_plan* plan = optimizer_->plan_for(grads);
        RLX_CHECK(rlx_plan_grad_norm(plan, max_norm, (void*)stream));
        float total_norm = 0.0f;
        RLX_CHECK(rlx_plan_norm_read(plan, &total_norm, nullptr, nullptr, (void*)stream));
        if (!config_.fused_clip && total_norm > max_norm) RLX_CHECK(rlx_plan_scale_grads(plan, (void*)stream));
        return total_norm;
    }

    // What training_step does after the backward passes.  embed_elems: size of the embedding at
    // the end of half_pool (only read when freeze_embed is set).  Returns the pre-clip norm.
    float apply(GradPools* grads, size_t embed_elems = 0, hipStream_t stream = 0) {
        optimizer_->set_embed_frozen(config_.freeze_embed && config_.freeze_in_plan);
        if (config_.freeze_embed && !config_.freeze_in_plan && embed_elems) {
            const size_t half_elems = grads->half_pool_bytes / sizeof(half);
            half* embed_grad = grads->half_pool + (half_elems - embed_elems);
            // zeros through a fill kernel (0 + 0 * z), which unlike a memset node is safe to capture
            RLX_CHECK(rlx_fill_f16(reinterpret_cast<uint16_t*>(embed_grad), (int64_t)embed_elems, 0, 0, 0.0f, 0.0f, 0,
                                   0, 0, (void*)stream));
        }
        float grad_norm = 0.0f;
        const bool clip = config_.max_grad_norm > 0.0f;
        if (clip) grad_norm = clip_grad_norm_(grads, config_.max_grad_norm, stream);
        optimizer_->step(grads, stream, clip && config_.fused_clip, config_.zero_grads);
        last_grad_norm_ = grad_norm;
        return grad_norm;
    }

    float last_grad_norm() const { return last_grad_norm_; }

private:
    AdamWOptimizer* optimizer_;
    OptimStepConfig config_;
    float last_grad_norm_ = 0.0f;
};
