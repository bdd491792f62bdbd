// Helpers around the optimizer for C++ callers without the reference's Trainer class.  (The header has a name of
// its own: the reference keeps its include/training/trainer.h, which this one must not shadow on the include path.)
// The optimizer end of Trainer::training_step for C++ callers (include/training/trainer.h:269-288
// and :323-352; GRPO_trainer.h:508-514 calls the same two functions): optional zeroing of the
// embedding gradients, gradient clipping by global L2 norm, one optimizer step.
#pragma once
#include <chrono>
#include <functional>

#include "logger.h"
#include "lr_scheduler.h"
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
    template <class Grads>
    float clip_grad_norm_(Grads* grads, float max_norm, hipStream_t stream = 0) {
        optimizer_->set_fused_clip(config_.fused_clip);
        return optimizer_->clip_grad_norm_(grads, max_norm, stream);
    }

    // What training_step does after the backward passes.  embed_elems: size of the embedding at
    // the end of half_pool (only read when freeze_embed is set).  Returns the pre-clip norm.
    template <class Grads>
    float apply(Grads* grads, size_t embed_elems = 0, hipStream_t stream = 0) {
        optimizer_->set_embed_frozen(config_.freeze_embed && config_.freeze_in_plan);
        optimizer_->set_fused_clip(config_.fused_clip);
        optimizer_->set_zero_grads(config_.zero_grads);
        if (config_.freeze_embed && !config_.freeze_in_plan && embed_elems) {
            const size_t half_elems = grads->half_pool_bytes / sizeof(half);
            half* embed_grad = grads->half_pool + (half_elems - embed_elems);
            // cleared by a kernel, which unlike a memset node is safe to record into a HIP graph
            RLX_CHECK(rlx_clear(embed_grad, (int64_t)(embed_elems * sizeof(half)), (void*)stream));
        }
        float grad_norm = 0.0f;
        const bool clip = config_.max_grad_norm > 0.0f;
        if (clip) grad_norm = clip_grad_norm_(grads, config_.max_grad_norm, stream);
        optimizer_->step(grads, stream);    // applies the scale itself after a fused clip_grad_norm_
        last_grad_norm_ = grad_norm;
        return grad_norm;
    }

    // Trainer::training_step around the optimizer (trainer.h:231-289): clear the gradient pools, run
    // grad_accum_steps micro-batches, then apply().  micro_batch(k, scale_loss_grad) stands for forward,
    // compute_loss and backward of micro-batch k and returns its loss; it calls scale_loss_grad(d_loss_grad, n)
    // where the reference launches scale_grad_kernel (trainer.h:261-263), before its backward pass adds
    // into the pools.  Returns the mean loss; the pre-clip norm is last_grad_norm().
    using ScaleLossGrad = std::function<void(float*, size_t)>;
    float training_step(GradPools* grads, int grad_accum_steps,
                        const std::function<float(int, const ScaleLossGrad&)>& micro_batch, size_t embed_elems = 0,
                        hipStream_t stream = 0) {
        const float scale = 1.0f / (float)grad_accum_steps;
        grad_pools_zero(grads, stream);
        const ScaleLossGrad scale_loss_grad = [scale, stream](float* d_loss_grad, size_t n) {
            RLX_CHECK(rlx_scale_f32(d_loss_grad, scale, (int64_t)n, (void*)stream));
        };
        float accum_loss = 0.0f;
        for (int acc = 0; acc < grad_accum_steps; acc++) accum_loss += micro_batch(acc, scale_loss_grad);
        apply(grads, embed_elems, stream);
        return accum_loss / (float)grad_accum_steps;
    }

    float last_grad_norm() const { return last_grad_norm_; }

private:
    AdamWOptimizer* optimizer_;
    OptimStepConfig config_;
    float last_grad_norm_ = 0.0f;
};

// The optimizer end of Trainer::train (include/training/trainer.h:183-225): per step set the scheduled
// rate, obtain gradients (produce_grads(step) stands for the forward/backward passes and returns the
// loss), clip and step, synchronise, log loss / lr / grad_norm / step_ms / tok_per_sec, commit every
// logging_steps, save the optimizer state every save_steps.  Returns the number of steps taken.
struct TrainLoopConfig {
    int total_steps = 0;
    int logging_steps = 1;
    int save_steps = 0;               // 0: never
    std::string save_path;            // optimizer state file
    float tokens_per_step = 0.0f;     // global_batch_size * sequence length
    size_t embed_elems = 0;
};

inline int run_train_loop(AdamWOptimizer& optimizer, const LRScheduler& scheduler, Logger& logger, OptimStep& tail,
                          GradPools* grads, const std::function<float(int)>& produce_grads,
                          const TrainLoopConfig& cfg, hipStream_t stream = 0) {
    int global_step = 0;
    while (global_step < cfg.total_steps) {
        const float cur_lr = scheduler.get_lr(global_step);
        optimizer.set_lr(cur_lr);
        const auto t0 = std::chrono::steady_clock::now();
        const float loss = produce_grads(global_step);
        const float grad_norm = tail.apply(grads, cfg.embed_elems, stream);
        HIP_CHECK(hipDeviceSynchronize());
        const auto t1 = std::chrono::steady_clock::now();
        const float step_ms = std::chrono::duration<float, std::milli>(t1 - t0).count();
        const float tok_per_sec = cfg.tokens_per_step / (step_ms * 1e-3f);
        global_step++;
        logger.log(global_step, "loss", loss);
        logger.log(global_step, "lr", cur_lr);
        logger.log(global_step, "grad_norm", grad_norm);
        logger.log(global_step, "step_ms", step_ms);
        logger.log(global_step, "tok_per_sec", tok_per_sec);
        if (cfg.logging_steps > 0 && global_step % cfg.logging_steps == 0) logger.commit(global_step);
        if (cfg.save_steps > 0 && !cfg.save_path.empty() && global_step % cfg.save_steps == 0)
            optimizer.save_state(cfg.save_path);
    }
    return global_step;
}
