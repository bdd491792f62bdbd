// Learning-rate schedule that feeds AdamWOptimizer::set_lr once per step: linear warm-up, then
// either a constant rate or a half-cosine decay to a floor.  Same class name, methods and FP32
// arithmetic as the reference's include/training/lr_scheduler.h:10-57, so that
// `optimizer_.set_lr(lr_scheduler_.get_lr(global_step))` (include/training/trainer.h:193-194)
// produces the same bits.
#pragma once
#include <cmath>

enum class LRScheduleType { Constant, Cosine };

class LRScheduler {
public:
    LRScheduler() = default;

    // Constant rate after an optional warm-up of `warmup_steps` steps.
    void init_constant(float base_lr, int warmup_steps = 0) {
        kind_ = LRScheduleType::Constant;
        peak_ = base_lr;
        floor_ = base_lr;
        warmup_ = warmup_steps;
        horizon_ = 0;
    }

    // Warm-up to base_lr, then cosine decay that reaches min_lr at step `total_steps`.
    void init_cosine(float base_lr, float min_lr, int warmup_steps, int total_steps) {
        kind_ = LRScheduleType::Cosine;
        peak_ = base_lr;
        floor_ = min_lr;
        warmup_ = warmup_steps;
        horizon_ = total_steps;
    }

    // Rate for optimizer step number `step` (0-based).
    float get_lr(int step) const {
        const bool warming = warmup_ > 0 && step < warmup_;
        if (warming) {
            const float done = (float)(step + 1) / (float)warmup_;    // first step already gets 1/warmup
            return peak_ * done;
        }
        const int span = horizon_ - warmup_;
        if (kind_ != LRScheduleType::Cosine || span <= 0) return peak_;
        const int into = step - warmup_;
        if (into >= span) return floor_;
        const float phase = (float)M_PI * (float)into / (float)span;
        const float weight = 0.5f * (1.0f + cosf(phase));
        return floor_ + (peak_ - floor_) * weight;
    }

private:
    LRScheduleType kind_ = LRScheduleType::Constant;
    float peak_ = 1e-5f;
    float floor_ = 0.0f;
    int warmup_ = 0;
    int horizon_ = 0;
};
