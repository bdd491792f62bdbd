// Learning-rate schedule feeding AdamWOptimizer::set_lr once per optimizer step.
//
// Two shapes, both with an optional linear warm-up: a constant rate, or a half-cosine that
// falls from the peak rate to a floor.  The class keeps the name, the three public methods and
// the exact FP32 arithmetic of the reference's scheduler (include/training/lr_scheduler.h:10-57),
// so that `optimizer_.set_lr(lr_scheduler_.get_lr(global_step))` (include/training/trainer.h:193-194)
// yields the same bits; the reference's own test (tests/test_lr_scheduler.cpp) compiles against
// this header and passes.
#pragma once
#include <cmath>

enum class LRScheduleType { Constant, Cosine };

namespace lr_detail {

// Rate during warm-up: step 0 already gets peak/warmup, step warmup-1 gets the peak.
inline float warmup_rate(float peak, int step, int warmup) {
    const float fraction = (float)(step + 1) / (float)warmup;
    return peak * fraction;
}

// Rate `into` steps into a cosine decay that lasts `span` steps.
inline float cosine_rate(float peak, float floor, int into, int span) {
    const float angle = (float)M_PI * (float)into / (float)span;
    const float blend = 0.5f * (1.0f + cosf(angle));
    return floor + (peak - floor) * blend;
}

}  // namespace lr_detail

class LRScheduler {
public:
    LRScheduler() = default;

    void init_constant(float base_lr, int warmup_steps = 0) {
        configure(LRScheduleType::Constant, base_lr, base_lr, warmup_steps, 0);
    }

    void init_cosine(float base_lr, float min_lr, int warmup_steps, int total_steps) {
        configure(LRScheduleType::Cosine, base_lr, min_lr, warmup_steps, total_steps);
    }

    // Rate for the optimizer step with 0-based index `step`.
    float get_lr(int step) const {
        if (in_warmup(step)) return lr_detail::warmup_rate(peak_, step, warmup_);
        const int span = horizon_ - warmup_;                 // length of the decay
        const bool decays = shape_ == LRScheduleType::Cosine && span > 0;
        if (!decays) return peak_;
        const int into = step - warmup_;
        return into < span ? lr_detail::cosine_rate(peak_, floor_, into, span) : floor_;
    }

    bool in_warmup(int step) const { return warmup_ > 0 && step < warmup_; }
    LRScheduleType type() const { return shape_; }

private:
    void configure(LRScheduleType shape, float peak, float floor, int warmup, int horizon) {
        shape_ = shape;
        peak_ = peak;
        floor_ = floor;
        warmup_ = warmup;
        horizon_ = horizon;
    }

    LRScheduleType shape_ = LRScheduleType::Constant;
    float peak_ = 1e-5f;      // rate after warm-up
    float floor_ = 0.0f;      // rate at and after `horizon_` (cosine only)
    int warmup_ = 0;          // warm-up steps
    int horizon_ = 0;         // step at which the cosine reaches the floor
};
