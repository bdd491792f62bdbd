// Operator API of the AdamW step for C++ callers: the reference's launch functions
// (include/kernels/adamw.cuh:24-57) with the same names, argument order and meaning,
// forwarding to the C ABI of librlx_adamw.so.  `bias_correctionK` is 1 - betaK^t, not its
// reciprocal; n <= 0 is a silent no-op.  The reference's launchers return void and check
// nothing; these abort with a message if the library reports an error, so that a bad call
// is never silent.
#pragma once
#include <hip/hip_fp16.h>
#include <hip/hip_runtime_api.h>

#include <cstdio>
#include <cstdlib>

#include "rlx_adamw.h"

#ifndef RLX_CHECK
#define RLX_CHECK(x)                                                                              \
    do {                                                                                          \
        int st_ = (x);                                                                            \
        if (st_ != RLX_OK) {                                                                      \
            fprintf(stderr, "rlx error %d (%s) %s at %s:%d\n", st_, rlx_status_string(st_),       \
                    rlx_last_hip_error(), __FILE__, __LINE__);                                    \
            exit(1);                                                                              \
        }                                                                                         \
    } while (0)
#endif

// FP16 weights with an FP32 master copy (master_w may be null: the FP16 weight is then the
// source of truth and the step moves 22 instead of 28 bytes per parameter).
inline void launch_adamw_fp16(float* master_w, half* model_w, const half* grad, float* m, float* v, int n,
                              float lr, float beta1, float beta2, float eps, float weight_decay,
                              float bias_correction1, float bias_correction2, hipStream_t stream = 0) {
    RLX_CHECK(rlx_adamw_fp16(master_w, reinterpret_cast<uint16_t*>(model_w),
                             reinterpret_cast<const uint16_t*>(grad), m, v, (int64_t)n, lr, beta1, beta2, eps,
                             weight_decay, bias_correction1, bias_correction2, (void*)stream));
}

// FP32 weights, in place.
inline void launch_adamw_fp32(float* w, const float* grad, float* m, float* v, int n,
                              float lr, float beta1, float beta2, float eps, float weight_decay,
                              float bias_correction1, float bias_correction2, hipStream_t stream = 0) {
    RLX_CHECK(rlx_adamw_fp32(w, grad, m, v, (int64_t)n, lr, beta1, beta2, eps, weight_decay, bias_correction1,
                             bias_correction2, (void*)stream));
}
