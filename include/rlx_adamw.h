/*
 * rlx_adamw.h — C ABI of the MI355X (gfx950) AdamW + gradient-norm/clip library.
 *
 * Plain pointers and sizes only; every pointer named "device" is HIP device memory,
 * `stream` is a hipStream_t passed as void* (NULL = the default stream).  All work is
 * stream-ordered and asynchronous unless a function says that it synchronises.  Every
 * function returns an rlx_status; nothing here exits the process.  FP16 values are
 * passed as uint16_t bit patterns (IEEE binary16).
 *
 * Each entry point names the reference interface (path inside the reference tree) that
 * it replaces.
 */
#ifndef RLX_ADAMW_H
#define RLX_ADAMW_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef enum {
    RLX_OK = 0,
    RLX_ERR_INVALID_ARG = 1,      /* null pointer, negative size, bad enum, bad plan */
    RLX_ERR_MISALIGNED = 2,       /* pointer not aligned to its element size */
    RLX_ERR_BAD_HYPER = 3,        /* bias correction of 0, or a non-finite hyper-parameter */
    RLX_ERR_HIP = 4,              /* a HIP runtime call failed; see rlx_last_hip_error() */
    RLX_ERR_NO_DEVICE = 5,
    RLX_ERR_TOO_LARGE = 6,        /* more chunks than one plan can address, or than rlx_grad_norm_static holds */
    RLX_ERR_NO_MEMORY = 7,        /* host allocation failed */
    RLX_ERR_WRONG_DEVICE = 8      /* the plan was made with another device current */
} rlx_status;

const char* rlx_status_string(int status);
/* Text of the last HIP error seen by this thread ("" if none). */
const char* rlx_last_hip_error(void);
/* ABI version of the loaded library (major*100 + minor). */
int rlx_version(void);

/* ------------------------------------------------------------------------------------
 * Operator API: one flat tensor per call.
 * ---------------------------------------------------------------------------------- */

/*
 * Replaces launch_adamw_fp16 (include/kernels/adamw.cuh:24-39, src/kernels/adamw.cu:42-58).
 * Same argument order and meaning: bias_correctionK = 1 - betaK^t (not the reciprocal);
 * n <= 0 is a no-op that returns RLX_OK.  n is 64-bit.
 * master_w may be NULL: the FP16 weight is then read as the source of truth
 * (22 bytes per parameter instead of 28).  With a master copy model_w is write-only,
 * as in the reference.
 */
int rlx_adamw_fp16(float* master_w, uint16_t* model_w, const uint16_t* grad,
                   float* m, float* v, int64_t n,
                   float lr, float beta1, float beta2, float eps, float weight_decay,
                   float bias_correction1, float bias_correction2, void* stream);

/* Replaces launch_adamw_fp32 (include/kernels/adamw.cuh:43-57, src/kernels/adamw.cu:93-108). */
int rlx_adamw_fp32(float* w, const float* grad, float* m, float* v, int64_t n,
                   float lr, float beta1, float beta2, float eps, float weight_decay,
                   float bias_correction1, float bias_correction2, void* stream);

/* Replaces fp16_to_fp32 (include/training/optimizer.h:46-57): dst[i] = (float)src[i]. */
int rlx_fp16_to_fp32(float* dst, const uint16_t* src, int64_t n, void* stream);

/*
 * x[i] *= scale over a plain FP32 buffer: replaces scale_grad_kernel (include/training/trainer.h:93-99),
 * with which training_step divides each micro-batch's loss gradient by grad_accum_steps before the
 * backward pass adds it into the gradient pools (trainer.h:261-263).
 */
int rlx_scale_f32(float* x, float scale, int64_t n, void* stream);

/*
 * Zero fill of nbytes at dst, any alignment, as kernels: replaces the two cudaMemsetAsync of
 * qwen3_gradients_zero (src/model/qwen3.cu:1109-1112) and the memset of the frozen embedding's
 * gradients (include/training/trainer.h:271-277) where the caller records its step into a HIP
 * graph (memset nodes are avoided there) or wants the same stream-ordered call either way.
 * nbytes <= 0 is a no-op.  (rlx_plan_adamw with RLX_STEP_ZERO_GRADS makes it unnecessary for
 * the gradient pools.)
 */
int rlx_clear(void* dst, int64_t nbytes, void* stream);

/* ------------------------------------------------------------------------------------
 * Multi-tensor plan: a whole model's tensors in one launch.
 * ---------------------------------------------------------------------------------- */

enum { RLX_DTYPE_F16 = 0, RLX_DTYPE_F32 = 1 };

enum {
    RLX_TENSOR_NO_DECAY  = 1,   /* weight_decay is 0 for this tensor (embedding and norm
                                   groups, include/training/optimizer.h:131-146) */
    RLX_TENSOR_GRAD_ONLY = 2,   /* no parameter: the buffer only takes part in the norm and
                                   in the scale pass (the D_buf tail of the reference's
                                   float_pool, include/training/trainer.h:330-337) */
    RLX_TENSOR_FROZEN    = 4    /* the tensor's gradient counts as zero: it is neither read by
                                   the norm nor scaled, and the update leaves p, m, v alone.
                                   Equals what the reference does for a frozen embedding
                                   (gradients cleared before the clip, then an identity
                                   update; include/training/trainer.h:269-277,
                                   optimizer.h:131-140) as long as the tensor's moments are
                                   zero and it has no weight decay. */
};

typedef struct rlx_tensor_desc {
    void*       param;    /* device; FP16 or FP32 weights [n]; NULL iff GRAD_ONLY */
    void*       grad;     /* device; same dtype as param [n]; written only by rlx_plan_scale_grads */
    float*      m;        /* device; first moment [n] */
    float*      v;        /* device; second moment [n] */
    float*      master;   /* device; FP32 master weights [n] or NULL (FP16 tensors only) */
    int64_t     n;        /* elements, > 0 */
    int32_t     dtype;    /* RLX_DTYPE_* */
    uint32_t    flags;    /* RLX_TENSOR_* */
} rlx_tensor_desc;

/* Hyper-parameters of one step; the same seven floats that launch_adamw_* take. */
typedef struct rlx_step_params {
    float lr, beta1, beta2, eps, weight_decay;
    float bias_correction1, bias_correction2;   /* 1 - beta^t */
} rlx_step_params;

typedef struct rlx_plan rlx_plan;

/*
 * Builds the device-resident work table for `count` tensors (the role that
 * AdamWOptimizer::init's offset bookkeeping has, include/training/optimizer.h:188-243).
 * Tensors are cut into chunks of `chunk_elems` elements (0 = chosen from the mean tensor
 * size: 8192, 2048 or 512, and up to 65536 for lists of billions of elements; otherwise a
 * power of two >= 512); the table order is the order of `descs`, which also fixes the order
 * of the norm reduction.  The plan borrows every pointer in `descs` and owns only
 * its tables and the reduction workspace.  Allocates; call outside the step loop.
 */
int rlx_plan_create(const rlx_tensor_desc* descs, int64_t count, int64_t chunk_elems, rlx_plan** out);
/*
 * The chunking that rlx_plan_create would use for these arguments, computed on the host without
 * touching a device: the chunk size (the chosen one if chunk_elems is 0), the number of chunks
 * (= device records = FP64 partials of the norm) and the number of elements.  Any out pointer may
 * be NULL.  Same argument checks and status codes as rlx_plan_create.  No counterpart in the
 * reference, whose launches are sized from flat pool lengths (include/training/optimizer.h:124-146).
 */
int rlx_plan_layout(const rlx_tensor_desc* descs, int64_t count, int64_t chunk_elems, int64_t* out_chunk_elems,
                    int64_t* out_num_chunks, int64_t* out_num_elements);
int rlx_plan_destroy(rlx_plan* plan);
int64_t rlx_plan_num_chunks(const rlx_plan* plan);
int64_t rlx_plan_num_elements(const rlx_plan* plan);
int64_t rlx_plan_chunk_elems(const rlx_plan* plan);

/*
 * Global gradient L2 norm and clip scale, entirely on the device:
 * replaces the reduce half of Trainer::clip_grad_norm_ (include/training/trainer.h:323-345,
 * sum_sq_half_kernel / sum_sq_float_kernel :103-133).  No value is ever added by an atomic:
 * one FP64 partial per chunk in table order (for plans with 512-element chunks, 16 consecutive
 * partials are then added, in order, into one group partial), then one workgroup adds these
 * in a fixed order, so that the result is the same bits on every run.  That last sum is a
 * second launch, or, for launches of up to 256 workgroups, the tail of the first one: the
 * workgroup that finishes last (found by counting tickets, which decides who adds but not in
 * which order) does it.  Both forms give the same bits ("norm_fused" below chooses).  Partials and tickets live
 * in the plan: norm launches of ONE plan must not overlap (two streams, two threads); launches that do spoil each
 * other's result, not those of later launches (the ticket counters only count up and need no reset).  Writes
 * {sum_sq, norm = sqrtf((float)sum_sq), scale} to the plan's device result, where
 * scale = max_norm / (norm + 1e-6f) iff norm > max_norm, else 1.0f (a NaN norm gives
 * 1.0f, as the reference's comparison does; max_norm = INFINITY measures without clipping).
 * No host synchronisation.  The plan must be used with the device current that it was
 * created on (RLX_ERR_WRONG_DEVICE otherwise; the same holds for every launch below).
 */
int rlx_plan_grad_norm(rlx_plan* plan, float max_norm, void* stream);

/*
 * Copies the last result of rlx_plan_grad_norm to the host and waits for it (the
 * blocking 4-byte copy of include/training/trainer.h:339-341).  Any out pointer may be NULL.
 */
int rlx_plan_norm_read(rlx_plan* plan, float* norm, float* scale, double* sum_sq, void* stream);

/* Device address of the result {double sum_sq; float norm; float scale;} (16 bytes). */
const void* rlx_plan_norm_device_ptr(const rlx_plan* plan);
/* Device address of the per-chunk FP64 partials (rlx_plan_num_chunks values); plans with 512-element chunks
 * keep one group partial per 16 chunks directly behind them. */
const double* rlx_plan_partials_device_ptr(const rlx_plan* plan);

/*
 * The same two-pass norm and clip rule over two flat gradient buffers (an FP16 one, then an FP32 one: the
 * shape of half_pool / float_pool) without a plan and without allocating anything.  It has no counterpart
 * in the reference; it is for callers that cannot allocate: code under HIP graph capture, tight serving
 * loops, harnesses that forbid hipMalloc.  The FP64 partials go to a 2.1 MiB array that is part of
 * the library's device image (every GPU the library runs on holds it until the process ends), so at most
 * 262,144 chunks fit: more returns RLX_ERR_TOO_LARGE (chunk_elems = 0 chooses the chunk as rlx_plan_create
 * would for these two tensors, which covers about 17e9 elements; otherwise a power of two >= 512).
 * Writes {double sum_sq; float norm; float scale;} (16 bytes, 8-byte aligned, device) to result_dev: the same
 * bits as rlx_plan_grad_norm leaves for a plan over these two tensors in this order with the same chunk size.
 * Either buffer may be empty (n = 0).  Calls no hipMalloc, hipFree or other allocating routine; the first call
 * on a device looks up the array's address there (make that call outside a graph capture).  All calls on one
 * GPU share the array: calls that overlap on one GPU (two streams, two threads) race; calls on one stream
 * do not.  Nothing in the array has to start at zero: every call writes each slot that it later reads (this
 * entry point always adds the partials in a second launch, whatever "norm_fused" says: the one-launch form keeps
 * counters that are only valid from call to call while the number of workgroups stays the same, and calls of any
 * size share this array).
 */
int rlx_grad_norm_static(const uint16_t* half_grads, int64_t n_half, const float* float_grads, int64_t n_float,
                         int64_t chunk_elems, float max_norm, void* result_dev, void* stream);

/*
 * In-place scale of all gradients by the device-resident clip scale: replaces
 * scale_half_kernel / scale_float_kernel (include/training/trainer.h:136-145,346-349).
 * FP16 gradients are re-rounded to FP16.  A scale of exactly 1.0f leaves every bit alone.
 */
int rlx_plan_scale_grads(rlx_plan* plan, void* stream);

/*
 * One AdamW step over every tensor of the plan in a single launch: replaces the three
 * launches of AdamWOptimizer::step (include/training/optimizer.h:124-146).
 * step_flags, any combination of:
 *   RLX_CLIP_FUSED       the scale left by rlx_plan_grad_norm on the device is applied to each
 *                        gradient in registers (FP16 gradients re-rounded to FP16 first, exactly
 *                        as rlx_plan_scale_grads would have stored them); without
 *                        RLX_STEP_ZERO_GRADS the gradient buffers are not written.
 *   RLX_STEP_ZERO_GRADS  every gradient buffer of the plan (grad-only and frozen ones too) is
 *                        cleared after it has been read: replaces the two memsets of
 *                        qwen3_gradients_zero at the start of the next step
 *                        (src/model/qwen3.cu:1109-1112, include/training/trainer.h:242).
 * 0 (RLX_CLIP_NONE) uses the gradients as stored and leaves them alone.
 */
enum { RLX_CLIP_NONE = 0, RLX_CLIP_FUSED = 1, RLX_STEP_ZERO_GRADS = 2 };
int rlx_plan_adamw(rlx_plan* plan, const rlx_step_params* params, int step_flags, void* stream);

/*
 * The same step with the hyper-parameters read from device memory at run time (28 bytes,
 * 4-byte aligned), so that a recorded launch (HIP graph) can be replayed with a new learning
 * rate and new bias corrections: the host only rewrites *dev_params between replays.  No
 * counterpart in the reference, whose step takes them by value (optimizer.h:119-147).
 * The values are not validated.
 */
int rlx_plan_adamw_dev(rlx_plan* plan, const rlx_step_params* dev_params, int step_flags, void* stream);

/*
 * Steps that need no host at all (a recorded norm + update replayed step after step): the host uploads, once, the
 * hyper-parameters of the next n_steps steps (learning rates from its scheduler, bias corrections
 * 1 - powf(beta, t) computed where the reference computes them, include/training/optimizer.h:120-122, so the
 * values are bit-equal), and every rlx_plan_adamw_scheduled launch reads the current entry from device memory
 * and then moves on to the next one with a one-lane kernel.  No counterpart in the reference, whose step takes
 * the values from the host each time (optimizer.h:119-147).
 *
 * rlx_plan_schedule_upload: every entry is validated like the arguments of rlx_plan_adamw (finite, bias
 * corrections not 0: RLX_ERR_BAD_HYPER otherwise, nothing uploaded).  Waits for the whole device
 * (hipDeviceSynchronize: scheduled updates of this plan that are still running, on `stream` or on any other
 * stream, replays of a recorded step included, read the old table), allocates when the table grows and copies
 * synchronously: call it outside the step loop and outside a graph capture.  `stream` is not otherwise used.
 * The next scheduled update reads entry 0.
 * A recorded rlx_plan_adamw_scheduled stays valid across uploads, of any length: the launch names only a small
 * header whose device address is fixed from the first upload until rlx_plan_destroy; the table's address and
 * length are read from that header when the kernel runs.  Record the step once, after the first upload, and
 * replay it through every later window.
 * rlx_plan_adamw_scheduled: the update of rlx_plan_adamw_dev with the current entry, then the advance.  After
 * the last entry has been used, that entry stays current (upload the next window before that happens);
 * updates that run with it again are counted (rlx_plan_schedule_overrun).
 * rlx_plan_schedule_position: how many scheduled steps have run since the upload (saturating at n_steps) and
 * the table's length; waits for `stream`.  Either out pointer may be NULL.
 * rlx_plan_schedule_overrun: how many scheduled updates since the upload ran after the table had been used up,
 * i.e. with the last entry's learning rate and bias corrections instead of their own (0 in a correct run);
 * waits for `stream`.
 */
int rlx_plan_schedule_upload(rlx_plan* plan, const rlx_step_params* steps, int64_t n_steps, void* stream);
int rlx_plan_adamw_scheduled(rlx_plan* plan, int step_flags, void* stream);
int rlx_plan_schedule_position(rlx_plan* plan, int64_t* steps_taken, int64_t* n_steps, void* stream);
int rlx_plan_schedule_overrun(rlx_plan* plan, int64_t* overrun, void* stream);

/* ------------------------------------------------------------------------------------
 * Launch tuning (process-wide; for measurement).  Unknown keys return RLX_ERR_INVALID_ARG.
 *   "update_variant"  0..N-1   which compiled form of the update kernel: tile shape, XCD swizzle,
 *                              store policy, loads and stores at once or two at a time (0 = default,
 *                              which picks between the last two by what the step writes); 10 = 128-bit
 *                              accesses (8 elements per lane), 11 = that in a persistent grid sized to the
 *                              CUs striding over the tiles, 12 = that with one workgroup walking a chunk
 *                              (10-12 with ordinary loads and stores; 13, 14 = 12, 11 with the shipped
 *                              kernel's non-temporal loads and system-scope non-temporal stores);
 *                              15, 16 = the shipped accesses with two / four 256-element sub-tiles per workgroup;
 *                              17 = the shipped tile with lane pairs sharing 128-bit accesses
 *   "norm_grid"       0 = one workgroup per chunk, >0 = that many persistent workgroups
 *   "norm_nt"         1 = non-temporal loads in the norm pass (default), 0 = plain
 *   "norm_pack"       512-element chunks per workgroup in the norm pass: 0 = one, 1 = eight (one per
 *                     wavefront), 2 = thirty-two (four per wavefront), 3 = sixteen (two per wavefront, default)
 *   "final_batch"     loads that a lane of the norm's second pass keeps in flight: 8, 16, 32, 40, or
 *                     0 = chosen from the number of partials (default)
 *   "norm_fused"      who adds the norm's partials: 0 = always a second launch of one workgroup; 1 = the
 *                     workgroup of the first launch that finishes last, whenever that launch has at most
 *                     8,192 workgroups; 2 = that for launches of up to 256 workgroups (default; beyond one
 *                     wave of workgroups the tickets cost more than the second launch).  Same bits.
 *   "norm_keep_mb"    > 0: the norm walks its chunks from the last to the first and reads the first that many
 *                     MB of gradients (the last it reads) with ordinary instead of non-temporal loads, so that
 *                     they are still in the last-level cache when the update starts; 0 = off (default).  Same bits.
 *   "update_reverse"  1 = the fused-clip update walks its tiles from the end of the table to its start (to meet
 *                     what a forward norm read last); 0 = off (default).  Same bits.
 *   "convert_variant" rlx_fp16_to_fp32: 0 = 128 lanes x 4 elements per workgroup (default),
 *                     1 = 128 lanes x 2 elements, 2 = one element per lane, grid-stride,
 *                     3 = 256 lanes x 4 elements x 2 rounds
 * ---------------------------------------------------------------------------------- */
int rlx_set_tuning(const char* key, int64_t value);
int64_t rlx_get_tuning(const char* key);
/* Name of the kernel instantiation behind an "update_variant" number ("" if out of range). */
const char* rlx_update_variant_name(int64_t variant);

/* ------------------------------------------------------------------------------------
 * Seeded synthetic inputs, generated on the device (no counterpart in the reference,
 * whose gradients come from its backward pass).  value(i) = mean + std * z(seed, first+i)
 * with z an integer-hash approximation of N(0,1); rows of row_len elements whose row
 * hash is below zero_rows_below / 2^32 are zero.  flags: 1 = use |z|.
 * ---------------------------------------------------------------------------------- */
int rlx_fill_f16(uint16_t* dst, int64_t n, uint64_t seed, int64_t first, float mean, float std,
                 uint32_t flags, int64_t row_len, uint32_t zero_rows_below, void* stream);
int rlx_fill_f32(float* dst, int64_t n, uint64_t seed, int64_t first, float mean, float std,
                 uint32_t flags, int64_t row_len, uint32_t zero_rows_below, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* RLX_ADAMW_H */
