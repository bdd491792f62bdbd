// MI355X (gfx950) AdamW step, deterministic gradient norm and clip: HIP kernels and the
// C ABI declared in include/rlx_adamw.h.
//
// Every kernel here is a pure stream over HBM: no LDS except for the cross-wave step of
// the norm reduction, no matrix cores.  A "chunk" is `chunk_elems` consecutive elements
// of one tensor; a workgroup of 256 lanes (four 64-lane wavefronts) handles one chunk at
// a time.  Inside a chunk lane t owns the 8-element groups t, t+256, t+512, ...: an FP16
// group is one 128-bit access, an FP32 group two.
//
// Arithmetic follows src/kernels/adamw.cu:25-39 of the reference operation by operation
// and is compiled without FMA contraction, with IEEE division and square root and with
// FP32 denormals kept, so that a CPU restatement built the same way agrees bit for bit.

#include <hip/hip_runtime.h>

#include <cmath>
#include <cstdint>
#include <cstdio>
#include <cstring>
#include <new>
#include <vector>

#include "rlx_adamw.h"

namespace {

constexpr int kBlock = 256;                   // lanes per workgroup
constexpr int kVec = 8;                       // elements per lane per group
constexpr int kGroup = kBlock * kVec;         // 2048 elements per workgroup-wide group
constexpr int64_t kDefaultChunk = 8192;
constexpr int kFinalBlock = 1024;

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef float f32x4 __attribute__((ext_vector_type(4)));

struct DevTensor {
    void* p;
    void* g;
    float* m;
    float* v;
    float* master;
    int64_t n;
    int32_t dtype;
    uint32_t flags;      // RLX_TENSOR_* | kAligned
    int64_t pad;
};
static_assert(sizeof(DevTensor) == 64, "DevTensor is one 64-byte record");
constexpr uint32_t kAligned = 0x100;          // every pointer of the tensor is 16-byte aligned

struct DevChunk {
    int32_t tensor;
    int32_t index;       // chunk number inside the tensor
};

struct NormResult {
    double sum_sq;
    float norm;
    float scale;
};

struct Hyper {
    float lr, beta1, beta2, eps, weight_decay, bc1_inv, bc2_inv;
};

// ---------------------------------------------------------------------------------------
// Small device helpers
// ---------------------------------------------------------------------------------------

__device__ __forceinline__ float h2f(uint32_t bits16) {
    return (float)__builtin_bit_cast(_Float16, (uint16_t)bits16);
}

__device__ __forceinline__ uint32_t f2h(float x) {
    return (uint32_t)__builtin_bit_cast(uint16_t, (_Float16)x);     // round to nearest even
}

// Every buffer handed to this library is HIP device memory, so all vector accesses go
// through global-address-space pointers (global_load/global_store rather than flat).
#define RLX_GLOBAL __attribute__((address_space(1)))

template <bool NT, typename T>
__device__ __forceinline__ T ldg(const T* p) {
    const RLX_GLOBAL T* gp = (const RLX_GLOBAL T*)p;
    if constexpr (NT) return __builtin_nontemporal_load(gp);
    else return *gp;
}

template <bool NT, typename T>
__device__ __forceinline__ void stg(T* p, T x) {
    RLX_GLOBAL T* gp = (RLX_GLOBAL T*)p;
    if constexpr (NT) __builtin_nontemporal_store(x, gp);
    else *gp = x;
}

// One element of the update, in the reference's operation order (adamw.cu:25-36).
__device__ __forceinline__ void adamw_elem(float g, float& m, float& v, float& w, const Hyper& h, float wd) {
    float mi = h.beta1 * m + (1.0f - h.beta1) * g;
    float vi = h.beta2 * v + (1.0f - h.beta2) * g * g;
    m = mi;
    v = vi;
    float m_hat = mi * h.bc1_inv;
    float v_hat = vi * h.bc2_inv;
    w = w * (1.0f - h.lr * wd) - h.lr * m_hat / (__builtin_sqrtf(v_hat) + h.eps);
}

// Clip as a preceding scale pass would have stored it (trainer.h:136-139): re-round to FP16.
__device__ __forceinline__ float clip_f16(float g, float scale) { return h2f(f2h(g * scale)); }

struct Group16 {          // eight FP16 parameters with their state, in registers
    u32x4 p, g;
    f32x4 m0, m1, v0, v1, w0, w1;
};

template <bool NT>
__device__ __forceinline__ void load_group16(Group16& r, const DevTensor& t, int64_t elem, bool has_master) {
    r.g = ldg<NT>((const u32x4*)((const uint16_t*)t.g + elem));
    r.m0 = ldg<NT>((const f32x4*)(t.m + elem));
    r.m1 = ldg<NT>((const f32x4*)(t.m + elem) + 1);
    r.v0 = ldg<NT>((const f32x4*)(t.v + elem));
    r.v1 = ldg<NT>((const f32x4*)(t.v + elem) + 1);
    if (has_master) {
        r.w0 = ldg<NT>((const f32x4*)(t.master + elem));
        r.w1 = ldg<NT>((const f32x4*)(t.master + elem) + 1);
    } else {
        r.p = ldg<NT>((const u32x4*)((const uint16_t*)t.p + elem));
    }
}

template <bool NT>
__device__ __forceinline__ void finish_group16(Group16& r, const DevTensor& t, int64_t elem, bool has_master,
                                               const Hyper& h, float wd, float scale, bool clip) {
    float g[8], m[8], v[8], w[8];
#pragma unroll
    for (int k = 0; k < 4; k++) {
        g[2 * k] = h2f(r.g[k] & 0xFFFFu);
        g[2 * k + 1] = h2f(r.g[k] >> 16);
        m[k] = r.m0[k]; m[4 + k] = r.m1[k];
        v[k] = r.v0[k]; v[4 + k] = r.v1[k];
    }
    if (has_master) {
#pragma unroll
        for (int k = 0; k < 4; k++) { w[k] = r.w0[k]; w[4 + k] = r.w1[k]; }
    } else {
#pragma unroll
        for (int k = 0; k < 4; k++) { w[2 * k] = h2f(r.p[k] & 0xFFFFu); w[2 * k + 1] = h2f(r.p[k] >> 16); }
    }
    if (clip) {
#pragma unroll
        for (int k = 0; k < 8; k++) g[k] = clip_f16(g[k], scale);
    }
#pragma unroll
    for (int k = 0; k < 8; k++) adamw_elem(g[k], m[k], v[k], w[k], h, wd);
    f32x4 a, b;
#pragma unroll
    for (int k = 0; k < 4; k++) { a[k] = m[k]; b[k] = m[4 + k]; }
    stg<NT>((f32x4*)(t.m + elem), a);
    stg<NT>((f32x4*)(t.m + elem) + 1, b);
#pragma unroll
    for (int k = 0; k < 4; k++) { a[k] = v[k]; b[k] = v[4 + k]; }
    stg<NT>((f32x4*)(t.v + elem), a);
    stg<NT>((f32x4*)(t.v + elem) + 1, b);
    if (has_master) {
#pragma unroll
        for (int k = 0; k < 4; k++) { a[k] = w[k]; b[k] = w[4 + k]; }
        stg<NT>((f32x4*)(t.master + elem), a);
        stg<NT>((f32x4*)(t.master + elem) + 1, b);
    }
    u32x4 out;
#pragma unroll
    for (int k = 0; k < 4; k++) out[k] = f2h(w[2 * k]) | (f2h(w[2 * k + 1]) << 16);
    stg<NT>((u32x4*)((uint16_t*)t.p + elem), out);
}

// Scalar path: unaligned tensors and the last, partial group of a tensor.
__device__ __forceinline__ void update_scalar16(const DevTensor& t, int64_t i, const Hyper& h, float wd,
                                                float scale, bool clip) {
    uint16_t* p = (uint16_t*)t.p;
    float g = h2f(((const uint16_t*)t.g)[i]);
    if (clip) g = clip_f16(g, scale);
    float m = t.m[i], v = t.v[i];
    float w = t.master ? t.master[i] : h2f(p[i]);
    adamw_elem(g, m, v, w, h, wd);
    t.m[i] = m;
    t.v[i] = v;
    if (t.master) t.master[i] = w;
    p[i] = (uint16_t)f2h(w);
}

__device__ __forceinline__ void update_scalar32(const DevTensor& t, int64_t i, const Hyper& h, float wd,
                                                float scale, bool clip) {
    float* p = (float*)t.p;
    float g = ((const float*)t.g)[i];
    if (clip) g = g * scale;                    // scale_float_kernel, trainer.h:142-145
    float m = t.m[i], v = t.v[i], w = p[i];
    adamw_elem(g, m, v, w, h, wd);
    t.m[i] = m;
    t.v[i] = v;
    p[i] = w;
}

// Eight FP32 parameters (norm weights): the same update, in place (adamw.cu:80-90).
template <bool NT>
__device__ __forceinline__ void update_group32(const DevTensor& t, int64_t elem, const Hyper& h, float wd,
                                               float scale, bool clip) {
    f32x4 pw[2], gw[2], mw[2], vw[2];
#pragma unroll
    for (int q = 0; q < 2; q++) {
        pw[q] = ldg<NT>((const f32x4*)((const float*)t.p + elem) + q);
        gw[q] = ldg<NT>((const f32x4*)((const float*)t.g + elem) + q);
        mw[q] = ldg<NT>((const f32x4*)(t.m + elem) + q);
        vw[q] = ldg<NT>((const f32x4*)(t.v + elem) + q);
    }
#pragma unroll
    for (int q = 0; q < 2; q++) {
#pragma unroll
        for (int k = 0; k < 4; k++) {
            float g = gw[q][k];
            if (clip) g = g * scale;
            float m = mw[q][k], v = vw[q][k], w = pw[q][k];
            adamw_elem(g, m, v, w, h, wd);
            mw[q][k] = m; vw[q][k] = v; pw[q][k] = w;
        }
        stg<NT>((f32x4*)(t.m + elem) + q, mw[q]);
        stg<NT>((f32x4*)(t.v + elem) + q, vw[q]);
        stg<NT>((f32x4*)((float*)t.p + elem) + q, pw[q]);
    }
}

// ---------------------------------------------------------------------------------------
// Update kernel.  U = groups per lane whose loads are all issued before the first use.
// SINGLE: one tensor passed by value (the operator API); otherwise the plan's tables.
// ---------------------------------------------------------------------------------------

template <int U, bool NT, bool SINGLE>
__global__ __launch_bounds__(kBlock) void adamw_update_kernel(
    const DevTensor* __restrict__ tensors, const DevChunk* __restrict__ chunks, DevTensor single,
    int64_t n_chunks, int64_t chunk_elems, Hyper h, const NormResult* __restrict__ norm)
{
    const int tid = threadIdx.x;
    const bool clip = norm != nullptr;
    const float scale = clip ? norm->scale : 1.0f;

    for (int64_t c = blockIdx.x; c < n_chunks; c += gridDim.x) {
        DevTensor t;
        int64_t start;
        if constexpr (SINGLE) {
            t = single;
            start = c * chunk_elems;
        } else {
            DevChunk ch = chunks[c];
            t = tensors[ch.tensor];
            start = (int64_t)ch.index * chunk_elems;
        }
        if (t.flags & RLX_TENSOR_GRAD_ONLY) continue;
        const float wd = (t.flags & RLX_TENSOR_NO_DECAY) ? 0.0f : h.weight_decay;
        const int64_t left = t.n - start;
        const int64_t count = left < chunk_elems ? left : chunk_elems;
        const bool aligned = (t.flags & kAligned) != 0;

        if (!aligned) {
            for (int64_t i = start + tid; i < start + count; i += kBlock) {
                if (t.dtype == RLX_DTYPE_F16) update_scalar16(t, i, h, wd, scale, clip);
                else update_scalar32(t, i, h, wd, scale, clip);
            }
            continue;
        }

        if (t.dtype == RLX_DTYPE_F16) {
            const bool has_master = t.master != nullptr;
            int64_t done = 0;
            // full tiles of U groups: every load of the tile is in flight before any use
            for (; done + (int64_t)U * kGroup <= count; done += (int64_t)U * kGroup) {
                Group16 r[U];
#pragma unroll
                for (int j = 0; j < U; j++)
                    load_group16<NT>(r[j], t, start + done + (int64_t)(j * kBlock + tid) * kVec, has_master);
#pragma unroll
                for (int j = 0; j < U; j++)
                    finish_group16<NT>(r[j], t, start + done + (int64_t)(j * kBlock + tid) * kVec, has_master,
                                       h, wd, scale, clip);
            }
            // remaining whole groups, then the last partial group element by element
            for (; done < count; done += kGroup) {
                const int64_t off = done + (int64_t)tid * kVec;
                if (off + kVec <= count) {
                    Group16 r;
                    load_group16<NT>(r, t, start + off, has_master);
                    finish_group16<NT>(r, t, start + off, has_master, h, wd, scale, clip);
                } else {
                    for (int64_t i = off; i < count; i++) update_scalar16(t, start + i, h, wd, scale, clip);
                }
            }
        } else {
            for (int64_t done = 0; done < count; done += kGroup) {
                const int64_t off = done + (int64_t)tid * kVec;
                if (off + kVec <= count) {
                    update_group32<NT>(t, start + off, h, wd, scale, clip);
                } else {
                    for (int64_t i = off; i < count; i++) update_scalar32(t, start + i, h, wd, scale, clip);
                }
            }
        }
    }
}

// ---------------------------------------------------------------------------------------
// Norm pass 1: one FP64 partial per chunk, written to the chunk's own slot.
// Order inside a chunk (restated on the CPU by the test oracle): lane t adds x*x of its
// groups t, t+256, ... element by element into one FP32 accumulator; the 64 lanes of a
// wavefront combine by xor butterfly with masks 32,16,8,4,2,1; the four wavefront sums
// go through LDS and are added in FP64 in wavefront order.
// ---------------------------------------------------------------------------------------

template <bool NT>
__global__ __launch_bounds__(kBlock) void sumsq_partials_kernel(
    const DevTensor* __restrict__ tensors, const DevChunk* __restrict__ chunks,
    int64_t n_chunks, int64_t chunk_elems, double* __restrict__ partials)
{
    __shared__ float wave_sum[kBlock / 64];
    const int tid = threadIdx.x;

    for (int64_t c = blockIdx.x; c < n_chunks; c += gridDim.x) {
        const DevChunk ch = chunks[c];
        const DevTensor t = tensors[ch.tensor];
        const int64_t start = (int64_t)ch.index * chunk_elems;
        const int64_t left = t.n - start;
        const int64_t count = left < chunk_elems ? left : chunk_elems;
        const bool aligned = (t.flags & kAligned) != 0;

        float acc = 0.0f;
        if (t.dtype == RLX_DTYPE_F16) {
            const uint16_t* g = (const uint16_t*)t.g + start;
            int64_t done = 0;
            if (aligned) {
                for (; done + 4 * (int64_t)kGroup <= count; done += 4 * (int64_t)kGroup) {
                    u32x4 r[4];
#pragma unroll
                    for (int j = 0; j < 4; j++)
                        r[j] = ldg<NT>((const u32x4*)(g + done + (int64_t)(j * kBlock + tid) * kVec));
#pragma unroll
                    for (int j = 0; j < 4; j++) {
#pragma unroll
                        for (int k = 0; k < 4; k++) {
                            float a = h2f(r[j][k] & 0xFFFFu), b = h2f(r[j][k] >> 16);
                            acc = acc + a * a;
                            acc = acc + b * b;
                        }
                    }
                }
            }
            for (; done < count; done += kGroup) {
                const int64_t off = done + (int64_t)tid * kVec;
                if (aligned && off + kVec <= count) {
                    u32x4 r = ldg<NT>((const u32x4*)(g + off));
#pragma unroll
                    for (int k = 0; k < 4; k++) {
                        float a = h2f(r[k] & 0xFFFFu), b = h2f(r[k] >> 16);
                        acc = acc + a * a;
                        acc = acc + b * b;
                    }
                } else {
                    for (int64_t i = off; i < off + kVec && i < count; i++) {
                        float a = h2f(g[i]);
                        acc = acc + a * a;
                    }
                }
            }
        } else {
            const float* g = (const float*)t.g + start;
            for (int64_t done = 0; done < count; done += kGroup) {
                const int64_t off = done + (int64_t)tid * kVec;
                if (aligned && off + kVec <= count) {
                    f32x4 r0 = ldg<NT>((const f32x4*)(g + off)), r1 = ldg<NT>((const f32x4*)(g + off) + 1);
#pragma unroll
                    for (int k = 0; k < 4; k++) acc = acc + r0[k] * r0[k];
#pragma unroll
                    for (int k = 0; k < 4; k++) acc = acc + r1[k] * r1[k];
                } else {
                    for (int64_t i = off; i < off + kVec && i < count; i++) acc = acc + g[i] * g[i];
                }
            }
        }

#pragma unroll
        for (int mask = 32; mask >= 1; mask >>= 1) acc = acc + __shfl_xor(acc, mask, 64);
        if ((tid & 63) == 0) wave_sum[tid >> 6] = acc;
        __syncthreads();
        if (tid == 0) {
            double total = 0.0;
#pragma unroll
            for (int w = 0; w < kBlock / 64; w++) total += (double)wave_sum[w];
            partials[c] = total;
        }
        __syncthreads();
    }
}

// Norm pass 2: one workgroup, fixed order.  Thread t adds partials t, t+1024, ... in FP64,
// then a halving tree through LDS.  Writes the sum, the norm and the clip scale
// (trainer.h:341-345: strict '>' and +1e-6f in the denominator).
__global__ __launch_bounds__(kFinalBlock) void sumsq_final_kernel(
    const double* __restrict__ partials, int64_t n_partials, float max_norm, NormResult* __restrict__ out)
{
    __shared__ double acc[kFinalBlock];
    const int tid = threadIdx.x;
    double a = 0.0;
    for (int64_t i = tid; i < n_partials; i += kFinalBlock) a += partials[i];
    acc[tid] = a;
    __syncthreads();
    for (int s = kFinalBlock / 2; s >= 1; s >>= 1) {
        if (tid < s) acc[tid] = acc[tid] + acc[tid + s];
        __syncthreads();
    }
    if (tid == 0) {
        const double sum_sq = acc[0];
        const float norm = __builtin_sqrtf((float)sum_sq);
        float scale = 1.0f;
        if (norm > max_norm) scale = max_norm / (norm + 1e-6f);
        out->sum_sq = sum_sq;
        out->norm = norm;
        out->scale = scale;
    }
}

// In-place scale of the gradients (trainer.h:136-145).  Exactly 1.0f: nothing is touched.
template <bool NT>
__global__ __launch_bounds__(kBlock) void scale_grads_kernel(
    const DevTensor* __restrict__ tensors, const DevChunk* __restrict__ chunks,
    int64_t n_chunks, int64_t chunk_elems, const NormResult* __restrict__ norm)
{
    const float scale = norm->scale;
    if (scale == 1.0f) return;
    const int tid = threadIdx.x;
    for (int64_t c = blockIdx.x; c < n_chunks; c += gridDim.x) {
        const DevChunk ch = chunks[c];
        const DevTensor t = tensors[ch.tensor];
        const int64_t start = (int64_t)ch.index * chunk_elems;
        const int64_t left = t.n - start;
        const int64_t count = left < chunk_elems ? left : chunk_elems;
        const bool aligned = (t.flags & kAligned) != 0;
        if (t.dtype == RLX_DTYPE_F16) {
            uint16_t* g = (uint16_t*)t.g + start;
            for (int64_t done = 0; done < count; done += kGroup) {
                const int64_t off = done + (int64_t)tid * kVec;
                if (aligned && off + kVec <= count) {
                    u32x4 r = ldg<NT>((const u32x4*)(g + off));
#pragma unroll
                    for (int k = 0; k < 4; k++)
                        r[k] = f2h(h2f(r[k] & 0xFFFFu) * scale) | (f2h(h2f(r[k] >> 16) * scale) << 16);
                    stg<NT>((u32x4*)(g + off), r);
                } else {
                    for (int64_t i = off; i < off + kVec && i < count; i++)
                        g[i] = (uint16_t)f2h(h2f(g[i]) * scale);
                }
            }
        } else {
            float* g = (float*)t.g + start;
            for (int64_t done = 0; done < count; done += kGroup) {
                const int64_t off = done + (int64_t)tid * kVec;
                for (int64_t i = off; i < off + kVec && i < count; i++) g[i] = g[i] * scale;
            }
        }
    }
}

__global__ __launch_bounds__(kBlock) void fp16_to_fp32_kernel(float* __restrict__ dst,
                                                              const uint16_t* __restrict__ src, int64_t n)
{
    for (int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x; i < n; i += (int64_t)gridDim.x * kBlock)
        dst[i] = h2f(src[i]);
}

// ---------------------------------------------------------------------------------------
// Seeded synthetic inputs: integer hash -> sum of eight 16-bit uniforms -> one FP32
// multiply and one FP32 add, so that a host restatement gives the same bits without libm.
// ---------------------------------------------------------------------------------------

__host__ __device__ inline uint64_t hash64(uint64_t seed, uint64_t idx) {
    uint64_t z = seed + idx * 0x9E3779B97F4A7C15ULL;
    z ^= z >> 30; z *= 0xBF58476D1CE4E5B9ULL;
    z ^= z >> 27; z *= 0x94D049BB133111EBULL;
    z ^= z >> 31;
    return z;
}

__device__ inline float fill_value(uint64_t seed, uint64_t i, float mean, float std, uint32_t flags,
                                   int64_t row_len, uint32_t zero_rows_below) {
    if (row_len > 0 && zero_rows_below) {
        const uint64_t row = i / (uint64_t)row_len;
        if ((uint32_t)(hash64(seed ^ 0xA5A5A5A55A5A5A5AULL, row) >> 32) < zero_rows_below) return 0.0f;
    }
    const uint64_t a = hash64(seed, 2 * i), b = hash64(seed, 2 * i + 1);
    uint32_t s = 0;
#pragma unroll
    for (int k = 0; k < 4; k++) {
        s += (uint32_t)((a >> (16 * k)) & 0xFFFFu);
        s += (uint32_t)((b >> (16 * k)) & 0xFFFFu);
    }
    float z = ((float)(int32_t)s - 262140.0f) * 0x1.3988e2p-16f;   // 1/sqrt(8*(65536^2-1)/12)
    if (flags & 1u) z = __builtin_fabsf(z);
    return mean + std * z;
}

template <typename T>
__global__ __launch_bounds__(kBlock) void fill_kernel(T* __restrict__ dst, int64_t n, uint64_t seed, int64_t first,
                                                      float mean, float std, uint32_t flags, int64_t row_len,
                                                      uint32_t zero_rows_below)
{
    for (int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x; i < n; i += (int64_t)gridDim.x * kBlock) {
        const float x = fill_value(seed, (uint64_t)(first + i), mean, std, flags, row_len, zero_rows_below);
        if constexpr (sizeof(T) == 2) dst[i] = (uint16_t)f2h(x);
        else dst[i] = x;
    }
}

// ---------------------------------------------------------------------------------------
// Host side
// ---------------------------------------------------------------------------------------

thread_local char g_hip_error[256] = "";

int hip_fail(hipError_t e, const char* what) {
    snprintf(g_hip_error, sizeof(g_hip_error), "%s: %s", what, hipGetErrorString(e));
    return RLX_ERR_HIP;
}

#define RLX_HIP(call)                                        \
    do {                                                     \
        hipError_t e_ = (call);                              \
        if (e_ != hipSuccess) return hip_fail(e_, #call);    \
    } while (0)

struct Tuning {
    int64_t update_variant = 0;
    int64_t update_grid = 0;
    int64_t norm_grid = 0;
    int64_t norm_nt = 0;
} g_tuning;

constexpr int64_t kMaxGrid = 1 << 22;     // grid * 256 lanes stays below 2^32

inline int64_t pick_grid(int64_t n_chunks, int64_t tuned) {
    int64_t g = tuned > 0 ? tuned : n_chunks;
    if (g > n_chunks) g = n_chunks;
    if (g > kMaxGrid) g = kMaxGrid;
    return g < 1 ? 1 : g;
}

inline bool is_aligned(const void* p, size_t a) { return ((uintptr_t)p & (a - 1)) == 0; }

int check_hyper(float lr, float beta1, float beta2, float eps, float wd, float bc1, float bc2) {
    const float all[] = {lr, beta1, beta2, eps, wd, bc1, bc2};
    for (float x : all)
        if (!std::isfinite(x)) return RLX_ERR_BAD_HYPER;
    if (bc1 == 0.0f || bc2 == 0.0f) return RLX_ERR_BAD_HYPER;
    return RLX_OK;
}

Hyper make_hyper(float lr, float beta1, float beta2, float eps, float wd, float bc1, float bc2) {
    Hyper h;
    h.lr = lr; h.beta1 = beta1; h.beta2 = beta2; h.eps = eps; h.weight_decay = wd;
    h.bc1_inv = 1.0f / bc1;       // host reciprocals, adamw.cu:52-53
    h.bc2_inv = 1.0f / bc2;
    return h;
}

// Fills the derived fields of a device record; returns a status for bad descriptors.
int make_dev_tensor(const rlx_tensor_desc& d, DevTensor& t) {
    if (d.n <= 0 || !d.grad) return RLX_ERR_INVALID_ARG;
    if (d.dtype != RLX_DTYPE_F16 && d.dtype != RLX_DTYPE_F32) return RLX_ERR_INVALID_ARG;
    if (d.flags & ~(uint32_t)(RLX_TENSOR_NO_DECAY | RLX_TENSOR_GRAD_ONLY)) return RLX_ERR_INVALID_ARG;
    const bool grad_only = (d.flags & RLX_TENSOR_GRAD_ONLY) != 0;
    if (!grad_only && (!d.param || !d.m || !d.v)) return RLX_ERR_INVALID_ARG;
    if (d.master && d.dtype != RLX_DTYPE_F16) return RLX_ERR_INVALID_ARG;
    const size_t es = d.dtype == RLX_DTYPE_F16 ? 2 : 4;
    if (!is_aligned(d.grad, es) || !is_aligned(d.param, es) || !is_aligned(d.m, 4) || !is_aligned(d.v, 4) ||
        !is_aligned(d.master, 4))
        return RLX_ERR_MISALIGNED;
    t.p = d.param; t.g = d.grad; t.m = d.m; t.v = d.v; t.master = d.master;
    t.n = d.n; t.dtype = d.dtype; t.flags = d.flags; t.pad = 0;
    if (is_aligned(d.grad, 16) && is_aligned(d.param, 16) && is_aligned(d.m, 16) && is_aligned(d.v, 16) &&
        is_aligned(d.master, 16))
        t.flags |= kAligned;
    return RLX_OK;
}

template <bool SINGLE>
int launch_update(const DevTensor* tensors, const DevChunk* chunks, const DevTensor& single, int64_t n_chunks,
                  int64_t chunk_elems, const Hyper& h, const NormResult* norm, hipStream_t s) {
    const dim3 grid((unsigned)pick_grid(n_chunks, g_tuning.update_grid)), block(kBlock);
    switch (g_tuning.update_variant) {
    default:
    case 0: adamw_update_kernel<4, false, SINGLE><<<grid, block, 0, s>>>(tensors, chunks, single, n_chunks, chunk_elems, h, norm); break;
    case 1: adamw_update_kernel<4, true, SINGLE><<<grid, block, 0, s>>>(tensors, chunks, single, n_chunks, chunk_elems, h, norm); break;
    case 2: adamw_update_kernel<2, false, SINGLE><<<grid, block, 0, s>>>(tensors, chunks, single, n_chunks, chunk_elems, h, norm); break;
    case 3: adamw_update_kernel<2, true, SINGLE><<<grid, block, 0, s>>>(tensors, chunks, single, n_chunks, chunk_elems, h, norm); break;
    case 4: adamw_update_kernel<1, false, SINGLE><<<grid, block, 0, s>>>(tensors, chunks, single, n_chunks, chunk_elems, h, norm); break;
    case 5: adamw_update_kernel<1, true, SINGLE><<<grid, block, 0, s>>>(tensors, chunks, single, n_chunks, chunk_elems, h, norm); break;
    }
    RLX_HIP(hipGetLastError());
    return RLX_OK;
}

int flat_update(void* p, const void* g, float* m, float* v, float* master, int64_t n, int dtype,
                float lr, float beta1, float beta2, float eps, float wd, float bc1, float bc2, void* stream) {
    if (n <= 0) return RLX_OK;                                   // adamw.cu:49,99
    rlx_tensor_desc d;
    d.param = p; d.grad = const_cast<void*>(g); d.m = m; d.v = v; d.master = master;
    d.n = n; d.dtype = dtype; d.flags = 0;
    if (!p || !g || !m || !v) return RLX_ERR_INVALID_ARG;
    int st = check_hyper(lr, beta1, beta2, eps, wd, bc1, bc2);
    if (st != RLX_OK) return st;
    DevTensor t;
    st = make_dev_tensor(d, t);
    if (st != RLX_OK) return st;
    const int64_t n_chunks = (n + kDefaultChunk - 1) / kDefaultChunk;
    return launch_update<true>(nullptr, nullptr, t, n_chunks, kDefaultChunk,
                               make_hyper(lr, beta1, beta2, eps, wd, bc1, bc2), nullptr, (hipStream_t)stream);
}

}  // namespace

struct rlx_plan {
    uint32_t magic;
    int device;
    int64_t n_tensors, n_chunks, n_elems, chunk_elems;
    DevTensor* d_tensors;
    DevChunk* d_chunks;
    double* d_partials;
    NormResult* d_norm;
    NormResult* h_norm;      // pinned
};

namespace {
constexpr uint32_t kPlanMagic = 0x524C5850u;   // "RLXP"
inline bool plan_ok(const rlx_plan* p) { return p && p->magic == kPlanMagic; }
}  // namespace

extern "C" {

const char* rlx_status_string(int status) {
    switch (status) {
    case RLX_OK: return "ok";
    case RLX_ERR_INVALID_ARG: return "invalid argument";
    case RLX_ERR_MISALIGNED: return "pointer not aligned to its element size";
    case RLX_ERR_BAD_HYPER: return "bias correction is zero or a hyper-parameter is not finite";
    case RLX_ERR_HIP: return "HIP runtime error";
    case RLX_ERR_NO_DEVICE: return "no HIP device";
    case RLX_ERR_TOO_LARGE: return "too many chunks for one plan";
    default: return "unknown status";
    }
}

const char* rlx_last_hip_error(void) { return g_hip_error; }

int rlx_version(void) { return 100; }

int rlx_adamw_fp16(float* master_w, uint16_t* model_w, const uint16_t* grad, float* m, float* v, int64_t n,
                   float lr, float beta1, float beta2, float eps, float weight_decay,
                   float bias_correction1, float bias_correction2, void* stream) {
    return flat_update(model_w, grad, m, v, master_w, n, RLX_DTYPE_F16, lr, beta1, beta2, eps, weight_decay,
                       bias_correction1, bias_correction2, stream);
}

int rlx_adamw_fp32(float* w, const float* grad, float* m, float* v, int64_t n,
                   float lr, float beta1, float beta2, float eps, float weight_decay,
                   float bias_correction1, float bias_correction2, void* stream) {
    return flat_update(w, grad, m, v, nullptr, n, RLX_DTYPE_F32, lr, beta1, beta2, eps, weight_decay,
                       bias_correction1, bias_correction2, stream);
}

int rlx_fp16_to_fp32(float* dst, const uint16_t* src, int64_t n, void* stream) {
    if (n <= 0) return RLX_OK;
    if (!dst || !src) return RLX_ERR_INVALID_ARG;
    if (!is_aligned(dst, 4) || !is_aligned(src, 2)) return RLX_ERR_MISALIGNED;
    int64_t grid = (n + kBlock - 1) / kBlock;
    if (grid > 65536) grid = 65536;
    fp16_to_fp32_kernel<<<dim3((unsigned)grid), dim3(kBlock), 0, (hipStream_t)stream>>>(dst, src, n);
    RLX_HIP(hipGetLastError());
    return RLX_OK;
}

int rlx_plan_create(const rlx_tensor_desc* descs, int64_t count, int64_t chunk_elems, rlx_plan** out) {
    if (!out) return RLX_ERR_INVALID_ARG;
    *out = nullptr;
    if (!descs || count <= 0 || count > INT32_MAX) return RLX_ERR_INVALID_ARG;
    if (chunk_elems == 0) chunk_elems = kDefaultChunk;
    if (chunk_elems < kGroup || chunk_elems % kGroup != 0 || chunk_elems > (1 << 24)) return RLX_ERR_INVALID_ARG;

    std::vector<DevTensor> tensors((size_t)count);
    int64_t n_chunks = 0, n_elems = 0;
    for (int64_t i = 0; i < count; i++) {
        int st = make_dev_tensor(descs[i], tensors[(size_t)i]);
        if (st != RLX_OK) return st;
        n_chunks += (descs[i].n + chunk_elems - 1) / chunk_elems;
        n_elems += descs[i].n;
    }
    if (n_chunks > INT32_MAX) return RLX_ERR_TOO_LARGE;
    std::vector<DevChunk> chunks;
    chunks.reserve((size_t)n_chunks);
    for (int64_t i = 0; i < count; i++) {
        const int64_t k = (descs[i].n + chunk_elems - 1) / chunk_elems;
        for (int64_t j = 0; j < k; j++) chunks.push_back(DevChunk{(int32_t)i, (int32_t)j});
    }

    rlx_plan* p = new (std::nothrow) rlx_plan();
    if (!p) return RLX_ERR_INVALID_ARG;
    p->magic = kPlanMagic;
    p->n_tensors = count; p->n_chunks = n_chunks; p->n_elems = n_elems; p->chunk_elems = chunk_elems;
    p->d_tensors = nullptr; p->d_chunks = nullptr; p->d_partials = nullptr; p->d_norm = nullptr; p->h_norm = nullptr;

    hipError_t e = hipGetDevice(&p->device);
    if (e == hipSuccess) e = hipMalloc((void**)&p->d_tensors, sizeof(DevTensor) * (size_t)count);
    if (e == hipSuccess) e = hipMalloc((void**)&p->d_chunks, sizeof(DevChunk) * (size_t)n_chunks);
    if (e == hipSuccess) e = hipMalloc((void**)&p->d_partials, sizeof(double) * (size_t)n_chunks);
    if (e == hipSuccess) e = hipMalloc((void**)&p->d_norm, sizeof(NormResult));
    if (e == hipSuccess) e = hipHostMalloc((void**)&p->h_norm, sizeof(NormResult), hipHostMallocDefault);
    if (e == hipSuccess) e = hipMemcpy(p->d_tensors, tensors.data(), sizeof(DevTensor) * (size_t)count, hipMemcpyHostToDevice);
    if (e == hipSuccess) e = hipMemcpy(p->d_chunks, chunks.data(), sizeof(DevChunk) * (size_t)n_chunks, hipMemcpyHostToDevice);
    if (e == hipSuccess) {
        const NormResult init = {0.0, 0.0f, 1.0f};
        *p->h_norm = init;
        e = hipMemcpy(p->d_norm, &init, sizeof(init), hipMemcpyHostToDevice);
    }
    if (e != hipSuccess) {
        int st = hip_fail(e, "rlx_plan_create");
        rlx_plan_destroy(p);
        return st;
    }
    *out = p;
    return RLX_OK;
}

int rlx_plan_destroy(rlx_plan* p) {
    if (!p) return RLX_OK;
    if (!plan_ok(p)) return RLX_ERR_INVALID_ARG;
    hipError_t first = hipSuccess, e;
    if (p->d_tensors && (e = hipFree(p->d_tensors)) != hipSuccess && first == hipSuccess) first = e;
    if (p->d_chunks && (e = hipFree(p->d_chunks)) != hipSuccess && first == hipSuccess) first = e;
    if (p->d_partials && (e = hipFree(p->d_partials)) != hipSuccess && first == hipSuccess) first = e;
    if (p->d_norm && (e = hipFree(p->d_norm)) != hipSuccess && first == hipSuccess) first = e;
    if (p->h_norm && (e = hipHostFree(p->h_norm)) != hipSuccess && first == hipSuccess) first = e;
    p->magic = 0;
    delete p;
    return first == hipSuccess ? RLX_OK : hip_fail(first, "rlx_plan_destroy");
}

int64_t rlx_plan_num_chunks(const rlx_plan* p) { return plan_ok(p) ? p->n_chunks : -1; }
int64_t rlx_plan_num_elements(const rlx_plan* p) { return plan_ok(p) ? p->n_elems : -1; }
int64_t rlx_plan_chunk_elems(const rlx_plan* p) { return plan_ok(p) ? p->chunk_elems : -1; }
const void* rlx_plan_norm_device_ptr(const rlx_plan* p) { return plan_ok(p) ? p->d_norm : nullptr; }
const double* rlx_plan_partials_device_ptr(const rlx_plan* p) { return plan_ok(p) ? p->d_partials : nullptr; }

int rlx_plan_grad_norm(rlx_plan* p, float max_norm, void* stream) {
    if (!plan_ok(p)) return RLX_ERR_INVALID_ARG;
    hipStream_t s = (hipStream_t)stream;
    const dim3 grid((unsigned)pick_grid(p->n_chunks, g_tuning.norm_grid)), block(kBlock);
    if (g_tuning.norm_nt)
        sumsq_partials_kernel<true><<<grid, block, 0, s>>>(p->d_tensors, p->d_chunks, p->n_chunks, p->chunk_elems, p->d_partials);
    else
        sumsq_partials_kernel<false><<<grid, block, 0, s>>>(p->d_tensors, p->d_chunks, p->n_chunks, p->chunk_elems, p->d_partials);
    RLX_HIP(hipGetLastError());
    sumsq_final_kernel<<<dim3(1), dim3(kFinalBlock), 0, s>>>(p->d_partials, p->n_chunks, max_norm, p->d_norm);
    RLX_HIP(hipGetLastError());
    return RLX_OK;
}

int rlx_plan_norm_read(rlx_plan* p, float* norm, float* scale, double* sum_sq, void* stream) {
    if (!plan_ok(p)) return RLX_ERR_INVALID_ARG;
    hipStream_t s = (hipStream_t)stream;
    RLX_HIP(hipMemcpyAsync(p->h_norm, p->d_norm, sizeof(NormResult), hipMemcpyDeviceToHost, s));
    RLX_HIP(hipStreamSynchronize(s));
    if (norm) *norm = p->h_norm->norm;
    if (scale) *scale = p->h_norm->scale;
    if (sum_sq) *sum_sq = p->h_norm->sum_sq;
    return RLX_OK;
}

int rlx_plan_scale_grads(rlx_plan* p, void* stream) {
    if (!plan_ok(p)) return RLX_ERR_INVALID_ARG;
    const dim3 grid((unsigned)pick_grid(p->n_chunks, g_tuning.update_grid)), block(kBlock);
    scale_grads_kernel<false><<<grid, block, 0, (hipStream_t)stream>>>(p->d_tensors, p->d_chunks, p->n_chunks,
                                                                       p->chunk_elems, p->d_norm);
    RLX_HIP(hipGetLastError());
    return RLX_OK;
}

int rlx_plan_adamw(rlx_plan* p, const rlx_step_params* sp, int clip_mode, void* stream) {
    if (!plan_ok(p) || !sp) return RLX_ERR_INVALID_ARG;
    if (clip_mode != RLX_CLIP_NONE && clip_mode != RLX_CLIP_FUSED) return RLX_ERR_INVALID_ARG;
    int st = check_hyper(sp->lr, sp->beta1, sp->beta2, sp->eps, sp->weight_decay, sp->bias_correction1,
                         sp->bias_correction2);
    if (st != RLX_OK) return st;
    const Hyper h = make_hyper(sp->lr, sp->beta1, sp->beta2, sp->eps, sp->weight_decay, sp->bias_correction1,
                               sp->bias_correction2);
    DevTensor none;
    memset(&none, 0, sizeof(none));
    return launch_update<false>(p->d_tensors, p->d_chunks, none, p->n_chunks, p->chunk_elems, h,
                                clip_mode == RLX_CLIP_FUSED ? p->d_norm : nullptr, (hipStream_t)stream);
}

int rlx_set_tuning(const char* key, int64_t value) {
    if (!key || value < 0) return RLX_ERR_INVALID_ARG;
    if (!strcmp(key, "update_variant")) { if (value > 5) return RLX_ERR_INVALID_ARG; g_tuning.update_variant = value; }
    else if (!strcmp(key, "update_grid")) g_tuning.update_grid = value;
    else if (!strcmp(key, "norm_grid")) g_tuning.norm_grid = value;
    else if (!strcmp(key, "norm_nt")) g_tuning.norm_nt = value ? 1 : 0;
    else return RLX_ERR_INVALID_ARG;
    return RLX_OK;
}

int64_t rlx_get_tuning(const char* key) {
    if (!key) return -1;
    if (!strcmp(key, "update_variant")) return g_tuning.update_variant;
    if (!strcmp(key, "update_grid")) return g_tuning.update_grid;
    if (!strcmp(key, "norm_grid")) return g_tuning.norm_grid;
    if (!strcmp(key, "norm_nt")) return g_tuning.norm_nt;
    return -1;
}

static int fill_common(void* dst, int elem_size, int64_t n, uint64_t seed, int64_t first, float mean, float std,
                       uint32_t flags, int64_t row_len, uint32_t zero_rows_below, void* stream) {
    if (n <= 0) return RLX_OK;
    if (!dst || first < 0 || row_len < 0) return RLX_ERR_INVALID_ARG;
    if (!is_aligned(dst, (size_t)elem_size)) return RLX_ERR_MISALIGNED;
    int64_t grid = (n + kBlock - 1) / kBlock;
    if (grid > 262144) grid = 262144;
    if (elem_size == 2)
        fill_kernel<uint16_t><<<dim3((unsigned)grid), dim3(kBlock), 0, (hipStream_t)stream>>>(
            (uint16_t*)dst, n, seed, first, mean, std, flags, row_len, zero_rows_below);
    else
        fill_kernel<float><<<dim3((unsigned)grid), dim3(kBlock), 0, (hipStream_t)stream>>>(
            (float*)dst, n, seed, first, mean, std, flags, row_len, zero_rows_below);
    RLX_HIP(hipGetLastError());
    return RLX_OK;
}

int rlx_fill_f16(uint16_t* dst, int64_t n, uint64_t seed, int64_t first, float mean, float std, uint32_t flags,
                 int64_t row_len, uint32_t zero_rows_below, void* stream) {
    return fill_common(dst, 2, n, seed, first, mean, std, flags, row_len, zero_rows_below, stream);
}

int rlx_fill_f32(float* dst, int64_t n, uint64_t seed, int64_t first, float mean, float std, uint32_t flags,
                 int64_t row_len, uint32_t zero_rows_below, void* stream) {
    return fill_common(dst, 4, n, seed, first, mean, std, flags, row_len, zero_rows_below, stream);
}

}  // extern "C"
