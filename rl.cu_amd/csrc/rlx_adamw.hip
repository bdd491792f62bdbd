// MI355X (gfx950) AdamW step, deterministic gradient norm and clip: HIP kernels and the
// C ABI declared in include/rlx_adamw.h.
//
// Every kernel here is a pure stream over HBM: no LDS except for the cross-wave step of
// the norm reduction, no matrix cores.
//
// Work is described by one 64-byte record per "chunk" (`chunk_elems` consecutive elements
// of one tensor) holding the chunk's resolved pointers, so that a workgroup needs a single
// scalar load to find its operands.
//
// Update kernel: a chunk is cut into tiles of 256 elements and every tile is one small
// workgroup (128 lanes, two elements per lane: one 32-bit access per FP16 stream and one
// 64-bit access per FP32 stream, each instruction contiguous across the wavefront, all
// marked non-temporal, the stores also system-scope).  On MI355X this shape measured
// ~6.8 TB/s on the seven streams of the update against ~5.3 TB/s for 128-bit accesses with
// several KB per workgroup: what matters for a mixed read/write stream is that the set of
// addresses in flight stays a narrow window, which many tiny workgroups dispatched in order
// give and fat workgroups or grid-stride loops do not.  Consecutive workgroups go round-robin
// to the 8 XCDs; an optional swizzle (K > 1) hands each XCD K neighbouring tiles, which did
// not pay in measurements.
//
// Norm kernel: one workgroup of up to 512 lanes per chunk with 128-bit reads; one FP64 partial
// per chunk in a fixed slot, then a single-workgroup pass in fixed order (no atomics).
//
// Arithmetic follows src/kernels/adamw.cu:25-39 of the reference operation by operation
// and is compiled without FMA contraction, with IEEE division and square root and with
// FP32 denormals kept, so that a CPU restatement built the same way agrees bit for bit.

#include <hip/hip_runtime.h>

#include <cmath>
#include <cstdint>
#include <cstdio>
#include <atomic>
#include <cstring>
#include <mutex>
#include <new>
#include <utility>
#include <vector>

#include "rlx_adamw.h"

// Intermediate sums of rlx_grad_norm_static, the entry point for callers that cannot allocate: part of the
// library's device image (2.1 MiB on every GPU the library runs on, until the process ends).  Layout, in
// doubles: [0, 2^18) per-chunk FP64 partials; [2^18, 2^18 + 2^14) group partials (one per 16 chunks, used with
// 512-element chunks).  Nothing in it has to start at zero: every call writes each slot that it later reads (the
// entry point always adds the partials in a second launch; the one-launch form needs counters that stay valid
// from call to call only while the number of workgroups stays the same, and calls of any size share this array).
// The name
// stands for the array only in device code; host code uses the address that hipGetSymbolAddress returns for the
// current device (static_scratch below), never the name.
constexpr int64_t kStaticMaxPartials = 1 << 18;
constexpr int64_t kStaticMaxGroups = kStaticMaxPartials / 16;
static __device__ __align__(256) double scratch[kStaticMaxPartials + kStaticMaxGroups];

namespace {

constexpr int kVec = 8;                       // elements per lane per group in the norm and scale passes
constexpr int kNormBlock = 512;               // most lanes per workgroup of the norm pass (8 wavefronts)
constexpr int kScaleBlock = 256;              // lanes per workgroup of the scale pass
constexpr int64_t kMinChunk = 512;             // the largest tile of any update variant
constexpr int64_t kSmallChunk = 2048;
constexpr int64_t kBigChunk = 8192;
constexpr int kFinalBlock = 1024;

typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x8 __attribute__((ext_vector_type(8)));

// One chunk of one tensor, pointers already advanced to the chunk's first element.
struct ChunkRec {
    void* p;
    void* g;
    float* m;
    float* v;
    float* master;
    uint32_t count;      // elements in this chunk (the last chunk of a tensor may be short)
    uint32_t flags;      // RLX_TENSOR_* | kF32 | valign << kValignShift | galign << kGalignShift
    int64_t pad[2];
};
static_assert(sizeof(ChunkRec) == 64, "ChunkRec is one 64-byte record");
constexpr uint32_t kF32 = 0x10;               // FP32 parameter and gradient
constexpr int kValignShift = 8;               // flags bits 8..11: widest lane vector (1,2,4,8 elements)
                                              // for which every stream of the chunk is aligned
constexpr int kGalignShift = 12;              // flags bits 12..15: the same for the gradient stream alone (the
                                              // norm and the scale pass touch nothing else)

struct NormResult {
    double sum_sq;
    float norm;
    float scale;
};

struct Hyper {
    float lr, beta1, beta2, eps, weight_decay, bc1_inv, bc2_inv;
};

// Device-resident state of a plan's step table (host-free replay).  One allocation whose address stays the same
// from the first upload until the plan is destroyed: recorded launches name it and nothing else.
struct SchedHeader {
    rlx_step_params current;         // the entry that the next scheduled update reads (first member: the update
                                     // kernel is handed the header's address as its hyper-parameters)
    uint32_t pad0;
    int64_t taken;                   // scheduled steps since the upload, saturating at len
    const rlx_step_params* table;    // the uploaded entries
    int64_t len;
    int64_t overrun;                 // scheduled updates that ran after the table had been used up
};
static_assert(sizeof(SchedHeader) == 64 && sizeof(rlx_step_params) == 28, "one 64-byte header");

// Two flat gradient buffers described by value (an FP16 one followed by an FP32 one, the shape of
// the reference's half_pool / float_pool): the chunks that a plan over these two tensors would
// hold, without a table in device memory.
struct PoolPair {
    const uint16_t* half_pool;
    const float* float_pool;
    int64_t n_half, n_float;
    int64_t chunks_half;             // chunks of the FP16 buffer; those of the FP32 buffer follow
    int chunk_log2;
    uint32_t flags_half, flags_float;   // ChunkRec::flags of every chunk of the buffer
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

// Every buffer handed to this library is HIP device memory, so all accesses go through
// global-address-space pointers (global_load/global_store rather than flat).
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

// Streaming store of the update kernel.  SP = 1 adds the sc1 bit to the non-temporal store
// (written as inline assembly: the compiler has no spelling for that combination); on MI355X it
// measured about 1 % faster than the plain non-temporal store for this kernel.  SP = 0: non-temporal
// store; SP = 2: ordinary store.
template <int SP, typename T>
__device__ __forceinline__ void st_stream(T* p, T x) {
    if constexpr (SP == 0) {
        stg<true>(p, x);
    } else if constexpr (SP == 2) {
        stg<false>(p, x);
    } else {
        RLX_GLOBAL T* gp = (RLX_GLOBAL T*)p;
        if constexpr (sizeof(T) == 2) {
            const uint32_t w = (uint32_t)x;
            asm volatile("global_store_short %0, %1, off sc1 nt" ::"v"(gp), "v"(w) : "memory");
        } else if constexpr (sizeof(T) == 4) {
            asm volatile("global_store_dword %0, %1, off sc1 nt" ::"v"(gp), "v"(x) : "memory");
        } else if constexpr (sizeof(T) == 8) {
            asm volatile("global_store_dwordx2 %0, %1, off sc1 nt" ::"v"(gp), "v"(x) : "memory");
        } else if constexpr (sizeof(T) == 16) {
            // the hardware needs two wait states between a store wider than 64 bits and a write to its data
            // registers; inside inline assembly the compiler does not insert them itself
            asm volatile("global_store_dwordx4 %0, %1, off sc1 nt\n\ts_nop 1" ::"v"(gp), "v"(x) : "memory");
        } else {
            static_assert(sizeof(T) == 32, "store of 2, 4, 8, 16 or 32 bytes");
            const f32x4 lo = {x[0], x[1], x[2], x[3]}, hi = {x[4], x[5], x[6], x[7]};
            asm volatile("global_store_dwordx4 %0, %1, off sc1 nt\n\tglobal_store_dwordx4 %0, %2, off offset:16 sc1 nt\n\ts_nop 1"
                         ::"v"(gp), "v"(lo), "v"(hi) : "memory");
        }
    }
}

// Every vector memory operation that this wavefront has issued so far has completed; later ones do not start before.
__device__ __forceinline__ void wait_for_memory() { asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); }

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

// FP16 gradient times the clip scale, as scale_half_kernel stores it (trainer.h:136-139): the
// product is rounded to FP32 and then to FP16.  Left to itself the compiler merges the multiply and
// the conversion into one v_fma_mixlo_f16, which rounds the exact product once and differs in the
// last FP16 bit for about one value in 10^4; the empty asm keeps the two roundings apart.
__device__ __forceinline__ uint32_t scaled_f16_bits(float g, float scale) {
    float t = g * scale;
    asm volatile("" : "+v"(t));
    return f2h(t);
}

// Clip as a preceding scale pass would have stored it: re-round to FP16, continue in FP32.
__device__ __forceinline__ float clip_f16(float g, float scale) { return h2f(scaled_f16_bits(g, scale)); }

// E packed FP16 values and E FP32 values as one access each.
template <int E> struct Lane;
template <> struct Lane<1> { typedef uint16_t H; typedef float F; };
template <> struct Lane<2> { typedef uint32_t H; typedef f32x2 F; };
template <> struct Lane<4> { typedef u32x2 H; typedef f32x4 F; };
template <> struct Lane<8> { typedef u32x4 H; typedef f32x8 F; };      // one 128-bit FP16 access, two 128-bit FP32 accesses

template <int E>
__device__ __forceinline__ void unpack_h(typename Lane<E>::H x, float* out) {
    if constexpr (E == 1) out[0] = h2f(x);
    else if constexpr (E == 2) { out[0] = h2f(x & 0xFFFFu); out[1] = h2f(x >> 16); }
    else {
#pragma unroll
        for (int k = 0; k < E / 2; k++) { out[2 * k] = h2f(x[k] & 0xFFFFu); out[2 * k + 1] = h2f(x[k] >> 16); }
    }
}

template <int E>
__device__ __forceinline__ typename Lane<E>::H pack_h(const float* w) {
    if constexpr (E == 1) return (uint16_t)f2h(w[0]);
    else if constexpr (E == 2) return f2h(w[0]) | (f2h(w[1]) << 16);
    else {
        typename Lane<E>::H o;
#pragma unroll
        for (int k = 0; k < E / 2; k++) o[k] = f2h(w[2 * k]) | (f2h(w[2 * k + 1]) << 16);
        return o;
    }
}

template <int E>
__device__ __forceinline__ void unpack_f(typename Lane<E>::F x, float* out) {
    if constexpr (E == 1) out[0] = x;
    else {
#pragma unroll
        for (int k = 0; k < E; k++) out[k] = x[k];
    }
}

template <int E>
__device__ __forceinline__ typename Lane<E>::F pack_f(const float* x) {
    if constexpr (E == 1) return x[0];
    else {
        typename Lane<E>::F o;
#pragma unroll
        for (int k = 0; k < E; k++) o[k] = x[k];
        return o;
    }
}

// Element-by-element path: chunks whose streams are not aligned for the lane vector, and the
// last, partial vector of a tensor.
__device__ __forceinline__ void update_scalar16(const ChunkRec& r, int64_t i, const Hyper& h, float wd,
                                                float scale, bool clip) {
    uint16_t* p = (uint16_t*)r.p + i;
    float g = h2f(ldg<true>((const uint16_t*)r.g + i));
    if (clip) g = clip_f16(g, scale);
    float m = ldg<true>(r.m + i), v = ldg<true>(r.v + i);
    float w = r.master ? ldg<true>(r.master + i) : h2f(ldg<true>(p));
    adamw_elem(g, m, v, w, h, wd);
    stg<true>(r.m + i, m);
    stg<true>(r.v + i, v);
    if (r.master) stg<true>(r.master + i, w);
    stg<true>(p, (uint16_t)f2h(w));
}

__device__ __forceinline__ void update_scalar32(const ChunkRec& r, int64_t i, const Hyper& h, float wd,
                                                float scale, bool clip) {
    float* p = (float*)r.p + i;
    float g = ldg<true>((const float*)r.g + i);
    if (clip) g = g * scale;                    // scale_float_kernel, trainer.h:142-145
    float m = ldg<true>(r.m + i), v = ldg<true>(r.v + i), w = ldg<true>(p);
    adamw_elem(g, m, v, w, h, wd);
    stg<true>(r.m + i, m);
    stg<true>(r.v + i, v);
    stg<true>(p, w);
}

// ---------------------------------------------------------------------------------------
// The update of a whole, aligned tile of an FP16 tensor without master copy, two elements per lane as in update_tile,
// but with half the memory instructions: the two lanes of a pair (2k, 2k+1) work on four consecutive elements, the
// even lane loads the four first moments (128 bits) and the four gradients (64 bits), the odd lane the four second
// moments and the four weights, each hands the other the half it needs (a swap inside the quad, no LDS), and the
// results go back the same way: even lanes store four first moments, odd lanes four second moments and four weights.
// One instruction then serves two streams, each half of the wavefront contiguous.  Same arithmetic per element.
// ---------------------------------------------------------------------------------------

template <int LANES, int SP, bool NTL, bool CLIP>
__device__ __forceinline__ void update_tile_paired(const ChunkRec& r, int64_t off, int lane, Hyper h,
                                                   const rlx_step_params* __restrict__ dev_params,
                                                   const NormResult* __restrict__ norm)
{
    if (dev_params) {
        h.lr = dev_params->lr; h.beta1 = dev_params->beta1; h.beta2 = dev_params->beta2; h.eps = dev_params->eps;
        h.weight_decay = dev_params->weight_decay;
        h.bc1_inv = 1.0f / dev_params->bias_correction1;
        h.bc2_inv = 1.0f / dev_params->bias_correction2;
    }
    float scale = 1.0f;
    if constexpr (CLIP) scale = norm->scale;
    const float wd = (r.flags & RLX_TENSOR_NO_DECAY) ? 0.0f : h.weight_decay;
    const bool odd = (lane & 1) != 0;
    const int64_t pair = off + (int64_t)(lane & ~1) * 2;          // first of the pair's four elements
    uint16_t* const p16 = (uint16_t*)r.p;
    const f32x4 f = ldg<NTL>((const f32x4*)((odd ? r.v : r.m) + pair));
    const u32x2 hw = ldg<NTL>((const u32x2*)((odd ? (const uint16_t*)p16 : (const uint16_t*)r.g) + pair));
    // the even lane works on elements 0, 1 of the pair and needs v[0..1], p[0..1]; the odd lane on 2, 3 and needs
    // m[2..3], g[2..3]
    const float rf0 = __shfl_xor(odd ? f[0] : f[2], 1, 64), rf1 = __shfl_xor(odd ? f[1] : f[3], 1, 64);
    const uint32_t rh = __shfl_xor(odd ? hw[0] : hw[1], 1, 64);
    float g[2], m[2], v[2], w[2];
    const uint32_t gbits = odd ? rh : hw[0], wbits = odd ? hw[1] : rh;
    g[0] = h2f(gbits & 0xFFFFu); g[1] = h2f(gbits >> 16);
    w[0] = h2f(wbits & 0xFFFFu); w[1] = h2f(wbits >> 16);
    m[0] = odd ? rf0 : f[0]; m[1] = odd ? rf1 : f[1];
    v[0] = odd ? f[2] : rf0; v[1] = odd ? f[3] : rf1;
    if constexpr (CLIP) { g[0] = clip_f16(g[0], scale); g[1] = clip_f16(g[1], scale); }
    adamw_elem(g[0], m[0], v[0], w[0], h, wd);
    adamw_elem(g[1], m[1], v[1], w[1], h, wd);
    // the even lane stores the pair's first moments, the odd lane its second moments and its weights
    const float x0 = __shfl_xor(odd ? m[0] : v[0], 1, 64), x1 = __shfl_xor(odd ? m[1] : v[1], 1, 64);
    const f32x4 out = odd ? f32x4{x0, x1, v[0], v[1]} : f32x4{m[0], m[1], x0, x1};
    st_stream<SP>((f32x4*)((odd ? r.v : r.m) + pair), out);
    const uint32_t mine = f2h(w[0]) | (f2h(w[1]) << 16);
    const uint32_t other = __shfl_xor(mine, 1, 64);
    if (odd) st_stream<SP>((u32x2*)(p16 + pair), u32x2{other, mine});
}

// ---------------------------------------------------------------------------------------
// Update of one tile: E elements per lane, LANES lanes, TILE = E * LANES elements starting `off` elements into
// the chunk `r`, of which `left` remain to the end of the chunk / tensor.  `lane` is this lane's index in the tile.
// SP: 1 = system-scope non-temporal stores, 0 = non-temporal stores, 2 = ordinary stores; NTL: non-temporal loads.
// PH: 0 = a lane issues the tile's four loads at once; 1 = tiles that write four streams (master copy,
// gradient clearing) issue their loads, and with a master copy their stores, two at a time.
// CLIP: the gradients are multiplied by the clip scale at `norm` first (a compile-time choice, so that the
// plain and the fused-clip update are two kernels with two names in a profile).
// ---------------------------------------------------------------------------------------

template <int E, int LANES, int SP, int PH, bool NTL, bool CLIP>
__device__ __forceinline__ void update_tile(const ChunkRec& r, int64_t off, int64_t left, int lane, Hyper h,
                                            const rlx_step_params* __restrict__ dev_params,
                                            const NormResult* __restrict__ norm, uint32_t step_flags)
{
    constexpr int TILE = E * LANES;
    if (left <= 0) return;
    const int n_here = left < TILE ? (int)left : TILE;
    const bool is_f32 = (r.flags & kF32) != 0;
    const int valign = (r.flags >> kValignShift) & 0xF;
    if constexpr (PH == 2 && E == 2) {
        // whole tiles of plain FP16 tensors whose streams are aligned for a pair's 128-bit accesses; everything
        // else (tails, FP32 tensors, master copy, gradient clearing, frozen and grad-only chunks) as below
        if (left >= TILE && valign >= 4 && r.master == nullptr &&
            !(r.flags & (kF32 | RLX_TENSOR_GRAD_ONLY | RLX_TENSOR_FROZEN)) && !(step_flags & RLX_STEP_ZERO_GRADS)) {
            update_tile_paired<LANES, SP, NTL, CLIP>(r, off, lane, h, dev_params, norm);
            return;
        }
    }
    const int e0 = lane * E;
    const int64_t i0 = off + e0;
    const bool zero_grads = (step_flags & RLX_STEP_ZERO_GRADS) != 0;
    const bool vec = valign >= E && e0 + E <= n_here;
    typedef typename Lane<E>::H HV;
    typedef typename Lane<E>::F FV;

    if (r.flags & (RLX_TENSOR_GRAD_ONLY | RLX_TENSOR_FROZEN)) {
        // no update here; the buffer is only cleared for the next accumulation
        if (zero_grads) {
            if (vec) {
                if (is_f32) st_stream<SP>((FV*)((float*)r.g + i0), FV{});
                else st_stream<SP>((HV*)((uint16_t*)r.g + i0), HV{});
            } else {
                for (int e = e0; e < e0 + E && e < n_here; e++) {
                    if (is_f32) st_stream<SP>((float*)r.g + off + e, 0.0f);
                    else st_stream<SP>((uint16_t*)r.g + off + e, (uint16_t)0);
                }
            }
        }
        return;
    }

    if (dev_params) {      // hyper-parameters resident on the device (replayable launches)
        h.lr = dev_params->lr; h.beta1 = dev_params->beta1; h.beta2 = dev_params->beta2; h.eps = dev_params->eps;
        h.weight_decay = dev_params->weight_decay;
        h.bc1_inv = 1.0f / dev_params->bias_correction1;
        h.bc2_inv = 1.0f / dev_params->bias_correction2;
    }
    constexpr bool clip = CLIP;
    float scale = 1.0f;
    if constexpr (CLIP) scale = norm->scale;
    const float wd = (r.flags & RLX_TENSOR_NO_DECAY) ? 0.0f : h.weight_decay;

    if (!vec) {
        for (int e = e0; e < e0 + E && e < n_here; e++) {
            if (is_f32) {
                update_scalar32(r, off + e, h, wd, scale, clip);
                if (zero_grads) st_stream<SP>((float*)r.g + off + e, 0.0f);
            } else {
                update_scalar16(r, off + e, h, wd, scale, clip);
                if (zero_grads) st_stream<SP>((uint16_t*)r.g + off + e, (uint16_t)0);
            }
        }
        return;
    }

    float g[E], m[E], v[E], w[E];
    if (!is_f32) {
        const bool has_master = r.master != nullptr;
        HV gw;
        FV mw, vw;
        const auto load_g = [&] { gw = ldg<NTL>((const HV*)((const uint16_t*)r.g + i0)); };
        const auto load_mv = [&] { mw = ldg<NTL>((const FV*)(r.m + i0)); vw = ldg<NTL>((const FV*)(r.v + i0)); };
        const auto load_w = [&] {
            if (has_master) unpack_f<E>(ldg<NTL>((const FV*)(r.master + i0)), w);
            else unpack_h<E>(ldg<NTL>((const HV*)((const uint16_t*)r.p + i0)), w);
        };
        // A tile that writes four streams (master copy, or gradients cleared) runs faster when a wavefront has
        // two loads in flight at a time instead of four: measured on Qwen3-0.6B with realistic values, 2.69 ->
        // 2.52 ms with a master copy and 2.157 -> 2.127 ms with gradient clearing.  With three streams written
        // the same split costs 1-4 %, so the plain update issues all four loads at once.
        // The host launches the PH = 1 form of the kernel only for such steps, so that the plain update keeps
        // its straight-line code (a run-time test here cost it 2 %).
        if constexpr (PH != 1) {
            load_g(); load_mv(); load_w();
        } else {
            if (has_master || zero_grads) { load_g(); load_w(); wait_for_memory(); load_mv(); }
            else { load_g(); load_mv(); load_w(); }
        }
        unpack_h<E>(gw, g);
        unpack_f<E>(mw, m);
        unpack_f<E>(vw, v);
        if (clip) {
#pragma unroll
            for (int k = 0; k < E; k++) g[k] = clip_f16(g[k], scale);
        }
#pragma unroll
        for (int k = 0; k < E; k++) adamw_elem(g[k], m[k], v[k], w[k], h, wd);
        st_stream<SP>((FV*)(r.m + i0), pack_f<E>(m));
        st_stream<SP>((FV*)(r.v + i0), pack_f<E>(v));
        if (has_master) {
            // likewise two stores at a time: another 2.52 -> 2.48 ms (with gradient clearing instead it costs 5 %)
            if constexpr (PH == 1) wait_for_memory();
            st_stream<SP>((FV*)(r.master + i0), pack_f<E>(w));
        }
        st_stream<SP>((HV*)((uint16_t*)r.p + i0), pack_h<E>(w));
        if (zero_grads) st_stream<SP>((HV*)((uint16_t*)r.g + i0), HV{});
    } else {
        // FP32 parameters (norm weights): the same update, in place (adamw.cu:80-90)
        unpack_f<E>(ldg<NTL>((const FV*)((const float*)r.g + i0)), g);
        unpack_f<E>(ldg<NTL>((const FV*)(r.m + i0)), m);
        unpack_f<E>(ldg<NTL>((const FV*)(r.v + i0)), v);
        unpack_f<E>(ldg<NTL>((const FV*)((const float*)r.p + i0)), w);
        if (clip) {
#pragma unroll
            for (int k = 0; k < E; k++) g[k] = g[k] * scale;
        }
#pragma unroll
        for (int k = 0; k < E; k++) adamw_elem(g[k], m[k], v[k], w[k], h, wd);
        st_stream<SP>((FV*)(r.m + i0), pack_f<E>(m));
        st_stream<SP>((FV*)(r.v + i0), pack_f<E>(v));
        st_stream<SP>((FV*)((float*)r.p + i0), pack_f<E>(w));
        if (zero_grads) st_stream<SP>((FV*)((float*)r.g + i0), FV{});
    }
}

// R sub-tiles of E * LANES elements per workgroup with the same narrow, wave-contiguous accesses as update_tile:
// the loads of all R sub-tiles are issued before the first is used.  Kept for comparison: on Qwen3-0.6B two
// sub-tiles per workgroup reach 6.38 TB/s and four 6.0 (a one-wavefront workgroup with two, and a 256-lane one
// with two, 6.18 and 6.36) against 6.76 for one: more bytes per workgroup widen the window of addresses in flight.  Tiles that are not whole, aligned FP16
// tensors with parameters go through update_tile one sub-tile after the other.
template <int E, int LANES, int R, int SP, bool CLIP>
__device__ __forceinline__ void update_tile_rounds(const ChunkRec& r, int64_t off, int64_t left, int lane, Hyper h,
                                                   const rlx_step_params* __restrict__ dev_params,
                                                   const NormResult* __restrict__ norm, uint32_t step_flags)
{
    constexpr int SUB = E * LANES;
    typedef typename Lane<E>::H HV;
    typedef typename Lane<E>::F FV;
    const int valign = (r.flags >> kValignShift) & 0xF;
    const bool fast = !(r.flags & (kF32 | RLX_TENSOR_GRAD_ONLY | RLX_TENSOR_FROZEN)) && valign >= E && left >= R * SUB;
    if (!fast) {
#pragma unroll
        for (int k = 0; k < R; k++)
            update_tile<E, LANES, SP, 0, true, CLIP>(r, off + k * SUB, left - k * SUB, lane, h, dev_params, norm, step_flags);
        return;
    }
    if (dev_params) {
        h.lr = dev_params->lr; h.beta1 = dev_params->beta1; h.beta2 = dev_params->beta2; h.eps = dev_params->eps;
        h.weight_decay = dev_params->weight_decay;
        h.bc1_inv = 1.0f / dev_params->bias_correction1;
        h.bc2_inv = 1.0f / dev_params->bias_correction2;
    }
    constexpr bool clip = CLIP;
    float scale = 1.0f;
    if constexpr (CLIP) scale = norm->scale;
    const float wd = (r.flags & RLX_TENSOR_NO_DECAY) ? 0.0f : h.weight_decay;
    const bool zero_grads = (step_flags & RLX_STEP_ZERO_GRADS) != 0;
    const bool has_master = r.master != nullptr;
    const int64_t i0 = off + lane * E;
    HV gw[R], pw[R];
    FV mw[R], vw[R], ww[R];
#pragma unroll
    for (int k = 0; k < R; k++) {
        const int64_t i = i0 + k * SUB;
        gw[k] = ldg<true>((const HV*)((const uint16_t*)r.g + i));
        mw[k] = ldg<true>((const FV*)(r.m + i));
        vw[k] = ldg<true>((const FV*)(r.v + i));
        if (has_master) ww[k] = ldg<true>((const FV*)(r.master + i));
        else pw[k] = ldg<true>((const HV*)((const uint16_t*)r.p + i));
    }
#pragma unroll
    for (int k = 0; k < R; k++) {
        const int64_t i = i0 + k * SUB;
        float g[E], m[E], v[E], w[E];
        unpack_h<E>(gw[k], g);
        unpack_f<E>(mw[k], m);
        unpack_f<E>(vw[k], v);
        if (has_master) unpack_f<E>(ww[k], w);
        else unpack_h<E>(pw[k], w);
        if (clip) {
#pragma unroll
            for (int e = 0; e < E; e++) g[e] = clip_f16(g[e], scale);
        }
#pragma unroll
        for (int e = 0; e < E; e++) adamw_elem(g[e], m[e], v[e], w[e], h, wd);
        st_stream<SP>((FV*)(r.m + i), pack_f<E>(m));
        st_stream<SP>((FV*)(r.v + i), pack_f<E>(v));
        if (has_master) st_stream<SP>((FV*)(r.master + i), pack_f<E>(w));
        st_stream<SP>((HV*)((uint16_t*)r.p + i), pack_h<E>(w));
        if (zero_grads) st_stream<SP>((HV*)((uint16_t*)r.g + i), HV{});
    }
}

template <int E, int BLOCK, int R, int SP, bool CLIP>
__global__ __launch_bounds__(BLOCK) void adamw_rounds_kernel(
    const ChunkRec* __restrict__ recs, int64_t first_tile, int64_t n_tiles, int tiles_per_chunk_log2, Hyper h,
    const rlx_step_params* __restrict__ dev_params, const NormResult* __restrict__ norm, uint32_t step_flags)
{
    constexpr int TILE = E * BLOCK * R;
    const int64_t tile = first_tile + blockIdx.x;
    if (tile >= n_tiles) return;
    const ChunkRec r = recs[tile >> tiles_per_chunk_log2];
    const int64_t off = (tile & ((1 << tiles_per_chunk_log2) - 1)) * TILE;
    update_tile_rounds<E, BLOCK, R, SP, CLIP>(r, off, (int64_t)r.count - off, threadIdx.x, h, dev_params, norm, step_flags);
}

// ---------------------------------------------------------------------------------------
// Update kernel, the shipped form: one workgroup of BLOCK lanes per tile of E*BLOCK elements.
// K > 1: workgroups b, b+8, ... land on the same XCD; groups of 8*K tiles are permuted so
// that each XCD gets K neighbouring tiles.
// SINGLE: one flat tensor passed by value (the operator API); otherwise the plan's records.
// ---------------------------------------------------------------------------------------

template <int E, int BLOCK, int K, bool SINGLE, int SP, int PH, bool NTL, bool CLIP, bool REV = false>
__global__ __launch_bounds__(BLOCK) void adamw_tile_kernel(
    const ChunkRec* __restrict__ recs, ChunkRec single, int64_t single_n, int64_t first_tile, int64_t n_tiles,
    int tiles_per_chunk_log2, Hyper h, const rlx_step_params* __restrict__ dev_params,
    const NormResult* __restrict__ norm, uint32_t step_flags)
{
    constexpr int TILE = E * BLOCK;
    int64_t b = blockIdx.x;
    if constexpr (K > 1) {
        const int64_t grp = b / (8 * K), r = b % (8 * K);
        b = grp * (8 * K) + (r % 8) * K + (r / 8);
    }
    int64_t tile = first_tile + b;
    if (tile >= n_tiles) return;
    if constexpr (REV) tile = n_tiles - 1 - tile;     // from the end of the table to its start

    ChunkRec r;
    int64_t off;         // first element of the tile, relative to r's pointers
    int64_t left;        // elements from there to the end of the chunk / tensor
    if constexpr (SINGLE) {
        r = single;
        off = tile * TILE;
        left = single_n - off;
    } else {
        r = recs[tile >> tiles_per_chunk_log2];
        off = (tile & ((1 << tiles_per_chunk_log2) - 1)) * TILE;
        left = (int64_t)r.count - off;
    }
    update_tile<E, BLOCK, SP, PH, NTL, CLIP>(r, off, left, threadIdx.x, h, dev_params, norm, step_flags);
}

// ---------------------------------------------------------------------------------------
// Two other shapes of the same update, kept compiled so that the choice of the shipped one can be measured
// again at any time (tuning key "update_variant"); they give the same bits.
//
// adamw_persistent_kernel: a grid sized to the device (a fixed number of workgroups per CU) whose wavefronts
// stride over the tiles, 8 elements per lane: one 128-bit access per FP16 stream and two per FP32 stream.
// adamw_chunk_kernel: one workgroup per chunk that walks its chunk in groups of E*BLOCK elements.
// ---------------------------------------------------------------------------------------

template <int E, int WAVES, int SP, bool NTL, bool CLIP>
__global__ __launch_bounds__(64 * WAVES) void adamw_persistent_kernel(
    const ChunkRec* __restrict__ recs, int64_t n_tiles, int tiles_per_chunk_log2, Hyper h,
    const rlx_step_params* __restrict__ dev_params, const NormResult* __restrict__ norm, uint32_t step_flags)
{
    constexpr int TILE = E * 64;                                  // one wavefront per tile
    const int wave = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6)), lane = threadIdx.x & 63;   // wave: uniform, so records come by scalar loads
    for (int64_t tile = (int64_t)blockIdx.x * WAVES + wave; tile < n_tiles; tile += (int64_t)gridDim.x * WAVES) {
        const ChunkRec r = recs[tile >> tiles_per_chunk_log2];
        const int64_t off = (tile & ((1 << tiles_per_chunk_log2) - 1)) * TILE;
        update_tile<E, 64, SP, 0, NTL, CLIP>(r, off, (int64_t)r.count - off, lane, h, dev_params, norm, step_flags);
    }
}

template <int E, int BLOCK, int SP, bool NTL, bool CLIP>
__global__ __launch_bounds__(BLOCK) void adamw_chunk_kernel(
    const ChunkRec* __restrict__ recs, int64_t first_chunk, int64_t n_chunks, Hyper h,
    const rlx_step_params* __restrict__ dev_params, const NormResult* __restrict__ norm, uint32_t step_flags)
{
    constexpr int TILE = E * BLOCK;
    const int64_t c = first_chunk + blockIdx.x;
    if (c >= n_chunks) return;
    const ChunkRec r = recs[c];
    for (int64_t off = 0; off < (int64_t)r.count; off += TILE)
        update_tile<E, BLOCK, SP, 0, NTL, CLIP>(r, off, (int64_t)r.count - off, threadIdx.x, h, dev_params, norm, step_flags);
}

// ---------------------------------------------------------------------------------------
// The norm.  Order of the sum (restated on the CPU by the test oracle), a pure function of the data and the plan:
//   1. per chunk: lane t of BLOCK = min(512, chunk_elems / 8) adds x*x of its 8-element groups t, t+BLOCK, ...
//      element by element into one FP32 accumulator; the 64 lanes of a wavefront combine by xor butterfly with
//      masks 32,16,8,4,2,1; the BLOCK/64 wavefront sums are added in FP64 in wavefront order: one FP64 partial
//      per chunk in the chunk's own slot;
//   2. plans with 512-element chunks (lists of thousands of small tensors) only: 16 consecutive chunk partials
//      are added in FP64, in index order, into one group partial (so that the last step reads a sixteenth);
//   3. the values of step 2 (of step 1 for larger chunks) are added in FP64 by 1,024 (virtual) threads, thread t
//      taking t, t+1024, ... in order, then by a halving tree.
// Steps 1-2 are one launch.  Step 3 is either a second launch of one workgroup, or the tail of the first launch:
// every workgroup takes a ticket when its partials are written, and the workgroup that draws the last ticket
// adds them up.  The tickets decide who adds, never in which order, so both forms give the same bits; no
// workgroup ever waits for another.
// ---------------------------------------------------------------------------------------

constexpr int kGroupChunks = 16;              // 512-element chunks per group partial
constexpr int kTicketGroup = 64;              // workgroups per first-level ticket counter
constexpr int kTicketStride = 16;             // 64-bit words from one counter to the next (128 bytes: a line each)
constexpr int64_t kMaxFusedWgs = 8192;        // largest grid whose last workgroup adds the partials itself
constexpr int64_t kTicketWords = (kMaxFusedWgs / kTicketGroup + 1) * kTicketStride;
static_assert(kStaticMaxGroups * kGroupChunks == kStaticMaxPartials, "the static scratch holds the partials and their groups");

// What the workgroup that finishes last needs for step 3.
struct NormTail {
    const double* values;        // per-chunk partials, or per-group partials for 512-element chunks
    int64_t n_values;
    float max_norm;
    NormResult* out;
    uint64_t* tickets;           // [0]: second-level counter; [(1 + g) * kTicketStride]: counter of workgroups
                                 // 64g .. 64g+63.  Never reset: every launch of the same grid adds the same
                                 // amount to each counter, and "last" is a ticket that completes a multiple of it.
    int64_t plain_below;         // > 0: the launch walks the chunks from the last to the first, and chunks with an
                                 // index below this are read with ordinary instead of non-temporal loads, so that
                                 // what the norm reads last, the start of the gradients, is what stays in the
                                 // last-level cache for the update that follows
};

// The sum, the norm and the clip scale (trainer.h:341-345: strict '>' and +1e-6f in the denominator).
__device__ __forceinline__ void write_norm_result(double sum_sq, float max_norm, NormResult* __restrict__ out) {
    const float norm = __builtin_sqrtf((float)sum_sq);
    float scale = 1.0f;
    if (norm > max_norm) scale = max_norm / (norm + 1e-6f);
    out->sum_sq = sum_sq;
    out->norm = norm;
    out->scale = scale;
}

// Step 3 by a workgroup of NTHREADS lanes: lane `tid` runs the virtual threads tid, tid + NTHREADS, ... of 1,024,
// each with an accumulator of its own, so the result does not depend on NTHREADS.  ROUNDS rounds of 1,024 values
// are requested before the first is added (in index order: the same sum as one at a time).  Slots beyond the end
// read as +0.0, which leaves a sum of squares (never negative zero) unchanged bit for bit.  COHERENT: the values
// were written by other workgroups of the same launch; they are read with device-scope loads.
// `lds`: 1,024 doubles.  Returns the total in every lane.
template <int NTHREADS, int ROUNDS, bool COHERENT>
__device__ __forceinline__ double fixed_order_sum(const double* vals, int64_t n, double* lds, int tid) {
    constexpr int V = kFinalBlock / NTHREADS;
    double a[V];
#pragma unroll
    for (int v = 0; v < V; v++) a[v] = 0.0;
    for (int64_t base = 0; base < n; base += (int64_t)ROUNDS * kFinalBlock) {
        double x[ROUNDS][V];
#pragma unroll
        for (int b = 0; b < ROUNDS; b++) {
#pragma unroll
            for (int v = 0; v < V; v++) {
                const int64_t j = base + (int64_t)b * kFinalBlock + v * NTHREADS + tid;
                double y = 0.0;
                if (j < n) {
                    if constexpr (COHERENT) y = __hip_atomic_load(vals + j, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                    else y = vals[j];
                }
                x[b][v] = y;
            }
        }
#pragma unroll
        for (int b = 0; b < ROUNDS; b++) {
#pragma unroll
            for (int v = 0; v < V; v++) a[v] += x[b][v];
        }
    }
#pragma unroll
    for (int v = 0; v < V; v++) lds[v * NTHREADS + tid] = a[v];
    __syncthreads();
    for (int s = kFinalBlock / 2; s >= 1; s >>= 1) {
        for (int i = tid; i < s; i += NTHREADS) lds[i] = lds[i] + lds[i + s];
        __syncthreads();
    }
    return lds[0];
}

// A value that the workgroup finishing last will add up: stored past the caches that other workgroups' loads
// could miss it in (a device-scope store).
__device__ __forceinline__ void publish(double* slot, double x) {
    __hip_atomic_store(slot, x, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// True in every lane of exactly one workgroup of the launch: the one that takes its ticket last.  Everything the
// final sum reads must have been stored with publish() by lanes of the workgroup's first wavefront before the call.
// Two levels of counters (64 workgroups share a first-level counter, the last of each 64 takes a second-level
// ticket), so that thousands of workgroups finishing together do not queue on one address (one counter for
// all: 12 ns per workgroup, 100 us for 8,192).
// The counters only ever count up (64 bits: they do not wrap): a launch of G workgroups adds the size of group g
// to counter g and the number of groups to the second-level counter, so as long as every launch on these counters
// has the same G (the host clears them when G changes), the ticket that completes a multiple of that amount is
// the launch's last.  Nothing has to be put back to zero, a recorded launch replays as it is, and two launches that
// overlap by mistake spoil each other's result but leave the counters at a multiple again for the launches after.
// Ordering: the published values are device-scope stores, the wavefront waits until they have been acknowledged
// and only then takes its ticket; the last workgroup reads them with device-scope loads after its ticket has
// come back.  A full device-scope fence in front of the ticket would do as well, but it writes the whole L2 back
// and measured 67 ns per workgroup, one after the other across the device (550 us for 8,192 workgroups).
__device__ __forceinline__ bool last_workgroup(uint64_t* tickets, int* lds_flag) {
    if (threadIdx.x < 64) {
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
        wait_for_memory();                  // this wavefront's published values have arrived before its ticket is taken
        if (threadIdx.x == 0) {
            const uint32_t n_wg = gridDim.x, grp = blockIdx.x / kTicketGroup;
            const uint32_t n_grp = (n_wg + kTicketGroup - 1) / kTicketGroup;
            const uint32_t in_grp = grp + 1 < n_grp ? (uint32_t)kTicketGroup : n_wg - grp * kTicketGroup;
            uint64_t* c1 = tickets + (size_t)(1 + grp) * kTicketStride;
            int last = 0;
            const uint64_t t1 = __hip_atomic_fetch_add(c1, (uint64_t)1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) + 1;
            if (t1 % in_grp == 0) {
                const uint64_t t0 = __hip_atomic_fetch_add(tickets, (uint64_t)1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) + 1;
                last = t0 % n_grp == 0;
            }
            *lds_flag = last;
        }
    }
    __syncthreads();
    const bool last = *lds_flag != 0;
    if (last) __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "agent");
    return last;
}

// Chunk c of a PoolPair as the record that a plan would hold for it (only the fields the norm reads).
__device__ __forceinline__ ChunkRec pool_chunk(const PoolPair& pp, int64_t c) {
    ChunkRec r;
    const int64_t chunk = (int64_t)1 << pp.chunk_log2;
    if (c < pp.chunks_half) {
        const int64_t start = c << pp.chunk_log2, left = pp.n_half - start;
        r.g = (void*)(pp.half_pool + start);
        r.count = (uint32_t)(left < chunk ? left : chunk);
        r.flags = pp.flags_half;
    } else {
        const int64_t start = (c - pp.chunks_half) << pp.chunk_log2, left = pp.n_float - start;
        r.g = (void*)(pp.float_pool + start);
        r.count = (uint32_t)(left < chunk ? left : chunk);
        r.flags = pp.flags_float;
    }
    return r;
}

// Sum of squares of this lane's share of one chunk: lane `tid` of BLOCK adds its 8-element groups tid,
// tid + BLOCK, ... element by element into one FP32 accumulator.
template <bool NT, int BLOCK>
__device__ __forceinline__ float chunk_lane_sumsq(const ChunkRec& r, int tid) {
    constexpr int kNormGroup = BLOCK * kVec;
    const int64_t count = r.count;
    const bool aligned = ((r.flags >> kGalignShift) & 0xF) >= 8;
    float acc = 0.0f;
    if (r.flags & RLX_TENSOR_FROZEN) {
        // gradients of a frozen tensor count as zero (the reference clears them before the norm)
    } else if (!(r.flags & kF32)) {
        const uint16_t* g = (const uint16_t*)r.g;
        int64_t done = 0;
        if (aligned) {
            for (; done + 2 * (int64_t)kNormGroup <= count; done += 2 * (int64_t)kNormGroup) {
                u32x4 x[2];
#pragma unroll
                for (int j = 0; j < 2; j++)
                    x[j] = ldg<NT>((const u32x4*)(g + done + (int64_t)(j * BLOCK + tid) * kVec));
#pragma unroll
                for (int j = 0; j < 2; j++) {
#pragma unroll
                    for (int k = 0; k < 4; k++) {
                        float a = h2f(x[j][k] & 0xFFFFu), b = h2f(x[j][k] >> 16);
                        acc = acc + a * a;
                        acc = acc + b * b;
                    }
                }
            }
        }
        for (; done < count; done += kNormGroup) {
            const int64_t off = done + (int64_t)tid * kVec;
            if (aligned && off + kVec <= count) {
                u32x4 x = ldg<NT>((const u32x4*)(g + off));
#pragma unroll
                for (int k = 0; k < 4; k++) {
                    float a = h2f(x[k] & 0xFFFFu), b = h2f(x[k] >> 16);
                    acc = acc + a * a;
                    acc = acc + b * b;
                }
            } else if (aligned && off < count) {
                // the tensor's last, partial group: its 16-byte granule starts inside the tensor, so one
                // aligned load cannot leave the tensor's last page; what lies beyond the end is read but
                // counts as zero (acc + 0 leaves a sum of squares as it is).  Element by element this
                // lane would wait for up to seven loads one after another, and its workgroup with it.
                u32x4 x = ldg<NT>((const u32x4*)(g + off));
                const int valid = (int)(count - off);
#pragma unroll
                for (int k = 0; k < 4; k++) {
                    float a = 2 * k < valid ? h2f(x[k] & 0xFFFFu) : 0.0f;
                    float b = 2 * k + 1 < valid ? h2f(x[k] >> 16) : 0.0f;
                    acc = acc + a * a;
                    acc = acc + b * b;
                }
            } else {
                for (int64_t i = off; i < off + kVec && i < count; i++) {
                    float a = h2f(ldg<NT>(g + i));
                    acc = acc + a * a;
                }
            }
        }
    } else {
        const float* g = (const float*)r.g;
        for (int64_t done = 0; done < count; done += kNormGroup) {
            const int64_t off = done + (int64_t)tid * kVec;
            if (aligned && off + kVec <= count) {
                f32x4 x0 = ldg<NT>((const f32x4*)(g + off)), x1 = ldg<NT>((const f32x4*)(g + off) + 1);
#pragma unroll
                for (int k = 0; k < 4; k++) acc = acc + x0[k] * x0[k];
#pragma unroll
                for (int k = 0; k < 4; k++) acc = acc + x1[k] * x1[k];
            } else if (aligned && off < count) {
                // partial last group, as above; the second 16-byte granule is only read if it starts inside
                const int valid = (int)(count - off);
                f32x4 x0 = ldg<NT>((const f32x4*)(g + off)), x1 = {0.0f, 0.0f, 0.0f, 0.0f};
                if (valid > 4) x1 = ldg<NT>((const f32x4*)(g + off) + 1);
#pragma unroll
                for (int k = 0; k < 4; k++) { const float a = k < valid ? x0[k] : 0.0f; acc = acc + a * a; }
#pragma unroll
                for (int k = 0; k < 4; k++) { const float a = 4 + k < valid ? x1[k] : 0.0f; acc = acc + a * a; }
            } else {
                for (int64_t i = off; i < off + kVec && i < count; i++) {
                    float a = ldg<NT>(g + i);
                    acc = acc + a * a;
                }
            }
        }
    }
    return acc;
}

// Step 1, general form: one workgroup of BLOCK lanes per chunk (512 lanes with two 128-bit reads each measured
// 7.3 TB/s as a stand-alone stream, 256 lanes with four 6.95).
// POOLS: the chunks come from `pools` (two flat buffers passed by value) instead of the table `recs`.
// PACK > 1 (only with BLOCK = 64, i.e. 512-element chunks; kept for comparison): the workgroup has PACK wavefronts
// and each takes a chunk of its own.
// FUSED (chunks of 1,024 elements and more): the workgroup that finishes last also runs step 3.
template <bool NT, int BLOCK, bool POOLS, int PACK, bool FUSED>
__global__ __launch_bounds__(BLOCK * PACK) void sumsq_partials_kernel(
    const ChunkRec* __restrict__ recs, PoolPair pools, int64_t n_chunks, double* partials, NormTail tail)
{
    static_assert(PACK == 1 || BLOCK == 64, "several chunks per workgroup only with one wavefront per chunk");
    static_assert(!FUSED || (PACK == 1 && BLOCK >= 128), "512-element chunks have a kernel of their own");
    __shared__ float wave_sum[BLOCK / 64];
    // which of the workgroup's PACK chunks: the wavefront's number, made known to the compiler as uniform
    // across the wavefront so that the chunk's record is still fetched with scalar loads
    const int tid = PACK == 1 ? (int)threadIdx.x : (int)(threadIdx.x & 63);
    const int sub = PACK == 1 ? 0 : __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));

    for (int64_t i = (int64_t)blockIdx.x * PACK + sub; i < n_chunks; i += (int64_t)gridDim.x * PACK) {
        const int64_t c = tail.plain_below > 0 ? n_chunks - 1 - i : i;      // the slot is the chunk's: same sum either way
        ChunkRec r;
        if constexpr (POOLS) r = pool_chunk(pools, c);
        else r = recs[c];
        float acc;
        if (NT && c < tail.plain_below) acc = chunk_lane_sumsq<false, BLOCK>(r, tid);
        else acc = chunk_lane_sumsq<NT, BLOCK>(r, tid);
#pragma unroll
        for (int mask = 32; mask >= 1; mask >>= 1) acc = acc + __shfl_xor(acc, mask, 64);
        if constexpr (BLOCK == 64) {
            // one wavefront per chunk: its sum is the chunk's partial (0.0 + x in FP64, as below, is x)
            if (tid == 0) partials[c] = (double)acc;
        } else {
            if ((tid & 63) == 0) wave_sum[tid >> 6] = acc;
            __syncthreads();
            if (tid == 0) {
                double total = 0.0;
#pragma unroll
                for (int w = 0; w < BLOCK / 64; w++) total += (double)wave_sum[w];
                if constexpr (FUSED) publish(&partials[c], total);
                else partials[c] = total;
            }
            __syncthreads();
        }
    }

    if constexpr (FUSED) {
        __shared__ double tree[kFinalBlock];
        __shared__ int last_flag;
        if (last_workgroup(tail.tickets, &last_flag)) {
            const double sum_sq = fixed_order_sum<BLOCK, 16 * BLOCK / kFinalBlock, true>(tail.values, tail.n_values, tree,
                                                                                       (int)threadIdx.x);
            if (threadIdx.x == 0) write_norm_result(sum_sq, tail.max_norm, tail.out);
        }
    }
}

// Steps 1 and 2 for 512-element chunks (lists of thousands of small tensors): a chunk is at most one 8-element
// group per lane of one wavefront, so a wavefront takes CPW consecutive chunks at once (records and data of all
// of them requested before the first is used) and a workgroup of WAVES wavefronts WAVES * CPW chunks, a whole
// number of groups.  With one chunk per wavefront the pass is bound by latency: record, data, butterfly, one
// after another, for each of tens of thousands of chunks.  The sum inside a chunk and its slot are those of the
// general kernel above with BLOCK = 64 (lane t adds its group's elements in order, xor butterfly).
// FUSED: the workgroup that finishes last also runs step 3 over the group partials.
template <bool NT, bool POOLS, int WAVES, int CPW, bool FUSED>
__global__ __launch_bounds__(64 * WAVES) void sumsq_small_chunks_kernel(
    const ChunkRec* __restrict__ recs, PoolPair pools, int64_t n_chunks, double* partials, double* groups, NormTail tail)
{
    constexpr int PER_WG = WAVES * CPW, GROUPS_PER_WG = PER_WG / kGroupChunks;
    static_assert(PER_WG % kGroupChunks == 0, "a workgroup covers whole groups of chunks");
    __shared__ double chunk_sum[PER_WG];
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));    // uniform: records by scalar loads
    const int64_t first = ((int64_t)blockIdx.x * WAVES + wave) * CPW;

    const char* g[CPW];
    int valid[CPW];          // elements of chunk j that belong to this lane's group (0..8)
    bool f32[CPW], fast[CPW];
    u32x4 a[CPW], b[CPW];
#pragma unroll
    for (int j = 0; j < CPW; j++) {
        ChunkRec r;
        r.g = nullptr; r.count = 0; r.flags = 0;
        if (first + j < n_chunks) {
            if constexpr (POOLS) r = pool_chunk(pools, first + j);
            else r = recs[first + j];
        }
        g[j] = (const char*)r.g;
        f32[j] = (r.flags & kF32) != 0;
        fast[j] = ((r.flags >> kGalignShift) & 0xF) >= 8;
        int left = (r.flags & RLX_TENSOR_FROZEN) ? 0 : (int)r.count - lane * kVec;   // a frozen tensor counts as zero
        valid[j] = left < 0 ? 0 : left > kVec ? kVec : left;
    }
#pragma unroll
    for (int j = 0; j < CPW; j++) {
        a[j] = u32x4{0u, 0u, 0u, 0u};
        b[j] = u32x4{0u, 0u, 0u, 0u};
        // aligned chunks: whole 16-byte granules that start inside the tensor (what lies beyond its end is
        // read but not used, see the general kernel)
        if (fast[j] && valid[j] > 0) {
            const u32x4* src = (const u32x4*)(g[j] + (size_t)lane * (f32[j] ? 32 : 16));
            a[j] = ldg<NT>(src);
            if (f32[j] && valid[j] > 4) b[j] = ldg<NT>(src + 1);
        }
    }
#pragma unroll
    for (int j = 0; j < CPW; j++) {
        float acc = 0.0f;
        if (fast[j]) {
            if (!f32[j]) {
#pragma unroll
                for (int k = 0; k < 4; k++) {
                    const float x = 2 * k < valid[j] ? h2f(a[j][k] & 0xFFFFu) : 0.0f;
                    const float y = 2 * k + 1 < valid[j] ? h2f(a[j][k] >> 16) : 0.0f;
                    acc = acc + x * x;
                    acc = acc + y * y;
                }
            } else {
#pragma unroll
                for (int k = 0; k < 4; k++) {
                    const uint32_t w = a[j][k];      // (a bit cast applied directly to a vector element took element 0 every time)
                    const float x = k < valid[j] ? __builtin_bit_cast(float, w) : 0.0f;
                    acc = acc + x * x;
                }
#pragma unroll
                for (int k = 0; k < 4; k++) {
                    const uint32_t w = b[j][k];
                    const float x = 4 + k < valid[j] ? __builtin_bit_cast(float, w) : 0.0f;
                    acc = acc + x * x;
                }
            }
        } else {
            for (int e = 0; e < valid[j]; e++) {          // a chunk that is not 16-byte aligned: element by element
                const float x = f32[j] ? ldg<NT>((const float*)g[j] + lane * kVec + e)
                                       : h2f(ldg<NT>((const uint16_t*)g[j] + lane * kVec + e));
                acc = acc + x * x;
            }
        }
#pragma unroll
        for (int mask = 32; mask >= 1; mask >>= 1) acc = acc + __shfl_xor(acc, mask, 64);
        if (lane == 0) {
            const bool exists = first + j < n_chunks;
            if (exists) partials[first + j] = (double)acc;
            chunk_sum[wave * CPW + j] = exists ? (double)acc : 0.0;     // +0.0 leaves the group's sum as it is
        }
    }
    __syncthreads();
    if (threadIdx.x < GROUPS_PER_WG) {
        const int64_t grp = (int64_t)blockIdx.x * GROUPS_PER_WG + threadIdx.x;
        if (grp * kGroupChunks < n_chunks) {
            double total = 0.0;
#pragma unroll
            for (int k = 0; k < kGroupChunks; k++) total += chunk_sum[threadIdx.x * kGroupChunks + k];
            if constexpr (FUSED) publish(&groups[grp], total);
            else groups[grp] = total;
        }
    }
    if constexpr (FUSED) {
        __shared__ double tree[kFinalBlock];
        __shared__ int last_flag;
        if (last_workgroup(tail.tickets, &last_flag)) {
            const double sum_sq = fixed_order_sum<64 * WAVES, 16 * 64 * WAVES / kFinalBlock, true>(
                tail.values, tail.n_values, tree, (int)threadIdx.x);
            if (threadIdx.x == 0) write_norm_result(sum_sq, tail.max_norm, tail.out);
        }
    }
}

// Step 2 as a launch of its own, for the forms of step 1 that have fewer than 16 chunks per workgroup (kept for
// comparison): one lane per group adds the group's chunk partials in index order.
__global__ __launch_bounds__(256) void sumsq_group_kernel(const double* __restrict__ partials, int64_t n_chunks,
                                                          double* __restrict__ groups)
{
    const int64_t grp = (int64_t)blockIdx.x * 256 + threadIdx.x;
    const int64_t first = grp * kGroupChunks;
    if (first >= n_chunks) return;
    double total = 0.0;
    for (int k = 0; k < kGroupChunks; k++) total += first + k < n_chunks ? partials[first + k] : 0.0;
    groups[grp] = total;
}

// Step 3 as a launch of its own: one workgroup of 1,024 lanes.  BATCH: rounds of loads in flight per lane.
template <int BATCH>
__global__ __launch_bounds__(kFinalBlock) void sumsq_final_kernel(
    const double* __restrict__ values, int64_t n_values, float max_norm, NormResult* __restrict__ out)
{
    __shared__ double tree[kFinalBlock];
    const double sum_sq = fixed_order_sum<kFinalBlock, BATCH, false>(values, n_values, tree, (int)threadIdx.x);
    if (threadIdx.x == 0) write_norm_result(sum_sq, max_norm, out);
}

// In-place scale of the gradients (trainer.h:136-145).  Exactly 1.0f: nothing is touched.
// One workgroup per 2,048 elements of a chunk (256 lanes, one 128-bit access each way per lane):
// 6.6 TB/s on Qwen3-0.6B against 5.7 TB/s for one workgroup looping over a whole chunk; 256-element
// tiles as in the update kernel are too small here (4 bytes per element: dispatch-bound, 2.8-4.7 TB/s).
template <int BLOCK>
__global__ __launch_bounds__(BLOCK) void scale_group_kernel(
    const ChunkRec* __restrict__ recs, int64_t first_tile, int64_t n_tiles, int tiles_per_chunk_log2,
    const NormResult* __restrict__ norm)
{
    constexpr int TILE = BLOCK * kVec;
    const float scale = norm->scale;
    if (scale == 1.0f) return;
    const int64_t tile = first_tile + blockIdx.x;
    if (tile >= n_tiles) return;
    const ChunkRec r = recs[tile >> tiles_per_chunk_log2];
    if (r.flags & RLX_TENSOR_FROZEN) return;
    const int64_t base = (tile & ((1 << tiles_per_chunk_log2) - 1)) * TILE;
    const int64_t count = r.count;
    const int64_t off = base + (int64_t)threadIdx.x * kVec;
    if (off >= count) return;
    const bool aligned = ((r.flags >> kGalignShift) & 0xF) >= 8;
    if (!(r.flags & kF32)) {
        uint16_t* g = (uint16_t*)r.g;
        if (aligned && off + kVec <= count) {
            u32x4 x = ldg<true>((const u32x4*)(g + off));
#pragma unroll
            for (int k = 0; k < 4; k++)
                x[k] = scaled_f16_bits(h2f(x[k] & 0xFFFFu), scale) | (scaled_f16_bits(h2f(x[k] >> 16), scale) << 16);
            st_stream<1>((u32x4*)(g + off), x);
        } else {
            for (int64_t i = off; i < off + kVec && i < count; i++) g[i] = (uint16_t)scaled_f16_bits(h2f(g[i]), scale);
        }
    } else {
        float* g = (float*)r.g;
        if (aligned && off + kVec <= count) {
            f32x4 x0 = ldg<true>((const f32x4*)(g + off)), x1 = ldg<true>((const f32x4*)(g + off) + 1);
#pragma unroll
            for (int k = 0; k < 4; k++) { x0[k] = x0[k] * scale; x1[k] = x1[k] * scale; }
            st_stream<1>((f32x4*)(g + off), x0);
            st_stream<1>((f32x4*)(g + off) + 1, x1);
        } else {
            for (int64_t i = off; i < off + kVec && i < count; i++) g[i] = g[i] * scale;
        }
    }
}

// x[i] *= scale for a plain FP32 buffer (the per-micro-batch loss-gradient scale, trainer.h:96-99).
// The buffer is small (one value per token); 128-bit accesses when it is 16-byte aligned.
__global__ __launch_bounds__(256) void scale_f32_kernel(float* __restrict__ x, float scale, int64_t n, int vec_ok) {
    const int64_t i = ((int64_t)blockIdx.x * 256 + threadIdx.x) * 4;
    if (i >= n) return;
    if (vec_ok && i + 4 <= n) {
        f32x4 v = ldg<false>((const f32x4*)(x + i));
#pragma unroll
        for (int k = 0; k < 4; k++) v[k] = v[k] * scale;
        stg<false>((f32x4*)(x + i), v);
    } else {
        for (int64_t j = i; j < i + 4 && j < n; j++) x[j] = x[j] * scale;
    }
}

// dst[i] = (float)src[i] as a stream (the FP32 master copy made from the FP16 weights, optimizer.h:46-57,242).
// One workgroup of LANES lanes per LANES*E*ROUNDS elements (shipped: 128 lanes x 4 elements, one round: a
// 64-bit load and a 128-bit store per lane); per lane and round one access of E halves and one of E floats, every instruction contiguous across the wavefront, all loads issued before the first use,
// non-temporal loads and system-scope non-temporal stores.  Workgroups whose span is not whole or not aligned
// go element by element.
template <int LANES, int E, int ROUNDS>
__global__ __launch_bounds__(LANES) void convert_tile_kernel(float* __restrict__ dst, const uint16_t* __restrict__ src,
                                                             int64_t n, int vec_ok)
{
    constexpr int PER = LANES * E;
    typedef typename Lane<E>::H HV;
    typedef typename Lane<E>::F FV;
    const int64_t base = (int64_t)blockIdx.x * (PER * ROUNDS) + (int64_t)threadIdx.x * E;
    if (vec_ok && (int64_t)(blockIdx.x + 1) * (PER * ROUNDS) <= n) {
        HV x[ROUNDS];
#pragma unroll
        for (int r = 0; r < ROUNDS; r++) x[r] = ldg<true>((const HV*)(src + base + r * PER));
#pragma unroll
        for (int r = 0; r < ROUNDS; r++) {
            float f[E];
            unpack_h<E>(x[r], f);
            st_stream<1>((FV*)(dst + base + r * PER), pack_f<E>(f));
        }
    } else {
        for (int r = 0; r < ROUNDS; r++)
            for (int e = 0; e < E; e++) {
                const int64_t i = base + r * PER + e;
                if (i < n) dst[i] = h2f(src[i]);
            }
    }
}

// The plain form: one element per lane, grid-stride (kept for comparison: tuning key "convert_variant" = 2).
__global__ __launch_bounds__(256) void fp16_to_fp32_kernel(float* __restrict__ dst,
                                                           const uint16_t* __restrict__ src, int64_t n)
{
    for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < n; i += (int64_t)gridDim.x * 256)
        dst[i] = h2f(src[i]);
}

// After an update that read the current entry of a plan's step table: move on to the next entry, so that the
// next (replayed) update reads new hyper-parameters without the host.  The launch names only the header, whose
// address never changes while the plan lives; the table's address and length are read from it at run time, so a
// recorded launch follows every later upload, whatever its length.  Beyond the end of the table the last entry
// stays current; `taken` counts the scheduled steps so far, saturating at the length, and `overrun` counts the
// updates that ran with the last entry again because the table had been used up.
__global__ __launch_bounds__(64) void schedule_advance_kernel(SchedHeader* __restrict__ hdr)
{
    if (threadIdx.x != 0 || blockIdx.x != 0) return;
    const int64_t n = hdr->len, done = hdr->taken;
    if (done >= n) { hdr->overrun = hdr->overrun + 1; return; }      // this update read a used-up table
    const int64_t next = done + 1;
    if (next < n) hdr->current = hdr->table[next];
    hdr->taken = next;
}

// Zero fill as a kernel (a memset node recorded into a HIP graph is not reliable on every
// runtime; a kernel is).  One workgroup of 256 lanes per 4 KiB: one 128-bit store per lane.
// `body` points at a 16-byte boundary; the few bytes before and after it are written by the host
// launcher's second, byte-wise launch.
__global__ __launch_bounds__(256) void clear_body_kernel(u32x4* __restrict__ body, int64_t n_vec) {
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i < n_vec) st_stream<1>(body + i, u32x4{0u, 0u, 0u, 0u});
}

__global__ __launch_bounds__(64) void clear_edges_kernel(uint8_t* __restrict__ head, int n_head,
                                                         uint8_t* __restrict__ tail, int n_tail) {
    const int t = threadIdx.x;
    if (t < n_head) head[t] = 0;
    if (t < n_tail) tail[t] = 0;
}

// ---------------------------------------------------------------------------------------
// Seeded synthetic inputs: integer hash -> sum of eight 16-bit uniforms -> one FP32
// multiply and one FP32 add, so that a host restatement gives the same bits without libm.
// ---------------------------------------------------------------------------------------

constexpr int kFillBlock = 256;

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
__global__ __launch_bounds__(kFillBlock) void fill_kernel(T* __restrict__ dst, int64_t n, uint64_t seed, int64_t first,
                                                      float mean, float std, uint32_t flags, int64_t row_len,
                                                      uint32_t zero_rows_below)
{
    for (int64_t i = (int64_t)blockIdx.x * kFillBlock + threadIdx.x; i < n; i += (int64_t)gridDim.x * kFillBlock) {
        const float x = fill_value(seed, (uint64_t)(first + i), mean, std, flags, row_len, zero_rows_below);
        if constexpr (sizeof(T) == 2) dst[i] = (uint16_t)f2h(x);
        else dst[i] = x;
    }
}

// ---------------------------------------------------------------------------------------
// Host side
// ---------------------------------------------------------------------------------------

thread_local char g_hip_error[256] = "";

constexpr int kMaxDevices = 64;
std::mutex g_scratch_mutex;
double* g_scratch_ptr[kMaxDevices];      // device address of `scratch` on each device; null until first used there

int hip_fail(hipError_t e, const char* what) {
    snprintf(g_hip_error, sizeof(g_hip_error), "%s: %s", what, hipGetErrorString(e));
    return RLX_ERR_HIP;
}

#define RLX_HIP(call)                                        \
    do {                                                     \
        hipError_t e_ = (call);                              \
        if (e_ != hipSuccess) return hip_fail(e_, #call);    \
    } while (0)

// Process-wide launch tuning (for measurement).  Atomic, so that a thread that changes a key while another
// launches is a defined race: every launch reads each key once and uses one consistent choice.
struct Tuning {
    std::atomic<int64_t> update_variant{0};
    std::atomic<int64_t> norm_grid{0};
    std::atomic<int64_t> norm_nt{1};
    std::atomic<int64_t> norm_pack{3};      // 512-element chunks per workgroup: 0 = one, 1 = eight (a wavefront each),
                                            // 2 = thirty-two (four per wavefront), 3 = sixteen (two per wavefront,
                                            // one group partial per workgroup: the default)
    std::atomic<int64_t> convert_variant{0};
    std::atomic<int64_t> final_batch{0};    // loads in flight per lane in the second pass of the norm; 0 = by the number of partials
    std::atomic<int64_t> norm_keep_mb{0};   // > 0: the norm walks its chunks backwards and reads the first that many MB of
                                            // gradients, last in time, with ordinary loads (they stay cached for the update)
    std::atomic<int64_t> update_reverse{0}; // 1: the fused-clip update walks the tile table from its end to its start
    std::atomic<int64_t> norm_fused{2};     // the fixed-order sum of the partials: 0 = always a second launch, 1 = by the
                                            // workgroup of the first launch that finishes last whenever that launch
                                            // has at most 8,192 workgroups, 2 = that up to 256 workgroups (default)
} g_tuning;

constexpr int kNumUpdateVariants = 18;
constexpr int kNumConvertVariants = 4;
constexpr int64_t kMaxTilesPerLaunch = 1 << 23;   // workgroups per launch; times 256 lanes stays below 2^32
constexpr int64_t kMaxNormGrid = 1 << 22;

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

int check_desc(const rlx_tensor_desc& d) {
    if (d.n <= 0 || !d.grad) return RLX_ERR_INVALID_ARG;
    if (d.dtype != RLX_DTYPE_F16 && d.dtype != RLX_DTYPE_F32) return RLX_ERR_INVALID_ARG;
    if (d.flags & ~(uint32_t)(RLX_TENSOR_NO_DECAY | RLX_TENSOR_GRAD_ONLY | RLX_TENSOR_FROZEN)) return RLX_ERR_INVALID_ARG;
    const bool grad_only = (d.flags & RLX_TENSOR_GRAD_ONLY) != 0;
    if (!grad_only && (!d.param || !d.m || !d.v)) return RLX_ERR_INVALID_ARG;
    if (d.master && d.dtype != RLX_DTYPE_F16) return RLX_ERR_INVALID_ARG;
    const size_t es = d.dtype == RLX_DTYPE_F16 ? 2 : 4;
    if (!is_aligned(d.grad, es) || !is_aligned(d.param, es) || !is_aligned(d.m, 4) || !is_aligned(d.v, 4) ||
        !is_aligned(d.master, 4))
        return RLX_ERR_MISALIGNED;
    return RLX_OK;
}

// Default chunk size: big chunks for big tensors; for a list of many small tensors a smaller chunk
// wastes fewer workgroups on the empty part of each tensor's last chunk.
int64_t default_chunk(int64_t n_elems, int64_t n_tensors) {
    const int64_t mean = n_elems / n_tensors;
    int64_t chunk = mean >= 4 * kBigChunk ? kBigChunk : mean >= 4 * kSmallChunk ? kSmallChunk : kMinChunk;
    // very large lists: keep the number of partials that the single-workgroup second pass of the norm
    // has to read near 2^18 (the update is equally fast with chunks from 8,192 to 65,536 elements)
    while (chunk >= kBigChunk && chunk < 65536 && n_elems / chunk > (1 << 18)) chunk *= 2;
    return chunk;
}

inline bool chunk_ok(int64_t chunk) { return chunk >= kMinChunk && chunk <= (1 << 24) && (chunk & (chunk - 1)) == 0; }

// Record of the chunk that starts `start` elements into the tensor.
ChunkRec make_rec(const rlx_tensor_desc& d, int64_t start, int64_t count) {
    const size_t es = d.dtype == RLX_DTYPE_F16 ? 2 : 4;
    ChunkRec r;
    r.p = d.param ? (char*)d.param + start * es : nullptr;
    r.g = (char*)d.grad + start * es;
    r.m = d.m ? d.m + start : nullptr;
    r.v = d.v ? d.v + start : nullptr;
    r.master = d.master ? d.master + start : nullptr;
    r.count = (uint32_t)count;
    r.flags = d.flags | (d.dtype == RLX_DTYPE_F32 ? kF32 : 0u);
    r.pad[0] = r.pad[1] = 0;
    uint32_t valign = 1;
    for (uint32_t e = 8; e > 1; e >>= 1) {
        if (is_aligned(r.p, e * es) && is_aligned(r.g, e * es) && is_aligned(r.m, e * 4) && is_aligned(r.v, e * 4) &&
            is_aligned(r.master, e * 4)) {
            valign = e;
            break;
        }
    }
    r.flags |= valign << kValignShift;
    uint32_t galign = 1;
    for (uint32_t e = 8; e > 1; e >>= 1) {
        if (is_aligned(r.g, e * es)) {
            galign = e;
            break;
        }
    }
    r.flags |= galign << kGalignShift;
    return r;
}

// Every launch is checked where it is made, so that a failure names the launch: returns hipSuccess or the
// first error.
template <int E, int BLOCK, int K, bool SINGLE, int SP, int PH = 0, bool NTL = true>
hipError_t launch_variant(const ChunkRec* recs, const ChunkRec& single, int64_t single_n, int64_t n_elems_or_chunks,
                          int chunk_log2, const Hyper& h, const rlx_step_params* dev_params, const NormResult* norm,
                          uint32_t step_flags, hipStream_t s) {
    constexpr int TILE = E * BLOCK;
    int64_t n_tiles;
    int tpc_log2 = 0;
    if constexpr (SINGLE) {
        n_tiles = (n_elems_or_chunks + TILE - 1) / TILE;
    } else {
        tpc_log2 = chunk_log2 - __builtin_ctz(TILE);
        n_tiles = n_elems_or_chunks << tpc_log2;          // n_chunks * tiles per chunk
    }
    for (int64_t first = 0; first < n_tiles; first += kMaxTilesPerLaunch) {
        int64_t here = n_tiles - first < kMaxTilesPerLaunch ? n_tiles - first : kMaxTilesPerLaunch;
        here = (here + 8 * K - 1) / (8 * K) * (8 * K);   // whole swizzle groups; the excess exits at once
        bool reversed = false;
        if constexpr (E == 2 && BLOCK == 128 && K == 1 && !SINGLE && SP == 1 && NTL) reversed = norm && g_tuning.update_reverse != 0;
        if (reversed) {
            if constexpr (E == 2 && BLOCK == 128 && K == 1 && !SINGLE && SP == 1 && NTL)
                adamw_tile_kernel<E, BLOCK, K, SINGLE, SP, PH, NTL, true, true><<<dim3((unsigned)here), dim3(BLOCK), 0, s>>>(
                    recs, single, single_n, first, n_tiles, tpc_log2, h, dev_params, norm, step_flags);
        } else if (norm)
            adamw_tile_kernel<E, BLOCK, K, SINGLE, SP, PH, NTL, true><<<dim3((unsigned)here), dim3(BLOCK), 0, s>>>(
                recs, single, single_n, first, n_tiles, tpc_log2, h, dev_params, norm, step_flags);
        else
            adamw_tile_kernel<E, BLOCK, K, SINGLE, SP, PH, NTL, false><<<dim3((unsigned)here), dim3(BLOCK), 0, s>>>(
                recs, single, single_n, first, n_tiles, tpc_log2, h, dev_params, norm, step_flags);
        const hipError_t e = hipGetLastError();
        if (e != hipSuccess) return e;
    }
    return hipSuccess;
}

// Workgroups per CU of the persistent form: four wavefronts each, eight fill a CU's wavefront slots.
constexpr int kPersistentWaves = 4, kPersistentPerCU = 8;

int compute_units() {
    static int cached[kMaxDevices];
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return 256;
    if (!cached[dev]) {
        int cu = 0;
        if (hipDeviceGetAttribute(&cu, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cu <= 0) cu = 256;
        cached[dev] = cu;
    }
    return cached[dev];
}

template <int SP, bool NTL>
hipError_t launch_persistent(const ChunkRec* recs, int64_t n_chunks, int chunk_log2, const Hyper& h,
                             const rlx_step_params* dev_params, const NormResult* norm, uint32_t step_flags,
                             hipStream_t s) {
    constexpr int E = 8, TILE = E * 64;
    const int tpc_log2 = chunk_log2 - __builtin_ctz(TILE);
    const int64_t n_tiles = n_chunks << tpc_log2;
    int64_t grid = (int64_t)compute_units() * kPersistentPerCU;
    const int64_t need = (n_tiles + kPersistentWaves - 1) / kPersistentWaves;
    if (grid > need) grid = need;
    if (norm)
        adamw_persistent_kernel<E, kPersistentWaves, SP, NTL, true><<<dim3((unsigned)grid), dim3(64 * kPersistentWaves), 0, s>>>(
            recs, n_tiles, tpc_log2, h, dev_params, norm, step_flags);
    else
        adamw_persistent_kernel<E, kPersistentWaves, SP, NTL, false><<<dim3((unsigned)grid), dim3(64 * kPersistentWaves), 0, s>>>(
            recs, n_tiles, tpc_log2, h, dev_params, norm, step_flags);
    return hipGetLastError();
}

template <int SP, bool NTL>
hipError_t launch_per_chunk(const ChunkRec* recs, int64_t n_chunks, const Hyper& h, const rlx_step_params* dev_params,
                            const NormResult* norm, uint32_t step_flags, hipStream_t s) {
    for (int64_t first = 0; first < n_chunks; first += kMaxTilesPerLaunch) {
        const int64_t here = n_chunks - first < kMaxTilesPerLaunch ? n_chunks - first : kMaxTilesPerLaunch;
        if (norm)
            adamw_chunk_kernel<8, 256, SP, NTL, true><<<dim3((unsigned)here), dim3(256), 0, s>>>(recs, first, n_chunks, h,
                                                                                         dev_params, norm, step_flags);
        else
            adamw_chunk_kernel<8, 256, SP, NTL, false><<<dim3((unsigned)here), dim3(256), 0, s>>>(recs, first, n_chunks, h,
                                                                                          dev_params, norm, step_flags);
        const hipError_t e = hipGetLastError();
        if (e != hipSuccess) return e;
    }
    return hipSuccess;
}

template <int E, int BLOCK, int R>
hipError_t launch_rounds(const ChunkRec* recs, int64_t n_chunks, int chunk_log2, const Hyper& h,
                         const rlx_step_params* dev_params, const NormResult* norm, uint32_t step_flags, hipStream_t s) {
    constexpr int TILE = E * BLOCK * R;
    const int tpc_log2 = chunk_log2 - __builtin_ctz(TILE);
    const int64_t n_tiles = n_chunks << tpc_log2;
    for (int64_t first = 0; first < n_tiles; first += kMaxTilesPerLaunch) {
        const int64_t here = n_tiles - first < kMaxTilesPerLaunch ? n_tiles - first : kMaxTilesPerLaunch;
        if (norm)
            adamw_rounds_kernel<E, BLOCK, R, 1, true><<<dim3((unsigned)here), dim3(BLOCK), 0, s>>>(recs, first, n_tiles, tpc_log2,
                                                                                            h, dev_params, norm, step_flags);
        else
            adamw_rounds_kernel<E, BLOCK, R, 1, false><<<dim3((unsigned)here), dim3(BLOCK), 0, s>>>(recs, first, n_tiles, tpc_log2,
                                                                                             h, dev_params, norm, step_flags);
        const hipError_t e = hipGetLastError();
        if (e != hipSuccess) return e;
    }
    return hipSuccess;
}

// The compiled forms of the update ("update_variant"), by number; 0 is what ships.  The names leave out the
// template arguments behind these: whether the clip scale is applied (false for the plain update, true for the
// fused-clip one) and, for adamw_tile_kernel, whether the tiles are walked backwards ("update_reverse").
const char* const kVariantNames[kNumUpdateVariants] = {
    "adamw_tile_kernel<2,128,1,*,1,0|1>",      // 0: 2 elements x 128 lanes, sc1 nt stores; loads at once, or two
                                               //    at a time when the step writes four streams
    "adamw_tile_kernel<2,128,2,*,1,0>",        // 1: with the XCD swizzle
    "adamw_tile_kernel<2,64,1,*,1,0>",         // 2
    "adamw_tile_kernel<4,64,1,*,1,0>",         // 3
    "adamw_tile_kernel<2,256,1,*,1,0>",        // 4
    "adamw_tile_kernel<1,256,1,*,1,0>",        // 5
    "adamw_tile_kernel<4,128,1,*,1,0>",        // 6
    "adamw_tile_kernel<2,128,1,*,0,0>",        // 7: plain nt stores
    "adamw_tile_kernel<2,128,1,*,1,0>",        // 8: always loads at once
    "adamw_tile_kernel<2,128,1,*,1,1>",        // 9: always the two-at-a-time form
    "adamw_tile_kernel<8,64,1,*,2,0,false>",   // 10: 128-bit FP16 / 2 x 128-bit FP32 accesses per lane, one wavefront per
                                               //     512-element tile, ordinary loads and stores
    "adamw_persistent_kernel<8,4,2,false>",    // 11: 128-bit accesses, grid sized to the CUs, wavefronts stride over the tiles
    "adamw_chunk_kernel<8,256,2,false>",       // 12: 128-bit accesses, one 256-lane workgroup walks a whole chunk
    "adamw_chunk_kernel<8,256,1,true>",        // 13: the same with the shipped kernel's non-temporal loads and sc1 nt stores
    "adamw_persistent_kernel<8,4,1,true>",     // 14: the persistent form with those
    "adamw_rounds_kernel<2,128,2,1>",          // 15: the shipped accesses, two 256-element sub-tiles per workgroup
    "adamw_rounds_kernel<2,128,4,1>",          // 16: four sub-tiles (chunks of 1,024 elements and more)
    "adamw_tile_kernel<2,128,1,*,1,2>",        // 17: the shipped tile with lane pairs sharing 128-bit accesses: half the
                                               //     memory instructions (whole aligned tiles of plain FP16 tensors)
};

// any_master: some tensor of the launch has an FP32 master copy.  Such launches, and those that clear the
// gradients, write four streams per tile and take the form of the kernel that splits its loads and stores.
template <bool SINGLE>
int launch_update(const ChunkRec* recs, const ChunkRec& single, int64_t single_n, int64_t n, int chunk_log2,
                  const Hyper& h, const rlx_step_params* dev_params, const NormResult* norm, uint32_t step_flags,
                  bool any_master, hipStream_t s) {
    const bool four_streams = any_master || (step_flags & RLX_STEP_ZERO_GRADS) != 0;
    hipError_t e = hipSuccess;
#define RLX_V(...) e = launch_variant<__VA_ARGS__>(recs, single, single_n, n, chunk_log2, h, dev_params, norm, step_flags, s)
    int64_t variant = g_tuning.update_variant;
    if (SINGLE && variant >= 11) variant = 0;      // the table-walking forms have no flat-tensor counterpart
    if (variant == 16 && chunk_log2 < 10) variant = 0;   // its tile is 1,024 elements
    switch (variant) {
    default:
    case 0:
        if (four_streams) RLX_V(2, 128, 1, SINGLE, 1, 1);
        else RLX_V(2, 128, 1, SINGLE, 1, 0);
        break;
    case 1: RLX_V(2, 128, 2, SINGLE, 1); break;
    case 2: RLX_V(2, 64, 1, SINGLE, 1); break;
    case 3: RLX_V(4, 64, 1, SINGLE, 1); break;
    case 4: RLX_V(2, 256, 1, SINGLE, 1); break;
    case 5: RLX_V(1, 256, 1, SINGLE, 1); break;
    case 6: RLX_V(4, 128, 1, SINGLE, 1); break;
    case 7: RLX_V(2, 128, 1, SINGLE, 0); break;
    case 8: RLX_V(2, 128, 1, SINGLE, 1, 0); break;
    case 9: RLX_V(2, 128, 1, SINGLE, 1, 1); break;
    case 10: RLX_V(8, 64, 1, SINGLE, 2, 0, false); break;
    case 11: if constexpr (!SINGLE) e = launch_persistent<2, false>(recs, n, chunk_log2, h, dev_params, norm, step_flags, s); break;
    case 12: if constexpr (!SINGLE) e = launch_per_chunk<2, false>(recs, n, h, dev_params, norm, step_flags, s); break;
    case 13: if constexpr (!SINGLE) e = launch_per_chunk<1, true>(recs, n, h, dev_params, norm, step_flags, s); break;
    case 14: if constexpr (!SINGLE) e = launch_persistent<1, true>(recs, n, chunk_log2, h, dev_params, norm, step_flags, s); break;
    case 15: if constexpr (!SINGLE) e = launch_rounds<2, 128, 2>(recs, n, chunk_log2, h, dev_params, norm, step_flags, s); break;
    case 16: if constexpr (!SINGLE) e = launch_rounds<2, 128, 4>(recs, n, chunk_log2, h, dev_params, norm, step_flags, s); break;
    case 17: RLX_V(2, 128, 1, SINGLE, 1, 2); break;
    }
#undef RLX_V
    if (e != hipSuccess) return hip_fail(e, "update kernel launch");
    return RLX_OK;
}

int flat_update(void* p, const void* g, float* m, float* v, float* master, int64_t n, int dtype,
                float lr, float beta1, float beta2, float eps, float wd, float bc1, float bc2, void* stream) {
    if (n <= 0) return RLX_OK;                                   // adamw.cu:49,99
    if (!p || !g || !m || !v) return RLX_ERR_INVALID_ARG;
    rlx_tensor_desc d;
    d.param = p; d.grad = const_cast<void*>(g); d.m = m; d.v = v; d.master = master;
    d.n = n; d.dtype = dtype; d.flags = 0;
    int st = check_desc(d);
    if (st != RLX_OK) return st;
    st = check_hyper(lr, beta1, beta2, eps, wd, bc1, bc2);
    if (st != RLX_OK) return st;
    const ChunkRec r = make_rec(d, 0, 0);
    return launch_update<true>(nullptr, r, n, n, 0, make_hyper(lr, beta1, beta2, eps, wd, bc1, bc2), nullptr, nullptr,
                               0, master != nullptr, (hipStream_t)stream);
}

// Zero fill of [dst, dst + nbytes): 128-bit stores over the 16-byte-aligned body, bytes at the edges.
// Returns the first launch error, if any.
hipError_t clear_range(void* dst, int64_t nbytes, hipStream_t s) {
    uint8_t* b = (uint8_t*)dst;
    int64_t n_head = (int64_t)((16 - ((uintptr_t)b & 15)) & 15);
    if (n_head > nbytes) n_head = nbytes;
    const int64_t n_vec = (nbytes - n_head) / 16;
    const int64_t n_tail = nbytes - n_head - n_vec * 16;
    u32x4* body = (u32x4*)(b + n_head);
    const int64_t per_launch = kMaxTilesPerLaunch * 256;         // vectors per launch
    for (int64_t first = 0; first < n_vec; first += per_launch) {
        const int64_t here = n_vec - first < per_launch ? n_vec - first : per_launch;
        clear_body_kernel<<<dim3((unsigned)((here + 255) / 256)), dim3(256), 0, s>>>(body + first, here);
        const hipError_t e = hipGetLastError();
        if (e != hipSuccess) return e;
    }
    if (n_head || n_tail)
        clear_edges_kernel<<<dim3(1), dim3(64), 0, s>>>(b, (int)n_head, b + n_head + n_vec * 16, (int)n_tail);
    return hipGetLastError();
}

}  // namespace

struct rlx_plan {
    uint32_t magic;
    int device;
    int chunk_log2;
    bool any_master;         // some tensor has an FP32 master copy
    int64_t n_tensors, n_chunks, n_elems, chunk_elems;
    ChunkRec* d_recs;        // every chunk, in tensor order (the order of the norm)
    ChunkRec* d_active;      // the chunks that the update changes (not frozen, not grad-only); == d_recs if all are
    int64_t n_active;
    // gradient buffers of the frozen and grad-only tensors, for steps that clear gradients; empty if there are
    // more than kMaxIdleRanges of them (such steps then run over the full table)
    std::vector<std::pair<void*, int64_t>> idle_grads;
    bool idle_by_range;
    double* d_partials;      // one allocation: per-chunk partials, then the group partials (one per 16 chunks),
    double* d_groups;        // then the ticket counters of the one-launch norm
    uint64_t* d_tickets;
    int64_t ticket_grid;     // workgroups of the last one-launch norm on these counters (0: none yet)
    NormResult* d_norm;
    NormResult* h_norm;      // pinned
    // host-free replay: a table of per-step hyper-parameters on the device, the entry that the next scheduled
    // update reads (d_current) and the count of scheduled steps taken (d_taken); all null until a table is uploaded
    rlx_step_params* d_sched;
    int64_t sched_cap, sched_len;
    SchedHeader* d_header;
};

namespace {
constexpr uint32_t kPlanMagic = 0x524C5850u;   // "RLXP"
constexpr size_t kMaxIdleRanges = 16;
inline bool plan_ok(const rlx_plan* p) { return p && p->magic == kPlanMagic; }

// A plan's tables and every pointer in them belong to the device that was current when the plan
// was made; launching it with another device current would hand that device foreign addresses.
int plan_launchable(const rlx_plan* p) {
    if (!plan_ok(p)) return RLX_ERR_INVALID_ARG;
    int dev = -1;
    RLX_HIP(hipGetDevice(&dev));
    return dev == p->device ? RLX_OK : RLX_ERR_WRONG_DEVICE;
}

template <int BLOCK>
hipError_t launch_scale_groups(const rlx_plan* p, hipStream_t s) {
    constexpr int TILE = BLOCK * kVec;
    // chunks smaller than one group: one workgroup per chunk, the lanes beyond its end drop out
    const int tpc_log2 = p->chunk_log2 > __builtin_ctz(TILE) ? p->chunk_log2 - __builtin_ctz(TILE) : 0;
    const int64_t n_tiles = p->n_chunks << tpc_log2;
    for (int64_t first = 0; first < n_tiles; first += kMaxTilesPerLaunch) {
        const int64_t here = n_tiles - first < kMaxTilesPerLaunch ? n_tiles - first : kMaxTilesPerLaunch;
        scale_group_kernel<BLOCK><<<dim3((unsigned)here), dim3(BLOCK), 0, s>>>(p->d_recs, first, n_tiles, tpc_log2,
                                                                             p->d_norm);
        const hipError_t e = hipGetLastError();
        if (e != hipSuccess) return e;
    }
    return hipSuccess;
}

// Step 3 of the norm as a launch of its own.  How many loads a lane keeps in flight only changes the speed, not
// the order of the sum.
hipError_t launch_final(const double* values, int64_t n, float max_norm, NormResult* result, hipStream_t s) {
    int64_t batch = g_tuning.final_batch;
    if (batch == 0) {          // automatic: about as many as a lane has values to add, so that few slots are empty
        const int64_t per_lane = (n + kFinalBlock - 1) / kFinalBlock;
        batch = per_lane <= 8 ? 8 : per_lane <= 16 ? 16 : per_lane <= 32 ? 32 : 40;
    }
    if (batch == 8) sumsq_final_kernel<8><<<dim3(1), dim3(kFinalBlock), 0, s>>>(values, n, max_norm, result);
    else if (batch == 32) sumsq_final_kernel<32><<<dim3(1), dim3(kFinalBlock), 0, s>>>(values, n, max_norm, result);
    else if (batch == 40) sumsq_final_kernel<40><<<dim3(1), dim3(kFinalBlock), 0, s>>>(values, n, max_norm, result);
    else sumsq_final_kernel<16><<<dim3(1), dim3(kFinalBlock), 0, s>>>(values, n, max_norm, result);
    return hipGetLastError();
}

// Where one norm launch reads its chunks and keeps its intermediate sums.
struct NormWork {
    const ChunkRec* recs;        // the chunk table, or
    PoolPair pools;              // two flat buffers by value (POOLS)
    int64_t n_chunks, chunk_elems;
    double* partials;            // one per chunk
    double* groups;              // one per 16 chunks; only used with 512-element chunks
    uint64_t* tickets;           // kTicketWords 64-bit counters; null: never the one-launch form
    int64_t* ticket_grid;        // workgroups of the last one-launch norm on these counters
    NormResult* result;
};

inline int64_t norm_groups(int64_t n_chunks) { return (n_chunks + kGroupChunks - 1) / kGroupChunks; }

// Workgroups up to which the automatic choice ("norm_fused" = 2) lets the last workgroup add the partials: as
// many as the device has CUs.  Measured on flat FP16 tensors of 8,192-element chunks, norm + fused-clip update:
// 64 and 128 workgroups 12.5 us against 16.0 us with the sum as a second launch (the norm alone 5.8 against
// 6.3); 256: 15.6 either way; 512: 22.1 against 21.3; 1,536: 52.4 against 51.4 (the norm alone 8.8 against 6.6);
// the 1,202 workgroups of the 4,096-tensor list: 14.2 against 11.9 for the norm alone.  Beyond one wave of
// workgroups the tickets cost more than the second launch.
constexpr int64_t kAutoFusedWgs = 256;

template <bool NT, bool POOLS, int BLOCK>
hipError_t launch_partials(const NormWork& w, int64_t grid, bool fused, const NormTail& tail, hipStream_t s) {
    if (fused)
        sumsq_partials_kernel<NT, BLOCK, POOLS, 1, true><<<dim3((unsigned)grid), dim3(BLOCK), 0, s>>>(
            w.recs, w.pools, w.n_chunks, w.partials, tail);
    else
        sumsq_partials_kernel<NT, BLOCK, POOLS, 1, false><<<dim3((unsigned)grid), dim3(BLOCK), 0, s>>>(
            w.recs, w.pools, w.n_chunks, w.partials, tail);
    return hipGetLastError();
}

template <bool NT, bool POOLS, int WAVES, int CPW>
hipError_t launch_small_chunks(const NormWork& w, int64_t grid, bool fused, const NormTail& tail, hipStream_t s) {
    if (fused)
        sumsq_small_chunks_kernel<NT, POOLS, WAVES, CPW, true><<<dim3((unsigned)grid), dim3(64 * WAVES), 0, s>>>(
            w.recs, w.pools, w.n_chunks, w.partials, w.groups, tail);
    else
        sumsq_small_chunks_kernel<NT, POOLS, WAVES, CPW, false><<<dim3((unsigned)grid), dim3(64 * WAVES), 0, s>>>(
            w.recs, w.pools, w.n_chunks, w.partials, w.groups, tail);
    return hipGetLastError();
}

// The whole norm: per-chunk partials (and group partials for 512-element chunks), then the fixed-order sum and
// the clip rule into w.result, as the tail of the same launch or as a second one ("norm_fused").
template <bool NT, bool POOLS>
int launch_norm_nt(const NormWork& w, float max_norm, hipStream_t s) {
    const int64_t norm_grid = g_tuning.norm_grid, norm_pack = g_tuning.norm_pack, norm_fused = g_tuning.norm_fused;
    const int64_t lanes = w.chunk_elems / kVec < kNormBlock ? w.chunk_elems / kVec : kNormBlock;
    const bool grouped = lanes == 64;
    NormTail tail;
    tail.values = grouped ? w.groups : w.partials;
    tail.n_values = grouped ? norm_groups(w.n_chunks) : w.n_chunks;
    tail.max_norm = max_norm;
    tail.out = w.result;
    tail.tickets = w.tickets;
    // "norm_keep_mb": that many MB of gradients at the start of the table (FP16 chunks assumed) are read last and
    // with ordinary loads
    const int64_t keep_mb = g_tuning.norm_keep_mb;
    tail.plain_below = keep_mb > 0 && !grouped ? (keep_mb << 20) / (w.chunk_elems * 2) + 1 : 0;
    const auto want_fused = [&](int64_t grid) {      // no ticket counters (w.tickets null): always a second launch
        return w.tickets && grid <= kMaxFusedWgs && (norm_fused == 1 || (norm_fused == 2 && grid <= kAutoFusedWgs));
    };
    bool fused = false;
    hipError_t e = hipSuccess;
    // the counters hold multiples of what one launch of the previous grid added: another grid starts from zero
    const auto same_grid = [&](int64_t grid) -> hipError_t {
        if (*w.ticket_grid == grid) return hipSuccess;
        *w.ticket_grid = grid;
        return clear_range(w.tickets, (int64_t)(sizeof(uint64_t) * kTicketWords), s);
    };
    if (!grouped) {
        int64_t g = norm_grid > 0 ? norm_grid : w.n_chunks;
        if (g > w.n_chunks) g = w.n_chunks;
        if (g > kMaxNormGrid) g = kMaxNormGrid;
        fused = want_fused(g);
        if (fused) e = same_grid(g);
        if (e != hipSuccess) return hip_fail(e, "norm ticket counters");
        if (lanes >= 512) e = launch_partials<NT, POOLS, 512>(w, g, fused, tail, s);
        else if (lanes == 256) e = launch_partials<NT, POOLS, 256>(w, g, fused, tail, s);
        else e = launch_partials<NT, POOLS, 128>(w, g, fused, tail, s);
    } else if (norm_pack == 0 || norm_pack == 1) {
        // 512-element chunks, one per workgroup or eight (a wavefront each): fewer chunks per workgroup than a
        // group has, so the group partials take a launch of their own (both kept for comparison)
        int64_t g = norm_grid > 0 ? norm_grid : w.n_chunks;
        if (g > w.n_chunks) g = w.n_chunks;
        if (g > kMaxNormGrid) g = kMaxNormGrid;
        if (norm_pack == 0)
            sumsq_partials_kernel<NT, 64, POOLS, 1, false><<<dim3((unsigned)g), dim3(64), 0, s>>>(
                w.recs, w.pools, w.n_chunks, w.partials, tail);
        else
            sumsq_partials_kernel<NT, 64, POOLS, 8, false><<<dim3((unsigned)((g + 7) / 8)), dim3(512), 0, s>>>(
                w.recs, w.pools, w.n_chunks, w.partials, tail);
        e = hipGetLastError();
        if (e == hipSuccess) {
            sumsq_group_kernel<<<dim3((unsigned)((tail.n_values + 255) / 256)), dim3(256), 0, s>>>(w.partials, w.n_chunks,
                                                                                                 w.groups);
            e = hipGetLastError();
        }
    } else {
        // 512-element chunks, the default: eight wavefronts per workgroup, two (or four) chunks each.  Measured on
        // the 4,096-tensor list, norm / norm + fused-clip update: two per wavefront 11.25 / 79.4 us, four 12.3 / 81.1,
        // four wavefronts x four 11.9 / 80.4, sixteen wavefronts x one 14.1 / 82.1
        const int64_t per_wg = norm_pack == 2 ? 32 : 16;
        const int64_t g = (w.n_chunks + per_wg - 1) / per_wg;
        if (g > kMaxNormGrid) return RLX_ERR_TOO_LARGE;
        fused = want_fused(g);
        if (fused) e = same_grid(g);
        if (e != hipSuccess) return hip_fail(e, "norm ticket counters");
        if (norm_pack == 3) e = launch_small_chunks<NT, POOLS, 8, 2>(w, g, fused, tail, s);
        else e = launch_small_chunks<NT, POOLS, 8, 4>(w, g, fused, tail, s);
    }
    if (e == hipSuccess && !fused) e = launch_final(tail.values, tail.n_values, max_norm, w.result, s);
    if (e != hipSuccess) return hip_fail(e, "norm kernel launch");
    return RLX_OK;
}

template <bool POOLS>
int launch_norm(const NormWork& w, float max_norm, hipStream_t s) {
    return g_tuning.norm_nt != 0 ? launch_norm_nt<true, POOLS>(w, max_norm, s) : launch_norm_nt<false, POOLS>(w, max_norm, s);
}

// The update launch of a plan.  Frozen and grad-only chunks have nothing to update, and a workgroup that only
// learns that from its record still costs its dispatch (0.3 ms for the frozen embedding of Qwen3-0.6B), so the
// update runs over the table without them; a step that clears gradients clears theirs by range.
int plan_update(const rlx_plan* p, const Hyper& h, const rlx_step_params* dev_params, int step_flags, hipStream_t s) {
    ChunkRec none;
    memset(&none, 0, sizeof(none));
    const NormResult* norm = (step_flags & RLX_CLIP_FUSED) ? p->d_norm : nullptr;
    const bool clear = (step_flags & RLX_STEP_ZERO_GRADS) != 0;
    if (clear && !p->idle_by_range)
        return launch_update<false>(p->d_recs, none, 0, p->n_chunks, p->chunk_log2, h, dev_params, norm,
                                    (uint32_t)step_flags, p->any_master, s);
    if (p->n_active > 0) {
        const int st = launch_update<false>(p->d_active, none, 0, p->n_active, p->chunk_log2, h, dev_params, norm,
                                            (uint32_t)step_flags, p->any_master, s);
        if (st != RLX_OK) return st;
    }
    if (clear) {
        for (const auto& r : p->idle_grads) RLX_HIP(clear_range(r.first, r.second, s));
    }
    return RLX_OK;
}

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
    case RLX_ERR_TOO_LARGE: return "too many chunks: more than one plan can address, or more than the 262,144 partials that the static scratch of rlx_grad_norm_static holds";
    case RLX_ERR_NO_MEMORY: return "out of host memory";
    case RLX_ERR_WRONG_DEVICE: return "the plan belongs to another device than the current one";
    default: return "unknown status";
    }
}

const char* rlx_last_hip_error(void) { return g_hip_error; }

int rlx_version(void) { return 109; }

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
    hipStream_t s = (hipStream_t)stream;
    const int64_t variant = g_tuning.convert_variant;
    if (variant == 2) {
        int64_t grid = (n + 255) / 256;
        if (grid > 65536) grid = 65536;
        fp16_to_fp32_kernel<<<dim3((unsigned)grid), dim3(256), 0, s>>>(dst, src, n);
        RLX_HIP(hipGetLastError());
        return RLX_OK;
    }
    // measured on 2^28 elements (1.6 GB): 128 lanes x 4 elements 6.76 TB/s; 256 x 4, one or two rounds, 6.64 / 6.40;
    // 64 x 4 x 2 6.58; 128 x 2 4.28 (too many workgroups for the dispatcher); one element per lane, grid-stride, 3.45
    int lanes = 128, e = 4, rounds = 1;                           // variant 0
    if (variant == 1) e = 2;
    else if (variant == 3) { lanes = 256; rounds = 2; }
    const int64_t span = (int64_t)lanes * e * rounds;
    const int vec_ok = is_aligned(src, 2 * (size_t)e) && is_aligned(dst, 4 * (size_t)e);
    const int64_t n_wg = (n + span - 1) / span;
    for (int64_t first = 0; first < n_wg; first += kMaxTilesPerLaunch) {
        const int64_t here = n_wg - first < kMaxTilesPerLaunch ? n_wg - first : kMaxTilesPerLaunch;
        float* d = dst + first * span;
        const uint16_t* q = src + first * span;
        const int64_t left = n - first * span;
        if (variant == 1) convert_tile_kernel<128, 2, 1><<<dim3((unsigned)here), dim3(128), 0, s>>>(d, q, left, vec_ok);
        else if (variant == 3) convert_tile_kernel<256, 4, 2><<<dim3((unsigned)here), dim3(256), 0, s>>>(d, q, left, vec_ok);
        else convert_tile_kernel<128, 4, 1><<<dim3((unsigned)here), dim3(128), 0, s>>>(d, q, left, vec_ok);
        RLX_HIP(hipGetLastError());
    }
    return RLX_OK;
}

int rlx_scale_f32(float* x, float scale, int64_t n, void* stream) {
    if (n <= 0) return RLX_OK;
    if (!x) return RLX_ERR_INVALID_ARG;
    if (!is_aligned(x, 4)) return RLX_ERR_MISALIGNED;
    const int64_t lanes = (n + 3) / 4;
    const int64_t per_launch = kMaxTilesPerLaunch * 256;         // lanes per launch
    for (int64_t first = 0; first < lanes; first += per_launch) {
        const int64_t here = lanes - first < per_launch ? lanes - first : per_launch;
        scale_f32_kernel<<<dim3((unsigned)((here + 255) / 256)), dim3(256), 0, (hipStream_t)stream>>>(
            x + first * 4, scale, n - first * 4, is_aligned(x, 16) ? 1 : 0);
        RLX_HIP(hipGetLastError());
    }
    return RLX_OK;
}

int rlx_clear(void* dst, int64_t nbytes, void* stream) {
    if (nbytes <= 0) return RLX_OK;
    if (!dst) return RLX_ERR_INVALID_ARG;
    RLX_HIP(clear_range(dst, nbytes, (hipStream_t)stream));
    return RLX_OK;
}

int rlx_plan_layout(const rlx_tensor_desc* descs, int64_t count, int64_t chunk_elems, int64_t* out_chunk_elems,
                    int64_t* out_num_chunks, int64_t* out_num_elements) {
    if (!descs || count <= 0 || count > INT32_MAX) return RLX_ERR_INVALID_ARG;
    int64_t n_elems = 0;
    for (int64_t i = 0; i < count; i++) {
        int st = check_desc(descs[i]);
        if (st != RLX_OK) return st;
        n_elems += descs[i].n;
    }
    if (chunk_elems == 0) chunk_elems = default_chunk(n_elems, count);
    if (!chunk_ok(chunk_elems)) return RLX_ERR_INVALID_ARG;
    int64_t n_chunks = 0;
    for (int64_t i = 0; i < count; i++) n_chunks += (descs[i].n + chunk_elems - 1) / chunk_elems;
    if (n_chunks > INT32_MAX) return RLX_ERR_TOO_LARGE;
    if (out_chunk_elems) *out_chunk_elems = chunk_elems;
    if (out_num_chunks) *out_num_chunks = n_chunks;
    if (out_num_elements) *out_num_elements = n_elems;
    return RLX_OK;
}

int rlx_plan_create(const rlx_tensor_desc* descs, int64_t count, int64_t chunk_elems, rlx_plan** out) {
    if (!out) return RLX_ERR_INVALID_ARG;
    *out = nullptr;
    int64_t n_elems = 0, n_chunks = 0;
    const int layout = rlx_plan_layout(descs, count, chunk_elems, &chunk_elems, &n_chunks, &n_elems);
    if (layout != RLX_OK) return layout;

    std::vector<ChunkRec> recs;
    try {
        recs.reserve((size_t)n_chunks);
    } catch (const std::bad_alloc&) {
        return RLX_ERR_NO_MEMORY;
    }
    for (int64_t i = 0; i < count; i++) {
        for (int64_t start = 0; start < descs[i].n; start += chunk_elems) {
            const int64_t left = descs[i].n - start;
            recs.push_back(make_rec(descs[i], start, left < chunk_elems ? left : chunk_elems));
        }
    }

    rlx_plan* p = new (std::nothrow) rlx_plan();
    if (!p) return RLX_ERR_NO_MEMORY;
    p->magic = kPlanMagic;
    p->chunk_log2 = __builtin_ctzll((unsigned long long)chunk_elems);
    p->n_tensors = count; p->n_chunks = n_chunks; p->n_elems = n_elems; p->chunk_elems = chunk_elems;
    p->any_master = false;
    p->idle_by_range = true;
    try {
        p->idle_grads.reserve(kMaxIdleRanges);
    } catch (const std::bad_alloc&) {
        delete p;
        return RLX_ERR_NO_MEMORY;
    }
    for (int64_t i = 0; i < count; i++) {
        p->any_master = p->any_master || descs[i].master != nullptr;
        if (descs[i].flags & (RLX_TENSOR_GRAD_ONLY | RLX_TENSOR_FROZEN)) {
            if (p->idle_grads.size() < kMaxIdleRanges)      // within the reserved capacity: cannot throw
                p->idle_grads.emplace_back(descs[i].grad, descs[i].n * (descs[i].dtype == RLX_DTYPE_F16 ? 2 : 4));
            else
                p->idle_by_range = false;
        }
    }
    p->d_recs = nullptr; p->d_active = nullptr; p->n_active = 0; p->d_partials = nullptr; p->d_groups = nullptr; p->d_tickets = nullptr; p->ticket_grid = 0; p->d_norm = nullptr; p->h_norm = nullptr;
    p->d_sched = nullptr; p->sched_cap = 0; p->sched_len = 0; p->d_header = nullptr;

    hipError_t e = hipGetDevice(&p->device);
    if (e == hipSuccess) e = hipMalloc((void**)&p->d_recs, sizeof(ChunkRec) * (size_t)n_chunks);
    const size_t n_sums = (size_t)n_chunks + (size_t)norm_groups(n_chunks);
    if (e == hipSuccess) e = hipMalloc((void**)&p->d_partials, sizeof(double) * n_sums + sizeof(uint64_t) * (size_t)kTicketWords);
    if (e == hipSuccess) {
        p->d_groups = p->d_partials + n_chunks;
        p->d_tickets = (uint64_t*)(p->d_partials + n_sums);
        e = hipMemset(p->d_tickets, 0, sizeof(uint64_t) * (size_t)kTicketWords);
    }
    if (e == hipSuccess) e = hipMalloc((void**)&p->d_norm, sizeof(NormResult));
    if (e == hipSuccess) e = hipHostMalloc((void**)&p->h_norm, sizeof(NormResult), hipHostMallocDefault);
    if (e == hipSuccess) e = hipMemcpy(p->d_recs, recs.data(), sizeof(ChunkRec) * (size_t)n_chunks, hipMemcpyHostToDevice);
    if (e == hipSuccess) {
        // A workgroup that only finds out from its record that it has nothing to do still costs its dispatch
        // (0.3 ms for the frozen embedding of Qwen3-0.6B): updates that do not clear gradients run over a
        // table without such chunks.
        size_t keep = 0;
        for (size_t i = 0; i < recs.size(); i++)
            if (!(recs[i].flags & (RLX_TENSOR_GRAD_ONLY | RLX_TENSOR_FROZEN))) recs[keep++] = recs[i];
        p->n_active = (int64_t)keep;
        if (keep == recs.size()) {
            p->d_active = p->d_recs;
        } else if (keep > 0) {
            e = hipMalloc((void**)&p->d_active, sizeof(ChunkRec) * keep);
            if (e == hipSuccess) e = hipMemcpy(p->d_active, recs.data(), sizeof(ChunkRec) * keep, hipMemcpyHostToDevice);
        }
    }
    if (e == hipSuccess) {
        const NormResult init = {0.0, 0.0f, 1.0f};
        *p->h_norm = init;
        e = hipMemcpy(p->d_norm, &init, sizeof(init), hipMemcpyHostToDevice);
    }
    if (e != hipSuccess) {
        int st = hip_fail(e, "rlx_plan_create");
        if (e == hipErrorNoDevice || e == hipErrorInvalidDevice) st = RLX_ERR_NO_DEVICE;
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
    if (p->d_active && p->d_active != p->d_recs && (e = hipFree(p->d_active)) != hipSuccess && first == hipSuccess) first = e;
    if (p->d_recs && (e = hipFree(p->d_recs)) != hipSuccess && first == hipSuccess) first = e;
    if (p->d_partials && (e = hipFree(p->d_partials)) != hipSuccess && first == hipSuccess) first = e;
    if (p->d_norm && (e = hipFree(p->d_norm)) != hipSuccess && first == hipSuccess) first = e;
    if (p->h_norm && (e = hipHostFree(p->h_norm)) != hipSuccess && first == hipSuccess) first = e;
    if (p->d_sched && (e = hipFree(p->d_sched)) != hipSuccess && first == hipSuccess) first = e;
    if (p->d_header && (e = hipFree(p->d_header)) != hipSuccess && first == hipSuccess) first = e;
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
    const int ready = plan_launchable(p);
    if (ready != RLX_OK) return ready;
    NormWork w;
    memset(&w, 0, sizeof(w));
    w.recs = p->d_recs; w.n_chunks = p->n_chunks; w.chunk_elems = p->chunk_elems;
    w.partials = p->d_partials; w.groups = p->d_groups; w.tickets = p->d_tickets; w.ticket_grid = &p->ticket_grid;
    w.result = p->d_norm;
    return launch_norm<false>(w, max_norm, (hipStream_t)stream);
}

/* Device address of the static scratch array on the current device, resolved once per device. */
static int static_scratch(double** out) {
    int dev = -1;
    RLX_HIP(hipGetDevice(&dev));
    if (dev < 0 || dev >= kMaxDevices) return RLX_ERR_INVALID_ARG;
    std::lock_guard<std::mutex> lock(g_scratch_mutex);
    if (!g_scratch_ptr[dev]) {
        void* ptr = nullptr;
        RLX_HIP(hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch)));
        if (!ptr) return RLX_ERR_HIP;
        g_scratch_ptr[dev] = (double*)ptr;
    }
    *out = g_scratch_ptr[dev];
    return RLX_OK;
}

int rlx_grad_norm_static(const uint16_t* half_grads, int64_t n_half, const float* float_grads, int64_t n_float,
                         int64_t chunk_elems, float max_norm, void* result_dev, void* stream) {
    if (n_half < 0 || n_float < 0 || !result_dev) return RLX_ERR_INVALID_ARG;
    if ((n_half > 0 && !half_grads) || (n_float > 0 && !float_grads)) return RLX_ERR_INVALID_ARG;
    if (!is_aligned(half_grads, 2) || !is_aligned(float_grads, 4) || !is_aligned(result_dev, 8)) return RLX_ERR_MISALIGNED;
    const int64_t n_tensors = (n_half > 0) + (n_float > 0);
    if (chunk_elems == 0) chunk_elems = n_tensors ? default_chunk(n_half + n_float, n_tensors) : kBigChunk;
    if (!chunk_ok(chunk_elems)) return RLX_ERR_INVALID_ARG;
    PoolPair pp;
    pp.half_pool = half_grads; pp.float_pool = float_grads; pp.n_half = n_half; pp.n_float = n_float;
    pp.chunk_log2 = __builtin_ctzll((unsigned long long)chunk_elems);
    pp.chunks_half = (n_half + chunk_elems - 1) / chunk_elems;
    const int64_t n_chunks = pp.chunks_half + (n_float + chunk_elems - 1) / chunk_elems;
    if (n_chunks > kStaticMaxPartials) return RLX_ERR_TOO_LARGE;
    // the flags that a plan's record of a gradient-only tensor at this address would carry
    rlx_tensor_desc d;
    memset(&d, 0, sizeof(d));
    d.flags = RLX_TENSOR_GRAD_ONLY;
    d.grad = const_cast<uint16_t*>(half_grads); d.dtype = RLX_DTYPE_F16;
    pp.flags_half = make_rec(d, 0, 0).flags;
    d.grad = const_cast<float*>(float_grads); d.dtype = RLX_DTYPE_F32;
    pp.flags_float = make_rec(d, 0, 0).flags;
    double* base = nullptr;
    const int st = static_scratch(&base);
    if (st != RLX_OK) return st;
    if (n_chunks == 0) {      // nothing to add up: sum 0, norm 0, scale by the rule
        RLX_HIP(launch_final(base, 0, max_norm, (NormResult*)result_dev, (hipStream_t)stream));
        return RLX_OK;
    }
    NormWork w;
    memset(&w, 0, sizeof(w));
    w.pools = pp; w.n_chunks = n_chunks; w.chunk_elems = chunk_elems;
    w.partials = base; w.groups = base + kStaticMaxPartials;
    w.tickets = nullptr; w.ticket_grid = nullptr;
    w.result = (NormResult*)result_dev;
    return launch_norm<true>(w, max_norm, (hipStream_t)stream);
}

int rlx_plan_norm_read(rlx_plan* p, float* norm, float* scale, double* sum_sq, void* stream) {
    const int ready = plan_launchable(p);
    if (ready != RLX_OK) return ready;
    hipStream_t s = (hipStream_t)stream;
    RLX_HIP(hipMemcpyAsync(p->h_norm, p->d_norm, sizeof(NormResult), hipMemcpyDeviceToHost, s));
    RLX_HIP(hipStreamSynchronize(s));
    if (norm) *norm = p->h_norm->norm;
    if (scale) *scale = p->h_norm->scale;
    if (sum_sq) *sum_sq = p->h_norm->sum_sq;
    return RLX_OK;
}

int rlx_plan_scale_grads(rlx_plan* p, void* stream) {
    const int ready = plan_launchable(p);
    if (ready != RLX_OK) return ready;
    RLX_HIP(launch_scale_groups<kScaleBlock>(p, (hipStream_t)stream));
    return RLX_OK;
}

int rlx_plan_adamw(rlx_plan* p, const rlx_step_params* sp, int step_flags, void* stream) {
    if (!plan_ok(p) || !sp) return RLX_ERR_INVALID_ARG;
    if (step_flags & ~(RLX_CLIP_FUSED | RLX_STEP_ZERO_GRADS)) return RLX_ERR_INVALID_ARG;
    const int ready = plan_launchable(p);
    if (ready != RLX_OK) return ready;
    int st = check_hyper(sp->lr, sp->beta1, sp->beta2, sp->eps, sp->weight_decay, sp->bias_correction1,
                         sp->bias_correction2);
    if (st != RLX_OK) return st;
    const Hyper h = make_hyper(sp->lr, sp->beta1, sp->beta2, sp->eps, sp->weight_decay, sp->bias_correction1,
                               sp->bias_correction2);
    return plan_update(p, h, nullptr, step_flags, (hipStream_t)stream);
}

int rlx_plan_adamw_dev(rlx_plan* p, const rlx_step_params* dev_params, int step_flags, void* stream) {
    if (!plan_ok(p) || !dev_params) return RLX_ERR_INVALID_ARG;
    if (step_flags & ~(RLX_CLIP_FUSED | RLX_STEP_ZERO_GRADS)) return RLX_ERR_INVALID_ARG;
    if (!is_aligned(dev_params, 4)) return RLX_ERR_MISALIGNED;
    const int ready = plan_launchable(p);
    if (ready != RLX_OK) return ready;
    Hyper h;
    memset(&h, 0, sizeof(h));
    return plan_update(p, h, dev_params, step_flags, (hipStream_t)stream);
}

int rlx_plan_schedule_upload(rlx_plan* p, const rlx_step_params* steps, int64_t n_steps, void* stream) {
    if (!plan_ok(p) || !steps || n_steps <= 0 || n_steps > ((int64_t)1 << 28)) return RLX_ERR_INVALID_ARG;
    const int ready = plan_launchable(p);
    if (ready != RLX_OK) return ready;
    for (int64_t i = 0; i < n_steps; i++) {
        const int st = check_hyper(steps[i].lr, steps[i].beta1, steps[i].beta2, steps[i].eps, steps[i].weight_decay,
                                   steps[i].bias_correction1, steps[i].bias_correction2);
        if (st != RLX_OK) return st;
    }
    (void)stream;
    // Scheduled updates of this plan that are still running, on whatever stream (replays of a recorded step
    // included), read the header and the old table: wait for the whole device, not only for `stream`.
    RLX_HIP(hipDeviceSynchronize());
    if (!p->d_header) RLX_HIP(hipMalloc((void**)&p->d_header, sizeof(SchedHeader)));   // address fixed from here on
    rlx_step_params* table = p->d_sched;
    rlx_step_params* retired = nullptr;
    if (n_steps > p->sched_cap) {
        // A longer table gets a new allocation.  Recorded launches hold the header's address, never the table's,
        // and nothing is running, so the old table can go once the header names the new one.
        RLX_HIP(hipMalloc((void**)&table, sizeof(rlx_step_params) * (size_t)n_steps));
        retired = p->d_sched;
    }
    hipError_t e = hipMemcpy(table, steps, sizeof(rlx_step_params) * (size_t)n_steps, hipMemcpyHostToDevice);
    if (e == hipSuccess) {
        SchedHeader h;
        memset(&h, 0, sizeof(h));
        h.current = steps[0];
        h.table = table;
        h.len = n_steps;
        e = hipMemcpy(p->d_header, &h, sizeof(h), hipMemcpyHostToDevice);
    }
    if (e != hipSuccess) {
        // the header still names the old table (or none): leave the plan as it was
        if (table != p->d_sched) (void)hipFree(table);
        return hip_fail(e, "rlx_plan_schedule_upload");
    }
    if (table != p->d_sched) { p->d_sched = table; p->sched_cap = n_steps; }
    p->sched_len = n_steps;
    if (retired) RLX_HIP(hipFree(retired));
    return RLX_OK;
}

int rlx_plan_adamw_scheduled(rlx_plan* p, int step_flags, void* stream) {
    if (!plan_ok(p) || !p->d_sched || p->sched_len <= 0) return RLX_ERR_INVALID_ARG;
    if (step_flags & ~(RLX_CLIP_FUSED | RLX_STEP_ZERO_GRADS)) return RLX_ERR_INVALID_ARG;
    const int ready = plan_launchable(p);
    if (ready != RLX_OK) return ready;
    Hyper h;
    memset(&h, 0, sizeof(h));
    const int st = plan_update(p, h, &p->d_header->current, step_flags, (hipStream_t)stream);
    if (st != RLX_OK) return st;
    schedule_advance_kernel<<<dim3(1), dim3(64), 0, (hipStream_t)stream>>>(p->d_header);
    RLX_HIP(hipGetLastError());
    return RLX_OK;
}

int rlx_plan_schedule_position(rlx_plan* p, int64_t* steps_taken, int64_t* n_steps, void* stream) {
    if (!plan_ok(p) || !p->d_sched) return RLX_ERR_INVALID_ARG;
    const int ready = plan_launchable(p);
    if (ready != RLX_OK) return ready;
    SchedHeader h;
    RLX_HIP(hipStreamSynchronize((hipStream_t)stream));
    RLX_HIP(hipMemcpy(&h, p->d_header, sizeof(h), hipMemcpyDeviceToHost));
    if (steps_taken) *steps_taken = h.taken;
    if (n_steps) *n_steps = h.len;
    return RLX_OK;
}

int rlx_plan_schedule_overrun(rlx_plan* p, int64_t* overrun, void* stream) {
    if (!plan_ok(p) || !p->d_sched || !overrun) return RLX_ERR_INVALID_ARG;
    const int ready = plan_launchable(p);
    if (ready != RLX_OK) return ready;
    SchedHeader h;
    RLX_HIP(hipStreamSynchronize((hipStream_t)stream));
    RLX_HIP(hipMemcpy(&h, p->d_header, sizeof(h), hipMemcpyDeviceToHost));
    *overrun = h.overrun;
    return RLX_OK;
}

const char* rlx_update_variant_name(int64_t variant) {
    return variant >= 0 && variant < kNumUpdateVariants ? kVariantNames[variant] : "";
}

int rlx_set_tuning(const char* key, int64_t value) {
    if (!key || value < 0) return RLX_ERR_INVALID_ARG;
    if (!strcmp(key, "update_variant")) {
        if (value >= kNumUpdateVariants) return RLX_ERR_INVALID_ARG;
        g_tuning.update_variant = value;
    } else if (!strcmp(key, "norm_grid")) g_tuning.norm_grid = value;
    else if (!strcmp(key, "norm_nt")) g_tuning.norm_nt = value ? 1 : 0;
    else if (!strcmp(key, "norm_pack")) {
        if (value > 3) return RLX_ERR_INVALID_ARG;
        g_tuning.norm_pack = value;
    }
    else if (!strcmp(key, "final_batch")) {
        if (value != 0 && value != 8 && value != 16 && value != 32 && value != 40) return RLX_ERR_INVALID_ARG;
        g_tuning.final_batch = value;
    }
    else if (!strcmp(key, "norm_fused")) {
        if (value > 2) return RLX_ERR_INVALID_ARG;
        g_tuning.norm_fused = value;
    }
    else if (!strcmp(key, "update_reverse")) g_tuning.update_reverse = value ? 1 : 0;
    else if (!strcmp(key, "norm_keep_mb")) {
        if (value > 4096) return RLX_ERR_INVALID_ARG;
        g_tuning.norm_keep_mb = value;
    }
    else if (!strcmp(key, "convert_variant")) {
        if (value >= kNumConvertVariants) return RLX_ERR_INVALID_ARG;
        g_tuning.convert_variant = value;
    } else return RLX_ERR_INVALID_ARG;
    return RLX_OK;
}

int64_t rlx_get_tuning(const char* key) {
    if (!key) return -1;
    if (!strcmp(key, "update_variant")) return g_tuning.update_variant;
    if (!strcmp(key, "norm_grid")) return g_tuning.norm_grid;
    if (!strcmp(key, "norm_nt")) return g_tuning.norm_nt;
    if (!strcmp(key, "norm_pack")) return g_tuning.norm_pack;
    if (!strcmp(key, "convert_variant")) return g_tuning.convert_variant;
    if (!strcmp(key, "final_batch")) return g_tuning.final_batch;
    if (!strcmp(key, "norm_fused")) return g_tuning.norm_fused;
    if (!strcmp(key, "update_reverse")) return g_tuning.update_reverse;
    if (!strcmp(key, "norm_keep_mb")) return g_tuning.norm_keep_mb;
    return -1;
}

static int fill_common(void* dst, int elem_size, int64_t n, uint64_t seed, int64_t first, float mean, float std,
                       uint32_t flags, int64_t row_len, uint32_t zero_rows_below, void* stream) {
    if (n <= 0) return RLX_OK;
    if (!dst || first < 0 || row_len < 0) return RLX_ERR_INVALID_ARG;
    if (!is_aligned(dst, (size_t)elem_size)) return RLX_ERR_MISALIGNED;
    int64_t grid = (n + kFillBlock - 1) / kFillBlock;
    if (grid > 262144) grid = 262144;
    if (elem_size == 2)
        fill_kernel<uint16_t><<<dim3((unsigned)grid), dim3(kFillBlock), 0, (hipStream_t)stream>>>(
            (uint16_t*)dst, n, seed, first, mean, std, flags, row_len, zero_rows_below);
    else
        fill_kernel<float><<<dim3((unsigned)grid), dim3(kFillBlock), 0, (hipStream_t)stream>>>(
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
