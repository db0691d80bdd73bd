// Shared device helpers for the gfx950 kernels: wave64 / workgroup reductions,
// 128-bit vector types and the launch-check macros used by every C-ABI entry.
#pragma once

#include <hip/hip_runtime.h>
#include <hip/hip_bf16.h>
#include <hip/hip_fp16.h>
#include <stdint.h>

#include "br_hip.h"

namespace brk {

constexpr int kWave = 64;  // CDNA wavefront width

// Returns from the enclosing extern "C" function with the hipError_t value.
#define BR_HIP_TRY(expr)                         \
    do {                                         \
        hipError_t br_err_ = (expr);             \
        if (br_err_ != hipSuccess) return (int)br_err_; \
    } while (0)

// After a kernel launch: report launch-configuration errors to the caller.
#define BR_HIP_LAUNCH_CHECK() BR_HIP_TRY(hipGetLastError())

inline hipStream_t as_stream(br_stream_t s) { return reinterpret_cast<hipStream_t>(s); }

inline bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }
inline bool aligned8(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 7u) == 0; }

// ---- wave64 reductions: butterfly over the 64 lanes --------------------
__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, kWave);
    return v;
}

__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v = fmaxf(v, __shfl_xor(v, off, kWave));
    return v;
}

// Workgroup sum of NV values per thread; every thread gets the result.
// `lds` must hold NV * (blockDim.x / 64) floats and must not be reused by the
// caller before the next __syncthreads() it issues itself (callers alternate
// between two such buffers to get away with one barrier per reduction).
template <int NV>
__device__ __forceinline__ void block_sum(float (&v)[NV], float* lds) {
    const int lane = threadIdx.x & (kWave - 1);
    const int wave = threadIdx.x >> 6;
    const int nwave = blockDim.x >> 6;
#pragma unroll
    for (int i = 0; i < NV; i++) v[i] = wave_sum(v[i]);
    if (nwave == 1) return;
    if (lane == 0) {
#pragma unroll
        for (int i = 0; i < NV; i++) lds[i * nwave + wave] = v[i];
    }
    __syncthreads();
#pragma unroll
    for (int i = 0; i < NV; i++) {
        float s = 0.f;
        for (int w = 0; w < nwave; w++) s += lds[i * nwave + w];
        v[i] = s;
    }
}


// ---- streaming (non-temporal) 128-bit accesses ------------------------------
// For data a kernel reads once or writes once and never touches again: the
// cache-policy hint keeps such lines from displacing what other kernels (or
// this one) reuse.  Which kernels use them was decided by measurement, kernel
// by kernel (MI355X, rotating buffers): streaming loads gain 2-10 % everywhere
// but in the log-softmax backward, where only loads and stores together do;
// streaming stores gain another 5-10 % in LayerNorm forward, bias-GELU and
// AdamW and LOSE in the 8-elements-per-thread conversion kernel used as a copy
// (-20 %) and in LayerNorm backward (-3 %), which therefore store normally (the
// one-granule-per-thread copy gains 2-4 % from them).  BR_STREAM=0 / BR_STREAM_STORES=0 compile the loads
// / the stores as ordinary accesses (for repeating that measurement).
#ifndef BR_STREAM
#define BR_STREAM 1
#endif
#ifndef BR_STREAM_STORES
#define BR_STREAM_STORES 1
#endif
typedef unsigned stream_u4 __attribute__((ext_vector_type(4)));
template <typename V>
__device__ __forceinline__ V load_stream(const V* p) {
    static_assert(sizeof(V) == 16, "128-bit vectors only");
#if BR_STREAM
    const stream_u4 v = __builtin_nontemporal_load(reinterpret_cast<const stream_u4*>(p));
    return __builtin_bit_cast(V, v);
#else
    return *p;
#endif
}
template <typename V>
__device__ __forceinline__ void store_stream(V* p, const V& v) {
    static_assert(sizeof(V) == 16, "128-bit vectors only");
#if BR_STREAM_STORES
    __builtin_nontemporal_store(__builtin_bit_cast(stream_u4, v), reinterpret_cast<stream_u4*>(p));
#else
    *p = v;
#endif
}

// ---- fp16 pack / unpack (8 halves <-> one 128-bit register quad) --------
struct alignas(16) half8 {
    __half2 v[4];
};
struct alignas(8) half4 {
    __half2 v[2];
};

__device__ __forceinline__ void unpack8(const half8& h, float (&f)[8]) {
#pragma unroll
    for (int i = 0; i < 4; i++) {
        float2 t = __half22float2(h.v[i]);
        f[2 * i] = t.x;
        f[2 * i + 1] = t.y;
    }
}

__device__ __forceinline__ half8 pack8(const float (&f)[8]) {
    half8 h;
#pragma unroll
    for (int i = 0; i < 4; i++) h.v[i] = __floats2half2_rn(f[2 * i], f[2 * i + 1]);
    return h;
}

// Optional second output of an fp32-producing kernel: the same values rounded
// to fp16 / bf16, for consumers that are 16-bit matrix products.  `base` is a
// dense array with the fp32 output's indexing; null = no copy.
struct Copy16 {
    void* base;
    int bf16;
};
// Stores v (4 consecutive fp32 results, already final) at 4-element index idx4.
// The barrier keeps the fp32 rounding: without it the compiler may fold the
// producing multiply-add into the conversion, and the copy would differ from
// the rounded fp32 output in the last bit.
__device__ __forceinline__ void store4_as16(const Copy16& c, int64_t idx4, float4& v) {
    asm volatile("" : "+v"(v.x), "+v"(v.y), "+v"(v.z), "+v"(v.w));
    if (!c.base) return;
    unsigned lo, hi;
    if (c.bf16) {
        lo = (unsigned)__builtin_bit_cast(unsigned short, __float2bfloat16(v.x)) |
             ((unsigned)__builtin_bit_cast(unsigned short, __float2bfloat16(v.y)) << 16);
        hi = (unsigned)__builtin_bit_cast(unsigned short, __float2bfloat16(v.z)) |
             ((unsigned)__builtin_bit_cast(unsigned short, __float2bfloat16(v.w)) << 16);
    } else {
        lo = (unsigned)__builtin_bit_cast(unsigned short, __float2half_rn(v.x)) |
             ((unsigned)__builtin_bit_cast(unsigned short, __float2half_rn(v.y)) << 16);
        hi = (unsigned)__builtin_bit_cast(unsigned short, __float2half_rn(v.z)) |
             ((unsigned)__builtin_bit_cast(unsigned short, __float2half_rn(v.w)) << 16);
    }
    reinterpret_cast<uint2*>(c.base)[idx4] = make_uint2(lo, hi);
}
inline bool copy16_ok(const void* y16, int dtype) {
    return y16 && (dtype == BR_F16 || dtype == BR_BF16) && (reinterpret_cast<uintptr_t>(y16) & 7u) == 0;
}

// gelu(v) = v * (0.5 + 0.5*tanh(u)),  u = v*(0.79788456 + 0.03567741 v^2)
//         = v * sigmoid(2u)            (no cancellation in the left tail)
// sigmoid(2u) = 1 / (1 + 2^w), w = -2*log2(e)*u: the factor is folded into the
// two polynomial constants, so the exponent costs no extra multiplies.
constexpr float kLog2e2 = 2.8853900817779268f;  // 2 * log2(e)
__device__ __forceinline__ float gelu_one(float v) {
    const float w = v * (-kLog2e2 * 0.79788456f + (-kLog2e2 * 0.03567741f) * (v * v));
    return v * __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(w));
}

// Grid size for a grid-stride elementwise kernel: one work item per thread wherever that fits a grid.  Workgroups
// are dispatched in order, so the launch then sweeps memory front to back as ONE stream; with the grid capped at a
// few thousand workgroups, each looping with a stride of megabytes, the same bytes arrive as thousands of streams.
// Measured with a plain copy of 134-537 MB: 6.0-6.5 TB/s one granule per thread, 4.4-5.5 TB/s for every persistent
// or chunked form tried (and 5.4 for the runtime's own device-to-device copy); AdamW over 67 M parameters 396 -> 340 us.
// The loops stay: they cover what the cap leaves over.
#ifndef BR_GRID_CAP
#define BR_GRID_CAP (1 << 24)
#endif
inline int grid_for(int64_t work_items, int block, int max_blocks = BR_GRID_CAP) {
    int64_t g = (work_items + block - 1) / block;
    if (g < 1) g = 1;
    if (g > max_blocks) g = max_blocks;
    return (int)g;
}

}  // namespace brk
