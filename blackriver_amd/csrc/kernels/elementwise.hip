// Memory-bound elementwise kernels for gfx950: fill, cast, broadcast add,
// (bias-)GELU forward / backward, transpose 0213, column sums and the
// data-preparation tables.  All of them move 128 bits per lane per access and
// are launched as grid-stride loops over a few thousand workgroups.
#include "common.hpp"

#include <type_traits>

#include <float.h>
#include <hip/hip_bf16.h>

using namespace brk;

namespace {

constexpr int kBlock = 256;

// ------------------------------------------------------------------ fill
template <typename T>
__global__ __launch_bounds__(kBlock) void fill_kernel(T* dst, T value, int64_t n) {
    const int64_t stride = (int64_t)gridDim.x * kBlock;
    for (int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x; i < n; i += stride) dst[i] = value;
}

// ------------------------------------------------------------------ cast
template <typename T>
__device__ __forceinline__ float to_f32(T v);
template <>
__device__ __forceinline__ float to_f32<float>(float v) { return v; }
template <>
__device__ __forceinline__ float to_f32<__half>(__half v) { return __half2float(v); }
template <>
__device__ __forceinline__ float to_f32<__hip_bfloat16>(__hip_bfloat16 v) { return __bfloat162float(v); }

template <typename T>
__device__ __forceinline__ T from_f32(float v);
template <>
__device__ __forceinline__ float from_f32<float>(float v) { return v; }
template <>
__device__ __forceinline__ __half from_f32<__half>(float v) { return __float2half_rn(v); }
template <>
__device__ __forceinline__ __hip_bfloat16 from_f32<__hip_bfloat16>(float v) { return __float2bfloat16(v); }

template <typename S, typename D>
__global__ __launch_bounds__(kBlock) void cast_kernel(const S* src, D* dst, int64_t n) {
    const int64_t stride = (int64_t)gridDim.x * kBlock * 4;
    for (int64_t i = ((int64_t)blockIdx.x * kBlock + threadIdx.x) * 4; i < n; i += stride) {
        if (i + 3 < n) {
            S s[4];
#pragma unroll
            for (int j = 0; j < 4; j++) s[j] = src[i + j];
#pragma unroll
            for (int j = 0; j < 4; j++) dst[i + j] = from_f32<D>(to_f32<S>(s[j]));
        } else {
            for (int64_t j = i; j < n; j++) dst[j] = from_f32<D>(to_f32<S>(src[j]));
        }
    }
}

// 8 elements per thread through 128-bit accesses (n % 8 == 0, 16-byte aligned).
template <typename S, typename D>
__global__ __launch_bounds__(kBlock) void cast_x8_kernel(const S* __restrict__ src, D* __restrict__ dst, int64_t n8) {
    struct alignas(16) SV { S v[8]; };
    struct alignas(16) DV { D v[8]; };
    const int64_t stride = (int64_t)gridDim.x * kBlock;
    for (int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x; i < n8; i += stride) {
        float f[8];
        if constexpr (sizeof(S) == 4) {
            const float4 a = load_stream(reinterpret_cast<const float4*>(src) + 2 * i),
                         b = load_stream(reinterpret_cast<const float4*>(src) + 2 * i + 1);
            f[0] = a.x; f[1] = a.y; f[2] = a.z; f[3] = a.w; f[4] = b.x; f[5] = b.y; f[6] = b.z; f[7] = b.w;
        } else {
            const uint4 raw = load_stream(reinterpret_cast<const uint4*>(src) + i);
            const unsigned w[4] = {raw.x, raw.y, raw.z, raw.w};
#pragma unroll
            for (int j = 0; j < 4; j++) {
                const unsigned short lo = (unsigned short)(w[j] & 0xffffu), hi = (unsigned short)(w[j] >> 16);
                f[2 * j] = to_f32<S>(__builtin_bit_cast(S, lo));
                f[2 * j + 1] = to_f32<S>(__builtin_bit_cast(S, hi));
            }
        }
        if constexpr (sizeof(D) == 4) {
            reinterpret_cast<float4*>(dst)[2 * i] = make_float4(f[0], f[1], f[2], f[3]);
            reinterpret_cast<float4*>(dst)[2 * i + 1] = make_float4(f[4], f[5], f[6], f[7]);
        } else {
            unsigned w[4];
#pragma unroll
            for (int j = 0; j < 4; j++) {
                const unsigned lo = __builtin_bit_cast(unsigned short, from_f32<D>(f[2 * j]));
                const unsigned hi = __builtin_bit_cast(unsigned short, from_f32<D>(f[2 * j + 1]));
                w[j] = lo | (hi << 16);
            }
            reinterpret_cast<uint4*>(dst)[i] = make_uint4(w[0], w[1], w[2], w[3]);
        }
    }
}

// Same type on both sides: a copy, one 16-byte granule per thread (the form that measured fastest: 5.3-5.6 TB/s at
// 2 x 34 MB, 6.0-6.5 TB/s from 2 x 134 MB up; two granules per thread as in cast_x8_kernel: 4.6 / 5.1-5.5).
__global__ __launch_bounds__(kBlock) void copy_x16_kernel(const uint4* __restrict__ src, uint4* __restrict__ dst, int64_t n16) {
    const int64_t stride = (int64_t)gridDim.x * kBlock;
    for (int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x; i < n16; i += stride)
        store_stream(dst + i, load_stream(src + i));
}

template <typename S, typename D>
void cast_launch(const void* src, void* dst, int64_t n, hipStream_t st) {
    if (std::is_same<S, D>::value && (n * (int64_t)sizeof(S)) % 16 == 0 && aligned16(src) && aligned16(dst)) {
        const int64_t n16 = n * (int64_t)sizeof(S) / 16;
        copy_x16_kernel<<<grid_for(n16, kBlock), kBlock, 0, st>>>((const uint4*)src, (uint4*)dst, n16);
        return;
    }
    if (n % 8 == 0 && aligned16(src) && aligned16(dst))
        cast_x8_kernel<S, D><<<grid_for(n / 8, kBlock), kBlock, 0, st>>>((const S*)src, (D*)dst, n / 8);
    else
        cast_kernel<S, D><<<grid_for((n + 3) / 4, kBlock), kBlock, 0, st>>>((const S*)src, (D*)dst, n);
}

template <typename S>
int cast_from(const void* src, void* dst, int dst_dtype, int64_t n, hipStream_t st) {
    switch (dst_dtype) {
        case BR_F32: cast_launch<S, float>(src, dst, n, st); break;
        case BR_F16: cast_launch<S, __half>(src, dst, n, st); break;
        case BR_BF16: cast_launch<S, __hip_bfloat16>(src, dst, n, st); break;
        default: return BR_ERR_TODO;
    }
    BR_HIP_LAUNCH_CHECK();
    return BR_OK;
}

// --------------------------------------------------------- broadcast add
// Same-shape fast path: 128-bit loads, no index arithmetic.
__global__ __launch_bounds__(kBlock) void add_same_f32x4(const float4* a, const float4* b, float4* c,
                                                          int64_t n4) {
    const int64_t stride = (int64_t)gridDim.x * kBlock;
    for (int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x; i < n4; i += stride) {
        float4 x = a[i], y = b[i];
        c[i] = make_float4(x.x + y.x, x.y + y.y, x.z + y.z, x.w + y.w);
    }
}

__global__ __launch_bounds__(kBlock) void add_same_f16x8(const half8* a, const half8* b, half8* c,
                                                          int64_t n8) {
    const int64_t stride = (int64_t)gridDim.x * kBlock;
    for (int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x; i < n8; i += stride) {
        half8 x = a[i], y = b[i], z;
#pragma unroll
        for (int j = 0; j < 4; j++) {
            // add in fp32 and round once, like a + b on fp16 values
            float2 fx = __half22float2(x.v[j]), fy = __half22float2(y.v[j]);
            z.v[j] = __floats2half2_rn(fx.x + fy.x, fx.y + fy.y);
        }
        c[i] = z;
    }
}

struct BcastDims {
    unsigned s1, s2, s3v;      // a's dims 1,2 and dim 3 in vectors
    long long bst0, bst1, bst2;  // b's element strides (0 where broadcast)
    int bst3;                    // 0 when b's last dim is broadcast, else 1
};

// General path over vectors of 4 fp32 along the last dimension.
__global__ __launch_bounds__(kBlock) void add_bcast_f32x4(const float* a, const float* b, float* c,
                                                           long long nvec, BcastDims d) {
    const long long stride = (long long)gridDim.x * kBlock;
    for (long long v = (long long)blockIdx.x * kBlock + threadIdx.x; v < nvec; v += stride) {
        unsigned long long r = (unsigned long long)v;
        const unsigned i3v = (unsigned)(r % d.s3v);
        r /= d.s3v;
        const unsigned i2 = (unsigned)(r % d.s2);
        r /= d.s2;
        const unsigned i1 = (unsigned)(r % d.s1);
        const unsigned long long i0 = r / d.s1;
        const float4 x = reinterpret_cast<const float4*>(a)[v];
        const float* bp = b + i0 * d.bst0 + i1 * d.bst1 + i2 * d.bst2;
        float4 y;
        if (d.bst3) {
            y = *reinterpret_cast<const float4*>(bp + (long long)i3v * 4);
        } else {
            const float s = bp[0];
            y = make_float4(s, s, s, s);
        }
        reinterpret_cast<float4*>(c)[v] = make_float4(x.x + y.x, x.y + y.y, x.z + y.z, x.w + y.w);
    }
}

// Fallback for shapes / pointers that do not allow 128-bit accesses.
template <typename T>
__global__ __launch_bounds__(kBlock) void add_bcast_scalar(const T* a, const T* b, T* c, long long n,
                                                            unsigned s1, unsigned s2, unsigned s3,
                                                            long long bst0, long long bst1,
                                                            long long bst2, int bst3) {
    const long long stride = (long long)gridDim.x * kBlock;
    for (long long v = (long long)blockIdx.x * kBlock + threadIdx.x; v < n; v += stride) {
        unsigned long long r = (unsigned long long)v;
        const unsigned i3 = (unsigned)(r % s3);
        r /= s3;
        const unsigned i2 = (unsigned)(r % s2);
        r /= s2;
        const unsigned i1 = (unsigned)(r % s1);
        const unsigned long long i0 = r / s1;
        const T y = b[i0 * bst0 + i1 * bst1 + i2 * bst2 + (long long)i3 * bst3];
        c[v] = from_f32<T>(to_f32<T>(a[v]) + to_f32<T>(y));
    }
}

// ------------------------------------------------------------------ GELU
// d/dv gelu(v) = s + 2 v s (1 - s) u',  s = sigmoid(2u),
//   u = 0.79788456 v (1 + 0.044715 v^2),  u' = 0.79788456 + 0.1070322243 v^2
// evaluated from e = exp(-2|u|) = 2^(-|w|), w = 2*log2(e)*u, in (0,1] so that s
// and s(1-s) keep full relative accuracy for large |v|.
__device__ __forceinline__ float gelu_grad_one(float v) {
    const float v2 = v * v;
    const float w = v * (kLog2e2 * 0.79788456f + (kLog2e2 * 0.79788456f * 0.044715f) * v2);
    const float e = __builtin_amdgcn_exp2f(-fabsf(w));
    const float inv = __builtin_amdgcn_rcpf(1.0f + e);
    const float ei = e * inv;
    const float s = w >= 0.f ? inv : ei;
    return s + v * (ei * inv) * (2.0f * 0.79788456f + (2.0f * 0.1070322243f) * v2);
}

__global__ __launch_bounds__(kBlock) void gelu_fwd_f32(const float* x, float* y, int64_t n4) {
    const int64_t stride = (int64_t)gridDim.x * kBlock;
    for (int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x; i < n4; i += stride) {
        const float4 v = reinterpret_cast<const float4*>(x)[i];
        reinterpret_cast<float4*>(y)[i] =
            make_float4(gelu_one(v.x), gelu_one(v.y), gelu_one(v.z), gelu_one(v.w));
    }
}

__global__ __launch_bounds__(kBlock) void gelu_fwd_f16(const half8* x, half8* y, int64_t n8) {
    const int64_t stride = (int64_t)gridDim.x * kBlock;
    for (int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x; i < n8; i += stride) {
        float f[8];
        unpack8(x[i], f);
#pragma unroll
        for (int j = 0; j < 8; j++) f[j] = gelu_one(f[j]);
        y[i] = pack8(f);
    }
}

// fp32 in, 16-bit out: the output of the 4h activation when it only feeds the
// next product (rounded once, exactly as that product would round an fp32 copy)
template <typename D>
__global__ __launch_bounds__(kBlock) void gelu_fwd_f32_to_16(const float4* x, uint4* y, int64_t n8) {
    const int64_t stride = (int64_t)gridDim.x * kBlock;
    for (int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x; i < n8; i += stride) {
        const float4 a = x[2 * i], b = x[2 * i + 1];
        float f[8] = {a.x, a.y, a.z, a.w, b.x, b.y, b.z, b.w};
        unsigned w[4];
#pragma unroll
        for (int j = 0; j < 4; j++) {
            float lo = gelu_one(f[2 * j]), hi = gelu_one(f[2 * j + 1]);
            // the fp32 results are rounded to fp32 first, then to the 16-bit type
            asm volatile("" : "+v"(lo), "+v"(hi));
            w[j] = (unsigned)__builtin_bit_cast(unsigned short, from_f32<D>(lo)) |
                   ((unsigned)__builtin_bit_cast(unsigned short, from_f32<D>(hi)) << 16);
        }
        y[i] = make_uint4(w[0], w[1], w[2], w[3]);
    }
}

__global__ __launch_bounds__(kBlock) void gelu_bwd_f32(const float* dy, const float* x, float* dx,
                                                        int64_t n4) {
    const int64_t stride = (int64_t)gridDim.x * kBlock;
    for (int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x; i < n4; i += stride) {
        const float4 v = reinterpret_cast<const float4*>(x)[i];
        const float4 g = reinterpret_cast<const float4*>(dy)[i];
        reinterpret_cast<float4*>(dx)[i] =
            make_float4(g.x * gelu_grad_one(v.x), g.y * gelu_grad_one(v.y),
                        g.z * gelu_grad_one(v.z), g.w * gelu_grad_one(v.w));
    }
}

__global__ __launch_bounds__(kBlock) void gelu_bwd_f16(const half8* dy, const half8* x, half8* dx,
                                                        int64_t n8) {
    const int64_t stride = (int64_t)gridDim.x * kBlock;
    for (int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x; i < n8; i += stride) {
        float v[8], g[8];
        unpack8(x[i], v);
        unpack8(dy[i], g);
#pragma unroll
        for (int j = 0; j < 8; j++) g[j] *= gelu_grad_one(v[j]);
        dx[i] = pack8(g);
    }
}

template <typename T>
__global__ __launch_bounds__(kBlock) void gelu_scalar(const T* dy, const T* x, const float* bias, T* out,
                                                       int64_t n, int64_t cols, bool backward) {
    const int64_t stride = (int64_t)gridDim.x * kBlock;
    for (int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x; i < n; i += stride) {
        float v = to_f32<T>(x[i]);
        if (bias) v += bias[i % cols];
        out[i] = from_f32<T>(backward ? to_f32<T>(dy[i]) * gelu_grad_one(v) : gelu_one(v));
    }
}

// Bias-GELU backward over a strip of rows.  A workgroup owns kBlock*VEC
// columns and `rows_per_block` rows; each thread keeps VEC running column
// sums of dx in registers and writes them to partial[blockIdx.y][col].
template <typename T, int VEC>
struct VecIO;
template <>
struct VecIO<float, 4> {
    static __device__ __forceinline__ void load(const float* p, float (&f)[4]) {
        const float4 v = load_stream(reinterpret_cast<const float4*>(p));
        f[0] = v.x; f[1] = v.y; f[2] = v.z; f[3] = v.w;
    }
    static __device__ __forceinline__ void store(float* p, const float (&f)[4]) {
        store_stream(reinterpret_cast<float4*>(p), make_float4(f[0], f[1], f[2], f[3]));
    }
    // store, and leave in f exactly the values that were stored
    static __device__ __forceinline__ void store_rounded(float* p, float (&f)[4]) { store(p, f); }
};
template <>
struct VecIO<__half, 8> {
    static __device__ __forceinline__ void load(const __half* p, float (&f)[8]) {
        unpack8(load_stream(reinterpret_cast<const half8*>(p)), f);
    }
    static __device__ __forceinline__ void store(__half* p, const float (&f)[8]) {
        store_stream(reinterpret_cast<half8*>(p), pack8(f));
    }
    // The compiler is free to fuse the producing multiply into the fp16
    // conversion (v_fma_mixlo_f16: one rounding) for one use and not for
    // another (v_mul_f32 + v_cvt: two roundings), which differ on rare inputs.
    // The empty asm makes the packed registers opaque, so the store and the
    // read-back see the very same bits.
    static __device__ __forceinline__ void store_rounded(__half* p, float (&f)[8]) {
        uint4 u = __builtin_bit_cast(uint4, pack8(f));
        asm volatile("" : "+v"(u.x), "+v"(u.y), "+v"(u.z), "+v"(u.w));
        const half8 h = __builtin_bit_cast(half8, u);
        store_stream(reinterpret_cast<half8*>(p), h);
        unpack8(h, f);
    }
};

template <>
struct VecIO<__hip_bfloat16, 8> {
    static __device__ __forceinline__ void load(const __hip_bfloat16* p, float (&f)[8]) {
        unpack(load_stream(reinterpret_cast<const uint4*>(p)), f);
    }
    static __device__ __forceinline__ void unpack(const uint4& u, float (&f)[8]) {
        const unsigned w[4] = {u.x, u.y, u.z, u.w};
#pragma unroll
        for (int i = 0; i < 4; i++) {
            f[2 * i] = __builtin_bit_cast(float, w[i] << 16);
            f[2 * i + 1] = __builtin_bit_cast(float, w[i] & 0xffff0000u);
        }
    }
    static __device__ __forceinline__ uint4 pack(const float (&f)[8]) {
        unsigned w[4];
#pragma unroll
        for (int i = 0; i < 4; i++)
            w[i] = (unsigned)__builtin_bit_cast(unsigned short, __float2bfloat16(f[2 * i])) |
                   ((unsigned)__builtin_bit_cast(unsigned short, __float2bfloat16(f[2 * i + 1])) << 16);
        return make_uint4(w[0], w[1], w[2], w[3]);
    }
    static __device__ __forceinline__ void store(__hip_bfloat16* p, const float (&f)[8]) {
        store_stream(reinterpret_cast<uint4*>(p), pack(f));
    }
    static __device__ __forceinline__ void store_rounded(__hip_bfloat16* p, float (&f)[8]) {
        uint4 u = pack(f);
        asm volatile("" : "+v"(u.x), "+v"(u.y), "+v"(u.z), "+v"(u.w));
        store_stream(reinterpret_cast<uint4*>(p), u);
        unpack(u, f);
    }
};

// The rows of one strip of a strip kernel (grid y = strips).  Strip s takes rows s, s + S, s + 2S, ... (S strips): all
// workgroups of the launch then read one window of S consecutive rows at a time and the launch sweeps memory front
// to back (see grid_for), instead of S windows a strip apart (bias-GELU backward at [2048,16384]: 43.0 -> 41.6 us).
// A strip's rows are summed in this order, whatever the kernel.
#ifndef BR_STRIPS_INTERLEAVED
#define BR_STRIPS_INTERLEAVED 1
#endif
struct StripWalk {
    int64_t first, end, step;
};
__device__ __forceinline__ StripWalk strip_walk(int64_t rows, int rows_per_block) {
    if (BR_STRIPS_INTERLEAVED) return StripWalk{(int64_t)blockIdx.y, rows, (int64_t)gridDim.y};
    const int64_t r0 = (int64_t)blockIdx.y * rows_per_block;
    return StripWalk{r0, r0 + rows_per_block < rows ? r0 + rows_per_block : rows, 1};
}

// Bias-GELU forward with the same tiling: the VEC bias values of a thread's
// columns stay in registers while it walks down its strip of rows.
template <typename T, int VEC>
__global__ __launch_bounds__(kBlock) void bias_gelu_fwd_kernel(const T* x, const float* bias, T* y,
                                                                int64_t rows, int64_t cols,
                                                                int rows_per_block) {
    const int64_t col = ((int64_t)blockIdx.x * kBlock + threadIdx.x) * VEC;
    if (col >= cols) return;
    float b[VEC];
#pragma unroll
    for (int j = 0; j < VEC; j++) b[j] = bias[col + j];
    const int64_t r0 = (int64_t)blockIdx.y * rows_per_block;
    const int64_t r1 = r0 + rows_per_block < rows ? r0 + rows_per_block : rows;
    // four rows of loads in flight per thread
    int64_t r = r0;
    for (; r + 4 <= r1; r += 4) {
        float v[4][VEC];
#pragma unroll
        for (int u = 0; u < 4; u++) VecIO<T, VEC>::load(x + (r + u) * cols + col, v[u]);
#pragma unroll
        for (int u = 0; u < 4; u++) {
#pragma unroll
            for (int j = 0; j < VEC; j++) v[u][j] = gelu_one(v[u][j] + b[j]);
            VecIO<T, VEC>::store(y + (r + u) * cols + col, v[u]);
        }
    }
    for (; r < r1; r++) {
        float v[VEC];
        VecIO<T, VEC>::load(x + r * cols + col, v);
#pragma unroll
        for (int j = 0; j < VEC; j++) v[j] = gelu_one(v[j] + b[j]);
        VecIO<T, VEC>::store(y + r * cols + col, v);
    }
}

template <typename T, int VEC>
__global__ __launch_bounds__(kBlock) void bias_gelu_bwd_kernel(const T* dy, const T* x, const float* bias,
                                                                T* dx, float* partial, int64_t rows,
                                                                int64_t cols, int rows_per_block) {
    const int64_t col = ((int64_t)blockIdx.x * kBlock + threadIdx.x) * VEC;
    if (col >= cols) return;
    float b[VEC], acc[VEC];
#pragma unroll
    for (int j = 0; j < VEC; j++) {
        b[j] = bias ? bias[col + j] : 0.f;
        acc[j] = 0.f;
    }
    const StripWalk w = strip_walk(rows, rows_per_block);
    const int64_t step = w.step, r1 = w.end;
    // four rows (eight loads) in flight per thread; a strip's rows are still summed in order
    int64_t r = w.first;
    for (; r + 3 * step < r1; r += 4 * step) {
        float v[4][VEC], g[4][VEC];
#pragma unroll
        for (int u = 0; u < 4; u++) {
            VecIO<T, VEC>::load(x + (r + u * step) * cols + col, v[u]);
            VecIO<T, VEC>::load(dy + (r + u * step) * cols + col, g[u]);
        }
#pragma unroll
        for (int u = 0; u < 4; u++) {
#pragma unroll
            for (int j = 0; j < VEC; j++) g[u][j] *= gelu_grad_one(v[u][j] + b[j]);
            // sum what was stored, i.e. after rounding to the storage type
            VecIO<T, VEC>::store_rounded(dx + (r + u * step) * cols + col, g[u]);
#pragma unroll
            for (int j = 0; j < VEC; j++) acc[j] += g[u][j];
        }
    }
    for (; r < r1; r += step) {
        float v[VEC], g[VEC];
        VecIO<T, VEC>::load(x + r * cols + col, v);
        VecIO<T, VEC>::load(dy + r * cols + col, g);
#pragma unroll
        for (int j = 0; j < VEC; j++) g[j] *= gelu_grad_one(v[j] + b[j]);
        VecIO<T, VEC>::store_rounded(dx + r * cols + col, g);
#pragma unroll
        for (int j = 0; j < VEC; j++) acc[j] += g[j];
    }
    if (partial) {
#pragma unroll
        for (int j = 0; j < VEC; j++) partial[(int64_t)blockIdx.y * cols + col + j] = acc[j];
    }
}

// --------------------------------------------------------------- colsum
// Stage 1: partial[g][c] = sum over the g-th strip of rows of x[r,c].
template <typename T>
__global__ __launch_bounds__(kBlock) void colsum_partial(const T* x, float* partial, int64_t rows,
                                                          int64_t cols, int rows_per_block) {
    const int64_t col = (int64_t)blockIdx.x * kBlock + threadIdx.x;
    if (col >= cols) return;
    const int64_t r0 = (int64_t)blockIdx.y * rows_per_block;
    const int64_t r1 = r0 + rows_per_block < rows ? r0 + rows_per_block : rows;
    float acc = 0.f;
    for (int64_t r = r0; r < r1; r++) acc += to_f32<T>(x[r * cols + col]);
    partial[(int64_t)blockIdx.y * cols + col] = acc;
}

// Stage 2: out[c] = sum_g partial[g][c]  (fixed order: deterministic).
__global__ __launch_bounds__(kBlock) void colsum_final(const float* partial, float* out, int groups,
                                                        int64_t cols, float scale) {
    const int64_t col = (int64_t)blockIdx.x * kBlock + threadIdx.x;
    if (col >= cols) return;
    float acc = 0.f;
    for (int g = 0; g < groups; g++) acc += partial[(int64_t)g * cols + col];
    out[col] = acc * scale;
}

// Vector forms of the two stages (cols % VEC == 0, 16-byte aligned rows).
// Stage 1: a thread owns VEC adjacent columns and sums a strip of rows, four
// rows of loads in flight at a time.
template <typename T, int VEC>
__global__ __launch_bounds__(kBlock) void colsum_partial_vec(const T* __restrict__ x, float* __restrict__ partial,
                                                              int64_t rows, int64_t cols, int rows_per_block) {
    const int64_t col = ((int64_t)blockIdx.x * kBlock + threadIdx.x) * VEC;
    if (col >= cols) return;
    const StripWalk w = strip_walk(rows, rows_per_block);
    const int64_t step = w.step, r1 = w.end;
    float acc[VEC];
#pragma unroll
    for (int j = 0; j < VEC; j++) acc[j] = 0.f;
    int64_t r = w.first;
    for (; r + 3 * step < r1; r += 4 * step) {
        float v[4][VEC];
#pragma unroll
        for (int u = 0; u < 4; u++) VecIO<T, VEC>::load(x + (r + u * step) * cols + col, v[u]);
#pragma unroll
        for (int u = 0; u < 4; u++)
#pragma unroll
            for (int j = 0; j < VEC; j++) acc[j] += v[u][j];
    }
    for (; r < r1; r += step) {
        float v[VEC];
        VecIO<T, VEC>::load(x + r * cols + col, v);
#pragma unroll
        for (int j = 0; j < VEC; j++) acc[j] += v[j];
    }
#pragma unroll
    for (int j = 0; j < VEC; j++) partial[(int64_t)blockIdx.y * cols + col + j] = acc[j];
}

// Stage 1 for fp32 x that is also wanted as a 16-bit copy (the gradient of a
// linear layer: its column sums are the bias gradient, its 16-bit copy is the
// operand of the two products that follow): one pass over x does both.
template <typename D>
__global__ __launch_bounds__(kBlock) void colsum_cast_partial(const float* __restrict__ x, float* __restrict__ partial,
                                                               D* __restrict__ x16, int64_t rows, int64_t cols,
                                                               int rows_per_block) {
    const int64_t col = ((int64_t)blockIdx.x * kBlock + threadIdx.x) * 4;
    if (col >= cols) return;
    const StripWalk w = strip_walk(rows, rows_per_block);
    const int64_t step = w.step, r1 = w.end;
    float acc[4] = {0.f, 0.f, 0.f, 0.f};
    auto emit = [&](int64_t r, const float (&v)[4]) {
        const unsigned lo = (unsigned)__builtin_bit_cast(unsigned short, from_f32<D>(v[0])) |
                            ((unsigned)__builtin_bit_cast(unsigned short, from_f32<D>(v[1])) << 16);
        const unsigned hi = (unsigned)__builtin_bit_cast(unsigned short, from_f32<D>(v[2])) |
                            ((unsigned)__builtin_bit_cast(unsigned short, from_f32<D>(v[3])) << 16);
        *reinterpret_cast<uint2*>(x16 + r * cols + col) = make_uint2(lo, hi);
    };
    int64_t r = w.first;
    for (; r + 3 * step < r1; r += 4 * step) {
        float v[4][4];
#pragma unroll
        for (int u = 0; u < 4; u++) VecIO<float, 4>::load(x + (r + u * step) * cols + col, v[u]);
#pragma unroll
        for (int u = 0; u < 4; u++) {
#pragma unroll
            for (int j = 0; j < 4; j++) acc[j] += v[u][j];
            emit(r + u * step, v[u]);
        }
    }
    for (; r < r1; r += step) {
        float v[4];
        VecIO<float, 4>::load(x + r * cols + col, v);
#pragma unroll
        for (int j = 0; j < 4; j++) acc[j] += v[j];
        emit(r, v);
    }
#pragma unroll
    for (int j = 0; j < 4; j++) partial[(int64_t)blockIdx.y * cols + col + j] = acc[j];
}

// The same pass with x produced on the fly: x = dy * gelu'(u), the GELU
// backward whose result is the gradient of the linear layer below it.  Writes
// the fp32 gradient (dx may be u's or dy's own buffer), its 16-bit copy and
// the column-sum partials; dx is rounded to fp32 before it is summed and
// converted, so all three equal what the separate kernels produce.
template <typename D>
__global__ __launch_bounds__(kBlock) void gelu_bwd_colsum_cast_partial(const float* dy, const float* u, float* dx,
                                                                        float* __restrict__ partial,
                                                                        D* __restrict__ dx16, int64_t rows,
                                                                        int64_t cols, int rows_per_block) {
    const int64_t col = ((int64_t)blockIdx.x * kBlock + threadIdx.x) * 4;
    if (col >= cols) return;
    const StripWalk w = strip_walk(rows, rows_per_block);
    const int64_t step = w.step, r1 = w.end;
    float acc[4] = {0.f, 0.f, 0.f, 0.f};
    auto emit = [&](int64_t r, const float (&g)[4], const float (&x)[4]) {
        float v[4];
#pragma unroll
        for (int j = 0; j < 4; j++) {
            v[j] = g[j] * gelu_grad_one(x[j]);
            asm volatile("" : "+v"(v[j]));
            acc[j] += v[j];
        }
        VecIO<float, 4>::store(dx + r * cols + col, v);
        const unsigned lo = (unsigned)__builtin_bit_cast(unsigned short, from_f32<D>(v[0])) |
                            ((unsigned)__builtin_bit_cast(unsigned short, from_f32<D>(v[1])) << 16);
        const unsigned hi = (unsigned)__builtin_bit_cast(unsigned short, from_f32<D>(v[2])) |
                            ((unsigned)__builtin_bit_cast(unsigned short, from_f32<D>(v[3])) << 16);
        *reinterpret_cast<uint2*>(dx16 + r * cols + col) = make_uint2(lo, hi);
    };
    int64_t r = w.first;
    for (; r + step < r1; r += 2 * step) {
        float g[2][4], x[2][4];
#pragma unroll
        for (int k = 0; k < 2; k++) {
            VecIO<float, 4>::load(dy + (r + k * step) * cols + col, g[k]);
            VecIO<float, 4>::load(u + (r + k * step) * cols + col, x[k]);
        }
#pragma unroll
        for (int k = 0; k < 2; k++) emit(r + k * step, g[k], x[k]);
    }
    for (; r < r1; r += step) {
        float g[4], x[4];
        VecIO<float, 4>::load(dy + r * cols + col, g);
        VecIO<float, 4>::load(u + r * cols + col, x);
        emit(r, g, x);
    }
#pragma unroll
    for (int j = 0; j < 4; j++) partial[(int64_t)blockIdx.y * cols + col + j] = acc[j];
}

// Stage 2 for cols % 4 == 0: 1024 threads = 16 column quads x 64 slices of
// groups, every load of a workgroup in flight at once; slices are combined in
// LDS in a fixed order.
__global__ __launch_bounds__(1024) void colsum_final_x4(const float4* __restrict__ partial, float4* __restrict__ out,
                                                        int groups, int cols4, float scale) {
    __shared__ float4 l[64][16];
    const int q = threadIdx.x & 15, sl = threadIdx.x >> 4;
    const int c4 = blockIdx.x * 16 + q;
    float4 s = make_float4(0.f, 0.f, 0.f, 0.f);
    if (c4 < cols4) {
#pragma unroll 4
        for (int g = sl; g < groups; g += 64) {
            const float4 a = partial[(int64_t)g * cols4 + c4];
            s.x += a.x; s.y += a.y; s.z += a.z; s.w += a.w;
        }
    }
    l[sl][q] = s;
    __syncthreads();
    if (sl < 8) {
        for (int k = sl + 8; k < 64; k += 8) {
            const float4 a = l[k][q];
            s.x += a.x; s.y += a.y; s.z += a.z; s.w += a.w;
        }
        l[sl][q] = s;
    }
    __syncthreads();
    if (sl == 0 && c4 < cols4) {
        for (int k = 1; k < 8; k++) {
            const float4 a = l[k][q];
            s.x += a.x; s.y += a.y; s.z += a.z; s.w += a.w;
        }
        out[c4] = make_float4(s.x * scale, s.y * scale, s.z * scale, s.w * scale);
    }
}

// Launches stage 2 in its vector form when the shapes allow.
int colsum_finish(const float* partial, float* out, int groups, int64_t cols, float scale, hipStream_t st) {
    if (cols % 4 == 0 && aligned16(partial) && aligned16(out))
        colsum_final_x4<<<(unsigned)((cols / 4 + 15) / 16), 1024, 0, st>>>(reinterpret_cast<const float4*>(partial),
                                                                            reinterpret_cast<float4*>(out), groups,
                                                                            (int)(cols / 4), scale);
    else
        colsum_final<<<(unsigned)((cols + kBlock - 1) / kBlock), kBlock, 0, st>>>(partial, out, groups, cols, scale);
    BR_HIP_LAUNCH_CHECK();
    return BR_OK;
}

// Row strips of the vector column sum: about 1024 workgroups in all, at most
// 256 strips.
constexpr int kMaxColsumGroups = 256;
int colsum_vec_rows_per_block(int64_t rows, int64_t blocks_x) {
    int64_t groups = 1024 / (blocks_x < 1 ? 1 : blocks_x);
    if (groups < 1) groups = 1;
    if (groups > kMaxColsumGroups) groups = kMaxColsumGroups;
    int64_t rpb = (rows + groups - 1) / groups;
    if (rpb < 4) rpb = 4;
    return (int)rpb;
}

// ------------------------------------------------ column sums in one launch
// A workgroup of 1024 threads owns 8 * VEC columns (128 bytes of a 16-bit row, 128 bytes of an fp32 row) and walks
// ALL rows: 8 lanes per row, 128 rows per pass, UNROLL passes in flight.  No partial sums leave the workgroup and
// there is no second launch; the 128 row slots are combined in LDS in a fixed order, so the result depends on the
// shape alone.  Measured against the two launches: 16-bit [2048,12288] 11.4 against 15.5 us, [2048,16384] 14.3
// against 18.9, [512,16384] 4.6 against 11.0; fp32 [512,4096] with a 16-bit copy 3.9 against 6.6 -- but fp32
// [2048,4096] 17 against 13.4 (128 workgroups are too few for 50 MB) and the fp16 bias-GELU backward at [2048,16384]
// 44.5 against 43.0 (its arithmetic wants more waves than 1024 threads per CU give), which therefore keep the two
// launches above 1024 rows (colsum_owner_applies).  Whole BLOOM-7B1 step at 512 tokens: -0.9 %.  What is summed, and what else is written on the way, is the Source's business:
//   load(at, in)      the loads of one row position (all of a pass's loads are issued before any is used)
//   finish(at, in)    leaves the values to be summed in in[0]; may store
template <typename T, int V>
struct OwnPlain {
    const T* x;
    static constexpr int VEC = V, NIN = 1;
    __device__ __forceinline__ void init(int64_t) {}
    __device__ __forceinline__ void load(int64_t at, float (&in)[NIN][VEC]) const { VecIO<T, V>::load(x + at, in[0]); }
    __device__ __forceinline__ void finish(int64_t, float (&)[NIN][VEC]) const {}
};
template <typename D>
__device__ __forceinline__ void store4_as16(D* p, const float (&v)[4]) {
    const unsigned lo = (unsigned)__builtin_bit_cast(unsigned short, from_f32<D>(v[0])) |
                        ((unsigned)__builtin_bit_cast(unsigned short, from_f32<D>(v[1])) << 16);
    const unsigned hi = (unsigned)__builtin_bit_cast(unsigned short, from_f32<D>(v[2])) |
                        ((unsigned)__builtin_bit_cast(unsigned short, from_f32<D>(v[3])) << 16);
    *reinterpret_cast<uint2*>(p) = make_uint2(lo, hi);
}
// fp32 x, summed as it is, with its 16-bit copy written (colsum_cast_partial)
template <typename D>
struct OwnCast {
    const float* x;
    D* x16;
    static constexpr int VEC = 4, NIN = 1;
    __device__ __forceinline__ void init(int64_t) {}
    __device__ __forceinline__ void load(int64_t at, float (&in)[NIN][VEC]) const { VecIO<float, 4>::load(x + at, in[0]); }
    __device__ __forceinline__ void finish(int64_t at, float (&in)[NIN][VEC]) const { store4_as16<D>(x16 + at, in[0]); }
};
// dx = dy * gelu'(u) in fp32, written as fp32 and as a 16-bit copy, summed (gelu_bwd_colsum_cast_partial)
template <typename D>
struct OwnGeluBwdCast {
    const float* dy;
    const float* u;
    float* dx;
    D* dx16;
    static constexpr int VEC = 4, NIN = 2;
    __device__ __forceinline__ void init(int64_t) {}
    __device__ __forceinline__ void load(int64_t at, float (&in)[NIN][VEC]) const {
        VecIO<float, 4>::load(dy + at, in[0]);
        VecIO<float, 4>::load(u + at, in[1]);
    }
    __device__ __forceinline__ void finish(int64_t at, float (&in)[NIN][VEC]) const {
#pragma unroll
        for (int j = 0; j < 4; j++) {
            in[0][j] = in[0][j] * gelu_grad_one(in[1][j]);
            asm volatile("" : "+v"(in[0][j]));   // one fp32 value for the store, the copy and the sum
        }
        VecIO<float, 4>::store(dx + at, in[0]);
        store4_as16<D>(dx16 + at, in[0]);
    }
};
// dx = dy * gelu'(x + bias) in the storage type; what was stored is what is summed (bias_gelu_bwd_kernel)
template <typename T, int V>
struct OwnBiasGeluBwd {
    const T* dy;
    const T* x;
    const float* bias;
    T* dx;
    float b[V];
    static constexpr int VEC = V, NIN = 2;
    __device__ __forceinline__ void init(int64_t col) {
#pragma unroll
        for (int j = 0; j < V; j++) b[j] = bias ? bias[col + j] : 0.f;
    }
    __device__ __forceinline__ void load(int64_t at, float (&in)[NIN][VEC]) const {
        VecIO<T, V>::load(dy + at, in[0]);
        VecIO<T, V>::load(x + at, in[1]);
    }
    __device__ __forceinline__ void finish(int64_t at, float (&in)[NIN][VEC]) const {
#pragma unroll
        for (int j = 0; j < V; j++) in[0][j] *= gelu_grad_one(in[1][j] + b[j]);
        VecIO<T, V>::store_rounded(dx + at, in[0]);
    }
};

constexpr int kOwnThreads = 1024, kOwnLanesPerRow = 8, kOwnRowsPerPass = kOwnThreads / kOwnLanesPerRow;

template <int UNROLL, typename Src>
__global__ __launch_bounds__(kOwnThreads) void colsum_owner_kernel(Src src_arg, float* __restrict__ out, int64_t rows,
                                                                   int64_t cols, float scale) {
    constexpr int VEC = Src::VEC, NIN = Src::NIN, RPP = kOwnRowsPerPass, CW = kOwnLanesPerRow * VEC;
    __shared__ float slots[RPP][CW + 1];
    Src src = src_arg;
    const int lr = threadIdx.x % kOwnLanesPerRow, rr = threadIdx.x / kOwnLanesPerRow;
    const int64_t col = (int64_t)blockIdx.x * CW + lr * VEC;
    float acc[VEC];
#pragma unroll
    for (int j = 0; j < VEC; j++) acc[j] = 0.f;
    if (col < cols) {
        src.init(col);
        int64_t r = rr;
        for (; r + (UNROLL - 1) * RPP < rows; r += UNROLL * RPP) {
            float in[UNROLL][NIN][VEC];
#pragma unroll
            for (int u = 0; u < UNROLL; u++) src.load((r + u * RPP) * cols + col, in[u]);
#pragma unroll
            for (int u = 0; u < UNROLL; u++) {
                src.finish((r + u * RPP) * cols + col, in[u]);
#pragma unroll
                for (int j = 0; j < VEC; j++) acc[j] += in[u][0][j];
            }
        }
        for (; r < rows; r += RPP) {
            float in[NIN][VEC];
            src.load(r * cols + col, in);
            src.finish(r * cols + col, in);
#pragma unroll
            for (int j = 0; j < VEC; j++) acc[j] += in[0][j];
        }
    }
#pragma unroll
    for (int j = 0; j < VEC; j++) slots[rr][lr * VEC + j] = acc[j];
    __syncthreads();
    // 1024 / CW threads per column take every (1024 / CW)-th slot, then one thread per column takes those
    constexpr int SLICES = kOwnThreads / CW;
    static_assert(SLICES <= RPP, "the second stage reuses the slots");
    const int c = threadIdx.x % CW, s = threadIdx.x / CW;
    float t = 0.f;
    for (int k = s; k < RPP; k += SLICES) t += slots[k][c];
    __syncthreads();
    slots[s][c] = t;
    __syncthreads();
    if (s == 0) {
        float z = 0.f;
        for (int k = 0; k < SLICES; k++) z += slots[k][c];
        const int64_t oc = (int64_t)blockIdx.x * CW + c;
        if (oc < cols) out[oc] = z * scale;
    }
}

// Where one launch beats two (measured, see above): enough column blocks to occupy the chip, and for 4-byte elements
// (32 columns per workgroup, half as many workgroups) and the bias-GELU backward only up to 1024 rows.  Depends on the shape and the element
// size alone, so entries that promise each other's bits (br_hip_colsum / br_hip_colsum_cast /
// br_hip_gelu_bwd_colsum_cast on fp32) always agree on the path.
#ifndef BR_COLSUM_OWNER
#define BR_COLSUM_OWNER 3   // bit 0: plain sums and sums with a copy; bit 1: the bias-GELU backward
#endif
bool colsum_owner_applies(int64_t rows, int64_t cols, int elem_bytes, int kind = 1) {
    if (!(BR_COLSUM_OWNER & kind)) return false;
    const int64_t cw = kOwnLanesPerRow * (elem_bytes == 4 ? 4 : 8);
    const int64_t blocks = (cols + cw - 1) / cw;
    if (cols % (elem_bytes == 4 ? 4 : 8) != 0 || blocks < 96 || blocks > 0x7fffffffLL) return false;
    return (elem_bytes == 2 && kind == 1) || rows <= 1024;
}

template <int UNROLL, typename Src>
int colsum_owner_launch(const Src& src, float* out, int64_t rows, int64_t cols, float scale, hipStream_t st) {
    const int64_t cw = kOwnLanesPerRow * Src::VEC;
    colsum_owner_kernel<UNROLL, Src><<<(unsigned)((cols + cw - 1) / cw), kOwnThreads, 0, st>>>(src, out, rows, cols, scale);
    BR_HIP_LAUNCH_CHECK();
    return BR_OK;
}

// ------------------------------------------------------- transpose 0213
// One 16-byte granule per thread, indexed by OUTPUT position so stores are
// fully coalesced; loads are contiguous runs of s3 elements.
__global__ __launch_bounds__(kBlock) void transpose_0213_x16(const uint4* x, uint4* y, long long n16,
                                                              unsigned s1, unsigned s2, unsigned s3g) {
    const long long stride = (long long)gridDim.x * kBlock;
    for (long long o = (long long)blockIdx.x * kBlock + threadIdx.x; o < n16; o += stride) {
        unsigned long long r = (unsigned long long)o;
        const unsigned i3 = (unsigned)(r % s3g);
        r /= s3g;
        const unsigned i1 = (unsigned)(r % s1);  // output dim 2 is input dim 1
        r /= s1;
        const unsigned i2 = (unsigned)(r % s2);
        const unsigned long long i0 = r / s2;
        y[o] = x[((i0 * s1 + i1) * s2 + i2) * s3g + i3];
    }
}

template <typename T>
__global__ __launch_bounds__(kBlock) void transpose_0213_scalar(const T* x, T* y, long long n, unsigned s1,
                                                                 unsigned s2, unsigned s3) {
    const long long stride = (long long)gridDim.x * kBlock;
    for (long long o = (long long)blockIdx.x * kBlock + threadIdx.x; o < n; o += stride) {
        unsigned long long r = (unsigned long long)o;
        const unsigned i3 = (unsigned)(r % s3);
        r /= s3;
        const unsigned i1 = (unsigned)(r % s1);
        r /= s1;
        const unsigned i2 = (unsigned)(r % s2);
        const unsigned long long i0 = r / s2;
        y[o] = x[((i0 * s1 + i1) * s2 + i2) * s3 + i3];
    }
}

// ------------------------------------------------------ data preparation
// One workgroup per output row; rows whose id is out of range are zeroed.
__global__ __launch_bounds__(kBlock) void gather_rows_x16(const uint4* table, const int32_t* ids, uint4* out,
                                                           int64_t row16, int64_t vocab) {
    const int64_t row = blockIdx.x;
    const int64_t id = ids[row];
    const bool ok = id >= 0 && id < vocab;
    for (int64_t i = threadIdx.x; i < row16; i += kBlock)
        out[row * row16 + i] = ok ? table[id * row16 + i] : make_uint4(0, 0, 0, 0);
}

__global__ __launch_bounds__(kBlock) void gather_rows_bytes(const unsigned char* table, const int32_t* ids,
                                                             unsigned char* out, int64_t row_bytes,
                                                             int64_t vocab) {
    const int64_t row = blockIdx.x;
    const int64_t id = ids[row];
    const bool ok = id >= 0 && id < vocab;
    for (int64_t i = threadIdx.x; i < row_bytes; i += kBlock)
        out[row * row_bytes + i] = ok ? table[id * row_bytes + i] : (unsigned char)0;
}

constexpr int kSlopeChunk = 128;
struct SlopeChunk {
    double v[kSlopeChunk];
};

__global__ __launch_bounds__(kBlock) void alibi_table_kernel(float* alibi, SlopeChunk slopes, int head0,
                                                              int nheads, int64_t tokens) {
    const int64_t n = (int64_t)nheads * tokens;
    const int64_t stride = (int64_t)gridDim.x * kBlock;
    for (int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x; i < n; i += stride) {
        const int h = (int)(i / tokens);
        const int64_t k = i % tokens;
        // fp64 product rounded once to fp32, as the host code it replaces does
        alibi[(int64_t)head0 * tokens + i] = (float)((double)k * 1.0 * slopes.v[h]);
    }
}

// One workgroup per (batch, query row).  valid = index of the first zero in
// mask[b,:] (tokens when there is none) is found by a min-reduction.
__global__ __launch_bounds__(kBlock) void xmask_table_kernel(const int32_t* mask, float* xmask,
                                                              int64_t tokens) {
    __shared__ int s_valid[kBlock / kWave];
    const int64_t b = blockIdx.y;
    const int64_t q = blockIdx.x;
    const int32_t* m = mask + b * tokens;
    int first_zero = (int)tokens;
    // keys beyond q are masked by causality anyway, so scanning [0, q] suffices
    for (int64_t k = threadIdx.x; k <= q; k += kBlock)
        if (m[k] == 0 && (int)k < first_zero) first_zero = (int)k;
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) {
        const int o = __shfl_xor(first_zero, off, kWave);
        first_zero = o < first_zero ? o : first_zero;
    }
    if ((threadIdx.x & 63) == 0) s_valid[threadIdx.x >> 6] = first_zero;
    __syncthreads();
    int valid = s_valid[0];
#pragma unroll
    for (int w = 1; w < kBlock / kWave; w++) valid = s_valid[w] < valid ? s_valid[w] : valid;
    float* row = xmask + (b * tokens + q) * tokens;
    for (int64_t k = threadIdx.x; k < tokens; k += kBlock)
        row[k] = (k <= q && k < valid) ? 0.0f : -FLT_MAX;
}

bool fits_u32(int64_t v) { return v > 0 && v <= 0xffffffffLL; }

// ---------------------------------------------------------- normal fill
// dst[i] = mean + std * z_i with z_i a standard normal that depends only on
// (seed, i): SplitMix64 of the pair gives two 24-bit uniforms, Box-Muller one
// normal.  The same (seed, i) gives the same value on any launch geometry.
__device__ __forceinline__ unsigned long long splitmix64(unsigned long long x) {
    x += 0x9E3779B97F4A7C15ull;
    x = (x ^ (x >> 30)) * 0xBF58476D1CE4E5B9ull;
    x = (x ^ (x >> 27)) * 0x94D049BB133111EBull;
    return x ^ (x >> 31);
}
template <typename T>
__global__ __launch_bounds__(kBlock) void normal_kernel(T* dst, float mean, float std, unsigned long long seed,
                                                         int64_t n) {
    const int64_t stride = (int64_t)gridDim.x * kBlock;
    for (int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x; i < n; i += stride) {
        const unsigned long long h = splitmix64(splitmix64(seed) ^ (unsigned long long)i);
        const float u1 = ((float)(unsigned)(h >> 40) + 1.0f) * (1.0f / 16777216.0f);  // (0, 1]
        const float u2 = (float)(unsigned)((h >> 8) & 0xffffffu) * (1.0f / 16777216.0f);
        const float z = sqrtf(-2.0f * __logf(u1)) * __cosf(6.28318530718f * u2);
        float value = mean + std * z;
        // keep the fp32 rounding: without the barrier the multiply-add is fused into
        // the 16-bit conversion and a 16-bit tensor would not be the rounded fp32 one
        asm volatile("" : "+v"(value));
        dst[i] = from_f32<T>(value);
    }
}

// Backward of the row gather: grad[ids[i], :] += dx[i, :] for i = 0 .. n-1, in
// that order, so that the result does not depend on scheduling when an id
// occurs several times.  Workgroup i owns id = ids[i] only if i is that id's
// first position; it then folds every later position with the same id into the
// row, in ascending position order, starting from the row's current value.
__global__ __launch_bounds__(kBlock) void scatter_add_rows(const float* __restrict__ dx,
                                                            const int32_t* __restrict__ ids, float* grad, int n,
                                                            int64_t hidden, int64_t vocab, float scale, bool vec) {
    const int i = blockIdx.x;
    const int32_t id = ids[i];
    if (id < 0 || (int64_t)id >= vocab) return;
    int seen = 0;
    for (int j = threadIdx.x; j < i; j += kBlock) seen |= ids[j] == id;
    if (__syncthreads_or(seen)) return;
    float* row = grad + (int64_t)id * hidden;
    if (vec) {
        const int64_t h4 = hidden / 4;
        for (int64_t c = threadIdx.x; c < h4; c += kBlock) {
            float4 acc = reinterpret_cast<float4*>(row)[c];
            for (int j = i; j < n; j++) {
                if (ids[j] != id) continue;
                const float4 d = reinterpret_cast<const float4*>(dx + (int64_t)j * hidden)[c];
                acc.x += d.x * scale; acc.y += d.y * scale; acc.z += d.z * scale; acc.w += d.w * scale;
            }
            reinterpret_cast<float4*>(row)[c] = acc;
        }
    } else {
        for (int64_t c = threadIdx.x; c < hidden; c += kBlock) {
            float acc = row[c];
            for (int j = i; j < n; j++)
                if (ids[j] == id) acc += dx[(int64_t)j * hidden + c] * scale;
            row[c] = acc;
        }
    }
}

}  // namespace

extern "C" {

int br_hip_fill(void* dst, int dtype, float value, int64_t n, br_stream_t stream) {
    if (n < 0) return BR_ERR_ATTR;
    if (n == 0) return BR_OK;
    if (!dst) return BR_ERR_OUTPUT;
    hipStream_t st = as_stream(stream);
    const int grid = grid_for(n, kBlock);
    switch (dtype) {
        case BR_F32: fill_kernel<float><<<grid, kBlock, 0, st>>>((float*)dst, value, n); break;
        case BR_F16: fill_kernel<__half><<<grid, kBlock, 0, st>>>((__half*)dst, __float2half_rn(value), n); break;
        case BR_BF16:
            fill_kernel<__hip_bfloat16><<<grid, kBlock, 0, st>>>((__hip_bfloat16*)dst, __float2bfloat16(value), n);
            break;
        case BR_I32: fill_kernel<int32_t><<<grid, kBlock, 0, st>>>((int32_t*)dst, (int32_t)value, n); break;
        default: return BR_ERR_TODO;
    }
    BR_HIP_LAUNCH_CHECK();
    return BR_OK;
}

int br_hip_normal(void* dst, int dtype, float mean, float std, uint64_t seed, int64_t n, br_stream_t stream) {
    if (n < 0) return BR_ERR_ATTR;
    if (n == 0) return BR_OK;
    if (!dst) return BR_ERR_OUTPUT;
    hipStream_t st = as_stream(stream);
    const int grid = grid_for(n, kBlock);
    switch (dtype) {
        case BR_F32: normal_kernel<float><<<grid, kBlock, 0, st>>>((float*)dst, mean, std, seed, n); break;
        case BR_F16: normal_kernel<__half><<<grid, kBlock, 0, st>>>((__half*)dst, mean, std, seed, n); break;
        case BR_BF16:
            normal_kernel<__hip_bfloat16><<<grid, kBlock, 0, st>>>((__hip_bfloat16*)dst, mean, std, seed, n);
            break;
        default: return BR_ERR_TODO;
    }
    BR_HIP_LAUNCH_CHECK();
    return BR_OK;
}

int br_hip_cast(const void* src, int src_dtype, void* dst, int dst_dtype, int64_t n, br_stream_t stream) {
    if (n < 0) return BR_ERR_ATTR;
    if (n == 0) return BR_OK;
    if (!src) return BR_ERR_INPUT;
    if (!dst) return BR_ERR_OUTPUT;
    hipStream_t st = as_stream(stream);
    switch (src_dtype) {
        case BR_F32: return cast_from<float>(src, dst, dst_dtype, n, st);
        case BR_F16: return cast_from<__half>(src, dst, dst_dtype, n, st);
        case BR_BF16: return cast_from<__hip_bfloat16>(src, dst, dst_dtype, n, st);
        default: return BR_ERR_TODO;
    }
}

int br_hip_add_bcast(const void* a, const void* b, void* c, int dtype, const int64_t as[4],
                     const int64_t bs[4], br_stream_t stream) {
    if (!a || !b || !as || !bs) return BR_ERR_INPUT;
    if (!c) return BR_ERR_OUTPUT;
    if (dtype != BR_F32 && dtype != BR_F16) return BR_ERR_TODO;
    bool same = true;
    for (int i = 0; i < 4; i++) {
        if (as[i] <= 0 || bs[i] <= 0) return BR_ERR_ATTR;
        if (bs[i] != as[i] && bs[i] != 1) return BR_ERR_INPUT;
        same = same && bs[i] == as[i];
    }
    const int64_t n = as[0] * as[1] * as[2] * as[3];
    hipStream_t st = as_stream(stream);
    const bool al = aligned16(a) && aligned16(b) && aligned16(c);
    if (same && al && dtype == BR_F32 && n % 4 == 0) {
        add_same_f32x4<<<grid_for(n / 4, kBlock), kBlock, 0, st>>>((const float4*)a, (const float4*)b,
                                                                   (float4*)c, n / 4);
        BR_HIP_LAUNCH_CHECK();
        return BR_OK;
    }
    if (same && al && dtype == BR_F16 && n % 8 == 0) {
        add_same_f16x8<<<grid_for(n / 8, kBlock), kBlock, 0, st>>>((const half8*)a, (const half8*)b,
                                                                   (half8*)c, n / 8);
        BR_HIP_LAUNCH_CHECK();
        return BR_OK;
    }
    if (!fits_u32(as[1]) || !fits_u32(as[2]) || !fits_u32(as[3])) return BR_ERR_ATTR;
    const long long bst3 = bs[3] == 1 ? 0 : 1;
    const long long bst2 = bs[2] == 1 ? 0 : bs[3];
    const long long bst1 = bs[1] == 1 ? 0 : bs[2] * bs[3];
    const long long bst0 = bs[0] == 1 ? 0 : bs[1] * bs[2] * bs[3];
    // 128-bit path: needs every row start of a, b and c to stay 16-byte aligned
    const bool vec_ok = dtype == BR_F32 && al && as[3] % 4 == 0 && (bst3 == 0 || bs[3] % 4 == 0);
    if (vec_ok) {
        BcastDims d;
        d.s1 = (unsigned)as[1];
        d.s2 = (unsigned)as[2];
        d.s3v = (unsigned)(as[3] / 4);
        d.bst0 = bst0; d.bst1 = bst1; d.bst2 = bst2; d.bst3 = (int)bst3;
        add_bcast_f32x4<<<grid_for(n / 4, kBlock), kBlock, 0, st>>>((const float*)a, (const float*)b,
                                                                    (float*)c, n / 4, d);
    } else if (dtype == BR_F32) {
        add_bcast_scalar<float><<<grid_for(n, kBlock), kBlock, 0, st>>>(
            (const float*)a, (const float*)b, (float*)c, n, (unsigned)as[1], (unsigned)as[2],
            (unsigned)as[3], bst0, bst1, bst2, (int)bst3);
    } else {
        add_bcast_scalar<__half><<<grid_for(n, kBlock), kBlock, 0, st>>>(
            (const __half*)a, (const __half*)b, (__half*)c, n, (unsigned)as[1], (unsigned)as[2],
            (unsigned)as[3], bst0, bst1, bst2, (int)bst3);
    }
    BR_HIP_LAUNCH_CHECK();
    return BR_OK;
}

static int strip_rows(int64_t rows) {
    // strips of rows per workgroup: about 64 strips, at least 8 rows each
    int64_t rpb = (rows + 63) / 64;
    if (rpb < 8) rpb = 8;
    return (int)rpb;
}

int br_hip_gelu_fwd_f32_to_16(const float* x, void* y, int y_dtype, int64_t n, br_stream_t stream) {
    if (n < 0) return BR_ERR_ATTR;
    if (n == 0) return BR_OK;
    if (!x) return BR_ERR_INPUT;
    if (!y) return BR_ERR_OUTPUT;
    if (y_dtype != BR_F16 && y_dtype != BR_BF16) return BR_ERR_TODO;
    if (n % 8 != 0 || !aligned16(x) || !aligned16(y)) return BR_ERR_TODO;
    const int grid = grid_for(n / 8, kBlock);
    if (y_dtype == BR_F16)
        gelu_fwd_f32_to_16<__half><<<grid, kBlock, 0, as_stream(stream)>>>((const float4*)x, (uint4*)y, n / 8);
    else
        gelu_fwd_f32_to_16<__hip_bfloat16><<<grid, kBlock, 0, as_stream(stream)>>>((const float4*)x, (uint4*)y, n / 8);
    BR_HIP_LAUNCH_CHECK();
    return BR_OK;
}

int br_hip_gelu_fwd(const void* x, void* y, int dtype, int64_t n, br_stream_t stream) {
    if (n < 0) return BR_ERR_ATTR;
    if (n == 0) return BR_OK;
    if (!x) return BR_ERR_INPUT;
    if (!y) return BR_ERR_OUTPUT;
    hipStream_t st = as_stream(stream);
    const bool al = aligned16(x) && aligned16(y);
    if (dtype == BR_F32 && al && n % 4 == 0) {
        gelu_fwd_f32<<<grid_for(n / 4, kBlock), kBlock, 0, st>>>((const float*)x, (float*)y, n / 4);
    } else if (dtype == BR_F16 && al && n % 8 == 0) {
        gelu_fwd_f16<<<grid_for(n / 8, kBlock), kBlock, 0, st>>>((const half8*)x, (half8*)y, n / 8);
    } else if (dtype == BR_F32) {
        gelu_scalar<float><<<grid_for(n, kBlock), kBlock, 0, st>>>(nullptr, (const float*)x, nullptr, (float*)y,
                                                                  n, 1, false);
    } else if (dtype == BR_F16) {
        gelu_scalar<__half><<<grid_for(n, kBlock), kBlock, 0, st>>>(nullptr, (const __half*)x, nullptr,
                                                                   (__half*)y, n, 1, false);
    } else {
        return BR_ERR_TODO;
    }
    BR_HIP_LAUNCH_CHECK();
    return BR_OK;
}

int br_hip_bias_gelu_fwd(const void* x, const float* bias, void* y, int dtype, int64_t rows, int64_t cols,
                         br_stream_t stream) {
    if (rows < 0 || cols <= 0) return BR_ERR_ATTR;
    if (rows == 0) return BR_OK;
    if (!x || !bias) return BR_ERR_INPUT;
    if (!y) return BR_ERR_OUTPUT;
    if (dtype != BR_F32 && dtype != BR_F16) return BR_ERR_TODO;
    hipStream_t st = as_stream(stream);
#ifndef BR_GELU_FWD_FLAT
#define BR_GELU_FWD_FLAT 1
#endif
    // one row per workgroup row of the grid (workgroups in memory order, see grid_for) while the grid allows
    const int rpb = BR_GELU_FWD_FLAT && rows <= 65535 ? 1 : strip_rows(rows);
    const unsigned groups = (unsigned)((rows + rpb - 1) / rpb);
    const bool al = aligned16(x) && aligned16(y);
    if (dtype == BR_F32 && al && cols % 4 == 0) {
        dim3 grid((unsigned)((cols / 4 + kBlock - 1) / kBlock), groups);
        bias_gelu_fwd_kernel<float, 4><<<grid, kBlock, 0, st>>>((const float*)x, bias, (float*)y, rows, cols, rpb);
    } else if (dtype == BR_F16 && al && cols % 8 == 0) {
        dim3 grid((unsigned)((cols / 8 + kBlock - 1) / kBlock), groups);
        bias_gelu_fwd_kernel<__half, 8><<<grid, kBlock, 0, st>>>((const __half*)x, bias, (__half*)y, rows, cols,
                                                                  rpb);
    } else {
        const int64_t n = rows * cols;
        if (dtype == BR_F32)
            gelu_scalar<float><<<grid_for(n, kBlock), kBlock, 0, st>>>(nullptr, (const float*)x, bias, (float*)y,
                                                                      n, cols, false);
        else
            gelu_scalar<__half><<<grid_for(n, kBlock), kBlock, 0, st>>>(nullptr, (const __half*)x, bias,
                                                                       (__half*)y, n, cols, false);
    }
    BR_HIP_LAUNCH_CHECK();
    return BR_OK;
}

int br_hip_gelu_bwd(const void* dy, const void* x, void* dx, int dtype, int64_t n, br_stream_t stream) {
    if (n < 0) return BR_ERR_ATTR;
    if (n == 0) return BR_OK;
    if (!dy || !x) return BR_ERR_INPUT;
    if (!dx) return BR_ERR_OUTPUT;
    hipStream_t st = as_stream(stream);
    const bool al = aligned16(dy) && aligned16(x) && aligned16(dx);
    if (dtype == BR_F32 && al && n % 4 == 0) {
        gelu_bwd_f32<<<grid_for(n / 4, kBlock), kBlock, 0, st>>>((const float*)dy, (const float*)x, (float*)dx,
                                                                n / 4);
    } else if (dtype == BR_F16 && al && n % 8 == 0) {
        gelu_bwd_f16<<<grid_for(n / 8, kBlock), kBlock, 0, st>>>((const half8*)dy, (const half8*)x, (half8*)dx,
                                                                n / 8);
    } else if (dtype == BR_F32) {
        gelu_scalar<float><<<grid_for(n, kBlock), kBlock, 0, st>>>((const float*)dy, (const float*)x, nullptr,
                                                                  (float*)dx, n, 1, true);
    } else if (dtype == BR_F16) {
        gelu_scalar<__half><<<grid_for(n, kBlock), kBlock, 0, st>>>((const __half*)dy, (const __half*)x, nullptr,
                                                                   (__half*)dx, n, 1, true);
    } else {
        return BR_ERR_TODO;
    }
    BR_HIP_LAUNCH_CHECK();
    return BR_OK;
}

size_t br_hip_bias_gelu_bwd_workspace(int64_t rows, int64_t cols) { return br_hip_colsum_workspace(rows, cols); }

int br_hip_bias_gelu_bwd(const void* dy, const void* x, const float* bias, void* dx, float* dbias, int dtype,
                         int64_t rows, int64_t cols, float dbias_scale, void* workspace, size_t workspace_bytes,
                         br_stream_t stream) {
    if (rows < 0 || cols <= 0) return BR_ERR_ATTR;
    if (rows == 0) return BR_OK;
    if (!dy || !x) return BR_ERR_INPUT;
    if (!dx) return BR_ERR_OUTPUT;
    if (dtype != BR_F32 && dtype != BR_F16 && dtype != BR_BF16) return BR_ERR_TODO;
    hipStream_t st = as_stream(stream);
    const int rpb = strip_rows(rows);
    const int groups = (int)((rows + rpb - 1) / rpb);
    float* partial = nullptr;
    if (dbias) {
        if (!workspace || workspace_bytes < br_hip_bias_gelu_bwd_workspace(rows, cols)) return BR_ERR_ATTR;
        partial = (float*)workspace;
    }
    const bool al = aligned16(dy) && aligned16(x) && aligned16(dx);
    if (dbias && al && colsum_owner_applies(rows, cols, dtype == BR_F32 ? 4 : 2, 2)) {
        // gradient and bias gradient from one launch
        if (dtype == BR_F32)
            return colsum_owner_launch<2>(OwnBiasGeluBwd<float, 4>{(const float*)dy, (const float*)x, bias, (float*)dx},
                                          dbias, rows, cols, dbias_scale, st);
        if (dtype == BR_F16)
            return colsum_owner_launch<2>(OwnBiasGeluBwd<__half, 8>{(const __half*)dy, (const __half*)x, bias, (__half*)dx},
                                          dbias, rows, cols, dbias_scale, st);
        return colsum_owner_launch<2>(OwnBiasGeluBwd<__hip_bfloat16, 8>{(const __hip_bfloat16*)dy, (const __hip_bfloat16*)x,
                                                                        bias, (__hip_bfloat16*)dx},
                                      dbias, rows, cols, dbias_scale, st);
    }
    if (dtype == BR_F32 && al && cols % 4 == 0) {
        dim3 grid((unsigned)((cols / 4 + kBlock - 1) / kBlock), (unsigned)groups);
        bias_gelu_bwd_kernel<float, 4><<<grid, kBlock, 0, st>>>((const float*)dy, (const float*)x, bias,
                                                                 (float*)dx, partial, rows, cols, rpb);
    } else if (dtype == BR_F16 && al && cols % 8 == 0) {
        dim3 grid((unsigned)((cols / 8 + kBlock - 1) / kBlock), (unsigned)groups);
        bias_gelu_bwd_kernel<__half, 8><<<grid, kBlock, 0, st>>>((const __half*)dy, (const __half*)x, bias,
                                                                  (__half*)dx, partial, rows, cols, rpb);
    } else if (dtype == BR_BF16 && al && cols % 8 == 0) {
        dim3 grid((unsigned)((cols / 8 + kBlock - 1) / kBlock), (unsigned)groups);
        bias_gelu_bwd_kernel<__hip_bfloat16, 8><<<grid, kBlock, 0, st>>>((const __hip_bfloat16*)dy,
                                                                         (const __hip_bfloat16*)x, bias,
                                                                         (__hip_bfloat16*)dx, partial, rows, cols, rpb);
    } else if (dtype == BR_BF16) {
        return BR_ERR_TODO;
    } else {
        // unaligned shapes: elementwise pass, then a separate column sum of dx
        const int64_t n = rows * cols;
        if (dtype == BR_F32)
            gelu_scalar<float><<<grid_for(n, kBlock), kBlock, 0, st>>>((const float*)dy, (const float*)x, bias,
                                                                      (float*)dx, n, cols, true);
        else
            gelu_scalar<__half><<<grid_for(n, kBlock), kBlock, 0, st>>>((const __half*)dy, (const __half*)x,
                                                                       bias, (__half*)dx, n, cols, true);
        BR_HIP_LAUNCH_CHECK();
        if (dbias) return br_hip_colsum(dx, dtype, dbias, rows, cols, dbias_scale, workspace, workspace_bytes, stream);
        return BR_OK;
    }
    BR_HIP_LAUNCH_CHECK();
    if (dbias) return colsum_finish(partial, dbias, groups, cols, dbias_scale, st);
    return BR_OK;
}

size_t br_hip_colsum_workspace(int64_t rows, int64_t cols) {
    if (rows <= 0 || cols <= 0) return 0;
    const int rpb = strip_rows(rows);
    const size_t strips = (size_t)((rows + rpb - 1) / rpb) * (size_t)cols * sizeof(float);
    const size_t vec = (size_t)kMaxColsumGroups * (size_t)cols * sizeof(float);
    return strips > vec ? strips : vec;
}

int br_hip_colsum(const void* x, int dtype, float* out, int64_t rows, int64_t cols, float out_scale, void* workspace,
                  size_t workspace_bytes, br_stream_t stream) {
    if (rows < 0 || cols <= 0) return BR_ERR_ATTR;
    if (!out) return BR_ERR_OUTPUT;
    hipStream_t st = as_stream(stream);
    if (rows == 0) return br_hip_fill(out, BR_F32, 0.f, cols, stream);
    if (!x) return BR_ERR_INPUT;
    if (!workspace || workspace_bytes < br_hip_colsum_workspace(rows, cols)) return BR_ERR_ATTR;
    if (dtype != BR_F32 && dtype != BR_F16 && dtype != BR_BF16) return BR_ERR_TODO;
    float* partial = (float*)workspace;
    const int vec = dtype == BR_F32 ? 4 : 8;
    if (cols % vec == 0 && aligned16(x) && (cols * (dtype == BR_F32 ? 4 : 2)) % 16 == 0) {
        if (colsum_owner_applies(rows, cols, dtype == BR_F32 ? 4 : 2)) {
            if (dtype == BR_F32) return colsum_owner_launch<4>(OwnPlain<float, 4>{(const float*)x}, out, rows, cols, out_scale, st);
            if (dtype == BR_F16) return colsum_owner_launch<4>(OwnPlain<__half, 8>{(const __half*)x}, out, rows, cols, out_scale, st);
            return colsum_owner_launch<4>(OwnPlain<__hip_bfloat16, 8>{(const __hip_bfloat16*)x}, out, rows, cols, out_scale, st);
        }
        const int64_t blocks_x = (cols / vec + kBlock - 1) / kBlock;
        const int rpb = colsum_vec_rows_per_block(rows, blocks_x);
        const int groups = (int)((rows + rpb - 1) / rpb);
        dim3 grid((unsigned)blocks_x, (unsigned)groups);
        if (dtype == BR_F32)
            colsum_partial_vec<float, 4><<<grid, kBlock, 0, st>>>((const float*)x, partial, rows, cols, rpb);
        else if (dtype == BR_F16)
            colsum_partial_vec<__half, 8><<<grid, kBlock, 0, st>>>((const __half*)x, partial, rows, cols, rpb);
        else
            colsum_partial_vec<__hip_bfloat16, 8><<<grid, kBlock, 0, st>>>((const __hip_bfloat16*)x, partial, rows, cols,
                                                                          rpb);
        BR_HIP_LAUNCH_CHECK();
        return colsum_finish(partial, out, groups, cols, out_scale, st);
    }
    const int rpb = strip_rows(rows);
    const int groups = (int)((rows + rpb - 1) / rpb);
    dim3 grid((unsigned)((cols + kBlock - 1) / kBlock), (unsigned)groups);
    if (dtype == BR_F32)
        colsum_partial<float><<<grid, kBlock, 0, st>>>((const float*)x, partial, rows, cols, rpb);
    else if (dtype == BR_F16)
        colsum_partial<__half><<<grid, kBlock, 0, st>>>((const __half*)x, partial, rows, cols, rpb);
    else
        colsum_partial<__hip_bfloat16><<<grid, kBlock, 0, st>>>((const __hip_bfloat16*)x, partial, rows, cols, rpb);
    BR_HIP_LAUNCH_CHECK();
    return colsum_finish(partial, out, groups, cols, out_scale, st);
}

int br_hip_colsum_cast(const float* x, float* out, void* x16, int x16_dtype, int64_t rows, int64_t cols,
                       float out_scale, void* workspace, size_t workspace_bytes, br_stream_t stream) {
    if (rows <= 0 || cols <= 0) return BR_ERR_ATTR;
    if (!x) return BR_ERR_INPUT;
    if (!out || !x16) return BR_ERR_OUTPUT;
    if (x16_dtype != BR_F16 && x16_dtype != BR_BF16) return BR_ERR_TODO;
    if (cols % 4 != 0 || !aligned16(x) || (reinterpret_cast<uintptr_t>(x16) & 7u) != 0) return BR_ERR_TODO;
    if (!workspace || workspace_bytes < br_hip_colsum_workspace(rows, cols)) return BR_ERR_ATTR;
    hipStream_t st = as_stream(stream);
    if (colsum_owner_applies(rows, cols, 4)) {
        if (x16_dtype == BR_F16) return colsum_owner_launch<4>(OwnCast<__half>{x, (__half*)x16}, out, rows, cols, out_scale, st);
        return colsum_owner_launch<4>(OwnCast<__hip_bfloat16>{x, (__hip_bfloat16*)x16}, out, rows, cols, out_scale, st);
    }
    float* partial = (float*)workspace;
    const int64_t blocks_x = (cols / 4 + kBlock - 1) / kBlock;
    const int rpb = colsum_vec_rows_per_block(rows, blocks_x);
    const int groups = (int)((rows + rpb - 1) / rpb);
    dim3 grid((unsigned)blocks_x, (unsigned)groups);
    if (x16_dtype == BR_F16)
        colsum_cast_partial<__half><<<grid, kBlock, 0, st>>>(x, partial, (__half*)x16, rows, cols, rpb);
    else
        colsum_cast_partial<__hip_bfloat16><<<grid, kBlock, 0, st>>>(x, partial, (__hip_bfloat16*)x16, rows, cols, rpb);
    BR_HIP_LAUNCH_CHECK();
    return colsum_finish(partial, out, groups, cols, out_scale, st);
}

int br_hip_gelu_bwd_colsum_cast(const float* dy, const float* x, float* dx, float* out, void* dx16, int dx16_dtype,
                                int64_t rows, int64_t cols, float out_scale, void* workspace, size_t workspace_bytes,
                                br_stream_t stream) {
    if (rows <= 0 || cols <= 0) return BR_ERR_ATTR;
    if (!dy || !x) return BR_ERR_INPUT;
    if (!dx || !out || !dx16) return BR_ERR_OUTPUT;
    if (dx16_dtype != BR_F16 && dx16_dtype != BR_BF16) return BR_ERR_TODO;
    if (cols % 4 != 0 || !aligned16(dy) || !aligned16(x) || !aligned16(dx) ||
        (reinterpret_cast<uintptr_t>(dx16) & 7u) != 0)
        return BR_ERR_TODO;
    if (!workspace || workspace_bytes < br_hip_colsum_workspace(rows, cols)) return BR_ERR_ATTR;
    hipStream_t st = as_stream(stream);
    if (colsum_owner_applies(rows, cols, 4)) {
        if (dx16_dtype == BR_F16)
            return colsum_owner_launch<2>(OwnGeluBwdCast<__half>{dy, x, dx, (__half*)dx16}, out, rows, cols, out_scale, st);
        return colsum_owner_launch<2>(OwnGeluBwdCast<__hip_bfloat16>{dy, x, dx, (__hip_bfloat16*)dx16}, out, rows, cols,
                                      out_scale, st);
    }
    float* partial = (float*)workspace;
    // same strips as br_hip_colsum_cast, hence the same summation order
    const int64_t blocks_x = (cols / 4 + kBlock - 1) / kBlock;
    const int rpb = colsum_vec_rows_per_block(rows, blocks_x);
    const int groups = (int)((rows + rpb - 1) / rpb);
    dim3 grid((unsigned)blocks_x, (unsigned)groups);
    if (dx16_dtype == BR_F16)
        gelu_bwd_colsum_cast_partial<__half><<<grid, kBlock, 0, st>>>(dy, x, dx, partial, (__half*)dx16, rows, cols, rpb);
    else
        gelu_bwd_colsum_cast_partial<__hip_bfloat16><<<grid, kBlock, 0, st>>>(dy, x, dx, partial,
                                                                             (__hip_bfloat16*)dx16, rows, cols, rpb);
    BR_HIP_LAUNCH_CHECK();
    return colsum_finish(partial, out, groups, cols, out_scale, st);
}

int br_hip_transpose_0213(const void* x, void* y, int elem_bytes, int64_t s0, int64_t s1, int64_t s2,
                          int64_t s3, br_stream_t stream) {
    if (s0 < 0 || s1 <= 0 || s2 <= 0 || s3 <= 0) return BR_ERR_ATTR;
    if (elem_bytes != 2 && elem_bytes != 4) return BR_ERR_ATTR;
    if (s0 == 0) return BR_OK;
    if (!x) return BR_ERR_INPUT;
    if (!y || x == y) return BR_ERR_OUTPUT;
    if (!fits_u32(s1) || !fits_u32(s2) || !fits_u32(s3)) return BR_ERR_ATTR;
    hipStream_t st = as_stream(stream);
    const int64_t n = s0 * s1 * s2 * s3;
    const int per16 = 16 / elem_bytes;
    if (s3 % per16 == 0 && aligned16(x) && aligned16(y)) {
        const int64_t n16 = n / per16;
        transpose_0213_x16<<<grid_for(n16, kBlock), kBlock, 0, st>>>((const uint4*)x, (uint4*)y, n16,
                                                                    (unsigned)s1, (unsigned)s2,
                                                                    (unsigned)(s3 / per16));
    } else if (elem_bytes == 4) {
        transpose_0213_scalar<uint32_t><<<grid_for(n, kBlock), kBlock, 0, st>>>(
            (const uint32_t*)x, (uint32_t*)y, n, (unsigned)s1, (unsigned)s2, (unsigned)s3);
    } else {
        transpose_0213_scalar<uint16_t><<<grid_for(n, kBlock), kBlock, 0, st>>>(
            (const uint16_t*)x, (uint16_t*)y, n, (unsigned)s1, (unsigned)s2, (unsigned)s3);
    }
    BR_HIP_LAUNCH_CHECK();
    return BR_OK;
}

int br_hip_embedding_gather(const void* table, const int32_t* ids, void* out, int elem_bytes, int64_t n,
                            int64_t hidden, int64_t vocab, br_stream_t stream) {
    if (n < 0 || hidden <= 0 || vocab <= 0 || (elem_bytes != 2 && elem_bytes != 4)) return BR_ERR_ATTR;
    if (n == 0) return BR_OK;
    if (!table || !ids) return BR_ERR_INPUT;
    if (!out) return BR_ERR_OUTPUT;
    if (n > 0x7fffffff) return BR_ERR_ATTR;
    hipStream_t st = as_stream(stream);
    const int64_t row_bytes = hidden * elem_bytes;
    if (row_bytes % 16 == 0 && aligned16(table) && aligned16(out))
        gather_rows_x16<<<(unsigned)n, kBlock, 0, st>>>((const uint4*)table, ids, (uint4*)out, row_bytes / 16,
                                                        vocab);
    else
        gather_rows_bytes<<<(unsigned)n, kBlock, 0, st>>>((const unsigned char*)table, ids, (unsigned char*)out,
                                                          row_bytes, vocab);
    BR_HIP_LAUNCH_CHECK();
    return BR_OK;
}

int br_hip_embedding_scatter_add(const float* dx, const int32_t* ids, float* grad, int64_t n, int64_t hidden,
                                 int64_t vocab, float dx_scale, br_stream_t stream) {
    if (n < 0 || hidden <= 0 || vocab <= 0 || n > 0x7fffffff) return BR_ERR_ATTR;
    if (n == 0) return BR_OK;
    if (!dx || !ids) return BR_ERR_INPUT;
    if (!grad || (const float*)grad == dx) return BR_ERR_OUTPUT;
    const bool vec = hidden % 4 == 0 && aligned16(dx) && aligned16(grad);
    scatter_add_rows<<<(unsigned)n, kBlock, 0, as_stream(stream)>>>(dx, ids, grad, (int)n, hidden, vocab, dx_scale, vec);
    BR_HIP_LAUNCH_CHECK();
    return BR_OK;
}

int br_hip_alibi_table(float* alibi, int64_t heads, int64_t tokens, br_stream_t stream) {
    if (heads <= 0 || tokens <= 0 || heads > 65536) return BR_ERR_ATTR;
    if (!alibi) return BR_ERR_OUTPUT;
    hipStream_t st = as_stream(stream);
    double* slopes = new double[heads];
    br_hip_alibi_slopes(slopes, heads);
    int rc = BR_OK;
    for (int64_t h0 = 0; h0 < heads && rc == BR_OK; h0 += kSlopeChunk) {
        SlopeChunk c;
        const int nh = (int)(heads - h0 < kSlopeChunk ? heads - h0 : kSlopeChunk);
        for (int i = 0; i < kSlopeChunk; i++) c.v[i] = i < nh ? slopes[h0 + i] : 0.0;
        alibi_table_kernel<<<grid_for((int64_t)nh * tokens, kBlock), kBlock, 0, st>>>(alibi, c, (int)h0, nh,
                                                                                      tokens);
        hipError_t e = hipGetLastError();
        if (e != hipSuccess) rc = (int)e;
    }
    delete[] slopes;
    return rc;
}

int br_hip_xmask_table(const int32_t* mask, float* xmask, int64_t batch, int64_t tokens, br_stream_t stream) {
    if (batch < 0 || tokens <= 0 || tokens > 0x7fffffff || batch > 65535) return BR_ERR_ATTR;
    if (batch == 0) return BR_OK;
    if (!mask) return BR_ERR_INPUT;
    if (!xmask) return BR_ERR_OUTPUT;
    dim3 grid((unsigned)tokens, (unsigned)batch);
    xmask_table_kernel<<<grid, kBlock, 0, as_stream(stream)>>>(mask, xmask, tokens);
    BR_HIP_LAUNCH_CHECK();
    return BR_OK;
}

}  // extern "C"
