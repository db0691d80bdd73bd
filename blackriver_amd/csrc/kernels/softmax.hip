// Softmax family for gfx950.
//
// Attention softmax (rows of a few hundred to a few thousand scores): one
// wave64 per row, the row held in registers, so HBM sees one read and one
// write; the ALiBi bias and the additive causal / padding mask are folded in
// either from their tables or analytically.
//
// Vocabulary log-softmax + NLL (rows of 250 880 logits, 1 MB each): one
// 1024-thread workgroup per row, a single online (max, sum) sweep with
// 128-bit loads; the backward re-reads the row and writes the gradient.
#include "common.hpp"

#include <float.h>

using namespace brk;

namespace {

constexpr int kBlock = 256;
constexpr int kRowsPerBlock = kBlock / kWave;  // one wave per row

enum MaskMode { kPlain = 0, kTables = 1, kAnalytic = 2 };

struct RowBias {
    const float* alibi;   // [heads, tk]            (kTables)
    const float* xmask;   // [batch, tq, tk]        (kTables)
    const double* slopes; // [heads]                (kAnalytic)
    const int32_t* valid; // [batch]                (kAnalytic)
    int heads, tq;
};

// Scores, probabilities and their gradients are read once and written once: streaming (non-temporal) accesses,
// measured at [4,32,512,512] fp32 on one box: forward 55.4 us plain, 54.5 with streaming loads, 51.0 with streaming
// stores too; backward 71 / 66.6 / 62.4.
#ifndef BR_SM_STREAM
#define BR_SM_STREAM 7   // one-wave-per-row kernels: bit 0 streaming loads, bit 1 streaming stores (forward), bit 2 (backward)
#endif
__device__ __forceinline__ float4 sm_load(const float4* p) {
#if BR_SM_STREAM & 1
    return load_stream(p);
#else
    return *p;
#endif
}
template <int BIT>
__device__ __forceinline__ void sm_store(float4* p, const float4& v) {
    if (BR_SM_STREAM & BIT) store_stream(p, v);
    else *p = v;
}

// exp(x - m) for x <= m, via the hardware exp2
__device__ __forceinline__ float exp_sub(float x, float m) { return __expf(x - m); }

// VPL = float4 vectors per lane; cols = 4 * cols4 <= 256 * VPL.
template <int VPL, int MODE>
__global__ __launch_bounds__(kBlock) void softmax_fwd_wave(const float* __restrict__ x, float* __restrict__ y,
                                                            int64_t rows, int cols4, RowBias rb, Copy16 y16) {
    const int lane = threadIdx.x & 63;
    const int64_t row = (int64_t)blockIdx.x * kRowsPerBlock + (threadIdx.x >> 6);
    if (row >= rows) return;
    const float4* xr = reinterpret_cast<const float4*>(x) + row * cols4;
    float4 v[VPL];
#pragma unroll
    for (int i = 0; i < VPL; i++) {
        const int idx = lane + i * kWave;
        v[i] = idx < cols4 ? sm_load(xr + idx) : make_float4(-INFINITY, -INFINITY, -INFINITY, -INFINITY);
    }
    if (MODE != kPlain) {
        // row = (b * heads + h) * tq + q
        const int q = (int)(row % rb.tq);
        const int64_t bh = row / rb.tq;
        const int h = (int)(bh % rb.heads);
        const int64_t b = bh / rb.heads;
        if (MODE == kTables) {
            const float4* ar = rb.alibi ? reinterpret_cast<const float4*>(rb.alibi) + (int64_t)h * cols4 : nullptr;
            const float4* mr =
                rb.xmask ? reinterpret_cast<const float4*>(rb.xmask) + (b * rb.tq + q) * cols4 : nullptr;
#pragma unroll
            for (int i = 0; i < VPL; i++) {
                const int idx = lane + i * kWave;
                if (idx < cols4) {
                    if (ar) {
                        const float4 a = ar[idx];
                        v[i].x += a.x; v[i].y += a.y; v[i].z += a.z; v[i].w += a.w;
                    }
                    if (mr) {
                        const float4 m = mr[idx];
                        v[i].x += m.x; v[i].y += m.y; v[i].z += m.z; v[i].w += m.w;
                    }
                }
            }
        } else {
            const double slope = rb.slopes[h];
            const int valid = rb.valid[b];
#pragma unroll
            for (int i = 0; i < VPL; i++) {
                const int idx = lane + i * kWave;
                if (idx < cols4) {
                    float* e = reinterpret_cast<float*>(&v[i]);
#pragma unroll
                    for (int j = 0; j < 4; j++) {
                        const int k = idx * 4 + j;
                        // same two additions, in the same order, as the table form
                        e[j] += (float)((double)k * 1.0 * slope);
                        e[j] += (k <= q && k < valid) ? 0.0f : -FLT_MAX;
                    }
                }
            }
        }
    }
    float m = -INFINITY;
#pragma unroll
    for (int i = 0; i < VPL; i++) m = fmaxf(m, fmaxf(fmaxf(v[i].x, v[i].y), fmaxf(v[i].z, v[i].w)));
    m = wave_max(m);
    float s = 0.f;
#pragma unroll
    for (int i = 0; i < VPL; i++) {
        v[i].x = exp_sub(v[i].x, m); v[i].y = exp_sub(v[i].y, m);
        v[i].z = exp_sub(v[i].z, m); v[i].w = exp_sub(v[i].w, m);
        s += (v[i].x + v[i].y) + (v[i].z + v[i].w);
    }
    s = wave_sum(s);
    const float inv = 1.0f / s;
    float4* yr = reinterpret_cast<float4*>(y) + row * cols4;
#pragma unroll
    for (int i = 0; i < VPL; i++) {
        const int idx = lane + i * kWave;
        if (idx < cols4) {
            float4 o = make_float4(v[i].x * inv, v[i].y * inv, v[i].z * inv, v[i].w * inv);
            store4_as16(y16, row * cols4 + idx, o);
            sm_store<2>(yr + idx, o);
        }
    }
}

template <int VPL>
__global__ __launch_bounds__(kBlock) void softmax_bwd_wave(const float* __restrict__ dy, const float* __restrict__ y,
                                                            float* __restrict__ dx, int64_t rows, int cols4,
                                                            Copy16 dx16) {
    const int lane = threadIdx.x & 63;
    const int64_t row = (int64_t)blockIdx.x * kRowsPerBlock + (threadIdx.x >> 6);
    if (row >= rows) return;
    const float4* gr = reinterpret_cast<const float4*>(dy) + row * cols4;
    const float4* yr = reinterpret_cast<const float4*>(y) + row * cols4;
    float4 g[VPL], p[VPL];
    float dot = 0.f;
#pragma unroll
    for (int i = 0; i < VPL; i++) {
        const int idx = lane + i * kWave;
        const bool ok = idx < cols4;
        g[i] = ok ? sm_load(gr + idx) : make_float4(0.f, 0.f, 0.f, 0.f);
        p[i] = ok ? sm_load(yr + idx) : make_float4(0.f, 0.f, 0.f, 0.f);
        dot += (g[i].x * p[i].x + g[i].y * p[i].y) + (g[i].z * p[i].z + g[i].w * p[i].w);
    }
    dot = wave_sum(dot);
    float4* dr = dx ? reinterpret_cast<float4*>(dx) + row * cols4 : nullptr;
#pragma unroll
    for (int i = 0; i < VPL; i++) {
        const int idx = lane + i * kWave;
        if (idx < cols4) {
            float4 o = make_float4(p[i].x * (g[i].x - dot), p[i].y * (g[i].y - dot), p[i].z * (g[i].z - dot),
                                   p[i].w * (g[i].w - dot));
            store4_as16(dx16, row * cols4 + idx, o);
            if (dx) sm_store<4>(dr + idx, o);  // dx == nullptr: only the 16-bit gradient is wanted
        }
    }
}

// Any width / alignment: one workgroup per row, three sweeps from global.
template <int MODE>
__global__ __launch_bounds__(kBlock) void softmax_fwd_generic(const float* x, float* y, int64_t cols, RowBias rb) {
    __shared__ float lds[2][kBlock / kWave];
    const int64_t row = blockIdx.x;
    const float* xr = x + row * cols;
    float* yr = y + row * cols;
    const int q = MODE != kPlain ? (int)(row % rb.tq) : 0;
    const int64_t bh = MODE != kPlain ? row / rb.tq : 0;
    const int h = MODE != kPlain ? (int)(bh % rb.heads) : 0;
    const int64_t b = MODE != kPlain ? bh / rb.heads : 0;
    auto value = [&](int64_t c) -> float {
        float v = xr[c];
        if (MODE == kTables) {
            if (rb.alibi) v += rb.alibi[(int64_t)h * cols + c];
            if (rb.xmask) v += rb.xmask[(b * rb.tq + q) * cols + c];
        } else if (MODE == kAnalytic) {
            v += (float)((double)c * 1.0 * rb.slopes[h]);
            v += (c <= q && c < rb.valid[b]) ? 0.0f : -FLT_MAX;
        }
        return v;
    };
    float m = -INFINITY;
    for (int64_t c = threadIdx.x; c < cols; c += kBlock) m = fmaxf(m, value(c));
    m = wave_max(m);
    if ((threadIdx.x & 63) == 0) lds[0][threadIdx.x >> 6] = m;
    __syncthreads();
    m = lds[0][0];
    for (int w = 1; w < kBlock / kWave; w++) m = fmaxf(m, lds[0][w]);
    float s[1] = {0.f};
    for (int64_t c = threadIdx.x; c < cols; c += kBlock) s[0] += exp_sub(value(c), m);
    block_sum<1>(s, lds[1]);
    const float inv = 1.0f / s[0];
    // y may alias x: every element is read (by value()) only by the thread that overwrites it
    for (int64_t c = threadIdx.x; c < cols; c += kBlock) yr[c] = exp_sub(value(c), m) * inv;
}

__global__ __launch_bounds__(kBlock) void softmax_bwd_generic(const float* dy, const float* y, float* dx,
                                                               int64_t cols) {
    __shared__ float lds[kBlock / kWave];
    const int64_t row = blockIdx.x;
    float s[1] = {0.f};
    for (int64_t c = threadIdx.x; c < cols; c += kBlock) s[0] += dy[row * cols + c] * y[row * cols + c];
    block_sum<1>(s, lds);
    for (int64_t c = threadIdx.x; c < cols; c += kBlock)
        dx[row * cols + c] = y[row * cols + c] * (dy[row * cols + c] - s[0]);
}

template <int MODE>
int launch_softmax_fwd(const float* x, float* y, int64_t rows, int64_t cols, const RowBias& rb, hipStream_t st,
                       Copy16 y16 = Copy16{nullptr, 0}) {
    bool vec = cols % 4 == 0 && cols <= 256 * 16 && aligned16(x) && aligned16(y);
    if (MODE == kTables)
        vec = vec && (!rb.alibi || aligned16(rb.alibi)) && (!rb.xmask || aligned16(rb.xmask));
    if (vec) {
        const int cols4 = (int)(cols / 4);
        const unsigned grid = (unsigned)((rows + kRowsPerBlock - 1) / kRowsPerBlock);
        const int vpl = (cols4 + kWave - 1) / kWave;
        if (vpl <= 1)
            softmax_fwd_wave<1, MODE><<<grid, kBlock, 0, st>>>(x, y, rows, cols4, rb, y16);
        else if (vpl <= 2)
            softmax_fwd_wave<2, MODE><<<grid, kBlock, 0, st>>>(x, y, rows, cols4, rb, y16);
        else if (vpl <= 4)
            softmax_fwd_wave<4, MODE><<<grid, kBlock, 0, st>>>(x, y, rows, cols4, rb, y16);
        else if (vpl <= 8)
            softmax_fwd_wave<8, MODE><<<grid, kBlock, 0, st>>>(x, y, rows, cols4, rb, y16);
        else
            softmax_fwd_wave<16, MODE><<<grid, kBlock, 0, st>>>(x, y, rows, cols4, rb, y16);
    } else {
        if (y16.base) return BR_ERR_TODO;  // the copy is only produced by the one-wave-per-row path
        softmax_fwd_generic<MODE><<<(unsigned)rows, kBlock, 0, st>>>(x, y, cols, rb);
    }
    BR_HIP_LAUNCH_CHECK();
    return BR_OK;
}

bool softmax_bwd_wave_ok(int64_t cols, const void* dy, const void* y, const void* dx) {
    return cols % 4 == 0 && cols <= 256 * 8 && aligned16(dy) && aligned16(y) && aligned16(dx);
}

int launch_softmax_bwd_wave(const float* dy, const float* y, float* dx, Copy16 dx16, int64_t rows, int64_t cols,
                            hipStream_t st) {
    const int cols4 = (int)(cols / 4);
    const unsigned grid = (unsigned)((rows + kRowsPerBlock - 1) / kRowsPerBlock);
    const int vpl = (cols4 + kWave - 1) / kWave;
    if (vpl <= 1)
        softmax_bwd_wave<1><<<grid, kBlock, 0, st>>>(dy, y, dx, rows, cols4, dx16);
    else if (vpl <= 2)
        softmax_bwd_wave<2><<<grid, kBlock, 0, st>>>(dy, y, dx, rows, cols4, dx16);
    else if (vpl <= 4)
        softmax_bwd_wave<4><<<grid, kBlock, 0, st>>>(dy, y, dx, rows, cols4, dx16);
    else
        softmax_bwd_wave<8><<<grid, kBlock, 0, st>>>(dy, y, dx, rows, cols4, dx16);
    BR_HIP_LAUNCH_CHECK();
    return BR_OK;
}

// ------------------------------------------------- vocabulary log-softmax
constexpr int kVBlock = 1024;
constexpr int kVWaves = kVBlock / kWave;

struct MaxSum {
    float m, s;
};

__device__ __forceinline__ MaxSum combine(MaxSum a, MaxSum b) {
    const float m = fmaxf(a.m, b.m);
    MaxSum r;
    r.m = m;
    // a side that has seen nothing carries m = -inf and s = 0
    r.s = (a.m == -INFINITY ? 0.f : a.s * __expf(a.m - m)) + (b.m == -INFINITY ? 0.f : b.s * __expf(b.m - m));
    return r;
}

// Online (max, sum) over one row; every thread returns the row's logsumexp.
__device__ __forceinline__ float row_logsumexp(const float* __restrict__ lr, int64_t vocab, bool vec_ok,
                                               MaxSum* lds) {
    MaxSum t;
    t.m = -INFINITY;
    t.s = 0.f;
    if (vec_ok) {
        const float4* l4 = reinterpret_cast<const float4*>(lr);
        const int64_t n4 = vocab / 4;
        for (int64_t i = threadIdx.x; i < n4; i += kVBlock) {
            const float4 v = load_stream(l4 + i);
            const float m4 = fmaxf(fmaxf(v.x, v.y), fmaxf(v.z, v.w));
            if (m4 > t.m) {
                t.s *= __expf(t.m - m4);  // exp(-inf) = 0 on the first vector
                t.m = m4;
            }
            t.s += (__expf(v.x - t.m) + __expf(v.y - t.m)) + (__expf(v.z - t.m) + __expf(v.w - t.m));
        }
    } else {
        for (int64_t i = threadIdx.x; i < vocab; i += kVBlock) {
            const float v = lr[i];
            if (v > t.m) {
                t.s *= __expf(t.m - v);
                t.m = v;
            }
            t.s += __expf(v - t.m);
        }
    }
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) {
        MaxSum o;
        o.m = __shfl_xor(t.m, off, kWave);
        o.s = __shfl_xor(t.s, off, kWave);
        t = combine(t, o);
    }
    if ((threadIdx.x & 63) == 0) lds[threadIdx.x >> 6] = t;
    __syncthreads();
    MaxSum r = lds[0];
    for (int w = 1; w < kVWaves; w++) r = combine(r, lds[w]);
    return r.m + __logf(r.s);
}

__global__ __launch_bounds__(kVBlock) void nll_fwd_kernel(const float* __restrict__ logits,
                                                           const int32_t* __restrict__ target,
                                                           const int32_t* __restrict__ keep,
                                                           float* __restrict__ lse, float* __restrict__ row_logp,
                                                           int64_t vocab, bool vec_ok) {
    __shared__ MaxSum lds[kVWaves];
    const int64_t row = blockIdx.x;
    const float* lr = logits + row * vocab;
    const float l = row_logsumexp(lr, vocab, vec_ok, lds);
    if (threadIdx.x == 0) {
        lse[row] = l;
        const int32_t t = target[row];
        const bool valid = keep[row] != 0 && t >= 0 && (int64_t)t < vocab;
        row_logp[row] = valid ? lr[t] - l : 0.f;
    }
}

// result[0] = sum(row_logp) / count, result[1] = count; one workgroup,
// fixed summation order.
__global__ __launch_bounds__(kVBlock) void nll_reduce_kernel(const float* __restrict__ row_logp,
                                                              const int32_t* __restrict__ keep,
                                                              float* __restrict__ result, int64_t rows) {
    __shared__ float lds[2 * kVWaves];
    float v[2] = {0.f, 0.f};
    for (int64_t r = threadIdx.x; r < rows; r += kVBlock) {
        v[0] += row_logp[r];
        v[1] += keep[r] != 0 ? 1.f : 0.f;
    }
    block_sum<2>(v, lds);
    if (threadIdx.x == 0) {
        result[0] = v[1] > 0.f ? v[0] / v[1] : 0.f;
        result[1] = v[1];
    }
}

template <typename OUT>
__device__ __forceinline__ void store4(OUT* p, float a, float b, float c, float d);
template <>
__device__ __forceinline__ void store4<float>(float* p, float a, float b, float c, float d) {
    store_stream(reinterpret_cast<float4*>(p), make_float4(a, b, c, d));
}
template <>
__device__ __forceinline__ void store4<__half>(__half* p, float a, float b, float c, float d) {
    half4 h;
    h.v[0] = __floats2half2_rn(a, b);
    h.v[1] = __floats2half2_rn(c, d);
    *reinterpret_cast<half4*>(p) = h;
}
template <typename OUT>
__device__ __forceinline__ OUT cvt_out(float v);
template <>
__device__ __forceinline__ float cvt_out<float>(float v) { return v; }
template <>
__device__ __forceinline__ __half cvt_out<__half>(float v) { return __float2half_rn(v); }
template <>
__device__ __forceinline__ void store4<__hip_bfloat16>(__hip_bfloat16* p, float a, float b, float c, float d) {
    auto bits = [](float v) { return (unsigned)__builtin_bit_cast(unsigned short, __float2bfloat16(v)); };
    *reinterpret_cast<uint2*>(p) = make_uint2(bits(a) | (bits(b) << 16), bits(c) | (bits(d) << 16));
}
template <>
__device__ __forceinline__ __hip_bfloat16 cvt_out<__hip_bfloat16>(float v) { return __float2bfloat16(v); }

template <typename OUT>
__global__ __launch_bounds__(kVBlock) void nll_bwd_kernel(const float* logits, const int32_t* __restrict__ target,
                                                           const int32_t* __restrict__ keep,
                                                           const float* __restrict__ lse, OUT* dlogits, float scale,
                                                           int64_t vocab, bool vec_ok) {
    const int64_t row = blockIdx.x;
    const float* lr = logits + row * vocab;
    OUT* dr = dlogits + row * vocab;
    const int32_t t = target[row];
    const bool on = keep[row] != 0 && t >= 0 && (int64_t)t < vocab;
    if (!on) {
        // rows without a label get an all-zero gradient and are never read
        if (vec_ok) {
            for (int64_t i = threadIdx.x; i < vocab / 4; i += kVBlock) store4<OUT>(dr + i * 4, 0.f, 0.f, 0.f, 0.f);
        } else {
            for (int64_t i = threadIdx.x; i < vocab; i += kVBlock) dr[i] = cvt_out<OUT>(0.f);
        }
        return;
    }
    const float l = lse[row];
    if (vec_ok) {
        const float4* l4 = reinterpret_cast<const float4*>(lr);
        const int64_t t4 = t >> 2;
        for (int64_t i = threadIdx.x; i < vocab / 4; i += kVBlock) {
            const float4 v = load_stream(l4 + i);
            float e[4] = {__expf(v.x - l), __expf(v.y - l), __expf(v.z - l), __expf(v.w - l)};
            if (i == t4) e[t & 3] -= 1.0f;
            store4<OUT>(dr + i * 4, e[0] * scale, e[1] * scale, e[2] * scale, e[3] * scale);
        }
    } else {
        for (int64_t i = threadIdx.x; i < vocab; i += kVBlock) {
            float e = __expf(lr[i] - l);
            if (i == t) e -= 1.0f;
            dr[i] = cvt_out<OUT>(e * scale);
        }
    }
}

// The same gradient with one quad per thread and the workgroups in memory order (blockIdx.x along a row, blockIdx.y
// over the rows): given lse the gradient is element-wise, and a launch that sweeps logits and gradient front to back
// as one stream moves 6.4 TB/s where a workgroup per 1 MB row moves 5.3 (see grid_for).  Same arithmetic, same bits.
#ifndef BR_NLL_BWD_FLAT
#define BR_NLL_BWD_FLAT 1
#endif
constexpr int kFlatBlock = 256;
template <typename OUT>
__global__ __launch_bounds__(kFlatBlock) void nll_bwd_flat_kernel(const float* logits, const int32_t* __restrict__ target,
                                                                  const int32_t* __restrict__ keep,
                                                                  const float* __restrict__ lse, OUT* dlogits,
                                                                  float scale, int64_t vocab) {
    const int64_t row = blockIdx.y;
    const int64_t i = (int64_t)blockIdx.x * kFlatBlock + threadIdx.x;   // quad of the row
    if (i >= vocab / 4) return;
    const int32_t t = target[row];
    const bool on = keep[row] != 0 && t >= 0 && (int64_t)t < vocab;
    OUT* dr = dlogits + row * vocab + i * 4;
    if (!on) {
        store4<OUT>(dr, 0.f, 0.f, 0.f, 0.f);   // rows without a label are not read
        return;
    }
    const float l = lse[row];
    const float4 v = load_stream(reinterpret_cast<const float4*>(logits + row * vocab) + i);
    float e[4] = {__expf(v.x - l), __expf(v.y - l), __expf(v.z - l), __expf(v.w - l)};
    if (i == (t >> 2)) e[t & 3] -= 1.0f;
    store4<OUT>(dr, e[0] * scale, e[1] * scale, e[2] * scale, e[3] * scale);
}

template <typename OUT>
void launch_nll_bwd(const float* logits, const int32_t* target, const int32_t* keep, const float* lse, OUT* dlogits,
                    float scale, int64_t rows, int64_t vocab, bool vec_ok, hipStream_t st) {
    const int64_t blocks_x = (vocab / 4 + kFlatBlock - 1) / kFlatBlock;
    if (BR_NLL_BWD_FLAT && vec_ok && rows <= 65535 && blocks_x <= 0x7fffffff) {
        nll_bwd_flat_kernel<OUT><<<dim3((unsigned)blocks_x, (unsigned)rows), kFlatBlock, 0, st>>>(logits, target, keep, lse,
                                                                                                  dlogits, scale, vocab);
    } else {
        nll_bwd_kernel<OUT><<<(unsigned)rows, kVBlock, 0, st>>>(logits, target, keep, lse, dlogits, scale, vocab, vec_ok);
    }
}

}  // namespace

extern "C" {

int br_hip_softmax_fwd(const float* x, float* y, int64_t rows, int64_t cols, br_stream_t stream) {
    if (rows < 0 || cols <= 0 || rows > 0x7fffffff) return BR_ERR_ATTR;
    if (rows == 0) return BR_OK;
    if (!x) return BR_ERR_INPUT;
    if (!y) return BR_ERR_OUTPUT;
    RowBias rb = {nullptr, nullptr, nullptr, nullptr, 1, 1};
    return launch_softmax_fwd<kPlain>(x, y, rows, cols, rb, as_stream(stream));
}

int br_hip_softmax_bwd(const float* dy, const float* y, float* dx, int64_t rows, int64_t cols,
                       br_stream_t stream) {
    if (rows < 0 || cols <= 0 || rows > 0x7fffffff) return BR_ERR_ATTR;
    if (rows == 0) return BR_OK;
    if (!dy || !y) return BR_ERR_INPUT;
    if (!dx) return BR_ERR_OUTPUT;
    hipStream_t st = as_stream(stream);
    if (softmax_bwd_wave_ok(cols, dy, y, dx)) return launch_softmax_bwd_wave(dy, y, dx, Copy16{nullptr, 0}, rows, cols, st);
    softmax_bwd_generic<<<(unsigned)rows, kBlock, 0, st>>>(dy, y, dx, cols);
    BR_HIP_LAUNCH_CHECK();
    return BR_OK;
}

int br_hip_softmax_bwd_to16(const float* dy, const float* y, void* dx16, int dx16_dtype, int64_t rows, int64_t cols,
                            br_stream_t stream) {
    if (rows < 0 || cols <= 0 || rows > 0x7fffffff) return BR_ERR_ATTR;
    if (rows == 0) return BR_OK;
    if (!dy || !y) return BR_ERR_INPUT;
    if (!dx16 || dx16 == (const void*)dy || dx16 == (const void*)y) return BR_ERR_OUTPUT;
    if (!copy16_ok(dx16, dx16_dtype) || !softmax_bwd_wave_ok(cols, dy, y, dy)) return BR_ERR_TODO;
    return launch_softmax_bwd_wave(dy, y, nullptr, Copy16{dx16, dx16_dtype == BR_BF16}, rows, cols, as_stream(stream));
}

int br_hip_alibi_masked_softmax_fwd(const float* s, const float* alibi, const float* xmask, float* p,
                                    int64_t batch, int64_t heads, int64_t tq, int64_t tk, br_stream_t stream) {
    if (batch < 0 || heads <= 0 || tq <= 0 || tk <= 0 || heads > 0x7fffffff || tq > 0x7fffffff)
        return BR_ERR_ATTR;
    const int64_t rows = batch * heads * tq;
    if (rows > 0x7fffffff) return BR_ERR_ATTR;
    if (rows == 0) return BR_OK;
    if (!s) return BR_ERR_INPUT;
    if (!p) return BR_ERR_OUTPUT;
    RowBias rb = {alibi, xmask, nullptr, nullptr, (int)heads, (int)tq};
    return launch_softmax_fwd<kTables>(s, p, rows, tk, rb, as_stream(stream));
}

int br_hip_alibi_masked_softmax_fwd_copy16(const float* s, const float* alibi, const float* xmask, float* p, void* p16,
                                           int p16_dtype, int64_t batch, int64_t heads, int64_t tq, int64_t tk,
                                           br_stream_t stream) {
    if (batch < 0 || heads <= 0 || tq <= 0 || tk <= 0 || heads > 0x7fffffff || tq > 0x7fffffff)
        return BR_ERR_ATTR;
    const int64_t rows = batch * heads * tq;
    if (rows > 0x7fffffff) return BR_ERR_ATTR;
    if (rows == 0) return BR_OK;
    if (!s) return BR_ERR_INPUT;
    if (!p || !p16) return BR_ERR_OUTPUT;
    if (!copy16_ok(p16, p16_dtype)) return BR_ERR_TODO;
    RowBias rb = {alibi, xmask, nullptr, nullptr, (int)heads, (int)tq};
    return launch_softmax_fwd<kTables>(s, p, rows, tk, rb, as_stream(stream), Copy16{p16, p16_dtype == BR_BF16});
}

int br_hip_alibi_causal_softmax_fwd(const float* s, const double* slopes, const int32_t* valid, float* p,
                                    int64_t batch, int64_t heads, int64_t tq, int64_t tk, br_stream_t stream) {
    if (batch < 0 || heads <= 0 || tq <= 0 || tk <= 0 || heads > 0x7fffffff || tq > 0x7fffffff)
        return BR_ERR_ATTR;
    const int64_t rows = batch * heads * tq;
    if (rows > 0x7fffffff) return BR_ERR_ATTR;
    if (rows == 0) return BR_OK;
    if (!s || !slopes || !valid) return BR_ERR_INPUT;
    if (!p) return BR_ERR_OUTPUT;
    RowBias rb = {nullptr, nullptr, slopes, valid, (int)heads, (int)tq};
    return launch_softmax_fwd<kAnalytic>(s, p, rows, tk, rb, as_stream(stream));
}

int br_hip_logsoftmax_nll_fwd(const float* logits, const int32_t* target, const int32_t* keep, float* lse,
                              float* row_logp, float* result, int64_t rows, int64_t vocab, br_stream_t stream) {
    if (rows < 0 || vocab <= 0 || rows > 0x7fffffff) return BR_ERR_ATTR;
    if (!result) return BR_ERR_OUTPUT;
    hipStream_t st = as_stream(stream);
    if (rows > 0) {
        if (!logits || !target || !keep) return BR_ERR_INPUT;
        if (!lse || !row_logp) return BR_ERR_OUTPUT;
        const bool vec_ok = vocab % 4 == 0 && aligned16(logits);
        nll_fwd_kernel<<<(unsigned)rows, kVBlock, 0, st>>>(logits, target, keep, lse, row_logp, vocab, vec_ok);
        BR_HIP_LAUNCH_CHECK();
    }
    nll_reduce_kernel<<<1, kVBlock, 0, st>>>(row_logp, keep, result, rows);
    BR_HIP_LAUNCH_CHECK();
    return BR_OK;
}

int br_hip_logsoftmax_nll_bwd(const float* logits, const int32_t* target, const int32_t* keep, const float* lse,
                              void* dlogits, int dlogits_dtype, float scale, int64_t rows, int64_t vocab,
                              br_stream_t stream) {
    if (rows < 0 || vocab <= 0 || rows > 0x7fffffff) return BR_ERR_ATTR;
    if (rows == 0) return BR_OK;
    if (!logits || !target || !keep || !lse) return BR_ERR_INPUT;
    if (!dlogits) return BR_ERR_OUTPUT;
    hipStream_t st = as_stream(stream);
    if (dlogits_dtype == BR_F32) {
        const bool vec_ok = vocab % 4 == 0 && aligned16(logits) && aligned16(dlogits);
        launch_nll_bwd<float>(logits, target, keep, lse, (float*)dlogits, scale, rows, vocab, vec_ok, st);
    } else if (dlogits_dtype == BR_F16) {
        if ((const void*)logits == dlogits) return BR_ERR_OUTPUT;
        const bool vec_ok = vocab % 4 == 0 && aligned16(logits) && aligned8(dlogits);
        launch_nll_bwd<__half>(logits, target, keep, lse, (__half*)dlogits, scale, rows, vocab, vec_ok, st);
    } else if (dlogits_dtype == BR_BF16) {
        if ((const void*)logits == dlogits) return BR_ERR_OUTPUT;
        const bool vec_ok = vocab % 4 == 0 && aligned16(logits) && aligned8(dlogits);
        launch_nll_bwd<__hip_bfloat16>(logits, target, keep, lse, (__hip_bfloat16*)dlogits, scale, rows, vocab, vec_ok, st);
    } else {
        return BR_ERR_TODO;
    }
    BR_HIP_LAUNCH_CHECK();
    return BR_OK;
}

}  // extern "C"
