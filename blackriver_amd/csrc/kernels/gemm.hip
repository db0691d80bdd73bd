// Strided-batched GEMM entry point of the C ABI.
//
//   C[b][i,j] = alpha * sum_p opA[b][i,p] * opB[b][p,j] (+ C) (+ bias[j])
//
// 16-bit multiplicands (fp16 / bf16, fp32 accumulation) go to the kernel
// templates in gemm_dtl16.hpp (both operands stored in the MFMA type, aligned:
// direct-to-LDS loads) and gemm_mfma16.hpp (everything else: fp32 operands
// converted on load, ragged sizes).  This file holds the argument checking,
// the staging of fp32 operands into a caller's workspace so that they too can
// take the direct-to-LDS kernel, and the kernel that keeps fp32 operands and
// multiplies with v_mfma_f32_32x32x2_f32 for callers that need fp32-faithful
// products (128x128x16 tiles, 4 wave64s x 2x2 MFMA blocks, register prefetch +
// LDS double buffering).
#include "common.hpp"

#include <hip/hip_bf16.h>

#include <stdlib.h>
#include <string.h>

#include "gemm_dtl16.hpp"

using namespace brk;

namespace brk {
int gemm16_launch_f16(const gemm16::GemmArgs& g, const gemm16::Problem& p, long long batch, hipStream_t st);
int gemm16_launch_bf16(const gemm16::GemmArgs& g, const gemm16::Problem& p, long long batch, hipStream_t st);
}  // namespace brk

namespace {

typedef float f32x16 __attribute__((ext_vector_type(16)));
using gemm16::GemmArgs;

constexpr int BM = 128, BN = 128;
constexpr int kThreads = 256;

// m varies fastest so that neighbouring workgroups share one panel of B
__device__ __forceinline__ void tile_coords32(const GemmArgs& g, long long& batch, int& tm, int& tn) {
    const long long per_batch = (long long)g.tiles_m * g.tiles_n;
    const long long id = blockIdx.x;
    batch = id / per_batch;
    const int rem = (int)(id % per_batch);
    tm = rem % g.tiles_m;
    tn = rem / g.tiles_m;
}

// ---- fp32 operands on v_mfma_f32_32x32x2_f32 ------------------------------
// Same tiling with BK = 16 fp32 values per step; LDS rows padded to 20 floats.
constexpr int BK32 = 16;
constexpr int kPitch32 = BK32 + 4;

template <bool KSTR>
struct TileLoader32 {
    float4 r[2];
    __device__ __forceinline__ void fetch(const float* base, long long ld, long long row0, long long rows,
                                          long long k0, long long kdim, bool vec) {
        const int t = threadIdx.x;
        if (!KSTR) {
            const int c = t & 3, r0 = t >> 2;  // 4 k-values per chunk, 64 rows per pass
#pragma unroll
            for (int p = 0; p < 2; p++) {
                const long long row = row0 + r0 + 64 * p;
                const long long off = row * ld + k0 + c * 4;
                if (vec && row < rows && k0 + c * 4 + 4 <= kdim) {
                    r[p] = *reinterpret_cast<const float4*>(base + off);
                } else {
                    float w[4];
#pragma unroll
                    for (int e = 0; e < 4; e++) w[e] = (row < rows && k0 + c * 4 + e < kdim) ? base[off + e] : 0.f;
                    r[p] = make_float4(w[0], w[1], w[2], w[3]);
                }
            }
        } else {
            const int r4 = t & 31, kg = t >> 5;  // 4 rows x 2 k-values per thread
            const long long row = row0 + 4 * r4;
#pragma unroll
            for (int kk = 0; kk < 2; kk++) {
                const long long kidx = k0 + 2 * kg + kk;
                const long long off = kidx * ld + row;
                if (vec && row + 4 <= rows && kidx < kdim) {
                    r[kk] = *reinterpret_cast<const float4*>(base + off);
                } else {
                    float w[4];
#pragma unroll
                    for (int e = 0; e < 4; e++) w[e] = (row + e < rows && kidx < kdim) ? base[off + e] : 0.f;
                    r[kk] = make_float4(w[0], w[1], w[2], w[3]);
                }
            }
        }
    }
    __device__ __forceinline__ void commit(float* tile) const {
        const int t = threadIdx.x;
        if (!KSTR) {
            const int c = t & 3, r0 = t >> 2;
#pragma unroll
            for (int p = 0; p < 2; p++) *reinterpret_cast<float4*>(tile + (r0 + 64 * p) * kPitch32 + c * 4) = r[p];
        } else {
            const int r4 = t & 31, kg = t >> 5;
            const float a[4] = {r[0].x, r[0].y, r[0].z, r[0].w};
            const float b[4] = {r[1].x, r[1].y, r[1].z, r[1].w};
#pragma unroll
            for (int e = 0; e < 4; e++)
                *reinterpret_cast<float2*>(tile + (4 * r4 + e) * kPitch32 + 2 * kg) = make_float2(a[e], b[e]);
        }
    }
};

template <bool A_KSTR, bool B_KSTR>
__global__ __launch_bounds__(kThreads) void gemm_mfma32_kernel(GemmArgs g) {
    __shared__ __attribute__((aligned(16))) float lds_a[2][BM * kPitch32];
    __shared__ __attribute__((aligned(16))) float lds_b[2][BN * kPitch32];
    long long batch;
    int tm, tn;
    tile_coords32(g, batch, tm, tn);
    const long long row0 = (long long)tm * BM, col0 = (long long)tn * BN;
    const float* a_base = static_cast<const float*>(g.a) + batch * g.sa;
    const float* b_base = static_cast<const float*>(g.b) + batch * g.sb;
    TileLoader32<A_KSTR> la;
    TileLoader32<B_KSTR> lb;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int wm = wave >> 1, wn = wave & 1;
    const int lrow = lane & 31, lk = (lane >> 5) * 4;

    f32x16 acc[2][2];
#pragma unroll
    for (int i = 0; i < 2; i++)
#pragma unroll
        for (int j = 0; j < 2; j++)
#pragma unroll
            for (int v = 0; v < 16; v++) acc[i][j][v] = 0.f;

    const long long nk = (g.k + BK32 - 1) / BK32;
    la.fetch(a_base, g.lda, row0, g.m, 0, g.k, g.vec_a);
    lb.fetch(b_base, g.ldb, col0, g.n, 0, g.k, g.vec_b);
    la.commit(lds_a[0]);
    lb.commit(lds_b[0]);
    __syncthreads();
    for (long long kt = 0; kt < nk; kt++) {
        const int cur = (int)(kt & 1);
        if (kt + 1 < nk) {
            la.fetch(a_base, g.lda, row0, g.m, (kt + 1) * BK32, g.k, g.vec_a);
            lb.fetch(b_base, g.ldb, col0, g.n, (kt + 1) * BK32, g.k, g.vec_b);
        }
        const float* ta = lds_a[cur] + (wm * 64 + lrow) * kPitch32 + lk;
        const float* tb = lds_b[cur] + (wn * 64 + lrow) * kPitch32 + lk;
#pragma unroll
        for (int ks = 0; ks < BK32 / 8; ks++) {
            // a lane holds k = ks*8 + (lane/32)*4 + s for s = 0..3; MFMA number s
            // multiplies slot s of both halves of the wave, i.e. two distinct k
            float4 fa[2], fb[2];
#pragma unroll
            for (int i = 0; i < 2; i++) {
                fa[i] = *reinterpret_cast<const float4*>(ta + i * 32 * kPitch32 + ks * 8);
                fb[i] = *reinterpret_cast<const float4*>(tb + i * 32 * kPitch32 + ks * 8);
            }
#pragma unroll
            for (int i = 0; i < 2; i++)
#pragma unroll
                for (int j = 0; j < 2; j++) {
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(fa[i].x, fb[j].x, acc[i][j], 0, 0, 0);
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(fa[i].y, fb[j].y, acc[i][j], 0, 0, 0);
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(fa[i].z, fb[j].z, acc[i][j], 0, 0, 0);
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(fa[i].w, fb[j].w, acc[i][j], 0, 0, 0);
                }
        }
        if (kt + 1 < nk) {
            la.commit(lds_a[cur ^ 1]);
            lb.commit(lds_b[cur ^ 1]);
        }
        __syncthreads();
    }
    float* c_base = static_cast<float*>(g.c) + batch * g.sc;
    const float* old_base = g.addend ? static_cast<const float*>(g.addend) + batch * g.sc : c_base;
#pragma unroll
    for (int j = 0; j < 2; j++) {
        const long long col = col0 + wn * 64 + j * 32 + lrow;
        if (col >= g.n) continue;
        const float bias = g.bias ? g.bias[col] : 0.f;
#pragma unroll
        for (int i = 0; i < 2; i++) {
#pragma unroll
            for (int v = 0; v < 16; v++) {
                const long long row = row0 + wm * 64 + i * 32 + (v >> 2) * 8 + (lane >> 5) * 4 + (v & 3);
                if (row < g.m) {
                    float* p = c_base + row * g.ldc + col;
                    float o = g.alpha * acc[i][j][v] + bias;
                    if (g.accumulate) o += old_base[row * g.ldc + col];
                    *p = o;
                }
            }
        }
    }
}

long long elem_size(int dtype) { return dtype == BR_F32 ? 4 : 2; }

// br_hip_gemm with the tensor an accumulating product adds to named separately (null = c itself).
int gemm_impl(int trans_a, int trans_b, int64_t m, int64_t n, int64_t k, float alpha, const void* a, int a_dtype,
              int64_t lda, int64_t stride_a, const void* b, int b_dtype, int64_t ldb, int64_t stride_b, int accumulate,
              const void* addend, void* c, int c_dtype, int64_t ldc, int64_t stride_c, const float* bias, int64_t batch,
              int compute, br_stream_t stream, float* partials = nullptr, size_t partial_bytes = 0) {
    if (m < 0 || n < 0 || k < 0 || batch < 0) return BR_ERR_ATTR;
    if (m == 0 || n == 0 || batch == 0) return BR_OK;
    if (!a || !b) return BR_ERR_INPUT;
    if (!c) return BR_ERR_OUTPUT;
    // minimal leading dimensions for the stated layouts
    if (lda < (trans_a ? m : k) || ldb < (trans_b ? k : n) || ldc < n) return BR_ERR_ATTR;
    const int native = compute == BR_GEMM_F16 ? BR_F16 : compute == BR_GEMM_BF16 ? BR_BF16 : BR_F32;
    if (compute != BR_GEMM_F16 && compute != BR_GEMM_BF16 && compute != BR_GEMM_F32) return BR_ERR_ATTR;
    if (a_dtype != BR_F32 && a_dtype != native) return BR_ERR_TODO;
    if (b_dtype != BR_F32 && b_dtype != native) return BR_ERR_TODO;
    if (c_dtype != BR_F32 && c_dtype != native) return BR_ERR_TODO;

    GemmArgs g;
    g.a = a; g.b = b; g.c = c; g.bias = bias;
    g.m = m; g.n = n; g.k = k;
    g.lda = lda; g.ldb = ldb; g.ldc = ldc;
    g.sa = stride_a; g.sb = stride_b; g.sc = stride_c;
    g.alpha = alpha;
    g.accumulate = accumulate ? 1 : 0;
    g.addend = accumulate ? addend : nullptr;
    g.partials = partials;   // room for the partial tiles of a K split (the direct-to-LDS kernel decides)
    g.partial_bytes = partials ? partial_bytes : 0;
    g.tiles_m = (int)((m + BM - 1) / BM);
    g.tiles_n = (int)((n + BN - 1) / BN);
    const long long blocks = (long long)g.tiles_m * g.tiles_n * batch;
    if (blocks > 0x7fffffffLL) return BR_ERR_ATTR;
    // 128-bit loads need 16-byte aligned bases, leading dimensions and batch strides
    auto vec_ok = [&](const void* p, int dtype, long long ld, long long stride) {
        const long long es = elem_size(dtype);
        return aligned16(p) && (ld * es) % 16 == 0 && (batch == 1 || (stride * es) % 16 == 0);
    };
    g.vec_a = vec_ok(a, a_dtype, lda, stride_a) ? 1 : 0;
    g.vec_b = vec_ok(b, b_dtype, ldb, stride_b) ? 1 : 0;
    hipStream_t st = as_stream(stream);
    // opA is k-strided in memory when A is stored [k,m]; opB when B is stored [k,n]
    const bool ak = trans_a != 0, bk = trans_b == 0;
    if (compute == BR_GEMM_F32) {
        if (ak && bk) gemm_mfma32_kernel<true, true><<<(unsigned)blocks, kThreads, 0, st>>>(g);
        else if (ak) gemm_mfma32_kernel<true, false><<<(unsigned)blocks, kThreads, 0, st>>>(g);
        else if (bk) gemm_mfma32_kernel<false, true><<<(unsigned)blocks, kThreads, 0, st>>>(g);
        else gemm_mfma32_kernel<false, false><<<(unsigned)blocks, kThreads, 0, st>>>(g);
        BR_HIP_LAUNCH_CHECK();
        return BR_OK;
    }
    gemm16::Problem p;
    p.a_f32 = a_dtype == BR_F32;
    p.b_f32 = b_dtype == BR_F32;
    p.a_kstr = ak;
    p.b_kstr = bk;
    p.c_dtype = c_dtype;
    // the fast kernel loads 128 bits at a time and never checks k
    const long long va = p.a_f32 ? 4 : 8, vb = p.b_f32 ? 4 : 8;
    p.guarded = !g.vec_a || !g.vec_b || k % 32 != 0 || (ak && m % va != 0) || (bk && n % vb != 0);
    if (compute == BR_GEMM_F16) return gemm16_launch_f16(g, p, batch, st);
    return gemm16_launch_bf16(g, p, batch, st);
}

}  // namespace

extern "C" int br_hip_gemm(int trans_a, int trans_b, int64_t m, int64_t n, int64_t k, float alpha, const void* a,
                           int a_dtype, int64_t lda, int64_t stride_a, const void* b, int b_dtype, int64_t ldb,
                           int64_t stride_b, int accumulate, void* c, int c_dtype, int64_t ldc, int64_t stride_c,
                           const float* bias, int64_t batch, int compute, br_stream_t stream) {
    return gemm_impl(trans_a, trans_b, m, n, k, alpha, a, a_dtype, lda, stride_a, b, b_dtype, ldb, stride_b, accumulate,
                     nullptr, c, c_dtype, ldc, stride_c, bias, batch, compute, stream);
}

extern "C" int br_hip_linear_gelu(const void* x, const void* w, const float* bias, void* u, void* y, int dtype,
                                  int64_t rows, int64_t out, int64_t in, br_stream_t stream) {
    if (rows < 0 || out <= 0 || in <= 0) return BR_ERR_ATTR;
    if (dtype != BR_F16 && dtype != BR_BF16) return BR_ERR_TODO;
    if (rows == 0) return BR_OK;
    if (!x || !w) return BR_ERR_INPUT;
    if (!u || !y || u == y) return BR_ERR_OUTPUT;
    // the GELU epilogue exists in the direct-to-LDS kernel only
    if (in % 32 != 0 || out % 8 != 0 || !aligned16(x) || !aligned16(w) || !aligned16(u) || !aligned16(y))
        return BR_ERR_TODO;
    GemmArgs g;
    g.a = x; g.b = w; g.c = u; g.c2 = y; g.bias = bias;
    g.m = rows; g.n = out; g.k = in;
    g.lda = in; g.ldb = in; g.ldc = out;
    g.sa = g.sb = g.sc = 0;
    g.alpha = 1.0f;
    g.accumulate = 0;
    g.tiles_m = g.tiles_n = 0;  // set by the launcher for the tile it picks
    g.vec_a = g.vec_b = 1;
    gemm16::Problem p;
    p.a_f32 = p.b_f32 = false;
    p.a_kstr = p.b_kstr = false;
    p.c_dtype = dtype;
    p.guarded = false;
    hipStream_t st = as_stream(stream);
    if (dtype == BR_F16) return gemm16_launch_f16(g, p, 1, st);
    return gemm16_launch_bf16(g, p, 1, st);
}

// ---- fp32 operands staged as 16-bit copies ----------------------------------
namespace {

// dst[b][r][c] (dense) = convert(src[b*stride + r*ld + c]); cols % 4 == 0 and
// 16-byte aligned rows take the vector path.
template <typename DST, bool VEC>
__global__ __launch_bounds__(256) void stage_rows_kernel(const float* __restrict__ src, long long ld,
                                                         long long stride, long long rows, long long cols,
                                                         long long batch, DST* __restrict__ dst) {
    const long long per_row = VEC ? cols / 4 : cols;
    const long long total = batch * rows * per_row;
    for (long long i = blockIdx.x * (long long)blockDim.x + threadIdx.x; i < total;
         i += (long long)gridDim.x * blockDim.x) {
        const long long c = i % per_row, r = (i / per_row) % rows, b = i / (per_row * rows);
        const float* s = src + b * stride + r * ld;
        DST* d = dst + (b * rows + r) * cols;
        if (VEC) {
            const float4 v = reinterpret_cast<const float4*>(s)[c];
            gemm16::u32x2 o;
            if (sizeof(DST) == 2 && __is_same(DST, __half)) {
                o.x = gemm16::pack2(gemm16::Cvt<BR_GEMM_F16>::from_f32(v.x), gemm16::Cvt<BR_GEMM_F16>::from_f32(v.y));
                o.y = gemm16::pack2(gemm16::Cvt<BR_GEMM_F16>::from_f32(v.z), gemm16::Cvt<BR_GEMM_F16>::from_f32(v.w));
            } else {
                o.x = gemm16::pack2(gemm16::Cvt<BR_GEMM_BF16>::from_f32(v.x), gemm16::Cvt<BR_GEMM_BF16>::from_f32(v.y));
                o.y = gemm16::pack2(gemm16::Cvt<BR_GEMM_BF16>::from_f32(v.z), gemm16::Cvt<BR_GEMM_BF16>::from_f32(v.w));
            }
            reinterpret_cast<gemm16::u32x2*>(d)[c] = o;
        } else {
            const unsigned short h = __is_same(DST, __half) ? gemm16::Cvt<BR_GEMM_F16>::from_f32(s[c])
                                                            : gemm16::Cvt<BR_GEMM_BF16>::from_f32(s[c]);
            reinterpret_cast<unsigned short*>(d)[c] = h;
        }
    }
}

// Dense operand (rows follow each other without gaps): a flat conversion, 8
// elements per thread, no index arithmetic.
template <bool BF>
__global__ __launch_bounds__(256) void stage_flat_kernel(const float4* __restrict__ src, gemm16::u32x4* __restrict__ dst,
                                                         long long n8) {
    for (long long i = blockIdx.x * (long long)blockDim.x + threadIdx.x; i < n8;
         i += (long long)gridDim.x * blockDim.x) {
        const float4 a = src[2 * i], b = src[2 * i + 1];
        constexpr int CT = BF ? BR_GEMM_BF16 : BR_GEMM_F16;
        gemm16::u32x4 o;
        o.x = gemm16::pack2(gemm16::Cvt<CT>::from_f32(a.x), gemm16::Cvt<CT>::from_f32(a.y));
        o.y = gemm16::pack2(gemm16::Cvt<CT>::from_f32(a.z), gemm16::Cvt<CT>::from_f32(a.w));
        o.z = gemm16::pack2(gemm16::Cvt<CT>::from_f32(b.x), gemm16::Cvt<CT>::from_f32(b.y));
        o.w = gemm16::pack2(gemm16::Cvt<CT>::from_f32(b.z), gemm16::Cvt<CT>::from_f32(b.w));
        dst[i] = o;
    }
}

int stage_rows(const float* src, long long ld, long long stride, long long rows, long long cols, long long batch,
               void* dst, int compute, hipStream_t st) {
    const long long total = batch * rows * cols;
    if (ld == cols && (batch == 1 || stride == rows * cols) && total % 8 == 0 && aligned16(src) && aligned16(dst)) {
        const unsigned grid = grid_for(total / 8, 256);
        if (compute == BR_GEMM_F16)
            stage_flat_kernel<false><<<grid, 256, 0, st>>>(reinterpret_cast<const float4*>(src),
                                                           static_cast<gemm16::u32x4*>(dst), total / 8);
        else
            stage_flat_kernel<true><<<grid, 256, 0, st>>>(reinterpret_cast<const float4*>(src),
                                                          static_cast<gemm16::u32x4*>(dst), total / 8);
        BR_HIP_LAUNCH_CHECK();
        return BR_OK;
    }
    const bool vec = cols % 4 == 0 && ld % 4 == 0 && stride % 4 == 0 && aligned16(src) && aligned16(dst);
    const long long work = batch * rows * (vec ? cols / 4 : cols);
    const unsigned grid = grid_for(work, 256);
    if (compute == BR_GEMM_F16) {
        if (vec) stage_rows_kernel<__half, true><<<grid, 256, 0, st>>>(src, ld, stride, rows, cols, batch, (__half*)dst);
        else stage_rows_kernel<__half, false><<<grid, 256, 0, st>>>(src, ld, stride, rows, cols, batch, (__half*)dst);
    } else {
        if (vec) stage_rows_kernel<__hip_bfloat16, true><<<grid, 256, 0, st>>>(src, ld, stride, rows, cols, batch, (__hip_bfloat16*)dst);
        else stage_rows_kernel<__hip_bfloat16, false><<<grid, 256, 0, st>>>(src, ld, stride, rows, cols, batch, (__hip_bfloat16*)dst);
    }
    BR_HIP_LAUNCH_CHECK();
    return BR_OK;
}

// ---- split-K ------------------------------------------------------------------
// A product with few output tiles and a long K leaves most CUs idle.  Two forms,
// both deterministic and free of floating-point atomics:
//  * many slices (products with M = 512 or fewer rows: 4-16 slices): run as a
//    strided-batched product over `splits` slices of K into fp32 partials (slice
//    s of A / B is the operand advanced by s * k/splits along k, which the batch
//    strides express), followed by a fixed-order sum in a second kernel;
//  * two slices (M = 2048, N = 4096, K >= 12288: 128 tiles of 256 x 256 on 256
//    CUs): inside the direct-to-LDS kernel, the slice that finishes last adds the
//    other's partial tile and runs the epilogue (gemm_dtl16.hpp).  Measured on
//    the same box, the in-kernel form loses to the two-kernel form when four or
//    more slices exchange partial tiles (its device-coherent accesses move
//    1.5-3 TB/s, ordinary stores 6-7) and wins with two, where only one of the
//    two slices writes anything.
// Which form, how many slices and which tile depend on the problem's sizes only,
// so a product's bits do not depend on where its operands or its workspace
// happen to live.
__global__ __launch_bounds__(256) void splitk_reduce_kernel(const float4* __restrict__ part, int splits,
                                                            long long mn4, long long n4, float alpha,
                                                            const float* __restrict__ bias, const void* old,
                                                            void* c, int c_dtype, long long ldc) {
    for (long long i = blockIdx.x * (long long)blockDim.x + threadIdx.x; i < mn4;
         i += (long long)gridDim.x * blockDim.x) {
        float4 s = part[i];
        for (int p = 1; p < splits; p++) {
            const float4 v = part[(long long)p * mn4 + i];
            s.x += v.x; s.y += v.y; s.z += v.z; s.w += v.w;
        }
        const long long row = i / n4, col = (i % n4) * 4;
        float o[4] = {alpha * s.x, alpha * s.y, alpha * s.z, alpha * s.w};
        if (bias) {
#pragma unroll
            for (int j = 0; j < 4; j++) o[j] += bias[col + j];
        }
        if (c_dtype == BR_F32) {
            // `old`: the tensor an accumulating product adds to (c itself or a tensor laid out like it), else null
            float* dst = static_cast<float*>(c) + row * ldc + col;
            const float* was = static_cast<const float*>(old) + row * ldc + col;
#pragma unroll
            for (int j = 0; j < 4; j++) dst[j] = old ? o[j] + was[j] : o[j];
        } else if (c_dtype == BR_F16) {
            __half* dst = static_cast<__half*>(c) + row * ldc + col;
            const __half* was = static_cast<const __half*>(old) + row * ldc + col;
#pragma unroll
            for (int j = 0; j < 4; j++) dst[j] = __float2half_rn(old ? o[j] + __half2float(was[j]) : o[j]);
        } else {
            __hip_bfloat16* dst = static_cast<__hip_bfloat16*>(c) + row * ldc + col;
            const __hip_bfloat16* was = static_cast<const __hip_bfloat16*>(old) + row * ldc + col;
#pragma unroll
            for (int j = 0; j < 4; j++) dst[j] = __float2bfloat16(old ? o[j] + __bfloat162float(was[j]) : o[j]);
        }
    }
}

// Number of K slices (1 = do not split) for an unbatched product on the
// direct-to-LDS kernel: the split whose estimated time, including the pass
// over the partials, is smallest.
int splitk_choice(int64_t m, int64_t n, int64_t k) {
    if (n % 4 != 0) return 1;
    double best = gemm16::dtl_tile_plan(m, n, k, 1).seconds;
    int pick = 1;
    for (int s = 2; s <= 16; s *= 2) {
        if (k % (64 * s) != 0 || k / s < 512) break;
        const double t = gemm16::dtl_tile_plan(m, n, k / s, s).seconds + 6e-6 + (double)(s + 1) * m * n * 4.0 / 4e12;
        if (t < 0.85 * best) {
            best = t;
            pick = s;
        }
    }
    return pick;
}


// Bytes of partial tiles the two-slice in-kernel form wants (0 = it does not apply or does not pay).
size_t pair_split_room(int64_t m, int64_t n, int64_t k, int64_t batch) {
    if (batch != 1 || splitk_choice(m, n, k) > 1) return 0;
    return gemm16::dtl_pair_split_bytes(m, n, k);
}

size_t staged_bytes(int64_t rows, int64_t cols, int64_t batch) {
    const size_t b = (size_t)rows * (size_t)cols * (size_t)batch * 2;
    return (b + 255) & ~(size_t)255;
}

}  // namespace

extern "C" size_t br_hip_gemm_staged_workspace(int trans_a, int trans_b, int64_t m, int64_t n, int64_t k, int a_dtype,
                                               int b_dtype, int64_t batch) {
    (void)trans_a;
    (void)trans_b;
    if (m <= 0 || n <= 0 || k <= 0 || batch <= 0) return 0;
    size_t need = 0;
    if (a_dtype == BR_F32) need += staged_bytes(m, k, batch);
    if (b_dtype == BR_F32) need += staged_bytes(k, n, batch);
    if (batch == 1) {
        const int splits = splitk_choice(m, n, k);
        if (splits > 1) need += (size_t)splits * (size_t)m * (size_t)n * sizeof(float);
    }
    need += pair_split_room(m, n, k, batch);
    return need;
}

namespace {
// br_hip_gemm_staged with the tensor an accumulating product adds to named separately (null = c itself).
int staged_impl(int trans_a, int trans_b, int64_t m, int64_t n, int64_t k, float alpha, const void* a, int a_dtype,
                int64_t lda, int64_t stride_a, const void* b, int b_dtype, int64_t ldb, int64_t stride_b, int accumulate,
                const void* addend, void* c, int c_dtype, int64_t ldc, int64_t stride_c, const float* bias,
                int64_t batch, int compute, void* workspace, size_t workspace_bytes, br_stream_t stream) {
    const bool f32_a = a_dtype == BR_F32, f32_b = b_dtype == BR_F32;
    const bool sixteen = compute == BR_GEMM_F16 || compute == BR_GEMM_BF16;
    // Stage (and consider splitting K) only when the converted problem meets the
    // direct-to-LDS kernel's rules; every other case is the plain entry point's
    // business.
    const int64_t a_rows = trans_a ? k : m, a_cols = trans_a ? m : k;
    const int64_t b_rows = trans_b ? n : k, b_cols = trans_b ? k : n;
    bool stage = sixteen && workspace && aligned16(workspace) && m > 0 && n > 0 && k > 0 && batch > 0 && a && b &&
                 k % 32 == 0;
    if (stage) {
        // dense 16-bit copies: leading dimension = cols, batch stride = rows*cols
        if (f32_a && a_cols % 8 != 0) stage = false;
        if (f32_b && b_cols % 8 != 0) stage = false;
        if (lda < a_cols || ldb < b_cols) stage = false;
        if (br_hip_gemm_staged_workspace(trans_a, trans_b, m, n, k, a_dtype, b_dtype, batch) > workspace_bytes)
            stage = false;
    }
    if (!stage)
        return gemm_impl(trans_a, trans_b, m, n, k, alpha, a, a_dtype, lda, stride_a, b, b_dtype, ldb, stride_b,
                         accumulate, addend, c, c_dtype, ldc, stride_c, bias, batch, compute, stream);
    const int native = compute == BR_GEMM_F16 ? BR_F16 : BR_BF16;
    hipStream_t st = as_stream(stream);
    char* ws = static_cast<char*>(workspace);
    if (f32_a) {
        const int rc = stage_rows(static_cast<const float*>(a), lda, stride_a, a_rows, a_cols, batch, ws, compute, st);
        if (rc != BR_OK) return rc;
        a = ws;
        a_dtype = native;
        lda = a_cols;
        stride_a = a_rows * a_cols;
        ws += staged_bytes(m, k, batch);
    }
    if (f32_b) {
        const int rc = stage_rows(static_cast<const float*>(b), ldb, stride_b, b_rows, b_cols, batch, ws, compute, st);
        if (rc != BR_OK) return rc;
        b = ws;
        b_dtype = native;
        ldb = b_cols;
        stride_b = b_rows * b_cols;
        ws += staged_bytes(k, n, batch);
    }
    const int splits = batch == 1 ? splitk_choice(m, n, k) : 1;
    if (splits > 1 && c) {
        // slices of K as batch entries: a k-contiguous operand advances by k/splits
        // elements per slice, a row-contiguous one by k/splits rows
        const int64_t ks = k / splits;
        float* part = reinterpret_cast<float*>(ws);
        const int rc = br_hip_gemm(trans_a, trans_b, m, n, ks, 1.0f, a, a_dtype, lda, trans_a ? ks * lda : ks, b,
                                   b_dtype, ldb, trans_b ? ks : ks * ldb, 0, part, BR_F32, n, m * n, nullptr, splits,
                                   compute, stream);
        if (rc != BR_OK) return rc;
        const long long mn4 = m * n / 4;
        splitk_reduce_kernel<<<grid_for(mn4, 256), 256, 0, st>>>(reinterpret_cast<const float4*>(part),
                                                                        splits, mn4, n / 4, alpha, bias,
                                                                        accumulate ? (addend ? addend : c) : nullptr,
                                                                        c, c_dtype, ldc);
        BR_HIP_LAUNCH_CHECK();
        return BR_OK;
    }
    // two slices inside the kernel: what is left of the workspace holds one partial tile per output tile; the
    // product is split only if the room the workspace function asked for is really there
    const size_t room = pair_split_room(m, n, k, batch);
    const size_t left = workspace_bytes - (size_t)(ws - static_cast<char*>(workspace));
    float* partials = room > 0 && room <= left ? reinterpret_cast<float*>(ws) : nullptr;
    return gemm_impl(trans_a, trans_b, m, n, k, alpha, a, a_dtype, lda, stride_a, b, b_dtype, ldb, stride_b, accumulate,
                     addend, c, c_dtype, ldc, stride_c, bias, batch, compute, stream, partials, room);
}
}  // namespace

extern "C" int br_hip_gemm_staged(int trans_a, int trans_b, int64_t m, int64_t n, int64_t k, float alpha, const void* a,
                                  int a_dtype, int64_t lda, int64_t stride_a, const void* b, int b_dtype, int64_t ldb,
                                  int64_t stride_b, int accumulate, void* c, int c_dtype, int64_t ldc,
                                  int64_t stride_c, const float* bias, int64_t batch, int compute, void* workspace,
                                  size_t workspace_bytes, br_stream_t stream) {
    return staged_impl(trans_a, trans_b, m, n, k, alpha, a, a_dtype, lda, stride_a, b, b_dtype, ldb, stride_b,
                       accumulate, nullptr, c, c_dtype, ldc, stride_c, bias, batch, compute, workspace, workspace_bytes,
                       stream);
}

extern "C" int br_hip_linear_residual(const void* x, int x_dtype, const void* w, int w_dtype, const float* bias,
                                      const void* r, void* y, int y_dtype, int64_t rows, int64_t out, int64_t in,
                                      int compute, void* workspace, size_t workspace_bytes, br_stream_t stream) {
    if (rows < 0 || out <= 0 || in <= 0) return BR_ERR_ATTR;
    if (rows == 0) return BR_OK;
    if (!x || !w || !r) return BR_ERR_INPUT;
    if (!y) return BR_ERR_OUTPUT;
    return staged_impl(0, 1, rows, out, in, 1.0f, x, x_dtype, in, 0, w, w_dtype, in, 0, 1, r, y, y_dtype, out, 0, bias, 1,
                       compute, workspace, workspace_bytes, stream);
}
