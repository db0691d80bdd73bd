// Strided-batched GEMM on the gfx950 matrix cores.
//
//   C[b][i,j] = alpha * sum_p opA[b][i,p] * opB[b][p,j] (+ C) (+ bias[j])
//
// Workgroup tile 128x128, K step 32, 256 threads = 4 wave64s in a 2x2 grid,
// each wave owning a 64x64 sub-tile as 2x2 v_mfma_f32_32x32x16 blocks with
// fp32 accumulators.  Operands may live in HBM as fp32, fp16 or bf16 and with
// either dimension contiguous; the loaders convert to the MFMA element type
// and lay every tile out in LDS as [row][k] (k contiguous, rows padded to 40
// elements), so the inner loop is the same for all layouts.  Global loads for
// tile t+1 are issued before the MFMAs of tile t and committed to the other
// LDS buffer afterwards (register prefetch + LDS double buffering, one
// barrier per K step).
//
// A second kernel keeps fp32 operands and multiplies with
// v_mfma_f32_32x32x2_f32 for callers that need fp32-faithful products.
#include "common.hpp"

#include <hip/hip_bf16.h>

using namespace brk;

namespace {

typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef unsigned short u16;

constexpr int BM = 128, BN = 128, BK = 32;
constexpr int kThreads = 256;
constexpr int kPitch = BK + 8;  // LDS row pitch in 16-bit elements (80 bytes)

struct GemmArgs {
    const void* a;
    const void* b;
    void* c;
    const float* bias;
    long long m, n, k;
    long long lda, ldb, ldc;
    long long sa, sb, sc;
    float alpha;
    int accumulate;
    int tiles_m, tiles_n;
    int vec_a, vec_b;  // 128-bit global loads allowed for this operand
};

// ---- element conversion ------------------------------------------------
template <int CT>
struct Cvt;
template <>
struct Cvt<BR_GEMM_F16> {
    static __device__ __forceinline__ u16 from_f32(float f) {
        return __builtin_bit_cast(u16, (_Float16)f);
    }
    static __device__ __forceinline__ f32x16 mfma(const uint4& a, const uint4& b, f32x16 c) {
        return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8, a), __builtin_bit_cast(f16x8, b), c,
                                                      0, 0, 0);
    }
};
template <>
struct Cvt<BR_GEMM_BF16> {
    static __device__ __forceinline__ u16 from_f32(float f) {
        return __builtin_bit_cast(u16, (__bf16)f);
    }
    static __device__ __forceinline__ f32x16 mfma(const uint4& a, const uint4& b, f32x16 c) {
        return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b),
                                                       c, 0, 0, 0);
    }
};

__device__ __forceinline__ unsigned pack2(u16 lo, u16 hi) { return (unsigned)lo | ((unsigned)hi << 16); }

// ---- operand tile loader -------------------------------------------------
// A "tile" is 128 rows x BK k-values of one operand.  `row` indexes the
// operand's non-reduction dimension.  KSTR == false: element (row, kk) sits
// at base[row*ld + kk]; KSTR == true: at base[kk*ld + row].
// F32SRC: the operand is stored as fp32 (converted on commit), otherwise it
// is already stored in the MFMA element type.
template <int CT, bool F32SRC, bool KSTR>
struct TileLoader {
    // raw registers fetched from global memory for one tile
    uint4 r[F32SRC ? 4 : 2];

    // ------------------------------------------------------------ fetch
    __device__ __forceinline__ void fetch(const void* base, long long ld, long long row0, long long rows,
                                          long long k0, long long kdim, bool vec) {
        const int t = threadIdx.x;
        if (!KSTR) {
            // thread -> (row r0 + 64*p, 8 consecutive k starting at c*8)
            const int c = t & 3, r0 = t >> 2;
            const bool k_in = k0 + c * 8 + 8 <= kdim;
#pragma unroll
            for (int p = 0; p < 2; p++) {
                const long long row = row0 + r0 + 64 * p;
                const long long off = row * ld + k0 + c * 8;
                if (vec && k_in && row < rows) {
                    if (F32SRC) {
                        const uint4* g = reinterpret_cast<const uint4*>(static_cast<const float*>(base) + off);
                        r[2 * p] = g[0];
                        r[2 * p + 1] = g[1];
                    } else {
                        r[p] = *reinterpret_cast<const uint4*>(static_cast<const u16*>(base) + off);
                    }
                } else {
                    unsigned w[8];
#pragma unroll
                    for (int e = 0; e < 8; e++) {
                        const bool ok = row < rows && k0 + c * 8 + e < kdim;
                        if (F32SRC)
                            w[e] = ok ? reinterpret_cast<const unsigned*>(base)[off + e] : 0u;
                        else
                            w[e] = ok ? static_cast<const u16*>(base)[off + e] : 0u;
                    }
                    if (F32SRC) {
                        r[2 * p] = make_uint4(w[0], w[1], w[2], w[3]);
                        r[2 * p + 1] = make_uint4(w[4], w[5], w[6], w[7]);
                    } else {
                        r[p] = make_uint4(w[0] | (w[1] << 16), w[2] | (w[3] << 16), w[4] | (w[5] << 16),
                                          w[6] | (w[7] << 16));
                    }
                }
            }
        } else {
            // thread -> (4 consecutive rows starting at 4*r4, 4 consecutive k starting at 4*kg)
            const int r4 = t & 31, kg = t >> 5;
            const long long row = row0 + 4 * r4;
            const bool rows_in = row + 4 <= rows;
#pragma unroll
            for (int kk = 0; kk < 4; kk++) {
                const long long kidx = k0 + 4 * kg + kk;
                const long long off = kidx * ld + row;
                unsigned w[4];
                if (vec && rows_in && kidx < kdim) {
                    if (F32SRC) {
                        const uint4 g = *reinterpret_cast<const uint4*>(static_cast<const float*>(base) + off);
                        w[0] = g.x; w[1] = g.y; w[2] = g.z; w[3] = g.w;
                    } else {
                        const uint2 g = *reinterpret_cast<const uint2*>(static_cast<const u16*>(base) + off);
                        w[0] = g.x & 0xffffu; w[1] = g.x >> 16; w[2] = g.y & 0xffffu; w[3] = g.y >> 16;
                    }
                } else {
#pragma unroll
                    for (int e = 0; e < 4; e++) {
                        const bool ok = row + e < rows && kidx < kdim;
                        if (F32SRC)
                            w[e] = ok ? reinterpret_cast<const unsigned*>(base)[off + e] : 0u;
                        else
                            w[e] = ok ? static_cast<const u16*>(base)[off + e] : 0u;
                    }
                }
                if (F32SRC) {
                    r[kk] = make_uint4(w[0], w[1], w[2], w[3]);
                } else {
                    // two k-rows per uint4: (.x,.y) hold kk even, (.z,.w) hold kk odd
                    const unsigned lo = w[0] | (w[1] << 16), hi = w[2] | (w[3] << 16);
                    if (kk & 1) {
                        r[kk >> 1].z = lo;
                        r[kk >> 1].w = hi;
                    } else {
                        r[kk >> 1].x = lo;
                        r[kk >> 1].y = hi;
                    }
                }
            }
        }
    }

    // ----------------------------------------------------------- commit
    // Convert and store into an LDS tile laid out [128][kPitch].
    __device__ __forceinline__ void commit(u16* tile) const {
        const int t = threadIdx.x;
        if (!KSTR) {
            const int c = t & 3, r0 = t >> 2;
#pragma unroll
            for (int p = 0; p < 2; p++) {
                uint4 h;
                if (F32SRC) {
                    const uint4 lo = r[2 * p], hi = r[2 * p + 1];
                    h.x = pack2(Cvt<CT>::from_f32(__uint_as_float(lo.x)), Cvt<CT>::from_f32(__uint_as_float(lo.y)));
                    h.y = pack2(Cvt<CT>::from_f32(__uint_as_float(lo.z)), Cvt<CT>::from_f32(__uint_as_float(lo.w)));
                    h.z = pack2(Cvt<CT>::from_f32(__uint_as_float(hi.x)), Cvt<CT>::from_f32(__uint_as_float(hi.y)));
                    h.w = pack2(Cvt<CT>::from_f32(__uint_as_float(hi.z)), Cvt<CT>::from_f32(__uint_as_float(hi.w)));
                } else {
                    h = r[p];
                }
                *reinterpret_cast<uint4*>(tile + (r0 + 64 * p) * kPitch + c * 8) = h;
            }
        } else {
            const int r4 = t & 31, kg = t >> 5;
            // element (row 4*r4 + e, k 4*kg + kk)
            u16 v[4][4];  // [kk][e]
#pragma unroll
            for (int kk = 0; kk < 4; kk++) {
                if (F32SRC) {
                    v[kk][0] = Cvt<CT>::from_f32(__uint_as_float(r[kk].x));
                    v[kk][1] = Cvt<CT>::from_f32(__uint_as_float(r[kk].y));
                    v[kk][2] = Cvt<CT>::from_f32(__uint_as_float(r[kk].z));
                    v[kk][3] = Cvt<CT>::from_f32(__uint_as_float(r[kk].w));
                } else {
                    const unsigned lo = (kk & 1) ? r[kk >> 1].z : r[kk >> 1].x;
                    const unsigned hi = (kk & 1) ? r[kk >> 1].w : r[kk >> 1].y;
                    v[kk][0] = (u16)(lo & 0xffffu); v[kk][1] = (u16)(lo >> 16);
                    v[kk][2] = (u16)(hi & 0xffffu); v[kk][3] = (u16)(hi >> 16);
                }
            }
#pragma unroll
            for (int e = 0; e < 4; e++) {
                uint2 h;
                h.x = pack2(v[0][e], v[1][e]);
                h.y = pack2(v[2][e], v[3][e]);
                *reinterpret_cast<uint2*>(tile + (4 * r4 + e) * kPitch + 4 * kg) = h;
            }
        }
    }
};

template <typename T>
__device__ __forceinline__ float c_load(const T* p);
template <>
__device__ __forceinline__ float c_load<float>(const float* p) { return *p; }
template <>
__device__ __forceinline__ float c_load<__half>(const __half* p) { return __half2float(*p); }
template <>
__device__ __forceinline__ float c_load<__hip_bfloat16>(const __hip_bfloat16* p) { return __bfloat162float(*p); }
template <typename T>
__device__ __forceinline__ void c_store(T* p, float v);
template <>
__device__ __forceinline__ void c_store<float>(float* p, float v) { *p = v; }
template <>
__device__ __forceinline__ void c_store<__half>(__half* p, float v) { *p = __float2half_rn(v); }
template <>
__device__ __forceinline__ void c_store<__hip_bfloat16>(__hip_bfloat16* p, float v) { *p = __float2bfloat16(v); }

// Tile index from the linear workgroup id: m varies fastest so that
// neighbouring workgroups share one panel of B (the weight matrix in the
// linear layers), which is then fetched from HBM once.
__device__ __forceinline__ void tile_coords(const GemmArgs& g, long long& batch, int& tm, int& tn) {
    const long long per_batch = (long long)g.tiles_m * g.tiles_n;
    const long long id = blockIdx.x;
    batch = id / per_batch;
    const int rem = (int)(id % per_batch);
    tm = rem % g.tiles_m;
    tn = rem / g.tiles_m;
}

template <int CT, bool A_F32, bool A_KSTR, bool B_F32, bool B_KSTR, typename TC>
__global__ __launch_bounds__(kThreads) void gemm_mfma16_kernel(GemmArgs g) {
    __shared__ __attribute__((aligned(16))) u16 lds_a[2][BM * kPitch];
    __shared__ __attribute__((aligned(16))) u16 lds_b[2][BN * kPitch];

    long long batch;
    int tm, tn;
    tile_coords(g, batch, tm, tn);
    const long long row0 = (long long)tm * BM, col0 = (long long)tn * BN;
    const void* a_base = A_F32 ? (const void*)(static_cast<const float*>(g.a) + batch * g.sa)
                               : (const void*)(static_cast<const u16*>(g.a) + batch * g.sa);
    const void* b_base = B_F32 ? (const void*)(static_cast<const float*>(g.b) + batch * g.sb)
                               : (const void*)(static_cast<const u16*>(g.b) + batch * g.sb);

    TileLoader<CT, A_F32, A_KSTR> la;
    TileLoader<CT, B_F32, B_KSTR> lb;

    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int wm = wave >> 1, wn = wave & 1;
    const int lrow = lane & 31, lk = (lane >> 5) * 8;

    f32x16 acc[2][2];
#pragma unroll
    for (int i = 0; i < 2; i++)
#pragma unroll
        for (int j = 0; j < 2; j++)
#pragma unroll
            for (int v = 0; v < 16; v++) acc[i][j][v] = 0.f;

    const long long nk = (g.k + BK - 1) / BK;
    la.fetch(a_base, g.lda, row0, g.m, 0, g.k, g.vec_a);
    lb.fetch(b_base, g.ldb, col0, g.n, 0, g.k, g.vec_b);
    la.commit(lds_a[0]);
    lb.commit(lds_b[0]);
    __syncthreads();

    for (long long kt = 0; kt < nk; kt++) {
        const int cur = (int)(kt & 1);
        if (kt + 1 < nk) {
            la.fetch(a_base, g.lda, row0, g.m, (kt + 1) * BK, g.k, g.vec_a);
            lb.fetch(b_base, g.ldb, col0, g.n, (kt + 1) * BK, g.k, g.vec_b);
        }
        const u16* ta = lds_a[cur] + (wm * 64 + lrow) * kPitch + lk;
        const u16* tb = lds_b[cur] + (wn * 64 + lrow) * kPitch + lk;
#pragma unroll
        for (int ks = 0; ks < BK / 16; ks++) {
            uint4 fa[2], fb[2];
#pragma unroll
            for (int i = 0; i < 2; i++) {
                fa[i] = *reinterpret_cast<const uint4*>(ta + i * 32 * kPitch + ks * 16);
                fb[i] = *reinterpret_cast<const uint4*>(tb + i * 32 * kPitch + ks * 16);
            }
#pragma unroll
            for (int i = 0; i < 2; i++)
#pragma unroll
                for (int j = 0; j < 2; j++) acc[i][j] = Cvt<CT>::mfma(fa[i], fb[j], acc[i][j]);
        }
        if (kt + 1 < nk) {
            la.commit(lds_a[cur ^ 1]);
            lb.commit(lds_b[cur ^ 1]);
        }
        __syncthreads();
    }

    // epilogue: acc[i][j][v] is C[row, col] with
    //   row = wm*64 + i*32 + (v/4)*8 + (lane/32)*4 + v%4,  col = wn*64 + j*32 + lane%32
    TC* c_base = static_cast<TC*>(g.c) + batch * g.sc;
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
                    TC* p = c_base + row * g.ldc + col;
                    float o = g.alpha * acc[i][j][v] + bias;
                    if (g.accumulate) o += c_load<TC>(p);
                    c_store<TC>(p, o);
                }
            }
        }
    }
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
    tile_coords(g, batch, tm, tn);
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
                    if (g.accumulate) o += *p;
                    *p = o;
                }
            }
        }
    }
}

// ---- dispatch ---------------------------------------------------------------
template <int CT, bool AF, bool AK, bool BF, bool BK_>
int launch_c(const GemmArgs& g, int c_dtype, unsigned grid, hipStream_t st) {
    if (c_dtype == BR_F32) {
        gemm_mfma16_kernel<CT, AF, AK, BF, BK_, float><<<grid, kThreads, 0, st>>>(g);
    } else if (c_dtype == BR_F16 && CT == BR_GEMM_F16) {
        gemm_mfma16_kernel<CT, AF, AK, BF, BK_, __half><<<grid, kThreads, 0, st>>>(g);
    } else if (c_dtype == BR_BF16 && CT == BR_GEMM_BF16) {
        gemm_mfma16_kernel<CT, AF, AK, BF, BK_, __hip_bfloat16><<<grid, kThreads, 0, st>>>(g);
    } else {
        return BR_ERR_TODO;
    }
    BR_HIP_LAUNCH_CHECK();
    return BR_OK;
}

template <int CT, bool AF, bool AK>
int launch_b(const GemmArgs& g, bool bf, bool bk, int c_dtype, unsigned grid, hipStream_t st) {
    if (bf) return bk ? launch_c<CT, AF, AK, true, true>(g, c_dtype, grid, st)
                      : launch_c<CT, AF, AK, true, false>(g, c_dtype, grid, st);
    return bk ? launch_c<CT, AF, AK, false, true>(g, c_dtype, grid, st)
              : launch_c<CT, AF, AK, false, false>(g, c_dtype, grid, st);
}

template <int CT>
int launch_a(const GemmArgs& g, bool af, bool ak, bool bf, bool bk, int c_dtype, unsigned grid, hipStream_t st) {
    if (af) return ak ? launch_b<CT, true, true>(g, bf, bk, c_dtype, grid, st)
                      : launch_b<CT, true, false>(g, bf, bk, c_dtype, grid, st);
    return ak ? launch_b<CT, false, true>(g, bf, bk, c_dtype, grid, st)
              : launch_b<CT, false, false>(g, bf, bk, c_dtype, grid, st);
}

long long elem_size(int dtype) { return dtype == BR_F32 ? 4 : 2; }

}  // namespace

extern "C" int br_hip_gemm(int trans_a, int trans_b, int64_t m, int64_t n, int64_t k, float alpha, const void* a,
                           int a_dtype, int64_t lda, int64_t stride_a, const void* b, int b_dtype, int64_t ldb,
                           int64_t stride_b, int accumulate, void* c, int c_dtype, int64_t ldc, int64_t stride_c,
                           const float* bias, int64_t batch, int compute, br_stream_t stream) {
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
    const bool af = a_dtype == BR_F32, bf = b_dtype == BR_F32;
    if (compute == BR_GEMM_F16) return launch_a<BR_GEMM_F16>(g, af, ak, bf, bk, c_dtype, (unsigned)blocks, st);
    return launch_a<BR_GEMM_BF16>(g, af, ak, bf, bk, c_dtype, (unsigned)blocks, st);
}
