// 16-bit MFMA GEMM kernel template (fp16 or bf16 multiplicands, fp32
// accumulation) shared by gemm_f16.hip and gemm_bf16.hip.
//
//   C[b][i,j] = alpha * sum_p opA[b][i,p] * opB[b][p,j] (+ C) (+ bias[j])
//
// Tiling.  A workgroup owns a BM x BN tile of C and walks K in steps of 32.
// Its wave64s form a (BM/WM) x (BN/WN) grid; a wave owns a WM x WN sub-tile as
// (WM/32) x (WN/32) v_mfma_f32_32x32x16 blocks.  Two configurations are
// built: 256x128 tiles with 128x64 wave tiles for the large linear-layer
// products and 128x128 / 64x64 for everything smaller.
//
// Operands may be stored as fp32 or as the MFMA element type, and with either
// dimension contiguous.  Whatever the source, the loader converts to the MFMA
// type on the way into LDS:
//   k contiguous in memory  -> LDS tile [row][k], rows padded to 40 elements,
//                              fragments read with one ds_read_b128;
//   row contiguous in memory-> LDS tile [k][row], rows padded by 16 elements,
//                              fragments read with two ds_read_b64_tr_b16,
//                              the gfx950 transposing LDS load, so a k-strided
//                              operand costs no scattered LDS traffic.
// Global loads run STAGES K steps ahead of the MFMAs in per-stage register
// sets (2 stages with an fp32 operand, 3 with 16-bit ones) and are committed
// to one of two LDS buffers right before their step, one barrier per K step.
// The fast kernel needs K % 32 == 0 and 16-byte aligned rows; a guarded
// variant of the same kernel (element-wise bounds checks, one stage) takes
// every other shape.
//
// Tile order.  Workgroup ids are first spread so that ids that land on the
// same XCD (id mod 8) are contiguous, then mapped to tiles in blocks of up to
// 8 x 4 tiles, so the workgroups resident on one XCD at a time share A and B
// panels in that XCD's L2.
#pragma once

#include "common.hpp"

#include <hip/hip_bf16.h>

namespace brk {
namespace gemm16 {

typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef short s16x4 __attribute__((ext_vector_type(4)));
typedef unsigned short u16;
// native vectors (not the u32x4 / u32x2 structs): copies of these are plain
// register moves, never memcpy through a private-memory temporary
typedef unsigned u32x4 __attribute__((ext_vector_type(4)));
typedef unsigned u32x2 __attribute__((ext_vector_type(2)));

constexpr int BK = 32;
constexpr int kPitchK = BK + 8;  // [row][k] tiles: row pitch in elements (80 bytes)
constexpr int kPadR = 16;        // [k][row] tiles: row pitch is rows + 16 elements

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
    // second output of the direct-to-LDS kernel's GELU epilogue: gelu of what
    // goes to c, same layout and type as c (null = plain epilogue)
    void* c2 = nullptr;
    // what an accumulating product adds to: a tensor laid out like c (same type, leading dimension and batch
    // stride), read where c is written; null = c itself
    const void* addend = nullptr;
    // K split of the direct-to-LDS kernel: with splits == 2 two workgroups share an output tile, each summing one
    // half of K; the first to finish leaves its fp32 partial tile in `partials`, the second adds it to its own and
    // runs the epilogue (see gemm_dtl16.hpp).  splits == 1: no split, partials unused.
    int splits = 1;
    float* partials = nullptr;
    size_t partial_bytes = 0;
    int split_slot = 0;   // which set of the library's arrival counters the two slices of a tile meet through (one per stream)
};

template <int CT>
struct Cvt;
template <>
struct Cvt<BR_GEMM_F16> {
    static __device__ __forceinline__ u16 from_f32(float f) { return __builtin_bit_cast(u16, (_Float16)f); }
    static __device__ __forceinline__ f32x16 mfma(const u32x4& a, const u32x4& b, f32x16 c) {
        return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8, a), __builtin_bit_cast(f16x8, b), c,
                                                      0, 0, 0);
    }
};
template <>
struct Cvt<BR_GEMM_BF16> {
    static __device__ __forceinline__ u16 from_f32(float f) { return __builtin_bit_cast(u16, (__bf16)f); }
    static __device__ __forceinline__ f32x16 mfma(const u32x4& a, const u32x4& b, f32x16 c) {
        return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b),
                                                       c, 0, 0, 0);
    }
};

__device__ __forceinline__ u32x4 mk4(unsigned a, unsigned b, unsigned c, unsigned d) {
    u32x4 v;
    v.x = a; v.y = b; v.z = c; v.w = d;
    return v;
}
__device__ __forceinline__ u32x2 mk2(unsigned a, unsigned b) {
    u32x2 v;
    v.x = a; v.y = b;
    return v;
}
__device__ __forceinline__ unsigned pack2(u16 lo, u16 hi) { return (unsigned)lo | ((unsigned)hi << 16); }

template <int CT>
__device__ __forceinline__ u32x2 cvt4(const u32x4& f) {
    return mk2(pack2(Cvt<CT>::from_f32(__uint_as_float(f.x)), Cvt<CT>::from_f32(__uint_as_float(f.y))),
                      pack2(Cvt<CT>::from_f32(__uint_as_float(f.z)), Cvt<CT>::from_f32(__uint_as_float(f.w))));
}

// ---- operand tile: ROWS x BK, staged through registers into LDS ----------
// GUARD = false: the fast kernel.  Every access is an unconditional 128-bit
// load; rows past the end of the operand are redirected to a valid row (their
// products land in rows / columns of C that are never stored).  The caller
// guarantees K % 32 == 0 and, for row-contiguous operands, rows % kVec == 0.
// GUARD = true: the generic kernel.  Every element is bounds-checked and
// zero-filled, any size and alignment.
template <int CT, int ROWS, int THREADS, bool F32SRC, bool KSTR>
struct Tile {
    // elements per global access: 8 along k (two float4 or one 128-bit fp16
    // load) for k-contiguous sources; along rows, 4 for fp32 and 8 for 16-bit
    static constexpr int kVec = KSTR ? (F32SRC ? 4 : 8) : 8;
    static constexpr int kChunks = ROWS * BK / kVec;
    static constexpr int kPasses = kChunks / THREADS;
    static_assert(kChunks % THREADS == 0, "tile does not divide among the threads");
    static constexpr int kRegs = (!KSTR && F32SRC) ? 2 : 1;  // u32x4 registers per pass
    static constexpr int kNumRegs = kPasses * kRegs;
    static constexpr int kLdsElems = KSTR ? BK * (ROWS + kPadR) : ROWS * kPitchK;

    template <bool GUARD>
    static __device__ __forceinline__ void fetch(u32x4 (&r)[kNumRegs], const void* base, long long ld,
                                                 long long row0, long long rows, long long k0, long long kdim) {
        const int t = threadIdx.x;
#pragma unroll
        for (int p = 0; p < kPasses; p++) {
            const int id = p * THREADS + t;
            if (!KSTR) {
                const int c = id % (BK / 8), rr = id / (BK / 8);
                long long row = row0 + rr;
                const long long kk = k0 + c * 8;
                if (!GUARD) {
                    row = row < rows ? row : rows - 1;
                    const long long off = row * ld + kk;
                    if (F32SRC) {
                        const u32x4* g = reinterpret_cast<const u32x4*>(static_cast<const float*>(base) + off);
                        r[p * kRegs] = g[0];
                        r[p * kRegs + (kRegs - 1)] = g[1];
                    } else {
                        r[p] = *reinterpret_cast<const u32x4*>(static_cast<const u16*>(base) + off);
                    }
                } else {
                    const long long off = row * ld + kk;
                    unsigned w[8];
#pragma unroll
                    for (int e = 0; e < 8; e++) {
                        const bool ok = row < rows && kk + e < kdim;
                        if (F32SRC)
                            w[e] = ok ? reinterpret_cast<const unsigned*>(base)[off + e] : 0u;
                        else
                            w[e] = ok ? (unsigned)static_cast<const u16*>(base)[off + e] : 0u;
                    }
                    if (F32SRC) {
                        r[p * kRegs] = mk4(w[0], w[1], w[2], w[3]);
                        r[p * kRegs + (kRegs - 1)] = mk4(w[4], w[5], w[6], w[7]);
                    } else {
                        r[p] = mk4(w[0] | (w[1] << 16), w[2] | (w[3] << 16), w[4] | (w[5] << 16),
                                          w[6] | (w[7] << 16));
                    }
                }
            } else {
                // chunk = kVec consecutive rows of one k
                const int rc = id % (ROWS / kVec), kk_ = id / (ROWS / kVec);
                long long row = row0 + rc * kVec;
                const long long kidx = k0 + kk_;
                if (!GUARD) {
                    row = row < rows ? row : 0;
                    const long long off = kidx * ld + row;
                    if (F32SRC)
                        r[p] = *reinterpret_cast<const u32x4*>(static_cast<const float*>(base) + off);
                    else
                        r[p] = *reinterpret_cast<const u32x4*>(static_cast<const u16*>(base) + off);
                } else {
                    const long long off = kidx * ld + row;
                    unsigned w[8] = {0u, 0u, 0u, 0u, 0u, 0u, 0u, 0u};
#pragma unroll
                    for (int e = 0; e < kVec; e++) {
                        const bool ok = row + e < rows && kidx < kdim;
                        if (F32SRC)
                            w[e] = ok ? reinterpret_cast<const unsigned*>(base)[off + e] : 0u;
                        else
                            w[e] = ok ? (unsigned)static_cast<const u16*>(base)[off + e] : 0u;
                    }
                    if (F32SRC)
                        r[p] = mk4(w[0], w[1], w[2], w[3]);
                    else
                        r[p] = mk4(w[0] | (w[1] << 16), w[2] | (w[3] << 16), w[4] | (w[5] << 16),
                                          w[6] | (w[7] << 16));
                }
            }
        }
    }

    static __device__ __forceinline__ void commit(const u32x4 (&r)[kNumRegs], u16* tile) {
        const int t = threadIdx.x;
#pragma unroll
        for (int p = 0; p < kPasses; p++) {
            const int id = p * THREADS + t;
            if (!KSTR) {
                const int c = id % (BK / 8), rr = id / (BK / 8);
                u32x4 h;
                if (F32SRC) {
                    const u32x2 lo = cvt4<CT>(r[p * kRegs]), hi = cvt4<CT>(r[p * kRegs + (kRegs - 1)]);
                    h = mk4(lo.x, lo.y, hi.x, hi.y);
                } else {
                    h = r[p];
                }
                *reinterpret_cast<u32x4*>(tile + rr * kPitchK + c * 8) = h;
            } else {
                const int rc = id % (ROWS / kVec), kk_ = id / (ROWS / kVec);
                u16* dst = tile + kk_ * (ROWS + kPadR) + rc * kVec;
                if (F32SRC)
                    *reinterpret_cast<u32x2*>(dst) = cvt4<CT>(r[p]);
                else
                    *reinterpret_cast<u32x4*>(dst) = r[p];
            }
        }
    }

    // MFMA operand for the 32 rows starting at `row_base` and the 16 k-values
    // of sub-step ks: lane l holds row (l % 32), k = ks*16 + (l / 32)*8 + 0..7.
    static __device__ __forceinline__ u32x4 fragment(const u16* tile, int row_base, int ks) {
        const int lane = threadIdx.x & 63;
        if (!KSTR) {
            return *reinterpret_cast<const u32x4*>(tile + (row_base + (lane & 31)) * kPitchK + ks * 16 +
                                                   (lane >> 5) * 8);
        } else {
            // Transposing read: within each group of 16 lanes, lane i supplies
            // the address of 4 consecutive rows at k-row (i / 4); the hardware
            // returns to lane l the 4 k-values of row l of the group.
            const int i = lane & 15, grp = lane >> 4;
            const int rows16 = row_base + (grp & 1) * 16 + (i & 3) * 4;
            const int kk = ks * 16 + (grp >> 1) * 8 + (i >> 2);
            const u16* p = tile + kk * (ROWS + kPadR) + rows16;
            typedef __attribute__((address_space(3))) s16x4 lds_s16x4;
            const s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4*)p);
            const s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4*)(p + 4 * (ROWS + kPadR)));
            const u32x2 l2 = __builtin_bit_cast(u32x2, lo), h2 = __builtin_bit_cast(u32x2, hi);
            return mk4(l2.x, l2.y, h2.x, h2.y);
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


// Tile number `rem` (0 .. tiles_m * tiles_n - 1) of one batch in the order workgroups take them.
// Panels of GN tile columns; inside a panel, blocks of GM x gn tiles with m
// fastest: the ~32 workgroups an XCD runs at a time cover a GM x GN block and
// share GM + GN operand strips in its L2 (8 x 4: 12 strips for 32 tiles; a
// column-first walk down a tall product would touch 33).
__device__ __forceinline__ void tile_in_order(const GemmArgs& g, int rem, int& tm, int& tn) {
    const int GM = g.tiles_m < 8 ? g.tiles_m : 8;
    const int GN = 32 / GM > 4 ? 32 / GM : 4;
    const int group = rem / (GN * g.tiles_m);
    const int first_n = group * GN;
    const int gn = g.tiles_n - first_n < GN ? g.tiles_n - first_n : GN;
    const int in_group = rem - group * GN * g.tiles_m;
    const int blk = in_group / (GM * gn);
    const int within = in_group - blk * GM * gn;
    const int gm = g.tiles_m - blk * GM < GM ? g.tiles_m - blk * GM : GM;
    tm = blk * GM + within % gm;
    tn = first_n + within / gm;
}

// Workgroup id -> (batch, tile_m, tile_n).
__device__ __forceinline__ void tile_coords(const GemmArgs& g, long long& batch, int& tm, int& tn) {
    const long long nb = gridDim.x;
    long long id = blockIdx.x;
    // ids are dealt to the 8 XCDs round-robin; make each XCD's share contiguous
    const long long per_xcd = nb / 8;
    if (per_xcd > 0 && id < per_xcd * 8) id = (id % 8) * per_xcd + id / 8;
    const long long per_batch = (long long)g.tiles_m * g.tiles_n;
    batch = id / per_batch;
    const int rem = (int)(id % per_batch);
    tile_in_order(g, rem, tm, tn);
}

// Where a tile starts its walk over K (an element index, a multiple of 64; the walk wraps round at the end of K).
// Workgroups that run side by side would otherwise all read the same 128-byte column of their operand rows at the
// same time; with row pitches that are large powers of two those lines fall on a few memory channels and the
// fetches queue behind one another (a [2048 x 4096] by [16384 x 4096] product, run back to back: 1105 TFLOP/s so,
// 1175 with the starts spread; the other shapes of the BLOOM-7B1 block measure the same either way).  The start depends only on the 256 x 256 block of C the tile lies in and on K, so every kernel and
// every tile shape in this library sums a given element of C in the same order and produces the same bits; the
// spread is kept to seven neighbouring columns so that tiles sharing an operand panel still meet in L2.
__device__ __forceinline__ long long k_walk_start(long long row0, long long col0, long long k) {
    const long long n64 = k >> 6;
    if (n64 < 2) return 0;
    const long long phase = ((row0 >> 8) & 3) + ((col0 >> 8) & 3);
    return 64 * (phase % n64);
}

// The K loop.  STAGES register sets: the global loads of K steps t+1 ..
// t+STAGES are in flight while step t is multiplied, which is what hides HBM /
// L2 latency.  Two LDS buffers, one barrier per step: a wave can only reach the
// commit of step t+2 (same buffer as t) after every wave has passed the barrier
// of step t+1, i.e. has finished multiplying step t.
template <bool GUARD, int CT, int BM, int BN, int WM, int WN, int STAGES, typename TA, typename TB>
__device__ __forceinline__ void main_loop(const GemmArgs& g, const void* a_base, const void* b_base, long long row0,
                                          long long col0, u16* lds_a, u16* lds_b,
                                          f32x16 (&acc)[WM / 32][WN / 32]) {
    constexpr int FM = WM / 32, FN = WN / 32;
    const int wave = threadIdx.x >> 6;
    const int wm = wave / (BN / WN), wn = wave % (BN / WN);
    static_assert(STAGES >= 1 && STAGES <= 3, "one to three prefetch stages");
    // one named register set per stage (no indexing across stages, so every
    // set stays in registers)
    u32x4 ra0[TA::kNumRegs], ra1[TA::kNumRegs], ra2[TA::kNumRegs];
    u32x4 rb0[TB::kNumRegs], rb1[TB::kNumRegs], rb2[TB::kNumRegs];
    const long long nk = (g.k + BK - 1) / BK;
    const long long first = k_walk_start(row0, col0, g.k) / BK;  // step `s` of the loop covers K step (s + first) mod nk

    auto fetch = [&](u32x4 (&xa)[TA::kNumRegs], u32x4 (&xb)[TB::kNumRegs], long long step) {
        if (step < nk) {
            const long long at = step + first < nk ? step + first : step + first - nk;
            TA::template fetch<GUARD>(xa, a_base, g.lda, row0, g.m, at * BK, g.k);
            TB::template fetch<GUARD>(xb, b_base, g.ldb, col0, g.n, at * BK, g.k);
        }
    };
    auto run = [&](u32x4 (&xa)[TA::kNumRegs], u32x4 (&xb)[TB::kNumRegs], long long step) {
        if (step >= nk) return;
        u16* ta = lds_a + (step & 1) * TA::kLdsElems;
        u16* tb = lds_b + (step & 1) * TB::kLdsElems;
        TA::commit(xa, ta);
        TB::commit(xb, tb);
        __syncthreads();
        fetch(xa, xb, step + STAGES);
#pragma unroll
        for (int ks = 0; ks < BK / 16; ks++) {
            u32x4 fa[FM], fb[FN];
#pragma unroll
            for (int i = 0; i < FM; i++) fa[i] = TA::fragment(ta, wm * WM + i * 32, ks);
#pragma unroll
            for (int j = 0; j < FN; j++) fb[j] = TB::fragment(tb, wn * WN + j * 32, ks);
#pragma unroll
            for (int i = 0; i < FM; i++)
#pragma unroll
                for (int j = 0; j < FN; j++) acc[i][j] = Cvt<CT>::mfma(fa[i], fb[j], acc[i][j]);
        }
    };

    fetch(ra0, rb0, 0);
    if (STAGES > 1) fetch(ra1, rb1, 1);
    if (STAGES > 2) fetch(ra2, rb2, 2);
    for (long long kt = 0; kt < nk; kt += STAGES) {
        run(ra0, rb0, kt);
        if (STAGES > 1) run(ra1, rb1, kt + 1);
        if (STAGES > 2) run(ra2, rb2, kt + 2);
    }
}

template <bool GUARD, int CT, int BM, int BN, int WM, int WN, int STAGES, bool A_F32, bool A_KSTR, bool B_F32,
          bool B_KSTR, typename TC>
__global__ __launch_bounds__((BM / WM) * (BN / WN) * 64) void gemm_kernel(GemmArgs g) {
    constexpr int THREADS = (BM / WM) * (BN / WN) * 64;
    constexpr int FM = WM / 32, FN = WN / 32;
    using TA = Tile<CT, BM, THREADS, A_F32, A_KSTR>;
    using TB = Tile<CT, BN, THREADS, B_F32, B_KSTR>;
    __shared__ __attribute__((aligned(16))) u16 lds_a[2][TA::kLdsElems];
    __shared__ __attribute__((aligned(16))) u16 lds_b[2][TB::kLdsElems];

    long long batch;
    int tm, tn;
    tile_coords(g, batch, tm, tn);
    const long long row0 = (long long)tm * BM, col0 = (long long)tn * BN;
    const void* a_base = A_F32 ? (const void*)(static_cast<const float*>(g.a) + batch * g.sa)
                               : (const void*)(static_cast<const u16*>(g.a) + batch * g.sa);
    const void* b_base = B_F32 ? (const void*)(static_cast<const float*>(g.b) + batch * g.sb)
                               : (const void*)(static_cast<const u16*>(g.b) + batch * g.sb);
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int wm = wave / (BN / WN), wn = wave % (BN / WN);

    f32x16 acc[FM][FN];
#pragma unroll
    for (int i = 0; i < FM; i++)
#pragma unroll
        for (int j = 0; j < FN; j++)
#pragma unroll
            for (int v = 0; v < 16; v++) acc[i][j][v] = 0.f;

    main_loop<GUARD, CT, BM, BN, WM, WN, STAGES, TA, TB>(g, a_base, b_base, row0, col0, lds_a[0], lds_b[0], acc);

    // acc[i][j][v] is C[row, col] with
    //   row = wm*WM + i*32 + (v/4)*8 + (lane/32)*4 + v%4,  col = wn*WN + j*32 + lane%32
    TC* c_base = static_cast<TC*>(g.c) + batch * g.sc;
    const TC* old_base = g.addend ? static_cast<const TC*>(g.addend) + batch * g.sc : c_base;
#pragma unroll
    for (int j = 0; j < FN; j++) {
        const long long col = col0 + wn * WN + j * 32 + (lane & 31);
        if (col >= g.n) continue;
        const float bias = g.bias ? g.bias[col] : 0.f;
#pragma unroll
        for (int i = 0; i < FM; i++) {
#pragma unroll
            for (int v = 0; v < 16; v++) {
                const long long row = row0 + wm * WM + i * 32 + (v >> 2) * 8 + (lane >> 5) * 4 + (v & 3);
                if (row < g.m) {
                    TC* p = c_base + row * g.ldc + col;
                    float o = g.alpha * acc[i][j][v] + bias;
                    if (g.accumulate) o += c_load<TC>(old_base + row * g.ldc + col);
                    c_store<TC>(p, o);
                }
            }
        }
    }
}

// ---- host-side dispatch over the template parameters ------------------------
struct Problem {
    bool a_f32, a_kstr, b_f32, b_kstr;
    int c_dtype;
    bool guarded;  // sizes / alignment rule out the fast kernel
};

template <bool GUARD, int CT, int BM, int BN, int WM, int WN, bool AF, bool AK, bool BF, bool BK_>
int launch_c(const GemmArgs& g, int c_dtype, unsigned grid, hipStream_t st) {
    constexpr int THREADS = (BM / WM) * (BN / WN) * 64;
    // prefetch depth: 16-bit operands need half the registers per stage
    constexpr int ST = GUARD ? 1 : ((AF || BF) ? 2 : 3);
    if (c_dtype == BR_F32) {
        gemm_kernel<GUARD, CT, BM, BN, WM, WN, ST, AF, AK, BF, BK_, float><<<grid, THREADS, 0, st>>>(g);
    } else if (CT == BR_GEMM_F16 && c_dtype == BR_F16) {
        gemm_kernel<GUARD, CT, BM, BN, WM, WN, ST, AF, AK, BF, BK_, __half><<<grid, THREADS, 0, st>>>(g);
    } else if (CT == BR_GEMM_BF16 && c_dtype == BR_BF16) {
        gemm_kernel<GUARD, CT, BM, BN, WM, WN, ST, AF, AK, BF, BK_, __hip_bfloat16><<<grid, THREADS, 0, st>>>(g);
    } else {
        return BR_ERR_TODO;
    }
    BR_HIP_LAUNCH_CHECK();
    return BR_OK;
}

template <bool GUARD, int CT, int BM, int BN, int WM, int WN>
int launch_layout(const GemmArgs& g, const Problem& p, unsigned grid, hipStream_t st) {
#define BR_GEMM_CASE(AF, AK, BF, BK_)                                         \
    if (p.a_f32 == AF && p.a_kstr == AK && p.b_f32 == BF && p.b_kstr == BK_)  \
        return launch_c<GUARD, CT, BM, BN, WM, WN, AF, AK, BF, BK_>(g, p.c_dtype, grid, st);
    BR_GEMM_CASE(true, true, true, true)
    BR_GEMM_CASE(true, true, true, false)
    BR_GEMM_CASE(true, true, false, true)
    BR_GEMM_CASE(true, true, false, false)
    BR_GEMM_CASE(true, false, true, true)
    BR_GEMM_CASE(true, false, true, false)
    BR_GEMM_CASE(true, false, false, true)
    BR_GEMM_CASE(true, false, false, false)
    BR_GEMM_CASE(false, true, true, true)
    BR_GEMM_CASE(false, true, true, false)
    BR_GEMM_CASE(false, true, false, true)
    BR_GEMM_CASE(false, true, false, false)
    BR_GEMM_CASE(false, false, true, true)
    BR_GEMM_CASE(false, false, true, false)
    BR_GEMM_CASE(false, false, false, true)
    BR_GEMM_CASE(false, false, false, false)
#undef BR_GEMM_CASE
    return BR_ERR_TODO;
}

// Fills in the tile counts and launches the register-staged kernel.
template <int CT>
int launch(GemmArgs g, const Problem& p, long long batch, hipStream_t st) {
    g.tiles_m = (int)((g.m + 127) / 128);
    g.tiles_n = (int)((g.n + 127) / 128);
    const long long blocks = (long long)g.tiles_m * g.tiles_n * batch;
    if (blocks > 0x7fffffffLL) return BR_ERR_ATTR;
    if (p.guarded) return launch_layout<true, CT, 128, 128, 64, 64>(g, p, (unsigned)blocks, st);
    return launch_layout<false, CT, 128, 128, 64, 64>(g, p, (unsigned)blocks, st);
}

}  // namespace gemm16
}  // namespace brk
