// Fused causal ALiBi attention for gfx950 (head size 128, fp16 / bf16 MFMA
// operands, fp32 accumulation): scores, probabilities and their gradients stay
// in registers, HBM sees q, k, v, o (and their gradients) once per pass.
//
// What it computes is the operator chain of the model scripts
// (bloomz-7b/train.words:154-166 forward, :217-226 backward):
//   s = (q . k^T) / sqrt(HD);  s += alibi[h, key];  s += mask(b, query, key);
//   p = softmax(s);  o = p . v
// with mask = 0 where key <= query and key < valid[b], else -FLT_MAX (the
// table blackriver/train_bloom.cpp:73-90 builds for a right-padded batch).
// Probabilities are rounded to the 16-bit type before p . v, as the unfused
// path does when it runs that product on the 16-bit MFMA.
//
// Layout.  q, k, v, o are addressed as [batch, token, head, 128] through
// explicit element strides, so the [B, T, H] outputs of the projections are
// read in place (no 0213 transposes).  lse[batch, head, token] keeps
// log(sum exp) of each score row for the backward pass.
//
// Forward kernel.  One workgroup = 4 waves = 128 queries of one (batch, head);
// each wave owns 32 queries (launches too small to fill the chip that way take
// 64-query workgroups whose waves share the keys of a tile, see the kernel).
// Keys / values stream through LDS in tiles of 64, global memory -> LDS direct;
// tiles wholly above the diagonal (or at / beyond valid[b]) are skipped, which
// is exact because their probabilities are exactly zero.  Per tile and wave:
//   S^T[key, query] = K . Q^T     16 x v_mfma_f32_32x32x16 (A = K rows from
//                                 LDS, B = Q held in registers)
//   online softmax on the accumulators: a lane holds 32 keys of ONE query
//   O^T[d, query] += V^T . P^T    16 MFMAs; P goes from the accumulators
//                                 straight into the B operand: the MFMA k index
//                                 is a summation index, so the key order the
//                                 accumulator layout implies is simply used
//                                 for the V^T operand as well (transposing LDS
//                                 reads pick the matching key rows).
// K and V tiles share one LDS image format [key][16 chunks of 8 d], chunk c of
// key r in slot c ^ g(r), g(r) = 4 * (r & 3) + ((r >> 2) & 3): 16 consecutive
// keys hit 16 different slots (128-bit row reads), 4 consecutive keys hit 4
// different 64-byte groups (transposing reads).
#include "common.hpp"
#include "gemm_mfma16.hpp"
#include "lds_direct.hpp"

#include <float.h>

#include <type_traits>

using namespace brk;
using namespace brk::gemm16;

namespace {

constexpr int kHD = 128;          // head size
constexpr int kChunks = kHD / 8;  // 16-byte chunks per row
constexpr int kBQ = 128;          // queries per workgroup (forward, dq pass)
constexpr int kBK = 64;           // keys per LDS tile
constexpr int kThreads = 256;

struct FlashArgs {
    const u16* q;
    const u16* k;
    const u16* v;
    u16* o;
    const u16* d_o;
    void* dq;  // fp32, or the operands' 16-bit type when grad16 is set
    void* dk;
    void* dv;
    int grad16;
    const float* alibi;    // [heads, tokens]
    const int32_t* valid;  // [batch]
    float* lse;            // [batch, heads, tokens]
    float* delta;          // [batch, heads, tokens]  rowsum(dO o O)
    long long row, head, batch_stride;  // element strides of q, k, v, dq, dk, dv
    long long orow, obatch;             // token / batch strides of o and d_o (same head stride)
    int heads, tokens, batch_heads;
    float scale;
};

__device__ __forceinline__ int swz(int r) { return ((r & 3) << 2) | ((r >> 2) & 3); }
// byte offset of chunk c of row r in a [rows][16 chunks] tile image
__device__ __forceinline__ unsigned slot(int r, int c) { return (unsigned)((r * kChunks + (c ^ swz(r))) * 16); }

// Direct-to-LDS fill of a tile image [64 rows][16 chunks] by the workgroup's four waves: wave w issues the
// wave-wide loads number w, w + 4, w + 8, w + 12 of the tile, each 1 KiB = 4 image rows; lane l of load L lands in
// image row 4 L + l / 16 at chunk position l % 16, so it fetches the chunk that `slot` puts there,
// (l % 16) ^ swz(row) -- and swz(row) = ((l / 16) << 2) | (L & 3), with L & 3 = w for every load of a wave: one
// per-lane offset serves all four loads, the 16-row blocks differ in the (scalar) base address only.  Rows past the
// end of the tensor read its last row, as the kernels' masks expect; only a ragged last tile takes that path.
struct TileFill {
    unsigned voff;  // this lane's byte offset inside a block of 16 rows
    unsigned cb;    // ... of which its chunk inside the row
    int lr;         // its row inside the block
    __device__ __forceinline__ TileFill(int lane, int wave, long long row_elems) {
        lr = 4 * wave + (lane >> 4);
        cb = (unsigned)(((lane & 15) ^ ((lane >> 4) << 2) ^ wave) * 16);
        voff = (unsigned)lr * (unsigned)(row_elems * 2) + cb;
    }
    // rows r0 .. r0 + 63 of `base` (row stride row_elems) into the image at LDS byte address lds_tile
    __device__ __forceinline__ void fill(unsigned lds_tile, const u16* base, long long row_elems, int r0, int rows,
                                         int wave) const {
        const u16* src = base + (long long)r0 * row_elems;
        if (r0 + kBK <= rows) {
#pragma unroll
            for (int n = 0; n < 4; n++) dtl_load(lds_tile + (4 * n + wave) * 1024, voff, src + 16 * n * row_elems);
        } else {
#pragma unroll
            for (int n = 0; n < 4; n++) {
                int r = 16 * n + lr;
                r = r < rows - r0 ? r : rows - 1 - r0;
                dtl_load(lds_tile + (4 * n + wave) * 1024, (unsigned)r * (unsigned)(row_elems * 2) + cb, src);
            }
        }
    }
};
// 64 floats src[r0 .. r0 + 63] (clamped to src[rows - 1]) to LDS byte address lds_row; one wave-wide load
__device__ __forceinline__ void fill_row(unsigned lds_row, const float* src, int r0, int rows, int lane) {
    const int r = lane < rows - r0 ? lane : rows - 1 - r0;
    dtl_load_dword(lds_row, (unsigned)r * 4u, src + r0);
}

// MFMA operand fragments of a tile image.  Every lane-dependent part of an
// address is computed once (constructor); inside the tile loops a read is that
// per-lane offset plus compile-time constants, i.e. no address arithmetic.
//   frag_rows: tile rows as MFMA rows (or columns), d as the k index: row
//       r0 + lane % 32, d = 16 * ks + 8 * (lane / 32) .. + 7; one 128-bit read.
//   frag_cols: d as the MFMA row (or column) index, tile rows as the k index:
//       d = 32 * db + lane % 32 and the eight tile rows r16 + 4 * half + 0..3 and
//       + 8 (half = lane / 32) -- the row order an accumulator block holds, so
//       that probabilities / score gradients go from accumulators straight into
//       the other operand; two transposing 64-bit reads.
struct FragOffsets {
    unsigned rows[8];
    unsigned cols_lo[4], cols_hi[4];
    // row_bias (a multiple of 16): tile rows are counted from there, for a wave that owns part of every tile
    __device__ __forceinline__ explicit FragOffsets(int lane, int row_bias = 0) {
        const int i = lane & 15, half = lane >> 5;
#pragma unroll
        for (int ks = 0; ks < 8; ks++) rows[ks] = slot(lane & 31, ks * 2 + half) + row_bias * 256;
#pragma unroll
        for (int db = 0; db < 4; db++) {
            // a group of 16 lanes reads 4 tile rows (i >> 2) x 16 d; lane i receives d column i
            const int d = db * 32 + ((lane >> 4) & 1) * 16 + (i & 3) * 4;
            const int ja = half * 4 + (i >> 2);
            cols_lo[db] = slot(ja, d >> 3) + (d & 7) * 2 + row_bias * 256;
            cols_hi[db] = slot(ja + 8, d >> 3) + (d & 7) * 2 + row_bias * 256;
        }
    }
    // rows r0 .. r0 + 31 (r0 a multiple of 32) of the tile at byte offset `tile`
    __device__ __forceinline__ u32x4 frag_rows(const lds_byte* lds, int tile, int r0, int ks) const {
        return *reinterpret_cast<const __attribute__((address_space(3))) u32x4*>(lds + rows[ks] + (tile + r0 * 256));
    }
    // r16 a multiple of 16
    __device__ __forceinline__ u32x4 frag_cols(const lds_byte* lds, int tile, int db, int r16) const {
        typedef __attribute__((address_space(3))) s16x4 lds_s16x4;
        const s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4*)(lds + cols_lo[db] + (tile + r16 * 256)));
        const s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4*)(lds + cols_hi[db] + (tile + r16 * 256)));
        const u32x2 l2 = __builtin_bit_cast(u32x2, lo), h2 = __builtin_bit_cast(u32x2, hi);
        return mk4(l2.x, l2.y, h2.x, h2.y);
    }
};

// Makes the compiler finish the global loads behind `x` here: it places its own s_waitcnt vmcnt in front of a load's
// first use, and a first use inside the tile loop would sit behind the direct-to-LDS loads issued at the top of the
// step (which the compiler does not count) -- the wave would wait for the NEXT tile in the middle of this one.
template <typename T>
__device__ __forceinline__ void landed(T& x) { asm volatile("" : "+v"(x)); }

// Row index (within a 32-row accumulator block) of accumulator element v.
__device__ __forceinline__ int acc_row(int v, int lane) { return (v >> 2) * 8 + (lane >> 5) * 4 + (v & 3); }

__device__ __forceinline__ float xor32(float x) { return __shfl_xor(x, 32, kWave); }

template <int CT>
__device__ __forceinline__ u32x4 pack8(const float* p) {
    return mk4(pack2(Cvt<CT>::from_f32(p[0]), Cvt<CT>::from_f32(p[1])), pack2(Cvt<CT>::from_f32(p[2]), Cvt<CT>::from_f32(p[3])),
               pack2(Cvt<CT>::from_f32(p[4]), Cvt<CT>::from_f32(p[5])), pack2(Cvt<CT>::from_f32(p[6]), Cvt<CT>::from_f32(p[7])));
}

// Number of keys a block of queries ending at q_end (exclusive) can see.
__device__ __forceinline__ int visible_keys(int q_end, int valid, int tokens) {
    if (valid <= 0) return tokens;  // every score is -FLT_MAX: uniform over all keys, as the unfused chain gives
    int n = q_end < tokens ? q_end : tokens;
    return n < valid ? n : valid;
}

// Masked, biased score of (query, key) from the raw dot product.
__device__ __forceinline__ float score(float dot, float scale, float bias, int query, int key, int valid, int tokens) {
    float x = dot * scale;
    x += bias;
    x += (key <= query && key < valid) ? 0.0f : -FLT_MAX;
    return key < tokens ? x : -INFINITY;  // tile overhang: not a key at all
}

// One LDS stage of the key loop: a K tile, a V tile and the tile's ALiBi row.
constexpr int kTileBytes = kBK * kHD * 2;
constexpr int kStageBytes = 2 * kTileBytes + kBK * 4;

// (G, KH) = (4, 1): four waves, each with 32 queries and every key of a tile; 128 queries per workgroup.
// (G, KH) = (2, 2): 64 queries per workgroup; wave (qg, kh) has the queries of group qg = wave % 2 and keys
// 32 * kh .. + 31 of every tile, with its own running maximum, sum and context; the two halves of a query group are
// merged through LDS at the end (the usual rescaling of two partial softmax sums).  Twice the workgroups, half the
// work per wave and tile: for launches whose 128-query workgroups would leave compute units empty (one sequence of
// 512 tokens and 32 heads: 128 of them), where a workgroup's walk over its key tiles is the whole kernel time.
template <int CT, int G, int KH>
__global__ __launch_bounds__(64 * G * KH, 2) void flash_fwd_kernel(FlashArgs a) {
    static_assert(G * KH == 4, "TileFill deals a tile to four waves");
    constexpr int BQ = 32 * G;         // queries per workgroup
    constexpr int NKB = 2 / KH;        // 32-key blocks of a tile per wave
    constexpr int kSpan = kBK / KH;    // keys of a tile per wave
    __shared__ __attribute__((aligned(1024))) unsigned char lds[2 * kStageBytes];
    static_assert(KH == 1 || 2 * kStageBytes >= G * (64 * 64 + 2 * 64) * 4, "the merge puts G contexts of 64 x 64 floats, their m and l into the stages");
    const int lane = threadIdx.x & 63, half = lane >> 5;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);  // wave-uniform: branches on it are scalar
    const int qg = KH == 1 ? wave : wave % G, kh = KH == 1 ? 0 : wave / G;
    // workgroups are numbered longest first: the query tiles with the most
    // visible keys of every (batch, head), then the next ones, ...
    const int tiles_q = (a.tokens + BQ - 1) / BQ;
    const int bh = (int)(blockIdx.x % a.batch_heads), b = bh / a.heads, h = bh % a.heads;
    const int qt = tiles_q - 1 - (int)(blockIdx.x / a.batch_heads);
    const long long base = (long long)b * a.batch_stride + (long long)h * a.head;
    const int valid = a.valid[b] < a.tokens ? a.valid[b] : a.tokens;
    const int q0 = qt * BQ + qg * 32;
    const int query = q0 + (lane & 31);
    const int qrow = query < a.tokens ? query : a.tokens - 1;
    const float* alibi_row = a.alibi + (long long)h * a.tokens;

    u32x4 qf[8];
#pragma unroll
    for (int ks = 0; ks < 8; ks++)
        qf[ks] = *reinterpret_cast<const u32x4*>(a.q + base + (long long)qrow * a.row + ks * 16 + half * 8);

    f32x16 o[4];
#pragma unroll
    for (int db = 0; db < 4; db++)
#pragma unroll
        for (int v = 0; v < 16; v++) o[db][v] = 0.f;
    float m = -INFINITY, l = 0.f;

    const int nkeys = visible_keys(qt * BQ + BQ, valid, a.tokens);
    const int ntiles = (nkeys + kBK - 1) / kBK;
    // keys this wave's queries can see (a wave may idle through the last tiles)
    const int wave_keys = visible_keys(q0 + 32, valid, a.tokens);

    const FragOffsets fo(lane, kh * 32);
    const lds_byte* ldsb = (const lds_byte*)lds;
    // Key tile t goes straight from global memory into stage t % 2 (K image, V image, the tile's ALiBi row): issued
    // at the start of step t - 1, when the barrier that ended step t - 2 has freed the stage, and waited for at the
    // end of step t - 1.  Every wave issues its quarter of the images and waits for its own loads before the barrier.
    const unsigned lds0 = (unsigned)(unsigned long long)ldsb;
    const TileFill kv_fill(lane, wave, a.row);
    auto issue = [&](int t, unsigned stage_bytes) {
        const unsigned st = lds0 + stage_bytes;
        kv_fill.fill(st, a.k + base, a.row, t * kBK, a.tokens, wave);
        kv_fill.fill(st + kTileBytes, a.v + base, a.row, t * kBK, a.tokens, wave);
        fill_row(st + 2 * kTileBytes, alibi_row, t * kBK, a.tokens, lane);
    };
#pragma unroll
    for (int ks = 0; ks < 8; ks++) landed(qf[ks]);
    issue(0, 0);
    wait_vmem<0>();
    __syncthreads();
    // one key tile; the stage is a compile-time constant so that every LDS
    // address is a per-lane offset computed once plus an immediate
    auto tile_step = [&](auto stage_c, int t) {
        constexpr int kStage = decltype(stage_c)::value * kStageBytes;
        const int k0 = t * kBK + kh * 32;   // this wave's first key of the tile
        if (t + 1 < ntiles) issue(t + 1, kStageBytes - kStage);
        if (k0 < wave_keys) {
            f32x16 s[NKB];
#pragma unroll
            for (int kb = 0; kb < NKB; kb++) {
#pragma unroll
                for (int v = 0; v < 16; v++) s[kb][v] = 0.f;
#pragma unroll
                for (int ks = 0; ks < 8; ks++)
                    s[kb] = Cvt<CT>::mfma(fo.frag_rows(ldsb, kStage, kb * 32, ks), qf[ks], s[kb]);
            }
            const float* tb = reinterpret_cast<const float*>(lds + kStage + 2 * kTileBytes) + kh * 32 + half * 4;
            float mt = -INFINITY;
            // keys wholly below the diagonal and inside the sequence need no mask
            if (k0 + kSpan - 1 <= q0 && k0 + kSpan <= valid) {
#pragma unroll
                for (int kb = 0; kb < NKB; kb++)
#pragma unroll
                    for (int g = 0; g < 4; g++) {
                        const float4 bv = *reinterpret_cast<const float4*>(tb + kb * 32 + g * 8);
                        const float bb[4] = {bv.x, bv.y, bv.z, bv.w};
#pragma unroll
                        for (int j = 0; j < 4; j++) {
                            float x = s[kb][g * 4 + j] * a.scale;
                            x += bb[j];
                            s[kb][g * 4 + j] = x;
                            mt = fmaxf(mt, x);
                        }
                    }
            } else {
#pragma unroll
                for (int kb = 0; kb < NKB; kb++)
#pragma unroll
                    for (int g = 0; g < 4; g++) {
                        const float4 bv = *reinterpret_cast<const float4*>(tb + kb * 32 + g * 8);
                        const float bb[4] = {bv.x, bv.y, bv.z, bv.w};
                        const int key = k0 + kb * 32 + g * 8 + half * 4;
#pragma unroll
                        for (int j = 0; j < 4; j++) {
                            const float x = score(s[kb][g * 4 + j], a.scale, bb[j], query, key + j, valid, a.tokens);
                            s[kb][g * 4 + j] = x;
                            mt = fmaxf(mt, x);
                        }
                    }
            }
            mt = fmaxf(mt, xor32(mt));
            const float m_new = fmaxf(m, mt);
            const float alpha = __expf(m - m_new);
            float sum = 0.f;
#pragma unroll
            for (int kb = 0; kb < NKB; kb++)
#pragma unroll
                for (int v = 0; v < 16; v++) {
                    const float p = __expf(s[kb][v] - m_new);
                    s[kb][v] = p;
                    sum += p;
                }
            sum += xor32(sum);
            l = l * alpha + sum;
            m = m_new;
            u32x4 pf[2 * NKB];
#pragma unroll
            for (int j = 0; j < 2 * NKB; j++) {
                const int kb = j >> 1, vb = (j & 1) * 8;
                float p8[8];
#pragma unroll
                for (int e = 0; e < 8; e++) p8[e] = s[kb][vb + e];
                pf[j] = pack8<CT>(p8);
            }
#pragma unroll
            for (int db = 0; db < 4; db++)
#pragma unroll
                for (int v = 0; v < 16; v++) o[db][v] *= alpha;
#pragma unroll
            for (int j = 0; j < 2 * NKB; j++)
#pragma unroll
                for (int db = 0; db < 4; db++)
                    o[db] = Cvt<CT>::mfma(fo.frag_cols(ldsb, kStage + kTileBytes, db, (j >> 1) * 32 + (j & 1) * 16), pf[j], o[db]);
        }
        wait_vmem<0>();   // this wave's part of tile t + 1 is in
        __syncthreads();
    };
    for (int t = 0; t < ntiles; t += 2) {
        tile_step(std::integral_constant<int, 0>(), t);
        if (t + 1 < ntiles) tile_step(std::integral_constant<int, 1>(), t + 1);
    }

    if (KH == 2) {
        // Merge the two key halves of each query group: the waves with the odd halves leave m, l and their context
        // in LDS (every wave is past the loop's last barrier: the stages are free), the others rescale both to the
        // common maximum.  A half that met no key has m = -inf, l = 0 and weighs nothing; key 0 is in the even half
        // and visible to every query of a non-empty sequence, so the common maximum is never -inf.
        float* const xo = reinterpret_cast<float*>(lds) + qg * (64 * 64);
        float* const xml = reinterpret_cast<float*>(lds) + G * 64 * 64 + qg * 128;
        if (kh == 1) {
#pragma unroll
            for (int db = 0; db < 4; db++)
#pragma unroll
                for (int v = 0; v < 16; v++) xo[(db * 16 + v) * 64 + lane] = o[db][v];
            xml[lane] = m;
            xml[64 + lane] = l;
        }
        __syncthreads();
        if (kh == 1) return;
        const float m1 = xml[lane], l1 = xml[64 + lane];
        const float m_all = fmaxf(m, m1);
        const float w0 = __expf(m - m_all), w1 = __expf(m1 - m_all);
        l = l * w0 + l1 * w1;
        m = m_all;
#pragma unroll
        for (int db = 0; db < 4; db++)
#pragma unroll
            for (int v = 0; v < 16; v++) o[db][v] = o[db][v] * w0 + xo[(db * 16 + v) * 64 + lane] * w1;
    }

    if (query < a.tokens) {
        const float inv = 1.0f / l;
        u16* orow = a.o + (long long)b * a.obatch + (long long)h * a.head + (long long)query * a.orow;
#pragma unroll
        for (int db = 0; db < 4; db++)
#pragma unroll
            for (int g = 0; g < 4; g++) {
                const int d = db * 32 + g * 8 + half * 4;
                const unsigned lo = pack2(Cvt<CT>::from_f32(o[db][g * 4 + 0] * inv), Cvt<CT>::from_f32(o[db][g * 4 + 1] * inv));
                const unsigned hi = pack2(Cvt<CT>::from_f32(o[db][g * 4 + 2] * inv), Cvt<CT>::from_f32(o[db][g * 4 + 3] * inv));
                *reinterpret_cast<uint2*>(orow + d) = make_uint2(lo, hi);
            }
        if (half == 0) a.lse[(long long)bh * a.tokens + query] = m + __logf(l);
    }
}

// ------------------------------------------------------------------ backward
template <int CT>
__device__ __forceinline__ float to_f32(u16 x);
template <>
__device__ __forceinline__ float to_f32<BR_GEMM_F16>(u16 x) { return (float)__builtin_bit_cast(_Float16, x); }
template <>
__device__ __forceinline__ float to_f32<BR_GEMM_BF16>(u16 x) { return __uint_as_float((unsigned)x << 16); }

// One LDS stage of the query loop of the dK / dV pass: a Q tile, a dO tile and
// the tile's lse and delta values.
constexpr int kQStageBytes = 2 * kTileBytes + 2 * kBK * 4;

// dK, dV of 128 keys (32 per wave) of one (batch, head): queries stream through
// LDS in tiles of 64.  Per wave and 32-query block:
//   S[query, key]  = Q . K^T        (A = Q rows from LDS, B = K in registers)
//   dP[query, key] = dO . V^T       (A = dO rows from LDS, B = V in registers)
//   P = exp(score - lse),  dS = P o (dP - delta)
//   dV[key, d] += P^T . dO,  dK[key, d] += dS^T . Q   (A from the accumulators,
//                                    B by transposing reads of the same tiles)
// (G, QH) = (4, 1): 128 keys per workgroup, 32 per wave, every query of a tile.  (2, 2): 64 keys per workgroup; wave
// (kg, qh) has the keys of group kg = wave % 2 and queries 32 * qh .. + 31 of every query tile; the two partial dK
// and dV of a key group are added through LDS at the end.
template <int CT, int G, int QH>
__global__ __launch_bounds__(64 * G * QH) void flash_bwd_dkv_kernel(FlashArgs a) {
    static_assert(G * QH == 4, "TileFill deals a tile to four waves");
    constexpr int BKEYS = 32 * G;      // keys per workgroup
    constexpr int NQB = 2 / QH;        // 32-query blocks of a tile per wave
    constexpr int kSpan = kBK / QH;    // queries of a tile per wave
    __shared__ __attribute__((aligned(1024))) unsigned char lds[2 * kQStageBytes];
    static_assert(2 * kQStageBytes >= G * 64 * 64 * 4, "the merge puts G blocks of 64 x 64 floats into the stages");
    const int lane = threadIdx.x & 63, half = lane >> 5;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);  // wave-uniform: branches on it are scalar
    const int kg = QH == 1 ? wave : wave % G, qh = QH == 1 ? 0 : wave / G;
    const int bh = (int)(blockIdx.x % a.batch_heads), b = bh / a.heads, h = bh % a.heads;
    const int kt = (int)(blockIdx.x / a.batch_heads);  // key tile 0 meets the most queries: longest first
    const long long base = (long long)b * a.batch_stride + (long long)h * a.head;
    const long long obase = (long long)b * a.obatch + (long long)h * a.head;
    const int valid = a.valid[b] < a.tokens ? a.valid[b] : a.tokens;
    const int key0 = kt * BKEYS + kg * 32;
    const int key = key0 + (lane & 31);
    const int krow = key < a.tokens ? key : a.tokens - 1;
    float bias = a.alibi[(long long)h * a.tokens + krow];
    const float uniform = 1.0f / (float)a.tokens;

    u32x4 kf[8], vf[8];
#pragma unroll
    for (int ks = 0; ks < 8; ks++) {
        kf[ks] = *reinterpret_cast<const u32x4*>(a.k + base + (long long)krow * a.row + ks * 16 + half * 8);
        vf[ks] = *reinterpret_cast<const u32x4*>(a.v + base + (long long)krow * a.row + ks * 16 + half * 8);
    }
    f32x16 dk[4], dv[4];
#pragma unroll
    for (int db = 0; db < 4; db++)
#pragma unroll
        for (int v = 0; v < 16; v++) dk[db][v] = dv[db][v] = 0.f;

    // queries that can see any key of this workgroup start at its first key
    // (none at all when the keys lie in the padding); an empty sequence has
    // uniform probabilities everywhere, so nothing is skipped for it
    const bool dead_group = valid > 0 && kt * BKEYS >= valid;
    const int q_begin = valid > 0 ? (kt * BKEYS / kBK) * kBK : 0;
    const int ntiles = dead_group ? 0 : (a.tokens - q_begin + kBK - 1) / kBK;
    const bool dead_wave = valid > 0 && key0 >= valid;

    const FragOffsets fo(lane, qh * 32);
    const lds_byte* ldsb = (const lds_byte*)lds;
    // query tile t (Q image, dO image, the tile's lse and delta rows) goes straight into stage t % 2, as the key
    // tiles of the forward kernel do
    const unsigned lds0 = (unsigned)(unsigned long long)ldsb;
    const TileFill q_fill(lane, wave, a.row), g_fill(lane, wave, a.orow);
    auto issue = [&](int t, unsigned stage_bytes) {
        const unsigned st = lds0 + stage_bytes;
        const int r0 = q_begin + t * kBK;
        q_fill.fill(st, a.q + base, a.row, r0, a.tokens, wave);
        g_fill.fill(st + kTileBytes, a.d_o + obase, a.orow, r0, a.tokens, wave);
        fill_row(st + 2 * kTileBytes, a.lse + (long long)bh * a.tokens, r0, a.tokens, lane);
        fill_row(st + 2 * kTileBytes + kBK * 4, a.delta + (long long)bh * a.tokens, r0, a.tokens, lane);
    };
#pragma unroll
    for (int ks = 0; ks < 8; ks++) {
        landed(kf[ks]);
        landed(vf[ks]);
    }
    landed(bias);
    if (ntiles > 0) issue(0, 0);
    wait_vmem<0>();
    __syncthreads();
    auto tile_step = [&](auto stage_c, int t) {
        constexpr int kStage = decltype(stage_c)::value * kQStageBytes;
        const int q0 = q_begin + t * kBK + qh * 32;   // this wave's first query of the tile
        if (t + 1 < ntiles) issue(t + 1, kQStageBytes - kStage);
        const float* tl = reinterpret_cast<const float*>(lds + kStage + 2 * kTileBytes) + qh * 32 + half * 4;
        const float* td = tl + kBK;
        // queries that all precede this wave's keys see none of them
        if (!dead_wave && !(valid > 0 && q0 + kSpan - 1 < key0)) {
            const bool open = q0 >= key0 + 31 && key0 + 32 <= valid && q0 + kSpan <= a.tokens;
#pragma unroll
            for (int qb = 0; qb < NQB; qb++) {
                f32x16 s, dp;
#pragma unroll
                for (int v = 0; v < 16; v++) s[v] = dp[v] = 0.f;
#pragma unroll
                for (int ks = 0; ks < 8; ks++) {
                    s = Cvt<CT>::mfma(fo.frag_rows(ldsb, kStage, qb * 32, ks), kf[ks], s);
                    dp = Cvt<CT>::mfma(fo.frag_rows(ldsb, kStage + kTileBytes, qb * 32, ks), vf[ks], dp);
                }
                if (open) {
#pragma unroll
                    for (int g = 0; g < 4; g++) {
                        const float4 l4 = *reinterpret_cast<const float4*>(tl + qb * 32 + g * 8);
                        const float4 d4 = *reinterpret_cast<const float4*>(td + qb * 32 + g * 8);
                        const float ll[4] = {l4.x, l4.y, l4.z, l4.w}, dd[4] = {d4.x, d4.y, d4.z, d4.w};
#pragma unroll
                        for (int j = 0; j < 4; j++) {
                            float x = s[g * 4 + j] * a.scale;
                            x += bias;
                            const float p = __expf(x - ll[j]);
                            s[g * 4 + j] = p;
                            dp[g * 4 + j] = p * (dp[g * 4 + j] - dd[j]);
                        }
                    }
                } else {
#pragma unroll
                    for (int g = 0; g < 4; g++) {
                        const float4 l4 = *reinterpret_cast<const float4*>(tl + qb * 32 + g * 8);
                        const float4 d4 = *reinterpret_cast<const float4*>(td + qb * 32 + g * 8);
                        const float ll[4] = {l4.x, l4.y, l4.z, l4.w}, dd[4] = {d4.x, d4.y, d4.z, d4.w};
#pragma unroll
                        for (int j = 0; j < 4; j++) {
                            const int query = q0 + qb * 32 + g * 8 + half * 4 + j;
                            const float x = score(s[g * 4 + j], a.scale, bias, query, key, valid, a.tokens);
                            float p = valid > 0 ? __expf(x - ll[j]) : uniform;
                            p = (query < a.tokens && key < a.tokens) ? p : 0.f;
                            s[g * 4 + j] = p;
                            dp[g * 4 + j] = p * (dp[g * 4 + j] - dd[j]);
                        }
                    }
                }
#pragma unroll
                for (int j = 0; j < 2; j++) {
                    float p8[8], s8[8];
#pragma unroll
                    for (int e = 0; e < 8; e++) {
                        p8[e] = s[j * 8 + e];
                        s8[e] = dp[j * 8 + e];
                    }
                    const u32x4 pf = pack8<CT>(p8), sf = pack8<CT>(s8);
#pragma unroll
                    for (int db = 0; db < 4; db++) {
                        dv[db] = Cvt<CT>::mfma(pf, fo.frag_cols(ldsb, kStage + kTileBytes, db, qb * 32 + j * 16), dv[db]);
                        dk[db] = Cvt<CT>::mfma(sf, fo.frag_cols(ldsb, kStage, db, qb * 32 + j * 16), dk[db]);
                    }
                }
            }
        }
        wait_vmem<0>();   // this wave's part of tile t + 1 is in
        __syncthreads();
    };
    for (int t = 0; t < ntiles; t += 2) {
        tile_step(std::integral_constant<int, 0>(), t);
        if (t + 1 < ntiles) tile_step(std::integral_constant<int, 1>(), t + 1);
    }

    if (QH == 2) {
        // the waves with the odd query halves hand their sums over, dK first, then dV (every wave is past the loop's
        // last barrier: the stages are free)
        float* const x = reinterpret_cast<float*>(lds) + kg * (64 * 64);
        if (qh == 1) {
#pragma unroll
            for (int db = 0; db < 4; db++)
#pragma unroll
                for (int v = 0; v < 16; v++) x[(db * 16 + v) * 64 + lane] = dk[db][v];
        }
        __syncthreads();
        if (qh == 0) {
#pragma unroll
            for (int db = 0; db < 4; db++)
#pragma unroll
                for (int v = 0; v < 16; v++) dk[db][v] += x[(db * 16 + v) * 64 + lane];
        }
        __syncthreads();
        if (qh == 1) {
#pragma unroll
            for (int db = 0; db < 4; db++)
#pragma unroll
                for (int v = 0; v < 16; v++) x[(db * 16 + v) * 64 + lane] = dv[db][v];
        }
        __syncthreads();
        if (qh == 1) return;
#pragma unroll
        for (int db = 0; db < 4; db++)
#pragma unroll
            for (int v = 0; v < 16; v++) dv[db][v] += x[(db * 16 + v) * 64 + lane];
    }

    // accumulator element v of block db: key key0 + acc_row(v), d = 32 * db + lane % 32
#pragma unroll
    for (int v = 0; v < 16; v++) {
        const int kk = key0 + acc_row(v, lane);
        if (kk < a.tokens) {
            const long long off = base + (long long)kk * a.row + (lane & 31);
#pragma unroll
            for (int db = 0; db < 4; db++) {
                if (a.grad16) {
                    static_cast<u16*>(a.dk)[off + db * 32] = Cvt<CT>::from_f32(dk[db][v] * a.scale);
                    static_cast<u16*>(a.dv)[off + db * 32] = Cvt<CT>::from_f32(dv[db][v]);
                } else {
                    static_cast<float*>(a.dk)[off + db * 32] = dk[db][v] * a.scale;
                    static_cast<float*>(a.dv)[off + db * 32] = dv[db][v];
                }
            }
        }
    }
}

// dQ of 128 queries (32 per wave) of one (batch, head): the forward's loop over
// key tiles, with  S^T = K . Q^T,  dP^T = V . dO^T  and
// dQ^T[d, query] += K^T . dS^T  (K^T by transposing reads of the K tile).
// (G, KH) = (2, 2): 64 queries per workgroup, the keys of every tile split between two waves as in the forward
// kernel; the two partial dQ of a query group are added through LDS at the end.
template <int CT, int G, int KH>
__global__ __launch_bounds__(64 * G * KH, 2) void flash_bwd_dq_kernel(FlashArgs a) {
    static_assert(G * KH == 4, "TileFill deals a tile to four waves");
    constexpr int BQ = 32 * G;
    constexpr int NKB = 2 / KH;
    constexpr int kSpan = kBK / KH;
    __shared__ __attribute__((aligned(1024))) unsigned char lds[2 * kStageBytes];
    static_assert(2 * kStageBytes >= G * 64 * 64 * 4, "the merge puts G blocks of 64 x 64 floats into the stages");
    const int lane = threadIdx.x & 63, half = lane >> 5;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);  // wave-uniform: branches on it are scalar
    const int qg = KH == 1 ? wave : wave % G, kh = KH == 1 ? 0 : wave / G;
    const int tiles_q = (a.tokens + BQ - 1) / BQ;
    const int bh = (int)(blockIdx.x % a.batch_heads), b = bh / a.heads, h = bh % a.heads;
    const int qt = tiles_q - 1 - (int)(blockIdx.x / a.batch_heads);
    const long long base = (long long)b * a.batch_stride + (long long)h * a.head;
    const int valid = a.valid[b] < a.tokens ? a.valid[b] : a.tokens;
    const int q0 = qt * BQ + qg * 32;
    const int query = q0 + (lane & 31);
    const int qrow = query < a.tokens ? query : a.tokens - 1;
    const float* alibi_row = a.alibi + (long long)h * a.tokens;
    float lse = a.lse[(long long)bh * a.tokens + qrow];
    const float uniform = 1.0f / (float)a.tokens;

    // The query's dO fragments, and on the way delta[query] = sum_d dO[query, d] * O[query, d]: the two halves of a
    // wave hold the two halves of every 16-wide slice of the row.  The dK / dV pass, which runs after this one,
    // reads the value from a.delta.
    u32x4 qf[8], gf[8];
    const long long orow = (long long)b * a.obatch + (long long)h * a.head + (long long)qrow * a.orow;
    float delta = 0.f;
#pragma unroll
    for (int ks = 0; ks < 8; ks++) {
        gf[ks] = *reinterpret_cast<const u32x4*>(a.d_o + orow + ks * 16 + half * 8);
        const u32x4 y = *reinterpret_cast<const u32x4*>(a.o + orow + ks * 16 + half * 8);
#pragma unroll
        for (int j = 0; j < 4; j++) {
            delta += to_f32<CT>((u16)(gf[ks][j] & 0xffffu)) * to_f32<CT>((u16)(y[j] & 0xffffu));
            delta += to_f32<CT>((u16)(gf[ks][j] >> 16)) * to_f32<CT>((u16)(y[j] >> 16));
        }
    }
    delta += __shfl_xor(delta, 32, kWave);
    if (half == 0 && kh == 0 && query < a.tokens) a.delta[(long long)bh * a.tokens + query] = delta;
#pragma unroll
    for (int ks = 0; ks < 8; ks++)
        qf[ks] = *reinterpret_cast<const u32x4*>(a.q + base + (long long)qrow * a.row + ks * 16 + half * 8);
    f32x16 dq[4];
#pragma unroll
    for (int db = 0; db < 4; db++)
#pragma unroll
        for (int v = 0; v < 16; v++) dq[db][v] = 0.f;

    const int nkeys = visible_keys(qt * BQ + BQ, valid, a.tokens);
    const int ntiles = (nkeys + kBK - 1) / kBK;
    const int wave_keys = visible_keys(q0 + 32, valid, a.tokens);

    const FragOffsets fo(lane, kh * 32);
    const lds_byte* ldsb = (const lds_byte*)lds;
    // Key tile t goes straight from global memory into stage t % 2 (K image, V image, the tile's ALiBi row): issued
    // at the start of step t - 1, when the barrier that ended step t - 2 has freed the stage, and waited for at the
    // end of step t - 1.  Every wave issues its quarter of the images and waits for its own loads before the barrier.
    const unsigned lds0 = (unsigned)(unsigned long long)ldsb;
    const TileFill kv_fill(lane, wave, a.row);
    auto issue = [&](int t, unsigned stage_bytes) {
        const unsigned st = lds0 + stage_bytes;
        kv_fill.fill(st, a.k + base, a.row, t * kBK, a.tokens, wave);
        kv_fill.fill(st + kTileBytes, a.v + base, a.row, t * kBK, a.tokens, wave);
        fill_row(st + 2 * kTileBytes, alibi_row, t * kBK, a.tokens, lane);
    };
#pragma unroll
    for (int ks = 0; ks < 8; ks++) {
        landed(qf[ks]);
        landed(gf[ks]);
    }
    landed(lse);
    issue(0, 0);
    wait_vmem<0>();
    __syncthreads();
    auto tile_step = [&](auto stage_c, int t) {
        constexpr int kStage = decltype(stage_c)::value * kStageBytes;
        const int k0 = t * kBK + kh * 32;   // this wave's first key of the tile
        if (t + 1 < ntiles) issue(t + 1, kStageBytes - kStage);
        const float* tb = reinterpret_cast<const float*>(lds + kStage + 2 * kTileBytes) + kh * 32 + half * 4;
        if (k0 < wave_keys) {
            const bool open = k0 + kSpan - 1 <= q0 && k0 + kSpan <= valid;
#pragma unroll
            for (int kb = 0; kb < NKB; kb++) {
                f32x16 s, dp;
#pragma unroll
                for (int v = 0; v < 16; v++) s[v] = dp[v] = 0.f;
#pragma unroll
                for (int ks = 0; ks < 8; ks++) {
                    s = Cvt<CT>::mfma(fo.frag_rows(ldsb, kStage, kb * 32, ks), qf[ks], s);
                    dp = Cvt<CT>::mfma(fo.frag_rows(ldsb, kStage + kTileBytes, kb * 32, ks), gf[ks], dp);
                }
                if (open) {
#pragma unroll
                    for (int g = 0; g < 4; g++) {
                        const float4 bv = *reinterpret_cast<const float4*>(tb + kb * 32 + g * 8);
                        const float bb[4] = {bv.x, bv.y, bv.z, bv.w};
#pragma unroll
                        for (int j = 0; j < 4; j++) {
                            float x = s[g * 4 + j] * a.scale;
                            x += bb[j];
                            dp[g * 4 + j] = __expf(x - lse) * (dp[g * 4 + j] - delta);
                        }
                    }
                } else {
#pragma unroll
                    for (int g = 0; g < 4; g++) {
                        const float4 bv = *reinterpret_cast<const float4*>(tb + kb * 32 + g * 8);
                        const float bb[4] = {bv.x, bv.y, bv.z, bv.w};
                        const int key = k0 + kb * 32 + g * 8 + half * 4;
#pragma unroll
                        for (int j = 0; j < 4; j++) {
                            const float x = score(s[g * 4 + j], a.scale, bb[j], query, key + j, valid, a.tokens);
                            float p = valid > 0 ? __expf(x - lse) : uniform;
                            p = key + j < a.tokens ? p : 0.f;
                            dp[g * 4 + j] = p * (dp[g * 4 + j] - delta);
                        }
                    }
                }
#pragma unroll
                for (int j = 0; j < 2; j++) {
                    float s8[8];
#pragma unroll
                    for (int e = 0; e < 8; e++) s8[e] = dp[j * 8 + e];
                    const u32x4 sf = pack8<CT>(s8);
#pragma unroll
                    for (int db = 0; db < 4; db++)
                        dq[db] = Cvt<CT>::mfma(fo.frag_cols(ldsb, kStage, db, kb * 32 + j * 16), sf, dq[db]);
                }
            }
        }
        wait_vmem<0>();   // this wave's part of tile t + 1 is in
        __syncthreads();
    };
    for (int t = 0; t < ntiles; t += 2) {
        tile_step(std::integral_constant<int, 0>(), t);
        if (t + 1 < ntiles) tile_step(std::integral_constant<int, 1>(), t + 1);
    }

    if (KH == 2) {
        float* const x = reinterpret_cast<float*>(lds) + qg * (64 * 64);
        if (kh == 1) {
#pragma unroll
            for (int db = 0; db < 4; db++)
#pragma unroll
                for (int v = 0; v < 16; v++) x[(db * 16 + v) * 64 + lane] = dq[db][v];
        }
        __syncthreads();
        if (kh == 1) return;
#pragma unroll
        for (int db = 0; db < 4; db++)
#pragma unroll
            for (int v = 0; v < 16; v++) dq[db][v] += x[(db * 16 + v) * 64 + lane];
    }

    if (query < a.tokens && !a.grad16) {
        float* row = static_cast<float*>(a.dq) + base + (long long)query * a.row;
#pragma unroll
        for (int db = 0; db < 4; db++)
#pragma unroll
            for (int g = 0; g < 4; g++)
                *reinterpret_cast<float4*>(row + db * 32 + g * 8 + half * 4) =
                    make_float4(dq[db][g * 4 + 0] * a.scale, dq[db][g * 4 + 1] * a.scale, dq[db][g * 4 + 2] * a.scale,
                                dq[db][g * 4 + 3] * a.scale);
    } else if (query < a.tokens) {
        u16* row = static_cast<u16*>(a.dq) + base + (long long)query * a.row;
#pragma unroll
        for (int db = 0; db < 4; db++)
#pragma unroll
            for (int g = 0; g < 4; g++) {
                const unsigned lo = (unsigned)Cvt<CT>::from_f32(dq[db][g * 4 + 0] * a.scale) |
                                    ((unsigned)Cvt<CT>::from_f32(dq[db][g * 4 + 1] * a.scale) << 16);
                const unsigned hi = (unsigned)Cvt<CT>::from_f32(dq[db][g * 4 + 2] * a.scale) |
                                    ((unsigned)Cvt<CT>::from_f32(dq[db][g * 4 + 3] * a.scale) << 16);
                *reinterpret_cast<uint2*>(row + db * 32 + g * 8 + half * 4) = make_uint2(lo, hi);
            }
    }
}

// Whether a launch that would take `workgroups` workgroups of 128 queries (or keys) runs on twice as many of 64
// instead, each tile's work split between two waves: where the wider ones would leave compute units empty or with
// one workgroup each.  Measured at 32 heads x 512 tokens, batch 1 / 2 / 4 (128 / 256 / 512 wide workgroups), wide
// against narrow: forward 19.5 -> 14.2, 19.5 -> 17.9, 27.5 -> 31.7 us; dQ + dK/dV passes 56.0 -> 37.9 (both narrow),
// 59.4 -> 54.1 and 86.4 -> 90.3 (dQ narrow).  The dK / dV pass needs more than 256 registers either way (one
// workgroup per CU) and was measured narrow at batch 1 only.
#ifndef BR_FA_SPLIT_UP_TO
#define BR_FA_SPLIT_UP_TO 256
#endif
#ifndef BR_FA_DKV_SPLIT_BELOW
#define BR_FA_DKV_SPLIT_BELOW 256
#endif
inline bool narrow_split(unsigned workgroups) { return workgroups <= (unsigned)BR_FA_SPLIT_UP_TO; }
inline bool narrow_split_dkv(unsigned workgroups) { return workgroups < (unsigned)BR_FA_DKV_SPLIT_BELOW; }

bool flash_shape_ok(int64_t batch, int64_t heads, int64_t tokens, int64_t head_dim, int64_t row, int64_t head,
                    int64_t batch_stride, int64_t orow, int64_t obatch) {
    return batch > 0 && heads > 0 && tokens >= 1 && head_dim == kHD && row % 8 == 0 &&
           head % 8 == 0 && batch_stride % 8 == 0 && orow % 8 == 0 && obatch % 8 == 0 && batch * heads <= (1 << 20) && tokens <= (1 << 20) &&
           row < (1 << 24) && orow < (1 << 24);   // 64 rows of a tile within a 32-bit byte offset
}

}  // namespace

extern "C" {

int br_hip_flash_attn_fwd(const void* q, const void* k, const void* v, int dtype, const float* alibi,
                          const int32_t* valid, void* o, float* lse, int64_t batch, int64_t heads, int64_t tokens,
                          int64_t head_dim, int64_t row_stride, int64_t head_stride, int64_t batch_stride,
                          int64_t o_row_stride, int64_t o_batch_stride, br_stream_t stream) {
    if (batch < 0 || heads <= 0 || tokens <= 0 || head_dim <= 0) return BR_ERR_ATTR;
    if (batch == 0) return BR_OK;
    if (!q || !k || !v || !alibi || !valid) return BR_ERR_INPUT;
    if (!o || !lse) return BR_ERR_OUTPUT;
    if ((dtype != BR_F16 && dtype != BR_BF16) ||
        !flash_shape_ok(batch, heads, tokens, head_dim, row_stride, head_stride, batch_stride, o_row_stride,
                        o_batch_stride) || !aligned16(q) ||
        !aligned16(k) || !aligned16(v) || !aligned16(o) || !aligned16(alibi))
        return BR_ERR_TODO;
    FlashArgs a = {};
    a.q = (const u16*)q;
    a.k = (const u16*)k;
    a.v = (const u16*)v;
    a.o = (u16*)o;
    a.alibi = alibi;
    a.valid = valid;
    a.lse = lse;
    a.row = row_stride;
    a.head = head_stride;
    a.batch_stride = batch_stride;
    a.orow = o_row_stride;
    a.obatch = o_batch_stride;
    a.heads = (int)heads;
    a.tokens = (int)tokens;
    a.batch_heads = (int)(batch * heads);
    a.scale = (float)(1.0 / sqrt((double)head_dim));
    const unsigned grid = (unsigned)(((tokens + kBQ - 1) / kBQ) * batch * heads);
    if (narrow_split(grid)) {
        const unsigned grid2 = (unsigned)(((tokens + 63) / 64) * batch * heads);
        if (dtype == BR_F16)
            flash_fwd_kernel<BR_GEMM_F16, 2, 2><<<grid2, kThreads, 0, as_stream(stream)>>>(a);
        else
            flash_fwd_kernel<BR_GEMM_BF16, 2, 2><<<grid2, kThreads, 0, as_stream(stream)>>>(a);
    } else {
        if (dtype == BR_F16)
            flash_fwd_kernel<BR_GEMM_F16, 4, 1><<<grid, kThreads, 0, as_stream(stream)>>>(a);
        else
            flash_fwd_kernel<BR_GEMM_BF16, 4, 1><<<grid, kThreads, 0, as_stream(stream)>>>(a);
    }
    BR_HIP_LAUNCH_CHECK();
    return BR_OK;
}

int br_hip_flash_attn_bwd(const void* q, const void* k, const void* v, const void* o, const void* d_o, int dtype,
                          const float* alibi, const int32_t* valid, const float* lse, float* delta, void* dq,
                          void* dk, void* dv, int grad_dtype, int64_t batch, int64_t heads, int64_t tokens,
                          int64_t head_dim,
                          int64_t row_stride, int64_t head_stride, int64_t batch_stride, int64_t o_row_stride,
                          int64_t o_batch_stride, br_stream_t stream) {
    if (batch < 0 || heads <= 0 || tokens <= 0 || head_dim <= 0) return BR_ERR_ATTR;
    if (batch == 0) return BR_OK;
    if (!q || !k || !v || !o || !d_o || !alibi || !valid || !lse) return BR_ERR_INPUT;
    if (!delta || !dq || !dk || !dv) return BR_ERR_OUTPUT;
    for (const void* out : {(const void*)dq, (const void*)dk, (const void*)dv})
        for (const void* in : {q, k, v, o, d_o})
            if (out == in) return BR_ERR_OUTPUT;   // both passes read every input
    if (grad_dtype != BR_F32 && grad_dtype != dtype) return BR_ERR_TODO;
    if ((dtype != BR_F16 && dtype != BR_BF16) ||
        !flash_shape_ok(batch, heads, tokens, head_dim, row_stride, head_stride, batch_stride, o_row_stride,
                        o_batch_stride) || !aligned16(q) ||
        !aligned16(k) || !aligned16(v) || !aligned16(o) || !aligned16(d_o) || !aligned16(alibi) || !aligned16(dq) ||
        !aligned16(dk) || !aligned16(dv))
        return BR_ERR_TODO;
    FlashArgs a = {};
    a.q = (const u16*)q;
    a.k = (const u16*)k;
    a.v = (const u16*)v;
    a.o = (u16*)const_cast<void*>(o);
    a.d_o = (const u16*)d_o;
    a.dq = dq;
    a.dk = dk;
    a.dv = dv;
    a.grad16 = grad_dtype != BR_F32;
    a.alibi = alibi;
    a.valid = valid;
    a.lse = const_cast<float*>(lse);
    a.delta = delta;
    a.row = row_stride;
    a.head = head_stride;
    a.batch_stride = batch_stride;
    a.orow = o_row_stride;
    a.obatch = o_batch_stride;
    a.heads = (int)heads;
    a.tokens = (int)tokens;
    a.batch_heads = (int)(batch * heads);
    a.scale = (float)(1.0 / sqrt((double)head_dim));
    hipStream_t st = as_stream(stream);
    const unsigned tiles = (unsigned)(((tokens + kBQ - 1) / kBQ) * batch * heads);
    // the dQ pass first: it leaves delta behind for the dK / dV pass
    const unsigned tiles2 = (unsigned)(((tokens + 63) / 64) * batch * heads);
    const bool split_q = narrow_split(tiles), split_kv = narrow_split_dkv(tiles);
    if (dtype == BR_F16) {
        if (split_q) flash_bwd_dq_kernel<BR_GEMM_F16, 2, 2><<<tiles2, kThreads, 0, st>>>(a);
        else flash_bwd_dq_kernel<BR_GEMM_F16, 4, 1><<<tiles, kThreads, 0, st>>>(a);
        if (split_kv) flash_bwd_dkv_kernel<BR_GEMM_F16, 2, 2><<<tiles2, kThreads, 0, st>>>(a);
        else flash_bwd_dkv_kernel<BR_GEMM_F16, 4, 1><<<tiles, kThreads, 0, st>>>(a);
    } else {
        if (split_q) flash_bwd_dq_kernel<BR_GEMM_BF16, 2, 2><<<tiles2, kThreads, 0, st>>>(a);
        else flash_bwd_dq_kernel<BR_GEMM_BF16, 4, 1><<<tiles, kThreads, 0, st>>>(a);
        if (split_kv) flash_bwd_dkv_kernel<BR_GEMM_BF16, 2, 2><<<tiles2, kThreads, 0, st>>>(a);
        else flash_bwd_dkv_kernel<BR_GEMM_BF16, 4, 1><<<tiles, kThreads, 0, st>>>(a);
    }
    BR_HIP_LAUNCH_CHECK();
    return BR_OK;
}

}  // extern "C"
