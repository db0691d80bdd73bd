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
// each wave owns 32 queries.  Keys / values stream through LDS in tiles of 64;
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

#include <float.h>

using namespace brk;
using namespace brk::gemm16;

namespace {

constexpr int kHD = 128;          // head size
constexpr int kChunks = kHD / 8;  // 16-byte chunks per row
constexpr int kBQ = 128;          // queries per workgroup (forward, dq pass)
constexpr int kBK = 64;           // keys per LDS tile
constexpr int kThreads = 256;

typedef __attribute__((address_space(3))) unsigned char lds_byte;

struct FlashArgs {
    const u16* q;
    const u16* k;
    const u16* v;
    u16* o;
    const u16* d_o;
    float* dq;
    float* dk;
    float* dv;
    const float* alibi;    // [heads, tokens]
    const int32_t* valid;  // [batch]
    float* lse;            // [batch, heads, tokens]
    float* delta;          // [batch, heads, tokens]  rowsum(dO o O)
    long long row, head, batch_stride;  // element strides of q, k, v, o, d_o, dq, dk, dv
    int heads, tokens;
    float scale;
};

__device__ __forceinline__ int swz(int r) { return ((r & 3) << 2) | ((r >> 2) & 3); }
// byte offset of chunk c of row r in a [rows][16 chunks] tile image
__device__ __forceinline__ unsigned slot(int r, int c) { return (unsigned)((r * kChunks + (c ^ swz(r))) * 16); }

// Cooperative load of ROWS x 128 16-bit elements (rows row0.., clamped to
// `rows` - 1) into registers, then into an LDS image.  256 threads, 16 bytes
// each per pass; 16 consecutive threads fetch one contiguous 256-byte row.
template <int ROWS>
struct TileLoader {
    static constexpr int kPasses = ROWS * kChunks / kThreads;
    u32x4 regs[kPasses];
    __device__ __forceinline__ void fetch(const u16* base, long long row_stride, int row0, int rows) {
#pragma unroll
        for (int i = 0; i < kPasses; i++) {
            const int idx = threadIdx.x + i * kThreads;
            int r = row0 + idx / kChunks;
            r = r < rows ? r : rows - 1;
            regs[i] = *reinterpret_cast<const u32x4*>(base + (long long)r * row_stride + (idx % kChunks) * 8);
        }
    }
    __device__ __forceinline__ void store(unsigned char* tile) const {
#pragma unroll
        for (int i = 0; i < kPasses; i++) {
            const int idx = threadIdx.x + i * kThreads;
            *reinterpret_cast<u32x4*>(tile + slot(idx / kChunks, idx % kChunks)) = regs[i];
        }
    }
};

// A operand, rows of the tile as MFMA rows, d as the k index: rows r0 + lane%32,
// d = 16 * ks + 8 * (lane / 32) .. + 7.
__device__ __forceinline__ u32x4 frag_rows(const lds_byte* tile, int r0, int ks, int lane) {
    const int r = r0 + (lane & 31);
    return *reinterpret_cast<const __attribute__((address_space(3))) u32x4*>(tile + slot(r, ks * 2 + (lane >> 5)));
}

// A / B operand with d as the MFMA row (or column) index and tile rows as the
// k index: lane gets d = d0 + 16 * ((lane >> 4) & 1) + lane % 16 and the eight
// tile rows  ra + 0..3  and  rb + 0..3  (ra, rb multiples of 4, per lane half).
__device__ __forceinline__ u32x4 frag_cols(const lds_byte* tile, int d0, int ra, int rb, int lane) {
    typedef __attribute__((address_space(3))) s16x4 lds_s16x4;
    const int i = lane & 15;
    const int d = d0 + ((lane >> 4) & 1) * 16 + (i & 3) * 4;
    const int ja = ra + (i >> 2), jb = rb + (i >> 2);
    const s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4*)(tile + slot(ja, d >> 3) + (d & 7) * 2));
    const s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4*)(tile + slot(jb, d >> 3) + (d & 7) * 2));
    const u32x2 l2 = __builtin_bit_cast(u32x2, lo), h2 = __builtin_bit_cast(u32x2, hi);
    return mk4(l2.x, l2.y, h2.x, h2.y);
}

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

template <int CT>
__global__ __launch_bounds__(kThreads) void flash_fwd_kernel(FlashArgs a) {
    __shared__ __attribute__((aligned(1024))) unsigned char lds_k[kBK * kHD * 2];
    __shared__ __attribute__((aligned(1024))) unsigned char lds_v[kBK * kHD * 2];
    const lds_byte* tk = (const lds_byte*)lds_k;
    const lds_byte* tv = (const lds_byte*)lds_v;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, half = lane >> 5;
    const int tiles_q = (a.tokens + kBQ - 1) / kBQ;
    const int qt = tiles_q - 1 - (int)blockIdx.x;  // longest rows first
    const int bh = blockIdx.y, b = bh / a.heads, h = bh % a.heads;
    const long long base = (long long)b * a.batch_stride + (long long)h * a.head;
    const int valid = a.valid[b];
    const int q0 = qt * kBQ + wave * 32;
    const int query = q0 + (lane & 31);
    const int qrow = query < a.tokens ? query : a.tokens - 1;
    const float* bias = a.alibi + (long long)h * a.tokens;

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

    const int nkeys = visible_keys(qt * kBQ + kBQ, valid, a.tokens);
    const int ntiles = (nkeys + kBK - 1) / kBK;
    // keys this wave's queries can see (a wave may idle through the last tiles)
    const int wave_keys = visible_keys(q0 + 32, valid, a.tokens);

    TileLoader<kBK> lk, lv;
    lk.fetch(a.k + base, a.row, 0, a.tokens);
    lv.fetch(a.v + base, a.row, 0, a.tokens);
    for (int t = 0; t < ntiles; t++) {
        const int k0 = t * kBK;
        __syncthreads();  // every wave has finished reading the previous tile
        lk.store(lds_k);
        lv.store(lds_v);
        __syncthreads();
        if (t + 1 < ntiles) {
            lk.fetch(a.k + base, a.row, k0 + kBK, a.tokens);
            lv.fetch(a.v + base, a.row, k0 + kBK, a.tokens);
        }
        if (k0 >= wave_keys) continue;

        f32x16 s[2];
#pragma unroll
        for (int kb = 0; kb < 2; kb++) {
#pragma unroll
            for (int v = 0; v < 16; v++) s[kb][v] = 0.f;
#pragma unroll
            for (int ks = 0; ks < 8; ks++) s[kb] = Cvt<CT>::mfma(frag_rows(tk, kb * 32, ks, lane), qf[ks], s[kb]);
        }
        float mt = -INFINITY;
#pragma unroll
        for (int kb = 0; kb < 2; kb++)
#pragma unroll
            for (int g = 0; g < 4; g++) {
                const int key = k0 + kb * 32 + g * 8 + half * 4;
                const int kidx = key + 3 < a.tokens ? key : a.tokens - 4;  // keep the 16-byte read inside the table
                const float4 bv = *reinterpret_cast<const float4*>(bias + (kidx > 0 ? kidx : 0));
                const float bb[4] = {bv.x, bv.y, bv.z, bv.w};
#pragma unroll
                for (int j = 0; j < 4; j++) {
                    const float x = score(s[kb][g * 4 + j], a.scale, bb[j], query, key + j, valid, a.tokens);
                    s[kb][g * 4 + j] = x;
                    mt = fmaxf(mt, x);
                }
            }
        mt = fmaxf(mt, xor32(mt));
        const float m_new = fmaxf(m, mt);
        const float alpha = __expf(m - m_new);
        float sum = 0.f;
#pragma unroll
        for (int kb = 0; kb < 2; kb++)
#pragma unroll
            for (int v = 0; v < 16; v++) {
                const float p = __expf(s[kb][v] - m_new);
                s[kb][v] = p;
                sum += p;
            }
        sum += xor32(sum);
        l = l * alpha + sum;
        m = m_new;
#pragma unroll
        for (int db = 0; db < 4; db++)
#pragma unroll
            for (int v = 0; v < 16; v++) o[db][v] *= alpha;
#pragma unroll
        for (int j = 0; j < 4; j++) {
            const int kb = j >> 1, vb = (j & 1) * 8;
            float p8[8];
#pragma unroll
            for (int e = 0; e < 8; e++) p8[e] = s[kb][vb + e];
            const u32x4 pf = pack8<CT>(p8);
            const int ra = kb * 32 + (j & 1) * 16 + half * 4;
#pragma unroll
            for (int db = 0; db < 4; db++) o[db] = Cvt<CT>::mfma(frag_cols(tv, db * 32, ra, ra + 8, lane), pf, o[db]);
        }
    }

    if (query < a.tokens) {
        const float inv = 1.0f / l;
        u16* orow = a.o + base + (long long)query * a.row;
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

bool flash_shape_ok(int64_t batch, int64_t heads, int64_t tokens, int64_t head_dim, int64_t row, int64_t head,
                    int64_t batch_stride) {
    return batch > 0 && heads > 0 && tokens >= 4 && tokens % 4 == 0 && head_dim == kHD && row % 8 == 0 &&
           head % 8 == 0 && batch_stride % 8 == 0 && batch * heads <= 65535 && tokens <= (1 << 20);
}

}  // namespace

extern "C" {

int br_hip_flash_attn_fwd(const void* q, const void* k, const void* v, int dtype, const float* alibi,
                          const int32_t* valid, void* o, float* lse, int64_t batch, int64_t heads, int64_t tokens,
                          int64_t head_dim, int64_t row_stride, int64_t head_stride, int64_t batch_stride,
                          br_stream_t stream) {
    if (batch < 0 || heads <= 0 || tokens <= 0 || head_dim <= 0) return BR_ERR_ATTR;
    if (batch == 0) return BR_OK;
    if (!q || !k || !v || !alibi || !valid) return BR_ERR_INPUT;
    if (!o || !lse) return BR_ERR_OUTPUT;
    if ((dtype != BR_F16 && dtype != BR_BF16) ||
        !flash_shape_ok(batch, heads, tokens, head_dim, row_stride, head_stride, batch_stride) || !aligned16(q) ||
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
    a.heads = (int)heads;
    a.tokens = (int)tokens;
    a.scale = (float)(1.0 / sqrt((double)head_dim));
    const dim3 grid((unsigned)((tokens + kBQ - 1) / kBQ), (unsigned)(batch * heads));
    if (dtype == BR_F16)
        flash_fwd_kernel<BR_GEMM_F16><<<grid, kThreads, 0, as_stream(stream)>>>(a);
    else
        flash_fwd_kernel<BR_GEMM_BF16><<<grid, kThreads, 0, as_stream(stream)>>>(a);
    BR_HIP_LAUNCH_CHECK();
    return BR_OK;
}

}  // extern "C"
