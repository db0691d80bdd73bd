// 16-bit MFMA GEMM, direct-to-LDS variant: the fast path for products whose
// two operands are both stored in the MFMA element type (fp16 or bf16).
//
//   C[b][i,j] = alpha * sum_p opA[b][i,p] * opB[b][p,j] (+ C) (+ bias[j])
//
// Operand tiles never pass through registers on their way in: every wave
// issues global_load_lds_dwordx4 (gfx950: 16 bytes per lane, 1 KiB per
// instruction, written to LDS at M0 + lane*16).  Because the LDS side of such
// a load is fixed to lane order, padding rows is not possible; bank conflicts
// are avoided by choosing WHICH 16-byte chunk of the tile each lane fetches
// (an XOR swizzle), and un-swizzling in the fragment reads:
//
//   k contiguous in memory  -> LDS image [row][4 chunks of 8 k], 64 bytes per
//       row; chunk c of row r sits in slot c ^ ((r >> 2) & 3).  A fragment is
//       one ds_read_b128 per lane; any 16 consecutive rows of one chunk column
//       cover all 64 banks exactly once.
//   row contiguous in memory-> LDS image [k][ROWS/8 chunks of 8 rows]; chunk c
//       of k-row k sits in slot c ^ (4 * (k & 3)).  Fragments are read with
//       ds_read_b64_tr_b16 (two per fragment); the 4 k-rows x 64 bytes that 32
//       lanes touch in one pass land in 16 different 16-byte bank groups.
//
// Pipeline.  STAGES tile buffers form a ring and are all filled up front.  A K
// step (KT = 32 or 64 k-values) is KT/16 sub-steps with two fragment register
// sets used alternately:
//   sub-step s < last:  issue the LDS reads of sub-step s+1, run the MFMAs of
//       sub-step s (whose fragments were read one sub-step ago);
//   last sub-step of tile t:  wait until this wave's loads of tile t+1 have
//       landed (s_waitcnt vmcnt(N), later tiles stay in flight); workgroup
//       barrier -- now tile t+1 is complete in LDS and every wave has read all
//       of tile t; issue the loads of tile t+STAGES into the buffer tile t
//       occupied; issue the LDS reads of (t+1, first sub-step); run the MFMAs.
// KT = 64 makes a k-contiguous operand row a full 128-byte cache line per
// step (with 32, each line is fetched from L2 twice, half used each time).
// One barrier per K step, no staging registers, LDS latency hidden behind 16+
// MFMAs inside the wave, HBM / L2 latency behind STAGES-1 K steps.  The loads
// and the vmcnt waits are inline assembly because the compiler would otherwise
// wait for ALL outstanding direct-to-LDS loads before any LDS read.
//
// Requirements (checked by the host dispatcher; everything else takes the
// register-staged kernel in gemm_mfma16.hpp): K % 32 == 0, 16-byte aligned
// operand bases / leading dimensions / batch strides, and for row-contiguous
// operands rows % 8 == 0.  Rows past the end of an operand are redirected to a
// valid row; their products land in rows / columns of C that are never stored.
#pragma once
#include <mutex>
#include <type_traits>

#include "gemm_mfma16.hpp"
#include "lds_direct.hpp"


namespace brk {
namespace gemm16 {

// Operand tile of ROWS x KT elements (KT = 32 or 64 k-values per K step).
template <int ROWS, int KT, int WAVES, bool KSTR>
struct DtlTile {
    static constexpr int kBytes = ROWS * KT * 2;
    static constexpr int kInstr = kBytes / 1024;     // wave-wide loads per tile
    static constexpr int kPerWave = kInstr / WAVES;  // ... issued by each wave
    static_assert(kInstr % WAVES == 0, "tile loads do not divide among the waves");
    static_assert(ROWS >= 128, "swizzle needs at least 16 chunks per k-row");
    // k contiguous: a row is KT/8 chunks; kRowsPer256 rows span the 64 banks
    static constexpr int kRowBytes = KT * 2;
    static constexpr int kChunksPerRow = KT / 8;
    static constexpr int kRowsPer256 = 256 / kRowBytes;
    static constexpr int kRowsPerInstr = 64 / kChunksPerRow;
    // row contiguous: a k-row is ROWS/8 chunks
    static constexpr int kChunksPerK = ROWS / 8;
    static constexpr int kKPerInstr = 64 / kChunksPerK;

    // Byte offset (from the tile origin at K step 0) of the chunk this lane
    // fetches in its q-th load of a tile; LDS slot = instruction*64 + lane.
    static __device__ __forceinline__ unsigned source_offset(int q, int wave, int lane, long long ld, long long row0,
                                                             long long rows) {
        const int j = q * WAVES + wave;
        if (!KSTR) {
            const int r = j * kRowsPerInstr + lane / kChunksPerRow;
            const int c = (lane % kChunksPerRow) ^ ((r / kRowsPer256) % kChunksPerRow);
            long long row = row0 + r;
            row = row < rows ? row : rows - 1;
            return (unsigned)(((row - row0) * ld + c * 8) * 2);
        } else {
            const int kk = j * kKPerInstr + lane / kChunksPerK;
            const int c = (lane % kChunksPerK) ^ (4 * (kk & 3));
            long long row = row0 + c * 8;
            row = row < rows ? row : row0;
            return (unsigned)((kk * ld + (row - row0)) * 2);
        }
    }

    // LDS byte offset (inside one tile image) this lane reads the fragment of
    // 32-row block `row_base` and 16-k sub-step ks from; row-contiguous tiles
    // read a second time 4 k-rows further on.
    static __device__ __forceinline__ unsigned frag_offset(int row_base, int ks, int lane) {
        if (!KSTR) {
            const int r = row_base + (lane & 31);
            const int c = ks * 2 + (lane >> 5);
            return (unsigned)(r * kRowBytes + ((c ^ ((r / kRowsPer256) % kChunksPerRow)) * 16));
        } else {
            const int i = lane & 15, grp = lane >> 4;
            const int kk = ks * 16 + (grp >> 1) * 8 + (i >> 2);
            const int row16 = row_base + (grp & 1) * 16 + (i & 3) * 4;
            const int c = (row16 >> 3) ^ (4 * (i >> 2));
            return (unsigned)(kk * (ROWS * 2) + c * 16 + (row16 & 7) * 2);
        }
    }

    static __device__ __forceinline__ u32x4 fragment(const lds_byte* tile, unsigned off) {
        if (!KSTR) {
            return *reinterpret_cast<const __attribute__((address_space(3))) u32x4*>(tile + off);
        } else {
            typedef __attribute__((address_space(3))) s16x4 lds_s16x4;
            const s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4*)(tile + off));
            const s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4*)(tile + off + 4 * ROWS * 2));
            const u32x2 l2 = __builtin_bit_cast(u32x2, lo), h2 = __builtin_bit_cast(u32x2, hi);
            return mk4(l2.x, l2.y, h2.x, h2.y);
        }
    }
};

// K split in two with the sum done in the kernel.  A product whose 256x256 tiles fill at most half the CUs and
// whose K is long runs two workgroups per tile, workgroup (tile, s) summing half s of K.  After its K loop a
// workgroup draws a ticket from the tile's counter.  The first to draw writes its fp32 partial tile to the caller's
// workspace (in the accumulators' own register order), reports in on a second counter and is done; the second
// waits until the first has reported -- it drew first, so it is past its K loop and its stores are in flight: a
// wait for work already under way, never for a workgroup that may not have started -- adds that partial to its own
// and runs the epilogue.  A sum of two terms is the same whichever is added to which, so the bits do not depend on
// which half finished first.
// The partial tile crosses from one XCD's L2 to another's.  Every access to it is made coherent at device scope by
// itself (the sc1 bit: the access goes to the level all XCDs share), so no fence has to write back or invalidate
// a whole L2 -- which a device-scope fence does on this part, and which costs more than the product when hundreds
// of workgroups do it.  Such accesses move 1.5-3 TB/s where ordinary stores move 6-7: with four or more slices
// (every slice writing, one reading them all) this form measured slower than partials written with ordinary
// stores and summed by a second kernel, which is what products with more slices use (gemm.hip).
// The counters live in the library, start at zero and are put back to zero by the second arrival, so a launch needs
// no clearing pass.  There is one set per stream (kSplitSlots of them, handed out in the order streams first ask:
// split_slot_of): products on one stream run one after the other and may share a set, products split at the same
// time on different streams meet through different sets; a stream beyond the last set gets no split.
constexpr int kMaxSplitTiles = 8192;
constexpr int kSplitSlots = 8;
static __device__ unsigned dtl_tickets[kSplitSlots][kMaxSplitTiles];
static __device__ unsigned dtl_arrived[kSplitSlots][kMaxSplitTiles];

typedef float f32x4 __attribute__((ext_vector_type(4)));
// The wait states after the store are part of the statement: a store of more than 64 bits reads its data
// registers a few cycles after it issues, and the compiler, which keeps such a store's data registers intact for
// that long when it emits the instruction itself, does not look into an asm statement -- it reused them for the
// next address at once, and single lanes of a partial tile came out as garbage.
__device__ __forceinline__ void store_device_coherent(f32x4* p, const f32x4& v) {
    asm volatile("global_store_dwordx4 %0, %1, off sc1\n\ts_nop 2" : : "v"(p), "v"(v) : "memory");
}
// Four such loads and the wait for them in ONE statement: the compiler takes an asm statement's outputs to be
// ready when the statement ends, so a wait in a statement of its own would let it copy the registers in between.
__device__ __forceinline__ void load4_device_coherent(f32x4 (&v)[4], const f32x4* p, int stride) {
    const f32x4 *p1 = p + stride, *p2 = p + 2 * stride, *p3 = p + 3 * stride;
    asm volatile(
        "global_load_dwordx4 %0, %4, off sc1\n\t"
        "global_load_dwordx4 %1, %5, off sc1\n\t"
        "global_load_dwordx4 %2, %6, off sc1\n\t"
        "global_load_dwordx4 %3, %7, off sc1\n\t"
        "s_waitcnt vmcnt(0)"
        : "=&v"(v[0]), "=&v"(v[1]), "=&v"(v[2]), "=&v"(v[3])
        : "v"(p), "v"(p1), "v"(p2), "v"(p3)
        : "memory");
}

// KW = 2: the sixteen-wide sub-steps of every K step are dealt to two groups of waves (group kw takes sub-steps
// kw * KS/2 ..), each group covering the whole tile with wave tiles twice as large; the groups' accumulators are
// added through LDS after the K loop (group 1 into group 0, which runs the epilogue).  For tiles too small to give
// eight waves a 64 x 128 block each: a 256 x 128 tile on eight 64 x 64 waves reads 128 KB of fragments per K step
// from LDS, on two groups of four 64 x 128 waves 96 KB.
template <int CT, int BM, int BN, int WM, int WN, int KT, int STAGES, bool A_KSTR, bool B_KSTR, typename TC,
          bool GELU = false, bool SPLIT = false, int KW = 1>
__global__ __launch_bounds__((BM / WM) * (BN / WN) * KW * 64) void gemm_dtl_kernel(GemmArgs g) {
    constexpr int WAVES_MN = (BM / WM) * (BN / WN);
    constexpr int WAVES = WAVES_MN * KW;
    constexpr int FM = WM / 32, FN = WN / 32, KS = KT / 16 / KW;   // KS: sub-steps of a K step per wave
    static_assert(KW == 1 || (KW == 2 && KT == 64 && !SPLIT), "two wave groups: 64-wide K steps, no K split across workgroups");
    using TA = DtlTile<BM, KT, WAVES, A_KSTR>;
    using TB = DtlTile<BN, KT, WAVES, B_KSTR>;
    constexpr int kStageBytes = TA::kBytes + TB::kBytes;
    constexpr int kLoads = TA::kPerWave + TB::kPerWave;  // per wave and tile
    static_assert(STAGES >= 2 && STAGES <= 6, "two to six tile buffers");
    static_assert(KT == 32 || KT == 64, "K tile of 32 or 64");
    static_assert(FM * FN >= FM + FN, "one LDS fragment read per MFMA slot");
    static_assert(STAGES * kStageBytes <= 160 * 1024, "LDS");
    __shared__ __attribute__((aligned(1024))) unsigned char lds_raw[STAGES * kStageBytes];
    const lds_byte* lds = (const lds_byte*)lds_raw;
    const unsigned lds0 = (unsigned)(unsigned long long)lds;

    long long batch;
    int tm, tn;
    tile_coords(g, batch, tm, tn);
    // The divisions in tile_coords run on the vector unit although their operands are wave-uniform.  Taking the
    // results back to scalar registers here keeps everything derived from them (operand tile origins, which the
    // load statement needs in scalar registers, and the row bases of C) on the scalar unit.
    tm = __builtin_amdgcn_readfirstlane(tm);
    tn = __builtin_amdgcn_readfirstlane(tn);
    batch = __builtin_amdgcn_readfirstlane((int)batch);
    // with a K split the slices take the place of the batch index in the tile order (slice-major: the workgroups
    // an XCD runs at a time still cover one block of tiles, of one slice)
    const int slice = SPLIT ? (int)batch : 0;
    if (SPLIT) batch = 0;
    const long long row0 = (long long)tm * BM, col0 = (long long)tn * BN;
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int kw = KW == 1 ? 0 : wave / WAVES_MN, wave_mn = KW == 1 ? wave : wave % WAVES_MN;
    const int wm = wave_mn / (BN / WN), wn = wave_mn % (BN / WN);

    // tile origins at K step 0 (wave-uniform, advanced once per step) and the
    // per-lane chunk offsets (fixed for the whole K loop)
    const unsigned char* a_src = reinterpret_cast<const unsigned char*>(g.a) +
                                 2 * (batch * g.sa + (A_KSTR ? row0 : row0 * g.lda));
    const unsigned char* b_src = reinterpret_cast<const unsigned char*>(g.b) +
                                 2 * (batch * g.sb + (B_KSTR ? col0 : col0 * g.ldb));
    const long long a_step = A_KSTR ? 2 * KT * g.lda : 2 * KT;
    const long long b_step = B_KSTR ? 2 * KT * g.ldb : 2 * KT;
    unsigned a_off[TA::kPerWave], b_off[TB::kPerWave];
#pragma unroll
    for (int q = 0; q < TA::kPerWave; q++) a_off[q] = TA::source_offset(q, wave, lane, g.lda, row0, g.m);
#pragma unroll
    for (int q = 0; q < TB::kPerWave; q++) b_off[q] = TB::source_offset(q, wave, lane, g.ldb, col0, g.n);

    unsigned fa_off[FM][KS], fb_off[FN][KS];
#pragma unroll
    for (int ks = 0; ks < KS; ks++) {
#pragma unroll
        for (int i = 0; i < FM; i++) fa_off[i][ks] = TA::frag_offset(wm * WM + i * 32, kw * KS + ks, lane);
#pragma unroll
        for (int j = 0; j < FN; j++) fb_off[j][ks] = TA::kBytes + TB::frag_offset(wn * WN + j * 32, kw * KS + ks, lane);
    }

    // this workgroup's K steps: [k_begin, k_begin + nk) of the g.k / KT steps (all of them without a split)
    const int nk_all = (int)(g.k / KT);
    const int k_begin = SPLIT ? slice * nk_all / 2 : 0;
    const int nk = SPLIT ? (slice + 1) * nk_all / 2 - k_begin : nk_all;
    // step `t` of the loop covers K step k_begin + (t + first) mod nk (see k_walk_start)
    const int first = SPLIT ? (int)(k_walk_start(row0, col0, g.k) / KT) % nk : (int)(k_walk_start(row0, col0, g.k) / KT);
    a_src += (k_begin + first) * a_step;
    b_src += (k_begin + first) * b_step;
    int until_wrap = nk - first;  // issues left before the walk returns to K step 0
    auto issue = [&](int tile) {
        const unsigned dst = lds0 + (unsigned)(tile % STAGES) * kStageBytes + (unsigned)wave * 1024u;
#pragma unroll
        for (int q = 0; q < TA::kPerWave; q++) dtl_load(dst + q * WAVES * 1024, a_off[q], a_src);
#pragma unroll
        for (int q = 0; q < TB::kPerWave; q++) dtl_load(dst + TA::kBytes + q * WAVES * 1024, b_off[q], b_src);
        const bool wraps = --until_wrap == 0;
        a_src += wraps ? a_step - nk * a_step : a_step;
        b_src += wraps ? b_step - nk * b_step : b_step;
    };
    auto read_frags = [&](u32x4 (&fa)[FM], u32x4 (&fb)[FN], int tile, int ks) {
        const lds_byte* stage = lds + (tile % STAGES) * kStageBytes;
#pragma unroll
        for (int i = 0; i < FM; i++) fa[i] = TA::fragment(stage, fa_off[i][ks]);
#pragma unroll
        for (int j = 0; j < FN; j++) fb[j] = TB::fragment(stage, fb_off[j][ks]);
    };

    f32x16 acc[FM][FN];
#pragma unroll
    for (int i = 0; i < FM; i++)
#pragma unroll
        for (int j = 0; j < FN; j++)
#pragma unroll
            for (int v = 0; v < 16; v++) acc[i][j][v] = 0.f;
    // One sub-step, in the instruction order the hardware is to see: the MFMAs of
    // the fragments in hand (fa, fb), with the LDS reads that fetch the next
    // sub-step's fragments (na, nb; from `tile`, sub-step `ks`) slotted in one
    // per MFMA.  The scheduling fences pin that order: left alone, the compiler
    // sinks the reads below the MFMAs to reuse their registers, and the next
    // sub-step's first MFMA then waits out the full LDS latency.
    auto step = [&](const u32x4 (&fa)[FM], const u32x4 (&fb)[FN], u32x4 (&na)[FM], u32x4 (&nb)[FN], int tile, int ks) {
        const lds_byte* stage = lds + (tile % STAGES) * kStageBytes;
#pragma unroll
        for (int idx = 0; idx < FM * FN; idx++) {
            // column-major walk over the wave's blocks: the first FM MFMAs need only fb[0];
            // fragments are fetched in the order the next sub-step uses them: fb[0], fa[0..], fb[1..]
            const int i = idx % FM, j = idx / FM;
            if (idx == 0) nb[0] = TB::fragment(stage, fb_off[0][ks]);
            else if (idx <= FM) na[idx - 1] = TA::fragment(stage, fa_off[idx - 1][ks]);
            else if (idx < FM + FN) nb[idx - FM] = TB::fragment(stage, fb_off[idx - FM][ks]);
            acc[i][j] = Cvt<CT>::mfma(fa[i], fb[j], acc[i][j]);
            __builtin_amdgcn_sched_barrier(0);
        }
    };

    // Fill the ring, wait for tile 0 and read its first sub-step of fragments.
#pragma unroll
    for (int s = 0; s < STAGES; s++)
        if (s < nk) issue(s);
    if (nk > STAGES - 1) {
        wait_vmem<(STAGES - 1) * kLoads>();
    } else {
        wait_vmem<0>();
    }
    __syncthreads();
    // Two fragment sets: while the MFMAs of one sub-step run, the LDS reads of
    // the next sub-step are in flight.
    u32x4 fa0[FM], fb0[FN], fa1[FM], fb1[FN];
    read_frags(fa0, fb0, 0, 0);
    __builtin_amdgcn_sched_barrier(0);

    // The MFMA stream is free of branches: the last tile's final sub-step also
    // fetches (from the buffer a tile nk would occupy; the values are never
    // used) and passes the barrier like every other.
    for (int t = 0; t < nk; t++) {
#pragma unroll
        for (int ks = 0; ks < KS; ks++) {
            u32x4(&fa_now)[FM] = (ks & 1) ? fa1 : fa0;
            u32x4(&fb_now)[FN] = (ks & 1) ? fb1 : fb0;
            u32x4(&fa_next)[FM] = (ks & 1) ? fa0 : fa1;
            u32x4(&fb_next)[FN] = (ks & 1) ? fb0 : fb1;
            if (ks + 1 < KS) {
                step(fa_now, fb_now, fa_next, fb_next, t, ks + 1);
            } else {
                // tile t+1 has to be in LDS; the tiles issued after it may stay in flight
                const int after = nk - 2 - t;
                if (after >= STAGES - 2) {
                    wait_vmem<(STAGES - 2) * kLoads>();
                } else if (STAGES > 3 && after == 1) {
                    wait_vmem<kLoads>();
                } else {
                    wait_vmem<0>();
                }
                // every wave has now read all of tile t (__syncthreads waits for the wave's own LDS reads to
                // complete, lgkmcnt(0), before the barrier), so its buffer can be refilled
                __syncthreads();
                if (t + STAGES < nk) issue(t + STAGES);
                __builtin_amdgcn_sched_barrier(0);
                step(fa_now, fb_now, fa_next, fb_next, t + 1, 0);
            }
        }
    }

    if constexpr (KW == 2) {
        // Every tile issued has landed and been read (the loop's last waits and barrier); the stages now carry
        // group 1's accumulators to group 0: quad q of thread t of wave w at quad index (w * 4 FM FN + q) * 64 + t.
        static_assert((size_t)STAGES * kStageBytes >= (size_t)WAVES_MN * FM * FN * 16 * 64 * 4, "the stages hold one group's sums");
        f32x4* const x = reinterpret_cast<f32x4*>(lds_raw) + (size_t)wave_mn * (4 * FM * FN) * 64 + lane;
        __syncthreads();   // the last sub-step's (unused) fragment reads are done too
        if (kw == 1) {
#pragma unroll
            for (int i = 0; i < FM; i++)
#pragma unroll
                for (int j = 0; j < FN; j++)
#pragma unroll
                    for (int q = 0; q < 4; q++) {
                        f32x4 v;
                        v.x = acc[i][j][4 * q]; v.y = acc[i][j][4 * q + 1]; v.z = acc[i][j][4 * q + 2]; v.w = acc[i][j][4 * q + 3];
                        x[((i * FN + j) * 4 + q) * 64] = v;
                    }
        }
        __syncthreads();
        if (kw == 1) return;
#pragma unroll
        for (int i = 0; i < FM; i++)
#pragma unroll
            for (int j = 0; j < FN; j++)
#pragma unroll
                for (int q = 0; q < 4; q++) {
                    const f32x4 v = x[((i * FN + j) * 4 + q) * 64];
                    acc[i][j][4 * q] += v.x; acc[i][j][4 * q + 1] += v.y; acc[i][j][4 * q + 2] += v.z; acc[i][j][4 * q + 3] += v.w;
                }
    }

    if constexpr (SPLIT) {
        constexpr int THREADS = WAVES * 64;
        constexpr size_t kTileQuads = (size_t)BM * BN / 4;
        const int tile_id = tm * g.tiles_n + tn;
        f32x4* const slot = reinterpret_cast<f32x4*>(g.partials) + (size_t)tile_id * kTileQuads;
        // everybody is through with the LDS tiles; one word of them carries the ticket to the workgroup
        __syncthreads();
        unsigned* const drawn = reinterpret_cast<unsigned*>(lds_raw);
        if (threadIdx.x == 0)
            *drawn = __hip_atomic_fetch_add(&dtl_tickets[g.split_slot][tile_id], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        __syncthreads();
        const bool last = *drawn == 1u;
        // Quad q of accumulator block (i, j) of thread t sits at quad index ((i*FN + j)*4 + q)*THREADS + t of the
        // partial tile (a kilobyte per wave and instruction).  One block at a time, with a running pointer and a
        // fence after each block: the kernel has no registers to spare for addresses formed ahead of time.
        if (!last) {
            f32x4* at = slot + threadIdx.x;
#pragma unroll
            for (int blk = 0; blk < FM * FN; blk++) {
                const int i = blk / FN, j = blk % FN;
#pragma unroll
                for (int q = 0; q < 4; q++) {
                    f32x4 v;
                    v.x = acc[i][j][4 * q]; v.y = acc[i][j][4 * q + 1]; v.z = acc[i][j][4 * q + 2]; v.w = acc[i][j][4 * q + 3];
                    store_device_coherent(at, v);
                    at += THREADS;
                }
                __builtin_amdgcn_sched_barrier(0);
            }
            wait_vmem<0>();   // this thread's stores have reached the level every XCD sees
            __syncthreads();  // ... and so have every other thread's of this workgroup
            if (threadIdx.x == 0)
                __hip_atomic_fetch_add(&dtl_arrived[g.split_slot][tile_id], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            return;
        }
        // The second to draw: the other slice drew first, so it is past its K loop and on its way through the few
        // lines above, which wait for nothing -- the wait below is for stores already in flight.  It is bounded all
        // the same (a second or so): should the counters ever be out of step -- a product killed half way leaves
        // them so -- the tile is filled with NaN rather than summed from a partial that is not there.
        if (threadIdx.x == 0) {
            unsigned seen = 0;
            for (int spin = 0; spin < (1 << 22); spin++) {
                seen = __hip_atomic_load(&dtl_arrived[g.split_slot][tile_id], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                if (seen >= 1u) break;
                __builtin_amdgcn_s_sleep(4);
            }
            *drawn = seen >= 1u ? 1u : 0u;
        }
        __syncthreads();
        if (*drawn == 0u) {
#pragma unroll
            for (int i = 0; i < FM; i++)
#pragma unroll
                for (int j = 0; j < FN; j++)
#pragma unroll
                    for (int v = 0; v < 16; v++) acc[i][j][v] = __builtin_nanf("");
        } else {
            // two terms: the sum is the same whichever of them is the one held in registers, so the bits do not
            // depend on which slice drew last
            const f32x4* at = slot + threadIdx.x;
#pragma unroll
            for (int blk = 0; blk < FM * FN; blk++) {
                const int i = blk / FN, j = blk % FN;
                f32x4 v[4];
                load4_device_coherent(v, at, THREADS);
                at += 4 * THREADS;
#pragma unroll
                for (int q = 0; q < 4; q++) {
                    acc[i][j][4 * q] += v[q].x;
                    acc[i][j][4 * q + 1] += v[q].y;
                    acc[i][j][4 * q + 2] += v[q].z;
                    acc[i][j][4 * q + 3] += v[q].w;
                }
                __builtin_amdgcn_sched_barrier(0);
            }
        }
        if (threadIdx.x == 0) {
            // ready for the next product; written the way the counters are read and added to (an ordinary store
            // would sit in this XCD's L2, out of sight of the other XCDs' atomics, until the kernel ends)
            __hip_atomic_store(&dtl_tickets[g.split_slot][tile_id], 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            __hip_atomic_store(&dtl_arrived[g.split_slot][tile_id], 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
    }

    // acc[i][j][v] is C[row, col] with
    //   row = wm*WM + i*32 + (v/4)*8 + (lane/32)*4 + v%4,  col = wn*WN + j*32 + lane%32
    TC* c_base = static_cast<TC*>(g.c) + batch * g.sc;
    TC* c2_base = GELU ? static_cast<TC*>(g.c2) + batch * g.sc : nullptr;
    const TC* old_base = g.addend ? static_cast<const TC*>(g.addend) + batch * g.sc : c_base;  // read when accumulating
    if (row0 + BM <= g.m && col0 + BN <= g.n) {
        // Interior tile: straight-line code without guards, one 32x32 block of accumulators at a time.  A block's
        // 16 stores leave back to back; when accumulating, the old C of the next block is read before the stores
        // of this one are issued, so the wait for those reads lets the stores stay in flight.  (In the guarded path
        // below, a read of C next to each store puts a wait for ALL outstanding memory operations in front of
        // every element: each store then completes before the next is issued.)  Addresses are a wave-uniform row
        // base plus one per-lane offset; dtl_applies has checked that the offset fits 32 bits.  The fences keep
        // the compiler from forming the addresses of all 128 elements ahead of the first store, which takes more
        // registers than there are.
        const unsigned lane_bytes = (unsigned)(((lane >> 5) * 4 * g.ldc + (lane & 31)) * (long long)sizeof(TC));
        const long long tile_at = (row0 + __builtin_amdgcn_readfirstlane(wm) * WM) * g.ldc + col0 +
                                  __builtin_amdgcn_readfirstlane(wn) * WN;
        char* const c_tile = reinterpret_cast<char*>(c_base + tile_at);
        char* const c2_tile = GELU ? reinterpret_cast<char*>(c2_base + tile_at) : nullptr;
        char* const old_tile = reinterpret_cast<char*>(const_cast<TC*>(old_base) + tile_at);
        auto element = [&](char* tile, int blk, int v) {
            const int i = blk / FN, j = blk % FN;
            return reinterpret_cast<TC*>(tile + (i * 32 + (v >> 2) * 8 + (v & 3)) * g.ldc * (long long)sizeof(TC) +
                                         j * 32 * sizeof(TC) + lane_bytes);
        };
        float bias[FN];
#pragma unroll
        for (int j = 0; j < FN; j++) bias[j] = g.bias ? g.bias[col0 + wn * WN + j * 32 + (lane & 31)] : 0.f;
        auto interior = [&](auto adds) {
            constexpr bool ADDS = decltype(adds)::value;
            // alpha made opaque per form, or the compiler merges the scaling of all 128 elements of the two forms
            // into one pass ahead of the branch and spills its results
            float alpha = g.alpha;
            asm volatile("" : "+v"(alpha));
            float was[2][16];
            auto fetch = [&](int blk) {
#pragma unroll
                for (int v = 0; v < 16; v++) was[blk & 1][v] = c_load<TC>(element(old_tile, blk, v));
            };
            if (ADDS) fetch(0);
#pragma unroll
            for (int blk = 0; blk < FM * FN; blk++) {
                const int i = blk / FN, j = blk % FN;
                if (ADDS && blk + 1 < FM * FN) fetch(blk + 1);
                __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                for (int v = 0; v < 16; v++) {
                    float o = alpha * acc[i][j][v] + bias[j];
                    if (ADDS) o += was[blk & 1][v];
                    // A 16-bit C is the rounded copy of this fp32 value, the same bits a later product would make
                    // of an fp32 C on loading it.  Left alone, the compiler merges the multiply-add and the
                    // narrowing into one mixed-precision instruction whose result differs in the last place.
                    if (sizeof(TC) == 2) asm volatile("" : "+v"(o));
                    c_store<TC>(element(c_tile, blk, v), o);
                    // the activation is taken of the fp32 value, not of its rounded copy
                    if (GELU) c_store<TC>(element(c2_tile, blk, v), gelu_one(o));
                }
                __builtin_amdgcn_sched_barrier(0);
            }
        };
        if (g.accumulate) {
            interior(std::true_type{});
        } else {
            interior(std::false_type{});
        }
        return;
    }
    // Edge tiles: element-wise guards.  The two forms are separate loops so that the plain one holds no read of C.
    auto guarded = [&](auto adds) {
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
                        if (decltype(adds)::value) o += c_load<TC>(old_base + row * g.ldc + col);
                        if (sizeof(TC) == 2) asm volatile("" : "+v"(o));  // as in the interior form
                        c_store<TC>(p, o);
                        if (GELU) c_store<TC>(c2_base + row * g.ldc + col, gelu_one(o));
                    }
                }
            }
        }
    };
    if (g.accumulate) {
        guarded(std::true_type{});
    } else {
        guarded(std::false_type{});
    }
}

// ---- the same product with workgroups that stay -------------------------------------------------
// 32 workgroups per XCD walk the tiles of that XCD's share instead of one workgroup being launched per tile; the
// tile order, the K walk and the order of every sum are those of gemm_dtl_kernel, so the bits are too.  What it
// buys: a workgroup issues the first two K stages of its NEXT tile before the C stores of the current one, and lets
// up to 63 of those stores stay in flight through the next tile's first K step -- the 2.3 us a fresh workgroup
// spends being launched and waiting for its first operand tile disappear behind the epilogue.  Measured on products
// of the BLOOM-7B1 block (same run, before / after): weight gradient [16384 x 4096] from K = 2048 253 -> 245 us,
// from K = 512 99 -> 95 us, [4096 x 4096] 66.2 -> 64.6, h -> 4h forward 241 -> 237.
// Memory operations complete in issue order on this target, which is what the partial waits rest on: after the 16
// operand loads of the next tile come the wave's 128 stores, so "at most 63 outstanding" means the loads are in.
// Plain products only: 256 x 256 tiles, all of them interior (m, n multiples of 256), one batch, no bias, nothing
// accumulated, no second output (walk_applies); everything else takes gemm_dtl_kernel.
template <int CT, bool A_KSTR, bool B_KSTR, typename TC>
__global__ __launch_bounds__(512) void gemm_dtl_walk_kernel(GemmArgs g) {
    constexpr int BM = 256, BN = 256, WM = 64, WN = 128, KT = 64, STAGES = 2;
    constexpr int WAVES = (BM / WM) * (BN / WN);
    constexpr int FM = WM / 32, FN = WN / 32, KS = KT / 16;
    using TA = DtlTile<BM, KT, WAVES, A_KSTR>;
    using TB = DtlTile<BN, KT, WAVES, B_KSTR>;
    constexpr int kStageBytes = TA::kBytes + TB::kBytes;
    constexpr int kLoads = TA::kPerWave + TB::kPerWave;
    static_assert(FM * FN * 16 >= 63, "the partial wait counts on at least 63 stores per wave and tile");
    __shared__ __attribute__((aligned(1024))) unsigned char lds_raw[STAGES * kStageBytes];
    const lds_byte* lds = (const lds_byte*)lds_raw;
    const unsigned lds0 = (unsigned)(unsigned long long)lds;
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int wm = wave / (BN / WN), wn = wave % (BN / WN);
    // workgroup ids are dealt to the 8 XCDs round-robin: this one is number `slot` of `slots` on XCD `xcd`, whose
    // share of the tile order is [xcd * per_xcd, (xcd + 1) * per_xcd), as in tile_coords
    const int per_xcd = g.tiles_m * g.tiles_n / 8;
    const int xcd = blockIdx.x & 7, slot = blockIdx.x >> 3, slots = gridDim.x >> 3;
    const int my_tiles = (per_xcd - slot + slots - 1) / slots;
    const int nk = (int)(g.k / KT);

    unsigned fa_off[FM][KS], fb_off[FN][KS];
#pragma unroll
    for (int ks = 0; ks < KS; ks++) {
#pragma unroll
        for (int i = 0; i < FM; i++) fa_off[i][ks] = TA::frag_offset(wm * WM + i * 32, ks, lane);
#pragma unroll
        for (int j = 0; j < FN; j++) fb_off[j][ks] = TA::kBytes + TB::frag_offset(wn * WN + j * 32, ks, lane);
    }
    // interior tiles: a lane's chunk offsets inside the operand tiles are the same for every tile
    unsigned a_off[TA::kPerWave], b_off[TB::kPerWave];
#pragma unroll
    for (int q = 0; q < TA::kPerWave; q++) a_off[q] = TA::source_offset(q, wave, lane, g.lda, 0, g.m);
#pragma unroll
    for (int q = 0; q < TB::kPerWave; q++) b_off[q] = TB::source_offset(q, wave, lane, g.ldb, 0, g.n);
    const long long a_step = A_KSTR ? 2 * KT * g.lda : 2 * KT;
    const long long b_step = B_KSTR ? 2 * KT * g.ldb : 2 * KT;

    const unsigned char* a_src = nullptr;
    const unsigned char* b_src = nullptr;
    int until_wrap = 0;
    long long row0 = 0, col0 = 0;
    auto setup = [&](int it) {   // the it-th tile of this workgroup: origins and the start of its K walk
        int tm, tn;
        tile_in_order(g, xcd * per_xcd + it * slots + slot, tm, tn);
        tm = __builtin_amdgcn_readfirstlane(tm);
        tn = __builtin_amdgcn_readfirstlane(tn);
        row0 = (long long)tm * BM;
        col0 = (long long)tn * BN;
        const int first = (int)(k_walk_start(row0, col0, g.k) / KT);
        a_src = reinterpret_cast<const unsigned char*>(g.a) + 2 * (A_KSTR ? row0 : row0 * g.lda) + first * a_step;
        b_src = reinterpret_cast<const unsigned char*>(g.b) + 2 * (B_KSTR ? col0 : col0 * g.ldb) + first * b_step;
        until_wrap = nk - first;
    };
    auto issue = [&](int tile) {
        const unsigned dst = lds0 + (unsigned)(tile % STAGES) * kStageBytes + (unsigned)wave * 1024u;
#pragma unroll
        for (int q = 0; q < kLoads; q++) {
            if (q < TA::kPerWave) dtl_load(dst + q * WAVES * 1024, a_off[q], a_src);
            else dtl_load(dst + TA::kBytes + (q - TA::kPerWave) * WAVES * 1024, b_off[q - TA::kPerWave], b_src);
        }
        const bool wraps = --until_wrap == 0;
        a_src += wraps ? a_step - nk * a_step : a_step;
        b_src += wraps ? b_step - nk * b_step : b_step;
    };
    f32x16 acc[FM][FN];
    auto step = [&](const u32x4 (&fa)[FM], const u32x4 (&fb)[FN], u32x4 (&na)[FM], u32x4 (&nb)[FN], int tile, int ks) {
        const lds_byte* stage = lds + (tile % STAGES) * kStageBytes;
#pragma unroll
        for (int idx = 0; idx < FM * FN; idx++) {
            const int i = idx % FM, j = idx / FM;
            if (idx == 0) nb[0] = TB::fragment(stage, fb_off[0][ks]);
            else if (idx <= FM) na[idx - 1] = TA::fragment(stage, fa_off[idx - 1][ks]);
            else if (idx < FM + FN) nb[idx - FM] = TB::fragment(stage, fb_off[idx - FM][ks]);
            acc[i][j] = Cvt<CT>::mfma(fa[i], fb[j], acc[i][j]);
            __builtin_amdgcn_sched_barrier(0);
        }
    };

    setup(0);
    issue(0);
    if (nk > 1) issue(1);
    for (int it = 0; it < my_tiles; it++) {
#pragma unroll
        for (int i = 0; i < FM; i++)
#pragma unroll
            for (int j = 0; j < FN; j++)
#pragma unroll
                for (int v = 0; v < 16; v++) acc[i][j][v] = 0.f;
        // K stage 0 of this tile has to be in LDS.  First tile: nothing but its two stages is outstanding.  Later
        // tiles: both stages were issued ahead of the previous tile's stores, so they have landed once at most 63
        // operations (all of them stores) are outstanding.
        if (nk == 1) wait_vmem<0>();
        else if (it == 0) wait_vmem<kLoads>();
        else wait_vmem<63>();
        __syncthreads();
        u32x4 fa0[FM], fb0[FN], fa1[FM], fb1[FN];
#pragma unroll
        for (int i = 0; i < FM; i++) fa0[i] = TA::fragment(lds, fa_off[i][0]);
#pragma unroll
        for (int j = 0; j < FN; j++) fb0[j] = TB::fragment(lds, fb_off[j][0]);
        __builtin_amdgcn_sched_barrier(0);
        for (int t = 0; t < nk; t++) {
#pragma unroll
            for (int ks = 0; ks < KS; ks++) {
                u32x4(&fa_now)[FM] = (ks & 1) ? fa1 : fa0;
                u32x4(&fb_now)[FN] = (ks & 1) ? fb1 : fb0;
                u32x4(&fa_next)[FM] = (ks & 1) ? fa0 : fa1;
                u32x4(&fb_next)[FN] = (ks & 1) ? fb0 : fb1;
                if (ks + 1 < KS) {
                    step(fa_now, fb_now, fa_next, fb_next, t, ks + 1);
                } else {
                    // K stage t+1 has to be in LDS: the only loads in flight, except during step 0 of a later tile,
                    // when stage 1 is already in and up to 63 of the previous tile's stores may go on draining
                    if (t == 0 && it > 0) wait_vmem<63>(); else wait_vmem<0>();
                    __syncthreads();
                    if (t + STAGES < nk) issue(t + STAGES);
                    __builtin_amdgcn_sched_barrier(0);
                    step(fa_now, fb_now, fa_next, fb_next, t + 1, 0);
                }
            }
        }
        // Every wave is past the last barrier of the K loop and nothing in LDS is read for its value any more (the
        // loop's trailing fragment reads fetch a stage that does not exist): the next tile's first stages may go.
        const long long st_row0 = row0, st_col0 = col0;
        if (it + 1 < my_tiles) {
            asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
            setup(it + 1);
            issue(0);
            if (nk > 1) issue(1);
        }
        // acc[i][j][v] is C[row, col] with row = wm*WM + i*32 + (v/4)*8 + (lane/32)*4 + v%4, col = wn*WN + j*32 + lane%32
        const unsigned lane_bytes = (unsigned)(((lane >> 5) * 4 * g.ldc + (lane & 31)) * (long long)sizeof(TC));
        const long long tile_at = (st_row0 + wm * WM) * g.ldc + st_col0 + wn * WN;
        char* const c_tile = reinterpret_cast<char*>(static_cast<TC*>(g.c) + tile_at);
        float alpha = g.alpha;
        asm volatile("" : "+v"(alpha));
#pragma unroll
        for (int blk = 0; blk < FM * FN; blk++) {
            const int i = blk / FN, j = blk % FN;
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int v = 0; v < 16; v++) {
                float o = alpha * acc[i][j][v] + 0.f;   // the plain epilogue's expression with its bias of zero
                if (sizeof(TC) == 2) asm volatile("" : "+v"(o));   // one fp32 value, then one rounding (see gemm_dtl_kernel)
                c_store<TC>(reinterpret_cast<TC*>(c_tile + (i * 32 + (v >> 2) * 8 + (v & 3)) * g.ldc * (long long)sizeof(TC) +
                                                  j * 32 * sizeof(TC) + lane_bytes), o);
            }
            __builtin_amdgcn_sched_barrier(0);
        }
    }
}

// Whether the walking form takes a product the plan has put on 256 x 256 tiles.
#ifndef BR_DTL_WALK
#define BR_DTL_WALK 1   // 0: every product on one workgroup per tile (for an A/B build)
#endif
inline bool walk_applies(const GemmArgs& g, long long batch) {
    if (!BR_DTL_WALK) return false;
    const long long tiles = (g.m / 256) * (g.n / 256);
    return batch == 1 && g.m % 256 == 0 && g.n % 256 == 0 && g.k % 64 == 0 && tiles >= 256 && tiles % 8 == 0 &&
           tiles <= 0x7fffffffLL && !g.bias && !g.accumulate && !g.c2 && !g.addend && g.splits == 1;
}

template <int CT>
int launch_dtl_walk(GemmArgs g, const Problem& p, hipStream_t st) {
    g.tiles_m = (int)(g.m / 256);
    g.tiles_n = (int)(g.n / 256);
    using F16 = __half;
    using BF16 = __hip_bfloat16;
#define BR_DTL_WALK_CASE(AK, BK_)                                                        \
    if (p.a_kstr == AK && p.b_kstr == BK_) {                                             \
        if (p.c_dtype == BR_F32)                                                         \
            gemm_dtl_walk_kernel<CT, AK, BK_, float><<<256, 512, 0, st>>>(g);            \
        else if (CT == BR_GEMM_F16)                                                      \
            gemm_dtl_walk_kernel<CT, AK, BK_, F16><<<256, 512, 0, st>>>(g);              \
        else                                                                             \
            gemm_dtl_walk_kernel<CT, AK, BK_, BF16><<<256, 512, 0, st>>>(g);             \
    }
    BR_DTL_WALK_CASE(false, false)
    BR_DTL_WALK_CASE(false, true)
    BR_DTL_WALK_CASE(true, false)
    BR_DTL_WALK_CASE(true, true)
#undef BR_DTL_WALK_CASE
    BR_HIP_LAUNCH_CHECK();
    return BR_OK;
}

// ---- host-side dispatch -------------------------------------------------------
#ifndef BR_DTL_KW
#define BR_DTL_KW 1
#endif
#ifndef BR_DTL_KW_MIN_STEPS
#define BR_DTL_KW_MIN_STEPS 24
#endif
template <int CT, int BM, int BN, int WM, int WN, int KT, int ST, int KW = 1>
int launch_dtl_config(GemmArgs g, const Problem& p, long long batch, hipStream_t st) {
    constexpr int THREADS = (BM / WM) * (BN / WN) * KW * 64;
    g.tiles_m = (int)((g.m + BM - 1) / BM);
    g.tiles_n = (int)((g.n + BN - 1) / BN);
    if (g.splits > 1) {
        // the plan only splits unbatched products whose partial tiles fit the workspace it was given
        const long long tiles = (long long)g.tiles_m * g.tiles_n;
        if (g.splits != 2 || batch != 1 || tiles > kMaxSplitTiles || !g.partials ||
            (size_t)tiles * BM * BN * sizeof(float) > g.partial_bytes)   // one partial tile per output tile
            return BR_ERR_ATTR;
    }
    const long long blocks = (long long)g.tiles_m * g.tiles_n * batch * g.splits;
    if (blocks > 0x7fffffffLL) return BR_ERR_ATTR;
    const unsigned grid = (unsigned)blocks;
    using F16 = __half;
    using BF16 = __hip_bfloat16;
    if (g.splits == 2) {
        // the two-slice form: its own instantiations (of the two 256-row tiles, the only ones it is planned on),
        // so that the unsplit kernels carry none of its code
        if (g.c2 || BM != 256 || KW != 1) return BR_ERR_TODO;
#define BR_DTL_SPLIT_CASE(AK, BK_)                                                                              \
    if constexpr (BM == 256 && KW == 1) if (p.a_kstr == AK && p.b_kstr == BK_) {                                                          \
        if (p.c_dtype == BR_F32)                                                                                 \
            gemm_dtl_kernel<CT, BM, BN, WM, WN, KT, ST, AK, BK_, float, false, true><<<grid, THREADS, 0, st>>>(g); \
        else if (CT == BR_GEMM_F16)                                                                              \
            gemm_dtl_kernel<CT, BM, BN, WM, WN, KT, ST, AK, BK_, F16, false, true><<<grid, THREADS, 0, st>>>(g);   \
        else                                                                                                     \
            gemm_dtl_kernel<CT, BM, BN, WM, WN, KT, ST, AK, BK_, BF16, false, true><<<grid, THREADS, 0, st>>>(g);  \
    }
        BR_DTL_SPLIT_CASE(false, false)
        BR_DTL_SPLIT_CASE(false, true)
        BR_DTL_SPLIT_CASE(true, false)
        BR_DTL_SPLIT_CASE(true, true)
#undef BR_DTL_SPLIT_CASE
        BR_HIP_LAUNCH_CHECK();
        return BR_OK;
    }
    if (g.c2) {
        // GELU epilogue: built for the linear layer's layout only (both operands k-contiguous, 16-bit outputs)
        if (p.a_kstr || p.b_kstr || p.c_dtype == BR_F32) return BR_ERR_TODO;
        if (CT == BR_GEMM_F16)
            gemm_dtl_kernel<CT, BM, BN, WM, WN, KT, ST, false, false, F16, true, false, KW><<<grid, THREADS, 0, st>>>(g);
        else
            gemm_dtl_kernel<CT, BM, BN, WM, WN, KT, ST, false, false, BF16, true, false, KW><<<grid, THREADS, 0, st>>>(g);
        BR_HIP_LAUNCH_CHECK();
        return BR_OK;
    }
#define BR_DTL_CASE(AK, BK_)                                                                           \
    if (p.a_kstr == AK && p.b_kstr == BK_) {                                                            \
        if (p.c_dtype == BR_F32)                                                                        \
            gemm_dtl_kernel<CT, BM, BN, WM, WN, KT, ST, AK, BK_, float, false, false, KW><<<grid, THREADS, 0, st>>>(g);   \
        else if (CT == BR_GEMM_F16)                                                                     \
            gemm_dtl_kernel<CT, BM, BN, WM, WN, KT, ST, AK, BK_, F16, false, false, KW><<<grid, THREADS, 0, st>>>(g);     \
        else                                                                                            \
            gemm_dtl_kernel<CT, BM, BN, WM, WN, KT, ST, AK, BK_, BF16, false, false, KW><<<grid, THREADS, 0, st>>>(g);    \
    }
    BR_DTL_CASE(false, false)
    BR_DTL_CASE(false, true)
    BR_DTL_CASE(true, false)
    BR_DTL_CASE(true, true)
#undef BR_DTL_CASE
    BR_HIP_LAUNCH_CHECK();
    return BR_OK;
}

// The direct-to-LDS kernel applies when both operands are 16-bit, the fast
// path's alignment rules hold and every per-lane source offset fits 32 bits.
inline bool dtl_applies(const GemmArgs& g, const Problem& p) {
    if (p.a_f32 || p.b_f32 || p.guarded) return false;
    const long long lim = 1LL << 31;
    const long long a_span = p.a_kstr ? 2 * 64 * g.lda : 2 * 256 * g.lda;
    const long long b_span = p.b_kstr ? 2 * 64 * g.ldb : 2 * 256 * g.ldb;
    return a_span < lim && b_span < lim && g.ldc < (1LL << 27);
}

// Tile choice by estimated time: rounds of workgroups over the 256 CUs x the
// MFMA work of one tile / the rate a workgroup of that configuration reaches
// (measured on the BLOOM-7B1 linear-layer shapes: ~1000 TFLOP/s chip-wide for
// 256x256, ~0.9 of that for 256x128, ~0.8 for 128x128 with two workgroups
// resident per CU).
struct DtlPlan {
    int config;      // 0: 256x256, 1: 256x128, 2: 128x128 (64-wide K steps), 3: 128x128 with 32-wide steps
    double seconds;  // estimate, for comparing plans only
};
inline DtlPlan dtl_tile_plan(long long m, long long n, long long k, long long batch) {
    const double per_cu = 1.0e15 / 256.0;  // flop/s of one CU at the 256x256 rate
    auto estimate = [&](long long bm, long long bn, long long slots, double rel) {
        const long long tiles = ((m + bm - 1) / bm) * ((n + bn - 1) / bn) * batch;
        const double rounds = (double)((tiles + slots - 1) / slots);
        const double per_block = per_cu * rel * 256.0 / (double)slots;  // co-resident workgroups share the CU
        return rounds * 2.0 * (double)bm * (double)bn * (double)k / per_block + 4e-6;
    };
    if (k % 64 != 0) return DtlPlan{3, estimate(128, 128, 512, 0.65)};
    DtlPlan best{0, estimate(256, 256, 256, 1.0)};
    const double t1 = estimate(256, 128, 256, 0.9), t2 = estimate(128, 128, 512, 0.8);
    if (t1 < best.seconds) best = DtlPlan{1, t1};
    if (t2 < best.seconds) best = DtlPlan{2, t2};
    return best;
}

// A product whose 256x256 tiles fill some rounds of workgroups and then at most half of one more (the q|k|v
// projection of 2048 tokens: 384 tiles, a round and a half) leaves half the chip idle for a whole tile time, and on
// 256x128 tiles throughout it pays their lower rate on every round.  Run in two launches -- the columns that make
// whole rounds on 256x256 tiles, the rest on 256x128 tiles, which then fill one round -- the projection takes 190 us
// instead of 210 either way.  Returns the first column of the second launch, or 0 where this does not apply or does
// not beat `best_seconds` (the estimate of the best single-launch plan, same model as dtl_tile_plan).  The split
// falls on a multiple of 1024 columns, the period of k_walk_start, so every element of C is still summed in the
// order every other plan sums it in.
inline long long dtl_column_tail(long long m, long long n, long long k, double best_seconds) {
    if (k % 64 != 0) return 0;
    const long long tm = (m + 255) / 256, tn = (n + 255) / 256;
    long long a = 256, b = tm;
    while (b) { const long long r = a % b; a = b; b = r; }   // a = gcd(256, tm)
    long long unit = 256 / a;                                // tile columns that make whole rounds
    if (unit < 4) unit = 4;                                  // a power of two; and a multiple of 1024 columns
    const long long tn_main = tn / unit * unit, tn_rest = tn - tn_main;
    if (tn_main == 0 || tn_rest == 0 || tm * tn_rest > 128) return 0;
    const double round256 = 2.0 * 256.0 * 256.0 * (double)k / (1.0e15 / 256.0);
    const double seconds = (double)(tm * tn_main / 256) * round256 + 0.5 * round256 / 0.9 + 6e-6;
    return seconds < best_seconds ? tn_main * 256 : 0;
}

// Whether the two-slice K split inside the kernel pays (-1 = no, else the tile configuration to run it with), from
// per-workgroup times measured on MI355X (fp16, all CUs busy): a 64-wide K step takes 1.8 us on a 256x256 tile and
// 1.15 us on 256x128; a round of workgroups costs 3 us to fill and drain; C leaves at 6.5 TB/s; the one partial tile
// per output tile is written and read back through device-coherent accesses at about 3 TB/s.  It pays where 256x256
// tiles would fill at most half the CUs and K is long: for [2048 x 4096] outputs from K = 12288 up (8-10 % there).
// Shorter M (few rows: many slices do better, see the caller) and shapes this timing was not taken on are left alone.
inline int dtl_pair_split(long long m, long long n, long long k) {
    if (m < 1024 || k % 64 != 0 || k / 64 < 16) return -1;
    auto estimate = [&](int config, int splits) {
        const long long bm = config == 0 ? 256 : 256, bn = config == 0 ? 256 : 128;
        const long long tiles = ((m + bm - 1) / bm) * ((n + bn - 1) / bn);
        const double rounds = (double)((tiles * splits + 255) / 256);
        const double steps = (double)(k / splits) / 64.0;
        double t = rounds * (steps * (config == 0 ? 1.8 : 1.15) + 3.0) * 1e-6 + (double)m * n * 4.0 / 6.5e12 + 4e-6;
        if (splits > 1) t += 2.0 * (double)tiles * bm * bn * 4.0 / 3e12 + 3e-6;
        return t;
    };
    const double unsplit = estimate(0, 1) < estimate(1, 1) ? estimate(0, 1) : estimate(1, 1);
    int pick = -1;
    double best = 0.97 * unsplit;
    for (int c = 0; c < 2; c++) {
        const long long bm = 256, bn = c == 0 ? 256 : 128;
        if (((m + bm - 1) / bm) * ((n + bn - 1) / bn) > kMaxSplitTiles) continue;
        const double t = estimate(c, 2);
        if (t < best) {
            best = t;
            pick = c;
        }
    }
    return pick;
}
// bytes of partial tiles the two-slice split needs in the caller's workspace (one per output tile; 0 when the
// split does not pay)
inline size_t dtl_pair_split_bytes(long long m, long long n, long long k) {
    const int c = dtl_pair_split(m, n, k);
    if (c < 0) return 0;
    const long long bm = 256, bn = c == 0 ? 256 : 128;
    return (size_t)(((m + bm - 1) / bm) * ((n + bn - 1) / bn)) * bm * bn * sizeof(float);
}

// The counter set of a stream (-1: all sets are taken by other streams).
inline int split_slot_of(hipStream_t st) {
    static std::mutex mu;
    static hipStream_t owner[kSplitSlots];
    static int used = 0;
    std::lock_guard<std::mutex> lock(mu);
    for (int i = 0; i < used; i++)
        if (owner[i] == st) return i;
    if (used == kSplitSlots) return -1;
    owner[used] = st;
    return used++;
}

template <int CT>
int launch_dtl(GemmArgs g, const Problem& p, long long batch, hipStream_t st) {
    g.splits = 1;
    if (batch == 1 && g.partials) {
        const int c = dtl_pair_split(g.m, g.n, g.k);
        const int slot = c >= 0 ? split_slot_of(st) : -1;
        if (c >= 0 && slot >= 0 && dtl_pair_split_bytes(g.m, g.n, g.k) <= g.partial_bytes) {
            g.splits = 2;
            g.split_slot = slot;
            if (c == 0) return launch_dtl_config<CT, 256, 256, 64, 128, 64, 2>(g, p, batch, st);
            return launch_dtl_config<CT, 256, 128, 64, 64, 64, 3>(g, p, batch, st);
        }
    }
    const DtlPlan plan = dtl_tile_plan(g.m, g.n, g.k, batch);
    const long long tail_from = batch == 1 ? dtl_column_tail(g.m, g.n, g.k, plan.seconds) : 0;
    if (tail_from > 0) {
        // whole rounds of 256x256 tiles, then the columns left over on 256x128 tiles (see dtl_column_tail)
        GemmArgs head = g;
        head.n = tail_from;
        const int rc = launch_dtl_config<CT, 256, 256, 64, 128, 64, 2>(head, p, batch, st);
        if (rc != BR_OK) return rc;
        GemmArgs tail = g;
        const size_t c_size = p.c_dtype == BR_F32 ? 4 : 2;
        tail.n = g.n - tail_from;
        tail.b = static_cast<const unsigned char*>(g.b) + 2 * (p.b_kstr ? tail_from : tail_from * g.ldb);
        tail.c = static_cast<unsigned char*>(g.c) + c_size * tail_from;
        if (g.c2) tail.c2 = static_cast<unsigned char*>(g.c2) + c_size * tail_from;
        if (g.addend) tail.addend = static_cast<const unsigned char*>(g.addend) + c_size * tail_from;
        if (g.bias) tail.bias = g.bias + tail_from;
        if (BR_DTL_KW && g.k / 64 >= BR_DTL_KW_MIN_STEPS) return launch_dtl_config<CT, 256, 128, 64, 128, 64, 3, 2>(tail, p, batch, st);
        return launch_dtl_config<CT, 256, 128, 64, 64, 64, 3>(tail, p, batch, st);
    }
    const int pick = plan.config;
    if (pick == 0 && walk_applies(g, batch)) return launch_dtl_walk<CT>(g, p, st);
    if (pick == 0) return launch_dtl_config<CT, 256, 256, 64, 128, 64, 2>(g, p, batch, st);
    if (pick == 1) {
        // long K: two groups of four 64 x 128 waves per tile (fewer fragment reads, a merge at the end)
        if (BR_DTL_KW && g.k / 64 >= BR_DTL_KW_MIN_STEPS) return launch_dtl_config<CT, 256, 128, 64, 128, 64, 3, 2>(g, p, batch, st);
        return launch_dtl_config<CT, 256, 128, 64, 64, 64, 3>(g, p, batch, st);
    }
    if (pick == 2) return launch_dtl_config<CT, 128, 128, 64, 64, 64, 2>(g, p, batch, st);
    return launch_dtl_config<CT, 128, 128, 64, 64, 32, 3>(g, p, batch, st);
}

template <int CT>
int launch_any(const GemmArgs& g, const Problem& p, long long batch, hipStream_t st) {
    if (dtl_applies(g, p)) return launch_dtl<CT>(g, p, batch, st);
    if (g.c2) return BR_ERR_TODO;  // only the direct-to-LDS kernel has the GELU epilogue
    return launch<CT>(g, p, batch, st);
}

}  // namespace gemm16
}  // namespace brk
