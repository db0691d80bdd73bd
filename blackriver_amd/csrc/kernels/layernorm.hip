// LayerNorm forward / backward for gfx950.
//
// Forward: one 256-thread workgroup per row; the row is read from HBM once
// into registers (128-bit loads), mean and centred variance are reduced with
// wave64 butterflies plus one LDS exchange, and the normalised row is written
// straight from registers.
//
// Backward: persistent workgroups walk over rows.  Each thread keeps gamma,
// beta and running dgamma / dbeta sums for its own columns in registers, so
// dy and y are read exactly once; per-workgroup partial column sums go to a
// workspace and a small second kernel adds them in a fixed order.
#include <mutex>

#include "common.hpp"

#include <stdlib.h>

using namespace brk;

namespace {

constexpr int kBlock = 256;
constexpr int kWaves = kBlock / kWave;

__device__ __forceinline__ float add_eps(float g, float eps) {
    return fabsf(g) > eps ? g : (g < 0.f ? -eps : eps);
}

// ---------------------------------------------------------------- forward
// VPT = float4 vectors per thread; cols4 = cols / 4 <= kBlock * VPT.
template <int VPT>
__global__ __launch_bounds__(kBlock) void ln_fwd_regs(const float* __restrict__ x,
                                                       const float* __restrict__ gamma,
                                                       const float* __restrict__ beta,
                                                       float* __restrict__ y, float* __restrict__ mean_out,
                                                       float* __restrict__ var_out, int cols4, float eps,
                                                       float inv_cols, Copy16 y16) {
    __shared__ float lds[2][kWaves];
    const int64_t row = blockIdx.x;
    const float4* xr = reinterpret_cast<const float4*>(x) + row * cols4;
    float4 v[VPT];
#pragma unroll
    for (int i = 0; i < VPT; i++) {
        const int idx = threadIdx.x + i * kBlock;
        v[i] = idx < cols4 ? load_stream(xr + idx) : make_float4(0.f, 0.f, 0.f, 0.f);
    }
    float s[1] = {0.f};
#pragma unroll
    for (int i = 0; i < VPT; i++) s[0] += (v[i].x + v[i].y) + (v[i].z + v[i].w);
    block_sum<1>(s, lds[0]);
    const float mean = s[0] * inv_cols;

    float q[1] = {0.f};
#pragma unroll
    for (int i = 0; i < VPT; i++) {
        const int idx = threadIdx.x + i * kBlock;
        if (idx < cols4) {
            const float a = v[i].x - mean, b = v[i].y - mean, c = v[i].z - mean, d = v[i].w - mean;
            q[0] += (a * a + b * b) + (c * c + d * d);
        }
    }
    block_sum<1>(q, lds[1]);
    const float var = q[0] * inv_cols + eps;  // the stored statistic includes eps
    const float rstd = 1.0f / sqrtf(var);
    if (threadIdx.x == 0) {
        if (mean_out) mean_out[row] = mean;
        if (var_out) var_out[row] = var;
    }
    float4* yr = reinterpret_cast<float4*>(y) + row * cols4;
#pragma unroll
    for (int i = 0; i < VPT; i++) {
        const int idx = threadIdx.x + i * kBlock;
        if (idx < cols4) {
            const float4 g = reinterpret_cast<const float4*>(gamma)[idx];
            const float4 b = reinterpret_cast<const float4*>(beta)[idx];
            float4 o;
            o.x = (v[i].x - mean) * rstd * g.x + b.x;
            o.y = (v[i].y - mean) * rstd * g.y + b.y;
            o.z = (v[i].z - mean) * rstd * g.z + b.z;
            o.w = (v[i].w - mean) * rstd * g.w + b.w;
            store4_as16(y16, row * cols4 + idx, o);
            store_stream(yr + idx, o);
        }
    }
}

// Any width / alignment: three sweeps over the row from global memory.
__global__ __launch_bounds__(kBlock) void ln_fwd_generic(const float* x, const float* gamma, const float* beta,
                                                          float* y, float* mean_out, float* var_out,
                                                          int64_t cols, float eps) {
    __shared__ float lds[2][kWaves];
    const int64_t row = blockIdx.x;
    const float* xr = x + row * cols;
    float s[1] = {0.f};
    for (int64_t c = threadIdx.x; c < cols; c += kBlock) s[0] += xr[c];
    block_sum<1>(s, lds[0]);
    const float mean = s[0] / (float)cols;
    float q[1] = {0.f};
    for (int64_t c = threadIdx.x; c < cols; c += kBlock) {
        const float d = xr[c] - mean;
        q[0] += d * d;
    }
    block_sum<1>(q, lds[1]);
    const float var = q[0] / (float)cols + eps;
    const float rstd = 1.0f / sqrtf(var);
    if (threadIdx.x == 0) {
        if (mean_out) mean_out[row] = mean;
        if (var_out) var_out[row] = var;
    }
    for (int64_t c = threadIdx.x; c < cols; c += kBlock)
        y[row * cols + c] = (xr[c] - mean) * rstd * gamma[c] + beta[c];
}

// --------------------------------------------------------------- backward
// A workgroup is GROUPS row walkers of 256 threads each: walker w of workgroup
// b takes rows (b*GROUPS + w), + gridDim.x*GROUPS, ...; each keeps gamma, beta,
// 1/gamma and its running dgamma / dbeta in registers and has the next row's
// loads in flight while it works on the current one.  At the end the walkers'
// running sums are added in LDS (walker order) and the workgroup writes ONE
// partial row pair, so the finalize pass reads gridDim.x partials.
// SUMS: the finished input gradient (residual included) is also summed over the rows, column by column, into a
// third partial row, and written a second time in 16 bit: what the backward of the linear layer that produced the
// LayerNorm's input needs of it (its bias gradient and the operand of its two products).
constexpr int kWalker = kBlock;  // threads per row walker
template <int VPT, int GROUPS, bool SUMS = false>
__global__ __launch_bounds__(kWalker * GROUPS) void ln_bwd_regs(const float* dy, const float* __restrict__ y,
                                                                 const float* __restrict__ gamma,
                                                                 const float* __restrict__ beta,
                                                                 const float* __restrict__ var, float* dx,
                                                                 float* __restrict__ part_dgamma,
                                                                 float* __restrict__ part_dbeta, int64_t rows,
                                                                 int cols4, float eps, float inv_cols,
                                                                 const float* residual,
                                                                 float* __restrict__ part_dx = nullptr,
                                                                 Copy16 dx16 = Copy16{nullptr, 0}) {
    __shared__ float lds[2][GROUPS][2 * kWaves];
    const int walker = threadIdx.x / kWalker, tid = threadIdx.x % kWalker;
    const int lane = tid & 63, wave = tid >> 6;
    float4 g[VPT], ginv[VPT], b[VPT], acc_g[VPT], acc_b[VPT], acc_x[SUMS ? VPT : 1];
    if (SUMS) {
#pragma unroll
        for (int i = 0; i < VPT; i++) acc_x[SUMS ? i : 0] = make_float4(0.f, 0.f, 0.f, 0.f);
    }
#pragma unroll
    for (int i = 0; i < VPT; i++) {
        const int idx = tid + i * kWalker;
        const bool ok = idx < cols4;
        g[i] = ok ? reinterpret_cast<const float4*>(gamma)[idx] : make_float4(1.f, 1.f, 1.f, 1.f);
        b[i] = ok ? reinterpret_cast<const float4*>(beta)[idx] : make_float4(0.f, 0.f, 0.f, 0.f);
        ginv[i] = make_float4(1.0f / add_eps(g[i].x, eps), 1.0f / add_eps(g[i].y, eps),
                              1.0f / add_eps(g[i].z, eps), 1.0f / add_eps(g[i].w, eps));
        acc_g[i] = make_float4(0.f, 0.f, 0.f, 0.f);
        acc_b[i] = make_float4(0.f, 0.f, 0.f, 0.f);
    }
    float4 d[VPT], xh[VPT], nd[VPT], nxh[VPT];
    // rows past the end read as dy = 0, y = 0: they add nothing to any sum
    auto request = [&](float4 (&rd)[VPT], float4 (&ry)[VPT], int64_t row) {
#pragma unroll
        for (int i = 0; i < VPT; i++) {
            const int idx = tid + i * kWalker;
            const bool ok = idx < cols4 && row < rows;
            // Dead lanes (columns or rows past the end) load element 0 and replace it by zeros: with dy = 0 they
            // add nothing to any sum whatever xhat comes out of y = 0.  (A choice `ok ? yr[idx] : b[i]` is turned
            // into a choice between two addresses, which puts b into private memory to give it one.)
            const int64_t at = ok ? row * cols4 + idx : 0;
            const float4 vd = load_stream(reinterpret_cast<const float4*>(dy) + at);
            const float4 vy = load_stream(reinterpret_cast<const float4*>(y) + at);
            rd[i] = ok ? vd : make_float4(0.f, 0.f, 0.f, 0.f);
            ry[i] = ok ? vy : make_float4(0.f, 0.f, 0.f, 0.f);
        }
    };
    const int64_t stride = (int64_t)gridDim.x * GROUPS;
    const int64_t first = (int64_t)blockIdx.x * GROUPS + walker;
    // every walker of a workgroup makes the same number of trips (they share barriers)
    const int64_t trips = (rows - (int64_t)blockIdx.x * GROUPS + stride - 1) / stride;
    request(d, xh, first);
    int flip = 0;
    for (int64_t trip = 0; trip < trips; trip++, flip ^= 1) {
        const int64_t row = first + trip * stride;
        const bool live = row < rows;
        request(nd, nxh, row + stride);
        // stored var already holds eps; the backward adds eps once more
        const float rstd = live ? 1.0f / sqrtf(var[row] + eps) : 0.f;
        // optional residual gradient added to dx (dx may be the same buffer):
        // requested here so that its latency hides behind the row reduction
        float4 res[VPT];
        if (residual) {
            const float4* rr = reinterpret_cast<const float4*>(residual) + row * cols4;
#pragma unroll
            for (int i = 0; i < VPT; i++) {
                const int idx = tid + i * kWalker;
                res[i] = (idx < cols4 && live) ? load_stream(rr + idx) : make_float4(0.f, 0.f, 0.f, 0.f);
            }
        }
        float s[2] = {0.f, 0.f};
#pragma unroll
        for (int i = 0; i < VPT; i++) {
            xh[i].x = (xh[i].x - b[i].x) * ginv[i].x;
            xh[i].y = (xh[i].y - b[i].y) * ginv[i].y;
            xh[i].z = (xh[i].z - b[i].z) * ginv[i].z;
            xh[i].w = (xh[i].w - b[i].w) * ginv[i].w;
            acc_b[i].x += d[i].x; acc_b[i].y += d[i].y; acc_b[i].z += d[i].z; acc_b[i].w += d[i].w;
            acc_g[i].x += d[i].x * xh[i].x; acc_g[i].y += d[i].y * xh[i].y;
            acc_g[i].z += d[i].z * xh[i].z; acc_g[i].w += d[i].w * xh[i].w;
            // from here on d holds dxhat = dy * gamma
            d[i].x *= g[i].x; d[i].y *= g[i].y; d[i].z *= g[i].z; d[i].w *= g[i].w;
            s[0] += (d[i].x + d[i].y) + (d[i].z + d[i].w);
            s[1] += (d[i].x * xh[i].x + d[i].y * xh[i].y) + (d[i].z * xh[i].z + d[i].w * xh[i].w);
        }
        // the walker's two row sums: wave butterflies, then its four waves through LDS
        s[0] = wave_sum(s[0]);
        s[1] = wave_sum(s[1]);
        if (lane == 0) {
            lds[flip][walker][wave] = s[0];
            lds[flip][walker][kWaves + wave] = s[1];
        }
        __syncthreads();
        s[0] = s[1] = 0.f;
#pragma unroll
        for (int w = 0; w < kWaves; w++) {
            s[0] += lds[flip][walker][w];
            s[1] += lds[flip][walker][kWaves + w];
        }
        const float m1 = s[0] * inv_cols, m2 = s[1] * inv_cols;
        float4* dxr = reinterpret_cast<float4*>(dx) + row * cols4;
#pragma unroll
        for (int i = 0; i < VPT; i++) {
            const int idx = tid + i * kWalker;
            if (idx < cols4 && live) {
                float4 o;
                o.x = (d[i].x - m1 - xh[i].x * m2) * rstd;
                o.y = (d[i].y - m1 - xh[i].y * m2) * rstd;
                o.z = (d[i].z - m1 - xh[i].z * m2) * rstd;
                o.w = (d[i].w - m1 - xh[i].w * m2) * rstd;
                if (residual) {
                    // dx is rounded to fp32 before the add, as a separate add kernel would see it
                    asm volatile("" : "+v"(o.x), "+v"(o.y), "+v"(o.z), "+v"(o.w));
                    o.x += res[i].x; o.y += res[i].y; o.z += res[i].z; o.w += res[i].w;
                }
                dxr[idx] = o;  // an ordinary store: measured faster here than the streaming form
                if (SUMS) {
                    store4_as16(dx16, row * cols4 + idx, o);   // o as stored, rounded once more
                    float4& ax = acc_x[SUMS ? i : 0];
                    ax.x += o.x; ax.y += o.y; ax.z += o.z; ax.w += o.w;
                }
            }
        }
#pragma unroll
        for (int i = 0; i < VPT; i++) {
            d[i] = nd[i];
            xh[i] = nxh[i];
        }
    }
    // walkers 1.. hand their running sums to walker 0 through LDS, in walker order
    if (GROUPS > 1) {
        __shared__ float4 hand[SUMS ? 3 : 2][VPT][kWalker];
        for (int w = 1; w < GROUPS; w++) {
            __syncthreads();
            if (walker == w) {
#pragma unroll
                for (int i = 0; i < VPT; i++) {
                    hand[0][i][tid] = acc_g[i];
                    hand[1][i][tid] = acc_b[i];
                    if (SUMS) hand[SUMS ? 2 : 0][i][tid] = acc_x[SUMS ? i : 0];
                }
            }
            __syncthreads();
            if (walker == 0) {
#pragma unroll
                for (int i = 0; i < VPT; i++) {
                    const float4 a = hand[0][i][tid], c = hand[1][i][tid];
                    acc_g[i].x += a.x; acc_g[i].y += a.y; acc_g[i].z += a.z; acc_g[i].w += a.w;
                    acc_b[i].x += c.x; acc_b[i].y += c.y; acc_b[i].z += c.z; acc_b[i].w += c.w;
                    if (SUMS) {
                        const float4 e = hand[SUMS ? 2 : 0][i][tid];
                        float4& ax = acc_x[SUMS ? i : 0];
                        ax.x += e.x; ax.y += e.y; ax.z += e.z; ax.w += e.w;
                    }
                }
            }
        }
    }
    if (walker == 0) {
        float4* pg = reinterpret_cast<float4*>(part_dgamma) + (int64_t)blockIdx.x * cols4;
        float4* pb = reinterpret_cast<float4*>(part_dbeta) + (int64_t)blockIdx.x * cols4;
#pragma unroll
        for (int i = 0; i < VPT; i++) {
            const int idx = tid + i * kWalker;
            if (idx < cols4) {
                pg[idx] = acc_g[i];
                pb[idx] = acc_b[i];
                if (SUMS) reinterpret_cast<float4*>(part_dx)[(int64_t)blockIdx.x * cols4 + idx] = acc_x[SUMS ? i : 0];
            }
        }
    }
}

// Any width / alignment: row pass from global memory (dx only).
__global__ __launch_bounds__(kBlock) void ln_bwd_dx_generic(const float* dy, const float* y, const float* gamma,
                                                             const float* beta, const float* var, float* dx,
                                                             int64_t cols, float eps) {
    __shared__ float lds[2 * kWaves];
    const int64_t row = blockIdx.x;
    const float rstd = 1.0f / sqrtf(var[row] + eps);
    float s[2] = {0.f, 0.f};
    for (int64_t c = threadIdx.x; c < cols; c += kBlock) {
        const float dxhat = dy[row * cols + c] * gamma[c];
        const float xhat = (y[row * cols + c] - beta[c]) / add_eps(gamma[c], eps);
        s[0] += dxhat;
        s[1] += dxhat * xhat;
    }
    block_sum<2>(s, lds);
    const float m1 = s[0] / (float)cols, m2 = s[1] / (float)cols;
    for (int64_t c = threadIdx.x; c < cols; c += kBlock) {
        const float dxhat = dy[row * cols + c] * gamma[c];
        const float xhat = (y[row * cols + c] - beta[c]) / add_eps(gamma[c], eps);
        dx[row * cols + c] = (dxhat - m1 - xhat * m2) * rstd;
    }
}

// Any width: partial column sums over a strip of rows, one column per thread.
__global__ __launch_bounds__(kBlock) void ln_bwd_cols_generic(const float* dy, const float* y, const float* gamma,
                                                               const float* beta, float* part_dgamma,
                                                               float* part_dbeta, int64_t rows, int64_t cols,
                                                               int rows_per_block, float eps) {
    const int64_t c = (int64_t)blockIdx.x * kBlock + threadIdx.x;
    if (c >= cols) return;
    const float ginv = 1.0f / add_eps(gamma[c], eps), b = beta[c];
    const int64_t r0 = (int64_t)blockIdx.y * rows_per_block;
    const int64_t r1 = r0 + rows_per_block < rows ? r0 + rows_per_block : rows;
    float sg = 0.f, sb = 0.f;
    for (int64_t r = r0; r < r1; r++) {
        const float d = dy[r * cols + c];
        sb += d;
        sg += d * ((y[r * cols + c] - b) * ginv);
    }
    part_dgamma[(int64_t)blockIdx.y * cols + c] = sg;
    part_dbeta[(int64_t)blockIdx.y * cols + c] = sb;
}

// dgamma[c] = sum_p part_dgamma[p][c] (and dbeta likewise), fixed order.
// blockDim = (64 columns, 4 slices of partials); slices are combined in LDS.
__global__ __launch_bounds__(kBlock) void ln_bwd_finalize(const float* part_dgamma, const float* part_dbeta,
                                                           float* dgamma, float* dbeta, int parts, int64_t cols,
                                                           float scale) {
    __shared__ float lg[4][64], lb[4][64];
    const int cx = threadIdx.x & 63, sl = threadIdx.x >> 6;
    const int64_t c = (int64_t)blockIdx.x * 64 + cx;
    float sg = 0.f, sb = 0.f;
    if (c < cols) {
        for (int p = sl; p < parts; p += 4) {
            sg += part_dgamma[(int64_t)p * cols + c];
            sb += part_dbeta[(int64_t)p * cols + c];
        }
    }
    lg[sl][cx] = sg;
    lb[sl][cx] = sb;
    __syncthreads();
    if (sl == 0 && c < cols) {
        dgamma[c] = ((lg[0][cx] + lg[1][cx]) + (lg[2][cx] + lg[3][cx])) * scale;
        dbeta[c] = ((lb[0][cx] + lb[1][cx]) + (lb[2][cx] + lb[3][cx])) * scale;
    }
}

// The same sums for the register path's partials (cols % 4 == 0, 16-byte
// aligned): 1024 threads = 16 column quads x 64 slices of partials, so that
// all of a workgroup's loads are in flight at once; slices are combined in LDS
// in a fixed order.
constexpr int kFinSlices = 64;
struct FinalSums {
    float4* out[3];   // dgamma, dbeta and (or null) the column sums of dx
};
// blockIdx.y picks the array: the partial arrays lie one after the other, parts x cols4 quads each
__global__ __launch_bounds__(1024) void ln_bwd_finalize_x4(const float4* __restrict__ partials, FinalSums sums,
                                                           int parts, int cols4, float scale) {
    __shared__ float4 ls[kFinSlices][16];
    const float4* __restrict__ part = partials + (int64_t)blockIdx.y * parts * cols4;
    float4* __restrict__ out = sums.out[blockIdx.y];
    const int q = threadIdx.x & 15, sl = threadIdx.x >> 4;
    const int c4 = blockIdx.x * 16 + q;
    float4 s = make_float4(0.f, 0.f, 0.f, 0.f);
    if (c4 < cols4) {
#pragma unroll 8
        for (int p = sl; p < parts; p += kFinSlices) {
            const float4 a = part[(int64_t)p * cols4 + c4];
            s.x += a.x; s.y += a.y; s.z += a.z; s.w += a.w;
        }
    }
    ls[sl][q] = s;
    __syncthreads();
    if (sl < 8) {
        for (int k = sl + 8; k < kFinSlices; k += 8) {
            const float4 a = ls[k][q];
            s.x += a.x; s.y += a.y; s.z += a.z; s.w += a.w;
        }
        ls[sl][q] = s;
    }
    __syncthreads();
    if (sl == 0 && c4 < cols4) {
        for (int k = 1; k < 8; k++) {
            const float4 a = ls[k][q];
            s.x += a.x; s.y += a.y; s.z += a.z; s.w += a.w;
        }
        out[c4] = make_float4(s.x * scale, s.y * scale, s.z * scale, s.w * scale);
    }
}

// Persistent workgroups of the register path: one per CU on a 256-CU part, two
// row walkers each (512 rows in flight chip-wide, 256 partial row pairs).
constexpr int kBwdWalkers = 2;
int bwd_parts(int64_t rows) {
    int64_t p = 256;
    const int64_t most = (rows + kBwdWalkers - 1) / kBwdWalkers;
    if (p > most) p = most;
    return (int)(p < 1 ? 1 : p);
}

int strip_rows(int64_t rows) {
    int64_t rpb = (rows + 127) / 128;
    if (rpb < 8) rpb = 8;
    return (int)rpb;
}

bool regs_path_ok(int64_t cols, const void* a, const void* b, const void* c, const void* d, const void* e) {
    return cols % 4 == 0 && cols / 4 <= kBlock * 8 && aligned16(a) && aligned16(b) && aligned16(c) &&
           aligned16(d) && aligned16(e);
}

}  // namespace

namespace {
int layernorm_fwd_launch(const float* x, const float* gamma, const float* beta, float* y, Copy16 y16, float* mean,
                         float* var, int64_t rows, int64_t cols, float eps, hipStream_t st) {
    const unsigned grid = (unsigned)rows;
    if (regs_path_ok(cols, x, gamma, beta, y, y)) {
        const int cols4 = (int)(cols / 4);
        const float inv = 1.0f / (float)cols;
        const int vpt = (cols4 + kBlock - 1) / kBlock;
        if (vpt <= 1)
            ln_fwd_regs<1><<<grid, kBlock, 0, st>>>(x, gamma, beta, y, mean, var, cols4, eps, inv, y16);
        else if (vpt <= 2)
            ln_fwd_regs<2><<<grid, kBlock, 0, st>>>(x, gamma, beta, y, mean, var, cols4, eps, inv, y16);
        else if (vpt <= 4)
            ln_fwd_regs<4><<<grid, kBlock, 0, st>>>(x, gamma, beta, y, mean, var, cols4, eps, inv, y16);
        else
            ln_fwd_regs<8><<<grid, kBlock, 0, st>>>(x, gamma, beta, y, mean, var, cols4, eps, inv, y16);
    } else {
        if (y16.base) return BR_ERR_TODO;  // the copy is only produced by the register path
        ln_fwd_generic<<<grid, kBlock, 0, st>>>(x, gamma, beta, y, mean, var, cols, eps);
    }
    BR_HIP_LAUNCH_CHECK();
    return BR_OK;
}
}  // namespace

// ---- scratch of the entry point that allocates nothing ---------------------
// Partial sums go to a file-scope device array instead of a caller workspace.
// Every GPU the library runs on holds its own copy of the array (until the
// process ends) at its own address; the address is looked up once per device,
// with that device current, and only that pointer is ever handed to kernels.
// (No `used` attribute on the array: with it the compiler keeps the symbol
// internal to the code object and the runtime's lookup by name cannot find it.)
constexpr size_t kStaticScratchBytes = (size_t)16 << 20;
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];

namespace {
constexpr int kMaxDevices = 64;
std::mutex g_scratch_mutex;
void* g_scratch_ptr[kMaxDevices] = {};

// Device address of `scratch` on the current device; hipError_t on failure.
int static_scratch(void** out) {
    int dev = -1;
    BR_HIP_TRY(hipGetDevice(&dev));
    if (dev < 0 || dev >= kMaxDevices) return BR_ERR_ATTR;
    std::lock_guard<std::mutex> lock(g_scratch_mutex);
    if (!g_scratch_ptr[dev]) {
        void* p = nullptr;
        BR_HIP_TRY(hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)));
        if (!p) return (int)hipErrorInvalidSymbol;
        g_scratch_ptr[dev] = p;
    }
    *out = g_scratch_ptr[dev];
    return BR_OK;
}
}  // namespace

extern "C" {

int br_hip_layernorm_fwd(const float* x, const float* gamma, const float* beta, float* y, float* mean,
                         float* var, int64_t rows, int64_t cols, float eps, br_stream_t stream) {
    if (rows < 0 || cols <= 0 || rows > 0x7fffffff) return BR_ERR_ATTR;
    if (rows == 0) return BR_OK;
    if (!x || !gamma || !beta) return BR_ERR_INPUT;
    if (!y) return BR_ERR_OUTPUT;
    return layernorm_fwd_launch(x, gamma, beta, y, Copy16{nullptr, 0}, mean, var, rows, cols, eps, as_stream(stream));
}

int br_hip_layernorm_fwd_copy16(const float* x, const float* gamma, const float* beta, float* y, void* y16,
                                int y16_dtype, float* mean, float* var, int64_t rows, int64_t cols, float eps,
                                br_stream_t stream) {
    if (rows < 0 || cols <= 0 || rows > 0x7fffffff) return BR_ERR_ATTR;
    if (rows == 0) return BR_OK;
    if (!x || !gamma || !beta) return BR_ERR_INPUT;
    if (!y || !y16) return BR_ERR_OUTPUT;
    if (!copy16_ok(y16, y16_dtype) || !regs_path_ok(cols, x, gamma, beta, y, y)) return BR_ERR_TODO;
    return layernorm_fwd_launch(x, gamma, beta, y, Copy16{y16, y16_dtype == BR_BF16}, mean, var, rows, cols, eps,
                                as_stream(stream));
}

size_t br_hip_layernorm_bwd_workspace(int64_t rows, int64_t cols) {
    if (rows <= 0 || cols <= 0) return 0;
    int64_t parts = bwd_parts(rows);
    const int64_t strips = (rows + strip_rows(rows) - 1) / strip_rows(rows);
    if (strips > parts) parts = strips;
    return (size_t)(2 * parts * cols) * sizeof(float);
}

size_t br_hip_layernorm_bwd_sums_workspace(int64_t rows, int64_t cols) {
    return br_hip_layernorm_bwd_workspace(rows, cols) / 2 * 3;   // a third partial array
}

// dx16 / dx_sum (both or neither): the 16-bit copy and the column sums of dx, register path only
static int layernorm_bwd_impl(const float* dy, const float* y, const float* gamma, const float* beta,
                              const float* var, const float* residual, float* dgamma, float* dbeta, float* dx,
                              int64_t rows, int64_t cols, float eps, float param_scale, void* workspace,
                              size_t workspace_bytes, br_stream_t stream, void* dx16 = nullptr, int dx16_dtype = 0,
                              float* dx_sum = nullptr) {
    if (rows < 0 || cols <= 0 || rows > 0x7fffffff) return BR_ERR_ATTR;
    if (!dgamma || !dbeta) return BR_ERR_OUTPUT;
    const bool sums = dx_sum != nullptr;
    if (rows == 0) {
        int rc = br_hip_fill(dgamma, BR_F32, 0.f, cols, stream);
        if (!rc && sums) rc = br_hip_fill(dx_sum, BR_F32, 0.f, cols, stream);
        return rc ? rc : br_hip_fill(dbeta, BR_F32, 0.f, cols, stream);
    }
    if (!dy || !y || !gamma || !beta || !var) return BR_ERR_INPUT;
    if (!dx) return BR_ERR_OUTPUT;
    const size_t need = sums ? br_hip_layernorm_bwd_sums_workspace(rows, cols) : br_hip_layernorm_bwd_workspace(rows, cols);
    if (!workspace || workspace_bytes < need) return BR_ERR_ATTR;
    hipStream_t st = as_stream(stream);
    int parts;
    float* part_g = (float*)workspace;
    const bool regs = regs_path_ok(cols, dy, y, gamma, beta, dx) && aligned16(workspace) &&
                      (!residual || aligned16(residual));
    if (residual && !regs) return BR_ERR_TODO;  // only the register path adds the residual
    const int cols4 = (int)(cols / 4);
    const int vpt = (cols4 + kBlock - 1) / kBlock;
    // ... and the sums: up to 4096 columns (wider rows run one walker with every register taken), all of dgamma,
    // dbeta and the sums aligned for the finalize pass that handles three arrays
    if (sums && !(regs && vpt <= 4 && aligned16(dgamma) && aligned16(dbeta) && aligned16(dx_sum) &&
                  copy16_ok(dx16, dx16_dtype)))
        return BR_ERR_TODO;
    if (regs) {
        parts = bwd_parts(rows);
        float* part_b = part_g + (int64_t)parts * cols;
        float* part_x = part_b + (int64_t)parts * cols;
        const float inv = 1.0f / (float)cols;
        constexpr int G = kBwdWalkers;
        const Copy16 c16{dx16, dx16_dtype == BR_BF16};
#define BR_LN_BWD(V, W)                                                                                              \
    do {                                                                                                             \
        if (sums)                                                                                                    \
            ln_bwd_regs<V, W, true><<<parts, kWalker * W, 0, st>>>(dy, y, gamma, beta, var, dx, part_g, part_b, rows, \
                                                                   cols4, eps, inv, residual, part_x, c16);          \
        else                                                                                                         \
            ln_bwd_regs<V, W><<<parts, kWalker * W, 0, st>>>(dy, y, gamma, beta, var, dx, part_g, part_b, rows,      \
                                                             cols4, eps, inv, residual);                             \
    } while (0)
        // Rows wider than 4096 floats keep 8 quads per thread in flight twice over; with two walkers (512
        // threads, 256 registers per wave) that spills, so they run one walker per workgroup.
        if (vpt <= 1) BR_LN_BWD(1, G);
        else if (vpt <= 2) BR_LN_BWD(2, G);
        else if (vpt <= 4) BR_LN_BWD(4, G);
        else ln_bwd_regs<8, 1><<<parts, kWalker, 0, st>>>(dy, y, gamma, beta, var, dx, part_g, part_b, rows, cols4, eps,
                                                          inv, residual);
#undef BR_LN_BWD
        BR_HIP_LAUNCH_CHECK();
        if (aligned16(dgamma) && aligned16(dbeta)) {
            const FinalSums out{{reinterpret_cast<float4*>(dgamma), reinterpret_cast<float4*>(dbeta),
                                 reinterpret_cast<float4*>(dx_sum)}};
            ln_bwd_finalize_x4<<<dim3((unsigned)((cols4 + 15) / 16), sums ? 3u : 2u), 1024, 0, st>>>(
                reinterpret_cast<const float4*>(part_g), out, parts, cols4, param_scale);
        } else {
            ln_bwd_finalize<<<(unsigned)((cols + 63) / 64), kBlock, 0, st>>>(part_g, part_b, dgamma, dbeta, parts, cols, param_scale);
        }
    } else {
        const int rpb = strip_rows(rows);
        parts = (int)((rows + rpb - 1) / rpb);
        float* part_b = part_g + (int64_t)parts * cols;
        dim3 grid((unsigned)((cols + kBlock - 1) / kBlock), (unsigned)parts);
        // column sums first: they read dy, which dx must not have replaced yet
        ln_bwd_cols_generic<<<grid, kBlock, 0, st>>>(dy, y, gamma, beta, part_g, part_b, rows, cols, rpb, eps);
        BR_HIP_LAUNCH_CHECK();
        ln_bwd_dx_generic<<<(unsigned)rows, kBlock, 0, st>>>(dy, y, gamma, beta, var, dx, cols, eps);
        BR_HIP_LAUNCH_CHECK();
        ln_bwd_finalize<<<(unsigned)((cols + 63) / 64), kBlock, 0, st>>>(part_g, part_b, dgamma, dbeta, parts, cols, param_scale);
    }
    BR_HIP_LAUNCH_CHECK();
    return BR_OK;
}

int br_hip_layernorm_bwd(const float* dy, const float* y, const float* gamma, const float* beta,
                         const float* var, float* dgamma, float* dbeta, float* dx, int64_t rows, int64_t cols,
                         float eps, float param_scale, void* workspace, size_t workspace_bytes, br_stream_t stream) {
    return layernorm_bwd_impl(dy, y, gamma, beta, var, nullptr, dgamma, dbeta, dx, rows, cols, eps, param_scale,
                              workspace, workspace_bytes, stream);
}

// ---- the entry point that allocates nothing -------------------------------
size_t br_hip_layernorm_bwd_static_limit(void) { return kStaticScratchBytes; }

int br_hip_layernorm_bwd_static(const float* dy, const float* y, const float* gamma, const float* beta,
                                const float* var, float* dgamma, float* dbeta, float* dx, int64_t rows, int64_t cols,
                                float eps, float param_scale, br_stream_t stream) {
    if (rows < 0 || cols <= 0 || rows > 0x7fffffff) return BR_ERR_ATTR;
    const size_t need = br_hip_layernorm_bwd_workspace(rows, cols);
    if (need > kStaticScratchBytes) return BR_ERR_SCRATCH;
    void* ws = nullptr;
    const int rc = static_scratch(&ws);
    if (rc != BR_OK) return rc;
    // every partial the finalize pass reads is written by the main pass of the
    // same call, so nothing in the array has to start at zero
    return layernorm_bwd_impl(dy, y, gamma, beta, var, nullptr, dgamma, dbeta, dx, rows, cols, eps, param_scale, ws,
                              kStaticScratchBytes, stream);
}

int br_hip_layernorm_bwd_residual_sums(const float* dy, const float* y, const float* gamma, const float* beta,
                                       const float* var, const float* residual, float* dgamma, float* dbeta,
                                       float* dx, void* dx16, int dx16_dtype, float* dx_sum, int64_t rows,
                                       int64_t cols, float eps, float param_scale, void* workspace,
                                       size_t workspace_bytes, br_stream_t stream) {
    if (rows > 0 && !residual) return BR_ERR_INPUT;
    if (!dx16 || !dx_sum) return BR_ERR_OUTPUT;
    if (rows == 0) residual = nullptr;
    return layernorm_bwd_impl(dy, y, gamma, beta, var, residual, dgamma, dbeta, dx, rows, cols, eps, param_scale,
                              workspace, workspace_bytes, stream, dx16, dx16_dtype, dx_sum);
}

int br_hip_layernorm_bwd_residual(const float* dy, const float* y, const float* gamma, const float* beta,
                                  const float* var, const float* residual, float* dgamma, float* dbeta, float* dx,
                                  int64_t rows, int64_t cols, float eps, float param_scale, void* workspace,
                                  size_t workspace_bytes, br_stream_t stream) {
    if (rows > 0 && !residual) return BR_ERR_INPUT;
    if (rows == 0) residual = nullptr;
    return layernorm_bwd_impl(dy, y, gamma, beta, var, residual, dgamma, dbeta, dx, rows, cols, eps, param_scale,
                              workspace, workspace_bytes, stream);
}

}  // extern "C"
