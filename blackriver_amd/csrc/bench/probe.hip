// Calibration probe: the rate of a bare v_mfma_f32_32x32x16_f16 loop (no
// memory traffic at all) with operands of zeros or of random values.  On
// MI355X the two differ by a third -- the clock follows the switching activity
// of the data -- so a GEMM on real data has to be read against the second
// figure as well as against the nominal peak.
//
// Built into libbr_probe.so, which only bench.py loads: a measuring aid, not
// part of the kernel library or of its C ABI.
#include <hip/hip_runtime.h>
#include <hip/hip_fp16.h>
#include <stdint.h>

namespace {

typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));

__device__ __forceinline__ unsigned mix(unsigned x) {
    x ^= x >> 16; x *= 0x7feb352du;
    x ^= x >> 15; x *= 0x846ca68bu;
    return x ^ (x >> 16);
}

// 8 waves per workgroup; every wave runs 64 MFMAs per pass over 8 accumulators
// and 8 x 8 operand pairs.
template <bool RANDOM>
__global__ __launch_bounds__(512) void mfma_loop_kernel(float* out, int passes) {
    f16x8 a[8], b[8];
#pragma unroll
    for (int p = 0; p < 8; p++) {
#pragma unroll
        for (int i = 0; i < 8; i++) {
            const unsigned h = mix(threadIdx.x * 64 + p * 8 + i + blockIdx.x * 77777u);
            a[p][i] = RANDOM ? (_Float16)(((h & 0xffff) / 65536.0f - 0.5f) * 3.4f) : (_Float16)0.f;
            b[p][i] = RANDOM ? (_Float16)(((h >> 16) / 65536.0f - 0.5f) * 3.4f) : (_Float16)0.f;
        }
        asm volatile("" : "+v"(a[p]));
        asm volatile("" : "+v"(b[p]));
    }
    f32x16 c[8];
#pragma unroll
    for (int j = 0; j < 8; j++)
#pragma unroll
        for (int i = 0; i < 16; i++) c[j][i] = 0.f;
    for (int it = 0; it < passes; it++) {
#pragma unroll
        for (int r = 0; r < 8; r++)
#pragma unroll
            for (int j = 0; j < 8; j++)
                c[j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a[j], b[(j + r) & 7], c[j], 0, 0, 0);
    }
    float s = 0.f;
#pragma unroll
    for (int j = 0; j < 8; j++)
#pragma unroll
        for (int i = 0; i < 16; i++) s += c[j][i];
    out[(size_t)blockIdx.x * 512 + threadIdx.x] = s;
}

}  // namespace

#define BR_HIP_TRY(expr)                                \
    do {                                                \
        hipError_t br_err_ = (expr);                    \
        if (br_err_ != hipSuccess) return (int)br_err_; \
    } while (0)

// Returns 0, a hipError_t, or -4 for bad arguments.  scratch: at least 131072
// floats of device memory; *tflops receives the rate of the timed launch.
extern "C" int br_probe_mfma_f16(int random_operands, int passes, float* scratch, int64_t scratch_floats,
                                 double* tflops, void* stream) {
    const int blocks = 256;
    if (passes < 1 || !scratch || scratch_floats < (int64_t)blocks * 512 || !tflops) return -4;
    hipStream_t st = reinterpret_cast<hipStream_t>(stream);
    hipEvent_t e0, e1;
    BR_HIP_TRY(hipEventCreate(&e0));
    BR_HIP_TRY(hipEventCreate(&e1));
    auto launch = [&](int n) {
        if (random_operands) mfma_loop_kernel<true><<<blocks, 512, 0, st>>>(scratch, n);
        else mfma_loop_kernel<false><<<blocks, 512, 0, st>>>(scratch, n);
    };
    launch(passes / 10 + 1);  // warm-up
    BR_HIP_TRY(hipEventRecord(e0, st));
    launch(passes);
    BR_HIP_TRY(hipEventRecord(e1, st));
    BR_HIP_TRY(hipEventSynchronize(e1));
    float ms = 0.f;
    BR_HIP_TRY(hipEventElapsedTime(&ms, e0, e1));
    BR_HIP_TRY(hipEventDestroy(e0));
    BR_HIP_TRY(hipEventDestroy(e1));
    BR_HIP_TRY(hipGetLastError());
    *tflops = (double)blocks * 8.0 * passes * 64.0 * 2.0 * 32 * 32 * 16 / ((double)ms * 1e-3) / 1e12;
    return 0;
}
