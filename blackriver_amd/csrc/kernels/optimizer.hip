// AdamW parameter update for gfx950: one pass over (param, grad, m, v), all
// arithmetic in fp32.  HBM-bound: 16 B read + 12 B written per fp32 parameter;
// a 16-bit parameter with an fp32 master copy reads 16 B and writes 14 B.
#include "common.hpp"

using namespace brk;

namespace {

constexpr int kBlock = 256;

struct AdamW {
    float lr, beta1, beta2, eps, decay;  // decay = 1 - lr * weight_decay
    float step_size;                     // lr / (1 - beta1^t)
    float sqrt_bc2;                      // sqrt(1 - beta2^t)
};

// The update of torch.optim.AdamW (decoupled weight decay), operation for
// operation: decay the parameter, update both moments, then
// p -= step_size * (m / (sqrt(v) / sqrt(1 - beta2^t) + eps)).
__device__ __forceinline__ float adamw_one(float p, float g, float& m, float& v, const AdamW& a) {
    p = p * a.decay;
    m = m + (g - m) * (1.0f - a.beta1);                  // lerp, as torch does it
    v = v * a.beta2 + ((1.0f - a.beta2) * g) * g;
    const float denom = sqrtf(v) / a.sqrt_bc2 + a.eps;
    return p - a.step_size * (m / denom);
}

template <typename T>
__device__ __forceinline__ float to_f32(T x);
template <>
__device__ __forceinline__ float to_f32<float>(float x) { return x; }
template <>
__device__ __forceinline__ float to_f32<__half>(__half x) { return __half2float(x); }
template <>
__device__ __forceinline__ float to_f32<__hip_bfloat16>(__hip_bfloat16 x) { return __bfloat162float(x); }
template <typename T>
__device__ __forceinline__ T from_f32(float x);
template <>
__device__ __forceinline__ float from_f32<float>(float x) { return x; }
template <>
__device__ __forceinline__ __half from_f32<__half>(float x) { return __float2half_rn(x); }
template <>
__device__ __forceinline__ __hip_bfloat16 from_f32<__hip_bfloat16>(float x) { return __float2bfloat16(x); }

// master == nullptr: the parameter itself is the state (read as T, written as T).
// master != nullptr: the fp32 master copy is updated and `param` receives its rounding.
// The contraction barrier keeps `next` an fp32 value before it is rounded to T.
template <typename T, int VEC>
__global__ __launch_bounds__(kBlock) void adamw_kernel(T* param, float* master, const float* __restrict__ grad,
                                                        float* m, float* v, int64_t n, AdamW a) {
    const int64_t stride = (int64_t)gridDim.x * kBlock * VEC;
    for (int64_t base = ((int64_t)blockIdx.x * kBlock + threadIdx.x) * VEC; base < n; base += stride) {
        if (VEC == 4) {
            const float4 g4 = load_stream(reinterpret_cast<const float4*>(grad + base));
            float4 m4 = load_stream(reinterpret_cast<const float4*>(m + base));
            float4 v4 = load_stream(reinterpret_cast<const float4*>(v + base));
            float p[4];
            if (master) {
                const float4 p4 = load_stream(reinterpret_cast<const float4*>(master + base));
                p[0] = p4.x; p[1] = p4.y; p[2] = p4.z; p[3] = p4.w;
            } else {
#pragma unroll
                for (int j = 0; j < 4; j++) p[j] = to_f32<T>(param[base + j]);
            }
            p[0] = adamw_one(p[0], g4.x, m4.x, v4.x, a);
            p[1] = adamw_one(p[1], g4.y, m4.y, v4.y, a);
            p[2] = adamw_one(p[2], g4.z, m4.z, v4.z, a);
            p[3] = adamw_one(p[3], g4.w, m4.w, v4.w, a);
            asm volatile("" : "+v"(p[0]), "+v"(p[1]), "+v"(p[2]), "+v"(p[3]));
            store_stream(reinterpret_cast<float4*>(m + base), m4);
            store_stream(reinterpret_cast<float4*>(v + base), v4);
            if (master) store_stream(reinterpret_cast<float4*>(master + base), make_float4(p[0], p[1], p[2], p[3]));
#pragma unroll
            for (int j = 0; j < 4; j++) param[base + j] = from_f32<T>(p[j]);
        } else {
            float mm = m[base], vv = v[base];
            float p = master ? master[base] : to_f32<T>(param[base]);
            p = adamw_one(p, grad[base], mm, vv, a);
            asm volatile("" : "+v"(p));
            m[base] = mm;
            v[base] = vv;
            if (master) master[base] = p;
            param[base] = from_f32<T>(p);
        }
    }
}

template <typename T>
int launch_adamw(void* param, float* master, const float* grad, float* m, float* v, int64_t n, const AdamW& a,
                 hipStream_t st) {
    const bool vec = n % 4 == 0 && aligned16(grad) && aligned16(m) && aligned16(v) &&
                     (!master || aligned16(master)) && (reinterpret_cast<uintptr_t>(param) % (4 * sizeof(T)) == 0);
    if (vec)
        adamw_kernel<T, 4><<<grid_for(n / 4, kBlock), kBlock, 0, st>>>((T*)param, master, grad, m, v, n, a);
    else
        adamw_kernel<T, 1><<<grid_for(n, kBlock), kBlock, 0, st>>>((T*)param, master, grad, m, v, n, a);
    BR_HIP_LAUNCH_CHECK();
    return BR_OK;
}

}  // namespace

extern "C" {

int br_hip_adamw(void* param, int param_dtype, float* master, const float* grad, float* m, float* v, int64_t n,
                 float lr, float beta1, float beta2, float eps, float weight_decay, int64_t step,
                 br_stream_t stream) {
    if (n < 0 || step < 1 || !(beta1 >= 0.f && beta1 < 1.f) || !(beta2 >= 0.f && beta2 < 1.f)) return BR_ERR_ATTR;
    if (n == 0) return BR_OK;
    if (!grad) return BR_ERR_INPUT;
    if (!param || !m || !v) return BR_ERR_OUTPUT;
    if (param_dtype == BR_F32 && master) return BR_ERR_ATTR;  // an fp32 parameter is its own master copy
    AdamW a;
    a.lr = lr;
    a.beta1 = beta1;
    a.beta2 = beta2;
    a.eps = eps;
    a.decay = 1.0f - lr * weight_decay;
    // bias corrections in fp64 on the host, as torch computes them for a python-number step
    const double bc1 = 1.0 - pow((double)beta1, (double)step);
    const double bc2 = 1.0 - pow((double)beta2, (double)step);
    a.step_size = (float)((double)lr / bc1);
    a.sqrt_bc2 = (float)sqrt(bc2);
    hipStream_t st = as_stream(stream);
    switch (param_dtype) {
        case BR_F32: return launch_adamw<float>(param, nullptr, grad, m, v, n, a, st);
        case BR_F16: return launch_adamw<__half>(param, master, grad, m, v, n, a, st);
        case BR_BF16: return launch_adamw<__hip_bfloat16>(param, master, grad, m, v, n, a, st);
        default: return BR_ERR_TODO;
    }
}

}  // extern "C"
