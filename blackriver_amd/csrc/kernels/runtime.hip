// Runtime plumbing of the C ABI: device selection, memory, streams, events
// and copies.  Thin pass-throughs to the HIP runtime so the C++ host above the
// ABI never includes a HIP header.
#include "common.hpp"

#include <math.h>

using namespace brk;

namespace {

// Byte fill as a kernel rather than hipMemsetAsync, so that a caller may record
// it into a HIP graph like any other launch: 16-byte stores over the aligned
// middle, single bytes at both ends.
__global__ __launch_bounds__(256) void memset_kernel(unsigned char* dst, unsigned char value, size_t bytes) {
    const size_t head = (16 - (reinterpret_cast<uintptr_t>(dst) & 15)) & 15;
    const size_t lead = head < bytes ? head : bytes;
    const size_t vecs = (bytes - lead) / 16;
    const size_t tid = (size_t)blockIdx.x * 256 + threadIdx.x, stride = (size_t)gridDim.x * 256;
    const unsigned w = value * 0x01010101u;
    uint4* mid = reinterpret_cast<uint4*>(dst + lead);
    for (size_t i = tid; i < vecs; i += stride) mid[i] = make_uint4(w, w, w, w);
    const size_t tail0 = lead + vecs * 16;
    for (size_t i = tid; i < lead; i += stride) dst[i] = value;
    for (size_t i = tail0 + tid; i < bytes; i += stride) dst[i] = value;
}

}  // namespace

extern "C" {

int br_hip_device_count(int* count) {
    if (!count) return BR_ERR_OUTPUT;
    BR_HIP_TRY(hipGetDeviceCount(count));
    return BR_OK;
}

int br_hip_set_device(int device) {
    BR_HIP_TRY(hipSetDevice(device));
    return BR_OK;
}

const char* br_hip_error_string(int code) {
    switch (code) {
        case BR_OK: return "ok";
        case BR_ERR_TODO: return "br_hip: combination not implemented";
        case BR_ERR_INPUT: return "br_hip: bad input argument";
        case BR_ERR_OUTPUT: return "br_hip: bad output argument";
        case BR_ERR_ATTR: return "br_hip: bad attribute or size";
        case BR_ERR_SCRATCH: return "br_hip: problem too large for the built-in scratch buffer of an allocation-free entry";
        default: break;
    }
    if (code > 0) return hipGetErrorString((hipError_t)code);
    return "br_hip: unknown error";
}

int br_hip_malloc(void** ptr, size_t bytes) {
    if (!ptr) return BR_ERR_OUTPUT;
    BR_HIP_TRY(hipMalloc(ptr, bytes ? bytes : 1));
    return BR_OK;
}

int br_hip_free(void* ptr) {
    BR_HIP_TRY(hipFree(ptr));
    return BR_OK;
}

int br_hip_host_malloc(void** ptr, size_t bytes) {
    if (!ptr) return BR_ERR_OUTPUT;
    BR_HIP_TRY(hipHostMalloc(ptr, bytes ? bytes : 1, hipHostMallocDefault));
    return BR_OK;
}

int br_hip_host_free(void* ptr) {
    BR_HIP_TRY(hipHostFree(ptr));
    return BR_OK;
}

int br_hip_stream_create(br_stream_t* stream) {
    if (!stream) return BR_ERR_OUTPUT;
    hipStream_t s;
    BR_HIP_TRY(hipStreamCreate(&s));  // default priority on purpose
    *stream = (br_stream_t)s;
    return BR_OK;
}

int br_hip_stream_destroy(br_stream_t stream) {
    BR_HIP_TRY(hipStreamDestroy(as_stream(stream)));
    return BR_OK;
}

int br_hip_stream_sync(br_stream_t stream) {
    BR_HIP_TRY(hipStreamSynchronize(as_stream(stream)));
    return BR_OK;
}

int br_hip_event_create(br_event_t* event) {
    if (!event) return BR_ERR_OUTPUT;
    hipEvent_t e;
    BR_HIP_TRY(hipEventCreate(&e));
    *event = (br_event_t)e;
    return BR_OK;
}

int br_hip_event_destroy(br_event_t event) {
    BR_HIP_TRY(hipEventDestroy((hipEvent_t)event));
    return BR_OK;
}

int br_hip_event_record(br_event_t event, br_stream_t stream) {
    BR_HIP_TRY(hipEventRecord((hipEvent_t)event, as_stream(stream)));
    return BR_OK;
}

int br_hip_event_sync(br_event_t event) {
    BR_HIP_TRY(hipEventSynchronize((hipEvent_t)event));
    return BR_OK;
}

int br_hip_event_elapsed_ms(br_event_t start, br_event_t stop, float* ms) {
    if (!ms) return BR_ERR_OUTPUT;
    BR_HIP_TRY(hipEventElapsedTime(ms, (hipEvent_t)start, (hipEvent_t)stop));
    return BR_OK;
}

int br_hip_memcpy_h2d(void* dst, const void* src, size_t bytes, br_stream_t stream) {
    if (bytes == 0) return BR_OK;
    BR_HIP_TRY(hipMemcpyAsync(dst, src, bytes, hipMemcpyHostToDevice, as_stream(stream)));
    return BR_OK;
}

int br_hip_memcpy_d2h(void* dst, const void* src, size_t bytes, br_stream_t stream) {
    if (bytes == 0) return BR_OK;
    BR_HIP_TRY(hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToHost, as_stream(stream)));
    return BR_OK;
}

int br_hip_memcpy_d2d(void* dst, const void* src, size_t bytes, br_stream_t stream) {
    if (bytes == 0 || dst == src) return BR_OK;
    BR_HIP_TRY(hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToDevice, as_stream(stream)));
    return BR_OK;
}

int br_hip_memset(void* dst, int byte_value, size_t bytes, br_stream_t stream) {
    if (bytes == 0) return BR_OK;
    if (!dst) return BR_ERR_OUTPUT;
    memset_kernel<<<grid_for((int64_t)(bytes / 16 + 1), 256), 256, 0, as_stream(stream)>>>(
        static_cast<unsigned char*>(dst), (unsigned char)byte_value, bytes);
    BR_HIP_LAUNCH_CHECK();
    return BR_OK;
}

int br_hip_alibi_slopes(double* slopes_host, int64_t heads) {
    if (!slopes_host) return BR_ERR_OUTPUT;
    if (heads <= 0) return BR_ERR_ATTR;
    // base = 2^(-2^(3 - log2(heads))); slope_h = base^(h+1), in fp64
    double base = 3.0 - log2((double)heads);
    base = -1.0 * pow(2.0, base);
    base = pow(2.0, base);
    for (int64_t h = 0; h < heads; h++) slopes_host[h] = pow(base, (double)(h + 1) * 1.0);
    return BR_OK;
}

}  // extern "C"
