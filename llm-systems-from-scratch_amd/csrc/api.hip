// Error bookkeeping and version string of the C ABI.
#include <hip/hip_runtime.h>
#include <string.h>

#include "launch.hpp"

static thread_local char g_last_error[256] = "";

int set_error(int code, const char* msg) {
    strncpy(g_last_error, msg ? msg : "", sizeof(g_last_error) - 1);
    g_last_error[sizeof(g_last_error) - 1] = '\0';
    return code;
}

extern "C" const char* mi355_last_error(void) { return g_last_error; }

extern "C" const char* mi355_version(void) { return "mi355attn 0.1 (gfx950)"; }

// Plain device-to-device copy of known size: the yardstick that HBM traffic counters
// (FETCH_SIZE / WRITE_SIZE) of the attention kernels are scaled by.
__global__ __launch_bounds__(256) void calib_copy_kernel(const uint4* __restrict__ src, uint4* __restrict__ dst,
                                                         size_t n) {
    size_t i = blockIdx.x * (size_t)blockDim.x + threadIdx.x;
    const size_t stride = (size_t)gridDim.x * blockDim.x;
    for (; i < n; i += stride) dst[i] = src[i];
}

extern "C" int mi355_calib_copy(const void* src, void* dst, size_t bytes, void* stream) {
    if (!src || !dst || (bytes & 15) || (((uintptr_t)src | (uintptr_t)dst) & 15))
        return set_error(MI355_EINVAL, "calib_copy: pointers and size must be 16-byte aligned");
    if (bytes == 0) return MI355_OK;
    hipLaunchKernelGGL(calib_copy_kernel, dim3(256 * 16), dim3(256), 0, (hipStream_t)stream, (const uint4*)src,
                       (uint4*)dst, bytes / 16);
    int rc = (int)hipGetLastError();
    if (rc != 0) return set_error(rc, hipGetErrorString((hipError_t)rc));
    return MI355_OK;
}
