// Library plumbing: version, thread-local error text, launch check, fill and copy kernels.
#include <stdio.h>
#include <string.h>

#include "mq_api_internal.hpp"
#include "mq_common.hpp"

static thread_local char g_err[256] = "";

int mq_fail(int code, const char* msg) {
    snprintf(g_err, sizeof(g_err), "%s", msg);
    return code;
}

int mq_check_launch(const char* what) {
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) {
        snprintf(g_err, sizeof(g_err), "%s: %s", what, hipGetErrorString(e));
        return MQ_ERR_HIP;
    }
    return MQ_OK;
}

extern "C" int mq_version(void) { return MQ_VERSION; }
extern "C" const char* mq_last_error(void) { return g_err; }

namespace mq {
__global__ void fill_u32_n_kernel(uint32_t* p, uint32_t v, int64_t n) {
    int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    const int64_t stride = (int64_t)gridDim.x * blockDim.x;
    for (; i < n; i += stride) p[i] = v;
}
__global__ __launch_bounds__(256) void copy16_kernel(const u32x4* __restrict__ src, u32x4* __restrict__ dst, int64_t n16) {
    int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    const int64_t stride = (int64_t)gridDim.x * blockDim.x;
    for (; i < n16; i += stride) dst[i] = src[i];
}
}  // namespace mq

extern "C" int mq_fill_u32(void* p, uint32_t value, int64_t n, void* stream) {
    if (!p || n < 0) return mq_fail(MQ_ERR_ARG, "bad argument");
    if (n == 0) return MQ_OK;
    int64_t blocks = (n + 255) / 256;
    if (blocks > mq_grid_cap()) blocks = mq_grid_cap();
    hipLaunchKernelGGL(mq::fill_u32_n_kernel, dim3((unsigned)blocks), dim3(256), 0, (hipStream_t)stream, (uint32_t*)p,
                       value, n);
    return mq_check_launch("fill");
}

extern "C" int mq_copy_bytes(const void* src, void* dst, int64_t nbytes, void* stream) {
    if (!src || !dst || nbytes < 0 || (nbytes % 16) || ((uintptr_t)src % 16) || ((uintptr_t)dst % 16))
        return mq_fail(MQ_ERR_ARG, "copy needs 16-byte aligned pointers and size");
    if (nbytes == 0) return MQ_OK;
    const int64_t n16 = nbytes / 16;
    int64_t blocks = (n16 + 255) / 256;
    if (blocks > 256 * 32) blocks = 256 * 32;
    hipLaunchKernelGGL(mq::copy16_kernel, dim3((unsigned)blocks), dim3(256), 0, (hipStream_t)stream,
                       (const mq::u32x4*)src, (mq::u32x4*)dst, n16);
    return mq_check_launch("copy");
}
