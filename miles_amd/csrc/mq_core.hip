// Library plumbing: version, thread-local error text, launch check, fill and copy kernels.
#include <stdio.h>
#include <string.h>

#include "mq_api_internal.hpp"
#include "mq_common.hpp"
#include "mq_group.hpp"

static thread_local char g_err[256] = "";
static thread_local uint32_t* g_amax_feedback = nullptr;
static thread_local uint32_t* g_amax_feedback_mirror = nullptr;
uint32_t* mq_amax_feedback() { return g_amax_feedback; }
uint32_t* mq_amax_feedback_mirror() { return g_amax_feedback_mirror; }
void mq_set_amax_feedback(uint32_t* device_counter, uint32_t* mirror) {
    g_amax_feedback = device_counter;
    g_amax_feedback_mirror = mirror;
}

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
// Grouped byte copies: a workgroup moves one 16 KiB chunk (four 16-byte units per lane) of one of up to 64 runs.
// Runs whose pointers are 16-byte aligned use 16-byte accesses with a byte tail; the others go byte by byte.
constexpr int kCopyUnits = 4;
constexpr int kCopyChunk = kCopyUnits * 4096;
__global__ __launch_bounds__(256) void copy_group_kernel(const CopyTable tab) {
    const int32_t item = blockIdx.x;
    const JobRef r = find_job(tab, item);
    const CopyJob& job = tab.job[r.ji];
    const int32_t local = item - r.start, row = local / job.chunks_per_row;
    const int64_t off0 = (int64_t)(local - row * job.chunks_per_row) * kCopyChunk;
    const uint8_t* __restrict__ src = job.src + row * job.src_pitch;
    uint8_t* __restrict__ dst = job.dst + row * job.dst_pitch;
    const bool aligned = (((uintptr_t)src | (uintptr_t)dst) & 15) == 0;
    if (aligned) {
        u32x4 v[kCopyUnits];
        bool full[kCopyUnits];
#pragma unroll
        for (int u = 0; u < kCopyUnits; u++) {
            const int64_t o = off0 + (u * 256 + threadIdx.x) * 16;
            full[u] = o + 16 <= job.bytes;
            if (full[u]) v[u] = ld16(src + o);
        }
#pragma unroll
        for (int u = 0; u < kCopyUnits; u++) {
            const int64_t o = off0 + (u * 256 + threadIdx.x) * 16;
            if (full[u]) st16(dst + o, v[u]);
            else for (int64_t b = o; b < job.bytes && b < o + 16; b++) dst[b] = src[b];
        }
    } else {
        const int64_t stop = off0 + kCopyChunk < job.bytes ? off0 + kCopyChunk : job.bytes;
        for (int64_t b = off0 + threadIdx.x; b < stop; b += 256) dst[b] = src[b];
    }
}
// one long aligned run: one 16-byte unit per lane, no table (the access pattern that streams fastest on MI355X)
__global__ __launch_bounds__(256) void copy_run_kernel(const uint8_t* __restrict__ src, uint8_t* __restrict__ dst,
                                                       int64_t bytes) {
    const int64_t o = ((int64_t)blockIdx.x * 256 + threadIdx.x) * 16;
    if (o + 16 <= bytes) st16(dst + o, ld16(src + o));
    else for (int64_t b = o; b < bytes; b++) dst[b] = src[b];
}
}  // namespace mq

int mq_copy_launch_run(const void* src, void* dst, int64_t bytes, hipStream_t st) {
    const int64_t blocks = (bytes + 4095) / 4096;
    if (blocks > 0x7FFFFFF0) return mq_fail(MQ_ERR_ARG, "copy too large");
    hipLaunchKernelGGL(mq::copy_run_kernel, dim3((unsigned)blocks), dim3(256), 0, st, (const uint8_t*)src, (uint8_t*)dst, bytes);
    return mq_check_launch("copy");
}

// tab.job[0..n) filled by the caller
int mq_copy_launch_group(mq::CopyTable& tab, hipStream_t st) {
    int64_t run = 0;
    for (int i = 0; i < tab.n; i++) {
        // chunks_per_row holds the row count on entry (0 or 1: a plain run)
        const int64_t rows = tab.job[i].chunks_per_row > 1 ? tab.job[i].chunks_per_row : 1;
        const int64_t per_row = (tab.job[i].bytes + mq::kCopyChunk - 1) / mq::kCopyChunk;
        if (per_row > 0x7FFFFFF0) return mq_fail(MQ_ERR_ARG, "copy group too large");
        tab.job[i].chunks_per_row = per_row > 0 ? (int32_t)per_row : 1;
        run += rows * per_row;
        if (run > 0x7FFFFFF0) return mq_fail(MQ_ERR_ARG, "copy group too large");
        tab.end[i] = (int32_t)run;
    }
    mq::seal_table(tab);
    if (tab.total == 0) return MQ_OK;
    hipLaunchKernelGGL(mq::copy_group_kernel, dim3((unsigned)tab.total), dim3(256), 0, st, tab);
    return mq_check_launch("grouped copy");
}

extern "C" int mq_fill_u32(void* p, uint32_t value, int64_t n, void* stream) {
    if (!p || n < 0) return mq_fail(MQ_ERR_ARG, "bad argument");
    if (n == 0) return MQ_OK;
    int64_t blocks = (n + 255) / 256;
    if (blocks > mq_grid_cap()) blocks = mq_grid_cap();
    hipLaunchKernelGGL(mq::fill_u32_n_kernel, dim3((unsigned)blocks), dim3(256), 0, (hipStream_t)stream, (uint32_t*)p,
                       value, n);
    return mq_check_launch("fill");
}
