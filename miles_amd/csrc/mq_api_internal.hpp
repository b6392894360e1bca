// Host-side plumbing shared by the entry points: error reporting and launch checks.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/miles_quant.h"

int mq_fail(int code, const char* msg);
int mq_check_launch(const char* what);
// Device counters that the amax fold kernels of the running mq_run_jobs_feedback call add to, and the device-visible
// address of the host mirror they refresh (both null outside such a call): set on entry, cleared on return, per host
// thread.
uint32_t* mq_amax_feedback();
uint32_t* mq_amax_feedback_mirror();
void mq_set_amax_feedback(uint32_t* device_counter, uint32_t* mirror);
// upper bound on the grid of a grid-stride kernel: enough workgroups to fill 256 CUs several times over
inline int64_t mq_grid_cap() { return 256 * 16; }

struct MqDequantArgs {
    const void* x;
    const float* s;
    void* y;
    int64_t M, N;
    int block;
};

struct MqRescaleArgs {
    const void* x;
    const float* s;
    void* q;
    uint8_t* scale;
    int64_t M, K, lds;
};

namespace mq {
__device__ __forceinline__ float load_f32(const void* p, int64_t i, int dtype) {
    if (dtype == MQ_BF16) return __builtin_bit_cast(float, (uint32_t)((const uint16_t*)p)[i] << 16);
    if (dtype == MQ_F16) return (float)((const _Float16*)p)[i];
    return ((const float*)p)[i];
}
__device__ __forceinline__ uint32_t f32_to_bf16_bits(float f) {
    uint32_t u = __builtin_bit_cast(uint32_t, f);
    if ((u & 0x7FFFFFFFu) > 0x7F800000u) return 0x7FC0u;
    return (u + 0x7FFFu + ((u >> 16) & 1u)) >> 16;
}
__device__ __forceinline__ float round_to_dtype(float f, int dtype) {
    if (dtype == MQ_BF16) return __builtin_bit_cast(float, f32_to_bf16_bits(f) << 16);
    if (dtype == MQ_F16) return (float)(_Float16)f;
    return f;
}
__device__ __forceinline__ void store_dtype(void* p, int64_t i, float f, int dtype) {
    if (dtype == MQ_BF16) ((uint16_t*)p)[i] = (uint16_t)f32_to_bf16_bits(f);
    else if (dtype == MQ_F16) ((_Float16*)p)[i] = (_Float16)f;
    else ((float*)p)[i] = f;
}
}  // namespace mq
