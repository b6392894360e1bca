// Exhaustive agreement check between the gfx950 convert instructions the kernels use and the
// software round-to-nearest-even forms in mq_common.hpp, over every fp32 bit pattern.  Built into libmq_probes.so
// (loaded by the GPU tests), not into the product library.
#include "mq_common.hpp"
#include "mq_probes_internal.hpp"

namespace mq {

__device__ __forceinline__ void tally(uint64_t* counts, int slot, bool bad) {
    const uint64_t mask = __ballot(bad);
    if (mask && (threadIdx.x & 63) == 0) atomicAdd((unsigned long long*)&counts[slot], (unsigned long long)__popcll(mask));
}

__global__ __launch_bounds__(256) void selftest_kernel(uint64_t* counts) {
    const uint32_t tid = blockIdx.x * blockDim.x + threadIdx.x;   // 2^20 lanes
    for (uint32_t it = 0; it < 4096; it++) {
        const uint32_t bits = it * (1u << 20) + tid;
        const float x = u2f(bits);
        const uint32_t a = bits & 0x7FFFFFFFu;
        const bool is_nan = a > 0x7F800000u;
        // e4m3: both slots of the packed convert, inputs the kernels can produce (|x| <= 448)
        const uint32_t hw8 = hw_e4m3x2<false>(x, x, 0u);
        const uint32_t hw8h = hw_e4m3x2<true>(x, x, 0u) >> 16;
        const uint32_t sw8 = sw_e4m3fn(x);
        const bool in_range = a <= 0x43E00000u;
        tally(counts, 0, in_range && ((hw8 & 0xFFu) != sw8 || ((hw8 >> 8) & 0xFFu) != sw8 || hw8h != (hw8 & 0xFFFFu)));
        tally(counts, 1, is_nan && (hw8 & 0x7Fu) != 0x7Fu);
        tally(counts, 6, !is_nan && a > 0x43E00000u && a <= 0x43E80000u && (hw8 & 0x7Fu) != 0x7Eu);
        // e2m1: every non-NaN input, all four byte slots
        const uint32_t sw4 = sw_e2m1(x);
        uint32_t hw4 = hw_e2m1x2<0>(x, x, 0u);
        hw4 = hw_e2m1x2<1>(x, x, hw4);
        hw4 = hw_e2m1x2<2>(x, x, hw4);
        hw4 = hw_e2m1x2<3>(x, x, hw4);
        tally(counts, 2, !is_nan && hw4 != sw4 * 0x11111111u);
        tally(counts, 5, is_nan && (hw4 & 0x7u) != 0x7u);
        // bf16
        const uint32_t hwb = hw_bf16x2(x, x);
        const uint32_t swb = sw_bf16(x);
        tally(counts, 3, !is_nan && hwb != (swb | (swb << 16)));
    }
    if (tid < 256) {
        const uint32_t word = tid | (tid << 8) | (tid << 16) | (tid << 24);
        const f32x2 lo = hw_e4m3x2_decode<false>(word), hi = hw_e4m3x2_decode<true>(word);
        const float want = sw_e4m3fn_decode(tid);
        const bool nan_code = (tid & 0x7Fu) == 0x7Fu;
        bool bad;
        if (nan_code) bad = !(lo.x != lo.x && lo.y != lo.y && hi.x != hi.x && hi.y != hi.y);
        else bad = f2u(lo.x) != f2u(want) || f2u(lo.y) != f2u(want) || f2u(hi.x) != f2u(want) || f2u(hi.y) != f2u(want);
        tally(counts, 4, bad);
    }
    if (tid == 0) {
        // nibble order of the packed e2m1 convert: first operand in the low nibble
        if (hw_e2m1x2<0>(1.0f, 2.0f, 0u) != 0x42u) atomicAdd((unsigned long long*)&counts[7], 1ull);
    }
}

// every divisor in the range of the shared-divisor sequence: refined hardware reciprocal against the IEEE division
__global__ __launch_bounds__(256) void selftest_reciprocal_kernel(uint64_t* count) {
    const uint32_t tid = blockIdx.x * blockDim.x + threadIdx.x;   // 2^20 lanes
    for (uint32_t it = 0; it < 4096; it++) {
        const uint32_t bits = it * (1u << 20) + tid;
        const float s = u2f(bits);
        float want = 1.0f / s;
        asm volatile("" : "+v"(want));
        tally(count, 0, shared_div_ok(s) && f2u(recip_shared(s)) != f2u(want));
    }
}

__global__ void selftest_clear_kernel(uint32_t* p, int n) {
    if ((int)threadIdx.x < n) p[threadIdx.x] = 0u;
}

}  // namespace mq

static int clear_words(void* p, int n, void* stream) {
    hipLaunchKernelGGL(mq::selftest_clear_kernel, dim3(1), dim3(64), 0, (hipStream_t)stream, (uint32_t*)p, n);
    return mqp_check_launch("selftest clear");
}

extern "C" int mqp_selftest_reciprocal(uint64_t* count, void* stream) {
    if (!count) return mqp_fail(MQP_ERR_ARG, "null pointer");
    hipStream_t st = (hipStream_t)stream;
    int rc = clear_words(count, 2, stream);
    if (rc) return rc;
    hipLaunchKernelGGL(mq::selftest_reciprocal_kernel, dim3(4096), dim3(256), 0, st, count);
    return mqp_check_launch("selftest reciprocal");
}

extern "C" int mqp_selftest_convert(uint64_t* counts, void* stream) {
    if (!counts) return mqp_fail(MQP_ERR_ARG, "null pointer");
    hipStream_t st = (hipStream_t)stream;
    int rc = clear_words(counts, 16, stream);
    if (rc) return rc;
    hipLaunchKernelGGL(mq::selftest_kernel, dim3(4096), dim3(256), 0, st, counts);
    return mqp_check_launch("selftest");
}
