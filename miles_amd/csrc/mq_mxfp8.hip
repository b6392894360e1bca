// MXFP8 (e4m3 codes, one E8M0 scale per 1x32 group along K) for gfx950.
// Reference: miles/utils/mxfp8.py:51-78 (layout: compact row-major scales [rows, K/32]); the arithmetic is
// Transformer Engine's rowwise MXFP8 quantizer:
//   amax = max|x| over the group; e = ceil_pow2_exponent(amax * f32(1/448)) (saturating at 0xFE, 0 for amax 0);
//   q = sat_e4m3(x * 2^(127-e)).
//
// The tensor is a flat run of groups.  Four lanes own one group (8 bf16 = 16 bytes each), so a wavefront
// reads 1 KiB of consecutive input per load instruction; the group amax is a two-step DPP max inside the
// quad.  Scaling by a power of two is exact, so the only rounding is the e4m3 conversion.
#include "mq_api_internal.hpp"
#include "mq_common.hpp"
#include "mq_group.hpp"

namespace mq {

constexpr int kMxThreads = 256;
#ifndef MQ_MX_UNROLL
#define MQ_MX_UNROLL 2
#endif
constexpr int kMxUnroll = MQ_MX_UNROLL;  // 16-byte units per lane (2 measured best on MI355X: 1 pays the prologue too often, 4 lowers occupancy)

// 16-bit inputs, bf16 or fp16 (F16): the two instances differ in the conversion to fp32 and in the infinity pattern
template <class Table, int F16>
__global__ __launch_bounds__(kMxThreads) void mxfp8_bf16_kernel(const Table tab) {
    constexpr uint32_t kInfBits = F16 ? 0x7C00u : 0x7F80u;
    const float inv448 = u2f(0x3B124925u);
    const FlatJob& job = flat_job(tab);
    const uint16_t* __restrict__ w = (const uint16_t*)job.w;
    uint8_t* __restrict__ q = (uint8_t*)job.q;
    uint8_t* __restrict__ scale = (uint8_t*)job.s;
    const int64_t total_units = job.units;
    const uint32_t t = threadIdx.x;
    const int64_t base = flat_block(tab) * (kMxThreads * kMxUnroll);
    if (base >= total_units) return;
    // everything a lane adds to the workgroup's (uniform) base addresses is a 32-bit offset
    const int64_t left = total_units - base;
    const uint32_t rem = left < kMxThreads * kMxUnroll ? (uint32_t)left : (uint32_t)(kMxThreads * kMxUnroll);
    const uint16_t* __restrict__ w0 = w + base * 8;
    uint8_t* __restrict__ q0 = q + base * 8;
    uint8_t* __restrict__ scale0 = scale + base / 4;        // `base` is a multiple of the four lanes of a group
    u32x4 v[kMxUnroll];
#pragma unroll
    for (int i = 0; i < kMxUnroll; i++) {
        const uint32_t off = t + i * kMxThreads;
        v[i] = off < rem ? ld16(w0 + off * 8u) : u32x4{0u, 0u, 0u, 0u};
    }
#pragma unroll
    for (int i = 0; i < kMxUnroll; i++) {
        const uint32_t off = t + i * kMxThreads;
        uint32_t m2 = max2_u16(max2_u16(abs2(v[i].x), abs2(v[i].y)), max2_u16(abs2(v[i].z), abs2(v[i].w)));
        uint32_t mb = group_max4(hmax_u16(m2));         // 16-bit pattern of the group amax, quad-uniform
        const bool plain = mb < kInfBits;               // no infinity and no NaN in the group
        if (mb > kInfBits) {
            // a NaN in the group (rare; the four lanes of a group branch together): the published kernel takes the
            // maximum with fmaxf, which skips a NaN, so the scale comes from the other elements and only the NaN
            // elements themselves become the NaN code
            const uint32_t u[4] = {v[i].x, v[i].y, v[i].z, v[i].w};
            uint32_t mf = 0;
#pragma unroll
            for (int k = 0; k < 4; k++) {
                const uint32_t lo = u[k] & 0x7FFFu, hi = (u[k] >> 16) & 0x7FFFu;
                mf = umax(mf, umax(lo > kInfBits ? 0u : lo, hi > kInfBits ? 0u : hi));
            }
            mb = group_max4(mf);
        }
        const float amax = elem_lo<F16>(mb);
        const uint32_t e = e8m0_ceil(amax * inv448);
        const float inv = e8m0_inverse(e);
        const float f[8] = {elem_lo<F16>(v[i].x), elem_hi<F16>(v[i].x), elem_lo<F16>(v[i].y), elem_hi<F16>(v[i].y),
                            elem_lo<F16>(v[i].z), elem_hi<F16>(v[i].z), elem_lo<F16>(v[i].w), elem_hi<F16>(v[i].w)};
        u32x2 o;
        if (plain) {
            // finite group: |x * inv| <= 448 by construction, no clamp needed
            o.x = hw_e4m3x4(f[0] * inv, f[1] * inv, f[2] * inv, f[3] * inv);
            o.y = hw_e4m3x4(f[4] * inv, f[5] * inv, f[6] * inv, f[7] * inv);
        } else {
            uint32_t c[8];
#pragma unroll
            for (int j = 0; j < 8; j++) c[j] = sw_e4m3fn_sat(f[j] * inv);
            o.x = c[0] | (c[1] << 8) | (c[2] << 16) | (c[3] << 24);
            o.y = c[4] | (c[5] << 8) | (c[6] << 16) | (c[7] << 24);
        }
        if (off < rem) {
            st8(q0 + off * 8u, o);
            if ((t & 3) == 0) scale0[off >> 2] = (uint8_t)e;
        }
    }
}

// any dtype: one lane per group
__global__ __launch_bounds__(256) void mxfp8_generic_kernel(const void* __restrict__ w, int dtype,
                                                            uint8_t* __restrict__ q, uint8_t* __restrict__ scale,
                                                            int64_t groups) {
    const float inv448 = u2f(0x3B124925u);
    const int64_t stride = (int64_t)gridDim.x * blockDim.x;
    for (int64_t g = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; g < groups; g += stride) {
        uint32_t m = 0;
        for (int j = 0; j < 32; j++) {
            const uint32_t a = f2u(load_f32(w, g * 32 + j, dtype)) & 0x7FFFFFFFu;
            m = umax(m, a > 0x7F800000u ? 0u : a);       // the published kernel's fmaxf skips a NaN
        }
        const uint32_t e = e8m0_ceil(u2f(m) * inv448);
        const float inv = e8m0_inverse(e);
        scale[g] = (uint8_t)e;
        for (int j = 0; j < 32; j++) q[g * 32 + j] = (uint8_t)sw_e4m3fn_sat(load_f32(w, g * 32 + j, dtype) * inv);
    }
}

}  // namespace mq

using namespace mq;

bool mq_mxfp8_fast_ok(const void* w, int dtype, const void* q) {
    return (dtype == MQ_BF16 || dtype == MQ_F16) && ((uintptr_t)w % 16) == 0 && ((uintptr_t)q % 8) == 0;
}

// tab.job[i].units set by the caller, every tensor of the one 16-bit dtype; fills tab.end and launches
int mq_mxfp8_launch_group(int dtype, FlatTable& tab, hipStream_t st) {
    if (!flat_grid(tab, kMxThreads * kMxUnroll)) return mq_fail(MQ_ERR_ARG, "tensor too large");
    if (tab.max_blocks == 0) return MQ_OK;
    const dim3 grid((unsigned)tab.max_blocks, (unsigned)tab.n), blk(kMxThreads);
    if (dtype == MQ_F16) hipLaunchKernelGGL((mxfp8_bf16_kernel<FlatTable, 1>), grid, blk, 0, st, tab);
    else hipLaunchKernelGGL((mxfp8_bf16_kernel<FlatTable, 0>), grid, blk, 0, st, tab);
    return mq_check_launch("mxfp8 quant");
}

// n descriptors in device memory; max_units: the largest tensor's 16-byte units
int mq_mxfp8_launch_table(int dtype, const FlatJob* device_jobs, int n, int64_t max_units, hipStream_t st) {
    FlatRef ref{device_jobs, 0, 0};
    if (!flat_grid(ref, max_units, kMxThreads * kMxUnroll)) return mq_fail(MQ_ERR_ARG, "tensor too large");
    if (ref.max_blocks == 0 || n == 0) return MQ_OK;
    const dim3 grid((unsigned)ref.max_blocks, (unsigned)n), blk(kMxThreads);
    if (dtype == MQ_F16) hipLaunchKernelGGL((mxfp8_bf16_kernel<FlatRef, 1>), grid, blk, 0, st, ref);
    else hipLaunchKernelGGL((mxfp8_bf16_kernel<FlatRef, 0>), grid, blk, 0, st, ref);
    return mq_check_launch("mxfp8 quant");
}

extern "C" int mq_mxfp8_quant(const void* w, int dtype, void* q, uint8_t* scale, int64_t rows, int64_t K,
                              void* stream) {
    if ((!w || !q || !scale) && rows != 0 && K != 0) return mq_fail(MQ_ERR_ARG, "null pointer");
    if (dtype < MQ_BF16 || dtype > MQ_F32 || rows < 0 || K < 0) return mq_fail(MQ_ERR_ARG, "bad argument");
    if (K % 32 != 0) return mq_fail(MQ_ERR_ARG, "Last dim must be divisible by 32 for MXFP8.");
    if (rows == 0 || K == 0) return MQ_OK;
    hipStream_t st = (hipStream_t)stream;
    const int64_t groups = rows * (K / 32);
    if (mq_mxfp8_fast_ok(w, dtype, q)) {
        FlatTable tab{};
        tab.n = 1;
        tab.job[0] = FlatJob{w, q, scale, nullptr, groups * 4, nullptr, 0, 0};
        return mq_mxfp8_launch_group(dtype, tab, st);
    }
    int64_t blocks = (groups + 255) / 256;
    if (blocks > mq_grid_cap()) blocks = mq_grid_cap();
    hipLaunchKernelGGL(mxfp8_generic_kernel, dim3((unsigned)blocks), dim3(256), 0, st, w, dtype, (uint8_t*)q, scale,
                       groups);
    return mq_check_launch("mxfp8 quant");
}
