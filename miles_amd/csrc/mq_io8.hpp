// Eight consecutive elements of a bf16 / fp16 / fp32 tensor as floats, and back: the per-lane unit of the row-wise
// kernels (16 bytes of a 16-bit tensor, 32 bytes of an fp32 one).
#pragma once
#include "mq_api_internal.hpp"
#include "mq_common.hpp"

namespace mq {

template <int DT>
__device__ __forceinline__ void fq_load8(const void* x, int64_t unit, float f[8]) {
    if (DT == MQ_F32) {
        const u32x4 a = ld16((const float*)x + unit * 8), b = ld16((const float*)x + unit * 8 + 4);
        f[0] = u2f(a.x); f[1] = u2f(a.y); f[2] = u2f(a.z); f[3] = u2f(a.w);
        f[4] = u2f(b.x); f[5] = u2f(b.y); f[6] = u2f(b.z); f[7] = u2f(b.w);
    } else {
        const u32x4 a = ld16((const uint16_t*)x + unit * 8);
        const uint32_t u[4] = {a.x, a.y, a.z, a.w};
#pragma unroll
        for (int i = 0; i < 4; i++) {
            if (DT == MQ_BF16) { f[2 * i] = bf16_lo(u[i]); f[2 * i + 1] = bf16_hi(u[i]); }
            else {
                f[2 * i] = (float)__builtin_bit_cast(_Float16, (uint16_t)(u[i] & 0xFFFFu));
                f[2 * i + 1] = (float)__builtin_bit_cast(_Float16, (uint16_t)(u[i] >> 16));
            }
        }
    }
}
template <int DT>
__device__ __forceinline__ void fq_store8(void* y, int64_t unit, const float f[8]) {
    if (DT == MQ_F32) {
        st16((float*)y + unit * 8, u32x4{f2u(f[0]), f2u(f[1]), f2u(f[2]), f2u(f[3])});
        st16((float*)y + unit * 8 + 4, u32x4{f2u(f[4]), f2u(f[5]), f2u(f[6]), f2u(f[7])});
    } else if (DT == MQ_BF16) {
        st16((uint16_t*)y + unit * 8, u32x4{hw_bf16x2(f[0], f[1]), hw_bf16x2(f[2], f[3]), hw_bf16x2(f[4], f[5]), hw_bf16x2(f[6], f[7])});
    } else {
        // The compiler would fold the preceding multiplication into the conversion as fma(q, scale, +0), and adding
        // +0 turns a -0 product into +0; the empty asm keeps the product a value of its own.
        uint32_t p[4];
#pragma unroll
        for (int i = 0; i < 4; i++) {
            float a = f[2 * i], b = f[2 * i + 1];
            asm volatile("" : "+v"(a), "+v"(b));
            p[i] = (uint32_t)__builtin_bit_cast(uint16_t, (_Float16)a) | ((uint32_t)__builtin_bit_cast(uint16_t, (_Float16)b) << 16);
        }
        st16((uint16_t*)y + unit * 8, u32x4{p[0], p[1], p[2], p[3]});
    }
}

}  // namespace mq
