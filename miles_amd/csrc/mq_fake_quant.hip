// Block fake quantization (quantize, then dequantize back to the input dtype in one pass) and the 1 x block FP8
// activation quantizer for gfx950.
// Reference: miles/kernels/quant/fake_quant.py:25-99 (`_fake_quant_kernel` and its three entry points):
//   mode 0  fp8, 1x32 blocks:  amax' = max(amax, 1e-4);        scale = ceil_pow2(amax' * f32(1/448))
//                              q = e4m3_rne(clamp(x / scale, +-448))
//   mode 1  fp4, 1x32 blocks:  amax' = max(amax, 6 * 2^-126);  scale = ceil_pow2(amax' * f32(1/6))
//                              q = e2m1_rne(clamp(x / scale, +-6)), an exact zero gives +0
//   mode 2  fp4 with e4m3 scales, 1x16 blocks ("compressed kv"):
//                              scale = f32(e4m3_rne(min(max(amax * f32(1/6), 2^-9), 448)));  q as mode 1 with the
//                              correctly rounded quotient x / scale
//   out = dtype(q * scale)
// A power-of-two scale makes x / scale exact, so it is a multiplication by the reciprocal power.  The hardware
// conversions saturate / round exactly as clamp-then-round does for the one or two ulp by which |x / scale| can
// exceed the format maximum.  Lanes own 8 consecutive elements; 4 (or 2) neighbouring lanes form a block.
#include "mq_api_internal.hpp"
#include "mq_common.hpp"
#include "mq_group.hpp"
#include "mq_io8.hpp"

namespace mq {

constexpr int kFqThreads = 256;

__device__ __forceinline__ float ceil_pow2_normal(float v) {   // v normal and positive
    const uint32_t u = f2u(v);
    return u2f(((u >> 23) + ((u & 0x7FFFFFu) != 0)) << 23);
}

// MODE as above; LANES = lanes per block (4 for 1x32, 2 for 1x16)
template <int DT, int MODE>
__global__ __launch_bounds__(kFqThreads) void fake_quant_kernel(const void* __restrict__ x, void* __restrict__ y,
                                                                int64_t units, int chunk) {
    constexpr int LANES = MODE == 2 ? 2 : 4;
    const int64_t unit = xcd_chunked_block(chunk) * kFqThreads + threadIdx.x;
    const bool live = unit < units;           // a block is a whole number of lanes: dead lanes never share one with live lanes
    float f[8];
    fq_load8<DT>(x, live ? unit : units - 1, f);
    uint32_t m = 0;
#pragma unroll
    for (int i = 0; i < 8; i++) m = umax(m, f2u(f[i]) & 0x7FFFFFFFu);
    m = LANES == 4 ? group_max4(m) : group_max2(m);
    const bool finite = m < 0x7F800000u;
    float amax = u2f(m), scale, q[8];
    if (MODE == 2) {
        const float hp = __builtin_fminf(__builtin_fmaxf(amax * u2f(0x3E2AAAABu), 0.001953125f), 448.0f);
        scale = finite ? hw_e4m3x2_decode<false>(hw_e4m3x2<false>(hp, hp, 0u)).x : sw_e4m3fn_decode(sw_e4m3fn(hp));
        const float r = 1.0f / scale;
        const bool fast = DT != MQ_F32;       // 16-bit numerators: the shared-divisor sequence is the exact quotient
#pragma unroll
        for (int i = 0; i < 8; i++) q[i] = fast ? div_by_shared(f[i], scale, r) : f[i] / scale;
    } else {
        amax = __builtin_fmaxf(amax, MODE == 0 ? 1e-4f : u2f(0x01C00000u) /* 6 * 2^-126 */);
        scale = ceil_pow2_normal(amax * u2f(MODE == 0 ? 0x3B124925u : 0x3E2AAAABu));
        const float r = u2f(0x7F000000u - f2u(scale));      // 2^-k for scale = 2^k
#pragma unroll
        for (int i = 0; i < 8; i++) q[i] = f[i] * r;
    }
    if (MODE == 0) {
        if (finite) {
            const uint32_t lo = hw_e4m3x4(q[0], q[1], q[2], q[3]), hi = hw_e4m3x4(q[4], q[5], q[6], q[7]);
            const f32x2 a = hw_e4m3x2_decode<false>(lo), b = hw_e4m3x2_decode<true>(lo);
            const f32x2 c = hw_e4m3x2_decode<false>(hi), d = hw_e4m3x2_decode<true>(hi);
            q[0] = a.x; q[1] = a.y; q[2] = b.x; q[3] = b.y; q[4] = c.x; q[5] = c.y; q[6] = d.x; q[7] = d.y;
        } else {
#pragma unroll
            for (int i = 0; i < 8; i++) q[i] = sw_e4m3fn_decode(sw_e4m3fn_sat(q[i]));
        }
    } else {
        const bool zero[8] = {q[0] == 0.0f, q[1] == 0.0f, q[2] == 0.0f, q[3] == 0.0f,
                              q[4] == 0.0f, q[5] == 0.0f, q[6] == 0.0f, q[7] == 0.0f};
        uint32_t w = 0;
        w = hw_e2m1x2<0>(q[0], q[1], w);
        w = hw_e2m1x2<1>(q[2], q[3], w);
        w = hw_e2m1x2<2>(q[4], q[5], w);
        w = hw_e2m1x2<3>(q[6], q[7], w);
        const f32x2 a = __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(w, 1.0f, 0), b = __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(w, 1.0f, 1);
        const f32x2 c = __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(w, 1.0f, 2), d = __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(w, 1.0f, 3);
        q[0] = a.x; q[1] = a.y; q[2] = b.x; q[3] = b.y; q[4] = c.x; q[5] = c.y; q[6] = d.x; q[7] = d.y;
        // an exact zero has sign 0 in the reference and comes out as +0; a negative value that rounds to zero keeps its sign
#pragma unroll
        for (int i = 0; i < 8; i++) q[i] = zero[i] ? 0.0f : q[i];
    }
#pragma unroll
    for (int i = 0; i < 8; i++) q[i] = q[i] * scale;
    if (live) fq_store8<DT>(y, unit, q);
}


// Tensors that do not start on a 16-byte boundary: one lane per block, element-wise accesses, software conversions.
__global__ __launch_bounds__(256) void fake_quant_generic_kernel(const void* __restrict__ x, int dtype,
                                                                 void* __restrict__ y, int64_t blocks, int mode) {
    const int64_t b = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (b >= blocks) return;
    const int n = mode == 2 ? 16 : 32;
    float amax = 0.0f;
    for (int j = 0; j < n; j++) amax = __builtin_fmaxf(amax, __builtin_fabsf(load_f32(x, b * n + j, dtype)));
    float scale;
    if (mode == 2) {
        const float hp = __builtin_fminf(__builtin_fmaxf(amax * u2f(0x3E2AAAABu), 0.001953125f), 448.0f);
        scale = sw_e4m3fn_decode(sw_e4m3fn(hp));
    } else {
        amax = __builtin_fmaxf(amax, mode == 0 ? 1e-4f : u2f(0x01C00000u));
        scale = ceil_pow2_normal(amax * u2f(mode == 0 ? 0x3B124925u : 0x3E2AAAABu));
    }
    const float top = mode == 0 ? 448.0f : 6.0f;
    for (int j = 0; j < n; j++) {
        const float v = __builtin_fminf(__builtin_fmaxf(load_f32(x, b * n + j, dtype) / scale, -top), top);
        float q;
        if (mode == 0) q = sw_e4m3fn_decode(sw_e4m3fn_sat(v));
        else {
            const uint32_t c = sw_e2m1(v);
            const float mag = (c & 7u) < 2u ? 0.5f * (float)(c & 7u) : u2f(0x3F000000u + ((c & 7u) << 22));
            q = v == 0.0f ? 0.0f : ((c & 8u) ? -mag : mag);     // an exact zero gives +0, a value rounded to zero keeps its sign
        }
        float o = q * scale;
        asm volatile("" : "+v"(o));            // keep the product apart from the fp16 conversion (see fq_store8)
        store_dtype(y, b * n + j, o, dtype);
    }
}

// ---- act_quant: FP8 codes + one scale per 1 x block group of consecutive elements -------------------------------
// Reference: miles/kernels/quant/fp8_act_quant.py:49-137 (`act_quant_kernel`, `act_quant`):
//   amax' = max(amax, 1e-4);  s = amax' * f32(1/448), with MQ_ACT_ROUND_SCALE rounded up to a power of two
//   code = e4m3_rne(clamp(x / s, +-448))  -- a true fp32 division --  and with MQ_ACT_INPLACE y = dtype(f32(code) * s)
// 16-bit inputs take the shared-divisor sequence (the correctly rounded quotient for numerators of at most 11
// significant bits; exact as well when s is a power of two); it returns +0 for a -0 numerator, and since s > 0 the
// quotient's sign is always the numerator's, so the sign is copied back with one v_bfi_b32.  LANES lanes of 8
// elements form a group.  x and y may be the same buffer: a lane writes only the 8 elements it has read.
template <int LANES>
__device__ __forceinline__ uint32_t group_max_lanes(uint32_t m) {
    return LANES == 16 ? group_max16(m) : LANES == 8 ? group_max8(m) : LANES == 4 ? group_max4(m) : group_max2(m);
}

// 8-element units per lane: two for the 2:1 read:write mix of the code path, one when as many bytes go out as come in
template <bool INPLACE> constexpr int kActUnits = INPLACE ? 1 : 2;

template <int DT, int LANES, bool INPLACE>
__device__ __forceinline__ void act_quant_unit(const float f[8], void* y, void* scale, int64_t unit, bool live, int flags) {
    float q[8];
    uint32_t m = 0;
#pragma unroll
    for (int i = 0; i < 8; i++) m = umax(m, f2u(f[i]) & 0x7FFFFFFFu);
    m = group_max_lanes<LANES>(m);
    const bool finite = m < 0x7F800000u;
    float s = __builtin_fmaxf(u2f(m), 1e-4f) * u2f(0x3B124925u);
    if ((flags & MQ_ACT_ROUND_SCALE) && finite) {             // power of two: the reciprocal is exact, so is the product
        s = ceil_pow2_normal(s);
        const float r = u2f(0x7F000000u - f2u(s));
#pragma unroll
        for (int i = 0; i < 8; i++) q[i] = f[i] * r;
    } else if (DT != MQ_F32 && finite && shared_div_ok(s)) {
        const float r = 1.0f / s;
#pragma unroll
        for (int i = 0; i < 8; i++) q[i] = div_by_shared(f[i], s, r);
    } else {
        if (flags & MQ_ACT_ROUND_SCALE) s = ceil_pow2_normal(s);
#pragma unroll
        for (int i = 0; i < 8; i++) q[i] = f[i] / s;
    }
    uint32_t lo, hi;
    if (finite) {                             // |x / s| <= 448 (1 + 2^-23): the conversion itself saturates
        lo = hw_e4m3x4(q[0], q[1], q[2], q[3]);
        hi = hw_e4m3x4(q[4], q[5], q[6], q[7]);
    } else {
        uint32_t c[8];
#pragma unroll
        for (int i = 0; i < 8; i++) c[i] = sw_e4m3fn_sat(__builtin_fminf(__builtin_fmaxf(q[i], -448.0f), 448.0f));
        lo = c[0] | (c[1] << 8) | (c[2] << 16) | (c[3] << 24);
        hi = c[4] | (c[5] << 8) | (c[6] << 16) | (c[7] << 24);
    }
    if (live && (threadIdx.x & (LANES - 1)) == 0) {
        const int64_t g = unit / LANES;
        if (flags & MQ_ACT_SCALE_E8M0) ((uint8_t*)scale)[g] = (uint8_t)(f2u(s) >> 23);
        else ((float*)scale)[g] = s;
    }
    if (!INPLACE) {
        if (live) st8((uint8_t*)y + unit * 8, u32x2{lo, hi});
        return;
    }
    if (finite) {
        const f32x2 a = hw_e4m3x2_decode<false>(lo), b = hw_e4m3x2_decode<true>(lo);
        const f32x2 c = hw_e4m3x2_decode<false>(hi), d = hw_e4m3x2_decode<true>(hi);
        q[0] = a.x; q[1] = a.y; q[2] = b.x; q[3] = b.y; q[4] = c.x; q[5] = c.y; q[6] = d.x; q[7] = d.y;
    } else {
#pragma unroll
        for (int i = 0; i < 4; i++) {
            q[i] = sw_e4m3fn_decode((lo >> (8 * i)) & 0xFFu);
            q[4 + i] = sw_e4m3fn_decode((hi >> (8 * i)) & 0xFFu);
        }
    }
#pragma unroll
    for (int i = 0; i < 8; i++) q[i] = q[i] * s;
    if (live) fq_store8<DT>(y, unit, q);
}

template <int DT, int LANES, bool INPLACE>
__global__ __launch_bounds__(kFqThreads) void act_quant_kernel(const void* x, void* y, void* scale, int64_t units,
                                                               int flags, int chunk) {
    const int64_t base = xcd_chunked_block(chunk) * (kFqThreads * kActUnits<INPLACE>) + threadIdx.x;
    float f[kActUnits<INPLACE>][8];
    // a group is a whole number of lanes, so dead lanes never share one with live lanes; they re-read the last unit
#pragma unroll
    for (int u = 0; u < kActUnits<INPLACE>; u++) {
        const int64_t unit = base + u * kFqThreads;
        fq_load8<DT>(x, unit < units ? unit : units - 1, f[u]);
    }
#pragma unroll
    for (int u = 0; u < kActUnits<INPLACE>; u++) {
        const int64_t unit = base + u * kFqThreads;
        act_quant_unit<DT, LANES, INPLACE>(f[u], y, scale, unit, unit < units, flags);
    }
}

// any block size, any alignment: one lane per group, software conversions
__global__ __launch_bounds__(256) void act_quant_generic_kernel(const void* x, int dtype, void* y, void* scale,
                                                                int64_t groups, int block, int flags) {
    const int64_t g = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (g >= groups) return;
    float amax = 0.0f;
    for (int j = 0; j < block; j++) amax = __builtin_fmaxf(amax, __builtin_fabsf(load_f32(x, g * block + j, dtype)));
    float s = __builtin_fmaxf(amax, 1e-4f) * u2f(0x3B124925u);
    if (flags & MQ_ACT_ROUND_SCALE) s = ceil_pow2_normal(s);
    if (flags & MQ_ACT_SCALE_E8M0) ((uint8_t*)scale)[g] = (uint8_t)(f2u(s) >> 23);
    else ((float*)scale)[g] = s;
    for (int j = 0; j < block; j++) {
        const int64_t i = g * block + j;
        const float r = load_f32(x, i, dtype) / s;
        const uint32_t code = sw_e4m3fn_sat(__builtin_fminf(__builtin_fmaxf(r, -448.0f), 448.0f));
        if (!(flags & MQ_ACT_INPLACE)) { ((uint8_t*)y)[i] = (uint8_t)code; continue; }
        float o = sw_e4m3fn_decode(code) * s;
        asm volatile("" : "+v"(o));           // keep the product apart from the fp16 conversion (see fq_store8)
        store_dtype(y, i, o, dtype);
    }
}

}  // namespace mq

using namespace mq;

template <int MODE>
static void launch_fq(const void* x, int dtype, void* y, int64_t units, hipStream_t st) {
    const int64_t blocks = (units + kFqThreads - 1) / kFqThreads;
    const int chunk = (int)flat_chunk(blocks);
    const dim3 grid((unsigned)flat_padded(blocks, chunk)), blk(kFqThreads);
    if (dtype == MQ_BF16) hipLaunchKernelGGL((fake_quant_kernel<MQ_BF16, MODE>), grid, blk, 0, st, x, y, units, chunk);
    else if (dtype == MQ_F16) hipLaunchKernelGGL((fake_quant_kernel<MQ_F16, MODE>), grid, blk, 0, st, x, y, units, chunk);
    else hipLaunchKernelGGL((fake_quant_kernel<MQ_F32, MODE>), grid, blk, 0, st, x, y, units, chunk);
}

extern "C" int mq_fake_quant(const void* x, int dtype, void* y, int64_t numel, int mode, void* stream) {
    if ((!x || !y) && numel != 0) return mq_fail(MQ_ERR_ARG, "null pointer");
    if (dtype < MQ_BF16 || dtype > MQ_F32 || numel < 0 || mode < 0 || mode > 2) return mq_fail(MQ_ERR_ARG, "bad argument");
    const int block = mode == 2 ? 16 : 32;
    if (numel % block != 0) return mq_fail(MQ_ERR_ARG, "element count must be a multiple of the block size");
    if (numel == 0) return MQ_OK;
    if ((((uintptr_t)x | (uintptr_t)y) & 15) != 0) {
        const int64_t blocks = numel / block;
        if ((blocks + 255) / 256 > 0x7FFFFFF0ll) return mq_fail(MQ_ERR_ARG, "tensor too large");
        hipLaunchKernelGGL(fake_quant_generic_kernel, dim3((unsigned)((blocks + 255) / 256)), dim3(256), 0,
                           (hipStream_t)stream, x, dtype, y, blocks, mode);
        return mq_check_launch("fake quant");
    }
    const int64_t units = numel / 8;
    if ((units + kFqThreads - 1) / kFqThreads > 0x7FFFFF00ll) return mq_fail(MQ_ERR_ARG, "tensor too large");
    hipStream_t st = (hipStream_t)stream;
    if (mode == 0) launch_fq<0>(x, dtype, y, units, st);
    else if (mode == 1) launch_fq<1>(x, dtype, y, units, st);
    else launch_fq<2>(x, dtype, y, units, st);
    return mq_check_launch("fake quant");
}

template <int DT, bool INPLACE>
static void launch_act(const void* x, void* y, void* scale, int64_t units, int lanes, int flags, hipStream_t st) {
    const int64_t blocks = (units + kFqThreads * kActUnits<INPLACE> - 1) / (kFqThreads * kActUnits<INPLACE>);
    const int chunk = 1;      // this kernel streams 1-2 % faster in plain block order (measured), unlike its neighbours
    const dim3 grid((unsigned)flat_padded(blocks, chunk)), blk(kFqThreads);
    if (lanes == 16) hipLaunchKernelGGL((act_quant_kernel<DT, 16, INPLACE>), grid, blk, 0, st, x, y, scale, units, flags, chunk);
    else if (lanes == 8) hipLaunchKernelGGL((act_quant_kernel<DT, 8, INPLACE>), grid, blk, 0, st, x, y, scale, units, flags, chunk);
    else if (lanes == 4) hipLaunchKernelGGL((act_quant_kernel<DT, 4, INPLACE>), grid, blk, 0, st, x, y, scale, units, flags, chunk);
    else hipLaunchKernelGGL((act_quant_kernel<DT, 2, INPLACE>), grid, blk, 0, st, x, y, scale, units, flags, chunk);
}
template <bool INPLACE>
static void launch_act_dt(const void* x, int dtype, void* y, void* scale, int64_t units, int lanes, int flags, hipStream_t st) {
    if (dtype == MQ_BF16) launch_act<MQ_BF16, INPLACE>(x, y, scale, units, lanes, flags, st);
    else if (dtype == MQ_F16) launch_act<MQ_F16, INPLACE>(x, y, scale, units, lanes, flags, st);
    else launch_act<MQ_F32, INPLACE>(x, y, scale, units, lanes, flags, st);
}

extern "C" int mq_fp8_act_quant(const void* x, int dtype, void* y, void* scale, int64_t numel, int block, int flags,
                                void* stream) {
    if ((!x || !y || !scale) && numel != 0) return mq_fail(MQ_ERR_ARG, "null pointer");
    if (dtype < MQ_BF16 || dtype > MQ_F32 || numel < 0 || block <= 0 || (flags & ~7) != 0) return mq_fail(MQ_ERR_ARG, "bad argument");
    if (numel % block != 0) return mq_fail(MQ_ERR_ARG, "element count must be a multiple of the block size");
    if ((flags & MQ_ACT_SCALE_E8M0) && !(flags & MQ_ACT_ROUND_SCALE))
        return mq_fail(MQ_ERR_ARG, "E8M0 scale storage needs power-of-two scales (MQ_ACT_ROUND_SCALE)");
    if (numel == 0) return MQ_OK;
    hipStream_t st = (hipStream_t)stream;
    const int64_t units = numel / 8;
    const bool inplace = (flags & MQ_ACT_INPLACE) != 0;
    const bool shaped = block == 16 || block == 32 || block == 64 || block == 128;
    const bool aligned = ((uintptr_t)x & 15) == 0 && ((uintptr_t)y & (inplace ? 15 : 7)) == 0 &&
                         ((flags & MQ_ACT_SCALE_E8M0) || ((uintptr_t)scale & 3) == 0);
    if (shaped && aligned && (units + kFqThreads - 1) / kFqThreads <= 0x7FFFFF00ll) {
        if (inplace) launch_act_dt<true>(x, dtype, y, scale, units, block / 8, flags, st);
        else launch_act_dt<false>(x, dtype, y, scale, units, block / 8, flags, st);
    } else {
        const int64_t groups = numel / block;
        if ((groups + 255) / 256 > 0x7FFFFFF0ll) return mq_fail(MQ_ERR_ARG, "tensor too large");
        hipLaunchKernelGGL(act_quant_generic_kernel, dim3((unsigned)((groups + 255) / 256)), dim3(256), 0, st, x, dtype, y,
                           scale, groups, block, flags);
    }
    return mq_check_launch("fp8 act quant");
}
