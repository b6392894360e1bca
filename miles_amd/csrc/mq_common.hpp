// Shared device helpers for the gfx950 weight-quantization kernels.
//
// Conventions used by every kernel in this directory:
//  * wavefront = 64 lanes; a 16-byte (8 x bf16) load per lane is the unit of coalescing;
//  * all floating-point arithmetic is IEEE binary32 round-to-nearest-even; the library is built
//    with -ffp-contract=off so a fused multiply-add appears only where __builtin_fmaf is written;
//  * conversions to e4m3 / e2m1 / bf16 use the gfx950 convert instructions; their agreement with
//    the software round-to-nearest-even forms below over every fp32 bit pattern is checked by
//    mq_selftest_convert, which the GPU test suite runs.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace mq {

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef uint16_t u16x2 __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));

constexpr int kWave = 64;
constexpr float kFp8Max = 448.0f;
constexpr float kFltMax = 3.402823466e+38f;

__device__ __forceinline__ float u2f(uint32_t u) { return __builtin_bit_cast(float, u); }
__device__ __forceinline__ uint32_t f2u(float f) { return __builtin_bit_cast(uint32_t, f); }

// ---- input element access -------------------------------------------------------------------
// A 32-bit word holds two 16-bit elements, element 0 in the low half.
__device__ __forceinline__ float bf16_lo(uint32_t w) { return u2f(w << 16); }
__device__ __forceinline__ float bf16_hi(uint32_t w) { return u2f(w & 0xFFFF0000u); }
// A 16-bit element of the input as a float: a bf16 is the upper half of the float, an fp16 goes through the converter
// (exact, subnormals included).  The absolute bit patterns of both formats order like the values they stand for, so
// kernels take maxima on the patterns and convert once.
template <int F16>
__device__ __forceinline__ float elem_lo(uint32_t w) {
    if (F16) return (float)__builtin_bit_cast(_Float16, (uint16_t)w);
    return bf16_lo(w);
}
template <int F16>
__device__ __forceinline__ float elem_hi(uint32_t w) {
    if (F16) return (float)__builtin_bit_cast(_Float16, (uint16_t)(w >> 16));
    return bf16_hi(w);
}

// |x| of both halves, compared as unsigned 16-bit integers: for bf16 (and fp16) the ordering of
// non-negative finite values equals the ordering of their bit patterns, and a NaN pattern is
// larger than every finite one, so a NaN input surfaces as a NaN amax.
__device__ __forceinline__ uint32_t abs2(uint32_t w) { return w & 0x7FFF7FFFu; }
__device__ __forceinline__ uint32_t max2_u16(uint32_t a, uint32_t b) {
    u16x2 r = __builtin_elementwise_max(__builtin_bit_cast(u16x2, a), __builtin_bit_cast(u16x2, b));
    return __builtin_bit_cast(uint32_t, r);
}
// larger half of a packed pair, as a 16-bit pattern in the low bits
__device__ __forceinline__ uint32_t hmax_u16(uint32_t p) {
    uint32_t lo = p & 0xFFFFu, hi = p >> 16;
    return lo > hi ? lo : hi;
}

// ---- cross-lane max (unsigned; used on non-negative float bit patterns) ----------------------
template <int CTRL>
__device__ __forceinline__ uint32_t dpp_u32(uint32_t v) {
    return (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, CTRL, 0xF, 0xF, false);
}
constexpr int kDppQuadXor1 = 0xB1;    // quad_perm:[1,0,3,2]
constexpr int kDppQuadXor2 = 0x4E;    // quad_perm:[2,3,0,1]
constexpr int kDppRowHalfMirror = 0x141;
constexpr int kDppRowMirror = 0x140;

__device__ __forceinline__ uint32_t umax(uint32_t a, uint32_t b) { return a > b ? a : b; }

// max over aligned groups of 2 / 4 / 8 / 16 lanes; every lane of the group gets the result
__device__ __forceinline__ uint32_t group_max2(uint32_t v) { return umax(v, dpp_u32<kDppQuadXor1>(v)); }
__device__ __forceinline__ uint32_t group_max4(uint32_t v) {
    v = umax(v, dpp_u32<kDppQuadXor1>(v));
    return umax(v, dpp_u32<kDppQuadXor2>(v));
}
__device__ __forceinline__ uint32_t group_max8(uint32_t v) {
    v = group_max4(v);
    return umax(v, dpp_u32<kDppRowHalfMirror>(v));
}
__device__ __forceinline__ uint32_t group_max16(uint32_t v) {
    v = group_max8(v);
    return umax(v, dpp_u32<kDppRowMirror>(v));
}
// max over the whole wavefront, returned wave-uniform
__device__ __forceinline__ uint32_t wave_max(uint32_t v) {
    v = group_max16(v);
    uint32_t a = (uint32_t)__builtin_amdgcn_readlane((int)v, 0);
    uint32_t b = (uint32_t)__builtin_amdgcn_readlane((int)v, 16);
    uint32_t c = (uint32_t)__builtin_amdgcn_readlane((int)v, 32);
    uint32_t d = (uint32_t)__builtin_amdgcn_readlane((int)v, 48);
    return umax(umax(a, b), umax(c, d));
}

// ---- exact division by a divisor shared by many elements -------------------------------------
// q = RN(w / s) from y = RN(1/s):  q0 = RN(w*y); e = q0*s - w (exact in an FMA); q = RN(q0 - e*y).
// For a numerator with at most 11 significant bits (bf16, fp16) this equals the correctly rounded
// quotient for every divisor mantissa (exhaustive check: 2^23 divisors x all numerator mantissas),
// provided no intermediate under/overflows; callers guard the exponent range of s.
// The residual is taken as q0*s - w and subtracted (a source negation, free on v_fma_f32) rather than
// w - q0*s added: for a zero numerator the first form gives e = +0 and q = q0 - (+0) = q0, which keeps
// the sign of a -0 numerator as the division itself does; the second form would return +0 for -0.
__device__ __forceinline__ float div_by_shared(float w, float s, float y) {
    float q0 = w * y;
    float e = __builtin_fmaf(q0, s, -w);
    return __builtin_fmaf(-e, y, q0);
}
// y = RN(1/s) for div_by_shared: the hardware reciprocal (within one ulp) and one Newton step, three instructions where
// the IEEE division 1.0f / s takes eleven.  On gfx950 the result equals that division for every divisor in the range
// of shared_div_ok (mq_selftest_reciprocal compares them over the whole range on the device); outside that range the
// callers do not use y.
__device__ __forceinline__ float recip_shared(float s) {
    const float r = __builtin_amdgcn_rcpf(s);
    const float e = __builtin_fmaf(-s, r, 1.0f);
    return __builtin_fmaf(e, r, r);
}
// divisor range in which div_by_shared is used; outside it kernels fall back to operator/
__device__ __forceinline__ bool shared_div_ok(float s) {
    uint32_t a = f2u(s) & 0x7FFFFFFFu;
    return a >= 0x12000000u /* 2^-91 */ && a <= 0x6C800000u /* 2^90 */;
}

// ---- software conversions (reference forms; also the fallbacks for special values) -----------
// float -> e4m3fn, round to nearest even, no saturation: values that round past 448 and NaN give
// 0x7F | sign (PyTorch float8_e4m3fn cast).
__device__ __forceinline__ uint32_t sw_e4m3fn(float x) {
    uint32_t u = f2u(x), sign = (u >> 24) & 0x80u, a = u & 0x7FFFFFFFu;
    if (a >= 0x43F00000u) return sign | 0x7Fu;
    if (a < 0x3C800000u) {
        float k = __builtin_rintf(u2f(a) * 512.0f);
        return sign | (uint32_t)k;
    }
    uint32_t lsb = (a >> 20) & 1u;
    a += 0x7FFFFu + lsb;                 // RNE at bit 20, carries into the exponent
    uint32_t code = (a >> 20) - (120u << 3);
    return sign | (code > 0x7Fu ? 0x7Fu : code);
}
// clamp that leaves NaN alone, like torch.clamp (v_med3_f32 alone would return the lower bound for a NaN)
__device__ __forceinline__ float clamp_keep_nan(float v, float lo, float hi) {
    return v != v ? v : __builtin_amdgcn_fmed3f(v, lo, hi);
}
// saturating form: |x| >= 448 and inf -> 0x7E | sign, NaN -> 0x7F
__device__ __forceinline__ uint32_t sw_e4m3fn_sat(float x) {
    uint32_t u = f2u(x), a = u & 0x7FFFFFFFu;
    if (a > 0x7F800000u) return 0x7Fu;
    if (a >= 0x43E00000u) return ((u >> 24) & 0x80u) | 0x7Eu;
    return sw_e4m3fn(x);
}
// float -> e2m1, round to nearest, ties to even code, saturating at 6, NaN -> 0x7
__device__ __forceinline__ uint32_t sw_e2m1(float x) {
    uint32_t u = f2u(x), sign = (u >> 28) & 0x8u, a = u & 0x7FFFFFFFu;
    if (a > 0x7F800000u) return 0x7u;
    float v = u2f(a);
    uint32_t c = (v > 0.25f) + (v >= 0.75f) + (v > 1.25f) + (v >= 1.75f) + (v > 2.5f) + (v >= 3.5f) + (v > 5.0f);
    return sign | c;
}
// float -> bf16 bits, round to nearest even, NaN -> 0x7FC0
__device__ __forceinline__ uint32_t sw_bf16(float f) {
    uint32_t u = f2u(f);
    if ((u & 0x7FFFFFFFu) > 0x7F800000u) return 0x7FC0u;
    return (u + 0x7FFFu + ((u >> 16) & 1u)) >> 16;
}
__device__ __forceinline__ float sw_e4m3fn_decode(uint32_t c) {
    uint32_t sign = (c & 0x80u) << 24, e = (c >> 3) & 0xFu, m = c & 7u;
    if (e == 15 && m == 7) return u2f(sign | 0x7FC00000u);
    if (e == 0) return u2f(f2u((float)m * 0.001953125f) | sign);
    return u2f(sign | ((e + 120u) << 23) | (m << 20));
}

// ---- E8M0 scales of the MX formats ---------------------------------------------------------------
// exponent byte of the smallest power of two >= v, for v >= 0: saturating at 0xFE (inf included), 0 for v == 0 and for
// subnormals up to 2^-127, 0xFF for a NaN
__device__ __forceinline__ uint32_t e8m0_ceil(float v) {
    const uint32_t u = f2u(v);
    uint32_t e = u >> 23, m = u & 0x7FFFFFu;
    if (u >= 0x7F800000u) return u == 0x7F800000u ? 0xFEu : 0xFFu;
    if ((m > 0 && e != 0xFEu) && !(e == 0 && m <= 0x400000u)) e++;
    return e;
}
// 2^(127 - e), exact (subnormal for the two largest bytes); 1 for byte 0
__device__ __forceinline__ float e8m0_inverse(uint32_t e) {
    if (e == 0) return 1.0f;
    if (e >= 254) return u2f(e == 254 ? 0x00400000u : 0x00200000u);
    return u2f((254u - e) << 23);
}

// ---- hardware conversions ---------------------------------------------------------------------
// two floats -> two e4m3 bytes in the low (hi=false) or high (hi=true) half of `old`.
// v_cvt_pk_fp8_f32 rounds to nearest even including into the subnormal range and rounds (448, 464]
// down to 448; inputs here are always within +-(448 + a few ulp) or NaN.
template <bool HI>
__device__ __forceinline__ uint32_t hw_e4m3x2(float a, float b, uint32_t old) {
    return (uint32_t)__builtin_amdgcn_cvt_pk_fp8_f32(a, b, (int)old, HI);
}
__device__ __forceinline__ uint32_t hw_e4m3x4(float a, float b, float c, float d) {
    uint32_t r = hw_e4m3x2<false>(a, b, 0u);
    return hw_e4m3x2<true>(c, d, r);
}
// two e4m3 bytes (low or high half of w) -> two floats
template <bool HI>
__device__ __forceinline__ f32x2 hw_e4m3x2_decode(uint32_t w) {
    return __builtin_amdgcn_cvt_pk_f32_fp8((int)w, HI);
}
// two floats -> one byte of two e2m1 codes (a in the low nibble) placed in byte SEL of `old`
template <int SEL>
__device__ __forceinline__ uint32_t hw_e2m1x2(float a, float b, uint32_t old) {
    return __builtin_amdgcn_cvt_scalef32_pk_fp4_f32(old, a, b, 1.0f, SEL);
}
// two floats -> packed bf16 pair (a in the low half), round to nearest even
__device__ __forceinline__ uint32_t hw_bf16x2(float a, float b) {
    f32x2 v = {a, b};
    bf16x2 r = __builtin_convertvector(v, bf16x2);
    return __builtin_bit_cast(uint32_t, r);
}

// ---- streaming global access -------------------------------------------------------------------
// Every byte on this path is touched exactly once, so loads and stores carry the non-temporal hint:
// measured on MI355X this adds about 5% of achieved HBM bandwidth over plain accesses.
__device__ __forceinline__ u32x4 ld16(const void* p) {
    return __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(p));
}
// A pointer that was itself loaded from device memory (a descriptor table) is a generic pointer to the compiler, and
// generic accesses are flat instructions, which measured 15 % slower than global ones in the streaming kernels.  Loading
// the pointer through a type that says "global" (the same 8 bytes) and converting it to a generic pointer afterwards
// lets the compiler's address-space inference turn every access through it into a global one.
#define MQ_GLOBAL __attribute__((address_space(1)))
template <class T>
__device__ __forceinline__ T* load_global_ptr(T* const* slot) {
    return (T*)*static_cast<MQ_GLOBAL T* const*>(static_cast<const void*>(slot));
}
// plain (cacheable) load for data that a following pass reads again
__device__ __forceinline__ u32x4 ld16_keep(const void* p) { return *reinterpret_cast<const u32x4*>(p); }
__device__ __forceinline__ void st16(void* p, u32x4 v) { __builtin_nontemporal_store(v, reinterpret_cast<u32x4*>(p)); }
__device__ __forceinline__ void st8(void* p, u32x2 v) { __builtin_nontemporal_store(v, reinterpret_cast<u32x2*>(p)); }
__device__ __forceinline__ void st4(void* p, uint32_t v) { __builtin_nontemporal_store(v, reinterpret_cast<uint32_t*>(p)); }

}  // namespace mq
