// MXFP4 (e2m1 codes, two per byte, one E8M0 scale per group) for gfx950.
// Reference: miles/utils/mxfp4.py:11-31 (quantize_mxfp4) and :34-59 (dequantize_mxfp4), plain tensor ops:
//   amax = max|x| over the group;  e = clamp(ceil(log2(amax / 6)), -127, 127);  scale byte = e + 127
//   n = f32(x) * 2^-e;  magnitude = #{b in (0.25, 0.75, 1.25, 1.75, 2.5, 3.5, 5) : |n| > b}   (ties round DOWN)
//   code = magnitude | signbit(n) << 3;  byte j = code(2j) | code(2j+1) << 4
//   dequantize: bf16(sign * {0, .5, 1, 1.5, 2, 3, 4, 6}[magnitude] * 2^(scale - 127))
//
// ceil(log2(q)) is taken from the bits of q = amax / 6.0f (exponent, plus one when the mantissa is not zero).
// For bf16 and fp16 inputs this is what a float log2 followed by ceil returns: q is either an exact power of
// two or at least 2^-11 away from one in relative terms, far more than the rounding of any log2.  For fp32
// inputs within a few ulp above a power of two a float log2 rounds to the integer below and the two differ;
// there the reference's own result depends on the device's log2.
//
// Packed fast path (bf16, group 32): four lanes own one group, 16 bytes in and 4 bytes out per lane.
#include "mq_api_internal.hpp"
#include "mq_common.hpp"
#include "mq_group.hpp"

namespace mq {

constexpr int kM4Threads = 256;
constexpr int kM4Unroll = 2;

// clamp(ceil(log2(q)), -127, 127) + 127 for q >= 0 (q == 0 -> -inf -> 0; inf -> 254)
__device__ __forceinline__ uint32_t mxfp4_scale_byte(float q) {
    const uint32_t u = f2u(q) & 0x7FFFFFFFu;
    const uint32_t e = u >> 23, m = u & 0x7FFFFFu;
    if (e == 0) return m > 0x400000u ? 1u : 0u;   // below 2^-126: -126 only above 2^-127
    uint32_t s = e + (m != 0);
    return s > 254u ? 254u : s;
}
// 2^(127 - byte): the multiplier that normalizes a group
__device__ __forceinline__ float mxfp4_normalizer(uint32_t byte) {
    return u2f(byte == 254u ? 0x00400000u : (254u - byte) << 23);
}
__device__ __forceinline__ uint32_t mxfp4_code(float x, float mult) {
    const float a = __builtin_fabsf(x * mult);
    const uint32_t mag = (a > 0.25f) + (a > 0.75f) + (a > 1.25f) + (a > 1.75f) + (a > 2.5f) + (a > 3.5f) + (a > 5.0f);
    return mag | ((f2u(x) >> 31) << 3);
}

// Scale byte straight from the bf16 pattern of the group amax: amax = m * 2^(E-127), so amax / 6 lies in
// (2^(E-130), 2^(E-129)] for m <= 1.5 and in (2^(E-129), 2^(E-128)) above, i.e. byte = E - 2 + (m > 1.5), floored at
// 0 (covers zero and subnormal amax) and 254 for inf.  Identical to mxfp4_scale_byte(amax / 6.0f) for every bf16
// pattern; no division.
__device__ __forceinline__ uint32_t mxfp4_scale_byte_bf16(uint32_t amax_bits) {
    const int e = (int)(amax_bits >> 7), gt = (amax_bits & 0x7Fu) > 0x40u;
    if (e == 255) return 254u;
    const int b = e - 2 + gt;
    return b < 0 ? 0u : (uint32_t)b;
}
// the same from the fp32 pattern of an amax that came from an fp16 tensor (its subnormals are normal fp32 values)
__device__ __forceinline__ uint32_t mxfp4_scale_byte_f32(uint32_t amax_f32_bits) {
    const int e = (int)(amax_f32_bits >> 23), gt = (amax_f32_bits & 0x7FFFFFu) > 0x400000u;
    if (e == 255) return 254u;
    const int b = e - 2 + gt;
    return b < 0 ? 0u : (uint32_t)b;
}
// The reference's thresholds send a value that sits exactly on a bound to the smaller magnitude, the hardware
// conversion rounds ties to even.  Stepping the magnitude down by one fp32 ulp first makes the two agree: a value
// on a bound lands just below it, and a scaled bf16 or fp16 value (8 / 11 significant bits) can never be the fp32 neighbour just
// above a bound, so nothing else moves across one.  Zero keeps its pattern (and its sign).
__device__ __forceinline__ float step_toward_zero(float n) {
    const uint32_t u = f2u(n);
    return u2f(u - ((u & 0x7FFFFFFFu) != 0));
}

template <class Table, int F16>
__global__ __launch_bounds__(kM4Threads) void mxfp4_bf16_kernel(const Table tab) {
    constexpr uint32_t kInfBits = F16 ? 0x7C00u : 0x7F80u;
    const FlatJob& job = flat_job(tab);
    const uint16_t* __restrict__ w = (const uint16_t*)job.w;
    uint32_t* __restrict__ packed = (uint32_t*)job.q;
    uint8_t* __restrict__ scale = (uint8_t*)job.s;
    const int64_t total_units = job.units;
    const uint32_t t = threadIdx.x;
    const int64_t base = flat_block(tab) * (kM4Threads * kM4Unroll);
    if (base >= total_units) return;
    // everything a lane adds to the workgroup's (uniform) base addresses is a 32-bit offset
    const int64_t left = total_units - base;
    const uint32_t rem = left < kM4Threads * kM4Unroll ? (uint32_t)left : (uint32_t)(kM4Threads * kM4Unroll);
    const uint16_t* __restrict__ w0 = w + base * 8;
    uint32_t* __restrict__ packed0 = packed + base;
    uint8_t* __restrict__ scale0 = scale + base / 4;        // `base` is a multiple of the four lanes of a group
    u32x4 v[kM4Unroll];
#pragma unroll
    for (int i = 0; i < kM4Unroll; i++) {
        const uint32_t off = t + i * kM4Threads;
        v[i] = off < rem ? ld16(w0 + off * 8u) : u32x4{0u, 0u, 0u, 0u};
    }
#pragma unroll
    for (int i = 0; i < kM4Unroll; i++) {
        const uint32_t off = t + i * kM4Threads;
        const uint32_t m2 = max2_u16(max2_u16(abs2(v[i].x), abs2(v[i].y)), max2_u16(abs2(v[i].z), abs2(v[i].w)));
        const uint32_t mb = group_max4(hmax_u16(m2));
        const uint32_t byte = F16 ? mxfp4_scale_byte_f32(f2u(elem_lo<1>(mb))) : mxfp4_scale_byte_bf16(mb);
        const float mult = mxfp4_normalizer(byte);
        const float f[8] = {elem_lo<F16>(v[i].x), elem_hi<F16>(v[i].x), elem_lo<F16>(v[i].y), elem_hi<F16>(v[i].y),
                            elem_lo<F16>(v[i].z), elem_hi<F16>(v[i].z), elem_lo<F16>(v[i].w), elem_hi<F16>(v[i].w)};
        uint32_t word = 0;
        if (mb < kInfBits) {
            float n[8];
#pragma unroll
            for (int j = 0; j < 8; j++) n[j] = step_toward_zero(f[j] * mult);
            word = hw_e2m1x2<0>(n[0], n[1], word);
            word = hw_e2m1x2<1>(n[2], n[3], word);
            word = hw_e2m1x2<2>(n[4], n[5], word);
            word = hw_e2m1x2<3>(n[6], n[7], word);
        } else {
#pragma unroll
            for (int j = 0; j < 8; j++) word |= mxfp4_code(f[j], mult) << (4 * j);
        }
        if (off < rem) {
            st4(packed0 + off, word);
            if ((t & 3) == 0) scale0[off >> 2] = (uint8_t)byte;
        }
    }
}

// any dtype, any group size: scales first (one lane per group), then one lane per output byte
__global__ __launch_bounds__(256) void mxfp4_scale_generic_kernel(const void* __restrict__ w, int dtype,
                                                                  uint8_t* __restrict__ scale, int64_t groups,
                                                                  int G) {
    const int64_t stride = (int64_t)gridDim.x * blockDim.x;
    for (int64_t g = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; g < groups; g += stride) {
        uint32_t m = 0;
        for (int j = 0; j < G; j++) m = umax(m, f2u(load_f32(w, g * G + j, dtype)) & 0x7FFFFFFFu);
        scale[g] = (uint8_t)mxfp4_scale_byte(u2f(m) / 6.0f);
    }
}
__global__ __launch_bounds__(256) void mxfp4_pack_generic_kernel(const void* __restrict__ w, int dtype,
                                                                 const uint8_t* __restrict__ scale,
                                                                 uint8_t* __restrict__ packed, int64_t bytes, int G) {
    const int64_t stride = (int64_t)gridDim.x * blockDim.x;
    for (int64_t b = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; b < bytes; b += stride) {
        const int64_t i0 = 2 * b, i1 = 2 * b + 1;
        const uint32_t lo = mxfp4_code(load_f32(w, i0, dtype), mxfp4_normalizer(scale[i0 / G]));
        const uint32_t hi = mxfp4_code(load_f32(w, i1, dtype), mxfp4_normalizer(scale[i1 / G]));
        packed[b] = (uint8_t)(lo | (hi << 4));
    }
}

// ---- dequantize ---------------------------------------------------------------------------------
// bf16 bit patterns of +{0, .5, 1, 1.5, 2, 3, 4, 6}
__device__ __forceinline__ uint32_t e2m1_bf16_bits(uint32_t mag) {
    const uint64_t lo = 0x3FC03F803F000000ull, hi = 0x40C0408040404000ull;
    return (uint32_t)(((mag & 4u) ? hi : lo) >> ((mag & 3u) * 16)) & 0xFFFFu;
}
// bf16(sign * value * 2^(s-127)): the product has at most two significant bits and bf16 shares fp32's exponent
// range, so it is exact whenever it is finite; s == 255 means 2^128 = inf (0 * inf = NaN, emitted as 0x7FC0).
__device__ __forceinline__ uint32_t mxfp4_decode(uint32_t code, uint32_t s) {
    const uint32_t mag = code & 7u, sign = (code & 8u) << 12;
    if (s == 255u) return mag == 0 ? 0x7FC0u : (sign | 0x7F80u);
    const float factor = u2f(s == 0 ? 0x00400000u : s << 23);
    const float v = u2f(e2m1_bf16_bits(mag) << 16) * factor;
    return sign | (f2u(v) >> 16);
}

// flat: one lane per 4 packed bytes (8 codes -> 16 bytes of bf16), kM4DqUnroll such units per lane; G = 8 << group_shift.
// Scale bytes 2..252 keep every product a normal, finite bf16 number: there the packed hardware conversion
// (two codes per instruction, scaled by 2^(s-127)) is used; the few bytes outside that range take the software form.
#ifndef MQ_M4DQ_UNROLL
#define MQ_M4DQ_UNROLL 2
#endif
constexpr int kM4DqUnroll = MQ_M4DQ_UNROLL;
typedef __bf16 hw_bf16x2_t __attribute__((ext_vector_type(2)));
template <int BYTE>
__device__ __forceinline__ uint32_t hw_e2m1x2_to_bf16x2(uint32_t word, float factor) {
    return __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(word, factor, BYTE));
}
// One tensor of a launch's table per blockIdx.y: w = packed words, q = bf16 output, s = E8M0 bytes, units = words,
// section = log2(words per group).
__global__ __launch_bounds__(256) void mxfp4_dequant_kernel(const FlatTable tab) {
    const FlatJob job = flat_job(tab);
    const uint32_t* __restrict__ packed = (const uint32_t*)job.w;
    const uint8_t* __restrict__ scale = (const uint8_t*)job.s;
    uint16_t* __restrict__ y = (uint16_t*)job.q;
    const int64_t units = job.units;
    const int group_shift = job.section;
    const int64_t first = flat_block(tab) * (256 * kM4DqUnroll);
    if (first >= units) return;          // a smaller tensor of the group
    // everything a lane adds to the workgroup's (uniform) base addresses is a 32-bit offset; `first` is a multiple of
    // the words of a group (at most 256 per unit of a lane, see mq_mxfp4_dequant_fast_ok)
    const int64_t left = units - first;
    const uint32_t rem = left < 256 * kM4DqUnroll ? (uint32_t)left : (uint32_t)(256 * kM4DqUnroll);
    const uint32_t* __restrict__ packed0 = packed + first;
    const uint8_t* __restrict__ scale0 = scale + (first >> group_shift);
    uint16_t* __restrict__ y0 = y + first * 8;
    uint32_t word[kM4DqUnroll], s[kM4DqUnroll];
#pragma unroll
    for (int i = 0; i < kM4DqUnroll; i++) {
        const uint32_t off = threadIdx.x + i * 256u;
        const uint32_t unit = off < rem ? off : 0u;       // past the end: re-read the workgroup's first unit
        word[i] = __builtin_nontemporal_load(packed0 + unit);
        s[i] = scale0[unit >> group_shift];
    }
    __builtin_amdgcn_sched_barrier(0);      // (the scheduler keeps the first unit's conversions below the last load)
#pragma unroll
    for (int i = 0; i < kM4DqUnroll; i++) {
        const uint32_t off = threadIdx.x + i * 256u;
        u32x4 o;
        if (s[i] >= 2u && s[i] <= 252u) {
            const float factor = u2f(s[i] << 23);
            o = u32x4{hw_e2m1x2_to_bf16x2<0>(word[i], factor), hw_e2m1x2_to_bf16x2<1>(word[i], factor),
                      hw_e2m1x2_to_bf16x2<2>(word[i], factor), hw_e2m1x2_to_bf16x2<3>(word[i], factor)};
        } else {
            uint32_t c[8];
#pragma unroll
            for (int j = 0; j < 8; j++) c[j] = mxfp4_decode((word[i] >> (4 * j)) & 0xFu, s[i]);
            o = u32x4{c[0] | (c[1] << 16), c[2] | (c[3] << 16), c[4] | (c[5] << 16), c[6] | (c[7] << 16)};
        }
        if (off < rem) st16(y0 + off * 8u, o);
    }
}
__global__ __launch_bounds__(256) void mxfp4_dequant_generic_kernel(const uint8_t* __restrict__ packed,
                                                                    const uint8_t* __restrict__ scale,
                                                                    uint16_t* __restrict__ y, int64_t bytes, int G) {
    const int64_t stride = (int64_t)gridDim.x * blockDim.x;
    for (int64_t b = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; b < bytes; b += stride) {
        const uint32_t p = packed[b];
        y[2 * b] = (uint16_t)mxfp4_decode(p & 0xFu, scale[(2 * b) / G]);
        y[2 * b + 1] = (uint16_t)mxfp4_decode(p >> 4, scale[(2 * b + 1) / G]);
    }
}

// ---- MXFP4 -> FP8 128x128 re-coder ------------------------------------------------------------------
// Reference: tools/convert_mxfp4_to_fp8.py:30-49 (cast_e2m1fn_to_e4m3fn).  Per 128x128 tile:
//   tile_scale = max(1x32 scales of the tile) / 64;  offset = scale / tile_scale (a power of two <= 64)
//   y = e4m3(fp4_value * offset);  one fp32 tile_scale per tile
// With E8M0 scale bytes s this is tile_scale = 2^(smax-133) and y = e4m3(value * 2^(s-smax+6)): |y| <= 384, so the
// e4m3 cast never overflows and only rounds when the product falls below 2^-6.
// One 256-lane workgroup per pair of tiles that are neighbours along `in` (128 rows x 256 columns).  16 lanes cover
// one row of the pair: a lane reads 8 packed bytes (16 codes) and writes 16 e4m3 bytes, so a row is one whole
// 128-byte line coming in and 256 contiguous bytes going out, and every load and store instruction of a wavefront is a
// run of consecutive 8- or 16-byte pieces.  A lane owns the same 16 columns of 8 rows; two neighbouring lanes share a
// 1x32 group and its scale byte.
// blockIdx.y selects the tensor of a launch of up to kMaxGroup of them (a checkpoint shard's experts); the grid's x
// extent is the largest tensor's, and a tensor deals its own tile pairs to the XCDs in its own chunk length.
__global__ __launch_bounds__(256) void mxfp4_to_fp8_kernel(const RecodeTable tab) {
    __shared__ uint32_t wave_smax[4][2];
    const RecodeJob& job = tab.job[blockIdx.y];
    const int32_t item = xcd_chunked_item(job.total_pairs, job.chunk);
    if (item < 0) return;
    const uint8_t* __restrict__ packed = job.packed;
    const uint8_t* __restrict__ scale = job.scale;
    uint8_t* __restrict__ y = job.y;
    float* __restrict__ tile_scale = job.tile_scale;
    const int64_t in_dim = job.in_dim;
    const int tiles_in = job.tiles_in, pairs_in = job.pairs_in;
    const int t = threadIdx.x;
    const int64_t ti = item / pairs_in, pj = item - ti * pairs_in;
    const int64_t groups_per_row = in_dim / 32;
    const int c = t & 15;                             // 16-column piece of the pair's row
    const int64_t g = pj * 8 + (c >> 1);              // 1x32 group of this lane
    const bool ok = g < groups_per_row;               // the second tile of the last pair may not exist
    const int half = c >> 3;                          // which tile of the pair
    const int64_t gl = ok ? g : groups_per_row - 1;   // lanes past the row re-read its last group: no branch around the loads
    const int64_t piece = ok ? pj * 16 + c : in_dim / 16 - 1;
    u32x2 v[8];
    uint32_t s[8];
#pragma unroll
    for (int i = 0; i < 8; i++) {
        const int64_t row = ti * 128 + i * 16 + (t >> 4);
        v[i] = __builtin_nontemporal_load((const u32x2*)(packed + row * (in_dim / 2)) + piece);
        s[i] = scale[row * groups_per_row + gl];
    }
    uint32_t own = 0;
#pragma unroll
    for (int i = 0; i < 8; i++) own = umax(own, s[i]);
    if (!ok) own = 0u;
    const uint32_t m0 = wave_max(half == 0 ? own : 0u), m1 = wave_max(half == 1 ? own : 0u);
    if ((t & 63) == 0) { wave_smax[t >> 6][0] = m0; wave_smax[t >> 6][1] = m1; }
    __syncthreads();
    const uint32_t smax = umax(umax(wave_smax[0][half], wave_smax[1][half]), umax(wave_smax[2][half], wave_smax[3][half]));
    // 2^(smax - 133): normal from smax = 7 up, an exact fp32 denormal below; byte 255 is E8M0's NaN
    if ((t >> 4) == 0 && (c & 7) == 0 && ok)
        tile_scale[ti * tiles_in + pj * 2 + half] =
            u2f(smax == 255u ? 0x7FC00000u : smax >= 7u ? (smax - 6u) << 23 : 1u << (smax + 16u));
#pragma unroll
    for (int i = 0; i < 8; i++) {
        const int64_t row = ti * 128 + i * 16 + (t >> 4);
        // offset = 2^(s - smax + 6) in (0, 64]; far below the e4m3 range every product rounds to (signed) zero anyway
        const int k = (int)s[i] - (int)smax + 6;
        const float factor = u2f((uint32_t)((k < -60 ? -60 : k) + 127) << 23);
        const uint32_t w[2] = {v[i].x, v[i].y};
        uint32_t o[4];
#pragma unroll
        for (int j = 0; j < 2; j++) {
            const f32x2 a = __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(w[j], 1.0f, 0), b = __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(w[j], 1.0f, 1);
            const f32x2 cc = __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(w[j], 1.0f, 2), d = __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(w[j], 1.0f, 3);
            o[2 * j] = hw_e4m3x4(a.x * factor, a.y * factor, b.x * factor, b.y * factor);
            o[2 * j + 1] = hw_e4m3x4(cc.x * factor, cc.y * factor, d.x * factor, d.y * factor);
        }
        // a NaN scale byte anywhere in the tile makes the tile scale, every offset and every product NaN: code 0x7F
        if (smax == 255u) o[0] = o[1] = o[2] = o[3] = 0x7F7F7F7Fu;
        if (ok) st16(y + row * in_dim + pj * 256 + c * 16, u32x4{o[0], o[1], o[2], o[3]});
    }
}

// ---- the same re-coding as two flat launches ----------------------------------------------------------------------
// The tile form writes 256-byte row pieces at the pitch of the matrix, and such writes stream at 5.5 TB/s on this part
// where a run of consecutive 16-byte stores reaches 6.9; the output is two thirds of the traffic.  Only the tile scale
// ties an element to its tile, and the scale bytes are 2 % of the bytes: a first launch reads them alone (a band of 128
// rows is one contiguous run, and each dword of it holds the four 1x32 groups of one tile row) and writes the fp32
// tile scales; the second launch is a flat stream -- a lane takes 16 consecutive elements, its group's scale byte is
// element index / 32, and the tile maximum comes back out of the fp32 tile scale's bit pattern.
// One workgroup per band of 128 rows: a lane owns a dword column (one tile) and keeps its running maximum in a
// register over the 32 rows of its wavefront; the four wavefronts meet in LDS.  Bands wider than 64 tiles go round again.
__global__ __launch_bounds__(256) void mxfp4_tile_smax_kernel(const RecodeTable tab) {
    __shared__ uint32_t part[4][64];
    const RecodeJob& job = tab.job[blockIdx.y];
    const int tiles_in = job.tiles_in;
    const int64_t band = blockIdx.x;
    if (band >= (job.pairs_in ? job.total_pairs / job.pairs_in : 0)) return;         // this tensor has fewer row bands
    const int t = threadIdx.x, lane = t & 63, wave = t >> 6;
    const uint32_t* __restrict__ words = (const uint32_t*)job.scale + band * 128 * tiles_in;
    for (int c0 = 0; c0 < tiles_in; c0 += 64) {
        const int c = c0 + lane;
        const bool live = c < tiles_in;
        uint32_t w[32];
#pragma unroll
        for (int i = 0; i < 32; i++) w[i] = live ? words[(wave * 32 + i) * tiles_in + c] : 0u;
        uint32_t m2 = 0;             // the even and the odd bytes as two pairs of 16-bit values
#pragma unroll
        for (int i = 0; i < 32; i++) m2 = max2_u16(m2, max2_u16(w[i] & 0x00FF00FFu, (w[i] >> 8) & 0x00FF00FFu));
        part[wave][lane] = hmax_u16(m2);
        __syncthreads();
        if (wave == 0 && live) {
            const uint32_t m = umax(umax(part[0][lane], part[1][lane]), umax(part[2][lane], part[3][lane]));
            // 2^(smax - 133): normal from smax = 7 up, an exact fp32 denormal below; byte 255 is E8M0's NaN
            job.tile_scale[band * tiles_in + c] = u2f(m == 255u ? 0x7FC00000u : m >= 7u ? (m - 6u) << 23 : 1u << (m + 16u));
        }
        __syncthreads();
    }
}
#ifndef MQ_RECODE_UNROLL
#define MQ_RECODE_UNROLL 2
#endif
// 16-element units per lane, 256 lanes apart, every load issued before the first conversion.  Measured on
// 8 x [16384, 7168] as one job list: 5.79 / 6.20 / 6.11 TB/s with one / two / four units.
constexpr int kRecodeUnroll = MQ_RECODE_UNROLL;
__global__ __launch_bounds__(256) void mxfp4_recode_flat_kernel(const RecodeTable tab) {
    const RecodeJob& job = tab.job[blockIdx.y];
    const int64_t base64 = xcd_chunked_block(job.flat_chunk) * (256 * kRecodeUnroll) + threadIdx.x;
    if (base64 >= job.units) return;
    const uint32_t base = (uint32_t)base64;
    const uint32_t upr = (uint32_t)(job.in_dim / 16);
    u32x2 v[kRecodeUnroll];
    uint32_t s[kRecodeUnroll], bits[kRecodeUnroll];
#pragma unroll
    for (int i = 0; i < kRecodeUnroll; i++) {
        const uint32_t u = base + i * 256;
        const uint32_t uc = u < job.units ? u : base;          // a dead unit repeats the lane's first one and stores nothing
        const uint32_t row = tile_div(uc, job.magic_upr, job.shift_upr), cu = uc - row * upr;
        v[i] = ((const u32x2*)job.packed)[uc];      // an ordinary load: 8-byte loads measured 0.5 % faster without the non-temporal hint
        s[i] = job.scale[uc >> 1];
        bits[i] = f2u(job.tile_scale[(uint64_t)(row >> 7) * job.tiles_in + (cu >> 3)]);
    }
    __builtin_amdgcn_sched_barrier(0);      // (the scheduler keeps the first unit's arithmetic below the last load)
#pragma unroll
    for (int i = 0; i < kRecodeUnroll; i++) {
        const uint32_t u = base + i * 256;
        if (u >= job.units) break;
        const uint32_t e = bits[i] >> 23;
        const uint32_t smax = bits[i] == 0x7FC00000u ? 255u : e != 0u ? e + 6u : (uint32_t)(31 - __builtin_clz(bits[i] | 1u)) - 16u;
        // offset = 2^(s - smax + 6) in (0, 64]; far below the e4m3 range every product rounds to (signed) zero anyway
        const int k = (int)s[i] - (int)smax + 6;
        const float factor = u2f((uint32_t)((k < -60 ? -60 : k) + 127) << 23);
        const uint32_t w[2] = {v[i].x, v[i].y};
        uint32_t o[4];
#pragma unroll
        for (int j = 0; j < 2; j++) {
            const f32x2 a = __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(w[j], 1.0f, 0), b = __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(w[j], 1.0f, 1);
            const f32x2 cc = __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(w[j], 1.0f, 2), d = __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(w[j], 1.0f, 3);
            o[2 * j] = hw_e4m3x4(a.x * factor, a.y * factor, b.x * factor, b.y * factor);
            o[2 * j + 1] = hw_e4m3x4(cc.x * factor, cc.y * factor, d.x * factor, d.y * factor);
        }
        // a NaN scale byte anywhere in the tile makes the tile scale, every offset and every product NaN: code 0x7F
        if (smax == 255u) o[0] = o[1] = o[2] = o[3] = 0x7F7F7F7Fu;
        st16(job.y + (uint64_t)u * 16, u32x4{o[0], o[1], o[2], o[3]});
    }
}

}  // namespace mq

using namespace mq;

bool mq_mxfp4_fast_ok(const void* w, int dtype, const void* packed, int group) {
    return (dtype == MQ_BF16 || dtype == MQ_F16) && group == 32 && ((uintptr_t)w % 16) == 0 && ((uintptr_t)packed % 4) == 0;
}

int mq_mxfp4_launch_group(int dtype, FlatTable& tab, hipStream_t st) {
    if (!flat_grid(tab, kM4Threads * kM4Unroll)) return mq_fail(MQ_ERR_ARG, "tensor too large");
    if (tab.max_blocks == 0) return MQ_OK;
    const dim3 grid((unsigned)tab.max_blocks, (unsigned)tab.n), blk(kM4Threads);
    if (dtype == MQ_F16) hipLaunchKernelGGL((mxfp4_bf16_kernel<FlatTable, 1>), grid, blk, 0, st, tab);
    else hipLaunchKernelGGL((mxfp4_bf16_kernel<FlatTable, 0>), grid, blk, 0, st, tab);
    return mq_check_launch("mxfp4 quant");
}

int mq_mxfp4_launch_table(int dtype, const FlatJob* device_jobs, int n, int64_t max_units, hipStream_t st) {
    FlatRef ref{device_jobs, 0, 0};
    if (!flat_grid(ref, max_units, kM4Threads * kM4Unroll)) return mq_fail(MQ_ERR_ARG, "tensor too large");
    if (ref.max_blocks == 0 || n == 0) return MQ_OK;
    const dim3 grid((unsigned)ref.max_blocks, (unsigned)n), blk(kM4Threads);
    if (dtype == MQ_F16) hipLaunchKernelGGL((mxfp4_bf16_kernel<FlatRef, 1>), grid, blk, 0, st, ref);
    else hipLaunchKernelGGL((mxfp4_bf16_kernel<FlatRef, 0>), grid, blk, 0, st, ref);
    return mq_check_launch("mxfp4 quant");
}

extern "C" int mq_mxfp4_quant(const void* w, int dtype, uint8_t* packed, uint8_t* scale, int64_t numel, int group,
                              void* stream) {
    if ((!w || !packed || !scale) && numel != 0) return mq_fail(MQ_ERR_ARG, "null pointer");
    if (dtype < MQ_BF16 || dtype > MQ_F32 || numel < 0 || group <= 0) return mq_fail(MQ_ERR_ARG, "bad argument");
    if (numel % group != 0 || numel % 2 != 0) return mq_fail(MQ_ERR_ARG, "element count must be a multiple of the group size and of 2");
    if (numel == 0) return MQ_OK;
    hipStream_t st = (hipStream_t)stream;
    if (mq_mxfp4_fast_ok(w, dtype, packed, group)) {
        FlatTable tab{};
        tab.n = 1;
        tab.job[0] = FlatJob{w, packed, scale, nullptr, numel / 8, nullptr, 0, 0};
        return mq_mxfp4_launch_group(dtype, tab, st);
    }
    const int64_t groups = numel / group, bytes = numel / 2;
    int64_t blocks = (groups + 255) / 256;
    if (blocks > mq_grid_cap()) blocks = mq_grid_cap();
    hipLaunchKernelGGL(mxfp4_scale_generic_kernel, dim3((unsigned)blocks), dim3(256), 0, st, w, dtype, scale, groups, group);
    int rc = mq_check_launch("mxfp4 scales");
    if (rc != MQ_OK) return rc;
    blocks = (bytes + 255) / 256;
    if (blocks > mq_grid_cap()) blocks = mq_grid_cap();
    hipLaunchKernelGGL(mxfp4_pack_generic_kernel, dim3((unsigned)blocks), dim3(256), 0, st, w, dtype, (const uint8_t*)scale, packed, bytes, group);
    return mq_check_launch("mxfp4 pack");
}

// the flat kernel takes whole words and groups of a power-of-two number of words
bool mq_mxfp4_dequant_fast_ok(const void* packed, const void* y, int64_t bytes, int group) {
    const int upg = group / 8;
    return group > 0 && group <= 2048 * kM4DqUnroll && group % 8 == 0 && (upg & (upg - 1)) == 0 && bytes % 4 == 0 &&
           ((uintptr_t)packed % 4) == 0 && ((uintptr_t)y % 16) == 0;
}
FlatJob mq_mxfp4_dequant_entry(const void* packed, const void* scale, void* y, int64_t bytes, int group) {
    int shift = 0;
    while ((1 << shift) < group / 8) shift++;
    return FlatJob{packed, y, (void*)scale, nullptr, bytes / 4, nullptr, shift, 0};
}
// up to kMaxGroup tensors in one launch
int mq_mxfp4_dequant_launch_group(FlatTable& tab, hipStream_t st) {
    if (!flat_grid(tab, 256 * kM4DqUnroll)) return mq_fail(MQ_ERR_ARG, "tensor too large");
    if (tab.max_blocks == 0) return MQ_OK;
    hipLaunchKernelGGL(mxfp4_dequant_kernel, dim3((unsigned)tab.max_blocks, (unsigned)tab.n), dim3(256), 0, st, tab);
    return mq_check_launch("mxfp4 dequant");
}

extern "C" int mq_mxfp4_dequant(const uint8_t* packed, const uint8_t* scale, void* y, int64_t bytes, int group,
                                void* stream) {
    if ((!packed || !scale || !y) && bytes != 0) return mq_fail(MQ_ERR_ARG, "null pointer");
    if (bytes < 0 || group <= 0) return mq_fail(MQ_ERR_ARG, "bad argument");
    if ((2 * bytes) % group != 0) return mq_fail(MQ_ERR_ARG, "element count must be a multiple of the group size");
    if (bytes == 0) return MQ_OK;
    hipStream_t st = (hipStream_t)stream;
    if (mq_mxfp4_dequant_fast_ok(packed, y, bytes, group)) {
        FlatTable tab{};
        tab.n = 1;
        tab.job[0] = mq_mxfp4_dequant_entry(packed, scale, y, bytes, group);
        return mq_mxfp4_dequant_launch_group(tab, st);
    }
    int64_t blocks = (bytes + 255) / 256;
    if (blocks > mq_grid_cap()) blocks = mq_grid_cap();
    hipLaunchKernelGGL(mxfp4_dequant_generic_kernel, dim3((unsigned)blocks), dim3(256), 0, st, packed, scale, (uint16_t*)y,
                       bytes, group);
    return mq_check_launch("mxfp4 dequant");
}

// fills one descriptor; the shape checks of mq_mxfp4_to_fp8_block
int mq_mxfp4_to_fp8_job(RecodeJob& job, const void* packed, const void* scale, void* y, void* tile_scale, int64_t out_dim,
                        int64_t in_dim) {
    if ((!packed || !scale || !y || !tile_scale) && out_dim != 0 && in_dim != 0) return mq_fail(MQ_ERR_ARG, "null pointer");
    if (out_dim < 0 || in_dim < 0 || out_dim % 128 != 0 || in_dim % 128 != 0)
        return mq_fail(MQ_ERR_ARG, "both dimensions must be multiples of 128");
    if ((((uintptr_t)packed | (uintptr_t)y) & 15) != 0) return mq_fail(MQ_ERR_ARG, "tensors must be 16-byte aligned");
    const int64_t tiles_in = in_dim / 128, pairs_in = (tiles_in + 1) / 2, pairs = (out_dim / 128) * pairs_in;
    // An XCD takes whole 128-row bands when there are enough of them: the band's scale bytes are one contiguous run,
    // and dealt out in smaller pieces every 128-byte line of them was fetched by four XCDs (measured: 0.625 bytes
    // read per element against 0.531 algorithmic).
    const int64_t chunk = (out_dim / 128 >= 2 * kXcds && pairs_in <= 4096) ? pairs_in : MQ_XCD_CHUNK;
    if (xcd_grid_chunked(pairs, chunk) > 0x7FFFFFF0ll) return mq_fail(MQ_ERR_ARG, "tensor too large");
    job = RecodeJob{(const uint8_t*)packed, (const uint8_t*)scale, (uint8_t*)y, (float*)tile_scale, in_dim,
                    (int32_t)tiles_in, (int32_t)pairs_in, (int32_t)pairs, (int32_t)chunk, 0u, 0u, 0u, 0};
    const int64_t units = out_dim * (in_dim / 16);
    if (units > 0 && units < 0x7FFFFFFFll && ((uintptr_t)scale & 3) == 0) {
        job.units = (uint32_t)units;
        tile_div_magic((uint32_t)(in_dim / 16), job.magic_upr, job.shift_upr);
        job.flat_chunk = (int32_t)flat_chunk((units + 256 * kRecodeUnroll - 1) / (256 * kRecodeUnroll));
    }
    return MQ_OK;
}
int mq_mxfp4_to_fp8_launch_group(const RecodeTable& tab, hipStream_t st) {
    // two tensors and more share the two launches of the flat form; a single call keeps the one launch of the tile form
    // (2 % faster alone: the second launch's start costs more than the write pattern)
    bool flat = tab.n > 1;
    int64_t bands = 0, blocks = 0;
    for (int i = 0; i < tab.n; i++) {
        const RecodeJob& j = tab.job[i];
        flat = flat && (j.units != 0 || j.total_pairs == 0);
        const int64_t b = j.pairs_in ? j.total_pairs / j.pairs_in : 0;
        bands = b > bands ? b : bands;
        const int64_t g = j.units ? flat_padded(((int64_t)j.units + 256 * kRecodeUnroll - 1) / (256 * kRecodeUnroll), j.flat_chunk) : 0;
        blocks = g > blocks ? g : blocks;
    }
    if (flat) {
        if (bands == 0) return MQ_OK;
        hipLaunchKernelGGL(mxfp4_tile_smax_kernel, dim3((unsigned)bands, (unsigned)tab.n), dim3(256), 0, st, tab);
        hipLaunchKernelGGL(mxfp4_recode_flat_kernel, dim3((unsigned)blocks, (unsigned)tab.n), dim3(256), 0, st, tab);
        return mq_check_launch("mxfp4 to fp8");
    }
    int64_t grid = 0;
    for (int i = 0; i < tab.n; i++) {
        const int64_t g = xcd_grid_chunked(tab.job[i].total_pairs, tab.job[i].chunk);
        grid = g > grid ? g : grid;
    }
    if (grid == 0 || tab.n == 0) return MQ_OK;
    hipLaunchKernelGGL(mxfp4_to_fp8_kernel, dim3((unsigned)grid, (unsigned)tab.n), dim3(256), 0, st, tab);
    return mq_check_launch("mxfp4 to fp8");
}

extern "C" int mq_mxfp4_to_fp8_block(const uint8_t* packed, const uint8_t* scale, void* y, float* tile_scale,
                                     int64_t out_dim, int64_t in_dim, void* stream) {
    RecodeTable tab{};
    tab.n = 1;
    int rc = mq_mxfp4_to_fp8_job(tab.job[0], packed, scale, y, tile_scale, out_dim, in_dim);
    if (rc != MQ_OK) return rc;
    return mq_mxfp4_to_fp8_launch_group(tab, (hipStream_t)stream);
}
