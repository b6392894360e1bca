// INT4 group quantization for gfx950.
//
//  mq_int4_fake_quant       restates fake_int4_quant_cuda for block (1, G)
//                           (reference: miles/kernels/quant/int4_fake/fake_int4_quant_cuda.cu:29-91,159-259):
//                             sym : scale = fmaxf(amax*(1/7), 1e-5);  out = rintf(x/scale)
//                             asym: scale = fmaxf((max-min)*(1/15), 1e-5); zero = clamp(-rintf(min/scale),0,15);
//                                   out = rintf(x/scale) + zero
//                           out / scale / zero are stored in the dtype of x.
//  mq_int4_group_quant_pack fuses the symmetric kernel with pack_layer's Python half
//                           (reference: .../processors/quantizer_compressed_tensors.py:137-265):
//                           code = rintf(x/scale_f32) + 8 in [1,15]; eight codes per int32, element 8j+i in bits
//                           4i..4i+3; scale stored as bf16.  The bf16 round trip that pack_layer performs
//                           (w = q*scale_b, q' = round(w/scale_b)) returns q for every |q| <= 7 and every scale
//                           below 4.8e37, so the codes come straight from the fp32 quotient; groups with a larger
//                           scale or a non-finite element run the round trip as written.
//
// Packed fast path (bf16, G = 8 * LANES): LANES lanes own one group, 16 bytes each; the group amax is a DPP
// max over the LANES-lane segment; x/scale uses the shared-divisor sequence (3 FMA-class ops per element,
// exactly rounded) and rint + the +8 offset are one fp32 add of 1.5*2^23 + 8.
#include "mq_api_internal.hpp"
#include "mq_common.hpp"
#include "mq_group.hpp"
#include "mq_io8.hpp"

namespace mq {

constexpr float kSymCons = 1.0f / 7.0f;
constexpr float kAsymCons = 1.0f / 15.0f;
constexpr int kI4Threads = 256;
#ifndef MQ_I4_UNROLL
#define MQ_I4_UNROLL 2
#endif
constexpr int kI4Unroll = MQ_I4_UNROLL;

template <int LANES>
__device__ __forceinline__ uint32_t seg_max(uint32_t v) {
    if (LANES == 16) return group_max16(v);
    if (LANES == 8) return group_max8(v);
    if (LANES == 4) return group_max4(v);
    if (LANES == 2) return group_max2(v);
    return v;
}

// nibble = (rint(q) + 8) & 15 taken from the low bits of q + (1.5*2^23 + 8)
__device__ __forceinline__ uint32_t code_bits(float q) { return f2u(q + 12582920.0f); }

// The fused form of the packed kernel relies on the round trip q -> bf16(q * scale_b) -> bf16(. / scale_b) being the
// identity.  It is for every group maximum below the largest finite bf16 (all maxima x all codes checked on the CPU);
// at that maximum 7 * scale_b overflows, and an infinity or a NaN breaks it too.  This function runs the chain as
// written for one unit: NaN skipped by the group maximum as the reference's fmaxf reduction does, codes above 15
// carrying into the next nibble as in its int32 sum.
// rounding of an fp32 value to the tensor's 16-bit dtype (as a float again, or as the stored pattern)
template <int F16>
__device__ __forceinline__ float round16(float x) {
    if (F16) return (float)(_Float16)x;
    return u2f(sw_bf16(x) << 16);
}
template <int F16>
__device__ __forceinline__ uint16_t bits16(float x) {
    if (F16) return __builtin_bit_cast(uint16_t, (_Float16)x);
    return (uint16_t)sw_bf16(x);
}
template <int LANES, int F16>
__device__ __forceinline__ void int4_pack_chain_unit(const u32x4 v, const int64_t unit, const bool live,
                                                               const int t, uint32_t* __restrict__ packed,
                                                               uint16_t* __restrict__ scale) {
    const float f[8] = {elem_lo<F16>(v.x), elem_hi<F16>(v.x), elem_lo<F16>(v.y), elem_hi<F16>(v.y),
                        elem_lo<F16>(v.z), elem_hi<F16>(v.z), elem_lo<F16>(v.w), elem_hi<F16>(v.w)};
    uint32_t m = 0;
#pragma unroll
    for (int j = 0; j < 8; j++) {
        const uint32_t a = f2u(f[j]) & 0x7FFFFFFFu;
        m = umax(m, a > 0x7F800000u ? 0u : a);
    }
    const float s = __builtin_fmaxf(u2f(seg_max<LANES>(m)) * kSymCons, 1e-5f);
    const float sb = round16<F16>(s);
    uint32_t word = 0;
#pragma unroll 1
    for (int j = 0; j < 8; j++) {
        const uint32_t pair = j < 2 ? v.x : j < 4 ? v.y : j < 6 ? v.z : v.w;
        const float x = (j & 1) ? elem_hi<F16>(pair) : elem_lo<F16>(pair);
        const float q0 = round16<F16>(__builtin_rintf(x / s));
        const float wv = round16<F16>(q0 * sb);
        const float rv = clamp_keep_nan(round16<F16>(wv / sb), -128.0f, 127.0f);
        word += (uint32_t)(((int)__builtin_rintf(rv) + 8) & 0xFF) << (4 * j);
    }
    if (live) {
        st4(packed + unit, word);
        if ((t & (LANES - 1)) == 0) scale[unit / LANES] = bits16<F16>(s);
    }
}

// 16-bit inputs, bf16 or fp16 (F16).  The fused form rests on the reference's dequantize / requantize round trip in the
// tensor's dtype being the identity on the codes: proved for bf16 scales, and checked over every fp16 scale from the
// floor fp16(1e-5) up (all 31 576 patterns x the fifteen codes): it fails only where 7 x scale overflows, which needs a
// group maximum of 65504, the largest fp16.
template <int LANES, class Table, int F16>
__global__ __launch_bounds__(kI4Threads) void int4_pack_bf16_kernel(const Table tab) {
    constexpr uint32_t kTopBits = F16 ? 0x7BFFu : 0x7F7Fu;      // the largest finite value; infinities and NaN lie above
    const FlatJob& job = flat_job(tab);
    const uint16_t* __restrict__ w = (const uint16_t*)job.w;
    uint32_t* __restrict__ packed = (uint32_t*)job.q;
    uint16_t* __restrict__ scale = (uint16_t*)job.s;
    const int64_t total_units = job.units;
    const uint32_t t = threadIdx.x;
    const int64_t base = flat_block(tab) * (kI4Threads * kI4Unroll);
    if (base >= total_units) return;
    // everything a lane adds to the workgroup's (uniform) base addresses is a 32-bit offset
    const int64_t left = total_units - base;
    const uint32_t rem = left < kI4Threads * kI4Unroll ? (uint32_t)left : (uint32_t)(kI4Threads * kI4Unroll);
    const uint16_t* __restrict__ w0 = w + base * 8;
    uint32_t* __restrict__ packed0 = packed + base;
    uint16_t* __restrict__ scale0 = scale + base / LANES;        // `base` is a multiple of the lanes per group
    u32x4 v[kI4Unroll];
#pragma unroll
    for (int i = 0; i < kI4Unroll; i++) {
        const uint32_t off = t + i * kI4Threads;
        v[i] = off < rem ? ld16(w0 + off * 8u) : u32x4{0u, 0u, 0u, 0u};
    }
    uint32_t top = 0;
#pragma unroll
    for (int i = 0; i < kI4Unroll; i++) {
        const int64_t unit = base + i * kI4Threads + t;
        const uint32_t m2 = max2_u16(max2_u16(abs2(v[i].x), abs2(v[i].y)), max2_u16(abs2(v[i].z), abs2(v[i].w)));
        const uint32_t mb = seg_max<LANES>(hmax_u16(m2));
        top = umax(top, mb);
        const float amax = elem_lo<F16>(mb);
        const float s = __builtin_fmaxf(amax * kSymCons, 1e-5f);
        const float y = recip_shared(s);
        const float f[8] = {elem_lo<F16>(v[i].x), elem_hi<F16>(v[i].x), elem_lo<F16>(v[i].y), elem_hi<F16>(v[i].y),
                            elem_lo<F16>(v[i].z), elem_hi<F16>(v[i].z), elem_lo<F16>(v[i].w), elem_hi<F16>(v[i].w)};
        const bool fast = shared_div_ok(s);
        // |x / s| <= 7 (1 + 2^-23), so the pattern of q + (1.5 * 2^23 + 8) is 0x4B400000 + nibble: the eight patterns
        // are summed at their nibble's place (one shift-add each, modulo 2^32) and what the high bits added up to is
        // taken off once.  (A wavefront that met an infinity, a NaN or the largest finite value writes its words again below.)
        constexpr uint32_t kMagicSum = 0x4B400000u + (0x4B400000u << 4) + (0x4B400000u << 8);     // further shifts: 0
        uint32_t word = 0;
        if (__builtin_amdgcn_ballot_w64(!fast) == 0) {         // every scale of the wavefront in range: one straight run
#pragma unroll
            for (int j = 0; j < 8; j++) word += code_bits(div_by_shared(f[j], s, y)) << (4 * j);
        } else {
#pragma unroll
            for (int j = 0; j < 8; j++) {
                const float qv = fast ? div_by_shared(f[j], s, y) : f[j] / s;
                word += code_bits(qv) << (4 * j);
            }
        }
        word -= kMagicSum;
        const uint32_t off = t + i * kI4Threads;
        if (off < rem) {
            st4(packed0 + off, word);
            if ((t & (LANES - 1)) == 0) scale0[off / LANES] = F16 ? bits16<1>(s) : (uint16_t)hw_bf16x2(s, 0.0f);
        }
    }
    // A group holding the largest finite value of the dtype, an infinity or a NaN is outside the fused form: a wavefront that met one
    // writes all of its groups again through the written-out chain (a scalar branch after the common path, which
    // therefore stays one straight instruction stream; the later store of a lane to the same address wins).
    if (__builtin_amdgcn_ballot_w64(top >= kTopBits) == 0) return;
#pragma unroll
    for (int i = 0; i < kI4Unroll; i++) {
        const int64_t unit = base + i * kI4Threads + t;
        int4_pack_chain_unit<LANES, F16>(v[i], unit, unit < total_units, t, packed, scale);
    }
}

// One wavefront per group, lanes stride its elements: any dtype, any block (BM, BN) -- a group is a BM x BN tile of
// the matrix, rows and columns past the edge count as 0 in the extrema -- symmetric and asymmetric.
__global__ __launch_bounds__(256) void int4_fake_generic_kernel(const void* __restrict__ x, int dtype,
                                                                void* __restrict__ out, void* __restrict__ scale_out,
                                                                void* __restrict__ zero_out, int64_t M, int64_t N,
                                                                int BM, int BN, int64_t groups_per_row, int64_t total,
                                                                int sym) {
    const int lane = threadIdx.x & 63;
    const int64_t wave = ((int64_t)blockIdx.x * blockDim.x + threadIdx.x) >> 6;
    const int64_t nwaves = ((int64_t)gridDim.x * blockDim.x) >> 6;
    const int elems = BM * BN;
    for (int64_t g = wave; g < total; g += nwaves) {
        const int64_t bi = g / groups_per_row, bj = g - bi * groups_per_row;
        const int64_t r0 = bi * BM, c0 = bj * BN;
        float mx = -__builtin_inff(), mn = __builtin_inff();
        for (int k = lane; k < elems; k += 64) {
            const int64_t r = r0 + k / BN, c = c0 + k % BN;
            const float val = (r < M && c < N) ? load_f32(x, r * N + c, dtype) : 0.0f;
            if (sym) mx = __builtin_fmaxf(mx, __builtin_fabsf(val));
            else { mx = __builtin_fmaxf(mx, val); mn = __builtin_fminf(mn, val); }
        }
        for (int off = 32; off > 0; off >>= 1) {
            mx = __builtin_fmaxf(mx, __shfl_xor(mx, off, 64));
            mn = __builtin_fminf(mn, __shfl_xor(mn, off, 64));
        }
        float s, zero = 0.0f;
        if (sym) s = __builtin_fmaxf(mx * kSymCons, 1e-5f);
        else {
            s = __builtin_fmaxf((mx - mn) * kAsymCons, 1e-5f);
            // max(-0, +0) is +0 in the reference's device code: adding +0 makes that explicit
            zero = __builtin_fminf(__builtin_fmaxf(-__builtin_rintf(mn / s), 0.0f), 15.0f) + 0.0f;
        }
        for (int k = lane; k < elems; k += 64) {
            const int64_t r = r0 + k / BN, c = c0 + k % BN;
            if (r < M && c < N) {
                float qv = __builtin_rintf(load_f32(x, r * N + c, dtype) / s);
                if (!sym) qv = qv + zero;
                store_dtype(out, r * N + c, qv, dtype);
            }
        }
        if (lane == 0) {
            store_dtype(scale_out, g, s, dtype);
            if (!sym) store_dtype(zero_out, g, zero, dtype);
        }
    }
}

// pack_layer for dtypes / group sizes the fast kernel does not take: follows the reference chain literally,
// one lane per packed word.
__global__ __launch_bounds__(256) void int4_pack_generic_kernel(const void* __restrict__ w, int dtype,
                                                                uint32_t* __restrict__ packed,
                                                                void* __restrict__ scale_out, int64_t M, int64_t K,
                                                                int G) {
    const int64_t words_per_row = K / 8, total = M * words_per_row, gpr = K / G;
    const int64_t stride = (int64_t)gridDim.x * blockDim.x;
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += stride) {
        const int64_t r = i / words_per_row, j = i - r * words_per_row;
        uint32_t word = 0;
        for (int k = 0; k < 8; k++) {
            const int64_t c = j * 8 + k;
            const int64_t g0 = (c / G) * G;
            float amax = -__builtin_inff();
            for (int e = 0; e < G; e++) amax = __builtin_fmaxf(amax, __builtin_fabsf(load_f32(w, r * K + g0 + e, dtype)));
            const float s = __builtin_fmaxf(amax * kSymCons, 1e-5f);
            const float q0 = round_to_dtype(__builtin_rintf(load_f32(w, r * K + c, dtype) / s), dtype);
            const float sb = round_to_dtype(s, dtype);
            const float wv = round_to_dtype(q0 * sb, dtype);
            float rv = round_to_dtype(wv / sb, dtype);
            rv = clamp_keep_nan(rv, -128.0f, 127.0f);
            const int qi = (int)__builtin_rintf(rv);                     // NaN converts to 0
            word += (uint32_t)((qi + 8) & 0xFF) << (4 * k);
            if (c == g0) store_dtype(scale_out, r * gpr + c / G, s, dtype);
        }
        packed[i] = word;
    }
}

// ---- asymmetric pack_layer ---------------------------------------------------------------------
// The reference runs the asymmetric fake-quant kernel and then dequantizes / requantizes in the weight's
// dtype D before packing (quantizer_compressed_tensors.py:235-264).  With rd() = round to D:
//   s = fmaxf((max-min)*(1/15), 1e-5);  z = clamp(-rintf(min/s), 0, 15)          (.cu:226-229)
//   w1 = rd(rintf(x/s) + z);  sb = rd(s)                                          (.cu:244-254)
//   w2 = rd(rd(w1 - z) * sb)                                                      (py:243)
//   r  = rd(rd(w2 / sb) + z);  code = uint8(round_half_even(clamp(r, 0, 255)))    (py:213-220,190)
//   word = sum_i code_i << 4i  (int32 wraparound: codes above 15 carry)           (py:173-175)
// Nothing clamps w1, so codes above 15 do occur (a group whose minimum is far above zero); the carry
// is part of the reference's result and is kept.
template <int DT>
__device__ __forceinline__ void load8(const void* p, int64_t word, float f[8]) {
    if (DT == MQ_F32) {
        const u32x4 a = ld16((const float*)p + word * 8), b = ld16((const float*)p + word * 8 + 4);
        f[0] = u2f(a.x); f[1] = u2f(a.y); f[2] = u2f(a.z); f[3] = u2f(a.w);
        f[4] = u2f(b.x); f[5] = u2f(b.y); f[6] = u2f(b.z); f[7] = u2f(b.w);
    } else {
        const u32x4 a = ld16((const uint16_t*)p + word * 8);
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

// the same for a tensor that does not start on a 16-byte boundary: element by element
template <int DT>
__device__ __forceinline__ void load8_any(const void* p, int64_t word, float f[8], bool aligned) {
    if (aligned) { load8<DT>(p, word, f); return; }
#pragma unroll
    for (int i = 0; i < 8; i++) f[i] = load_f32(p, word * 8 + i, DT);
}

// 16 lanes own one group; a lane handles the 8-element words lane, lane+16, ... of it.
template <int DT>
__global__ __launch_bounds__(256) void int4_pack_asym_kernel(const void* __restrict__ w,
                                                             uint32_t* __restrict__ packed,
                                                             void* __restrict__ scale_out,
                                                             uint8_t* __restrict__ zero_out, int64_t total_groups,
                                                             int words_per_group, bool aligned) {
    const int lane = threadIdx.x & 15;
    const int64_t team = ((int64_t)blockIdx.x * blockDim.x + threadIdx.x) >> 4;
    const int64_t nteams = ((int64_t)gridDim.x * blockDim.x) >> 4;
    // every lane of a wavefront runs the same number of trips so the shuffles below always see all 64 lanes
    const int64_t trips = (total_groups + nteams - 1) / nteams;
    for (int64_t it = 0; it < trips; it++) {
        const int64_t g = team + it * nteams;
        const bool live = g < total_groups;
        const int64_t word0 = live ? g * words_per_group : 0;
        float mx = -__builtin_inff(), mn = __builtin_inff();
        float f[8];
        if (live)
            for (int k = lane; k < words_per_group; k += 16) {
                load8_any<DT>(w, word0 + k, f, aligned);
#pragma unroll
                for (int i = 0; i < 8; i++) { mx = __builtin_fmaxf(mx, f[i]); mn = __builtin_fminf(mn, f[i]); }
            }
        for (int off = 8; off > 0; off >>= 1) {
            mx = __builtin_fmaxf(mx, __shfl_xor(mx, off, 64));
            mn = __builtin_fminf(mn, __shfl_xor(mn, off, 64));
        }
        if (!live) continue;
        const float s = __builtin_fmaxf((mx - mn) * kAsymCons, 1e-5f);
        const float z = __builtin_fminf(__builtin_fmaxf(-__builtin_rintf(mn / s), 0.0f), 15.0f) + 0.0f;
        const float sb = round_to_dtype(s, DT);
        const float ys = 1.0f / s, yb = 1.0f / sb;
        // the shared-divisor sequence needs finite intermediates: quotients stay far below 2^100
        const float big = __builtin_fmaxf(__builtin_fabsf(mx), __builtin_fabsf(mn));
        const bool fast = DT != MQ_F32 && shared_div_ok(s) && shared_div_ok(sb) && big * ys < 1e30f;
        for (int k = lane; k < words_per_group; k += 16) {
            load8_any<DT>(w, word0 + k, f, aligned);
            uint32_t word = 0;
#pragma unroll
            for (int i = 0; i < 8; i++) {
                const float q = fast ? div_by_shared(f[i], s, ys) : f[i] / s;
                const float w1 = round_to_dtype(__builtin_rintf(q) + z, DT);
                const float w2 = round_to_dtype(round_to_dtype(w1 - z, DT) * sb, DT);
                // w1 * sb may have overflowed the dtype: the sequence needs a finite numerator
                const float d = (fast && __builtin_fabsf(w2) < __builtin_inff()) ? div_by_shared(w2, sb, yb) : w2 / sb;
                float r = round_to_dtype(round_to_dtype(d, DT) + z, DT);
                r = clamp_keep_nan(r, 0.0f, 255.0f);
                word += (uint32_t)__builtin_rintf(r) << (4 * i);
            }
            packed[word0 + k] = word;
        }
        if (lane == 0) {
            store_dtype(scale_out, g, s, DT);
            zero_out[g] = (uint8_t)z;
        }
    }
}

// bf16 fast path of the asymmetric packer: LANES lanes own one group (16 bytes each, G = 8 * LANES) and the data
// stays in registers between the min/max pass and the coding pass.  In the written-out chain min and max travel
// through the unsigned DPP reduction as order-preserving integer keys, and every rounding to bf16 is the packed
// hardware conversion.
__device__ __forceinline__ uint32_t order_key(float f) {
    const uint32_t u = f2u(f);
    return u ^ ((u >> 31) ? 0xFFFFFFFFu : 0x80000000u);
}
__device__ __forceinline__ float order_unkey(uint32_t k) {
    return u2f(k ^ ((k >> 31) ? 0x80000000u : 0xFFFFFFFFu));
}
// two values rounded to the tensor's 16-bit dtype (bf16: the packed hardware conversion)
template <int F16>
__device__ __forceinline__ void rd16x2(float& a, float& b) {
    if (F16) {
        a = (float)(_Float16)a;
        b = (float)(_Float16)b;
    } else {
        const uint32_t p = hw_bf16x2(a, b);
        a = bf16_lo(p);
        b = bf16_hi(p);
    }
}
// One 16-byte unit of one lane, LANES neighbouring lanes hold the rest of the group: the chain as written, with IEEE
// divisions.  The packed kernel sends here the wavefronts that met a group outside its fused form (minimum above zero
// or far below it, huge scales, infinities, NaN).
template <int LANES, int F16>
__device__ __forceinline__ void int4_asym_unit(const u32x4 v, const bool live, const int64_t unit, const int t,
                                               uint32_t* __restrict__ packed, uint16_t* __restrict__ scale_out,
                                               uint8_t* __restrict__ zero_out) {
    float f[8] = {elem_lo<F16>(v.x), elem_hi<F16>(v.x), elem_lo<F16>(v.y), elem_hi<F16>(v.y),
                  elem_lo<F16>(v.z), elem_hi<F16>(v.z), elem_lo<F16>(v.w), elem_hi<F16>(v.w)};
    float mx = f[0], mn = f[0];
#pragma unroll
    for (int i = 1; i < 8; i++) { mx = __builtin_fmaxf(mx, f[i]); mn = __builtin_fminf(mn, f[i]); }
    mx = mx != mx ? -__builtin_inff() : mx;         // eight NaNs in one lane: the group reduction skips them
    mn = mn != mn ? __builtin_inff() : mn;
    mx = order_unkey(seg_max<LANES>(order_key(mx)));
    mn = order_unkey(~seg_max<LANES>(~order_key(mn)));
    const float s = __builtin_fmaxf((mx - mn) * kAsymCons, 1e-5f);
    const float sb = round16<F16>(s);
    const float z = __builtin_fminf(__builtin_fmaxf(-__builtin_rintf(mn / s), 0.0f), 15.0f) + 0.0f;
    uint32_t word = 0;
    float q[8];
#pragma unroll
    for (int i = 0; i < 8; i++) q[i] = __builtin_rintf(f[i] / s) + z;
#pragma unroll
    for (int i = 0; i < 8; i += 2) rd16x2<F16>(q[i], q[i + 1]);
#pragma unroll
    for (int i = 0; i < 8; i++) q[i] = q[i] - z;
#pragma unroll
    for (int i = 0; i < 8; i += 2) rd16x2<F16>(q[i], q[i + 1]);
#pragma unroll
    for (int i = 0; i < 8; i++) q[i] = q[i] * sb;
#pragma unroll
    for (int i = 0; i < 8; i += 2) rd16x2<F16>(q[i], q[i + 1]);
#pragma unroll
    for (int i = 0; i < 8; i++) q[i] = q[i] / sb;
#pragma unroll
    for (int i = 0; i < 8; i += 2) rd16x2<F16>(q[i], q[i + 1]);
#pragma unroll
    for (int i = 0; i < 8; i++) q[i] = q[i] + z;
#pragma unroll
    for (int i = 0; i < 8; i += 2) rd16x2<F16>(q[i], q[i + 1]);
#pragma unroll
    for (int i = 0; i < 8; i++)
        word += (uint32_t)__builtin_rintf(clamp_keep_nan(q[i], 0.0f, 255.0f)) << (4 * i);
    if (live) {
        st4(packed + unit, word);
        if ((t & (LANES - 1)) == 0) {
            scale_out[unit / LANES] = bits16<F16>(s);
            zero_out[unit / LANES] = (uint8_t)z;
        }
    }
}
// Max of `mx` and min of `mn` over aligned groups of LANES lanes, for floats that are not NaN.  Written as instructions:
// through the builtins every step costs a move, a quieting of the moved value and the max itself.  A DPP operand must
// have been written two issue slots earlier (whatever the compiler put in front of the block included), so the block
// opens with two idle slots and the two chains alternate with one idle slot per step.
#define MQ_EXTREMA_FIRST(ctrl)                                               \
    "v_max_f32_dpp %0, %2, %2 " ctrl " row_mask:0xf bank_mask:0xf\n\t"        \
    "v_min_f32_dpp %1, %3, %3 " ctrl " row_mask:0xf bank_mask:0xf\n\t"
#define MQ_EXTREMA_STEP(ctrl)                                                \
    "v_max_f32_dpp %0, %0, %0 " ctrl " row_mask:0xf bank_mask:0xf\n\t"        \
    "v_min_f32_dpp %1, %1, %1 " ctrl " row_mask:0xf bank_mask:0xf\n\t"
template <int LANES>
__device__ __forceinline__ void seg_extrema(float& mx, float& mn) {
    static_assert(LANES == 4 || LANES == 8 || LANES == 16, "group of 32, 64 or 128 elements");
    float gx, gn;          // results in registers of their own: tied operands made the compiler copy the inputs first
    if (LANES == 4)
        asm volatile("s_nop 1\n\t" MQ_EXTREMA_FIRST("quad_perm:[1,0,3,2]") "s_nop 0\n\t" MQ_EXTREMA_STEP("quad_perm:[2,3,0,1]")
                     : "=&v"(gx), "=&v"(gn) : "v"(mx), "v"(mn));
    else if (LANES == 8)
        asm volatile("s_nop 1\n\t" MQ_EXTREMA_FIRST("quad_perm:[1,0,3,2]") "s_nop 0\n\t" MQ_EXTREMA_STEP("quad_perm:[2,3,0,1]")
                     "s_nop 0\n\t" MQ_EXTREMA_STEP("row_half_mirror")
                     : "=&v"(gx), "=&v"(gn) : "v"(mx), "v"(mn));
    else
        asm volatile("s_nop 1\n\t" MQ_EXTREMA_FIRST("quad_perm:[1,0,3,2]") "s_nop 0\n\t" MQ_EXTREMA_STEP("quad_perm:[2,3,0,1]")
                     "s_nop 0\n\t" MQ_EXTREMA_STEP("row_half_mirror") "s_nop 0\n\t" MQ_EXTREMA_STEP("row_mirror")
                     : "=&v"(gx), "=&v"(gn) : "v"(mx), "v"(mn));
    mx = gx;
    mn = gn;
}
#undef MQ_EXTREMA_FIRST
#undef MQ_EXTREMA_STEP
// job: w, q = packed codes, s = scales, aux = zero points (one byte per group, read again by the zero-point packer),
// aux2 = packed zero points, units, section = groups per row
//
// Every group first runs the fused form as one straight instruction stream: scale and zero point from the group's
// extrema, codes = rint(x / s) + z through the shared-divisor sequence.  The form is final when the scale is in the
// range of that sequence, the zero point was not clamped (lo = rint(min / s) in [-15, 0]) and bf16(s) <= 1e37: then
// every rint(x / s) + z is an integer in [0, 16] -- (max - min) / s <= 15 (1 + 2^-22) because s >= RN(RN(max - min) / 15),
// and two roundings to integer lie at most one further apart than their arguments -- and for such codes the reference's
// dequantize / requantize round trip in bf16 returns the code itself (checked exhaustively on the CPU: all scales x
// all codes x all zero points).  A wavefront that met any other group (minimum above zero or far below it, huge or
// non-finite values) writes its groups again through int4_asym_unit, the chain as written; the later store wins.
// (fp16 instance, F16: the same check over every fp16 scale from fp16(1e-5) upwards holds for all scales below 4096,
// where 16 x scale stays finite; a group with a larger scale takes the chain.)
template <int LANES, class Table, int F16>
__global__ __launch_bounds__(kI4Threads) void int4_pack_asym_bf16_kernel(const Table tab) {
    const FlatJob& job = flat_job(tab);
    const uint16_t* __restrict__ w = (const uint16_t*)job.w;
    uint32_t* __restrict__ packed = (uint32_t*)job.q;
    uint16_t* __restrict__ scale_out = (uint16_t*)job.s;
    uint8_t* __restrict__ zero_out = (uint8_t*)job.aux;
    const int64_t total_units = job.units;
    const uint32_t t = threadIdx.x;
    const int64_t first = flat_block(tab) * (kI4Threads * kI4Unroll);
    if (first >= total_units) return;
    // everything a lane adds to the workgroup's (uniform) base addresses is a 32-bit offset
    const int64_t left = total_units - first;
    const uint32_t rem = left < kI4Threads * kI4Unroll ? (uint32_t)left : (uint32_t)(kI4Threads * kI4Unroll);
    const uint16_t* __restrict__ w0 = w + first * 8;
    uint32_t* __restrict__ packed0 = packed + first;
    uint16_t* __restrict__ scale0 = scale_out + first / LANES;        // `first` is a multiple of the lanes per group
    uint8_t* __restrict__ zero0 = zero_out + first / LANES;
    // a group is a whole number of lanes, so dead lanes never share one with live lanes; they re-read the last unit
    u32x4 v[kI4Unroll];
#pragma unroll
    for (int i = 0; i < kI4Unroll; i++) {
        const uint32_t off = t + i * kI4Threads;
        v[i] = ld16(w0 + (off < rem ? off : rem - 1) * 8u);
    }
    // wavefronts with a group outside the fused form: the tests are collected as wavefront masks (scalar registers)
    uint64_t odd = 0;
    uint32_t word[kI4Unroll], sb[kI4Unroll], z[kI4Unroll];
#pragma unroll
    for (int i = 0; i < kI4Unroll; i++) {
        const float f[8] = {elem_lo<F16>(v[i].x), elem_hi<F16>(v[i].x), elem_lo<F16>(v[i].y), elem_hi<F16>(v[i].y),
                            elem_lo<F16>(v[i].z), elem_hi<F16>(v[i].z), elem_lo<F16>(v[i].w), elem_hi<F16>(v[i].w)};
        float mx = f[0], mn = f[0];
#pragma unroll
        for (int j = 1; j < 8; j++) { mx = __builtin_fmaxf(mx, f[j]); mn = __builtin_fminf(mn, f[j]); }
        // a NaN element is skipped by the extrema but is not coded like a number: its wavefront takes the chain below,
        // whatever the fused form makes of the group (an unordered compare takes two elements at a time)
#pragma unroll
        for (int j = 0; j < 8; j += 2) odd |= __builtin_amdgcn_ballot_w64(!(f[j] == f[j]) || !(f[j + 1] == f[j + 1]));
        seg_extrema<LANES>(mx, mn);
        const float s = __builtin_fmaxf((mx - mn) * kAsymCons, 1e-5f);
        const float ys = recip_shared(s);
        sb[i] = F16 ? (uint32_t)bits16<1>(s) : hw_bf16x2(s, 0.0f);
        if (F16) odd |= __builtin_amdgcn_ballot_w64(!(s < 4094.0f));        // fp16(s) below 4096: 16 x scale stays finite
        // The zero point unclamped: lo = rint(min / s) in [-15, 0].  Every quotient of the group then lies within +-16,
        // far from the range limits of the shared-divisor sequence, and bf16(s) <= 2^90 (1 + 2^-8) is far below 1e37.
        // One infinite extremum makes s infinite, which shared_div_ok refuses; a group of equal infinities has the
        // floor scale and lo = NaN, which fails both comparisons.
        const float lo = __builtin_rintf(div_by_shared(mn, s, ys));
        z[i] = (uint32_t)(int)(0.0f - lo);
        odd |= __builtin_amdgcn_ballot_w64(!shared_div_ok(s));
        odd |= __builtin_amdgcn_ballot_w64(!(lo <= 0.0f));
        odd |= __builtin_amdgcn_ballot_w64(!(lo >= -15.0f));
        // rint through one add of 1.5 * 2^23: the low bits of the sum's pattern are the (signed) integer.  The zero point
        // is added as an integer afterwards (inside the float add an odd zero point would turn the ties around);
        // everything is arithmetic modulo 2^32, like the reference's int32 sum.
        constexpr uint32_t kMagicSum = 0x4B400000u + (0x4B400000u << 4) + (0x4B400000u << 8);     // further shifts: 0
        uint32_t sum = 0;
#pragma unroll
        for (int j = 0; j < 8; j++) sum += f2u(div_by_shared(f[j], s, ys) + 12582912.0f) << (4 * j);
        // z in every nibble (z <= 15 where the word is kept): z * 0x11 in the low byte, the byte copied to all four
        const uint32_t zz = __builtin_amdgcn_perm(0u, z[i] | (z[i] << 4), 0u);
        word[i] = sum - kMagicSum + zz;
    }
    // all stores after all loads have been used: a store between them would have to complete before the next unit's
    // data counts as arrived (loads and stores return in order)
#pragma unroll
    for (int i = 0; i < kI4Unroll; i++) {
        const uint32_t off = t + i * kI4Threads;
        if (off < rem) {
            st4(packed0 + off, word[i]);
            if ((t & (LANES - 1)) == 0) {
                scale0[off / LANES] = (uint16_t)sb[i];
                zero0[off / LANES] = (uint8_t)z[i];
            }
        }
    }
    const int64_t base = first + t;
    if (odd == 0) return;
#pragma unroll
    for (int i = 0; i < kI4Unroll; i++) {
        const int64_t unit = base + i * kI4Threads;
        int4_asym_unit<LANES, F16>(v[i], unit < total_units, unit, t, packed, scale_out, zero_out);
    }
}

// packed_zp[g, j] = sum_i zero[8j+i, g] << 4*order[i], order = {0,4,1,5,2,6,3,7}   (py:249-254)
// `zero` is [rows, groups_per_row] bytes and the packed words are its transpose, eight rows to a word.  A workgroup
// takes a tile of 256 rows x 64 groups through LDS: the bytes are read along the rows (neighbouring lanes, neighbouring
// bytes) and the words written along j (32 consecutive words of one group per half wavefront).
constexpr int kZpRows = 256, kZpCols = 64, kZpPitch = kZpCols + 4;
__host__ __device__ __forceinline__ int64_t int4_zero_tiles(int64_t rows8, int64_t groups_per_row) {
    return ((rows8 * 8 + kZpRows - 1) / kZpRows) * ((groups_per_row + kZpCols - 1) / kZpCols);
}
__device__ __forceinline__ void int4_zero_pack_tile(const uint8_t* __restrict__ zero, uint32_t* __restrict__ packed_zp,
                                                    const int64_t rows8, const int64_t groups_per_row, const int64_t tile,
                                                    uint8_t* lds) {
    const int64_t col_tiles = (groups_per_row + kZpCols - 1) / kZpCols;
    const int64_t row0 = (tile / col_tiles) * kZpRows, g0 = (tile % col_tiles) * kZpCols;
    const int64_t rows = rows8 * 8;
    const int t = threadIdx.x;
    if ((groups_per_row & 3) == 0 && ((uintptr_t)zero & 3) == 0) {
        // four bytes per lane and every load of the tile issued before the first is used: one memory round trip
        const int c = (t & 15) * 4;
        const bool col_live = g0 + c < groups_per_row;
        uint32_t v[kZpRows / 16];
#pragma unroll
        for (int i = 0; i < kZpRows / 16; i++) {
            const int r = (t >> 4) + 16 * i;
            const bool live = col_live && row0 + r < rows;
            v[i] = live ? *(const uint32_t*)(zero + (row0 + r) * groups_per_row + g0 + c) : 0u;
        }
#pragma unroll
        for (int i = 0; i < kZpRows / 16; i++) *(uint32_t*)(lds + ((t >> 4) + 16 * i) * kZpPitch + c) = v[i];
    } else {
        const int c = t & (kZpCols - 1);
        const bool col_live = g0 + c < groups_per_row;
#pragma unroll 8
        for (int r = t / kZpCols; r < kZpRows; r += 256 / kZpCols) {
            const bool live = col_live && row0 + r < rows;
            lds[r * kZpPitch + c] = live ? zero[(row0 + r) * groups_per_row + g0 + c] : (uint8_t)0;
        }
    }
    __syncthreads();
    const int j = t & (kZpRows / 8 - 1);
    const int64_t jj = row0 / 8 + j;
    if (jj >= rows8) return;
#pragma unroll
    for (int g = t / (kZpRows / 8); g < kZpCols; g += 256 / (kZpRows / 8)) {
        if (g0 + g >= groups_per_row) break;
        uint32_t word = 0;
#pragma unroll
        for (int k = 0; k < 8; k++) {
            const int nib = (k >> 1) + 4 * (k & 1);
            word += (uint32_t)lds[(j * 8 + k) * kZpPitch + g] << (4 * nib);
        }
        packed_zp[(g0 + g) * rows8 + jj] = word;
    }
}
__global__ __launch_bounds__(256) void int4_zero_pack_kernel(const uint8_t* __restrict__ zero,
                                                             uint32_t* __restrict__ packed_zp, int64_t M,
                                                             int64_t groups_per_row) {
    __shared__ __align__(4) uint8_t lds[kZpRows * kZpPitch];
    int4_zero_pack_tile(zero, packed_zp, M / 8, groups_per_row, blockIdx.x, lds);
}
// the zero points of a group of tensors (descriptors as for int4_pack_asym_bf16_kernel): blockIdx.y selects the tensor;
// a tensor of `units` 16-byte units has units / units_per_group groups, groups_per_row of them in each row
template <class Table>
__global__ __launch_bounds__(256) void int4_zero_pack_group_kernel(const Table tab, int units_per_group) {
    __shared__ __align__(4) uint8_t lds[kZpRows * kZpPitch];
    const FlatJob& job = flat_job(tab);
    const int64_t groups_per_row = job.section;
    if (groups_per_row <= 0) return;
    const int64_t rows8 = job.units / units_per_group / groups_per_row / 8;
    if (blockIdx.x >= int4_zero_tiles(rows8, groups_per_row)) return;
    int4_zero_pack_tile((const uint8_t*)job.aux, (uint32_t*)job.aux2, rows8, groups_per_row, blockIdx.x, lds);
}

// ---- fake INT4 quantization of row blocks (1, G), G = 32 / 64 / 128 ------------------------------------------------
// The standalone form of the reference's extension (fake_int4_quant_cuda.cu:29-91 for G = 32, :159-259 otherwise):
// `out` holds the integer codes as values of the input dtype, `scale` (and `zero`) one value per block in that dtype.
//   symmetric:  s = max(amax * f32(1/7), 1e-5);   out = rint(x / s)
//   asymmetric: s = max((max - min) * f32(1/15), 1e-5);   z = min(max(-rint(min / s), +0), 15);   out = rint(x / s) + z
// Lanes own 8 consecutive elements, G / 8 neighbouring lanes a block; x / s is the exact quotient (shared-divisor
// sequence for 16-bit inputs, the sign of a -0 numerator put back; the division itself otherwise).
template <int DT, int LANES, bool SYM>
__global__ __launch_bounds__(kI4Threads) void int4_fake_rows_kernel(const void* __restrict__ x, void* __restrict__ out,
                                                                    void* __restrict__ scale_out,
                                                                    void* __restrict__ zero_out, int64_t units, int chunk) {
    const int64_t unit = xcd_chunked_block(chunk) * kI4Threads + threadIdx.x;
    const bool live = unit < units;            // a block is a whole number of lanes: dead lanes never share one with live lanes
    float f[8], q[8];
    fq_load8<DT>(x, live ? unit : units - 1, f);
    float mx, mn = 0.0f, s, zero = 0.0f;
    if (SYM) {
        mx = __builtin_fabsf(f[0]);
#pragma unroll
        for (int i = 1; i < 8; i++) mx = __builtin_fmaxf(mx, __builtin_fabsf(f[i]));
        mx = mx != mx ? 0.0f : mx;             // eight NaNs in one lane: fmaxf over the group skips them
        mx = u2f(seg_max<LANES>(f2u(mx)));     // non-negative floats order like their bit patterns
        s = __builtin_fmaxf(mx * kSymCons, 1e-5f);
    } else {
        mx = mn = f[0];
#pragma unroll
        for (int i = 1; i < 8; i++) { mx = __builtin_fmaxf(mx, f[i]); mn = __builtin_fminf(mn, f[i]); }
        mx = mx != mx ? -__builtin_inff() : mx;     // eight NaNs in one lane: the group reduction skips them
        mn = mn != mn ? __builtin_inff() : mn;
        mx = order_unkey(seg_max<LANES>(order_key(mx)));
        mn = order_unkey(~seg_max<LANES>(~order_key(mn)));
        s = __builtin_fmaxf((mx - mn) * kAsymCons, 1e-5f);
        // max(-0, +0) is +0 in the reference's device code: adding +0 makes that explicit
        zero = __builtin_fminf(__builtin_fmaxf(-__builtin_rintf(mn / s), 0.0f), 15.0f) + 0.0f;
    }
    const float y = 1.0f / s;
    const float top = SYM ? mx : __builtin_fmaxf(__builtin_fabsf(mx), __builtin_fabsf(mn));
    if (DT != MQ_F32 && shared_div_ok(s) && top * y < 1e30f) {
#pragma unroll
        for (int i = 0; i < 8; i++) q[i] = __builtin_rintf(div_by_shared(f[i], s, y));
    } else {
#pragma unroll
        for (int i = 0; i < 8; i++) q[i] = __builtin_rintf(f[i] / s);
    }
    if (!SYM) {
#pragma unroll
        for (int i = 0; i < 8; i++) q[i] = q[i] + zero;
    }
    if (!live) return;
    fq_store8<DT>(out, unit, q);
    if ((threadIdx.x & (LANES - 1)) == 0) {
        store_dtype(scale_out, unit / LANES, s, DT);
        if (!SYM) store_dtype(zero_out, unit / LANES, zero, DT);
    }
}

// ---- unpack + dequantize (symmetric codes) ------------------------------------------------------
// Inverse of the symmetric pack: tools/convert_kimi_int4_to_bf16.py:57-86 unpacks nibble i of word j into
// element 8j+i, subtracts the offset 8 (compressed-tensors' unpack_from_int32), multiplies by the group's scale
// in fp32 and rounds to bf16.  The product of a 4-bit integer and a bf16/fp16 scale is exact in fp32, so the only
// rounding is the final one.
#ifndef MQ_I4_UNPACK_UNROLL
#define MQ_I4_UNPACK_UNROLL 2
#endif
constexpr int kI4UnpackUnroll = MQ_I4_UNPACK_UNROLL;   // words per lane, 256 lanes apart so every load and store instruction stays contiguous
// One tensor of a launch's table per blockIdx.y: w = packed words, q = bf16 output, s = scales, units = words,
// section = log2(words per group).
template <int SDT>
__global__ __launch_bounds__(256) void int4_unpack_kernel(const FlatTable tab) {
    const FlatJob job = flat_job(tab);
    const uint32_t* __restrict__ packed = (const uint32_t*)job.w;
    const void* __restrict__ scale = job.s;
    uint16_t* __restrict__ y = (uint16_t*)job.q;
    const int64_t words = job.units;
    const int group_shift = job.section;
    const int64_t first = flat_block(tab) * (256 * kI4UnpackUnroll);
    if (first >= words) return;          // a smaller tensor of the group
    // everything a lane adds to the workgroup's (uniform) base addresses is a 32-bit offset; `first` is a multiple of
    // the words of a group (at most 256 per unit of a lane, see mq_int4_unpack_fast_ok)
    const int64_t left = words - first;
    const uint32_t rem = left < 256 * kI4UnpackUnroll ? (uint32_t)left : (uint32_t)(256 * kI4UnpackUnroll);
    const uint32_t* __restrict__ packed0 = packed + first;
    uint16_t* __restrict__ y0 = y + first * 8;
    const int64_t group0 = first >> group_shift;
    uint32_t word[kI4UnpackUnroll], sraw[kI4UnpackUnroll];
    // every load is issued before the first use: lanes past the end re-read the workgroup's first word instead of branching
#pragma unroll
    for (int u = 0; u < kI4UnpackUnroll; u++) {
        const uint32_t off = threadIdx.x + u * 256u;
        const uint32_t i = off < rem ? off : 0u;
        word[u] = __builtin_nontemporal_load(packed0 + i);
        if (SDT == MQ_F32) sraw[u] = ((const uint32_t*)scale + group0)[i >> group_shift];
        else sraw[u] = ((const uint16_t*)scale + group0)[i >> group_shift];
    }
    // (the scheduler otherwise moves the first word's unpacking, and with it the wait for that word, above the second
    // word's loads)
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int u = 0; u < kI4UnpackUnroll; u++) {
        const uint32_t off = threadIdx.x + u * 256u;
        const float sc = SDT == MQ_F32 ? u2f(sraw[u]) : SDT == MQ_BF16 ? u2f(sraw[u] << 16)
                                                                       : (float)__builtin_bit_cast(_Float16, (uint16_t)sraw[u]);
        // even nibbles and odd nibbles as bytes: one byte-to-float conversion each.  (n - 8) * scale as
        // fma(n, scale, -8 * scale): 8 * scale is exact and the FMA rounds the exact n * scale - 8 * scale once, which
        // is the rounding of the product (itself exact for a bf16 or fp16 scale).
        const uint32_t ev = word[u] & 0x0F0F0F0Fu, od = (word[u] >> 4) & 0x0F0F0F0Fu;
        const float minus8 = -8.0f * sc;
        float f[8];
#pragma unroll
        for (int k = 0; k < 4; k++) {
            f[2 * k] = __builtin_fmaf((float)((ev >> (8 * k)) & 0xFFu), sc, minus8);
            f[2 * k + 1] = __builtin_fmaf((float)((od >> (8 * k)) & 0xFFu), sc, minus8);
        }
        u32x4 o = {hw_bf16x2(f[0], f[1]), hw_bf16x2(f[2], f[3]), hw_bf16x2(f[4], f[5]), hw_bf16x2(f[6], f[7])};
        // A NaN or infinite scale (decided for the wavefront): the products may be NaN -- the scale's own, or 0 x inf --
        // and the reference's rounding to bf16 writes the one quiet NaN 0x7FC0 whatever the sign and the payload.  A
        // scale of 2^124 and more, whose eightfold is no longer finite, takes the same path, with the product as written,
        // and so does a zero or negative one (the FMA's zeros are all +0; the product's carry the sign of n - 8 and of
        // the scale).  One unsigned comparison covers them all.
        if (__builtin_amdgcn_ballot_w64(f2u(sc) - 1u >= 0x7D800000u - 1u) != 0) {
            uint32_t h[8];
#pragma unroll
            for (int k = 0; k < 4; k++) {
                f[2 * k] = ((float)((ev >> (8 * k)) & 0xFFu) - 8.0f) * sc;
                f[2 * k + 1] = ((float)((od >> (8 * k)) & 0xFFu) - 8.0f) * sc;
            }
#pragma unroll
            for (int k = 0; k < 8; k++) h[k] = f[k] != f[k] ? 0x7FC0u : hw_bf16x2(f[k], 0.0f) & 0xFFFFu;
            o = u32x4{h[0] | (h[1] << 16), h[2] | (h[3] << 16), h[4] | (h[5] << 16), h[6] | (h[7] << 16)};
        }
        if (off < rem) st16(y0 + off * 8u, o);
    }
}
// any K (rows padded to whole words), any group size, any scale dtype: one lane per element
__global__ __launch_bounds__(256) void int4_unpack_generic_kernel(const uint32_t* __restrict__ packed,
                                                                  const void* __restrict__ scale, int sdt,
                                                                  uint16_t* __restrict__ y, int64_t M, int64_t K,
                                                                  int G) {
    const int64_t wpr = (K + 7) / 8, gpr = K / G, total = M * K;
    const int64_t stride = (int64_t)gridDim.x * blockDim.x;
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += stride) {
        const int64_t r = i / K, c = i - r * K;
        const uint32_t word = packed[r * wpr + c / 8];
        const float v = (float)((int)((word >> (4 * (c & 7))) & 0xFu) - 8) * load_f32(scale, r * gpr + c / G, sdt);
        y[i] = (uint16_t)f32_to_bf16_bits(v);
    }
}

}  // namespace mq

using namespace mq;

template <int DT, int LANES>
static void launch_fake_rows_sym(const void* x, void* out, void* scale, void* zero, int64_t units, bool sym, int chunk,
                                 unsigned blocks, hipStream_t st) {
    if (sym) hipLaunchKernelGGL((int4_fake_rows_kernel<DT, LANES, true>), dim3(blocks), dim3(kI4Threads), 0, st, x, out, scale, zero, units, chunk);
    else hipLaunchKernelGGL((int4_fake_rows_kernel<DT, LANES, false>), dim3(blocks), dim3(kI4Threads), 0, st, x, out, scale, zero, units, chunk);
}
template <int DT>
static void launch_fake_rows_dt(const void* x, void* out, void* scale, void* zero, int64_t units, int lanes, bool sym,
                                int chunk, unsigned blocks, hipStream_t st) {
    if (lanes == 16) launch_fake_rows_sym<DT, 16>(x, out, scale, zero, units, sym, chunk, blocks, st);
    else if (lanes == 8) launch_fake_rows_sym<DT, 8>(x, out, scale, zero, units, sym, chunk, blocks, st);
    else launch_fake_rows_sym<DT, 4>(x, out, scale, zero, units, sym, chunk, blocks, st);
}
static void launch_fake_rows(const void* x, int dtype, void* out, void* scale, void* zero, int64_t units, int lanes,
                             bool sym, int chunk, unsigned blocks, hipStream_t st) {
    if (dtype == MQ_BF16) launch_fake_rows_dt<MQ_BF16>(x, out, scale, zero, units, lanes, sym, chunk, blocks, st);
    else if (dtype == MQ_F16) launch_fake_rows_dt<MQ_F16>(x, out, scale, zero, units, lanes, sym, chunk, blocks, st);
    else launch_fake_rows_dt<MQ_F32>(x, out, scale, zero, units, lanes, sym, chunk, blocks, st);
}

extern "C" int mq_int4_fake_quant(const void* x, int dtype, void* out, void* scale, void* zero, int64_t M, int64_t N,
                                  int block_m, int block_n, int sym, void* stream) {
    if ((!x || !out || !scale || (!sym && !zero)) && M != 0 && N != 0) return mq_fail(MQ_ERR_ARG, "null pointer");
    if (dtype < MQ_BF16 || dtype > MQ_F32 || M < 0 || N < 0 || block_m <= 0 || block_n <= 0) return mq_fail(MQ_ERR_ARG, "bad argument");
    if (((int64_t)block_m * block_n) % 32 != 0 || (int64_t)block_m * block_n > (1 << 24))
        return mq_fail(MQ_ERR_ARG, "block_m * block_n must be divisible by 32");
    if (M == 0 || N == 0) return MQ_OK;
    const bool rows_fast = block_m == 1 && (block_n == 32 || block_n == 64 || block_n == 128) &&
                           N % block_n == 0 && ((((uintptr_t)x | (uintptr_t)out)) & 15) == 0 && M * (N / 8) < (1ll << 38);
    if (rows_fast) {
        const int64_t units = M * (N / 8);
        int64_t blocks = (units + kI4Threads - 1) / kI4Threads;
        const int chunk = (int)flat_chunk(blocks);
        blocks = flat_padded(blocks, chunk);
        launch_fake_rows(x, dtype, out, scale, zero, units, block_n / 8, sym != 0, chunk, (unsigned)blocks, (hipStream_t)stream);
        return mq_check_launch("int4 fake quant");
    }
    const int64_t gpr = (N + block_n - 1) / block_n;
    const int64_t waves = ((M + block_m - 1) / block_m) * gpr;
    int64_t blocks = (waves + 3) / 4;
    if (blocks > mq_grid_cap()) blocks = mq_grid_cap();
    hipLaunchKernelGGL(int4_fake_generic_kernel, dim3((unsigned)blocks), dim3(256), 0, (hipStream_t)stream, x, dtype,
                       out, scale, zero, M, N, block_m, block_n, gpr, waves, sym);
    return mq_check_launch("int4 fake quant");
}

bool mq_int4_pack_fast_ok(const void* w, int dtype, int group) {
    return (dtype == MQ_BF16 || dtype == MQ_F16) && ((uintptr_t)w % 16) == 0 && (group == 128 || group == 64 || group == 32);
}

template <class Table>
static void int4_pack_launch(int dtype, int group, dim3 grid, hipStream_t st, const Table& tab) {
    const dim3 blk(kI4Threads);
    if (dtype == MQ_F16) {
        if (group == 128) hipLaunchKernelGGL((int4_pack_bf16_kernel<16, Table, 1>), grid, blk, 0, st, tab);
        else if (group == 64) hipLaunchKernelGGL((int4_pack_bf16_kernel<8, Table, 1>), grid, blk, 0, st, tab);
        else hipLaunchKernelGGL((int4_pack_bf16_kernel<4, Table, 1>), grid, blk, 0, st, tab);
    } else {
        if (group == 128) hipLaunchKernelGGL((int4_pack_bf16_kernel<16, Table, 0>), grid, blk, 0, st, tab);
        else if (group == 64) hipLaunchKernelGGL((int4_pack_bf16_kernel<8, Table, 0>), grid, blk, 0, st, tab);
        else hipLaunchKernelGGL((int4_pack_bf16_kernel<4, Table, 0>), grid, blk, 0, st, tab);
    }
}

// every tensor of a launch has the one 16-bit dtype
int mq_int4_pack_launch_group(int dtype, FlatTable& tab, int group, hipStream_t st) {
    if (!flat_grid(tab, kI4Threads * kI4Unroll)) return mq_fail(MQ_ERR_ARG, "tensor too large");
    if (tab.max_blocks == 0) return MQ_OK;
    int4_pack_launch(dtype, group, dim3((unsigned)tab.max_blocks, (unsigned)tab.n), st, tab);
    return mq_check_launch("int4 pack");
}

int mq_int4_pack_launch_table(int dtype, const FlatJob* device_jobs, int n, int64_t max_units, int group, hipStream_t st) {
    FlatRef ref{device_jobs, 0, 0};
    if (!flat_grid(ref, max_units, kI4Threads * kI4Unroll)) return mq_fail(MQ_ERR_ARG, "tensor too large");
    if (ref.max_blocks == 0 || n == 0) return MQ_OK;
    int4_pack_launch(dtype, group, dim3((unsigned)ref.max_blocks, (unsigned)n), st, ref);
    return mq_check_launch("int4 pack");
}

extern "C" int mq_int4_group_quant_pack(const void* w, int dtype, int32_t* packed, void* scale, int64_t M, int64_t K,
                                        int group, void* stream) {
    if ((!w || !packed || !scale) && M != 0 && K != 0) return mq_fail(MQ_ERR_ARG, "null pointer");
    if (dtype < MQ_BF16 || dtype > MQ_F32 || M < 0 || K < 0 || group <= 0) return mq_fail(MQ_ERR_ARG, "bad argument");
    if (K % group != 0 || K % 8 != 0) return mq_fail(MQ_ERR_ARG, "K must be a multiple of the group size and of 8");
    if (M == 0 || K == 0) return MQ_OK;
    hipStream_t st = (hipStream_t)stream;
    const int64_t units = M * (K / 8);
    if (mq_int4_pack_fast_ok(w, dtype, group)) {
        FlatTable tab{};
        tab.n = 1;
        tab.job[0] = FlatJob{w, packed, scale, nullptr, units, nullptr, 0, 0};
        return mq_int4_pack_launch_group(dtype, tab, group, st);
    }
    int64_t blocks = (units + 255) / 256;
    if (blocks > mq_grid_cap()) blocks = mq_grid_cap();
    hipLaunchKernelGGL(int4_pack_generic_kernel, dim3((unsigned)blocks), dim3(256), 0, st, w, dtype, (uint32_t*)packed,
                       scale, M, K, group);
    return mq_check_launch("int4 pack");
}

bool mq_int4_pack_asym_fast_ok(const void* w, int dtype, int group, int64_t M) {
    return (dtype == MQ_BF16 || dtype == MQ_F16) && ((uintptr_t)w % 16) == 0 && (group == 128 || group == 64 || group == 32) && M % 8 == 0;
}

// tiles of the zero-point packer for a [rows, cols] tensor with groups of `group` elements
int64_t mq_int4_zero_tiles(int64_t rows, int64_t cols, int group) { return int4_zero_tiles(rows / 8, cols / group); }

// The two launches of an asymmetric pack for a group of tensors: codes + scales + zero points, then the zero points
// packed eight rows to a word.  max_tiles: the most tiles the second launch has to cover in one tensor.
template <class Table>
static int int4_pack_asym_launch(int dtype, const Table& tab, int n, int64_t max_tiles, int group, hipStream_t st) {
    const dim3 grid((unsigned)tab.max_blocks, (unsigned)n), blk(kI4Threads);
    if (dtype == MQ_F16) {
        if (group == 128) hipLaunchKernelGGL((int4_pack_asym_bf16_kernel<16, Table, 1>), grid, blk, 0, st, tab);
        else if (group == 64) hipLaunchKernelGGL((int4_pack_asym_bf16_kernel<8, Table, 1>), grid, blk, 0, st, tab);
        else hipLaunchKernelGGL((int4_pack_asym_bf16_kernel<4, Table, 1>), grid, blk, 0, st, tab);
    } else {
        if (group == 128) hipLaunchKernelGGL((int4_pack_asym_bf16_kernel<16, Table, 0>), grid, blk, 0, st, tab);
        else if (group == 64) hipLaunchKernelGGL((int4_pack_asym_bf16_kernel<8, Table, 0>), grid, blk, 0, st, tab);
        else hipLaunchKernelGGL((int4_pack_asym_bf16_kernel<4, Table, 0>), grid, blk, 0, st, tab);
    }
    int rc = mq_check_launch("int4 asymmetric pack");
    if (rc != MQ_OK) return rc;
    hipLaunchKernelGGL(int4_zero_pack_group_kernel<Table>, dim3((unsigned)max_tiles, (unsigned)n), dim3(256), 0, st, tab, group / 8);
    return mq_check_launch("int4 zero-point pack");
}
int mq_int4_pack_asym_launch_group(int dtype, FlatTable& tab, int group, hipStream_t st) {
    if (!flat_grid(tab, kI4Threads * kI4Unroll)) return mq_fail(MQ_ERR_ARG, "tensor too large");
    if (tab.max_blocks == 0) return MQ_OK;
    int64_t max_tiles = 1;
    for (int i = 0; i < tab.n; i++) {
        const int64_t gpr = tab.job[i].section;
        if (gpr <= 0) continue;
        const int64_t tiles = int4_zero_tiles(tab.job[i].units / (group / 8) / gpr / 8, gpr);
        max_tiles = tiles > max_tiles ? tiles : max_tiles;
    }
    if (max_tiles >= 0x7FFFFFFF) return mq_fail(MQ_ERR_ARG, "tensor too large");
    return int4_pack_asym_launch(dtype, tab, tab.n, max_tiles, group, st);
}
// max_units: the largest tensor's 16-byte units; max_zero_tiles: the largest mq_int4_zero_tiles of the tensors
int mq_int4_pack_asym_launch_table(int dtype, const FlatJob* device_jobs, int n, int64_t max_units, int64_t max_zero_tiles,
                                   int group, hipStream_t st) {
    FlatRef ref{device_jobs, 0, 0};
    if (!flat_grid(ref, max_units, kI4Threads * kI4Unroll) || max_zero_tiles >= 0x7FFFFFFF) return mq_fail(MQ_ERR_ARG, "tensor too large");
    if (ref.max_blocks == 0 || n == 0) return MQ_OK;
    return int4_pack_asym_launch(dtype, ref, n, max_zero_tiles < 1 ? 1 : max_zero_tiles, group, st);
}

extern "C" int mq_int4_group_quant_pack_asym(const void* w, int dtype, int32_t* packed, void* scale, uint8_t* zero,
                                             int32_t* packed_zp, int64_t M, int64_t K, int group, void* stream) {
    if ((!w || !packed || !scale || !zero || !packed_zp) && M != 0 && K != 0) return mq_fail(MQ_ERR_ARG, "null pointer");
    if (dtype < MQ_BF16 || dtype > MQ_F32 || M < 0 || K < 0 || group <= 0) return mq_fail(MQ_ERR_ARG, "bad argument");
    if (K % group != 0 || group % 8 != 0) return mq_fail(MQ_ERR_ARG, "K must be a multiple of the group size and the group size of 8");
    if (M % 8 != 0) return mq_fail(MQ_ERR_ARG, "asymmetric packing needs a multiple of 8 rows");
    const bool aligned = ((uintptr_t)w % 16) == 0;
    if (M == 0 || K == 0) return MQ_OK;
    hipStream_t st = (hipStream_t)stream;
    const int64_t gpr = K / group, groups = M * gpr;
    int64_t blocks = (groups + 15) / 16;
    if (blocks > mq_grid_cap() * 4) blocks = mq_grid_cap() * 4;
    const int wpg = group / 8;
    if (mq_int4_pack_asym_fast_ok(w, dtype, group, M)) {
        FlatTable tab{};
        tab.n = 1;
        tab.job[0] = FlatJob{w, packed, scale, zero, M * (K / 8), packed_zp, (int32_t)gpr, 0};
        return mq_int4_pack_asym_launch_group(dtype, tab, group, st);
    } else if (dtype == MQ_BF16)
        hipLaunchKernelGGL(int4_pack_asym_kernel<MQ_BF16>, dim3((unsigned)blocks), dim3(256), 0, st, w, (uint32_t*)packed, scale, zero, groups, wpg, aligned);
    else if (dtype == MQ_F16)
        hipLaunchKernelGGL(int4_pack_asym_kernel<MQ_F16>, dim3((unsigned)blocks), dim3(256), 0, st, w, (uint32_t*)packed, scale, zero, groups, wpg, aligned);
    else
        hipLaunchKernelGGL(int4_pack_asym_kernel<MQ_F32>, dim3((unsigned)blocks), dim3(256), 0, st, w, (uint32_t*)packed, scale, zero, groups, wpg, aligned);
    int rc = mq_check_launch("int4 asymmetric pack");
    if (rc != MQ_OK) return rc;
    const int64_t zblocks = int4_zero_tiles(M / 8, gpr);
    if (zblocks >= 0x7FFFFFFF) return mq_fail(MQ_ERR_ARG, "tensor too large");
    hipLaunchKernelGGL(int4_zero_pack_kernel, dim3((unsigned)zblocks), dim3(256), 0, st, zero, (uint32_t*)packed_zp, M, gpr);
    return mq_check_launch("int4 zero-point pack");
}

// the flat kernel takes whole words and groups of a power-of-two number of words
bool mq_int4_unpack_fast_ok(const void* packed, const void* y, int64_t K, int group) {
    const int upg = group / 8;
    return group > 0 && group <= 2048 * kI4UnpackUnroll && K % 8 == 0 && group % 8 == 0 && (upg & (upg - 1)) == 0 &&
           ((uintptr_t)packed % 4) == 0 && ((uintptr_t)y % 16) == 0;
}
FlatJob mq_int4_unpack_entry(const void* packed, const void* scale, void* y, int64_t M, int64_t K, int group) {
    int shift = 0;
    while ((1 << shift) < group / 8) shift++;
    return FlatJob{packed, y, (void*)scale, nullptr, M * (K / 8), nullptr, shift, 0};
}
// up to kMaxGroup tensors with scales of one dtype in one launch
int mq_int4_unpack_launch_group(int scale_dtype, FlatTable& tab, hipStream_t st) {
    if (!flat_grid(tab, 256 * kI4UnpackUnroll)) return mq_fail(MQ_ERR_ARG, "tensor too large");
    if (tab.max_blocks == 0) return MQ_OK;
    const dim3 grid((unsigned)tab.max_blocks, (unsigned)tab.n), blk(256);
    if (scale_dtype == MQ_BF16) hipLaunchKernelGGL(int4_unpack_kernel<MQ_BF16>, grid, blk, 0, st, tab);
    else if (scale_dtype == MQ_F16) hipLaunchKernelGGL(int4_unpack_kernel<MQ_F16>, grid, blk, 0, st, tab);
    else hipLaunchKernelGGL(int4_unpack_kernel<MQ_F32>, grid, blk, 0, st, tab);
    return mq_check_launch("int4 unpack");
}

extern "C" int mq_int4_unpack_dequant(const int32_t* packed, const void* scale, int scale_dtype, void* y, int64_t M,
                                      int64_t K, int group, void* stream) {
    if ((!packed || !scale || !y) && M != 0 && K != 0) return mq_fail(MQ_ERR_ARG, "null pointer");
    if (scale_dtype < MQ_BF16 || scale_dtype > MQ_F32 || M < 0 || K < 0 || group <= 0) return mq_fail(MQ_ERR_ARG, "bad argument");
    if (K % group != 0) return mq_fail(MQ_ERR_ARG, "K must be a multiple of the group size");
    if (M == 0 || K == 0) return MQ_OK;
    hipStream_t st = (hipStream_t)stream;
    if (mq_int4_unpack_fast_ok(packed, y, K, group)) {
        FlatTable tab{};
        tab.n = 1;
        tab.job[0] = mq_int4_unpack_entry(packed, scale, y, M, K, group);
        return mq_int4_unpack_launch_group(scale_dtype, tab, st);
    }
    int64_t blocks = (M * K + 255) / 256;
    if (blocks > mq_grid_cap()) blocks = mq_grid_cap();
    hipLaunchKernelGGL(int4_unpack_generic_kernel, dim3((unsigned)blocks), dim3(256), 0, st, (const uint32_t*)packed, scale,
                       scale_dtype, (uint16_t*)y, M, K, group);
    return mq_check_launch("int4 unpack");
}
