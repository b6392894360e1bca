// NVFP4 (e2m1 codes, one e4m3 scale per 1x16 block, one fp32 scale per tensor) for gfx950.
// Reference: miles/utils/nvfp4.py:19-114 (layout, global scale); block arithmetic as restated in
// miles/kernels/quant/nvfp4_qdq.py:716-743,859-889,1079-1081:
//   S_enc = min(e4m3_max*6 / amax, FLT_MAX), 1 if amax == 0 or the quotient is 0;  S_dec = 1 / S_enc
//   per block: bmax = max|x|; s8 = sat_e4m3(bmax == 0 ? 0 : bmax * (S_enc * f32(1/6)))
//              inv = min(1 / (f32(s8) * S_dec), FLT_MAX);  code = sat_e2m1(x * inv)
//   published global scale: 1 / min(e4m3_max*6/amax, FLT_MAX) with only the ==0 repair (nvfp4.py:19-39)
//
// Pass 1 (mq_nvfp4_amax): 256 workgroups per tensor stream its elements and each writes one partial maximum
// into the tensor's section of the amax record: plain stores, no atomics (thousands of agent-scope atomics
// on one address serialise at ~8 ns each on this multi-XCD part) and nothing to clear.  A one-workgroup-per-
// record fold kernel turns the partial maxima into the amax, S_enc/6, 1/S_enc and the published global scale.
// Pass 2 (mq_nvfp4_quant) reads those two factors with a scalar load; two lanes own one 16-element block
// (16 bytes each), the block amax is one DPP step, and each lane emits four bytes of codes.  A gate/up pair
// writes two sections of one record.
#include <type_traits>

#include "mq_api_internal.hpp"
#include "mq_common.hpp"
#include "mq_group.hpp"

namespace mq {

constexpr int kNvThreads = 256;
#ifndef MQ_NV_UNROLL
#define MQ_NV_UNROLL 2
#endif
constexpr int kNvUnroll = MQ_NV_UNROLL;
constexpr float kSixth = 0.16666667163372040f;  // 0x3E2AAAAB

static_assert(kSectionWords == MQ_NVFP4_SECTION_WORDS && kRecordSections == MQ_NVFP4_SECTIONS, "record layout");
#ifndef MQ_AMAX_UNROLL
#define MQ_AMAX_UNROLL 4
#endif
#ifndef MQ_AMAX_NT
#define MQ_AMAX_NT 1
#endif
constexpr int kAmaxUnroll = MQ_AMAX_UNROLL;             // 16-byte units per lane per loop trip

// grid (kSectionWords, tensors): workgroup b of a tensor strides over its 16 KiB chunks and writes word b of
// the section.  job.units counts whole 16-byte units; job.s carries the element count for the sub-unit tail.
// (descriptors of a device table are in the quantizer's form, whose tensors are whole units: no tail, and job.s is the
// block-scale pointer there)
// (16-bit inputs, bf16 or fp16: the maximum is taken on the absolute bit patterns and converted to the fp32 pattern once)
template <class Table, int F16>
__global__ __launch_bounds__(256) void nvfp4_amax_bf16_kernel(const Table tab) {
    __shared__ uint32_t wave_amax[4];
    const FlatJob job = flat_job(tab);       // a copy in registers: a descriptor in device memory must not be re-read after the stores
    const uint16_t* __restrict__ w = (const uint16_t*)job.w;
    uint32_t* __restrict__ section = (uint32_t*)job.aux + job.section * kSectionWords;
    const int64_t n16 = job.units, numel = std::is_same<Table, FlatRef>::value ? n16 * 8 : (int64_t)(uintptr_t)job.s;
    const int t = threadIdx.x;
    uint32_t m2 = 0;
    for (int64_t base = (int64_t)blockIdx.x * (256 * kAmaxUnroll); base < n16; base += (int64_t)kSectionWords * 256 * kAmaxUnroll) {
        u32x4 v[kAmaxUnroll];
#pragma unroll
        for (int i = 0; i < kAmaxUnroll; i++) {
            const int64_t unit = base + i * 256 + t;
            v[i] = unit < n16 ? (MQ_AMAX_NT ? ld16(w + unit * 8) : ld16_keep(w + unit * 8)) : u32x4{0u, 0u, 0u, 0u};
        }
#pragma unroll
        for (int i = 0; i < kAmaxUnroll; i++)
            m2 = max2_u16(m2, max2_u16(max2_u16(abs2(v[i].x), abs2(v[i].y)), max2_u16(abs2(v[i].z), abs2(v[i].w))));
    }
    uint32_t m = hmax_u16(m2);
    if (blockIdx.x == 0 && t == 0)
        for (int64_t i = n16 * 8; i < numel; i++) m = umax(m, (uint32_t)(w[i] & 0x7FFFu));
    m = wave_max(m);
    if ((t & 63) == 0) wave_amax[t >> 6] = m;
    __syncthreads();
    if (t == 0) section[blockIdx.x] = f2u(elem_lo<F16>(umax(umax(wave_amax[0], wave_amax[1]), umax(wave_amax[2], wave_amax[3]))));
}

__global__ __launch_bounds__(256) void nvfp4_amax_generic_kernel(const void* __restrict__ w, int dtype, int64_t numel,
                                                                 uint32_t* __restrict__ section) {
    __shared__ uint32_t wave_amax[4];
    const int t = threadIdx.x;
    const int64_t stride = (int64_t)gridDim.x * blockDim.x;
    uint32_t m = 0;
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + t; i < numel; i += stride)
        m = umax(m, f2u(load_f32(w, i, dtype)) & 0x7FFFFFFFu);
    m = wave_max(m);
    if ((t & 63) == 0) wave_amax[t >> 6] = m;
    __syncthreads();
    if (t == 0) section[blockIdx.x] = umax(umax(wave_amax[0], wave_amax[1]), umax(wave_amax[2], wave_amax[3]));
}

struct NvScales {
    float enc_sixth;  // S_enc * (1/6)
    float s_dec;      // 1 / S_enc
    float enc;        // S_enc
};
__device__ __forceinline__ NvScales nv_scales(float amax, float numer) {
    float enc = __builtin_fminf(numer / amax, kFltMax);
    if (amax == 0.0f || enc == 0.0f) enc = 1.0f;
    NvScales r;
    r.enc_sixth = enc * kSixth;
    r.s_dec = 1.0f / enc;
    r.enc = enc;
    return r;
}
__device__ __forceinline__ float nv_published_scale(float amax, float numer) {
    float enc = numer / amax;
    if (enc > kFltMax) enc = kFltMax;  // NaN stays NaN
    if (enc == 0.0f) enc = 1.0f;
    return 1.0f / enc;
}

// words of a record behind its sections
constexpr int kRecEncSixth = kRecAmax + 1;                     // S_enc * (1/6)
constexpr int kRecSDec = kRecAmax + 2;                         // 1 / S_enc
constexpr int kRecEnc = kRecAmax + 3;                          // S_enc

// Fold kernel, one workgroup per tensor.
// MODE 0 (single calls): fold the first job.section sections of the record and publish the scales.  Tensors that share
//   a record compute the same values and write them twice.
// MODE 1 / 2 (the job driver): job.section is the tensor's place inside its record and job.pad the number of tensors
//   sharing it; they sit next to each other in the table.  Only the workgroup of the last one works: it folds all their
//   sections, writes every one's global scale and then clears the sections, so that the next sync may collect its
//   partial maxima with atomic max (see the carried-over amax below).  MODE 2 additionally checks the amax and scales
//   the record held before against the new ones: all four words equal means the codes just written with the old values
//   are final (kRecRedo = 0); otherwise the new values are stored and kRecRedo = 1 asks for a second quantization.
//   A record whose amax moved on two syncs in a row is marked volatile (kRecVolatile): on the next carried sync the
//   single pass only collects its partial maxima (no codes are written with an amax that is likely stale again) and the
//   second pass quantizes it with the fresh amax -- the cost of the plain two-pass form, instead of two full
//   quantizations.  The mark is dropped as soon as the amax has held still for one sync (amax_record_after_carried_run).
template <int MODE, class Table>
__global__ __launch_bounds__(256) void nvfp4_fold_kernel(const Table tab, float numer, uint32_t* moved_counter, uint32_t* moved_mirror) {
    __shared__ uint32_t lds4[4];
    const int ji = blockIdx.x;
    const FlatJob& job = tab.job[ji];
    const int sections = MODE == 0 ? job.section : job.pad;
    if (MODE != 0) amax_feedback_folded(moved_counter, moved_mirror, gridDim.x);
    if (MODE != 0 && job.section != job.pad - 1) return;
    uint32_t* rec = (uint32_t*)job.aux;
    uint32_t m = 0;
    for (int i = threadIdx.x; i < sections * kSectionWords; i += 256) m = umax(m, rec[i]);
    m = wave_max(m);
    if ((threadIdx.x & 63) == 0) lds4[threadIdx.x >> 6] = m;
    __syncthreads();
    if (MODE != 0)
        for (int i = threadIdx.x; i < sections * kSectionWords; i += 256) rec[i] = 0;
    if (threadIdx.x == 0) {
        const float amax = u2f(umax(umax(lds4[0], lds4[1]), umax(lds4[2], lds4[3])));
        const NvScales gs = nv_scales(amax, numer);
        if (MODE == 2) {
            const bool moved = !(rec[kRecAmax] == f2u(amax) && rec[kRecEncSixth] == f2u(gs.enc_sixth) &&
                                 rec[kRecSDec] == f2u(gs.s_dec) && rec[kRecEnc] == f2u(gs.enc));
            amax_record_after_carried_run(rec, moved);
            amax_feedback(moved_counter, moved, (uint32_t)sections);
        } else if (MODE == 1) {
            rec[kRecRedo] = 0;
            rec[kRecVolatile] = 0;
            rec[kRecMovedRuns] = 0;
            amax_feedback(moved_counter, rec[kRecAmax] != f2u(amax), (uint32_t)sections);
        }
        rec[kRecAmax] = f2u(amax);
        rec[kRecEncSixth] = f2u(gs.enc_sixth);
        rec[kRecSDec] = f2u(gs.s_dec);
        rec[kRecEnc] = f2u(gs.enc);
        const float published = nv_published_scale(amax, numer);
        if (MODE == 0) {
            if (job.aux2) *(float*)job.aux2 = published;
        } else {
            for (int k = 0; k < sections; k++)
                if (tab.job[ji - k].aux2) *(float*)tab.job[ji - k].aux2 = published;
        }
    }
}

// ---- Four Over Six block scaling (miles/kernels/quant/nvfp4_qdq.py:893-990) --------------------------------
// Every block is quantized twice: "map to 6" with scale6 = e4m3(min(RN(RN(bmax / 6) * S_enc), 448)) and "map to 4"
// with scale4 = e4m3(min(RN(that product * 1.5), 448)); the candidate with the strictly smaller reconstruction
// error wins, ties go to map-to-6.  The error is an fp32 sum over the 16 elements in element order:
//   default   | RN(RN(RN(value * f32(scale)) * amax) / (6 * e4m3_max)) - x |   (MQ_NVFP4_ERR_MSE: its square)
//   ERR_FP16  | f32(RN_f16(f16(value) * f16(scale))) - RN(x * S_enc) |
struct NvCandidate {
    uint32_t sc;     // e4m3 byte
    uint32_t word;   // this lane's eight codes
    float s_f;       // f32(sc)
};
__device__ __forceinline__ NvCandidate nv_candidate(const float f[8], float s_hp, float s_dec) {
    NvCandidate c;
    c.sc = hw_e4m3x2<false>(__builtin_fminf(s_hp, kFp8Max), 0.0f, 0u) & 0xFFu;
    c.s_f = hw_e4m3x2_decode<false>(c.sc).x;
    // the refined hardware reciprocal where it equals the division, decided for the wavefront (see nvfp4_quant_units)
    const float d = c.s_f * s_dec;
    float inv;
    if (__builtin_amdgcn_ballot_w64(!shared_div_ok(d)) == 0) inv = recip_shared(d);
    else inv = __builtin_fminf(1.0f / d, kFltMax);
    c.word = hw_e2m1x2<0>(f[0] * inv, f[1] * inv, 0u);
    c.word = hw_e2m1x2<1>(f[2] * inv, f[3] * inv, c.word);
    c.word = hw_e2m1x2<2>(f[4] * inv, f[5] * inv, c.word);
    c.word = hw_e2m1x2<3>(f[6] * inv, f[7] * inv, c.word);
    return c;
}
__device__ __forceinline__ void nv_decode8(uint32_t word, float q[8]) {
    const f32x2 a = __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(word, 1.0f, 0), b = __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(word, 1.0f, 1);
    const f32x2 c = __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(word, 1.0f, 2), d = __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(word, 1.0f, 3);
    q[0] = a.x; q[1] = a.y; q[2] = b.x; q[3] = b.y; q[4] = c.x; q[5] = c.y; q[6] = d.x; q[7] = d.y;
}
// x / d for d = 2688 or 1536 with y = RN(1/d): q0 = RN(x*y); r = x - q0*d (exact in an FMA); q = RN(q0 + r*y) is the
// correctly rounded quotient for every fp32 mantissa of x and both divisors (exhaustive CPU check, 2^23 mantissas
// each), provided no intermediate leaves the normal range, i.e. for |x| in 2^-91 .. 2^89 (and for zero, which comes
// out as +0 whatever its sign: no error term can see that).  The numerators here are RN(RN(value * f32(scale)) * amax)
// with value * f32(scale) either zero or in 2^-10 .. 2688, so one test of the tensor amax covers every element:
// nv_fast_division(amax) allows the sequence for the whole tensor, otherwise every quotient is the IEEE division.
// 0: IEEE divisions; 1: the sequence; 2: the sequence, and the amax has at most 12 significant bits (the amax of a bf16 or
// fp16 tensor has), so that value x f32(scale) x amax -- 2, 4 and 12 bits -- is exact in whatever order it is taken
__device__ __forceinline__ int nv_fast_division(float amax) {
    const uint32_t e = f2u(amax) & 0x7F800000u;
    if (!(e >= 0x17800000u /* 2^-80 */ && e <= 0x65800000u /* 2^76 */)) return 0;
    return (f2u(amax) & 0xFFFu) == 0 ? 2 : 1;
}
template <int FASTDIV>
__device__ __forceinline__ float div_by_numer(float x, float d, float y) {
    if (!FASTDIV) return x / d;
    const float q0 = x * y;
    const float r = __builtin_fmaf(-q0, d, x);
    return __builtin_fmaf(r, y, q0);
}
// error terms of this lane's eight elements; EM bit 0: squared error, bit 1: fp16 candidate error
template <int EM, int FASTDIV>
__device__ __forceinline__ void nv_error_terms(const float f[8], const NvCandidate& c, float amax, float enc, float denom, float denom_inv,
                                               float term[8]) {
    float q[8];
    nv_decode8(c.word, q);
    // FASTDIV 2: every partial product of value x f32(scale) x amax is exact, one multiplication per element
    const float scale_amax = c.s_f * amax;
#pragma unroll
    for (int j = 0; j < 8; j++) {
        float diff;
        if (EM & 2) {
            _Float16 h = (_Float16)q[j] * (_Float16)c.s_f;        // both factors exact in fp16; one fp16 rounding
            float hf = (float)h;
            asm volatile("" : "+v"(hf));                          // keep the fp16 product a value of its own
            diff = hf - f[j] * enc;
        } else {
            diff = div_by_numer<FASTDIV>(FASTDIV == 2 ? q[j] * scale_amax : (q[j] * c.s_f) * amax, denom, denom_inv) - f[j];
        }
        term[j] = (EM & 1) ? diff * diff : __builtin_fabsf(diff);
    }
}
// Sum of the block's sixteen terms in element order.  The even lane of the pair holds elements 0..7: its partial
// sum from zero seeds the odd lane's accumulation, and the odd lane's total goes back to the even lane.
__device__ __forceinline__ float nv_pair_error(const float term[8], bool odd_lane) {
    float from_zero = 0.0f;
#pragma unroll
    for (int j = 0; j < 8; j++) from_zero = from_zero + term[j];
    float seeded = u2f(dpp_u32<kDppQuadXor1>(f2u(from_zero)));
#pragma unroll
    for (int j = 0; j < 8; j++) seeded = seeded + term[j];
    const float partner_total = u2f(dpp_u32<kDppQuadXor1>(f2u(seeded)));
    return odd_lane ? seeded : partner_total;
}
// the winning candidate for this lane's block; bmax is the block amax (pair-uniform)
template <int EM, int FASTDIV>
__device__ __forceinline__ NvCandidate nv_four_over_six(const float f[8], float bmax, float amax, const NvScales& gs,
                                                        float denom, bool odd_lane) {
    // bmax / 6: a bf16 numerator and a shared divisor, so the three-instruction sequence gives the IEEE quotient
    // wherever its intermediates stay normal (decided for the wavefront; zero blocks and extreme maxima divide)
    const bool plain_bmax = shared_div_ok(bmax);
    const float s6_hp = (__builtin_amdgcn_ballot_w64(!plain_bmax) == 0 ? div_by_shared(bmax, 6.0f, 0x1.555556p-3f) : bmax / 6.0f) * gs.enc;
    const float s4_hp = s6_hp * 1.5f;
    const NvCandidate c4 = nv_candidate(f, s4_hp, gs.s_dec), c6 = nv_candidate(f, s6_hp, gs.s_dec);
    float t4[8], t6[8];
    const float denom_inv = 1.0f / denom;
    nv_error_terms<EM, FASTDIV>(f, c4, amax, gs.enc, denom, denom_inv, t4);
    nv_error_terms<EM, FASTDIV>(f, c6, amax, gs.enc, denom, denom_inv, t6);
    const float e4 = nv_pair_error(t4, odd_lane), e6 = nv_pair_error(t6, odd_lane);
    return e4 < e6 ? c4 : c6;
}
// ---- the same with one lane per block (the quantizer's form) ------------------------------------------------
// With two lanes per block every block-level step (the two candidate scales, their reciprocals, the comparison) is
// done twice, and the error sum, which has to run through the sixteen terms in element order, takes sixteen additions
// in each lane of the pair.  The quantizer therefore regroups its data first: a lane ends up with the thirty-two
// bytes of one whole block, and this kernel is bound by vector instructions, not by memory.
struct NvCandidate16 {
    uint32_t sc;        // e4m3 byte
    uint32_t lo, hi;    // codes of elements 0..7 and 8..15
    float a;            // RN(f32(sc) * amax / denom): what one unit of the code grid is worth (tensors that take the estimate)
};
// A candidate's block scale is one of 128 bytes, and what the quantizer needs of it -- the reciprocal
// min(1 / (f32(byte) * S_dec), FLT_MAX) and, for the error estimate, RN(f32(byte) * amax / denom) -- depends on the byte
// and the tensor only.  A workgroup therefore computes both for every byte once (128 lanes, one IEEE division each,
// while its loads are in flight) into LDS, and a candidate is one 8-byte LDS read instead of a decode, a multiplication,
// a range test, a refined reciprocal and a three-instruction division per block and candidate.
struct NvScaleEntry {
    float inv, a;
};
__device__ __forceinline__ void nv_fill_scale_table(NvScaleEntry* table, int t, float amax, float s_dec, bool estimate,
                                                    float denom, float denom_inv) {
    if (t < 128) {
        const float s_f = hw_e4m3x2_decode<false>((uint32_t)t).x;
        NvScaleEntry e;
        e.inv = __builtin_fminf(1.0f / (s_f * s_dec), kFltMax);
        // (only read where f32(byte) * amax is exact and the sequence gives its correctly rounded quotient)
        e.a = estimate ? div_by_numer<2>(s_f * amax, denom, denom_inv) : 0.0f;
        table[t] = e;
    }
}
__device__ __forceinline__ NvCandidate16 nv_candidate16(const float f[16], float s_hp, const NvScaleEntry* table) {
    NvCandidate16 c;
    c.sc = hw_e4m3x2<false>(__builtin_fminf(s_hp, kFp8Max), 0.0f, 0u) & 0xFFu;
    const NvScaleEntry e = table[c.sc & 0x7Fu];      // s_hp is not negative: the byte has no sign bit
    const float inv = e.inv;
    c.a = e.a;
    c.lo = hw_e2m1x2<0>(f[0] * inv, f[1] * inv, 0u);
    c.lo = hw_e2m1x2<1>(f[2] * inv, f[3] * inv, c.lo);
    c.lo = hw_e2m1x2<2>(f[4] * inv, f[5] * inv, c.lo);
    c.lo = hw_e2m1x2<3>(f[6] * inv, f[7] * inv, c.lo);
    c.hi = hw_e2m1x2<0>(f[8] * inv, f[9] * inv, 0u);
    c.hi = hw_e2m1x2<1>(f[10] * inv, f[11] * inv, c.hi);
    c.hi = hw_e2m1x2<2>(f[12] * inv, f[13] * inv, c.hi);
    c.hi = hw_e2m1x2<3>(f[14] * inv, f[15] * inv, c.hi);
    return c;
}
template <int EM, int FASTDIV>
__device__ __forceinline__ float nv_block_error(const float f[16], const NvCandidate16& c, float amax, float enc, float denom,
                                                float denom_inv) {
    float term[8], error = 0.0f;
    NvCandidate half{c.sc, c.lo, hw_e4m3x2_decode<false>(c.sc).x};
    nv_error_terms<EM, FASTDIV>(f, half, amax, enc, denom, denom_inv, term);
#pragma unroll
    for (int j = 0; j < 8; j++) error = error + term[j];
    half.word = c.hi;
    nv_error_terms<EM, FASTDIV>(f + 8, half, amax, enc, denom, denom_inv, term);
#pragma unroll
    for (int j = 0; j < 8; j++) error = error + term[j];
    return error;
}
// A cheaper error sum that decides almost every block.  With a = RN(f32(scale) * amax / denom), the exact term's
// dequantized value RN(q * f32(scale) * amax / denom) IS q * a for the codes that are powers of two (0.5, 1, 2, 4: scaling
// by a power of two commutes with the rounding) and differs from q * a by at most 2^-23 of its size for 1.5, 3 and 6.
// The estimate sums |q * a - x|, each term rounded once (an FMA), in element order.  Every step is within a few units in
// the last place of the exact computation, so the estimated sum S' and the exact sum S of a candidate differ by at most
//   2^-20 (31.4 a + 2 bmax) + 30.3 * 2^-24 S'
// (per element: 2.01 * 2^-24 |deq| between the two dequantized values, 2^-24 (|deq| + |x|) for each of the two roundings
// of the difference, |deq| <= 6 a (1 + 2^-22), |x| <= bmax; for the sums: recursive summation of sixteen non-negative
// terms is within 15.1 * 2^-24 of their true sum, on both sides).  Whenever the two estimates are further apart than
// the two bounds together, the exact sums compare the same way.
//
// The squared error (SQUARED) has the same estimate with each difference d' = RN(q * a - x) squared.  Per element the
// exact difference d and d' are within E = 2^-24 (24.1 a + 2 bmax) of each other (the three contributions above), so
// the squares differ by at most E (2 |d'| + E) and, rounded, by 2^-23 d'^2 more; over the block, with
// sum |d'| <= 4 sqrt(sum d'^2), the estimated and the exact sum of a candidate differ by at most
//   8.1 E sqrt(S') + 16.1 E^2 + 32.5 * 2^-24 S'.
template <bool SQUARED>
__device__ __forceinline__ float nv_block_error_estimate(const float f[16], const NvCandidate16& c, float a) {
    float q[8], sum = 0.0f;
    nv_decode8(c.lo, q);
#pragma unroll
    for (int j = 0; j < 8; j++) {
        const float d = __builtin_fmaf(q[j], a, -f[j]);
        sum = sum + (SQUARED ? d * d : __builtin_fabsf(d));
    }
    nv_decode8(c.hi, q);
#pragma unroll
    for (int j = 0; j < 8; j++) {
        const float d = __builtin_fmaf(q[j], a, -f[8 + j]);
        sum = sum + (SQUARED ? d * d : __builtin_fabsf(d));
    }
    return sum;
}
template <int EM, int FASTDIV>
__device__ __forceinline__ NvCandidate16 nv_four_over_six16(const float f[16], float bmax, float amax, const NvScales& gs,
                                                            float denom, float denom_inv, const NvScaleEntry* table) {
    const bool plain_bmax = shared_div_ok(bmax);
    const float s6_hp = (__builtin_amdgcn_ballot_w64(!plain_bmax) == 0 ? div_by_shared(bmax, 6.0f, 0x1.555556p-3f) : bmax / 6.0f) * gs.enc;
    const float s4_hp = s6_hp * 1.5f;
    const NvCandidate16 c4 = nv_candidate16(f, s4_hp, table), c6 = nv_candidate16(f, s6_hp, table);
    if ((EM == 0 || EM == 1) && FASTDIV == 2) {
        // (FASTDIV 2: f32(scale) * amax is exact and its quotient by denom comes correctly rounded from the sequence)
        const float a4 = c4.a, a6 = c6.a;
        const float g4 = nv_block_error_estimate<EM == 1>(f, c4, a4), g6 = nv_block_error_estimate<EM == 1>(f, c6, a6);
        float guard;
        if (EM == 0) {
            // twice the bound's first part and four times its second: rounding in this line cannot bring it below the bound
            guard = 0x1p-19f * (32.0f * (a4 + a6) + 4.0f * bmax + 4.0f * (g4 + g6));
        } else {
            // twice the squared error's bound for both candidates, and more (the hardware square root is within one unit
            // in the last place; the small constant keeps a denormal sum from dropping out of it and is the floor below
            // which two sums are too small to call)
            const float e4 = 0x1p-24f * (25.0f * a4 + 2.0f * bmax), e6 = 0x1p-24f * (25.0f * a6 + 2.0f * bmax);
            guard = 17.0f * (e4 * __builtin_amdgcn_sqrtf(g4 + 0x1p-100f) + e6 * __builtin_amdgcn_sqrtf(g6 + 0x1p-100f)) +
                    33.0f * (e4 * e4 + e6 * e6) + 0x1p-17f * (g4 + g6) + 0x1p-100f;
        }
        // (an all-zero block, or two candidates with one scale byte -- the block that holds the tensor's maximum, whose
        // scales both saturate: the candidates are the same, the tie goes to map-to-6, as g4 < g6 says; a NaN compares false)
        const bool decided = __builtin_fabsf(g4 - g6) > guard || bmax == 0.0f || c4.sc == c6.sc;
        if (__builtin_amdgcn_ballot_w64(!decided) == 0) return g4 < g6 ? c4 : c6;
        // a wavefront with a block too close to call (a few blocks in 10 000, most of them exact ties) takes the exact sums below
    }
    const float e4 = nv_block_error<EM, FASTDIV>(f, c4, amax, gs.enc, denom, denom_inv);
    const float e6 = nv_block_error<EM, FASTDIV>(f, c6, amax, gs.enc, denom, denom_inv);
    return e4 < e6 ? c4 : c6;
}
// error mode of a flags word, as the EM template argument
static inline int nv_error_mode(int flags) { return ((flags & MQ_NVFP4_ERR_MSE) ? 1 : 0) | ((flags & MQ_NVFP4_ERR_FP16) ? 2 : 0); }

// Four Over Six over kNvThreads * 2 units starting at `base`: loaded as the standard quantizer loads them (lane t takes
// units t and kNvThreads + t, so a wavefront's loads are contiguous), then regrouped through LDS inside each wavefront so
// that the even lane of a pair holds the block made of units 2p, 2p + 1 and the odd lane the block kNvThreads + 2p, + 1.
// Returns the largest |element| of the lane's block (bf16 bits).
#ifndef MQ_NV_FOS_ROUNDS
#define MQ_NV_FOS_ROUNDS 2
#endif
// consecutive pieces of kNvThreads * 2 units one Four Over Six workgroup takes.  Measured on 96 DeepSeek-V3 expert
// matrices, steady state: 4.74 / 4.95 / 4.83 TB/s with one / two / three pieces (78 and 86 registers with two and three:
// six and five wavefronts per SIMD instead of seven).
constexpr int kFosRounds = MQ_NV_FOS_ROUNDS;
// units a workgroup of the quantizer covers (FOS as in nvfp4_quant_units)
constexpr int64_t nv_units_per_block(int fos) { return (int64_t)kNvThreads * kNvUnroll * (fos ? kFosRounds : 1); }
template <int EM, int F16>
__device__ __forceinline__ uint32_t nvfp4_fos_units(const FlatJob& job, const int64_t base, const int t, const float denom) {
    static_assert(kNvUnroll == 2, "the regrouping pairs the two units of a lane");
    constexpr uint32_t kPiece = kNvThreads * 2;
    __shared__ u32x4 stage[kPiece];
    __shared__ NvScaleEntry scale_table[128];
    const uint16_t* __restrict__ w = (const uint16_t*)job.w;
    uint32_t* __restrict__ q = (uint32_t*)job.q;
    uint8_t* __restrict__ s8 = (uint8_t*)job.s;
    const uint32_t* __restrict__ amax_bits = (const uint32_t*)job.aux;
    const int64_t left = job.units - base;
    const uint32_t rem_all = left < kPiece * kFosRounds ? (uint32_t)left : kPiece * kFosRounds;
    const uint16_t* __restrict__ w0 = w + base * 8;
    uint32_t* __restrict__ q0 = q + base;
    uint8_t* __restrict__ s80 = s8 + base / 2;
    // every load of every piece is issued before the first is waited for: this kernel is bound by its arithmetic, some
    // two hundred vector instructions per block, and a wavefront that computes on one piece while nothing of its own is
    // in flight leaves the memory system idle.  A lane past the end reads the workgroup's first unit again (always
    // there) and drops it.
    u32x4 in[kFosRounds][2];
#pragma unroll
    for (int r = 0; r < kFosRounds; r++)
#pragma unroll
        for (int i = 0; i < 2; i++) {
            const uint32_t off = r * kPiece + (uint32_t)t + i * kNvThreads;
            in[r][i] = ld16(w0 + (off < rem_all ? off : 0u) * 8u);
        }
    NvScales gs;
    gs.enc_sixth = u2f(amax_bits[kRecEncSixth]);
    gs.s_dec = u2f(amax_bits[kRecSDec]);
    gs.enc = u2f(amax_bits[kRecEnc]);
    const float amax = u2f(amax_bits[kRecAmax]);
    const int fastdiv = nv_fast_division(amax);
    // the error's divisor 6 * e4m3_max is one of two constants and the same for the whole launch: its reciprocal is
    // picked on the scalar unit
    constexpr float kInv2688 = 1.0f / 2688.0f, kInv1536 = 1.0f / 1536.0f;
    const float denom_inv = denom == 2688.0f ? kInv2688 : denom == 1536.0f ? kInv1536 : 1.0f / denom;
    // (a workgroup that comes here again, in the striding second pass, writes the same values over the table: one tensor)
    nv_fill_scale_table(scale_table, t, amax, gs.s_dec, fastdiv == 2 && EM < 2, denom, denom_inv);
    __syncthreads();
    uint32_t seen = 0;
#pragma unroll
    for (int r = 0; r < kFosRounds; r++) {
        if (r * kPiece >= rem_all) break;      // the same for the whole workgroup
        const uint32_t rem = rem_all - r * kPiece;
#pragma unroll
        for (int i = 0; i < 2; i++) {
            const uint32_t off = (uint32_t)t + i * kNvThreads;
            stage[off] = in[r][i];      // (a unit past the end holds the workgroup's first unit: real data, nothing new to any maximum)
        }
        // A wavefront reads back only what its own lanes wrote, and the LDS serves one wavefront's accesses in the order
        // it issued them: no workgroup barrier, only the compiler is told not to move the reads above the writes.
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
        const uint32_t first = ((t & 1) ? (uint32_t)kNvThreads : 0u) + ((uint32_t)t & ~1u);      // the block's first unit
        const u32x4 lo = stage[first], hi = stage[first + 1];
        // (and the next piece's writes stay below these reads)
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        const uint32_t m2 = max2_u16(max2_u16(max2_u16(abs2(lo.x), abs2(lo.y)), max2_u16(abs2(lo.z), abs2(lo.w))),
                                     max2_u16(max2_u16(abs2(hi.x), abs2(hi.y)), max2_u16(abs2(hi.z), abs2(hi.w))));
        const uint32_t mb = hmax_u16(m2);
        seen = umax(seen, mb);
        const float bmax = elem_lo<F16>(mb);
        const float f[16] = {elem_lo<F16>(lo.x), elem_hi<F16>(lo.x), elem_lo<F16>(lo.y), elem_hi<F16>(lo.y),
                             elem_lo<F16>(lo.z), elem_hi<F16>(lo.z), elem_lo<F16>(lo.w), elem_hi<F16>(lo.w),
                             elem_lo<F16>(hi.x), elem_hi<F16>(hi.x), elem_lo<F16>(hi.y), elem_hi<F16>(hi.y),
                             elem_lo<F16>(hi.z), elem_hi<F16>(hi.z), elem_lo<F16>(hi.w), elem_hi<F16>(hi.w)};
        const NvCandidate16 c = fastdiv == 2   ? nv_four_over_six16<EM, 2>(f, bmax, amax, gs, denom, denom_inv, scale_table)
                                : fastdiv == 1 ? nv_four_over_six16<EM, 1>(f, bmax, amax, gs, denom, denom_inv, scale_table)
                                               : nv_four_over_six16<EM, 0>(f, bmax, amax, gs, denom, denom_inv, scale_table);
        if (first < rem) {      // the tensor is whole blocks: both units of a block are inside or outside
            st8(q0 + r * kPiece + first, u32x2{c.lo, c.hi});      // `first` is even and `base` a multiple of the piece
            s80[(r * kPiece + first) >> 1] = (uint8_t)c.sc;
        }
    }
    return seen;
}

// kNvThreads * kNvUnroll units starting at `base` of one tensor; returns the largest |element| this lane saw (bf16 bits)
// FOS = 0: standard quantizer; FOS = 1 + error mode: Four Over Six
template <int FOS, int F16>
__device__ __forceinline__ uint32_t nvfp4_quant_units(const FlatJob& job, const int64_t base, const int t, const float denom) {
    if (FOS) return nvfp4_fos_units<(FOS > 0 ? FOS - 1 : 0), F16>(job, base, t, denom);
    constexpr uint32_t kInfBits = F16 ? 0x7C00u : 0x7F80u;
    const uint16_t* __restrict__ w = (const uint16_t*)job.w;
    uint32_t* __restrict__ q = (uint32_t*)job.q;
    uint8_t* __restrict__ s8 = (uint8_t*)job.s;
    const uint32_t* __restrict__ amax_bits = (const uint32_t*)job.aux;
    const int64_t total_units = job.units;
    // everything a lane adds to the workgroup's (uniform) base addresses is a 32-bit offset
    const int64_t left = total_units - base;
    const uint32_t rem = left < kNvThreads * kNvUnroll ? (uint32_t)left : (uint32_t)(kNvThreads * kNvUnroll);
    const uint16_t* __restrict__ w0 = w + base * 8;
    uint32_t* __restrict__ q0 = q + base;
    uint8_t* __restrict__ s80 = s8 + base / 2;        // `base` is a multiple of the two lanes of a block
    u32x4 v[kNvUnroll];
#pragma unroll
    for (int i = 0; i < kNvUnroll; i++) {
        const uint32_t off = (uint32_t)t + i * kNvThreads;
        v[i] = off < rem ? ld16(w0 + off * 8u) : u32x4{0u, 0u, 0u, 0u};
    }
    NvScales gs;
    gs.enc_sixth = u2f(amax_bits[kRecEncSixth]);
    gs.s_dec = u2f(amax_bits[kRecSDec]);
    gs.enc = u2f(amax_bits[kRecEnc]);
    const float amax = u2f(amax_bits[kRecAmax]);
    const int fastdiv = nv_fast_division(amax);
    uint32_t seen = 0;
#pragma unroll
    for (int i = 0; i < kNvUnroll; i++) {
        const uint32_t off = (uint32_t)t + i * kNvThreads;
        const uint32_t m2 = max2_u16(max2_u16(abs2(v[i].x), abs2(v[i].y)), max2_u16(abs2(v[i].z), abs2(v[i].w)));
        const uint32_t mb = group_max2(hmax_u16(m2));
        seen = umax(seen, mb);
        const float bmax = elem_lo<F16>(mb);
        const float s_hp = bmax == 0.0f ? 0.0f : bmax * gs.enc_sixth;
        const float f[8] = {elem_lo<F16>(v[i].x), elem_hi<F16>(v[i].x), elem_lo<F16>(v[i].y), elem_hi<F16>(v[i].y),
                            elem_lo<F16>(v[i].z), elem_hi<F16>(v[i].z), elem_lo<F16>(v[i].w), elem_hi<F16>(v[i].w)};
        uint32_t sc, word;
        if (mb < kInfBits && s_hp == s_hp) {
            sc = hw_e4m3x2<false>(__builtin_fminf(s_hp, kFp8Max), 0.0f, 0u) & 0xFFu;
            const float s_f = hw_e4m3x2_decode<false>(sc).x;
            // 1 / (block scale x global decode scale): the refined hardware reciprocal where it equals the division (every
            // divisor in 2^-91 .. 2^90, far below FLT_MAX), decided for the wavefront; an all-zero block has divisor 0
            const float d = s_f * gs.s_dec;
            float inv;
            if (__builtin_amdgcn_ballot_w64(!shared_div_ok(d)) == 0) inv = recip_shared(d);
            else inv = __builtin_fminf(1.0f / d, kFltMax);
            word = hw_e2m1x2<0>(f[0] * inv, f[1] * inv, 0u);
            word = hw_e2m1x2<1>(f[2] * inv, f[3] * inv, word);
            word = hw_e2m1x2<2>(f[4] * inv, f[5] * inv, word);
            word = hw_e2m1x2<3>(f[6] * inv, f[7] * inv, word);
        } else {
            sc = sw_e4m3fn_sat(s_hp);
            const float s_f = sw_e4m3fn_decode(sc);
            const float inv = __builtin_fminf(1.0f / (s_f * gs.s_dec), kFltMax);
            word = 0;
#pragma unroll
            for (int j = 0; j < 8; j++) word |= sw_e2m1(f[j] * inv) << (4 * j);
        }
        if (off < rem) {
            st4(q0 + off, word);
            if ((t & 1) == 0) s80[off >> 1] = (uint8_t)sc;
        }
    }
    return seen;
}

// the largest |element| (bf16 bits) this lane sees in kNvThreads * kNvUnroll units starting at `base`: what the single
// pass does for a record marked volatile
__device__ __forceinline__ uint32_t nvfp4_amax_units(const FlatJob& job, const int64_t base, const int t) {
    const uint16_t* __restrict__ w = (const uint16_t*)job.w;
    uint32_t m2 = 0;
#pragma unroll
    for (int i = 0; i < kNvUnroll; i++) {
        const int64_t unit = base + i * kNvThreads + t;
        const u32x4 v = unit < job.units ? ld16(w + unit * 8) : u32x4{0u, 0u, 0u, 0u};
        m2 = max2_u16(m2, max2_u16(max2_u16(abs2(v.x), abs2(v.y)), max2_u16(abs2(v.z), abs2(v.w))));
    }
    return hmax_u16(m2);
}

// Carried-over amax.  A weight tensor's amax rarely changes from one sync to the next (the largest element has to move
// to another bf16 value), and the amax record of a replayed job list still holds the last sync's amax and scales.
// PASS 1 quantizes with those in a single read of the tensor and collects this sync's partial maxima on the way (one
// atomic max per workgroup into the tensor's section, cleared by the previous fold); the fold kernel then compares, and
// PASS 2, a small grid striding over the blocks, quantizes again only the tensors whose amax did change.
// PASS 0 is the second pass of the plain two-pass form (amax kernel, fold, quantize).
template <int FOS, int PASS, class Table, int F16>
__global__ __launch_bounds__(kNvThreads) void nvfp4_quant_bf16_kernel(const Table tab, float denom) {
    const FlatJob job = flat_job(tab);       // a copy in registers: a descriptor in device memory must not be re-read after the stores
    const int t = threadIdx.x;
    constexpr int64_t kPerBlock = nv_units_per_block(FOS);
    if (PASS == 2) {
        if (((const uint32_t*)job.aux)[kRecRedo] == 0) return;
        // an XCD takes a run of consecutive blocks in every trip of the grid, as the flat grids do (second pass 2 pct faster)
        const int64_t first = xcd_chunked_block(gridDim.x == kSectionWords ? kSectionWords / kXcds : tab.chunk);
        for (int64_t base = first * kPerBlock; base < job.units; base += (int64_t)gridDim.x * kPerBlock)
            nvfp4_quant_units<FOS, F16>(job, base, t, denom);
        return;
    }
    const int64_t base = flat_block(tab) * kPerBlock;
    if (base >= job.units) return;
    uint32_t seen;
    if (PASS == 1 && ((const uint32_t*)job.aux)[kRecVolatile] != 0) {
        seen = 0;
        for (int64_t piece = base; piece < base + kPerBlock && piece < job.units; piece += kNvThreads * kNvUnroll)
            seen = umax(seen, nvfp4_amax_units(job, piece, t));
    } else seen = nvfp4_quant_units<FOS, F16>(job, base, t, denom);
    if (PASS == 1) {
        __shared__ uint32_t wave_seen[kNvThreads / 64];
        seen = wave_max(seen);
        if ((t & 63) == 0) wave_seen[t >> 6] = seen;
        __syncthreads();
        if (t == 0) {
            uint32_t m = 0;
#pragma unroll
            for (int k = 0; k < kNvThreads / 64; k++) m = umax(m, wave_seen[k]);
            atomicMax((uint32_t*)job.aux + job.section * kSectionWords + (blockIdx.x & (kSectionWords - 1)), f2u(elem_lo<F16>(m)));
        }
    }
}

// software candidate of the one-lane-per-block kernel: codes of sixteen values and their error
__device__ __forceinline__ float nv_candidate_sw(const float x[16], uint32_t sc, float amax, const NvScales& gs, float denom,
                                                 int flags, uint32_t codes[16]) {
    const float s_f = sw_e4m3fn_decode(sc);
    const float inv = __builtin_fminf(1.0f / (s_f * gs.s_dec), kFltMax);
    float error = 0.0f;
    for (int j = 0; j < 16; j++) {
        const uint32_t c = sw_e2m1(x[j] * inv);
        codes[j] = c;
        const float mag = (c & 7u) < 2u ? 0.5f * (float)(c & 7u) : u2f(0x3F000000u + ((c & 7u) << 22));
        const float cand = (c & 8u) ? -mag : mag;
        float diff;
        if (flags & MQ_NVFP4_ERR_FP16) {
            float hf = (float)((_Float16)cand * (_Float16)s_f);
            asm volatile("" : "+v"(hf));
            diff = hf - x[j] * gs.enc;
        } else {
            diff = ((cand * s_f) * amax) / denom - x[j];
        }
        error = error + ((flags & MQ_NVFP4_ERR_MSE) ? diff * diff : __builtin_fabsf(diff));
    }
    return error;
}

__global__ __launch_bounds__(256) void nvfp4_quant_generic_kernel(const void* __restrict__ w, int dtype,
                                                                  const uint32_t* __restrict__ amax_bits,
                                                                  uint8_t* __restrict__ q, uint8_t* __restrict__ s8,
                                                                  int64_t blocks16, int flags, float denom) {
    NvScales gs;
    gs.enc_sixth = u2f(amax_bits[kRecEncSixth]);
    gs.s_dec = u2f(amax_bits[kRecSDec]);
    gs.enc = u2f(amax_bits[kRecEnc]);
    const float amax = u2f(amax_bits[kRecAmax]);
    const int64_t stride = (int64_t)gridDim.x * blockDim.x;
    for (int64_t b = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; b < blocks16; b += stride) {
        uint32_t m = 0;
        for (int j = 0; j < 16; j++) m = umax(m, f2u(load_f32(w, b * 16 + j, dtype)) & 0x7FFFFFFFu);
        const float bmax = u2f(m);
        if (flags & MQ_NVFP4_4OVER6) {
            float x[16];
            for (int j = 0; j < 16; j++) x[j] = load_f32(w, b * 16 + j, dtype);
            const float s6_hp = (bmax / 6.0f) * gs.enc, s4_hp = s6_hp * 1.5f;
            const uint32_t sc4 = sw_e4m3fn_sat(__builtin_fminf(s4_hp, kFp8Max)), sc6 = sw_e4m3fn_sat(__builtin_fminf(s6_hp, kFp8Max));
            uint32_t c4[16], c6[16];
            const float e4 = nv_candidate_sw(x, sc4, amax, gs, denom, flags, c4);
            const float e6 = nv_candidate_sw(x, sc6, amax, gs, denom, flags, c6);
            const bool pick4 = e4 < e6;
            s8[b] = (uint8_t)(pick4 ? sc4 : sc6);
            for (int j = 0; j < 16; j += 2)
                q[b * 8 + j / 2] = (uint8_t)(pick4 ? (c4[j] | (c4[j + 1] << 4)) : (c6[j] | (c6[j + 1] << 4)));
            continue;
        }
        const float s_hp = bmax == 0.0f ? 0.0f : bmax * gs.enc_sixth;
        const uint32_t sc = sw_e4m3fn_sat(s_hp);
        s8[b] = (uint8_t)sc;
        const float inv = __builtin_fminf(1.0f / (sw_e4m3fn_decode(sc) * gs.s_dec), kFltMax);
        for (int j = 0; j < 16; j += 2) {
            const uint32_t lo = sw_e2m1(load_f32(w, b * 16 + j, dtype) * inv);
            const uint32_t hi = sw_e2m1(load_f32(w, b * 16 + j + 1, dtype) * inv);
            q[b * 8 + j / 2] = (uint8_t)(lo | (hi << 4));
        }
    }
}

// ---- fused quantize + dequantize (training-forward fake quantization) -------------------------------
// Reference: miles/kernels/quant/nvfp4_qdq.py:877-890 (standard quantize), :993-1029 (dequantize), kernel :1067-1105.
// Given the tensor amax (a device scalar): codes and block scale exactly as the quantizer above, then
//   final = RN(RN(f32(s8) * amax) * f32(1 / (6 * e4m3_max)));  y = dtype(RN(e2m1_value * final))
// Two lanes own one 1x16 block; nothing but x is read and nothing but y written.
template <int DT, int FOS>
__global__ __launch_bounds__(kNvThreads) void nvfp4_qdq_kernel(const uint16_t* __restrict__ x,
                                                               const float* __restrict__ amax_ptr,
                                                               uint16_t* __restrict__ y, int64_t total_units,
                                                               float numer, float inv_numer, int chunk) {
    const int t = threadIdx.x;
    const int64_t unit = xcd_chunked_block(chunk) * kNvThreads + t;
    const bool live = unit < total_units;
    const u32x4 v = ld16(x + (live ? unit : total_units - 1) * 8);
    const float amax = *amax_ptr;
    const NvScales gs = nv_scales(amax, numer);
    float f[8];
    const uint32_t u[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
    for (int i = 0; i < 4; i++) {
        if (DT == MQ_BF16) { f[2 * i] = bf16_lo(u[i]); f[2 * i + 1] = bf16_hi(u[i]); }
        else {
            f[2 * i] = (float)__builtin_bit_cast(_Float16, (uint16_t)(u[i] & 0xFFFFu));
            f[2 * i + 1] = (float)__builtin_bit_cast(_Float16, (uint16_t)(u[i] >> 16));
        }
    }
    uint32_t m = 0;
#pragma unroll
    for (int i = 0; i < 8; i++) m = umax(m, f2u(f[i]) & 0x7FFFFFFFu);
    m = group_max2(m);
    const float bmax = u2f(m);
    const float s_hp = bmax == 0.0f ? 0.0f : bmax * gs.enc_sixth;
    float s_f, q[8];
    if (FOS) {
        constexpr int EM = FOS > 0 ? FOS - 1 : 0;
        const int fastdiv = nv_fast_division(amax);
        const NvCandidate c = fastdiv == 2   ? nv_four_over_six<EM, 2>(f, bmax, amax, gs, numer, (t & 1) != 0)
                              : fastdiv == 1 ? nv_four_over_six<EM, 1>(f, bmax, amax, gs, numer, (t & 1) != 0)
                                             : nv_four_over_six<EM, 0>(f, bmax, amax, gs, numer, (t & 1) != 0);
        s_f = c.s_f;
        nv_decode8(c.word, q);
    } else if (m < 0x7F800000u && s_hp == s_hp) {
        const uint32_t sc = hw_e4m3x2<false>(__builtin_fminf(s_hp, kFp8Max), 0.0f, 0u) & 0xFFu;
        s_f = hw_e4m3x2_decode<false>(sc).x;
        const float inv = __builtin_fminf(1.0f / (s_f * gs.s_dec), kFltMax);
        uint32_t word = hw_e2m1x2<0>(f[0] * inv, f[1] * inv, 0u);
        word = hw_e2m1x2<1>(f[2] * inv, f[3] * inv, word);
        word = hw_e2m1x2<2>(f[4] * inv, f[5] * inv, word);
        word = hw_e2m1x2<3>(f[6] * inv, f[7] * inv, word);
        const f32x2 a = __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(word, 1.0f, 0), b = __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(word, 1.0f, 1);
        const f32x2 c = __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(word, 1.0f, 2), d = __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(word, 1.0f, 3);
        q[0] = a.x; q[1] = a.y; q[2] = b.x; q[3] = b.y; q[4] = c.x; q[5] = c.y; q[6] = d.x; q[7] = d.y;
    } else {
        const uint32_t sc = sw_e4m3fn_sat(s_hp);
        s_f = sw_e4m3fn_decode(sc);
        const float inv = __builtin_fminf(1.0f / (s_f * gs.s_dec), kFltMax);
#pragma unroll
        for (int j = 0; j < 8; j++) {
            const uint32_t c = sw_e2m1(f[j] * inv);
            const float mag = (c & 7u) < 2u ? 0.5f * (float)(c & 7u) : u2f(0x3F000000u + ((c & 7u) << 22));
            q[j] = (c & 8u) ? -mag : mag;
        }
    }
    const float final_scale = (s_f * amax) * inv_numer;
#pragma unroll
    for (int j = 0; j < 8; j++) q[j] = q[j] * final_scale;
    if (!live) return;
    if (DT == MQ_BF16) {
        st16(y + unit * 8, u32x4{hw_bf16x2(q[0], q[1]), hw_bf16x2(q[2], q[3]), hw_bf16x2(q[4], q[5]), hw_bf16x2(q[6], q[7])});
    } else {
        uint32_t p[4];
#pragma unroll
        for (int i = 0; i < 4; i++) {
            float a = q[2 * i], b = q[2 * i + 1];
            asm volatile("" : "+v"(a), "+v"(b));     // keep the product apart from the conversion: a fused fma(.., +0) loses -0
            p[i] = (uint32_t)__builtin_bit_cast(uint16_t, (_Float16)a) | ((uint32_t)__builtin_bit_cast(uint16_t, (_Float16)b) << 16);
        }
        st16(y + unit * 8, u32x4{p[0], p[1], p[2], p[3]});
    }
}

}  // namespace mq

using namespace mq;

bool mq_nvfp4_fast_ok(const void* w, int dtype, const void* q) {
    return (dtype == MQ_BF16 || dtype == MQ_F16) && ((uintptr_t)w % 16) == 0 && ((uintptr_t)q % 4) == 0;
}

// the 16-bit dtype of a launch's tensors rides in the flags word of the launch helpers below (not a public flag)
constexpr int kNvFlagF16 = 1 << 30;

// tab.job[i]: w, aux = amax record, section, units = numel / 8, s = (void*)numel; every tensor of the one 16-bit dtype
int mq_nvfp4_amax_launch_group(int dtype, FlatTable& tab, hipStream_t st) {
    const dim3 grid(kSectionWords, (unsigned)tab.n), blk(256);
    if (dtype == MQ_F16) hipLaunchKernelGGL((nvfp4_amax_bf16_kernel<FlatTable, 1>), grid, blk, 0, st, tab);
    else hipLaunchKernelGGL((nvfp4_amax_bf16_kernel<FlatTable, 0>), grid, blk, 0, st, tab);
    return mq_check_launch("nvfp4 amax");
}
// the same over n descriptors of a device table (the quantizer's form: whole units, section = place inside the record)
int mq_nvfp4_amax_launch_table(int dtype, const FlatJob* device_jobs, int n, hipStream_t st) {
    if (n == 0) return MQ_OK;
    const FlatRef ref{device_jobs, 0, 0};
    const dim3 grid(kSectionWords, (unsigned)n), blk(256);
    if (dtype == MQ_F16) hipLaunchKernelGGL((nvfp4_amax_bf16_kernel<FlatRef, 1>), grid, blk, 0, st, ref);
    else hipLaunchKernelGGL((nvfp4_amax_bf16_kernel<FlatRef, 0>), grid, blk, 0, st, ref);
    return mq_check_launch("nvfp4 amax");
}

template <int PASS, class Table, int F16>
static void launch_nvfp4_quant_dtype(const Table& tab, int flags, float numer, dim3 grid, hipStream_t st) {
    const dim3 blk(kNvThreads);
    // Four Over Six keeps to launches of kernel-argument tables (its five error modes are not built in the other form)
    const int fos = (flags & MQ_NVFP4_4OVER6) ? 1 + nv_error_mode(flags) : 0;
    if constexpr (std::is_same<Table, FlatRef>::value) {
        hipLaunchKernelGGL((nvfp4_quant_bf16_kernel<0, PASS, Table, F16>), grid, blk, 0, st, tab, numer);
    } else {
        switch (fos) {
            case 0: hipLaunchKernelGGL((nvfp4_quant_bf16_kernel<0, PASS, Table, F16>), grid, blk, 0, st, tab, numer); break;
            case 1: hipLaunchKernelGGL((nvfp4_quant_bf16_kernel<1, PASS, Table, F16>), grid, blk, 0, st, tab, numer); break;
            case 2: hipLaunchKernelGGL((nvfp4_quant_bf16_kernel<2, PASS, Table, F16>), grid, blk, 0, st, tab, numer); break;
            case 3: hipLaunchKernelGGL((nvfp4_quant_bf16_kernel<3, PASS, Table, F16>), grid, blk, 0, st, tab, numer); break;
            default: hipLaunchKernelGGL((nvfp4_quant_bf16_kernel<4, PASS, Table, F16>), grid, blk, 0, st, tab, numer); break;
        }
    }
}
template <int PASS, class Table>
static void launch_nvfp4_quant(const Table& tab, int flags, float numer, dim3 grid, hipStream_t st) {
    if (flags & kNvFlagF16) launch_nvfp4_quant_dtype<PASS, Table, 1>(tab, flags, numer, grid, st);
    else launch_nvfp4_quant_dtype<PASS, Table, 0>(tab, flags, numer, grid, st);
}

// fold + quantize (+ second pass) over a table whose grid is known: tab.chunk / tab.max_blocks are set
template <class Table>
static int nvfp4_quant_launch(const Table& tab, int n, int e4m3_max, int flags, int mode, hipStream_t st) {
    const float numer = (float)e4m3_max * 6.0f;
    const dim3 folds((unsigned)n), blk(256);
    const dim3 grid((unsigned)tab.max_blocks, (unsigned)n);
    if (mode == 2) {
        if (tab.max_blocks > 0) launch_nvfp4_quant<1>(tab, flags, numer, grid, st);
        hipLaunchKernelGGL((nvfp4_fold_kernel<2, Table>), folds, blk, 0, st, tab, numer, mq_amax_feedback(), mq_amax_feedback_mirror());
        if (tab.max_blocks > 0) {
            const unsigned redo_blocks = tab.max_blocks < kSectionWords ? (unsigned)tab.max_blocks : (unsigned)kSectionWords;
            launch_nvfp4_quant<2>(tab, flags, numer, dim3(redo_blocks, (unsigned)n), st);
        }
        return mq_check_launch("nvfp4 quant (carried-over amax)");
    }
    if (mode == 1) hipLaunchKernelGGL((nvfp4_fold_kernel<1, Table>), folds, blk, 0, st, tab, numer, mq_amax_feedback(), mq_amax_feedback_mirror());
    else hipLaunchKernelGGL((nvfp4_fold_kernel<0, Table>), folds, blk, 0, st, tab, numer, (uint32_t*)nullptr, (uint32_t*)nullptr);
    if (tab.max_blocks > 0) launch_nvfp4_quant<0>(tab, flags, numer, grid, st);
    return mq_check_launch("nvfp4 quant");
}

// tab.job[i]: w, q, s = block scales, aux = amax record, aux2 = fp32 global scale out (may be null), units = numel / 8.
// mode 0 (single calls): section = sections to fold; fold, then quantize.
// mode 1 (job driver, after its amax launch): section = place of the tensor inside its record, pad = tensors sharing the
//   record (adjacent entries); fold once per record, clear the sections, quantize.
// mode 2 (job driver, carried-over amax; the sections were cleared by the previous sync's fold): quantize with the
//   record's old scales while collecting the new partial maxima, fold and compare, quantize again where they differ.
int mq_nvfp4_quant_launch_group(int dtype, FlatTable& tab, int e4m3_max, int flags, int mode, hipStream_t st) {
    if (!flat_grid(tab, nv_units_per_block(flags & MQ_NVFP4_4OVER6))) return mq_fail(MQ_ERR_ARG, "tensor too large");
    return nvfp4_quant_launch(tab, tab.n, e4m3_max, flags | (dtype == MQ_F16 ? kNvFlagF16 : 0), mode, st);
}
// modes 1 and 2 over n descriptors of a device table (standard block scaling only); max_units: the largest tensor's units
int mq_nvfp4_quant_launch_table(int dtype, const FlatJob* device_jobs, int n, int64_t max_units, int e4m3_max, int mode,
                                hipStream_t st) {
    FlatRef ref{device_jobs, 0, 0};
    if (!flat_grid(ref, max_units, kNvThreads * kNvUnroll)) return mq_fail(MQ_ERR_ARG, "tensor too large");
    if (n == 0) return MQ_OK;
    return nvfp4_quant_launch(ref, n, e4m3_max, dtype == MQ_F16 ? kNvFlagF16 : 0, mode, st);
}

extern "C" int mq_nvfp4_amax(const void* w, int dtype, int64_t numel, void* record, int section, void* stream) {
    if ((!w && numel != 0) || !record) return mq_fail(MQ_ERR_ARG, "null pointer");
    if (dtype < MQ_BF16 || dtype > MQ_F32 || numel < 0) return mq_fail(MQ_ERR_ARG, "bad argument");
    if (section < 0 || section >= MQ_NVFP4_SECTIONS) return mq_fail(MQ_ERR_ARG, "bad amax record section");
    hipStream_t st = (hipStream_t)stream;
    if ((dtype == MQ_BF16 || dtype == MQ_F16) && ((uintptr_t)w % 16) == 0) {
        FlatTable tab{};
        tab.n = 1;
        tab.job[0] = FlatJob{w, nullptr, (void*)(uintptr_t)numel, record, numel / 8, nullptr, section, 0};
        return mq_nvfp4_amax_launch_group(dtype, tab, st);
    }
    hipLaunchKernelGGL(nvfp4_amax_generic_kernel, dim3(kSectionWords), dim3(256), 0, st, w, dtype, numel,
                       (uint32_t*)record + section * kSectionWords);
    return mq_check_launch("nvfp4 amax");
}

extern "C" int mq_nvfp4_quant(const void* w, int dtype, const void* record, int n_sections, void* q, void* block_scale,
                              float* global_scale, int64_t M, int64_t K, int e4m3_max, int flags, void* stream) {
    if (((!w || !q || !block_scale) && M != 0 && K != 0) || !record) return mq_fail(MQ_ERR_ARG, "null pointer");
    if (dtype < MQ_BF16 || dtype > MQ_F32 || M < 0 || K < 0) return mq_fail(MQ_ERR_ARG, "bad argument");
    if (n_sections < 1 || n_sections > MQ_NVFP4_SECTIONS) return mq_fail(MQ_ERR_ARG, "bad amax record section count");
    if (K % 16 != 0) return mq_fail(MQ_ERR_ARG, "Last dim must be divisible by 16 for NVFP4");
    if (e4m3_max != 448 && e4m3_max != 256) return mq_fail(MQ_ERR_ARG, "e4m3_max must be 448 or 256");
    if (flags & ~(MQ_NVFP4_4OVER6 | MQ_NVFP4_ERR_MSE | MQ_NVFP4_ERR_FP16)) return mq_fail(MQ_ERR_ARG, "unknown NVFP4 flag");
    hipStream_t st = (hipStream_t)stream;
    const float numer = (float)e4m3_max * 6.0f;
    const int64_t blocks16 = M * (K / 16);
    if (blocks16 == 0 || mq_nvfp4_fast_ok(w, dtype, q)) {
        FlatTable tab{};
        tab.n = 1;
        tab.job[0] = FlatJob{w, q, block_scale, const_cast<void*>(record), blocks16 * 2, global_scale, n_sections, 0};
        return mq_nvfp4_quant_launch_group(blocks16 == 0 ? MQ_BF16 : dtype, tab, e4m3_max, flags, 0, st);
    }
    FlatTable fold{};
    fold.n = 1;
    fold.job[0] = FlatJob{w, q, block_scale, const_cast<void*>(record), 0, global_scale, n_sections, 0};
    hipLaunchKernelGGL((nvfp4_fold_kernel<0, FlatTable>), dim3(1), dim3(256), 0, st, fold, numer, (uint32_t*)nullptr, (uint32_t*)nullptr);
    int64_t nb = (blocks16 + 255) / 256;
    if (nb > mq_grid_cap()) nb = mq_grid_cap();
    hipLaunchKernelGGL(nvfp4_quant_generic_kernel, dim3((unsigned)nb), dim3(256), 0, st, w, dtype,
                       (const uint32_t*)record, (uint8_t*)q, (uint8_t*)block_scale, blocks16, flags, numer);
    return mq_check_launch("nvfp4 quant");
}

extern "C" int mq_nvfp4_fold(void* record, int n_sections, int e4m3_max, void* stream) {
    if (!record) return mq_fail(MQ_ERR_ARG, "null pointer");
    if (n_sections < 1 || n_sections > MQ_NVFP4_SECTIONS) return mq_fail(MQ_ERR_ARG, "bad amax record section count");
    if (e4m3_max != 448 && e4m3_max != 256) return mq_fail(MQ_ERR_ARG, "e4m3_max must be 448 or 256");
    FlatTable tab{};
    tab.n = 1;
    tab.job[0] = FlatJob{nullptr, nullptr, nullptr, record, 0, nullptr, n_sections, 0};
    hipLaunchKernelGGL((nvfp4_fold_kernel<0, FlatTable>), dim3(1), dim3(256), 0, (hipStream_t)stream, tab, (float)e4m3_max * 6.0f, (uint32_t*)nullptr, (uint32_t*)nullptr);
    return mq_check_launch("nvfp4 fold");
}

extern "C" int mq_nvfp4_qdq(const void* x, int dtype, const float* amax, void* y, int64_t numel, int e4m3_max,
                            int flags, void* stream) {
    if (((!x || !y) && numel != 0) || !amax) return mq_fail(MQ_ERR_ARG, "null pointer");
    if ((dtype != MQ_BF16 && dtype != MQ_F16) || numel < 0) return mq_fail(MQ_ERR_ARG, "input must be bfloat16 or float16");
    if (numel % 16 != 0) return mq_fail(MQ_ERR_ARG, "element count must be a multiple of 16");
    if (e4m3_max != 448 && e4m3_max != 256) return mq_fail(MQ_ERR_ARG, "e4m3_max must be 448 or 256");
    if ((((uintptr_t)x | (uintptr_t)y) & 15) != 0) return mq_fail(MQ_ERR_ARG, "tensors must be 16-byte aligned");
    if (flags & ~(MQ_NVFP4_4OVER6 | MQ_NVFP4_ERR_MSE | MQ_NVFP4_ERR_FP16)) return mq_fail(MQ_ERR_ARG, "unknown NVFP4 flag");
    if (numel == 0) return MQ_OK;
    const int64_t units = numel / 8;
    int64_t blocks = (units + kNvThreads - 1) / kNvThreads;
    const int chunk = (int)flat_chunk(blocks);
    blocks = flat_padded(blocks, chunk);
    if (blocks > 0x7FFFFFF0ll) return mq_fail(MQ_ERR_ARG, "tensor too large");
    const float numer = (float)e4m3_max * 6.0f, inv_numer = (float)(1.0 / (double)(6 * e4m3_max));
    const dim3 grid((unsigned)blocks), blk(kNvThreads);
    hipStream_t st = (hipStream_t)stream;
    const uint16_t* xi = (const uint16_t*)x;
    uint16_t* yo = (uint16_t*)y;
    const int fos = (flags & MQ_NVFP4_4OVER6) ? 1 + nv_error_mode(flags) : 0;
#define MQ_QDQ_LAUNCH(DT, FOS) hipLaunchKernelGGL((nvfp4_qdq_kernel<DT, FOS>), grid, blk, 0, st, xi, amax, yo, units, numer, inv_numer, chunk)
#define MQ_QDQ_SWITCH(DT)                           \
    switch (fos) {                                  \
        case 0: MQ_QDQ_LAUNCH(DT, 0); break;        \
        case 1: MQ_QDQ_LAUNCH(DT, 1); break;        \
        case 2: MQ_QDQ_LAUNCH(DT, 2); break;        \
        case 3: MQ_QDQ_LAUNCH(DT, 3); break;        \
        default: MQ_QDQ_LAUNCH(DT, 4); break;       \
    }
    if (dtype == MQ_BF16) { MQ_QDQ_SWITCH(MQ_BF16) } else { MQ_QDQ_SWITCH(MQ_F16) }
#undef MQ_QDQ_SWITCH
#undef MQ_QDQ_LAUNCH
    return mq_check_launch("nvfp4 qdq");
}
