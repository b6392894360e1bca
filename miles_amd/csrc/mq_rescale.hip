// FP8 128x128 block-scaled weights -> MXFP8 (e4m3 codes, one E8M0 scale per 1x32 group) for gfx950.
// Reference: tools/convert_hf_to_mxfp8.py:56-102 (the source's tile scales: fp32 or exponent bytes, the power-of-two
// test, one exponent per tile repeated to one per group) and :180-195 (a source whose scales are powers of two keeps
// its codes and is relabelled; any other source is dequantized to fp32 with SGLang's block_quant_dequant -- the tile
// scales repeated 128 x 128 and ONE fp32 multiply f32(code) * s[i/128, j/128] -- and quantized again by mxfp8_quantize).
//
// The re-quantizer keeps the fp32 tensor in registers: a lane takes 16 consecutive codes (one 16-byte load), two
// neighbouring lanes share a 1x32 group, which lies inside one 128-column tile, so both hold the same tile scale.
// The group maximum of |f32(code) * s| is taken on the codes: rounding is monotonic, so the largest product is the
// product of the largest code magnitude, and the 7-bit magnitudes of e4m3 order like the values they stand for -- with
// the NaN code 0x7F as the largest pattern, which sends a group that holds one to the written-out form.  HBM traffic is
// one read of the codes and one write of codes and scale bytes: 2 + 1/32 bytes per element, plus the tile scales.
#include "mq_api_internal.hpp"
#include "mq_common.hpp"
#include "mq_group.hpp"

namespace mq {

constexpr int kRsThreads = 256;
#ifndef MQ_RS_UNROLL
#define MQ_RS_UNROLL 2
#endif
constexpr int kRsUnroll = MQ_RS_UNROLL;       // 16-code units per lane

struct RescaleJob {
    const uint8_t* x;        // [M, K] e4m3 codes
    const float* s;          // fp32 tile scales, rows lds elements apart
    uint8_t* q;              // [M, K] e4m3 codes
    uint8_t* scale;          // [M, K / 32] E8M0 bytes
    uint32_t units;          // M * K / 16
    uint32_t units_per_row;  // K / 16, at least 2
    uint32_t magic, shift;   // tile_div constants for units_per_row
    int32_t lds;
    int32_t pad;
};
struct RescaleTable {
    int32_t n;
    int32_t max_blocks;
    int32_t chunk;           // blocks per XCD chunk (xcd_chunked_block); max_blocks is a multiple of 8 * chunk
    int32_t pad;
    RescaleJob job[kMaxGroup];
};

__global__ __launch_bounds__(kRsThreads) void fp8_to_mxfp8_kernel(const RescaleTable tab) {
    const float inv448 = u2f(0x3B124925u);
    const RescaleJob& job = tab.job[blockIdx.y];
    const int64_t base64 = xcd_chunked_block(tab.chunk) * (kRsThreads * kRsUnroll);
    if (base64 >= job.units) return;
    const uint32_t base = (uint32_t)base64, t = threadIdx.x;
    u32x4 in[kRsUnroll];
    float sc[kRsUnroll];
#pragma unroll
    for (int i = 0; i < kRsUnroll; i++) {
        const uint32_t unit = base + i * kRsThreads + t;
        // past the end a lane reads the last unit again (the units come in pairs, so a group is whole or absent)
        const uint32_t u = unit < job.units ? unit : job.units - 1u;
        in[i] = ld16(job.x + (int64_t)u * 16);
        const uint32_t row = tile_div(u, job.magic, job.shift);
        const uint32_t cu = u - row * job.units_per_row;
        sc[i] = job.s[(int64_t)(row >> 7) * job.lds + (cu >> 3)];
    }
#pragma unroll
    for (int i = 0; i < kRsUnroll; i++) {
        const uint32_t unit = base + i * kRsThreads + t;
        const uint32_t w[4] = {in[i].x, in[i].y, in[i].z, in[i].w};
        uint32_t m2 = 0;
#pragma unroll
        for (int k = 0; k < 4; k++) m2 = max2_u16(m2, max2_u16(w[k] & 0x007F007Fu, (w[k] >> 8) & 0x007F007Fu));
        const uint32_t mb = group_max2(hmax_u16(m2));      // largest magnitude pattern of the group's 32 codes
        const uint32_t sbits = f2u(sc[i]) & 0x7FFFFFFFu;
        // no NaN code, and a scale whose products stay finite (448 * 2^118 < 2^127): the maximum can be taken on the codes
        const bool plain = mb != 0x7Fu && sbits <= 0x7A800000u;
        uint32_t e, o[4];
        if (plain) {
            const float amax = hw_e4m3x2_decode<false>(mb).x * u2f(sbits);
            e = e8m0_ceil(amax * inv448);
            const float inv = e8m0_inverse(e);
            const float s = sc[i];
#pragma unroll
            for (int k = 0; k < 4; k++) {
                const f32x2 a = hw_e4m3x2_decode<false>(w[k]), b = hw_e4m3x2_decode<true>(w[k]);
                // two roundings, as the reference makes them: the fp32 tensor, then its scaling (exact bar underflow);
                // |product| <= 448 (1 + 2^-22), which the convert rounds to 448
                o[k] = hw_e4m3x4((a.x * s) * inv, (a.y * s) * inv, (b.x * s) * inv, (b.y * s) * inv);
            }
        } else {
            // a NaN code or a huge / non-finite scale (rare; both lanes of a group branch together): element by element,
            // the maximum skipping NaN and keeping an infinity, the conversion saturating
            float f[16];
            uint32_t m = 0;
#pragma unroll
            for (int j = 0; j < 16; j++) {
                f[j] = sw_e4m3fn_decode((w[j >> 2] >> (8 * (j & 3))) & 0xFFu) * sc[i];
                const uint32_t a = f2u(f[j]) & 0x7FFFFFFFu;
                m = umax(m, a > 0x7F800000u ? 0u : a);
            }
            m = group_max2(m);
            e = e8m0_ceil(u2f(m) * inv448);
            const float inv = e8m0_inverse(e);
#pragma unroll
            for (int k = 0; k < 4; k++) {
                o[k] = 0;
#pragma unroll
                for (int b = 0; b < 4; b++) o[k] |= sw_e4m3fn_sat(f[4 * k + b] * inv) << (8 * b);
            }
        }
        if (unit < job.units) {
            st16(job.q + (int64_t)unit * 16, u32x4{o[0], o[1], o[2], o[3]});
            if ((t & 1u) == 0) job.scale[unit >> 1] = (uint8_t)e;
        }
    }
}

// any alignment: one lane per 1x32 group, byte accesses
__global__ __launch_bounds__(256) void fp8_to_mxfp8_generic_kernel(const uint8_t* __restrict__ x, const float* __restrict__ s,
                                                                   int64_t lds, uint8_t* __restrict__ q,
                                                                   uint8_t* __restrict__ scale, int64_t groups,
                                                                   int64_t groups_per_row) {
    const float inv448 = u2f(0x3B124925u);
    const int64_t stride = (int64_t)gridDim.x * blockDim.x;
    for (int64_t g = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; g < groups; g += stride) {
        const int64_t row = g / groups_per_row, cg = g - row * groups_per_row;
        const float sc = s[(row >> 7) * lds + (cg >> 2)];
        uint32_t m = 0;
        for (int j = 0; j < 32; j++) {
            const uint32_t a = f2u(sw_e4m3fn_decode(x[g * 32 + j]) * sc) & 0x7FFFFFFFu;
            m = umax(m, a > 0x7F800000u ? 0u : a);
        }
        const uint32_t e = e8m0_ceil(u2f(m) * inv448);
        const float inv = e8m0_inverse(e);
        scale[g] = (uint8_t)e;
        for (int j = 0; j < 32; j++) q[g * 32 + j] = (uint8_t)sw_e4m3fn_sat((sw_e4m3fn_decode(x[g * 32 + j]) * sc) * inv);
    }
}

// One exponent byte per 128x128 tile -> one per 1x32 group: out[r, g] = byte(s[r / 128, g / 4]).  WORDS: a lane writes
// the four equal bytes of one tile's piece of a row as one word (K % 128 == 0, aligned output), else one byte.
template <bool F32, bool WORDS>
__global__ __launch_bounds__(256) void e8m0_expand_kernel(const void* __restrict__ s, int64_t lds, uint8_t* __restrict__ out,
                                                          int64_t total, int64_t per_row) {
    const int64_t stride = (int64_t)gridDim.x * blockDim.x;
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += stride) {
        const int64_t r = i / per_row, j = i - r * per_row;
        const int64_t at = (r >> 7) * lds + (WORDS ? j : (j >> 2));
        const uint32_t byte = F32 ? (f2u(((const float*)s)[at]) >> 23) & 0xFFu : ((const uint8_t*)s)[at];
        if (WORDS) ((uint32_t*)out)[i] = byte * 0x01010101u;
        else out[i] = (uint8_t)byte;
    }
}

// flag <- 1 when every scale of the grid is a power of two with its sign bit clear (mantissa bits all zero), else 0
__global__ __launch_bounds__(256) void fp8_scales_pow2_kernel(const float* __restrict__ s, int64_t rows, int64_t cols,
                                                              int64_t lds, uint32_t* __restrict__ flag) {
    uint32_t bad = 0;
    for (int64_t i = threadIdx.x; i < rows * cols; i += 256) {
        const int64_t r = i / cols, c = i - r * cols;
        const uint32_t u = f2u(s[r * lds + c]);
        bad |= (u & 0x007FFFFFu) | (u >> 31);
    }
    const int any = __syncthreads_or(bad != 0u);
    if (threadIdx.x == 0) *flag = any ? 0u : 1u;
}

// exponent bytes as the fp32 numbers with those exponent fields: bits = byte << 23 (byte 0 gives 0.0, byte 255 +inf)
__global__ __launch_bounds__(256) void e8m0_to_f32_kernel(const uint8_t* __restrict__ s, float* __restrict__ out, int64_t n) {
    const int64_t stride = (int64_t)gridDim.x * blockDim.x;
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride) out[i] = u2f((uint32_t)s[i] << 23);
}

}  // namespace mq

using namespace mq;

bool mq_fp8_to_mxfp8_fast_ok(const void* x, const void* q, int64_t M, int64_t K) {
    return K % 32 == 0 && ((uintptr_t)x % 16) == 0 && ((uintptr_t)q % 16) == 0 && M * (K / 16) < 0xFFFFFFF0ll;
}

int mq_fp8_to_mxfp8_launch_group(const MqRescaleArgs* a, int n, hipStream_t st) {
    RescaleTable tab{};
    tab.n = n;
    int64_t mx = 0;
    for (int i = 0; i < n; i++) {
        RescaleJob& j = tab.job[i];
        j.x = (const uint8_t*)a[i].x;
        j.s = a[i].s;
        j.q = (uint8_t*)a[i].q;
        j.scale = a[i].scale;
        j.units = (uint32_t)(a[i].M * (a[i].K / 16));
        j.units_per_row = (uint32_t)(a[i].K / 16);
        tile_div_magic(j.units_per_row, j.magic, j.shift);
        j.lds = (int32_t)a[i].lds;
        const int64_t b = ((int64_t)j.units + kRsThreads * kRsUnroll - 1) / (kRsThreads * kRsUnroll);
        if (b > mx) mx = b;
    }
    if (mx == 0) return MQ_OK;
    const int64_t chunk = flat_chunk(mx);
    mx = flat_padded(mx, chunk);
    tab.chunk = (int32_t)chunk;
    tab.max_blocks = (int32_t)mx;
    hipLaunchKernelGGL(fp8_to_mxfp8_kernel, dim3((unsigned)mx, (unsigned)n), dim3(kRsThreads), 0, st, tab);
    return mq_check_launch("fp8 block to mxfp8");
}

extern "C" int mq_fp8_block_to_mxfp8(const void* x, const float* s, int64_t lds, void* q, uint8_t* scale, int64_t M,
                                     int64_t K, void* stream) {
    if ((!x || !s || !q || !scale) && M != 0 && K != 0) return mq_fail(MQ_ERR_ARG, "null pointer");
    if (M < 0 || K < 0) return mq_fail(MQ_ERR_ARG, "bad shape");
    if (K % 32 != 0) return mq_fail(MQ_ERR_ARG, "Last dim must be divisible by 32 for MXFP8.");
    if (M == 0 || K == 0) return MQ_OK;
    if (lds < (K + 127) / 128 || lds > 0x7FFFFFFF) return mq_fail(MQ_ERR_ARG, "tile-scale rows overlap (lds below ceil(K / 128))");
    hipStream_t st = (hipStream_t)stream;
    if (mq_fp8_to_mxfp8_fast_ok(x, q, M, K)) {
        const MqRescaleArgs a{x, s, q, scale, M, K, lds};
        return mq_fp8_to_mxfp8_launch_group(&a, 1, st);
    }
    const int64_t groups = M * (K / 32);
    int64_t blocks = (groups + 255) / 256;
    if (blocks > mq_grid_cap()) blocks = mq_grid_cap();
    hipLaunchKernelGGL(fp8_to_mxfp8_generic_kernel, dim3((unsigned)blocks), dim3(256), 0, st, (const uint8_t*)x, s, lds,
                       (uint8_t*)q, scale, groups, K / 32);
    return mq_check_launch("fp8 block to mxfp8");
}

extern "C" int mq_e8m0_expand_tile_scales(const void* s, int scales_are_f32, int64_t lds, uint8_t* out, int64_t M,
                                          int64_t groups, void* stream) {
    if ((!s || !out) && M != 0 && groups != 0) return mq_fail(MQ_ERR_ARG, "null pointer");
    if (M < 0 || groups < 0) return mq_fail(MQ_ERR_ARG, "bad shape");
    if (M == 0 || groups == 0) return MQ_OK;
    if (lds < (groups + 3) / 4) return mq_fail(MQ_ERR_ARG, "tile-scale rows overlap (lds below ceil(groups / 4))");
    const bool words = groups % 4 == 0 && ((uintptr_t)out % 4) == 0;
    const int64_t per_row = words ? groups / 4 : groups, total = M * per_row;
    int64_t blocks = (total + 255) / 256;
    if (blocks > mq_grid_cap()) blocks = mq_grid_cap();
    const dim3 grid((unsigned)blocks), blk(256);
    hipStream_t st = (hipStream_t)stream;
    if (scales_are_f32) {
        if (words) hipLaunchKernelGGL((e8m0_expand_kernel<true, true>), grid, blk, 0, st, s, lds, out, total, per_row);
        else hipLaunchKernelGGL((e8m0_expand_kernel<true, false>), grid, blk, 0, st, s, lds, out, total, per_row);
    } else {
        if (words) hipLaunchKernelGGL((e8m0_expand_kernel<false, true>), grid, blk, 0, st, s, lds, out, total, per_row);
        else hipLaunchKernelGGL((e8m0_expand_kernel<false, false>), grid, blk, 0, st, s, lds, out, total, per_row);
    }
    return mq_check_launch("e8m0 scale expansion");
}

extern "C" int mq_fp8_scales_pow2_flag(const float* s, int64_t rows, int64_t cols, int64_t lds, uint32_t* flag,
                                       void* stream) {
    if (!flag || (!s && rows != 0 && cols != 0)) return mq_fail(MQ_ERR_ARG, "null pointer");
    if (rows < 0 || cols < 0 || (rows > 0 && lds < cols)) return mq_fail(MQ_ERR_ARG, "bad shape");
    hipLaunchKernelGGL(fp8_scales_pow2_kernel, dim3(1), dim3(256), 0, (hipStream_t)stream, s, rows, cols, lds, flag);
    return mq_check_launch("fp8 scale power-of-two test");
}

extern "C" int mq_e8m0_bytes_to_f32(const uint8_t* s, float* out, int64_t n, void* stream) {
    if ((!s || !out) && n != 0) return mq_fail(MQ_ERR_ARG, "null pointer");
    if (n < 0) return mq_fail(MQ_ERR_ARG, "bad size");
    if (n == 0) return MQ_OK;
    int64_t blocks = (n + 255) / 256;
    if (blocks > mq_grid_cap()) blocks = mq_grid_cap();
    hipLaunchKernelGGL(e8m0_to_f32_kernel, dim3((unsigned)blocks), dim3(256), 0, (hipStream_t)stream, s, out, n);
    return mq_check_launch("e8m0 bytes to fp32");
}
