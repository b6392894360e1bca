// FP8 e4m3 block-scale quantizers and the block dequantizer for gfx950.
//
//   mode 0  "block_fp8"          scale = amax/448 (true division), q = e4m3(clamp(w/scale)); an all-zero
//                                tile has scale 0 and every byte 0xFF   (reference: tools/convert_hf_to_fp8.py:39-70)
//   mode 1  "fp8_blockwise_cast" absmax = max(amax,1e-10), x_s = absmax/448, q = e4m3(clamp(x * (1/x_s)))
//                                                                       (reference: miles/kernels/quant/fp8_blockwise.py:43-58)
//   mode 2  "per_block_cast_to_fp8" (power-of-two scales) absmax = max(amax,1e-4), sf = 2^ceil(log2(absmax/448)),
//                                q = e4m3(x * (1/sf)).  SGLang's function (third party, not in the reference tree; called at
//                                .../processors/quantizer_fp8.py:139-147); restated from its published source
//   dequant y = bf16(float(q) * s[i/B][j/B])                            (reference: tools/fp8_cast_bf16.py:15-40)
//
// Fast path (bf16 or fp16, 128x128 tiles, 16-byte aligned rows): one 512-lane workgroup (eight wavefronts) owns one tile.
// Lane t loads four 16-byte row segments (rows t/16 + 32 i, columns 8 (t%16) ..+8) so that sixteen lanes read one
// contiguous 256-byte tile row; the 32 values stay in registers, the tile amax is reduced with DPP inside each
// wavefront and through eight LDS words across the wavefronts, and the tile is quantized from registers:
// HBM traffic is one read of the input and one write of the codes and scale.
#include <mutex>

#include "mq_api_internal.hpp"
#include "mq_common.hpp"
#include "mq_group.hpp"

namespace mq {

constexpr int kTile = 128;
#ifndef MQ_TILE_THREADS
#define MQ_TILE_THREADS 512
#endif
constexpr int kTileThreads = MQ_TILE_THREADS;            // 8 wavefronts per 128x128 tile
constexpr int kRowsPerThread = 2048 / kTileThreads;     // 16-byte row segments per lane
constexpr int kRowStep = kTileThreads / 16;             // tile rows covered per pass of the workgroup
constexpr int kTileWaves = kTileThreads / kWave;

// 2^ceil(log2 v) for a normal positive v (the floor of 1e-4 / 448 keeps it normal): exponent, plus one when the
// mantissa is not zero.  For bf16 / fp16 inputs this is what pow(2, ceil(log2(v))) evaluates to in floating point
// as well: v is either an exact power of two or far from one.
__device__ __forceinline__ float ceil_pow2_scale(float v) {
    const uint32_t u = f2u(v);
    return u2f(((u >> 23) + ((u & 0x7FFFFFu) != 0)) << 23);
}

// Everything that is the same for the whole workgroup stays on the scalar unit (with the job lookup and the tile
// addressing in vector instructions the kernel issued 460 of them per wavefront; it issues about 200 now and the
// vector unit is busy a third of the time, the memory system being what bounds it): the job lookup, the tile's row and column (a
// multiply-high division with constants from the host), the 64-bit base addresses of the tile in the input and in the
// output.  A lane adds 32-bit offsets to those bases.  Interior tiles take a path with no bounds tests at all; edge
// tiles load from clamped (always valid) addresses and zero what lies outside, so that in both cases the four loads of
// a lane are issued back to back.
// which tensor and which of its tiles a workgroup works on: searched in the running counts of a kernel-argument table, or
// read off the two-dimensional grid of a device table (the workgroup then leaves if its tensor has fewer tiles)
struct TilePick {
    int32_t ji;         // index into tab.job
    int32_t tile;       // -1: nothing to do
};
__device__ __forceinline__ TilePick pick_tile(const TileTable& tab) {
    const int32_t item = xcd_contiguous_item(tab.total);
    if (item < 0) return TilePick{0, -1};
    const JobRef ref = find_job(tab, item);
    return TilePick{ref.ji, item - ref.start};
}
__device__ __forceinline__ TilePick pick_tile(const TileRef& tab) {
    const TileJob& job = tab.job[blockIdx.y];
    const int32_t tiles = ((job.M + kTile - 1) / kTile) * ((job.K + kTile - 1) / kTile);
    return TilePick{(int32_t)blockIdx.y, xcd_contiguous_item(tiles)};
}
template <int MODE, class Table, int F16>
__global__ __launch_bounds__(kTileThreads) void fp8_block128_kernel(const Table tab) {
    constexpr uint32_t kInfBits = F16 ? 0x7C00u : 0x7F80u;      // pattern of +inf; anything above is a NaN
    __shared__ uint32_t wave_amax[kTileWaves];
    const TilePick pick = pick_tile(tab);
    if (pick.tile < 0) return;
    const TileJob& job = tab.job[pick.ji];
    const uint32_t tile = (uint32_t)pick.tile;
    const uint32_t M = (uint32_t)job.M, K = (uint32_t)job.K, ldw = (uint32_t)job.ldw;
    const uint32_t tiles_k = (K + kTile - 1) / kTile;
    uint32_t ti = tile, tj = 0;
    if (tiles_k > 1) {
        ti = tile_div(tile, job.magic_k, job.shifts & 0xFFu);
        tj = tile - ti * tiles_k;
    }
    // row-blocked input: the tile's rows sit in block ti / tiles_per_block, at the same offset inside it
    const uint16_t* __restrict__ wt = (const uint16_t*)load_global_ptr(&job.w);
    uint32_t wti = ti;
    if (job.tiles_per_block > 0) {
        const uint32_t tpb = (uint32_t)job.tiles_per_block;
        const uint32_t blk = tpb > 1 ? tile_div(ti, job.magic_b, job.shifts >> 8) : ti;
        wt += (int64_t)blk * job.block_stride;
        wti = ti - blk * tpb;
    }
    wt += (int64_t)wti * kTile * ldw + (int64_t)tj * kTile;
    uint8_t* __restrict__ qt = (uint8_t*)load_global_ptr(&job.q) + (int64_t)ti * kTile * K + (int64_t)tj * kTile;
    float* __restrict__ tile_scales = load_global_ptr(&job.scale);
    const uint32_t rows_left = M - ti * kTile, cols_left = K - tj * kTile;     // both at least 1
    const bool full = rows_left >= (uint32_t)kTile && cols_left >= (uint32_t)kTile;

    const uint32_t t = threadIdx.x, r0 = t >> 4, c0 = (t & 15u) * 8u;
    const bool col_ok = full || c0 < cols_left;  // K % 8 == 0: an 8-wide segment is entirely inside or outside
    u32x4 v[kRowsPerThread];
    if (full) {
        const uint32_t off = (r0 * ldw + c0) * 2u;
#pragma unroll
        for (int i = 0; i < kRowsPerThread; i++) {
            v[i] = ld16((const char*)wt + (off + (uint32_t)i * (2u * kRowStep) * ldw));
            // The first quarter of the tile is waited for before the other three are requested.  With all four loads
            // of every lane in flight at once the sync ran 0.5 - 1.2 % slower (alternating runs on one GPU): the
            // memory queues are full either way, and the narrower front of requests keeps more of them on open pages.
            if (i == 0 && kRowsPerThread > 2) asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        }
    } else {
        const uint32_t c = col_ok ? c0 : 0u;
#pragma unroll
        for (int i = 0; i < kRowsPerThread; i++) {
            const uint32_t r = r0 + kRowStep * i;
            const uint32_t rr = r < rows_left ? r : rows_left - 1u;
            const u32x4 x = ld16((const char*)wt + (rr * ldw + c) * 2u);
            v[i] = (col_ok && r < rows_left) ? x : u32x4{0u, 0u, 0u, 0u};
        }
    }
    const uint32_t qoff = r0 * K + c0;
    auto row_ok = [&](int i) { return full || (col_ok && r0 + kRowStep * i < rows_left); };

    uint32_t m2 = 0;
#pragma unroll
    for (int i = 0; i < kRowsPerThread; i++) {
        m2 = max2_u16(m2, abs2(v[i].x));
        m2 = max2_u16(m2, abs2(v[i].y));
        m2 = max2_u16(m2, abs2(v[i].z));
        m2 = max2_u16(m2, abs2(v[i].w));
    }
    uint32_t m = wave_max(hmax_u16(m2));
    if ((t & (kWave - 1)) == 0) wave_amax[t >> 6] = m;
    __syncthreads();
    m = 0;
#pragma unroll
    for (int k = 0; k < kTileWaves; k++) m = umax(m, wave_amax[k]);
    if (MODE != 0 && m >= kInfBits) {
        // An infinity or a NaN in the tile (rare, and uniform over the workgroup).  Mode 1: Triton's max, maximum and
        // clamp return the operand that is not NaN, so the tile maximum skips NaN and a NaN product clamps to -448.
        // Mode 2: torch's amax hands a NaN on, 2^ceil(log2(.)) of inf / NaN is inf / NaN, and nothing clamps.
        float sx;
        if (MODE == 1) {
            uint32_t mf = 0;
#pragma unroll
            for (int i = 0; i < kRowsPerThread; i++) {
                const uint32_t u[4] = {v[i].x, v[i].y, v[i].z, v[i].w};
#pragma unroll
                for (int k = 0; k < 4; k++) {
                    const uint32_t lo = u[k] & 0x7FFFu, hi = (u[k] >> 16) & 0x7FFFu;
                    mf = umax(mf, umax(lo > kInfBits ? 0u : lo, hi > kInfBits ? 0u : hi));
                }
            }
            mf = wave_max(mf);
            __syncthreads();                    // every wavefront has read the first set of maxima
            if ((t & (kWave - 1)) == 0) wave_amax[t >> 6] = mf;
            __syncthreads();
            mf = 0;
#pragma unroll
            for (int k = 0; k < kTileWaves; k++) mf = umax(mf, wave_amax[k]);
            const float finite_max = elem_lo<F16>(mf);
            sx = (finite_max > 1e-10f ? finite_max : 1e-10f) / kFp8Max;
        } else {
            sx = u2f(m > kInfBits ? 0x7FC00000u : 0x7F800000u);
        }
        const float yx = 1.0f / sx;
        if (t == 0) tile_scales[tile] = sx;
#pragma unroll 1
        for (int i = 0; i < kRowsPerThread; i++) {
            const float f[8] = {elem_lo<F16>(v[i].x), elem_hi<F16>(v[i].x), elem_lo<F16>(v[i].y), elem_hi<F16>(v[i].y),
                                elem_lo<F16>(v[i].z), elem_hi<F16>(v[i].z), elem_lo<F16>(v[i].w), elem_hi<F16>(v[i].w)};
            uint32_t c[8];
#pragma unroll
            for (int j = 0; j < 8; j++) {
                float p = f[j] * yx;
                if (MODE == 1) p = __builtin_fminf(__builtin_fmaxf(p, -kFp8Max), kFp8Max);
                c[j] = sw_e4m3fn(p);
            }
            if (row_ok(i))
                st8(qt + (qoff + (uint32_t)i * kRowStep * K),
                    u32x2{c[0] | (c[1] << 8) | (c[2] << 16) | (c[3] << 24), c[4] | (c[5] << 8) | (c[6] << 16) | (c[7] << 24)});
        }
        return;
    }
    const float amax = elem_lo<F16>(m);

    float s;
    if (MODE == 0) s = amax / kFp8Max;
    else if (MODE == 1) s = (amax > 1e-10f ? amax : 1e-10f) / kFp8Max;
    else s = ceil_pow2_scale((amax > 1e-4f ? amax : 1e-4f) / kFp8Max);
    const float y = 1.0f / s;
    if (t == 0) tile_scales[tile] = s;

    if (MODE == 0 && !(amax > 0.0f) && amax == amax) {
        // all-zero tile: 0/0 on every element; the reference's CPU result is the negative NaN code
#pragma unroll
        for (int i = 0; i < kRowsPerThread; i++)
            if (row_ok(i)) st8(qt + (qoff + (uint32_t)i * kRowStep * K), u32x2{0xFFFFFFFFu, 0xFFFFFFFFu});
        return;
    }
    const bool fast_div = (MODE != 0) || shared_div_ok(s);

#pragma unroll
    for (int i = 0; i < kRowsPerThread; i++) {
        float f[8] = {elem_lo<F16>(v[i].x), elem_hi<F16>(v[i].x), elem_lo<F16>(v[i].y), elem_hi<F16>(v[i].y),
                      elem_lo<F16>(v[i].z), elem_hi<F16>(v[i].z), elem_lo<F16>(v[i].w), elem_hi<F16>(v[i].w)};
#pragma unroll
        for (int j = 0; j < 8; j++) {
            // |w/s| <= 448 (1 + 2^-22): no clamp is needed, the convert rounds anything up to 464 to 448
            if (MODE != 0) f[j] = f[j] * y;
            else f[j] = fast_div ? div_by_shared(f[j], s, y) : f[j] / s;
        }
        u32x2 o;
        o.x = hw_e4m3x4(f[0], f[1], f[2], f[3]);
        o.y = hw_e4m3x4(f[4], f[5], f[6], f[7]);
        if (row_ok(i)) st8(qt + (qoff + (uint32_t)i * kRowStep * K), o);
    }
}

constexpr int kGenThreads = 256;
// Any dtype, any strides, any block size: one workgroup per tile, two passes over the tile (the second
// one is served by the caches).  Correctness path for shapes the fast kernel does not take.
template <int MODE>
__global__ __launch_bounds__(kGenThreads) void fp8_block_generic_kernel(const void* __restrict__ w, int dtype,
                                                                         int64_t sxm, int64_t sxn,
                                                                         uint8_t* __restrict__ q, int64_t ldq,
                                                                         float* __restrict__ scale, int64_t M,
                                                                         int64_t K, int bm, int bk, int tiles_k) {
    __shared__ uint32_t wave_amax[kGenThreads / kWave];
    const int t = threadIdx.x;
    const int64_t tile = blockIdx.x;
    const int64_t ti = tile / tiles_k, tj = tile - ti * tiles_k;
    const int64_t r0 = ti * bm, c0 = tj * bk;
    const int n = bm * bk;
    uint32_t m = 0;
    for (int idx = t; idx < n; idx += kGenThreads) {
        const int64_t r = r0 + idx / bk, c = c0 + idx % bk;
        if (r < M && c < K) {
            const uint32_t a = f2u(load_f32(w, r * sxm + c * sxn, dtype)) & 0x7FFFFFFFu;
            m = umax(m, (MODE == 1 && a > 0x7F800000u) ? 0u : a);      // Triton's max skips NaN, torch's amax hands it on
        }
    }
    m = wave_max(m);
    if ((t & (kWave - 1)) == 0) wave_amax[t >> 6] = m;
    __syncthreads();
    m = umax(umax(wave_amax[0], wave_amax[1]), umax(wave_amax[2], wave_amax[3]));
    const float amax = u2f(m);
    float s, y;
    if (MODE == 0) {
        s = amax / kFp8Max;
        y = 0.0f;
    } else if (MODE == 1) {
        const float absmax = amax > 1e-10f ? amax : 1e-10f;
        s = absmax / kFp8Max;
        y = 1.0f / s;
    } else {
        s = m >= 0x7F800000u ? amax : ceil_pow2_scale((amax > 1e-4f ? amax : 1e-4f) / kFp8Max);   // inf / NaN stay
        y = 1.0f / s;
    }
    if (t == 0) scale[tile] = s;
    const bool zero_tile = MODE == 0 && !(amax > 0.0f) && amax == amax;
    for (int idx = t; idx < n; idx += kGenThreads) {
        const int64_t r = r0 + idx / bk, c = c0 + idx % bk;
        if (r < M && c < K) {
            uint32_t code;
            if (zero_tile) code = 0xFFu;
            else {
                const float x = load_f32(w, r * sxm + c * sxn, dtype);
                float v = MODE != 0 ? x * y : x / s;
                if (MODE == 0) v = clamp_keep_nan(v, -kFp8Max, kFp8Max);                              // torch.clamp
                else if (MODE == 1) v = __builtin_fminf(__builtin_fmaxf(v, -kFp8Max), kFp8Max);        // tl.clamp: NaN -> -448
                code = sw_e4m3fn(v);
            }
            q[r * ldq + c] = (uint8_t)code;
        }
    }
}

// ---- per-tensor / per-channel (reference: tools/convert_hf_to_fp8.py:73-86,
//      quantizer_fp8.py:153-158) ---------------------------------------------------------------
// pass 1: amax per row (per_channel) or per tensor (atomic max on the float bit pattern)
__global__ __launch_bounds__(256) void fp8_row_amax_kernel(const void* __restrict__ w, int dtype, int64_t ldw,
                                                           int64_t K, uint32_t* __restrict__ amax_bits,
                                                           int per_channel) {
    __shared__ uint32_t wave_amax[4];
    const int t = threadIdx.x;
    const int64_t r = blockIdx.x;
    uint32_t m = 0;
    for (int64_t c = t; c < K; c += 256) m = umax(m, f2u(load_f32(w, r * ldw + c, dtype)) & 0x7FFFFFFFu);
    m = wave_max(m);
    if ((t & 63) == 0) wave_amax[t >> 6] = m;
    __syncthreads();
    if (t == 0) {
        m = umax(umax(wave_amax[0], wave_amax[1]), umax(wave_amax[2], wave_amax[3]));
        if (per_channel) amax_bits[r] = m;
        else atomicMax(amax_bits, m);
    }
}
// pass 2: scale = max(amax, floor)/448 ; q = e4m3(clamp(w/scale)).  With one scale for the whole
// tensor the quotient is first rounded to the weight's dtype (torch keeps `weight / zero_dim_scale`
// in the weight's dtype).
__global__ __launch_bounds__(256) void fp8_row_quant_kernel(const void* __restrict__ w, int dtype, int64_t ldw,
                                                            int64_t K, const uint32_t* __restrict__ amax_bits,
                                                            float floor_v, int per_channel,
                                                            uint8_t* __restrict__ q, float* __restrict__ scale) {
    const int t = threadIdx.x;
    const int64_t r = blockIdx.x;
    float amax = u2f(per_channel ? amax_bits[r] : amax_bits[0]);
    if (amax < floor_v) amax = floor_v;
    const float s = amax / kFp8Max;
    if (t == 0 && (per_channel || r == 0)) scale[per_channel ? r : 0] = s;
    for (int64_t c = t; c < K; c += 256) {
        float v = load_f32(w, r * ldw + c, dtype) / s;
        if (!per_channel) v = round_to_dtype(v, dtype);
        v = clamp_keep_nan(v, -kFp8Max, kFp8Max);
        q[r * K + c] = (uint8_t)sw_e4m3fn(v);
    }
}
// bf16 fast paths of the two.  The quotient x / s is the exact one (shared-divisor sequence, which keeps the sign of a
// -0 numerator; the division itself when s leaves the guarded range).
//
// per channel: a row lives in the registers of ROWLANES lanes (up to 8 sixteen-byte units each), so it is read once:
// amax across the lanes, one scale, codes.  ROWLANES = 64: four rows per workgroup, no LDS; 256: one row.
template <int ROWLANES, int F16>
__global__ __launch_bounds__(256) void fp8_channel_bf16_kernel(const uint16_t* __restrict__ w, int64_t ldw, int64_t K,
                                                               int64_t M, float floor_v, uint8_t* __restrict__ q,
                                                               float* __restrict__ scale, int chunk) {
    __shared__ uint32_t wave_amax[4];
    constexpr int kRows = 256 / ROWLANES, kMaxUnits = 8;
    const int t = threadIdx.x, lane = t % ROWLANES;
    // an XCD takes runs of consecutive rows, as the flat kernels take runs of consecutive blocks
    const int64_t row = xcd_chunked_block(chunk) * kRows + t / ROWLANES;
    const int64_t units = K / 8;
    const bool row_ok = row < M;
    const uint16_t* __restrict__ src = w + (row_ok ? row : M - 1) * ldw;
    u32x4 v[kMaxUnits];
    uint32_t m2 = 0;
#pragma unroll
    for (int u = 0; u < kMaxUnits; u++) {
        const int64_t unit = lane + (int64_t)u * ROWLANES;
        v[u] = unit < units ? ld16(src + unit * 8) : u32x4{0u, 0u, 0u, 0u};
        m2 = max2_u16(m2, max2_u16(max2_u16(abs2(v[u].x), abs2(v[u].y)), max2_u16(abs2(v[u].z), abs2(v[u].w))));
    }
    uint32_t m = wave_max(hmax_u16(m2));
    if (ROWLANES == 256) {
        if ((t & 63) == 0) wave_amax[t >> 6] = m;
        __syncthreads();
        m = umax(umax(wave_amax[0], wave_amax[1]), umax(wave_amax[2], wave_amax[3]));
    }
    float amax = elem_lo<F16>(m);
    if (amax < floor_v) amax = floor_v;
    const float s = amax / kFp8Max, y = 1.0f / s;
    const bool fast_div = shared_div_ok(s);
    // the hardware conversion takes finite quotients: an infinity or a NaN in the row, or a zero scale (fp16 has no
    // 1e-12 floor, so a row of zeros divides 0 by 0), goes through the software conversion
    const bool plain = m < (F16 ? 0x7C00u : 0x7F80u) && s > 0.0f;
    if (!row_ok) return;
    if (lane == 0) scale[row] = s;
#pragma unroll
    for (int u = 0; u < kMaxUnits; u++) {
        const int64_t unit = lane + (int64_t)u * ROWLANES;
        if (unit >= units) continue;
        float f[8] = {elem_lo<F16>(v[u].x), elem_hi<F16>(v[u].x), elem_lo<F16>(v[u].y), elem_hi<F16>(v[u].y),
                      elem_lo<F16>(v[u].z), elem_hi<F16>(v[u].z), elem_lo<F16>(v[u].w), elem_hi<F16>(v[u].w)};
#pragma unroll
        for (int j = 0; j < 8; j++) f[j] = fast_div ? div_by_shared(f[j], s, y) : f[j] / s;
        u32x2 o;
        if (plain) {
            o.x = hw_e4m3x4(f[0], f[1], f[2], f[3]);
            o.y = hw_e4m3x4(f[4], f[5], f[6], f[7]);
        } else {                                  // inf / NaN in the row: clamp and convert in software
            uint32_t c[8];
#pragma unroll
            for (int j = 0; j < 8; j++) c[j] = sw_e4m3fn(clamp_keep_nan(f[j], -kFp8Max, kFp8Max));
            o.x = c[0] | (c[1] << 8) | (c[2] << 16) | (c[3] << 24);
            o.y = c[4] | (c[5] << 8) | (c[6] << 16) | (c[7] << 24);
        }
        st8(q + row * K + unit * 8, o);
    }
}

// per tensor, pass 1: every workgroup strides over 8 KiB pieces and ends with one atomic max on the bf16 amax
__global__ __launch_bounds__(256) void fp8_tensor_amax_bf16_kernel(const uint16_t* __restrict__ w, int64_t units,
                                                                   uint32_t* __restrict__ amax_bits) {
    __shared__ uint32_t wave_amax[4];
    const int t = threadIdx.x;
    uint32_t m2 = 0;
    for (int64_t base = (int64_t)blockIdx.x * 512; base < units; base += (int64_t)gridDim.x * 512) {
        const int64_t a = base + t, b = base + 256 + t;
        const u32x4 va = a < units ? ld16(w + a * 8) : u32x4{0u, 0u, 0u, 0u};
        const u32x4 vb = b < units ? ld16(w + b * 8) : u32x4{0u, 0u, 0u, 0u};
        m2 = max2_u16(m2, max2_u16(max2_u16(abs2(va.x), abs2(va.y)), max2_u16(abs2(va.z), abs2(va.w))));
        m2 = max2_u16(m2, max2_u16(max2_u16(abs2(vb.x), abs2(vb.y)), max2_u16(abs2(vb.z), abs2(vb.w))));
    }
    const uint32_t m = wave_max(hmax_u16(m2));
    if ((t & 63) == 0) wave_amax[t >> 6] = m;
    __syncthreads();
    if (t == 0) atomicMax(amax_bits, umax(umax(wave_amax[0], wave_amax[1]), umax(wave_amax[2], wave_amax[3])) << 16);
}
// per tensor, pass 2: flat.  torch divides by a zero-dimensional scale in the weight's dtype, so the quotient is
// rounded to bf16 before it is clamped and converted.
__global__ __launch_bounds__(256) void fp8_tensor_quant_bf16_kernel(const uint16_t* __restrict__ w,
                                                                    const uint32_t* __restrict__ amax_bits, float floor_v,
                                                                    uint8_t* __restrict__ q, float* __restrict__ scale,
                                                                    int64_t units, int chunk) {
    const int64_t base = xcd_chunked_block(chunk) * 512 + threadIdx.x;
    u32x4 v[2];
#pragma unroll
    for (int i = 0; i < 2; i++) {
        const int64_t unit = base + i * 256;
        v[i] = ld16(w + (unit < units ? unit : units - 1) * 8);
    }
    const uint32_t abits = amax_bits[0];
    float amax = u2f(abits);
    if (amax < floor_v) amax = floor_v;
    const float s = amax / kFp8Max, y = 1.0f / s;
    const bool fast_div = shared_div_ok(s);
    if (base == 0) scale[0] = s;
#pragma unroll
    for (int i = 0; i < 2; i++) {
        const int64_t unit = base + i * 256;
        float f[8] = {bf16_lo(v[i].x), bf16_hi(v[i].x), bf16_lo(v[i].y), bf16_hi(v[i].y),
                      bf16_lo(v[i].z), bf16_hi(v[i].z), bf16_lo(v[i].w), bf16_hi(v[i].w)};
#pragma unroll
        for (int j = 0; j < 8; j++) f[j] = fast_div ? div_by_shared(f[j], s, y) : f[j] / s;
#pragma unroll
        for (int j = 0; j < 8; j += 2) {           // the rounding to bf16
            const uint32_t p = hw_bf16x2(f[j], f[j + 1]);
            f[j] = bf16_lo(p);
            f[j + 1] = bf16_hi(p);
        }
        u32x2 o;
        if (abits < 0x7F800000u) {
            o.x = hw_e4m3x4(f[0], f[1], f[2], f[3]);
            o.y = hw_e4m3x4(f[4], f[5], f[6], f[7]);
        } else {
            uint32_t c[8];
#pragma unroll
            for (int j = 0; j < 8; j++) c[j] = sw_e4m3fn(clamp_keep_nan(f[j], -kFp8Max, kFp8Max));
            o.x = c[0] | (c[1] << 8) | (c[2] << 16) | (c[3] << 24);
            o.y = c[4] | (c[5] << 8) | (c[6] << 16) | (c[7] << 24);
        }
        if (unit < units) st8(q + unit * 8, o);
    }
}

__global__ void fill_u32_kernel(uint32_t* p, uint32_t v, int n) {
    int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) p[i] = v;
}

// ---- dequant ----------------------------------------------------------------------------------
// Fast path: N % 8 == 0, block a power of two >= 8, aligned pointers.  The tensor is a flat run of 8-code
// units; each lane turns kDqUnroll units (8-byte loads, kDqThreads units apart) into bf16 (16-byte stores), so a
// wavefront writes 1 KiB of consecutive output per store instruction.  Row and column of a unit come from a multiply-high
// division by the row length (exact for every 32-bit unit index), not from an integer divide.
constexpr int kDqThreads = 256;
// (units per lane, alternating runs, one / two / four: 6.53-6.57 / 6.47-6.50 / 6.23-6.27 TB/s on 96 DeepSeek-V3 expert
// matrices, 6.21-6.23 / 6.17-6.22 / 6.11-6.14 on eight [16384, 7168] tensors)
#ifndef MQ_DQ_UNROLL
#define MQ_DQ_UNROLL 1
#endif
constexpr int kDqUnroll = MQ_DQ_UNROLL;
struct DequantJob {
    const uint8_t* x;
    const float* s;
    uint16_t* y;
    uint32_t units;          // M * N / 8
    uint32_t units_per_row;  // N / 8
    uint32_t magic, shift;   // floor(n / units_per_row) == (t + ((n - t) >> 1)) >> shift, t = mulhi(magic, n)
    int32_t block_shift;     // log2(block)
    int32_t tiles_n;
};
struct DequantTable {
    int32_t n;
    int32_t max_blocks;
    int32_t chunk;           // blocks per XCD chunk (xcd_chunked_block); max_blocks is a multiple of 8 * chunk
    int32_t pad;
    DequantJob job[kMaxGroup];
};

__global__ __launch_bounds__(kDqThreads) void fp8_dequant_kernel(const DequantTable tab) {
    const DequantJob& job = tab.job[blockIdx.y];
    const int64_t base64 = xcd_chunked_block(tab.chunk) * (kDqThreads * kDqUnroll);
    if (base64 >= job.units) return;
    const uint32_t base = (uint32_t)base64;
    u32x2 in[kDqUnroll];
    float scale[kDqUnroll];
    // every load is issued before the first use: a lane past the end reads the workgroup's first unit again (always
    // there) and stores nothing
#pragma unroll
    for (int i = 0; i < kDqUnroll; i++) {
        const uint32_t unit = base + i * kDqThreads + threadIdx.x;
        const uint32_t uc = unit < job.units ? unit : base;
        // an ordinary (cached) load: with the non-temporal hint the 8-byte code loads of this kernel, which writes
        // twice what it reads, ran 2 % slower (6.36 against 6.50 TB/s on 36 tensors of [4096, 2560]); the 4- and
        // 16-byte code loads of the other unpacking kernels measured the other way round and keep the hint
        in[i] = *reinterpret_cast<const u32x2*>(job.x + (int64_t)uc * 8);
        const uint32_t th = __umulhi(job.magic, uc);
        const uint32_t r = (th + ((uc - th) >> 1)) >> job.shift;
        const uint32_t c = (uc - r * job.units_per_row) * 8u;
        scale[i] = job.s[(int64_t)(r >> job.block_shift) * job.tiles_n + (c >> job.block_shift)];
    }
    __builtin_amdgcn_sched_barrier(0);      // (and the scheduler keeps the first unit's arithmetic below the last load)
#pragma unroll
    for (int i = 0; i < kDqUnroll; i++) {
        const uint32_t unit = base + i * kDqThreads + threadIdx.x;
        if (unit >= job.units) continue;
        const float sc = scale[i];
        const uint32_t wd[2] = {in[i].x, in[i].y};
        uint32_t o[4];
        // a NaN code (0x7F / 0xFF) or a non-finite scale must give the canonical bf16 NaN 0x7FC0
        bool special = (f2u(sc) & 0x7F800000u) == 0x7F800000u;
#pragma unroll
        for (int k = 0; k < 2; k++) special |= (((wd[k] & 0x7F7F7F7Fu) + 0x01010101u) & 0x80808080u) != 0u;
        if (!special) {
#pragma unroll
            for (int k = 0; k < 2; k++) {
                const f32x2 a = hw_e4m3x2_decode<false>(wd[k]);
                const f32x2 b = hw_e4m3x2_decode<true>(wd[k]);
                o[2 * k] = hw_bf16x2(a.x * sc, a.y * sc);
                o[2 * k + 1] = hw_bf16x2(b.x * sc, b.y * sc);
            }
        } else {
#pragma unroll
            for (int k = 0; k < 2; k++) {
                uint32_t h[4];
#pragma unroll
                for (int b = 0; b < 4; b++) h[b] = sw_bf16(sw_e4m3fn_decode((wd[k] >> (8 * b)) & 0xFFu) * sc);
                o[2 * k] = h[0] | (h[1] << 16);
                o[2 * k + 1] = h[2] | (h[3] << 16);
            }
        }
        st16(job.y + (int64_t)unit * 8, u32x4{o[0], o[1], o[2], o[3]});
    }
}

__global__ __launch_bounds__(256) void fp8_dequant_generic_kernel(const uint8_t* __restrict__ x,
                                                                  const float* __restrict__ s,
                                                                  uint16_t* __restrict__ y, int64_t M, int64_t N,
                                                                  int block, int tiles_n) {
    const int64_t total = M * N;
    const int64_t stride = (int64_t)gridDim.x * blockDim.x;
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += stride) {
        const int64_t r = i / N, c = i - r * N;
        y[i] = (uint16_t)sw_bf16(sw_e4m3fn_decode(x[i]) * s[(r / block) * tiles_n + c / block]);
    }
}

}  // namespace mq

using namespace mq;

bool mq_fp8_tile_fast_ok(const void* w, int dtype, int64_t sxm, int64_t sxn, const void* q, int64_t M, int64_t K,
                         int bm, int bk) {
    // rows and columns below 2^24: a lane addresses its tile with 32-bit byte offsets from the tile's base
    return (dtype == MQ_BF16 || dtype == MQ_F16) && bm == kTile && bk == kTile && sxn == 1 && (K % 8) == 0 && (sxm % 8) == 0 &&
           ((uintptr_t)w % 16) == 0 && ((uintptr_t)q % 8) == 0 && M <= 0x7FFFFFFF && K < (1 << 24) && sxm > 0 &&
           sxm < (1 << 24);
}

// fills the division constants of a descriptor whose w, q, scale, ldw, M, K and row blocks are set; returns its tile count
int64_t mq_fp8_tile_job_finish(TileJob& j) {
    const uint32_t tiles_k = (uint32_t)((j.K + kTile - 1) / kTile);
    uint32_t shift_k = 0, shift_b = 0;
    if (tiles_k > 1) tile_div_magic(tiles_k, j.magic_k, shift_k);
    if (j.tiles_per_block > 1) tile_div_magic((uint32_t)j.tiles_per_block, j.magic_b, shift_b);
    j.shifts = shift_k | (shift_b << 8);
    return (int64_t)((j.M + kTile - 1) / kTile) * tiles_k;
}

template <class Table>
static void tile_launch(int mode, bool f16, dim3 grid, hipStream_t st, const Table& tab) {
    const dim3 blk(kTileThreads);
    if (f16) {
        if (mode == 0) hipLaunchKernelGGL((fp8_block128_kernel<0, Table, 1>), grid, blk, 0, st, tab);
        else if (mode == 1) hipLaunchKernelGGL((fp8_block128_kernel<1, Table, 1>), grid, blk, 0, st, tab);
        else hipLaunchKernelGGL((fp8_block128_kernel<2, Table, 1>), grid, blk, 0, st, tab);
    } else {
        if (mode == 0) hipLaunchKernelGGL((fp8_block128_kernel<0, Table, 0>), grid, blk, 0, st, tab);
        else if (mode == 1) hipLaunchKernelGGL((fp8_block128_kernel<1, Table, 0>), grid, blk, 0, st, tab);
        else hipLaunchKernelGGL((fp8_block128_kernel<2, Table, 0>), grid, blk, 0, st, tab);
    }
}

// n finished descriptors in device memory, all of one 16-bit dtype; max_tiles: the largest tensor's tile count
int mq_fp8_tile_launch_table(int mode, int dtype, const TileJob* device_jobs, int n, int64_t max_tiles, hipStream_t st) {
    if (n == 0 || max_tiles == 0) return MQ_OK;
    const int64_t gx = xcd_grid(max_tiles);
    if (gx >= 0x7FFFFFF0) return mq_fail(MQ_ERR_ARG, "too many tiles");
    tile_launch(mode, dtype == MQ_F16, dim3((unsigned)gx, (unsigned)n), st, TileRef{device_jobs});
    return mq_check_launch("fp8 block quant");
}

// tab.job[i] filled by the caller (w, q, scale, ldw, M, K, row blocks), all of one 16-bit dtype; fills the division
// constants and `end`, launches
int mq_fp8_tile_launch_group(int mode, int dtype, TileTable& tab, hipStream_t st) {
    int64_t tiles = 0;
    for (int i = 0; i < tab.n; i++) {
        tiles += mq_fp8_tile_job_finish(tab.job[i]);
        if (tiles >= 0x7FFFFFF0) return mq_fail(MQ_ERR_ARG, "too many tiles");
        tab.end[i] = (int32_t)tiles;
    }
    if (tiles == 0) return MQ_OK;
    seal_table(tab);
    tile_launch(mode, dtype == MQ_F16, dim3((unsigned)xcd_grid(tiles)), st, tab);
    return mq_check_launch("fp8 block quant");
}

static int fp8_block_launch(int mode, const void* w, int dtype, int64_t sxm, int64_t sxn, void* q, float* scale,
                            int64_t M, int64_t K, int bm, int bk, hipStream_t stream) {
    if ((!w || !q || !scale) && M != 0 && K != 0) return mq_fail(MQ_ERR_ARG, "null pointer");
    if (M < 0 || K < 0 || bm <= 0 || bk <= 0) return mq_fail(MQ_ERR_ARG, "bad shape or block size");
    if (dtype < MQ_BF16 || dtype > MQ_F32) return mq_fail(MQ_ERR_ARG, "unsupported dtype");
    if (M == 0 || K == 0) return MQ_OK;
    if (mq_fp8_tile_fast_ok(w, dtype, sxm, sxn, q, M, K, bm, bk)) {
        TileTable tab{};
        tab.n = 1;
        tab.job[0] = TileJob{w, q, scale, (int32_t)sxm, (int32_t)M, (int32_t)K, 0, 0, 0, 0, 0};
        return mq_fp8_tile_launch_group(mode, dtype, tab, stream);
    }
    const int64_t tiles_m = (M + bm - 1) / bm, tiles_k = (K + bk - 1) / bk;
    const int64_t tiles = tiles_m * tiles_k;
    if (tiles > 0x7FFFFFFF || tiles_k > 0x7FFFFFFF) return mq_fail(MQ_ERR_ARG, "too many tiles");
    if ((int64_t)bm * bk > (1 << 24)) return mq_fail(MQ_ERR_ARG, "block too large");
    dim3 grid((unsigned)tiles), blk(kGenThreads);
    if (mode == 0)
        hipLaunchKernelGGL(fp8_block_generic_kernel<0>, grid, blk, 0, stream, w, dtype, sxm, sxn, (uint8_t*)q, K, scale,
                           M, K, bm, bk, (int)tiles_k);
    else if (mode == 1)
        hipLaunchKernelGGL(fp8_block_generic_kernel<1>, grid, blk, 0, stream, w, dtype, sxm, sxn, (uint8_t*)q, K, scale,
                           M, K, bm, bk, (int)tiles_k);
    else
        hipLaunchKernelGGL(fp8_block_generic_kernel<2>, grid, blk, 0, stream, w, dtype, sxm, sxn, (uint8_t*)q, K, scale,
                           M, K, bm, bk, (int)tiles_k);
    return mq_check_launch("fp8 block quant");
}

extern "C" int mq_fp8_block_quant(const void* w, int dtype, int64_t ldw, void* q, float* scale, int64_t M, int64_t K,
                                  int block_m, int block_k, void* stream) {
    return fp8_block_launch(0, w, dtype, ldw, 1, q, scale, M, K, block_m, block_k, (hipStream_t)stream);
}

extern "C" int mq_fp8_blockwise_cast(const void* x, int dtype, int64_t stride_m, int64_t stride_n, void* y, float* s,
                                     int64_t M, int64_t N, int block_m, int block_n, void* stream) {
    return fp8_block_launch(1, x, dtype, stride_m, stride_n, y, s, M, N, block_m, block_n, (hipStream_t)stream);
}

extern "C" int mq_fp8_block_quant_pow2(const void* w, int dtype, int64_t ldw, void* q, float* scale, int64_t M, int64_t K,
                                       void* stream) {
    return fp8_block_launch(2, w, dtype, ldw, 1, q, scale, M, K, kTile, kTile, (hipStream_t)stream);
}

static int fp8_scaled_quant(const void* w, int dtype, int64_t ldw, void* q, float* scale, void* amax_ws, int64_t M,
                            int64_t K, int per_channel, float floor_in_dtype, void* stream) {
    if ((!w || !q) && M != 0 && K != 0) return mq_fail(MQ_ERR_ARG, "null pointer");
    if ((!scale || !amax_ws) && (M != 0 || !per_channel)) return mq_fail(MQ_ERR_ARG, "null pointer");
    if (dtype < MQ_BF16 || dtype > MQ_F32 || M < 0 || K < 0) return mq_fail(MQ_ERR_ARG, "bad argument");
    if (M == 0 || K == 0) return MQ_OK;
    if (M > 0x7FFFFFFF) return mq_fail(MQ_ERR_ARG, "too many rows");
    hipStream_t st = (hipStream_t)stream;
    const bool aligned16 = (dtype == MQ_BF16 || dtype == MQ_F16) && K % 8 == 0 && ldw % 8 == 0 && ((uintptr_t)w % 16) == 0 &&
                           ((uintptr_t)q % 8) == 0;
    const bool aligned = aligned16 && dtype == MQ_BF16;
    if (aligned16 && per_channel && K / 8 <= 2048) {
        const uint16_t* wi = (const uint16_t*)w;
        const bool four_rows = K / 8 <= 256;
        const int64_t blocks = four_rows ? (M + 3) / 4 : M;
        const int chunk = (int)flat_chunk(blocks);
        const dim3 grid((unsigned)flat_padded(blocks, chunk)), blk(256);
        if (dtype == MQ_F16) {
            if (four_rows) hipLaunchKernelGGL((fp8_channel_bf16_kernel<64, 1>), grid, blk, 0, st, wi, ldw, K, M, floor_in_dtype, (uint8_t*)q, scale, chunk);
            else hipLaunchKernelGGL((fp8_channel_bf16_kernel<256, 1>), grid, blk, 0, st, wi, ldw, K, M, floor_in_dtype, (uint8_t*)q, scale, chunk);
        } else {
            if (four_rows) hipLaunchKernelGGL((fp8_channel_bf16_kernel<64, 0>), grid, blk, 0, st, wi, ldw, K, M, floor_in_dtype, (uint8_t*)q, scale, chunk);
            else hipLaunchKernelGGL((fp8_channel_bf16_kernel<256, 0>), grid, blk, 0, st, wi, ldw, K, M, floor_in_dtype, (uint8_t*)q, scale, chunk);
        }
        return mq_check_launch("fp8 scaled quant");
    }
    if (aligned && !per_channel && ldw == K && M * (K / 8) < (1ll << 38)) {
        const int64_t units = M * (K / 8);
        int64_t blocks = (units + 511) / 512;
        hipLaunchKernelGGL(fill_u32_kernel, dim3(1), dim3(64), 0, st, (uint32_t*)amax_ws, 0u, 1);
        hipLaunchKernelGGL(fp8_tensor_amax_bf16_kernel, dim3((unsigned)(blocks < 2048 ? blocks : 2048)), dim3(256), 0, st,
                           (const uint16_t*)w, units, (uint32_t*)amax_ws);
        const int chunk = (int)flat_chunk(blocks);
        blocks = flat_padded(blocks, chunk);
        hipLaunchKernelGGL(fp8_tensor_quant_bf16_kernel, dim3((unsigned)blocks), dim3(256), 0, st, (const uint16_t*)w,
                           (const uint32_t*)amax_ws, floor_in_dtype, (uint8_t*)q, scale, units, chunk);
        return mq_check_launch("fp8 scaled quant");
    }
    if (!per_channel) hipLaunchKernelGGL(fill_u32_kernel, dim3(1), dim3(64), 0, st, (uint32_t*)amax_ws, 0u, 1);
    hipLaunchKernelGGL(fp8_row_amax_kernel, dim3((unsigned)M), dim3(256), 0, st, w, dtype, ldw, K,
                       (uint32_t*)amax_ws, per_channel);
    hipLaunchKernelGGL(fp8_row_quant_kernel, dim3((unsigned)M), dim3(256), 0, st, w, dtype, ldw, K,
                       (const uint32_t*)amax_ws, floor_in_dtype, per_channel, (uint8_t*)q, scale);
    return mq_check_launch("fp8 scaled quant");
}

extern "C" int mq_fp8_scaled_quant(const void* w, int dtype, int64_t ldw, void* q, float* scale, void* amax_ws,
                                   int64_t M, int64_t K, int per_channel, float floor_in_dtype, void* stream) {
    return fp8_scaled_quant(w, dtype, ldw, q, scale, amax_ws, M, K, per_channel, floor_in_dtype, stream);
}

// ---- the same quantizer for callers that cannot allocate ------------------------------------------------------
// The amax workspace (one word per tensor, or one per row with per-channel scales) lives in a file-scope device
// array instead of coming from the caller.  `scratch` names the array in host code only as a symbol: its address in
// device memory differs per GPU and is looked up once per device with hipGetSymbolAddress; kernels and fills get
// that address, never the symbol.
static __device__ __align__(256) uint32_t scratch[MQ_FP8_STATIC_MAX_ROWS];
static constexpr int kMaxDevices = 64;
static std::mutex g_scratch_lock;
static uint32_t* g_scratch_ptr[kMaxDevices];      // device address of `scratch` on each GPU, 0 until first use there
static int64_t g_scratch_next[kMaxDevices];       // first word of the array that the next call on that GPU takes

// `words` words of `scratch` on the current device for one call, or null with the error text set.  Calls take
// consecutive pieces of the array (whole 256-byte lines), starting over at its beginning when a piece no longer fits:
// two calls that are in flight together -- on two streams, from two host threads -- only share words when the pieces
// handed out between them add up to more than the array.
static uint32_t* scratch_on_current_device(int64_t words) {
    int dev = -1;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess || dev < 0 || dev >= kMaxDevices) {
        mq_fail(MQ_ERR_HIP, "mq_fp8_scaled_quant_static: no current device (or a device index above 63)");
        return nullptr;
    }
    std::lock_guard<std::mutex> hold(g_scratch_lock);
    if (!g_scratch_ptr[dev]) {
        void* p = nullptr;
        e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
        if (e != hipSuccess || !p) {
            mq_fail(MQ_ERR_HIP, "mq_fp8_scaled_quant_static: hipGetSymbolAddress failed for the amax workspace");
            return nullptr;
        }
        g_scratch_ptr[dev] = (uint32_t*)p;
    }
    const int64_t piece = (words + 63) / 64 * 64;
    if (g_scratch_next[dev] + piece > MQ_FP8_STATIC_MAX_ROWS) g_scratch_next[dev] = 0;
    uint32_t* at = g_scratch_ptr[dev] + g_scratch_next[dev];
    g_scratch_next[dev] += piece;
    return at;
}

extern "C" int mq_fp8_scaled_quant_static(const void* w, int dtype, int64_t ldw, void* q, float* scale, int64_t M,
                                          int64_t K, int per_channel, float floor_in_dtype, void* stream) {
    if (per_channel && M > MQ_FP8_STATIC_MAX_ROWS)
        return mq_fail(MQ_ERR_ARG, "mq_fp8_scaled_quant_static: per-channel scales take at most MQ_FP8_STATIC_MAX_ROWS "
                                   "(262144) rows; use mq_fp8_scaled_quant with a workspace of its own");
    uint32_t* ws = scratch_on_current_device(per_channel && M > 0 ? M : 1);
    if (!ws) return MQ_ERR_HIP;
    return fp8_scaled_quant(w, dtype, ldw, q, scale, ws, M, K, per_channel, floor_in_dtype, stream);
}

bool mq_fp8_dequant_fast_ok(const void* x, const void* y, int64_t M, int64_t N, int block) {
    const bool pow2 = block >= 8 && (block & (block - 1)) == 0;
    return (N % 8) == 0 && N >= 16 && pow2 && ((uintptr_t)x % 8) == 0 && ((uintptr_t)y % 16) == 0 &&
           M * (N / 8) < 0xFFFFFFF0ll;
}

int mq_fp8_dequant_launch_group(const MqDequantArgs* a, int n, hipStream_t st) {
    DequantTable tab{};
    tab.n = n;
    int64_t mx = 0;
    for (int i = 0; i < n; i++) {
        DequantJob& j = tab.job[i];
        j.x = (const uint8_t*)a[i].x;
        j.s = a[i].s;
        j.y = (uint16_t*)a[i].y;
        j.units = (uint32_t)(a[i].M * (a[i].N / 8));
        const uint32_t d = (uint32_t)(a[i].N / 8);   // >= 2
        j.units_per_row = d;
        uint32_t l = 0;
        while ((1ull << l) < d) l++;                 // ceil(log2 d) >= 1
        j.magic = (uint32_t)((((1ull << l) - d) << 32) / d + 1);
        j.shift = l - 1;
        int bs = 0;
        while ((1 << bs) < a[i].block) bs++;
        j.block_shift = bs;
        j.tiles_n = (int32_t)((a[i].N + a[i].block - 1) / a[i].block);
        const int64_t b = ((int64_t)j.units + kDqThreads * kDqUnroll - 1) / (kDqThreads * kDqUnroll);
        if (b > mx) mx = b;
    }
    if (mx == 0) return MQ_OK;
    const int64_t chunk = flat_chunk(mx);
    mx = flat_padded(mx, chunk);
    tab.chunk = (int32_t)chunk;
    tab.max_blocks = (int32_t)mx;
    hipLaunchKernelGGL(fp8_dequant_kernel, dim3((unsigned)mx, (unsigned)n), dim3(kDqThreads), 0, st, tab);
    return mq_check_launch("fp8 block dequant");
}

// One lane per output word.  ROW_MAJOR = false: DeepGEMM's layout [batch][ceil(kb/4)][align(mn,4)], consecutive lanes
// take consecutive rows; true: the same words as a contiguous [batch][mn][ceil(kb/4)] array (what `.contiguous()` makes
// of the transposed view, e.g. inside a flattened transport payload).
template <bool ROW_MAJOR>
__global__ __launch_bounds__(256) void ue8m0_pack_scales_kernel(const float* __restrict__ sf, uint32_t* __restrict__ out,
                                                                int64_t total, int64_t mn, int64_t amn, int64_t kb,
                                                                int64_t kw, int64_t tile_rows) {
    const int64_t stride = (int64_t)gridDim.x * blockDim.x;
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += stride) {
        int64_t r, j, b;
        if (ROW_MAJOR) {
            j = i % kw;
            r = (i / kw) % mn;
            b = i / (kw * mn);
        } else {
            r = i % amn;
            j = (i / amn) % kw;
            b = i / (amn * kw);
        }
        uint32_t word = 0;
        if (r < mn) {
            const float* row = sf + (b * tile_rows + r / 128) * kb;
#pragma unroll
            for (int e = 0; e < 4; e++)
                if (4 * j + e < kb) word |= ((__float_as_uint(row[4 * j + e]) >> 23) & 0xFFu) << (8 * e);
        }
        out[i] = word;
    }
}

extern "C" int mq_ue8m0_pack_scales(const float* sf, int32_t* out, int64_t batch, int64_t mn, int64_t kb,
                                    int64_t tile_rows, int row_major, void* stream) {
    if ((!sf || !out) && batch != 0 && mn != 0 && kb != 0) return mq_fail(MQ_ERR_ARG, "null pointer");
    if (batch < 0 || mn < 0 || kb < 0 || tile_rows < (mn + 127) / 128) return mq_fail(MQ_ERR_ARG, "bad shape");
    const int64_t amn = (mn + 3) / 4 * 4, kw = (kb + 3) / 4, total = batch * kw * (row_major ? mn : amn);
    if (total == 0) return MQ_OK;
    int64_t blocks = (total + 255) / 256;
    if (blocks > mq_grid_cap()) blocks = mq_grid_cap();
    const dim3 grid((unsigned)blocks), blk(256);
    if (row_major)
        hipLaunchKernelGGL(ue8m0_pack_scales_kernel<true>, grid, blk, 0, (hipStream_t)stream, sf, (uint32_t*)out, total, mn, amn, kb, kw, tile_rows);
    else
        hipLaunchKernelGGL(ue8m0_pack_scales_kernel<false>, grid, blk, 0, (hipStream_t)stream, sf, (uint32_t*)out, total, mn, amn, kb, kw, tile_rows);
    return mq_check_launch("ue8m0 scale pack");
}

extern "C" int mq_fp8_block_dequant(const void* x, const float* s, void* y, int64_t M, int64_t N, int block,
                                    void* stream) {
    if ((!x || !s || !y) && M != 0 && N != 0) return mq_fail(MQ_ERR_ARG, "null pointer");
    if (M < 0 || N < 0 || block <= 0) return mq_fail(MQ_ERR_ARG, "bad shape or block size");
    if (M == 0 || N == 0) return MQ_OK;
    const int64_t tiles_n = (N + block - 1) / block;
    if (tiles_n > 0x7FFFFFFF) return mq_fail(MQ_ERR_ARG, "too many tiles");
    hipStream_t st = (hipStream_t)stream;
    if (mq_fp8_dequant_fast_ok(x, y, M, N, block)) {
        MqDequantArgs a{x, s, y, M, N, block};
        return mq_fp8_dequant_launch_group(&a, 1, st);
    }
    int64_t blocks = (M * N + 255) / 256;
    if (blocks > mq_grid_cap()) blocks = mq_grid_cap();
    hipLaunchKernelGGL(fp8_dequant_generic_kernel, dim3((unsigned)blocks), dim3(256), 0, st, (const uint8_t*)x, s,
                       (uint16_t*)y, M, N, block, (int)tiles_n);
    return mq_check_launch("fp8 block dequant");
}
