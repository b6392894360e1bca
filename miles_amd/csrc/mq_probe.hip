// Streaming probes: kernels that only move bytes, in the access shapes the quantizers use.  They exist to calibrate what
// a shape can reach on a given GPU (bench.py --stream-ceilings), next to the plain copy; they are built into
// libmq_probes.so, not into the product library.  All read `src` and write `dst` with non-temporal accesses; the
// values written are meaningless.
#include <stdio.h>

#include "mq_common.hpp"
#include "mq_group.hpp"
#include "mq_probes_internal.hpp"

static thread_local char g_probe_err[256] = "";
int mqp_fail(int code, const char* msg) {
    snprintf(g_probe_err, sizeof(g_probe_err), "%s", msg);
    return code;
}
int mqp_check_launch(const char* what) {
    const hipError_t e = hipGetLastError();
    if (e == hipSuccess) return MQP_OK;
    snprintf(g_probe_err, sizeof(g_probe_err), "%s: %s", what, hipGetErrorString(e));
    return MQP_ERR_HIP;
}
extern "C" const char* mqp_last_error(void) { return g_probe_err; }

namespace mq {

// flat, 16-byte units: IN bytes read and OUT bytes written per unit (16 / 8: the 2:1 mix of the FP8 quantizers;
// 8 / 16: the 1:2 mix of the FP8 dequantizer), U units per lane, one-shot workgroups of 256 lanes
template <int U, bool WIDE_OUT>
__global__ __launch_bounds__(256) void probe_flat_kernel(const uint8_t* __restrict__ s, uint8_t* __restrict__ d, int64_t n,
                                                         int chunk) {
    const int64_t base = xcd_chunked_block(chunk) * (256 * U) + threadIdx.x;
    u32x4 v[U];
#pragma unroll
    for (int u = 0; u < U; u++) {
        const int64_t i = base + u * 256;
        if (WIDE_OUT) {
            const u32x2 h = i < n ? __builtin_nontemporal_load((const u32x2*)s + i) : u32x2{0u, 0u};
            v[u] = u32x4{h.x, h.y, h.x ^ 1u, h.y ^ 1u};
        } else {
            v[u] = i < n ? ld16(s + i * 16) : u32x4{0u, 0u, 0u, 0u};
        }
    }
#pragma unroll
    for (int u = 0; u < U; u++) {
        const int64_t i = base + u * 256;
        if (i >= n) continue;
        if (WIDE_OUT) st16(d + i * 16, v[u]);
        else st8(d + i * 8, u32x2{v[u].x ^ v[u].y, v[u].z ^ v[u].w});
    }
}
// the 2:1 mix as a loop: gridDim.x workgroups stride over the buffer, two units per lane and trip
__global__ __launch_bounds__(256) void probe_loop_kernel(const uint8_t* __restrict__ s, uint8_t* __restrict__ d, int64_t n,
                                                         int chunk) {
    const int64_t step = (int64_t)gridDim.x * 512;
    for (int64_t base = xcd_chunked_block(chunk) * 512 + threadIdx.x; base < n; base += step) {
        u32x4 v[2];
#pragma unroll
        for (int u = 0; u < 2; u++) v[u] = base + u * 256 < n ? ld16(s + (base + u * 256) * 16) : u32x4{0u, 0u, 0u, 0u};
#pragma unroll
        for (int u = 0; u < 2; u++)
            if (base + u * 256 < n) st8(d + (base + u * 256) * 8, u32x2{v[u].x ^ v[u].y, v[u].z ^ v[u].w});
    }
}
// the 128 x 128 tile shape of the FP8 block quantizer on a row-major [M, K] matrix of 2-byte elements: 512 lanes per
// tile, four 16-byte row pieces per lane, a workgroup-wide exchange between the loads and the stores, 8-byte stores
// into a [M, K] matrix of bytes.  MODE 0: read and write, 1: read only, 2: write only.
template <int MODE>
__global__ __launch_bounds__(512) void probe_tile_kernel(const uint8_t* __restrict__ s, uint8_t* __restrict__ d, int64_t K,
                                                         int32_t tiles) {
    __shared__ uint32_t wave_word[8];
    const int32_t item = xcd_contiguous_item(tiles);
    if (item < 0) return;
    const int32_t tiles_k = (int32_t)(K / 128);
    const int64_t ti = item / tiles_k, tj = item - ti * tiles_k;
    const int t = threadIdx.x, r0 = t >> 4, c = (t & 15) * 8;
    const uint8_t* sp = s + ((ti * 128 + r0) * K + tj * 128 + c) * 2;
    uint8_t* dp = d + (ti * 128 + r0) * K + tj * 128 + c;
    u32x4 v[4];
#pragma unroll
    for (int p = 0; p < 4; p++) v[p] = MODE == 2 ? u32x4{(uint32_t)p, 1u, 2u, 3u} : ld16(sp + (int64_t)p * 32 * K * 2);
    uint32_t m = 0;
#pragma unroll
    for (int p = 0; p < 4; p++) m |= v[p].x | v[p].y | v[p].z | v[p].w;
    m = wave_max(m);
    if ((t & 63) == 0) wave_word[t >> 6] = m;
    __syncthreads();
    uint32_t all = 0;
#pragma unroll
    for (int k = 0; k < 8; k++) all |= wave_word[k];
    if (MODE == 1) {
        if (all == 0x12345678u && t == 0) d[item] = 1;      // keeps the loads alive; never true for the probe's input
        return;
    }
#pragma unroll
    for (int p = 0; p < 4; p++) st8(dp + (int64_t)p * 32 * K, u32x2{v[p].x ^ v[p].y ^ all, v[p].z ^ v[p].w});
}

// one 16-byte unit per lane, no loop: the access pattern that streams fastest on MI355X
__global__ __launch_bounds__(256) void probe_copy_kernel(const uint8_t* __restrict__ src, uint8_t* __restrict__ dst) {
    const int64_t o = ((int64_t)blockIdx.x * 256 + threadIdx.x) * 16;
    st16(dst + o, ld16(src + o));
}

}  // namespace mq

using namespace mq;

extern "C" int mqp_copy_bytes(const void* src, void* dst, int64_t nbytes, void* stream) {
    if (!src || !dst || nbytes < 0 || (nbytes % 4096) || ((uintptr_t)src % 16) || ((uintptr_t)dst % 16))
        return mqp_fail(MQP_ERR_ARG, "copy needs 16-byte aligned pointers and a size that is a multiple of 4096");
    if (nbytes == 0) return MQP_OK;
    if (nbytes / 4096 > 0x7FFFFFF0ll) return mqp_fail(MQP_ERR_ARG, "copy too large");
    hipLaunchKernelGGL(probe_copy_kernel, dim3((unsigned)(nbytes / 4096)), dim3(256), 0, (hipStream_t)stream,
                       (const uint8_t*)src, (uint8_t*)dst);
    return mqp_check_launch("copy");
}

extern "C" int mqp_stream_probe(int shape, const void* src, void* dst, int64_t nbytes, int64_t param, void* stream) {
    if (!src || !dst || nbytes <= 0 || (nbytes % 16) || ((uintptr_t)src % 16) || ((uintptr_t)dst % 16))
        return mqp_fail(MQP_ERR_ARG, "probe needs 16-byte aligned pointers and a positive size that is a multiple of 16");
    hipStream_t st = (hipStream_t)stream;
    const uint8_t* s = (const uint8_t*)src;
    uint8_t* d = (uint8_t*)dst;
    if (shape == MQP_FLAT_2_1 || shape == MQP_FLAT_1_2) {
        // nbytes: the larger of the two sides (read for 2:1, written for 1:2)
        const int64_t n = nbytes / 16;
        if (param != 1 && param != 2 && param != 4 && param != 8) return mqp_fail(MQP_ERR_ARG, "units per lane: 1, 2, 4 or 8");
        int64_t blocks = (n + 256 * param - 1) / (256 * param);
        const int chunk = (int)flat_chunk(blocks);
        blocks = flat_padded(blocks, chunk);
        if (blocks > 0x7FFFFFF0ll) return mqp_fail(MQP_ERR_ARG, "buffer too large");
        const dim3 grid((unsigned)blocks), blk(256);
#define MQ_PROBE_FLAT(U)                                                                                      \
    if (shape == MQP_FLAT_2_1) hipLaunchKernelGGL((probe_flat_kernel<U, false>), grid, blk, 0, st, s, d, n, chunk); \
    else hipLaunchKernelGGL((probe_flat_kernel<U, true>), grid, blk, 0, st, s, d, n, chunk)
        if (param == 1) { MQ_PROBE_FLAT(1); } else if (param == 2) { MQ_PROBE_FLAT(2); }
        else if (param == 4) { MQ_PROBE_FLAT(4); } else { MQ_PROBE_FLAT(8); }
#undef MQ_PROBE_FLAT
        return mqp_check_launch("stream probe");
    }
    if (shape == MQP_LOOP_2_1) {
        if (param < 512 || param % 512 != 0 || param > (1 << 24)) return mqp_fail(MQP_ERR_ARG, "workgroups: a multiple of 512");
        hipLaunchKernelGGL(probe_loop_kernel, dim3((unsigned)param), dim3(256), 0, st, s, d, nbytes / 16, 64);
        return mqp_check_launch("stream probe");
    }
    if (shape == MQP_TILE_2_1 || shape == MQP_TILE_READ || shape == MQP_TILE_WRITE) {
        // nbytes: size of the 2-byte matrix; param: its row length K in elements
        if (param < 128 || param % 128 != 0) return mqp_fail(MQP_ERR_ARG, "row length: a multiple of 128");
        const int64_t rows = nbytes / 2 / param / 128 * 128, tiles = (rows / 128) * (param / 128);
        if (tiles <= 0 || tiles > 0x7FFFFFF0ll) return mqp_fail(MQP_ERR_ARG, "bad matrix size");
        const dim3 grid((unsigned)xcd_grid(tiles)), blk(512);
        if (shape == MQP_TILE_2_1) hipLaunchKernelGGL(probe_tile_kernel<0>, grid, blk, 0, st, s, d, param, (int32_t)tiles);
        else if (shape == MQP_TILE_READ) hipLaunchKernelGGL(probe_tile_kernel<1>, grid, blk, 0, st, s, d, param, (int32_t)tiles);
        else hipLaunchKernelGGL(probe_tile_kernel<2>, grid, blk, 0, st, s, d, param, (int32_t)tiles);
        return mqp_check_launch("stream probe");
    }
    return mqp_fail(MQP_ERR_ARG, "unknown probe shape");
}
