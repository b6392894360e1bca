// NVFP4 (e2m1 codes, one e4m3 scale per 1x16 block, one fp32 scale per tensor) for gfx950.
// Reference: miles/utils/nvfp4.py:19-114 (layout, global scale); block arithmetic as restated in
// miles/kernels/quant/nvfp4_qdq.py:716-743,859-889,1079-1081:
//   S_enc = min(e4m3_max*6 / amax, FLT_MAX), 1 if amax == 0 or the quotient is 0;  S_dec = 1 / S_enc
//   per block: bmax = max|x|; s8 = sat_e4m3(bmax == 0 ? 0 : bmax * (S_enc * f32(1/6)))
//              inv = min(1 / (f32(s8) * S_dec), FLT_MAX);  code = sat_e2m1(x * inv)
//   published global scale: 1 / min(e4m3_max*6/amax, FLT_MAX) with only the ==0 repair (nvfp4.py:19-39)
//
// Pass 1 (mq_nvfp4_amax) reduces max|x| to one uint32 with one atomic per workgroup; a gate/up pair calls
// it twice on the same word.  Pass 2 (mq_nvfp4_quant): two lanes own one block (16 bytes each), the block
// amax is one DPP step, and each lane emits four bytes of codes.
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

// kAmaxUnroll 16-byte units per lane; job.units counts whole units, job.s holds the element count so that
// the first workgroup of a tensor can fold in a tail shorter than one unit
constexpr int kAmaxUnroll = 8;
__global__ __launch_bounds__(256) void nvfp4_amax_bf16_kernel(const FlatTable tab) {
    __shared__ uint32_t wave_amax[4];
    const FlatJob& job = tab.job[blockIdx.y];
    const uint16_t* __restrict__ w = (const uint16_t*)job.w;
    uint32_t* __restrict__ amax_bits = (uint32_t*)job.aux;
    const int64_t n16 = job.units, numel = (int64_t)(uintptr_t)job.s;
    const int t = threadIdx.x;
    const int64_t base = (int64_t)blockIdx.x * (256 * kAmaxUnroll);
    if (base >= n16 && !(blockIdx.x == 0 && numel > 0)) return;
    uint32_t m2 = 0;
#pragma unroll
    for (int i = 0; i < kAmaxUnroll; i++) {
        const int64_t unit = base + i * 256 + t;
        if (unit < n16) {
            const u32x4 v = ld16_keep(w + unit * 8);
            m2 = max2_u16(m2, max2_u16(max2_u16(abs2(v.x), abs2(v.y)), max2_u16(abs2(v.z), abs2(v.w))));
        }
    }
    uint32_t m = hmax_u16(m2);
    if (blockIdx.x == 0 && t == 0)
        for (int64_t i = n16 * 8; i < numel; i++) m = umax(m, (uint32_t)(w[i] & 0x7FFFu));
    m = wave_max(m);
    if ((t & 63) == 0) wave_amax[t >> 6] = m;
    __syncthreads();
    if (t == 0) {
        m = umax(umax(wave_amax[0], wave_amax[1]), umax(wave_amax[2], wave_amax[3])) << 16;
        // most workgroups lose against the running maximum: read it first, touch the atomic only to raise it
        if (m > __hip_atomic_load(amax_bits, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT)) atomicMax(amax_bits, m);
    }
}

__global__ __launch_bounds__(256) void nvfp4_amax_generic_kernel(const void* __restrict__ w, int dtype, int64_t numel,
                                                                 uint32_t* __restrict__ amax_bits) {
    __shared__ uint32_t wave_amax[4];
    const int t = threadIdx.x;
    const int64_t stride = (int64_t)gridDim.x * blockDim.x;
    uint32_t m = 0;
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + t; i < numel; i += stride)
        m = umax(m, f2u(load_f32(w, i, dtype)) & 0x7FFFFFFFu);
    m = wave_max(m);
    if ((t & 63) == 0) wave_amax[t >> 6] = m;
    __syncthreads();
    if (t == 0) {
        m = umax(umax(wave_amax[0], wave_amax[1]), umax(wave_amax[2], wave_amax[3]));
        if (m) atomicMax(amax_bits, m);
    }
}

struct NvScales {
    float enc_sixth;  // S_enc * (1/6)
    float s_dec;      // 1 / S_enc
};
__device__ __forceinline__ NvScales nv_scales(float amax, float numer) {
    float enc = __builtin_fminf(numer / amax, kFltMax);
    if (amax == 0.0f || enc == 0.0f) enc = 1.0f;
    NvScales r;
    r.enc_sixth = enc * kSixth;
    r.s_dec = 1.0f / enc;
    return r;
}
__device__ __forceinline__ float nv_published_scale(float amax, float numer) {
    float enc = numer / amax;
    if (enc > kFltMax) enc = kFltMax;  // NaN stays NaN
    if (enc == 0.0f) enc = 1.0f;
    return 1.0f / enc;
}

__global__ __launch_bounds__(kNvThreads) void nvfp4_quant_bf16_kernel(const FlatTable tab, float numer) {
    const FlatJob& job = tab.job[blockIdx.y];
    const uint16_t* __restrict__ w = (const uint16_t*)job.w;
    uint32_t* __restrict__ q = (uint32_t*)job.q;
    uint8_t* __restrict__ s8 = (uint8_t*)job.s;
    const uint32_t* __restrict__ amax_bits = (const uint32_t*)job.aux;
    const int64_t total_units = job.units;
    const int t = threadIdx.x;
    const int64_t base = (int64_t)blockIdx.x * (kNvThreads * kNvUnroll);
    if (base >= total_units) return;
    u32x4 v[kNvUnroll];
#pragma unroll
    for (int i = 0; i < kNvUnroll; i++) {
        const int64_t unit = base + i * kNvThreads + t;
        v[i] = unit < total_units ? ld16(w + unit * 8) : u32x4{0u, 0u, 0u, 0u};
    }
    const float amax = u2f(amax_bits[0]);
    const NvScales gs = nv_scales(amax, numer);
#pragma unroll
    for (int i = 0; i < kNvUnroll; i++) {
        const int64_t unit = base + i * kNvThreads + t;
        const uint32_t m2 = max2_u16(max2_u16(abs2(v[i].x), abs2(v[i].y)), max2_u16(abs2(v[i].z), abs2(v[i].w)));
        const uint32_t mb = group_max2(hmax_u16(m2));
        const float bmax = u2f(mb << 16);
        const float s_hp = bmax == 0.0f ? 0.0f : bmax * gs.enc_sixth;
        const float f[8] = {bf16_lo(v[i].x), bf16_hi(v[i].x), bf16_lo(v[i].y), bf16_hi(v[i].y),
                            bf16_lo(v[i].z), bf16_hi(v[i].z), bf16_lo(v[i].w), bf16_hi(v[i].w)};
        uint32_t sc, word;
        if (mb < 0x7F80u && s_hp == s_hp) {
            sc = hw_e4m3x2<false>(__builtin_fminf(s_hp, kFp8Max), 0.0f, 0u) & 0xFFu;
            const float s_f = hw_e4m3x2_decode<false>(sc).x;
            const float inv = __builtin_fminf(1.0f / (s_f * gs.s_dec), kFltMax);
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
        if (unit < total_units) {
            st4(q + unit, word);
            if ((t & 1) == 0) s8[unit >> 1] = (uint8_t)sc;
        }
    }
}

// weight_scale_2 of every tensor of a group: out[i] = 1 / min(numer / amax_i, FLT_MAX) (zero repaired to 1)
struct NvGlobalTable {
    int32_t n;
    int32_t pad;
    const uint32_t* amax[kMaxGroup];
    float* out[kMaxGroup];
};
__global__ void nvfp4_global_scale_kernel(const NvGlobalTable tab, float numer) {
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < tab.n && tab.out[i]) *tab.out[i] = nv_published_scale(u2f(*tab.amax[i]), numer);
}

__global__ __launch_bounds__(256) void nvfp4_quant_generic_kernel(const void* __restrict__ w, int dtype,
                                                                  const uint32_t* __restrict__ amax_bits,
                                                                  uint8_t* __restrict__ q, uint8_t* __restrict__ s8,
                                                                  float* __restrict__ global_scale, float numer,
                                                                  int64_t blocks16) {
    const float amax = u2f(amax_bits[0]);
    const NvScales gs = nv_scales(amax, numer);
    if (global_scale && blockIdx.x == 0 && threadIdx.x == 0) *global_scale = nv_published_scale(amax, numer);
    const int64_t stride = (int64_t)gridDim.x * blockDim.x;
    for (int64_t b = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; b < blocks16; b += stride) {
        uint32_t m = 0;
        for (int j = 0; j < 16; j++) m = umax(m, f2u(load_f32(w, b * 16 + j, dtype)) & 0x7FFFFFFFu);
        const float bmax = u2f(m);
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

}  // namespace mq

using namespace mq;

bool mq_nvfp4_fast_ok(const void* w, int dtype, const void* q) {
    return dtype == MQ_BF16 && ((uintptr_t)w % 16) == 0 && ((uintptr_t)q % 4) == 0;
}

// tab.job[i]: w, aux = amax word, units = numel / 8, s = (void*)numel
int mq_nvfp4_amax_launch_group(FlatTable& tab, hipStream_t st) {
    if (!flat_grid(tab, 256 * kAmaxUnroll)) return mq_fail(MQ_ERR_ARG, "tensor too large");
    if (tab.max_blocks == 0) tab.max_blocks = 1;   // tensors shorter than one unit still have a tail
    hipLaunchKernelGGL(nvfp4_amax_bf16_kernel, dim3((unsigned)tab.max_blocks, (unsigned)tab.n), dim3(256), 0, st, tab);
    return mq_check_launch("nvfp4 amax");
}

// tab.job[i]: w, q, s = block scales, aux = amax word, units = numel / 8; global_out[i] may be null
int mq_nvfp4_quant_launch_group(FlatTable& tab, float* const* global_out, int e4m3_max, hipStream_t st) {
    const float numer = (float)e4m3_max * 6.0f;
    NvGlobalTable gt{};
    gt.n = tab.n;
    bool any_global = false;
    for (int i = 0; i < tab.n; i++) {
        gt.amax[i] = (const uint32_t*)tab.job[i].aux;
        gt.out[i] = global_out ? global_out[i] : nullptr;
        any_global |= gt.out[i] != nullptr;
    }
    if (any_global) hipLaunchKernelGGL(nvfp4_global_scale_kernel, dim3(1), dim3(64), 0, st, gt, numer);
    if (!flat_grid(tab, kNvThreads * kNvUnroll)) return mq_fail(MQ_ERR_ARG, "tensor too large");
    if (tab.max_blocks > 0)
        hipLaunchKernelGGL(nvfp4_quant_bf16_kernel, dim3((unsigned)tab.max_blocks, (unsigned)tab.n), dim3(kNvThreads), 0,
                           st, tab, numer);
    return mq_check_launch("nvfp4 quant");
}

extern "C" int mq_nvfp4_amax(const void* w, int dtype, int64_t numel, void* amax_bits, void* stream) {
    if (!w || !amax_bits) return mq_fail(MQ_ERR_ARG, "null pointer");
    if (dtype < MQ_BF16 || dtype > MQ_F32 || numel < 0) return mq_fail(MQ_ERR_ARG, "bad argument");
    if (numel == 0) return MQ_OK;
    hipStream_t st = (hipStream_t)stream;
    if (dtype == MQ_BF16 && ((uintptr_t)w % 16) == 0) {
        FlatTable tab{};
        tab.n = 1;
        tab.job[0] = FlatJob{w, nullptr, (void*)(uintptr_t)numel, amax_bits, numel / 8};
        return mq_nvfp4_amax_launch_group(tab, st);
    }
    int64_t blocks = (numel + 255) / 256;
    if (blocks > 2048) blocks = 2048;
    hipLaunchKernelGGL(nvfp4_amax_generic_kernel, dim3((unsigned)blocks), dim3(256), 0, st, w, dtype, numel,
                       (uint32_t*)amax_bits);
    return mq_check_launch("nvfp4 amax");
}

extern "C" int mq_nvfp4_quant(const void* w, int dtype, const void* amax_bits, void* q, void* block_scale,
                              float* global_scale, int64_t M, int64_t K, int e4m3_max, void* stream) {
    if (!w || !amax_bits || !q || !block_scale) return mq_fail(MQ_ERR_ARG, "null pointer");
    if (dtype < MQ_BF16 || dtype > MQ_F32 || M < 0 || K < 0) return mq_fail(MQ_ERR_ARG, "bad argument");
    if (K % 16 != 0) return mq_fail(MQ_ERR_ARG, "Last dim must be divisible by 16 for NVFP4");
    if (e4m3_max != 448 && e4m3_max != 256) return mq_fail(MQ_ERR_ARG, "e4m3_max must be 448 or 256");
    hipStream_t st = (hipStream_t)stream;
    const float numer = (float)e4m3_max * 6.0f;
    const int64_t blocks16 = M * (K / 16);
    if (blocks16 == 0 || mq_nvfp4_fast_ok(w, dtype, q)) {
        FlatTable tab{};
        tab.n = 1;
        tab.job[0] = FlatJob{w, q, block_scale, const_cast<void*>(amax_bits), blocks16 * 2};
        return mq_nvfp4_quant_launch_group(tab, &global_scale, e4m3_max, st);
    }
    int64_t nb = (blocks16 + 255) / 256;
    if (nb > mq_grid_cap()) nb = mq_grid_cap();
    hipLaunchKernelGGL(nvfp4_quant_generic_kernel, dim3((unsigned)nb), dim3(256), 0, st, w, dtype,
                       (const uint32_t*)amax_bits, (uint8_t*)q, (uint8_t*)block_scale, global_scale, numer, blocks16);
    return mq_check_launch("nvfp4 quant");
}
