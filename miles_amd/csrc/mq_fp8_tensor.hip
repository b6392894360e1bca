// Per-tensor FP8 (one fp32 scale for the whole tensor) as a job of the batched driver, for gfx950.
// Reference: the per-tensor branch of the sync path, .../processors/quantizer_fp8.py:153-158, and tensor_fp8,
// tools/convert_hf_to_fp8.py:73-77:
//   scale = max(max|w|, dtype(1e-12)) / 448;  q = e4m3(clamp(dtype(w / scale), -448, 448))
// (torch divides by the zero-dimensional scale in the weight's dtype, hence the rounding of the quotient to bf16).
//
// bf16 tensors, up to 64 per launch.  The first run of a job list takes two passes: the grouped amax kernel shared
// with NVFP4 (256 partial maxima per tensor, plain stores), a fold kernel (one workgroup per tensor: amax, scale out,
// sections cleared) and the flat quantize kernel.  Later runs of the same list carry the amax over like NVFP4 does:
// pass 1 quantizes with the amax the record kept, collecting the new partial maxima with one atomic max per workgroup;
// the fold compares; pass 2 quantizes again only the tensors whose amax moved.  A tensor whose amax moved takes the
// two-pass form on the next run (pass 1 only collects its amax) and returns to the single pass once the amax has held.
#include "mq_api_internal.hpp"
#include "mq_common.hpp"
#include "mq_group.hpp"

namespace mq {

constexpr int kFtThreads = 256;
constexpr int kFtUnroll = 2;

// job.s = fp32 scale output, job.aux = amax record (section 0)
template <int MODE, class Table>   // 1: fold and clear; 2: also compare with the amax the record held
__global__ __launch_bounds__(256) void fp8_tensor_fold_kernel(const Table tab, float floor_v, uint32_t* moved_counter, uint32_t* moved_mirror) {
    __shared__ uint32_t lds4[4];
    const FlatJob& job = tab.job[blockIdx.x];
    uint32_t* rec = (uint32_t*)job.aux;
    amax_feedback_folded(moved_counter, moved_mirror, gridDim.x);
    uint32_t m = rec[threadIdx.x];
    rec[threadIdx.x] = 0;
    m = wave_max(m);
    if ((threadIdx.x & 63) == 0) lds4[threadIdx.x >> 6] = m;
    __syncthreads();
    if (threadIdx.x == 0) {
        m = umax(umax(lds4[0], lds4[1]), umax(lds4[2], lds4[3]));
        if (MODE == 2) {
            // a record whose amax moved twice in a row is marked volatile: the next carried run only collects its amax in the
            // single pass and quantizes in the second one (the two-pass cost instead of two quantizations), until it holds still
            const bool moved = rec[kRecAmax] != m;
            amax_record_after_carried_run(rec, moved);
            amax_feedback(moved_counter, moved, 1u);
        } else {
            rec[kRecRedo] = 0;
            rec[kRecVolatile] = 0;
            rec[kRecMovedRuns] = 0;
            amax_feedback(moved_counter, rec[kRecAmax] != m, 1u);
        }
        rec[kRecAmax] = m;
        float amax = u2f(m);
        if (amax < floor_v) amax = floor_v;          // a NaN amax stays NaN, as torch's clamp leaves it
        *(float*)job.s = amax / kFp8Max;
    }
}

template <int F16>
__device__ __forceinline__ uint32_t fp8_tensor_quant_units(const FlatJob& job, const int64_t base, const int t, const float floor_v) {
    const uint16_t* __restrict__ w = (const uint16_t*)job.w;
    uint8_t* __restrict__ q = (uint8_t*)job.q;
    const int64_t units = job.units;
    u32x4 v[kFtUnroll];
#pragma unroll
    for (int i = 0; i < kFtUnroll; i++) {
        const int64_t unit = base + i * kFtThreads + t;
        v[i] = unit < units ? ld16(w + unit * 8) : u32x4{0u, 0u, 0u, 0u};
    }
    const uint32_t abits = ((const uint32_t*)job.aux)[kRecAmax];
    float amax = u2f(abits);
    if (amax < floor_v) amax = floor_v;
    const float s = amax / kFp8Max, y = 1.0f / s;
    const bool fast_div = shared_div_ok(s);
    uint32_t seen = 0;
#pragma unroll
    for (int i = 0; i < kFtUnroll; i++) {
        const int64_t unit = base + i * kFtThreads + t;
        seen = umax(seen, hmax_u16(max2_u16(max2_u16(abs2(v[i].x), abs2(v[i].y)), max2_u16(abs2(v[i].z), abs2(v[i].w)))));
        float f[8] = {elem_lo<F16>(v[i].x), elem_hi<F16>(v[i].x), elem_lo<F16>(v[i].y), elem_hi<F16>(v[i].y),
                      elem_lo<F16>(v[i].z), elem_hi<F16>(v[i].z), elem_lo<F16>(v[i].w), elem_hi<F16>(v[i].w)};
#pragma unroll
        for (int j = 0; j < 8; j++) f[j] = fast_div ? div_by_shared(f[j], s, y) : f[j] / s;
#pragma unroll
        for (int j = 0; j < 8; j += 2) {           // the rounding to the weight's dtype
            if (F16) {
                f[j] = (float)(_Float16)f[j];
                f[j + 1] = (float)(_Float16)f[j + 1];
            } else {
                const uint32_t p = hw_bf16x2(f[j], f[j + 1]);
                f[j] = bf16_lo(p);
                f[j + 1] = bf16_hi(p);
            }
        }
        u32x2 o;
        if (abits < 0x7F800000u && s > 0.0f) {      // (a zero scale -- fp16 has no 1e-12 floor -- makes every quotient NaN)
            o.x = hw_e4m3x4(f[0], f[1], f[2], f[3]);
            o.y = hw_e4m3x4(f[4], f[5], f[6], f[7]);
        } else {                                   // inf / NaN amax: clamp and convert in software
            uint32_t c[8];
#pragma unroll
            for (int j = 0; j < 8; j++) c[j] = sw_e4m3fn(clamp_keep_nan(f[j], -kFp8Max, kFp8Max));
            o.x = c[0] | (c[1] << 8) | (c[2] << 16) | (c[3] << 24);
            o.y = c[4] | (c[5] << 8) | (c[6] << 16) | (c[7] << 24);
        }
        if (unit < units) st8(q + unit * 8, o);
    }
    return seen;
}

// PASS 0: second pass of the two-pass form; 1: single pass with the carried-over amax, new partial maxima collected;
// 2: grid-stride second quantization of the tensors whose amax moved
template <int PASS, class Table, int F16>
__global__ __launch_bounds__(kFtThreads) void fp8_tensor_quant_kernel(const Table tab, float floor_v) {
    const FlatJob job = flat_job(tab);       // a copy in registers: a descriptor in device memory must not be re-read after the stores
    const int t = threadIdx.x;
    constexpr int64_t kPerBlock = kFtThreads * kFtUnroll;
    if (PASS == 2) {
        if (((const uint32_t*)job.aux)[kRecRedo] == 0) return;
        // an XCD takes a run of consecutive blocks in every trip of the grid, as the flat grids do (second pass 2 pct faster)
        const int64_t first = xcd_chunked_block(gridDim.x == kSectionWords ? kSectionWords / kXcds : tab.chunk);
        for (int64_t base = first * kPerBlock; base < job.units; base += (int64_t)gridDim.x * kPerBlock)
            fp8_tensor_quant_units<F16>(job, base, t, floor_v);
        return;
    }
    const int64_t base = flat_block(tab) * kPerBlock;
    if (base >= job.units) return;
    uint32_t seen;
    if (PASS == 1 && ((const uint32_t*)job.aux)[kRecVolatile] != 0) {
        const uint16_t* __restrict__ w = (const uint16_t*)job.w;
        uint32_t m2 = 0;
#pragma unroll
        for (int i = 0; i < kFtUnroll; i++) {
            const int64_t unit = base + i * kFtThreads + t;
            const u32x4 v = unit < job.units ? ld16(w + unit * 8) : u32x4{0u, 0u, 0u, 0u};
            m2 = max2_u16(m2, max2_u16(max2_u16(abs2(v.x), abs2(v.y)), max2_u16(abs2(v.z), abs2(v.w))));
        }
        seen = hmax_u16(m2);
    } else {
        seen = fp8_tensor_quant_units<F16>(job, base, t, floor_v);
    }
    if (PASS == 1) {
        __shared__ uint32_t wave_seen[kFtThreads / 64];
        seen = wave_max(seen);
        if ((t & 63) == 0) wave_seen[t >> 6] = seen;
        __syncthreads();
        if (t == 0) {
            uint32_t m = 0;
#pragma unroll
            for (int k = 0; k < kFtThreads / 64; k++) m = umax(m, wave_seen[k]);
            atomicMax((uint32_t*)job.aux + (blockIdx.x & (kSectionWords - 1)), f2u(elem_lo<F16>(m)));
        }
    }
}

}  // namespace mq

using namespace mq;

int mq_nvfp4_amax_launch_group(int dtype, FlatTable& tab, hipStream_t st);
int mq_nvfp4_amax_launch_table(int dtype, const FlatJob* device_jobs, int n, hipStream_t st);

bool mq_fp8_tensor_fast_ok(const void* w, int dtype, const void* q, int64_t rows, int64_t cols, int64_t ld) {
    return (dtype == MQ_BF16 || dtype == MQ_F16) && cols % 8 == 0 && ld == cols && ((uintptr_t)w % 16) == 0 && ((uintptr_t)q % 8) == 0 &&
           rows * (cols / 8) < (1ll << 38);
}

// fold + quantize (+ second pass) over a table whose grid is known
template <class Table, int F16>
static int fp8_tensor_launch_dtype(const Table& tab, int n, float floor_v, bool carry, hipStream_t st) {
    const dim3 folds((unsigned)n), blk(256), grid((unsigned)tab.max_blocks, (unsigned)n);
    if (carry) {
        if (tab.max_blocks > 0) hipLaunchKernelGGL((fp8_tensor_quant_kernel<1, Table, F16>), grid, dim3(kFtThreads), 0, st, tab, floor_v);
        hipLaunchKernelGGL((fp8_tensor_fold_kernel<2, Table>), folds, blk, 0, st, tab, floor_v, mq_amax_feedback(), mq_amax_feedback_mirror());
        if (tab.max_blocks > 0) {
            const unsigned redo = tab.max_blocks < kSectionWords ? (unsigned)tab.max_blocks : (unsigned)kSectionWords;
            hipLaunchKernelGGL((fp8_tensor_quant_kernel<2, Table, F16>), dim3(redo, (unsigned)n), dim3(kFtThreads), 0, st, tab, floor_v);
        }
        return mq_check_launch("fp8 per-tensor quant (carried-over amax)");
    }
    hipLaunchKernelGGL((fp8_tensor_fold_kernel<1, Table>), folds, blk, 0, st, tab, floor_v, mq_amax_feedback(), mq_amax_feedback_mirror());
    if (tab.max_blocks > 0) hipLaunchKernelGGL((fp8_tensor_quant_kernel<0, Table, F16>), grid, dim3(kFtThreads), 0, st, tab, floor_v);
    return mq_check_launch("fp8 per-tensor quant");
}
template <class Table>
static int fp8_tensor_launch(int dtype, const Table& tab, int n, float floor_v, bool carry, hipStream_t st) {
    return dtype == MQ_F16 ? fp8_tensor_launch_dtype<Table, 1>(tab, n, floor_v, carry, st)
                           : fp8_tensor_launch_dtype<Table, 0>(tab, n, floor_v, carry, st);
}

// tab.job[i]: w, q, s = fp32 scale out, aux = amax record, units = numel / 8.  carry: see the file header.
int mq_fp8_tensor_launch_group(int dtype, FlatTable& tab, float floor_v, bool carry, hipStream_t st) {
    if (!carry) {
        FlatTable amax = tab;
        for (int i = 0; i < tab.n; i++) {
            amax.job[i].s = (void*)(uintptr_t)(tab.job[i].units * 8);      // element count, for the amax kernel's tail
            amax.job[i].section = 0;
        }
        int rc = mq_nvfp4_amax_launch_group(dtype, amax, st);
        if (rc) return rc;
    }
    if (!flat_grid(tab, kFtThreads * kFtUnroll)) return mq_fail(MQ_ERR_ARG, "tensor too large");
    return fp8_tensor_launch(dtype, tab, tab.n, floor_v, carry, st);
}
// the same over n descriptors of a device table (section 0 in every entry); max_units: the largest tensor's units
int mq_fp8_tensor_launch_table(int dtype, const FlatJob* device_jobs, int n, int64_t max_units, float floor_v, bool carry,
                               hipStream_t st) {
    if (n == 0) return MQ_OK;
    if (!carry) {
        int rc = mq_nvfp4_amax_launch_table(dtype, device_jobs, n, st);
        if (rc) return rc;
    }
    FlatRef ref{device_jobs, 0, 0};
    if (!flat_grid(ref, max_units, kFtThreads * kFtUnroll)) return mq_fail(MQ_ERR_ARG, "tensor too large");
    return fp8_tensor_launch(dtype, ref, n, floor_v, carry, st);
}
