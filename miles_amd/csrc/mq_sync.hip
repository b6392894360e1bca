// Batched driver: turns a list of per-tensor quantization jobs into grouped kernel launches.
//
// One launch carries up to kMaxGroup tensors (descriptors in the kernel argument segment), so a weight sync
// issues a few launches per layer instead of several per tensor.  Jobs that do not qualify for a grouped
// fast path (other dtypes, block sizes, strides, alignment) run through the single-tensor entry points, in
// list order.
#include <atomic>
#include <vector>

#include <stdlib.h>
#include <string.h>

#include "mq_api_internal.hpp"
#include "mq_common.hpp"
#include "mq_group.hpp"

using namespace mq;

// grouped launchers implemented next to their kernels
bool mq_fp8_tile_fast_ok(const void* w, int dtype, int64_t sxm, int64_t sxn, const void* q, int64_t M, int64_t K,
                         int bm, int bk);
int mq_fp8_tile_launch_group(int mode, int dtype, TileTable& tab, hipStream_t st);
int64_t mq_fp8_tile_job_finish(TileJob& j);
int mq_fp8_tile_launch_table(int mode, int dtype, const TileJob* device_jobs, int n, int64_t max_tiles, hipStream_t st);
bool mq_fp8_dequant_fast_ok(const void* x, const void* y, int64_t M, int64_t N, int block);
int mq_fp8_dequant_launch_group(const MqDequantArgs* a, int n, hipStream_t st);
bool mq_mxfp8_fast_ok(const void* w, int dtype, const void* q);
int mq_mxfp8_launch_group(int dtype, FlatTable& tab, hipStream_t st);
bool mq_int4_pack_fast_ok(const void* w, int dtype, int group);
int mq_int4_pack_launch_group(int dtype, FlatTable& tab, int group, hipStream_t st);
bool mq_nvfp4_fast_ok(const void* w, int dtype, const void* q);
int mq_nvfp4_amax_launch_group(int dtype, FlatTable& tab, hipStream_t st);
int mq_nvfp4_quant_launch_group(int dtype, FlatTable& tab, int e4m3_max, int flags, int mode, hipStream_t st);
bool mq_mxfp4_fast_ok(const void* w, int dtype, const void* packed, int group);
int mq_mxfp4_launch_group(int dtype, FlatTable& tab, hipStream_t st);
bool mq_fp8_tensor_fast_ok(const void* w, int dtype, const void* q, int64_t rows, int64_t cols, int64_t ld);
int mq_fp8_tensor_launch_group(int dtype, FlatTable& tab, float floor_v, bool carry, hipStream_t st);
int mq_fp8_tensor_launch_table(int dtype, const FlatJob* device_jobs, int n, int64_t max_units, float floor_v, bool carry,
                               hipStream_t st);
int mq_nvfp4_amax_launch_table(int dtype, const FlatJob* device_jobs, int n, hipStream_t st);
int mq_nvfp4_quant_launch_table(int dtype, const FlatJob* device_jobs, int n, int64_t max_units, int e4m3_max, int mode,
                                hipStream_t st);
int mq_mxfp8_launch_table(int dtype, const FlatJob* device_jobs, int n, int64_t max_units, hipStream_t st);
int mq_mxfp4_launch_table(int dtype, const FlatJob* device_jobs, int n, int64_t max_units, hipStream_t st);
int mq_int4_pack_launch_table(int dtype, const FlatJob* device_jobs, int n, int64_t max_units, int group, hipStream_t st);
bool mq_int4_pack_asym_fast_ok(const void* w, int dtype, int group, int64_t M);
int mq_int4_pack_asym_launch_group(int dtype, FlatTable& tab, int group, hipStream_t st);
int mq_int4_pack_asym_launch_table(int dtype, const FlatJob* device_jobs, int n, int64_t max_units, int64_t max_zero_tiles, int group,
                                   hipStream_t st);
int64_t mq_int4_zero_tiles(int64_t rows, int64_t cols, int group);
int mq_mxfp4_to_fp8_job(RecodeJob& job, const void* packed, const void* scale, void* y, void* tile_scale, int64_t out_dim,
                        int64_t in_dim);
int mq_mxfp4_to_fp8_launch_group(const RecodeTable& tab, hipStream_t st);
bool mq_fp8_to_mxfp8_fast_ok(const void* x, const void* q, int64_t M, int64_t K);
int mq_fp8_to_mxfp8_launch_group(const MqRescaleArgs* a, int n, hipStream_t st);
bool mq_int4_unpack_fast_ok(const void* packed, const void* y, int64_t K, int group);
FlatJob mq_int4_unpack_entry(const void* packed, const void* scale, void* y, int64_t M, int64_t K, int group);
int mq_int4_unpack_launch_group(int scale_dtype, FlatTable& tab, hipStream_t st);
bool mq_mxfp4_dequant_fast_ok(const void* packed, const void* y, int64_t bytes, int group);
FlatJob mq_mxfp4_dequant_entry(const void* packed, const void* scale, void* y, int64_t bytes, int group);
int mq_mxfp4_dequant_launch_group(FlatTable& tab, hipStream_t st);
int mq_copy_launch_group(CopyTable& tab, hipStream_t st);
int mq_copy_launch_run(const void* src, void* dst, int64_t bytes, hipStream_t st);

// Upper bound on the input bytes of one NVFP4 group (amax launch + fold + quantize launch).  Measured on
// MI355X the second read of a tensor gains nothing from the memory-side cache at any group size, so groups
// are as large as the 64-tensor table allows: fewer launch boundaries.
#ifndef MQ_NV_GROUP_MB
#define MQ_NV_GROUP_MB (1 << 20)
#endif
static const int64_t kNvfp4GroupBytes = (int64_t)MQ_NV_GROUP_MB << 20;

static bool job_fast(const mq_job& j) {
    switch (j.kind) {
        case MQ_JOB_FP8_BLOCK:
        case MQ_JOB_FP8_BLOCKWISE_CAST:
        case MQ_JOB_FP8_BLOCK_POW2:
            return mq_fp8_tile_fast_ok(j.in, j.dtype, j.ld, 1, j.out, j.rows, j.cols, j.p0, j.p1) &&
                   (j.block_stride % 8) == 0 && j.block_stride >= 0 && j.block_stride <= 0x7FFFFFFF &&
                   j.rows_per_block / 128 <= 0x7FFFFFFF;
        case MQ_JOB_FP8_DEQUANT:
            return mq_fp8_dequant_fast_ok(j.in, j.out, j.rows, j.cols, j.p0);
        case MQ_JOB_MXFP8:
            return mq_mxfp8_fast_ok(j.in, j.dtype, j.out) && j.cols % 32 == 0;
        case MQ_JOB_INT4_PACK:
            return mq_int4_pack_fast_ok(j.in, j.dtype, j.p0) && j.cols % j.p0 == 0 && j.cols % 8 == 0;
        case MQ_JOB_INT4_PACK_ASYM:
            return mq_int4_pack_asym_fast_ok(j.in, j.dtype, j.p0, j.rows) && j.cols % j.p0 == 0;
        case MQ_JOB_NVFP4:
            return mq_nvfp4_fast_ok(j.in, j.dtype, j.out) && j.cols % 16 == 0 && (j.p0 == 448 || j.p0 == 256);
        case MQ_JOB_MXFP4:
            return mq_mxfp4_fast_ok(j.in, j.dtype, j.out, j.p0);
        case MQ_JOB_COPY:
            return true;
        case MQ_JOB_FP8_TENSOR:
            return mq_fp8_tensor_fast_ok(j.in, j.dtype, j.out, j.rows, j.cols, j.ld);
        case MQ_JOB_MXFP4_TO_FP8:
            return true;               // check_job has refused what the kernel does not take
        case MQ_JOB_FP8_TO_MXFP8:
            return mq_fp8_to_mxfp8_fast_ok(j.in, j.out, j.rows, j.cols) && j.ld >= (j.cols + 127) / 128 && j.ld <= 0x7FFFFFFF;
        case MQ_JOB_INT4_UNPACK:
            return mq_int4_unpack_fast_ok(j.in, j.out, j.cols, j.p0);
        case MQ_JOB_MXFP4_DEQUANT:
            return mq_mxfp4_dequant_fast_ok(j.in, j.out, j.rows * j.cols / 2, j.p0);
        default:
            return false;
    }
}

static int64_t copy_dst_pitch(const mq_job& j);
static int check_job(const mq_job& j) {
    if (j.kind < MQ_JOB_FP8_BLOCK || j.kind > MQ_JOB_MXFP4_DEQUANT) return mq_fail(MQ_ERR_ARG, "unknown job kind");
    if (j.rows < 0 || j.cols < 0) return mq_fail(MQ_ERR_ARG, "job with a negative shape");
    const bool empty = j.rows == 0 || j.cols == 0;       // an empty tensor has no address
    if ((!j.in || !j.out) && !empty) return mq_fail(MQ_ERR_ARG, "job with a null tensor pointer");
    if (j.kind == MQ_JOB_COPY) {
        if (j.rows > 1 && (j.ld < j.cols || copy_dst_pitch(j) < j.cols || j.rows > 0x7FFFFFF0))
            return mq_fail(MQ_ERR_ARG, "rows of a copy job overlap");
        return MQ_OK;
    }
    if (j.kind == MQ_JOB_UE8M0_PACK)
        return j.p0 >= 0 && j.rows_per_block == 0 ? MQ_OK : mq_fail(MQ_ERR_ARG, "bad scale-pack job");
    if (j.kind == MQ_JOB_E8M0_EXPAND)
        return j.rows_per_block == 0 ? MQ_OK : mq_fail(MQ_ERR_ARG, "bad scale-expansion job");
    if (j.kind == MQ_JOB_FP8_TO_MXFP8 && !empty && (!j.aux || j.rows_per_block != 0))
        return mq_fail(MQ_ERR_ARG, "FP8 to MXFP8 job without tile scales");
    if (j.kind == MQ_JOB_INT4_UNPACK || j.kind == MQ_JOB_MXFP4_DEQUANT) {
        // the entry points' own checks, made before anything of the list runs
        if (j.rows_per_block != 0 || j.p0 <= 0 || (!empty && !j.aux)) return mq_fail(MQ_ERR_ARG, "unpacking job without scales or a group size");
        if (j.kind == MQ_JOB_INT4_UNPACK && (j.dtype < MQ_BF16 || j.dtype > MQ_F32)) return mq_fail(MQ_ERR_ARG, "bad scale dtype");
        if (j.kind == MQ_JOB_INT4_UNPACK ? j.cols % j.p0 != 0 : (j.rows * j.cols) % j.p0 != 0 || (j.rows * j.cols) % 2 != 0)
            return mq_fail(MQ_ERR_ARG, "the element count must be a multiple of the group size");
        return MQ_OK;
    }
    if (j.kind == MQ_JOB_MXFP4_TO_FP8) {
        if (j.rows_per_block != 0) return mq_fail(MQ_ERR_ARG, "bad MXFP4 to FP8 job");
        RecodeJob probe;
        return mq_mxfp4_to_fp8_job(probe, j.in, j.aux, j.out, j.scale, j.rows, j.cols);
    }
    if (!empty && (j.kind == MQ_JOB_FP8_DEQUANT ? !j.aux : !j.scale)) return mq_fail(MQ_ERR_ARG, "job without a scale pointer");
    if (j.kind == MQ_JOB_NVFP4 && !j.aux) return mq_fail(MQ_ERR_ARG, "NVFP4 job without an amax record");
    if (j.kind == MQ_JOB_INT4_PACK_ASYM && !empty && (!j.aux || !j.aux2)) return mq_fail(MQ_ERR_ARG, "asymmetric INT4 job without zero-point outputs");
    if (j.kind == MQ_JOB_FP8_TENSOR) {
        if (!j.aux || !j.scale) return mq_fail(MQ_ERR_ARG, "per-tensor FP8 job without an amax record or a scale pointer");
        if (!empty && !job_fast(j)) return mq_fail(MQ_ERR_ARG, "per-tensor FP8 jobs take contiguous bf16 or fp16 tensors (cols % 8 == 0, 16-byte aligned)");
    }
    if (j.rows_per_block != 0) {
        const bool fp8q = j.kind == MQ_JOB_FP8_BLOCK || j.kind == MQ_JOB_FP8_BLOCKWISE_CAST || j.kind == MQ_JOB_FP8_BLOCK_POW2;
        if (!fp8q || j.rows_per_block < 0 || j.rows_per_block % 128 != 0 || j.p0 != 128 || j.p1 != 128 ||
            (j.dtype != MQ_BF16 && j.dtype != MQ_F16))
            return mq_fail(MQ_ERR_ARG, "row-blocked input needs a bf16 or fp16 FP8 128x128 job with rows_per_block % 128 == 0");
    }
    return MQ_OK;
}

static int run_single(const mq_job& j, void* stream) {
    switch (j.kind) {
        case MQ_JOB_FP8_BLOCK:
            return mq_fp8_block_quant(j.in, j.dtype, j.ld, j.out, (float*)j.scale, j.rows, j.cols, j.p0, j.p1, stream);
        case MQ_JOB_FP8_BLOCKWISE_CAST:
            return mq_fp8_blockwise_cast(j.in, j.dtype, j.ld, 1, j.out, (float*)j.scale, j.rows, j.cols, j.p0, j.p1,
                                         stream);
        case MQ_JOB_FP8_BLOCK_POW2:
            if (j.p0 != 128 || j.p1 != 128) return mq_fail(MQ_ERR_ARG, "power-of-two FP8 scales use 128x128 blocks");
            return mq_fp8_block_quant_pow2(j.in, j.dtype, j.ld, j.out, (float*)j.scale, j.rows, j.cols, stream);
        case MQ_JOB_FP8_DEQUANT:
            return mq_fp8_block_dequant(j.in, (const float*)j.aux, j.out, j.rows, j.cols, j.p0, stream);
        case MQ_JOB_MXFP8:
            return mq_mxfp8_quant(j.in, j.dtype, j.out, (uint8_t*)j.scale, j.rows, j.cols, stream);
        case MQ_JOB_INT4_PACK:
            return mq_int4_group_quant_pack(j.in, j.dtype, (int32_t*)j.out, j.scale, j.rows, j.cols, j.p0, stream);
        case MQ_JOB_MXFP4:
            return mq_mxfp4_quant(j.in, j.dtype, (uint8_t*)j.out, (uint8_t*)j.scale, j.rows * j.cols, j.p0, stream);
        case MQ_JOB_INT4_PACK_ASYM:
            return mq_int4_group_quant_pack_asym(j.in, j.dtype, (int32_t*)j.out, j.scale, (uint8_t*)j.aux, (int32_t*)j.aux2,
                                                 j.rows, j.cols, j.p0, stream);
        case MQ_JOB_UE8M0_PACK:
            return mq_ue8m0_pack_scales((const float*)j.in, (int32_t*)j.out, j.p0, j.rows, j.cols, j.p1, j.ld != 0, stream);
        case MQ_JOB_FP8_TO_MXFP8:
            return mq_fp8_block_to_mxfp8(j.in, (const float*)j.aux, j.ld, j.out, (uint8_t*)j.scale, j.rows, j.cols, stream);
        case MQ_JOB_E8M0_EXPAND:
            return mq_e8m0_expand_tile_scales(j.in, j.dtype == MQ_F32, j.ld, (uint8_t*)j.out, j.rows, j.cols, stream);
        case MQ_JOB_MXFP4_TO_FP8:
            return mq_mxfp4_to_fp8_block((const uint8_t*)j.in, (const uint8_t*)j.aux, j.out, (float*)j.scale, j.rows, j.cols, stream);
        case MQ_JOB_INT4_UNPACK:
            return mq_int4_unpack_dequant((const int32_t*)j.in, j.aux, j.dtype, j.out, j.rows, j.cols, j.p0, stream);
        case MQ_JOB_MXFP4_DEQUANT:
            return mq_mxfp4_dequant((const uint8_t*)j.in, (const uint8_t*)j.aux, j.out, j.rows * j.cols / 2, j.p0, stream);
        default:
            return mq_fail(MQ_ERR_ARG, "unknown job kind");
    }
}

static_assert(kMaxGroup == MQ_MAX_GROUP, "the public group size must match the launch tables");
static_assert(sizeof(FlatJob) == MQ_JOB_TABLE_ENTRY_BYTES && sizeof(TileJob) == MQ_JOB_TABLE_ENTRY_BYTES &&
              kTableGroup == MQ_TABLE_GROUP, "the public table entry must match FlatJob and TileJob");

// job kinds whose grouped launch can read its descriptors from a device table: the flat kernels and the FP8 tile kernel
static bool tile_kind(int kind) {
    return kind == MQ_JOB_FP8_BLOCK || kind == MQ_JOB_FP8_BLOCKWISE_CAST || kind == MQ_JOB_FP8_BLOCK_POW2;
}
static bool table_kind(int kind) {
    return kind == MQ_JOB_MXFP8 || kind == MQ_JOB_MXFP4 || kind == MQ_JOB_INT4_PACK || kind == MQ_JOB_INT4_PACK_ASYM ||
           kind == MQ_JOB_FP8_TENSOR || kind == MQ_JOB_NVFP4 || tile_kind(kind);
}
// NVFP4 jobs that share an amax record are neighbours in the list: the place of job t among them, and how many they are
static void nvfp4_sections(const mq_job* jobs, int64_t n, int64_t t, int& section, int& sections) {
    section = 0;
    for (int64_t b = t; b > 0 && section < 2 * MQ_NVFP4_SECTIONS && jobs[b - 1].kind == MQ_JOB_NVFP4 && jobs[b - 1].aux == jobs[t].aux; b--)
        section++;
    sections = section + 1;
    for (int64_t f = t + 1; f < n && sections < 2 * MQ_NVFP4_SECTIONS && jobs[f].kind == MQ_JOB_NVFP4 && jobs[f].aux == jobs[t].aux; f++)
        sections++;
}
static TileJob tile_entry(const mq_job& jb) {
    return TileJob{jb.in, jb.out, (float*)jb.scale, (int32_t)jb.ld, (int32_t)jb.rows, (int32_t)jb.cols,
                   (int32_t)jb.block_stride, (int32_t)(jb.rows_per_block / 128), 0, 0, 0};
}
// The tile kernel streams a few percent faster in launches of moderate length than in very long ones (measured on the
// Qwen3-4B tensors: 0.770 of peak at 98 000 tiles per launch, 0.784 at 49 000, 0.790 at 31 000, 0.792 at 18 000; each
// launch boundary costs about 4 us).  A run of tile jobs longer than this many tiles goes out as launches of equal size.
#ifndef MQ_TILE_LAUNCH_TILES
#define MQ_TILE_LAUNCH_TILES 36864
#endif
static int64_t tiles_of(const mq_job& jb) { return ((jb.rows + 127) / 128) * ((jb.cols + 127) / 128); }
static FlatJob flat_entry(const mq_job& jb) {
    if (jb.kind == MQ_JOB_INT4_PACK_ASYM)       // zero points, packed zero points, groups per row
        return FlatJob{jb.in, jb.out, jb.scale, jb.aux, jb.rows * jb.cols / 8, jb.aux2, jb.p0 > 0 ? (int32_t)(jb.cols / jb.p0) : 0, 0};
    if (jb.kind == MQ_JOB_FP8_TENSOR)           // amax record, one section
        return FlatJob{jb.in, jb.out, jb.scale, jb.aux, jb.rows * jb.cols / 8, nullptr, 0, 1};
    return FlatJob{jb.in, jb.out, jb.scale, nullptr, jb.rows * jb.cols / 8, nullptr, 0, 0};
}

// The cut length of this process: the compiled-in value, unless the environment variable MQ_TILE_LAUNCH_TILES held a
// whole number when the library first needed it (anything else in the variable is ignored), or until
// mq_tune_tile_launch_tiles sets another.  0 switches the cutting off.
static std::atomic<int64_t>& tile_launch_cap() {
    static std::atomic<int64_t> cap{[] {
        int64_t v = MQ_TILE_LAUNCH_TILES;
        if (const char* env = getenv("MQ_TILE_LAUNCH_TILES")) {
            char* end = nullptr;
            const long long parsed = strtoll(env, &end, 10);
            if (end != env && *end == '\0' && parsed >= 0) v = parsed;
        }
        return v;
    }()};
    return cap;
}
extern "C" int mq_tune_tile_launch_tiles(int64_t tiles, int64_t* previous) {
    if (tiles < 0) return mq_fail(MQ_ERR_ARG, "the launch length is a tile count, 0 for no cutting");
    const int64_t old = tile_launch_cap().exchange(tiles);
    if (previous) *previous = old;
    return MQ_OK;
}

// jobs [i, j) hold `tiles` tiles: where the first of the equal launches they are cut into ends
static int64_t tile_run_end(const mq_job* jobs, int64_t i, int64_t j, int64_t tiles) {
    const int64_t cap = tile_launch_cap().load(std::memory_order_relaxed);
    if (cap <= 0 || tiles <= cap) return j;
    const int64_t launches = (tiles + cap - 1) / cap;
    const int64_t target = (tiles + launches - 1) / launches;
    int64_t acc = 0, t = i;
    while (t < j && acc < target) acc += tiles_of(jobs[t++]);
    return t;
}

static bool same_group(const mq_job& a, const mq_job& b) {
    // the quantizer kernels are compiled per 16-bit input dtype; the other kinds' fast paths take one dtype, or any
    // (copies)
    const bool per_dtype = tile_kind(a.kind) || a.kind == MQ_JOB_MXFP8 || a.kind == MQ_JOB_MXFP4 || a.kind == MQ_JOB_INT4_PACK ||
                           a.kind == MQ_JOB_INT4_PACK_ASYM || a.kind == MQ_JOB_INT4_UNPACK;
    return a.kind == b.kind && a.p0 == b.p0 && a.p1 == b.p1 && (!per_dtype || a.dtype == b.dtype);
}

// Copy jobs of one launch run in no particular order: a job that reads what an earlier job of the group writes (a
// regrouped tensor that is then copied into a payload), or writes what one reads or writes, has to start a new group.
// A copy job is `rows` rows of `cols` bytes; with more than one row the source rows are `ld` bytes apart and the
// destination rows `block_stride` bytes (0: back to back).  Its footprints are taken as the whole span of the rows.
static int64_t copy_dst_pitch(const mq_job& j) { return j.block_stride != 0 ? j.block_stride : j.cols; }
static uintptr_t copy_span(const mq_job& j, int64_t pitch) {
    return (uintptr_t)(j.rows > 1 ? (j.rows - 1) * pitch + j.cols : j.rows * j.cols);
}
static bool copy_depends_on_group(const mq_job* jobs, int64_t first, int64_t candidate) {
    const mq_job& c = jobs[candidate];
    const uintptr_t cin = (uintptr_t)c.in, cout = (uintptr_t)c.out;
    const uintptr_t cib = copy_span(c, c.ld), cob = copy_span(c, copy_dst_pitch(c));
    for (int64_t t = first; t < candidate; t++) {
        const uintptr_t tin = (uintptr_t)jobs[t].in, tout = (uintptr_t)jobs[t].out;
        const uintptr_t tib = copy_span(jobs[t], jobs[t].ld), tob = copy_span(jobs[t], copy_dst_pitch(jobs[t]));
        const bool reads_written = cin < tout + tob && tout < cin + cib;
        const bool writes_touched = (cout < tout + tob && tout < cout + cob) || (cout < tin + tib && tin < cout + cob);
        if (reads_written || writes_touched) return true;
    }
    return false;
}

// per-tensor FP8 run [i, j): chunks of up to kMaxGroup tensors of similar size with the same floor and flags
// (`table`: the device descriptors of jobs[0..), or null)
static int run_fp8_tensor(const mq_job* jobs, int64_t i, int64_t j, const FlatJob* table, void* stream) {
    const int64_t cap = table ? kTableGroup : kMaxGroup;
    while (i < j) {
        int64_t k = i, sum = 0, mx = 0;
        while (k < j && k - i < cap && jobs[k].p0 == jobs[i].p0 && jobs[k].p1 == jobs[i].p1 && jobs[k].dtype == jobs[i].dtype) {
            const int64_t e = jobs[k].rows * jobs[k].cols;
            const int64_t nmx = e > mx ? e : mx;
            if (k > i && nmx * (k - i + 1) * 4 > (sum + e) * 5) break;       // padding of the 2-D grid under 25 %
            sum += e;
            mx = nmx;
            k++;
        }
        const uint32_t floor_bits = (uint32_t)jobs[i].p0;
        float floor_v;
        memcpy(&floor_v, &floor_bits, 4);
        const bool carry = (jobs[i].p1 & MQ_NVFP4_CARRY_AMAX) != 0;
        int rc;
        if (k - i > kMaxGroup) {
            rc = mq_fp8_tensor_launch_table(jobs[i].dtype, table + i, (int)(k - i), mx / 8, floor_v, carry, (hipStream_t)stream);
        } else {
            FlatTable tab{};
            tab.n = (int)(k - i);
            for (int64_t t = i; t < k; t++) tab.job[t - i] = flat_entry(jobs[t]);
            rc = mq_fp8_tensor_launch_group(jobs[i].dtype, tab, floor_v, carry, (hipStream_t)stream);
        }
        if (rc) return rc;
        i = k;
    }
    return MQ_OK;
}

// NVFP4 run [i, j): all jobs fast or not, processed as amax-phase then quantize-phase per chunk
// (`table`: the device descriptors of jobs[0..), or null; n_all: length of the whole list, for the section lookup)
static int run_nvfp4(const mq_job* jobs, int64_t n_all, int64_t i, int64_t j, const FlatJob* table, void* stream) {
    hipStream_t st = (hipStream_t)stream;
    while (i < j) {
        // a chunk ends at the group / byte limit, but never between two jobs that share an amax word
        auto form = [&](int64_t cap) {
            int64_t k = i, bytes = 0, mx = 0;
            while (k < j) {
                int64_t r = k + 1;                               // the jobs of one record: k .. r-1
                while (r < j && jobs[r].aux == jobs[k].aux) r++;
                int64_t b = 0, nmx = mx;
                for (int64_t t = k; t < r; t++) {
                    const int64_t bt = jobs[t].rows * jobs[t].cols * (jobs[t].dtype == MQ_F32 ? 4 : 2);
                    b += bt;
                    nmx = bt > nmx ? bt : nmx;
                }
                const bool ragged = nmx * (r - i) * 4 > (bytes + b) * 5;
                if (k > i && (r - i > cap || bytes + b > kNvfp4GroupBytes || jobs[k].p0 != jobs[i].p0 ||
                              jobs[k].p1 != jobs[i].p1 || jobs[k].dtype != jobs[i].dtype || ragged))
                    break;
                mx = nmx;
                bytes += b;
                k = r;
            }
            return k;
        };
        auto all_fast_in = [&](int64_t k) {
            for (int64_t t = i; t < k; t++)       // (the packed kernels are compiled per 16-bit dtype: one per launch)
                if (!job_fast(jobs[t]) || jobs[t].dtype != jobs[i].dtype) return false;
            return true;
        };
        // a device table lifts the limit for standard block scaling when every job takes the packed kernels
        const bool standard = (jobs[i].p1 & (MQ_NVFP4_4OVER6 | MQ_NVFP4_ERR_MSE | MQ_NVFP4_ERR_FP16)) == 0;
        int64_t k = form(table && standard ? kTableGroup : kMaxGroup);
        bool all_fast = all_fast_in(k);
        if (k - i > kMaxGroup && !all_fast) {
            k = form(kMaxGroup);
            all_fast = all_fast_in(k);
        }
        const int n = (int)(k - i);
        const bool from_table = table && standard && all_fast && n > kMaxGroup;
        if (n > kMaxGroup && !from_table) return mq_fail(MQ_ERR_ARG, "too many NVFP4 jobs share one amax record");
        std::vector<int> section(n), sections(n);
        for (int t = 0; t < n; t++) {
            nvfp4_sections(jobs, n_all, i + t, section[t], sections[t]);
            if (sections[t] > MQ_NVFP4_SECTIONS) return mq_fail(MQ_ERR_ARG, "too many NVFP4 jobs share one amax record");
        }
        if (all_fast) {
            // MQ_NVFP4_CARRY_AMAX (set by a caller that replays this very list, records included, after a first plain
            // run): one pass with last sync's amax instead of the amax pass; every job of the chunk must ask for it
            bool carry = true;
            for (int t = 0; t < n; t++) carry &= (jobs[i + t].p1 & MQ_NVFP4_CARRY_AMAX) != 0;
            int rc = MQ_OK;
            if (from_table) {
                int64_t max_units = 0;
                for (int t = 0; t < n; t++) {
                    const int64_t u = jobs[i + t].rows * jobs[i + t].cols / 8;
                    max_units = u > max_units ? u : max_units;
                }
                if (!carry) rc = mq_nvfp4_amax_launch_table(jobs[i].dtype, table + i, n, st);
                if (rc) return rc;
                rc = mq_nvfp4_quant_launch_table(jobs[i].dtype, table + i, n, max_units, jobs[i].p0, carry ? 2 : 1, st);
                if (rc) return rc;
                i = k;
                continue;
            }
            FlatTable tab{};
            tab.n = n;
            if (!carry) {
                for (int t = 0; t < n; t++) {
                    const mq_job& jb = jobs[i + t];
                    const int64_t numel = jb.rows * jb.cols;
                    tab.job[t] = FlatJob{jb.in, nullptr, (void*)(uintptr_t)numel, jb.aux, numel / 8, nullptr, section[t], 0};
                }
                rc = mq_nvfp4_amax_launch_group(jobs[i].dtype, tab, st);
                if (rc) return rc;
            }
            for (int t = 0; t < n; t++) {
                const mq_job& jb = jobs[i + t];
                tab.job[t] = FlatJob{jb.in, jb.out, jb.scale, jb.aux, jb.rows * jb.cols / 8, jb.aux2, section[t], sections[t]};
            }
            rc = mq_nvfp4_quant_launch_group(jobs[i].dtype, tab, jobs[i].p0, jobs[i].p1 & ~MQ_NVFP4_CARRY_AMAX, carry ? 2 : 1, st);
            if (rc) return rc;
        } else {
            for (int t = 0; t < n; t++) {
                const mq_job& jb = jobs[i + t];
                int rc = mq_nvfp4_amax(jb.in, jb.dtype, jb.rows * jb.cols, jb.aux, section[t], stream);
                if (rc) return rc;
            }
            for (int t = 0; t < n; t++) {
                const mq_job& jb = jobs[i + t];
                int rc = mq_nvfp4_quant(jb.in, jb.dtype, jb.aux, sections[t], jb.out, jb.scale, (float*)jb.aux2, jb.rows,
                                        jb.cols, jb.p0, jb.p1 & ~MQ_NVFP4_CARRY_AMAX, stream);
                if (rc) return rc;
            }
        }
        i = k;
    }
    return mq_check_launch("nvfp4 group");
}

extern "C" int mq_job_table_fill(const mq_job* jobs, int64_t n, void* host_table) {
    if (n < 0 || (n > 0 && (!jobs || !host_table))) return mq_fail(MQ_ERR_ARG, "bad job list");
    for (int64_t i = 0; i < n; i++) {
        char* slot = (char*)host_table + i * MQ_JOB_TABLE_ENTRY_BYTES;
        if (tile_kind(jobs[i].kind) && job_fast(jobs[i])) {
            TileJob e = tile_entry(jobs[i]);
            mq_fp8_tile_job_finish(e);
            memcpy(slot, &e, sizeof(e));
        } else if (jobs[i].kind == MQ_JOB_NVFP4) {
            const mq_job& jb = jobs[i];
            int section, sections;
            nvfp4_sections(jobs, n, i, section, sections);
            const FlatJob e{jb.in, jb.out, jb.scale, jb.aux, jb.rows * jb.cols / 8, jb.aux2, section, sections};
            memcpy(slot, &e, sizeof(e));
        } else {
            const FlatJob e = table_kind(jobs[i].kind) && !tile_kind(jobs[i].kind) ? flat_entry(jobs[i]) : FlatJob{};
            memcpy(slot, &e, sizeof(e));
        }
    }
    return MQ_OK;
}

extern "C" int mq_run_jobs(const mq_job* jobs, int64_t n, void* stream) { return mq_run_jobs_tabled(jobs, n, nullptr, stream); }

extern "C" int mq_run_jobs_feedback(const mq_job* jobs, int64_t n, const void* device_table, uint32_t* device_moved,
                                    uint32_t* host_mirror, void* stream) {
    if ((uintptr_t)device_moved % 4 != 0 || (uintptr_t)host_mirror % 4 != 0)
        return mq_fail(MQ_ERR_ARG, "feedback counters and their mirror must be 4-byte aligned");
    if (host_mirror && !device_moved) return mq_fail(MQ_ERR_ARG, "a feedback mirror needs the device counters it mirrors");
    uint32_t* mirror = nullptr;
    if (host_mirror) {
        // the fold kernels store through this address: it has to be host memory the GPU can write (pinned, mapped)
        hipPointerAttribute_t attr;
        if (hipPointerGetAttributes(&attr, host_mirror) != hipSuccess || attr.type != hipMemoryTypeHost || !attr.devicePointer) {
            (void)hipGetLastError();
            return mq_fail(MQ_ERR_ARG, "the feedback mirror must be pinned host memory (hipHostMalloc)");
        }
        mirror = (uint32_t*)attr.devicePointer;
    }
    mq_set_amax_feedback(device_moved, mirror);
    const int rc = mq_run_jobs_tabled(jobs, n, device_table, stream);
    mq_set_amax_feedback(nullptr, nullptr);
    return rc;
}

extern "C" int mq_run_jobs_tabled(const mq_job* jobs, int64_t n, const void* device_table, void* stream) {
    if (n < 0 || (n > 0 && !jobs)) return mq_fail(MQ_ERR_ARG, "bad job list");
    if ((uintptr_t)device_table % 8 != 0) return mq_fail(MQ_ERR_ARG, "job table must be 8-byte aligned");
    const FlatJob* table = (const FlatJob*)device_table;
    hipStream_t st = (hipStream_t)stream;
    for (int64_t i = 0; i < n; i++) {
        int rc = check_job(jobs[i]);
        if (rc) return rc;
    }
    int64_t i = 0;
    while (i < n) {
        const mq_job& head = jobs[i];
        if (head.kind == MQ_JOB_NVFP4 || head.kind == MQ_JOB_FP8_TENSOR) {
            int64_t j = i + 1;
            while (j < n && jobs[j].kind == head.kind) j++;
            int rc = head.kind == MQ_JOB_NVFP4 ? run_nvfp4(jobs, n, i, j, table, stream) : run_fp8_tensor(jobs, i, j, table, stream);
            if (rc) return rc;
            i = j;
            continue;
        }
        if (head.rows == 0 || head.cols == 0) { i++; continue; }
        if (!job_fast(head)) {
            if (head.rows_per_block != 0) return mq_fail(MQ_ERR_ARG, "row-blocked input must be 16-byte aligned, with fewer than 2^24 columns and a block stride below 2^31 elements");
            int rc = run_single(head, stream);
            if (rc) return rc;
            i++;
            continue;
        }
        // flat kinds run on a (largest tensor) x (tensors) grid: keep the padding of a group under 25 %
        const bool flat = head.kind != MQ_JOB_FP8_BLOCK && head.kind != MQ_JOB_FP8_BLOCKWISE_CAST &&
                          head.kind != MQ_JOB_FP8_BLOCK_POW2 && head.kind != MQ_JOB_COPY;
        const bool tabled = table != nullptr && table_kind(head.kind);
        if (tabled && tile_kind(head.kind)) {
            // tile jobs of similar tile counts (an MoE layer's experts) beyond what the kernel arguments hold: one launch
            // on a (largest tile count) x (tensors) grid; mixed shapes keep the searched form below, 64 tensors at a time
            int64_t j = i + 1, sum = tiles_of(head), mx = sum;
            while (j < n && j - i < kTableGroup && same_group(head, jobs[j]) && job_fast(jobs[j]) && jobs[j].rows > 0 &&
                   jobs[j].cols > 0) {
                const int64_t e = tiles_of(jobs[j]);
                const int64_t nmx = e > mx ? e : mx;
                if (nmx * (j - i + 1) * 4 > (sum + e) * 5) break;
                sum += e;
                mx = nmx;
                j++;
            }
            j = tile_run_end(jobs, i, j, sum);
            // (tensors of 256 tiles and more fill a searched launch of 64 well enough, and run 1-2 % faster in that form)
            if (j - i > kMaxGroup && mx < 256) {
                const int mode = head.kind == MQ_JOB_FP8_BLOCK ? 0 : head.kind == MQ_JOB_FP8_BLOCKWISE_CAST ? 1 : 2;
                int rc = mq_fp8_tile_launch_table(mode, head.dtype, (const TileJob*)table + i, (int)(j - i), mx, st);
                if (rc) return rc;
                i = j;
                continue;
            }
        }
        const int64_t group_cap = tabled && !tile_kind(head.kind) ? kTableGroup : kMaxGroup;
        int64_t j = i + 1, sum = head.rows * head.cols, mx = sum;
        while (j < n && j - i < group_cap && same_group(head, jobs[j]) && job_fast(jobs[j]) && jobs[j].rows > 0 &&
               jobs[j].cols > 0) {
            const int64_t e = jobs[j].rows * jobs[j].cols;
            const int64_t nmx = e > mx ? e : mx;
            if (flat && nmx * (j - i + 1) * 4 > (sum + e) * 5) break;
            if (head.kind == MQ_JOB_COPY && copy_depends_on_group(jobs, i, j)) break;
            sum += e;
            mx = nmx;
            j++;
        }
        if (tile_kind(head.kind)) {
            int64_t tiles = 0;
            for (int64_t t = i; t < j; t++) tiles += tiles_of(jobs[t]);
            j = tile_run_end(jobs, i, j, tiles);
        }
        const int cnt = (int)(j - i);
        int rc = MQ_OK;
        switch (head.kind) {
            case MQ_JOB_FP8_BLOCK:
            case MQ_JOB_FP8_BLOCKWISE_CAST:
            case MQ_JOB_FP8_BLOCK_POW2: {
                TileTable tab{};
                tab.n = cnt;
                for (int t = 0; t < cnt; t++) {
                    const mq_job& jb = jobs[i + t];
                    tab.job[t] = tile_entry(jb);
                }
                rc = mq_fp8_tile_launch_group(head.kind == MQ_JOB_FP8_BLOCK ? 0 : head.kind == MQ_JOB_FP8_BLOCKWISE_CAST ? 1 : 2, head.dtype, tab, st);
                break;
            }
            case MQ_JOB_FP8_DEQUANT: {
                MqDequantArgs a[kMaxGroup];
                for (int t = 0; t < cnt; t++) {
                    const mq_job& jb = jobs[i + t];
                    a[t] = MqDequantArgs{jb.in, (const float*)jb.aux, jb.out, jb.rows, jb.cols, jb.p0};
                }
                rc = mq_fp8_dequant_launch_group(a, cnt, st);
                break;
            }
            case MQ_JOB_MXFP8:
            case MQ_JOB_MXFP4:
            case MQ_JOB_INT4_PACK:
            case MQ_JOB_INT4_PACK_ASYM: {
                if (tabled && cnt > kMaxGroup) {        // small groups keep the kernel-argument form (no pointer chase)
                    int64_t zero_tiles = 0;
                    if (head.kind == MQ_JOB_INT4_PACK_ASYM)
                        for (int t = 0; t < cnt; t++) {
                            const int64_t tiles = mq_int4_zero_tiles(jobs[i + t].rows, jobs[i + t].cols, head.p0);
                            zero_tiles = tiles > zero_tiles ? tiles : zero_tiles;
                        }
                    rc = head.kind == MQ_JOB_MXFP8       ? mq_mxfp8_launch_table(head.dtype, table + i, cnt, mx / 8, st)
                         : head.kind == MQ_JOB_MXFP4     ? mq_mxfp4_launch_table(head.dtype, table + i, cnt, mx / 8, st)
                         : head.kind == MQ_JOB_INT4_PACK ? mq_int4_pack_launch_table(head.dtype, table + i, cnt, mx / 8, head.p0, st)
                                                         : mq_int4_pack_asym_launch_table(head.dtype, table + i, cnt, mx / 8, zero_tiles, head.p0, st);
                    break;
                }
                FlatTable tab{};
                tab.n = cnt;
                for (int t = 0; t < cnt; t++) tab.job[t] = flat_entry(jobs[i + t]);
                rc = head.kind == MQ_JOB_MXFP8       ? mq_mxfp8_launch_group(head.dtype, tab, st)
                     : head.kind == MQ_JOB_MXFP4     ? mq_mxfp4_launch_group(head.dtype, tab, st)
                     : head.kind == MQ_JOB_INT4_PACK ? mq_int4_pack_launch_group(head.dtype, tab, head.p0, st)
                                                     : mq_int4_pack_asym_launch_group(head.dtype, tab, head.p0, st);
                break;
            }
            case MQ_JOB_FP8_TO_MXFP8: {
                MqRescaleArgs a[kMaxGroup];
                for (int t = 0; t < cnt; t++) {
                    const mq_job& jb = jobs[i + t];
                    a[t] = MqRescaleArgs{jb.in, (const float*)jb.aux, jb.out, (uint8_t*)jb.scale, jb.rows, jb.cols, jb.ld};
                }
                rc = mq_fp8_to_mxfp8_launch_group(a, cnt, st);
                break;
            }
            case MQ_JOB_INT4_UNPACK:
            case MQ_JOB_MXFP4_DEQUANT: {
                FlatTable tab{};
                tab.n = cnt;
                for (int t = 0; t < cnt; t++) {
                    const mq_job& jb = jobs[i + t];
                    tab.job[t] = head.kind == MQ_JOB_INT4_UNPACK
                                     ? mq_int4_unpack_entry(jb.in, jb.aux, jb.out, jb.rows, jb.cols, jb.p0)
                                     : mq_mxfp4_dequant_entry(jb.in, jb.aux, jb.out, jb.rows * jb.cols / 2, jb.p0);
                }
                rc = head.kind == MQ_JOB_INT4_UNPACK ? mq_int4_unpack_launch_group(head.dtype, tab, st)
                                                     : mq_mxfp4_dequant_launch_group(tab, st);
                break;
            }
            case MQ_JOB_MXFP4_TO_FP8: {
                RecodeTable tab{};
                tab.n = cnt;
                for (int t = 0; t < cnt && rc == MQ_OK; t++) {
                    const mq_job& jb = jobs[i + t];
                    rc = mq_mxfp4_to_fp8_job(tab.job[t], jb.in, jb.aux, jb.out, jb.scale, jb.rows, jb.cols);
                }
                if (rc == MQ_OK) rc = mq_mxfp4_to_fp8_launch_group(tab, st);
                break;
            }
            case MQ_JOB_COPY: {
                // long aligned runs stream best from a launch of their own; everything else shares one grouped launch
                CopyTable tab{};
                for (int t = 0; t < cnt && rc == MQ_OK; t++) {
                    const mq_job& jb = jobs[i + t];
                    const int64_t bytes = jb.rows * jb.cols;
                    const bool aligned = (((uintptr_t)jb.in | (uintptr_t)jb.out) & 15) == 0;
                    const bool one_run = jb.rows == 1 || (jb.ld == jb.cols && copy_dst_pitch(jb) == jb.cols);
                    if (one_run && aligned && bytes >= (64 << 20)) rc = mq_copy_launch_run(jb.in, jb.out, bytes, st);
                    else if (one_run) tab.job[tab.n++] = CopyJob{(const uint8_t*)jb.in, (uint8_t*)jb.out, bytes, 0, 0, 1, 0};
                    else tab.job[tab.n++] = CopyJob{(const uint8_t*)jb.in, (uint8_t*)jb.out, jb.cols, jb.ld, copy_dst_pitch(jb),
                                                    (int32_t)jb.rows, 0};
                }
                if (rc == MQ_OK && tab.n > 0) rc = mq_copy_launch_group(tab, st);
                break;
            }
            default:
                rc = mq_fail(MQ_ERR_ARG, "unknown job kind");
        }
        if (rc) return rc;
        i = j;
    }
    return MQ_OK;
}
