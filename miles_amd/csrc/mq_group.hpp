// Grouped launches: one kernel launch covers up to kMaxGroup tensors.  The per-tensor descriptors travel
// in the kernel argument segment (no device allocation, no host-to-device copy); a workgroup finds its
// tensor by scanning the running workgroup counts, which the compiler keeps in scalar registers.
//
// Workgroup ids are first remapped: the eight XCDs receive consecutive workgroup ids round-robin, and each XCD has
// its own L2.  Work items are dealt to the XCDs in small chunks of consecutive items (four 128x128 tiles = 1 KiB
// of every tile row), so the workgroups an XCD runs at any moment touch neighbouring addresses, while every XCD sees
// the same mix of tensors and none of them finishes long after the others.
#pragma once
#include <stdint.h>

namespace mq {

constexpr int kMaxGroup = 64;
constexpr int kXcds = 8;

// work item (after remap) of this workgroup, or -1 if it falls past the end
// Measured on the Qwen3-4B FP8 sync (MI355X): chunks of 4 tiles 6.28 TB/s, 16: 6.27, 64: 6.21, 512: 5.74, one contiguous
// eighth per XCD 5.97, no remap at all (chunk 1) 5.9.
#ifndef MQ_XCD_CHUNK
#define MQ_XCD_CHUNK 4
#endif
__device__ __forceinline__ int32_t xcd_contiguous_item(int32_t total) {
    const int32_t bid = blockIdx.x;
    const int32_t x = bid % kXcds, k = bid / kXcds;
    if (MQ_XCD_CHUNK > 0) {
        // chunks of MQ_XCD_CHUNK consecutive items go to the XCDs round-robin: locality inside a chunk, and every XCD
        // sees the same mix of tensors, so none of them finishes long after the others
        const int32_t item = ((k / MQ_XCD_CHUNK) * kXcds + x) * MQ_XCD_CHUNK + (k % MQ_XCD_CHUNK);
        return item < total ? item : -1;
    }
    const int32_t per = (total + kXcds - 1) / kXcds;
    const int32_t item = x * per + k;
    return (k < per && item < total) ? item : -1;
}
inline int64_t xcd_grid(int64_t total) {
    const int64_t unit = (int64_t)kXcds * (MQ_XCD_CHUNK > 0 ? MQ_XCD_CHUNK : 1);
    return ((total + unit - 1) / unit) * unit;
}

// the same dealing with a chunk length chosen at launch time (a whole row band of a matrix, say)
__device__ __forceinline__ int32_t xcd_chunked_item(int32_t total, int32_t chunk) {
    const int32_t bid = blockIdx.x;
    const int32_t x = bid % kXcds, k = bid / kXcds;
    const int32_t item = ((k / chunk) * kXcds + x) * chunk + (k % chunk);
    return item < total ? item : -1;
}
inline int64_t xcd_grid_chunked(int64_t total, int64_t chunk) {
    const int64_t unit = (int64_t)kXcds * chunk;
    return ((total + unit - 1) / unit) * unit;
}

struct TileJob {      // one 2-D tensor cut into 128x128 tiles
    const void* w;
    void* q;
    float* scale;
    int32_t ldw;              // input row stride, elements (below 2^24)
    int32_t M, K;
    int32_t block_stride;     // elements between the first rows of consecutive row blocks (row-blocked inputs)
    int32_t tiles_per_block;  // tile rows per input row block, 0 = plain matrix
    uint32_t magic_k, magic_b;  // tile_div constants for division by the tiles per row and by tiles_per_block
    uint32_t shifts;            // their shifts: the first in bits 0-7, the second in bits 8-15
};
// n / d for any 32-bit n from constants made on the host for a divisor d >= 2 (round-up multiply-high method):
// t = mulhi(magic, n); n / d = (t + ((n - t) >> 1)) >> shift.  Both values are uniform over a workgroup, so the three
// operations run on the scalar unit.
inline void tile_div_magic(uint32_t d, uint32_t& magic, uint32_t& shift) {
    uint32_t l = 0;
    while ((1ull << l) < d) l++;                 // ceil(log2 d) >= 1
    magic = (uint32_t)((((1ull << l) - d) << 32) / d + 1);
    shift = l - 1;
}
__device__ __forceinline__ uint32_t tile_div(uint32_t n, uint32_t magic, uint32_t shift) {
    const uint32_t t = __umulhi(magic, n);
    return (t + ((n - t) >> 1)) >> shift;
}
struct TileTable {
    int32_t n;
    int32_t total;            // all work items of the launch
    int32_t end[kMaxGroup];   // running count of tiles: tensor i owns [end[i-1], end[i]); INT32_MAX past n
    TileJob job[kMaxGroup];
};

// Tile descriptors in device memory (see FlatRef below): tensors of similar tile counts on a two-dimensional grid,
// blockIdx.y the tensor and blockIdx.x the tile (gridDim.x is the largest count, rounded up for the XCD dealing), so no
// search is needed however many tensors the launch covers.
struct TileRef {
    const TileJob* job;
};

struct FlatJob {      // one tensor seen as a flat run of 16-byte input units
    const void* w;
    void* q;
    void* s;
    void* aux;        // NVFP4: amax record; unused otherwise
    int64_t units;
    void* aux2;       // NVFP4: fp32 global scale output; unused otherwise
    int32_t section;  // NVFP4 amax: section of the record to write; quantize: number of sections to read
    int32_t pad;
};
// Flat kernels are launched on a 2-D grid: blockIdx.y selects the tensor, blockIdx.x the workgroup inside
// it, so a workgroup reads its descriptor with one scalar load and no search.  grid.x is the largest
// per-tensor workgroup count of the group; the batched driver only groups tensors of similar size.
struct FlatTable {
    int32_t n;
    int32_t max_blocks;
    int32_t chunk;            // workgroups per XCD chunk (see flat_block); max_blocks is a multiple of 8 * chunk
    int32_t pad;
    FlatJob job[kMaxGroup];
};
// Flat kernels stream a tensor front to back.  Consecutive workgroup ids go to the eight XCDs in turn; the block a
// workgroup works on is remapped so that an XCD takes runs of `chunk` consecutive blocks (up to MQ_FLAT_CHUNK,
// 512 KiB of bf16 input at two units per lane) instead of every eighth one.  Measured on MI355X with chunks of
// up to 64: MXFP4 quantize 6.42 -> 6.75 TB/s, MXFP8 on [768,2048] experts 6.20 -> 6.35, INT4 pack 6.40 -> 6.48.
// The grid is padded to a whole number of 8 * chunk workgroups (surplus ones exit); the chunk is the largest of
// 1, 2, 3, 4, 6, 8, ... 48, 64 whose padding stays under 3 %.
#ifndef MQ_FLAT_CHUNK
#define MQ_FLAT_CHUNK 64
#endif
// `chunk` is a power of two or three times one (flat_chunk makes no other), so the division is a shift, or a shift and
// the multiply-high division by three, which is exact for every 32-bit value: a division by a run-time value costs every
// wavefront some forty dependent scalar instructions before its first load (the shift measured 0.5 to 3 % faster on every
// flat kernel).  The threefold chunks matter for tensors such as the [768, 2048] experts of Qwen3-30B-A3B: 384
// workgroups, which a power of two above 16 would pad by a third, split into runs of 48 exactly (MXFP8 6.49 -> 6.8 TB/s).
__device__ __forceinline__ int64_t xcd_chunked_block(int32_t chunk) {
    const int32_t bid = blockIdx.x, x = bid % kXcds, k = bid / kXcds;
    const int32_t shift = __builtin_ctz((uint32_t)chunk);
    const uint32_t shifted = (uint32_t)k >> shift;
    const uint32_t run = (chunk >> shift) == 3 ? __umulhi(shifted, 0xAAAAAAABu) >> 1 : shifted;      // k / chunk
    return (int64_t)(run * kXcds + x) * chunk + (k - (int32_t)run * chunk);
}
// The same descriptors kept in device memory by a caller that submits one job list again and again: a launch is then not
// bound to the kMaxGroup tensors that fit the kernel arguments.  A model of thousands of small tensors (MoE experts of
// 3 MB) otherwise pays a launch boundary -- the chip draining and filling again, about 4 us -- per 64 of them, 8 % of
// such a sync.  Kernels are templates over the two forms and read their descriptor with scalar loads either way.
struct FlatRef {
    const FlatJob* job;       // device memory, one entry per tensor of the launch (blockIdx.y)
    int32_t chunk;
    int32_t max_blocks;
};
constexpr int kTableGroup = 8192;         // tensors per launch of the device-table form (gridDim.y stays below 65 536)
// the descriptor of this workgroup's tensor, copied into registers (a descriptor in device memory must not be read
// again after the kernel's own stores) with its pointers loaded as global ones (see load_global_ptr)
template <class Table>
__device__ __forceinline__ FlatJob flat_job(const Table& tab) {
    const FlatJob& src = tab.job[blockIdx.y];
    FlatJob j;
    j.w = load_global_ptr(&src.w);
    j.q = load_global_ptr(&src.q);
    j.s = load_global_ptr(&src.s);
    j.aux = load_global_ptr(&src.aux);
    j.units = src.units;
    j.aux2 = load_global_ptr(&src.aux2);
    j.section = src.section;
    j.pad = src.pad;
    return j;
}
template <class Table>
__device__ __forceinline__ int64_t flat_block(const Table& tab) { return xcd_chunked_block(tab.chunk); }
// largest chunk of the form 2^a or 3 * 2^a (up to MQ_FLAT_CHUNK) whose grid padding stays under 3 % of `blocks` workgroups
inline int64_t flat_chunk(int64_t blocks) {
    int64_t chunk = 1;
    for (int64_t c : {2, 3, 4, 6, 8, 12, 16, 24, 32, 48, 64}) {
        if (c > MQ_FLAT_CHUNK) break;
        const int64_t padded = (blocks + c * kXcds - 1) / (c * kXcds) * (c * kXcds);
        if ((padded - blocks) * 32 <= blocks) chunk = c;
    }
    return chunk;
}
inline int64_t flat_padded(int64_t blocks, int64_t chunk) {
    return (blocks + chunk * kXcds - 1) / (chunk * kXcds) * (chunk * kXcds);
}
// workgroups a tensor of `units` 16-byte units needs when each covers `per_block` units; fills max_blocks
inline bool flat_grid(FlatTable& tab, int64_t per_block) {
    int64_t mx = 0;
    for (int i = 0; i < tab.n; i++) {
        const int64_t b = (tab.job[i].units + per_block - 1) / per_block;
        if (b > mx) mx = b;
    }
    const int64_t chunk = flat_chunk(mx);
    mx = flat_padded(mx, chunk);
    tab.chunk = (int32_t)chunk;
    tab.max_blocks = (int32_t)mx;
    return mx < 0x7FFFFFF0;
}
// the same for a device table whose largest tensor has `max_units` units
inline bool flat_grid(FlatRef& ref, int64_t max_units, int64_t per_block) {
    int64_t mx = (max_units + per_block - 1) / per_block;
    const int64_t chunk = flat_chunk(mx);
    mx = flat_padded(mx, chunk);
    ref.chunk = (int32_t)chunk;
    ref.max_blocks = (int32_t)mx;
    return mx < 0x7FFFFFF0;
}

// one MXFP4 tensor re-coded as FP8 with 128 x 128 scales: a workgroup takes a pair of tiles, neighbours along `in`
struct RecodeJob {
    const uint8_t* packed;    // [out, in / 2] e2m1 pairs
    const uint8_t* scale;     // [out, in / 32] E8M0 bytes
    uint8_t* y;               // [out, in] e4m3
    float* tile_scale;        // [out / 128, in / 128]
    int64_t in_dim;
    int32_t tiles_in, pairs_in, total_pairs;
    int32_t chunk;            // tile pairs an XCD takes in a row (tile form)
    // flat form: 16-element units, tile_div constants for units per row, XCD run length of the flat grid
    uint32_t units, magic_upr, shift_upr;
    int32_t flat_chunk;
};
struct RecodeTable {
    int32_t n;
    RecodeJob job[kMaxGroup];
};

// The amax record of the quantizers that need a whole-tensor maximum (NVFP4, per-tensor FP8): kRecordSections
// sections of kSectionWords partial maxima (float bit patterns), then the folded amax and what is derived from it.
constexpr int kSectionWords = 256;      // MQ_NVFP4_SECTION_WORDS: workgroups of an amax pass per tensor
constexpr int kRecordSections = 4;      // MQ_NVFP4_SECTIONS
constexpr int kRecAmax = kRecordSections * kSectionWords;      // folded amax (float bits)
constexpr int kRecRedo = kRecAmax + 4;  // the amax carried over from the last run turned out stale: quantize again
constexpr int kRecVolatile = kRecAmax + 5;  // the amax moved on the last two runs: the next carried run collects the amax first
constexpr int kRecMovedRuns = kRecAmax + 6; // carried runs in a row on which the amax moved (counted up to two)
// What a fold of a carried run does with a record once it knows whether the amax moved.  A record that moved is
// quantized a second time on this run (its codes were written with the stale amax).  Only a record that moved on two
// runs in a row is marked volatile: the next carried run then just collects its amax in the single pass and quantizes
// in the second one -- the plain two-pass cost, 4.56 bytes per element where a wasted quantization costs 5.12 -- until
// the amax has held still for one run.  One move alone does not mark it: with an optimizer step between the syncs a
// tensor's amax moves on one sync in five or so, mostly not on the next one too, and a record marked after a single move
// paid the two-pass cost for nothing on the sync after every move.
__device__ __forceinline__ void amax_record_after_carried_run(uint32_t* rec, bool moved) {
    rec[kRecRedo] = (moved || rec[kRecVolatile] != 0) ? 1u : 0u;     // a volatile record has no codes yet
    const uint32_t runs = moved ? (rec[kRecMovedRuns] >= 1u ? 2u : 1u) : 0u;
    rec[kRecMovedRuns] = runs;
    rec[kRecVolatile] = runs >= 2u ? 1u : 0u;
}
// A fold launched by the job driver also tells its caller how many tensors' records held another amax before, and how
// many tensors it folded (two counters in device memory that only ever grow: a copy taken at any time gives a
// consistent rate): a caller whose every amax keeps moving can then submit the plain two-pass form.
__device__ __forceinline__ void amax_feedback(uint32_t* counter, bool moved, uint32_t tensors) {
    if (counter && moved) atomicAdd(counter, tensors);
}
// Once per fold launch: first the two counters as the launches before left them (a consistent pair) go to the caller's
// host-visible mirror, if the call named one (a kernel argument: the host checked that it is pinned memory), then this
// launch's tensors are added to the second counter.
__device__ __forceinline__ void amax_feedback_folded(uint32_t* counter, uint32_t* mirror_words, uint32_t tensors) {
    if (counter && blockIdx.x == 0 && threadIdx.x == 0) {
        if (mirror_words) {
            volatile uint32_t* mirror = mirror_words;
            const uint32_t moved = atomicAdd(counter, 0u), folded = atomicAdd(counter + 1, 0u);
            mirror[0] = moved;
            mirror[1] = folded;
        }
        atomicAdd(counter + 1, tensors);
    }
}

struct CopyJob {      // rows of `bytes` bytes each (one row: a plain run), chunks_per_row chunks of the copy kernel per row
    const uint8_t* src;
    uint8_t* dst;
    int64_t bytes;
    int64_t src_pitch, dst_pitch;
    int32_t chunks_per_row;
    int32_t pad;
};
struct CopyTable {
    int32_t n;
    int32_t total;            // all chunks of the launch
    int32_t end[kMaxGroup];   // running chunk counts, as in TileTable
    CopyJob job[kMaxGroup];
};

// Index of the tensor that owns work item `item`: the number of running counts not above it.  The loop has
// a fixed trip count and no early exit, so the compiler fetches the whole `end` array with a few wide scalar
// loads and the comparison chain runs on the scalar unit: a short, latency-free prologue even for
// workgroups that only move a few KiB.
struct JobRef {
    int ji;         // index into tab.job
    int32_t start;  // first work item of that tensor
};
template <class Table>
__device__ __forceinline__ JobRef find_job(const Table& tab, int32_t item) {
    // `item` is uniform over the workgroup, and so is everything here: the count is kept on the scalar unit with a
    // compare and an add-with-carry per entry.  (Left to the compiler the chain ended up on the vector unit -- two
    // vector operations per entry, or, with the descriptor selected inside the loop, a vector multiply-add per entry
    // to build its address: a quarter to a half of the vector work of a whole 128x128 tile.)
    int32_t ji = 0;
#pragma unroll
    for (int i = 0; i < kMaxGroup - 1; i++) {
        const int32_t e = tab.end[i];
        asm("s_cmp_ge_i32 %1, %2\n\ts_addc_u32 %0, %0, 0" : "+s"(ji) : "s"(item), "s"(e) : "scc");
    }
    return JobRef{ji, ji > 0 ? tab.end[ji - 1] : 0};
}
// host side: after end[0..n) holds the running counts, record the total and pad the rest of `end`
template <class Table>
inline void seal_table(Table& tab) {
    tab.total = tab.n > 0 ? tab.end[tab.n - 1] : 0;
    for (int i = tab.n > 0 ? tab.n - 1 : 0; i < kMaxGroup; i++) tab.end[i] = 0x7FFFFFFF;
}

}  // namespace mq
