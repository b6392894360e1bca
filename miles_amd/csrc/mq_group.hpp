// Grouped launches: one kernel launch covers up to kMaxGroup tensors.  The per-tensor descriptors travel
// in the kernel argument segment (no device allocation, no host-to-device copy); a workgroup finds its
// tensor by scanning the running workgroup counts, which the compiler keeps in scalar registers.
//
// Workgroup ids are first remapped so that each of the eight XCDs (which receive consecutive workgroup
// ids round-robin) works on one contiguous eighth of the launch's work: the workgroups resident on an
// XCD at any moment then touch neighbouring addresses, which measurably raises achieved HBM bandwidth
// for the 128x128-tile access pattern.
#pragma once
#include <stdint.h>

namespace mq {

constexpr int kMaxGroup = 64;
constexpr int kXcds = 8;

// work item (after remap) of this workgroup, or -1 if it falls past the end
__device__ __forceinline__ int64_t xcd_contiguous_item(int64_t total) {
    const int64_t per = (total + kXcds - 1) / kXcds;
    const int64_t bid = blockIdx.x;
    const int64_t x = bid % kXcds, k = bid / kXcds;
    const int64_t item = x * per + k;
    return (k < per && item < total) ? item : -1;
}
inline int64_t xcd_grid(int64_t total) { return ((total + kXcds - 1) / kXcds) * kXcds; }

struct TileJob {      // one 2-D tensor cut into 128x128 tiles
    const void* w;
    void* q;
    float* scale;
    int64_t ldw;      // input row stride, elements
    int32_t M, K;
    int32_t tiles_k;
    int32_t pad;
};
struct TileTable {
    int32_t n;
    int32_t pad;
    int64_t end[kMaxGroup];   // running count of tiles: tensor i owns [end[i-1], end[i])
    TileJob job[kMaxGroup];
};

struct FlatJob {      // one tensor seen as a flat run of 16-byte input units
    const void* w;
    void* q;
    void* s;
    void* aux;        // NVFP4: amax word; unused otherwise
    int64_t units;
};
struct FlatTable {
    int32_t n;
    int32_t pad;
    int64_t end[kMaxGroup];   // running count of workgroups
    FlatJob job[kMaxGroup];
};

template <class Table>
__device__ __forceinline__ int find_job(const Table& tab, int64_t item) {
    int i = 0;
    while (i < tab.n - 1 && item >= tab.end[i]) i++;
    return i;
}

}  // namespace mq
