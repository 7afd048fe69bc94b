// join_device.hpp -- device-side pieces shared by the join kernels: parameter block, counter layout, the
// fused distance test.  Included by the .hip files only.
#pragma once
#include <hip/hip_runtime.h>

#include "tile_order.hpp"

namespace fasted {
namespace {

typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef float floatx4 __attribute__((ext_vector_type(4)));
typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));

// Counter block of one join: word 0 = pairs found, word 1 = non-finite flag, word 2 = a clock reading, word 3 =
// workgroups of the join kernel that have signed off; then the 8 queue heads, each on its own 128-byte line; then,
// on a line of its own again (it is read by every workgroup while the first line is busy with atomics), where the
// join kernel reports to the host.
constexpr int kCounterFound = 0;
constexpr int kCounterNonFinite = 1;  // == the join's epoch: some point of the join has a non-finite squared norm
constexpr int kCounterStampNorms = 2;  // the device's constant-rate clock when the join's first norm kernel started
constexpr int kCounterDone = 3;        // workgroups of the join kernel that are through (the last one reports to the host)
constexpr int kQueueBase = 16, kQueueStride = 16;
// Set once by the owner of the block and never cleared by a kernel: the address (as the device sees it) of 4 words
// of pinned host memory, or 0: [0] pairs found, [1]-[3] clock readings (norms started, join kernel started, join
// kernel through).  It sits here and not among the kernel's arguments because the tile loop has no scalar
// registers to spare.
constexpr int kCounterHostWords = kQueueBase + kQueues * kQueueStride;
constexpr int kCounterWords = kCounterHostWords + 16;

struct JoinParams {
    const u32x4* ptsQ;  // query rows
    const u32x4* ptsC;  // candidate rows (the same buffer for a self-join)
    long long ldQ16, ldC16;  // row strides in 16-byte units
    int nQ, nC;
    int selfStride;  // != 0: (q, q * selfStride) is always a pair -- 1 for a self-join ((i, i) is a pair)
    int symmetric; // self-join only: compute tiles on and above the diagonal, emit (q,c) and (c,q)
    int nSlabs;    // 64-wide k-slabs per tile
    int direct;    // != 0: no more tiles than workgroups: workgroup b computes tile b and nothing else (no queues)
    const float* halfQ;  // per query point: eps^2/4 - s/2, s = squared norm
    const float* halfC;  // ... per candidate point
    unsigned long long* counters;
    unsigned long long epoch;  // number of this join (never 0): the value of the non-finite flag that counts
    int2* pairs;
    unsigned long long cap;
    TileOrder raster;
};

// Lane number 0..63, re-derived from the execution mask where it is needed.  Volatile on purpose: the
// optimiser then cannot hoist it (and what is derived from it) out of the tile loop, where it would
// occupy registers, or spill, across the k loop.
__device__ __forceinline__ int lane_now() {
    int l;
    asm volatile("v_mbcnt_lo_u32_b32 %0, -1, 0\n\tv_mbcnt_hi_u32_b32 %0, -1, %0" : "=v"(l));
    return l;
}

}  // namespace
}  // namespace fasted
