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

// Counter block of one join: word 0 = pairs found, then the 8 queue heads, each on its own 128-byte line.
constexpr int kCounterFound = 0;
constexpr int kQueueBase = 16, kQueueStride = 16;
constexpr int kCounterWords = kQueueBase + kQueues * kQueueStride;

struct JoinParams {
    const u32x4* ptsQ;  // query rows
    const u32x4* ptsC;  // candidate rows (the same buffer for a self-join)
    long long ldQ16, ldC16;  // row strides in 16-byte units
    int nQ, nC;
    int selfJoin;  // queries and candidates are the same set: (i, i) is always a pair
    int symmetric; // self-join only: compute tiles on and above the diagonal, emit (q,c) and (c,q)
    int nSlabs;    // 64-wide k-slabs per tile
    float eps2;
    const float* sumsQ;
    const float* sumsC;
    unsigned long long* counters;
    int2* pairs;
    unsigned long long cap;
    TileOrder raster;
};

// Distance test of one wave's block of accumulators (kFragRows x kFragCols MFMA blocks of 16x16, kFragCols = 4:
// 128x64 or 64x64 points).  acc[fi][fj] is a 16x16 MFMA block:
// lane l holds column l%16 and rows 4*(l/16) .. +3, i.e. 4 elements per block.
//
// The accumulators start at -(s_q + s_c)/2 instead of 0, so what arrives here is
//     a = q.c - (s_q + s_c)/2 = -dist^2 / 2
// and the reference's test  s_q + s_c - 2 q.c <= eps^2  (source/warpMma.cuh:241-257) reads
//     a >= -eps^2/2,
// one threshold for every element, exact in FP32 (the scaling by 2 is exact), and symmetric in q and c
// like the reference's.  Screening, about 1/2 VALU op per element: the maximum of the lane's 128 elements
// (formed per row of blocks) against the threshold; a wave in which no lane has a hit is done.  Otherwise
// the rows of blocks with a hit somewhere in the wave yield their per-element bits, branch-free.
//
// kEdge: the tile touches the diagonal of a self-join or the ragged end of a dataset; self pairs are
// forced and padded rows/cols are masked (source/warpMma.cuh:257-259).
// Returns per-lane hit bits, shifted in from the right in evaluation order: element e = (fi&1)*16 + fj*4 + r
// of the pair of row blocks fi/2 ends up in bit 31 - e of mask[fi/2].
template <int kFragRows, int kFragCols, bool kEdge>
__device__ __forceinline__ void test_block(const floatx4 (&acc)[kFragRows][kFragCols], const int (&cand)[kFragCols],
                                           int qBase, int quad, int nQ, int nC, int selfJoin, float thr,
                                           unsigned (&mask)[kFragRows / 2]) {
    if (kEdge) {
        // every element is tested; branch-free, in the form of the fast path below: the sign of x - thr is
        // shifted in, where x is the accumulator, +inf for a self pair, -inf for a padded row or column
        // (and for a NaN); thr is finite
        const float inf = __builtin_inff();
        bool candReal[kFragCols];
#pragma unroll
        for (int fj = 0; fj < kFragCols; ++fj) candReal[fj] = cand[fj] < nC;
#pragma unroll
        for (int fp = 0; fp < kFragRows / 2; ++fp) {
            unsigned m = 0;
#pragma unroll
            for (int h = 0; h < 2; ++h) {
                const int fi = fp * 2 + h;
#pragma unroll
                for (int fj = 0; fj < kFragCols; ++fj) {
#pragma unroll
                    for (int r = 0; r < 4; ++r) {
                        const int q = qBase + fi * 16 + quad * 4 + r;
                        float x = __builtin_fmaxf(acc[fi][fj][r], -inf);
                        x = ((selfJoin != 0) & (q == cand[fj])) ? inf : x;
                        x = ((q < nQ) & candReal[fj]) ? x : -inf;
                        m = __builtin_amdgcn_alignbit(m, __builtin_bit_cast(unsigned, x - thr), 31);
                    }
                }
            }
            mask[fp] = ~m;
        }
        return;
    }
    // maximum of every row of blocks (16 elements per lane), then of all of them
    float rowBest[kFragRows];
#pragma unroll
    for (int fi = 0; fi < kFragRows; ++fi) {
        float best = acc[fi][0][0];
#pragma unroll
        for (int fj = 0; fj < kFragCols; ++fj)
#pragma unroll
            for (int r = 0; r < 4; ++r) best = __builtin_fmaxf(best, acc[fi][fj][r]);
        rowBest[fi] = best;
    }
    float best = rowBest[0];
#pragma unroll
    for (int fi = 1; fi < kFragRows; ++fi) best = __builtin_fmaxf(best, rowBest[fi]);
    if (__builtin_amdgcn_ballot_w64(best >= thr) == 0ull) {
#pragma unroll
        for (int fp = 0; fp < kFragRows / 2; ++fp) mask[fp] = 0u;
        return;
    }
    // some lane has a hit: rows of blocks without one (wave-wide) are skipped, the others yield their
    // bits: the sign of acc - thr (set = no hit) is shifted in; the maximum with -inf turns a NaN
    // (points with infinite coordinates) into "no hit", as every comparison with NaN is false
    unsigned long long rowHit[kFragRows];
#pragma unroll
    for (int fi = 0; fi < kFragRows; ++fi) rowHit[fi] = __builtin_amdgcn_ballot_w64(rowBest[fi] >= thr);
#pragma unroll
    for (int fp = 0; fp < kFragRows / 2; ++fp) {
        unsigned m = 0;
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            const int fi = fp * 2 + h;
            if (rowHit[fi] != 0ull) {
#pragma unroll
                for (int fj = 0; fj < kFragCols; ++fj)
#pragma unroll
                    for (int r = 0; r < 4; ++r)
                        m = __builtin_amdgcn_alignbit(
                            m, __builtin_bit_cast(unsigned, __builtin_fmaxf(acc[fi][fj][r], -__builtin_inff()) - thr), 31);
            } else {
                m = (m << 16) | 0xffffu;
            }
        }
        mask[fp] = ~m;
    }
}

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
