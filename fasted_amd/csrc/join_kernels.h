// join_kernels.h -- host-callable launchers of the gfx950 kernels (internal to libfasted).
#pragma once
#include <hip/hip_runtime.h>

#include <cstdint>

namespace fasted {

constexpr int kTile = 256;       // points per tile side (queries x candidates)
constexpr int kSlabK = 64;       // halves of K staged in LDS per pipeline stage
constexpr int kSquareTiles = 256; // tiles of a super-square of the work queues: one per workgroup of a full chip

struct JoinLaunch {
    const void* queries;         // FP16 rows
    const void* candidates;      // FP16 rows; the same buffer for a self-join
    long long ldQ, ldC;          // row strides in halves (multiples of 8)
    int nQ, nC;                  // real points
    bool selfJoin;               // same set on both sides: (i, i) always counts as a pair
    int forcedStride = 0;        // two sets where query i IS candidate i * forcedStride (a sample of the
                                 // candidates joined against all of them): that pair always counts
    bool symmetric;              // self-join: only tiles on/above the diagonal are computed, pairs mirrored
    int dPad;                    // K extent, multiple of kSlabK
    const float* halfQ;          // per query point: eps^2/4 - s/2 (s = squared norm), see launch_sum_squared
    const float* halfC;          // ... per candidate point
    unsigned long long* counters;  // counter_words() words: [0] pairs found, [1] non-finite flag, ..., then the queue
                                   // heads.  Word host_words_slot() is the owner's: the device-side address of 4
                                   // words of pinned host memory, or 0.  If set, the join kernel's last workgroup
                                   // writes [0] = pairs found and the device's constant-rate clock [1] when the
                                   // join's first norm kernel started and [3] (never 0) when it was through itself,
                                   // its first workgroup [2] when it started; every pair record of the join is in
                                   // memory when [3] appears.  The kernels of this file never clear that word.
    unsigned long long epoch = 1;  // number of the join: what the norm kernels of THIS join write into the
                                   // non-finite flag (a flag left by an earlier join is not seen)
    void* pairs;                 // FastedPair[cap]
    unsigned long long cap;
    bool epilogue;               // false: contraction only (measurement)
};

// Host mirror of the device tile order.
// upperOnly: the order of a symmetric self-join (super-squares on and above the diagonal only).
unsigned long long raster_count(long long nQ, long long nC, bool upperOnly = false);
int raster_coord(unsigned long long idx, long long nQ, long long nC, bool upperOnly, int* row, int* col);
int counter_words();
int host_words_slot();
unsigned long long tile_count(long long nQ, long long nC);  // 256x256 tiles the kernel processes
// Slot (0..7) of 16-byte chunk `chunk` of slab row `row` in LDS (host mirror of the device swizzle).
int lds_chunk_slot(int row, int chunk);

// Squared norms of n points into `sums` (may be null) and, when `halves` is given, the per-point start value of
// the join's accumulators  h = eps2/4 - s/2  (eps2 = (float)(eps*eps), source/findPairs.cuh:678): the join kernel
// tests  h_q + h_c + q.c >= 0.  A non-finite norm raises the flag in `counters` (the join then tests element
// by element): the flag word receives `epoch`.  With `reset` the kernel also clears the pair counter and the
// queue heads for the join that follows (no launch_reset_counters needed).
hipError_t launch_sum_squared(const void* points, long long ld, int n, int dPad, float* sums, float* halves, float eps2,
                              unsigned long long* counters, hipStream_t stream, unsigned long long epoch = 1,
                              bool reset = false);
// The same halves from norms that are already there.
hipError_t launch_halves(const float* sums, int n, float eps2, float* halves, unsigned long long* counters,
                         hipStream_t stream, unsigned long long epoch = 1, bool reset = false);
// *badRows += number of rows whose columns d .. dPad-1 are not all zeros.
hipError_t launch_padding_check(const void* points, long long ld, int n, int d, int dPad, unsigned long long* badRows,
                                hipStream_t stream);
// Clears the queue heads and, unless keepFound, the pair counter (word 0 of `counters`).
hipError_t launch_reset_counters(unsigned long long* counters, bool keepFound, hipStream_t stream);
// pairs[first, last): QueryPoint += qOffset, CandidatePoint += cOffset.
hipError_t launch_offset_pairs(void* pairs, unsigned long long first, unsigned long long last, int qOffset, int cOffset,
                               hipStream_t stream);
// The same for the pairs [min(mark[0], cap), min(counter, cap)) that the join before this launch appended; leaves
// the counter in mark[1].  No host round trip: the range is read on the device.
hipError_t launch_offset_appended_pairs(void* pairs, unsigned long long* mark, const unsigned long long* counters,
                                        unsigned long long cap, int qOffset, int cOffset, hipStream_t stream);
hipError_t launch_join(const JoinLaunch& p, hipStream_t stream);
// "" for the library proper; a measurement build of the join kernel (parts compiled out) names itself here.
const char* build_tag();


// Device buffers of the row-major sort (a second key buffer and the radix sort's own storage).  They only
// grow; a caller that keeps a SortBuffers across calls sorts without allocating.
struct SortBuffers {
    void* alt = nullptr;
    size_t altBytes = 0;
    void* temp = nullptr;
    size_t tempBytes = 0;
    void release();
};
// Row-major sort of `count` stored pairs (pair_sort.hip); synchronises the stream.  With ws == nullptr the
// buffers are allocated and freed inside the call.  On failure (no memory for the buffers) the pairs are left
// as they were, unsorted.  nQueries / nCandidates bound the indices (0: unknown): the sort then only runs over
// the bits the indices can occupy.
hipError_t sort_pairs_row_major(void* pairs, unsigned long long count, hipStream_t stream, SortBuffers* ws = nullptr,
                                long long nQueries = 0, long long nCandidates = 0);
// Device bytes a sort of `count` pairs needs beside the pairs themselves.
size_t sort_scratch_bytes(unsigned long long count);

// out[i] = Euclidean distance of pair i (FP32 sum of squared differences over dPad dimensions); NaN for a
// pair that names a point outside [0, nQ) x [0, nC).
hipError_t launch_pair_distances(const void* queries, long long ldQ, int nQ, const void* candidates, long long ldC,
                                 int nC, int dPad, const void* pairs, unsigned long long count, float* out,
                                 hipStream_t stream);

}  // namespace fasted
