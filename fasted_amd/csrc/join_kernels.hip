// join_kernels.hip -- the gfx950 (CDNA4, wave64) kernels of the epsilon self-join.
//
//   sum_squared_kernel   FP32 squared norm of every FP16 point; HBM-bound, 16-byte
//                        coalesced loads, lane-group shuffle reduction.  Stands where the
//                        reference has SumSqd::SquaredSumsKernel (source/sumSquared.cuh:53-73).
//   join_kernel          persistent workgroups pull 256x256 tiles of the distance matrix from
//                        per-XCD atomic work queues (the reference's on-demand rasterizer,
//                        source/rasterizer/onDemandRasterizer.cuh:78-108), form Q.C^T with
//                        v_mfma_f32_16x16x32_f16 from XOR-swizzled, double-buffered LDS slabs that
//                        global_load_lds_dwordx4 fills without passing through registers
//                        (source/findPairs.cuh:360-546 is the reference's kernel), and run the
//                        fused test  (s_q + s_c) - 2 q.c <= eps^2  (source/warpMma.cuh:220-273)
//                        with wave-level compaction into an LDS staging area: one global
//                        reservation per workgroup flush instead of two atomics per pair
//                        (source/pair.cuh:123-133).  The first slab and the squared norms of the
//                        next tile travel during the last slab and the epilogue of the current one.
//                        Variants of the same code: tiles of 128 query rows and one workgroup per tile
//                        without the queues for matrices of few tiles (the reference runs smaller tiles
//                        on more blocks, source/findPairs.cuh:55-63,656), and a mailbox that runs one tile
//                        further ahead for tiles of a single slab (D <= 64).
//
// Data layout: points are row-major FP16, one point per row, row stride `ld` halves.  Both
// MFMA operands are "row = point, 8 consecutive k per lane", so the query tile and the
// candidate tile are staged in LDS in the same [256 rows][64 halves] form.
//
// The kernel is written so that it needs no scratch memory: a scratch reload in the epilogue would
// have to wait for every outstanding vector-memory operation of the wave, i.e. for the transfers of
// the next tile that are meant to stay in flight there.  Build with
// -mllvm -amdgpu-atomic-optimizer-strategy=None: the queue reservation is made by one lane a whole
// tile before its result is used, and the optimiser's wave-reduction form would wait for it on the spot.
#include "join_kernels.h"

#include <cstdlib>
#include <type_traits>

#include "join_device.hpp"
#include "tile_order.hpp"

namespace fasted {
namespace {


constexpr int kThreads = 512;                       // 8 waves: 2 (rows) x 4 (cols)
constexpr int kRowBytes = kSlabK * 2;               // one LDS row of a slab: 128 B = 8 chunks of 16 B
constexpr int kOperandBytes = kTile * kRowBytes;    // 32 KiB per operand per stage
constexpr int kStageBytes = 2 * kOperandBytes;      // queries then candidates: 64 KiB
constexpr int kLdsSums = 2 * kStageBytes;           // two buffers of s_q[256] then s_c[256] (current / next tile)
constexpr int kSumsBytes = 2 * kTile * 4;
constexpr int kLdsNext = kLdsSums + 2 * kSumsBytes; // the next two tiles of this workgroup: two slots of (row, col) as u32
constexpr int kLdsStage = kLdsNext + 16;            // staged pairs: one private region per wave
constexpr int kWaveStagePairs = 384;                // 3 KiB of 8-byte records per wave
constexpr int kLdsBytes = kLdsStage + 8 * kWaveStagePairs * 8;
static_assert(kLdsBytes <= 160 * 1024, "LDS budget of one CU");
constexpr int kWaveCols = 64;                       // columns of a wave's output sub-tile (its rows: half the tile's)

// Measurement builds (`make ablation`): the join kernel with parts compiled out, to see what each part
// costs in time and in power.  Such a build computes wrong results; the library proper is built with 0.
//   FASTED_ABLATE bit 0: the accumulators are not initialised
//                 bit 1: no global -> LDS transfers once both LDS stages hold the first two slabs of the
//                        workgroup's first tile (the matrix cores keep seeing real operand values)
//                 bit 2: no LDS fragment reads (the operand registers hold whatever they held)
//                 bit 3: the hit bits of a tile are formed but no pair is extracted from them
//                 bit 4: only the screening of a tile (is there any hit in the wave?), no hit bits, no pairs
//   FASTED_ABLATE_PANELS k > 0: every tile reads the panels (row % k, col % k): the whole join touches
//                        k panels of 256 points only, so they stay in the Infinity Cache (or the L2)
#ifndef FASTED_ABLATE
#define FASTED_ABLATE 0
#endif
#ifndef FASTED_ABLATE_PANELS
#define FASTED_ABLATE_PANELS 0
#endif
constexpr bool kNoInit = (FASTED_ABLATE & 1) != 0, kNoTransfers = (FASTED_ABLATE & 2) != 0,
               kNoFragments = (FASTED_ABLATE & 4) != 0, kNoExtract = (FASTED_ABLATE & 24) != 0,
               kNoHits = (FASTED_ABLATE & 16) != 0;
__device__ __forceinline__ unsigned panel_of(unsigned tile) {
    return FASTED_ABLATE_PANELS > 0 ? tile % (unsigned)(FASTED_ABLATE_PANELS > 0 ? FASTED_ABLATE_PANELS : 1) : tile;
}
__device__ __forceinline__ half8 fragment(const unsigned char* p) {
    if (kNoFragments) {
        half8 v;
        asm volatile("" : "=v"(v) : "v"((unsigned)(size_t)p));
        return v;
    }
    return *reinterpret_cast<const half8*>(p);
}
constexpr int kFragCols = kWaveCols / 16;  // a wave's sub-tile: 8 (or 4) x 4 MFMA 16x16 blocks

// Operand rows of the 256x256 kernel are 128 bytes (a 64-wide k-slab): see lds_swizzle128 in
// tile_order.hpp (conflict freedom is checked exhaustively on the host by tests, and with the
// SQ_LDS_BANK_CONFLICT counter on the device).
__host__ __device__ __forceinline__ int swz(int row) { return lds_swizzle128(row); }

// Work queues of the 256x256 kernel (tile_order.hpp).  From 64 x 64 tiles on, an XCD's sub-rectangle is
// 8 x 4 tiles: the 32 workgroups resident on one XCD work on 8 query panels and 4 candidate panels at a time,
// and a super-square is 32 x 8 tiles, so a round of the 256 workgroups brings 8 new candidate panels from HBM
// while the 32 query panels stay in the Infinity Cache.  Measured against 4 x 8 sub-rectangles (16 x 16
// super-squares, 16 new candidate panels per round): memory-controller activity 2 % instead of 4 %, 1.5 %
// faster at 1M x 4096, 2 % at 500k x 960 and 100k x 4096, 2.5 % at 2M x 384; still taller super-squares
// (64 x 4) gain nothing more at D = 384, flatter ones lose (2 x 16: -8 %, 1 x 32: -15 %).
// Small matrices keep 4 x 8 sub-rectangles (16 x 16 super-squares): fewer padding tiles, and no XCD whose
// own queue holds nothing but padding.  The join kernel is compiled for both shapes.
// An XCD whose queue is exhausted takes from the next XCD's queue, so the tail stays balanced.
typedef TileOrder Raster;
constexpr int kSubTiles = 32;  // per sub-rectangle: the workgroups resident on one XCD
static_assert(kSubTiles * kQueues == kSquareTiles, "8 sub-rectangles tile a super-square");
template <bool kTall>
struct SubShape {
    static constexpr int rows = kTall ? 8 : 4, cols = kTall ? 4 : 8;
};

inline bool tall_order(long long nQueries, int tileRows = kTile) {
    return (nQueries + tileRows - 1) / tileRows >= 64;
}

inline Raster make_raster(long long nQueries, long long nCandidates, bool upperOnly = false, int tileRows = kTile) {
    const bool tall = tall_order(nQueries, tileRows);
    return tall ? make_tile_order(nQueries, nCandidates, tileRows, kTile, SubShape<true>::rows, SubShape<true>::cols, upperOnly)
                : make_tile_order(nQueries, nCandidates, tileRows, kTile, SubShape<false>::rows, SubShape<false>::cols, upperOnly);
}

// host mirror of the kernels' decoding
inline void raster_decode(const Raster& r, bool tall, unsigned q, unsigned long long t, unsigned* tr, unsigned* tc) {
    if (tall)
        tile_order_decode(r, SubShape<true>::rows, SubShape<true>::cols, q, t, tr, tc);
    else
        tile_order_decode(r, SubShape<false>::rows, SubShape<false>::cols, q, t, tr, tc);
}

// ------------------------------------------------------------------------------------------
// Optionally also writes, per point, h = quarterEps2 - s/2 (what the join kernel starts its accumulators
// from) and raises the non-finite flag of the counter block when a squared norm is infinite or NaN: the flag
// word receives `epoch`, the number of the join this launch belongs to, so that it never has to be cleared
// (clearing it in this kernel would race with raising it).  With `reset`, the first workgroup clears the pair
// counter and the queue heads for the join kernel that follows in the stream: no launch of its own for that.
__device__ __forceinline__ void reset_for_join(unsigned long long* __restrict__ counters) {
    if (blockIdx.x != 0) return;
    const int t = threadIdx.x;
    if (t == 0) counters[kCounterStampNorms] = wall_clock64();  // the timed region of a small join starts here
    if (t < kCounterWords && t != kCounterNonFinite && t != kCounterStampNorms && t != kCounterHostWords) counters[t] = 0ull;
}

__global__ void __launch_bounds__(256) sum_squared_kernel(const u32x4* __restrict__ pts, long long ld16, int n,
                                                          int chunksPerRow, int lanesPerRow,
                                                          float* __restrict__ sums, float* __restrict__ halves,
                                                          float quarterEps2, unsigned long long* __restrict__ counters,
                                                          unsigned long long epoch, int reset) {
    if (reset) reset_for_join(counters);
    const int lane = threadIdx.x & 63;
    const long long wave = ((long long)blockIdx.x * blockDim.x + threadIdx.x) >> 6;
    const int rowsPerWave = 64 / lanesPerRow;
    const long long row = wave * rowsPerWave + lane / lanesPerRow;
    const int sub = lane % lanesPerRow;
    float acc = 0.0f;
    if (row < n) {
        const u32x4* p = pts + row * ld16;
        auto square_add = [](u32x4 v, float a) {
            const half8 h = __builtin_bit_cast(half8, v);
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                const float x = (float)h[e];
                a = __builtin_fmaf(x, x, a);
            }
            return a;
        };
        // four independent 16-byte loads in flight per lane (one alone leaves the memory pipe idle
        // for most of its latency), four partial sums
        float part[4] = {0.0f, 0.0f, 0.0f, 0.0f};
        int c = sub;
        for (; c + 3 * lanesPerRow < chunksPerRow; c += 4 * lanesPerRow) {
            // streaming loads: every byte is read once, nothing should displace other lines in the caches
            const u32x4 v0 = __builtin_nontemporal_load(p + c), v1 = __builtin_nontemporal_load(p + c + lanesPerRow),
                        v2 = __builtin_nontemporal_load(p + c + 2 * lanesPerRow),
                        v3 = __builtin_nontemporal_load(p + c + 3 * lanesPerRow);
            part[0] = square_add(v0, part[0]);
            part[1] = square_add(v1, part[1]);
            part[2] = square_add(v2, part[2]);
            part[3] = square_add(v3, part[3]);
        }
        for (; c < chunksPerRow; c += lanesPerRow) part[0] = square_add(__builtin_nontemporal_load(p + c), part[0]);
        acc = (part[0] + part[1]) + (part[2] + part[3]);
    }
    for (int off = lanesPerRow >> 1; off > 0; off >>= 1) acc += __shfl_xor(acc, off, 64);
    if (sub == 0 && row < n) {
        if (sums) sums[row] = acc;
        if (halves) {
            halves[row] = __builtin_fmaf(acc, -0.5f, quarterEps2);
            if (!(__builtin_fabsf(acc) < __builtin_inff())) counters[kCounterNonFinite] = epoch;
        }
    }
}

// The same per-point halves from squared norms that are already there.
__global__ void __launch_bounds__(256) halves_kernel(const float* __restrict__ sums, int n, float quarterEps2,
                                                     float* __restrict__ halves, unsigned long long* __restrict__ counters,
                                                     unsigned long long epoch, int reset) {
    if (reset) reset_for_join(counters);
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n) return;
    const float s = sums[i];
    halves[i] = __builtin_fmaf(s, -0.5f, quarterEps2);
    if (!(__builtin_fabsf(s) < __builtin_inff())) counters[kCounterNonFinite] = epoch;
}

// Rows whose padding columns d .. dPad-1 hold anything but zeros (the kernels read them unmasked, so they must
// be zeros: a caller's mistake that would otherwise show up as silently wrong norms and pairs).
__global__ void __launch_bounds__(256) padding_check_kernel(const unsigned short* __restrict__ pts, long long ld, int n, int d,
                                                            int dPad, unsigned long long* __restrict__ badRows) {
    const int row = blockIdx.x * blockDim.x + threadIdx.x;
    if (row >= n) return;
    const unsigned short* p = pts + (long long)row * ld;
    bool bad = false;
    for (int k = d; k < dPad; ++k) bad |= (p[k] & 0x7fffu) != 0u;  // +0 and -0 are both fine
    if (bad) atomicAdd(badRows, 1ull);
}

// Clears the queue heads and, unless `keepFound`, the pair counter (word 0): a launch that keeps it appends its
// pairs behind those of the launch before.  The non-finite flag (word 1) is never cleared: it holds the number
// of the join that raised it.  (A join that computes its norms first needs no launch of this: the norm kernel's
// first workgroup does the clearing.)
__global__ void reset_counters_kernel(unsigned long long* c, int keepFound) {
    if (threadIdx.x < kCounterWords && threadIdx.x != kCounterNonFinite && threadIdx.x != kCounterHostWords &&
        !(keepFound && threadIdx.x == kCounterFound))
        c[threadIdx.x] = 0ull;
}

// Adds the first row of the query block and of the candidate block to the pairs [first, last) that a
// join of two row blocks of a larger dataset has appended with block-local indices.
__global__ void __launch_bounds__(256) offset_pairs_kernel(int2* pairs, unsigned long long first,
                                                           unsigned long long last, int qOffset, int cOffset) {
    const unsigned long long stride = (unsigned long long)gridDim.x * blockDim.x;
    for (unsigned long long i = first + (unsigned long long)blockIdx.x * blockDim.x + threadIdx.x; i < last; i += stride) {
        int2 v = pairs[i];
        v.x += qOffset;
        v.y += cOffset;
        pairs[i] = v;
    }
}

// The same for the pairs a join has just appended, with the range taken from device memory, so that a series of
// block joins needs no host round trip in between: the range starts at *mark (where the join before this one
// ended; the caller zeroes the first mark) and ends at the pair counter, both clipped to the capacity; the
// counter is then left in mark[1] for the launch after the next join.
__global__ void __launch_bounds__(256) offset_appended_pairs_kernel(int2* pairs, unsigned long long* mark,
                                                                    const unsigned long long* __restrict__ counters,
                                                                    unsigned long long cap, int qOffset, int cOffset) {
    const unsigned long long found = counters[kCounterFound];
    const unsigned long long first = mark[0] < cap ? mark[0] : cap, last = found < cap ? found : cap;
    if (blockIdx.x == 0 && threadIdx.x == 0) mark[1] = found;
    const unsigned long long stride = (unsigned long long)gridDim.x * blockDim.x;
    for (unsigned long long i = first + (unsigned long long)blockIdx.x * blockDim.x + threadIdx.x; i < last; i += stride) {
        int2 v = pairs[i];
        v.x += qOffset;
        v.y += cOffset;
        pairs[i] = v;
    }
}

// ------------------------------------------------------------------------------------------
// The barrier of the tile loop: every global->LDS transfer this wave has issued has landed (they are vector
// memory operations: vmcnt), every LDS operation of the wave is complete, then the workgroup meets.  The wait
// is written out because it is part of the algorithm: __syncthreads() alone only promises the LDS counter at
// workgroup scope, and the transfers are hand-written instructions the compiler knows nothing about.  It is the
// s_waitcnt builtin and not assembly text, so that the compiler's own bookkeeping of outstanding operations
// sees it (behind an opaque wait it assumes the worst and waits for every LDS read of a slab before the first
// MFMA).
__device__ __forceinline__ void transfers_landed_barrier() {
    __builtin_amdgcn_s_waitcnt(0x0070);  // vmcnt(0) lgkmcnt(0), export counter left alone
    __syncthreads();
}

// f(integral_constant<int, kBegin>) ... f(integral_constant<int, kEnd - 1>): a loop whose index is a constant
// expression inside the body (an immediate operand of hand-written instructions needs one)
template <int kBegin, int kEnd, class F>
__device__ __forceinline__ void static_for(F&& f) {
    if constexpr (kBegin < kEnd) {
        f(std::integral_constant<int, kBegin>{});
        static_for<kBegin + 1, kEnd>(f);
    }
}

// kTileRows = 256, or 128 for matrices of few tiles: the tile grid is then twice as fine along the queries (a wave's
// sub-tile is 64 x 64, 4 x 4 blocks), so that twice as many workgroups find work.  The transfers stay as they
// are -- 256 query rows from the tile's first row on are staged, the lower half unused -- which costs nothing
// that matters at such sizes and keeps one set of addresses.
// kOneSlab: D <= 64, a tile is one slab.  No barrier inside such a tile could publish the next tile's coordinates, so
// the mailbox that carries them runs one tile further ahead there (two slots).
// kBitsInLastSlab: the hit bits of a tile are gathered between the MFMAs of its last slab instead of behind the
// k-loop (tiles of up to 16 slabs; see slab_step).
template <bool kEpilogue, bool kTall, int kTileRows, bool kOneSlab, bool kBitsInLastSlab = false>
__global__ void __launch_bounds__(kThreads, 1) join_kernel(JoinParams p) {
    static_assert(!kBitsInLastSlab || kEpilogue, "hit bits are gathered only when there is an epilogue");
    static_assert(kTileRows == 256 || kTileRows == 128, "tile rows");
    constexpr int kWaveRows = kTileRows / 2;    // rows of a wave's output sub-tile (2 x 4 waves)
    constexpr int kFragRows = kWaveRows / 16;   // its rows of 16x16 blocks
    constexpr int kHalfRows = kFragRows / 2;    // a k-step goes through them in two halves
    // Tiles of up to 16 slabs gather their hit bits between the MFMAs of their last slab (see slab_step).  Against
    // screening the accumulators behind the k-loop, on workloads with neighbours to report: +9 % at 200k x 64 and
    // +6.6 % at 100k x 128 (64 neighbours), +2.1 % at 2M x 384 (1000), +3 / +2 / +1 % at D = 256 / 512 / 1024 (100);
    // when no tile has a hit it costs instead: -2 % at D = 64, -0.6 % at 256, -0.2 % at 1024.  Longer tiles keep
    // the screening, which is the cheaper of the two when hardly any tile has a hit (0.1 - 0.3 % at D = 4096 with 16
    // neighbours); a run-time choice between the two inside one kernel made the register allocator spill.
    constexpr bool kFusedBits = kBitsInLastSlab;
    __shared__ __align__(16) unsigned char lds[kLdsBytes];
    const int wave = __builtin_amdgcn_readfirstlane((int)threadIdx.x >> 6);  // wave-uniform, lives in an SGPR
    const int wr = wave >> 2, wc = wave & 3;

    // fragment role (v_mfma_f32_16x16x32_f16): lane reads row l%16 of a 16-row block and the
    // 8 halves k = 8*(l/16) .. +7 of a 32-wide k-step, i.e. chunk 4*ks + l/16 of the slab row.
    int aOff[2], bOff[2];
    {
        const int lane = lane_now();
        const int l16 = lane & 15, quad = lane >> 4;
#pragma unroll
        for (int ks = 0; ks < 2; ++ks) {
            const int slot = ((ks * 4 + quad) ^ swz(l16)) << 4;
            aOff[ks] = (wr * kWaveRows + l16) * kRowBytes + slot;
            bOff[ks] = kOperandBytes + (wc * kWaveCols + l16) * kRowBytes + slot;
        }
    }

    // LDS byte address of lds[0], for the LDS instructions written out by hand below
    const unsigned ldsBase = (unsigned)(size_t)(__attribute__((address_space(3))) unsigned char*)lds;
    unsigned* const sNext = reinterpret_cast<unsigned*>(lds + kLdsNext);  // two slots of [0] row, [1] col
    const int2* const sStage = reinterpret_cast<const int2*>(lds + kLdsStage) + wave * kWaveStagePairs;  // this wave's region

    // (timing of small joins: the first workgroup notes when the kernel started, straight into the host's words)
    auto host_words = [&]() { return reinterpret_cast<unsigned long long*>(p.counters[kCounterHostWords]); };
    if (blockIdx.x == 0 && threadIdx.x == 0) {
        unsigned long long* const hostWords = host_words();
        if (hostWords) __hip_atomic_store(&hostWords[2], wall_clock64(), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
    }

    // Every workgroup signs off when it has nothing left to do, and the one that signs off last hands the pair
    // count and the clock readings to the host (pinned memory that the device writes): no launch and no copy
    // command behind the join for that, and the host may take a small join for finished when word 3 turns
    // non-zero, without waiting for the stream.  So a workgroup is counted only when its pair records have
    // arrived in memory: they are written through (store_pair), each wave waits for its own, the barrier
    // collects the waves.  (A release fence per workgroup would do the same by writing the whole L2 back, once
    // per workgroup: measured, 2 us on a join of 13 us and 11 us on one of 190 us.)  A workgroup's additions to the
    // pair counter are over by then as well -- their old values have come back and been used -- so the last to
    // sign off reads the final count.
    auto sign_off = [&]() {
        unsigned long long* const hostWords = host_words();
        if (!hostWords) return;
        __builtin_amdgcn_s_waitcnt(0x0f70);  // vmcnt(0)
        __syncthreads();
        // (Not `threadIdx.x != 0`: the thread number would stay in a vector register until here, across the tile
        // loop, and move the accumulators and the MFMA operand tuples off their 4-register alignment.)
        if (wave != 0 || lane_now() != 0) return;
        if (atomicAdd(&p.counters[kCounterDone], 1ull) + 1 != gridDim.x) return;
        const unsigned long long through = wall_clock64() | 1ull;  // every workgroup is through (never 0)
        __hip_atomic_store(&hostWords[0], atomicAdd(&p.counters[kCounterFound], 0ull), __ATOMIC_RELAXED,
                           __HIP_MEMORY_SCOPE_SYSTEM);
        __hip_atomic_store(&hostWords[1], p.counters[kCounterStampNorms], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
        __builtin_amdgcn_s_waitcnt(0x0f70);  // both are on their way before the word that the host watches
        __hip_atomic_store(&hostWords[3], through, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
    };

    // set by the kernel that formed this join's per-point halves: some point has a non-finite squared norm
    const bool nonFinite = p.counters[kCounterNonFinite] == p.epoch;

    // Which XCD this workgroup runs on (hardware register XCC_ID, low 3 bits).
    // (thread 0 moves on to the queue it last found work in once its own is exhausted)
    unsigned home = __builtin_amdgcn_s_getreg(20 | (0 << 6) | ((4 - 1) << 11)) & (kQueues - 1);
    constexpr unsigned kNoTile = ~0u;

    // Thread 0 only.  `pos` was popped from the home queue; walks on (and on to the other queues
    // once a queue is exhausted) until a tile that has to be computed turns up.  Skipped on the way:
    // padding tiles of the last super-squares and, in symmetric mode, tiles below the diagonal.
    auto find_tile = [&](unsigned long long pos, unsigned* row, unsigned* col) {
        // the divisors pass through an empty volatile statement so that the reciprocals the division
        // needs are formed here, once per tile, instead of living in registers across the k loop
        Raster ras = p.raster;
        asm volatile("" : "+s"(ras.squareCols));
        unsigned q = home;
        int hops = 0;
        *row = kNoTile;
        *col = 0u;
        for (;;) {
            if (pos < ras.perQueue) {
                unsigned tr, tc;
                tile_order_decode(ras, SubShape<kTall>::rows, SubShape<kTall>::cols, q, pos, &tr, &tc);
                if (tr < ras.tileRows && tc < ras.tileCols && !(p.symmetric && tc < tr)) {
                    *row = tr;
                    *col = tc;
                    home = q;  // the next reservation goes where this tile came from
                    return;
                }
            } else {
                if (++hops == kQueues) return;  // every queue is exhausted
                q = (q + 1) & (kQueues - 1);
            }
            pos = atomicAdd(&p.counters[kQueueBase + q * kQueueStride], 1ull);
        }
    };

    // Pairs are staged in LDS, in a region private to each wave whose fill count lives in a scalar
    // register: appending needs no atomic and no barrier.  A region goes to the global list with one
    // reservation on the global counter (same-address atomics serialise at about 12 ns each: one per pair,
    // or per wave and tile, is what would bound output-heavy joins) and coalesced 8-byte stores.
    int staged = 0;
    // Pair records are written through to memory (a store at system scope) instead of staying dirty in the L2 of
    // the XCD until the kernel ends: the host may take a small join for finished as soon as the last workgroup
    // has reported, and a record is written once and not read again by this kernel.
    auto store_pair = [&](unsigned long long slot, int2 rec) {
        __hip_atomic_store(reinterpret_cast<unsigned long long*>(p.pairs + slot),
                           (unsigned long long)(unsigned)rec.x | ((unsigned long long)(unsigned)rec.y << 32),
                           __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
    };
    auto flush_wave = [&]() {
        const int ln = lane_now();
        unsigned long long base = 0;
        if (ln == 0) base = atomicAdd(&p.counters[kCounterFound], (unsigned long long)staged);
        base = ((unsigned long long)__builtin_amdgcn_readfirstlane((unsigned)(base >> 32)) << 32) |
               __builtin_amdgcn_readfirstlane((unsigned)base);
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");  // the staged records are in LDS
        for (int i = ln; i < staged; i += 64)
            if (base + i < p.cap) store_pair(base + i, sStage[i]);  // past the capacity: counted, not stored
        staged = 0;
    };

    // Byte offsets, from the tile's first row, of the 16-byte chunks this lane copies: 4 query rows and
    // 4 candidate rows per slab.  The swizzle is applied here, on the global side.  Rows past the end of
    // the dataset re-read the last real row (their results are masked), so only the ragged last tiles have
    // offsets of their own: the offsets are formed again only when a ragged tile comes or goes.
    bool clampedA = false, clampedB = false;  // the current offsets belong to a ragged tile
    auto side_offsets = [&](int base, int n, long long ld16, unsigned (&o)[4]) {
        const int ln = lane_now();
        const int row0 = wave * 32 + (ln >> 3);
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int r = row0 + 8 * i;
            const int chunk = (ln & 7) ^ swz(r);
            o[i] = (unsigned)(min(r, n - 1 - base) * (int)ld16 + chunk) * 16u;
        }
    };
    auto tile_offsets = [&](int rowBase, int colBase, unsigned (&oA)[4], unsigned (&oB)[4], bool first) {
        const bool raggedA = rowBase + kTile > p.nQ, raggedB = colBase + kTile > p.nC;
        if (first || raggedA || clampedA) {
            side_offsets(rowBase, p.nQ, p.ldQ16, oA);
            clampedA = raggedA;
        }
        if (first || raggedB || clampedB) {
            side_offsets(colBase, p.nC, p.ldC16, oB);
            clampedB = raggedB;
        }
    };

    // One 1-KiB global->LDS transfer of this wave (global_load_lds_dwordx4: no registers in between);
    // j = 0..7 alternates query / candidate rows.  Lane l lands in row l/8, chunk slot l%8 of the
    // 8 rows the instruction fills.
    bool filling = true;  // (measurement builds only)
    // LDS byte address of this wave's first row in stage 0: wave w owns rows [32w, 32w+32) of both operands
    const unsigned waveRows = ldsBase + (unsigned)(wave * 32 * kRowBytes);
    auto issue_load = [&](auto jc, const char* slabA, const char* slabB, const unsigned (&oA)[4], const unsigned (&oB)[4],
                          int stage) {
        if (kNoTransfers && !filling) return;
        constexpr int j = decltype(jc)::value;
        constexpr int i = j >> 1;
        constexpr unsigned within = (unsigned)((j & 1) * kOperandBytes + i * 8 * kRowBytes);
        const unsigned stageRows = waveRows + (unsigned)(stage * kStageBytes);
        // Written as instructions: M0 (the LDS destination) is formed by one scalar add with an immediate, the
        // slab's address sits in scalar registers, the lane's offset is a 32-bit vector register that never
        // changes -- no vector arithmetic per transfer (left to the compiler, the addresses become
        // loop-carried 64-bit vector pointers, and M0 costs a scalar instruction or two more).
        if (j & 1)
            asm volatile("s_add_u32 m0, %0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %2, %3" ::"s"(stageRows), "n"(within),
                         "v"(oB[i]), "s"(slabB)
                         : "memory", "m0", "scc");
        else
            asm volatile("s_add_u32 m0, %0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %2, %3" ::"s"(stageRows), "n"(within),
                         "v"(oA[i]), "s"(slabA)
                         : "memory", "m0", "scc");
    };

    // Per-point halves (eps^2/4 - s/2) of a tile's 256 queries (waves 0-3) and 256 candidates (waves 4-7),
    // 64 floats per wave, straight into the buffer `which`.
    auto issue_sums = [&](int rowBase, int colBase, int which) {
        const int ln = lane_now();
        const int part = wave & 3;
        const float* src = wave < 4 ? p.halfQ + min(rowBase + part * 64 + ln, p.nQ - 1)
                                    : p.halfC + min(colBase + part * 64 + ln, p.nC - 1);
        unsigned char* const dst = lds + kLdsSums + which * kSumsBytes + wave * 256;
        __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)src,
                                         (__attribute__((address_space(3))) void*)dst, 4, 0, 0);
    };

    // ---- first tile
    if (wave == 0 && lane_now() == 0) {
        unsigned r, c, r1 = kNoTile, c1 = 0u;
        if (p.direct) {
            // A matrix of no more tiles than workgroups: one tile each, by workgroup number.  Through the queues,
            // every workgroup would reserve a second tile while it starts its first (the reservation runs one
            // tile ahead), and the workgroups of XCDs with short queues would find the work already taken.
            r = blockIdx.x / p.raster.tileCols;
            c = blockIdx.x % p.raster.tileCols;
            if (p.symmetric && c < r) r = kNoTile;
        } else {
            find_tile(atomicAdd(&p.counters[kQueueBase + home * kQueueStride], 1ull), &r, &c);
            if (kOneSlab && r != kNoTile) find_tile(atomicAdd(&p.counters[kQueueBase + home * kQueueStride], 1ull), &r1, &c1);
        }
        // Single-slab tiles use two mailbox slots: during tile t, slot (t + 1) % 2 names tile t + 1 (written during
        // tile t - 1 and published by the barrier at the top of tile t) and thread 0 writes tile t + 2 into slot
        // t % 2.  With more slabs, slot 0 is written at the top of a tile and published by its first slab's barrier.
        sNext[0] = r;
        sNext[1] = c;
        sNext[2] = r1;
        sNext[3] = c1;
    }
    __syncthreads();
    unsigned tr = __builtin_amdgcn_readfirstlane(sNext[0]);
    unsigned tc = __builtin_amdgcn_readfirstlane(sNext[1]);
    if (tr == kNoTile) {
        sign_off();
        return;
    }

    unsigned offA[4], offB[4];
    tile_offsets((int)tr * kTileRows, (int)tc * kTile, offA, offB, true);
    const char* gA = reinterpret_cast<const char*>(p.ptsQ + (long long)panel_of(tr) * kTileRows * p.ldQ16);
    const char* gB = reinterpret_cast<const char*>(p.ptsC + (long long)panel_of(tc) * kTile * p.ldC16);
    static_for<0, 8>([&](auto jc) { issue_load(jc, gA, gB, offA, offB, 0); });
    if (kNoTransfers) {
        const int second = kOneSlab ? 0 : kRowBytes;
        static_for<0, 8>([&](auto jc) { issue_load(jc, gA + second, gB + second, offA, offB, 1); });
        filling = false;
    }
    issue_sums((int)tr * kTileRows, (int)tc * kTile, 0);
    unsigned long long popped = 0;  // thread 0: the home queue position reserved for the tile after the next one to be decoded
    if (wave == 0 && lane_now() == 0 && !p.direct) popped = atomicAdd(&p.counters[kQueueBase + home * kQueueStride], 1ull);

    int stage = 0;  // LDS stage that holds slab 0 of the current tile
    int sumsBuf = 0;

    for (;;) {
        // slab 0 of this tile (issued during the previous tile's last slab) has landed
        transfers_landed_barrier();
        if (wave == 0 && lane_now() == 0) {
            // the reservation made a whole tile ago has long arrived: no wait here
            unsigned r, c;
            if (p.direct) {
                r = kNoTile;
                c = 0u;
            } else {
                find_tile(popped, &r, &c);
                popped = atomicAdd(&p.counters[kQueueBase + home * kQueueStride], 1ull);
            }
            const int slot = kOneSlab ? 2 * sumsBuf : 0;  // (sumsBuf is the tile count's parity)
            sNext[slot] = r;
            sNext[slot + 1] = c;
        }

        // The accumulators start at h_q + h_c, h = eps^2/4 - s/2 per point (see the epilogue): the tile's
        // 512 values landed together with slab 0.  Only the first row of blocks is set here; the others are
        // set between the MFMAs of the tile's first k-step, one row of blocks ahead of the MFMAs that need it
        // (a wave's vector instructions between its own MFMAs cost far less than on their own).
        floatx4 acc[kFragRows][kFragCols];
        // Per-lane hit bits of the 4 pairs of block rows: element e = (fi & 1) * 16 + fj * 4 + r of the pair
        // fi / 2 is bit 31 - e.
        unsigned hits[kFragRows / 2];
        float hc[kFragCols];
        const float* sQw;
        {
            const int ln = lane_now();
            sQw = reinterpret_cast<const float*>(lds + kLdsSums + sumsBuf * kSumsBytes) + wr * kWaveRows + (ln >> 4) * 4;
            const float* const sCw =
                reinterpret_cast<const float*>(lds + kLdsSums + sumsBuf * kSumsBytes) + kTile + wc * kWaveCols + (ln & 15);
#pragma unroll
            for (int fj = 0; fj < kFragCols; ++fj) hc[fj] = sCw[fj * 16];
        }
        auto init_row = [&](int fi) {
            const floatx4 hq = *reinterpret_cast<const floatx4*>(sQw + fi * 16);
#pragma unroll
            for (int fj = 0; fj < kFragCols; ++fj) {
                if (kNoInit)
                    asm volatile("" : "=v"(acc[fi][fj]));
                else
                    acc[fi][fj] = hq + hc[fj];  // commutative: the same for (q, c) and (c, q)
            }
        };
        init_row(0);

        // One slab = 2 k-steps of 32; a k-step is two halves of 16 MFMAs (query blocks 0-3, then
        // 4-7, each against the 4 candidate blocks, query fragment held for 4 MFMAs, candidate blocks
        // in snake order: consecutive MFMAs always share an operand, which the power-limited clock
        // rewards with about 1.5 %).  The instruction order is pinned with
        // scheduling barriers: the LDS reads for the next half are issued ahead of the MFMAs of
        // the current half, and the 8 global->LDS transfers of the following slab are issued during
        // the first k-step, four at the start of each of its halves: early, so that an L2 miss has the
        // whole second k-step to land before the slab's barrier (one transfer pinned in front of every 4 MFMAs
        // instead measured 1-3 % slower on the 1M x 4096 workload).
        auto slab_step = [&](auto modec, int stg, bool prefetch, const char* pA, const char* pB,
                             const unsigned (&oA)[4], const unsigned (&oB)[4]) {
            constexpr int mode = decltype(modec)::value;
            constexpr bool first = mode == 1;     // the tile's first slab also sets the accumulators
            constexpr bool withBits = mode == 2;  // the tile's last slab also gathers the hit bits
            const unsigned char* const buf = lds + stg * kStageBytes;
            half8 aLo[kHalfRows], aHi[kHalfRows], b[2][kFragCols];

            if constexpr (withBits) {
                // The tile's last slab goes through the rows of blocks one after the other like the first, both
                // k-steps of a row together: after its 8 MFMAs a row of blocks is final, and the sign bits of its
                // 16 elements per lane (set = no hit) are shifted into the lane's hit words between the 8 MFMAs of
                // the row after it, two vector instructions behind every MFMA, where they cost next to nothing
                // -- instead of a screening pass over all accumulators and a conditional pass over the rows with
                // a hit behind the k-loop, where nothing hides them.  Only the last row's 16 shifts are exposed.
                // (Both k-steps visit the candidate blocks in ascending order, so that the blocks of a row become
                // final in the order in which their bits are gathered.)
                half8 a[2][2];
#pragma unroll
                for (int ks = 0; ks < 2; ++ks) {
                    a[0][ks] = fragment(buf + aOff[ks]);
#pragma unroll
                    for (int fj = 0; fj < kFragCols; ++fj) b[ks][fj] = fragment(buf + bOff[ks] + fj * 16 * kRowBytes);
                    __builtin_amdgcn_sched_barrier(0);
                }
                unsigned m = ~0u;
                auto gather_row = [&](int fi) {
#pragma unroll
                    for (int fj = 0; fj < kFragCols; ++fj)
#pragma unroll
                        for (int r = 0; r < 4; ++r) {
                            const float v = acc[fi][fj][r];
                            m = __builtin_amdgcn_alignbit(m, __float_as_uint(v), 31);
                        }
                    // (an anchor: without it the shifts are sunk to where the hit words are used, behind the k-loop)
                    asm volatile("" : "+v"(m));
                    if (fi & 1) {
                        hits[fi >> 1] = kNoHits ? 0u : ~m;
                        m = ~0u;
                    }
                };
                static_for<0, kFragRows>([&](auto fic) {
                    constexpr int fi = decltype(fic)::value;
                    __builtin_amdgcn_sched_barrier(0);
                    if constexpr (fi < 4) {
                        if (prefetch) {
                            issue_load(std::integral_constant<int, 2 * fi>{}, pA, pB, oA, oB, stg ^ 1);
                            issue_load(std::integral_constant<int, 2 * fi + 1>{}, pA, pB, oA, oB, stg ^ 1);
                        }
                    }
                    __builtin_amdgcn_sched_barrier(0);
                    if constexpr (fi + 1 < kFragRows) {
                        a[(fi + 1) & 1][0] = fragment(buf + aOff[0] + (fi + 1) * 16 * kRowBytes);
                        a[(fi + 1) & 1][1] = fragment(buf + aOff[1] + (fi + 1) * 16 * kRowBytes);
                    }
#pragma unroll
                    for (int ks = 0; ks < 2; ++ks)
#pragma unroll
                        for (int fj = 0; fj < kFragCols; ++fj)
                            acc[fi][fj] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a[fi & 1][ks], b[ks][fj], acc[fi][fj], 0, 0, 0);
                    if constexpr (fi >= 1) {
                        gather_row(fi - 1);
                        // the order asked of the scheduler: the fragment reads, then MFMA, 2 shifts, MFMA, 2 shifts ...
                        if constexpr (fi + 1 < kFragRows) __builtin_amdgcn_sched_group_barrier(0x100, 2, 0);
#pragma unroll
                        for (int k = 0; k < 8; ++k) {
                            __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
                            __builtin_amdgcn_sched_group_barrier(0x002, 2, 0);
                        }
                    }
                });
                __builtin_amdgcn_sched_barrier(0);
                gather_row(kFragRows - 1);
                return;
            }

            if constexpr (first) {
                // The tile's first slab goes through the rows of blocks one after the other, both k-steps of a
                // row together (an element still receives k-step 0 before k-step 1): the 16 start values of row
                // fi + 1 are formed between the 8 MFMAs of row fi, two vector instructions behind every MFMA,
                // which is about what a wave issues for free there.  The rows' h_q are read ahead of the slab
                // (into registers of accumulators that are not live yet).
                floatx4 hq[kFragRows];
                half8 a[2][2];
                // what the first MFMAs need is read first (LDS reads complete in order)
#pragma unroll
                for (int ks = 0; ks < 2; ++ks) {
                    a[0][ks] = fragment(buf + aOff[ks]);
#pragma unroll
                    for (int fj = 0; fj < kFragCols; ++fj) b[ks][fj] = fragment(buf + bOff[ks] + fj * 16 * kRowBytes);
                    __builtin_amdgcn_sched_barrier(0);
                }
#pragma unroll
                for (int fi = 1; fi < kFragRows; ++fi) hq[fi] = *reinterpret_cast<const floatx4*>(sQw + fi * 16);
                static_for<0, kFragRows>([&](auto fic) {
                    constexpr int fi = decltype(fic)::value;
                    __builtin_amdgcn_sched_barrier(0);
                    if constexpr (fi < 4) {
                        if (prefetch) {
                            issue_load(std::integral_constant<int, 2 * fi>{}, pA, pB, oA, oB, stg ^ 1);
                            issue_load(std::integral_constant<int, 2 * fi + 1>{}, pA, pB, oA, oB, stg ^ 1);
                        }
                    }
                    __builtin_amdgcn_sched_barrier(0);
                    if constexpr (fi + 1 < kFragRows) {
                        a[(fi + 1) & 1][0] = fragment(buf + aOff[0] + (fi + 1) * 16 * kRowBytes);
                        a[(fi + 1) & 1][1] = fragment(buf + aOff[1] + (fi + 1) * 16 * kRowBytes);
                    }
#pragma unroll
                    for (int ks = 0; ks < 2; ++ks)
#pragma unroll
                        for (int fs = 0; fs < kFragCols; ++fs) {
                            const int fj = ((fi + ks) & 1) ? kFragCols - 1 - fs : fs;
                            acc[fi][fj] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a[fi & 1][ks], b[ks][fj], acc[fi][fj], 0, 0, 0);
                        }
                    if constexpr (fi + 1 < kFragRows) {
#pragma unroll
                        for (int fj = 0; fj < kFragCols; ++fj) {
                            if (kNoInit)
                                asm volatile("" : "=v"(acc[fi + 1][fj]));
                            else
                                acc[fi + 1][fj] = hq[fi + 1] + hc[fj];
                        }
                        // the order asked of the scheduler: the two fragment reads, then MFMA, 2 adds, MFMA, 2 adds ...
                        __builtin_amdgcn_sched_group_barrier(0x100, 2, 0);
#pragma unroll
                        for (int m = 0; m < 8; ++m) {
                            __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
                            __builtin_amdgcn_sched_group_barrier(0x002, 2, 0);
                        }
                    }
                });
                __builtin_amdgcn_sched_barrier(0);
                return;
            }

#pragma unroll
            for (int fj = 0; fj < kFragCols; ++fj)
                b[0][fj] = fragment(buf + bOff[0] + fj * 16 * kRowBytes);
#pragma unroll
            for (int fi = 0; fi < kHalfRows; ++fi)
                aLo[fi] = fragment(buf + aOff[0] + fi * 16 * kRowBytes);
#pragma unroll
            for (int ks = 0; ks < 2; ++ks) {
#pragma unroll
                for (int fi = 0; fi < kHalfRows; ++fi)
                    aHi[fi] = fragment(buf + aOff[ks] + (fi + kHalfRows) * 16 * kRowBytes);
                __builtin_amdgcn_sched_barrier(0);
                if (ks == 0 && prefetch) static_for<0, 4>([&](auto jc) { issue_load(jc, pA, pB, oA, oB, stg ^ 1); });
#pragma unroll
                for (int fi = 0; fi < kHalfRows; ++fi) {
#pragma unroll
                    for (int fs = 0; fs < kFragCols; ++fs) {
                        const int fj = (fi & 1) ? kFragCols - 1 - fs : fs;  // snake order: one operand in common with the MFMA before
                        acc[fi][fj] = __builtin_amdgcn_mfma_f32_16x16x32_f16(aLo[fi], b[ks][fj], acc[fi][fj], 0, 0, 0);
                    }
                }
                __builtin_amdgcn_sched_barrier(0);
                if (ks == 0) {
#pragma unroll
                    for (int fj = 0; fj < kFragCols; ++fj)
                        b[1][fj] = fragment(buf + bOff[1] + fj * 16 * kRowBytes);
#pragma unroll
                    for (int fi = 0; fi < kHalfRows; ++fi)
                        aLo[fi] = fragment(buf + aOff[1] + fi * 16 * kRowBytes);
                }
                __builtin_amdgcn_sched_barrier(0);
                if (ks == 0 && prefetch) static_for<4, 8>([&](auto jc) { issue_load(jc, pA, pB, oA, oB, stg ^ 1); });
#pragma unroll
                for (int fi = 0; fi < kHalfRows; ++fi) {
#pragma unroll
                    for (int fs = 0; fs < kFragCols; ++fs) {
                        const int fj = (fi & 1) ? kFragCols - 1 - fs : fs;
                        acc[fi + kHalfRows][fj] =
                            __builtin_amdgcn_mfma_f32_16x16x32_f16(aHi[fi], b[ks][fj], acc[fi + kHalfRows][fj], 0, 0, 0);
                    }
                }
                __builtin_amdgcn_sched_barrier(0);
            }
        };

        constexpr std::integral_constant<int, 1> kFirstSlab{};
        constexpr std::integral_constant<int, 0> kLaterSlab{};
        constexpr std::integral_constant<int, kFusedBits ? 2 : 0> kLastSlab{};
        if (!kOneSlab && p.nSlabs > 1) {  // (the run-time test is always true here; the register allocator does better with it)
            slab_step(kFirstSlab, stage, true, gA + kRowBytes, gB + kRowBytes, offA, offB);
            stage ^= 1;
            transfers_landed_barrier();
        }
        for (int s = 1; s + 1 < p.nSlabs; ++s) {
            slab_step(kLaterSlab, stage, true, gA + (s + 1) * kRowBytes, gB + (s + 1) * kRowBytes, offA, offB);
            stage ^= 1;
            transfers_landed_barrier();
        }

        // The tile after this one: its first slab and its squared norms travel during this tile's last
        // slab and epilogue.  The current tile's offsets are not needed any more, so the next tile's
        // take their registers.
        const int slot = kOneSlab ? 2 * (sumsBuf ^ 1) : 0;
        const unsigned ntr = __builtin_amdgcn_readfirstlane(sNext[slot]);
        const unsigned ntc = __builtin_amdgcn_readfirstlane(sNext[slot + 1]);
        const bool more = ntr != kNoTile;
        if (more) {
            tile_offsets((int)ntr * kTileRows, (int)ntc * kTile, offA, offB, false);
            gA = reinterpret_cast<const char*>(p.ptsQ + (long long)panel_of(ntr) * kTileRows * p.ldQ16);
            gB = reinterpret_cast<const char*>(p.ptsC + (long long)panel_of(ntc) * kTile * p.ldC16);
            issue_sums((int)ntr * kTileRows, (int)ntc * kTile, sumsBuf ^ 1);
        }
        if (kOneSlab || p.nSlabs == 1) {  // a single slab: all rows are set before it
#pragma unroll
            for (int fi = 1; fi < kFragRows; ++fi) init_row(fi);
        }
        slab_step(kLastSlab, stage, more, gA, gB, offA, offB);
        stage ^= 1;

        if (kEpilogue) {
            // Fused test (source/warpMma.cuh:220-273).  The accumulators started at h_q + h_c with
            // h = eps^2/4 - s/2 per point, so an element now holds a = q.c - (s_q + s_c)/2 + eps^2/2 =
            // (eps^2 - dist^2)/2 and the reference's test  s_q + s_c - 2 q.c <= eps^2  reads  a >= 0: the sign
            // bit of the accumulator, symmetric in q and c like the reference's test.
            const int rowBase = (int)tr * kTileRows, colBase = (int)tc * kTile;
            const int ln = lane_now();
            const int qLane = rowBase + wr * kWaveRows + (ln >> 4) * 4;  // row of element r = 0 of block row 0
            const int cLane = colBase + wc * kWaveCols + (ln & 15);      // column in block column 0
            // Every element is tested one by one when the tile touches the diagonal of a self-join or the ragged
            // end of a dataset (self pairs are forced, padded rows/columns masked: source/warpMma.cuh:257-259)
            // or when the dataset holds points with non-finite norms (a NaN must compare as "no hit").
            // (forced pairs: query q with candidate q * selfStride -- the diagonal of a self-join, or the sampled
            // points among all points)
            const bool diagonal = p.selfStride != 0 && colBase <= (rowBase + kTileRows - 1) * p.selfStride &&
                                  rowBase * p.selfStride <= colBase + kTile - 1;
            const bool edge = nonFinite || diagonal || rowBase + kTileRows > p.nQ || colBase + kTile > p.nC;
            const bool mirror = p.symmetric && tr != tc;  // a tile above the diagonal also stands for its mirror image

            bool any;
            if (kFusedBits && !edge) {
                // the hit bits came out of the last slab: is there one in the wave at all?
                unsigned some = hits[0];
#pragma unroll
                for (int fp = 1; fp < kFragRows / 2; ++fp) some |= hits[fp];
                any = __builtin_amdgcn_ballot_w64(some != 0u) != 0ull;
            } else if (!edge) {
                // Screening, about 1/2 vector instruction per element: the maximum of the lane's 128 elements,
                // formed per row of blocks; a wave in which no lane has a hit is done.
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
                any = __builtin_amdgcn_ballot_w64(best >= 0.0f) != 0ull;
                if (kNoHits) asm volatile("" ::"v"(best));
                if (any && !kNoHits) {
                    // the rows of blocks with a hit somewhere in the wave yield their bits, one instruction per
                    // element: the sign of the accumulator (set = no hit) is shifted in.  (The eight compares are
                    // issued together: one at a time, each branch waits for its compare.)
                    unsigned long long rowHit[kFragRows];
#pragma unroll
                    for (int fi = 0; fi < kFragRows; ++fi) rowHit[fi] = __builtin_amdgcn_ballot_w64(rowBest[fi] >= 0.0f);
#pragma unroll
                    for (int fi = 0; fi < kFragRows; ++fi) asm volatile("" : "+s"(rowHit[fi]));
#pragma unroll
                    for (int fp = 0; fp < kFragRows / 2; ++fp) {
                        unsigned m = ~0u;
#pragma unroll
                        for (int h = 0; h < 2; ++h) {
                            const int fi = fp * 2 + h;
                            if (rowHit[fi] != 0ull) {
#pragma unroll
                                for (int fj = 0; fj < kFragCols; ++fj)
#pragma unroll
                                    for (int r = 0; r < 4; ++r) {
                                        const float a = acc[fi][fj][r];  // (a bit cast of the vector element itself reads element 0)
                                        m = __builtin_amdgcn_alignbit(m, __float_as_uint(a), 31);
                                    }
                            } else {
                                m = (m << 16) | 0xffffu;
                            }
                        }
                        hits[fp] = ~m;
                    }
                }
            } else {
                any = true;
#pragma unroll
                for (int fp = 0; fp < kFragRows / 2; ++fp) {
                    unsigned m = 0u;
#pragma unroll
                    for (int h = 0; h < 2; ++h) {
                        const int fi = fp * 2 + h;
#pragma unroll
                        for (int fj = 0; fj < kFragCols; ++fj) {
#pragma unroll
                            for (int r = 0; r < 4; ++r) {
                                const int q = qLane + fi * 16 + r, c = cLane + fj * 16;
                                const bool hit =
                                    ((acc[fi][fj][r] >= 0.0f) | ((p.selfStride != 0) & (q * p.selfStride == c))) & (q < p.nQ) & (c < p.nC);
                                m = (m << 1) | (hit ? 1u : 0u);
                            }
                        }
                    }
                    hits[fp] = m;
                }
            }
            if (kNoExtract) {
                if (any && !kNoHits) {
#pragma unroll
                    for (int fp = 0; fp < kFragRows / 2; ++fp) asm volatile("" ::"v"(hits[fp]));
                }
            } else if (any) {
                // Extraction.  A round takes the first remaining hit of every lane that has one among its 128
                // elements (all four words of hit bits at once: most lanes have no hit and nearly all others
                // exactly one, so one round is the rule): the lanes form a mask in scalar registers, a lane's
                // record goes behind those of the lanes before it, the wave's fill count moves on by the number of
                // lanes.  The index of a lane's first hit is a chain of vector instructions without compares
                // (v_ffbh_u32 yields all ones for an empty word, so the minimum over the words, each with its
                // word number in bits 5-6, is the first hit or all ones), and the two masks a round branches on --
                // lanes with a hit, lanes with more than one -- are formed together: a branch waits for the
                // compare that forms its mask, and one wait serves both.
                constexpr int kWords = kFragRows / 2;
                for (;;) {
                    unsigned first = ~0u, total = 0u;
#pragma unroll
                    for (int fp = kWords - 1; fp >= 0; --fp) {
                        unsigned lead;
                        asm("v_ffbh_u32 %0, %1" : "=v"(lead) : "v"(hits[fp]));
                        first = min(first, lead | (unsigned)(fp * 32));
                        total += (unsigned)__builtin_popcount(hits[fp]);
                    }
                    unsigned long long lanes = __builtin_amdgcn_ballot_w64((int)first >= 0);
                    unsigned long long again = __builtin_amdgcn_ballot_w64(total > 1u);
                    asm volatile("" : "+s"(lanes), "+s"(again));
                    if (lanes == 0ull) break;
                    const int count = __builtin_popcountll(lanes) << (mirror ? 1 : 0);
                    if (staged + count > kWaveStagePairs) flush_wave();
                    if ((int)first >= 0) {
                        // element `first` of the lane: block row first / 16, block column (first / 4) % 4, row first % 4
                        const int q = qLane + (int)((first & ~15u) + (first & 3u));
                        const int c = cLane + (int)((first & 12u) << 2);
                        const unsigned before = __builtin_amdgcn_mbcnt_hi(
                            (unsigned)(lanes >> 32), __builtin_amdgcn_mbcnt_lo((unsigned)lanes, 0u));
                        const unsigned at = (unsigned)staged + (mirror ? 2u * before : before);
                        // written as an instruction: for an ordinary LDS store the compiler first waits until
                        // this wave's global->LDS transfers of the next tile have landed
                        auto put = [&](unsigned idx, int a0, int a1) {
                            const unsigned long long rec =
                                (unsigned long long)(unsigned)a0 | ((unsigned long long)(unsigned)a1 << 32);
                            asm volatile("ds_write_b64 %0, %1" ::"v"(ldsBase + (unsigned)kLdsStage +
                                                                     ((unsigned)wave * kWaveStagePairs + idx) * 8u),
                                         "v"(rec)
                                         : "memory");
                        };
                        put(at, q, c);
                        if (mirror) put(at + 1, c, q);
                    }
                    staged += count;
                    if (again == 0ull) break;
                    // some lane has another hit: every lane drops the one it has just written
#pragma unroll
                    for (int fp = 0; fp < kWords; ++fp)
                        if ((first >> 5) == (unsigned)fp) hits[fp] &= ~(0x80000000u >> (first & 31u));
                }
            }
        } else {
            // keep the accumulators observable without spending instructions on them
#pragma unroll
            for (int fi = 0; fi < kFragRows; ++fi)
#pragma unroll
                for (int fj = 0; fj < kFragCols; ++fj) asm volatile("" ::"v"(acc[fi][fj]));
        }

        if (!more) break;
        tr = ntr;
        tc = ntc;
        sumsBuf ^= 1;
    }
    if (kEpilogue) {
        // What is left in the eight regions goes out with one reservation for the workgroup: every workgroup
        // ends at about the same time, and one atomic per wave, all on one address, would serialise for
        // longer than a small join takes.  No transfer is in flight any more, so ordinary LDS accesses do.
        unsigned* const sLeft = reinterpret_cast<unsigned*>(lds);  // the operand stages are free now
        unsigned long long* const sBase = reinterpret_cast<unsigned long long*>(lds + 64);
        const int ln = lane_now();
        __syncthreads();  // every wave is past its last fragment read
        if (ln == 0) sLeft[wave] = (unsigned)staged;
        __syncthreads();
        unsigned before = 0, total = 0;
#pragma unroll
        for (int w = 0; w < kThreads / 64; ++w) {
            const unsigned left = __builtin_amdgcn_readfirstlane(sLeft[w]);
            if (w < wave) before += left;
            total += left;
        }
        if (total != 0) {
            if (wave == 0 && ln == 0) *sBase = atomicAdd(&p.counters[kCounterFound], (unsigned long long)total);
            __syncthreads();
            const unsigned long long base = *sBase + before;
            for (int i = ln; i < staged; i += 64)
                if (base + i < p.cap) store_pair(base + i, sStage[i]);
        }
    }
    sign_off();
}

}  // namespace

unsigned long long raster_count(long long nQ, long long nC, bool upperOnly) {
    return make_raster(nQ, nC, upperOnly).perQueue * kQueues;
}

// Index idx enumerates the queues round-robin: queue idx % 8, position idx / 8 -- the order in
// which eight equally fast XCDs would take the tiles.  Returns 0 past the end, 2 for a padding
// tile that the kernel skips, 1 for a real tile.
// With upperOnly (symmetric self-join) the tiles below the diagonal count as skipped as well.
int raster_coord(unsigned long long idx, long long nQ, long long nC, bool upperOnly, int* row, int* col) {
    const Raster r = make_raster(nQ, nC, upperOnly);
    if (idx >= r.perQueue * kQueues) return 0;
    unsigned tr, tc;
    raster_decode(r, tall_order(nQ), (unsigned)(idx % kQueues), idx / kQueues, &tr, &tc);
    *row = (int)tr * kTile;
    *col = (int)tc * kTile;
    return (tr < r.tileRows && tc < r.tileCols && !(upperOnly && tc < tr)) ? 1 : 2;
}

int counter_words() { return kCounterWords; }
int host_words_slot() { return kCounterHostWords; }

// "" for the library proper; a measurement build names what it leaves out (its results are wrong by construction)
#define FASTED_STR2(x) #x
#define FASTED_STR(x) FASTED_STR2(x)
const char* build_tag() {
    return (FASTED_ABLATE != 0 || FASTED_ABLATE_PANELS != 0)
               ? "ABLATION BUILD (ablate=" FASTED_STR(FASTED_ABLATE) ", panels=" FASTED_STR(FASTED_ABLATE_PANELS) "): results are wrong by construction"
               : "";
}

unsigned long long tile_count(long long nQ, long long nC) {
    const Raster r = make_raster(nQ, nC);
    return (unsigned long long)r.tileRows * r.tileCols;
}

int lds_chunk_slot(int row, int chunk) { return (chunk ^ swz(row)) & 7; }

// (float)(eps*eps) / 4, kept finite: the kernels rely on finite accumulator start values, so an infinite
// epsilon (every pair of finite points is a hit) is clamped.  The host entries refuse a NaN epsilon; should one
// arrive here all the same, the start values become hugely negative: no distance passes the test, as no
// distance compares <= NaN in the reference (source/warpMma.cuh:257), and only the forced self pairs remain.
float quarter_eps2(float eps2) { return (eps2 != eps2 ? -3.0e38f : (eps2 > 3.0e38f ? 3.0e38f : eps2)) * 0.25f; }

hipError_t launch_sum_squared(const void* points, long long ld, int n, int dPad, float* sums, float* halves, float eps2,
                              unsigned long long* counters, hipStream_t stream, unsigned long long epoch, bool reset) {
    const int chunksPerRow = dPad / 8;
    int lanesPerRow = 64;
    while (lanesPerRow > chunksPerRow) lanesPerRow >>= 1;
    const int rowsPerWave = 64 / lanesPerRow;
    const long long waves = ((long long)n + rowsPerWave - 1) / rowsPerWave;
    const long long blocks = (waves + 3) / 4;
    sum_squared_kernel<<<dim3((unsigned)blocks), dim3(256), 0, stream>>>(static_cast<const u32x4*>(points), ld / 8, n,
                                                                        chunksPerRow, lanesPerRow, sums, halves,
                                                                        quarter_eps2(eps2), counters, epoch, reset ? 1 : 0);
    return hipGetLastError();
}

hipError_t launch_halves(const float* sums, int n, float eps2, float* halves, unsigned long long* counters,
                         hipStream_t stream, unsigned long long epoch, bool reset) {
    halves_kernel<<<dim3((unsigned)((n + 255) / 256)), dim3(256), 0, stream>>>(sums, n, quarter_eps2(eps2), halves, counters,
                                                                               epoch, reset ? 1 : 0);
    return hipGetLastError();
}

hipError_t launch_padding_check(const void* points, long long ld, int n, int d, int dPad, unsigned long long* badRows,
                                hipStream_t stream) {
    if (dPad > d)
        padding_check_kernel<<<dim3((unsigned)((n + 255) / 256)), dim3(256), 0, stream>>>(
            static_cast<const unsigned short*>(points), ld, n, d, dPad, badRows);
    return hipGetLastError();
}

hipError_t launch_reset_counters(unsigned long long* counters, bool keepFound, hipStream_t stream) {
    reset_counters_kernel<<<1, 256, 0, stream>>>(counters, keepFound ? 1 : 0);
    return hipGetLastError();
}

hipError_t launch_offset_pairs(void* pairs, unsigned long long first, unsigned long long last, int qOffset, int cOffset,
                               hipStream_t stream) {
    if (last <= first || (qOffset == 0 && cOffset == 0)) return hipSuccess;
    const unsigned long long count = last - first;
    const unsigned blocks = (unsigned)((count + 255) / 256 < 4096 ? (count + 255) / 256 : 4096);
    offset_pairs_kernel<<<dim3(blocks), dim3(256), 0, stream>>>(static_cast<int2*>(pairs), first, last, qOffset, cOffset);
    return hipGetLastError();
}

hipError_t launch_offset_appended_pairs(void* pairs, unsigned long long* mark, const unsigned long long* counters,
                                        unsigned long long cap, int qOffset, int cOffset, hipStream_t stream) {
    offset_appended_pairs_kernel<<<dim3(512), dim3(256), 0, stream>>>(static_cast<int2*>(pairs), mark, counters, cap, qOffset,
                                                                     cOffset);
    return hipGetLastError();
}

namespace {

// One launch of the join kernel over the tile grid described by p.raster, in the queue or the direct mode, with
// tiles of 256 or 128 query rows.
hipError_t launch_join_grid(JoinParams p, bool rows128, bool tall, bool epilogue, int numCUs, hipStream_t stream) {
    const unsigned long long realTiles = (unsigned long long)p.raster.tileRows * p.raster.tileCols;
    // Up to two tiles per CU, workgroup b computes tile b and ends, one workgroup per tile (the hardware places
    // the second round as CUs fall free); from there on, one persistent workgroup per CU draws from the queues.
    p.direct = realTiles <= 2ull * (unsigned long long)numCUs ? 1 : 0;
    unsigned grid = (unsigned)(p.direct ? realTiles : (unsigned long long)numCUs);
    if (grid == 0) grid = 1;
    const dim3 g(grid), b(kThreads);
    const bool oneSlab = p.nSlabs == 1;
    // Tiles of up to 16 slabs gather their hit bits in their last slab; longer ones screen behind the k-loop.
    const bool bitsInLastSlab = epilogue && p.nSlabs <= 16;
    const int variant = (oneSlab ? 8 : 0) | (tall ? 2 : 0) | (rows128 ? 1 : 0);
    if (bitsInLastSlab) {
        switch (variant) {
            case 11: join_kernel<true, true, 128, true, true><<<g, b, 0, stream>>>(p); break;
            case 10: join_kernel<true, true, 256, true, true><<<g, b, 0, stream>>>(p); break;
            case 9: join_kernel<true, false, 128, true, true><<<g, b, 0, stream>>>(p); break;
            case 8: join_kernel<true, false, 256, true, true><<<g, b, 0, stream>>>(p); break;
            case 3: join_kernel<true, true, 128, false, true><<<g, b, 0, stream>>>(p); break;
            case 2: join_kernel<true, true, 256, false, true><<<g, b, 0, stream>>>(p); break;
            case 1: join_kernel<true, false, 128, false, true><<<g, b, 0, stream>>>(p); break;
            default: join_kernel<true, false, 256, false, true><<<g, b, 0, stream>>>(p); break;
        }
    } else if (epilogue) {  // more than 16 slabs
        switch (variant) {
            case 3: join_kernel<true, true, 128, false><<<g, b, 0, stream>>>(p); break;
            case 2: join_kernel<true, true, 256, false><<<g, b, 0, stream>>>(p); break;
            case 1: join_kernel<true, false, 128, false><<<g, b, 0, stream>>>(p); break;
            default: join_kernel<true, false, 256, false><<<g, b, 0, stream>>>(p); break;
        }
    } else {
        switch (variant) {
            case 11: join_kernel<false, true, 128, true><<<g, b, 0, stream>>>(p); break;
            case 10: join_kernel<false, true, 256, true><<<g, b, 0, stream>>>(p); break;
            case 9: join_kernel<false, false, 128, true><<<g, b, 0, stream>>>(p); break;
            case 8: join_kernel<false, false, 256, true><<<g, b, 0, stream>>>(p); break;
            case 3: join_kernel<false, true, 128, false><<<g, b, 0, stream>>>(p); break;
            case 2: join_kernel<false, true, 256, false><<<g, b, 0, stream>>>(p); break;
            case 1: join_kernel<false, false, 128, false><<<g, b, 0, stream>>>(p); break;
            default: join_kernel<false, false, 256, false><<<g, b, 0, stream>>>(p); break;
        }
    }
    return hipGetLastError();
}

}  // namespace

hipError_t launch_join(const JoinLaunch& launch, hipStream_t stream) {
    // (the compute units of the current device, looked up at every launch: the device may change between calls)
    int dev = 0, numCUs = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return e;
    e = hipDeviceGetAttribute(&numCUs, hipDeviceAttributeMultiprocessorCount, dev);
    if (e != hipSuccess) return e;
    const JoinLaunch& l = launch;
    JoinParams p;
    p.ptsQ = static_cast<const u32x4*>(l.queries);
    p.ptsC = static_cast<const u32x4*>(l.candidates);
    p.ldQ16 = l.ldQ / 8;
    p.ldC16 = l.ldC / 8;
    p.nQ = l.nQ;
    p.nC = l.nC;
    p.selfStride = l.forcedStride > 0 ? l.forcedStride : (l.selfJoin ? 1 : 0);
    p.symmetric = (l.selfJoin && l.symmetric) ? 1 : 0;
    p.nSlabs = l.dPad / kSlabK;
    p.halfQ = l.halfQ;
    p.halfC = l.halfC;
    p.counters = l.counters;
    p.epoch = l.epoch;
    p.pairs = static_cast<int2*>(l.pairs);
    p.cap = l.cap;
    // Tiles of 128 query rows when the matrix then still has no more tiles than the chip has workgroups (never
    // in symmetric mode, whose diagonal logic assumes square tiles): twice as many workgroups work, each on half a
    // tile.  A 128-row tile costs about 0.7 of a 256-row one (64 x 64 wave sub-tiles need a third more LDS fragment
    // reads per MFMA), so the finer grid only pays while it fits one round: measured on Exp(40) data, 1000 and 2154
    // points 1.1x - 1.4x faster, 3000 points (288 tiles of 128 rows: two rounds) 1.4x slower.
    // FASTED_TILE_ROWS=256 or 128 in the environment overrides the choice (tests run both).
    const unsigned long long tiles128 = (unsigned long long)((l.nQ + 127) / 128) * ((l.nC + kTile - 1) / kTile);
    bool rows128 = p.symmetric == 0 && tiles128 <= (unsigned long long)numCUs;
    const char* const forced = getenv("FASTED_TILE_ROWS");  // read at every launch: a test sets it per case
    const int forcedRows = forced ? atoi(forced) : 0;
    if (forcedRows == 256) rows128 = false;
    if (forcedRows == 128 && p.symmetric == 0) rows128 = true;
    const int tileRows = rows128 ? 128 : kTile;
    p.raster = make_raster(l.nQ, l.nC, p.symmetric != 0, tileRows);
    return launch_join_grid(p, rows128, tall_order(l.nQ, tileRows), l.epilogue, numCUs, stream);
}

}  // namespace fasted
