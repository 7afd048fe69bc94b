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
constexpr int kLdsNext = kLdsSums + 2 * kSumsBytes; // next tile of this workgroup: (row, col) as two u32
constexpr int kLdsStageCount = kLdsNext + 16;       // pairs waiting in the LDS staging area (u32) + flush base (u64)
constexpr int kLdsStage = kLdsStageCount + 16;      // staged pairs
constexpr int kStagePairs = 3072;                   // 24 KiB of 8-byte records
constexpr int kLdsBytes = kLdsStage + kStagePairs * 8;
static_assert(kLdsBytes <= 160 * 1024, "LDS budget of one CU");
constexpr int kWaveRows = 128, kWaveCols = 64;      // output sub-tile of one wave
constexpr int kFragRows = kWaveRows / 16, kFragCols = kWaveCols / 16;  // 8 x 4 MFMA 16x16 blocks

// Operand rows of the 256x256 kernel are 128 bytes (a 64-wide k-slab): see lds_swizzle128 in
// tile_order.hpp (conflict freedom is checked exhaustively on the host by tests, and with the
// SQ_LDS_BANK_CONFLICT counter on the device).
__host__ __device__ __forceinline__ int swz(int row) { return lds_swizzle128(row); }

// Work queues of the 256x256 kernel (tile_order.hpp): an XCD's sub-rectangle is 4 x 8 tiles, so the 32
// workgroups resident on one XCD work on 4 query panels and 8 candidate panels at a time.  An XCD whose
// queue is exhausted steals from the next XCD's queue, so the tail stays balanced.
typedef TileOrder Raster;
constexpr int kSubRows = 4, kSubCols = 8;  // sub-rectangle of one XCD inside a super-square
constexpr int kSubTiles = kSubRows * kSubCols;
static_assert(kRaster == 16 && kSubTiles * kQueues == kRaster * kRaster, "8 sub-rectangles tile a super-square");

__host__ __device__ inline Raster make_raster(long long nQueries, long long nCandidates, bool upperOnly = false) {
    return make_tile_order(nQueries, nCandidates, kTile, kTile, kSubRows, kSubCols, upperOnly);
}

__host__ __device__ inline void raster_decode(const Raster& r, unsigned q, unsigned long long t, unsigned* tr,
                                              unsigned* tc) {
    tile_order_decode(r, kSubRows, kSubCols, q, t, tr, tc);
}

// ------------------------------------------------------------------------------------------
__global__ void __launch_bounds__(256) sum_squared_kernel(const u32x4* __restrict__ pts, long long ld16, int n,
                                                          int chunksPerRow, int lanesPerRow,
                                                          float* __restrict__ sums) {
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
    if (sub == 0 && row < n) sums[row] = acc;
}

// Clears the queue heads and, unless `keepFound`, the pair counter (word 0): a launch that keeps it
// appends its pairs behind those of the launch before.
__global__ void reset_counters_kernel(unsigned long long* c, int keepFound) {
    if (threadIdx.x < kCounterWords && !(keepFound && threadIdx.x == kCounterFound)) c[threadIdx.x] = 0ull;
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

// ------------------------------------------------------------------------------------------
template <bool kEpilogue>
__global__ void __launch_bounds__(kThreads, 1) join_kernel(JoinParams p) {
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
    unsigned* const sNext = reinterpret_cast<unsigned*>(lds + kLdsNext);  // next tile: [0] row, [1] col
    unsigned* const sStageCount = reinterpret_cast<unsigned*>(lds + kLdsStageCount);
    unsigned long long* const sFlushBase = reinterpret_cast<unsigned long long*>(lds + kLdsStageCount + 8);
    int2* const sStage = reinterpret_cast<int2*>(lds + kLdsStage);

    // Which XCD this workgroup runs on (hardware register XCC_ID, low 3 bits).
    const unsigned home = __builtin_amdgcn_s_getreg(20 | (0 << 6) | ((4 - 1) << 11)) & (kQueues - 1);
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
                raster_decode(ras, q, pos, &tr, &tc);
                if (tr < ras.tileRows && tc < ras.tileCols && !(p.symmetric && tc < tr)) {
                    *row = tr;
                    *col = tc;
                    return;
                }
            } else {
                if (++hops == kQueues) return;  // every queue is exhausted
                q = (q + 1) & (kQueues - 1);
            }
            pos = atomicAdd(&p.counters[kQueueBase + q * kQueueStride], 1ull);
        }
    };

    // Pairs are staged in LDS and appended to the global list by the whole workgroup: one
    // reservation on the global counter per flush instead of one per wave and tile, which is what
    // bounds output-heavy joins (same-address atomics serialise at about 12 ns each).
    auto flush_stage = [&](unsigned staged) {
        const unsigned cnt = staged < (unsigned)kStagePairs ? staged : (unsigned)kStagePairs;
        const unsigned tid = (unsigned)(wave * 64 + lane_now());
        if (tid == 0) *sFlushBase = atomicAdd(&p.counters[kCounterFound], (unsigned long long)cnt);
        __syncthreads();
        const unsigned long long gb = *sFlushBase;
        for (unsigned i = tid; i < cnt; i += kThreads)
            if (gb + i < p.cap) p.pairs[gb + i] = sStage[i];  // past the capacity: counted, not stored
        __syncthreads();
        if (tid == 0) *sStageCount = 0u;
        __syncthreads();
    };

    // Byte offsets, from the tile's first row, of the 16-byte chunks this lane copies: 4 query rows and
    // 4 candidate rows per slab.  Rows past the end of the dataset re-read the last real row; their
    // results are masked.  The swizzle is applied here, on the global side.
    auto tile_offsets = [&](int rowBase, int colBase, unsigned (&oA)[4], unsigned (&oB)[4]) {
        const int ln = lane_now();
        const int row0 = wave * 32 + (ln >> 3);
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int r = row0 + 8 * i;
            const int chunk = (ln & 7) ^ swz(r);
            oA[i] = (unsigned)(min(r, p.nQ - 1 - rowBase) * (int)p.ldQ16 + chunk) * 16u;
            oB[i] = (unsigned)(min(r, p.nC - 1 - colBase) * (int)p.ldC16 + chunk) * 16u;
        }
    };

    // One 1-KiB global->LDS transfer of this wave (global_load_lds_dwordx4: no registers in between);
    // j = 0..7 alternates query / candidate rows.  Lane l lands in row l/8, chunk slot l%8 of the
    // 8 rows the instruction fills; wave w owns rows [32w, 32w+32) of both operands.
    auto issue_load = [&](const char* gA, const char* gB, const unsigned (&oA)[4], const unsigned (&oB)[4],
                          unsigned slabByte, int stage, int j) {
        const int i = j >> 1;
        unsigned char* const dst = lds + stage * kStageBytes + (j & 1) * kOperandBytes + (wave * 32 + i * 8) * kRowBytes;
        // uniform 64-bit base + 32-bit lane offset (formed here so it stays a 32-bit add)
        const char* const src = (j & 1) ? gB + (oB[i] + slabByte) : gA + (oA[i] + slabByte);
        __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)src,
                                         (__attribute__((address_space(3))) void*)dst, 16, 0, 0);
    };

    // Squared norms of a tile's 256 queries (waves 0-3) and 256 candidates (waves 4-7), 64 floats per
    // wave, straight into the sums buffer `which`.
    auto issue_sums = [&](int rowBase, int colBase, int which) {
        const int ln = lane_now();
        const int part = wave & 3;
        const float* src = wave < 4 ? p.sumsQ + min(rowBase + part * 64 + ln, p.nQ - 1)
                                    : p.sumsC + min(colBase + part * 64 + ln, p.nC - 1);
        unsigned char* const dst = lds + kLdsSums + which * kSumsBytes + wave * 256;
        __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)src,
                                         (__attribute__((address_space(3))) void*)dst, 4, 0, 0);
    };

    // ---- first tile
    if (wave == 0 && lane_now() == 0) {
        *sStageCount = 0u;
        unsigned r, c;
        find_tile(atomicAdd(&p.counters[kQueueBase + home * kQueueStride], 1ull), &r, &c);
        sNext[0] = r;
        sNext[1] = c;
    }
    __syncthreads();
    unsigned tr = __builtin_amdgcn_readfirstlane(sNext[0]);
    unsigned tc = __builtin_amdgcn_readfirstlane(sNext[1]);
    if (tr == kNoTile) return;
    __syncthreads();  // everybody has read sNext before thread 0 writes the second tile there

    unsigned offA[4], offB[4];
    tile_offsets((int)tr * kTile, (int)tc * kTile, offA, offB);
    const char* gA = reinterpret_cast<const char*>(p.ptsQ + (long long)tr * kTile * p.ldQ16);
    const char* gB = reinterpret_cast<const char*>(p.ptsC + (long long)tc * kTile * p.ldC16);
#pragma unroll
    for (int j = 0; j < 8; ++j) issue_load(gA, gB, offA, offB, 0u, 0, j);
    issue_sums((int)tr * kTile, (int)tc * kTile, 0);
    unsigned long long popped = 0;  // thread 0: the home queue position reserved for the tile after the current one
    if (wave == 0 && lane_now() == 0) popped = atomicAdd(&p.counters[kQueueBase + home * kQueueStride], 1ull);

    int stage = 0;  // LDS stage that holds slab 0 of the current tile
    int sumsBuf = 0;

    for (;;) {
        // slab 0 of this tile (issued during the previous tile's last slab) has landed
        __syncthreads();
        if (kEpilogue) {
            const unsigned staged = __builtin_amdgcn_readfirstlane(*sStageCount);
            if (staged >= (unsigned)kStagePairs / 2) flush_stage(staged);
        }
        if (wave == 0 && lane_now() == 0) {
            // the reservation made a whole tile ago has long arrived: no wait here
            unsigned r, c;
            find_tile(popped, &r, &c);
            sNext[0] = r;
            sNext[1] = c;
            popped = atomicAdd(&p.counters[kQueueBase + home * kQueueStride], 1ull);
        }

        // the accumulators start at -(s_q + s_c)/2 (see test_block): the tile's squared norms landed
        // together with slab 0
        floatx4 acc[kFragRows][kFragCols];
        {
            const int ln = lane_now();
            const float* const sQw =
                reinterpret_cast<const float*>(lds + kLdsSums + sumsBuf * kSumsBytes) + wr * kWaveRows + (ln >> 4) * 4;
            const float* const sCw =
                reinterpret_cast<const float*>(lds + kLdsSums + sumsBuf * kSumsBytes) + kTile + wc * kWaveCols + (ln & 15);
            float hc[kFragCols];
#pragma unroll
            for (int fj = 0; fj < kFragCols; ++fj) hc[fj] = -0.5f * sCw[fj * 16];
#pragma unroll
            for (int fi = 0; fi < kFragRows; ++fi) {
                const floatx4 hq = *reinterpret_cast<const floatx4*>(sQw + fi * 16) * -0.5f;
#pragma unroll
                for (int fj = 0; fj < kFragCols; ++fj) acc[fi][fj] = hq + hc[fj];
            }
        }

        // One slab = 2 k-steps of 32; a k-step is two halves of 16 MFMAs (query blocks 0-3, then
        // 4-7, each against the 4 candidate blocks, query fragment held for 4 MFMAs, candidate blocks
        // in snake order: consecutive MFMAs always share an operand, which the power-limited clock
        // rewards with about 1.5 %).  The instruction order is pinned with
        // scheduling barriers: the LDS reads for the next half are issued ahead of the MFMAs of
        // the current half, and the 8 global->LDS transfers of the following slab are issued one per
        // 4 MFMAs during the first k-step: spaced so that the texture-address queue never makes a
        // wave wait with the matrix pipe idle, early so that an L2 miss has the whole second
        // k-step to land before the slab's barrier.
        auto slab_step = [&](int stg, bool prefetch, const char* pA, const char* pB, const unsigned (&oA)[4],
                             const unsigned (&oB)[4], unsigned nextByte) {
            const unsigned char* const buf = lds + stg * kStageBytes;
            half8 aLo[4], aHi[4], b[2][kFragCols];
#pragma unroll
            for (int fj = 0; fj < kFragCols; ++fj)
                b[0][fj] = *reinterpret_cast<const half8*>(buf + bOff[0] + fj * 16 * kRowBytes);
#pragma unroll
            for (int fi = 0; fi < 4; ++fi)
                aLo[fi] = *reinterpret_cast<const half8*>(buf + aOff[0] + fi * 16 * kRowBytes);
#pragma unroll
            for (int ks = 0; ks < 2; ++ks) {
#pragma unroll
                for (int fi = 0; fi < 4; ++fi)
                    aHi[fi] = *reinterpret_cast<const half8*>(buf + aOff[ks] + (fi + 4) * 16 * kRowBytes);
                __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                for (int fi = 0; fi < 4; ++fi) {
                    if (ks == 0 && prefetch) issue_load(pA, pB, oA, oB, nextByte, stg ^ 1, fi);
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
                        b[1][fj] = *reinterpret_cast<const half8*>(buf + bOff[1] + fj * 16 * kRowBytes);
#pragma unroll
                    for (int fi = 0; fi < 4; ++fi)
                        aLo[fi] = *reinterpret_cast<const half8*>(buf + aOff[1] + fi * 16 * kRowBytes);
                }
                __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                for (int fi = 0; fi < 4; ++fi) {
                    if (ks == 0 && prefetch) issue_load(pA, pB, oA, oB, nextByte, stg ^ 1, 4 + fi);
#pragma unroll
                    for (int fs = 0; fs < kFragCols; ++fs) {
                        const int fj = (fi & 1) ? kFragCols - 1 - fs : fs;
                        acc[fi + 4][fj] =
                            __builtin_amdgcn_mfma_f32_16x16x32_f16(aHi[fi], b[ks][fj], acc[fi + 4][fj], 0, 0, 0);
                    }
                }
                __builtin_amdgcn_sched_barrier(0);
            }
        };

        for (int s = 0; s + 1 < p.nSlabs; ++s) {
            slab_step(stage, true, gA, gB, offA, offB, (unsigned)(s + 1) * kRowBytes);
            stage ^= 1;
            __syncthreads();
        }
        if (p.nSlabs == 1) __syncthreads();  // with a single slab no barrier has published sNext yet

        // The tile after this one: its first slab and its squared norms travel during this tile's last
        // slab and epilogue.  The current tile's offsets are not needed any more, so the next tile's
        // take their registers.
        const unsigned ntr = __builtin_amdgcn_readfirstlane(sNext[0]);
        const unsigned ntc = __builtin_amdgcn_readfirstlane(sNext[1]);
        const bool more = ntr != kNoTile;
        if (more) {
            tile_offsets((int)ntr * kTile, (int)ntc * kTile, offA, offB);
            gA = reinterpret_cast<const char*>(p.ptsQ + (long long)ntr * kTile * p.ldQ16);
            gB = reinterpret_cast<const char*>(p.ptsC + (long long)ntc * kTile * p.ldC16);
            issue_sums((int)ntr * kTile, (int)ntc * kTile, sumsBuf ^ 1);
        }
        slab_step(stage, more, gA, gB, offA, offB, 0u);
        stage ^= 1;

        if (kEpilogue) {
            const int rowBase = (int)tr * kTile, colBase = (int)tc * kTile;
            const int ln = lane_now();
            const int l16 = ln & 15, quad = ln >> 4;
            const int qBase = rowBase + wr * kWaveRows;
            int cand[kFragCols];
#pragma unroll
            for (int fj = 0; fj < kFragCols; ++fj) cand[fj] = colBase + wc * kWaveCols + fj * 16 + l16;
            const float thr = -0.5f * p.eps2;
            const bool edge = (p.selfJoin && tr == tc) || rowBase + kTile > p.nQ || colBase + kTile > p.nC;
            unsigned mask[kFragRows / 2];
            if (edge)
                test_block<kFragRows, kFragCols, true>(acc, cand, qBase, quad, p.nQ, p.nC, p.selfJoin, thr, mask);
            else
                test_block<kFragRows, kFragCols, false>(acc, cand, qBase, quad, p.nQ, p.nC, p.selfJoin, thr, mask);

            // symmetric mode: a tile above the diagonal also stands for its mirror image
            const bool mirror = p.symmetric && tr != tc;
            int mine = 0;
#pragma unroll
            for (int fp = 0; fp < kFragRows / 2; ++fp) mine += __builtin_popcount(mask[fp]);
            if (mirror) mine *= 2;
            if (__builtin_amdgcn_ballot_w64(mine != 0) != 0ull) {
                // wave-level compaction: inclusive prefix sum of per-lane counts, one reservation
                // (data-parallel-primitive moves inside the vector ALU: shifts within rows of 16 lanes, then the
                // last lane of row 0/2 added to row 1/3, then lane 31 to the upper half)
                int incl = mine;
                incl += __builtin_amdgcn_update_dpp(0, incl, 0x111, 0xf, 0xf, false);  // row_shr:1
                incl += __builtin_amdgcn_update_dpp(0, incl, 0x112, 0xf, 0xf, false);  // row_shr:2
                incl += __builtin_amdgcn_update_dpp(0, incl, 0x114, 0xf, 0xf, false);  // row_shr:4
                incl += __builtin_amdgcn_update_dpp(0, incl, 0x118, 0xf, 0xf, false);  // row_shr:8
                incl += __builtin_amdgcn_update_dpp(0, incl, 0x142, 0xa, 0xf, false);  // row_bcast:15 -> rows 1, 3
                incl += __builtin_amdgcn_update_dpp(0, incl, 0x143, 0xc, 0xf, false);  // row_bcast:31 -> rows 2, 3
                const unsigned total = (unsigned)__builtin_amdgcn_readlane(incl, 63);
                // reserve room in the staging area (LDS atomic); what does not fit goes straight
                // to the global list with a reservation of this wave's own
                // (LDS atomic and LDS stores below are written as instructions: for ordinary LDS writes the
                // compiler first waits until this wave's global->LDS transfers of the next tile have landed)
                unsigned pos = 0;
                if (ln == 0)
                    asm volatile("ds_add_rtn_u32 %0, %1, %2\n\ts_waitcnt lgkmcnt(0)"
                                 : "=v"(pos)
                                 : "v"(ldsBase + (unsigned)kLdsStageCount), "v"(total)
                                 : "memory");
                pos = __builtin_amdgcn_readfirstlane(pos);
                const unsigned room = pos < (unsigned)kStagePairs ? (unsigned)kStagePairs - pos : 0u;
                const unsigned fit = total < room ? total : room;
                unsigned long long gbase = 0;
                if (fit < total) {
                    if (ln == 0) gbase = atomicAdd(&p.counters[kCounterFound], (unsigned long long)(total - fit));
                    gbase = ((unsigned long long)__builtin_amdgcn_readfirstlane((unsigned)(gbase >> 32)) << 32) |
                            __builtin_amdgcn_readfirstlane((unsigned)gbase);
                }
                unsigned idx = (unsigned)(incl - mine);
#pragma unroll
                for (int fp = 0; fp < kFragRows / 2; ++fp) {
                    unsigned m = mask[fp];
                    while (m) {
                        const int low = __builtin_ctz(m);
                        m &= m - 1;
                        const int bit = 31 - low;  // element number inside the pair of row blocks
                        const int fi = fp * 2 + (bit >> 4), fj = (bit >> 2) & 3, r = bit & 3;
                        const int q = qBase + fi * 16 + quad * 4 + r;
                        const int c = colBase + wc * kWaveCols + fj * 16 + l16;
                        auto put = [&](unsigned at, int first, int second) {
                            if (at < fit) {
                                const unsigned long long rec =
                                    (unsigned long long)(unsigned)first | ((unsigned long long)(unsigned)second << 32);
                                asm volatile("ds_write_b64 %0, %1" ::"v"(ldsBase + (unsigned)kLdsStage + (pos + at) * 8u), "v"(rec)
                                             : "memory");
                            } else {
                                const unsigned long long slot = gbase + (at - fit);
                                if (slot < p.cap) p.pairs[slot] = make_int2(first, second);
                            }
                        };
                        put(idx++, q, c);
                        if (mirror) put(idx++, c, q);
                    }
                }
                asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");  // the staged records are in LDS
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
        __syncthreads();
        const unsigned staged = __builtin_amdgcn_readfirstlane(*sStageCount);
        if (staged > 0) flush_stage(staged);
    }
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
    raster_decode(r, (unsigned)(idx % kQueues), idx / kQueues, &tr, &tc);
    *row = (int)tr * kTile;
    *col = (int)tc * kTile;
    return (tr < r.tileRows && tc < r.tileCols && !(upperOnly && tc < tr)) ? 1 : 2;
}

int counter_words() { return kCounterWords; }

unsigned long long tile_count(long long nQ, long long nC) {
    const Raster r = make_raster(nQ, nC);
    return (unsigned long long)r.tileRows * r.tileCols;
}

int lds_chunk_slot(int row, int chunk) { return (chunk ^ swz(row)) & 7; }

hipError_t launch_sum_squared(const void* points, long long ld, int n, int dPad, float* sums, hipStream_t stream) {
    const int chunksPerRow = dPad / 8;
    int lanesPerRow = 64;
    while (lanesPerRow > chunksPerRow) lanesPerRow >>= 1;
    const int rowsPerWave = 64 / lanesPerRow;
    const long long waves = ((long long)n + rowsPerWave - 1) / rowsPerWave;
    const long long blocks = (waves + 3) / 4;
    sum_squared_kernel<<<dim3((unsigned)blocks), dim3(256), 0, stream>>>(static_cast<const u32x4*>(points), ld / 8, n,
                                                                        chunksPerRow, lanesPerRow, sums);
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

hipError_t launch_join(const JoinLaunch& launch, hipStream_t stream) {
    static int numCUs = 0;
    static bool configured = false;
    if (!configured) {
        int dev = 0;
        hipError_t e = hipGetDevice(&dev);
        if (e != hipSuccess) return e;
        hipDeviceProp_t prop;
        e = hipGetDeviceProperties(&prop, dev);
        if (e != hipSuccess) return e;
        numCUs = prop.multiProcessorCount;
        configured = true;
    }
    JoinLaunch l = launch;
    // the kernels compare against -eps^2/2 and rely on that threshold being finite
    if (!(l.eps2 < 3.0e38f)) l.eps2 = 3.0e38f;
    JoinParams p;
    p.ptsQ = static_cast<const u32x4*>(l.queries);
    p.ptsC = static_cast<const u32x4*>(l.candidates);
    p.ldQ16 = l.ldQ / 8;
    p.ldC16 = l.ldC / 8;
    p.nQ = l.nQ;
    p.nC = l.nC;
    p.selfJoin = l.selfJoin ? 1 : 0;
    p.symmetric = (l.selfJoin && l.symmetric) ? 1 : 0;
    p.nSlabs = l.dPad / kSlabK;
    p.eps2 = l.eps2;
    p.sumsQ = l.sumsQ;
    p.sumsC = l.sumsC;
    p.counters = l.counters;
    p.pairs = static_cast<int2*>(l.pairs);
    p.cap = l.cap;
    p.raster = make_raster(l.nQ, l.nC, p.symmetric != 0);
    unsigned long long realTiles = (unsigned long long)p.raster.tileRows * p.raster.tileCols;
    unsigned grid = (unsigned)(realTiles < (unsigned long long)numCUs ? realTiles : (unsigned long long)numCUs);
    if (grid == 0) grid = 1;
    if (l.epilogue)
        join_kernel<true><<<dim3(grid), dim3(kThreads), 0, stream>>>(p);
    else
        join_kernel<false><<<dim3(grid), dim3(kThreads), 0, stream>>>(p);
    return hipGetLastError();
}

}  // namespace fasted
