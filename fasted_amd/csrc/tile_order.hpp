// tile_order.hpp -- the order in which the join kernels walk the tiles of the distance matrix, and where
// the 16-byte chunks of an operand row go in LDS.  Plain C++ (host and device): the kernels use it with
// compile-time tile shapes, the library exports host mirrors of it, and a host-only build checks it
// under the address and undefined-behaviour sanitizers.
//
// Counterpart of Raster::OnDemandRasterizer (source/rasterizer/onDemandRasterizer.cuh:50-108) and
// SimSearch::SwizzleAddress (source/findPairs.cuh:161-166), re-cut for 8 accelerator dies (XCDs) with
// private L2 caches and for the 64-bank LDS of gfx950.
#pragma once

#if defined(__HIPCC__)
#define FASTED_HD __host__ __device__
#else
#define FASTED_HD
#endif

namespace fasted {

constexpr int kQueues = 8;  // one work queue per XCD

// Work queues.  The matrix of tiles is cut into super-squares of 4096 x 4096 points; a super-square is
// cut into 8 sub-rectangles of 1024 x 2048 points (`subRows` x `subCols` tiles), one per XCD, arranged
// 4 (down) x 2 (across).  Each XCD has its own queue head: position t of queue q is tile t % (subRows *
// subCols), row-major, of sub-rectangle q of super-square t / (subRows * subCols).  The workgroups
// resident on one XCD therefore work on a few query panels and candidate panels at a time and share them
// through that XCD's L2, and all 8 XCDs stay inside one super-square, which the Infinity Cache holds.
struct TileOrder {
    unsigned tileRows, tileCols;  // tiles along the queries / the candidates
    unsigned squareCols;          // super-squares per row of super-squares
    unsigned upperOnly;           // symmetric self-join: only the super-squares on and above the diagonal
    unsigned long long perQueue;  // positions each queue serves
};

FASTED_HD inline TileOrder make_tile_order(long long nQueries, long long nCandidates, int tileM, int tileN,
                                           int subRows, int subCols, bool upperOnly) {
    TileOrder r;
    r.tileRows = (unsigned)((nQueries + tileM - 1) / tileM);
    r.tileCols = (unsigned)((nCandidates + tileN - 1) / tileN);
    const unsigned squareRows = (r.tileRows + 4 * subRows - 1) / (4 * subRows);
    r.squareCols = (r.tileCols + 2 * subCols - 1) / (2 * subCols);
    r.upperOnly = (upperOnly && squareRows == r.squareCols) ? 1u : 0u;
    const unsigned long long squares = r.upperOnly ? (unsigned long long)squareRows * (squareRows + 1) / 2
                                                   : (unsigned long long)squareRows * r.squareCols;
    r.perQueue = squares * (unsigned)(subRows * subCols);
    return r;
}

// Position t of queue q -> tile (row, col) in tile units.  Tiles outside the tileRows x tileCols grid
// are padding of the last super-squares: the caller skips them.
FASTED_HD inline void tile_order_decode(const TileOrder& r, int subRows, int subCols, unsigned q,
                                        unsigned long long t, unsigned* tr, unsigned* tc) {
    const unsigned subTiles = (unsigned)(subRows * subCols);
    const unsigned long long sq = t / subTiles;
    const unsigned local = (unsigned)(t % subTiles);
    unsigned squareRow, squareCol;
    if (r.upperOnly) {
        // row-major over the upper triangle: row i starts at i*S - i*(i-1)/2; estimate, then correct
        const unsigned long long S = r.squareCols;
        const double b = 2.0 * (double)S + 1.0;
        long long i = (long long)((b - __builtin_sqrt(b * b - 8.0 * (double)sq)) * 0.5);
        if (i < 0) i = 0;
        if (i >= (long long)S) i = (long long)S - 1;
        auto start = [S](long long row) {
            return (unsigned long long)row * S - (unsigned long long)(row * (row - 1) / 2);
        };
        while (i > 0 && start(i) > sq) --i;
        while (i + 1 < (long long)S && start(i + 1) <= sq) ++i;
        squareRow = (unsigned)i;
        squareCol = (unsigned)(i + (long long)(sq - start(i)));
    } else {
        squareRow = (unsigned)(sq / r.squareCols);
        squareCol = (unsigned)(sq % r.squareCols);
    }
    *tr = squareRow * (unsigned)(4 * subRows) + (q >> 1) * (unsigned)subRows + local / (unsigned)subCols;
    *tc = squareCol * (unsigned)(2 * subCols) + (q & 1) * (unsigned)subCols + local % (unsigned)subCols;
}

// LDS placement of operand rows.  gfx950 serves a ds_read_b128 in four phases of 16 lanes --
// {0-3,12-15,20-23,24-27}, {4-7,8-11,16-19,28-31} and the same two groups +32 -- and the fragment read
// of v_mfma_f32_16x16x32_f16 has lane l on row l%16, 16-byte chunk l/16 of a 32-wide k-step.  A phase is
// conflict free when its 16 lanes touch all 64 four-byte banks once.
//
// Rows of 128 bytes (a 64-wide k-slab, 8 chunks): chunk c of row r is stored at slot c ^ ((r>>1)&7).
FASTED_HD inline int lds_swizzle128(int row) { return (row >> 1) & 7; }
// Rows of 64 bytes (a 32-wide k-step, 4 chunks): chunk c of row r is stored at slot c ^ ((r>>2)&2).
FASTED_HD inline int lds_swizzle64(int row) { return (row >> 2) & 2; }

}  // namespace fasted
