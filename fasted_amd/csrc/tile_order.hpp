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

// Work queues.  The matrix of tiles is cut into super-squares of 4 * subRows x 2 * subCols tiles; a
// super-square is cut into 8 sub-rectangles of subRows x subCols
// tiles, one per XCD, arranged 4 (down) x 2 (across).  Each XCD has its own queue head: position t of
// queue q is tile t % (subRows * subCols), row-major, of sub-rectangle q of super-square t / (subRows *
// subCols); the super-squares follow each other along a row of the matrix.  The workgroups resident on one
// XCD therefore work on a few query panels and candidate panels at a time and share them through that
// XCD's L2, all 8 XCDs stay inside one super-square, and from one super-square to the next the query
// panels stay (the Infinity Cache holds them) while only the candidate panels are new: the taller the
// super-square, the fewer bytes come from HBM.
struct TileOrder {
    unsigned tileRows, tileCols;  // tiles along the queries / the candidates
    unsigned squareCols;          // super-squares per row of super-squares
    unsigned upperOnly;           // symmetric self-join: only the super-squares that reach the diagonal or lie above it
    unsigned long long perQueue;  // positions each queue serves
};

// With `upperOnly` (square matrix, square tiles, super-squares a whole number of times taller than wide:
// ratio = height / width) row i of super-squares keeps the squares from column ratio * i on: those hold
// every tile on or above the diagonal.  Row i starts at position i * S - ratio * i * (i - 1) / 2 of that order.
FASTED_HD inline unsigned long long tile_order_row_start(unsigned long long squareCols, unsigned ratio, long long row) {
    return (unsigned long long)row * squareCols - (unsigned long long)ratio * (unsigned long long)(row * (row - 1) / 2);
}

FASTED_HD inline TileOrder make_tile_order(long long nQueries, long long nCandidates, int tileM, int tileN,
                                           int subRows, int subCols, bool upperOnly) {
    TileOrder r;
    r.tileRows = (unsigned)((nQueries + tileM - 1) / tileM);
    r.tileCols = (unsigned)((nCandidates + tileN - 1) / tileN);
    const unsigned height = 4u * (unsigned)subRows, width = 2u * (unsigned)subCols;  // of a super-square, in tiles
    const unsigned squareRows = (r.tileRows + height - 1) / height;
    r.squareCols = (r.tileCols + width - 1) / width;
    r.upperOnly = (upperOnly && height % width == 0 && tileM == tileN && r.tileRows == r.tileCols) ? 1u : 0u;
    const unsigned long long squares = r.upperOnly ? tile_order_row_start(r.squareCols, height / width, squareRows)
                                                   : (unsigned long long)squareRows * r.squareCols;
    r.perQueue = squares * (unsigned)(subRows * subCols);
    return r;
}

// Position t of queue q -> tile (row, col) in tile units, for the sub-rectangle shape the order was made
// with.  Tiles outside the tileRows x tileCols grid are padding of the last super-squares: the caller
// skips them.
FASTED_HD inline void tile_order_decode(const TileOrder& r, int subRows, int subCols, unsigned q,
                                        unsigned long long t, unsigned* tr, unsigned* tc) {
    const unsigned subTiles = (unsigned)(subRows * subCols);
    const unsigned long long sq = t / subTiles;
    const unsigned local = (unsigned)(t % subTiles);
    const unsigned height = 4u * (unsigned)subRows, width = 2u * (unsigned)subCols;
    unsigned squareRow, squareCol;
    if (r.upperOnly) {
        // smaller root of  ratio/2 * i^2 - (S + ratio/2) * i + sq = 0  as an estimate, then corrected
        const unsigned ratio = height / width;
        const unsigned long long S = r.squareCols;
        const long long rowsOfSquares = (long long)((r.tileRows + height - 1) / height);
        const double b = (double)S + 0.5 * (double)ratio;
        const double disc = b * b - 2.0 * (double)ratio * (double)sq;
        long long i = (long long)((b - __builtin_sqrt(disc > 0.0 ? disc : 0.0)) / (double)ratio);
        if (i < 0) i = 0;
        if (i >= rowsOfSquares) i = rowsOfSquares - 1;
        while (i > 0 && tile_order_row_start(S, ratio, i) > sq) --i;
        while (i + 1 < rowsOfSquares && tile_order_row_start(S, ratio, i + 1) <= sq) ++i;
        squareRow = (unsigned)i;
        squareCol = (unsigned)((long long)ratio * i + (long long)(sq - tile_order_row_start(S, ratio, i)));
    } else {
        squareRow = (unsigned)(sq / r.squareCols);
        squareCol = (unsigned)(sq % r.squareCols);
    }
    *tr = squareRow * height + (q >> 1) * (unsigned)subRows + local / (unsigned)subCols;
    *tc = squareCol * width + (q & 1) * (unsigned)subCols + local % (unsigned)subCols;
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
