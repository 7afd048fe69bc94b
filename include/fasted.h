/*
 * fasted.h -- C ABI of libfasted.so, the MI355X (gfx950) epsilon self-join.
 *
 * Two groups of entry points:
 *
 *  1. The four symbols the reference's `make shared` library (main.so) exports and that
 *     results/scripts/experiment/find_pairs.py:93-127 binds with ctypes.  Same names,
 *     argument order, `Results` layout (returned by value) and process-global dataset
 *     residency, so `ctypes.CDLL("libfasted.so")` can stand in for `main.so`.
 *
 *  2. Raw-buffer entry points ("points, N, D, epsilon in; pair list and count out") that
 *     the reference does not have: its pairs only leave the library through a text file.
 *     They report failure through a return code instead of exiting the process.
 *
 * All pointers are plain C pointers; sizes are explicit; nothing here depends on torch.
 * The library is not re-entrant (process-global resident dataset, one device, one stream
 * at a time), exactly like the reference (source/main.cu:33, source/findPairs.cuh:52).
 */
#ifndef FASTED_H
#define FASTED_H

#include <stdbool.h>
#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* source/ptxMma.cuh:27-31 */
typedef struct mmaShape {
    int m, n, k;
} mmaShape;

/* source/findPairs.cuh:37-46; mirrored by find_pairs.py:24-44.  56 bytes. */
typedef struct Results {
    double totalTime;              /* seconds: upload + kernels + sort + download and, with savePairs, the writing of
                                      the .pairs file (as source/findPairs.cuh:700-726 times it) */
    double TFLOPS;                 /* 2*N*N*D / (counter reset + sumSquared + join kernel time) / 1e12, unpadded N, D.
                                      The reference's window (source/findPairs.cuh:625-697,729) also spans its pair-buffer
                                      allocation and rasterizer set-up; here the pair buffer is kept between calls */
    unsigned long long pairsFound; /* every ordered pair with dist <= eps, self pairs included */
    unsigned long long pairsStored; /* <= pairsFound when the pair buffer overflowed */
    mmaShape inputProblemShape;    /* (N, N, D) as given */
    mmaShape paddedProblemShape;   /* (N_pad, N_pad, D_pad) as resident on the device */
} Results;

/* source/pair.cuh:27-46.  8 bytes, ordered row-major (QueryPoint, then CandidatePoint). */
typedef struct FastedPair {
    int QueryPoint;
    int CandidatePoint;
} FastedPair;

/* ---- group 1: drop-in for main.so ------------------------------------------------- */

/* source/main.cu:66-67,250-261.  Seeded Exp(lambda) points rejected to [0, max], FP16. */
Results runFromExponentialDataset(int size, int dimensionality, double lambda, double max, double epsilon,
                                  bool savePairs);

/* source/main.cu:54,263-273.  One point per line, comma separated. */
Results runFromFile(const char* filename, double epsilon, bool savePairs);

/* source/main.cu:45,275-278.  New epsilon on the dataset already resident on host+device. */
Results reRun(double epsilon, bool savePairs);

/* source/main.cu:74,280 (there it recurses into itself; here it frees the resident
 * dataset as its comment intends, source/findPairs.cuh:766-776). */
void releaseResources(void);

/* ---- group 2: raw buffers ----------------------------------------------------------
 * Return 0 on success, non-zero on failure; fasted_last_error() then describes it.     */

/* The two kernel times are HIP-event times on the stream, as the reference measures them
 * (source/findPairs.cuh:625-639,695-697); for joins of at most 512 tiles of 256 x 256, where three event records
 * would cost a third of the call, they are differences of the device's constant-rate clock, read by the kernels
 * themselves (hipDeviceAttributeWallClockRate ticks): by the first norm kernel and the join kernel as they start,
 * and by the join kernel's last workgroup when it has nothing left to do. */
typedef struct FastedJoinStats {
    float sumSquaredMs; /* squared-norm pre-pass (which also clears the counters): its start to the join kernel's start */
    float joinMs;       /* the join kernel: its start to the event behind it (small joins: to its last workgroup's report) */
    float sortMs;       /* host wall time of the row-major sort, stream synchronisation included (0 when not sorted) */
    int paddedN;        /* rows covered by the tile grid */
    int paddedD;        /* K extent the kernel looped over */
    unsigned long long tiles;      /* size of the distance matrix in 256x256 tiles (with FASTED_SYMMETRIC: those on and
                                      above the diagonal); small matrices are computed in 128x256 tiles, two per unit */
    unsigned long long pairsFound;
    unsigned long long pairsStored;
} FastedJoinStats;

/* Flags for fasted_self_join_device. */
enum {
    FASTED_SORT_PAIRS = 1,  /* sort stored pairs row-major, as source/pair.cuh:151-158 */
    FASTED_NO_EPILOGUE = 2, /* measurement only: run the contraction, skip test + emit */
    FASTED_SKIP_SUMS = 4,   /* d_sums already holds the squared norms */
    FASTED_SYMMETRIC = 8,   /* self-join only, off by default: dist(q,c) = dist(c,q), so compute only the tiles
                               on and above the diagonal and emit both orientations of every pair found there.
                               Same pair set, about half the matrix-core work; the reference always computes the
                               full matrix (source/findPairs.cuh:650-653), which is also this library's default
                               and what its TFLOPS figure assumes. */
    FASTED_EVENT_TIMING = 16 /* time the kernels with HIP events and wait for the stream whatever the size of the
                               join, as the reference does (source/findPairs.cuh:625-639,695-697): for joins of at
                               most 512 tiles this costs the call about 15 us and is what a profiler's kernel
                               durations compare with. */
};

/* Host buffers in, host buffers out.  `points` is N x D row-major IEEE binary16 bit
 * patterns (what source/DataLoader/PointListBuilder.hpp:57-73 produces, before padding);
 * up to `cap` pairs are written to `out` sorted row-major; *found counts every pair
 * (source/pair.cuh:123-133), *stored = min(found, cap).  Replaces the body of
 * SimSearch::FindPairs (source/findPairs.cuh:615-764) for a caller that owns its data. */
int fasted_self_join(const uint16_t* points, long long n, int d, double epsilon, FastedPair* out,
                     unsigned long long cap, unsigned long long* found, unsigned long long* stored);

/* The same join for a dataset that does not fit the device (or should not occupy it): the host-resident
 * points are streamed through the device in blocks of `block_rows` points (rounded up to a multiple of
 * 256).  Device memory used: three blocks, 4 bytes per point of the whole dataset (each point's squared norm
 * enters the join through one float, formed when its block is first uploaded), and a pair buffer of
 * min(cap, block_rows*256) records (about three times that while sorting).  Blocks that a later join still
 * needs stay on the device: with B blocks about B*(B-2)+2 block uploads instead of B*B.  Output as fasted_self_join: row-major, *found counts every pair,
 * at most `cap` are written; in addition the pairs of one block of query points beyond block_rows*256 are
 * counted but not written.  The reference has no such path: its dataset, twice, and N*256 pair records
 * must fit the device (source/findPairs.cuh:568-600,644-647); "batching" is named as future work in its
 * paper. */
int fasted_self_join_blocked(const uint16_t* points, long long n, int d, double epsilon, long long block_rows,
                             FastedPair* out, unsigned long long cap, unsigned long long* found,
                             unsigned long long* stored);

/* Everything already in device memory (HBM-resident dataset, caller-owned pair buffer).
 *   d_points   N rows of FP16, row stride `ld` halves (ld % 8 == 0, ld >= D rounded up to
 *              64; the columns D..roundup(D,64) of every row must be readable zeros, or
 *              D % 64 == 0)
 *   d_sums     N floats of workspace/result for the squared norms (may be NULL: library
 *              workspace is used)
 *   d_pairs    room for `cap` pairs
 *   stream     hipStream_t (NULL = default stream)
 * The call waits for the join before returning and fills *stats: it synchronises the stream, except that a join
 * of at most 512 tiles of 256 x 256 returns as soon as the join kernel's last workgroup has reported the pair
 * count to the host (a few microseconds before the stream itself reports idle, a fifth of such a call).  Every
 * pair record and squared norm is in device memory by then, for any stream, copy or kernel that reads them next;
 * the stream may still answer hipStreamQuery with hipErrorNotReady for a moment.  With FASTED_SORT_PAIRS the sort's
 * device buffers (a second key buffer and the radix sort's storage, about twice the bytes of the stored
 * pairs) are allocated by the library and kept for the next sort; so are the counters and, without d_sums,
 * the squared norms.  releaseResources() frees all of it.  Replaces the
 * kernel launches of source/findPairs.cuh:632-687 (ComputeSquaredSums x2,
 * initOnDemandRasterizer, FindPairsKernel) and the sort of :703-704. */
int fasted_self_join_device(const void* d_points, long long n, int d, long long ld, double epsilon, float* d_sums,
                            FastedPair* d_pairs, unsigned long long cap, unsigned flags, void* stream,
                            FastedJoinStats* stats);

/* fasted_self_join_device for callers that cannot allocate device memory (tight serving loops, harnesses that
 * forbid hipMalloc, programs that must not disturb a memory pool or a graph they captured elsewhere).  No
 * counterpart in the reference.  Like fasted_self_join_device it synchronises the stream before it returns
 * (it times itself with events and reads the pair count back), so the call itself cannot be recorded into a
 * HIP graph capture.  The queue
 * heads, the pair counter, the squared norms and the per-point accumulator start values live in a device
 * array that is part of the library image (4 KiB + 32 MiB per GPU, held until the process ends) instead of
 * allocated workspace; the call makes no
 * hipMalloc / hipFree and calls no allocating library routine.  Limits, each refused with an error:
 * n <= 4 194 304 points; FASTED_SORT_PAIRS (the sort needs device buffers; the pairs come back in
 * arbitrary order) and FASTED_SKIP_SUMS are not accepted.  Every call on one GPU shares that GPU's array:
 * calls that overlap on one GPU race.  Same results as fasted_self_join_device otherwise; the first call on
 * a device looks up the array's address and creates three timing events. */
int fasted_self_join_device_noalloc(const void* d_points, long long n, int d, long long ld, double epsilon,
                                    FastedPair* d_pairs, unsigned long long cap, unsigned flags, void* stream,
                                    FastedJoinStats* stats);

/* Join of two different sets: every pair (q, c), q indexing the queries and c the candidates, with
 * dist <= epsilon; no pair is forced (there are no self pairs).  Same buffer rules per set as
 * fasted_self_join_device.  The reference's device parameters already carry distinct query and
 * candidate pointers (source/findPairs.cuh:90-100) although its host code always passes one set twice
 * (source/findPairs.cuh:619); joining a dataset block by block through this entry is how a dataset
 * larger than the device memory would be handled. */
int fasted_join_device(const void* d_queries, long long n_queries, long long ld_queries, const void* d_candidates,
                       long long n_candidates, long long ld_candidates, int d, double epsilon, float* d_sums_queries,
                       float* d_sums_candidates, FastedPair* d_pairs, unsigned long long cap, unsigned flags,
                       void* stream, FastedJoinStats* stats);

/* Euclidean distance of each of `count` listed pairs (QueryPoint indexes the queries, CandidatePoint the
 * candidates; pass the same set twice for the output of a self-join): d_distances[i] in FP32, formed as
 * the sum of squared differences, NaN for a pair that names a point outside its set.  The reference never
 * reports distances, but its neighbour-table script reads an optional third column "q, c, dist"
 * (results/scripts/neighbor_tables.py:102-115); this fills it. */
int fasted_pair_distances_device(const void* d_queries, long long n_queries, long long ld_queries,
                                 const void* d_candidates, long long n_candidates, long long ld_candidates, int d,
                                 const FastedPair* d_pairs, unsigned long long count, float* d_distances, void* stream);

/* Checks the one precondition of the device entries that they cannot see for themselves: with D % 64 != 0 the
 * columns D .. roundup(D,64)-1 of every row must be zeros (the kernels read whole 64-wide slabs unmasked, as the
 * reference reads its zero padding, source/DataLoader/PointListBuilder.hpp:149-179).  *bad_rows = number of rows
 * that hold anything else there (0 = fine; always 0 when D % 64 == 0).  No counterpart in the reference, whose
 * only data path pads on the host. */
int fasted_check_padding_device(const void* d_points, long long n, int d, long long ld, unsigned long long* bad_rows,
                                void* stream);

/* Squared norms only: sums[i] = sum_k x_ik^2 in FP32.  Replaces
 * SumSqd::ComputeSquaredSums (source/sumSquared.cuh:84-118). */
int fasted_sum_squared_device(const void* d_points, long long n, int d, long long ld, float* d_sums, void* stream);

/* Tile order of the work queues: writes the (row, col) origin, in points, of the 256x256 tile
 * that queue index `idx` stands for in an n-point problem.  idx enumerates the eight per-XCD
 * queues round-robin (queue idx % 8, position idx / 8).  Returns 0 past the end, 1 for a real
 * tile, 2 for a padding tile of the last raster squares (the kernel skips those).  Host-side
 * mirror of the device rasterizer, the counterpart of Raster::OnDemandRasterizer::nextChunk
 * (source/rasterizer/onDemandRasterizer.cuh:78-108). */
int fasted_raster_coord(unsigned long long idx, long long n, int* row, int* col);
unsigned long long fasted_raster_count(long long n);
/* The same for a FASTED_SYMMETRIC join: only the super-squares (32 x 8 tiles) that reach the diagonal or
 * lie above it are enumerated (row by row), and tiles below the diagonal inside those squares
 * return 2 like padding tiles.  No counterpart in the reference, which always walks the full grid
 * (source/rasterizer/onDemandRasterizer.cuh:50-71). */
int fasted_raster_coord_symmetric(unsigned long long idx, long long n, int* row, int* col);
unsigned long long fasted_raster_count_symmetric(long long n);

/* LDS placement of the kernel's operand tiles: the 16-byte chunk `chunk` (0..7) of row `row` of a
 * 64-wide k-slab is stored at the returned slot (0..7) of that row's 128 bytes.  Host mirror of the
 * device swizzle, the counterpart of SimSearch::SwizzleAddress (source/findPairs.cuh:161-166); exported
 * so that its bank-conflict freedom can be checked without a GPU. */
int fasted_lds_chunk_slot(int row, int chunk);

/* Build the resident host dataset only (no GPU work): what runFromExponentialDataset /
 * runFromFile do before the join (source/main.cu:205-208), so that reRun() can follow.
 * Counterparts of ExponentialPointGenerator + PointListBuilder::build
 * (source/DataLoader/ExponentialPointGenerator.hpp:35-57, PointListBuilder.hpp:132-192) and
 * FilePointGenerator (source/DataLoader/FilePointGenerator.hpp:33-56). */
int fasted_load_exponential_dataset(int size, int dimensionality, double lambda, double max);
int fasted_load_file(const char* filename);

/* Count-only join on the resident dataset (no pair buffer, no sort, no download): *pairsFound as
 * reRun() would report it, *kernelSeconds = squared norms + join kernel.  The probe an epsilon
 * search needs; the reference pays a full reRun for it (results/scripts/experiment/
 * experiments.py:153-281 call find_pairs once per probe).  The probe computes only the tiles on and above the
 * diagonal and counts their off-diagonal hits twice (the test is bitwise the same for (q, c) and (c, q)): the same
 * count as the full join in about half its time. */
int fasted_count_pairs(double epsilon, unsigned long long* pairsFound, double* kernelSeconds);

/* Epsilon for a target selectivity (mean neighbours per point, self pairs excluded) on the resident
 * dataset: the bound-then-bisect search of the reference's find_epsilon_binary
 * (results/scripts/experiment/experiments.py:153-281: double from `initialEpsilon` (0 -> 2) until
 * the target is reached, then half steps until within 1 %), with count-only probes.  Fails instead
 * of looping forever when the selectivity cannot come within 1 % of the target. */
int fasted_find_epsilon(double targetSelectivity, double initialEpsilon, double* epsilon, double* selectivity,
                        int* probes);

/* Epsilon for a target selectivity by volume scaling, the reference's find_epsilon_volumetric with
 * adjust_epsilon_volume (results/scripts/experiment/experiments.py:100-150,284-323): each count-only probe with
 * selectivity s at epsilon e predicts e * (target / s)^(1/D), an empty probe doubles epsilon, the search ends
 * within 10 % of the target.  `initialEpsilon` must be positive (the reference's default is 0.1).  The reference's
 * loop probes the initial epsilon again instead of the adjusted one (experiments.py:314); the adjusted one is
 * probed here.  Fails after 200 probes. */
int fasted_find_epsilon_volumetric(double targetSelectivity, double initialEpsilon, double* epsilon, double* selectivity,
                                   int* probes);

/* The same probe and the same search on an evenly spaced sample of `sample_rows` query points against all
 * points (sample_rows/N of the work per probe): *pairsFound - *sampledRows estimates sampledRows x
 * selectivity.  fasted_find_epsilon_sampled runs the search of fasted_find_epsilon on sampled probes and
 * ends with one full count, so *selectivity is the dataset's; it can miss the 1 % window by the sampling
 * error (about 1/sqrt(sample_rows x selectivity)).  The reference pays a full run per probe
 * (results/scripts/experiment/experiments.py:228-281 via find_pairs). */
int fasted_count_pairs_sampled(double epsilon, int sample_rows, unsigned long long* pairsFound, int* sampledRows,
                               double* kernelSeconds);
int fasted_find_epsilon_sampled(double targetSelectivity, double initialEpsilon, int sample_rows, double* epsilon,
                                double* selectivity, int* probes);

/* Resident dataset: padded FP16 bit patterns (host copy) and its name
 * (PointGenerator::getName, source/DataLoader/PointGenerator.hpp:27-30). */
const uint16_t* fasted_resident_points(int* n, int* d, int* n_pad, int* d_pad);
const char* fasted_resident_name(void);

/* Where `savePairs` writes "<name>_<epsilon>.pairs" (default: $FASTED_PAIRS_DIR or ".").
 * The reference hard-codes a cluster path at source/main.cu:214-215. */
void fasted_set_output_dir(const char* dir);

/* With a non-zero argument (or $FASTED_PAIRS_DISTANCES set) `savePairs` writes "q, c, dist" lines, the
 * three-column form results/scripts/neighbor_tables.py:102-115 accepts; default "q, c" as
 * source/pair.cuh:51-54. */
void fasted_set_save_distances(int enabled);

/* The reference copies the whole pair list to the host after every run, saved or not
 * (source/findPairs.cuh:711-713: 16 GB per reRun at 2M x 384 with 1000 neighbours).  With a zero argument (or
 * $FASTED_DOWNLOAD_PAIRS=0) a run that does not save leaves the pairs on the device; Results is unchanged.
 * fasted_last_pairs_device: the sorted pairs of the last runFrom... / reRun in device memory (*stored of them),
 * owned by the library, valid until the next run or releaseResources(). */
void fasted_set_download_pairs(int enabled);
const FastedPair* fasted_last_pairs_device(unsigned long long* stored);

const char* fasted_last_error(void);
/* Name and version of the library.  A measurement build of the join kernel (parts of it compiled out, results
 * wrong by construction) carries the words "ABLATION BUILD" and what it leaves out in this string. */
const char* fasted_version(void);

#ifdef __cplusplus
}
#endif
#endif /* FASTED_H */
