// fasted_api.cpp -- host driver and C ABI of libfasted.so (declarations: include/fasted.h).
//
// Host orchestration of one join, the counterpart of SimSearch::FindPairs
// (source/findPairs.cuh:615-764): upload once, time squared norms and the join kernel with
// device events, sort the stored pairs row-major, hand the pairs back (or write the
// ".pairs" text file), report Results.  The resident dataset lives in process globals so
// that reRun() can change epsilon without touching the data (source/main.cu:33,198-248).
#include <hip/hip_runtime.h>

#include <algorithm>
#include <atomic>
#include <chrono>
#include <cmath>
#include <climits>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <fstream>
#include <iostream>
#include <memory>
#include <string>
#include <thread>
#include <vector>

#include "../../include/fasted.h"
#include "join_kernels.h"
#include "point_table.hpp"

static_assert(sizeof(mmaShape) == 12, "mmaShape layout is part of the ABI");
static_assert(sizeof(Results) == 56, "Results layout is part of the ABI");
static_assert(offsetof(Results, pairsFound) == 16 && offsetof(Results, inputProblemShape) == 32 &&
                  offsetof(Results, paddedProblemShape) == 44,
              "Results layout is part of the ABI");
static_assert(sizeof(FastedPair) == 8, "pair record is 8 bytes");

namespace {

std::string g_error;
std::string g_outDir;

struct HipFailure : std::runtime_error {
    using std::runtime_error::runtime_error;
};

void hip_check(hipError_t e, const char* what) {
    if (e != hipSuccess) throw HipFailure(std::string(what) + ": " + hipGetErrorString(e));
}
#define HIP_CHECK(expr) hip_check((expr), #expr)

int round_up(long long v, int m) { return (int)(((v + m - 1) / m) * m); }

bool quiet() {
    static const bool q = [] {
        const char* v = std::getenv("FASTED_QUIET");
        return v && *v && *v != '0';
    }();
    return q;
}

// Small device workspace that survives between calls: counters, a squared-norm buffer and the buffer of
// per-point accumulator start values (eps^2/4 - s/2) that the join kernel reads.
struct Workspace {
    unsigned long long* counters = nullptr;
    float* sums = nullptr;
    float* halves = nullptr;
    size_t cap = 0;
    // kept between calls, so that a small join does not pay for them every time: the three timing events and a
    // pinned word the pair counter is copied into behind the join kernel (one wait for kernels and count)
    hipEvent_t ev[3] = {nullptr, nullptr, nullptr};
    unsigned long long* hostCount = nullptr;
    unsigned long long* hostCountDev = nullptr;  // the same words as the device addresses them
    double clockRate = 0.0;

    // ticks per millisecond of the clock the kernels read (a constant-rate counter, independent of the shader clock)
    double clockKHz() {
        if (clockRate == 0.0) {
            int dev = 0, khz = 0;
            HIP_CHECK(hipGetDevice(&dev));
            HIP_CHECK(hipDeviceGetAttribute(&khz, hipDeviceAttributeWallClockRate, dev));
            clockRate = khz > 0 ? (double)khz : 100000.0;
        }
        return clockRate;
    }

    void ensure(size_t n) {
        if (!hostCount) {
            // coherent whatever the environment says: the host watches these words while the kernel still runs
            HIP_CHECK(hipHostMalloc(reinterpret_cast<void**>(&hostCount), 64, hipHostMallocCoherent));
            HIP_CHECK(hipHostGetDevicePointer(reinterpret_cast<void**>(&hostCountDev), hostCount, 0));
        }
        if (!counters) {
            // all zero (the non-finite flag is compared with join numbers, which start at 1), except for the word
            // that tells the join kernel where to report the pair count and its clock readings
            const size_t bytes = fasted::counter_words() * sizeof(unsigned long long);
            HIP_CHECK(hipMalloc(&counters, bytes));
            HIP_CHECK(hipMemset(counters, 0, bytes));
            HIP_CHECK(hipMemcpy(counters + fasted::host_words_slot(), &hostCountDev, sizeof hostCountDev, hipMemcpyHostToDevice));
        }
        for (auto& e : ev)
            if (!e) HIP_CHECK(hipEventCreate(&e));
        if (n > cap) {
            if (sums) HIP_CHECK(hipFree(sums));
            if (halves) HIP_CHECK(hipFree(halves));
            sums = halves = nullptr;
            cap = 0;
            HIP_CHECK(hipMalloc(&sums, n * sizeof(float)));
            HIP_CHECK(hipMalloc(&halves, n * sizeof(float)));
            cap = n;
        }
    }
    void release() {
        if (counters) (void)hipFree(counters);
        if (sums) (void)hipFree(sums);
        if (halves) (void)hipFree(halves);
        if (hostCount) (void)hipHostFree(hostCount);
        for (auto& e : ev) {
            if (e) (void)hipEventDestroy(e);
            e = nullptr;
        }
        counters = nullptr;
        sums = halves = nullptr;
        hostCount = hostCountDev = nullptr;
        cap = 0;
    }
} g_ws;

// ---- the entry point that allocates nothing --------------------------------------------------
// Its kernels use the same two pieces of device memory beyond inputs and outputs as every other join here:
// the counter block (pair counter + queue heads) and the squared norms.  They live in one file-scope device
// array instead of hipMalloc'ed memory; each GPU the library runs on holds its own copy at its own address,
// looked up once per device.  Host code never uses the array's name as an address: only `base`.
constexpr size_t kNoAllocMaxPoints = (size_t)1 << 22;  // 4 Mi points: 2 x 16 MiB (squared norms, accumulator start values)
constexpr size_t kNoAllocCounterBytes = 4096;          // counter block (1152 bytes used)
constexpr size_t kNoAllocScratchBytes = kNoAllocCounterBytes + 2 * kNoAllocMaxPoints * sizeof(float);  // norms, halves
static __device__ __align__(256) unsigned char scratch[kNoAllocScratchBytes];

constexpr int kMaxDevices = 64;
struct DeviceScratch {
    unsigned char* base = nullptr;  // device address of `scratch` on this device
    hipEvent_t ev[3] = {nullptr, nullptr, nullptr};
} g_deviceScratch[kMaxDevices];

// First call on the current device: looks up the device's copy of `scratch` and creates the timing
// events.  Later calls only read the table.
DeviceScratch& device_scratch() {
    int dev = 0;
    HIP_CHECK(hipGetDevice(&dev));
    if (dev < 0 || dev >= kMaxDevices) throw std::invalid_argument("device index out of range");
    DeviceScratch& ds = g_deviceScratch[dev];
    if (!ds.base) {
        void* ptr = nullptr;
        HIP_CHECK(hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch)));
        for (auto& e : ds.ev) HIP_CHECK(hipEventCreate(&e));
        ds.base = static_cast<unsigned char*>(ptr);
    }
    return ds;
}

// Where a join keeps its counters and (unless the caller brings a buffer) its squared norms, and the
// events it times itself with.  Default: the library workspace, events created for the call.
struct JoinScratch {
    unsigned long long* counters;
    float* sums;
    float* halves;
    hipEvent_t* ev;  // three events
};

// Joins are numbered: the norm kernels of a join write its number into the non-finite flag of the counter
// block, the join kernel compares with it, and so the flag never has to be cleared between joins.
unsigned long long g_epoch = 0;

fasted::SortBuffers g_sortWs;  // device buffers of the row-major sort, kept between calls

// Three events around the two timed stages; created for the call, or borrowed from the caller.
struct EventTimer {
    hipEvent_t ev[3] = {nullptr, nullptr, nullptr};
    bool owned;
    explicit EventTimer(hipEvent_t* borrowed = nullptr) : owned(borrowed == nullptr) {
        for (int i = 0; i < 3; ++i) {
            if (borrowed)
                ev[i] = borrowed[i];
            else
                HIP_CHECK(hipEventCreate(&ev[i]));
        }
    }
    EventTimer(const EventTimer&) = delete;
    EventTimer& operator=(const EventTimer&) = delete;
    ~EventTimer() {
        if (!owned) return;
        for (auto& e : ev)
            if (e) (void)hipEventDestroy(e);
    }
    float ms(int a, int b) {
        float t = 0.f;
        HIP_CHECK(hipEventElapsedTime(&t, ev[a], ev[b]));
        return t;
    }
};

// A NaN epsilon compares false with every distance in the reference (source/warpMma.cuh:257: no pairs at all);
// here the accumulator start values are formed from epsilon, so it is refused before any launch.
void validate_epsilon(double epsilon) {
    if (std::isnan(epsilon)) throw std::invalid_argument("epsilon is NaN");
}

void validate_shape(long long n, int d, long long ld) {
    if (n < 1) throw std::invalid_argument("number of points must be at least 1");
    if (n > (long long)INT_MAX - 2 * fasted::kTile) throw std::invalid_argument("number of points exceeds int range");
    if (d < 1) throw std::invalid_argument("dimensionality must be at least 1");
    const long long dPad = round_up(d, fasted::kSlabK);
    if (ld % 8 != 0) throw std::invalid_argument("row stride must be a multiple of 8 halves (16 bytes)");
    if (ld < dPad) throw std::invalid_argument("row stride must cover the dimensionality rounded up to 64");
    // the kernel addresses a tile's rows with 32-bit byte offsets from the tile's first row
    if (ld * 2 * fasted::kTile >= (1ll << 32)) throw std::invalid_argument("row stride too large");
}

// One side of a join: `n` FP16 rows of `d` dimensions, row stride `ld` halves.
struct PointSet {
    const void* ptr;
    long long n;
    long long ld;
    float* sums;  // caller's buffer for the squared norms, or null
};

// The timed region of the reference (source/findPairs.cuh:625-697): squared norms, then
// queue/pair-counter reset and the join kernel; then counters come back and the stored pairs
// are sorted outside the TFLOPS window.  `c.ptr == q.ptr` with selfJoin computes the norms once.
void join_on_device(PointSet q, PointSet c, bool selfJoin, int d, double epsilon, void* dPairs,
                    unsigned long long cap, unsigned flags, hipStream_t stream, FastedJoinStats* stats,
                    const JoinScratch* fixed = nullptr, bool sortMayFail = false, int forcedStride = 0) {
    validate_epsilon(epsilon);
    validate_shape(q.n, d, q.ld);
    validate_shape(c.n, d, c.ld);
    if (cap > 0 && !dPairs) throw std::invalid_argument("pair buffer is null");
    const int dPad = round_up(d, fasted::kSlabK);
    if (!fixed) g_ws.ensure((size_t)q.n + (selfJoin ? 0 : (size_t)c.n));
    EventTimer t(fixed ? fixed->ev : g_ws.ev);
    unsigned long long* counters = nullptr;
    float* wsSums = nullptr;
    float* wsHalves = nullptr;
    if (fixed) {
        counters = fixed->counters;
        wsSums = fixed->sums;
        wsHalves = fixed->halves;
    } else {
        counters = g_ws.counters;
        wsSums = g_ws.sums;
        wsHalves = g_ws.halves;
    }
    float* sumsQ = q.sums ? q.sums : wsSums;
    float* sumsC = selfJoin ? sumsQ : (c.sums ? c.sums : wsSums + q.n);
    float* halfQ = wsHalves;
    float* halfC = selfJoin ? halfQ : wsHalves + q.n;
    if ((flags & FASTED_SKIP_SUMS) && (!q.sums || (!selfJoin && !c.sums)))
        throw std::invalid_argument("FASTED_SKIP_SUMS needs the squared-norm buffers");
    const float eps2 = static_cast<float>(epsilon * epsilon);  // product in double, then narrowed (findPairs.cuh:678)

    // squared norms and, from them, each point's accumulator start value eps^2/4 - s/2
    // (the first of these launches also clears the pair counter and the queue heads)
    const unsigned long long epoch = ++g_epoch;
    // Timing.  Three event records cost a call about 10 us, a third of a join of a few thousand points, so a
    // join of at most two tiles per compute unit is timed by the kernels themselves instead: the first norm
    // kernel and the join kernel note the device's constant-rate clock when they start, and the join kernel's
    // last workgroup when it hands the pair count to the host.  Larger joins, and the entry
    // that owns no pinned memory, are timed with events on the stream as the reference is
    // (source/findPairs.cuh:625-639,695-697,728-736).
    const bool stamped = !fixed && !(flags & FASTED_EVENT_TIMING) && fasted::tile_count(q.n, c.n) <= 512;
    const bool events = !stamped && stats != nullptr;
    if (events) HIP_CHECK(hipEventRecord(t.ev[0], stream));
    if (!(flags & FASTED_SKIP_SUMS)) {
        HIP_CHECK(fasted::launch_sum_squared(q.ptr, q.ld, (int)q.n, dPad, sumsQ, halfQ, eps2, counters, stream, epoch, true));
        if (!selfJoin)
            HIP_CHECK(fasted::launch_sum_squared(c.ptr, c.ld, (int)c.n, dPad, sumsC, halfC, eps2, counters, stream, epoch));
    } else {
        HIP_CHECK(fasted::launch_halves(sumsQ, (int)q.n, eps2, halfQ, counters, stream, epoch, true));
        if (!selfJoin) HIP_CHECK(fasted::launch_halves(sumsC, (int)c.n, eps2, halfC, counters, stream, epoch));
    }
    if (events) HIP_CHECK(hipEventRecord(t.ev[1], stream));

    fasted::JoinLaunch jl;
    jl.queries = q.ptr;
    jl.candidates = c.ptr;
    jl.ldQ = q.ld;
    jl.ldC = c.ld;
    jl.nQ = (int)q.n;
    jl.nC = (int)c.n;
    jl.selfJoin = selfJoin;
    jl.forcedStride = forcedStride;
    jl.symmetric = selfJoin && (flags & FASTED_SYMMETRIC);
    jl.dPad = dPad;
    jl.halfQ = halfQ;
    jl.halfC = halfC;
    jl.counters = counters;
    jl.epoch = epoch;
    jl.pairs = dPairs;
    jl.cap = cap;
    jl.epilogue = !(flags & FASTED_NO_EPILOGUE);
    if (!fixed) static_cast<volatile unsigned long long*>(g_ws.hostCount)[3] = 0;  // the kernel's report turns it non-zero
    HIP_CHECK(fasted::launch_join(jl, stream));
    if (events) HIP_CHECK(hipEventRecord(t.ev[2], stream));
    // c[0] = pairs found; every slot below the capacity received exactly one pair, the rest were
    // counted only (source/pair.cuh:123-133), so stored = min(found, capacity)
    unsigned long long cnt[4] = {0, 0, 0, 0};
    if (fixed) {
        HIP_CHECK(hipStreamSynchronize(stream));
        HIP_CHECK(hipMemcpy(cnt, counters, sizeof(unsigned long long), hipMemcpyDeviceToHost));
    } else {
        // The join kernel's last workgroup writes the count (and the kernels' clock readings) into pinned memory:
        // no launch or copy command behind the join.  A small join is over when that report is there -- every
        // workgroup has released its stores at system scope before it was counted -- and the few microseconds
        // until the stream itself reports idle, a fifth of such a call, are not waited for.  (A kernel that never
        // reports, because it failed, falls through to the stream's own wait, which returns the error.)
        volatile unsigned long long* const w = g_ws.hostCount;
        bool reported = false;
        if (stamped) {
            const auto t0 = std::chrono::steady_clock::now();
            for (unsigned spins = 1; !(reported = w[3] != 0); ++spins)
                if ((spins & 1023u) == 0 && std::chrono::steady_clock::now() - t0 > std::chrono::milliseconds(2)) break;
            std::atomic_thread_fence(std::memory_order_acquire);
        }
        if (!reported) HIP_CHECK(hipStreamSynchronize(stream));
        if (w[3] != 0) {
            cnt[0] = w[0];
        } else {
            // the stream has drained without a report (a counter block that names no host words): the count is
            // still where the kernel keeps it
            HIP_CHECK(hipMemcpy(cnt, counters, sizeof(unsigned long long), hipMemcpyDeviceToHost));
        }
    }
    cnt[1] = (jl.epilogue && cnt[0] > cap) ? cap : cnt[0];
    cnt[2] = fasted::tile_count(q.n, c.n);
    if (jl.symmetric) {
        const unsigned long long side = ((unsigned long long)q.n + fasted::kTile - 1) / fasted::kTile;
        cnt[2] = side * (side + 1) / 2;
    }
    float sortMs = 0.f;
    if ((flags & FASTED_SORT_PAIRS) && cnt[1] > 1) {
        const auto w0 = std::chrono::steady_clock::now();
        const hipError_t e = fasted::sort_pairs_row_major(dPairs, cnt[1], stream, &g_sortWs, q.n, c.n);
        if (e != hipSuccess) {
            (void)hipGetLastError();
            if (!sortMayFail) hip_check(e, "row-major sort of the pairs");
            std::cout << "Failed to sort pairs: " << hipGetErrorString(e) << std::endl;
        }
        sortMs = std::chrono::duration<float, std::milli>(std::chrono::steady_clock::now() - w0).count();
    }
    if (stats) {
        if (stamped) {
            const volatile unsigned long long* const w = g_ws.hostCount;  // [1] norms start, [2] join start, [3] join over
            const bool reportedTimes = w[3] != 0;  // (no report, no clock readings: the times stay 0)
            stats->sumSquaredMs = reportedTimes ? (float)((double)(w[2] - w[1]) / g_ws.clockKHz()) : 0.f;
            stats->joinMs = reportedTimes ? (float)((double)(w[3] - w[2]) / g_ws.clockKHz()) : 0.f;
        } else {
            stats->sumSquaredMs = t.ms(0, 1);
            stats->joinMs = t.ms(1, 2);
        }
        stats->sortMs = sortMs;
        stats->paddedN = round_up(q.n, fasted::kTile);
        stats->paddedD = dPad;
        stats->tiles = cnt[2];
        stats->pairsFound = cnt[0];
        stats->pairsStored = cnt[1];
    }
}

// Host rows of `rowBytes` bytes -> device rows of `pitch` bytes (pitch >= rowBytes; the bytes past rowBytes
// are written as zeros).  Rows that are already contiguous go up in one copy; otherwise they are packed
// into two pinned staging buffers in turn, so that packing one chunk overlaps the transfer of the other
// (a strided 2-D copy from pageable memory moves row by row, at about 1 GB/s).
void upload_rows(void* dst, size_t pitch, const void* src, size_t rowBytes, size_t rows, hipStream_t stream) {
    if (rows == 0) return;
    if (rowBytes == pitch) {
        HIP_CHECK(hipMemcpyAsync(dst, src, rows * pitch, hipMemcpyHostToDevice, stream));
        return;
    }
    const size_t chunkRows = std::max<size_t>(1, std::min(rows, ((size_t)32 << 20) / pitch));
    struct Staging {
        void* buf[2] = {nullptr, nullptr};
        hipEvent_t done[2] = {nullptr, nullptr};
        ~Staging() {
            for (int i = 0; i < 2; ++i) {
                if (buf[i]) (void)hipHostFree(buf[i]);
                if (done[i]) (void)hipEventDestroy(done[i]);
            }
        }
    } st;
    for (int i = 0; i < 2; ++i) {
        HIP_CHECK(hipHostMalloc(&st.buf[i], chunkRows * pitch, hipHostMallocDefault));
        HIP_CHECK(hipEventCreateWithFlags(&st.done[i], hipEventDisableTiming));
    }
    int slot = 0;
    for (size_t r0 = 0; r0 < rows; r0 += chunkRows, slot ^= 1) {
        const size_t count = std::min(chunkRows, rows - r0);
        HIP_CHECK(hipEventSynchronize(st.done[slot]));  // the transfer that last read this buffer is over
        char* out = static_cast<char*>(st.buf[slot]);
        const char* in = static_cast<const char*>(src) + r0 * rowBytes;
        for (size_t r = 0; r < count; ++r) {
            std::memcpy(out + r * pitch, in + r * rowBytes, rowBytes);
            std::memset(out + r * pitch + rowBytes, 0, pitch - rowBytes);
        }
        HIP_CHECK(hipMemcpyAsync(static_cast<char*>(dst) + r0 * pitch, out, count * pitch, hipMemcpyHostToDevice, stream));
        HIP_CHECK(hipEventRecord(st.done[slot], stream));
    }
    HIP_CHECK(hipStreamSynchronize(stream));  // the staging buffers go away with this frame
}

// The largest pair count <= `want` whose records fit the free device memory together with what the sort of
// that many records needs beside them (a second key buffer and the radix sort's storage), as Pairs::init
// shrinks the reference's buffer to the free memory (source/pair.cuh:69-85).
unsigned long long fit_pairs_with_sort(unsigned long long want) {
    size_t freeB = 0, totalB = 0;
    HIP_CHECK(hipMemGetInfo(&freeB, &totalB));
    const size_t usable = freeB - freeB / 16;  // leave some room for the runtime
    unsigned long long maxPairs = want;
    for (int round = 0; round < 4; ++round) {
        const size_t need = (size_t)maxPairs * sizeof(FastedPair) + fasted::sort_scratch_bytes(maxPairs);
        if (need <= usable) break;
        maxPairs = (unsigned long long)((double)maxPairs * (double)usable / (double)need * 0.98);
    }
    return maxPairs;
}

// Self-join of a host-resident dataset that is streamed through the device in blocks of `blockRows`
// points: for every query block (held on the device) every candidate block is uploaded in turn, on a
// copy stream, while the join of the block before it runs.  The pairs of one query block are appended
// to one device buffer across the candidate blocks, get their global indices, are sorted row-major and
// go back to the host; query blocks are processed in order, so the whole output is row-major.
struct DeviceBuffers {
    std::vector<void*> owned;
    hipStream_t compute = nullptr, copy = nullptr;
    ~DeviceBuffers() {
        for (void* p : owned) (void)hipFree(p);
        if (compute) (void)hipStreamDestroy(compute);
        if (copy) (void)hipStreamDestroy(copy);
    }
    void* alloc(size_t bytes) {
        void* p = nullptr;
        HIP_CHECK(hipMalloc(&p, bytes ? bytes : 1));
        owned.push_back(p);
        return p;
    }
};

void self_join_blocked(const uint16_t* points, long long n, int d, double epsilon, long long blockRows, FastedPair* out,
                       unsigned long long cap, unsigned long long* found, unsigned long long* stored) {
    if (!points) throw std::invalid_argument("points pointer is null");
    if (cap > 0 && !out) throw std::invalid_argument("output buffer is null");
    if (blockRows < 1) throw std::invalid_argument("block size must be at least 1 point");
    validate_epsilon(epsilon);
    const int dPad = round_up(d, fasted::kSlabK);
    validate_shape(n, d, dPad);
    // blocks start on tile boundaries, so a block join sees the same tiles as the whole join would
    const long long rows = std::min<long long>(round_up(blockRows, fasted::kTile), round_up(n, fasted::kTile));
    const long long blocks = (n + rows - 1) / rows;
    const size_t pitch = (size_t)dPad * 2, blockBytes = (size_t)rows * pitch;

    // Three block buffers.  One holds the query block; the candidate blocks pass through the other two, and
    // the order of the candidates is chosen so that nothing is uploaded twice in a row: the last candidate of
    // query block i is block i + 1, whose buffer then becomes the query buffer, and the old query block is
    // still resident as the first off-diagonal candidate of block i + 1.  Uploads run on a copy stream while
    // joins run on the compute stream; events, not the host, order a buffer's upload behind the last join
    // that read it and a join behind the upload of its candidates.
    DeviceBuffers dev;
    HIP_CHECK(hipStreamCreateWithFlags(&dev.compute, hipStreamNonBlocking));
    HIP_CHECK(hipStreamCreateWithFlags(&dev.copy, hipStreamNonBlocking));
    struct BlockBuffer {
        void* rows = nullptr;
        long long block = -1;           // which block of the dataset it holds
        hipEvent_t uploaded = nullptr;  // recorded on the copy stream behind the upload
        hipEvent_t released = nullptr;  // recorded on the compute stream behind the last join that read it
    } buf[3];
    struct Events {
        BlockBuffer* b;
        ~Events() {
            for (int i = 0; i < 3; ++i) {
                if (b[i].uploaded) (void)hipEventDestroy(b[i].uploaded);
                if (b[i].released) (void)hipEventDestroy(b[i].released);
            }
        }
    } eventGuard{buf};
    for (auto& b : buf) {
        b.rows = dev.alloc(blockBytes);
        HIP_CHECK(hipEventCreateWithFlags(&b.uploaded, hipEventDisableTiming));
        HIP_CHECK(hipEventCreateWithFlags(&b.released, hipEventDisableTiming));
    }
    // accumulator start values eps^2/4 - s/2 of every point of the dataset: formed when a block is uploaded
    // for the first time (all of them during the first query block), read again for every later query block
    float* const halves = static_cast<float*>(dev.alloc((size_t)blocks * rows * sizeof(float)));
    std::vector<char> haveHalves((size_t)blocks, 0);
    // where the pairs of the joins of one query block begin: mark[k] = pair counter before its k-th join
    unsigned long long* const marks =
        static_cast<unsigned long long*>(dev.alloc((size_t)(blocks + 1) * sizeof(unsigned long long)));
    // pair buffer of one query block: rows*256 records as the reference sizes its buffer per point
    // (source/findPairs.cuh:644-647), shrunk to what is free together with the sort's own buffers
    unsigned long long devCap = std::min<unsigned long long>((unsigned long long)rows * 256ull, cap);
    devCap = fit_pairs_with_sort(devCap);
    void* dPairs = dev.alloc((size_t)devCap * sizeof(FastedPair));
    g_ws.ensure(1);

    auto block_rows = [&](long long b) { return std::min<long long>(rows, n - b * rows); };
    const float eps2 = static_cast<float>(epsilon * epsilon);
    const unsigned long long epoch = ++g_epoch;  // one number for all block joins of this call
    // Block b into buffer `into`, on the copy stream, once the joins that still read the buffer are through.
    auto upload = [&](BlockBuffer& into, long long b) {
        HIP_CHECK(hipStreamWaitEvent(dev.copy, into.released, 0));
        upload_rows(into.rows, pitch, points + (size_t)b * rows * d, (size_t)d * 2, (size_t)block_rows(b), dev.copy);
        HIP_CHECK(hipEventRecord(into.uploaded, dev.copy));
        into.block = b;
    };
    // The compute stream waits for the upload of a buffer and forms the block's start values if they are new.
    auto make_ready = [&](BlockBuffer& b) {
        HIP_CHECK(hipStreamWaitEvent(dev.compute, b.uploaded, 0));
        if (!haveHalves[(size_t)b.block]) {
            HIP_CHECK(fasted::launch_sum_squared(b.rows, dPad, (int)block_rows(b.block), dPad, nullptr,
                                                 halves + (size_t)b.block * rows, eps2, g_ws.counters, dev.compute, epoch));
            haveHalves[(size_t)b.block] = 1;
        }
    };

    unsigned long long foundAll = 0, storedAll = 0;
    BlockBuffer* query = &buf[0];
    BlockBuffer* spare[2] = {&buf[1], &buf[2]};
    for (auto& b : buf) HIP_CHECK(hipEventRecord(b.released, dev.compute));
    upload(*query, 0);
    for (long long i = 0; i < blocks; ++i) {
        const int nQ = (int)block_rows(i);
        make_ready(*query);
        HIP_CHECK(fasted::launch_reset_counters(g_ws.counters, false, dev.compute));
        HIP_CHECK(hipMemsetAsync(marks, 0, sizeof(unsigned long long), dev.compute));
        // Candidates in this order: block i itself (the query buffer), then what the two spare buffers still
        // hold from the query block before (block i - 1 in spare[0], some other block in spare[1]), then the
        // rest, block i + 1 last.  Position p >= 1 of the order lives in spare[(p - 1) % 2]: the joins read
        // the two buffers in turn, and a buffer receives position p behind join p - 2, which read it.
        std::vector<long long> order{i};
        const bool keep0 = i > 0 && spare[0]->block == i - 1;
        if (keep0) order.push_back(i - 1);
        const long long held = spare[1]->block;
        const bool keep1 = keep0 && held >= 0 && held != i && held != i - 1 && held != i + 1;
        if (keep1) order.push_back(held);
        for (long long j = 0; j < blocks; ++j)
            if (j != i && j != i + 1 && !(keep0 && j == i - 1) && !(keep1 && j == held)) order.push_back(j);
        if (i + 1 < blocks) order.push_back(i + 1);
        size_t next = 1 + (keep0 ? 1 : 0) + (keep1 ? 1 : 0);  // first position that has to be uploaded
        for (size_t k = 0; k < order.size(); ++k) {
            const long long j = order[k];
            const bool diagonal = (k == 0);
            BlockBuffer& cand = diagonal ? *query : *spare[(k - 1) % 2];
            if (cand.block != j) throw std::logic_error("blocked join: a candidate block is not where it should be");
            if (!diagonal) make_ready(cand);
            fasted::JoinLaunch jl;
            jl.queries = query->rows;
            jl.candidates = cand.rows;
            jl.ldQ = jl.ldC = dPad;
            jl.nQ = nQ;
            jl.nC = (int)block_rows(j);
            jl.selfJoin = diagonal;
            jl.symmetric = false;
            jl.dPad = dPad;
            jl.halfQ = halves + (size_t)i * rows;
            jl.halfC = halves + (size_t)j * rows;
            jl.counters = g_ws.counters;
            jl.epoch = epoch;
            jl.pairs = dPairs;
            jl.cap = devCap;
            jl.epilogue = true;
            HIP_CHECK(fasted::launch_reset_counters(g_ws.counters, /*keepFound=*/true, dev.compute));
            HIP_CHECK(fasted::launch_join(jl, dev.compute));
            // block-local indices -> indices of the whole dataset, for the pairs this join appended
            HIP_CHECK(fasted::launch_offset_appended_pairs(dPairs, marks + k, g_ws.counters, devCap, (int)(i * rows),
                                                           (int)(j * rows), dev.compute));
            if (!diagonal) HIP_CHECK(hipEventRecord(cand.released, dev.compute));
            // With join k queued, the host turns to the upload of candidate k + 1 (if it is not resident): into
            // the buffer join k - 1 read, behind that join, while join k runs.  (An upload from pageable memory
            // holds the host until it is through, so it must not come before the join it overlaps is queued.)
            if (next == k + 1 && next < order.size()) {
                upload(*spare[(next - 1) % 2], order[next]);
                ++next;
            }
        }
        HIP_CHECK(hipEventRecord(query->released, dev.compute));
        HIP_CHECK(hipStreamSynchronize(dev.compute));
        unsigned long long before = 0;
        HIP_CHECK(hipMemcpy(&before, g_ws.counters, sizeof before, hipMemcpyDeviceToHost));
        const unsigned long long kept = std::min(before, devCap);
        if (kept > 1) HIP_CHECK(fasted::sort_pairs_row_major(dPairs, kept, dev.compute, &g_sortWs, n, n));
        HIP_CHECK(hipStreamSynchronize(dev.compute));
        const unsigned long long take = std::min(kept, cap - storedAll);
        if (take)
            HIP_CHECK(hipMemcpy(out + storedAll, dPairs, (size_t)take * sizeof(FastedPair), hipMemcpyDeviceToHost));
        storedAll += take;
        foundAll += before;
        // roles for query block i + 1: its rows are in the buffer read last; the old query block stays resident
        if (i + 1 < blocks) {
            const size_t lastPos = order.size() - 1;
            BlockBuffer* const last = spare[(lastPos - 1) % 2];
            BlockBuffer* const other = spare[lastPos % 2];
            if (last->block != i + 1) throw std::logic_error("blocked join: the next query block is not resident");
            spare[0] = query;
            spare[1] = other;
            query = last;
        }
    }
    if (found) *found = foundAll;
    if (stored) *stored = storedAll;
}

// ---- resident dataset of the reference-compatible entry points -------------------------
struct Resident {
    fasted::PointTable table;
    void* dPoints = nullptr;
    bool uploaded = false;
    void* dSample = nullptr;  // every (n / sampleRows)-th point, for the sampled epsilon search
    int sampleRows = 0;
    void drop_device() {
        if (dPoints) (void)hipFree(dPoints);
        if (dSample) (void)hipFree(dSample);
        dPoints = dSample = nullptr;
        sampleRows = 0;
        uploaded = false;
    }
} g_res;

std::string output_dir() {
    if (!g_outDir.empty()) return g_outDir;
    const char* env = std::getenv("FASTED_PAIRS_DIR");
    return env && *env ? std::string(env) : std::string(".");
}

bool g_saveDistances = false;
bool g_downloadPairs = true;
unsigned long long g_lastStored = 0;  // pairs the last resident run left, sorted, in the device pair buffer

// The reference always copies the pair list to the host, saved or not (source/findPairs.cuh:711-713).  A caller
// that only wants the counts, or goes on working with the pairs on the device, switches that off.
bool download_pairs() {
    if (!g_downloadPairs) return false;
    const char* v = std::getenv("FASTED_DOWNLOAD_PAIRS");
    return !(v && v[0] == '0');
}

bool save_distances() {
    if (g_saveDistances) return true;
    const char* v = std::getenv("FASTED_PAIRS_DISTANCES");
    return v && *v && *v != '0';
}

// Decimal digits of a non-negative int, written backwards from `end`; returns the first character.
char* write_index(char* end, int value) {
    unsigned v = static_cast<unsigned>(value);
    do {
        *--end = static_cast<char>('0' + v % 10u);
        v /= 10u;
    } while (v);
    return end;
}

// "q, c\n" per pair, the format of operator<< in source/pair.cuh:51-54; with distances
// "q, c, dist\n", the three-column form results/scripts/neighbor_tables.py:102-115 also reads.
// Pairs arrive in pieces (the download of the next piece runs while this one is written).  The lines of a
// piece are formatted by several threads, a slice each, into buffers that are then written in order (one
// formatted-print call per pair made large lists take minutes).
class PairsTextFile {
public:
    explicit PairsTextFile(const std::string& path) : path_(path), f_(std::fopen(path.c_str(), "w")) {
        if (!f_) throw std::ios_base::failure("Failed to open output file: " + path);
    }
    PairsTextFile(const PairsTextFile&) = delete;
    PairsTextFile& operator=(const PairsTextFile&) = delete;
    ~PairsTextFile() {
        if (f_) (void)std::fclose(f_);
    }
    // `dist` may be null: two columns
    void append(const FastedPair* pairs, const float* dist, size_t count) {
        const size_t slice = 1u << 20;  // pairs per buffer
        const unsigned threads = std::max(1u, std::min(fasted::host_threads("FASTED_CSV_THREADS"),
                                                       static_cast<unsigned>((count + slice - 1) / slice)));
        text_.resize(std::max<size_t>(text_.size(), threads));
        for (size_t base = 0; base < count && !failed_; base += slice * threads) {
            auto format = [&](unsigned w) {
                const size_t lo = std::min(count, base + w * slice), hi = std::min(count, lo + slice);
                std::string& out = text_[w];
                out.clear();
                out.reserve((hi - lo) * (dist ? 40 : 24));
                char line[64];
                for (size_t i = lo; i < hi; ++i) {
                    char* end = line + sizeof line;
                    *--end = '\n';
                    if (dist) {
                        char number[32];
                        const int len = std::snprintf(number, sizeof number, "%.7g", dist[i]);
                        end -= len;
                        std::memcpy(end, number, static_cast<size_t>(len));
                        *--end = ' ';
                        *--end = ',';
                    }
                    end = write_index(end, pairs[i].CandidatePoint);
                    *--end = ' ';
                    *--end = ',';
                    end = write_index(end, pairs[i].QueryPoint);
                    out.append(end, static_cast<size_t>(line + sizeof line - end));
                }
            };
            std::vector<std::thread> pool;
            for (unsigned w = 1; w < threads; ++w) pool.emplace_back(format, w);
            format(0);
            for (auto& t : pool) t.join();
            for (unsigned w = 0; w < threads && !failed_; ++w)
                if (!text_[w].empty() && std::fwrite(text_[w].data(), 1, text_[w].size(), f_) != text_[w].size())
                    failed_ = true;
        }
    }
    void close() {
        const bool bad = std::fclose(f_) != 0 || failed_;
        f_ = nullptr;
        if (bad) throw std::ios_base::failure("Failed to write output file: " + path_);
    }

private:
    std::string path_;
    std::FILE* f_;
    std::vector<std::string> text_;
    bool failed_ = false;
};

// Device and pinned host memory of the drop-in entry points that outlives a call: the pair buffer, the
// distance column, and two pinned pieces through which the sorted pairs leave the device.  reRun() on a
// resident dataset allocates nothing.
struct PairWorkspace {
    void* dPairs = nullptr;
    unsigned long long capPairs = 0;
    float* dDist = nullptr;
    unsigned long long capDist = 0;
    static constexpr size_t kPiecePairs = (size_t)4 << 20;  // 32 MiB of records per piece
    FastedPair* hPairs[2] = {nullptr, nullptr};
    float* hDist[2] = {nullptr, nullptr};
    hipEvent_t landed[2] = {nullptr, nullptr};
    hipStream_t copy = nullptr;

    void ensure_host() {
        if (copy) return;
        HIP_CHECK(hipStreamCreateWithFlags(&copy, hipStreamNonBlocking));  // default priority
        for (int i = 0; i < 2; ++i) {
            HIP_CHECK(hipHostMalloc(reinterpret_cast<void**>(&hPairs[i]), kPiecePairs * sizeof(FastedPair), hipHostMallocDefault));
            HIP_CHECK(hipHostMalloc(reinterpret_cast<void**>(&hDist[i]), kPiecePairs * sizeof(float), hipHostMallocDefault));
            HIP_CHECK(hipEventCreateWithFlags(&landed[i], hipEventDisableTiming));
        }
    }
    void release() {
        if (dPairs) (void)hipFree(dPairs);
        if (dDist) (void)hipFree(dDist);
        dPairs = nullptr;
        dDist = nullptr;
        capPairs = capDist = 0;
        for (int i = 0; i < 2; ++i) {
            if (hPairs[i]) (void)hipHostFree(hPairs[i]);
            if (hDist[i]) (void)hipHostFree(hDist[i]);
            if (landed[i]) (void)hipEventDestroy(landed[i]);
            hPairs[i] = nullptr;
            hDist[i] = nullptr;
            landed[i] = nullptr;
        }
        if (copy) (void)hipStreamDestroy(copy);
        copy = nullptr;
    }
} g_pairWs;

// Pair buffer of N*256 records (source/findPairs.cuh:644-647), shrunk to what the device can hold together
// with what the sort of a full buffer needs (a second key buffer and the radix sort's storage), as
// Pairs::init shrinks it to the free memory (source/pair.cuh:69-85).  Kept until a larger one is needed.
unsigned long long ensure_pair_buffer(int n) {
    const unsigned long long want = (unsigned long long)n * 256ull;
    if (g_pairWs.dPairs && g_pairWs.capPairs >= want) return want;
    if (g_pairWs.dPairs) {
        HIP_CHECK(hipFree(g_pairWs.dPairs));
        g_pairWs.dPairs = nullptr;
        g_pairWs.capPairs = 0;
    }
    g_sortWs.release();
    const unsigned long long maxPairs = fit_pairs_with_sort(want);
    if (maxPairs < want)
        std::printf("Failed to allocate enough space for %llu pairs. Reducing max number of pairs to %llu\n", want, maxPairs);
    HIP_CHECK(hipMalloc(&g_pairWs.dPairs, (size_t)(maxPairs ? maxPairs : 1) * sizeof(FastedPair)));
    g_pairWs.capPairs = maxPairs;
    return maxPairs;
}

Results find_pairs_resident(double epsilon, bool savePairs, bool skipUpload, const std::string& datasetName) {
    const auto wall0 = std::chrono::steady_clock::now();
    const fasted::PointTable& tb = g_res.table;
    if (tb.empty()) throw std::runtime_error("no dataset is resident: call runFromFile or runFromExponentialDataset first");
    HIP_CHECK(hipSetDevice(0));
    const size_t bytes = tb.bits.size() * sizeof(uint16_t);
    if (!skipUpload || !g_res.uploaded) {
        g_res.drop_device();
        if (!quiet()) std::printf("Allocating %zu bytes for the points (queries and candidates share one copy)\n", bytes);
        HIP_CHECK(hipMalloc(&g_res.dPoints, bytes));
        HIP_CHECK(hipMemcpy(g_res.dPoints, tb.bits.data(), bytes, hipMemcpyHostToDevice));
        g_res.uploaded = true;
    }
    HIP_CHECK(hipDeviceSynchronize());

    g_lastStored = 0;  // the buffer may move or be overwritten from here on
    const unsigned long long maxPairs = std::min(ensure_pair_buffer(tb.n), g_pairWs.capPairs);
    g_pairWs.ensure_host();
    void* const dPairs = g_pairWs.dPairs;

    FastedJoinStats st{};
    const PointSet all{g_res.dPoints, tb.n, tb.dPad, nullptr};
    // a sort that fails (no memory for its buffers) is reported and the pairs leave unsorted, as the
    // reference carries on after "Failed to sort pairs" (source/findPairs.cuh:701-718)
    join_on_device(all, all, true, tb.dPad, epsilon, dPairs, maxPairs, FASTED_SORT_PAIRS, nullptr, &st, nullptr,
                   /*sortMayFail=*/true);
    if (!quiet()) {
        std::printf("Number of pairs found %llu\n", st.pairsFound);
        std::printf("Number of pairs stored %llu\n", st.pairsStored);
    }
    const bool withDistance = savePairs && save_distances() && st.pairsStored > 0;
    if (withDistance) {
        if (g_pairWs.capDist < st.pairsStored) {
            if (g_pairWs.dDist) HIP_CHECK(hipFree(g_pairWs.dDist));
            g_pairWs.dDist = nullptr;
            g_pairWs.capDist = 0;
            HIP_CHECK(hipMalloc(reinterpret_cast<void**>(&g_pairWs.dDist), (size_t)st.pairsStored * sizeof(float)));
            g_pairWs.capDist = st.pairsStored;
        }
        HIP_CHECK(fasted::launch_pair_distances(g_res.dPoints, tb.dPad, tb.n, g_res.dPoints, tb.dPad, tb.n, tb.dPad, dPairs,
                                                st.pairsStored, g_pairWs.dDist, nullptr));
        HIP_CHECK(hipStreamSynchronize(nullptr));
    }

    g_lastStored = st.pairsStored;
    // The pairs leave the device, saved or not (source/findPairs.cuh:705-714; unless the caller has switched the
    // download off and does not save): piece by piece through two pinned buffers, the next piece travelling while
    // the current one is written as text.
    std::unique_ptr<PairsTextFile> file;
    if (savePairs) {
        const std::string path = output_dir() + "/" + datasetName + "_" + std::to_string(epsilon) + ".pairs";
        std::cout << "Output file is: " << path << std::endl;
        file.reset(new PairsTextFile(path));
    }
    const size_t piece = PairWorkspace::kPiecePairs;
    const size_t total = (savePairs || download_pairs()) ? (size_t)st.pairsStored : 0;
    auto fetch = [&](size_t first, int slot) {
        const size_t count = std::min(piece, total - first);
        HIP_CHECK(hipMemcpyAsync(g_pairWs.hPairs[slot], static_cast<const FastedPair*>(dPairs) + first,
                                 count * sizeof(FastedPair), hipMemcpyDeviceToHost, g_pairWs.copy));
        if (withDistance)
            HIP_CHECK(hipMemcpyAsync(g_pairWs.hDist[slot], g_pairWs.dDist + first, count * sizeof(float),
                                     hipMemcpyDeviceToHost, g_pairWs.copy));
        HIP_CHECK(hipEventRecord(g_pairWs.landed[slot], g_pairWs.copy));
    };
    if (total) fetch(0, 0);
    int slot = 0;
    for (size_t first = 0; first < total; first += piece, slot ^= 1) {
        HIP_CHECK(hipEventSynchronize(g_pairWs.landed[slot]));
        if (first + piece < total) fetch(first + piece, slot ^ 1);
        if (file) file->append(g_pairWs.hPairs[slot], withDistance ? g_pairWs.hDist[slot] : nullptr, std::min(piece, total - first));
    }
    if (file) file->close();

    // the reference's total also spans the writing of the file (source/findPairs.cuh:700-726)
    const double totalTime = std::chrono::duration<double>(std::chrono::steady_clock::now() - wall0).count();
    const float kernelSec = (st.sumSquaredMs + st.joinMs) / 1000.0f;
    // unpadded shape: padded zeros are not useful work (source/findPairs.cuh:745-747)
    const float tflops = static_cast<float>(tb.n) * tb.n * tb.d * 2 / kernelSec / 1e12f;
    if (!quiet()) {
        std::printf("Total Elapsed time: %f seconds\n", totalTime);
        std::printf("Total Kernel Elapsed time: %f seconds\n", kernelSec);
        std::printf("SumSquared Kernel Elapsed time: %f seconds\n", st.sumSquaredMs / 1000.0f);
        std::printf("FindPairs Kernel Elapsed time: %f seconds\n", st.joinMs / 1000.0f);
        std::printf("Pairs sort Elapsed time: %f seconds\n", st.sortMs / 1000.0f);
        std::printf("Pairs found: %llu\n", st.pairsFound);
        std::printf("Estimated TFLOPS %.3f\n", tflops);
        std::fflush(stdout);
    }
    Results r;
    r.totalTime = static_cast<float>(totalTime);
    r.TFLOPS = tflops;
    r.pairsFound = st.pairsFound;
    r.pairsStored = st.pairsStored;
    r.inputProblemShape = mmaShape{tb.n, tb.n, tb.d};
    r.paddedProblemShape = mmaShape{tb.nPad, tb.nPad, tb.dPad};
    return r;
}

// Shared body of the three run entry points, the counterpart of run() in
// source/main.cu:198-248: failures are printed and end the process, as there.  `fresh` is a newly
// built dataset that becomes the resident one; without it the resident dataset is reused (reRun).
Results run_resident(fasted::PointTable* fresh, double epsilon, bool savePairs) {
    try {
        if (fresh) {
            g_res.table = std::move(*fresh);
            g_res.uploaded = false;
            if (!quiet()) {
                std::cout << "Number of points is: " << g_res.table.n << std::endl;
                std::cout << "Padding with " << g_res.table.nPad - g_res.table.n << " points" << std::endl;
            }
        }
        const fasted::PointTable& tb = g_res.table;
        if (!quiet() && !tb.empty()) {
            std::cout << "Padded Search Dimensions:\nM: " << tb.nPad << "\nN: " << tb.nPad << "\nK: " << tb.dPad
                      << std::endl;
            std::cout << "Input Search Dimensions:\nM: " << tb.n << "\nN: " << tb.n << "\nK: " << tb.d << std::endl;
        }
        // the output file of a reRun keeps the dataset's name (the reference names it "_<epsilon>.pairs":
        // source/main.cu:203-211 clears the name there, with a note that this is not right)
        return find_pairs_resident(epsilon, savePairs, fresh == nullptr, tb.name);
    } catch (const std::exception& e) {
        std::cout << "Error: Failed to run. " << e.what() << std::endl;
        std::exit(EXIT_FAILURE);
    }
}

template <typename Build>
Results run_built(Build&& build, double epsilon, bool savePairs) {
    fasted::PointTable table;
    try {
        if (!quiet()) std::cout << "Building point list" << std::endl;
        table = build();
    } catch (const std::exception& e) {
        std::cout << "Error: Failed to run. " << e.what() << std::endl;
        std::exit(EXIT_FAILURE);
    }
    return run_resident(&table, epsilon, savePairs);
}

// Uploads the resident dataset if it is not on the device yet.
void ensure_resident_uploaded() {
    const fasted::PointTable& tb = g_res.table;
    if (tb.empty()) throw std::runtime_error("no dataset is resident: call runFromFile or runFromExponentialDataset first");
    if (g_res.uploaded) return;
    HIP_CHECK(hipSetDevice(0));
    g_res.drop_device();
    const size_t bytes = tb.bits.size() * sizeof(uint16_t);
    HIP_CHECK(hipMalloc(&g_res.dPoints, bytes));
    HIP_CHECK(hipMemcpy(g_res.dPoints, tb.bits.data(), bytes, hipMemcpyHostToDevice));
    g_res.uploaded = true;
}

// One join on the resident dataset that only counts: no pair buffer, no sort, no download.  Only the count
// matters, and the test is the same bit for bit for (q, c) and (c, q), so the probe computes the tiles on and above
// the diagonal only and counts every hit off the diagonal twice: the same number in about half the time.
FastedJoinStats count_resident(double epsilon) {
    ensure_resident_uploaded();
    const fasted::PointTable& tb = g_res.table;
    FastedJoinStats st{};
    const PointSet all{g_res.dPoints, tb.n, tb.dPad, nullptr};
    join_on_device(all, all, true, tb.dPad, epsilon, nullptr, 0, FASTED_SYMMETRIC, nullptr, &st);
    return st;
}

// Count-only join of an evenly spaced sample of the resident points against all of them.  Every sampled
// point meets itself among the candidates -- that pair is forced like the self pairs of the full join, so the
// sampled and the full count treat a point's own pair alike -- and found - sampleRows estimates
// sampleRows x selectivity.
FastedJoinStats count_resident_sampled(double epsilon, int sampleRows) {
    ensure_resident_uploaded();
    const fasted::PointTable& tb = g_res.table;
    if (sampleRows < 1) throw std::invalid_argument("sample size must be at least 1 point");
    sampleRows = std::min(sampleRows, tb.n);
    if (!g_res.dSample || g_res.sampleRows != sampleRows) {
        if (g_res.dSample) (void)hipFree(g_res.dSample);
        g_res.dSample = nullptr;
        g_res.sampleRows = 0;
        const size_t pitch = (size_t)tb.dPad * 2;
        const size_t stride = (size_t)(tb.n / sampleRows);
        HIP_CHECK(hipMalloc(&g_res.dSample, (size_t)sampleRows * pitch));
        HIP_CHECK(hipMemcpy2D(g_res.dSample, pitch, g_res.dPoints, pitch * stride, pitch, (size_t)sampleRows,
                              hipMemcpyDeviceToDevice));
        g_res.sampleRows = sampleRows;
    }
    FastedJoinStats st{};
    const PointSet sample{g_res.dSample, sampleRows, tb.dPad, nullptr};
    const PointSet all{g_res.dPoints, tb.n, tb.dPad, nullptr};
    join_on_device(sample, all, false, tb.dPad, epsilon, nullptr, 0, 0, nullptr, &st, nullptr, false,
                   /*forcedStride=*/tb.n / sampleRows);
    return st;
}

double selectivity_of(unsigned long long pairsFound, int n) {
    // (|R| - |D|) / |D|, never negative (results/scripts/experiment/find_pairs.py:9-21)
    const double r = (double)pairsFound - (double)n;
    return (r > 0 ? r : 0.0) / (double)n;
}

// Epsilon for a target selectivity by the reference's procedure (results/scripts/experiment/
// experiments.py:153-281): double epsilon (0 -> 2) until the target is reached, then half steps until the
// selectivity is within 1 % of the target.  `probe` maps epsilon to a selectivity.
template <typename Probe>
double search_epsilon(double targetSelectivity, double initialEpsilon, double* selectivity, Probe&& probe) {
    if (!(targetSelectivity > 0.0)) throw std::invalid_argument("target selectivity must be positive");
    if (initialEpsilon < 0.0) throw std::invalid_argument("initial epsilon must not be negative");
    const double maxEpsilon = 100000.0;
    double lower = initialEpsilon, upper = initialEpsilon, current = 0.0;
    while (current < targetSelectivity) {
        lower = upper;
        upper = (lower == 0.0) ? 2.0 : lower * 2.0;
        if (upper > maxEpsilon)
            throw std::runtime_error("Epsilon of " + std::to_string(upper) + " exceed the maximum value of " +
                                     std::to_string(maxEpsilon) + ". Giving up trying to find the upper bound.");
        current = probe(upper);
    }
    double eps = (upper - lower) / 2.0 + lower, last = upper;
    current = probe(eps);
    int guard = 0;
    while (!(std::fabs(current - targetSelectivity) / targetSelectivity < 0.01)) {
        const double step = std::fabs(eps - last);
        const double next = current > targetSelectivity ? eps - 0.5 * step : eps + 0.5 * step;
        last = eps;
        eps = next;
        if (++guard > 200 || next == last)  // the reference would loop forever on a plateau
            throw std::runtime_error("epsilon search did not converge to within 1% of the target selectivity");
        current = probe(eps);
    }
    if (selectivity) *selectivity = current;
    return eps;
}

// Epsilon for a target selectivity by volume scaling (results/scripts/experiment/experiments.py:100-150,
// 284-323): the number of neighbours is taken to grow like the volume of the epsilon ball, so a probe with
// selectivity s at epsilon e predicts  e * (target / s)^(1/D)  -- the reference forms the two ball volumes with
// pi^(D/2) / Gamma(D/2 + 1) in decimal arithmetic; the constants cancel -- and an empty probe doubles epsilon.
// Ends within 10 % of the target, the reference's threshold for this search.  The reference's loop probes the
// initial epsilon again instead of the adjusted one (experiments.py:314) and so never ends unless the first
// probe is already close enough; here the adjusted epsilon is probed.
template <typename Probe>
double search_epsilon_volumetric(double targetSelectivity, double initialEpsilon, int dims, double* selectivity,
                                 Probe&& probe) {
    if (!(targetSelectivity > 0.0)) throw std::invalid_argument("target selectivity must be positive");
    if (!(initialEpsilon > 0.0)) throw std::invalid_argument("initial epsilon must be positive");
    if (dims < 1) throw std::invalid_argument("no resident dataset");
    double eps = initialEpsilon, current = probe(eps);
    int guard = 0;
    while (!(std::fabs(current - targetSelectivity) / targetSelectivity < 0.1)) {
        const double next = current == 0.0 ? eps * 2.0 : eps * std::pow(targetSelectivity / current, 1.0 / (double)dims);
        if (++guard > 200 || next == eps || !std::isfinite(next))
            throw std::runtime_error("volumetric epsilon search did not converge to within 10% of the target selectivity");
        eps = next;
        current = probe(eps);
    }
    if (selectivity) *selectivity = current;
    return eps;
}

template <typename F>
int guarded(F&& body) {
    try {
        body();
        g_error.clear();
        return 0;
    } catch (const std::exception& e) {
        g_error = e.what();
        (void)hipGetLastError();
        return 1;
    }
}

}  // namespace

extern "C" {

Results runFromExponentialDataset(int size, int dimensionality, double lambda, double max, double epsilon,
                                  bool savePairs) {
    if (!quiet()) std::cout << "Running from a generated exponential dataset" << std::endl;
    return run_built(
        [&] {
            return fasted::build_exponential_table(size, dimensionality, lambda, max, fasted::kSlabK, fasted::kTile);
        },
        epsilon, savePairs);
}

Results runFromFile(const char* filename, double epsilon, bool savePairs) {
    const std::string path(filename ? filename : "");
    if (!quiet()) std::cout << "Running from file: " << path << std::endl;
    // a missing file ends the process here as it does in the reference
    return run_built([&] { return fasted::load_csv_table(path, ',', fasted::kSlabK, fasted::kTile); }, epsilon,
                     savePairs);
}

Results reRun(double epsilon, bool savePairs) { return run_resident(nullptr, epsilon, savePairs); }

void releaseResources(void) {
    g_res.drop_device();
    g_res.table = fasted::PointTable();
    g_ws.release();
    g_pairWs.release();
    g_sortWs.release();
}

int fasted_self_join_device(const void* d_points, long long n, int d, long long ld, double epsilon, float* d_sums,
                            FastedPair* d_pairs, unsigned long long cap, unsigned flags, void* stream,
                            FastedJoinStats* stats) {
    return guarded([&] {
        if (!d_points) throw std::invalid_argument("points pointer is null");
        const PointSet all{d_points, n, ld, d_sums};
        join_on_device(all, all, true, d, epsilon, d_pairs, cap, flags, static_cast<hipStream_t>(stream), stats);
    });
}

int fasted_self_join_device_noalloc(const void* d_points, long long n, int d, long long ld, double epsilon,
                                    FastedPair* d_pairs, unsigned long long cap, unsigned flags, void* stream,
                                    FastedJoinStats* stats) {
    return guarded([&] {
        if (!d_points) throw std::invalid_argument("points pointer is null");
        if (n > (long long)kNoAllocMaxPoints)
            throw std::invalid_argument("fasted_self_join_device_noalloc holds the squared norms of at most " +
                                        std::to_string(kNoAllocMaxPoints) + " points; got " + std::to_string(n));
        if (flags & FASTED_SORT_PAIRS)
            throw std::invalid_argument("fasted_self_join_device_noalloc cannot sort: the sort allocates device memory");
        if (flags & FASTED_SKIP_SUMS)
            throw std::invalid_argument("fasted_self_join_device_noalloc computes the squared norms itself");
        validate_epsilon(epsilon);
        validate_shape(n, d, ld);
        DeviceScratch& ds = device_scratch();
        float* const norms = reinterpret_cast<float*>(ds.base + kNoAllocCounterBytes);
        const JoinScratch js{reinterpret_cast<unsigned long long*>(ds.base), norms, norms + kNoAllocMaxPoints, ds.ev};
        const PointSet all{d_points, n, ld, nullptr};
        join_on_device(all, all, true, d, epsilon, d_pairs, cap, flags, static_cast<hipStream_t>(stream), stats, &js);
    });
}

int fasted_join_device(const void* d_queries, long long n_queries, long long ld_queries, const void* d_candidates,
                       long long n_candidates, long long ld_candidates, int d, double epsilon, float* d_sums_queries,
                       float* d_sums_candidates, FastedPair* d_pairs, unsigned long long cap, unsigned flags,
                       void* stream, FastedJoinStats* stats) {
    return guarded([&] {
        if (!d_queries || !d_candidates) throw std::invalid_argument("points pointer is null");
        const PointSet q{d_queries, n_queries, ld_queries, d_sums_queries};
        const PointSet c{d_candidates, n_candidates, ld_candidates, d_sums_candidates};
        join_on_device(q, c, false, d, epsilon, d_pairs, cap, flags, static_cast<hipStream_t>(stream), stats);
    });
}

int fasted_pair_distances_device(const void* d_queries, long long n_queries, long long ld_queries,
                                 const void* d_candidates, long long n_candidates, long long ld_candidates, int d,
                                 const FastedPair* d_pairs, unsigned long long count, float* d_distances, void* stream) {
    return guarded([&] {
        if (!d_queries || !d_candidates) throw std::invalid_argument("points pointer is null");
        if (count > 0 && (!d_pairs || !d_distances)) throw std::invalid_argument("pair or distance buffer is null");
        validate_shape(n_queries, d, ld_queries);
        validate_shape(n_candidates, d, ld_candidates);
        HIP_CHECK(fasted::launch_pair_distances(d_queries, ld_queries, (int)n_queries, d_candidates, ld_candidates,
                                                (int)n_candidates, round_up(d, fasted::kSlabK), d_pairs, count,
                                                d_distances, static_cast<hipStream_t>(stream)));
        HIP_CHECK(hipStreamSynchronize(static_cast<hipStream_t>(stream)));
    });
}

int fasted_check_padding_device(const void* d_points, long long n, int d, long long ld, unsigned long long* bad_rows,
                                void* stream) {
    return guarded([&] {
        if (!d_points || !bad_rows) throw std::invalid_argument("null pointer");
        validate_shape(n, d, ld);
        g_ws.ensure(1);
        unsigned long long* const word = g_ws.counters;  // word 0 of the counter block is free between joins
        hipStream_t s = static_cast<hipStream_t>(stream);
        HIP_CHECK(fasted::launch_reset_counters(g_ws.counters, false, s));
        HIP_CHECK(fasted::launch_padding_check(d_points, ld, (int)n, d, round_up(d, fasted::kSlabK), word, s));
        HIP_CHECK(hipStreamSynchronize(s));
        HIP_CHECK(hipMemcpy(bad_rows, word, sizeof *bad_rows, hipMemcpyDeviceToHost));
    });
}

int fasted_sum_squared_device(const void* d_points, long long n, int d, long long ld, float* d_sums, void* stream) {
    return guarded([&] {
        if (!d_points || !d_sums) throw std::invalid_argument("null pointer");
        validate_shape(n, d, ld);
        HIP_CHECK(fasted::launch_sum_squared(d_points, ld, (int)n, round_up(d, fasted::kSlabK), d_sums, nullptr, 0.0f,
                                             nullptr, static_cast<hipStream_t>(stream)));
        HIP_CHECK(hipStreamSynchronize(static_cast<hipStream_t>(stream)));
    });
}

int fasted_self_join(const uint16_t* points, long long n, int d, double epsilon, FastedPair* out,
                     unsigned long long cap, unsigned long long* found, unsigned long long* stored) {
    return guarded([&] {
        if (!points) throw std::invalid_argument("points pointer is null");
        if (cap > 0 && !out) throw std::invalid_argument("output buffer is null");
        if (n < 1 || d < 1) throw std::invalid_argument("empty dataset");
        validate_epsilon(epsilon);
        const int dPad = round_up(d, fasted::kSlabK);
        validate_shape(n, d, dPad);
        void* dPoints = nullptr;
        void* dPairs = nullptr;
        try {
            const size_t pitch = (size_t)dPad * 2;
            HIP_CHECK(hipMalloc(&dPoints, (size_t)n * pitch));
            upload_rows(dPoints, pitch, points, (size_t)d * 2, (size_t)n, nullptr);
            HIP_CHECK(hipStreamSynchronize(nullptr));
            HIP_CHECK(hipMalloc(&dPairs, (size_t)(cap ? cap : 1) * sizeof(FastedPair)));
            FastedJoinStats st{};
            const PointSet all{dPoints, n, dPad, nullptr};
            join_on_device(all, all, true, d, epsilon, dPairs, cap, FASTED_SORT_PAIRS, nullptr, &st);
            if (st.pairsStored)
                HIP_CHECK(hipMemcpy(out, dPairs, (size_t)st.pairsStored * sizeof(FastedPair), hipMemcpyDeviceToHost));
            if (found) *found = st.pairsFound;
            if (stored) *stored = st.pairsStored;
        } catch (...) {
            if (dPoints) (void)hipFree(dPoints);
            if (dPairs) (void)hipFree(dPairs);
            throw;
        }
        (void)hipFree(dPoints);
        (void)hipFree(dPairs);
    });
}

int fasted_self_join_blocked(const uint16_t* points, long long n, int d, double epsilon, long long block_rows,
                             FastedPair* out, unsigned long long cap, unsigned long long* found,
                             unsigned long long* stored) {
    return guarded([&] { self_join_blocked(points, n, d, epsilon, block_rows, out, cap, found, stored); });
}

int fasted_load_exponential_dataset(int size, int dimensionality, double lambda, double max) {
    return guarded([&] {
        g_res.drop_device();
        g_res.table = fasted::build_exponential_table(size, dimensionality, lambda, max, fasted::kSlabK, fasted::kTile);
    });
}

int fasted_load_file(const char* filename) {
    return guarded([&] {
        fasted::PointTable table = fasted::load_csv_table(std::string(filename ? filename : ""), ',', fasted::kSlabK,
                                                          fasted::kTile);
        g_res.drop_device();
        g_res.table = std::move(table);
    });
}

const char* fasted_resident_name(void) { return g_res.table.name.c_str(); }

int fasted_count_pairs(double epsilon, unsigned long long* pairsFound, double* kernelSeconds) {
    return guarded([&] {
        const FastedJoinStats st = count_resident(epsilon);
        if (pairsFound) *pairsFound = st.pairsFound;
        if (kernelSeconds) *kernelSeconds = (st.sumSquaredMs + st.joinMs) / 1000.0;
    });
}

int fasted_find_epsilon(double targetSelectivity, double initialEpsilon, double* epsilon, double* selectivity,
                        int* probes) {
    return guarded([&] {
        const int n = g_res.table.n;
        int count = 0;
        const double eps = search_epsilon(targetSelectivity, initialEpsilon, selectivity, [&](double e) {
            ++count;
            return selectivity_of(count_resident(e).pairsFound, n);
        });
        if (epsilon) *epsilon = eps;
        if (probes) *probes = count;
    });
}

int fasted_find_epsilon_volumetric(double targetSelectivity, double initialEpsilon, double* epsilon, double* selectivity,
                                   int* probes) {
    return guarded([&] {
        const int n = g_res.table.n;
        int count = 0;
        const double eps = search_epsilon_volumetric(targetSelectivity, initialEpsilon, g_res.table.d, selectivity, [&](double e) {
            ++count;
            return selectivity_of(count_resident(e).pairsFound, n);
        });
        if (epsilon) *epsilon = eps;
        if (probes) *probes = count;
    });
}

int fasted_count_pairs_sampled(double epsilon, int sample_rows, unsigned long long* pairsFound, int* sampledRows,
                               double* kernelSeconds) {
    return guarded([&] {
        const FastedJoinStats st = count_resident_sampled(epsilon, sample_rows);
        if (pairsFound) *pairsFound = st.pairsFound;
        if (sampledRows) *sampledRows = g_res.sampleRows;
        if (kernelSeconds) *kernelSeconds = (st.sumSquaredMs + st.joinMs) / 1000.0;
    });
}

int fasted_find_epsilon_sampled(double targetSelectivity, double initialEpsilon, int sample_rows, double* epsilon,
                                double* selectivity, int* probes) {
    return guarded([&] {
        int count = 0;
        double estimate = 0.0;
        const double eps = search_epsilon(targetSelectivity, initialEpsilon, &estimate, [&](double e) {
            ++count;
            const FastedJoinStats st = count_resident_sampled(e, sample_rows);
            return selectivity_of(st.pairsFound, g_res.sampleRows);
        });
        // one full count at the end: the selectivity reported is the dataset's, not the sample's
        ++count;
        const double full = selectivity_of(count_resident(eps).pairsFound, g_res.table.n);
        if (epsilon) *epsilon = eps;
        if (selectivity) *selectivity = full;
        if (probes) *probes = count;
    });
}

int fasted_raster_coord(unsigned long long idx, long long n, int* row, int* col) {
    if (n < 1 || !row || !col) return 0;
    return fasted::raster_coord(idx, n, n, false, row, col);
}

int fasted_raster_coord_symmetric(unsigned long long idx, long long n, int* row, int* col) {
    if (n < 1 || !row || !col) return 0;
    return fasted::raster_coord(idx, n, n, true, row, col);
}

unsigned long long fasted_raster_count_symmetric(long long n) { return n < 1 ? 0ull : fasted::raster_count(n, n, true); }

int fasted_lds_chunk_slot(int row, int chunk) { return fasted::lds_chunk_slot(row, chunk); }

unsigned long long fasted_raster_count(long long n) { return n < 1 ? 0ull : fasted::raster_count(n, n); }

const uint16_t* fasted_resident_points(int* n, int* d, int* n_pad, int* d_pad) {
    const fasted::PointTable& tb = g_res.table;
    if (n) *n = tb.n;
    if (d) *d = tb.d;
    if (n_pad) *n_pad = tb.nPad;
    if (d_pad) *d_pad = tb.dPad;
    return tb.empty() ? nullptr : tb.bits.data();
}

void fasted_set_output_dir(const char* dir) { g_outDir = dir ? dir : ""; }

void fasted_set_save_distances(int enabled) { g_saveDistances = enabled != 0; }

void fasted_set_download_pairs(int enabled) { g_downloadPairs = enabled != 0; }

const FastedPair* fasted_last_pairs_device(unsigned long long* stored) {
    if (stored) *stored = g_pairWs.dPairs ? g_lastStored : 0;
    return static_cast<const FastedPair*>(g_pairWs.dPairs);
}

const char* fasted_last_error(void) { return g_error.c_str(); }

const char* fasted_version(void) {
    static const std::string version = [] {
        std::string v = "fasted-mi355x 0.1 (gfx950)";
        const char* const tag = fasted::build_tag();
        if (tag[0]) v += std::string(" ") + tag;
        return v;
    }();
    return version.c_str();
}

}  // extern "C"
