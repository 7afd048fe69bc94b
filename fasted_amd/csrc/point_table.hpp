// point_table.hpp -- host data layer: point sources and the padded FP16 point table.
//
// Behavioural counterpart of the reference's source/DataLoader/*.hpp:
//   PointSource        <- SimSearch::PointGenerator            (PointGenerator.hpp:18-30)
//   ExponentialSource  <- SimSearch::ExponentialPointGenerator (ExponentialPointGenerator.hpp:18-72)
//   load_csv_table     <- SimSearch::FilePointGenerator        (FilePointGenerator.hpp:17-74) + build
//   build_point_table  <- Points::PointListBuilder<half>::build (PointListBuilder.hpp:132-192)
//   PointTable         <- Points::PointList<half>              (PointList.hpp:12-42)
// Same seeds, same draw order, same double -> float -> half rounding, same padding rule,
// same dataset names and the same error texts, so a caller sees the same dataset.
#pragma once
#include <algorithm>
#include <cerrno>
#include <cmath>
#include <cstdint>
#include <cstring>
#include <cstdlib>
#include <condition_variable>
#include <functional>
#include <mutex>
#include <fstream>
#include <ios>
#include <iterator>
#include <iostream>
#include <random>
#include <stdexcept>
#include <string>
#include <thread>
#include <vector>

namespace fasted {

class PointSource {
   public:
    virtual ~PointSource() = default;
    // Fills `row` with the next point; false when the source is exhausted.
    virtual bool next(std::vector<double>& row) = 0;
    virtual std::string name() const = 0;
};

// Exp(lambda) coordinates, redrawn until they fall in [0, maxValue]; std::mt19937 with the
// reference's fixed seed and std::exponential_distribution<double>, drawn point by point.
class ExponentialSource final : public PointSource {
   public:
    static constexpr uint32_t kSeed = 2137834274u;  // ExponentialPointGenerator.hpp:11

    ExponentialSource(int numPoints, int numDims, double lambda, double maxValue)
        : remaining_(numPoints), total_(numPoints), dims_(numDims), lambda_(lambda), max_(maxValue), engine_(kSeed),
          dist_(lambda) {}

    bool next(std::vector<double>& row) override {
        if (remaining_ <= 0) return false;
        row.resize(dims_ > 0 ? dims_ : 0);
        for (int k = 0; k < dims_; ++k) {
            double v;
            do {
                v = dist_(engine_);
            } while (v < 0.0 || v > max_);
            row[k] = v;
        }
        --remaining_;
        return true;
    }

    std::string name() const override {
        return "Exponential_" + std::to_string(total_) + "_" + std::to_string(dims_) + "_" + std::to_string(lambda_);
    }

   private:
    int remaining_, total_, dims_;
    double lambda_, max_;
    std::mt19937 engine_;
    std::exponential_distribution<double> dist_;
};

struct PointTable {
    std::vector<uint16_t> bits;  // [nPad][dPad] IEEE binary16, zero padded
    int n = 0, d = 0;            // real points / dimensions
    int nPad = 0, dPad = 0;
    std::string name;
    bool empty() const { return bits.empty(); }
};

// double -> float -> half, both round-to-nearest-even.  The float is kept in a volatile so that the
// compiler cannot merge the two conversions into one double -> half rounding, which differs on
// values whose float image is an exact tie between two halves (e.g. 0.01198196413320991).
inline uint16_t quantize_half(double v) {
    volatile float narrowed = static_cast<float>(v);
    const _Float16 h = static_cast<_Float16>(narrowed);
    uint16_t b;
    std::memcpy(&b, &h, sizeof b);
    return b;
}

inline int round_up_to(int value, int multiple) {
    return static_cast<int>(std::ceil(1.0 * value / multiple) * multiple);
}

// Drains `src` into a table whose dimensionality is padded to a multiple of `dimMultiple`
// and whose point count is padded to a multiple of `pointMultiple`, all padding zero.
inline PointTable build_point_table(PointSource& src, int dimMultiple, int pointMultiple, int maxPoints = 0) {
    PointTable t;
    t.name = src.name();
    std::vector<double> row;
    int count = 0;
    try {
        while ((maxPoints == 0 || count < maxPoints) && src.next(row)) {
            const int dims = static_cast<int>(row.size());
            if (count == 0) {
                t.d = dims;
                t.dPad = round_up_to(dims, dimMultiple);
            } else if (dims != t.d) {
                throw std::runtime_error("Dimensions of subsequent points didn't match the first point");
            }
            const size_t base = t.bits.size();
            t.bits.resize(base + static_cast<size_t>(t.dPad), 0);
            for (int k = 0; k < dims; ++k) t.bits[base + k] = quantize_half(row[k]);
            ++count;
        }
    } catch (const std::exception&) {
        std::cout << "Failed to build point list at line: " << count << std::endl;
        throw;
    }
    if (count == 0) throw std::runtime_error("No points were generated.");
    t.n = count;
    t.nPad = round_up_to(count, pointMultiple);
    t.bits.resize(static_cast<size_t>(t.nPad) * static_cast<size_t>(t.dPad), 0);
    return t;
}

inline unsigned host_threads(const char* specificEnv) {
    const char* env = std::getenv(specificEnv);
    if (!env) env = std::getenv("FASTED_HOST_THREADS");
    unsigned t = env ? static_cast<unsigned>(std::atoi(env)) : std::thread::hardware_concurrency();
    if (t == 0) t = 1;
    return t > 16 ? 16 : t;
}

// ---------------------------------------------------------------------------------------------
// The seeded exponential dataset, built by several threads, value for value what
// build_point_table(ExponentialSource) gives.  What makes that possible: every candidate value of
// std::exponential_distribution<double> over std::mt19937 consumes exactly two engine outputs
// (std::generate_canonical<double, 53> with a 32-bit engine), whether it is then rejected or not, so
// candidate i is a function of outputs 2i and 2i+1 alone and the dataset is the accepted candidates
// in order.  One thread runs the engine (the only sequential part, 1 to 1.5 ns per output), the
// others turn blocks of raw outputs into candidates (logarithm, range test, quantisation), and the
// accepted values of each block are copied to their place once the blocks before it are counted.
namespace detail {

// The output stream of std::mt19937 (MT19937, 32 bit), produced a state block of 624 words at a time:
// the same recurrence and tempering, written as plain loops over the block, about ten times faster than
// one engine call per output.
class Mt19937Stream {
   public:
    explicit Mt19937Stream(uint32_t seed) {
        state_[0] = seed;
        for (uint32_t i = 1; i < kWords; ++i) state_[i] = 1812433253u * (state_[i - 1] ^ (state_[i - 1] >> 30)) + i;
    }
    void generate(uint32_t* out, size_t count) {
        while (count > 0) {
            if (next_ == kWords) refill();
            const size_t run = std::min<size_t>(count, kWords - next_);
            std::memcpy(out, tempered_ + next_, run * sizeof(uint32_t));
            out += run;
            next_ += static_cast<uint32_t>(run);
            count -= run;
        }
    }

   private:
    static constexpr uint32_t kWords = 624, kShift = 397;
    static uint32_t mix(uint32_t upper, uint32_t lower) {
        const uint32_t y = (upper & 0x80000000u) | (lower & 0x7fffffffu);
        return (y >> 1) ^ ((lower & 1u) ? 0x9908b0dfu : 0u);
    }
    void refill() {
        uint32_t i = 0;
        for (; i < kWords - kShift; ++i) state_[i] = state_[i + kShift] ^ mix(state_[i], state_[i + 1]);
        for (; i < kWords - 1; ++i) state_[i] = state_[i + kShift - kWords] ^ mix(state_[i], state_[i + 1]);
        state_[kWords - 1] = state_[kShift - 1] ^ mix(state_[kWords - 1], state_[0]);
        for (i = 0; i < kWords; ++i) {
            uint32_t y = state_[i];
            y ^= y >> 11;
            y ^= (y << 7) & 0x9d2c5680u;
            y ^= (y << 15) & 0xefc60000u;
            y ^= y >> 18;
            tempered_[i] = y;
        }
        next_ = 0;
    }
    uint32_t state_[kWords];
    uint32_t tempered_[kWords];
    uint32_t next_ = kWords;
};

// A few worker threads that run one job after another: start(body) has worker w call body(b) for the blocks
// b = w, w + workers, ... < blocks; wait() returns when all of them are through.  (Threads are kept
// because creating one per round costs more than a round's work.)
class RoundPool {
   public:
    RoundPool(unsigned workers, size_t blocks) : workers_(workers), blocks_(blocks) {
        for (unsigned w = 0; w < workers_; ++w) threads_.emplace_back([this, w] { loop(w); });
    }
    ~RoundPool() {
        {
            std::lock_guard<std::mutex> lock(mutex_);
            stop_ = true;
        }
        wake_.notify_all();
        for (auto& t : threads_) t.join();
    }
    void start(std::function<void(size_t)> body) {
        {
            std::lock_guard<std::mutex> lock(mutex_);
            body_ = std::move(body);
            pending_ = workers_;
            ++round_;
        }
        wake_.notify_all();
    }
    void wait() {
        std::unique_lock<std::mutex> lock(mutex_);
        done_.wait(lock, [this] { return pending_ == 0; });
    }

   private:
    void loop(unsigned w) {
        unsigned long long seen = 0;
        for (;;) {
            std::function<void(size_t)> body;
            {
                std::unique_lock<std::mutex> lock(mutex_);
                wake_.wait(lock, [&] { return stop_ || round_ != seen; });
                if (stop_) return;
                seen = round_;
                body = body_;
            }
            for (size_t b = w; b < blocks_; b += workers_) body(b);
            std::lock_guard<std::mutex> lock(mutex_);
            if (--pending_ == 0) done_.notify_all();
        }
    }
    unsigned workers_;
    size_t blocks_;
    std::vector<std::thread> threads_;
    std::mutex mutex_;
    std::condition_variable wake_, done_;
    std::function<void(size_t)> body_;
    unsigned pending_ = 0;
    unsigned long long round_ = 0;
    bool stop_ = false;
};

// libstdc++'s generate_canonical<double, 53>(mt19937) followed by exponential_distribution<double>
inline double exponential_from_outputs(uint32_t first, uint32_t second, double lambda) {
    double sum = static_cast<double>(first) * 1.0;
    sum += static_cast<double>(second) * 4294967296.0;
    double u = sum / 18446744073709551616.0;
    if (u >= 1.0) u = std::nextafter(1.0, 0.0);
    return -std::log(1.0 - u) / lambda;
}

}  // namespace detail

inline PointTable build_exponential_table(int numPoints, int numDims, double lambda, double maxValue, int dimMultiple,
                                          int pointMultiple, unsigned threads = 0) {
    if (threads == 0) threads = host_threads("FASTED_GEN_THREADS");
    const unsigned long long total = numPoints > 0 && numDims > 0 ? 1ull * numPoints * numDims : 0ull;
    if (threads < 2 || total < (1ull << 20)) {  // small or degenerate: the plain sequential builder
        ExponentialSource src(numPoints, numDims, lambda, maxValue);
        return build_point_table(src, dimMultiple, pointMultiple);
    }
    PointTable t;
    t.name = ExponentialSource(numPoints, numDims, lambda, maxValue).name();
    t.n = numPoints;
    t.d = numDims;
    t.dPad = round_up_to(numDims, dimMultiple);
    t.nPad = round_up_to(numPoints, pointMultiple);
    t.bits.assign(static_cast<size_t>(t.nPad) * static_cast<size_t>(t.dPad), 0);

    constexpr size_t kBlock = 1u << 15;  // candidates per block
    const unsigned workers = threads - 1;  // one thread runs the engine
    const size_t roundBlocks = static_cast<size_t>(workers) * 4;
    std::vector<uint32_t> raw[2];
    raw[0].resize(2 * kBlock * roundBlocks);
    raw[1].resize(2 * kBlock * roundBlocks);
    std::vector<uint16_t> values(kBlock * roundBlocks);
    std::vector<size_t> counts(roundBlocks), offsets(roundBlocks);
    detail::Mt19937Stream engine(ExponentialSource::kSeed);
    auto fill = [&](std::vector<uint32_t>& out) { engine.generate(out.data(), out.size()); };
    detail::RoundPool pool(workers, roundBlocks);
    fill(raw[0]);
    unsigned long long produced = 0;
    int cur = 0;
    while (produced < total) {
        const uint32_t* const in = raw[cur].data();
        pool.start([&, in](size_t b) {
            const uint32_t* r = in + 2 * kBlock * b;
            uint16_t* out = values.data() + kBlock * b;
            size_t kept = 0;
            for (size_t i = 0; i < kBlock; ++i) {
                const double v = detail::exponential_from_outputs(r[2 * i], r[2 * i + 1], lambda);
                if (v < 0.0 || v > maxValue) continue;  // redrawn by the sequential generator
                out[kept++] = quantize_half(v);
            }
            counts[b] = kept;
        });
        fill(raw[cur ^ 1]);  // the engine runs ahead while the workers convert
        pool.wait();
        unsigned long long at = produced;
        for (size_t b = 0; b < roundBlocks; ++b) {
            offsets[b] = static_cast<size_t>(at);
            at += counts[b];
        }
        pool.start([&](size_t b) {
            unsigned long long j = offsets[b];
            const uint16_t* src = values.data() + kBlock * b;
            size_t left = counts[b];
            while (left > 0 && j < total) {  // contiguous run inside one row of the padded table
                const size_t row = static_cast<size_t>(j / numDims), col = static_cast<size_t>(j % numDims);
                const size_t run = std::min<unsigned long long>({left, static_cast<unsigned long long>(numDims - col), total - j});
                std::memcpy(t.bits.data() + row * t.dPad + col, src, run * sizeof(uint16_t));
                src += run;
                left -= run;
                j += run;
            }
        });
        pool.wait();
        produced = at;
        cur ^= 1;
    }
    return t;
}

// ---------------------------------------------------------------------------------------------
// CSV files: one point per line, fields separated by `delimiter`, each field parsed like std::stod
// (leading blanks skipped, trailing characters after the number ignored, no number -> error).  The
// file is read once and its lines are parsed by several threads straight into the padded table; the
// result and the error texts are those of the reference's sequential reader + builder.
inline std::string csv_dataset_name(const std::string& path) {  // file name without directory and last extension
    const size_t slash = path.find_last_of("/\\");
    const std::string file = path.substr(slash + 1);
    return file.substr(0, file.find_last_of('.'));
}

namespace detail {

struct CsvError {
    long long line = -1;  // first failing line (0-based), -1 = none
    std::string what;
    bool outOfRange = false;
    bool mismatch = false;
    std::string field;
};

// Parses one line into `out` (quantised) or just counts its fields when out == nullptr.
// Returns the number of fields; on a malformed field fills `err` and returns -1.
inline int parse_csv_line(const char* p, const char* end, char delim, uint16_t* out, int maxFields, CsvError& err) {
    int count = 0;
    while (p < end) {  // a trailing delimiter yields no empty last field, as std::getline
        const char* stop = static_cast<const char*>(std::memchr(p, delim, static_cast<size_t>(end - p)));
        if (!stop) stop = end;
        // strtod needs a terminated buffer; fields are short, so copy
        char buf[64];
        const size_t len = static_cast<size_t>(stop - p);
        std::string big;
        const char* text = buf;
        if (len < sizeof buf) {
            std::memcpy(buf, p, len);
            buf[len] = 0;
        } else {
            big.assign(p, len);
            text = big.c_str();
        }
        char* after = nullptr;
        errno = 0;
        const double v = std::strtod(text, &after);
        if (after == text || errno == ERANGE) {
            err.field.assign(p, len);
            err.outOfRange = after != text;
            err.what = "stod";
            return -1;
        }
        if (out && count < maxFields) out[count] = quantize_half(v);
        ++count;
        p = stop + 1;
    }
    return count;
}

}  // namespace detail

inline PointTable load_csv_table(const std::string& path, char delim, int dimMultiple, int pointMultiple,
                                 unsigned threads = 0) {
    if (path.empty()) throw std::invalid_argument("filepath must be set.");
    std::ifstream in(path, std::ios::binary);
    if (!in.is_open()) throw std::ios_base::failure("Failed to open file: " + path);
    std::string text((std::istreambuf_iterator<char>(in)), std::istreambuf_iterator<char>());
    in.close();

    // line starts; the last line may lack its newline, a final newline opens no further line
    std::vector<size_t> starts;
    for (size_t pos = 0; pos < text.size();) {
        starts.push_back(pos);
        const void* nl = std::memchr(text.data() + pos, '\n', text.size() - pos);
        pos = nl ? static_cast<size_t>(static_cast<const char*>(nl) - text.data()) + 1 : text.size();
    }
    const long long lines = static_cast<long long>(starts.size());
    auto line_end = [&](long long i) {
        size_t e = (i + 1 < lines) ? starts[i + 1] - 1 : text.size();
        if (e > starts[i] && i + 1 == lines && text[e - 1] == '\n') --e;
        return e;
    };

    PointTable t;
    t.name = csv_dataset_name(path);
    if (lines == 0) throw std::runtime_error("No points were generated.");
    detail::CsvError first;
    const int dims = detail::parse_csv_line(text.data() + starts[0], text.data() + line_end(0), delim, nullptr, 0, first);
    if (dims < 0) {
        std::cout << "Failed to parse value: " << first.field << " from dataset" << std::endl;
        std::cout << "Failed to build point list at line: 0" << std::endl;
        if (first.outOfRange) throw std::out_of_range(first.what);
        throw std::invalid_argument(first.what);
    }
    t.n = static_cast<int>(lines);
    t.d = dims;
    t.dPad = round_up_to(dims, dimMultiple);
    t.nPad = round_up_to(t.n, pointMultiple);
    t.bits.assign(static_cast<size_t>(t.nPad) * static_cast<size_t>(t.dPad), 0);

    if (threads == 0) threads = host_threads("FASTED_CSV_THREADS");
    if (static_cast<long long>(threads) > lines) threads = static_cast<unsigned>(lines);
    std::vector<detail::CsvError> errors(threads);
    auto work = [&](unsigned w) {
        const long long lo = lines * w / threads, hi = lines * (w + 1) / threads;
        for (long long i = lo; i < hi; ++i) {
            detail::CsvError e;
            const int got = detail::parse_csv_line(text.data() + starts[i], text.data() + line_end(i), delim,
                                                   t.bits.data() + static_cast<size_t>(i) * t.dPad, dims, e);
            if (got == dims) continue;
            e.line = i;
            if (got >= 0) {
                e.mismatch = true;
                e.what = "Dimensions of subsequent points didn't match the first point";
            }
            errors[w] = e;
            return;  // the sequential reader stops at its first bad line too
        }
    };
    std::vector<std::thread> pool;
    for (unsigned w = 1; w < threads; ++w) pool.emplace_back(work, w);
    work(0);
    for (auto& th : pool) th.join();

    const detail::CsvError* bad = nullptr;
    for (const auto& e : errors)
        if (e.line >= 0 && (!bad || e.line < bad->line)) bad = &e;
    if (bad) {
        if (!bad->mismatch) std::cout << "Failed to parse value: " << bad->field << " from dataset" << std::endl;
        std::cout << "Failed to build point list at line: " << bad->line << std::endl;
        if (bad->mismatch) throw std::runtime_error(bad->what);
        if (bad->outOfRange) throw std::out_of_range(bad->what);
        throw std::invalid_argument(bad->what);
    }
    return t;
}

}  // namespace fasted
