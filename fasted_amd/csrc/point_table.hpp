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
#include <cerrno>
#include <cmath>
#include <cstdint>
#include <cstring>
#include <cstdlib>
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

    if (threads == 0) {
        const char* env = std::getenv("FASTED_CSV_THREADS");
        threads = env ? static_cast<unsigned>(std::atoi(env)) : std::thread::hardware_concurrency();
        if (threads == 0) threads = 1;
        if (threads > 16) threads = 16;
    }
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
