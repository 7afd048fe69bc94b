// point_table.hpp -- host data layer: point sources and the padded FP16 point table.
//
// Behavioural counterpart of the reference's source/DataLoader/*.hpp:
//   PointSource        <- SimSearch::PointGenerator            (PointGenerator.hpp:18-30)
//   ExponentialSource  <- SimSearch::ExponentialPointGenerator (ExponentialPointGenerator.hpp:18-72)
//   CsvSource          <- SimSearch::FilePointGenerator        (FilePointGenerator.hpp:17-74)
//   build_point_table  <- Points::PointListBuilder<half>::build (PointListBuilder.hpp:132-192)
//   PointTable         <- Points::PointList<half>              (PointList.hpp:12-42)
// Same seeds, same draw order, same double -> float -> half rounding, same padding rule,
// same dataset names and the same error texts, so a caller sees the same dataset.
#pragma once
#include <cmath>
#include <cstdint>
#include <cstring>
#include <fstream>
#include <ios>
#include <iostream>
#include <random>
#include <stdexcept>
#include <string>
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

// One point per line, fields separated by `delimiter`, each parsed like std::stod.
class CsvSource final : public PointSource {
   public:
    explicit CsvSource(const std::string& path, char delimiter = ',') : path_(path), in_(path), delim_(delimiter) {
        if (path.empty()) throw std::invalid_argument("filepath must be set.");
        if (!in_.is_open()) throw std::ios_base::failure("Failed to open file: " + path);
    }

    bool next(std::vector<double>& row) override {
        if (!std::getline(in_, line_)) return false;
        row.clear();
        size_t pos = 0;
        const size_t len = line_.size();
        while (pos < len) {  // a trailing delimiter yields no empty last field, as std::getline
            size_t end = line_.find(delim_, pos);
            if (end == std::string::npos) end = len;
            const std::string field = line_.substr(pos, end - pos);
            try {
                row.push_back(std::stod(field));
            } catch (const std::exception&) {
                std::cout << "Failed to parse value: " << field << " from dataset" << std::endl;
                throw;
            }
            pos = end + 1;
        }
        return true;
    }

    std::string name() const override {  // file name without directory and last extension
        const size_t slash = path_.find_last_of("/\\");
        const std::string file = path_.substr(slash + 1);
        return file.substr(0, file.find_last_of('.'));
    }

   private:
    std::string path_;
    std::ifstream in_;
    std::string line_;
    char delim_;
};

struct PointTable {
    std::vector<uint16_t> bits;  // [nPad][dPad] IEEE binary16, zero padded
    int n = 0, d = 0;            // real points / dimensions
    int nPad = 0, dPad = 0;
    std::string name;
    bool empty() const { return bits.empty(); }
};

inline uint16_t quantize_half(double v) {  // double -> float -> half, both round-to-nearest-even
    const _Float16 h = static_cast<_Float16>(static_cast<float>(v));
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

}  // namespace fasted
