// ref_shim.cpp -- C entry points around the REFERENCE's own host data-loader headers.
//
// TEST INFRASTRUCTURE ONLY.  Compiled by oracle/Makefile with
//   -I$(REFERENCE)/source  (the headers are used where they lie; nothing is copied)
// into oracle/_ref/libfasted_ref.so, which is only ever loaded by the tests and by
// tests/golden/make_golden.py to pin the CPU restatement in fasted_oracle.c.
//
// The reference's GPU sources (findPairs.cuh, warpMma.cuh, ptxMma.cuh, sumSquared.cuh,
// pair.cuh, onDemandRasterizer.cuh) need nvcc, CUDA headers, thrust and inline PTX and are
// not buildable here; only DataLoader/*.hpp is plain C++17.
#include <cmath>
#include <cstdint>
#include <cstring>
#include <string>
#include <vector>

#include "DataLoader/ExponentialPointGenerator.hpp"
#include "DataLoader/FilePointGenerator.hpp"
#include "DataLoader/PointListBuilder.hpp"

using half = half_float::half;

namespace {
Points::PointList<half> g_list;
std::string g_name;
std::string g_error;

int finish(Points::PointListBuilder<half>& builder, int dimFactor, int pointsFactor) {
    g_name = builder.getDatasetName();
    g_list = builder.build(dimFactor, pointsFactor);
    return 0;
}
}  // namespace

extern "C" {

// half(float(double)) exactly as PointListBuilder<half>::castValue does it.
uint16_t ref_cast_value(double v) {
    half h(static_cast<float>(v));
    uint16_t bits;
    std::memcpy(&bits, &h, 2);
    return bits;
}

int ref_build_exponential(int n, int d, double lambda, double maxValue, int dimFactor, int pointsFactor) {
    try {
        SimSearch::ExponentialPointGenerator gen(n, d, lambda, maxValue);
        Points::PointListBuilder<half> builder(&gen);
        return finish(builder, dimFactor, pointsFactor);
    } catch (const std::exception& e) {
        g_error = e.what();
        return 1;
    }
}

int ref_build_file(const char* path, int dimFactor, int pointsFactor) {
    try {
        SimSearch::FilePointGenerator gen(path, ',');
        Points::PointListBuilder<half> builder(&gen);
        return finish(builder, dimFactor, pointsFactor);
    } catch (const std::exception& e) {
        g_error = e.what();
        return 1;
    }
}

const char* ref_last_error() { return g_error.c_str(); }
const char* ref_dataset_name() { return g_name.c_str(); }
int ref_num_points() { return g_list.getNumPoints(); }
int ref_actual_num_points() { return g_list.getActualNumPoints(); }
int ref_dimensions() { return g_list.getDimensions(); }
int ref_actual_dimensions() { return g_list.getActualDimensions(); }

// Copies the padded FP16 bit patterns of the last built list.
void ref_copy_values(uint16_t* out) { std::memcpy(out, g_list.values.data(), g_list.values.size() * 2); }
}
