// mfma_probe.hip -- what rate the matrix cores sustain on their own: register-only loops of the two FP16
// MFMA shapes of gfx950 with the accumulator footprint of the join kernel's wave tile (128 x 64), no LDS
// and no memory traffic, on all-zero operands and on operands distributed like the benchmark data.
// The chip is power limited on this instruction stream, so the answer depends on the operand values and
// on the shape; it is the ceiling the join kernel's MFMA utilisation x clock has to be read against.
//
//   mfma_probe [iterations]     (default 100000; one line per variant)
#include <hip/hip_runtime.h>

#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <vector>

typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef float floatx16 __attribute__((ext_vector_type(16)));
typedef float floatx4 __attribute__((ext_vector_type(4)));

#define CHECK(x)                                                                              \
    do {                                                                                      \
        hipError_t e_ = (x);                                                                  \
        if (e_ != hipSuccess) {                                                               \
            std::printf("HIP error %s at line %d\n", hipGetErrorString(e_), __LINE__);        \
            std::exit(1);                                                                     \
        }                                                                                     \
    } while (0)

constexpr int kThreads = 512;    // 8 waves per CU, 2 per SIMD, as the join kernel
constexpr int kFragments = 12;   // operand fragments a wave holds (8 + 4)

// kShape 0: v_mfma_f32_16x16x32_f16, 8 x 4 blocks;  1: v_mfma_f32_32x32x16_f16, 4 x 2 blocks.
// Both cover a 128 x 64 tile with 128 accumulator registers and 2 x 128 x 64 x 32 FLOP per pass.
template <int kShape>
__global__ void __launch_bounds__(kThreads, 1) mfma_loop(const half8* __restrict__ operands, float* __restrict__ out,
                                                         int iterations) {
    half8 frag[kFragments];
    for (int i = 0; i < kFragments; ++i) frag[i] = operands[threadIdx.x + kThreads * i];
    float sum = 0.0f;
    if (kShape == 0) {
        floatx4 acc[8][4];
        for (int i = 0; i < 8; ++i)
            for (int j = 0; j < 4; ++j)
                for (int r = 0; r < 4; ++r) acc[i][j][r] = 0.0f;
        for (int it = 0; it < iterations; ++it) {
#pragma unroll
            for (int j = 0; j < 4; ++j)
#pragma unroll
                for (int i = 0; i < 8; ++i)
                    acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_f16(frag[i], frag[8 + j], acc[i][j], 0, 0, 0);
        }
        for (int i = 0; i < 8; ++i)
            for (int j = 0; j < 4; ++j)
                for (int r = 0; r < 4; ++r) sum += acc[i][j][r];
    } else {
        floatx16 acc[4][2];
        for (int i = 0; i < 4; ++i)
            for (int j = 0; j < 2; ++j)
                for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.0f;
        for (int it = 0; it < iterations; ++it) {
#pragma unroll
            for (int half = 0; half < 2; ++half)  // two k = 16 steps make the k = 32 of the other shape
#pragma unroll
                for (int j = 0; j < 2; ++j)
#pragma unroll
                    for (int i = 0; i < 4; ++i)
                        acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(frag[i + 4 * half], frag[8 + j + 2 * half],
                                                                           acc[i][j], 0, 0, 0);
        }
        for (int i = 0; i < 4; ++i)
            for (int j = 0; j < 2; ++j)
                for (int r = 0; r < 16; ++r) sum += acc[i][j][r];
    }
    out[blockIdx.x * kThreads + threadIdx.x] = sum;
}

template <int kShape>
void run(const char* shape, const char* data, const half8* operands, float* out, int iterations, int workgroups) {
    hipEvent_t e0, e1;
    CHECK(hipEventCreate(&e0));
    CHECK(hipEventCreate(&e1));
    float ms = 0.0f;
    for (int rep = 0; rep < 2; ++rep) {  // the first launch warms up
        CHECK(hipEventRecord(e0, nullptr));
        mfma_loop<kShape><<<workgroups, kThreads>>>(operands, out, iterations);
        CHECK(hipEventRecord(e1, nullptr));
        CHECK(hipDeviceSynchronize());
        CHECK(hipEventElapsedTime(&ms, e0, e1));
    }
    const double flop = 2.0 * 128 * 64 * 32 * 8.0 * workgroups * iterations;
    std::printf("%-24s %-10s %8.2f ms  %7.1f TFLOP/s  %5.1f %% of 2516.6\n", shape, data, ms, flop / ms / 1e9,
                100.0 * flop / ms / 1e9 / 2516.6);
    CHECK(hipEventDestroy(e0));
    CHECK(hipEventDestroy(e1));
}

int main(int argc, char** argv) {
    const int iterations = argc > 1 ? std::atoi(argv[1]) : 100000;
    hipDeviceProp_t prop;
    CHECK(hipGetDeviceProperties(&prop, 0));
    const int workgroups = prop.multiProcessorCount;
    const size_t halves = (size_t)kThreads * kFragments * 8;
    half8* operands;
    float* out;
    CHECK(hipMalloc(&operands, halves * 2));
    CHECK(hipMalloc(&out, (size_t)workgroups * kThreads * sizeof(float)));
    std::vector<_Float16> host(halves);
    std::printf("%s, %d CUs, %d iterations\n", prop.name, workgroups, iterations);
    for (int mode = 0; mode < 2; ++mode) {
        unsigned state = 12345u;
        for (auto& h : host) {
            state = state * 1664525u + 1013904223u;
            const float u = ((state >> 8) + 0.5f) / 16777216.0f;
            h = (_Float16)(mode == 0 ? 0.0f : std::fmin(-std::log(1.0f - u) / 40.0f, 1.0f));
        }
        CHECK(hipMemcpy(operands, host.data(), halves * 2, hipMemcpyHostToDevice));
        const char* data = mode == 0 ? "zeros" : "Exp(40)";
        run<0>("v_mfma_f32_16x16x32_f16", data, operands, out, iterations, workgroups);
        run<1>("v_mfma_f32_32x32x16_f16", data, operands, out, iterations, workgroups);
    }
    return 0;
}
