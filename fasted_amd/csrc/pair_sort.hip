// pair_sort.hip -- what happens to the stored pairs on the device after the join: the row-major
// ordering, and the optional distance of every pair.
//
// The reference sorts its pair buffer with thrust::sort and Pair::operator< (query index,
// then candidate index; source/pair.cuh:39-45,151-158).  A pair is 8 bytes with the query
// index in the low word; packed as (query << bits of a candidate index) | candidate that order is plain
// unsigned order on the low bits of a 64-bit key: pack, radix sort over just those bits (42 instead of 64
// for two million points: 6 passes of 8 bits instead of 8), unpack.
#include <cstring>

#include <rocprim/device/device_radix_sort.hpp>

#include "join_kernels.h"

namespace fasted {
namespace {

// record (candidate << 32 | query) -> key (query << candidateBits | candidate), and back
__global__ void pack_pairs_kernel(const unsigned long long* __restrict__ in, unsigned long long* __restrict__ out,
                                  unsigned long long count, int candidateBits) {
    const unsigned long long stride = (unsigned long long)gridDim.x * blockDim.x;
    for (unsigned long long i = (unsigned long long)blockIdx.x * blockDim.x + threadIdx.x; i < count; i += stride) {
        const unsigned long long v = in[i];
        out[i] = ((v & 0xffffffffull) << candidateBits) | (v >> 32);
    }
}
__global__ void unpack_pairs_kernel(const unsigned long long* __restrict__ in, unsigned long long* __restrict__ out,
                                    unsigned long long count, int candidateBits) {
    const unsigned long long stride = (unsigned long long)gridDim.x * blockDim.x;
    for (unsigned long long i = (unsigned long long)blockIdx.x * blockDim.x + threadIdx.x; i < count; i += stride) {
        const unsigned long long k = in[i];
        out[i] = ((k & ((1ull << candidateBits) - 1ull)) << 32) | (k >> candidateBits);
    }
}

int index_bits(long long n) {  // bits of the largest index of n items; 32 when n is not known
    if (n <= 0 || n > (1ll << 32)) return 32;
    int b = 1;
    while ((1ll << b) < n) ++b;
    return b;
}

typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));

// Euclidean distance of every listed pair, sum of squared differences in FP32 (no cancellation, unlike
// the expansion the join itself tests).  16 lanes share a pair: 16-byte chunks of both rows, strided.
// Pairs that name a point outside its set get NaN.
__global__ void __launch_bounds__(256) pair_distances_kernel(const u32x4* __restrict__ ptsQ, long long ldQ16, int nQ,
                                                             const u32x4* __restrict__ ptsC, long long ldC16, int nC,
                                                             int chunksPerRow, const int2* __restrict__ pairs,
                                                             unsigned long long count, float* __restrict__ out) {
    const int sub = threadIdx.x & 15;
    const unsigned long long groups = ((unsigned long long)gridDim.x * blockDim.x) >> 4;
    for (unsigned long long g = ((unsigned long long)blockIdx.x * blockDim.x + threadIdx.x) >> 4; g < count; g += groups) {
        const int2 pr = pairs[g];
        const bool valid = pr.x >= 0 && pr.x < nQ && pr.y >= 0 && pr.y < nC;
        float acc = 0.0f;
        if (valid) {
            const u32x4* a = ptsQ + (long long)pr.x * ldQ16;
            const u32x4* b = ptsC + (long long)pr.y * ldC16;
            for (int c = sub; c < chunksPerRow; c += 16) {
                const half8 x = __builtin_bit_cast(half8, a[c]);
                const half8 y = __builtin_bit_cast(half8, b[c]);
#pragma unroll
                for (int e = 0; e < 8; ++e) {
                    const float diff = (float)x[e] - (float)y[e];
                    acc = __builtin_fmaf(diff, diff, acc);
                }
            }
        }
#pragma unroll
        for (int off = 8; off > 0; off >>= 1) acc += __shfl_xor(acc, off, 64);
        if (sub == 0) out[g] = valid ? __builtin_sqrtf(acc) : __builtin_nanf("");
    }
}

unsigned grid_for(unsigned long long count) {
    unsigned long long blocks = (count + 255) / 256;
    return (unsigned)(blocks > 65536ull ? 65536ull : (blocks ? blocks : 1));
}

}  // namespace

void SortBuffers::release() {
    if (alt) (void)hipFree(alt);
    if (temp) (void)hipFree(temp);
    alt = temp = nullptr;
    altBytes = tempBytes = 0;
}

// Grows the two buffers of `ws` to what `count` records need; they are kept for the next sort.
static hipError_t reserve_sort_buffers(SortBuffers* ws, unsigned long long count, hipStream_t stream) {
    size_t needTemp = 0;
    hipError_t e = rocprim::radix_sort_keys(nullptr, needTemp, static_cast<unsigned long long*>(nullptr),
                                            static_cast<unsigned long long*>(nullptr), (size_t)count, 0u, 64u, stream);
    if (e != hipSuccess) return e;
    if (needTemp == 0) needTemp = 16;
    const size_t needAlt = (size_t)count * sizeof(unsigned long long);
    if (needAlt > ws->altBytes) {
        if (ws->alt) (void)hipFree(ws->alt);
        ws->alt = nullptr;
        ws->altBytes = 0;
        e = hipMalloc(&ws->alt, needAlt);
        if (e != hipSuccess) return e;
        ws->altBytes = needAlt;
    }
    if (needTemp > ws->tempBytes) {
        if (ws->temp) (void)hipFree(ws->temp);
        ws->temp = nullptr;
        ws->tempBytes = 0;
        e = hipMalloc(&ws->temp, needTemp);
        if (e != hipSuccess) return e;
        ws->tempBytes = needTemp;
    }
    return hipSuccess;
}

size_t sort_scratch_bytes(unsigned long long count) {
    size_t needTemp = 0;
    if (rocprim::radix_sort_keys(nullptr, needTemp, static_cast<unsigned long long*>(nullptr),
                                 static_cast<unsigned long long*>(nullptr), (size_t)count, 0u, 64u, nullptr) != hipSuccess)
        return 0;
    return needTemp + (size_t)count * sizeof(unsigned long long);
}

hipError_t sort_pairs_row_major(void* pairs, unsigned long long count, hipStream_t stream, SortBuffers* ws,
                                long long nQueries, long long nCandidates) {
    if (count < 2) return hipSuccess;
    SortBuffers local;
    SortBuffers* const b = ws ? ws : &local;
    hipError_t e = reserve_sort_buffers(b, count, stream);
    auto* keys = static_cast<unsigned long long*>(pairs);
    auto* alt = static_cast<unsigned long long*>(b->alt);
    if (e == hipSuccess) {
        const int candidateBits = index_bits(nCandidates);
        const unsigned keyBits = (unsigned)(candidateBits + index_bits(nQueries));
        size_t tempBytes = b->tempBytes;
        pack_pairs_kernel<<<grid_for(count), 256, 0, stream>>>(keys, keys, count, candidateBits);
        e = rocprim::radix_sort_keys(b->temp, tempBytes, keys, alt, (size_t)count, 0u, keyBits, stream);
        if (e == hipSuccess) {
            unpack_pairs_kernel<<<grid_for(count), 256, 0, stream>>>(alt, keys, count, candidateBits);
            e = hipGetLastError();
        } else {
            // the keys are still in place, packed: put the records back as they were
            unpack_pairs_kernel<<<grid_for(count), 256, 0, stream>>>(keys, keys, count, candidateBits);
        }
    }
    const hipError_t s = hipStreamSynchronize(stream);
    if (e == hipSuccess) e = s;
    if (!ws) local.release();
    return e;
}

hipError_t launch_pair_distances(const void* queries, long long ldQ, int nQ, const void* candidates, long long ldC,
                                 int nC, int dPad, const void* pairs, unsigned long long count, float* out,
                                 hipStream_t stream) {
    if (count == 0) return hipSuccess;
    const unsigned long long blocks = (count * 16 + 255) / 256;
    pair_distances_kernel<<<dim3((unsigned)(blocks > 16384ull ? 16384ull : blocks)), dim3(256), 0, stream>>>(
        static_cast<const u32x4*>(queries), ldQ / 8, nQ, static_cast<const u32x4*>(candidates), ldC / 8, nC, dPad / 8,
        static_cast<const int2*>(pairs), count, out);
    return hipGetLastError();
}

}  // namespace fasted
