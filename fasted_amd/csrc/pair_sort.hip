// pair_sort.hip -- row-major ordering of the stored pairs on the device.
//
// The reference sorts its pair buffer with thrust::sort and Pair::operator< (query index,
// then candidate index; source/pair.cuh:39-45,151-158).  A pair is 8 bytes with the query
// index in the low word, so rotating each record by 32 bits turns that order into plain
// unsigned 64-bit order: rotate, radix sort, rotate back.
#include <cstring>

#include <rocprim/device/device_radix_sort.hpp>

#include "join_kernels.h"

namespace fasted {
namespace {

__global__ void rotate_pairs_kernel(const unsigned long long* __restrict__ in, unsigned long long* __restrict__ out,
                                    unsigned long long count) {
    const unsigned long long stride = (unsigned long long)gridDim.x * blockDim.x;
    for (unsigned long long i = (unsigned long long)blockIdx.x * blockDim.x + threadIdx.x; i < count; i += stride) {
        const unsigned long long v = in[i];
        out[i] = (v << 32) | (v >> 32);
    }
}

unsigned grid_for(unsigned long long count) {
    unsigned long long blocks = (count + 255) / 256;
    return (unsigned)(blocks > 65536ull ? 65536ull : (blocks ? blocks : 1));
}

}  // namespace

hipError_t sort_pairs_row_major(void* pairs, unsigned long long count, hipStream_t stream) {
    if (count < 2) return hipSuccess;
    auto* keys = static_cast<unsigned long long*>(pairs);
    unsigned long long* alt = nullptr;
    void* temp = nullptr;
    size_t tempBytes = 0;
    hipError_t e = hipMalloc(&alt, count * sizeof(unsigned long long));
    if (e != hipSuccess) return e;
    e = rocprim::radix_sort_keys(nullptr, tempBytes, keys, alt, (size_t)count, 0u, 64u, stream);
    if (e == hipSuccess) e = hipMalloc(&temp, tempBytes ? tempBytes : 16);
    if (e == hipSuccess) {
        rotate_pairs_kernel<<<grid_for(count), 256, 0, stream>>>(keys, keys, count);
        e = rocprim::radix_sort_keys(temp, tempBytes, keys, alt, (size_t)count, 0u, 64u, stream);
    }
    if (e == hipSuccess) {
        rotate_pairs_kernel<<<grid_for(count), 256, 0, stream>>>(alt, keys, count);
        e = hipGetLastError();
    }
    hipError_t s = hipStreamSynchronize(stream);
    if (e == hipSuccess) e = s;
    if (temp) (void)hipFree(temp);
    (void)hipFree(alt);
    return e;
}

}  // namespace fasted
