// Yardstick for the memory-bound kernels: what this device gives a kernel that does nothing but read a buffer
// once.  The flat GEMM is judged against the published HBM peak; this kernel measures, on the same box and the
// same buffers, the read bandwidth that is actually attainable, in the manner of the reference's
// bandwidth_memread/bandwidth_kernel.cu:68-92 (a grid sized to the machine, every thread looping over 16-byte
// non-temporal loads UNROLL at a time, the values folded into a register that is stored only if it takes a
// value it cannot take).
#pragma once
#include "a8w8_device.hpp"

namespace a8w8 {

constexpr int HBM_PROBE_THREADS = 256;
constexpr int HBM_PROBE_UNROLL = 16;     // with eight workgroups per compute unit the best of the configurations tried (unroll 4 / 8 / 16, 1 .. 64 workgroups per compute unit)

__global__ void __launch_bounds__(HBM_PROBE_THREADS) hbm_read_probe_kernel(const v4i* src, size_t n16, int* sink)
{
    const size_t stride = (size_t)gridDim.x * HBM_PROBE_THREADS;
    size_t i = (size_t)blockIdx.x * HBM_PROBE_THREADS + threadIdx.x;
    v4i folded = {0, 0, 0, 0};
    // UNROLL loads in flight per thread, each instruction of a wave covering 1 KiB of contiguous memory
    for (; i + (HBM_PROBE_UNROLL - 1) * stride < n16; i += HBM_PROBE_UNROLL * stride) {
        v4i v[HBM_PROBE_UNROLL];
#pragma unroll
        for (int u = 0; u < HBM_PROBE_UNROLL; ++u) v[u] = __builtin_nontemporal_load(src + i + u * stride);
#pragma unroll
        for (int u = 0; u < HBM_PROBE_UNROLL; ++u) folded ^= v[u];
    }
    for (; i < n16; i += stride) folded ^= __builtin_nontemporal_load(src + i);
    // never true for data that is not crafted for it; keeps the loads alive
    if ((folded.x ^ folded.y ^ folded.z ^ folded.w) == 0x5ca1ab1e && (folded.x & folded.y) == 0x0defaced) sink[0] = folded.z;
}

}  // namespace a8w8
