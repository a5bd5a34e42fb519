// A hand-tuned streaming copy, the yardstick bench.py puts beside every bandwidth-bound kernel: what a kernel that
// only moves the same number of bytes (half read, half written) reaches on this GPU, timed the same way.
// Built into lib/libmase_bench.so; not part of the product's C ABI.
//
// Both forms use 128-bit non-temporal loads and stores (every byte is touched once).  Measured on one MI355X at 51, 134
// and 178 MB per launch: the persistent form (two workgroups per compute unit striding through the buffer, two loads in
// flight per lane) is the fastest at the smaller sizes (5.3 / 6.1 / 6.1 TB/s), one 16-byte step per lane in workgroups of
// 512 the fastest at the largest (5.2 / 5.9 / 6.2 TB/s); plain (cached) accesses, contiguous chunks per workgroup, longer
// unrolls and smaller or larger grids were slower.  bench.py times both and reports the better one.
#include <hip/hip_runtime.h>
#include <stdint.h>

typedef unsigned int u4v __attribute__((ext_vector_type(4)));

template <int TPB, int UNROLL>
__global__ __launch_bounds__(TPB) void stream_copy_kernel(const u4v* __restrict__ src, u4v* __restrict__ dst, int64_t n16) {
    int64_t i = (int64_t)blockIdx.x * TPB + threadIdx.x;
    const int64_t stride = (int64_t)gridDim.x * TPB;
    for (; i + (UNROLL - 1) * stride < n16; i += UNROLL * stride) {
        u4v v[UNROLL];
#pragma unroll
        for (int u = 0; u < UNROLL; ++u) v[u] = __builtin_nontemporal_load(src + i + u * stride);
#pragma unroll
        for (int u = 0; u < UNROLL; ++u) __builtin_nontemporal_store(v[u], dst + i + u * stride);
    }
    for (; i < n16; i += stride) __builtin_nontemporal_store(__builtin_nontemporal_load(src + i), dst + i);
}

// form 0: persistent, 2 workgroups of 256 per compute unit; form 1: one 16-byte step per lane, workgroups of 512.
// nbytes must be a multiple of 16 and the pointers 16-byte aligned.  Returns 0, or -1 for bad arguments.
extern "C" int mase_bench_stream_copy(const void* src, void* dst, int64_t nbytes, int form, void* stream) {
    if (!src || !dst || nbytes <= 0 || nbytes % 16 != 0 || ((uintptr_t)src & 15) || ((uintptr_t)dst & 15)) return -1;
    const int64_t n16 = nbytes / 16;
    hipStream_t s = static_cast<hipStream_t>(stream);
    if (form == 0) {
        int dev = 0, cus = 256;
        if (hipGetDevice(&dev) == hipSuccess) hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev);
        hipLaunchKernelGGL((stream_copy_kernel<256, 2>), dim3((unsigned)(2 * cus)), dim3(256), 0, s, static_cast<const u4v*>(src),
                           static_cast<u4v*>(dst), n16);
    } else {
        hipLaunchKernelGGL((stream_copy_kernel<512, 1>), dim3((unsigned)((n16 + 511) / 512)), dim3(512), 0, s,
                           static_cast<const u4v*>(src), static_cast<u4v*>(dst), n16);
    }
    return hipGetLastError() == hipSuccess ? 0 : -3;
}
