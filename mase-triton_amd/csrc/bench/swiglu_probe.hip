// Test helper, not part of the product's C ABI: the SwiGLU arithmetic of the operand kernel (swiglu.h) on its own,
// out[i] = silu(gate[i]) * up[i] in bfloat16, so that a test can compare every bf16 gate value with a tensor library.
#include <hip/hip_runtime.h>
#include <stdint.h>
#include "../swiglu.h"

namespace {
__global__ __launch_bounds__(256) void swiglu_probe_kernel(const uint4* __restrict__ gate, const uint4* __restrict__ up, uint4* __restrict__ out,
                                                           int64_t n8) {
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    // every lane takes part in the wave-uniform test inside: lanes past the end work on zeros
    const uint4 zero = make_uint4(0, 0, 0, 0);
    const uint4 h = mase::swiglu_x8(i < n8 ? gate[i] : zero, i < n8 ? up[i] : zero);
    if (i < n8) out[i] = h;
}
}  // namespace

extern "C" int mase_bench_swiglu_bf16(const void* gate, const void* up, void* out, int64_t n, void* stream) {
    if (!gate || !up || !out || n <= 0 || n % 8 != 0 || (((uintptr_t)gate | (uintptr_t)up | (uintptr_t)out) & 15)) return -1;
    const int64_t n8 = n / 8;
    hipLaunchKernelGGL(swiglu_probe_kernel, dim3((unsigned)((n8 + 255) / 256)), dim3(256), 0, static_cast<hipStream_t>(stream),
                       static_cast<const uint4*>(gate), static_cast<const uint4*>(up), static_cast<uint4*>(out), n8);
    return hipGetLastError() == hipSuccess ? 0 : -3;
}
