// Bit-packing of MXFP / minifloat element codes for storage: 4-bit codes two to a byte, 6-bit codes four to three
// bytes.  The codes form a little-endian bit stream: code i occupies bits [w i, w i + w) of the packed buffer, w the
// code width.  The reference keeps one byte per code everywhere (src/mase_triton/mxfp/layers.py:69-80 stores
// w_elements as uint8 [n / B, B]); these kernels only change how a stored layer is laid out on disk or at rest in
// HBM, and unpack restores the reference's layout bit for bit.  HBM-bound byte work: a lane moves 16 codes.
#include "../../include/mase_hip.h"
#include "mase_host.h"

namespace mase {
namespace {

constexpr int kPackThreads = 256;

__device__ inline uint32_t squeeze4(uint32_t w, int bits) {  // 4 codes, one per byte -> 4 bits-wide fields, packed
    const uint32_t m = (1u << bits) - 1u;
    return (w & m) | (((w >> 8) & m) << bits) | (((w >> 16) & m) << (2 * bits)) | (((w >> 24) & m) << (3 * bits));
}
__device__ inline uint32_t spread4(uint32_t t, int bits) {   // inverse of squeeze4
    const uint32_t m = (1u << bits) - 1u;
    return (t & m) | (((t >> bits) & m) << 8) | (((t >> (2 * bits)) & m) << 16) | (((t >> (3 * bits)) & m) << 24);
}

template <int BITS>
__global__ __launch_bounds__(kPackThreads) void pack_codes_kernel(const uint4* __restrict__ codes, uint32_t* __restrict__ packed,
                                                                  int64_t n_chunks) {
    const int64_t c = (int64_t)blockIdx.x * kPackThreads + threadIdx.x;
    if (c >= n_chunks) return;
    const uint4 v = codes[c];
    const uint32_t t0 = squeeze4(v.x, BITS), t1 = squeeze4(v.y, BITS), t2 = squeeze4(v.z, BITS), t3 = squeeze4(v.w, BITS);
    if (BITS == 4) {
        *reinterpret_cast<uint2*>(packed + 2 * c) = make_uint2(t0 | (t1 << 16), t2 | (t3 << 16));
    } else {  // 6 bits: four 24-bit groups -> three words
        uint32_t* o = packed + 3 * c;
        o[0] = t0 | (t1 << 24);
        o[1] = (t1 >> 8) | (t2 << 16);
        o[2] = (t2 >> 16) | (t3 << 8);
    }
}

template <int BITS>
__global__ __launch_bounds__(kPackThreads) void unpack_codes_kernel(const uint32_t* __restrict__ packed, uint4* __restrict__ codes,
                                                                    int64_t n_chunks) {
    const int64_t c = (int64_t)blockIdx.x * kPackThreads + threadIdx.x;
    if (c >= n_chunks) return;
    uint32_t t0, t1, t2, t3;
    if (BITS == 4) {
        const uint2 p = *reinterpret_cast<const uint2*>(packed + 2 * c);
        t0 = p.x & 0xFFFFu; t1 = p.x >> 16; t2 = p.y & 0xFFFFu; t3 = p.y >> 16;
    } else {
        const uint32_t* p = packed + 3 * c;
        const uint32_t a = p[0], b = p[1], d = p[2];
        t0 = a & 0xFFFFFFu;
        t1 = (a >> 24) | ((b & 0xFFFFu) << 8);
        t2 = (b >> 16) | ((d & 0xFFu) << 16);
        t3 = d >> 8;
    }
    codes[c] = make_uint4(spread4(t0, BITS), spread4(t1, BITS), spread4(t2, BITS), spread4(t3, BITS));
}

int check_pack_args(const void* a, const void* b, int64_t n, int bits) {
    if (bits != 4 && bits != 6) return fail(ERR_INVALID, "code width must be 4 or 6 bits (8-bit codes are stored as they are)");
    if (n < 0 || n % 16 != 0) return fail(ERR_INVALID, "code count must be a non-negative multiple of 16");
    if (n == 0) return OK;
    if (!a || !b) return fail(ERR_INVALID, "null pointer");
    return OK;
}

}  // namespace
}  // namespace mase

using namespace mase;

extern "C" {

int mase_hip_pack_codes(const uint8_t* elements, uint8_t* packed, int64_t n, int bits, void* stream) {
    if (int rc = check_pack_args(elements, packed, n, bits)) return rc;
    if (n == 0) return OK;
    if (!aligned(elements, 16) || !aligned(packed, 8)) return fail(ERR_INVALID, "elements must be 16-byte and packed 8-byte aligned");
    const int64_t chunks = n / 16;
    const unsigned grid = (unsigned)((chunks + kPackThreads - 1) / kPackThreads);
    hipStream_t s = static_cast<hipStream_t>(stream);
    if (bits == 4)
        hipLaunchKernelGGL(pack_codes_kernel<4>, dim3(grid), dim3(kPackThreads), 0, s, reinterpret_cast<const uint4*>(elements),
                           reinterpret_cast<uint32_t*>(packed), chunks);
    else
        hipLaunchKernelGGL(pack_codes_kernel<6>, dim3(grid), dim3(kPackThreads), 0, s, reinterpret_cast<const uint4*>(elements),
                           reinterpret_cast<uint32_t*>(packed), chunks);
    return check_launch("pack_codes");
}

int mase_hip_unpack_codes(const uint8_t* packed, uint8_t* elements, int64_t n, int bits, void* stream) {
    if (int rc = check_pack_args(packed, elements, n, bits)) return rc;
    if (n == 0) return OK;
    if (!aligned(elements, 16) || !aligned(packed, 8)) return fail(ERR_INVALID, "elements must be 16-byte and packed 8-byte aligned");
    const int64_t chunks = n / 16;
    const unsigned grid = (unsigned)((chunks + kPackThreads - 1) / kPackThreads);
    hipStream_t s = static_cast<hipStream_t>(stream);
    if (bits == 4)
        hipLaunchKernelGGL(unpack_codes_kernel<4>, dim3(grid), dim3(kPackThreads), 0, s, reinterpret_cast<const uint32_t*>(packed),
                           reinterpret_cast<uint4*>(elements), chunks);
    else
        hipLaunchKernelGGL(unpack_codes_kernel<6>, dim3(grid), dim3(kPackThreads), 0, s, reinterpret_cast<const uint32_t*>(packed),
                           reinterpret_cast<uint4*>(elements), chunks);
    return check_launch("unpack_codes");
}

}  // extern "C"
