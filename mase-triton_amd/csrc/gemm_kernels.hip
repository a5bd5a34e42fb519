// Dequant-fused MXFP GEMM for gfx950:  y[M,N] = A[M,K] * W[N,K]^T (+ bias), fp32 accumulation
// on v_mfma_f32_32x32x16_bf16.
//
// W (and optionally A) arrive as MXFP components: one uint8 code per element, one uint8 scale
// per 32 elements along K.  A workgroup owns a BM x BN tile of y.  Per K-step it stages a
// BM x BK slab of A and a BN x BK slab of W in LDS as bf16; MXFP operands are composed to bf16
// in registers on the way (code -> fp32 by exponent-field placement, times the block scale,
// -> bf16; exact, every MXFP value has at most 4 significant bits).  Each wavefront then feeds
// 32x32x16 MFMA tiles from LDS with 128-bit fragment reads.
//
// MFMA operand layout (wave64): lane l supplies row/column l%32 and the 8 consecutive k values
// starting at 8*(l/32); accumulator register v of lane l is y[8*(v/4) + 4*(l/32) + v%4][l%32].
#include "../../include/mase_hip.h"
#include "mase_host.h"

namespace mase {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float floatx16 __attribute__((ext_vector_type(16)));
typedef float floatx2_t __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));

__device__ inline uint32_t cvt_pk_bf16(float a, float b) {
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(floatx2_t{a, b}, bf16x2_t));
}

// 16 MXFP codes (one 128-bit word) of one block -> 16 bf16 (two 128-bit words).
template <class F>
__device__ inline void compose16(const uint4& codes, uint32_t scale, const F& f, uint4& lo, uint4& hi) {
    const float s = scale_f32(scale);
    const uint32_t w[4] = {codes.x, codes.y, codes.z, codes.w};
    uint32_t o[8];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const float v0 = decode_f32(w[j] & 0xFFu, f) * s;
        const float v1 = decode_f32((w[j] >> 8) & 0xFFu, f) * s;
        const float v2 = decode_f32((w[j] >> 16) & 0xFFu, f) * s;
        const float v3 = decode_f32(w[j] >> 24, f) * s;
        o[2 * j] = cvt_pk_bf16(v0, v1);
        o[2 * j + 1] = cvt_pk_bf16(v2, v3);
    }
    lo = make_uint4(o[0], o[1], o[2], o[3]);
    hi = make_uint4(o[4], o[5], o[6], o[7]);
}

constexpr int BM = 128, BN = 128, BK = 32;
constexpr int kGemmThreads = 256;
constexpr int LDS_STRIDE = BK + 8;  // bf16 elements per tile row: 80 bytes, conflict-free 128-bit reads

// A_MODE: 0 = dense bf16 A, 1 = MXFP A (format FA).  W is always MXFP (format FW).
template <int A_MODE, class FA, class FW, int DT_OUT>
__global__ __launch_bounds__(kGemmThreads) void mxfp_gemm_kernel(
    const uint16_t* __restrict__ a_dense, const uint8_t* __restrict__ a_scales, const uint8_t* __restrict__ a_elements,
    const uint8_t* __restrict__ w_scales, const uint8_t* __restrict__ w_elements, const void* __restrict__ bias,
    int bias_dtype, void* __restrict__ y, int M, int N, int K, FA fa, FW fw) {
    __shared__ __attribute__((aligned(16))) uint16_t lds_a[BM * LDS_STRIDE];
    __shared__ __attribute__((aligned(16))) uint16_t lds_w[BN * LDS_STRIDE];

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wave_m = wave >> 1, wave_n = wave & 1;  // 2 x 2 waves, 64 x 64 each
    const int m0 = blockIdx.y * BM, n0 = blockIdx.x * BN;
    const int kblocks = K / 32;

    // staging assignment: thread t handles tile row t/2, k-half t%2 (16 elements)
    const int srow = tid >> 1, shalf = tid & 1;
    const bool a_row_ok = m0 + srow < M, w_row_ok = n0 + srow < N;
    const int64_t a_row = (int64_t)(m0 + srow), w_row = (int64_t)(n0 + srow);

    floatx16 acc[2][2];
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.0f;

    uint4 ra0 = make_uint4(0, 0, 0, 0), ra1 = ra0, rw = ra0;
    uint32_t sa = 0, sw = 0;
    auto fetch = [&](int kt) {
        const int64_t k = (int64_t)kt * BK + shalf * 16;
        if (a_row_ok) {
            if (A_MODE == 0) {
                const uint4* p = reinterpret_cast<const uint4*>(a_dense + a_row * K + k);
                ra0 = p[0];
                ra1 = p[1];
            } else {
                ra0 = *reinterpret_cast<const uint4*>(a_elements + a_row * K + k);
                sa = a_scales[a_row * kblocks + kt];
            }
        }
        if (w_row_ok) {
            rw = *reinterpret_cast<const uint4*>(w_elements + w_row * K + k);
            sw = w_scales[w_row * kblocks + kt];
        }
    };

    const int ktiles = K / BK;
    fetch(0);
    for (int kt = 0; kt < ktiles; ++kt) {
        __syncthreads();  // everyone finished reading the previous slab
        {
            uint4 lo, hi;
            if (A_MODE == 0) { lo = ra0; hi = ra1; }
            else compose16(ra0, sa, fa, lo, hi);
            uint4* pa = reinterpret_cast<uint4*>(&lds_a[srow * LDS_STRIDE + shalf * 16]);
            pa[0] = lo; pa[1] = hi;
            compose16(rw, sw, fw, lo, hi);
            uint4* pw = reinterpret_cast<uint4*>(&lds_w[srow * LDS_STRIDE + shalf * 16]);
            pw[0] = lo; pw[1] = hi;
        }
        __syncthreads();
        if (kt + 1 < ktiles) fetch(kt + 1);
#pragma unroll
        for (int ks = 0; ks < BK / 16; ++ks) {
            bf16x8 af[2], bf[2];
            const int kofs = ks * 16 + (lane >> 5) * 8;
#pragma unroll
            for (int i = 0; i < 2; ++i)
                af[i] = *reinterpret_cast<const bf16x8*>(&lds_a[(wave_m * 64 + i * 32 + (lane & 31)) * LDS_STRIDE + kofs]);
#pragma unroll
            for (int j = 0; j < 2; ++j)
                bf[j] = *reinterpret_cast<const bf16x8*>(&lds_w[(wave_n * 64 + j * 32 + (lane & 31)) * LDS_STRIDE + kofs]);
#pragma unroll
            for (int i = 0; i < 2; ++i)
#pragma unroll
                for (int j = 0; j < 2; ++j) acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(af[i], bf[j], acc[i][j], 0, 0, 0);
        }
    }

    // epilogue: bias, rounding, store
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            const int col = n0 + wave_n * 64 + j * 32 + (lane & 31);
            if (col >= N) continue;
            float b = 0.0f;
            if (bias) {
                if (bias_dtype == F32) b = static_cast<const float*>(bias)[col];
                else {
                    const uint32_t h = static_cast<const uint16_t*>(bias)[col];
                    b = bits_f32(bias_dtype == BF16 ? h << 16 : half_bits_to_f32_bits(h));
                }
            }
#pragma unroll
            for (int v = 0; v < 16; ++v) {
                const int row = m0 + wave_m * 64 + i * 32 + 8 * (v >> 2) + 4 * (lane >> 5) + (v & 3);
                if (row >= M) continue;
                const float r = acc[i][j][v] + b;
                const int64_t o = (int64_t)row * N + col;
                if (DT_OUT == F32) static_cast<float*>(y)[o] = r;
                else if (DT_OUT == BF16) static_cast<uint16_t*>(y)[o] = (uint16_t)(cvt_pk_bf16(r, 0.0f) & 0xFFFFu);
                else static_cast<uint16_t*>(y)[o] = (uint16_t)f32_bits_to_half_bits(f32_bits(r));
            }
        }
}

template <class Fn>
inline int dispatch_preset(int E, int M, Fn&& fn) {
    if (E == 4 && M == 3) return fn(SFmt<4, 3>{});
    if (E == 5 && M == 2) return fn(SFmt<5, 2>{});
    if (E == 2 && M == 3) return fn(SFmt<2, 3>{});
    if (E == 3 && M == 2) return fn(SFmt<3, 2>{});
    if (E == 2 && M == 1) return fn(SFmt<2, 1>{});
    return fail(ERR_INVALID, "MXFP element (exp_bits, frac_bits) must be one of (4,3) (5,2) (2,3) (3,2) (2,1)");
}

}  // namespace mase

using namespace mase;

extern "C" int mase_hip_mxfp_gemm(const void* a_dense, int a_dtype, const uint8_t* a_scales, const uint8_t* a_elements,
                                  int a_exp_bits, int a_frac_bits, const uint8_t* w_scales, const uint8_t* w_elements,
                                  int w_exp_bits, int w_frac_bits, const void* bias, int bias_dtype, void* y, int out_dtype,
                                  int64_t M, int64_t N, int64_t K, int block_size, void* stream) {
    if (M < 1 || N < 1 || K < 1) return fail(ERR_INVALID, "M, N, K must be positive");
    if (M > 0x7FFFFFFF || N > 0x7FFFFFFF || K > 0x7FFFFFFF) return fail(ERR_INVALID, "M, N, K must fit in 31 bits");
    if (block_size != 32) return fail(ERR_UNSUPPORTED, "the GEMM supports block_size 32 only");
    if (K % 32 != 0) return fail(ERR_INVALID, "K must be a multiple of the block size");
    if (!w_scales || !w_elements || !y) return fail(ERR_INVALID, "null pointer");
    if (int rc = check_dtype(out_dtype, "output")) return rc;
    if (bias) if (int rc = check_dtype(bias_dtype, "bias")) return rc;
    const bool a_is_dense = a_dense != nullptr;
    if (a_is_dense) {
        if (a_dtype != BF16) return fail(ERR_UNSUPPORTED, "a dense A operand must be bfloat16");
        if (!aligned(a_dense, 16)) return fail(ERR_INVALID, "A must be 16-byte aligned");
    } else {
        if (!a_scales || !a_elements) return fail(ERR_INVALID, "A needs either a dense pointer or scales and elements");
        if (!aligned(a_elements, 16)) return fail(ERR_INVALID, "a_elements must be 16-byte aligned");
    }
    if (!aligned(w_elements, 16)) return fail(ERR_INVALID, "w_elements must be 16-byte aligned");
    hipStream_t s = static_cast<hipStream_t>(stream);
    const dim3 grid((unsigned)((N + BN - 1) / BN), (unsigned)((M + BM - 1) / BM));
    if (grid.y > 65535u) return fail(ERR_UNSUPPORTED, "M too large for the launch grid");
    return dispatch_preset(w_exp_bits, w_frac_bits, [&](auto fw) {
        return dispatch_dtype(out_dtype, [&](auto dout) {
            if (a_is_dense) {
                hipLaunchKernelGGL((mxfp_gemm_kernel<0, SFmt<4, 3>, decltype(fw), decltype(dout)::value>), grid, dim3(kGemmThreads), 0, s,
                                   static_cast<const uint16_t*>(a_dense), nullptr, nullptr, w_scales, w_elements, bias, bias_dtype, y,
                                   (int)M, (int)N, (int)K, SFmt<4, 3>{}, fw);
                return check_launch("mxfp_gemm");
            }
            return dispatch_preset(a_exp_bits, a_frac_bits, [&](auto fa) {
                hipLaunchKernelGGL((mxfp_gemm_kernel<1, decltype(fa), decltype(fw), decltype(dout)::value>), grid, dim3(kGemmThreads), 0, s,
                                   nullptr, a_scales, a_elements, w_scales, w_elements, bias, bias_dtype, y, (int)M, (int)N, (int)K, fa,
                                   fw);
                return check_launch("mxfp_gemm");
            });
        });
    });
}
