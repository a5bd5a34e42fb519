// C-ABI entry point of the block-scaled MXFP GEMM; the kernel is in gemm_scaled.h.
#include "gemm_impl.h"

using namespace mase;

static int scaled_entry(const uint8_t* a_codes, const uint32_t* a_scales, const uint8_t* w_codes, const uint32_t* w_scales,
                        const void* bias, int bias_dtype, void* y, int out_dtype, int64_t M, int64_t N, int64_t K, void* workspace,
                        int64_t workspace_bytes, void* stream) {
    if (M < 0 || N < 1 || K < 1) return fail(ERR_INVALID, "M must not be negative, N and K must be positive");
    if (M == 0) return OK;   // no rows of A: nothing to compute
    if (M > 0x7FFFFFFF || N > 0x7FFFFFFF || K >= ((int64_t)1 << 27)) return fail(ERR_INVALID, "M, N must fit in 31 bits and K in 27");
    if (K % 256 != 0 || K < 512) return fail(ERR_UNSUPPORTED, "the block-scaled GEMM needs K to be a multiple of 256, at least 512");
    if (!a_codes || !a_scales || !w_codes || !w_scales || !y) return fail(ERR_INVALID, "null pointer");
    if (int rc = check_dtype(out_dtype, "output")) return rc;
    if (bias) if (int rc = check_dtype(bias_dtype, "bias")) return rc;
    if (!aligned(a_codes, 16) || !aligned(w_codes, 16) || !aligned(a_scales, 4) || !aligned(w_scales, 4) || !aligned(y, 16))
        return fail(ERR_INVALID, "codes and y must be 16-byte aligned, scales 4-byte aligned");
    if (N % (16 / dtype_size(out_dtype)) != 0) return fail(ERR_UNSUPPORTED, "the block-scaled GEMM stores 16 bytes at a time: N must be a multiple of 8 (4 for fp32 output)");
    if (workspace_bytes < 0) return fail(ERR_INVALID, "workspace_bytes must not be negative");
    if (workspace && !aligned(workspace, 16)) return fail(ERR_INVALID, "workspace must be 16-byte aligned");
    hipStream_t s = static_cast<hipStream_t>(stream);
    return dispatch_dtype(out_dtype, [&](auto dout) {
        return launch_gemm_scaled<decltype(dout)::value>(a_codes, a_scales, w_codes, w_scales, bias, bias_dtype, y, (int)M, (int)N, (int)K,
                                                         workspace, workspace ? workspace_bytes : 0, s);
    });
}

extern "C" int mase_hip_mxfp_gemm_scaled(const uint8_t* a_codes, const uint32_t* a_scales, const uint8_t* w_codes, const uint32_t* w_scales,
                                         const void* bias, int bias_dtype, void* y, int out_dtype, int64_t M, int64_t N, int64_t K,
                                         void* stream) {
    return scaled_entry(a_codes, a_scales, w_codes, w_scales, bias, bias_dtype, y, out_dtype, M, N, K, nullptr, 0, stream);
}

extern "C" int mase_hip_mxfp_gemm_scaled_ws(const uint8_t* a_codes, const uint32_t* a_scales, const uint8_t* w_codes, const uint32_t* w_scales,
                                            const void* bias, int bias_dtype, void* y, int out_dtype, int64_t M, int64_t N, int64_t K,
                                            void* workspace, int64_t workspace_bytes, void* stream) {
    return scaled_entry(a_codes, a_scales, w_codes, w_scales, bias, bias_dtype, y, out_dtype, M, N, K, workspace, workspace_bytes, stream);
}

extern "C" int64_t mase_hip_mxfp_gemm_scaled_workspace_bytes(int64_t M, int64_t N, int64_t K) {
    if (M < 1 || N < 1 || K < 512 || K % 256 != 0 || M > 0x7FFFFFFF || N > 0x7FFFFFFF || K >= ((int64_t)1 << 27)) return 0;
    if (const int slices = scaled_rows_slices((int)M, (int)N, (int)K)) return (int64_t)slices * M * N * 4;
    const int splits = plan_scaled_splits((int)M, (int)N, (int)K, device_cu_count());
    return splits > 1 ? (int64_t)splits * M * N * 4 : 0;
}

extern "C" int mase_hip_mxfp_gemm_prepared_w(const void* a_dense, int a_dtype, const uint8_t* w_codes, const uint32_t* w_scales, const void* bias,
                                             int bias_dtype, void* y, int out_dtype, int64_t M, int64_t N, int64_t K, void* stream) {
    if (M < 0 || N < 1 || K < 1) return fail(ERR_INVALID, "M must not be negative, N and K must be positive");
    if (M == 0) return OK;   // no rows of A: nothing to compute
    if (M > 0x7FFFFFFF || N > 0x7FFFFFFF || K > 0x7FFFFFFF) return fail(ERR_INVALID, "M, N, K must fit in 31 bits");
    if (!a_dense || !w_codes || !w_scales || !y) return fail(ERR_INVALID, "null pointer");
    if (a_dtype != BF16) return fail(ERR_UNSUPPORTED, "a dense A operand must be bfloat16");
    if (int rc = check_dtype(out_dtype, "output")) return rc;
    if (bias) if (int rc = check_dtype(bias_dtype, "bias")) return rc;
    if (!aligned(a_dense, 16) || !aligned(w_codes, 16) || !aligned(w_scales, 4) || !aligned(y, 16))
        return fail(ERR_INVALID, "A, codes and y must be 16-byte aligned, scales 4-byte aligned");
    hipStream_t s = static_cast<hipStream_t>(stream);
    return dispatch_dtype(out_dtype, [&](auto dout) {
        return launch_gemm_tall_prepared<decltype(dout)::value>(a_dense, w_codes, w_scales, bias, bias_dtype, y, (int)M, (int)N, (int)K, s);
    });
}

// ---- activations straight through: operand of x, then the product, in one call
static int64_t linear_scaled_operand_bytes(int64_t M, int64_t K) {
    const int64_t rows_pad = mase_hip_scaled_padded_rows(M);
    return (rows_pad * K + (K / 128) * rows_pad * 4 + 255) / 256 * 256;      // codes, scale dwords; the workspace behind them stays aligned
}

extern "C" int64_t mase_hip_mxfp_linear_scaled_scratch_bytes(int64_t M, int64_t N, int64_t K) {
    if (M < 1 || N < 1 || K < 512 || K % 256 != 0 || M > 0x7FFFFFFF || N > 0x7FFFFFFF || K >= ((int64_t)1 << 27)) return 0;
    return linear_scaled_operand_bytes(M, K) + mase_hip_mxfp_gemm_scaled_workspace_bytes(M, N, K);
}

extern "C" int mase_hip_mxfp_linear_scaled(const void* x, int x_dtype, int x_exp_bits, int x_frac_bits, int x_is_minifloat, const uint8_t* w_codes,
                                           const uint32_t* w_scales, const void* bias, int bias_dtype, void* y, int out_dtype, int64_t M, int64_t N,
                                           int64_t K, void* scratch, int64_t scratch_bytes, void* stream) {
    if (M < 0 || N < 1 || K < 1) return fail(ERR_INVALID, "M must not be negative, N and K must be positive");
    if (M == 0) return OK;   // no rows of x: nothing to compute
    if (K % 256 != 0 || K < 512) return fail(ERR_UNSUPPORTED, "the block-scaled GEMM needs K to be a multiple of 256, at least 512");
    if (!scratch || !aligned(scratch, 256)) return fail(ERR_INVALID, "scratch must be given, 256-byte aligned");
    const int64_t operand = linear_scaled_operand_bytes(M, K);
    if (scratch_bytes < operand) return fail(ERR_INVALID, "scratch is smaller than the operand of x: ask mase_hip_mxfp_linear_scaled_scratch_bytes");
    uint8_t* const a_codes = static_cast<uint8_t*>(scratch);
    uint32_t* const a_scales = reinterpret_cast<uint32_t*>(a_codes + mase_hip_scaled_padded_rows(M) * K);
    if (int rc = x_is_minifloat ? mase_hip_scaled_operand_from_dense_minifloat(x, x_dtype, x_exp_bits, x_frac_bits, M, K, a_codes, a_scales, stream)
                                : mase_hip_scaled_operand_from_dense(x, x_dtype, x_exp_bits, x_frac_bits, M, K, a_codes, a_scales, stream))
        return rc;
    const int64_t rest = scratch_bytes - operand;
    return scaled_entry(a_codes, a_scales, w_codes, w_scales, bias, bias_dtype, y, out_dtype, M, N, K, rest > 0 ? a_codes + operand : nullptr, rest, stream);
}
