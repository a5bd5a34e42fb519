// C-ABI entry point of the MXFP GEMM; the kernels are in gemm_impl.h, instantiated per weight
// format in gemm_w_*.hip.
#include "gemm_impl.h"

using namespace mase;

extern "C" int64_t mase_hip_mxfp_gemm_workspace_bytes(int a_is_dense, int64_t M, int64_t N, int64_t K);

static int gemm_entry(const void* a_dense, int a_dtype, const uint8_t* a_scales, const uint8_t* a_elements, int a_exp_bits,
                      int a_frac_bits, const uint8_t* w_scales, const uint8_t* w_elements, int w_exp_bits, int w_frac_bits,
                      const void* bias, int bias_dtype, void* y, int out_dtype, int64_t M, int64_t N, int64_t K, int block_size,
                      void* workspace, int64_t workspace_bytes, void* stream, int64_t batches = 1, int64_t a_batch_stride = 0,
                      int64_t w_batch_stride = 0, int64_t y_batch_stride = 0) {
    if (M < 0 || N < 1 || K < 1) return fail(ERR_INVALID, "M must not be negative, N and K must be positive");
    if (M == 0) return OK;   // no rows of A: nothing to compute
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
    if (workspace_bytes < 0) return fail(ERR_INVALID, "workspace_bytes must not be negative");
    if (workspace && !aligned(workspace, 16)) return fail(ERR_INVALID, "workspace must be 16-byte aligned");
    if (!workspace) workspace_bytes = 0;
    GemmBatch gb{0, 0, 0, 0};
    if (batches != 1) {
        if (batches < 1 || batches > 65535) return fail(ERR_INVALID, "batches must be between 1 and 65535");
        if (!a_is_dense) return fail(ERR_UNSUPPORTED, "a batched product takes a dense A");
        const int64_t ysz = dtype_size(out_dtype);
        if (a_batch_stride != 0 && a_batch_stride < M * K) return fail(ERR_INVALID, "a_batch_stride must be 0 (A shared by every product) or at least M * K");
        if (w_batch_stride != 0 && w_batch_stride < N * K) return fail(ERR_INVALID, "w_batch_stride must be 0 (W shared by every product) or at least N * K");
        if (y_batch_stride < M * N) return fail(ERR_INVALID, "y_batch_stride must be at least M * N");
        // every product's operands must be aligned like the first one's
        if (a_batch_stride % 8 != 0 || w_batch_stride % 32 != 0 || (y_batch_stride * ysz) % 16 != 0)
            return fail(ERR_INVALID, "batch strides must be multiples of 8 (A), 32 (W) and 16 bytes (y)");
        gb = GemmBatch{a_batch_stride, w_batch_stride / 32, w_batch_stride, y_batch_stride * ysz};
    }
    const GemmArgs g{a_dense, a_scales, a_elements, a_is_dense ? 0 : a_exp_bits, a_frac_bits, w_scales, w_elements, bias, bias_dtype,
                     y, out_dtype, (int)M, (int)N, (int)K, workspace, workspace_bytes, static_cast<hipStream_t>(stream), (int)batches, gb};
    if (w_exp_bits == 4 && w_frac_bits == 3) return gemm_w_e4m3(g);
    if (w_exp_bits == 5 && w_frac_bits == 2) return gemm_w_e5m2(g);
    if (w_exp_bits == 2 && w_frac_bits == 3) return gemm_w_e2m3(g);
    if (w_exp_bits == 3 && w_frac_bits == 2) return gemm_w_e3m2(g);
    if (w_exp_bits == 2 && w_frac_bits == 1) return gemm_w_e2m1(g);
    return fail(ERR_INVALID, "MXFP element (exp_bits, frac_bits) must be one of (4,3) (5,2) (2,3) (3,2) (2,1)");
}

extern "C" int mase_hip_mxfp_gemm(const void* a_dense, int a_dtype, const uint8_t* a_scales, const uint8_t* a_elements,
                                  int a_exp_bits, int a_frac_bits, const uint8_t* w_scales, const uint8_t* w_elements,
                                  int w_exp_bits, int w_frac_bits, const void* bias, int bias_dtype, void* y, int out_dtype,
                                  int64_t M, int64_t N, int64_t K, int block_size, void* stream) {
    return gemm_entry(a_dense, a_dtype, a_scales, a_elements, a_exp_bits, a_frac_bits, w_scales, w_elements, w_exp_bits, w_frac_bits,
                      bias, bias_dtype, y, out_dtype, M, N, K, block_size, nullptr, 0, stream);
}

extern "C" int mase_hip_mxfp_gemm_ws(const void* a_dense, int a_dtype, const uint8_t* a_scales, const uint8_t* a_elements,
                                     int a_exp_bits, int a_frac_bits, const uint8_t* w_scales, const uint8_t* w_elements,
                                     int w_exp_bits, int w_frac_bits, const void* bias, int bias_dtype, void* y, int out_dtype,
                                     int64_t M, int64_t N, int64_t K, int block_size, void* workspace, int64_t workspace_bytes,
                                     void* stream) {
    return gemm_entry(a_dense, a_dtype, a_scales, a_elements, a_exp_bits, a_frac_bits, w_scales, w_elements, w_exp_bits, w_frac_bits,
                      bias, bias_dtype, y, out_dtype, M, N, K, block_size, workspace, workspace_bytes, stream);
}

extern "C" int mase_hip_mxfp_gemm_batched(const void* a_dense, int a_dtype, const uint8_t* w_scales, const uint8_t* w_elements, int w_exp_bits,
                                          int w_frac_bits, void* y, int out_dtype, int64_t M, int64_t N, int64_t K, int block_size,
                                          int64_t batches, int64_t a_batch_stride, int64_t w_batch_stride, int64_t y_batch_stride,
                                          void* stream) {
    if (!a_dense) return fail(ERR_INVALID, "a batched product takes a dense A");
    return gemm_entry(a_dense, a_dtype, nullptr, nullptr, 0, 0, w_scales, w_elements, w_exp_bits, w_frac_bits, nullptr, 0, y, out_dtype, M, N,
                      K, block_size, nullptr, 0, stream, batches, a_batch_stride, w_batch_stride, y_batch_stride);
}

// ---- the same product for callers that cannot allocate: the partial sums of the K split live in a static device array
static __device__ __align__(256) unsigned char scratch[MASE_HIP_STATIC_WORKSPACE_BYTES];

// Device address of `scratch` on the current device (every device has its own copy of the array at its own address),
// looked up once per device.  In host code the array's name is only a handle for this lookup, never an address.
static int static_workspace(void** out) {
    static std::atomic<void*> known[64];
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return fail(ERR_RUNTIME, std::string("hipGetDevice: ") + hipGetErrorString(e));
    if (dev < 0 || dev >= 64) return fail(ERR_UNSUPPORTED, "the static workspace serves device ordinals 0..63");
    void* p = known[dev].load(std::memory_order_acquire);
    if (!p) {
        e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
        if (e != hipSuccess || !p) return fail(ERR_RUNTIME, std::string("hipGetSymbolAddress(scratch): ") + hipGetErrorString(e));
        known[dev].store(p, std::memory_order_release);
    }
    *out = p;
    return OK;
}

extern "C" int mase_hip_mxfp_gemm_static_ws(const void* a_dense, int a_dtype, const uint8_t* a_scales, const uint8_t* a_elements,
                                            int a_exp_bits, int a_frac_bits, const uint8_t* w_scales, const uint8_t* w_elements,
                                            int w_exp_bits, int w_frac_bits, const void* bias, int bias_dtype, void* y, int out_dtype,
                                            int64_t M, int64_t N, int64_t K, int block_size, void* stream) {
    const int64_t need = mase_hip_mxfp_gemm_workspace_bytes(a_dense != nullptr, M, N, K);
    if (need > (int64_t)MASE_HIP_STATIC_WORKSPACE_BYTES)
        return fail(ERR_UNSUPPORTED, "this shape splits K into " + std::to_string(need) + " bytes of partial sums, more than the " +
                                         std::to_string((long long)MASE_HIP_STATIC_WORKSPACE_BYTES) +
                                         " bytes of the static workspace: pass a workspace to mase_hip_mxfp_gemm_ws, or call mase_hip_mxfp_gemm (no split, no workspace)");
    // looked up on every call (one atomic load after the first): the first call on a device, whatever its shape, is the one
    // that may load the code object, so a caller who warms up outside a capture has done it
    void* ws = nullptr;
    if (int rc = static_workspace(&ws)) return rc;
    if (need == 0) ws = nullptr;
    // every split writes all of its [M, N] array before the second kernel reads it: nothing has to start at zero
    return gemm_entry(a_dense, a_dtype, a_scales, a_elements, a_exp_bits, a_frac_bits, w_scales, w_elements, w_exp_bits, w_frac_bits,
                      bias, bias_dtype, y, out_dtype, M, N, K, block_size, ws, ws ? (int64_t)MASE_HIP_STATIC_WORKSPACE_BYTES : 0, stream);
}

extern "C" int64_t mase_hip_mxfp_gemm_workspace_bytes(int a_is_dense, int64_t M, int64_t N, int64_t K) {
    if (!a_is_dense || M < 1 || N < 1 || K < 1 || M > 0x7FFFFFFF || N > 0x7FFFFFFF || K > 0x7FFFFFFF) return 0;
    return plan_split_k((int)M, (int)N, (int)K, device_cu_count()).workspace_bytes((int)M, (int)N);
}
