/*
 * mase_hip.h - C ABI of libmase_hip.so: MXFP / minifloat quantisation and the MXFP GEMM for
 * AMD MI355X (gfx950).
 *
 * The reference (DeepWok/mase-triton) has no FFI of its own: its seam is the Python "kernels"
 * modules that the functional layer calls for GPU tensors.  Every entry point below replaces
 * one of those module functions (cited per function, paths relative to the reference
 * checkout) and takes what that function takes, flattened to plain pointers and sizes.
 *
 * Conventions
 *   - All pointers are DEVICE pointers on the current HIP device, and `stream` (a hipStream_t,
 *     NULL for the default stream) belongs to it: make the device current (hipSetDevice) before
 *     the call.  The library never allocates, frees or synchronises; work is enqueued on
 *     `stream` and the call returns immediately.  Calls may come from several host threads and
 *     for several devices of one process.
 *   - dtype codes:      0 = float32, 1 = float16, 2 = bfloat16   (MASE_F32/F16/BF16)
 *   - round_mode codes: 0 = rn (nearest even), 1 = ru, 2 = rd, 3 = rz
 *   - is_finite != 0: the all-ones exponent is an ordinary binade (the reference's "_fn"
 *     presets); 0: it encodes inf/NaN.
 *   - Element codes: uint16 for minifloat, uint8 (one code per byte, never bit-packed) for MXFP.
 *     MXFP scales: one uint8 biased exponent per block of `block_size` consecutive elements.
 *   - Return value: 0 on success; -1 invalid argument, -2 unsupported combination, -3 HIP
 *     runtime error.  mase_hip_last_error() gives the message of the calling thread's last
 *     failure.
 *   - Inputs are never written.  Buffers must not overlap unless stated.
 */
#ifndef MASE_HIP_H
#define MASE_HIP_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define MASE_F32 0
#define MASE_F16 1
#define MASE_BF16 2

#define MASE_RN 0
#define MASE_RU 1
#define MASE_RD 2
#define MASE_RZ 3

#define MASE_OK 0
#define MASE_ERR_INVALID (-1)
#define MASE_ERR_UNSUPPORTED (-2)
#define MASE_ERR_RUNTIME (-3)

/* ABI version of the loaded library (bumped on any signature change). */
int mase_hip_abi_version(void);

/* Message of the last failure on the calling thread ("" if none). */
const char* mase_hip_last_error(void);

/*
 * x[n] (x_dtype) -> codes[n] (uint16).
 * Replaces extract_minifloat_component(x, minifloat_meta)
 *   src/mase_triton/minifloat/kernels/cast.py:148-170, numerics of minifloat/fake.py:7-78.
 * The reference's functional layer upcasts to float32 first (minifloat/functional/cast.py:27);
 * here the 16-bit dtypes are read directly, which gives the same codes.
 */
int mase_hip_extract_minifloat(const void* x, int x_dtype, uint16_t* codes, int64_t n,
                               int exp_bits, int frac_bits, int is_finite, int round_mode,
                               void* stream);

/*
 * codes[n] (uint16) -> out[n] (out_dtype).
 * Replaces compose_minifloat_component(elements, minifloat_meta, output_dtype)
 *   src/mase_triton/minifloat/kernels/cast.py:263-288, numerics of minifloat/fake.py:81-125.
 */
int mase_hip_compose_minifloat(const uint16_t* codes, void* out, int out_dtype, int64_t n,
                               int exp_bits, int frac_bits, int is_finite, void* stream);

/*
 * out[n] = compose(extract(x[n])) in one pass, codes never stored.  `out` may alias `x` when
 * both dtypes have the same size.
 * Replaces quantize_dequantize(tensor, minifloat_meta, output_dtype)
 *   src/mase_triton/minifloat/functional/cast.py:72-90.
 */
int mase_hip_qdq_minifloat(const void* x, int x_dtype, void* out, int out_dtype, int64_t n,
                           int exp_bits, int frac_bits, int is_finite, int round_mode,
                           void* stream);

/*
 * x[n] -> scales[n / block_size] (uint8), elements[n] (uint8); blocks are consecutive runs of
 * block_size elements of the flat array; n must be a multiple of block_size.
 * Replaces extract_mxfp_components(x, mxfp_meta)
 *   src/mase_triton/mxfp/kernels/cast.py:126-160, numerics of mxfp/fake.py:11-59.
 * (exp_bits, frac_bits) must be one of (4,3) (5,2) (2,3) (3,2) (2,1)  (mxfp/meta.py:21-34);
 * the scale has 8 exponent bits.
 */
int mase_hip_extract_mxfp(const void* x, int x_dtype, uint8_t* scales, uint8_t* elements,
                          int64_t n, int block_size, int exp_bits, int frac_bits, int is_finite,
                          int round_mode, void* stream);

/*
 * scales[n / block_size], elements[n] -> out[n] (out_dtype).
 * Replaces compose_mxfp_tensor(scales, elements, mxfp_meta, output_dtype)
 *   src/mase_triton/mxfp/kernels/cast.py:237-272, numerics of mxfp/fake.py:62-79.
 */
int mase_hip_compose_mxfp(const uint8_t* scales, const uint8_t* elements, void* out,
                          int out_dtype, int64_t n, int block_size, int exp_bits, int frac_bits,
                          int is_finite, void* stream);

/*
 * out[n] = compose(extract(x[n])) in one pass.  `out` may alias `x` when both dtypes have the
 * same size.
 * Replaces quantize_dequantize(tensor, block_dim, mxfp_meta, output_dtype) for a flat,
 * block-contiguous tensor  src/mase_triton/mxfp/functional/cast.py:103-129 (and the activation
 * half of mxfp_linear_XqWq, mxfp/functional/linear.py:50-53).
 */
int mase_hip_qdq_mxfp(const void* x, int x_dtype, void* out, int out_dtype, int64_t n,
                      int block_size, int exp_bits, int frac_bits, int is_finite, int round_mode,
                      void* stream);

/*
 * Blocks along the middle axis of a row-major [outer, k_len, inner] tensor: block b of column
 * (o, i) is x[o, 32*b .. 32*b+31, i].  Same scales and elements, in the same order
 * (scales[outer, inner, k_len/32], elements[outer, inner, k_len]), as permuting the block axis
 * last, copying and calling mase_hip_extract_mxfp, without the copy.
 * Replaces extract_mxfp_components(tensor, block_dim, mxfp_meta) for block_dim other than the last
 * axis  src/mase_triton/mxfp/functional/cast.py:11-44 with its flatten_for_quantize
 * src/mase_triton/mxfp/helpers.py:4-24, as used on `other` by mxfp_matmul
 * src/mase_triton/mxfp/functional/matmul.py:24-29.
 * Needs block_size == 32 and k_len % 32 == 0 (a block never straddles columns), else -2.
 */
int mase_hip_extract_mxfp_strided(const void* x, int x_dtype, uint8_t* scales, uint8_t* elements,
                                  int64_t outer, int64_t k_len, int64_t inner, int block_size,
                                  int exp_bits, int frac_bits, int is_finite, int round_mode,
                                  void* stream);

/*
 * out[outer, k_len, inner] = compose(extract(x)) with blocks along the middle axis, in one pass,
 * written in x's own layout.  `out` may alias `x` when both dtypes have the same size.
 * Replaces quantize_dequantize(tensor, block_dim, ...) for block_dim other than the last axis
 * src/mase_triton/mxfp/functional/cast.py:103-129 (flatten, cast, permute back).
 * Same restrictions as mase_hip_extract_mxfp_strided.
 */
int mase_hip_qdq_mxfp_strided(const void* x, int x_dtype, void* out, int out_dtype, int64_t outer,
                              int64_t k_len, int64_t inner, int block_size, int exp_bits,
                              int frac_bits, int is_finite, int round_mode, void* stream);

/*
 * Storage form of element codes: n codes of `bits` (4 or 6) significant bits, one per byte in `elements`, as a
 * little-endian bit stream in `packed` (code i at bits [bits*i, bits*i + bits); n*bits/8 bytes).  n % 16 == 0;
 * `elements` 16-byte and `packed` 8-byte aligned.  unpack restores exactly the bytes pack read (with the bits above
 * `bits` cleared).
 * No counterpart in the reference, which keeps one byte per code in memory and in state_dict
 * (src/mase_triton/mxfp/layers.py:69-80, src/mase_triton/mxfp/fake.py:71-79); these serve a packed on-disk /
 * at-rest form of a quantised layer.
 */
int mase_hip_pack_codes(const uint8_t* elements, uint8_t* packed, int64_t n, int bits, void* stream);
int mase_hip_unpack_codes(const uint8_t* packed, uint8_t* elements, int64_t n, int bits, void* stream);

/*
 * y[M,N] (out_dtype) = A[M,K] * W[N,K]^T (+ bias[N]), fp32 accumulation on bf16 MFMA.
 *
 *   A: either dense (a_dense != NULL, dtype a_dtype, row-major [M,K], NOT yet quantised: it is
 *      used as is), or MXFP components (a_dense == NULL; a_scales[M*K/block], a_elements[M*K],
 *      blocks along K).  The dense form is the fast one: mxfp_linear quantises its activations to
 *      bfloat16 with mase_hip_qdq_mxfp (exact: MXFP values have at most 4 significant bits) and
 *      passes them dense, which lets every tile kernel stream A straight into LDS.  A in component
 *      form is a compatibility path for callers that hold pre-quantised activations: it always
 *      takes the general 256 x 256 tile kernel (about 0.7 of the dense form's rate on large
 *      shapes) and is never split over K.
 *   W: MXFP components w_scales[N*K/block], w_elements[N*K], blocks along K, as produced by
 *      mase_hip_extract_mxfp on the row-major [N,K] weight.
 *   bias: NULL or bias[N] of dtype bias_dtype, added in fp32 before the output rounding.
 *
 * K must be a multiple of block_size, block_size must be 32, N, K >= 1; M == 0 (no rows of A) is a
 * valid call that does nothing, here and in every GEMM entry point below.
 * Replaces the body of mxfp_linear_XqWq / mxfp_linear_XWq with backend="fused", which the
 * reference leaves unimplemented (src/mase_triton/mxfp/functional/linear.py:31-32,63-64); the
 * result equals the "separate" backend (compose, then torch.nn.functional.linear, :50-61) up
 * to the summation order of the fp32 accumulation.
 */
int mase_hip_mxfp_gemm(const void* a_dense, int a_dtype, const uint8_t* a_scales,
                       const uint8_t* a_elements, int a_exp_bits, int a_frac_bits,
                       const uint8_t* w_scales, const uint8_t* w_elements, int w_exp_bits,
                       int w_frac_bits, const void* bias, int bias_dtype, void* y, int out_dtype,
                       int64_t M, int64_t N, int64_t K, int block_size, void* stream);

/*
 * The same product with room for partial sums.  A product with few output tiles and a long K
 * (say a [256, 4096] output over K = 14336: 64 tiles of 128 x 128 for 256 compute units) runs
 * several times faster when K is split over several workgroups per tile; the splits leave fp32
 * partial sums in `workspace` and a second kernel on the same stream adds them, adds the bias
 * and rounds to out_dtype.  The library allocates nothing, so the caller brings the memory:
 *
 *   mase_hip_mxfp_gemm_workspace_bytes(a_is_dense, M, N, K)
 *       bytes with which this shape would be split on the current device, 0 if it would not
 *       (MXFP A, enough tiles, short K, sizes the split kernel does not take).
 *   mase_hip_mxfp_gemm_ws(..., workspace, workspace_bytes, stream)
 *       `workspace`: 16-byte aligned device memory of at least that many bytes, or NULL.  With
 *       NULL, or fewer bytes than the shape asks for, the call is mase_hip_mxfp_gemm.  The
 *       contents before the call do not matter and are undefined after it; calls that share
 *       a workspace must be ordered on one stream.
 *
 * The result differs from mase_hip_mxfp_gemm's only in the order of the fp32 additions.
 * Same reference counterpart as mase_hip_mxfp_gemm (src/mase_triton/mxfp/functional/linear.py:
 * 31-32,50-64); the reference has no workspace argument because its GEMM is torch's, which
 * allocates its own.
 */
int64_t mase_hip_mxfp_gemm_workspace_bytes(int a_is_dense, int64_t M, int64_t N, int64_t K);
int mase_hip_mxfp_gemm_ws(const void* a_dense, int a_dtype, const uint8_t* a_scales,
                          const uint8_t* a_elements, int a_exp_bits, int a_frac_bits,
                          const uint8_t* w_scales, const uint8_t* w_elements, int w_exp_bits,
                          int w_frac_bits, const void* bias, int bias_dtype, void* y,
                          int out_dtype, int64_t M, int64_t N, int64_t K, int block_size,
                          void* workspace, int64_t workspace_bytes, void* stream);

/*
 * `batches` products in one launch: y_b[M,N] = A_b[M,K] * W_b[N,K]^T for b = 0 .. batches-1, with A_b, the components of
 * W_b and y_b lying a_batch_stride, w_batch_stride and y_batch_stride ELEMENTS after those of product b-1 (the scales
 * of W_b: w_batch_stride / 32 bytes).  A stride of 0 shares that operand between all products (a_batch_stride = 0: one
 * A against many weights; w_batch_stride = 0: equivalent to one product with batches * M rows when the A_b are
 * contiguous).  A is dense bfloat16; no bias; K is never split (no workspace).  Strides must be multiples of 8 (A),
 * 32 (W) and 16 bytes (y) so that every product's operands are aligned like the first one's; batches <= 65535.
 * Replaces the torch.matmul over leading batch axes at the end of mxfp_matmul
 *   src/mase_triton/mxfp/functional/matmul.py:24-35
 * (with `other` already extracted along its second-to-last axis into [.., N, K] order by
 * mase_hip_extract_mxfp_strided, and `input` quantised by mase_hip_qdq_mxfp); the reference's 4-D use is
 * test/test_mxfp_functional.py:229-230.
 */
int mase_hip_mxfp_gemm_batched(const void* a_dense, int a_dtype, const uint8_t* w_scales,
                               const uint8_t* w_elements, int w_exp_bits, int w_frac_bits, void* y,
                               int out_dtype, int64_t M, int64_t N, int64_t K, int block_size,
                               int64_t batches, int64_t a_batch_stride, int64_t w_batch_stride,
                               int64_t y_batch_stride, void* stream);

/*
 * The same product as mase_hip_mxfp_gemm_ws for callers that cannot allocate device memory at all (code under HIP
 * graph capture, tight serving loops, harnesses that forbid hipMalloc): the partial sums of the K split live in a
 * device array that is part of the library image, MASE_HIP_STATIC_WORKSPACE_BYTES on every GPU the library runs on,
 * held until the process ends.  The call allocates and frees nothing.  A shape whose split asks for more
 * (mase_hip_mxfp_gemm_workspace_bytes; on a 256-CU device the largest request of any shape is 64 MiB, made by 512-row
 * tiles split two to four ways, e.g. [1024, 4096] over K = 14336) is refused with -2: pass your own workspace to
 * mase_hip_mxfp_gemm_ws then, or call mase_hip_mxfp_gemm, which does not split and needs none.
 * A shape that is not split does not touch the array.
 * Every call on a GPU shares that GPU's array, which keeps the last call's partial sums (nothing in it has to start
 * at zero): calls on one GPU must be ordered on one stream, calls that overlap there race.  The first call on a
 * device looks up the array's address (it loads the library's code object there if nothing has yet): make it once
 * outside any stream capture.
 * No counterpart in the reference, whose GEMM is torch's and allocates its own workspace; it exists for the callers
 * above, those that cannot allocate.
 */
#define MASE_HIP_STATIC_WORKSPACE_BYTES (32 * 1024 * 1024)
int mase_hip_mxfp_gemm_static_ws(const void* a_dense, int a_dtype, const uint8_t* a_scales,
                                 const uint8_t* a_elements, int a_exp_bits, int a_frac_bits,
                                 const uint8_t* w_scales, const uint8_t* w_elements, int w_exp_bits,
                                 int w_frac_bits, const void* bias, int bias_dtype, void* y,
                                 int out_dtype, int64_t M, int64_t N, int64_t K, int block_size,
                                 void* stream);

/*
 * ---- The same product on the block-scaled matrix instruction (v_mfma_scale_f32_16x16x128_f8f6f4).
 *
 * Both operands stay MXFP up to the matrix unit: FP8 (E4M3) bytes and one E8M0 scale per 32 elements along K, which
 * the instruction applies itself; products are exact and accumulate in fp32.  Nothing is composed to bfloat16, so
 * an operand byte costs half the LDS and cache traffic of the bf16 kernels and the instruction runs at twice the
 * bf16 rate.  The operands are handed over in a prepared form, built by one of two calls:
 *
 *   mase_hip_scaled_operand_from_dense(x, BF16, E, M, rows, K, out_codes, out_scales, stream)
 *       extract of the row-major [rows, K] bfloat16 matrix x (blocks of 32 along K, element format (E, M), finite,
 *       round to nearest: what mase_hip_extract_mxfp computes) written straight into the prepared form;
 *   mase_hip_scaled_operand_from_mxfp(scales, elements, E, M, rows, K, out_codes, out_scales, stream)
 *       the same from MXFP components in the reference's layout (scales[rows * K / 32], elements[rows * K]).
 *
 * Prepared form: out_codes [rows_pad, K] bytes, out_scales [K / 128, rows_pad] dwords, rows_pad =
 * mase_hip_scaled_padded_rows(rows) (the next multiple of 256; rows past `rows` are never written and may hold
 * anything).  Byte (k / 32) % 4 of dword [k / 128][row] is the scale of block k / 32 of that row.  Element formats
 * (2,1) (2,3) (3,2) are embedded into E4M3 bytes of the same value under the same scale (exact).  E4M3 itself: the
 * matrix unit reads the code S.1111.111 as NaN where the reference has +-480, so a block that holds it is stored one
 * scale step up with every code halved.  That is exact except for a block's odd codes below 16 (elements 2^13 and
 * more below the block's largest), which round half to even: a change of at most 2^-14 of the block's largest
 * element.  E5M2 is not taken (-2): every block of it reaches the binade the matrix unit reads as inf / NaN.
 * A block with scale byte 255 (it held inf or NaN) makes its row of the product NaN, as in the reference whenever
 * the block also holds a zero code (always, unless all 32 inputs were inf / NaN).
 *
 *   mase_hip_mxfp_gemm_scaled(a_codes, a_scales, w_codes, w_scales, bias, bias_dtype, y, out_dtype, M, N, K, stream)
 *       y[M,N] = A[M,K] * W[N,K]^T (+ bias), A and W prepared as above with rows M and N.
 *
 * K % 256 == 0 and K >= 512; N a multiple of 8 (4 for fp32 output); codes and y 16-byte aligned.  Other shapes: -2,
 * use mase_hip_mxfp_gemm.  Up to 64 rows of A take weight-streaming kernels (the product is a read of W; 17 - 64 rows
 * against a K beyond 4096 only through mase_hip_mxfp_gemm_scaled_ws, which brings the room for their K slices' sums),
 * more rows 256 x 256 tiles.
 * Replaces, like mase_hip_mxfp_gemm, the unimplemented backend="fused" of mxfp_linear_XqWq
 *   src/mase_triton/mxfp/functional/linear.py:36-64
 * (extract of x :50-52, the two composes :53-54 and the linear :61 in one prepare call and one GEMM).
 */
int64_t mase_hip_scaled_padded_rows(int64_t rows);
int mase_hip_scaled_operand_from_dense(const void* x, int x_dtype, int exp_bits, int frac_bits, int64_t rows,
                                       int64_t K, uint8_t* out_codes, uint32_t* out_scales, void* stream);
int mase_hip_scaled_operand_from_mxfp(const uint8_t* scales, const uint8_t* elements, int exp_bits,
                                      int frac_bits, int64_t rows, int64_t K, uint8_t* out_codes,
                                      uint32_t* out_scales, void* stream);
/*
 * The activations of a minifloat linear layer as an operand of the same GEMM: every element of the row-major [rows, K]
 * bfloat16 matrix x is rounded by itself to the minifloat format (E, M) (finite, round to nearest: the codes of
 * mase_hip_extract_minifloat, one byte each) and every block carries the scale 2^0, under which a minifloat code is an
 * MXFP element of the same value.  The weight codes of such a layer go through mase_hip_scaled_operand_from_mxfp with
 * scale bytes of 127.  Formats and the E4M3 re-encoding as above.
 * Replaces, with mase_hip_mxfp_gemm_scaled, the unimplemented backend="fused" of minifloat_linear_XqWq
 *   src/mase_triton/minifloat/functional/linear.py:33-58
 * (extract and compose of x :45-46, compose of W :47 and the linear :55 in one prepare call and one GEMM).
 */
int mase_hip_scaled_operand_from_dense_minifloat(const void* x, int x_dtype, int exp_bits, int frac_bits,
                                                 int64_t rows, int64_t K, uint8_t* out_codes,
                                                 uint32_t* out_scales, void* stream);
/*
 * The activations of the down projection of a SwiGLU block, quantised where they are formed: the matrix that is
 * extracted is silu(gate) * up (gate, up: row-major [rows, K] bfloat16 with a common row stride of `row_stride`
 * elements, e.g. the two halves of a stacked gate / up projection's output, row_stride = 2 K), each of the two
 * operations rounded to bfloat16 as a tensor library rounds it; the bfloat16 product itself is never stored.
 * No counterpart in the reference, where the caller writes  down(silu(gate(x)) * up(x))  between two MXFPLinearPTQ
 * layers (src/mase_triton/mxfp/layers.py:150-165 is the layer's forward) and the extract of
 * src/mase_triton/mxfp/functional/linear.py:50-52 then reads the product back from memory.
 */
int mase_hip_scaled_operand_from_swiglu(const void* gate, const void* up, int dtype, int64_t row_stride,
                                        int exp_bits, int frac_bits, int64_t rows, int64_t K,
                                        uint8_t* out_codes, uint32_t* out_scales, void* stream);
int mase_hip_mxfp_gemm_scaled(const uint8_t* a_codes, const uint32_t* a_scales, const uint8_t* w_codes,
                              const uint32_t* w_scales, const void* bias, int bias_dtype, void* y,
                              int out_dtype, int64_t M, int64_t N, int64_t K, void* stream);
/*
 * The same with room for partial sums, as mase_hip_mxfp_gemm_ws: a product with few 256 x 256 tiles and a long K, or with
 * 17 - 64 rows of A and a K beyond 4096, is split over K into fp32 partial sums in `workspace` (mase_hip_mxfp_gemm_scaled_workspace_bytes(M, N, K) bytes, 0 when
 * the shape is not split; 16-byte aligned; NULL or too small: no split), and a second kernel adds them, the bias, and
 * rounds.  Same reference counterpart as mase_hip_mxfp_gemm_scaled.
 */
int64_t mase_hip_mxfp_gemm_scaled_workspace_bytes(int64_t M, int64_t N, int64_t K);
int mase_hip_mxfp_gemm_scaled_ws(const uint8_t* a_codes, const uint32_t* a_scales, const uint8_t* w_codes,
                                 const uint32_t* w_scales, const void* bias, int bias_dtype, void* y,
                                 int out_dtype, int64_t M, int64_t N, int64_t K, void* workspace,
                                 int64_t workspace_bytes, void* stream);

/*
 * The whole XqWq linear in one call for a caller that keeps W in the prepared form: the operand of x
 * (mase_hip_scaled_operand_from_dense, or ..._from_dense_minifloat when x_is_minifloat != 0) built in `scratch`, then
 * mase_hip_mxfp_gemm_scaled_ws with the rest of `scratch` as its workspace.  `scratch`: 256-byte aligned,
 * mase_hip_mxfp_linear_scaled_scratch_bytes(M, N, K) bytes (the operand of x plus whatever the product's K split asks
 * for; with less than the operand: -1, with the operand alone: no split).  Nothing in it has to survive the call.
 * A decode-sized product takes less time on the GPU than two calls through a binding take on the host; this is
 * the one call.  Shapes, formats and results as of the two calls it makes.
 * Replaces the body of mxfp_linear_XqWq / minifloat_linear_XqWq with backend="fused"
 *   src/mase_triton/mxfp/functional/linear.py:36-64, src/mase_triton/minifloat/functional/linear.py:33-58.
 */
int64_t mase_hip_mxfp_linear_scaled_scratch_bytes(int64_t M, int64_t N, int64_t K);
int mase_hip_mxfp_linear_scaled(const void* x, int x_dtype, int x_exp_bits, int x_frac_bits, int x_is_minifloat,
                                const uint8_t* w_codes, const uint32_t* w_scales, const void* bias,
                                int bias_dtype, void* y, int out_dtype, int64_t M, int64_t N, int64_t K,
                                void* scratch, int64_t scratch_bytes, void* stream);

/*
 * y[M,N] = A[M,K] * W[N,K]^T (+ bias) with a DENSE bfloat16 A (used as is, like a_dense of mase_hip_mxfp_gemm) and W in
 * the prepared form above (mase_hip_scaled_operand_from_mxfp with rows = N), on the bf16 matrix instruction: the
 * 512 x 128 tile kernel of mase_hip_mxfp_gemm composing W to bfloat16 in registers, with what the prepared form saves it
 * (one convert per pair of codes, because no byte holds the code the convert reads as NaN; the scales of a 128-k step
 * of 128 rows as 512 contiguous bytes).  For layers that keep the prepared weight anyway and whose activations are not
 * quantised (layer types XWq*) or are quantised to a format the block-scaled GEMM does not take.
 * M >= 512, N % 128 == 0, K % 128 == 0, else -2 (use mase_hip_mxfp_gemm with the components).
 * Replaces the body of mxfp_linear_XWq with backend="fused"  src/mase_triton/mxfp/functional/linear.py:10-33.
 */
int mase_hip_mxfp_gemm_prepared_w(const void* a_dense, int a_dtype, const uint8_t* w_codes,
                                  const uint32_t* w_scales, const void* bias, int bias_dtype, void* y,
                                  int out_dtype, int64_t M, int64_t N, int64_t K, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* MASE_HIP_H */
