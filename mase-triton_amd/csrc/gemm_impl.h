// Dequant-fused MXFP GEMM for gfx950:  y[M,N] = A[M,K] * W[N,K]^T (+ bias), fp32 accumulation
// on v_mfma_f32_32x32x16_bf16.
//
// W (and optionally A) arrive as MXFP components: one uint8 code per element, one uint8 scale
// per 32 elements along K.  A workgroup owns a TM x TN tile of y.  Per K-step it stages a
// TM x TK slab of A and a TN x TK slab of W in LDS as bf16; MXFP operands are composed to bf16
// in registers on the way (code -> fp16 by field placement, -> fp32, times 2^(scale - bias'),
// -> bf16; exact, every MXFP value has at most 4 significant bits).  LDS is double buffered:
// while the MFMAs consume slab k, slab k+1 (already in registers) is composed and written to the
// other buffer and the global loads of slab k+2 are in flight; one barrier per K-step.
//
// MFMA operand layout (wave64): lane l supplies row l%32 of the first operand / column l%32 of
// the second and the 8 consecutive k values starting at 8*(l/32); accumulator register v of
// lane l is D[8*(v/4) + 4*(l/32) + v%4][l%32].  W is fed as the FIRST operand, so a lane ends
// up with runs of 4 consecutive n for one m and can store 8 contiguous bytes of bf16 output.
#pragma once
#include "../../include/mase_hip.h"
#include "mase_host.h"
#include "mxfp_compose.h"

namespace mase {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float floatx16 __attribute__((ext_vector_type(16)));

// Offsets between consecutive products of a batched launch (grid plane z = product z): elements of A, bytes of the W
// scales, of the W codes and of y.  All zero for a single product; an operand shared by every product has offset 0.
struct GemmBatch {
    int64_t a, ws, we, y;
};

// Workgroup barrier that orders LDS traffic only.  __syncthreads() also fences global memory, which
// would make every wave wait for its outstanding output stores; here those are meant to drain in
// the background while the next tile starts.
__device__ inline void lds_barrier() {
    __builtin_amdgcn_s_waitcnt(0xC07F);  // lgkmcnt(0): this wave's LDS reads and writes are done
    __builtin_amdgcn_s_barrier();
}

__device__ inline float load_bias(const void* bias, int bias_dtype, int col) {
    if (bias_dtype == F32) return static_cast<const float*>(bias)[col];
    const uint32_t h = static_cast<const uint16_t*>(bias)[col];
    return bits_f32(bias_dtype == BF16 ? h << 16 : half_bits_to_f32_bits(h));
}

template <int DT_OUT>
__device__ inline void store_out(void* y, int64_t o, float r) {
    if (DT_OUT == F32) static_cast<float*>(y)[o] = r;
    else if (DT_OUT == BF16) static_cast<uint16_t*>(y)[o] = (uint16_t)(cvt_pk_bf16(r, 0.0f) & 0xFFFFu);
    else static_cast<uint16_t*>(y)[o] = (uint16_t)f32_bits_to_half_bits(f32_bits(r));
}

// 4 consecutive outputs of one row, starting at a column that is a multiple of 4
template <int DT_OUT>
__device__ inline void store_out4(void* y, int64_t o, const float (&r)[4], bool vec_ok, int valid) {
    if (vec_ok && valid == 4) {
        if (DT_OUT == F32) *reinterpret_cast<float4*>(static_cast<float*>(y) + o) = make_float4(r[0], r[1], r[2], r[3]);
        else if (DT_OUT == BF16)
            *reinterpret_cast<uint2*>(static_cast<uint16_t*>(y) + o) = make_uint2(cvt_pk_bf16(r[0], r[1]), cvt_pk_bf16(r[2], r[3]));
        else
            *reinterpret_cast<uint2*>(static_cast<uint16_t*>(y) + o) =
                make_uint2(f32_bits_to_half_bits(f32_bits(r[0])) | (f32_bits_to_half_bits(f32_bits(r[1])) << 16),
                           f32_bits_to_half_bits(f32_bits(r[2])) | (f32_bits_to_half_bits(f32_bits(r[3])) << 16));
    } else {
        for (int t = 0; t < valid; ++t) store_out<DT_OUT>(y, o + t, r[t]);
    }
}

// ---------------------------------------------------------------------------------------------
// Main kernel: 256 x 256 x 64 tiles, 4 waves (2 x 2), each wave 128 x 128 = 4 x 4 MFMA tiles.
// ---------------------------------------------------------------------------------------------
constexpr int TM = 256, TN = 256, TK = 64;
constexpr int kGemmThreads = 256;
constexpr int ROW_BYTES = TK * 2 + 16;  // 144: rows 16 B apart modulo 256 -> conflict-free 128-bit reads
constexpr int SLAB_BYTES = TM * ROW_BYTES;  // one operand, one buffer (TM == TN)

// A_MODE: 0 = dense bf16 A, 1 = MXFP A (format FA).  W is always MXFP (format FW).
template <int A_MODE, class FA, class FW, int DT_OUT, bool GUARD_K>
__global__ __launch_bounds__(kGemmThreads) __attribute__((amdgpu_waves_per_eu(1, 1))) void mxfp_gemm_kernel(
    const uint16_t* __restrict__ a_dense0, const uint8_t* __restrict__ a_scales, const uint8_t* __restrict__ a_elements,
    const uint8_t* __restrict__ w_scales0, const uint8_t* __restrict__ w_elements0, const void* __restrict__ bias,
    int bias_dtype, void* __restrict__ y0, int M, int N, int K, int tiles_m, int tiles_n, GemmBatch gb) {
    extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
    // batched launches: workgroups of grid plane z work on product z (offsets are zero for a single product)
    const uint16_t* __restrict__ const a_dense = a_dense0 + (int64_t)blockIdx.z * gb.a;
    const uint8_t* __restrict__ const w_scales = w_scales0 + (int64_t)blockIdx.z * gb.ws;
    const uint8_t* __restrict__ const w_elements = w_elements0 + (int64_t)blockIdx.z * gb.we;
    void* __restrict__ const y = static_cast<uint8_t*>(y0) + (int64_t)blockIdx.z * gb.y;
    uint8_t* const lds_a = lds;                    // [2][TM][ROW_BYTES]
    uint8_t* const lds_w = lds + 2 * SLAB_BYTES;   // [2][TN][ROW_BYTES]

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wave_m = wave >> 1, wave_n = wave & 1;

    // Persistent workgroups: the grid is one workgroup per CU (a multiple of 8) and each walks a list
    // of tiles, so a tile's output stores drain while the next tile is already loading.
    // Tile order.  Workgroup ids are dealt round-robin to the 8 XCDs, each with its own L2, so XCD x
    // owns the contiguous range of positions [x * per_xcd, (x+1) * per_xcd) and its workgroups take
    // them in turn; positions walk the tile grid in groups of 4 tile-rows, rows fastest, so the tiles
    // an XCD runs at once form a 4 x 8 patch that shares 4 A slabs and 8 W slabs through that L2.
    const int n_tiles = tiles_m * tiles_n;
    const int per_xcd = (n_tiles + 7) >> 3;
    const int slots = gridDim.x >> 3;
    for (int local = blockIdx.x >> 3; local < per_xcd; local += slots) {
    const int pos = (blockIdx.x & 7) * per_xcd + local;
    if (pos >= n_tiles) break;
    int tile_m, tile_n;
    {
        constexpr int GROUP = 4;
        const int in_group = GROUP * tiles_n;
        const int first_m = (pos / in_group) * GROUP;
        const int rows = min(tiles_m - first_m, GROUP);
        const int r = pos % in_group;
        tile_m = first_m + r % rows;
        tile_n = r / rows;
    }
    const int m0 = tile_m * TM, n0 = tile_n * TN;
    const int kblocks = K / 32;
    const int ksteps = (K + TK - 1) / TK;  // K % 32 == 0; a last half step is zero-filled

    // ---- global -> register staging assignment, in 4 parts (one per MFMA phase of a K-step)
    // dense A: 8 lanes cover one 128-byte row slab; load j (0..7) takes row j*32 + tid/8; part p owns j = 2p, 2p+1
    // MXFP operands: 4 lanes cover one 64-code row slab; load j (0..3) takes row j*64 + tid/4; part p owns j = p
    const int a_chunk = tid & 7, a_row0 = tid >> 3;
    const int c_chunk = tid & 3, c_row0 = tid >> 2;
    const int last_step = ksteps - 1;

    uint4 ra[A_MODE == 0 ? 8 : 4];
    uint4 rw[4];
    uint32_t sa[4], sw[4];

    // Rows past the matrix edge are clamped to the last row: they only feed outputs that are never
    // stored.  Offsets are 32-bit (the host checks the operand sizes) and constant over the K loop;
    // the slab's k0 is folded into a uniform base pointer.
    uint32_t a_off[A_MODE == 0 ? 8 : 4], as_off[4], w_off[4], ws_off[4];
#pragma unroll
    for (int j = 0; j < (A_MODE == 0 ? 8 : 4); ++j) {
        if (A_MODE == 0) {
            const int row = min(m0 + j * 32 + a_row0, M - 1);
            a_off[j] = ((uint32_t)row * (uint32_t)K + a_chunk * 8) * 2u;
        } else {
            const int row = min(m0 + j * 64 + c_row0, M - 1);
            a_off[j] = (uint32_t)row * (uint32_t)K + c_chunk * 16;
            as_off[j] = (uint32_t)row * (uint32_t)kblocks + (c_chunk >> 1);
        }
    }
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const int row = min(n0 + j * 64 + c_row0, N - 1);
        w_off[j] = (uint32_t)row * (uint32_t)K + c_chunk * 16;
        ws_off[j] = (uint32_t)row * (uint32_t)kblocks + (c_chunk >> 1);
    }
    const uint8_t* const a_bytes = A_MODE == 0 ? reinterpret_cast<const uint8_t*>(a_dense) : a_elements;

    auto fetch_part = [&](int p, int kt) {
        const int ktc = kt < last_step ? kt : last_step;  // past the end: reload the last slab (never used)
        const bool k_ok = !GUARD_K || ktc * TK + c_chunk * 16 < K;  // only a trailing half slab can fail
        if (A_MODE == 0) {
            const uint8_t* const base = a_bytes + (size_t)ktc * (TK * 2);
            const bool ak_ok = !GUARD_K || ktc * TK + a_chunk * 8 < K;
#pragma unroll
            for (int jj = 0; jj < 2; ++jj) {
                const int j = 2 * p + jj;
                // a chunk past K is never dereferenced: its address could lie beyond the last row
                ra[j] = ak_ok ? *reinterpret_cast<const uint4*>(base + a_off[j]) : make_uint4(0, 0, 0, 0);
            }
        } else {
            ra[p] = k_ok ? *reinterpret_cast<const uint4*>(a_bytes + (size_t)ktc * TK + a_off[p]) : make_uint4(0, 0, 0, 0);
            sa[p] = k_ok ? (a_scales + (size_t)ktc * (TK / 32))[as_off[p]] : 0u;
        }
        rw[p] = k_ok ? *reinterpret_cast<const uint4*>(w_elements + (size_t)ktc * TK + w_off[p]) : make_uint4(0, 0, 0, 0);
        sw[p] = k_ok ? (w_scales + (size_t)ktc * (TK / 32))[ws_off[p]] : 0u;
    };

    auto stage_part = [&](auto safe, int p, int buf) {
        constexpr bool SAFE = decltype(safe)::value;
        uint8_t* const pa = lds_a + buf * SLAB_BYTES;
        uint8_t* const pw = lds_w + buf * SLAB_BYTES;
        if (A_MODE == 0) {
#pragma unroll
            for (int jj = 0; jj < 2; ++jj) {
                const int j = 2 * p + jj;
                *reinterpret_cast<uint4*>(pa + (j * 32 + a_row0) * ROW_BYTES + a_chunk * 16) = ra[j];
            }
        } else {
            uint4 lo, hi;
            Composer<FA>::template compose16<SAFE>(ra[p], sa[p], lo, hi);
            uint4* q = reinterpret_cast<uint4*>(pa + (p * 64 + c_row0) * ROW_BYTES + c_chunk * 32);
            q[0] = lo; q[1] = hi;
        }
        {
            uint4 lo, hi;
            Composer<FW>::template compose16<SAFE>(rw[p], sw[p], lo, hi);
            uint4* q = reinterpret_cast<uint4*>(pw + (p * 64 + c_row0) * ROW_BYTES + c_chunk * 32);
            q[0] = lo; q[1] = hi;
        }
    };

    floatx16 acc[4][4];  // [n-tile j][m-tile i]
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
        for (int i = 0; i < 4; ++i)
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[j][i][v] = 0.0f;

    const int frag_off = (lane & 31) * ROW_BYTES + (lane >> 5) * 16;  // the lane's row and its 8 k values
    const uint8_t* const frag_a = lds_a + wave_m * 128 * ROW_BYTES + frag_off;
    const uint8_t* const frag_w = lds_w + wave_n * 128 * ROW_BYTES + frag_off;
    auto load_frags = [&](int buf, int ks, bf16x8 (&af)[4], bf16x8 (&wf)[4]) {
#pragma unroll
        for (int i = 0; i < 4; ++i) af[i] = *reinterpret_cast<const bf16x8*>(frag_a + buf * SLAB_BYTES + i * 32 * ROW_BYTES + ks * 32);
#pragma unroll
        for (int j = 0; j < 4; ++j) wf[j] = *reinterpret_cast<const bf16x8*>(frag_w + buf * SLAB_BYTES + j * 32 * ROW_BYTES + ks * 32);
    };
    auto mfma16 = [&](const bf16x8 (&af)[4], const bf16x8 (&wf)[4]) {
#pragma unroll
        for (int j = 0; j < 4; ++j)
#pragma unroll
            for (int i = 0; i < 4; ++i) acc[j][i] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(wf[j], af[i], acc[j][i], 0, 0, 0);
    };
    // one MFMA, then a slice of the phase's other work: keeps the matrix pipe fed while the
    // vector ALU composes, the LDS is read and written and the next global loads are issued
    auto interleave = [&]() {
#pragma unroll
        for (int i = 0; i < 16; ++i) {
            __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);   // MFMA
            if (i < 8) __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);  // DS read
            __builtin_amdgcn_sched_group_barrier(0x002, 7, 0);   // VALU
            if (i >= 8 && i < 12) __builtin_amdgcn_sched_group_barrier(0x200, 1, 0);  // DS write
            if (i >= 12) __builtin_amdgcn_sched_group_barrier(0x020, 1, 0);  // VMEM read
        }
    };

    // ---- does any scale this tile will read need the slow compose (255, a block that held inf/NaN, or nearly)?  Decided once per
    //      tile so that the K loop itself carries no test: thread t scans the scale row of W row
    //      n0 + t (and of A row m0 + t when A is MXFP).
    bool saw_slow = false;
    {
        const uint8_t* const wr = w_scales + (size_t)min(n0 + tid, N - 1) * kblocks;
        for (int b = 0; b < kblocks; ++b) saw_slow |= Composer<FW>::is_slow(wr[b]);
        if (A_MODE == 1) {
            const uint8_t* const ar = a_scales + (size_t)min(m0 + tid, M - 1) * kblocks;
            for (int b = 0; b < kblocks; ++b) saw_slow |= Composer<FA>::is_slow(ar[b]);
        }
    }
    const bool tile_has_slow = __syncthreads_or(saw_slow) != 0;

    auto run_tile = [&](auto safe) {
    // ---- prologue: slab 0 complete in LDS[0], part 0 of slab 1 in LDS[1]; registers hold parts
    //      1..3 of slab 1 and part 0 of slab 2
#pragma unroll
    for (int p = 0; p < 4; ++p) fetch_part(p, 0);
#pragma unroll
    for (int p = 0; p < 4; ++p) stage_part(safe, p, 0);
#pragma unroll
    for (int p = 0; p < 4; ++p) fetch_part(p, 1);
    stage_part(safe, 0, 1);
    fetch_part(0, 2);
    lds_barrier();

    bf16x8 fa0[4], fw0[4], fa1[4], fw1[4];
    load_frags(0, 0, fa0, fw0);

    // ---- main loop.  Step kt multiplies slab kt (LDS[cur]).  Its phases 0..2 finish staging slab
    //      kt+1 into LDS[nxt]; after the barrier LDS[cur] is free and phase 3 starts staging slab kt+2.
    //      Each register part is refilled from global memory right after it has been staged, one
    //      whole K-step before it is needed again.
    for (int kt = 0; kt < ksteps; ++kt) {
        const int cur = kt & 1, nxt = cur ^ 1;
        load_frags(cur, 1, fa1, fw1);
        mfma16(fa0, fw0);
        stage_part(safe, 1, nxt);
        fetch_part(1, kt + 2);
        interleave();
        __builtin_amdgcn_sched_barrier(0);

        load_frags(cur, 2, fa0, fw0);
        mfma16(fa1, fw1);
        stage_part(safe, 2, nxt);
        fetch_part(2, kt + 2);
        interleave();
        __builtin_amdgcn_sched_barrier(0);

        load_frags(cur, 3, fa1, fw1);
        mfma16(fa0, fw0);
        stage_part(safe, 3, nxt);
        fetch_part(3, kt + 2);
        interleave();
        __builtin_amdgcn_sched_barrier(0);

        lds_barrier();

        load_frags(nxt, 0, fa0, fw0);
        mfma16(fa1, fw1);
        stage_part(safe, 0, cur);
        fetch_part(0, kt + 3);
        interleave();
        __builtin_amdgcn_sched_barrier(0);
    }

    };
    if (tile_has_slow) run_tile(IntC<1>{});
    else run_tile(IntC<0>{});

    // ---- epilogue: lane holds, for tile (j, i) and g = 0..3, y[m][n .. n+3] with
    //      m = m0 + wave_m*128 + i*32 + lane%32,  n = n0 + wave_n*128 + j*32 + 8*g + 4*(lane/32)
    const bool vec_ok = (N % 4 == 0) && (reinterpret_cast<uintptr_t>(y) & 15) == 0;
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
        for (int g = 0; g < 4; ++g) {
            const int n = n0 + wave_n * 128 + j * 32 + 8 * g + 4 * (lane >> 5);
            const int valid = N - n >= 4 ? 4 : (N - n > 0 ? N - n : 0);
            float b[4] = {0.0f, 0.0f, 0.0f, 0.0f};
            if (bias)
                for (int t = 0; t < valid; ++t) b[t] = load_bias(bias, bias_dtype, n + t);
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const int m = m0 + wave_m * 128 + i * 32 + (lane & 31);
                if (m >= M || valid == 0) continue;
                const float r[4] = {acc[j][i][4 * g] + b[0], acc[j][i][4 * g + 1] + b[1], acc[j][i][4 * g + 2] + b[2],
                                    acc[j][i][4 * g + 3] + b[3]};
                store_out4<DT_OUT>(y, (int64_t)m * N + n, r, vec_ok, valid);
            }
        }
    lds_barrier();  // nobody may still be reading this tile's last slabs when the next tile stages
    }  // tile loop
}

#include "gemm_tall.h"
#include "gemm_skinny.h"
#include "gemm_rows16.h"
#include "gemm_mid.h"
#include "gemm_wide.h"
#include "gemm_split_k.h"
#include "gemm_scaled.h"

// ---------------------------------------------------------------------------------------------
// Small-shape kernel: 128 x 128 x 32 tiles, single LDS buffer.  Used when the problem cannot
// fill the chip with 256 x 256 tiles.
// ---------------------------------------------------------------------------------------------
constexpr int SBM = 128, SBN = 128, SBK = 32;
constexpr int S_STRIDE = SBK + 8;  // bf16 elements per tile row: 80 bytes

template <int A_MODE, class FA, class FW, int DT_OUT>
__global__ __launch_bounds__(kGemmThreads) void mxfp_gemm_small_kernel(
    const uint16_t* __restrict__ a_dense0, const uint8_t* __restrict__ a_scales, const uint8_t* __restrict__ a_elements,
    const uint8_t* __restrict__ w_scales0, const uint8_t* __restrict__ w_elements0, const void* __restrict__ bias,
    int bias_dtype, void* __restrict__ y0, int M, int N, int K, GemmBatch gb) {
    // batched launches: workgroups of grid plane z work on product z (offsets are zero for a single product)
    const uint16_t* __restrict__ const a_dense = a_dense0 + (int64_t)blockIdx.z * gb.a;
    const uint8_t* __restrict__ const w_scales = w_scales0 + (int64_t)blockIdx.z * gb.ws;
    const uint8_t* __restrict__ const w_elements = w_elements0 + (int64_t)blockIdx.z * gb.we;
    void* __restrict__ const y = static_cast<uint8_t*>(y0) + (int64_t)blockIdx.z * gb.y;
    __shared__ __attribute__((aligned(16))) uint16_t lds_a[SBM * S_STRIDE];
    __shared__ __attribute__((aligned(16))) uint16_t lds_w[SBN * S_STRIDE];

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wave_m = wave >> 1, wave_n = wave & 1;  // 2 x 2 waves, 64 x 64 each
    const int m0 = blockIdx.y * SBM, n0 = blockIdx.x * SBN;
    const int kblocks = K / 32;

    const int srow = tid >> 1, shalf = tid & 1;  // thread stages tile row tid/2, 16 k values
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
        const int64_t k = (int64_t)kt * SBK + shalf * 16;
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

    const int ktiles = K / SBK;
    fetch(0);
    for (int kt = 0; kt < ktiles; ++kt) {
        __syncthreads();  // everyone finished reading the previous slab
        {
            uint4 lo, hi;
            if (A_MODE == 0) { lo = ra0; hi = ra1; }
            else Composer<FA>::template compose16<true>(ra0, sa, lo, hi);
            uint4* pa = reinterpret_cast<uint4*>(&lds_a[srow * S_STRIDE + shalf * 16]);
            pa[0] = lo; pa[1] = hi;
            Composer<FW>::template compose16<true>(rw, sw, lo, hi);
            uint4* pw = reinterpret_cast<uint4*>(&lds_w[srow * S_STRIDE + shalf * 16]);
            pw[0] = lo; pw[1] = hi;
        }
        __syncthreads();
        if (kt + 1 < ktiles) fetch(kt + 1);
#pragma unroll
        for (int ks = 0; ks < SBK / 16; ++ks) {
            bf16x8 af[2], wf[2];
            const int kofs = ks * 16 + (lane >> 5) * 8;
#pragma unroll
            for (int i = 0; i < 2; ++i)
                af[i] = *reinterpret_cast<const bf16x8*>(&lds_a[(wave_m * 64 + i * 32 + (lane & 31)) * S_STRIDE + kofs]);
#pragma unroll
            for (int j = 0; j < 2; ++j)
                wf[j] = *reinterpret_cast<const bf16x8*>(&lds_w[(wave_n * 64 + j * 32 + (lane & 31)) * S_STRIDE + kofs]);
#pragma unroll
            for (int i = 0; i < 2; ++i)
#pragma unroll
                for (int j = 0; j < 2; ++j) acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(af[i], wf[j], acc[i][j], 0, 0, 0);
        }
    }

#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            const int col = n0 + wave_n * 64 + j * 32 + (lane & 31);
            if (col >= N) continue;
            const float b = bias ? load_bias(bias, bias_dtype, col) : 0.0f;
#pragma unroll
            for (int v = 0; v < 16; ++v) {
                const int row = m0 + wave_m * 64 + i * 32 + 8 * (v >> 2) + 4 * (lane >> 5) + (v & 3);
                if (row < M) store_out<DT_OUT>(y, (int64_t)row * N + col, acc[i][j][v] + b);
            }
        }
}

template <int A_MODE, class FA, class FW, int DT_OUT>
int launch_gemm(const void* a_dense, const uint8_t* a_scales, const uint8_t* a_elements, const uint8_t* w_scales,
                const uint8_t* w_elements, const void* bias, int bias_dtype, void* y, int M, int N, int K, void* workspace,
                int64_t workspace_bytes, int batches, const GemmBatch& gb, hipStream_t s) {
    // batches > 1: the same product for `batches` operand sets, gb apart, in one launch (grid plane z = product z); dense A only,
    // never split over K (the caller checks both)
    const int tiles_m = (M + TM - 1) / TM, tiles_n = (N + TN - 1) / TN;
    const int64_t big_tiles = (int64_t)tiles_m * tiles_n;
    // 256 x 256 tiles need enough of them to occupy the 256 CUs; smaller problems use 128 x 128
    const bool fits32 = (int64_t)M * K * 2 < ((int64_t)1 << 32) && (int64_t)N * K < ((int64_t)1 << 32);  // 32-bit operand offsets
    const bool use_big = fits32 && (big_tiles >= 128 || (int64_t)M * N >= (int64_t)4096 * 4096);
    if constexpr (A_MODE == 0) {
        // few tiles and a long K: with a workspace, K is split over several workgroups per tile
        if (workspace && batches == 1 && K <= (1 << 23) && (reinterpret_cast<uintptr_t>(a_dense) & 15) == 0 && (reinterpret_cast<uintptr_t>(w_elements) & 15) == 0) {
            // (the 512 x 128 kernel reads four scale bytes at a time)
            const SplitPlan plan = plan_split_k(M, N, K, device_cu_count(), (reinterpret_cast<uintptr_t>(w_scales) & 3) == 0);
            if (plan.splits > 1 && workspace_bytes >= plan.workspace_bytes(M, N))
                return launch_gemm_split_k<FW, DT_OUT>(a_dense, w_scales, w_elements, bias, bias_dtype, y, M, N, K, plan, workspace, s);
        }
    }
    if constexpr (A_MODE == 0) {
        // fewest rows of A and not many rows of W: one workgroup per 16 rows of W, so that there are enough workgroups
        // (the 32-row kernel below has N / 32; measured better up to N = 12288 for M <= 16 and up to N = 8192 for M <= 64)
        if (M <= 64 && N % R16_N == 0 && N <= (M <= 16 ? 12288 : 8192) && K % 128 == 0 && K <= (1 << 24) &&
            (reinterpret_cast<uintptr_t>(a_dense) & 15) == 0 && (reinterpret_cast<uintptr_t>(w_elements) & 7) == 0) {
            if (M <= 16) return launch_gemm_rows16<FW, DT_OUT, 1, 8>(a_dense, w_scales, w_elements, bias, bias_dtype, y, M, N, K, batches, gb, s);
            if (M <= 32) return launch_gemm_rows16<FW, DT_OUT, 2, 4>(a_dense, w_scales, w_elements, bias, bias_dtype, y, M, N, K, batches, gb, s);
            return launch_gemm_rows16<FW, DT_OUT, 4, 2>(a_dense, w_scales, w_elements, bias, bias_dtype, y, M, N, K, batches, gb, s);
        }
    }
    if constexpr (A_MODE == 0) {
        // few rows of A: bound by streaming W; one workgroup per 32 rows of W
        // (K bound: both kernels address a row of A or W with a 32-bit byte offset from a per-workgroup base)
        if (M <= 128 && N % SK_N == 0 && K % SK_MAC == 0 && K <= (1 << 24) && (reinterpret_cast<uintptr_t>(a_dense) & 15) == 0 &&
            (reinterpret_cast<uintptr_t>(w_elements) & 15) == 0)
            return launch_gemm_skinny<FW, DT_OUT>(a_dense, w_scales, w_elements, bias, bias_dtype, y, M, N, K, batches, gb, s);
    }
    if constexpr (A_MODE == 0) {
        // More rows: three tile shapes.  The larger the tile the fewer instructions per MFMA (a composed W row serves more
        // rows of A), but the fewer tiles there are to spread over the CUs.  Pick the shape with the least estimated time:
        // (rounds of one tile per CU) x (time of one tile, relative, measured at K = 4096: 48 / 67 / 98 us for
        // 128 x 128 / 256 x 128 / 512 x 128); ties go to the larger tile.
        const bool al = (reinterpret_cast<uintptr_t>(a_dense) & 15) == 0 && (reinterpret_cast<uintptr_t>(w_elements) & 15) == 0;
        // (these kernels address with a 64-bit base per tile and 32-bit offsets within the tile's rows: operands of any
        // size, as long as 256 rows of A, or a few rows of y, stay below 4 GiB)
        const bool reach = K <= (1 << 23) && N <= (1 << 26);
        const bool mid_ok = reach && al && M > 128 && N % MD_N == 0 && K % MD_MAC == 0;
        const bool wide_ok = reach && al && M > 128 && N % WD_N == 0 && K % WD_K == 0;
        const bool tall_ok = reach && al && M >= UM && N % UN == 0 && K % UMAC == 0 && (reinterpret_cast<uintptr_t>(y) & 15) == 0 &&
                             (reinterpret_cast<uintptr_t>(w_scales) & 3) == 0 && (gb.ws & 3) == 0 &&
                             (int64_t)((M + UM - 1) / UM) * (N / UN) < (1 << 30);
        if (mid_ok || wide_ok || tall_ok) {
            const int cus = device_cu_count();
            if (cus <= 0) return fail(ERR_RUNTIME, "cannot read the compute-unit count of the current device");
            const int64_t n128 = N / 128;
            auto cost = [&](int tile_rows, double tile_time) {
                const int64_t tiles = (int64_t)((M + tile_rows - 1) / tile_rows) * n128;
                return tile_time * (double)((tiles + cus - 1) / cus);
            };
            int pick = -1;
            double best = 0.0;
            if (mid_ok) { pick = 0; best = cost(MD_M, 1.0); }
            if (wide_ok) { const double c = cost(WD_M, 1.4); if (pick < 0 || c <= best) { pick = 1; best = c; } }
            if (tall_ok) { const double c = cost(UM, 2.05); if (pick < 0 || c <= best) { pick = 2; best = c; } }
            if (pick == 0) return launch_gemm_mid<FW, DT_OUT, 2>(a_dense, w_scales, w_elements, bias, bias_dtype, y, M, N, K, batches, gb, s);
            if (pick == 1) return launch_gemm_wide<FW, DT_OUT>(a_dense, w_scales, w_elements, bias, bias_dtype, y, M, N, K, batches, gb, s);
            const int tall_tiles_m = (M + UM - 1) / UM;
            const int64_t tall_tiles = (int64_t)tall_tiles_m * (N / UN);
            const bool sc4 = K % 512 == 0;
            auto kern = sc4 ? mxfp_gemm_tall_kernel<FW, DT_OUT, true> : mxfp_gemm_tall_kernel<FW, DT_OUT, false>;
            static std::atomic<uint64_t> lds_allowed[2] = {{0}, {0}};
            if (int rc = allow_dynamic_lds(reinterpret_cast<const void*>(kern), U_LDS_BYTES, lds_allowed[sc4])) return rc;
            // one persistent workgroup per CU (a multiple of the 8 XCDs), never more than tiles
            const unsigned grid = (unsigned)(tall_tiles < cus ? ((tall_tiles + 7) / 8) * 8 : (cus / 8) * 8);
            hipLaunchKernelGGL(kern, dim3(grid, 1u, (unsigned)batches), dim3(kGemmThreads), U_LDS_BYTES, s, static_cast<const uint16_t*>(a_dense),
                               w_scales, w_elements, bias, bias_dtype, y, M, N, K, tall_tiles_m, N / UN, 1, (int64_t)0, gb, 0);
            return check_launch("mxfp_gemm");
        }
    }
    if (use_big) {
        const bool guard_k = K % TK != 0;
        auto kern = guard_k ? mxfp_gemm_kernel<A_MODE, FA, FW, DT_OUT, true> : mxfp_gemm_kernel<A_MODE, FA, FW, DT_OUT, false>;
        constexpr int lds_bytes = 4 * SLAB_BYTES;
        static std::atomic<uint64_t> lds_allowed[2];
        if (int rc = allow_dynamic_lds(reinterpret_cast<const void*>(kern), lds_bytes, lds_allowed[guard_k])) return rc;
        const int n_cus = device_cu_count();
        if (n_cus <= 0) return fail(ERR_RUNTIME, "cannot read the compute-unit count of the current device");
        // one persistent workgroup per CU (rounded down to a multiple of 8 XCD slots), never more than tiles
        const int64_t want = big_tiles < n_cus ? ((big_tiles + 7) / 8) * 8 : (n_cus / 8) * 8;
        const unsigned grid = (unsigned)want;
        hipLaunchKernelGGL(kern, dim3(grid, 1u, (unsigned)batches), dim3(kGemmThreads), lds_bytes, s, static_cast<const uint16_t*>(a_dense), a_scales,
                           a_elements, w_scales, w_elements, bias, bias_dtype, y, M, N, K, tiles_m, tiles_n, gb);
    } else {
        const dim3 grid((unsigned)((N + SBN - 1) / SBN), (unsigned)((M + SBM - 1) / SBM), (unsigned)batches);
        if (grid.y > 65535u) return fail(ERR_UNSUPPORTED, "M too large for the launch grid");
        hipLaunchKernelGGL((mxfp_gemm_small_kernel<A_MODE, FA, FW, DT_OUT>), grid, dim3(kGemmThreads), 0, s,
                           static_cast<const uint16_t*>(a_dense), a_scales, a_elements, w_scales, w_elements, bias, bias_dtype, y, M,
                           N, K, gb);
    }
    return check_launch("mxfp_gemm");
}


// Dense bf16 A against a weight in prepared form (the operand of the block-scaled GEMM: E4M3 bytes [rows_pad, K] without the
// NaN code, scales dword [K / 128][rows_pad]) on the 512 x 128 bf16 kernel: the compose is one convert per pair of
// codes and the scales of a macro step come as whole lines.
inline bool tall_prepared_shape_ok(int64_t M, int64_t N, int64_t K) {
    return M >= UM && N % UN == 0 && K % UMAC == 0 && K <= (1 << 23) && N <= (1 << 26) && ((M + UM - 1) / UM) * (N / UN) < (1 << 30);
}
template <int DT_OUT>
int launch_gemm_tall_prepared(const void* a_dense, const uint8_t* w_codes, const uint32_t* w_scales, const void* bias, int bias_dtype, void* y,
                              int M, int N, int K, hipStream_t s) {
    if (!tall_prepared_shape_ok(M, N, K)) return fail(ERR_UNSUPPORTED, "the prepared-weight bf16 GEMM takes M >= 512, N % 128 == 0, K % 128 == 0");
    const int cus = device_cu_count();
    if (cus <= 0) return fail(ERR_RUNTIME, "cannot read the compute-unit count of the current device");
    const int tiles_m = (M + UM - 1) / UM;
    const int64_t tiles = (int64_t)tiles_m * (N / UN);
    auto kern = mxfp_gemm_tall_kernel<PreparedE4M3, DT_OUT, false>;
    static std::atomic<uint64_t> lds_allowed{0};
    if (int rc = allow_dynamic_lds(reinterpret_cast<const void*>(kern), U_LDS_BYTES, lds_allowed)) return rc;
    const unsigned grid = (unsigned)(tiles < cus ? ((tiles + 7) / 8) * 8 : (cus / 8) * 8);
    const int rows_pad = (N + SN - 1) / SN * SN;
    hipLaunchKernelGGL(kern, dim3(grid), dim3(kGemmThreads), U_LDS_BYTES, s, static_cast<const uint16_t*>(a_dense), reinterpret_cast<const uint8_t*>(w_scales),
                       w_codes, bias, bias_dtype, y, M, N, K, tiles_m, N / UN, 1, (int64_t)0, GemmBatch{0, 0, 0, 0}, rows_pad);
    return check_launch("mxfp_gemm_prepared_w");
}

// One entry per weight format; each lives in its own translation unit (gemm_w_*.hip) so that the
// formats compile in parallel.  a_exp_bits == 0 selects the dense-A kernel.
struct GemmArgs {
    const void* a_dense; const uint8_t* a_scales; const uint8_t* a_elements; int a_exp_bits, a_frac_bits;
    const uint8_t* w_scales; const uint8_t* w_elements; const void* bias; int bias_dtype; void* y; int out_dtype;
    int M, N, K; void* workspace; int64_t workspace_bytes; hipStream_t stream;
    int batches; GemmBatch batch;   // batches > 1: one launch for that many products, operands `batch` apart (dense A only)
};
int gemm_w_e4m3(const GemmArgs& g);
int gemm_w_e5m2(const GemmArgs& g);
int gemm_w_e2m3(const GemmArgs& g);
int gemm_w_e3m2(const GemmArgs& g);
int gemm_w_e2m1(const GemmArgs& g);

template <class FW>
int gemm_for_weight_format(const GemmArgs& g) {
    return dispatch_dtype(g.out_dtype, [&](auto dout) {
        constexpr int DO = decltype(dout)::value;
        if (g.a_dense)
            return launch_gemm<0, SFmt<4, 3>, FW, DO>(g.a_dense, nullptr, nullptr, g.w_scales, g.w_elements, g.bias, g.bias_dtype, g.y,
                                                      g.M, g.N, g.K, g.workspace, g.workspace_bytes, g.batches, g.batch, g.stream);
        const int E = g.a_exp_bits, M = g.a_frac_bits;
#define MASE_A_FMT(e, m)                                                                                                       \
        if (E == e && M == m)                                                                                                  \
            return launch_gemm<1, SFmt<e, m>, FW, DO>(nullptr, g.a_scales, g.a_elements, g.w_scales, g.w_elements, g.bias,     \
                                                      g.bias_dtype, g.y, g.M, g.N, g.K, nullptr, 0, 1, GemmBatch{0, 0, 0, 0}, g.stream);
        MASE_A_FMT(4, 3) MASE_A_FMT(5, 2) MASE_A_FMT(2, 3) MASE_A_FMT(3, 2) MASE_A_FMT(2, 1)
#undef MASE_A_FMT
        return fail(ERR_INVALID, "MXFP element (exp_bits, frac_bits) must be one of (4,3) (5,2) (2,3) (3,2) (2,1)");
    });
}

}  // namespace mase
