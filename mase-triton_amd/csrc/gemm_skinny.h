// Skinny MXFP GEMM kernel for gfx950: M <= 128 (decode / small-batch shapes), dense bf16 A, MXFP W.
//
// With few rows of A the product is bound by streaming W from HBM, and the point of the fused path is
// that W is read as one byte per element and never written back as bf16.  One workgroup owns 32 rows of
// W (N / 32 workgroups, several resident per CU) and walks K in macro steps of 128:
//   * W codes come as whole 128-byte lines (lane = 16 codes of one row), are composed to bf16 in
//     registers and written to LDS in the MFMA fragment-friendly layout below;
//   * the matching 128 k of all A rows come global -> LDS by DMA (whole lines; A is small and stays in L2);
//   * the macro step's eight 16-k MFMA steps are split over the four wavefronts (two each, all rows),
//     so every wavefront ends with partial sums that are added through LDS once, at the end.
// The loads of macro step m+D (W codes and scales into registers, A by DMA into one of D+1 LDS stages) are issued
// before the MFMAs of step m; HBM latency is covered by this depth, since a CU holds fewer than two of these
// workgroups when N / 32 is a few hundred.  All of them are inline asm, waited for with a counted s_waitcnt
// (vector memory completes in issue order).  The composed W is double buffered; one barrier per macro step.
//
// LDS rows are 256 bytes (128 k of bf16), the 16-byte chunk c of row r at position c ^ (r & 15): the LDS
// serves a 128-bit read 16 lanes at a time from 64 banks, and 16 consecutive rows then hit 16 different
// bank groups.
// (included from gemm_impl.h, inside namespace mase, after gemm_tall.h, whose asm helpers it uses)

constexpr int SK_N = 32;        // W rows per workgroup
constexpr int SK_MAC = 128;     // k granularity the launcher requires

template <class FW, int DT_OUT, int MT, int D, int L, int AR>
__global__ __launch_bounds__(kGemmThreads) void mxfp_gemm_skinny_kernel(
    const uint16_t* __restrict__ a_dense0, const uint8_t* __restrict__ w_scales0, const uint8_t* __restrict__ w_elements0,
    const void* __restrict__ bias, int bias_dtype, void* __restrict__ y0, int M, int N, int K, GemmBatch gb) {
    // batched launches: workgroups of grid plane z work on product z (offsets are zero for a single product)
    const uint16_t* __restrict__ const a_dense = a_dense0 + (int64_t)blockIdx.z * gb.a;
    const uint8_t* __restrict__ const w_scales = w_scales0 + (int64_t)blockIdx.z * gb.ws;
    const uint8_t* __restrict__ const w_elements = w_elements0 + (int64_t)blockIdx.z * gb.we;
    void* __restrict__ const y = static_cast<uint8_t*>(y0) + (int64_t)blockIdx.z * gb.y;
    // L = 128-byte lines of W codes per row and macro step: the macro step covers KM = 128 L k, LDS rows are 256 L bytes
    // AR = rows of A kept per m-tile: 32, or 16 when M <= 16 (rows 16..31 of the MFMA operand then re-read rows 0..15)
    static_assert(AR == 32 || (AR == 16 && MT == 1), "16-row stages only with one m-tile");
    constexpr int KM = 128 * L, ROW = 2 * KM, CH = ROW / 16;
    constexpr int R = D + 1;                                  // ring size: registers sets of W, LDS stages of A
    constexpr int A_DMAS = AR * MT * ROW / 1024 / 4;          // A DMAs per wavefront and macro step
    constexpr int OPS = A_DMAS + 2 * L;                       // vector-memory operations per wavefront and macro step
    constexpr int A_STAGE = AR * MT * ROW, W_STAGE = SK_N * ROW;
    constexpr int QW = KM / 16 / 4;                           // 16-k MFMA steps per wavefront and macro step
    static_assert((D - 1) * OPS < 64, "vmcnt is a 6-bit counter");
    extern __shared__ __attribute__((aligned(1024))) uint8_t lds[];
    uint8_t* const lds_a = lds;                    // [R][32 MT rows][ROW]
    uint8_t* const lds_w = lds + R * A_STAGE;      // [2][32 rows][ROW]
    const uint32_t lds_a_addr = (uint32_t)(uintptr_t)lds;

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int n0 = blockIdx.x * SK_N;
    const int kblocks = K / 32, nmac = K / KM;

    // A DMA: an instruction moves 1 KB = 1024 / ROW rows; lane l fills position l % CH of row (1 KB index) * (1024 / ROW)
    // + l / CH, which must hold chunk (l % CH) ^ (row & 15).  Rows past M re-read row M - 1.
    uint32_t a_voff[A_DMAS];
#pragma unroll
    for (int j = 0; j < A_DMAS; ++j) {
        const int row = (wave * A_DMAS + j) * (1024 / ROW) + lane / CH;
        a_voff[j] = (uint32_t)min(row, M - 1) * (uint32_t)K * 2u + (uint32_t)((((lane % CH) ^ (row & 15))) * 16);
    }
    // W: the wavefront loads rows 8w .. 8w+7 as whole lines, lane = 16 codes (16 k) of row 8w + (l >> 3), L times
    const int w_row = wave * 8 + (lane >> 3), w_chunk = lane & 7;
    const uint8_t* const w_base = w_elements + (size_t)(n0 + wave * 8) * K;          // wave-uniform
    const uint8_t* const ws_base = w_scales + (size_t)(n0 + wave * 8) * kblocks;
    const uint32_t w_voff = (uint32_t)(lane >> 3) * (uint32_t)K + (uint32_t)w_chunk * 16u;
    const uint32_t ws_voff = (uint32_t)(lane >> 3) * (uint32_t)kblocks + (uint32_t)(w_chunk >> 1);
    uint32_t w_lds_off[L][2];
#pragma unroll
    for (int li = 0; li < L; ++li)
#pragma unroll
        for (int e = 0; e < 2; ++e)
            w_lds_off[li][e] = (uint32_t)w_row * ROW + (uint32_t)(((16 * li + 2 * w_chunk + e) ^ (w_row & 15)) * 16);
    // fragment reads: lane (g = l >> 5, r = l & 31) reads chunk 2q + g of row 32 t + r; this wavefront owns q = QW w .. QW w + QW - 1
    uint32_t f_off[QW], fa_off[QW];
#pragma unroll
    for (int e = 0; e < QW; ++e) {
        f_off[e] = (uint32_t)(lane & 31) * ROW + (uint32_t)(((2 * (QW * wave + e) + (lane >> 5)) ^ (lane & 15)) * 16);
        fa_off[e] = (uint32_t)(lane & (AR - 1)) * ROW + (uint32_t)(((2 * (QW * wave + e) + (lane >> 5)) ^ (lane & 15)) * 16);
    }

    floatx16 acc[MT];
#pragma unroll
    for (int t = 0; t < MT; ++t)
#pragma unroll
        for (int v = 0; v < 16; ++v) acc[t][v] = 0.0f;

    u32x4 w_raw[R][L];
    uint32_t w_scale[R][L];
    // workgroups start at different macro steps of K (and wrap around): at any moment they then read different
    // columns of W, i.e. addresses that do not all differ by multiples of the row pitch and so spread over the
    // memory channels
    const int rot = (int)(blockIdx.x % (unsigned)nmac);
    // loads of macro step `mac` into ring slot `slot_c`; past the end the last macro step is read again (unused),
    // which keeps the number of operations per step, and with it the wait counts, the same
    auto issue_loads = [&](int mac, auto slot_c) {
        constexpr int slot = decltype(slot_c)::value;
        int mc = min(mac, nmac - 1) + rot;
        if (mc >= nmac) mc -= nmac;
#pragma unroll
        for (int li = 0; li < L; ++li) {
            async_load16(w_raw[slot][li], w_voff, w_base + (size_t)mc * KM + li * 128);
            async_load_u8(w_scale[slot][li], ws_voff, ws_base + mc * (KM / 32) + li * 4);
        }
        const uint8_t* const a_src = reinterpret_cast<const uint8_t*>(a_dense) + (size_t)mc * (KM * 2);
        const uint32_t dst = lds_a_addr + (uint32_t)slot * A_STAGE + (uint32_t)wave * (A_DMAS * 1024);
#pragma unroll
        for (int j = 0; j < A_DMAS; ++j) dma_1kb(dst + j * 1024, a_voff[j], a_src);
    };
    // the loads of the macro step in ring slot `slot_c` have arrived (D - 1 younger steps may still be in flight):
    // compose its W into stage `mac & 1`
    auto stage_w = [&](int mac, auto slot_c) {
        constexpr int slot = decltype(slot_c)::value;
        wait_vmcnt<(D - 1) * OPS>(w_raw[slot][0], w_scale[slot][0]);
        if (L == 2) wait_vmcnt<(D - 1) * OPS>(w_raw[slot][L - 1], w_scale[slot][L - 1]);
        uint8_t* const st = lds_w + (mac & 1) * W_STAGE;
#pragma unroll
        for (int li = 0; li < L; ++li) {
            uint4 lo, hi;
            Composer<FW>::template compose16<true>(make_uint4(w_raw[slot][li].x, w_raw[slot][li].y, w_raw[slot][li].z, w_raw[slot][li].w),
                                                   w_scale[slot][li], lo, hi);
            *reinterpret_cast<uint4*>(st + w_lds_off[li][0]) = lo;
            *reinterpret_cast<uint4*>(st + w_lds_off[li][1]) = hi;
        }
    };

    static_for<D>([&](auto d_c) { issue_loads(decltype(d_c)::value, d_c); });
    stage_w(0, IntC<0>{});
    for (int base = 0; base < nmac; base += R) {
        static_for<R>([&](auto r_c) {
            constexpr int r = decltype(r_c)::value;
            const int mac = base + r;
            if (mac < nmac) {
                __builtin_amdgcn_s_waitcnt(0xC07F);  // lgkmcnt(0): this wavefront's LDS reads and writes are done
                __builtin_amdgcn_s_barrier();        // W stage mac & 1 and A slot r are complete; slot r - 1 is no longer read
                issue_loads(mac + D, IntC<(r + D) % R>{});
                const uint8_t* const pa = lds_a + r * A_STAGE;
                const uint8_t* const pw = lds_w + (mac & 1) * W_STAGE;
                if constexpr (MT <= 2) {
                    // few MFMAs: the fragment reads go out, the next step's W is composed while they are in flight, then
                    // the MFMAs (nothing waits for their results before the next step's MFMAs)
                    bf16x8 wf[QW], af[QW][MT];
#pragma unroll
                    for (int e = 0; e < QW; ++e) {
                        wf[e] = *reinterpret_cast<const bf16x8*>(pw + f_off[e]);
#pragma unroll
                        for (int t = 0; t < MT; ++t) af[e][t] = *reinterpret_cast<const bf16x8*>(pa + t * (32 * ROW) + fa_off[e]);
                    }
                    __builtin_amdgcn_sched_barrier(0);
                    stage_w(mac + 1, IntC<(r + 1) % R>{});  // (past the end: composes the re-read step into the unused stage)
                    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                    for (int e = 0; e < QW; ++e)
#pragma unroll
                        for (int t = 0; t < MT; ++t) acc[t] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(wf[e], af[e][t], acc[t], 0, 0, 0);
                } else {
#pragma unroll
                    for (int e = 0; e < QW; ++e) {
                        const bf16x8 wf = *reinterpret_cast<const bf16x8*>(pw + f_off[e]);
#pragma unroll
                        for (int t = 0; t < MT; ++t) {
                            const bf16x8 af = *reinterpret_cast<const bf16x8*>(pa + t * (32 * ROW) + fa_off[e]);
                            acc[t] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(wf, af, acc[t], 0, 0, 0);
                        }
                    }
                    stage_w(mac + 1, IntC<(r + 1) % R>{});
                }
            }
        });
    }
    // the look-ahead loads still target LDS and registers: let them finish
    wait_vmcnt<0>(w_raw[0][0], w_scale[0][0]);

    // ---- add the four wavefronts' partial sums: wavefronts 1..3 park theirs in LDS ([w-1][t][v][lane]), 0 adds
    __syncthreads();  // every fragment read is done: the stages can be reused
    float* const red = reinterpret_cast<float*>(lds);
    if (wave != 0) {
#pragma unroll
        for (int t = 0; t < MT; ++t)
#pragma unroll
            for (int v = 0; v < 16; ++v) red[(((wave - 1) * MT + t) * 16 + v) * 64 + lane] = acc[t][v];
    }
    __syncthreads();
    if (wave != 0) return;
#pragma unroll 1
    for (int w = 0; w < 3; ++w)  // one wavefront's sums at a time: all three at once would cost 48 MT registers
#pragma unroll
        for (int t = 0; t < MT; ++t)
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[t][v] += red[((w * MT + t) * 16 + v) * 64 + lane];

    // lane holds, for m-tile t and g = 0..3, y[m][n .. n+3] with m = 32 t + lane % 32, n = n0 + 8 g + 4 (lane / 32)
    const bool vec_ok = (N % 4 == 0) && (reinterpret_cast<uintptr_t>(y) & 15) == 0;
#pragma unroll
    for (int g = 0; g < 4; ++g) {
        const int n = n0 + 8 * g + 4 * (lane >> 5);
        float b[4] = {0.0f, 0.0f, 0.0f, 0.0f};
        if (bias)
            for (int t = 0; t < 4; ++t) b[t] = load_bias(bias, bias_dtype, n + t);
#pragma unroll
        for (int t = 0; t < MT; ++t) {
            const int m = 32 * t + (lane & 31);
            if (m < M) {
                const float r[4] = {acc[t][4 * g] + b[0], acc[t][4 * g + 1] + b[1], acc[t][4 * g + 2] + b[2], acc[t][4 * g + 3] + b[3]};
                store_out4<DT_OUT>(y, (int64_t)m * N + n, r, vec_ok, 4);
            }
        }
    }
}

template <class FW, int DT_OUT>
int launch_gemm_skinny(const void* a_dense, const uint8_t* w_scales, const uint8_t* w_elements, const void* bias, int bias_dtype,
                       void* y, int M, int N, int K, int batches, const GemmBatch& gb, hipStream_t s) {
    const dim3 grid((unsigned)(N / SK_N), 1u, (unsigned)batches);
    auto go = [&](auto mt_c, auto d_c) {
        constexpr int MT = decltype(mt_c)::value, D = decltype(d_c)::value, L = 1, AR = 32;
        constexpr int lds_bytes = (D + 1) * AR * MT * 256 * L + 2 * SK_N * 256 * L;
        auto kern = mxfp_gemm_skinny_kernel<FW, DT_OUT, MT, D, L, AR>;
        static std::atomic<uint64_t> lds_allowed{0};
        if (int rc = allow_dynamic_lds(reinterpret_cast<const void*>(kern), lds_bytes, lds_allowed)) return rc;
        hipLaunchKernelGGL(kern, grid, dim3(kGemmThreads), lds_bytes, s, static_cast<const uint16_t*>(a_dense), w_scales, w_elements,
                           bias, bias_dtype, y, M, N, K, gb);
        return check_launch("mxfp_gemm");
    };
    if (M <= 16) {  // 16-row A stages leave LDS for a look-ahead of 8 macro steps
        constexpr int D = 8, L = 1, AR = 16;
        constexpr int lds_bytes = (D + 1) * AR * 256 * L + 2 * SK_N * 256 * L;
        auto kern = mxfp_gemm_skinny_kernel<FW, DT_OUT, 1, D, L, AR>;
        static std::atomic<uint64_t> lds_allowed{0};
        if (int rc = allow_dynamic_lds(reinterpret_cast<const void*>(kern), lds_bytes, lds_allowed)) return rc;
        hipLaunchKernelGGL(kern, grid, dim3(kGemmThreads), lds_bytes, s, static_cast<const uint16_t*>(a_dense), w_scales, w_elements,
                           bias, bias_dtype, y, M, N, K, gb);
        return check_launch("mxfp_gemm");
    }
    // Look-ahead in macro steps.  With more workgroups than CUs the A stages must leave LDS for two workgroups per CU, which
    // then cover each other's waits; a workgroup alone on its CU needs the deeper ring to cover memory latency itself
    // (four m-tiles, N = 4096, K = 14336: 110 -> 81 us).
    const int cus = device_cu_count();
    if (cus <= 0) return fail(ERR_RUNTIME, "cannot read the compute-unit count of the current device");
    const bool alone = (int)grid.x <= cus;
    if (M <= 32) return go(IntC<1>{}, IntC<4>{});
    if (M <= 64) return go(IntC<2>{}, IntC<2>{});
    return alone ? go(IntC<4>{}, IntC<3>{}) : go(IntC<4>{}, IntC<1>{});
}
