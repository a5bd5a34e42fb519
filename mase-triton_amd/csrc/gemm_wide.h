// MXFP GEMM kernel for gfx950 for a few hundred rows of A (256 < M <= 512): dense bf16 A, MXFP W.
//
// The 128 x 128 tile kernel composes every W row once per 128 rows of A and is bound by that compose.  Here a
// workgroup owns a 256 x 128 tile, so the compose per MFMA halves; eight wavefronts own 64 x 64 pieces of it (4 along
// M x 2 along N, two wavefronts per SIMD, no partial sums to add).  K is walked in steps of 64:
//   * W codes (128 rows x 64 k: one 16-byte load per lane) go through a three-slot register ring, are composed to
//     bf16 between the MFMAs of the step before and written to one of two 16 KB LDS stages;
//   * the matching 64 k of the tile's 256 A rows come global -> LDS by DMA as whole 128-byte lines into one of three
//     32 KB stages, two steps ahead;
//   * 16 MFMAs (32x32x16) per wavefront and step; one barrier.
// Step s issues the DMAs of A(s + 2), then the loads of W(s + 3).  Vector memory completes in issue order, so one
// counted wait at the top of a step (all but the youngest step's operations) covers A(s) and W(s + 1).
//
// LDS rows are 128 bytes (64 k of bf16), the 16-byte chunk c of row r at position c ^ ((r >> 1) & 7).
// (included from gemm_impl.h, inside namespace mase, after gemm_mid.h)

constexpr int WD_M = 256, WD_N = 128, WD_K = 64;
constexpr int WD_ROW = 2 * WD_K;                         // bytes per LDS row
constexpr int WD_A_STAGE = WD_M * WD_ROW;                // 32 KB
constexpr int WD_W_STAGE = WD_N * WD_ROW;                // 16 KB
constexpr int WD_LDS_BYTES = 3 * WD_A_STAGE + 2 * WD_W_STAGE;  // 128 KB
constexpr int WD_THREADS = 512;

template <class FW, int DT_OUT>
__global__ __launch_bounds__(WD_THREADS) void mxfp_gemm_wide_kernel(
    const uint16_t* __restrict__ a_dense0, const uint8_t* __restrict__ w_scales0, const uint8_t* __restrict__ w_elements0,
    const void* __restrict__ bias, int bias_dtype, void* __restrict__ y_all, int M, int N, int K, int tiles_m, int k_len, int64_t y_split_bytes,
    GemmBatch gb) {
    // batched launches: workgroups of grid plane z work on product z (offsets are zero for a single product)
    const uint16_t* __restrict__ const a_dense = a_dense0 + (int64_t)blockIdx.z * gb.a;
    const uint8_t* __restrict__ const w_scales = w_scales0 + (int64_t)blockIdx.z * gb.ws;
    const uint8_t* __restrict__ const w_elements = w_elements0 + (int64_t)blockIdx.z * gb.we;
    constexpr int A_DMAS = WD_A_STAGE / 1024 / 8;          // 4 per wavefront and step
    constexpr int OPS = A_DMAS + 2;                        // vector-memory operations per wavefront and step
    extern __shared__ __attribute__((aligned(1024))) uint8_t lds[];
    uint8_t* const lds_a = lds;                            // [3][256 rows][128 B]
    uint8_t* const lds_w = lds + 3 * WD_A_STAGE;           // [2][128 rows][128 B]
    const uint32_t lds_a_addr = (uint32_t)(uintptr_t)lds;

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wave_m = wave >> 1, wave_n = wave & 1;
    // m-tile fastest: the workgroups that share 128 rows of W run next to each other in time, and, workgroups being dealt
    // to the 8 XCDs in turn, on the same XCD (one L2): XCD x takes the x-th eighth of the tiles
    const unsigned n_wg = gridDim.x, per_xcd = n_wg >> 3;
    const unsigned tile = (n_wg & 7u) == 0 ? (blockIdx.x & 7u) * per_xcd + (blockIdx.x >> 3) : blockIdx.x;
    const int tile_m = (int)(tile % (unsigned)tiles_m), tile_n = (int)(tile / (unsigned)tiles_m);
    const int m0 = tile_m * WD_M, n0 = tile_n * WD_N;
    // blockIdx.y = split of K: this workgroup multiplies k in [k_begin, k_begin + k_len) (the last split may be shorter)
    // and writes its sums to its own [M, N] array, y_split_bytes apart.  One split: k_len = K.
    const int k_begin = (int)blockIdx.y * k_len;
    const int kblocks = K / 32, nsteps = min(k_len, K - k_begin) / WD_K;
    void* const y = static_cast<uint8_t*>(y_all) + (size_t)blockIdx.y * (size_t)y_split_bytes + (int64_t)blockIdx.z * gb.y;
    // 64-bit base of the tile's first row (and the split's first k): the per-lane offsets below stay within the tile's rows
    const uint8_t* const a_tile = reinterpret_cast<const uint8_t*>(a_dense) + ((size_t)m0 * K + k_begin) * 2;

    // A DMA: an instruction moves 1 KB = 8 rows; lane l fills position l & 7 of row 8 (4 w + j) + (l >> 3), which must
    // hold chunk (l & 7) ^ ((row >> 1) & 7).  Rows past M re-read row M - 1 (their products are never stored).
    uint32_t a_voff[A_DMAS];
#pragma unroll
    for (int j = 0; j < A_DMAS; ++j) {
        const int row = (wave * A_DMAS + j) * 8 + (lane >> 3);
        a_voff[j] = (uint32_t)(min(m0 + row, M - 1) - m0) * (uint32_t)K * 2u + (uint32_t)(((lane & 7) ^ ((row >> 1) & 7)) * 16);
    }
    // W: thread t loads the 16 codes at k 16 (t & 3) .. + 15 of row t >> 2
    const int w_row = tid >> 2, w_piece = tid & 3;
    const uint8_t* const w_base = w_elements + (size_t)n0 * K + k_begin;
    const uint8_t* const ws_base = w_scales + (size_t)n0 * kblocks + k_begin / 32;
    const uint32_t w_voff = (uint32_t)w_row * (uint32_t)K + (uint32_t)w_piece * 16u;
    const uint32_t ws_voff = (uint32_t)w_row * (uint32_t)kblocks + (uint32_t)(w_piece >> 1);
    uint32_t w_lds_off[2];
#pragma unroll
    for (int e = 0; e < 2; ++e) w_lds_off[e] = (uint32_t)w_row * WD_ROW + (uint32_t)(((2 * w_piece + e) ^ ((w_row >> 1) & 7)) * 16);
    // fragment reads: lane (g = l >> 5, r = l & 31) reads chunk 2 q + g of row 32 t + r for the 16-k step q
    uint32_t f_off[4];
#pragma unroll
    for (int q = 0; q < 4; ++q) f_off[q] = (uint32_t)(lane & 31) * WD_ROW + (uint32_t)(((2 * q + (lane >> 5)) ^ ((lane >> 1) & 7)) * 16);

    floatx16 acc[2][2];  // [m-tile of the wavefront][n-tile]
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.0f;

    u32x4 w_raw[3];
    uint32_t w_scale[3];
    // workgroups start at different steps of K (and wrap around), so that at any moment they read different columns
    // of W and A: addresses that spread over the memory channels
    const int rot = (int)((unsigned)(tile_n + blockIdx.y) % (unsigned)nsteps);
    // past the end the last step is read again (unused), which keeps the operation count per step, and with it the
    // wait counts, the same
    auto k_of = [&](int s) __attribute__((always_inline)) {
        const int kc = min(s, nsteps - 1) + rot;
        return kc >= nsteps ? kc - nsteps : kc;
    };
    // (compile-time indices and forced inlining throughout: a run-time loop, even one that is unrolled later, or a
    // real call leaves the register ring and the accumulators in scratch memory, whose traffic the wait counts below
    // do not expect)
    auto issue_a = [&](int s, auto stage_c) __attribute__((always_inline)) {
        constexpr int stage = decltype(stage_c)::value;
        const uint8_t* const a_src = a_tile + (size_t)k_of(s) * (WD_K * 2);
        const uint32_t dst = lds_a_addr + (uint32_t)stage * WD_A_STAGE + (uint32_t)wave * (A_DMAS * 1024);
        static_for<A_DMAS>([&](auto j_c) __attribute__((always_inline)) {
            constexpr int j = decltype(j_c)::value;
            dma_1kb(dst + j * 1024, a_voff[j], a_src);
        });
    };
    auto issue_w = [&](int s, auto slot_c) __attribute__((always_inline)) {
        constexpr int slot = decltype(slot_c)::value;
        const int kc = k_of(s);
        async_load16(w_raw[slot], w_voff, w_base + (size_t)kc * WD_K);
        async_load_u8(w_scale[slot], ws_voff, ws_base + kc * (WD_K / 32));
    };

    // Issue groups: step s issues {A(s + 2), W(s + 3)}.  At the top of step s everything but the group of step s - 1
    // has arrived: A(s) is in LDS and W(s + 1) in registers; W(s + 1) is composed between the MFMAs of step s.
    issue_w(0, IntC<0>{});
    issue_a(0, IntC<0>{});
    issue_w(1, IntC<1>{});
    wait_vmcnt<0>(w_raw[0], w_scale[0]);
    wait_vmcnt<0>(w_raw[1], w_scale[1]);
    {
        uint4 lo, hi;
        Composer<FW>::template compose16<true>(make_uint4(w_raw[0].x, w_raw[0].y, w_raw[0].z, w_raw[0].w), w_scale[0], lo, hi);
        *reinterpret_cast<uint4*>(lds_w + w_lds_off[0]) = lo;
        *reinterpret_cast<uint4*>(lds_w + w_lds_off[1]) = hi;
    }
    issue_a(1, IntC<1>{});
    issue_w(2, IntC<2>{});
    for (int base = 0; base < nsteps; base += 6) {
        // (forced inline: as a call, the step would take the accumulators and the ring through memory)
        static_for<6>([&](auto r_c) __attribute__((always_inline)) {
            constexpr int r = decltype(r_c)::value;
            const int s = base + r;
            if (s < nsteps) {
                constexpr int ns = r % 3, cs = (r + 1) % 3, a_stage = (r + 2) % 3, w_stage = (r + 1) % 2;
                wait_vmcnt<OPS>(w_raw[cs], w_scale[cs]);
                __builtin_amdgcn_s_waitcnt(0xC07F);  // lgkmcnt(0): this wavefront's LDS reads and writes are done
                __builtin_amdgcn_s_barrier();        // this step's W and A stages are complete; last step's are no longer read
                // this step's loads (A(s + 2) into the stage read last step, W(s + 3) into the ring slot composed last
                // step) and the compose of W(s + 1) are spread over the step's 16 MFMAs: instructions issue in order, so
                // work placed behind a run of MFMAs would wait for the whole run
                const uint8_t* const a_src = a_tile + (size_t)k_of(s + 2) * (WD_K * 2);
                const uint32_t a_dst = lds_a_addr + (uint32_t)a_stage * WD_A_STAGE + (uint32_t)wave * (A_DMAS * 1024);
                const int kw = k_of(s + 3);
                const uint8_t* const w_src = w_base + (size_t)kw * WD_K;
                const uint8_t* const ws_src = ws_base + kw * (WD_K / 32);
                auto vmem = [&](auto k_c) __attribute__((always_inline)) {  // operation k of the step's 6, A first
                    constexpr int k = decltype(k_c)::value;
                    if constexpr (k < A_DMAS) dma_1kb(a_dst + k * 1024, a_voff[k], a_src);
                    else if constexpr (k == A_DMAS) async_load16(w_raw[ns], w_voff, w_src);
                    else async_load_u8(w_scale[ns], ws_voff, ws_src);
                };
                const bool any_slow = __builtin_amdgcn_ballot_w64(Composer<FW>::is_slow(w_scale[cs])) != 0;
                const Composer<FW> cmp(w_scale[cs]);
                const uint8_t* const pa = lds_a + (r % 3) * WD_A_STAGE + wave_m * (64 * WD_ROW);
                const uint8_t* const pw = lds_w + (r % 2) * WD_W_STAGE + wave_n * (64 * WD_ROW);
                uint8_t* const st = lds_w + w_stage * WD_W_STAGE;
                bf16x8 wf[2][2], af[2][2];
                auto load_frags = [&](auto q_c) __attribute__((always_inline)) {
                    constexpr int q = decltype(q_c)::value;
#pragma unroll
                    for (int j = 0; j < 2; ++j) wf[q & 1][j] = *reinterpret_cast<const bf16x8*>(pw + j * (32 * WD_ROW) + f_off[q]);
#pragma unroll
                    for (int i = 0; i < 2; ++i) af[q & 1][i] = *reinterpret_cast<const bf16x8*>(pa + i * (32 * WD_ROW) + f_off[q]);
                };
                uint32_t o[8];
                load_frags(IntC<0>{});
                static_for<4>([&](auto q_c) __attribute__((always_inline)) {
                    constexpr int q = decltype(q_c)::value, b = q & 1;
                    // the next 16-k step's fragments are requested before this step's MFMAs; word q of the step's four
                    // code words is composed beside them, and the first six MFMAs of the step carry its loads
                    if constexpr (q < 3) load_frags(IntC<q + 1>{});
                    const uint32_t cw = w_raw[cs][q];
                    __builtin_amdgcn_sched_barrier(0);
                    acc[0][0] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(wf[b][0], af[b][0], acc[0][0], 0, 0, 0);
                    o[2 * q] = cmp.pair_lo(cw);
                    if constexpr (4 * q < OPS) vmem(IntC<4 * q>{});
                    __builtin_amdgcn_sched_barrier(0);
                    acc[0][1] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(wf[b][1], af[b][0], acc[0][1], 0, 0, 0);
                    if constexpr (4 * q + 1 < OPS) vmem(IntC<4 * q + 1>{});
                    __builtin_amdgcn_sched_barrier(0);
                    acc[1][0] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(wf[b][0], af[b][1], acc[1][0], 0, 0, 0);
                    o[2 * q + 1] = cmp.pair_hi(cw);
                    if constexpr (4 * q + 2 < OPS) vmem(IntC<4 * q + 2>{});
                    __builtin_amdgcn_sched_barrier(0);
                    acc[1][1] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(wf[b][1], af[b][1], acc[1][1], 0, 0, 0);
                    if constexpr (4 * q + 3 < OPS) vmem(IntC<4 * q + 3>{});
                    __builtin_amdgcn_sched_barrier(0);
                });
                uint4 lo = make_uint4(o[0], o[1], o[2], o[3]), hi = make_uint4(o[4], o[5], o[6], o[7]);
                if (any_slow) Composer<FW>::fix_slow(w_scale[cs], make_uint4(w_raw[cs].x, w_raw[cs].y, w_raw[cs].z, w_raw[cs].w), lo, hi);
                *reinterpret_cast<uint4*>(st + w_lds_off[0]) = lo;
                *reinterpret_cast<uint4*>(st + w_lds_off[1]) = hi;
            }
        });
    }
    // the look-ahead loads still target LDS and registers: let them finish
    wait_vmcnt<0>(w_raw[0], w_scale[0]);

    // lane holds, for its m-tile i, n-tile j and g = 0..3, y[m][n .. n+3] with m = m0 + 64 wave_m + 32 i + lane % 32,
    // n = n0 + 64 wave_n + 32 j + 8 g + 4 (lane / 32)
    const bool vec_ok = (N % 4 == 0) && (reinterpret_cast<uintptr_t>(y) & 15) == 0;
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
        for (int g = 0; g < 4; ++g) {
            const int n = n0 + 64 * wave_n + 32 * j + 8 * g + 4 * (lane >> 5);
            float b[4] = {0.0f, 0.0f, 0.0f, 0.0f};
            if (bias)
                for (int t = 0; t < 4; ++t) b[t] = load_bias(bias, bias_dtype, n + t);
#pragma unroll
            for (int i = 0; i < 2; ++i) {
                const int m = m0 + 64 * wave_m + 32 * i + (lane & 31);
                if (m < M) {
                    const float r[4] = {acc[i][j][4 * g] + b[0], acc[i][j][4 * g + 1] + b[1], acc[i][j][4 * g + 2] + b[2],
                                        acc[i][j][4 * g + 3] + b[3]};
                    store_out4<DT_OUT>(y, (int64_t)m * N + n, r, vec_ok, 4);
                }
            }
        }
}

template <class FW, int DT_OUT>
int launch_gemm_wide(const void* a_dense, const uint8_t* w_scales, const uint8_t* w_elements, const void* bias, int bias_dtype,
                     void* y, int M, int N, int K, int batches, const GemmBatch& gb, hipStream_t s) {
    auto kern = mxfp_gemm_wide_kernel<FW, DT_OUT>;
    static std::atomic<uint64_t> lds_allowed{0};
    if (int rc = allow_dynamic_lds(reinterpret_cast<const void*>(kern), WD_LDS_BYTES, lds_allowed)) return rc;
    const int tiles_m = (M + WD_M - 1) / WD_M;
    const int64_t tiles = (int64_t)tiles_m * (N / WD_N);
    if (tiles > 0x7FFFFFFFll) return fail(ERR_UNSUPPORTED, "too many tiles for one launch");
    hipLaunchKernelGGL(kern, dim3((unsigned)tiles, 1u, (unsigned)batches), dim3(WD_THREADS), WD_LDS_BYTES, s, static_cast<const uint16_t*>(a_dense),
                       w_scales, w_elements, bias, bias_dtype, y, M, N, K, tiles_m, K, (int64_t)0, gb);
    return check_launch("mxfp_gemm");
}
