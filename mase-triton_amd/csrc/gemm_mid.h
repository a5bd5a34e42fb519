// Mid-size MXFP GEMM kernel for gfx950: more rows of A than the weight-streaming kernel takes (M > 128), fewer than
// a 512-row tile; dense bf16 A, MXFP W.
//
// One workgroup owns a 128 x 128 tile and walks K in macro steps of 128.  Four wavefronts own the four 64 x 64
// quadrants; with KS = 2 four more own the same quadrants for the upper half of every macro step's k range (two
// wavefronts per SIMD fill each other's issue gaps), and the two halves are added through LDS at the end.
// Per macro step:
//   * W codes come as whole 128-byte lines (lane = 16 codes of one row), are composed to bf16 in registers and
//     written to one of two LDS stages;
//   * the matching 128 k of the tile's 128 A rows come global -> LDS by DMA into one of three 32 KB stages;
//   * 32 MFMAs (32x32x16) per quadrant; one barrier.
// The tile is square because a flatter one re-reads more of A through the vector-memory path (here 48 KB per macro
// step and workgroup).  Step s issues the DMAs of A(s + 2) and the loads of W(s + 3).  Vector memory completes in
// issue order, so one counted wait at the top of a step (all but the youngest step's operations) covers A(s) and
// W(s + 1) and leaves one step's loads in flight.  W(s + 1) is composed in pieces between the MFMAs of step s, the
// step's loads are issued between them too, and the fragments of every 16-k step are requested one step ahead:
// instructions issue in order, so anything placed behind a run of MFMAs would wait for the whole run.
// With 64 x 64 per wavefront the compose (4 instructions per code) and the fragment reads (1 KB per MFMA) weigh
// four and two times what they do in the 512 x 128 kernel; this kernel is bound by them, not by the MFMA pipe.
//
// LDS rows are 256 bytes (128 k of bf16), the 16-byte chunk c of row r at position c ^ (r & 15), as in the
// weight-streaming kernel.
// (included from gemm_impl.h, inside namespace mase, after gemm_skinny.h)

constexpr int MD_M = 128, MD_N = 128, MD_MAC = 128;
constexpr int MD_ROW = 2 * MD_MAC;                         // bytes per LDS row
constexpr int MD_A_STAGES = 3;
constexpr int MD_A_STAGE = MD_M * MD_ROW;                  // 32 KB
constexpr int MD_W_STAGE = MD_N * MD_ROW;                  // 32 KB
constexpr int MD_LDS_BYTES = MD_A_STAGES * MD_A_STAGE + 2 * MD_W_STAGE;  // 160 KB

template <class FW, int DT_OUT, int KS>
__global__ __launch_bounds__(256 * KS) void mxfp_gemm_mid_kernel(
    const uint16_t* __restrict__ a_dense0, const uint8_t* __restrict__ w_scales0, const uint8_t* __restrict__ w_elements0,
    const void* __restrict__ bias, int bias_dtype, void* __restrict__ y_all, int M, int N, int K, int tiles_m, int k_len,
    int64_t y_split_bytes, GemmBatch gb) {
    // batched launches: workgroups of grid plane z work on product z (offsets are zero for a single product)
    const uint16_t* __restrict__ const a_dense = a_dense0 + (int64_t)blockIdx.z * gb.a;
    const uint8_t* __restrict__ const w_scales = w_scales0 + (int64_t)blockIdx.z * gb.ws;
    const uint8_t* __restrict__ const w_elements = w_elements0 + (int64_t)blockIdx.z * gb.we;
    constexpr int WAVES = 4 * KS, QW = 8 / KS;             // 16-k steps per wavefront and macro step
    constexpr int A_DMAS = MD_A_STAGE / 1024 / WAVES;      // per wavefront and macro step
    constexpr int W_LOADS = MD_N * MD_MAC / 16 / (64 * WAVES);  // code loads (and as many scale loads) per lane
    constexpr int OPS = A_DMAS + 2 * W_LOADS;              // vector-memory operations per wavefront and macro step
    extern __shared__ __attribute__((aligned(1024))) uint8_t lds[];
    uint8_t* const lds_a = lds;                                // [3][128 rows][256 B]
    uint8_t* const lds_w = lds + MD_A_STAGES * MD_A_STAGE;     // [2][128 rows][256 B]
    const uint32_t lds_a_addr = (uint32_t)(uintptr_t)lds;

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wave_m = (wave >> 1) & 1, wave_n = wave & 1, wave_k = wave >> 2;
    // m-tile fastest: the workgroups that share 128 rows of W run next to each other in time, and, workgroups being dealt
    // to the 8 XCDs in turn, on the same XCD (one L2): XCD x takes the x-th eighth of the tiles
    const unsigned n_wg = gridDim.x, per_xcd = n_wg >> 3;
    const unsigned tile = (n_wg & 7u) == 0 ? (blockIdx.x & 7u) * per_xcd + (blockIdx.x >> 3) : blockIdx.x;
    const int tile_m = (int)(tile % (unsigned)tiles_m), tile_n = (int)(tile / (unsigned)tiles_m);
    const int m0 = tile_m * MD_M, n0 = tile_n * MD_N;
    // blockIdx.y = split of K: this workgroup multiplies k in [k_begin, k_begin + k_len) (the last split may be shorter)
    // and writes its sums to its own [M, N] array, y_split_bytes apart.  One split: k_len = K.
    const int k_begin = (int)blockIdx.y * k_len;
    const int kblocks = K / 32, nmac = min(k_len, K - k_begin) / MD_MAC;
    // 64-bit base of the tile's first row (and the split's first k): the per-lane offsets below stay within the tile's rows
    const uint8_t* const a_tile = reinterpret_cast<const uint8_t*>(a_dense) + ((size_t)m0 * K + k_begin) * 2;
    void* const y = static_cast<uint8_t*>(y_all) + (size_t)blockIdx.y * (size_t)y_split_bytes + (int64_t)blockIdx.z * gb.y;

    // A DMA: an instruction moves 1 KB = 4 rows; lane l fills position l % 16 of row 4 (8 w + j) + l / 16, which must
    // hold chunk (l % 16) ^ (row & 15).  Rows past M re-read row M - 1 (their products are never stored).
    uint32_t a_voff[A_DMAS];
#pragma unroll
    for (int j = 0; j < A_DMAS; ++j) {
        const int row = (wave * A_DMAS + j) * 4 + (lane >> 4);
        a_voff[j] = (uint32_t)(min(m0 + row, M - 1) - m0) * (uint32_t)K * 2u + (uint32_t)(((lane & 15) ^ (row & 15)) * 16);
    }
    // W: the wavefront loads 8 W_LOADS rows as whole lines: lane = 16 codes (16 k) of its row 8 h + (l >> 3)
    const int w_chunk = lane & 7;
    const uint8_t* const w_base = w_elements + (size_t)(n0 + wave * (8 * W_LOADS)) * K + k_begin;          // wave-uniform
    const uint8_t* const ws_base = w_scales + (size_t)(n0 + wave * (8 * W_LOADS)) * kblocks + k_begin / 32;
    uint32_t w_voff[W_LOADS], ws_voff[W_LOADS], w_lds_off[W_LOADS][2];
#pragma unroll
    for (int h = 0; h < W_LOADS; ++h) {
        const int rl = 8 * h + (lane >> 3), w_row = wave * (8 * W_LOADS) + rl;
        w_voff[h] = (uint32_t)rl * (uint32_t)K + (uint32_t)w_chunk * 16u;
        ws_voff[h] = (uint32_t)rl * (uint32_t)kblocks + (uint32_t)(w_chunk >> 1);
#pragma unroll
        for (int e = 0; e < 2; ++e) w_lds_off[h][e] = (uint32_t)w_row * MD_ROW + (uint32_t)(((2 * w_chunk + e) ^ (w_row & 15)) * 16);
    }
    // fragment reads: lane (g = l >> 5, r = l & 31) reads chunk 2 q + g of row 32 t + r for the 16-k step q
    uint32_t f_off[QW];
#pragma unroll
    for (int q = 0; q < QW; ++q)
        f_off[q] = (uint32_t)(lane & 31) * MD_ROW + (uint32_t)(((2 * (QW * wave_k + q) + (lane >> 5)) ^ (lane & 15)) * 16);

    floatx16 acc[2][2];  // [m-tile of the wavefront][n-tile]
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.0f;

    u32x4 w_raw[3][W_LOADS];
    uint32_t w_scale[3][W_LOADS];
    // workgroups start at different macro steps of K (and wrap around), so that at any moment they read different
    // columns of W and A: addresses that spread over the memory channels
    const int rot = (int)((unsigned)(tile_n + blockIdx.y) % (unsigned)nmac);
    // past the end the last macro step is read again (unused), which keeps the operation count per step, and with
    // it the wait counts, the same
    auto k_of = [&](int mac) __attribute__((always_inline)) {
        const int mc = min(mac, nmac - 1) + rot;
        return mc >= nmac ? mc - nmac : mc;
    };
    // (compile-time indices and forced inlining throughout: a run-time loop, even one that is unrolled later, or a
    // real call leaves the register ring and the accumulators in scratch memory, whose traffic the wait counts below
    // do not expect)
    auto issue_a = [&](int mac, auto stage_c) __attribute__((always_inline)) {
        constexpr int stage = decltype(stage_c)::value;
        const uint8_t* const a_src = a_tile + (size_t)k_of(mac) * (MD_MAC * 2);
        const uint32_t dst = lds_a_addr + (uint32_t)stage * MD_A_STAGE + (uint32_t)wave * (A_DMAS * 1024);
        static_for<A_DMAS>([&](auto j_c) __attribute__((always_inline)) {
            constexpr int j = decltype(j_c)::value;
            dma_1kb(dst + j * 1024, a_voff[j], a_src);
        });
    };
    auto issue_w = [&](int mac, auto slot_c) __attribute__((always_inline)) {
        constexpr int slot = decltype(slot_c)::value;
        const int mc = k_of(mac);
        static_for<W_LOADS>([&](auto h_c) __attribute__((always_inline)) {
            constexpr int h = decltype(h_c)::value;
            async_load16(w_raw[slot][h], w_voff[h], w_base + (size_t)mc * MD_MAC);
            async_load_u8(w_scale[slot][h], ws_voff[h], ws_base + mc * (MD_MAC / 32));
        });
    };
    // all but the N youngest vector-memory operations are done; ties ring slot `slot_c` to this point
    auto wait_slot = [&](auto slot_c, auto n_c) __attribute__((always_inline)) {
        constexpr int slot = decltype(slot_c)::value, PENDING = decltype(n_c)::value;
        static_for<W_LOADS>([&](auto h_c) __attribute__((always_inline)) {
            constexpr int h = decltype(h_c)::value;
            wait_vmcnt<PENDING>(w_raw[slot][h], w_scale[slot][h]);
        });
    };
    // compose the 16 codes of load h of ring slot `slot_c` into W stage `wstage_c`
    auto compose_h = [&](auto slot_c, auto wstage_c, auto h_c) __attribute__((always_inline)) {
        constexpr int slot = decltype(slot_c)::value, wstage = decltype(wstage_c)::value, h = decltype(h_c)::value;
        uint8_t* const st = lds_w + wstage * MD_W_STAGE;
        uint4 lo, hi;
        Composer<FW>::template compose16<true>(make_uint4(w_raw[slot][h].x, w_raw[slot][h].y, w_raw[slot][h].z, w_raw[slot][h].w),
                                               w_scale[slot][h], lo, hi);
        *reinterpret_cast<uint4*>(st + w_lds_off[h][0]) = lo;
        *reinterpret_cast<uint4*>(st + w_lds_off[h][1]) = hi;
    };

    // Issue groups: step s issues {A(s + 2), W(s + 3)}.  At the top of step s everything but the group of step s - 1
    // has arrived: A(s) is in LDS and W(s + 1) in registers; W(s + 1) is composed between the MFMAs of step s.
    issue_w(0, IntC<0>{});
    issue_a(0, IntC<0>{});
    issue_w(1, IntC<1>{});
    wait_slot(IntC<0>{}, IntC<0>{});
    wait_slot(IntC<1>{}, IntC<0>{});
    static_for<W_LOADS>([&](auto h_c) __attribute__((always_inline)) { compose_h(IntC<0>{}, IntC<0>{}, h_c); });
    issue_a(1, IntC<1>{});
    issue_w(2, IntC<2>{});
    for (int base = 0; base < nmac; base += 6) {
        static_for<6>([&](auto r_c) __attribute__((always_inline)) {
            constexpr int r = decltype(r_c)::value;
            const int mac = base + r;
            if (mac < nmac) {
                wait_slot(IntC<(r + 1) % 3>{}, IntC<OPS>{});
                __builtin_amdgcn_s_waitcnt(0xC07F);  // lgkmcnt(0): this wavefront's LDS reads and writes are done
                __builtin_amdgcn_s_barrier();        // this step's W and A stages are complete; last step's are no longer read
                // this step's loads (A(mac + 2) into the stage read last step, W(mac + 3) into the ring slot composed last
                // step) and the compose of W(mac + 1) are spread over the step's 32 MFMAs, a few instructions beside each:
                // instructions issue in order, so work placed behind a run of MFMAs would wait for the whole run
                constexpr int ns = r % 3, cs = (r + 1) % 3, a_stage = (r + 2) % 3, w_stage = (r + 1) % 2;
                const int mc_a = k_of(mac + 2), mc_w = k_of(mac + 3);
                const uint8_t* const a_src = a_tile + (size_t)mc_a * (MD_MAC * 2);
                const uint32_t a_dst = lds_a_addr + (uint32_t)a_stage * MD_A_STAGE + (uint32_t)wave * (A_DMAS * 1024);
                const uint8_t* const w_src = w_base + (size_t)mc_w * MD_MAC;
                const uint8_t* const ws_src = ws_base + mc_w * (MD_MAC / 32);
                auto vmem = [&](auto k_c) __attribute__((always_inline)) {  // operation k of the step's 16, A first
                    constexpr int k = decltype(k_c)::value;
                    if constexpr (k < A_DMAS) dma_1kb(a_dst + k * 1024, a_voff[k], a_src);
                    else if constexpr ((k - A_DMAS) % 2 == 0) async_load16(w_raw[ns][(k - A_DMAS) / 2], w_voff[(k - A_DMAS) / 2], w_src);
                    else async_load_u8(w_scale[ns][(k - A_DMAS) / 2], ws_voff[(k - A_DMAS) / 2], ws_src);
                };
                static_assert(OPS == 2 * QW, "two vector-memory operations beside each 16-k step");
                bool any_slow = false;
                static_for<W_LOADS>([&](auto h_c) __attribute__((always_inline)) { any_slow |= Composer<FW>::is_slow(w_scale[cs][decltype(h_c)::value]); });
                any_slow = __builtin_amdgcn_ballot_w64(any_slow) != 0;
                const uint8_t* const pa = lds_a + (r % 3) * MD_A_STAGE + wave_m * (64 * MD_ROW);
                const uint8_t* const pw = lds_w + (r % 2) * MD_W_STAGE + wave_n * (64 * MD_ROW);
                uint8_t* const st = lds_w + w_stage * MD_W_STAGE;
                bf16x8 wf[2][2], af[2][2];
                auto load_frags = [&](auto q_c) __attribute__((always_inline)) {
                    constexpr int q = decltype(q_c)::value;
#pragma unroll
                    for (int j = 0; j < 2; ++j) wf[q & 1][j] = *reinterpret_cast<const bf16x8*>(pw + j * (32 * MD_ROW) + f_off[q]);
#pragma unroll
                    for (int i = 0; i < 2; ++i) af[q & 1][i] = *reinterpret_cast<const bf16x8*>(pa + i * (32 * MD_ROW) + f_off[q]);
                };
                uint32_t o[8];
                load_frags(IntC<0>{});
                static_for<QW>([&](auto q_c) __attribute__((always_inline)) {
                    constexpr int q = decltype(q_c)::value, h = q / 2, d0 = 2 * (q % 2), b = q & 1;
                    // the next 16-k step's fragments are requested before this step's MFMAs
                    if constexpr (q < QW - 1) load_frags(IntC<q + 1>{});
                    const Composer<FW> cmp(w_scale[cs][h]);
                    const uint32_t c0 = w_raw[cs][h][d0], c1 = w_raw[cs][h][d0 + 1];
                    __builtin_amdgcn_sched_barrier(0);
                    acc[0][0] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(wf[b][0], af[b][0], acc[0][0], 0, 0, 0);
                    o[2 * d0] = cmp.pair_lo(c0);
                    vmem(IntC<2 * q>{});
                    __builtin_amdgcn_sched_barrier(0);
                    acc[0][1] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(wf[b][1], af[b][0], acc[0][1], 0, 0, 0);
                    o[2 * d0 + 1] = cmp.pair_hi(c0);
                    vmem(IntC<2 * q + 1>{});
                    __builtin_amdgcn_sched_barrier(0);
                    acc[1][0] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(wf[b][0], af[b][1], acc[1][0], 0, 0, 0);
                    o[2 * d0 + 2] = cmp.pair_lo(c1);
                    __builtin_amdgcn_sched_barrier(0);
                    acc[1][1] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(wf[b][1], af[b][1], acc[1][1], 0, 0, 0);
                    o[2 * d0 + 3] = cmp.pair_hi(c1);
                    if constexpr (q % 2 == 1) {  // the 16 codes of load h are done
                        uint4 lo = make_uint4(o[0], o[1], o[2], o[3]), hi = make_uint4(o[4], o[5], o[6], o[7]);
                        if (any_slow)
                            Composer<FW>::fix_slow(w_scale[cs][h], make_uint4(w_raw[cs][h].x, w_raw[cs][h].y, w_raw[cs][h].z, w_raw[cs][h].w), lo, hi);
                        *reinterpret_cast<uint4*>(st + w_lds_off[h][0]) = lo;
                        *reinterpret_cast<uint4*>(st + w_lds_off[h][1]) = hi;
                    }
                    __builtin_amdgcn_sched_barrier(0);
                });
            }
        });
    }
    // the look-ahead loads still target LDS and registers: let them finish
    wait_slot(IntC<0>{}, IntC<0>{});

    if constexpr (KS == 2) {
        // the upper-k wavefronts park their sums in LDS ([quadrant][i][j][v][lane]); the lower-k ones add them
        __syncthreads();  // every fragment read is done: the stages can be reused
        float* const red = reinterpret_cast<float*>(lds) + (wave & 3) * (64 * 64);
        if (wave_k == 1) {
#pragma unroll
            for (int i = 0; i < 2; ++i)
#pragma unroll
                for (int j = 0; j < 2; ++j)
#pragma unroll
                    for (int v = 0; v < 16; ++v) red[((i * 2 + j) * 16 + v) * 64 + lane] = acc[i][j][v];
        }
        __syncthreads();
        if (wave_k == 1) return;
#pragma unroll
        for (int i = 0; i < 2; ++i)
#pragma unroll
            for (int j = 0; j < 2; ++j)
#pragma unroll
                for (int v = 0; v < 16; ++v) acc[i][j][v] += red[((i * 2 + j) * 16 + v) * 64 + lane];
    }

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

template <class FW, int DT_OUT, int KS>
int launch_gemm_mid(const void* a_dense, const uint8_t* w_scales, const uint8_t* w_elements, const void* bias, int bias_dtype,
                    void* y, int M, int N, int K, int batches, const GemmBatch& gb, hipStream_t s) {
    auto kern = mxfp_gemm_mid_kernel<FW, DT_OUT, KS>;
    static std::atomic<uint64_t> lds_allowed{0};
    if (int rc = allow_dynamic_lds(reinterpret_cast<const void*>(kern), MD_LDS_BYTES, lds_allowed)) return rc;
    const int tiles_m = (M + MD_M - 1) / MD_M;
    const int64_t tiles = (int64_t)tiles_m * (N / MD_N);
    if (tiles > 0x7FFFFFFFll) return fail(ERR_UNSUPPORTED, "too many tiles for one launch");
    hipLaunchKernelGGL(kern, dim3((unsigned)tiles, 1u, (unsigned)batches), dim3(256 * KS), MD_LDS_BYTES, s, static_cast<const uint16_t*>(a_dense),
                       w_scales, w_elements, bias, bias_dtype, y, M, N, K, tiles_m, K, (int64_t)0, gb);
    return check_launch("mxfp_gemm");
}
