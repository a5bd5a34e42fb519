// Weight-streaming MXFP GEMM kernel for the fewest rows of A (decode shapes) and a moderate number of W rows: one
// workgroup per 16 rows of W.
//
// With a handful of A rows the product is a single pass over W.  A workgroup of the 32-row kernel walks K as a chain of
// macro steps (wait for the codes, compose, LDS round trip, barrier, MFMA), and there are only N / 32 of them: for
// N = 4096 half the CUs have none, and a long K makes every chain long.  This kernel halves the rows per workgroup
// (twice as many workgroups, half the compose per lane in the chain) by using the 16x16x32 MFMA: W rows are the 16
// rows of its first operand, up to 16 rows of A the 16 columns of its second, and one MFMA covers 32 k.
//   * W codes come as whole 128-byte lines (lane = 8 codes of one row, 16 lanes per row), are composed to bf16 in
//     registers and written to one of two 4 KB LDS stages;
//   * the matching 128 k of the A rows come global -> LDS by DMA into a ring of stages, D macro steps ahead;
//   * the macro step's four 32-k MFMA steps are split over the four wavefronts, whose partial sums are added
//     through LDS at the end.
// Loads are inline asm waited for with a counted s_waitcnt (vector memory completes in issue order); one barrier per
// macro step; workgroups start at different macro steps of K so that they read different columns at any moment.
// N = 4096, K = 14336: 28 / 40 us at M = 16 / 64 against 37 / 57 us for the 32-row kernels; no gain once N / 32 is a few
// hundred (N = 14336).
//
// LDS rows are 256 bytes (128 k of bf16), the 16-byte chunk c of row r at position c ^ (r & 15).
// (included from gemm_impl.h, inside namespace mase, after gemm_skinny.h)

constexpr int R16_N = 16;

typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
typedef float floatx4_t __attribute__((ext_vector_type(4)));

__device__ inline void async_load8(u32x2& dst, uint32_t voff, const void* sbase) {
    asm volatile("global_load_dwordx2 %0, %1, %2" : "=v"(dst) : "v"(voff), "s"(sbase) : "memory");
}
template <int N>
__device__ inline void wait_vmcnt8(u32x2& a, uint32_t& b) {
    asm volatile("s_waitcnt vmcnt(%2)" : "+v"(a), "+v"(b) : "n"(N) : "memory");
}

// MT = 16-row tiles of A (M <= 16 MT), D = look-ahead in macro steps
template <class FW, int DT_OUT, int MT, int D>
__global__ __launch_bounds__(kGemmThreads) void mxfp_gemm_rows16_kernel(
    const uint16_t* __restrict__ a_dense0, const uint8_t* __restrict__ w_scales0, const uint8_t* __restrict__ w_elements0,
    const void* __restrict__ bias, int bias_dtype, void* __restrict__ y0, int M, int N, int K, GemmBatch gb) {
    // batched launches: workgroups of grid plane z work on product z (offsets are zero for a single product)
    const uint16_t* __restrict__ const a_dense = a_dense0 + (int64_t)blockIdx.z * gb.a;
    const uint8_t* __restrict__ const w_scales = w_scales0 + (int64_t)blockIdx.z * gb.ws;
    const uint8_t* __restrict__ const w_elements = w_elements0 + (int64_t)blockIdx.z * gb.we;
    void* __restrict__ const y = static_cast<uint8_t*>(y0) + (int64_t)blockIdx.z * gb.y;
    constexpr int KM = 128, ROW = 2 * KM;
    constexpr int R = D + 1;                       // ring size: register sets of W, LDS stages of A
    constexpr int A_DMAS = MT;                     // per wavefront and macro step: 16 MT rows x 256 B / 1 KB / 4
    constexpr int OPS = A_DMAS + 2;                // vector-memory operations per wavefront and macro step
    constexpr int A_STAGE = 16 * MT * ROW, W_STAGE = R16_N * ROW;
    static_assert((D - 1) * OPS < 64, "vmcnt is a 6-bit counter");
    extern __shared__ __attribute__((aligned(1024))) uint8_t lds[];
    uint8_t* const lds_a = lds;                    // [R][16 MT rows][ROW]
    uint8_t* const lds_w = lds + R * A_STAGE;      // [2][16 rows][ROW]
    const uint32_t lds_a_addr = (uint32_t)(uintptr_t)lds;

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int n0 = blockIdx.x * R16_N;
    const int kblocks = K / 32, nmac = K / KM;

    // A DMA: an instruction moves 1 KB = 4 rows; lane l fills position l % 16 of row 4 (A_DMAS w + j) + l / 16, which must
    // hold chunk (l % 16) ^ (row & 15).  Rows past M re-read row M - 1.
    uint32_t a_voff[A_DMAS];
#pragma unroll
    for (int j = 0; j < A_DMAS; ++j) {
        const int row = (wave * A_DMAS + j) * 4 + (lane >> 4);
        a_voff[j] = (uint32_t)min(row, M - 1) * (uint32_t)K * 2u + (uint32_t)(((lane & 15) ^ (row & 15)) * 16);
    }
    // W: thread t loads the 8 codes at k 8 (t & 15) .. + 7 of row t >> 4; a wavefront covers four whole lines
    const int w_row = tid >> 4, w_piece = tid & 15;
    const uint8_t* const w_base = w_elements + (size_t)n0 * K;
    const uint8_t* const ws_base = w_scales + (size_t)n0 * kblocks;
    const uint32_t w_voff = (uint32_t)w_row * (uint32_t)K + (uint32_t)w_piece * 8u;
    const uint32_t ws_voff = (uint32_t)w_row * (uint32_t)kblocks + (uint32_t)(w_piece >> 2);
    const uint32_t w_lds_off = (uint32_t)w_row * ROW + (uint32_t)((w_piece ^ (w_row & 15)) * 16);
    // fragment reads of the 16x16x32 MFMA: lane (g = l >> 4, r = l & 15) holds k 8 g .. 8 g + 7 of row r of the 32-k
    // step; this wavefront owns step `wave` of the macro step's four: chunk 4 wave + g
    const uint32_t f_off = (uint32_t)(lane & 15) * ROW + (uint32_t)(((4 * wave + (lane >> 4)) ^ (lane & 15)) * 16);

    floatx4_t acc[MT];
#pragma unroll
    for (int t = 0; t < MT; ++t) acc[t] = floatx4_t{0.0f, 0.0f, 0.0f, 0.0f};

    u32x2 w_raw[R];
    uint32_t w_scale[R];
    const int rot = (int)(blockIdx.x % (unsigned)nmac);
    // loads of macro step `mac` into ring slot `slot_c`; past the end the last macro step is read again (unused),
    // which keeps the number of operations per step, and with it the wait counts, the same
    auto issue_loads = [&](int mac, auto slot_c) __attribute__((always_inline)) {
        constexpr int slot = decltype(slot_c)::value;
        int mc = min(mac, nmac - 1) + rot;
        if (mc >= nmac) mc -= nmac;
        async_load8(w_raw[slot], w_voff, w_base + (size_t)mc * KM);
        async_load_u8(w_scale[slot], ws_voff, ws_base + mc * (KM / 32));
        const uint8_t* const a_src = reinterpret_cast<const uint8_t*>(a_dense) + (size_t)mc * (KM * 2);
        const uint32_t dst = lds_a_addr + (uint32_t)slot * A_STAGE + (uint32_t)wave * (A_DMAS * 1024);
        static_for<A_DMAS>([&](auto j_c) __attribute__((always_inline)) {
            constexpr int j = decltype(j_c)::value;
            dma_1kb(dst + j * 1024, a_voff[j], a_src);
        });
    };
    // the loads of the macro step in ring slot `slot_c` have arrived (D - 1 younger steps may still be in flight):
    // compose its W into stage `mac & 1`
    auto stage_w = [&](int mac, auto slot_c) __attribute__((always_inline)) {
        constexpr int slot = decltype(slot_c)::value;
        wait_vmcnt8<(D - 1) * OPS>(w_raw[slot], w_scale[slot]);
        const uint32_t scale = w_scale[slot];
        const Composer<FW> cmp(scale);
        uint32_t o[4];
        cmp.pair2(w_raw[slot].x, o[0], o[1]);
        cmp.pair2(w_raw[slot].y, o[2], o[3]);
        if (__builtin_amdgcn_ballot_w64(Composer<FW>::is_slow(scale)) != 0 && Composer<FW>::is_slow(scale)) {
            // rare scales (255, "times +inf" in the reference, among them) that the fast compose does not take
            cmp.pair2_slow(w_raw[slot].x, o[0], o[1]);
            cmp.pair2_slow(w_raw[slot].y, o[2], o[3]);
        }
        *reinterpret_cast<uint4*>(lds_w + (mac & 1) * W_STAGE + w_lds_off) = make_uint4(o[0], o[1], o[2], o[3]);
    };

    static_for<D>([&](auto d_c) __attribute__((always_inline)) { issue_loads(decltype(d_c)::value, d_c); });
    stage_w(0, IntC<0>{});
    for (int base = 0; base < nmac; base += R) {
        static_for<R>([&](auto r_c) __attribute__((always_inline)) {
            constexpr int r = decltype(r_c)::value;
            const int mac = base + r;
            if (mac < nmac) {
                __builtin_amdgcn_s_waitcnt(0xC07F);  // lgkmcnt(0): this wavefront's LDS reads and writes are done
                __builtin_amdgcn_s_barrier();        // W stage mac & 1 and A slot r are complete; slot r - 1 is no longer read
                issue_loads(mac + D, IntC<(r + D) % R>{});
                const uint8_t* const pa = lds_a + r * A_STAGE;
                const uint8_t* const pw = lds_w + (mac & 1) * W_STAGE;
                // the fragment reads go out, the next step's W is composed while they are in flight, then the MFMAs
                const bf16x8 wf = *reinterpret_cast<const bf16x8*>(pw + f_off);
                bf16x8 af[MT];
#pragma unroll
                for (int t = 0; t < MT; ++t) af[t] = *reinterpret_cast<const bf16x8*>(pa + t * (16 * ROW) + f_off);
                __builtin_amdgcn_sched_barrier(0);
                stage_w(mac + 1, IntC<(r + 1) % R>{});  // (past the end: composes the re-read step into the unused stage)
                __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                for (int t = 0; t < MT; ++t) acc[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wf, af[t], acc[t], 0, 0, 0);
            }
        });
    }
    // the look-ahead loads still target LDS and registers: let them finish
    wait_vmcnt8<0>(w_raw[0], w_scale[0]);

    // ---- add the four wavefronts' partial sums: wavefronts 1..3 park theirs in LDS ([w-1][t][v][lane]), 0 adds
    __syncthreads();  // every fragment read is done: the stages can be reused
    float* const red = reinterpret_cast<float*>(lds);
    if (wave != 0) {
#pragma unroll
        for (int t = 0; t < MT; ++t)
#pragma unroll
            for (int v = 0; v < 4; ++v) red[(((wave - 1) * MT + t) * 4 + v) * 64 + lane] = acc[t][v];
    }
    __syncthreads();
    if (wave != 0) return;
#pragma unroll
    for (int w = 0; w < 3; ++w)
#pragma unroll
        for (int t = 0; t < MT; ++t)
#pragma unroll
            for (int v = 0; v < 4; ++v) acc[t][v] += red[((w * MT + t) * 4 + v) * 64 + lane];

    // lane holds, for m-tile t, y[m][n .. n+3] with m = 16 t + lane % 16, n = n0 + 4 (lane / 16)
    const bool vec_ok = (N % 4 == 0) && (reinterpret_cast<uintptr_t>(y) & 15) == 0;
    const int n = n0 + 4 * (lane >> 4);
    float b[4] = {0.0f, 0.0f, 0.0f, 0.0f};
    if (bias)
        for (int t = 0; t < 4; ++t) b[t] = load_bias(bias, bias_dtype, n + t);
#pragma unroll
    for (int t = 0; t < MT; ++t) {
        const int m = 16 * t + (lane & 15);
        if (m < M) {
            const float r[4] = {acc[t][0] + b[0], acc[t][1] + b[1], acc[t][2] + b[2], acc[t][3] + b[3]};
            store_out4<DT_OUT>(y, (int64_t)m * N + n, r, vec_ok, 4);
        }
    }
}

template <class FW, int DT_OUT, int MT, int D>
int launch_gemm_rows16(const void* a_dense, const uint8_t* w_scales, const uint8_t* w_elements, const void* bias, int bias_dtype,
                       void* y, int M, int N, int K, int batches, const GemmBatch& gb, hipStream_t s) {
    constexpr int lds_bytes = (D + 1) * 16 * MT * 256 + 2 * R16_N * 256;  // >= the 3 MT KB the final reduction needs
    auto kern = mxfp_gemm_rows16_kernel<FW, DT_OUT, MT, D>;
    static std::atomic<uint64_t> lds_allowed{0};
    if (int rc = allow_dynamic_lds(reinterpret_cast<const void*>(kern), lds_bytes, lds_allowed)) return rc;
    hipLaunchKernelGGL(kern, dim3((unsigned)(N / R16_N), 1u, (unsigned)batches), dim3(kGemmThreads), lds_bytes, s,
                       static_cast<const uint16_t*>(a_dense), w_scales, w_elements, bias, bias_dtype, y, M, N, K, gb);
    return check_launch("mxfp_gemm");
}
