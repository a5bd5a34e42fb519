// Block-scaled MXFP GEMM for a few rows of A (decode-sized calls: M <= 64):  y[M,N] = A[M,K] * W[N,K]^T (+ bias) as a
// read of W.  Operands in the prepared form of gemm_scaled.h (FP8 bytes [rows_pad, K], scales [K/128][rows_pad] dwords).
//
// The product is bound by HBM: W is N * K * 33/32 bytes, read once, against 2 M N K flop.  With the block-scaled
// instruction a wavefront turns 2 KB of W (16 rows x 128 k) into one MFMA without a single VALU instruction on the
// codes (the bf16 kernels for this size compose every code to bf16 first and are bound by that), so the kernel is
// loads and a few MFMAs.  What decides its speed is the shape of the loads.  Measured with bare read kernels on 58.7 MB
// (N x K = 14336 x 4096), a workgroup per 16 rows: a lane-for-lane load of the instruction's operand layout (16 rows x 64
// bytes per load instruction, the rows K bytes apart: rows a power of two apart land on the same L2 channel) takes
// 15.6 us, 1 KB of one row per instruction 14.1 us, the plain linear read of the same bytes 9.8 us.  So:
//   * a workgroup owns 16 rows of W over all of K and walks K in chunks of 1 KB per row; a load instruction of a wavefront
//     is 1 KB of ONE row (wave w: rows 4 w .. 4 w + 3 of W, and of each 16-row tile of A), two chunks ahead in registers;
//   * the chunk goes through LDS (rows 1040 bytes apart: conflict-free 128-bit writes and fragment reads) and comes
//     back as operand fragments: lane 16 g + r reads pieces g and g + 4 of row r of a 128-k macro step; wave w multiplies
//     the chunk's macro steps 2 w and 2 w + 1, its scale dwords straight from global memory (16 rows = 64 contiguous bytes);
//   * the wavefronts' partial sums meet in LDS at the end.
// A (at most a few hundred KB, shared by every workgroup) takes the same route from L2.  Two kernels: this one streams A
// beside W (any K, M <= 32); the other keeps A in registers (M <= 64, K <= 4096, or from 17 rows a longer K in slices).
// (included from gemm_impl.h's namespace, after gemm_scaled.h's typedefs)

// the same instruction as mfma_scaled with the accumulator in ordinary registers (a kernel that asks for accumulation
// registers gets its register budget split in two halves, and this one needs the ordinary half whole); the leading s_nop
// keeps VALU writes of the scale operands (v_bfe) clear of the matrix instruction's read of them, which the compiler cannot
// see inside an asm statement
__device__ inline void mfma_scaled_after_valu(floatx4& c, const intx8& w, const intx8& a, uint32_t sw, uint32_t sa) {
    asm volatile("s_nop 3\n\tv_mfma_scale_f32_16x16x128_f8f6f4 %0, %1, %2, %0, %3, %4 op_sel_hi:[0,0,0]" : "+v"(c) : "v"(w), "v"(a), "v"(sw), "v"(sa));
}

constexpr int SR_CHUNK = 1024;            // bytes of k per row and chunk: 8 macro steps
constexpr int SR_ROW = SR_CHUNK + 16;     // LDS row pitch

template <int MB>
struct RowsChunk {
    intx4 w[4], a[MB][4];                 // this wave's four rows of W and of each A tile: 16 bytes per lane and row
    uint32_t w_sc[2], a_sc[MB][2];        // scale dwords of the wave's two macro steps (row = lane & 15)
};

// OCC: wavefronts per SIMD the register budget is set for (workgroups per CU)
template <int DT_OUT, int MB, int OCC>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(OCC, OCC))) void mxfp_gemm_scaled_rows_kernel(const uint8_t* __restrict__ a_codes, const uint32_t* __restrict__ a_scales,
                                                                    const uint8_t* __restrict__ w_codes, const uint32_t* __restrict__ w_scales,
                                                                    const void* __restrict__ bias, int bias_dtype, void* __restrict__ y, int M, int N,
                                                                    int K, int rows_a, int rows_w) {
    __shared__ __attribute__((aligned(16))) uint8_t tile[(16 + 16 * MB) * SR_ROW];   // W rows 0..15, then the A tiles
    __shared__ float red[3][MB][256];
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int g = lane >> 4, r = lane & 15;
    const int n0 = blockIdx.x * 16;
    const int nmac = K / 128;
    const int nchunk = (K + SR_CHUNK - 1) / SR_CHUNK;

    // global side: lane l reads bytes 16 l .. 16 l + 15 of a row's chunk (uniform row addresses, a 32-bit lane offset)
    const uint8_t* const w_src = w_codes + (size_t)(n0 + 4 * wave) * K;
    const uint8_t* const a_src = a_codes + (size_t)(4 * wave) * K;
    const uint32_t* const w_sc_src = w_scales + n0;
    // Every step issues the same loads, whatever its chunk (the compiler can then count exactly which loads a step has to
    // wait for and leaves the younger chunk in flight): a chunk past the end reads one line, the lanes past the end of a K
    // that is not a multiple of 1 KB their row's first bytes; what they bring is never multiplied.
    auto issue = [&](RowsChunk<MB>& c, int chunk) __attribute__((always_inline)) {
        const bool live = chunk < nchunk;                                   // uniform
        const uint32_t k = live ? (uint32_t)chunk * SR_CHUNK : 0u;
        const uint32_t off = live && k + 16u * lane < (uint32_t)K ? k + 16u * lane : 0u;
        const size_t pitch = live ? (size_t)K : 0;                          // a chunk past the end: one line for the whole wavefront
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            c.w[i] = __builtin_nontemporal_load(reinterpret_cast<const intx4*>(w_src + i * pitch + off));
#pragma unroll
            for (int mb = 0; mb < MB; ++mb) c.a[mb][i] = *reinterpret_cast<const intx4*>(a_src + (16 * mb + i) * pitch + off);
        }
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            const int mac = min(chunk * 8 + 2 * wave + j, nmac - 1);
            c.w_sc[j] = __builtin_nontemporal_load(w_sc_src + (size_t)mac * rows_w + r);
#pragma unroll
            for (int mb = 0; mb < MB; ++mb) c.a_sc[mb][j] = a_scales[(size_t)mac * rows_a + 16 * mb + r];
        }
    };
    // LDS side
    uint8_t* const st_w = tile + (4 * wave) * SR_ROW + 16 * lane;
    uint8_t* const st_a = tile + (16 + 4 * wave) * SR_ROW + 16 * lane;
    const uint8_t* const frag_w = tile + r * SR_ROW + 16 * g;
    const uint8_t* const frag_a = tile + (16 + r) * SR_ROW + 16 * g;

    floatx4 acc[MB];
#pragma unroll
    for (int mb = 0; mb < MB; ++mb) acc[mb] = floatx4{0.0f, 0.0f, 0.0f, 0.0f};

    auto step = [&](RowsChunk<MB>& c, int chunk) __attribute__((always_inline)) {
        __syncthreads();                                   // the fragment reads of the chunk before are done
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            *reinterpret_cast<intx4*>(st_w + i * SR_ROW) = c.w[i];
#pragma unroll
            for (int mb = 0; mb < MB; ++mb) *reinterpret_cast<intx4*>(st_a + (16 * mb + i) * SR_ROW) = c.a[mb][i];
        }
        uint32_t w_sc[2], a_sc[MB][2];
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            w_sc[j] = c.w_sc[j];
#pragma unroll
            for (int mb = 0; mb < MB; ++mb) a_sc[mb][j] = c.a_sc[mb][j];
        }
        issue(c, chunk + 2);
        __builtin_amdgcn_sched_barrier(0);
        __syncthreads();
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            const int ms = 2 * wave + j;
            if (chunk * 8 + ms < nmac) {
                const intx4 w_lo = *reinterpret_cast<const intx4*>(frag_w + ms * 128), w_hi = *reinterpret_cast<const intx4*>(frag_w + ms * 128 + 64);
                const intx8 wf = __builtin_shufflevector(w_lo, w_hi, 0, 1, 2, 3, 4, 5, 6, 7);
                const uint32_t sw = (w_sc[j] >> (8 * g)) & 0xFFu;
#pragma unroll
                for (int mb = 0; mb < MB; ++mb) {
                    const uint8_t* fa = frag_a + 16 * mb * SR_ROW + ms * 128;
                    const intx4 a_lo = *reinterpret_cast<const intx4*>(fa), a_hi = *reinterpret_cast<const intx4*>(fa + 64);
                    const intx8 af = __builtin_shufflevector(a_lo, a_hi, 0, 1, 2, 3, 4, 5, 6, 7);
                    mfma_scaled_after_valu(acc[mb], wf, af, sw, (a_sc[mb][j] >> (8 * g)) & 0xFFu);
                }
            }
        }
    };

    RowsChunk<MB> c0, c1;
    issue(c0, 0);
    __builtin_amdgcn_sched_barrier(0);
    issue(c1, 1);
    __builtin_amdgcn_sched_barrier(0);
    for (int chunk = 0; chunk < nchunk; chunk += 2) {      // (an odd count ends with a step that multiplies nothing)
        step(c0, chunk);
        step(c1, chunk + 1);
    }
    // the matrix unit's last results must have left its pipeline before ordinary instructions read the accumulators
    asm volatile("s_nop 15\n\ts_nop 15" ::: "memory");

    // ---- add the wavefronts' partial sums (lane l holds n = 4 (l >> 4) + v, m = l & 15 of each 16 x 16 tile) and store
    if (wave > 0) {
#pragma unroll
        for (int mb = 0; mb < MB; ++mb) *reinterpret_cast<floatx4*>(&red[wave - 1][mb][lane * 4]) = acc[mb];
    }
    __syncthreads();
    if (wave == 0) {
        const int n = n0 + 4 * g;
#pragma unroll
        for (int mb = 0; mb < MB; ++mb) {
            floatx4 s = acc[mb];
#pragma unroll
            for (int w = 0; w < 3; ++w) s += *reinterpret_cast<const floatx4*>(&red[w][mb][lane * 4]);
            const int m = 16 * mb + r;
            if (m < M && n < N) {
                float out[4] = {s[0], s[1], s[2], s[3]};
                const int valid = min(4, N - n);
                if (bias)
                    for (int t = 0; t < valid; ++t) out[t] += load_bias(bias, bias_dtype, n + t);
                store_out4<DT_OUT>(y, (int64_t)m * N + n, out, true, valid);
            }
        }
    }
}

// ---- The persistent kernels: K <= 4096 (or a slice of K that long), workgroups that stay (one per CU) and take 16 whole
// rows of W x all of K per unit, as whole rows (the shape that reads fastest), one unit ahead in registers.
constexpr int SRR_ROW = 4096 + 16;        // LDS row pitch: K <= 4096 bytes and 16 of padding (conflict-free 128-bit accesses)

// How the persistent kernels below deal the row groups of W (16 rows each) to their workgroups.  Whole rounds first: group
// b + u * grid is unit u of workgroup b.  What is left after the whole rounds, when it is at most half a round, is dealt in
// HALF units: eight rows of a group each (the matrix instruction still multiplies sixteen; the other eight are whatever
// the buffer holds and their results are not stored), two workgroups to a group, so that a tail of L groups keeps 2 L CUs
// busy for half a unit's time instead of L CUs for a whole one (N = 14336 on 256 CUs: 3.5 rounds instead of 4).
struct RowsDeal {
    int grid, full_rounds, tail_halves;   // workgroups; units every workgroup takes; workgroups that take a half unit after them
};
inline RowsDeal deal_row_groups(int groups, int cus) {
    const int full = groups / cus, left = groups - full * cus;
    if (left > 0 && 2 * left <= cus) return RowsDeal{full > 0 ? cus : 2 * left, full, 2 * left};
    return RowsDeal{min(groups, cus), 0, 0};      // whole units only: unit u of workgroup b is group b + u * grid while there are groups
}
// unit u of workgroup b: its group, and which half of it (-1: all sixteen rows)
struct RowsUnit { int group, half; };
__device__ inline int rows_unit_count(int b, int grid, int groups, int full_rounds, int tail_halves) {
    if (tail_halves > 0) return full_rounds + (b < tail_halves ? 1 : 0);
    return b < groups ? (groups - b + grid - 1) / grid : 0;
}
__device__ inline RowsUnit rows_unit(int b, int u, int grid, int full_rounds, int tail_halves) {
    if (tail_halves > 0 && u >= full_rounds) return RowsUnit{full_rounds * grid + (b >> 1), b & 1};
    return RowsUnit{b + u * grid, -1};
}

// ---- A in registers (K <= 4096, M <= 16 MT, MT = 1, 2 or 4 operand tiles of 16 rows: up to 64 rows of A).  A wavefront
// multiplies the same macro steps of every unit (wave w: SPW w .. SPW w + SPW - 1, SPW = 32 / WAVES), so the fragments of
// A it needs are the same for the whole launch: MT x SPW x 8 registers (128 for four tiles on eight wavefronts), filled
// once.  LDS holds W alone (rows 4112 bytes apart: conflict-free 128-bit writes and fragment reads) and no byte of A is
// read a second time.  W: 1 KB of one row per load instruction, one unit ahead in registers, through LDS; so does A on its
// way to the registers, tile by tile through W's place in LDS (read straight from global memory in the operand layout, 64
// bytes of a row at a time, every cache line is fetched twice, and with every CU of an XCD asking its L2 for the same A
// that is what the prologue costs: 22 against 19 us at 64 rows, N x K = 14336 x 4096).  The wavefronts' partial sums meet
// in LDS; wavefront t adds and stores tile t.  Eight wavefronts: 15.6 against 18.4 us with four at 32 rows (sixteen: the
// same, and the registers of four tiles no longer fit).  N x K = 14336 x 4096: 14.0 / 15.6 / 19.2 us at 16 / 32 / 64 rows against
// 20.9 / 23.2 / 30.8 on the bf16 weight-streaming kernels (23.8 / 26.9 at 32 / 64 rows on the chunked and the tile kernel); 4096 x
// 4096: 6.8 / 7.6 / 10.0 against 9.7 / 10.7 / 16.9.  (A build that kept 16 rows of A in LDS instead, four wavefronts: 14.8 us at
// 16 rows where this one takes 14.0, same box.)
// W by DMA into two LDS units, the next but one asked for before the wait for the next (one to two units in flight per CU,
// no registers on the way), measured 15.1 / 16.4 / 19.9 us at 16 / 32 / 64 rows: no faster, so the time is not in a pipe that runs
// dry between units; nor is it in the last round (half units, above: 0.1 - 0.4 us).  Launch, the first unit's latency,
// the prologue of A and the last reduction are about 4 of the 14 us.
constexpr int SRG_WAVES = 8;

template <int DT_OUT, int MT, int WAVES>
__global__ __launch_bounds__(WAVES * 64) __attribute__((amdgpu_waves_per_eu(WAVES / 4, WAVES / 4))) void mxfp_gemm_scaled_rows_regs_kernel(
    const uint8_t* __restrict__ a_codes, const uint32_t* __restrict__ a_scales, const uint8_t* __restrict__ w_codes,
    const uint32_t* __restrict__ w_scales, const void* __restrict__ bias, int bias_dtype, void* __restrict__ y, int M, int N, int K, int rows_a,
    int rows_w, int slices, int slice_macs, float* __restrict__ partial, int full_rounds, int tail_halves) {
    constexpr int SPW = 32 / WAVES;          // macro steps of a unit per wavefront
    constexpr int RPW = 16 / WAVES;          // rows of W a wavefront carries from global memory to LDS
    extern __shared__ __attribute__((aligned(16))) uint8_t lds[];            // W [16][SRR_ROW], partial sums [WAVES][MT][256]
    uint8_t* const tile_w = lds;
    float (*const red)[MT][256] = reinterpret_cast<float (*)[MT][256]>(lds + 16 * SRR_ROW);
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int g = lane >> 4, r = lane & 15;
    // A K beyond 4096 is cut into `slices` pieces of `slice_macs` macro steps (the last one may be shorter): a workgroup stays
    // with ONE slice (its share of A in registers is that slice's) and walks the row groups of W with the workgroups of the
    // same slice; the slices' sums go to `partial` [slices][M][N] as fp32 and a second kernel adds them.  slices == 1: the
    // whole K, results straight to y.
    const int slice = (int)blockIdx.x % slices, first_group = (int)blockIdx.x / slices, group_step = (int)gridDim.x / slices;
    const int mac0 = slice * slice_macs;
    const int nmac = min(slice_macs, K / 128 - mac0);            // this slice's macro steps: at most 32
    const size_t k0 = (size_t)mac0 * 128;
    const int groups = (N + 15) / 16;
    const int units = rows_unit_count(first_group, group_step, groups, full_rounds, tail_halves);      // (half units: one slice only)
    uint32_t off[4];
#pragma unroll
    for (int q = 0; q < 4; ++q) off[q] = min(1024u * q + 16u * lane, (uint32_t)nmac * 128u - 16u);
    a_codes += k0;
    w_codes += k0;
    a_scales += (size_t)mac0 * rows_a;
    w_scales += (size_t)mac0 * rows_w;

    intx4 wreg[RPW][4];
    uint32_t w_sc_next[SPW];
    auto issue = [&](int u) __attribute__((always_inline)) {
        // (plain arithmetic: a unit past the end, or the rows of the half that a half unit leaves out, have pitch 0 and
        // offset 0: every lane of a wavefront reads the same line)
        const RowsUnit ru = rows_unit(first_group, u, group_step, full_rounds, tail_halves);
        const uint32_t live = u < units && (ru.half < 0 || (RPW * wave >> 3) == ru.half) ? 1u : 0u;      // this wavefront's rows: RPW wave .. + RPW - 1
        const int group = u < units ? ru.group : 0;
        const uint8_t* row0 = w_codes + (size_t)live * (size_t)(group * 16 + RPW * wave) * K;
        const size_t pitch = (size_t)live * (size_t)K;
#pragma unroll
        for (int i = 0; i < RPW; ++i)
#pragma unroll
            for (int q = 0; q < 4; ++q) wreg[i][q] = __builtin_nontemporal_load(reinterpret_cast<const intx4*>(row0 + i * pitch + live * off[q]));
#pragma unroll
        for (int j = 0; j < SPW; ++j)
            w_sc_next[j] = __builtin_nontemporal_load(w_scales + (size_t)min(SPW * wave + j, nmac - 1) * rows_w + group * 16 + r);
    };
    // ---- this wavefront's fragments of A and their scale bytes, once.  A tile takes W's route (whole 1 KB pieces of a row per
    // load instruction, through LDS): read in the operand layout straight from global memory, 64 bytes of a row at a time,
    // every cache line is fetched twice, and with every CU of an XCD asking for the same A that is what the prologue costs
    // (a macro step past the end of K: the last one's bytes, under scale bytes 0 on W's side)
    const uint8_t* const frag_w = tile_w + r * SRR_ROW + 16 * g;
    intx8 af[MT][SPW];
    uint32_t a_sc[MT][SPW], keep[SPW];
#pragma unroll
    for (int j = 0; j < SPW; ++j) keep[j] = SPW * wave + j < nmac ? 0xFFu : 0u;
    intx4 areg[2][RPW][4];                                      // a tile's rows on their way to LDS, the next tile's behind them
    auto load_a = [&](int t) __attribute__((always_inline)) {
#pragma unroll
        for (int i = 0; i < RPW; ++i)
#pragma unroll
            for (int q = 0; q < 4; ++q) areg[t & 1][i][q] = *reinterpret_cast<const intx4*>(a_codes + (size_t)(16 * t + RPW * wave + i) * K + off[q]);
#pragma unroll
        for (int j = 0; j < SPW; ++j) a_sc[t][j] = a_scales[(size_t)min(SPW * wave + j, nmac - 1) * rows_a + 16 * t + r];
    };
    load_a(0);
#pragma unroll
    for (int t = 0; t < MT; ++t) {
        __builtin_amdgcn_sched_barrier(0);
        if (t + 1 < MT) load_a(t + 1);
        __builtin_amdgcn_sched_barrier(0);
        if (t > 0) __syncthreads();                              // the fragment reads of the tile before are done
#pragma unroll
        for (int i = 0; i < RPW; ++i)
#pragma unroll
            for (int q = 0; q < 4; ++q) *reinterpret_cast<intx4*>(tile_w + (RPW * wave + i) * SRR_ROW + 1024 * q + 16 * lane) = areg[t & 1][i][q];
        if (t == MT - 1) {
            __builtin_amdgcn_sched_barrier(0);
            issue(0);
            __builtin_amdgcn_sched_barrier(0);
        }
        __syncthreads();
#pragma unroll
        for (int j = 0; j < SPW; ++j) {
            const int ms = min(SPW * wave + j, nmac - 1);
            const intx4 lo = *reinterpret_cast<const intx4*>(frag_w + ms * 128), hi = *reinterpret_cast<const intx4*>(frag_w + ms * 128 + 64);
            af[t][j] = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
            a_sc[t][j] = (a_sc[t][j] >> (8 * g)) & keep[j];     // (both sides' scale bytes 0 past the end of K: the product underflows to 0)
        }
    }
    for (int u = 0; u < units; ++u) {
        const RowsUnit ru = rows_unit(first_group, u, group_step, full_rounds, tail_halves);
        const int group = ru.group;
        __syncthreads();                                         // the reads of the unit before (fragments, partial sums) are done
#pragma unroll
        for (int i = 0; i < RPW; ++i)
#pragma unroll
            for (int q = 0; q < 4; ++q) *reinterpret_cast<intx4*>(tile_w + (RPW * wave + i) * SRR_ROW + 1024 * q + 16 * lane) = wreg[i][q];
        uint32_t w_sc[SPW];
#pragma unroll
        for (int j = 0; j < SPW; ++j) w_sc[j] = (w_sc_next[j] >> (8 * g)) & keep[j];
        __builtin_amdgcn_sched_barrier(0);
        issue(u + 1);
        __builtin_amdgcn_sched_barrier(0);
        __syncthreads();
        floatx4 acc[MT];
#pragma unroll
        for (int t = 0; t < MT; ++t) acc[t] = floatx4{0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
        for (int j = 0; j < SPW; ++j) {
            const int ms = SPW * wave + j;
            const intx4 w_lo = *reinterpret_cast<const intx4*>(frag_w + ms * 128), w_hi = *reinterpret_cast<const intx4*>(frag_w + ms * 128 + 64);
            const intx8 wf = __builtin_shufflevector(w_lo, w_hi, 0, 1, 2, 3, 4, 5, 6, 7);
#pragma unroll
            for (int t = 0; t < MT; ++t) mfma_scaled_after_valu(acc[t], wf, af[t][j], w_sc[j], a_sc[t][j]);
        }
        asm volatile("s_nop 15\n\ts_nop 15" ::: "memory");     // the matrix unit's last results have left its pipeline
#pragma unroll
        for (int t = 0; t < MT; ++t) *reinterpret_cast<floatx4*>(&red[wave][t][lane * 4]) = acc[t];
        __syncthreads();
        // wavefront t adds tile t (lane l holds n = 4 (l >> 4) + v, m = l & 15 of it) and stores it
        if (wave < MT) {
            const int t = wave;
            floatx4 s = *reinterpret_cast<const floatx4*>(&red[0][t][lane * 4]);
#pragma unroll
            for (int w = 1; w < WAVES; ++w) s += *reinterpret_cast<const floatx4*>(&red[w][t][lane * 4]);
            const int n = group * 16 + 4 * g, m = 16 * t + r;
            if (m < M && n < N && (ru.half < 0 || (g >> 1) == ru.half)) {
                float out[4] = {s[0], s[1], s[2], s[3]};
                const int valid = min(4, N - n);
                if (partial) {
                    float* const dst = partial + ((size_t)slice * M + m) * N + n;
                    for (int v = 0; v < valid; ++v) dst[v] = out[v];
                } else {
                    if (bias)
                        for (int v = 0; v < valid; ++v) out[v] += load_bias(bias, bias_dtype, n + v);
                    store_out4<DT_OUT>(y, (int64_t)m * N + n, out, true, valid);
                }
            }
        }
    }
}

// the shapes these kernels take without room for partial sums: up to 32 rows of A (two 16-row operand tiles), up to 64 when
// a wavefront's share of A fits its registers in one piece
inline bool scaled_rows_shape_ok(int M, int K) { return K >= 128 && (M <= 32 || (M <= 64 && K <= 4096)); }

// K beyond what a wavefront's registers hold of A in one piece, 17 - 64 rows: slices of at most 32 macro steps, their sums added
// by a second kernel (room for them: slices * M * N * 4 bytes).  0: not a shape for this.  N x K = 4096 x 14336: 18.4 / 23.0 us
// at 32 / 64 rows against 23.3 (the chunked kernel) / 31.0 (the tile kernel, K split) and 27.8 / 49.4 on the bf16 kernels; 8192 x
// 8192: 19.4 / 24.4 against 23.2 / 30.2 and 29.5 / 42.6.  (Up to 16 rows the chunked kernel is level: 17.7 us, one launch.)
inline int scaled_rows_slices(int M, int N, int K) {
    if (M <= 16 || M > 64 || K <= 4096 || K % 128 != 0 || N % 4 != 0) return 0;
    return (K / 128 + 31) / 32;
}

template <int DT_OUT>
int launch_gemm_scaled_rows_sliced(const uint8_t* a_codes, const uint32_t* a_scales, const uint8_t* w_codes, const uint32_t* w_scales, const void* bias,
                                   int bias_dtype, void* y, int M, int N, int K, float* partial, hipStream_t s) {
    const int rows_a = (M + 255) / 256 * 256, rows_w = (N + 255) / 256 * 256;
    const int groups = (N + 15) / 16, slices = scaled_rows_slices(M, N, K), slice_macs = (K / 128 + slices - 1) / slices;
    const int cus = device_cu_count();
    if (cus <= 0) return fail(ERR_RUNTIME, "cannot read the compute-unit count of the current device");
    auto go = [&](auto kern, int mt, std::atomic<uint64_t>& allowed) {
        const int lds_bytes = max(16 * SRR_ROW + SRG_WAVES * mt * 256 * (int)sizeof(float), 84 * 1024);
        if (int rc = allow_dynamic_lds(reinterpret_cast<const void*>(kern), lds_bytes, allowed)) return rc;
        // as many workgroups per slice as fill the CUs between them (every slice the same count)
        const int per_slice = max(1, min(groups, cus / slices));
        hipLaunchKernelGGL(kern, dim3((unsigned)(per_slice * slices)), dim3(SRG_WAVES * 64), lds_bytes, s, a_codes, a_scales, w_codes, w_scales,
                           static_cast<const void*>(nullptr), 0, static_cast<void*>(nullptr), M, N, K, rows_a, rows_w, slices, slice_macs, partial, 0, 0);
        return check_launch("mxfp_gemm_scaled");
    };
    static std::atomic<uint64_t> allowed2{0}, allowed4{0};
    if (int rc = M <= 32 ? go(mxfp_gemm_scaled_rows_regs_kernel<F32, 2, SRG_WAVES>, 2, allowed2) : go(mxfp_gemm_scaled_rows_regs_kernel<F32, 4, SRG_WAVES>, 4, allowed4))
        return rc;
    const int64_t mn = (int64_t)M * N;
    hipLaunchKernelGGL(split_k_reduce_kernel<DT_OUT>, dim3((unsigned)((mn / 4 + 255) / 256)), dim3(256), 0, s, static_cast<const float*>(partial), slices, mn, N, bias,
                       bias_dtype, y);
    return check_launch("mxfp_gemm_scaled");
}

template <int DT_OUT>
int launch_gemm_scaled_rows(const uint8_t* a_codes, const uint32_t* a_scales, const uint8_t* w_codes, const uint32_t* w_scales, const void* bias,
                            int bias_dtype, void* y, int M, int N, int K, hipStream_t s) {
    const int rows_a = (M + 255) / 256 * 256, rows_w = (N + 255) / 256 * 256;
    const unsigned groups = (unsigned)((N + 15) / 16);
    if (K <= 4096) {
        // a wavefront's share of A stays in its registers: persistent workgroups of eight wavefronts, one per CU
        const int cus = device_cu_count();
        if (cus <= 0) return fail(ERR_RUNTIME, "cannot read the compute-unit count of the current device");
        auto go = [&](auto kern, int mt, std::atomic<uint64_t>& allowed) {
            // (more than half a CU's LDS, so that no CU is given two of these workgroups while another has none)
            const int lds_bytes = max(16 * SRR_ROW + SRG_WAVES * mt * 256 * (int)sizeof(float), 84 * 1024);
            if (int rc = allow_dynamic_lds(reinterpret_cast<const void*>(kern), lds_bytes, allowed)) return rc;
            const RowsDeal d = deal_row_groups((int)groups, cus);
            hipLaunchKernelGGL(kern, dim3((unsigned)d.grid), dim3(SRG_WAVES * 64), lds_bytes, s, a_codes, a_scales, w_codes, w_scales, bias, bias_dtype, y, M, N,
                               K, rows_a, rows_w, 1, K / 128, static_cast<float*>(nullptr), d.full_rounds, d.tail_halves);
            return check_launch("mxfp_gemm_scaled");
        };
        static std::atomic<uint64_t> allowed1{0}, allowed2{0}, allowed4{0};
        if (M <= 16) return go(mxfp_gemm_scaled_rows_regs_kernel<DT_OUT, 1, SRG_WAVES>, 1, allowed1);
        if (M <= 32) return go(mxfp_gemm_scaled_rows_regs_kernel<DT_OUT, 2, SRG_WAVES>, 2, allowed2);
        return go(mxfp_gemm_scaled_rows_regs_kernel<DT_OUT, 4, SRG_WAVES>, 4, allowed4);
    }
    if (M <= 16)
        hipLaunchKernelGGL((mxfp_gemm_scaled_rows_kernel<DT_OUT, 1, 4>), dim3(groups), dim3(256), 0, s, a_codes, a_scales, w_codes, w_scales, bias, bias_dtype, y,
                           M, N, K, rows_a, rows_w);
    else
        hipLaunchKernelGGL((mxfp_gemm_scaled_rows_kernel<DT_OUT, 2, 2>), dim3(groups), dim3(256), 0, s, a_codes, a_scales, w_codes, w_scales, bias, bias_dtype, y,
                           M, N, K, rows_a, rows_w);
    return check_launch("mxfp_gemm_scaled");
}
