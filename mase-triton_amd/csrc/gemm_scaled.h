// Block-scaled MXFP GEMM for gfx950:  y[M,N] = A[M,K] * W[N,K]^T (+ bias) on v_mfma_scale_f32_16x16x128_f8f6f4.
//
// Both operands stay MXFP all the way into the matrix unit: one FP8 (E4M3) code per element and one E8M0 scale per
// 32 elements along K, which the instruction applies itself.  Nothing is composed to bf16, no operand byte passes
// through a VGPR on its way to LDS, and an operand row costs one byte per element of LDS and L2 traffic instead of two.
// The operands come from the operand kernels (cast_kernels.hip), which
//   * re-encode every block that holds the code S.1111.111 one scale step up (the instruction reads that code as NaN,
//     the reference as +-480) and embed the narrower element formats into E4M3 bytes (exact),
//   * pad the rows to a multiple of 256 and store the scales transposed: dword [K/128][rows], the four bytes of a dword
//     being the scales of the four 32-k blocks of one 128-k macro step of one row.
//
// What the instruction expects (measured with a one-wavefront probe): lane l = 16 g + r supplies row r of a 16-row
// operand tile; its first 16 bytes are k 16 g .. 16 g + 15 and its second 16 bytes k 64 + 16 g .. 64 + 16 g + 15 of the
// 128 k; byte `opsel` of its scale register is the scale of k block g (k 32 g .. 32 g + 31) of that row.  The first
// operand's rows are the result's rows in lane groups of four (c[4 (l >> 4) + v][l & 15] in element v), so W is fed
// first and a lane ends up with four consecutive n of one m, as in the bf16 kernels.
//
// Tile 256 x 256, four wavefronts 2 x 2, each 128 x 128 (8 x 8 MFMA tiles, 256 accumulator AGPRs), macro steps of 128 k.
// A macro step is worked off in two periods of four m-tiles (32 MFMAs); the eight W fragments of a macro step live in
// registers (they are read from LDS during the macro step before).  The data of one period is a "chunk": 128 rows of A
// (the period's four m-tiles of both wave rows) and 128 rows of W (four n-tiles of the NEXT macro step, both wave
// columns), 16 KB each, plus 1 KB of scales, all by DMA (global_load_lds).  LDS holds a ring of four chunks:
//
//   period c    multiplies chunk c's A rows, reads chunk c's W rows into the registers of the next macro step,
//               and issues the DMAs of chunk c + 3 (into the slot that chunk c - 1 left), spread over the period
//   barrier c+1 sits before the last eight MFMAs of period c: every wave has finished reading chunk c, and has waited
//               until its own DMAs of chunk c + 1 (issued two periods earlier: vmcnt(20)) have landed
//
// so a DMA has between two and three periods (2000 - 3000 cycles) to land and the address unit sees an even stream.
// (included from gemm_impl.h's namespace, after gemm_tall.h whose asm helpers it shares)

constexpr int SM = 256, SN = 256, SMAC = 128;
constexpr int S_RING = 4;
constexpr int S_PART_BYTES = 128 * 128;                       // 128 rows of one operand, 128 k
constexpr int S_A_OFF = 0;                                    // [4 chunks][128 rows][128 B]
constexpr int S_W_OFF = S_RING * S_PART_BYTES;                // the same for W: both below 64 KB offsets from their base
constexpr int S_SC_OFF = 2 * S_RING * S_PART_BYTES;           // [4 chunks][4 waves][64 dwords]: 32 A rows, 32 W rows per wave
constexpr int S_SC_BYTES = 1024;
constexpr int S_OUT_OFF = S_SC_OFF + S_RING * S_SC_BYTES;     // [4 waves][32 rows][128 B] output staging
constexpr int S_LDS_BYTES = S_OUT_OFF + 4 * 4096;             // 148 KB

typedef int intx8 __attribute__((ext_vector_type(8)));
typedef int intx4 __attribute__((ext_vector_type(4)));

// c += w (16 n x 128 k, scales sw) * a (16 m x 128 k, scales sa)^T
__device__ inline void mfma_scaled(floatx4& c, const intx8& w, const intx8& a, uint32_t sw, uint32_t sa) {
    asm volatile("v_mfma_scale_f32_16x16x128_f8f6f4 %0, %1, %2, %0, %3, %4 op_sel_hi:[0,0,0]" : "+a"(c) : "v"(w), "v"(a), "v"(sw), "v"(sa));
}
__device__ inline void mfma_scaled_first(floatx4& c, const intx8& w, const intx8& a, uint32_t sw, uint32_t sa) {
    asm volatile("v_mfma_scale_f32_16x16x128_f8f6f4 %0, %1, %2, 0, %3, %4 op_sel_hi:[0,0,0]" : "=a"(c) : "v"(w), "v"(a), "v"(sw), "v"(sa));
}
// for the lanes in `mask`: 4 bytes from (sbase + voff) to LDS lds_addr + 4 * lane.  (The mask is applied here and not by
// a branch around the call: the LDS address has to stay in a scalar register.)
__device__ inline void dma_dwords_masked(uint32_t lds_addr, uint32_t voff, const void* sbase, uint64_t mask) {
    uint64_t saved;
    asm volatile("s_mov_b64 %0, exec\n\ts_mov_b64 exec, %4\n\ts_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dword %2, %3\n\ts_mov_b64 exec, %0"
                 : "=&s"(saved) : "s"(lds_addr), "v"(voff), "s"(sbase), "s"(mask) : "memory");
}

// 16 bytes to a per-lane address (non-temporal: the output is not read again by this kernel); the trailing s_nop keeps a
// following VALU write of the data registers out of the store's read window
__device__ inline void store16_nt(void* dst, const u32x4& v) {
    asm volatile("global_store_dwordx4 %0, %1, off nt\n\ts_nop 0" ::"v"(dst), "v"(v) : "memory");
}

struct ScaledTile {
    int m0, n0;
    int mac0;        // first macro step of this walk (K split: walk z of a tile takes macro steps z * nmac .. )
    size_t y_off;    // byte offset of the walk's output array (K split: one fp32 [M, N] array per split)
};

template <int DT_OUT>
__global__ __launch_bounds__(kGemmThreads) __attribute__((amdgpu_waves_per_eu(1, 1))) void mxfp_gemm_scaled_kernel(
    const uint8_t* __restrict__ a_codes, const uint32_t* __restrict__ a_scales, const uint8_t* __restrict__ w_codes,
    const uint32_t* __restrict__ w_scales, const void* __restrict__ bias, int bias_dtype, void* __restrict__ y, int M, int N, int K,
    int rows_a, int rows_w, int tiles_m, int tiles_n, int splits, int64_t y_split_bytes) {
    // splits > 1: every tile is walked `splits` times, each time over K / splits of k and into its own [M, N] array of y
    extern __shared__ __attribute__((aligned(1024))) uint8_t lds[];
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wave_m = wave >> 1, wave_n = wave & 1;
    const int nmac = K / SMAC / splits;   // macro steps per walk: even and at least 4 (the launcher checks)
    const uint32_t lds_base = (uint32_t)(uintptr_t)lds;

    // ---- per-lane constants
    // data DMA d (0..3) of a wave covers rows 32 wave + 8 d .. + 7 of a chunk part; lane l fills position l & 7 of row
    // 8 d + (l >> 3), which must hold the row's 16-byte piece (l & 7) ^ (row >> 1 & 7) = (l & 7) ^ ((4 d + (l >> 4)) & 7)
    uint32_t dma_voff[4];
#pragma unroll
    for (int d = 0; d < 4; ++d)
        dma_voff[d] = (uint32_t)(8 * d + (lane >> 3)) * (uint32_t)K + (uint32_t)((((lane & 7) ^ ((4 * d + (lane >> 4)) & 7))) << 4);
    // fragment reads: lane (g = l >> 4, r = l & 15) reads pieces g and g + 4 of row r of its 16-row tile
    const uint32_t f_off = (uint32_t)(lane & 15) * 128u + (uint32_t)((((lane >> 4) ^ ((lane >> 1) & 7)) & 7) << 4);
    const uint8_t* const a_frag0 = lds + S_A_OFF + wave_m * (64 * 128) + f_off;
    const uint8_t* const a_frag1 = lds + S_A_OFF + wave_m * (64 * 128) + (f_off ^ 64u);
    const uint8_t* const w_frag0 = lds + S_W_OFF + wave_n * (64 * 128) + f_off;
    const uint8_t* const w_frag1 = lds + S_W_OFF + wave_n * (64 * 128) + (f_off ^ 64u);
    // scale bytes: the dword of chunk row q sits at (q >> 5) * 256 + (q & 31) * 4 (A) or + 128 (W); a lane wants byte g
    const uint8_t* const a_sc = lds + S_SC_OFF + wave_m * 512 + (lane & 15) * 4 + (lane >> 4);
    const uint8_t* const w_sc = lds + S_SC_OFF + wave_n * 512 + 128 + (lane & 15) * 4 + (lane >> 4);

    const int n_tiles = tiles_m * tiles_n * splits;   // walks
    const int per_xcd = (n_tiles + 7) >> 3;
    const int slots = gridDim.x >> 3;
    auto has_tile = [&](int local) __attribute__((always_inline)) { return local < per_xcd && (int)(blockIdx.x & 7) * per_xcd + local < n_tiles; };
    auto tile_at = [&](int local) __attribute__((always_inline)) {
        const int walk = (blockIdx.x & 7) * per_xcd + local;
        const int pos = walk / splits, z = walk - pos * splits;      // the splits of a tile run next to each other
        // groups of 4 tile rows, rows fastest: the 32 tiles an XCD runs at once form a 4 x 8 patch
        constexpr int GROUP = 4;
        const int in_group = GROUP * tiles_n;
        const int first_m = (pos / in_group) * GROUP;
        const int rows = min(tiles_m - first_m, GROUP);
        const int rr = pos % in_group;
        ScaledTile t;
        t.m0 = (first_m + rr % rows) * SM;
        t.n0 = (rr / rows) * SN;
        t.mac0 = z * nmac;
        t.y_off = (size_t)z * (size_t)y_split_bytes;
        return t;
    };

    int local = blockIdx.x >> 3;
    if (!has_tile(local)) return;
    ScaledTile cur = tile_at(local), next = cur;

    // ---- The DMA streams.  A chunk = (macro step ma of A, macro step ma + 1 of W, half h): ten operations per wave, its
    //      32 rows of A and of W (four of 8 rows each) and the scale dwords of those rows (lanes 0..31 those of A, lanes
    //      32..63 those of W).  Each half of each operand is a stream of its own that moves one macro step along K per
    //      chunk and jumps to the next tile when it passes the end of this one (the W streams one macro step before the
    //      A streams).
    const int row0_w = 128 * (wave >> 1) + 32 * (wave & 1);   // this wave's first row of a part, as a row of the tile, for half 0
    const uint32_t wave_lds = lds_base + (uint32_t)wave * 4096u;   // ... and its place within a chunk part
    const uint32_t wave_lds_sc = lds_base + (uint32_t)wave * 256u;
    const uint32_t sc_voff = (uint32_t)(lane & 31) * 4u;
    const uint8_t *pa[2], *pw[2];      // where the next chunk of half h reads its codes ...
    const uint32_t *pas[2], *pws[2];   // ... and its scales
    auto a_stream_to = [&](const ScaledTile& t, int h) __attribute__((always_inline)) {
        const int row = t.m0 + row0_w + 64 * h;
        pa[h] = a_codes + (size_t)row * K + (size_t)t.mac0 * SMAC;
        pas[h] = a_scales + (size_t)t.mac0 * rows_a + row;
    };
    auto w_stream_to = [&](const ScaledTile& t, int h) __attribute__((always_inline)) {
        const int row = t.n0 + row0_w + 64 * h;
        pw[h] = w_codes + (size_t)row * K + (size_t)t.mac0 * SMAC;
        pws[h] = w_scales + (size_t)t.mac0 * rows_w + row;
    };
    // operation q (0..9) of the next chunk of half H into ring slot SLOT
    auto chunk_dma = [&](auto h_c, auto slot_c, auto q_c) __attribute__((always_inline)) {
        constexpr int H = decltype(h_c)::value, SLOT = decltype(slot_c)::value, q = decltype(q_c)::value;
        if constexpr (q < 4) dma_1kb(wave_lds + (S_A_OFF + SLOT * S_PART_BYTES + q * 1024), dma_voff[q], pa[H]);
        else if constexpr (q < 8) dma_1kb(wave_lds + (S_W_OFF + SLOT * S_PART_BYTES + (q - 4) * 1024), dma_voff[q - 4], pw[H]);
        else if constexpr (q == 8) dma_dwords_masked(wave_lds_sc + (S_SC_OFF + SLOT * S_SC_BYTES), sc_voff, pas[H], 0x00000000FFFFFFFFull);
        else dma_dwords_masked(wave_lds_sc + (S_SC_OFF + SLOT * S_SC_BYTES), sc_voff, pws[H], 0xFFFFFFFF00000000ull);
    };
    auto a_advance = [&](int h) __attribute__((always_inline)) { pa[h] += SMAC; pas[h] += rows_a; };
    auto w_advance = [&](int h) __attribute__((always_inline)) { pw[h] += SMAC; pws[h] += rows_w; };

    floatx4 acc[8][8];        // [n-tile j][m-tile i]
    intx8 wreg[2][8];         // the W fragments of the macro step in flight and of the next one
    uint32_t wsc[2][8];       // their scale bytes
    intx8 areg[2];            // A fragment ring
    uint32_t asc[2][4];       // scale bytes of the period's four m-tiles, and of the next period's

    // halves of fragment t (0..3) of ring slot `slot`
    auto read_a_lo = [&](intx8& dst, int slot, int t) __attribute__((always_inline)) { dst.lo = *reinterpret_cast<const intx4*>(a_frag0 + slot * S_PART_BYTES + t * 2048); };
    auto read_a_hi = [&](intx8& dst, int slot, int t) __attribute__((always_inline)) { dst.hi = *reinterpret_cast<const intx4*>(a_frag1 + slot * S_PART_BYTES + t * 2048); };
    auto read_w_lo = [&](intx8& dst, int slot, int t) __attribute__((always_inline)) { dst.lo = *reinterpret_cast<const intx4*>(w_frag0 + slot * S_PART_BYTES + t * 2048); };
    auto read_w_hi = [&](intx8& dst, int slot, int t) __attribute__((always_inline)) { dst.hi = *reinterpret_cast<const intx4*>(w_frag1 + slot * S_PART_BYTES + t * 2048); };
    auto read_w_sc = [&](uint32_t& sc, int slot, int t) __attribute__((always_inline)) { sc = w_sc[slot * S_SC_BYTES + (t >> 1) * 256 + (t & 1) * 64]; };
    auto read_a_sc = [&](uint32_t& sc, int slot, int t) __attribute__((always_inline)) { sc = a_sc[slot * S_SC_BYTES + (t >> 1) * 256 + (t & 1) * 64]; };

    // ---- prologue of the stream: W macro step 0 of the first tile travels alone through slots 2 and 3 (as the W halves
    //      of chunks "-2" and "-1"); then chunks 0, 1, 2.  The waits here are total: only the steady state counts.
    a_stream_to(cur, 0); a_stream_to(cur, 1); w_stream_to(cur, 0); w_stream_to(cur, 1);
    auto issue_w_half = [&](auto h_c, auto slot_c) __attribute__((always_inline)) {
        chunk_dma(h_c, slot_c, IntC<4>{}); chunk_dma(h_c, slot_c, IntC<5>{}); chunk_dma(h_c, slot_c, IntC<6>{});
        chunk_dma(h_c, slot_c, IntC<7>{}); chunk_dma(h_c, slot_c, IntC<9>{});
        w_advance(decltype(h_c)::value);
    };
    auto issue_a_half = [&](auto h_c, auto slot_c) __attribute__((always_inline)) {
        chunk_dma(h_c, slot_c, IntC<0>{}); chunk_dma(h_c, slot_c, IntC<1>{}); chunk_dma(h_c, slot_c, IntC<2>{});
        chunk_dma(h_c, slot_c, IntC<3>{}); chunk_dma(h_c, slot_c, IntC<8>{});
        a_advance(decltype(h_c)::value);
    };
    issue_w_half(IntC<0>{}, IntC<2>{});
    issue_w_half(IntC<1>{}, IntC<3>{});
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __builtin_amdgcn_s_barrier();
#pragma unroll
    for (int t = 0; t < 4; ++t) {
        read_w_lo(wreg[0][t], 2, t); read_w_hi(wreg[0][t], 2, t); read_w_sc(wsc[0][t], 2, t);
        read_w_lo(wreg[0][4 + t], 3, t); read_w_hi(wreg[0][4 + t], 3, t); read_w_sc(wsc[0][4 + t], 3, t);
    }
    lds_barrier();   // slots 2 and 3 are free again
    issue_a_half(IntC<0>{}, IntC<0>{}); issue_w_half(IntC<0>{}, IntC<0>{});
    issue_a_half(IntC<1>{}, IntC<1>{}); issue_w_half(IntC<1>{}, IntC<1>{});
    issue_a_half(IntC<0>{}, IntC<2>{}); issue_w_half(IntC<0>{}, IntC<2>{});
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __builtin_amdgcn_s_barrier();
    read_a_lo(areg[0], 0, 0); read_a_hi(areg[0], 0, 0);
#pragma unroll
    for (int t = 0; t < 4; ++t) read_a_sc(asc[0][t], 0, t);

    // One period: H = half of the macro step (m-tiles 4 H .. 4 H + 3), C4 = ring slot of its chunk, WC = register set of
    // the macro step's W fragments.  ma = macro step (of the current tile).  Every MFMA is followed by at most a few
    // other instructions (a wave can issue about six under one 32-cycle MFMA), in this order, pinned by scheduling
    // barriers: the period's ten DMAs, the reads of the next A fragment and of the next macro step's W fragments.
    auto period = [&](int ma, auto h_c, auto c4_c, auto wc_c, auto first_c) __attribute__((always_inline)) {
        constexpr int H = decltype(h_c)::value, C4 = decltype(c4_c)::value, WC = decltype(wc_c)::value;
        constexpr bool FIRST = decltype(first_c)::value != 0;
        constexpr int WN = WC ^ 1, NEXT_SLOT = (C4 + 1) & 3, ISSUE_SLOT = (C4 + 3) & 3;
        constexpr int AS = H, ASN = H ^ 1;   // scale register set of this period, of the next
        // the chunk issued during this period: three periods ahead, the other half; its streams may have to move on to
        // the next tile first
        constexpr int IH = H ^ 1;
        {
            const int issue_ma = H == 0 ? ma + 1 : ma + 2;
            if (issue_ma == nmac) a_stream_to(next, IH);
            if (issue_ma == nmac - 1) w_stream_to(next, IH);
        }
        auto dma = [&](auto q_c) __attribute__((always_inline)) { chunk_dma(IntC<IH>{}, IntC<ISSUE_SLOT>{}, q_c); };
        auto mm = [&](const intx8& a, uint32_t sa, auto i_c, auto j_c) __attribute__((always_inline)) {
            constexpr int i = decltype(i_c)::value, j = decltype(j_c)::value;
            if (FIRST) mfma_scaled_first(acc[j][i], wreg[WC][j], a, wsc[WC][j], sa);
            else mfma_scaled(acc[j][i], wreg[WC][j], a, wsc[WC][j], sa);
        };
#define S_SLOT_END() __builtin_amdgcn_sched_barrier(0)
        // rows 0..2: m-tile 4 H + r against the eight n-tiles; beside them the A fragment of row r + 1, W fragment(s) of the
        // next macro step, three or four DMAs
        static_for<3>([&](auto r_c) __attribute__((always_inline)) {
            constexpr int r = decltype(r_c)::value;
            constexpr int i = 4 * H + r;
            intx8& a_now = areg[r & 1];
            intx8& a_nxt = areg[(r + 1) & 1];
            const uint32_t sa = asc[AS][r];
            constexpr int wt = r == 0 ? 0 : r + 1;          // W fragment read in this row (row 0 reads two: 0 and 1)
            mm(a_now, sa, IntC<i>{}, IntC<0>{}); read_a_lo(a_nxt, C4, r + 1); S_SLOT_END();
            mm(a_now, sa, IntC<i>{}, IntC<1>{}); read_a_hi(a_nxt, C4, r + 1); S_SLOT_END();
            mm(a_now, sa, IntC<i>{}, IntC<2>{}); dma(IntC<r == 0 ? 0 : r == 1 ? 3 : 7>{}); S_SLOT_END();
            mm(a_now, sa, IntC<i>{}, IntC<3>{}); read_w_lo(wreg[WN][4 * H + wt], C4, wt); S_SLOT_END();
            mm(a_now, sa, IntC<i>{}, IntC<4>{}); read_w_hi(wreg[WN][4 * H + wt], C4, wt); read_w_sc(wsc[WN][4 * H + wt], C4, wt); S_SLOT_END();
            mm(a_now, sa, IntC<i>{}, IntC<5>{}); dma(IntC<r == 0 ? 1 : r == 1 ? 4 : 8>{}); S_SLOT_END();
            mm(a_now, sa, IntC<i>{}, IntC<6>{});
            if constexpr (r == 0) { read_w_lo(wreg[WN][4 * H + 1], C4, 1); read_w_hi(wreg[WN][4 * H + 1], C4, 1); read_w_sc(wsc[WN][4 * H + 1], C4, 1); }
            else dma(IntC<r == 1 ? 5 : 9>{});
            S_SLOT_END();
            mm(a_now, sa, IntC<i>{}, IntC<7>{});
            if constexpr (r < 2) dma(IntC<r == 0 ? 2 : 6>{});
            if constexpr (r == 2) { a_advance(IH); w_advance(IH); }
            S_SLOT_END();
        });
        // row 3: the next chunk has landed everywhere (this wave's part of it was issued two periods ago: 20 younger
        // operations), this one is no longer read
        {
            constexpr int i = 4 * H + 3;
            intx8& a_now = areg[1];
            const uint32_t sa = asc[AS][3];
            asm volatile("s_waitcnt vmcnt(20)" ::: "memory");
            lds_barrier();
            mm(a_now, sa, IntC<i>{}, IntC<0>{}); read_a_lo(areg[0], NEXT_SLOT, 0); S_SLOT_END();
            mm(a_now, sa, IntC<i>{}, IntC<1>{}); read_a_hi(areg[0], NEXT_SLOT, 0); S_SLOT_END();
            mm(a_now, sa, IntC<i>{}, IntC<2>{}); read_a_sc(asc[ASN][0], NEXT_SLOT, 0); S_SLOT_END();
            mm(a_now, sa, IntC<i>{}, IntC<3>{}); read_a_sc(asc[ASN][1], NEXT_SLOT, 1); S_SLOT_END();
            mm(a_now, sa, IntC<i>{}, IntC<4>{}); read_a_sc(asc[ASN][2], NEXT_SLOT, 2); S_SLOT_END();
            mm(a_now, sa, IntC<i>{}, IntC<5>{}); read_a_sc(asc[ASN][3], NEXT_SLOT, 3); S_SLOT_END();
            mm(a_now, sa, IntC<i>{}, IntC<6>{}); S_SLOT_END();
            mm(a_now, sa, IntC<i>{}, IntC<7>{}); S_SLOT_END();
        }
#undef S_SLOT_END
    };

    for (;;) {
        const int next_local = local + slots;
        const bool more = has_tile(next_local);
        if (more) next = tile_at(next_local);  // else the look-ahead re-reads this tile's first operands (unused)

        // macro steps in pairs: the register sets of W and the ring slots alternate at compile time
        period(0, IntC<0>{}, IntC<0>{}, IntC<0>{}, IntC<1>{});
        period(0, IntC<1>{}, IntC<1>{}, IntC<0>{}, IntC<1>{});
        period(1, IntC<0>{}, IntC<2>{}, IntC<1>{}, IntC<0>{});
        period(1, IntC<1>{}, IntC<3>{}, IntC<1>{}, IntC<0>{});
        for (int ma = 2; ma < nmac; ma += 2) {
            period(ma, IntC<0>{}, IntC<0>{}, IntC<0>{}, IntC<0>{});
            period(ma, IntC<1>{}, IntC<1>{}, IntC<0>{}, IntC<0>{});
            period(ma + 1, IntC<0>{}, IntC<2>{}, IntC<1>{}, IntC<0>{});
            period(ma + 1, IntC<1>{}, IntC<3>{}, IntC<1>{}, IntC<0>{});
        }

        // ---- output: lane holds, for tile (j, i), y[m][n .. n+3] with m = m0 + 128 wave_m + 16 i + lane % 16,
        //      n = n0 + 128 wave_n + 16 j + 4 (lane / 16); staged through LDS so that a store instruction writes whole lines
        uint8_t* const lds_out = lds + S_OUT_OFF + wave * 4096;
        const int row_base = cur.m0 + wave_m * 128, col_base = cur.n0 + wave_n * 128;
        uint32_t ol = (uint32_t)lane;
        asm volatile("s_nop 15\n\ts_nop 15" : "+v"(ol));  // also: the last MFMA results are readable after this
        const uint32_t o_row = ol & 15u, o_q = ol >> 4;
        const uint32_t o_rd_off = (ol >> 3) * 128u + (((ol & 7u) ^ (ol >> 3)) * 16u);
        auto write_tile = [&](auto has_bias_c) __attribute__((always_inline)) {
            constexpr bool HAS_BIAS = decltype(has_bias_c)::value != 0;
            float bv[2] = {0.0f, 0.0f};
            if (HAS_BIAS) {
                bv[0] = col_base + (int)ol < N ? load_bias(bias, bias_dtype, col_base + (int)ol) : 0.0f;
                bv[1] = col_base + 64 + (int)ol < N ? load_bias(bias, bias_dtype, col_base + 64 + (int)ol) : 0.0f;
            }
            auto values = [&](auto j_c, auto i_c, float(&r)[4]) {
                constexpr int j = decltype(j_c)::value, i = decltype(i_c)::value;
                static_for<4>([&](auto t_c) __attribute__((always_inline)) {
                    constexpr int t = decltype(t_c)::value;
                    r[t] = acc_read(acc[j][i][t]);
                    if (HAS_BIAS) {
                        const int src = (int)(((uint32_t)(16 * j + t) + 4u * o_q) & 63u);
                        r[t] += __builtin_bit_cast(float, __builtin_amdgcn_ds_bpermute(src * 4, __builtin_bit_cast(int, bv[j >> 2])));
                    }
                });
            };
            constexpr int OB = DT_OUT == F32 ? 4 : 2;           // bytes per output
            constexpr int PASS_COLS = 128 / OB;                 // columns of a 128-byte staged row: 32 (fp32) or 64
            constexpr int NPASS_J = 128 / PASS_COLS;            // passes across the wave's 128 columns
            constexpr int JT = PASS_COLS / 16;                  // n-tiles per pass
            // store: lane covers 16 bytes (16 / OB columns) of row (ol >> 3) of each 8-row group
            const int st_col = col_base + (int)(ol & 7u) * (16 / OB);
            static_for<4>([&](auto ip_c) __attribute__((always_inline)) {
                static_for<NPASS_J>([&](auto jp_c) __attribute__((always_inline)) {
                    constexpr int ip = decltype(ip_c)::value, jp = decltype(jp_c)::value;
                    static_for<2 * JT>([&](auto x_c) __attribute__((always_inline)) {
                        constexpr int ii = decltype(x_c)::value / JT, jj = decltype(x_c)::value % JT;
                        float r[4];
                        values(IntC<JT * jp + jj>{}, IntC<2 * ip + ii>{}, r);
                        const uint32_t row = 16u * ii + o_row;
                        if constexpr (DT_OUT == F32) {
                            const uint32_t chunk = ((uint32_t)(4 * jj) + o_q) ^ (row & 7u);
                            *reinterpret_cast<uint4*>(lds_out + row * 128u + chunk * 16u) = make_uint4(f32_bits(r[0]), f32_bits(r[1]), f32_bits(r[2]), f32_bits(r[3]));
                        } else {
                            const uint2 p = pack_out4<DT_OUT>(r[0], r[1], r[2], r[3]);
                            const uint32_t chunk = ((uint32_t)(2 * jj) + (o_q >> 1)) ^ (row & 7u);
                            *reinterpret_cast<uint2*>(lds_out + row * 128u + chunk * 16u + (o_q & 1u) * 8u) = p;
                        }
                    });
                    u32x4 v[4];
                    static_for<4>([&](auto t_c) __attribute__((always_inline)) {
                        constexpr int t = decltype(t_c)::value;
                        v[t] = *reinterpret_cast<const u32x4*>(lds_out + o_rd_off + t * 1024);
                    });
                    static_for<4>([&](auto t_c) __attribute__((always_inline)) {
                        constexpr int t = decltype(t_c)::value;
                        const int row = row_base + ip * 32 + 8 * t + (int)(ol >> 3);
                        const int col = st_col + jp * PASS_COLS;
                        if (row < M && col < N) {
                            uint8_t* const dst = static_cast<uint8_t*>(y) + cur.y_off + ((size_t)row * N + col) * OB;
                            store16_nt(dst, v[t]);
                        }
                    });
                    __builtin_amdgcn_sched_barrier(0);  // one pass at a time
                });
            });
        };
        if (bias) write_tile(IntC<1>{});
        else write_tile(IntC<0>{});

        if (!more) break;
        cur = next;
        local = next_local;
    }
    // the look-ahead DMAs of the last periods still target LDS: let them finish
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
}

#include "gemm_scaled_rows.h"   // the weight-streaming kernels for up to 64 rows of A


// K split for few tiles and a long K (a [1024, 4096] output has 64 tiles for 256 CUs): the number of walks per tile, chosen so
// that the walks about fill the CUs; a walk takes an even number of macro steps, at least 4.  Priced like the bf16 kernels'
// split: macro steps per walk at about 1 us, rounds of walks over the CUs, and for a split the second launch plus the
// partial sums written and read once.
inline int plan_scaled_splits(int M, int N, int K, int cus) {
    const int64_t tiles = (int64_t)((M + SM - 1) / SM) * ((N + SN - 1) / SN);
    const int nmac = K / SMAC;
    if (tiles * 2 > cus || cus <= 0 || scaled_rows_shape_ok(M, K)) return 1;
    const double mn_mb = (double)M * N * 4.0 / 1e6;
    auto price = [&](int s) {
        const double rounds = (double)((tiles * s + cus - 1) / cus);
        return rounds * (nmac / s + 3) * 1.0 + (s > 1 ? 4.0 + (2.0 * s + 0.5) * mn_mb * 0.21 : 0.0);
    };
    int best = 1;
    double best_t = price(1);
    for (int s = 2; s <= 16 && tiles * s <= cus; ++s) {
        if (nmac % s != 0 || (nmac / s) % 2 != 0 || nmac / s < 4) continue;
        const double t = price(s);
        if (t < best_t) { best_t = t; best = s; }
    }
    return best;
}

// a_codes [rows_a, K], w_codes [rows_w, K]: rows padded to multiples of 256; scales [K / 128][rows] dwords.  `workspace`
// (may be null): room for the fp32 partial sums of a K split, splits * M * N * 4 bytes.
template <int DT_OUT>
int launch_gemm_scaled(const uint8_t* a_codes, const uint32_t* a_scales, const uint8_t* w_codes, const uint32_t* w_scales, const void* bias,
                       int bias_dtype, void* y, int M, int N, int K, void* workspace, int64_t workspace_bytes, hipStream_t s) {
    const int tiles_m = (M + SM - 1) / SM, tiles_n = (N + SN - 1) / SN;
    const int64_t tiles = (int64_t)tiles_m * tiles_n;
    if (tiles >= (1 << 26)) return fail(ERR_UNSUPPORTED, "too many tiles");
    const int cus = device_cu_count();
    if (cus <= 0) return fail(ERR_RUNTIME, "cannot read the compute-unit count of the current device");
    if (const int slices = scaled_rows_slices(M, N, K); slices > 0 && workspace && workspace_bytes >= (int64_t)slices * M * N * 4)
        return launch_gemm_scaled_rows_sliced<DT_OUT>(a_codes, a_scales, w_codes, w_scales, bias, bias_dtype, y, M, N, K, static_cast<float*>(workspace), s);
    if (scaled_rows_shape_ok(M, K)) return launch_gemm_scaled_rows<DT_OUT>(a_codes, a_scales, w_codes, w_scales, bias, bias_dtype, y, M, N, K, s);
    int splits = workspace ? plan_scaled_splits(M, N, K, cus) : 1;
    const int64_t mn = (int64_t)M * N;
    if (splits > 1 && workspace_bytes < splits * mn * 4) splits = 1;
    const int64_t walks = tiles * splits;
    const unsigned grid = (unsigned)(walks < cus ? ((walks + 7) / 8) * 8 : (cus / 8) * 8);
    if (splits > 1) {
        auto kern = mxfp_gemm_scaled_kernel<F32>;
        static std::atomic<uint64_t> lds_allowed{0};
        if (int rc = allow_dynamic_lds(reinterpret_cast<const void*>(kern), S_LDS_BYTES, lds_allowed)) return rc;
        hipLaunchKernelGGL(kern, dim3(grid), dim3(kGemmThreads), S_LDS_BYTES, s, a_codes, a_scales, w_codes, w_scales, static_cast<const void*>(nullptr), 0,
                           workspace, M, N, K, tiles_m * SM, tiles_n * SN, tiles_m, tiles_n, splits, mn * 4);
        if (int rc = check_launch("mxfp_gemm_scaled")) return rc;
        hipLaunchKernelGGL(split_k_reduce_kernel<DT_OUT>, dim3((unsigned)((mn / 4 + 255) / 256)), dim3(256), 0, s,
                           static_cast<const float*>(workspace), splits, mn, N, bias, bias_dtype, y);
        return check_launch("mxfp_gemm_scaled");
    }
    auto kern = mxfp_gemm_scaled_kernel<DT_OUT>;
    static std::atomic<uint64_t> lds_allowed{0};
    if (int rc = allow_dynamic_lds(reinterpret_cast<const void*>(kern), S_LDS_BYTES, lds_allowed)) return rc;
    hipLaunchKernelGGL(kern, dim3(grid), dim3(kGemmThreads), S_LDS_BYTES, s, a_codes, a_scales, w_codes, w_scales, bias, bias_dtype, y, M, N, K,
                       tiles_m * SM, tiles_n * SN, tiles_m, tiles_n, 1, (int64_t)0);
    return check_launch("mxfp_gemm_scaled");
}
