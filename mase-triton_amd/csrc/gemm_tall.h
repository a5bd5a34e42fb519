// Tall-tile MXFP GEMM kernel for gfx950: 512 (M) x 128 (N) tiles, dense bf16 A, 16-bit output.
//
// Why this shape.  One wavefront can issue only two other instructions per 16-cycle 16x16x32 MFMA
// (six per 32-cycle 32x32x16 MFMA) without slowing the matrix pipe, so the K loop has to be lean:
//   * the dense A operand goes from global memory straight into LDS (global_load_lds_dwordx4, no
//     VGPRs, no ds_write), always as whole 128-byte lines: a CU's vector memory path moves about
//     2.5 cycles per cache line an instruction touches, whatever part of the line is used, so
//     64-byte row pieces would halve its rate;
//   * the MXFP weight slab is composed to bf16 once per 512 output rows instead of once per 256;
//   * all global traffic is issued by hand (inline asm) and waited for with explicit s_waitcnt
//     counts, so the compiler inserts no conservative waits of its own;
//   * every K step is laid out by hand in 16 slots of four MFMAs each, the other work spread over
//     them one vector-memory instruction at a time (a burst of them stalls the issuing wave for
//     as long as the address unit needs to drain it).
// Four wavefronts stacked along M, each 128 x 128 (8 x 8 MFMA tiles of 16 x 16, 256 accumulator AGPRs).
// A wave only ever reads the 128 A rows it loaded itself; the 128-row W slab is shared by all four.
// The MFMA is v_mfma_f32_16x16x32_bf16: under the chip's power limit (which, not stalls, bounds this
// kernel on real data) it does the same work as 32x32x16 for less accumulator traffic; measured on
// 16384 x 14336 x 4096 it is 1 to 3 % faster than the same schedule on 32x32x16.
//
// A workgroup walks its tiles as ONE stream of macro steps of 128 k (four K steps of 32): the last
// macro step of a tile already fetches the first operands of the next one, the output tile is
// converted and stored between two steps, and its stores drain while the next tile is being
// multiplied.  Vector-memory operations complete in issue order, so a wait only has to let the
// younger ones stay outstanding.
//
// LDS (160 KB):
//   A   [2 stages][4 waves][128 rows][128 B]  stage d holds k 64d .. 64d+63 of the macro step; the
//       16-byte chunk c of row r sits at position c ^ ((r >> 1) & 7): the LDS serves a 128-bit read 16 lanes
//       at a time from 64 banks, and 16 consecutive rows then land in 16 different 16-byte bank groups
//   W   [2 stages][128 rows][128 B]           composed bf16, same split of the macro step and same swizzle.  A wave
//       composes rows 32w .. 32w+31; between tiles it uses that part of stage 1 to turn the accumulator
//       layout into whole output lines
//
// Macro step m, K step S = 0..3 (slab 4m+S is multiplied; A and W stage S/2).  Slot s multiplies n-tiles
// 4 (s/4 % 2) .. +3 by m-tile s % 4 + 4 (s / 8), so every fragment is read at least four slots before its first use:
//   slots 0-3    read the A fragments of m-tiles 4..7 of slab S (used from slot 8 on)
//   slots 0-7    compose W slab S+2, two codes a slot
//   slot  8      write the composed W slab to its stage (S0, S1: stage 1; S2, S3: stage 0 of macro step m+1)
//   slot  9      S1, S3 only: barrier (the W stage written last is complete, the other one no longer read)
//   slots 10-15  read the eight W fragments of slab S+1
//   slots 12-15  read the A fragments of m-tiles 0..3 of slab S+1
// Global traffic of macro step m (per wave): one A DMA per slot in slots 8..15 of every step -
//   S3 of m-1 and S0     A stage 1 of m     [rows 0..63 first: the MFMAs of S3 slots 0-7 have consumed them]
//   S1 and S2            A stage 0 of m+1   [the same with S1]
//   S0 slots 0..4        W codes (4 x 16 B per thread) and scales (4 bytes) of m+1
// Waits: S1 and S3 slot 12 need the A stage whose last DMA went out in the previous step's slot 15 (4 younger
// operations); the top of S2 needs the W registers of m+1 (16 younger).
// (included from gemm_impl.h, inside namespace mase, after the shared helpers)

constexpr int UM = 512, UN = 128, UK = 32;
constexpr int UMAC = 128;                         // k per macro step: four K steps, one 128-byte line of W codes, two of A
constexpr int U_A_STAGES = 2, U_W_STAGES = 2;
constexpr int U_A_STAGE_BYTES = UM * 64 * 2;      // 64 KB: 512 rows x 64 k
constexpr int U_A_WAVE_BYTES = 128 * 128;         // one wave's 128 rows of a stage
constexpr int U_W_STAGE_BYTES = UN * 64 * 2;      // 16 KB: 128 rows x 64 k, composed
constexpr int U_OUT_WAVE_BYTES = 32 * 128;        // 32 rows x 64 outputs of 2 bytes
constexpr int U_LDS_BYTES = U_A_STAGES * U_A_STAGE_BYTES + U_W_STAGES * U_W_STAGE_BYTES;  // 160 KB

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef float floatx4 __attribute__((ext_vector_type(4)));

// 64 lanes x 16 bytes from per-lane global addresses (sbase + voff) to LDS [lds_addr, lds_addr + 1024)
__device__ inline void dma_1kb(uint32_t lds_addr, uint32_t voff, const void* sbase) {
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2" ::"s"(lds_addr), "v"(voff), "s"(sbase) : "memory");
}
// the same with M0 left as the previous dma_1kb_set_m0 / dma_1kb set it: LDS [m0 + OFF, m0 + OFF + 1024) from
// (sbase + voff + OFF); the immediate offset counts on both sides, so the caller pre-subtracts it from voff
template <int OFF>
__device__ inline void dma_1kb_keep_m0(uint32_t voff, const void* sbase) {
    asm volatile("global_load_lds_dwordx4 %0, %1 offset:%2" ::"v"(voff), "s"(sbase), "n"(OFF) : "memory");
}
__device__ inline void async_load16(u32x4& dst, uint32_t voff, const void* sbase) {
    asm volatile("global_load_dwordx4 %0, %1, %2" : "=v"(dst) : "v"(voff), "s"(sbase) : "memory");
}
__device__ inline void async_load_u8(uint32_t& dst, uint32_t voff, const void* sbase) {
    asm volatile("global_load_ubyte %0, %1, %2" : "=v"(dst) : "v"(voff), "s"(sbase) : "memory");
}
__device__ inline void async_store16(uint32_t voff, const void* sbase, const u32x4& v) {
    // the trailing s_nop keeps a following VALU write of the data registers out of the store's read window
    // (non-temporal: the output is not read again by this kernel and should not displace the operands in L2)
    asm volatile("global_store_dwordx4 %0, %1, %2 nt\n\ts_nop 0" ::"v"(voff), "v"(v), "s"(sbase) : "memory");
}
// wait until at most N vector-memory operations are outstanding; the operands tie the registers
// that the waited-for loads fill to this point of the program
template <int N>
__device__ inline void wait_vmcnt(u32x4& a, uint32_t& b) {
    asm volatile("s_waitcnt vmcnt(%2)" : "+v"(a), "+v"(b) : "n"(N) : "memory");
}

// accumulator register -> VGPR, pinned to this point of the program (a plain read lets the register
// allocator pull hundreds of these copies ahead of the stores that should free their registers)
__device__ inline float acc_read(float a) {
    float v;
    asm volatile("v_accvgpr_read_b32 %0, %1" : "=v"(v) : "a"(a));
    return v;
}

// c += w (16 n x 32 k) * a (16 m x 32 k)^T: lane l supplies k 8 (l >> 4) .. +7 of row l & 15 of either operand and
// holds c[n = 4 (l >> 4) + v][m = l & 15] in element v.  Written as asm so that the accumulators stay in AGPRs and the
// instructions stay in program order.
__device__ inline void mfma16(floatx4& c, const bf16x8& w, const bf16x8& a) {
    asm volatile("v_mfma_f32_16x16x32_bf16 %0, %1, %2, %0" : "+a"(c) : "v"(w), "v"(a));
}
// the same into a zero accumulator
__device__ inline void mfma16_first(floatx4& c, const bf16x8& w, const bf16x8& a) {
    asm volatile("v_mfma_f32_16x16x32_bf16 %0, %1, %2, 0" : "=a"(c) : "v"(w), "v"(a));
}

template <int DT_OUT>
__device__ inline uint2 pack_out4(float r0, float r1, float r2, float r3) {
    static_assert(DT_OUT == BF16 || DT_OUT == F16, "16-bit outputs only");
    if (DT_OUT == BF16) return make_uint2(cvt_pk_bf16(r0, r1), cvt_pk_bf16(r2, r3));
    return make_uint2(f32_bits_to_half_bits(f32_bits(r0)) | (f32_bits_to_half_bits(f32_bits(r1)) << 16),
                      f32_bits_to_half_bits(f32_bits(r2)) | (f32_bits_to_half_bits(f32_bits(r3)) << 16));
}

template <class F, int... I>
__device__ __attribute__((always_inline)) inline void static_for_impl(F&& f, std::integer_sequence<int, I...>) {
    (f(IntC<I>{}), ...);
}
// f(IntC<0>{}), ..., f(IntC<N-1>{}): a loop whose index is a compile-time constant in the body
template <int N, class F>
__device__ __attribute__((always_inline)) inline void static_for(F&& f) {
    static_for_impl(f, std::make_integer_sequence<int, N>{});
}

struct TallTile {
    const uint8_t* a;   // this wave's first A row
    const uint8_t* w;   // first W row (codes)
    const uint8_t* ws;  // first W row (scales)
    size_t y_off;       // byte offset of this tile's output array (K split: one [M, N] array per split)
    int m0, n0;
};

// SC4: the k range of a walk is a multiple of 512, and the scales are fetched 16 bytes per row every fourth macro step
// (a load of 4 bytes per row touches as many cache lines, one per row, and the address unit's time goes by lines)
template <class FW, int DT_OUT, bool SC4>
__global__ __launch_bounds__(kGemmThreads) __attribute__((amdgpu_waves_per_eu(1, 1))) void mxfp_gemm_tall_kernel(
    const uint16_t* __restrict__ a_dense0, const uint8_t* __restrict__ w_scales0, const uint8_t* __restrict__ w_elements0,
    const void* __restrict__ bias, int bias_dtype, void* __restrict__ y0, int M, int N, int K, int tiles_m, int tiles_n, int splits, int64_t y_split_bytes,
    GemmBatch gb, int w_rows_pad) {
    // WT: the weight is a prepared operand (see scaled_operand_kernel): E4M3 bytes without the NaN code and its scales
    // transposed, dword [k / 128][row of w_rows_pad]: the 128 rows' scales of a macro step are 512 contiguous bytes
    constexpr bool WT = has_no_top_code<FW>::value;
    static_assert(!(WT && SC4), "transposed scales come one dword per row and macro step");
    // batched launches: workgroups of grid plane z work on product z (offsets are zero for a single product)
    const uint16_t* __restrict__ const a_dense = a_dense0 + (int64_t)blockIdx.z * gb.a;
    const uint8_t* __restrict__ const w_scales = w_scales0 + (int64_t)blockIdx.z * gb.ws;
    const uint8_t* __restrict__ const w_elements = w_elements0 + (int64_t)blockIdx.z * gb.we;
    void* __restrict__ const y = static_cast<uint8_t*>(y0) + (int64_t)blockIdx.z * gb.y;
    // splits > 1: every tile is walked `splits` times, each time over K / splits of k and into its own [M, N] output array
    extern __shared__ __attribute__((aligned(1024))) uint8_t lds[];
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int k_len = K / splits;                 // the launcher guarantees K % (128 splits) == 0
    const int kblocks = K / 32, nmac = k_len / UMAC;
    const uint32_t lds_aw = (uint32_t)(uintptr_t)lds + (uint32_t)wave * U_A_WAVE_BYTES;  // this wave's rows of stage 0
    uint8_t* const lds_a_ptr = lds + wave * U_A_WAVE_BYTES;
    uint8_t* const lds_w_ptr = lds + U_A_STAGES * U_A_STAGE_BYTES;
    // output staging: the wave's own 32 rows of W stage 1, which nobody reads between the last barrier of a tile
    // and this wave's next write of them
    uint8_t* const lds_out = lds_w_ptr + U_W_STAGE_BYTES + wave * U_OUT_WAVE_BYTES;

    // ---- per-lane constants
    // A DMA: instruction i of a wave covers its rows 8i .. 8i+7; lane l fills position l & 7 of row
    // 8i + (l >> 3), which must hold chunk (l & 7) ^ (row >> 1 & 7) = (l & 7) ^ ((4i + (l >> 4)) & 7)
    uint32_t a_voff[16];
#pragma unroll
    for (int i = 0; i < 16; ++i)
        a_voff[i] = (uint32_t)(8 * i + (lane >> 3)) * (uint32_t)K * 2u + (uint32_t)(((lane & 7) ^ ((4 * i + (lane >> 4)) & 7)) * 16) -
                    (uint32_t)((i & 3) * 1024);  // DMAs 4q+1 .. 4q+3 reuse the M0 of DMA 4q and add an immediate instead
    // fragment reads (A and W alike: same row length and swizzle): for the 16 x 32 operand tile t of K step p (0 / 1
    // within the 64-k stage) lane (q = l >> 4, r = l & 15) reads chunk 4p + q of row 16 t + r
    uint32_t f_off[2];
#pragma unroll
    for (int pp = 0; pp < 2; ++pp)
        f_off[pp] = (uint32_t)(lane & 15) * 128u + (uint32_t)(((4 * pp + (lane >> 4)) ^ ((lane >> 1) & 7)) * 16);
    // W staging: thread t owns codes [16 h, 16 h + 16) of row t >> 1 in every K step, h = t & 1
    const int w_row = tid >> 1, w_half = tid & 1;
    const uint32_t w_voff = (uint32_t)w_row * (uint32_t)K + (uint32_t)w_half * 16u;
    const uint32_t ws_voff = WT ? (uint32_t)w_row * 4u : (uint32_t)w_row * (uint32_t)kblocks;
    const size_t ws_mac_stride = WT ? (size_t)w_rows_pad * 4u : (size_t)(UMAC / 32);   // bytes between a row's scales of consecutive macro steps
    // its 16 bf16 of K step p (0 / 1 within the 64-k stage) are chunks 4p + 2h and 4p + 2h + 1 of the row
    uint32_t w_lds_off[2][2];
#pragma unroll
    for (int pp = 0; pp < 2; ++pp)
#pragma unroll
        for (int e = 0; e < 2; ++e)
            w_lds_off[pp][e] = (uint32_t)w_row * 128u + (uint32_t)(((4 * pp + 2 * w_half + e) ^ ((w_row >> 1) & 7)) * 16);

    const int n_tiles = tiles_m * tiles_n * splits;
    const int per_xcd = (n_tiles + 7) >> 3;
    const int slots = gridDim.x >> 3;
    auto has_tile = [&](int local) __attribute__((always_inline)) { return local < per_xcd && (int)(blockIdx.x & 7) * per_xcd + local < n_tiles; };
    auto tile_at = [&](int local) __attribute__((always_inline)) {
        const int walk = (blockIdx.x & 7) * per_xcd + local;
        const int pos = walk / splits, z = walk - pos * splits;      // the splits of a tile run next to each other
        // groups of 2 tile-rows, rows fastest: the 32 tiles an XCD runs at once form a 2 x 16 patch
        constexpr int GROUP = 2;
        const int in_group = GROUP * tiles_n;
        const int first_m = (pos / in_group) * GROUP;
        const int rows = min(tiles_m - first_m, GROUP);
        const int rr = pos % in_group;
        TallTile t;
        // M need not be a multiple of 512: the last tile row is shifted up to end at row M - 1; the rows it shares with
        // its neighbour are computed twice, identically
        t.m0 = min((first_m + rr % rows) * UM, M - UM);
        t.n0 = (rr / rows) * UN;
        const size_t k0 = (size_t)z * k_len;
        t.a = reinterpret_cast<const uint8_t*>(a_dense) + ((size_t)(t.m0 + wave * 128) * K + k0) * 2;
        t.w = w_elements + (size_t)t.n0 * K + k0;
        t.ws = WT ? w_scales + (size_t)t.n0 * 4u + (k0 / UMAC) * ws_mac_stride : w_scales + (size_t)t.n0 * kblocks + k0 / 32;
        t.y_off = (size_t)z * (size_t)y_split_bytes;
        return t;
    };

    int local = blockIdx.x >> 3;
    if (!has_tile(local)) return;
    TallTile cur = tile_at(local), next = cur;

    // raw W codes and scales: `wn` is the landing area of the next macro step's (its slabs 0, 1 are composed
    // during steps 2, 3 of the current one), `wc[2..3]`, `sc` keep slabs 2, 3 of the current one
    u32x4 wc[4], wn[4];
    uint32_t sc, sn;
    bool any_slow_cur = true, any_slow_nxt = true;  // wave-uniform: a scale among the macro step's four that the fast compose does not take
    auto issue_w_codes = [&](const uint8_t* w_src, auto q_c) __attribute__((always_inline)) {
        constexpr int q = decltype(q_c)::value;
        async_load16(wn[q], w_voff, w_src + q * 32);
    };
    // SC4: the scale bytes of four macro steps (16 per row) arrive in one load every fourth macro step; in the other three
    // the same instruction reads one address for all lanes (one cache line instead of one per row), so that the number
    // of vector-memory operations per macro step, which the waits count, stays the same
    u32x4 sq, sn4;               // landing area of that load; the four dwords in use
    uint32_t ws_voff_now = ws_voff;
    bool sc_fresh = true;        // wave-uniform: the load in flight carries new scales
    int sc_j = 0;                // which dword of sn4 the next macro step uses
    auto issue_w_scales = [&](const uint8_t* ws_src) __attribute__((always_inline)) {
        if constexpr (SC4) asm volatile("global_load_dwordx4 %0, %1, %2" : "=v"(sq) : "v"(ws_voff_now), "s"(ws_src) : "memory");
        else asm volatile("global_load_dword %0, %1, %2" : "=v"(sn) : "v"(ws_voff), "s"(ws_src) : "memory");
    };
    auto take_scales = [&]() __attribute__((always_inline)) {   // after the wait for that load
        if constexpr (SC4) {
            if (sc_fresh) sn4 = sq;
            sn = sc_j == 0 ? sn4.x : sc_j == 1 ? sn4.y : sc_j == 2 ? sn4.z : sn4.w;
        }
    };
    auto issue_w = [&](const uint8_t* w_src, const uint8_t* ws_src) __attribute__((always_inline)) {
#pragma unroll
        for (int q = 0; q < 4; ++q) async_load16(wn[q], w_voff, w_src + q * 32);
        issue_w_scales(ws_src);
    };
    // DMA i (rows 8i .. 8i+7 of the wave) of the 64-k half at `src` into stage `stage`
    auto issue_a = [&](const uint8_t* src, int stage, auto i_c) __attribute__((always_inline)) {
        constexpr int i = decltype(i_c)::value;
        if (i % 4 == 0) dma_1kb(lds_aw + (uint32_t)stage * U_A_STAGE_BYTES + (uint32_t)i * 1024u, a_voff[i], src);
        else dma_1kb_keep_m0<(i % 4) * 1024>(a_voff[i], src);
    };
    auto compose_to = [&](const u32x4& codes, uint32_t scale, int w_stage, int pp) __attribute__((always_inline)) {
        uint4 lo, hi;
        Composer<FW>::template compose16<true>(make_uint4(codes.x, codes.y, codes.z, codes.w), scale, lo, hi);
        uint8_t* const st = lds_w_ptr + w_stage * U_W_STAGE_BYTES;
        *reinterpret_cast<uint4*>(st + w_lds_off[pp][0]) = lo;
        *reinterpret_cast<uint4*>(st + w_lds_off[pp][1]) = hi;
    };

    floatx4 acc[8][8];       // [n-tile j of 16 columns][m-tile i of 16 rows]
    bf16x8 fw_even[8], fw_odd[8];  // the eight W fragments of the K step in flight and of the one after it
    bf16x8 far[8];           // A fragments, one per m-tile

    // ---- prologue of the stream: what a macro step expects to find: A stage 0 landed, the first 8 DMAs
    //      of A stage 1 issued, W slabs 0, 1 composed, wc = the codes of slabs 2, 3, fragments k 0..15 of slab 0
    {
        issue_w(cur.w, cur.ws);
        static_for<16>([&](auto i_c) __attribute__((always_inline)) { issue_a(cur.a, 0, i_c); });
        wait_vmcnt<0>(wn[0], sn);
        wait_vmcnt<0>(wn[1], sn);
        wait_vmcnt<0>(wn[2], sn);
        wait_vmcnt<0>(wn[3], sn);
        if constexpr (SC4) wait_vmcnt<0>(sq, sn);
        take_scales();
        static_for<8>([&](auto i_c) __attribute__((always_inline)) { issue_a(cur.a + 128, 1, i_c); });
        compose_to(wn[0], sn & 0xFFu, 0, 0);
        compose_to(wn[1], (sn >> 8) & 0xFFu, 0, 1);
        wc[2] = wn[2];
        wc[3] = wn[3];
        sc = sn;
        lds_barrier();
#pragma unroll
        for (int j = 0; j < 8; ++j) fw_even[j] = *reinterpret_cast<const bf16x8*>(lds_w_ptr + f_off[0] + j * 2048);
#pragma unroll
        for (int i = 0; i < 4; ++i) far[i] = *reinterpret_cast<const bf16x8*>(lds_a_ptr + f_off[0] + i * 2048);
    }

    // pointers of the macro step in flight: a1_cur = second 64-k half of the current macro step; *_nxt = the
    // next macro step (of this tile or, past its end, of the next one)
    const uint8_t *a1_cur, *a0_nxt, *a1_nxt, *w_nxt, *ws_nxt;

    // K step S of a macro step; FIRST: the accumulators start from zero
    auto step = [&](auto s_c, auto first_c) __attribute__((always_inline)) {
        constexpr int S = decltype(s_c)::value;
        constexpr bool FIRST = decltype(first_c)::value != 0;
        // this step composes slab S+2 (S0, S1: second 64-k half of this macro step, W stage 1; S2, S3: first half
        // of the next macro step, W stage 0)
        constexpr int WST_WRITE = S < 2 ? 1 : 0, PP = S & 1;
        constexpr int ST_NOW = S >> 1, ST_NEXT = ((S + 1) >> 1) & 1;
        const uint8_t* const pa_now = lds_a_ptr + ST_NOW * U_A_STAGE_BYTES + f_off[S & 1];           // slab S
        const uint8_t* const pa_next = lds_a_ptr + ST_NEXT * U_A_STAGE_BYTES + f_off[(S + 1) & 1];   // slab S+1
        const uint8_t* const pw_next = lds_w_ptr + ST_NEXT * U_W_STAGE_BYTES + f_off[(S + 1) & 1];
        bf16x8(&fw_now)[8] = (S & 1) ? fw_odd : fw_even;
        bf16x8(&fw_next)[8] = (S & 1) ? fw_even : fw_odd;
        uint8_t* const wst = lds_w_ptr + WST_WRITE * U_W_STAGE_BYTES;

        if (S == 2) {  // the next macro step's codes and scales are about to be composed
            wait_vmcnt<16>(wn[0], sn);
            wait_vmcnt<16>(wn[1], sn);
            wait_vmcnt<16>(wn[2], sn);
            wait_vmcnt<16>(wn[3], sn);
            if constexpr (SC4) wait_vmcnt<16>(sq, sn);
            take_scales();
            // does any wavefront lane hold a scale among these four that needs the slow compose (255, a block that held inf /
            // NaN, or one so large that the product leaves the bf16 range)?  Checked once
            // per macro step; the patch-up code below runs only then.
            any_slow_nxt = __builtin_amdgcn_ballot_w64(Composer<FW>::any_slow4(sn)) != 0;
        }
        const u32x4& codes = S < 2 ? wc[(S + 2) & 3] : wn[(S + 2) & 3];
        const uint32_t scale = ((S < 2 ? sc : sn) >> (8 * ((S + 2) & 3))) & 0xFFu;
        const Composer<FW> cmp(scale);
        const uint32_t cw[4] = {codes.x, codes.y, codes.z, codes.w};
        uint32_t o[8];

        // the global traffic of slot `slot` of this step
        auto vmem = [&](auto slot_c) __attribute__((always_inline)) {
            constexpr int slot = decltype(slot_c)::value;
            // A: one DMA per slot in the second half of every step (the first half carries the compose).
            // Stage 0 of the next macro step in S1, S2; stage 1 in S3 and S0 of the next macro step.
            if constexpr (slot >= 8) {
                constexpr int h = slot - 8;
                if constexpr (S == 3) issue_a(a1_nxt, 1, IntC<h>{});
                if constexpr (S == 0) issue_a(a1_cur, 1, IntC<8 + h>{});
                if constexpr (S == 1) issue_a(a0_nxt, 0, IntC<h>{});
                if constexpr (S == 2) issue_a(a0_nxt, 0, IntC<8 + h>{});
            }
            // W codes and scales of the next macro step: S0, slots 0..4
            if constexpr (S == 0 && slot < 4) issue_w_codes(w_nxt, IntC<slot>{});
            if constexpr (S == 0 && slot == 4) issue_w_scales(ws_nxt);
        };
        // slot s: the four MFMAs of n-tiles 4 (s >> 2 & 1) .. +3 against m-tile (s & 3) + 4 (s >> 3)
        auto mm4 = [&](auto slot_c) __attribute__((always_inline)) {
            constexpr int slot = decltype(slot_c)::value, i = (slot & 3) + 4 * (slot >> 3), j0 = 4 * ((slot >> 2) & 1);
#pragma unroll
            for (int j = j0; j < j0 + 4; ++j) {
                if (FIRST) mfma16_first(acc[j][i], fw_now[j], far[i]);
                else mfma16(acc[j][i], fw_now[j], far[i]);
            }
        };
        // slots 0..3 fetch the A fragments of m-tiles 4..7 (used from slot 8 on), slots 12..15 those of m-tiles 0..3 of the next slab
        auto a_frag = [&](auto slot_c) __attribute__((always_inline)) {
            constexpr int slot = decltype(slot_c)::value;
            if constexpr (slot < 4) far[4 + slot] = *reinterpret_cast<const bf16x8*>(pa_now + (4 + slot) * 2048);
            if constexpr (slot >= 12) far[slot - 12] = *reinterpret_cast<const bf16x8*>(pa_next + (slot - 12) * 2048);
        };
        auto w_frag = [&](auto j_c) __attribute__((always_inline)) {
            constexpr int j = decltype(j_c)::value;
            fw_next[j] = *reinterpret_cast<const bf16x8*>(pw_next + j * 2048);
        };
#define U_SLOT_END() __builtin_amdgcn_sched_barrier(0)
        // ---- slots 0..7: one pair of the next W slab per slot
        auto pair_at = [&](auto k_c) __attribute__((always_inline)) {
            constexpr int k = decltype(k_c)::value;
            if (k & 1) o[k] = cmp.pair_hi(cw[k >> 1]);
            else o[k] = cmp.pair_lo(cw[k >> 1]);
        };
        static_for<8>([&](auto s_c2) __attribute__((always_inline)) {
            a_frag(s_c2);
            pair_at(s_c2);
            vmem(s_c2);
            mm4(s_c2);
            U_SLOT_END();
        });
        // ---- slots 8..15: the composed slab goes to LDS; the W fragments of the next slab, its first two A fragments.
        //      From here on steps 1 and 3 hand rows 0..63 of the A stage they read back to the DMA engine (rows 64..127
        //      follow in the next step): the MFMAs of slots 0..7 have consumed every fragment of those rows, so the
        //      reads are complete
        {
            uint4 lo = make_uint4(o[0], o[1], o[2], o[3]), hi = make_uint4(o[4], o[5], o[6], o[7]);
            if (S < 2 ? any_slow_cur : any_slow_nxt) Composer<FW>::fix_slow(scale, make_uint4(cw[0], cw[1], cw[2], cw[3]), lo, hi);
            *reinterpret_cast<uint4*>(wst + w_lds_off[PP][0]) = lo;
            *reinterpret_cast<uint4*>(wst + w_lds_off[PP][1]) = hi;
        }
        if (S == 3) {
            any_slow_cur = any_slow_nxt;
            wc[2] = wn[2];
            wc[3] = wn[3];
            sc = sn;
        }
        a_frag(IntC<8>{});
        vmem(IntC<8>{});
        mm4(IntC<8>{});
        U_SLOT_END();
        vmem(IntC<9>{});
        mm4(IntC<9>{});
        U_SLOT_END();
        // S1: W stage 1 is complete and W stage 0 is no longer read; S3: the other way round
        if (S & 1) lds_barrier();
        U_SLOT_END();
        a_frag(IntC<10>{});
        w_frag(IntC<0>{});
        w_frag(IntC<1>{});
        vmem(IntC<10>{});
        mm4(IntC<10>{});
        U_SLOT_END();
        w_frag(IntC<2>{});
        w_frag(IntC<3>{});
        vmem(IntC<11>{});
        mm4(IntC<11>{});
        U_SLOT_END();
        // the A stage read next has landed: steps 1 and 3 start a stage whose last DMA was issued in slot 2
        if (S & 1) asm volatile("s_waitcnt vmcnt(4)" ::: "memory");
        a_frag(IntC<12>{});
        w_frag(IntC<4>{});
        vmem(IntC<12>{});
        mm4(IntC<12>{});
        U_SLOT_END();
        a_frag(IntC<13>{});
        w_frag(IntC<5>{});
        vmem(IntC<13>{});
        mm4(IntC<13>{});
        U_SLOT_END();
        a_frag(IntC<14>{});
        w_frag(IntC<6>{});
        vmem(IntC<14>{});
        mm4(IntC<14>{});
        U_SLOT_END();
        a_frag(IntC<15>{});
        w_frag(IntC<7>{});
        vmem(IntC<15>{});
        mm4(IntC<15>{});
        U_SLOT_END();
#undef U_SLOT_END
    };
    auto macro_step = [&](int mi, auto first_c) __attribute__((always_inline)) {
        a1_cur = cur.a + (size_t)mi * (UMAC * 2) + 128;
        const bool wrap = mi + 1 == nmac;
        const int mn = wrap ? 0 : mi + 1;
        a0_nxt = (wrap ? next.a : cur.a) + (size_t)mn * (UMAC * 2);
        a1_nxt = a0_nxt + 128;
        w_nxt = (wrap ? next.w : cur.w) + (size_t)mn * UMAC;
        if constexpr (SC4) {
            sc_j = mn & 3;
            sc_fresh = sc_j == 0;
            ws_voff_now = sc_fresh ? ws_voff : 0u;
            ws_nxt = (wrap ? next.ws : cur.ws) + (mn >> 2) * 16;
        } else {
            ws_nxt = (wrap ? next.ws : cur.ws) + mn * ws_mac_stride;
        }
        step(IntC<0>{}, first_c);
        step(IntC<1>{}, IntC<0>{});
        step(IntC<2>{}, IntC<0>{});
        step(IntC<3>{}, IntC<0>{});
    };

    for (;;) {
        const int next_local = local + slots;
        const bool more = has_tile(next_local);
        if (more) next = tile_at(next_local);  // else the look-ahead re-reads this tile's first operands (unused)

        macro_step(0, IntC<1>{});
        for (int mi = 1; mi < nmac; ++mi) macro_step(mi, IntC<0>{});

        // ---- output: lane holds, for tile (j, i), y[m][n .. n+3] with
        //      m = m0 + wave*128 + 16 i + lane%16,  n = n0 + 16 j + 4*(lane/16).
        //      Staged through LDS in 8 passes of 32 rows x 64 columns so that every store instruction
        //      writes 8 whole 128-byte lines.
        uint8_t* const y_wave = static_cast<uint8_t*>(y) + cur.y_off + ((size_t)(cur.m0 + wave * 128) * N + cur.n0) * 2;
        // output staging (per wave, 32 rows of 128 bytes, 16-byte chunk c of row r at position c ^ (r & 7)):
        // a lane writes 8 bytes of rows l & 15 and 16 + (l & 15) and reads 16 bytes of row 8 t + (l >> 3).  The lane
        // number goes through an asm so that these addresses are recomputed here instead of living in registers
        // through the K loop.
        uint32_t ol = (uint32_t)lane;
        asm volatile("s_nop 15\n\ts_nop 15" : "+v"(ol));  // also: the last MFMA results are readable after this
        const uint32_t o_row = ol & 15u, o_q = ol >> 4;
        const uint32_t o_rd_off = (ol >> 3) * 128u + (((ol & 7u) ^ (ol >> 3)) * 16u);
        const uint32_t o_st_voff = ((ol >> 3) * (uint32_t)N + (ol & 7u) * 8u) * 2u;
        auto write_tile = [&](auto has_bias_c) __attribute__((always_inline)) {
            constexpr bool HAS_BIAS = decltype(has_bias_c)::value != 0;
            // the tile's 128 bias values, two per lane: column c sits in register c / 64 of lane c % 64
            float bv[2] = {0.0f, 0.0f};
            if (HAS_BIAS) {
                bv[0] = load_bias(bias, bias_dtype, cur.n0 + (int)ol);
                bv[1] = load_bias(bias, bias_dtype, cur.n0 + 64 + (int)ol);
            }
            // the four values of tile (j, i), bias added: columns 16 j + 4 q + t of the workgroup's 128
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
            if constexpr (DT_OUT == F32) {
                // fp32 output: 16 passes of 32 rows x 32 columns (128 bytes per row again); a lane writes the 16 bytes of
                // its four consecutive columns as chunk 4 jj + q of rows 16 ii + (l & 15)
                uint8_t* const y_wave32 = static_cast<uint8_t*>(y) + cur.y_off + ((size_t)(cur.m0 + wave * 128) * N + cur.n0) * 4;
                const uint32_t o_st_voff32 = ((ol >> 3) * (uint32_t)N + (ol & 7u) * 4u) * 4u;
                static_for<4>([&](auto ip_c) __attribute__((always_inline)) {
                    static_for<4>([&](auto jq_c) __attribute__((always_inline)) {
                        constexpr int ip = decltype(ip_c)::value, jq = decltype(jq_c)::value;
                        static_for<4>([&](auto x_c) __attribute__((always_inline)) {
                            constexpr int ii = decltype(x_c)::value >> 1, jj = decltype(x_c)::value & 1;
                            float r[4];
                            values(IntC<2 * jq + jj>{}, IntC<2 * ip + ii>{}, r);
                            const uint32_t row = 16u * ii + o_row;
                            const uint32_t chunk = ((uint32_t)(4 * jj) + o_q) ^ (row & 7u);
                            *reinterpret_cast<uint4*>(lds_out + row * 128u + chunk * 16u) =
                                make_uint4(f32_bits(r[0]), f32_bits(r[1]), f32_bits(r[2]), f32_bits(r[3]));
                        });
                        u32x4 v[4];
                        static_for<4>([&](auto t_c) __attribute__((always_inline)) {
                            constexpr int t = decltype(t_c)::value;
                            v[t] = *reinterpret_cast<const u32x4*>(lds_out + o_rd_off + t * 1024);
                        });
                        static_for<4>([&](auto t_c) __attribute__((always_inline)) {
                            constexpr int t = decltype(t_c)::value;
                            async_store16(o_st_voff32, y_wave32 + ((size_t)(ip * 32 + 8 * t) * N + jq * 32) * 4, v[t]);
                        });
                        __builtin_amdgcn_sched_barrier(0);  // one pass at a time
                    });
                });
            } else
            static_for<4>([&](auto ip_c) __attribute__((always_inline)) {
                static_for<2>([&](auto jh_c) __attribute__((always_inline)) {
                    constexpr int ip = decltype(ip_c)::value, jh = decltype(jh_c)::value;
                    static_for<8>([&](auto x_c) __attribute__((always_inline)) {
                        constexpr int ii = decltype(x_c)::value >> 2, jj = decltype(x_c)::value & 3;
                        float r[4];
                        values(IntC<4 * jh + jj>{}, IntC<2 * ip + ii>{}, r);
                        const uint2 p = pack_out4<DT_OUT>(r[0], r[1], r[2], r[3]);
                        // its 8 bytes are half q & 1 of chunk 2 jj + (q >> 1) of the staged row
                        const uint32_t row = 16u * ii + o_row;
                        const uint32_t chunk = ((uint32_t)(2 * jj) + (o_q >> 1)) ^ (row & 7u);
                        *reinterpret_cast<uint2*>(lds_out + row * 128u + chunk * 16u + (o_q & 1u) * 8u) = p;
                    });
                    u32x4 v[4];
                    static_for<4>([&](auto t_c) __attribute__((always_inline)) {
                        constexpr int t = decltype(t_c)::value;
                        v[t] = *reinterpret_cast<const u32x4*>(lds_out + o_rd_off + t * 1024);
                    });
                    static_for<4>([&](auto t_c) __attribute__((always_inline)) {
                        constexpr int t = decltype(t_c)::value;
                        async_store16(o_st_voff, y_wave + ((size_t)(ip * 32 + 8 * t) * N + jh * 64) * 2, v[t]);
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
    // the look-ahead loads of the last macro step still target LDS and registers: let them finish
    wait_vmcnt<0>(wn[0], sn);
    wait_vmcnt<0>(wn[1], sn);
    wait_vmcnt<0>(wn[2], sn);
    wait_vmcnt<0>(wn[3], sn);
}
