// Tall-tile MXFP GEMM kernel for gfx950: 512 (M) x 128 (N) x 32 (K) tiles, dense bf16 A, 16-bit output, no bias.
//
// Why this shape.  One wavefront can issue only about three other instructions per 32-cycle
// 32x32x16 MFMA without slowing the matrix pipe, so the K loop has to be lean:
//   * the dense A slab goes from global memory straight into LDS (global_load_lds_dwordx4, no
//     VGPRs, no ds_write), four slabs deep;
//   * the MXFP weight slab is composed to bf16 once per 512 output rows instead of once per 256;
//   * all global traffic is issued by hand (inline asm) three K-steps ahead and waited for with
//     one s_waitcnt per step, so the compiler inserts no conservative waits of its own;
//   * every step is laid out by hand in 16 slots of two MFMAs each, the other work spread over
//     them one vector-memory instruction at a time (a burst of them stalls the issuing wave for
//     as long as the address unit needs to drain it).
// Four wavefronts stacked along M, each 128 x 128 (4 x 4 MFMA tiles, 256 accumulator AGPRs).  A wave
// only ever reads the 128 A rows it loaded itself; the 128-row W slab is shared by all four.
//
// A workgroup walks its tiles as ONE stream of K steps: the last three steps of a tile already
// fetch the first three slabs of the next one, the output tile is converted and stored between two
// steps, and its stores drain while the next tile is being multiplied.  Vector-memory operations
// complete in issue order, so a wait only has to let the younger ones stay outstanding.
//
// LDS (160 KB): A stages [4][4 waves][128 rows][64 B], W stages [2][128 rows][64 B], and 4 KB per
// wave to turn the accumulator layout into whole 128-byte output lines.  Rows of 64 bytes carry no
// padding (the DMA writes 1 KB contiguous per instruction); the 16-byte chunk c of row r is kept
// at position c ^ ((r >> 2) & 3), which makes the 128-bit fragment reads of 16 consecutive rows
// hit 16 distinct bank groups.
//
// Step kt (slab kt is being multiplied; A slab s -> stage s % 4 counted over the whole stream,
// W slab s -> stage s % 2, its raw codes in register set s % 2):
//   top         s_waitcnt: slab kt+1 has landed (W codes in registers, A rows in LDS)
//   slots 0-7   MFMAs on k 0..15 of slab kt | read fragments k 16..31 of slab kt | compose W slab
//               kt+1 into its stage | issue the W loads and the first A DMAs of slab kt+3
//   barrier
//   slots 8-15  MFMAs on k 16..31 | read fragments k 0..15 of slab kt+1 | remaining A DMAs
// (included from gemm_impl.h, inside namespace mase, after the shared helpers)

constexpr int UM = 512, UN = 128, UK = 32;
constexpr int U_A_STAGES = 4, U_W_STAGES = 2;
constexpr int U_A_STAGE_BYTES = UM * UK * 2;  // 32 KB
constexpr int U_W_STAGE_BYTES = UN * UK * 2;  // 8 KB
constexpr int U_OUT_WAVE_BYTES = 32 * 128;    // 32 rows x 64 outputs of 2 bytes
constexpr int U_LDS_BYTES = U_A_STAGES * U_A_STAGE_BYTES + U_W_STAGES * U_W_STAGE_BYTES + 4 * U_OUT_WAVE_BYTES;  // 160 KB
constexpr int U_VMEM_PER_STEP = 10;    // 1 code load + 1 scale load + 8 DMAs per wave
constexpr int U_STORES_PER_TILE = 32;  // 16-byte output stores per lane and tile

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

// 64 lanes x 16 bytes from per-lane global addresses (sbase + voff) to LDS [lds_addr, lds_addr + 1024)
__device__ inline void dma_1kb(uint32_t lds_addr, uint32_t voff, const void* sbase) {
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2" ::"s"(lds_addr), "v"(voff), "s"(sbase) : "memory");
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

template <int DT_OUT>
__device__ inline uint2 pack_out4(float r0, float r1, float r2, float r3) {
    static_assert(DT_OUT == BF16 || DT_OUT == F16, "16-bit outputs only");
    if (DT_OUT == BF16) return make_uint2(cvt_pk_bf16(r0, r1), cvt_pk_bf16(r2, r3));
    return make_uint2(f32_bits_to_half_bits(f32_bits(r0)) | (f32_bits_to_half_bits(f32_bits(r1)) << 16),
                      f32_bits_to_half_bits(f32_bits(r2)) | (f32_bits_to_half_bits(f32_bits(r3)) << 16));
}

template <class F, int... I>
__device__ inline void static_for_impl(F&& f, std::integer_sequence<int, I...>) {
    (f(IntC<I>{}), ...);
}
// f(IntC<0>{}), ..., f(IntC<N-1>{}): a loop whose index is a compile-time constant in the body
template <int N, class F>
__device__ inline void static_for(F&& f) {
    static_for_impl(f, std::make_integer_sequence<int, N>{});
}

struct TallTile {
    const uint8_t* a;   // this wave's first A row
    const uint8_t* w;   // first W row (codes)
    const uint8_t* ws;  // first W row (scales)
    int m0, n0;
};

template <class FW, int DT_OUT>
__global__ __launch_bounds__(kGemmThreads) __attribute__((amdgpu_waves_per_eu(1, 1))) void mxfp_gemm_tall_kernel(
    const uint16_t* __restrict__ a_dense, const uint8_t* __restrict__ w_scales, const uint8_t* __restrict__ w_elements,
    void* __restrict__ y, int M, int N, int K, int tiles_m, int tiles_n) {
    extern __shared__ __attribute__((aligned(1024))) uint8_t lds[];
    const uint32_t lds_a = (uint32_t)(uintptr_t)lds;
    uint8_t* const lds_w_ptr = lds + U_A_STAGES * U_A_STAGE_BYTES;

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int kblocks = K / 32, ksteps = K / UK;  // the launcher guarantees an even ksteps >= 4
    uint8_t* const lds_out = lds_w_ptr + U_W_STAGES * U_W_STAGE_BYTES + wave * U_OUT_WAVE_BYTES;

    // ---- per-lane constants
    // A DMA: instruction i of a wave covers its rows 16i .. 16i+15; lane l fills position l & 3 of row
    // 16i + (l >> 2), which must hold chunk (l & 3) ^ (row >> 2 & 3) = (l & 3) ^ (l >> 4 & 3)
    uint32_t a_voff[8];
#pragma unroll
    for (int i = 0; i < 8; ++i)
        a_voff[i] = (uint32_t)(16 * i + (lane >> 2)) * (uint32_t)K * 2u + (uint32_t)(((lane & 3) ^ ((lane >> 4) & 3)) * 16);
    // W staging: thread t owns codes [16 h, 16 h + 16) of row t >> 1, h = t & 1
    const int w_row = tid >> 1, w_half = tid & 1;
    const uint32_t w_voff = (uint32_t)w_row * (uint32_t)K + (uint32_t)w_half * 16u;
    const uint32_t ws_voff = (uint32_t)w_row * (uint32_t)kblocks;
    const uint32_t w_swz = (uint32_t)((w_row >> 2) & 3);
    const uint32_t w_lds_off0 = (uint32_t)w_row * 64u + (((2u * w_half) ^ w_swz) * 16u);
    const uint32_t w_lds_off1 = (uint32_t)w_row * 64u + (((2u * w_half + 1u) ^ w_swz) * 16u);
    // fragment reads: lane (g = l >> 5, r = l & 31) reads chunk 2q + g of row 32 t + r
    const uint32_t f_swz = (uint32_t)((lane >> 2) & 3);
    const uint32_t f_row = (uint32_t)(lane & 31) * 64u;
    const uint32_t f_off_q0 = f_row + ((((uint32_t)(lane >> 5)) ^ f_swz) * 16u);
    const uint32_t f_off_q1 = f_row + (((2u + (uint32_t)(lane >> 5)) ^ f_swz) * 16u);
    const int n_tiles = tiles_m * tiles_n;
    const int per_xcd = (n_tiles + 7) >> 3;
    const int slots = gridDim.x >> 3;
    auto has_tile = [&](int local) { return local < per_xcd && (int)(blockIdx.x & 7) * per_xcd + local < n_tiles; };
    auto tile_at = [&](int local) {
        const int pos = (blockIdx.x & 7) * per_xcd + local;
        // groups of 2 tile-rows, rows fastest: the 32 tiles an XCD runs at once form a 2 x 16 patch
        constexpr int GROUP = 2;
        const int in_group = GROUP * tiles_n;
        const int first_m = (pos / in_group) * GROUP;
        const int rows = min(tiles_m - first_m, GROUP);
        const int rr = pos % in_group;
        TallTile t;
        t.m0 = (first_m + rr % rows) * UM;
        t.n0 = (rr / rows) * UN;
        t.a = reinterpret_cast<const uint8_t*>(a_dense) + ((size_t)(t.m0 + wave * 128) * K) * 2;
        t.w = w_elements + (size_t)t.n0 * K;
        t.ws = w_scales + (size_t)t.n0 * kblocks;
        return t;
    };

    int local = blockIdx.x >> 3;
    if (!has_tile(local)) return;
    TallTile cur = tile_at(local), next = cur;
    int gbase = 0;  // stream number of the current tile's slab 0 (mod 4 is all that matters)

    u32x4 rw[2];
    uint32_t sw[2];
    // W codes + scale of `slab` of tile `t` into register set `set`
    auto issue_w = [&](const TallTile& t, int slab, auto set_c) {
        constexpr int set = decltype(set_c)::value;
        async_load16(rw[set], w_voff, t.w + (size_t)slab * UK);
        async_load_u8(sw[set], ws_voff, t.ws + slab);
    };
    // DMA i (rows 16i .. 16i+15 of the wave) of the slab at `src` into the stage at `dst`
    auto issue_a = [&](const uint8_t* src, uint32_t dst, int i) { dma_1kb(dst + i * 1024, a_voff[i], src); };
    auto a_src_of = [&](const TallTile& t, int slab) { return t.a + (size_t)slab * (UK * 2); };
    auto a_dst_of = [&](int stream_slab) {
        return lds_a + (uint32_t)(stream_slab & (U_A_STAGES - 1)) * U_A_STAGE_BYTES + (uint32_t)wave * (128 * 64);
    };
    auto compose_all = [&](int w_stage, auto set_c) {
        constexpr int set = decltype(set_c)::value;
        uint4 lo, hi;
        const uint4 codes = make_uint4(rw[set].x, rw[set].y, rw[set].z, rw[set].w);
        Composer<FW>::template compose16<true>(codes, sw[set], lo, hi);
        uint8_t* const st = lds_w_ptr + w_stage * U_W_STAGE_BYTES;
        *reinterpret_cast<uint4*>(st + w_lds_off0) = lo;
        *reinterpret_cast<uint4*>(st + w_lds_off1) = hi;
    };

    floatx16 acc[4][4];  // [n-tile j][m-tile i]
    bf16x8 fa0[4], fw0[4], fa1[4], fw1[4];

    // ---- prologue of the stream: slabs 0..2 of the first tile landed, W slab 0 composed,
    //      fragments k 0..15 of slab 0 in registers
    {
        issue_w(cur, 0, IntC<0>{});
#pragma unroll
        for (int i = 0; i < 8; ++i) issue_a(a_src_of(cur, 0), a_dst_of(0), i);
        issue_w(cur, 1, IntC<1>{});
#pragma unroll
        for (int i = 0; i < 8; ++i) issue_a(a_src_of(cur, 1), a_dst_of(1), i);
        wait_vmcnt<U_VMEM_PER_STEP>(rw[0], sw[0]);
        compose_all(0, IntC<0>{});
        issue_w(cur, 2, IntC<0>{});
#pragma unroll
        for (int i = 0; i < 8; ++i) issue_a(a_src_of(cur, 2), a_dst_of(2), i);
        wait_vmcnt<0>(rw[1], sw[1]);
        wait_vmcnt<0>(rw[0], sw[0]);
        lds_barrier();
        const uint8_t* const pa = lds + wave * (128 * 64) + f_off_q0;
        const uint8_t* const pw = lds_w_ptr + f_off_q0;
#pragma unroll
        for (int i = 0; i < 4; ++i) fa0[i] = *reinterpret_cast<const bf16x8*>(pa + i * 2048);
#pragma unroll
        for (int j = 0; j < 4; ++j) fw0[j] = *reinterpret_cast<const bf16x8*>(pw + j * 2048);
    }

    // one K step; FIRST: the accumulators start from zero; WAITN: operations younger than slab kt+1
    auto step = [&](auto first_c, auto set_c, auto wait_c, int kt) {
        constexpr bool FIRST = decltype(first_c)::value != 0;
        constexpr int set = decltype(set_c)::value;  // (kt + 1) & 1
        constexpr int WAITN = decltype(wait_c)::value;
        wait_vmcnt<WAITN>(rw[set], sw[set]);

        const int s_now = gbase + kt;
        const uint8_t* const pa1 = lds + (s_now & 3) * U_A_STAGE_BYTES + wave * (128 * 64) + f_off_q1;
        const uint8_t* const pw1 = lds_w_ptr + (set ^ 1) * U_W_STAGE_BYTES + f_off_q1;
        const uint8_t* const pa0 = lds + ((s_now + 1) & 3) * U_A_STAGE_BYTES + wave * (128 * 64) + f_off_q0;
        const uint8_t* const pw0 = lds_w_ptr + set * U_W_STAGE_BYTES + f_off_q0;
        uint8_t* const wst = lds_w_ptr + set * U_W_STAGE_BYTES;
        int s3 = kt + 3;
        const bool wrap = s3 >= ksteps;
        if (wrap) s3 -= ksteps;
        const uint8_t* const a_src = (wrap ? next.a : cur.a) + (size_t)s3 * (UK * 2);
        const uint8_t* const w_src = (wrap ? next.w : cur.w) + (size_t)s3 * UK;
        const uint8_t* const ws_src = (wrap ? next.ws : cur.ws) + s3;
        const uint32_t a_dst = a_dst_of(s_now + 3);

        const Composer<FW> cmp(sw[set]);
        const uint32_t cw[4] = {rw[set].x, rw[set].y, rw[set].z, rw[set].w};
        uint32_t o[8];

        auto mm = [&](const bf16x8(&af)[4], const bf16x8(&wf)[4], int j, int i, bool zero) {
            if (zero) {
                floatx16 z;
#pragma unroll
                for (int v = 0; v < 16; ++v) z[v] = 0.0f;
                acc[j][i] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(wf[j], af[i], z, 0, 0, 0);
            } else {
                acc[j][i] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(wf[j], af[i], acc[j][i], 0, 0, 0);
            }
        };
#define U_SLOT_END() __builtin_amdgcn_sched_barrier(0)
        // ---- slots 0..7: k 0..15
        fa1[0] = *reinterpret_cast<const bf16x8*>(pa1);
        fa1[1] = *reinterpret_cast<const bf16x8*>(pa1 + 2048);
        cmp.pair2(cw[0], o[0], o[1]);
        mm(fa0, fw0, 0, 0, FIRST);
        mm(fa0, fw0, 0, 1, FIRST);
        U_SLOT_END();
        fa1[2] = *reinterpret_cast<const bf16x8*>(pa1 + 4096);
        fa1[3] = *reinterpret_cast<const bf16x8*>(pa1 + 6144);
        cmp.pair2(cw[1], o[2], o[3]);
        mm(fa0, fw0, 0, 2, FIRST);
        mm(fa0, fw0, 0, 3, FIRST);
        U_SLOT_END();
        fw1[0] = *reinterpret_cast<const bf16x8*>(pw1);
        fw1[1] = *reinterpret_cast<const bf16x8*>(pw1 + 2048);
        cmp.pair2(cw[2], o[4], o[5]);
        mm(fa0, fw0, 1, 0, FIRST);
        mm(fa0, fw0, 1, 1, FIRST);
        U_SLOT_END();
        fw1[2] = *reinterpret_cast<const bf16x8*>(pw1 + 4096);
        fw1[3] = *reinterpret_cast<const bf16x8*>(pw1 + 6144);
        cmp.pair2(cw[3], o[6], o[7]);
        mm(fa0, fw0, 1, 2, FIRST);
        mm(fa0, fw0, 1, 3, FIRST);
        U_SLOT_END();
        {
            uint4 lo = make_uint4(o[0], o[1], o[2], o[3]), hi = make_uint4(o[4], o[5], o[6], o[7]);
            Composer<FW>::fix255(sw[set], make_uint4(cw[0], cw[1], cw[2], cw[3]), lo, hi);
            *reinterpret_cast<uint4*>(wst + w_lds_off0) = lo;
            *reinterpret_cast<uint4*>(wst + w_lds_off1) = hi;
        }
        U_SLOT_END();
        async_load16(rw[set], w_voff, w_src);  // the set's old contents were consumed above
        async_load_u8(sw[set], ws_voff, ws_src);
        mm(fa0, fw0, 2, 0, FIRST);
        mm(fa0, fw0, 2, 1, FIRST);
        U_SLOT_END();
        issue_a(a_src, a_dst, 0);
        mm(fa0, fw0, 2, 2, FIRST);
        mm(fa0, fw0, 2, 3, FIRST);
        U_SLOT_END();
        issue_a(a_src, a_dst, 1);
        mm(fa0, fw0, 3, 0, FIRST);
        mm(fa0, fw0, 3, 1, FIRST);
        U_SLOT_END();
        issue_a(a_src, a_dst, 2);
        mm(fa0, fw0, 3, 2, FIRST);
        mm(fa0, fw0, 3, 3, FIRST);
        U_SLOT_END();
        lds_barrier();  // every wave's part of W slab kt+1 is in LDS; W slab kt is no longer read
        U_SLOT_END();
        // ---- slots 8..15: k 16..31
        fa0[0] = *reinterpret_cast<const bf16x8*>(pa0);
        fa0[1] = *reinterpret_cast<const bf16x8*>(pa0 + 2048);
        issue_a(a_src, a_dst, 3);
        mm(fa1, fw1, 0, 0, false);
        mm(fa1, fw1, 0, 1, false);
        U_SLOT_END();
        fa0[2] = *reinterpret_cast<const bf16x8*>(pa0 + 4096);
        fa0[3] = *reinterpret_cast<const bf16x8*>(pa0 + 6144);
        issue_a(a_src, a_dst, 4);
        mm(fa1, fw1, 0, 2, false);
        mm(fa1, fw1, 0, 3, false);
        U_SLOT_END();
        fw0[0] = *reinterpret_cast<const bf16x8*>(pw0);
        fw0[1] = *reinterpret_cast<const bf16x8*>(pw0 + 2048);
        issue_a(a_src, a_dst, 5);
        mm(fa1, fw1, 1, 0, false);
        mm(fa1, fw1, 1, 1, false);
        U_SLOT_END();
        fw0[2] = *reinterpret_cast<const bf16x8*>(pw0 + 4096);
        fw0[3] = *reinterpret_cast<const bf16x8*>(pw0 + 6144);
        issue_a(a_src, a_dst, 6);
        mm(fa1, fw1, 1, 2, false);
        mm(fa1, fw1, 1, 3, false);
        U_SLOT_END();
        issue_a(a_src, a_dst, 7);
        mm(fa1, fw1, 2, 0, false);
        mm(fa1, fw1, 2, 1, false);
        U_SLOT_END();
        mm(fa1, fw1, 2, 2, false);
        mm(fa1, fw1, 2, 3, false);
        mm(fa1, fw1, 3, 0, false);
        mm(fa1, fw1, 3, 1, false);
        mm(fa1, fw1, 3, 2, false);
        mm(fa1, fw1, 3, 3, false);
        U_SLOT_END();
#undef U_SLOT_END
    };

    // after a tile's stores, the first two steps of the next tile may leave them outstanding
    typedef IntC<U_VMEM_PER_STEP> WaitSteady;
    typedef IntC<U_VMEM_PER_STEP + U_STORES_PER_TILE> WaitAfterStores;

    for (;;) {
        const int next_local = local + slots;
        const bool more = has_tile(next_local);
        if (more) next = tile_at(next_local);  // else the look-ahead re-reads this tile's first slabs (unused)

        step(IntC<1>{}, IntC<1>{}, WaitAfterStores{}, 0);
        step(IntC<0>{}, IntC<0>{}, WaitAfterStores{}, 1);
        for (int kt = 2; kt < ksteps; kt += 2) {
            step(IntC<0>{}, IntC<1>{}, WaitSteady{}, kt);
            step(IntC<0>{}, IntC<0>{}, WaitSteady{}, kt + 1);
        }

        // ---- output: lane holds, for tile (j, i) and g = 0..3, y[m][n .. n+3] with
        //      m = m0 + wave*128 + i*32 + lane%32,  n = n0 + j*32 + 8*g + 4*(lane/32).
        //      Staged through LDS in 8 passes of 32 rows x 64 columns so that every store instruction
        //      writes 8 whole 128-byte lines.
        uint8_t* const y_wave = static_cast<uint8_t*>(y) + ((size_t)(cur.m0 + wave * 128) * N + cur.n0) * 2;
        // output staging (per wave, 32 rows of 128 bytes, 16-byte chunk c of row r at position c ^ (r & 7)):
        // a lane writes 8 bytes of row l & 31 and reads 16 bytes of row 8 t + (l >> 3).  The lane number goes
        // through an empty asm so that these addresses are recomputed here instead of living in registers
        // through the K loop.
        uint32_t ol = (uint32_t)lane;
        asm volatile("s_nop 15\n\ts_nop 15" : "+v"(ol));  // also: the last MFMA results are readable after this
        const uint32_t o_row = ol & 31u, o_half = ol >> 5;
        const uint32_t o_rd_off = (ol >> 3) * 128u + (((ol & 7u) ^ (ol >> 3)) * 16u);
        const uint32_t o_st_voff = ((ol >> 3) * (uint32_t)N + (ol & 7u) * 8u) * 2u;
        static_for<4>([&](auto i_c) {
            static_for<2>([&](auto jh_c) {
                constexpr int i = decltype(i_c)::value, jh = decltype(jh_c)::value;
                static_for<8>([&](auto jg_c) {
                    constexpr int jj = decltype(jg_c)::value >> 2, g = decltype(jg_c)::value & 3, j = 2 * jh + jj;
                    const uint2 p = pack_out4<DT_OUT>(acc_read(acc[j][i][4 * g]), acc_read(acc[j][i][4 * g + 1]),
                                                      acc_read(acc[j][i][4 * g + 2]), acc_read(acc[j][i][4 * g + 3]));
                    const uint32_t chunk = (uint32_t)(jj * 4 + g) ^ (o_row & 7u);
                    *reinterpret_cast<uint2*>(lds_out + o_row * 128u + chunk * 16u + o_half * 8u) = p;
                });
                static_for<4>([&](auto t_c) {
                    constexpr int t = decltype(t_c)::value;
                    const u32x4 v = *reinterpret_cast<const u32x4*>(lds_out + o_rd_off + t * 1024);
                    async_store16(o_st_voff, y_wave + ((size_t)(i * 32 + 8 * t) * N + jh * 64) * 2, v);
                });
                __builtin_amdgcn_sched_barrier(0);  // one pass at a time: keeps the accumulator reads from piling up in VGPRs
            });
        });

        if (!more) break;
        cur = next;
        local = next_local;
        gbase = (gbase + ksteps) & 3;
    }
    // the look-ahead loads of the last steps still target LDS and registers: let them finish
    wait_vmcnt<0>(rw[0], sw[0]);
    wait_vmcnt<0>(rw[1], sw[1]);
}
