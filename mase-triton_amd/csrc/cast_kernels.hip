// Bandwidth-bound cast kernels for gfx950: minifloat extract / compose / fused QDQ and MXFP
// extract / compose / fused QDQ, plus their C-ABI entry points.
//
// Data layout: every tensor is a flat array in HBM.  A lane moves EPT consecutive elements per
// step with 128-bit accesses; consecutive lanes take consecutive EPT-runs, so a wavefront reads
// and writes whole contiguous segments.  An MXFP block of B elements is owned by B/EPT adjacent
// lanes, which agree on the block maximum with xor-shuffles; one of them stores the scale byte.
#include "../../include/mase_hip.h"
#include "mase_host.h"
#include "mxfp_compose.h"
#include "swiglu.h"

namespace mase {

constexpr int kThreads = 256;
// 128-bit steps per lane and launch: one is fastest on every measured size (more, smaller workgroups in flight)
#ifndef MASE_QDQ_NT
#define MASE_QDQ_NT 1
#endif
#ifndef MASE_UNROLL_COMPOSE
#define MASE_UNROLL_COMPOSE 2
#endif
#ifndef MASE_UNROLL_SMALL
#define MASE_UNROLL_SMALL 1
#endif
#ifndef MASE_UNROLL_MXFP
#define MASE_UNROLL_MXFP 1
#endif
#ifndef MASE_UNROLL_EXTRACT
#define MASE_UNROLL_EXTRACT 2
#endif
#ifndef MASE_UNROLL_PACKED
#define MASE_UNROLL_PACKED 2
#endif

typedef float floatx2 __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef _Float16 halfx2 __attribute__((ext_vector_type(2)));

// ------------------------------------------------------------------------------ vector I/O
// 128- and 64-bit accesses of the streaming kernels.  Every byte is touched once, so loads and stores are
// marked non-temporal (no reuse to keep in the caches); measured faster on all kernels but the fp32 -> fp32
// fused minifloat pass, which passes NT = false.
typedef uint32_t u32v4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32v2 __attribute__((ext_vector_type(2)));
template <bool NT = true>
__device__ inline uint4 ld128(const void* p) {
    if (NT) {
        const u32v4 v = __builtin_nontemporal_load(static_cast<const u32v4*>(p));
        return make_uint4(v.x, v.y, v.z, v.w);
    }
    return *static_cast<const uint4*>(p);
}
__device__ inline uint2 ld64(const void* p) {
    const u32v2 v = __builtin_nontemporal_load(static_cast<const u32v2*>(p));
    return make_uint2(v.x, v.y);
}
template <bool NT = true>
__device__ inline void st128(void* p, uint4 v) {
    if (NT) __builtin_nontemporal_store(u32v4{v.x, v.y, v.z, v.w}, static_cast<u32v4*>(p));
    else *static_cast<uint4*>(p) = v;
}
__device__ inline void st64(void* p, uint2 v) { __builtin_nontemporal_store(u32v2{v.x, v.y}, static_cast<u32v2*>(p)); }

// EPT elements starting at element index `off` of a flat array, as fp32 bit patterns.
template <int DT, int EPT, bool NT = true>
__device__ inline void load_bits(const void* base, int64_t off, uint32_t (&u)[EPT]) {
    if (DT == F32) {
        const uint4* p = reinterpret_cast<const uint4*>(static_cast<const uint32_t*>(base) + off);
#pragma unroll
        for (int v = 0; v < EPT / 4; ++v) {
            const uint4 r = ld128<NT>(p + v);
            u[4 * v + 0] = r.x; u[4 * v + 1] = r.y; u[4 * v + 2] = r.z; u[4 * v + 3] = r.w;
        }
    } else {
        const uint4* p = reinterpret_cast<const uint4*>(static_cast<const uint16_t*>(base) + off);
#pragma unroll
        for (int v = 0; v < EPT / 8; ++v) {
            const uint4 r = ld128<NT>(p + v);
            const uint32_t w[4] = {r.x, r.y, r.z, r.w};
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                if (DT == BF16) {
                    u[8 * v + 2 * j] = w[j] << 16;
                    u[8 * v + 2 * j + 1] = w[j] & 0xFFFF0000u;
                } else {
                    u[8 * v + 2 * j] = half_bits_to_f32_bits(w[j] & 0xFFFFu);
                    u[8 * v + 2 * j + 1] = half_bits_to_f32_bits(w[j] >> 16);
                }
            }
        }
    }
}

template <int DT>
__device__ inline uint32_t load_bits_scalar(const void* base, int64_t i) {
    if (DT == F32) return static_cast<const uint32_t*>(base)[i];
    const uint32_t h = static_cast<const uint16_t*>(base)[i];
    return DT == BF16 ? h << 16 : half_bits_to_f32_bits(h);
}

__device__ inline uint32_t pack_bf16(float a, float b) {
    const bf16x2 r = __builtin_convertvector(floatx2{a, b}, bf16x2);
    return __builtin_bit_cast(uint32_t, r);
}
__device__ inline uint32_t pack_f16(float a, float b) {
    return f32_bits_to_half_bits(f32_bits(a)) | (f32_bits_to_half_bits(f32_bits(b)) << 16);
}

template <int DT, int EPT, bool NT = true>
__device__ inline void store_vals(void* base, int64_t off, const float (&y)[EPT]) {
    if (DT == F32) {
        uint4* p = reinterpret_cast<uint4*>(static_cast<float*>(base) + off);
#pragma unroll
        for (int v = 0; v < EPT / 4; ++v)
            st128<NT>(p + v, make_uint4(f32_bits(y[4 * v]), f32_bits(y[4 * v + 1]), f32_bits(y[4 * v + 2]), f32_bits(y[4 * v + 3])));
    } else {
        uint4* p = reinterpret_cast<uint4*>(static_cast<uint16_t*>(base) + off);
#pragma unroll
        for (int v = 0; v < EPT / 8; ++v) {
            uint32_t w[4];
#pragma unroll
            for (int j = 0; j < 4; ++j)
                w[j] = DT == BF16 ? pack_bf16(y[8 * v + 2 * j], y[8 * v + 2 * j + 1])
                                  : pack_f16(y[8 * v + 2 * j], y[8 * v + 2 * j + 1]);
            st128<NT>(p + v, make_uint4(w[0], w[1], w[2], w[3]));
        }
    }
}

template <int DT>
__device__ inline void store_val_scalar(void* base, int64_t i, float y) {
    if (DT == F32) static_cast<float*>(base)[i] = y;
    else if (DT == BF16) static_cast<uint16_t*>(base)[i] = (uint16_t)(pack_bf16(y, 0.0f) & 0xFFFFu);
    else static_cast<uint16_t*>(base)[i] = (uint16_t)f32_bits_to_half_bits(f32_bits(y));
}

// ------------------------------------------------------------------------------ minifloat
template <int DT_IN, class F, int UNROLL>
__global__ __launch_bounds__(kThreads) void extract_minifloat_kernel(const void* __restrict__ x,
                                                                      uint16_t* __restrict__ codes, int64_t n, F f) {
    constexpr int EPT = 8;
    const int64_t n_chunks = n / EPT;
    const int64_t chunk0 = (int64_t)blockIdx.x * (UNROLL * kThreads) + threadIdx.x;
    uint32_t u[UNROLL][EPT];
#pragma unroll
    for (int r = 0; r < UNROLL; ++r) {
        const int64_t c = chunk0 + (int64_t)r * kThreads;
        if (c < n_chunks) load_bits<DT_IN, EPT>(x, c * EPT, u[r]);
    }
#pragma unroll
    for (int r = 0; r < UNROLL; ++r) {
        const int64_t c = chunk0 + (int64_t)r * kThreads;
        if (c < n_chunks) {
            uint32_t w[4];
#pragma unroll
            for (int j = 0; j < 4; ++j)
                w[j] = encode_f32_bits(u[r][2 * j], f) | (encode_f32_bits(u[r][2 * j + 1], f) << 16);
            st128(codes + c * EPT, make_uint4(w[0], w[1], w[2], w[3]));
        }
    }
    if (blockIdx.x == 0 && threadIdx.x < (n % EPT)) {
        const int64_t i = n_chunks * EPT + threadIdx.x;
        codes[i] = (uint16_t)encode_f32_bits(load_bits_scalar<DT_IN>(x, i), f);
    }
}

template <int DT_OUT, class F, int UNROLL>
__global__ __launch_bounds__(kThreads) void compose_minifloat_kernel(const uint16_t* __restrict__ codes,
                                                                      void* __restrict__ out, int64_t n, F f) {
    constexpr int EPT = 8;
    const int64_t n_chunks = n / EPT;
    const int64_t chunk0 = (int64_t)blockIdx.x * (UNROLL * kThreads) + threadIdx.x;
    uint4 raw[UNROLL];
#pragma unroll
    for (int r = 0; r < UNROLL; ++r) {
        const int64_t c = chunk0 + (int64_t)r * kThreads;
        if (c < n_chunks) raw[r] = ld128(codes + c * EPT);
    }
#pragma unroll
    for (int r = 0; r < UNROLL; ++r) {
        const int64_t c = chunk0 + (int64_t)r * kThreads;
        if (c < n_chunks) {
            const uint32_t w[4] = {raw[r].x, raw[r].y, raw[r].z, raw[r].w};
            float y[EPT];
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                y[2 * j] = decode_f32(w[j] & 0xFFFFu, f);
                y[2 * j + 1] = decode_f32(w[j] >> 16, f);
            }
            store_vals<DT_OUT, EPT>(out, c * EPT, y);
        }
    }
    if (blockIdx.x == 0 && threadIdx.x < (n % EPT)) {
        const int64_t i = n_chunks * EPT + threadIdx.x;
        store_val_scalar<DT_OUT>(out, i, decode_f32(codes[i], f));
    }
}

template <int DT_IN, int DT_OUT, class F, int UNROLL>
__global__ __launch_bounds__(kThreads) void qdq_minifloat_kernel(const void* x, void* out, int64_t n, F f) {
    constexpr int EPT = 8;
    const int64_t n_chunks = n / EPT;
    const int64_t chunk0 = (int64_t)blockIdx.x * (UNROLL * kThreads) + threadIdx.x;
    uint32_t u[UNROLL][EPT];
#pragma unroll
    for (int r = 0; r < UNROLL; ++r) {
        const int64_t c = chunk0 + (int64_t)r * kThreads;
        if (c < n_chunks) load_bits<DT_IN, EPT, false>(x, c * EPT, u[r]);
    }
    // the scalar tail reads before anything is written, so that `out` may alias `x`
    uint32_t tail_bits = 0;
    const bool has_tail = blockIdx.x == 0 && threadIdx.x < (n % EPT);
    if (has_tail) tail_bits = load_bits_scalar<DT_IN>(x, n_chunks * EPT + threadIdx.x);
#pragma unroll
    for (int r = 0; r < UNROLL; ++r) {
        const int64_t c = chunk0 + (int64_t)r * kThreads;
        if (c < n_chunks) {
            float y[EPT];
#pragma unroll
            for (int j = 0; j < EPT; ++j) y[j] = decode_f32(encode_f32_bits(u[r][j], f), f);
            store_vals<DT_OUT, EPT, false>(out, c * EPT, y);
        }
    }
    if (has_tail) store_val_scalar<DT_OUT>(out, n_chunks * EPT + threadIdx.x, decode_f32(encode_f32_bits(tail_bits, f), f));
}

// fp32 sides.  With 8 consecutive elements per lane a lane's two 16-byte fp32 accesses are 32 bytes apart from its neighbour's, so
// every load or store instruction of a wavefront covers 2 KB and uses half of it (the stores then reach memory as partial
// lines: 1.10 x the output bytes measured).  Here a wavefront owns 512 consecutive elements and a lane two runs of four, 256
// elements apart: every instruction covers one contiguous kilobyte on the fp32 side (512 bytes on the 16-bit side).
// MODE 0: fp32 -> codes, 1: codes -> fp32, 2: fp32 -> fp32 (quantise-dequantise; `out` may alias `x`: a lane reads what it writes).
// n must be a multiple of 512; the callers give the rest to the kernels above.
template <int MODE, class F>
__global__ __launch_bounds__(kThreads) void minifloat_f32_kernel(const void* x, void* out, int64_t n, F f) {
    const int64_t wave_first = ((int64_t)blockIdx.x * (kThreads / 64) + (threadIdx.x >> 6)) * 512;
    if (wave_first >= n) return;
    const int lane = threadIdx.x & 63;
    uint32_t code[8];
    if (MODE == 1) {
        const uint16_t* c = static_cast<const uint16_t*>(x) + wave_first + 4 * lane;
        const uint2 a = ld64(c), b = ld64(c + 256);
        const uint32_t w[4] = {a.x, a.y, b.x, b.y};
#pragma unroll
        for (int j = 0; j < 4; ++j) { code[2 * j] = w[j] & 0xFFFFu; code[2 * j + 1] = w[j] >> 16; }
    } else {
        const uint32_t* p = static_cast<const uint32_t*>(x) + wave_first + 4 * lane;
        const uint4 a = ld128<MASE_QDQ_NT || MODE == 0>(p), b = ld128<MASE_QDQ_NT || MODE == 0>(p + 256);
        const uint32_t u[8] = {a.x, a.y, a.z, a.w, b.x, b.y, b.z, b.w};
        // inf / NaN anywhere in the wavefront's 512 elements: the per-element routine for all of them
        uint32_t amax = 0;
#pragma unroll
        for (int j = 0; j < 8; ++j) amax = max(amax, u[j] & 0x7FFFFFFFu);
        bool fast = false;
        if constexpr (F::kStatic) {
            fast = __builtin_amdgcn_ballot_w64(amax >= 0x7F800000u) == 0;
            if (fast) {
#pragma unroll
                for (int j = 0; j < 8; ++j) code[j] = encode_f32_finite_rn(u[j], f);
            }
        }
        if (!fast) {
#pragma unroll
            for (int j = 0; j < 8; ++j) code[j] = encode_f32_bits(u[j], f);
        }
    }
    if (MODE == 0) {
        uint16_t* c = static_cast<uint16_t*>(out) + wave_first + 4 * lane;
        st64(c, make_uint2(code[0] | (code[1] << 16), code[2] | (code[3] << 16)));
        st64(c + 256, make_uint2(code[4] | (code[5] << 16), code[6] | (code[7] << 16)));
    } else {
        float y[8];
#pragma unroll
        for (int j = 0; j < 8; ++j) y[j] = decode_f32(code[j], f);
        float* o = static_cast<float*>(out) + wave_first + 4 * lane;
        st128<MASE_QDQ_NT || MODE == 1>(o, make_uint4(f32_bits(y[0]), f32_bits(y[1]), f32_bits(y[2]), f32_bits(y[3])));
        st128<MASE_QDQ_NT || MODE == 1>(o + 256, make_uint4(f32_bits(y[4]), f32_bits(y[5]), f32_bits(y[6]), f32_bits(y[7])));
    }
}

// ------------------------------------------------------------------------------ MXFP
// Largest |x| bit pattern over the `lpb` adjacent lanes that share a block.
__device__ inline uint32_t block_max(uint32_t amax, int lpb) {
    for (int off = 1; off < lpb; off <<= 1) {
        const uint32_t o = (uint32_t)__shfl_xor((int)amax, off);
        amax = o > amax ? o : amax;
    }
    return amax;
}

template <int DT_IN, class F, int EPT>
__device__ inline void mxfp_encode_run(const uint32_t (&u)[EPT], int lpb, const F& f, uint32_t (&code)[EPT],
                                       uint32_t& scale) {
    uint32_t amax = 0;
#pragma unroll
    for (int j = 0; j < EPT; ++j) {
        const uint32_t a = u[j] & 0x7FFFFFFFu;
        amax = a > amax ? a : amax;
    }
    amax = block_max(amax, lpb);
    const int se = shared_exponent<F, DT_IN != F32>(amax, f);
    scale = amax < 0x00800000u ? 0u : (uint32_t)(se + 127);  // all elements flushed -> 0
#pragma unroll
    for (int j = 0; j < EPT; ++j) code[j] = encode_mxfp_element(u[j], se, f);
}

// Vector path: B % EPT == 0, B / EPT a power of two <= 64.  lpb = lanes per block.
template <int DT_IN, class F, int EPT, int UNROLL>
__global__ __launch_bounds__(kThreads) void extract_mxfp_kernel(const void* __restrict__ x, uint8_t* __restrict__ scales,
                                                                 uint8_t* __restrict__ elements, int64_t n, int lpb,
                                                                 int lpb_shift, F f) {
    const int64_t n_chunks = n / EPT;
    const int64_t chunk0 = (int64_t)blockIdx.x * (UNROLL * kThreads) + threadIdx.x;
    uint32_t u[UNROLL][EPT];
#pragma unroll
    for (int r = 0; r < UNROLL; ++r) {
        const int64_t c = chunk0 + (int64_t)r * kThreads;
        if (c < n_chunks) load_bits<DT_IN, EPT>(x, c * EPT, u[r]);
        else {
#pragma unroll
            for (int j = 0; j < EPT; ++j) u[r][j] = 0u;
        }
    }
#pragma unroll
    for (int r = 0; r < UNROLL; ++r) {
        const int64_t c = chunk0 + (int64_t)r * kThreads;
        uint32_t code[EPT], scale;
        mxfp_encode_run<DT_IN, F, EPT>(u[r], lpb, f, code, scale);  // all lanes take part in the shuffles
        if (c < n_chunks) {
            uint32_t w[EPT / 4];
#pragma unroll
            for (int j = 0; j < EPT / 4; ++j)
                w[j] = code[4 * j] | (code[4 * j + 1] << 8) | (code[4 * j + 2] << 16) | (code[4 * j + 3] << 24);
            if constexpr (EPT == 16) st128(elements + c * EPT, make_uint4(w[0], w[1], w[2], w[3]));
            else st64(elements + c * EPT, make_uint2(w[0], w[1]));
            if ((c & (lpb - 1)) == 0) scales[c >> lpb_shift] = (uint8_t)scale;
        }
    }
}

template <class F>
__device__ inline float mxfp_value(uint32_t code, float scale, const F& f) {
    return decode_f32(code, f) * scale;
}

// ------------------------------------------------------------------------------ bf16 fast path
// bfloat16 input, block size 32, compile-time format.  A lane owns 8 consecutive elements (one
// 128-bit load), four adjacent lanes own a block.  Two elements are processed per 32-bit
// register with packed 16-bit integer instructions; there is no per-element branch.
//
// With h the bf16 bits, a = h & 0x7FFF and scale the block's biased shared exponent, the value
//     t = a - ((scale - bias) << 7)        (signed, clamped at 0)
// is  (ye << 7) | f7 : the element's exponent field in the target format above its 7 mantissa
// bits.  Rounding to M bits, the reference's "(ye << M) | yf" with its lost carry, the one
// reachable subnormal binade (ye == 0) and underflow (t < 0) are all functions of t alone.
// Not covered, and sent to the exact per-element routine by a wave-uniform test: blocks holding
// inf/NaN, and scales >= 151 (only there can a quotient underflow to exactly zero).
typedef unsigned short u16x2 __attribute__((ext_vector_type(2)));
typedef short i16x2 __attribute__((ext_vector_type(2)));

__device__ inline uint32_t as_u32(u16x2 v) { return __builtin_bit_cast(uint32_t, v); }
__device__ inline uint32_t as_u32(i16x2 v) { return __builtin_bit_cast(uint32_t, v); }
__device__ inline u16x2 as_u16x2(uint32_t v) { return __builtin_bit_cast(u16x2, v); }
__device__ inline i16x2 as_i16x2(uint32_t v) { return __builtin_bit_cast(i16x2, v); }

template <class F>
struct PackedBf16 {
    static constexpr int E = F{}.E(), M = F{}.M(), SH = 7 - M;
    static constexpr uint32_t LSB = 0x00010001u;
    // code magnitudes (exponent and mantissa fields, no sign) of two elements, one per 16-bit half,
    // plus, through `t_q`, the quantised magnitude back in the t domain for the fused QDQ
    // Packed 16-bit operations written as asm: given the plain expressions the compiler replaces each of them by one
    // compare and one conditional move per 16-bit half plus a byte permute to put the halves together again.
    __device__ static inline uint32_t pk_min_u16(uint32_t a, uint32_t b) {
        uint32_t d;
        asm("v_pk_min_u16 %0, %1, %2" : "=v"(d) : "v"(a), "v"(b));
        return d;
    }
    // all ones in the halves where a < b (as signed 16-bit numbers whose difference fits 16 bits)
    __device__ static inline uint32_t pk_less_mask(uint32_t a, uint32_t b) {
        uint32_t d;
        asm("v_pk_sub_i16 %0, %1, %2\n\tv_pk_ashrrev_i16 %0, 15, %0 op_sel_hi:[0,1]" : "=&v"(d) : "v"(a), "v"(b));
        return d;
    }
    __device__ static inline uint32_t magnitude(uint32_t a, uint32_t ssb2, uint32_t& t_q) {
        // t = a - ssb2 clamped at 0 (underflow -> 0); the caller guarantees ssb2 >= 0 in both halves
        const uint32_t tu = as_u32(__builtin_elementwise_sub_sat(as_u16x2(a), as_u16x2(ssb2)));
        const uint32_t u = as_u32(as_u16x2(tu) >> (unsigned short)SH);    // (ye << M) | truncated mantissa
        const uint32_t r = tu + (((1u << (SH - 1)) - 1u) * LSB) + (u & LSB);  // round half to even
        const uint32_t v = as_u32(as_u16x2(r) >> (unsigned short)SH);     // (ye << M) + rounded mantissa
        // the reference ORs the exponent field with the rounded mantissa, so a carry out of the mantissa into an odd
        // exponent field is lost
        const uint32_t ef = u & (0xFFFFu & ~((1u << M) - 1u)) * LSB;
        const uint32_t code_n = ef | (v - ef);
        // ye == 0: the mantissa (with its carry) is shifted down under an explicit leading one; zero stays zero
        const uint32_t m01 = pk_min_u16(v, LSB);
        const uint32_t code_s = as_u32(as_u16x2((m01 << M) | v) >> (unsigned short)1);
        // all ones where ye >= 1, i.e. u >= 2^M
        const uint32_t is_norm = pk_less_mask(((1u << M) - 1u) * LSB, u);
        // t-domain value of the code: normal codes keep their fields; subnormal code xf' (>= 2^(M-1))
        // is 2^-bias * xf' / 2^(M-1), i.e. exponent field 0 and mantissa (xf' << (8 - M)) & 0x7F
        const uint32_t tq_n = code_n << SH;
        const uint32_t tq_s = (code_s << (8 - M)) & (0x7Fu * LSB);
        t_q = (is_norm & tq_n) | (~is_norm & tq_s);
        return (is_norm & code_n) | (~is_norm & code_s);
    }
    // all ones in the halves whose input has a non-zero exponent field (everything else is flushed
    // to +0.0 by the reference before encoding and gets code 0, sign included)
    __device__ static inline uint32_t live_mask(uint32_t a) { return as_u32(as_i16x2(a + 0x7F807F80u) >> (short)15); }
    __device__ static inline uint32_t codes(uint32_t h, uint32_t ssb2) {
        const uint32_t a = h & 0x7FFF7FFFu;
        uint32_t t_q;
        const uint32_t mag = magnitude(a, ssb2, t_q);
        const uint32_t sgn = (h >> (15 - (E + M))) & ((1u << (E + M)) * LSB);
        return (mag | sgn) & live_mask(a);
    }
    // quantise-dequantise of two bf16 values; valid when every non-zero code lands in the bf16
    // normal range, i.e. scale > bias (smaller scales give subnormal results: slow path)
    __device__ static inline uint32_t qdq(uint32_t h, uint32_t ssb2) {
        const uint32_t a = h & 0x7FFF7FFFu;
        uint32_t t_q;
        const uint32_t mag = magnitude(a, ssb2, t_q);
        const uint32_t nonzero = pk_less_mask(0u, mag);                    // code magnitudes are small positive numbers
        const uint32_t body = (t_q + ssb2) & nonzero;                      // code 0 -> +-0.0
        return (body | (h & 0x80008000u)) & live_mask(a);
    }
};

// ------------------------------------------------------------------------------ operands of the block-scaled GEMM
// The block-scaled matrix instruction takes FP8 (E4M3) bytes and one E8M0 scale per 32 of them.  It reads the code
// S.1111.111 as NaN where the reference's finite E4M3 has +-480, so a block that holds that code is stored one scale
// step up with every code halved: exact for codes of 16 and more (exponent field - 1) and for even codes below 16
// (whose value is code * 2^-9 in units of the block scale); an odd code below 16 rounds half to even.  The narrower
// element formats are embedded into E4M3 bytes with the same value and the same block scale (their subnormals are
// E4M3 normals).  Scales go out transposed for the GEMM's DMA: dword [k / 128][row], byte (k / 32) % 4.
__device__ inline uint32_t e4m3_top_bits(uint32_t w) { return ((w & 0x7F7F7F7Fu) + 0x01010101u) & 0x80808080u; }
__device__ inline uint32_t e4m3_halve4(uint32_t w) {
    const uint32_t mag = w & 0x7F7F7F7Fu, sign = w & 0x80808080u;
    const uint32_t big = (((mag + 0x70707070u) & 0x80808080u) >> 7) * 0xFFu;      // all ones in the bytes with mag >= 16
    const uint32_t mag_n = ((mag | 0x80808080u) - 0x08080808u) & 0x7F7F7F7Fu;     // exponent field - 1 (the guard bit stops the borrow)
    const uint32_t q = (mag >> 1) & 0x7F7F7F7Fu;
    const uint32_t mag_s = q + (mag & q & 0x01010101u);                           // mag / 2, half to even
    return sign | (big & mag_n) | (~big & mag_s);
}
// one code of format F as the E4M3 byte of the same value
template <class F>
__device__ inline uint32_t embed_e4m3(uint32_t c, const F& f) {
    constexpr int E = F{}.E(), M = F{}.M(), bias = (1 << (E - 1)) - 1;
    if constexpr (E == 4 && M == 3) return c & 0xFFu;
    const uint32_t s = (c >> (E + M)) & 1u, e = (c >> M) & ((1u << E) - 1u), fr = c & ((1u << M) - 1u);
    uint32_t mag = 0;
    if (e != 0) mag = ((e + 7 - bias) << 3) | (fr << (3 - M));
    else if (fr != 0) {
        const int p = 31 - __clz(fr);   // value 2^(p - M + 1 - bias) * (1 + rest / 2^p)
        mag = ((uint32_t)(p - M + 8 - bias) << 3) | ((fr << (3 - p)) & 7u);
    }
    return (s << 7) | mag;
}
template <class F>
__device__ inline uint32_t embed_e4m3_x4(uint32_t w, const F& f) {
    return embed_e4m3(w & 0xFFu, f) | (embed_e4m3((w >> 8) & 0xFFu, f) << 8) | (embed_e4m3((w >> 16) & 0xFFu, f) << 16) |
           (embed_e4m3(w >> 24, f) << 24);
}
// ---- code tables of the bf16 kernels
// With t as above ((ye << 7) | f7: the element's exponent field in the target format above the 7 mantissa bits of its
// bf16 magnitude), the code magnitude is a function of t alone: 2^(E + 7) entries, built at compile time by the same steps
// as PackedBf16::magnitude (round half to even on the M-bit mantissa, the reference's OR that loses a carry into an odd
// exponent field, the one reachable subnormal binade).  A workgroup copies its format's table into LDS and looks every
// element up there: half the vector instructions of the arithmetic.
template <int E, int M>
struct CodeLut {
    static constexpr int N = 1 << (E + 7);
    uint8_t code[N];
    constexpr CodeLut() : code{} {
        constexpr int SH = 7 - M;
        for (int t = 0; t < N; ++t) {
            const int ye = t >> 7, f7 = t & 127;
            const int q = f7 >> SH, r = f7 & ((1 << SH) - 1), half = 1 << (SH - 1);
            const int yf = q + ((r > half || (r == half && (q & 1))) ? 1 : 0);   // in [0, 2^M]
            const int c = ye != 0 ? ((ye << M) | yf) : (yf != 0 ? ((yf | (1 << M)) >> 1) : 0);
            code[t] = (uint8_t)c;
        }
    }
};
template <int E, int M>
__device__ const CodeLut<E, M> kCodeLut{};

// LDS copy of the table (the code-producing modes; the fused quantise-dequantise pass does not use one: BYTES = 16 there);
// all threads of the workgroup call it, before the first bf16_block_step.
template <class F, bool QDQ>
struct LdsLut {
    static constexpr int E = F{}.E(), M = F{}.M();
    static constexpr int BYTES = QDQ ? 16 : (1 << (E + 7));
    __device__ static inline void fill(uint8_t* lds) {
        if (QDQ) return;
        for (int i = threadIdx.x * 16; i < BYTES; i += kThreads * 16)
            *reinterpret_cast<uint4*>(lds + i) = *reinterpret_cast<const uint4*>(kCodeLut<E, M>.code + i);
        __syncthreads();
    }
};

// two table entries, for the t values in the halves of `t2` (issued here, valid after the caller's s_waitcnt; plain loads into
// two registers: a load into half a register does not keep the other half on this hardware)
template <bool UNUSED>
__device__ inline void lut_pair(uint32_t& lo, uint32_t& hi, uint32_t lds_base, uint32_t t2) {
    const uint32_t a_lo = lds_base + (t2 & 0xFFFFu), a_hi = lds_base + (t2 >> 16);
    asm volatile("ds_read_u8 %0, %2\n\tds_read_u8 %1, %3" : "=&v"(lo), "=&v"(hi) : "v"(a_lo), "v"(a_hi));
}

// The arithmetic of one 128-bit step of the bf16 kernels below: 8 elements of a lane whose three quad neighbours hold the
// rest of the block.  QDQ false: o[j] = two codes in the low bytes of the halves; true: two quantised bf16 values.
// `lut`: LDS address of the table (LdsLut<F, QDQ>).  Every lane of a quad must call it (DPP).
template <class F, bool QDQ>
__device__ inline void bf16_block_step(const uint4& raw, const F& f, uint32_t (&o)[4], uint32_t& scale, uint32_t lut) {
    constexpr int E = F{}.E(), M = F{}.M();
    const uint32_t h[4] = {raw.x, raw.y, raw.z, raw.w};
    // block maximum of |x| bits: packed max over the lane's four registers, then the two halves,
    // then the four lanes of the block (DPP quad permutes)
    u16x2 m2 = __builtin_elementwise_max(__builtin_elementwise_max(as_u16x2(h[0] & 0x7FFF7FFFu), as_u16x2(h[1] & 0x7FFF7FFFu)),
                                         __builtin_elementwise_max(as_u16x2(h[2] & 0x7FFF7FFFu), as_u16x2(h[3] & 0x7FFF7FFFu)));
    uint32_t amax = max((uint32_t)m2[0], (uint32_t)m2[1]);
    amax = max(amax, (uint32_t)__builtin_amdgcn_mov_dpp((int)amax, 0xB1, 0xF, 0xF, true));  // lane ^ 1
    amax = max(amax, (uint32_t)__builtin_amdgcn_mov_dpp((int)amax, 0x4E, 0xF, 0xF, true));  // lane ^ 2
    const int ef_max = (int)(amax >> 7);
    const int scale_n = max(ef_max - fmt_emax_unb(f), 0);  // amax == 0 gives 0: the all-flushed rule
    // (scale_n < bias: the packed arithmetic subtracts (scale_n - bias) << 7 with unsigned saturation)
    const bool hard = amax >= 0x7F80u || scale_n >= 151 || (amax != 0u && scale_n < fmt_bias(f) + (QDQ ? 1 : 0));
    scale = (uint32_t)scale_n;
    if (__builtin_amdgcn_ballot_w64(hard) == 0) {
        const uint32_t ssb = (uint32_t)((scale_n - fmt_bias(f)) << 7) & 0xFFFFu;
        const uint32_t ssb2 = ssb | (ssb << 16);
        if constexpr (QDQ) {
            // (the fused pass stays on the packed arithmetic: a lane has as many stores as loads to hide it under, and a
            // workgroup would copy a table half the size of its input; measured slower with the table)
#pragma unroll
            for (int j = 0; j < 4; ++j) o[j] = PackedBf16<F>::qdq(h[j], ssb2);
            return;
        }
        uint32_t hl[4], lo[4], hi[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            // inputs with a zero exponent field are flushed to +0.0 before encoding (code 0, sign included): clear them here
            hl[j] = h[j] & PackedBf16<F>::live_mask(h[j] & 0x7FFF7FFFu);
            const uint32_t t2 = as_u32(__builtin_elementwise_sub_sat(as_u16x2(hl[j] & 0x7FFF7FFFu), as_u16x2(ssb2)));
            lut_pair<false>(lo[j], hi[j], lut, t2);
        }
        asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(lo[0]), "+v"(lo[1]), "+v"(lo[2]), "+v"(lo[3]), "+v"(hi[0]), "+v"(hi[1]), "+v"(hi[2]), "+v"(hi[3]));
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            o[j] = lo[j] | (hi[j] << 16) | ((hl[j] >> (15 - (E + M))) & ((1u << (E + M)) * 0x00010001u));
        }
    } else {
        // exact per-element routine (the block's lanes agree on amax, so they agree on the result)
        const uint32_t amax32 = amax << 16;
        const int se = shared_exponent<F, true>(amax32, f);
        scale = amax32 < 0x00800000u ? 0u : (uint32_t)(se + 127);
        const float sc = scale_f32(scale);
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const uint32_t c0 = encode_mxfp_element(h[j] << 16, se, f), c1 = encode_mxfp_element(h[j] & 0xFFFF0000u, se, f);
            o[j] = QDQ ? pack_bf16(mxfp_value(c0, sc, f), mxfp_value(c1, sc, f)) : (c0 | (c1 << 16));
        }
    }
}

// MODE 0: extract (scales + elements); MODE 1: fused quantise-dequantise to bf16
template <class F, int UNROLL, int MODE>
__global__ __launch_bounds__(kThreads) void mxfp_bf16_b32_kernel(const uint4* __restrict__ x, uint8_t* __restrict__ scales,
                                                                  uint2* __restrict__ elements, uint4* __restrict__ out,
                                                                  int64_t n_chunks, F f) {
    __shared__ __attribute__((aligned(16))) uint8_t lut[LdsLut<F, MODE == 1>::BYTES];
    const int64_t chunk0 = (int64_t)blockIdx.x * (UNROLL * kThreads) + threadIdx.x;
    uint4 raw[UNROLL];
#pragma unroll
    for (int r = 0; r < UNROLL; ++r) {
        const int64_t c = chunk0 + (int64_t)r * kThreads;
        raw[r] = c < n_chunks ? ld128(x + c) : make_uint4(0, 0, 0, 0);
    }
    LdsLut<F, MODE == 1>::fill(lut);
    const uint32_t lut_addr = (uint32_t)(uintptr_t)lut;
#pragma unroll
    for (int r = 0; r < UNROLL; ++r) {
        const int64_t c = chunk0 + (int64_t)r * kThreads;
        uint32_t o[4], scale;
        bf16_block_step<F, MODE == 1>(raw[r], f, o, scale, lut_addr);
        if (c < n_chunks) {
            if (MODE == 0) {
                // o[j] holds two codes in the low bytes of its halves: gather the 8 code bytes
                st64(elements + c, make_uint2(__builtin_amdgcn_perm(o[1], o[0], 0x06040200u), __builtin_amdgcn_perm(o[3], o[2], 0x06040200u)));
                if ((c & 3) == 0) scales[c >> 2] = (uint8_t)scale;
            } else {
                st128(out + c, make_uint4(o[0], o[1], o[2], o[3]));
            }
        }
    }
}

// bf16 matrix x [rows, K] (row stride ld elements) -> operand of the block-scaled GEMM in one pass (extract, then the
// re-encoding / embedding above).  A workgroup owns 32 rows x 128 k, the unit whose scale dwords fill one 128-byte line of
// the transposed scale array: 16 lanes read the 256 bytes of one row (8 elements each, four lanes to a block), a
// wavefront four rows per step, two steps.  The four scale bytes of a row are gathered into one lane and stored as a dword.
// MODE 1 (SwiGLU): the matrix that is quantised is silu(x) * up (up [rows, K] with the same row stride), formed in registers.
// MODE 2 (minifloat): every element is rounded by itself to the minifloat format F (what extract_minifloat_kernel computes)
// and every block carries the scale 2^0: a minifloat code is the MXFP element of a block with that scale.
enum { FROM_DENSE = 0, FROM_SWIGLU = 1, FROM_DENSE_MINIFLOAT = 2 };
template <class F, int MODE>
__global__ __launch_bounds__(kThreads) void scaled_from_dense_kernel(const uint16_t* __restrict__ x, const uint16_t* __restrict__ up, size_t ld,
                                                                      uint8_t* __restrict__ codes, uint32_t* __restrict__ scales, int rows,
                                                                      int K, int nmac, uint32_t rows_pad, F f) {
    constexpr bool SWIGLU = MODE == FROM_SWIGLU, MINIFLOAT = MODE == FROM_DENSE_MINIFLOAT;
    __shared__ __attribute__((aligned(16))) uint8_t lut[LdsLut<F, false>::BYTES + 16];   // (one more entry in the minifloat mode)
    const uint32_t ms = blockIdx.x % (uint32_t)nmac, row_base = (blockIdx.x / (uint32_t)nmac) * 32u;
    const int t = threadIdx.x;
    uint4 raw[2], raw_up[2];
    size_t off[2];
    bool live[2];
#pragma unroll
    for (int r = 0; r < 2; ++r) {
        const uint32_t row = row_base + 16u * r + (uint32_t)(t >> 4);
        const uint32_t col = ms * 128u + (uint32_t)(t & 15) * 8u;
        live[r] = row < (uint32_t)rows;
        off[r] = (size_t)row * K + col;
        raw[r] = live[r] ? ld128(x + (size_t)row * ld + col) : make_uint4(0, 0, 0, 0);
        if (SWIGLU) raw_up[r] = live[r] ? ld128(up + (size_t)row * ld + col) : make_uint4(0, 0, 0, 0);
    }
    // minifloat mode: the same table serves (with the scale fixed at 2^0 the rounding of the reference's minifloat extract
    // is the MXFP element's, step for step); values past the top binade, which a block's own scale rules out, saturate
    // through one more entry
    constexpr int LUT_N = LdsLut<F, false>::BYTES;
    if (MINIFLOAT && t == 0) lut[LUT_N] = (uint8_t)((1u << (F{}.E() + F{}.M())) - 1u);
    LdsLut<F, false>::fill(lut);
    const uint32_t lut_addr = (uint32_t)(uintptr_t)lut;
#pragma unroll
    for (int r = 0; r < 2; ++r) {
        if (SWIGLU) raw[r] = swiglu_x8(raw[r], raw_up[r]);
        uint32_t o[4], scale;
        if constexpr (MINIFLOAT) {
            const uint32_t h[4] = {raw[r].x, raw[r].y, raw[r].z, raw[r].w};
            constexpr int E = F{}.E(), M = F{}.M();
            // inf / NaN anywhere in the wavefront's elements: the per-element routine for all of them
            const u16x2 m2 = __builtin_elementwise_max(__builtin_elementwise_max(as_u16x2(h[0] & 0x7FFF7FFFu), as_u16x2(h[1] & 0x7FFF7FFFu)),
                                                       __builtin_elementwise_max(as_u16x2(h[2] & 0x7FFF7FFFu), as_u16x2(h[3] & 0x7FFF7FFFu)));
            if (__builtin_amdgcn_ballot_w64(max((uint32_t)m2[0], (uint32_t)m2[1]) >= 0x7F80u) == 0) {
                constexpr uint32_t OFF = (uint32_t)(127 - ((1 << (E - 1)) - 1)) << 7;   // t = |x| bits - OFF, saturating: below the format's range gives entry 0
                uint32_t lo[4], hi[4];
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    const u16x2 d = __builtin_elementwise_sub_sat(as_u16x2(h[j] & 0x7FFF7FFFu), as_u16x2(OFF * 0x00010001u));
                    lut_pair<false>(lo[j], hi[j], lut_addr, as_u32(__builtin_elementwise_min(d, as_u16x2((uint32_t)LUT_N * 0x00010001u))));
                }
                asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(lo[0]), "+v"(lo[1]), "+v"(lo[2]), "+v"(lo[3]), "+v"(hi[0]), "+v"(hi[1]), "+v"(hi[2]), "+v"(hi[3]));
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    // the sign code goes with every negative input but -0.0, flushed ones included
                    const uint32_t sign = h[j] & ((h[j] & 0x7FFF7FFFu) + 0x7FFF7FFFu) & 0x80008000u;
                    o[j] = lo[j] | (hi[j] << 16) | (sign >> (15 - (E + M)));
                }
            } else {
#pragma unroll
                for (int j = 0; j < 4; ++j) o[j] = encode_f32_bits(h[j] << 16, f) | (encode_f32_bits(h[j] & 0xFFFF0000u, f) << 16);
            }
            scale = 127u;
        } else {
            bf16_block_step<F, false>(raw[r], f, o, scale, lut_addr);
        }
        uint32_t w0 = __builtin_amdgcn_perm(o[1], o[0], 0x06040200u), w1 = __builtin_amdgcn_perm(o[3], o[2], 0x06040200u);
        if constexpr (F{}.E() == 4 && F{}.M() == 3) {
            uint32_t top = e4m3_top_bits(w0) | e4m3_top_bits(w1);
            top |= (uint32_t)__builtin_amdgcn_mov_dpp((int)top, 0xB1, 0xF, 0xF, true);
            top |= (uint32_t)__builtin_amdgcn_mov_dpp((int)top, 0x4E, 0xF, 0xF, true);
            if (top != 0u && scale < 254u) {   // (a block of scale 255 holds inf / NaN: its row of the product is NaN either way)
                w0 = e4m3_halve4(w0);
                w1 = e4m3_halve4(w1);
                scale += 1u;
            }
        } else {
            w0 = embed_e4m3_x4(w0, f);
            w1 = embed_e4m3_x4(w1, f);
        }
        // the row's four scale bytes (lanes 0, 4, 8, 12 of its 16) into its first lane: row_shl 4, 8, 12
        uint32_t dw = scale;
        dw |= (uint32_t)__builtin_amdgcn_update_dpp(0, (int)scale, 0x104, 0xF, 0xF, true) << 8;
        dw |= (uint32_t)__builtin_amdgcn_update_dpp(0, (int)scale, 0x108, 0xF, 0xF, true) << 16;
        dw |= (uint32_t)__builtin_amdgcn_update_dpp(0, (int)scale, 0x10C, 0xF, 0xF, true) << 24;
        if (live[r]) {
            st64(codes + off[r], make_uint2(w0, w1));
            if ((t & 15) == 0) scales[(size_t)ms * rows_pad + row_base + 16u * r + (uint32_t)(t >> 4)] = dw;
        }
    }
}

// Fallback for any block size / alignment: one lane owns one block.
template <int DT_IN, class F>
__global__ __launch_bounds__(kThreads) void extract_mxfp_block_kernel(const void* __restrict__ x, uint8_t* __restrict__ scales,
                                                                       uint8_t* __restrict__ elements, int64_t n_blocks, int B,
                                                                       F f) {
    const int64_t b = (int64_t)blockIdx.x * kThreads + threadIdx.x;
    if (b >= n_blocks) return;
    uint32_t amax = 0;
    for (int j = 0; j < B; ++j) {
        const uint32_t a = load_bits_scalar<DT_IN>(x, b * B + j) & 0x7FFFFFFFu;
        amax = a > amax ? a : amax;
    }
    const int se = shared_exponent<F, DT_IN != F32>(amax, f);
    scales[b] = amax < 0x00800000u ? (uint8_t)0 : (uint8_t)(se + 127);
    for (int j = 0; j < B; ++j) elements[b * B + j] = (uint8_t)encode_mxfp_element(load_bits_scalar<DT_IN>(x, b * B + j), se, f);
}

// block index of chunk c with `per_block` chunks to a block: a shift when per_block is a power of two (a 64-bit
// division costs more instructions than the rest of a lane's work); the test is uniform over the launch
__device__ inline int64_t block_of_chunk(int64_t c, int per_block) {
    if ((per_block & (per_block - 1)) == 0) return c >> (31 - __builtin_clz((unsigned)per_block));
    return c / per_block;
}

// Vector path: B % EPT == 0 (a lane's run lies inside one block).
template <int DT_OUT, class F, int EPT, int UNROLL>
__global__ __launch_bounds__(kThreads) void compose_mxfp_kernel(const uint8_t* __restrict__ scales,
                                                                 const uint8_t* __restrict__ elements, void* __restrict__ out,
                                                                 int64_t n, int chunks_per_block, F f) {
    const int64_t n_chunks = n / EPT;
    const int64_t chunk0 = (int64_t)blockIdx.x * (UNROLL * kThreads) + threadIdx.x;
    uint32_t w[UNROLL][EPT / 4];
    uint32_t sc[UNROLL];
#pragma unroll
    for (int r = 0; r < UNROLL; ++r) {
        const int64_t c = chunk0 + (int64_t)r * kThreads;
        if (c < n_chunks) {
            if constexpr (EPT == 16) {
                const uint4 v = ld128(elements + c * EPT);
                w[r][0] = v.x; w[r][1] = v.y; w[r][2] = v.z; w[r][3] = v.w;
            } else {
                const uint2 v = ld64(elements + c * EPT);
                w[r][0] = v.x; w[r][1] = v.y;
            }
            sc[r] = scales[block_of_chunk(c, chunks_per_block)];
        }
    }
#pragma unroll
    for (int r = 0; r < UNROLL; ++r) {
        const int64_t c = chunk0 + (int64_t)r * kThreads;
        if (c < n_chunks) {
            const float s = scale_f32(sc[r]);
            float y[EPT];
#pragma unroll
            for (int j = 0; j < EPT; ++j) y[j] = mxfp_value((w[r][j / 4] >> (8 * (j % 4))) & 0xFFu, s, f);
            store_vals<DT_OUT, EPT>(out, c * EPT, y);
        }
    }
}

// does the format have a compile-time Composer that takes the hardware convert route?
template <class F, bool STATIC = F::kStatic> struct HwCompose { static constexpr bool value = false; };
template <class F> struct HwCompose<F, true> { static constexpr bool value = Composer<F>::HW; };

// bf16 output, a preset format with at most four exponent bits: the hardware's scaled fp8 -> bf16 convert does a pair of
// codes per instruction (Composer, mxfp_compose.h).  A lane owns 8 codes (one 64-bit load) of one block; lanes whose scale
// the convert does not take (from Composer::SLOW_FROM up: 255, "times +inf", among them) redo theirs with the exact
// per-element routine, behind a wave-uniform test.
template <class F, int UNROLL>
__global__ __launch_bounds__(kThreads) void compose_mxfp_bf16_kernel(const uint8_t* __restrict__ scales,
                                                                      const uint8_t* __restrict__ elements, void* __restrict__ out,
                                                                      int64_t n, int chunks_per_block, F f) {
    typedef Composer<F> C;
    constexpr uint32_t KEEP4 = ((1u << (1 + C::E + C::M)) - 1u) * 0x01010101u;   // the reference ignores the bits above the code
    const int64_t n_chunks = n / 8;
    const int64_t chunk0 = (int64_t)blockIdx.x * (UNROLL * kThreads) + threadIdx.x;
    uint2 w[UNROLL];
    uint32_t sc[UNROLL];
#pragma unroll
    for (int r = 0; r < UNROLL; ++r) {
        const int64_t c = chunk0 + (int64_t)r * kThreads;
        w[r] = make_uint2(0u, 0u);
        sc[r] = 127u;
        if (c < n_chunks) {
            w[r] = ld64(elements + c * 8);
            sc[r] = scales[block_of_chunk(c, chunks_per_block)];
        }
    }
#pragma unroll
    for (int r = 0; r < UNROLL; ++r) {
        const int64_t c = chunk0 + (int64_t)r * kThreads;
        const uint32_t w0 = w[r].x & KEEP4, w1 = w[r].y & KEEP4;
        const C cmp(sc[r]);
        uint32_t o[4];
        cmp.pair2(w0, o[0], o[1]);
        cmp.pair2(w1, o[2], o[3]);
        if (__builtin_amdgcn_ballot_w64(C::is_slow(sc[r])) != 0 && C::is_slow(sc[r])) {
            const float s = scale_f32(sc[r]);
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const uint32_t ww = j < 2 ? w0 : w1;
                const int b0 = 16 * (j & 1);
                o[j] = pack_bf16(mxfp_value((ww >> b0) & 0xFFu, s, f), mxfp_value((ww >> (b0 + 8)) & 0xFFu, s, f));
            }
        }
        if (c < n_chunks) st128(static_cast<uint8_t*>(out) + c * 16, make_uint4(o[0], o[1], o[2], o[3]));
    }
}

template <int DT_OUT, class F>
__global__ __launch_bounds__(kThreads) void compose_mxfp_scalar_kernel(const uint8_t* __restrict__ scales,
                                                                        const uint8_t* __restrict__ elements,
                                                                        void* __restrict__ out, int64_t n, int B, F f) {
    const int64_t i = (int64_t)blockIdx.x * kThreads + threadIdx.x;
    if (i >= n) return;
    store_val_scalar<DT_OUT>(out, i, mxfp_value(elements[i], scale_f32(scales[i / B]), f));
}

template <int DT_IN, int DT_OUT, class F, int EPT, int UNROLL>
__global__ __launch_bounds__(kThreads) void qdq_mxfp_kernel(const void* x, void* out, int64_t n, int lpb, F f) {
    const int64_t n_chunks = n / EPT;
    const int64_t chunk0 = (int64_t)blockIdx.x * (UNROLL * kThreads) + threadIdx.x;
    uint32_t u[UNROLL][EPT];
#pragma unroll
    for (int r = 0; r < UNROLL; ++r) {
        const int64_t c = chunk0 + (int64_t)r * kThreads;
        if (c < n_chunks) load_bits<DT_IN, EPT>(x, c * EPT, u[r]);
        else {
#pragma unroll
            for (int j = 0; j < EPT; ++j) u[r][j] = 0u;
        }
    }
#pragma unroll
    for (int r = 0; r < UNROLL; ++r) {
        const int64_t c = chunk0 + (int64_t)r * kThreads;
        uint32_t code[EPT], scale;
        mxfp_encode_run<DT_IN, F, EPT>(u[r], lpb, f, code, scale);
        if (c < n_chunks) {
            const float s = scale_f32(scale);
            float y[EPT];
#pragma unroll
            for (int j = 0; j < EPT; ++j) y[j] = mxfp_value(code[j], s, f);
            store_vals<DT_OUT, EPT>(out, c * EPT, y);
        }
    }
}

template <int DT_IN, int DT_OUT, class F>
__global__ __launch_bounds__(kThreads) void qdq_mxfp_block_kernel(const void* x, void* out, int64_t n_blocks, int B, F f) {
    const int64_t b = (int64_t)blockIdx.x * kThreads + threadIdx.x;
    if (b >= n_blocks) return;
    uint32_t amax = 0;
    for (int j = 0; j < B; ++j) {
        const uint32_t a = load_bits_scalar<DT_IN>(x, b * B + j) & 0x7FFFFFFFu;
        amax = a > amax ? a : amax;
    }
    const int se = shared_exponent<F, DT_IN != F32>(amax, f);
    const float s = scale_f32(amax < 0x00800000u ? 0u : (uint32_t)(se + 127));
    // a lane reads and writes only its own block, element by element, so in-place use is safe
    for (int j = 0; j < B; ++j) {
        const uint32_t code = encode_mxfp_element(load_bits_scalar<DT_IN>(x, b * B + j), se, f);
        store_val_scalar<DT_OUT>(out, b * B + j, mxfp_value(code, s, f));
    }
}

// ------------------------------------------------------------------------------ blocks along a non-last axis
// The tensor is [outer, K, inner] row-major and blocks of 32 run along K (element stride
// `inner`), K % 32 == 0: what the reference reaches by permuting the block axis last and
// copying (src/mase_triton/mxfp/helpers.py:4-24) before its flat kernel.  Here a lane owns
// adjacent positions of the inner axis and walks down K one block at a time; a block sits in
// one lane's registers, so its maximum needs no cross-lane traffic, and adjacent lanes read
// adjacent addresses of a row.  Outputs keep the reference's order: scales [outer, inner, K/32]
// and elements [outer, inner, K] (extract), or the input's own layout (quantise-dequantise).
// Work item (one per lane) -> (outer, group of kb_per k-blocks, chunk of the inner axis), chunk
// fastest, so a short inner axis still fills a wavefront with several k-groups.
struct StridedGeom {
    int64_t K, inner, nkb;  // nkb = K / 32
    int64_t chunks, kgroups, items;
    int kb_per;
};

__device__ inline bool strided_origin(const StridedGeom& g, int vec, int64_t& o, int64_t& kb0, int64_t& i0) {
    const int64_t item = (int64_t)blockIdx.x * kThreads + threadIdx.x;
    const int64_t rest = item / g.chunks;
    i0 = (item - rest * g.chunks) * vec;
    o = rest / g.kgroups;
    kb0 = (rest - o * g.kgroups) * g.kb_per;
    return item < g.items;
}

// 32 codes (one per entry, low byte) -> 32 consecutive bytes at dst
__device__ inline void store_block_codes(uint8_t* dst, const uint32_t (&code)[32], bool aligned16) {
    if (aligned16) {
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            uint32_t w[4];
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const int b = 16 * h + 4 * j;
                w[j] = code[b] | (code[b + 1] << 8) | (code[b + 2] << 16) | (code[b + 3] << 24);
            }
            st128<false>(dst + 16 * h, make_uint4(w[0], w[1], w[2], w[3]));
        }
    } else {
#pragma unroll
        for (int j = 0; j < 32; ++j) dst[j] = (uint8_t)code[j];
    }
}

// Any dtype, any format: one position of the inner axis per lane.  MODE 0 extract, 1 QDQ.
template <int DT_IN, int DT_OUT, class F, int MODE>
__global__ __launch_bounds__(kThreads) void mxfp_strided_kernel(const void* x, uint8_t* __restrict__ scales,
                                                                 uint8_t* __restrict__ elements, void* out, StridedGeom g,
                                                                 bool elements_aligned16, F f) {
    int64_t o, kb0, i;
    if (!strided_origin(g, 1, o, kb0, i)) return;
    for (int q = 0; q < g.kb_per; ++q) {
        const int64_t kb = kb0 + q;
        if (kb >= g.nkb) break;
        const int64_t first = (o * g.K + kb * 32) * g.inner + i;
        uint32_t u[32], amax = 0;
#pragma unroll
        for (int j = 0; j < 32; ++j) {
            u[j] = load_bits_scalar<DT_IN>(x, first + j * g.inner);
            const uint32_t a = u[j] & 0x7FFFFFFFu;
            amax = a > amax ? a : amax;
        }
        const int se = shared_exponent<F, DT_IN != F32>(amax, f);
        const uint32_t scale = amax < 0x00800000u ? 0u : (uint32_t)(se + 127);
        uint32_t code[32];
#pragma unroll
        for (int j = 0; j < 32; ++j) code[j] = encode_mxfp_element(u[j], se, f);
        if (MODE == 0) {
            const int64_t col = o * g.inner + i;
            store_block_codes(elements + col * g.K + kb * 32, code, elements_aligned16);
            scales[col * g.nkb + kb] = (uint8_t)scale;
        } else {
            // the lane has read its whole block before it writes: in-place use is safe
            const float sc = scale_f32(scale);
#pragma unroll
            for (int j = 0; j < 32; ++j) store_val_scalar<DT_OUT>(out, first + j * g.inner, mxfp_value(code[j], sc, f));
        }
    }
}

// bfloat16 in (and out), compile-time format: two positions of the inner axis per lane (one
// 32-bit load per row), packed 16-bit arithmetic as in mxfp_bf16_b32_kernel with one scale per
// 16-bit half.  Needs inner % 2 == 0 and 4-byte aligned x / out.
// One block of 32 rows for the lane's two columns, read at x + first (+ j * inner).  res[j]: MODE 0 the two codes
// of row j (low byte of each 16-bit half), MODE 1 the two bf16 results; scale[t]: the scale byte of column t.
template <class F, int MODE>
__device__ inline void strided_bf16_block(const uint16_t* x, int64_t first, int64_t inner, const F& f, uint32_t (&res)[32],
                                          uint32_t (&scale)[2]) {
    uint32_t h[32];
    u16x2 m = {0, 0};
#pragma unroll
    for (int j = 0; j < 32; ++j) {
        h[j] = *reinterpret_cast<const uint32_t*>(x + first + j * inner);
        m = __builtin_elementwise_max(m, as_u16x2(h[j] & 0x7FFF7FFFu));
    }
    uint32_t amax[2];
    bool hard = false;
#pragma unroll
    for (int c = 0; c < 2; ++c) {
        amax[c] = m[c];
        const int scale_n = max((int)(amax[c] >> 7) - fmt_emax_unb(f), 0);  // amax == 0 gives 0: the all-flushed rule
        hard |= amax[c] >= 0x7F80u || scale_n >= 151 || (amax[c] != 0u && scale_n < fmt_bias(f) + (MODE == 1 ? 1 : 0));
        scale[c] = (uint32_t)scale_n;
    }
    if (__builtin_amdgcn_ballot_w64(hard) == 0) {
        const uint32_t lo = (uint32_t)(((int)scale[0] - fmt_bias(f)) << 7) & 0xFFFFu;
        const uint32_t hi = (uint32_t)(((int)scale[1] - fmt_bias(f)) << 7) & 0xFFFFu;
        const uint32_t ssb2 = lo | (hi << 16);
#pragma unroll
        for (int j = 0; j < 32; ++j) res[j] = MODE == 0 ? PackedBf16<F>::codes(h[j], ssb2) : PackedBf16<F>::qdq(h[j], ssb2);
    } else {
        // exact per-element routine
        int se[2];
        float sc[2];
#pragma unroll
        for (int t = 0; t < 2; ++t) {
            const uint32_t amax32 = amax[t] << 16;
            se[t] = shared_exponent<F, true>(amax32, f);
            scale[t] = amax32 < 0x00800000u ? 0u : (uint32_t)(se[t] + 127);
            sc[t] = scale_f32(scale[t]);
        }
#pragma unroll
        for (int j = 0; j < 32; ++j) {
            const uint32_t c0 = encode_mxfp_element(h[j] << 16, se[0], f);
            const uint32_t c1 = encode_mxfp_element(h[j] & 0xFFFF0000u, se[1], f);
            res[j] = MODE == 0 ? (c0 | (c1 << 16)) : pack_bf16(mxfp_value(c0, sc[0], f), mxfp_value(c1, sc[1], f));
        }
    }
}

// bytes 0 / 2 of res[j] are the codes of the lane's first / second column in row j -> 32 code bytes per column
__device__ inline void gather_column_codes(const uint32_t (&res)[32], uint32_t (&cd)[2][8]) {
#pragma unroll
    for (int w = 0; w < 8; ++w) {
        const uint32_t t01 = __builtin_amdgcn_perm(res[4 * w + 1], res[4 * w], 0x06020400u);
        const uint32_t t23 = __builtin_amdgcn_perm(res[4 * w + 3], res[4 * w + 2], 0x06020400u);
        cd[0][w] = __builtin_amdgcn_perm(t23, t01, 0x05040100u);
        cd[1][w] = __builtin_amdgcn_perm(t23, t01, 0x07060302u);
    }
}

template <class F, int MODE>
__global__ __launch_bounds__(kThreads) void mxfp_strided_bf16_kernel(const uint16_t* x, uint8_t* __restrict__ scales,
                                                                      uint8_t* __restrict__ elements, uint16_t* out,
                                                                      StridedGeom g, bool elements_aligned16, F f) {
    int64_t o, kb0, i0;
    if (!strided_origin(g, 2, o, kb0, i0)) return;
    for (int q = 0; q < g.kb_per; ++q) {
        const int64_t kb = kb0 + q;
        if (kb >= g.nkb) break;
        const int64_t first = (o * g.K + kb * 32) * g.inner + i0;
        uint32_t res[32], scale[2];
        strided_bf16_block<F, MODE>(x, first, g.inner, f, res, scale);
        if (MODE == 0) {
            uint32_t cd[2][8];
            gather_column_codes(res, cd);
#pragma unroll
            for (int t = 0; t < 2; ++t) {
                const int64_t col = o * g.inner + i0 + t;
                uint8_t* dst = elements + col * g.K + kb * 32;
                if (elements_aligned16) {
                    st128<false>(dst, make_uint4(cd[t][0], cd[t][1], cd[t][2], cd[t][3]));
                    st128<false>(dst + 16, make_uint4(cd[t][4], cd[t][5], cd[t][6], cd[t][7]));
                } else {
#pragma unroll
                    for (int b = 0; b < 32; ++b) dst[b] = (uint8_t)(cd[t][b >> 2] >> (8 * (b & 3)));
                }
                scales[col * g.nkb + kb] = (uint8_t)scale[t];
            }
        } else {
#pragma unroll
            for (int j = 0; j < 32; ++j) *reinterpret_cast<uint32_t*>(out + first + j * g.inner) = res[j];
        }
    }
}

// Extract with whole-line stores: a workgroup takes 128 adjacent columns and four consecutive k-blocks (one per
// wavefront), i.e. one 128-byte line of codes per column.  The lanes' 32-byte pieces meet in LDS ([column][128 B],
// row of column c = 64 (c & 1) + (c >> 1), 16-byte chunk k of a row at position k ^ ((row >> 1) & 7): conflict-free
// for the lane-per-column writes and for the 8-lanes-per-line reads), and every store instruction then writes 8
// whole lines instead of 64 quarter lines; the four scale bytes of a column leave as one dword.
// Needs inner % 128 == 0, K % 128 == 0, 16-byte aligned elements and 4-byte aligned scales.
constexpr int kStridedTCols = 128;
template <class F>
__global__ __launch_bounds__(kThreads) void mxfp_strided_bf16_lines_kernel(const uint16_t* x, uint8_t* __restrict__ scales,
                                                                            uint8_t* __restrict__ elements, int64_t K, int64_t inner,
                                                                            int64_t nkb, F f) {
    __shared__ __attribute__((aligned(16))) uint8_t tile[kStridedTCols * 128];
    __shared__ __attribute__((aligned(4))) uint8_t sc_tile[kStridedTCols * 4];
    const int lane = threadIdx.x & 63, q = threadIdx.x >> 6;
    // workgroup -> (outer, group of 4 k-blocks, chunk of 128 columns), column chunk fastest
    const int64_t col_chunks = inner / kStridedTCols, kgroups = nkb / 4;
    int64_t bid = blockIdx.x;
    const int64_t cc = bid % col_chunks;
    bid /= col_chunks;
    const int64_t kg = bid % kgroups, o = bid / kgroups;
    const int64_t iw = cc * kStridedTCols, kb0 = kg * 4;
    {
        const int64_t first = (o * K + (kb0 + q) * 32) * inner + iw + 2 * lane;
        uint32_t res[32], scale[2], cd[2][8];
        strided_bf16_block<F, 0>(x, first, inner, f, res, scale);
        gather_column_codes(res, cd);
#pragma unroll
        for (int t = 0; t < 2; ++t) {
            const int row = 64 * t + lane;
            uint8_t* const r = tile + row * 128;
            const int sw = (row >> 1) & 7;
            *reinterpret_cast<uint4*>(r + (((2 * q) ^ sw) * 16)) = make_uint4(cd[t][0], cd[t][1], cd[t][2], cd[t][3]);
            *reinterpret_cast<uint4*>(r + (((2 * q + 1) ^ sw) * 16)) = make_uint4(cd[t][4], cd[t][5], cd[t][6], cd[t][7]);
            sc_tile[(2 * lane + t) * 4 + q] = (uint8_t)scale[t];
        }
    }
    __syncthreads();
    const int64_t col0 = o * inner + iw;
#pragma unroll
    for (int p = 0; p < 4; ++p) {
        const int row = 8 * (4 * q + p) + (lane >> 3), k = lane & 7;
        const int col = 2 * (row & 63) + (row >> 6);
        const uint4 v = *reinterpret_cast<const uint4*>(tile + row * 128 + ((k ^ ((row >> 1) & 7)) * 16));
        st128<false>(elements + (col0 + col) * K + kb0 * 32 + k * 16, v);
    }
    if (lane < 32) {
        const int col = 32 * q + lane;
        *reinterpret_cast<uint32_t*>(scales + (col0 + col) * nkb + kb0) = *reinterpret_cast<const uint32_t*>(sc_tile + col * 4);
    }
}

// MXFP components (reference layout: one code byte per element, scales [rows, K / 32]) -> operand of the block-scaled
// GEMM.  A workgroup owns 32 rows x 512 k (four lines of the transposed scale array, one per 128 k): a lane 16 codes per
// 128 k, two lanes a block, eight lanes the 128 bytes of a row.  A row's sixteen scale bytes of the 512 k are one 128-bit
// load (a dword per 128 k where the row ends before that or is not 16-byte aligned there) and four dwords on the way out.
template <class F>
__global__ __launch_bounds__(kThreads) void scaled_operand_kernel(const uint8_t* __restrict__ scales, const uint8_t* __restrict__ elements,
                                                                   uint8_t* __restrict__ out_codes, uint32_t* __restrict__ out_scales,
                                                                   int rows, int K, int nmac, uint32_t rows_pad, uint32_t units, bool scales_by_16, F f) {
    // Workgroups are dealt to the eight XCDs (each with its own L2) round-robin.  The workgroups of one row set read
    // different 16-byte pieces of the same scale lines, so they are renumbered to follow each other on ONE XCD:
    // seven eighths of the scale fetches came from that otherwise (1.21 x the kernel's bytes).
    const uint32_t groups = ((uint32_t)nmac + 3u) / 4u, per_xcd = gridDim.x / 8u;
    const uint32_t unit = (blockIdx.x % 8u) * per_xcd + blockIdx.x / 8u;
    if (unit >= units) return;
    const uint32_t ms0 = (unit % groups) * 4u, row = (unit / groups) * 32u + (threadIdx.x >> 3);
    const int piece = threadIdx.x & 7;                  // 16 codes of the row's 128
    const bool live = row < (uint32_t)rows;
    const size_t off = (size_t)row * K + ms0 * 128u + (uint32_t)piece * 16u;
    const uint8_t* srow = scales + ((size_t)row * (K / 32) + ms0 * 4u);
    uint4 w[4];
    uint32_t sc4[4] = {0u, 0u, 0u, 0u};
#pragma unroll
    for (int j = 0; j < 4; ++j) w[j] = live && ms0 + j < (uint32_t)nmac ? ld128(elements + off + j * 128) : make_uint4(0, 0, 0, 0);
    if (live) {
        if (scales_by_16 && ms0 + 3u < (uint32_t)nmac) {
            const uint4 v = *reinterpret_cast<const uint4*>(srow);
            sc4[0] = v.x; sc4[1] = v.y; sc4[2] = v.z; sc4[3] = v.w;
        } else {
#pragma unroll
            for (int j = 0; j < 4; ++j)
                if (ms0 + j < (uint32_t)nmac) sc4[j] = *reinterpret_cast<const uint32_t*>(srow + 4 * j);
        }
    }
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        uint32_t scale = (sc4[j] >> (8 * (piece >> 1))) & 0xFFu;
        if constexpr (F{}.E() == 4 && F{}.M() == 3) {
            uint32_t top = e4m3_top_bits(w[j].x) | e4m3_top_bits(w[j].y) | e4m3_top_bits(w[j].z) | e4m3_top_bits(w[j].w);
            top |= (uint32_t)__builtin_amdgcn_mov_dpp((int)top, 0xB1, 0xF, 0xF, true);  // lane ^ 1
            if (top != 0u && scale < 254u) {
                w[j] = make_uint4(e4m3_halve4(w[j].x), e4m3_halve4(w[j].y), e4m3_halve4(w[j].z), e4m3_halve4(w[j].w));
                scale += 1u;
            }
        } else {
            w[j] = make_uint4(embed_e4m3_x4(w[j].x, f), embed_e4m3_x4(w[j].y, f), embed_e4m3_x4(w[j].z, f), embed_e4m3_x4(w[j].w, f));
        }
        // the row's four scale bytes (lanes 0, 2, 4, 6 of its 8) into its first lane: row_shl 2, 4, 6
        uint32_t dw = scale;
        dw |= (uint32_t)__builtin_amdgcn_update_dpp(0, (int)scale, 0x102, 0xF, 0xF, true) << 8;
        dw |= (uint32_t)__builtin_amdgcn_update_dpp(0, (int)scale, 0x104, 0xF, 0xF, true) << 16;
        dw |= (uint32_t)__builtin_amdgcn_update_dpp(0, (int)scale, 0x106, 0xF, 0xF, true) << 24;
        if (live && ms0 + j < (uint32_t)nmac) {
            st128(out_codes + off + j * 128, w[j]);
            if (piece == 0) out_scales[(size_t)(ms0 + j) * rows_pad + row] = dw;
        }
    }
}

// ------------------------------------------------------------------------------ launch helpers
inline unsigned grid_for(int64_t items, int per_block) {
    return (unsigned)((items + per_block - 1) / per_block);
}

inline bool pow2(int v) { return v > 0 && (v & (v - 1)) == 0; }
inline int ilog2(int v) { int s = 0; while ((1 << s) < v) ++s; return s; }

}  // namespace mase

using namespace mase;

namespace mase {
std::string& last_error() {
    static thread_local std::string msg;
    return msg;
}
}  // namespace mase

extern "C" {

int mase_hip_abi_version(void) { return 1; }

const char* mase_hip_last_error(void) { return last_error().c_str(); }

int mase_hip_extract_minifloat(const void* x, int x_dtype, uint16_t* codes, int64_t n, int exp_bits, int frac_bits,
                               int is_finite, int round_mode, void* stream) {
    if (int rc = check_minifloat_fmt(exp_bits, frac_bits, round_mode)) return rc;
    if (int rc = check_dtype(x_dtype, "input")) return rc;
    if (n < 0) return fail(ERR_INVALID, "n must be non-negative");
    if (n == 0) return OK;
    if (!x || !codes) return fail(ERR_INVALID, "null pointer");
    if (!aligned(x, 16) || !aligned(codes, 16)) return fail(ERR_INVALID, "x and codes must be 16-byte aligned");
    hipStream_t s = static_cast<hipStream_t>(stream);
    constexpr int UNROLL = MASE_UNROLL_SMALL;
    const unsigned grid = grid_for(n / 8 + 1, UNROLL * kThreads);
    return dispatch_fmt(exp_bits, frac_bits, is_finite, round_mode, [&](auto f) {
        return dispatch_dtype(x_dtype, [&](auto dt) {
            if constexpr (decltype(dt)::value == F32) {
                // whole runs of 512 elements: the kernel whose fp32 accesses are contiguous over the wavefront; the rest below
                const int64_t n_main = n & ~(int64_t)511;
                if (n_main > 0) {
                    hipLaunchKernelGGL((minifloat_f32_kernel<0, decltype(f)>), dim3(grid_for(n_main / 512, kThreads / 64)), dim3(kThreads), 0,
                                       s, x, static_cast<void*>(codes), n_main, f);
                    if (n_main == n) return check_launch("extract_minifloat");
                    hipLaunchKernelGGL((extract_minifloat_kernel<F32, decltype(f), UNROLL>), dim3(1), dim3(kThreads), 0, s,
                                       static_cast<const void*>(static_cast<const float*>(x) + n_main), codes + n_main, n - n_main, f);
                    return check_launch("extract_minifloat");
                }
            }
            hipLaunchKernelGGL((extract_minifloat_kernel<decltype(dt)::value, decltype(f), UNROLL>), dim3(grid), dim3(kThreads), 0, s, x,
                               codes, n, f);
            return check_launch("extract_minifloat");
        });
    });
}

int mase_hip_compose_minifloat(const uint16_t* codes, void* out, int out_dtype, int64_t n, int exp_bits, int frac_bits,
                               int is_finite, void* stream) {
    if (int rc = check_minifloat_fmt(exp_bits, frac_bits, RN)) return rc;
    if (int rc = check_dtype(out_dtype, "output")) return rc;
    if (n < 0) return fail(ERR_INVALID, "n must be non-negative");
    if (n == 0) return OK;
    if (!codes || !out) return fail(ERR_INVALID, "null pointer");
    if (!aligned(codes, 16) || !aligned(out, 16)) return fail(ERR_INVALID, "codes and out must be 16-byte aligned");
    hipStream_t s = static_cast<hipStream_t>(stream);
    constexpr int UNROLL = MASE_UNROLL_SMALL;
    const unsigned grid = grid_for(n / 8 + 1, UNROLL * kThreads);
    return dispatch_fmt(exp_bits, frac_bits, is_finite, RN, [&](auto f) {
        return dispatch_dtype(out_dtype, [&](auto dt) {
            if constexpr (decltype(dt)::value == F32) {
                const int64_t n_main = n & ~(int64_t)511;
                if (n_main > 0) {
                    hipLaunchKernelGGL((minifloat_f32_kernel<1, decltype(f)>), dim3(grid_for(n_main / 512, kThreads / 64)), dim3(kThreads), 0,
                                       s, static_cast<const void*>(codes), out, n_main, f);
                    if (n_main == n) return check_launch("compose_minifloat");
                    hipLaunchKernelGGL((compose_minifloat_kernel<F32, decltype(f), UNROLL>), dim3(1), dim3(kThreads), 0, s, codes + n_main,
                                       static_cast<void*>(static_cast<float*>(out) + n_main), n - n_main, f);
                    return check_launch("compose_minifloat");
                }
            }
            hipLaunchKernelGGL((compose_minifloat_kernel<decltype(dt)::value, decltype(f), UNROLL>), dim3(grid), dim3(kThreads), 0, s,
                               codes, out, n, f);
            return check_launch("compose_minifloat");
        });
    });
}

int mase_hip_qdq_minifloat(const void* x, int x_dtype, void* out, int out_dtype, int64_t n, int exp_bits, int frac_bits,
                           int is_finite, int round_mode, void* stream) {
    if (int rc = check_minifloat_fmt(exp_bits, frac_bits, round_mode)) return rc;
    if (int rc = check_dtype(x_dtype, "input")) return rc;
    if (int rc = check_dtype(out_dtype, "output")) return rc;
    if (n < 0) return fail(ERR_INVALID, "n must be non-negative");
    if (n == 0) return OK;
    if (!x || !out) return fail(ERR_INVALID, "null pointer");
    if (!aligned(x, 16) || !aligned(out, 16)) return fail(ERR_INVALID, "x and out must be 16-byte aligned");
    if (x == out && dtype_size(x_dtype) != dtype_size(out_dtype)) return fail(ERR_INVALID, "in-place use needs equal element sizes");
    hipStream_t s = static_cast<hipStream_t>(stream);
    constexpr int UNROLL = MASE_UNROLL_SMALL;
    const unsigned grid = grid_for(n / 8 + 1, UNROLL * kThreads);
    return dispatch_fmt(exp_bits, frac_bits, is_finite, round_mode, [&](auto f) {
        return dispatch_dtype(x_dtype, [&](auto di) {
            return dispatch_dtype(out_dtype, [&](auto dout) {
                if constexpr (decltype(di)::value == F32 && decltype(dout)::value == F32) {
                    const int64_t n_main = n & ~(int64_t)511;
                    if (n_main > 0) {
                        hipLaunchKernelGGL((minifloat_f32_kernel<2, decltype(f)>), dim3(grid_for(n_main / 512, kThreads / 64)), dim3(kThreads),
                                           0, s, x, out, n_main, f);
                        if (n_main == n) return check_launch("qdq_minifloat");
                        hipLaunchKernelGGL((qdq_minifloat_kernel<F32, F32, decltype(f), UNROLL>), dim3(1), dim3(kThreads), 0, s,
                                           static_cast<const void*>(static_cast<const float*>(x) + n_main),
                                           static_cast<void*>(static_cast<float*>(out) + n_main), n - n_main, f);
                        return check_launch("qdq_minifloat");
                    }
                }
                hipLaunchKernelGGL((qdq_minifloat_kernel<decltype(di)::value, decltype(dout)::value, decltype(f), UNROLL>), dim3(grid),
                                   dim3(kThreads), 0, s, x, out, n, f);
                return check_launch("qdq_minifloat");
            });
        });
    });
}

int mase_hip_extract_mxfp(const void* x, int x_dtype, uint8_t* scales, uint8_t* elements, int64_t n, int block_size,
                          int exp_bits, int frac_bits, int is_finite, int round_mode, void* stream) {
    if (int rc = check_mxfp_fmt(exp_bits, frac_bits, round_mode, n, block_size)) return rc;
    if (int rc = check_dtype(x_dtype, "input")) return rc;
    if (n == 0) return OK;
    if (!x || !scales || !elements) return fail(ERR_INVALID, "null pointer");
    hipStream_t s = static_cast<hipStream_t>(stream);
    constexpr int EPT = 8, UNROLL = MASE_UNROLL_MXFP;
    const int B = block_size;
    const bool vec = B % EPT == 0 && pow2(B / EPT) && B / EPT <= 64 && aligned(x, 16) && aligned(elements, 8);
    return dispatch_fmt(exp_bits, frac_bits, is_finite, round_mode, [&](auto f) {
        if constexpr (decltype(f)::kStatic) {
            if (x_dtype == BF16 && B == 32 && vec) {
                constexpr int U = MASE_UNROLL_EXTRACT;
                hipLaunchKernelGGL((mxfp_bf16_b32_kernel<decltype(f), U, 0>), dim3(grid_for(n / 8, U * kThreads)), dim3(kThreads), 0, s,
                                   static_cast<const uint4*>(x), scales, reinterpret_cast<uint2*>(elements), nullptr, n / 8, f);
                return check_launch("extract_mxfp");
            }
        }
        return dispatch_dtype(x_dtype, [&](auto dt) {
            if (vec) {
                const int lpb = B / EPT;
                hipLaunchKernelGGL((extract_mxfp_kernel<decltype(dt)::value, decltype(f), EPT, UNROLL>),
                                   dim3(grid_for(n / EPT, UNROLL * kThreads)), dim3(kThreads), 0, s, x, scales, elements, n, lpb,
                                   ilog2(lpb), f);
            } else {
                hipLaunchKernelGGL((extract_mxfp_block_kernel<decltype(dt)::value, decltype(f)>), dim3(grid_for(n / B, kThreads)),
                                   dim3(kThreads), 0, s, x, scales, elements, n / B, B, f);
            }
            return check_launch("extract_mxfp");
        });
    });
}

int mase_hip_compose_mxfp(const uint8_t* scales, const uint8_t* elements, void* out, int out_dtype, int64_t n,
                          int block_size, int exp_bits, int frac_bits, int is_finite, void* stream) {
    if (int rc = check_mxfp_fmt(exp_bits, frac_bits, RN, n, block_size)) return rc;
    if (int rc = check_dtype(out_dtype, "output")) return rc;
    if (n == 0) return OK;
    if (!scales || !elements || !out) return fail(ERR_INVALID, "null pointer");
    hipStream_t s = static_cast<hipStream_t>(stream);
    constexpr int UNROLL = MASE_UNROLL_COMPOSE;
    const int B = block_size;
    const bool al = aligned(elements, 8) && aligned(out, 16);
    return dispatch_fmt(exp_bits, frac_bits, is_finite, RN, [&](auto f) {
        return dispatch_dtype(out_dtype, [&](auto dt) {
            // 8 codes per lane: a wavefront then stores 1 KB contiguous per instruction (16 per lane would leave gaps)
            if constexpr (decltype(dt)::value == BF16 && HwCompose<decltype(f)>::value) {
                if (al && B % 8 == 0) {
                    hipLaunchKernelGGL((compose_mxfp_bf16_kernel<decltype(f), UNROLL>), dim3(grid_for(n / 8, UNROLL * kThreads)),
                                       dim3(kThreads), 0, s, scales, elements, out, n, B / 8, f);
                    return check_launch("compose_mxfp");
                }
            }
            if (al && B % 8 == 0) {
                hipLaunchKernelGGL((compose_mxfp_kernel<decltype(dt)::value, decltype(f), 8, UNROLL>),
                                   dim3(grid_for(n / 8, UNROLL * kThreads)), dim3(kThreads), 0, s, scales, elements, out, n, B / 8, f);
            } else {
                hipLaunchKernelGGL((compose_mxfp_scalar_kernel<decltype(dt)::value, decltype(f)>), dim3(grid_for(n, kThreads)),
                                   dim3(kThreads), 0, s, scales, elements, out, n, B, f);
            }
            return check_launch("compose_mxfp");
        });
    });
}

int mase_hip_qdq_mxfp(const void* x, int x_dtype, void* out, int out_dtype, int64_t n, int block_size, int exp_bits,
                      int frac_bits, int is_finite, int round_mode, void* stream) {
    if (int rc = check_mxfp_fmt(exp_bits, frac_bits, round_mode, n, block_size)) return rc;
    if (int rc = check_dtype(x_dtype, "input")) return rc;
    if (int rc = check_dtype(out_dtype, "output")) return rc;
    if (n == 0) return OK;
    if (!x || !out) return fail(ERR_INVALID, "null pointer");
    if (x == out && dtype_size(x_dtype) != dtype_size(out_dtype)) return fail(ERR_INVALID, "in-place use needs equal element sizes");
    hipStream_t s = static_cast<hipStream_t>(stream);
    constexpr int EPT = 8, UNROLL = MASE_UNROLL_MXFP;
    const int B = block_size;
    const bool vec = B % EPT == 0 && pow2(B / EPT) && B / EPT <= 64 && aligned(x, 16) && aligned(out, 16);
    return dispatch_fmt(exp_bits, frac_bits, is_finite, round_mode, [&](auto f) {
        if constexpr (decltype(f)::kStatic) {
            if (x_dtype == BF16 && out_dtype == BF16 && B == 32 && vec) {
                constexpr int U = MASE_UNROLL_PACKED;
                hipLaunchKernelGGL((mxfp_bf16_b32_kernel<decltype(f), U, 1>), dim3(grid_for(n / 8, U * kThreads)), dim3(kThreads), 0, s,
                                   static_cast<const uint4*>(x), nullptr, nullptr, static_cast<uint4*>(out), n / 8, f);
                return check_launch("qdq_mxfp");
            }
        }
        return dispatch_dtype(x_dtype, [&](auto di) {
            return dispatch_dtype(out_dtype, [&](auto dout) {
                if (vec) {
                    hipLaunchKernelGGL((qdq_mxfp_kernel<decltype(di)::value, decltype(dout)::value, decltype(f), EPT, UNROLL>),
                                       dim3(grid_for(n / EPT, UNROLL * kThreads)), dim3(kThreads), 0, s, x, out, n, B / EPT, f);
                } else {
                    hipLaunchKernelGGL((qdq_mxfp_block_kernel<decltype(di)::value, decltype(dout)::value, decltype(f)>),
                                       dim3(grid_for(n / B, kThreads)), dim3(kThreads), 0, s, x, out, n / B, B, f);
                }
                return check_launch("qdq_mxfp");
            });
        });
    });
}

// Blocks along the middle axis of an [outer, K, inner] tensor (no counterpart kernel in the
// reference, which permutes and copies first; same outputs as that route).
static int strided_args(int64_t outer, int64_t k_len, int64_t inner, int block_size) {
    if (outer < 0 || k_len < 0 || inner < 0) return fail(ERR_INVALID, "negative extent");
    if (block_size != 32) return fail(ERR_UNSUPPORTED, "strided blocks need block_size 32");
    if (k_len % 32 != 0) return fail(ERR_UNSUPPORTED, "strided blocks need the block axis to be a multiple of 32");
    if (outer != 0 && k_len != 0 && inner != 0 && (outer > INT64_MAX / k_len || outer * k_len > INT64_MAX / inner))
        return fail(ERR_INVALID, "extent overflow");
    return OK;
}

// k-blocks handled in sequence by one lane: up to 4 (a lane then fills whole 128-byte lines of
// codes), fewer while that leaves less than a few wavefronts per SIMD
static StridedGeom strided_geom(int64_t outer, int64_t k_len, int64_t inner, int vec, unsigned& grid, bool& ok) {
    StridedGeom g;
    g.K = k_len; g.inner = inner; g.nkb = k_len / 32;
    g.chunks = inner / vec;
    int kb_per = 4;
    while (kb_per > 1 && outer * ((g.nkb + kb_per - 1) / kb_per) * g.chunks < (int64_t)256 * 16 * 64) kb_per >>= 1;
    g.kb_per = kb_per;
    g.kgroups = (g.nkb + kb_per - 1) / kb_per;
    g.items = outer * g.kgroups * g.chunks;
    const int64_t blocks = (g.items + kThreads - 1) / kThreads;
    ok = blocks <= 0x7FFFFFFFll;
    grid = (unsigned)blocks;
    return g;
}

int mase_hip_extract_mxfp_strided(const void* x, int x_dtype, uint8_t* scales, uint8_t* elements, int64_t outer,
                                  int64_t k_len, int64_t inner, int block_size, int exp_bits, int frac_bits, int is_finite,
                                  int round_mode, void* stream) {
    if (int rc = strided_args(outer, k_len, inner, block_size)) return rc;
    if (int rc = check_mxfp_fmt(exp_bits, frac_bits, round_mode, 0, block_size)) return rc;
    if (int rc = check_dtype(x_dtype, "input")) return rc;
    if (outer == 0 || k_len == 0 || inner == 0) return OK;
    if (!x || !scales || !elements) return fail(ERR_INVALID, "null pointer");
    hipStream_t s = static_cast<hipStream_t>(stream);
    const bool el16 = aligned(elements, 16);
    return dispatch_fmt(exp_bits, frac_bits, is_finite, round_mode, [&](auto f) {
        unsigned grid; bool ok;
        if constexpr (decltype(f)::kStatic) {
            if (x_dtype == BF16 && inner % 2 == 0 && aligned(x, 4)) {
                if (inner % kStridedTCols == 0 && k_len % 128 == 0 && el16 && aligned(scales, 4)) {
                    const int64_t blocks = outer * (k_len / 128) * (inner / kStridedTCols);
                    if (blocks > 0x7FFFFFFFll) return fail(ERR_UNSUPPORTED, "tensor too large for one launch");
                    hipLaunchKernelGGL((mxfp_strided_bf16_lines_kernel<decltype(f)>), dim3((unsigned)blocks), dim3(kThreads), 0, s,
                                       static_cast<const uint16_t*>(x), scales, elements, k_len, inner, k_len / 32, f);
                    return check_launch("extract_mxfp_strided");
                }
                const StridedGeom g = strided_geom(outer, k_len, inner, 2, grid, ok);
                if (!ok) return fail(ERR_UNSUPPORTED, "tensor too large for one launch");
                hipLaunchKernelGGL((mxfp_strided_bf16_kernel<decltype(f), 0>), dim3(grid), dim3(kThreads), 0, s,
                                   static_cast<const uint16_t*>(x), scales, elements, nullptr, g, el16, f);
                return check_launch("extract_mxfp_strided");
            }
        }
        const StridedGeom g = strided_geom(outer, k_len, inner, 1, grid, ok);
        if (!ok) return fail(ERR_UNSUPPORTED, "tensor too large for one launch");
        return dispatch_dtype(x_dtype, [&](auto dt) {
            hipLaunchKernelGGL((mxfp_strided_kernel<decltype(dt)::value, F32, decltype(f), 0>), dim3(grid), dim3(kThreads), 0, s, x,
                               scales, elements, nullptr, g, el16, f);
            return check_launch("extract_mxfp_strided");
        });
    });
}

int mase_hip_qdq_mxfp_strided(const void* x, int x_dtype, void* out, int out_dtype, int64_t outer, int64_t k_len,
                              int64_t inner, int block_size, int exp_bits, int frac_bits, int is_finite, int round_mode,
                              void* stream) {
    if (int rc = strided_args(outer, k_len, inner, block_size)) return rc;
    if (int rc = check_mxfp_fmt(exp_bits, frac_bits, round_mode, 0, block_size)) return rc;
    if (int rc = check_dtype(x_dtype, "input")) return rc;
    if (int rc = check_dtype(out_dtype, "output")) return rc;
    if (outer == 0 || k_len == 0 || inner == 0) return OK;
    if (!x || !out) return fail(ERR_INVALID, "null pointer");
    if (x == out && dtype_size(x_dtype) != dtype_size(out_dtype)) return fail(ERR_INVALID, "in-place use needs equal element sizes");
    hipStream_t s = static_cast<hipStream_t>(stream);
    return dispatch_fmt(exp_bits, frac_bits, is_finite, round_mode, [&](auto f) {
        unsigned grid; bool ok;
        if constexpr (decltype(f)::kStatic) {
            if (x_dtype == BF16 && out_dtype == BF16 && inner % 2 == 0 && aligned(x, 4) && aligned(out, 4)) {
                const StridedGeom g = strided_geom(outer, k_len, inner, 2, grid, ok);
                if (!ok) return fail(ERR_UNSUPPORTED, "tensor too large for one launch");
                hipLaunchKernelGGL((mxfp_strided_bf16_kernel<decltype(f), 1>), dim3(grid), dim3(kThreads), 0, s,
                                   static_cast<const uint16_t*>(x), nullptr, nullptr, static_cast<uint16_t*>(out), g, false, f);
                return check_launch("qdq_mxfp_strided");
            }
        }
        const StridedGeom g = strided_geom(outer, k_len, inner, 1, grid, ok);
        if (!ok) return fail(ERR_UNSUPPORTED, "tensor too large for one launch");
        return dispatch_dtype(x_dtype, [&](auto di) {
            return dispatch_dtype(out_dtype, [&](auto dout) {
                hipLaunchKernelGGL((mxfp_strided_kernel<decltype(di)::value, decltype(dout)::value, decltype(f), 1>), dim3(grid),
                                   dim3(kThreads), 0, s, x, nullptr, nullptr, out, g, false, f);
                return check_launch("qdq_mxfp_strided");
            });
        });
    });
}

// ---- operands of the block-scaled GEMM (mase_hip_mxfp_gemm_scaled)
int64_t mase_hip_scaled_padded_rows(int64_t rows) { return rows <= 0 ? 0 : (rows + 255) / 256 * 256; }

static int scaled_operand_args(int64_t rows, int64_t K, int exp_bits, int frac_bits, uint32_t& rows_pad) {
    if (rows < 1 || K < 1) return fail(ERR_INVALID, "rows and K must be positive");
    if (K % 128 != 0) return fail(ERR_UNSUPPORTED, "the block-scaled GEMM needs K to be a multiple of 128");
    if (K >= ((int64_t)1 << 27) || rows * (K / 32) >= ((int64_t)1 << 31)) return fail(ERR_UNSUPPORTED, "operand too large for the block-scaled GEMM");
    const bool ok = (exp_bits == 4 && frac_bits == 3) || (exp_bits == 2 && frac_bits == 3) || (exp_bits == 3 && frac_bits == 2) ||
                    (exp_bits == 2 && frac_bits == 1);
    if (!ok) return fail(ERR_UNSUPPORTED, "the block-scaled GEMM takes element formats (4,3) (2,3) (3,2) (2,1)");
    rows_pad = (uint32_t)mase_hip_scaled_padded_rows(rows);
    return OK;
}

int mase_hip_scaled_operand_from_mxfp(const uint8_t* scales, const uint8_t* elements, int exp_bits, int frac_bits, int64_t rows, int64_t K,
                                      uint8_t* out_codes, uint32_t* out_scales, void* stream) {
    uint32_t rows_pad;
    if (int rc = scaled_operand_args(rows, K, exp_bits, frac_bits, rows_pad)) return rc;
    if (!scales || !elements || !out_codes || !out_scales) return fail(ERR_INVALID, "null pointer");
    if (!aligned(elements, 16) || !aligned(out_codes, 16) || !aligned(out_scales, 4) || !aligned(scales, 4))
        return fail(ERR_INVALID, "elements and out_codes must be 16-byte aligned, scales and out_scales 4-byte aligned");
    hipStream_t s = static_cast<hipStream_t>(stream);
    return dispatch_fmt(exp_bits, frac_bits, 1, RN, [&](auto f) {
        if constexpr (decltype(f)::kStatic && decltype(f){}.E() != 5) {
            const int nmac = (int)(K / 128);
            const int64_t blocks = (rows + 31) / 32 * ((nmac + 3) / 4);
            if (blocks > 0x7FFFFFF0ll) return fail(ERR_UNSUPPORTED, "operand too large for one launch");
            const bool scales_by_16 = aligned(scales, 16) && (K / 32) % 16 == 0;   // every row's scales of 512 k are one aligned 128-bit word
            hipLaunchKernelGGL((scaled_operand_kernel<decltype(f)>), dim3((unsigned)((blocks + 7) / 8 * 8)), dim3(kThreads), 0, s, scales, elements,
                               out_codes, out_scales, (int)rows, (int)K, nmac, rows_pad, (uint32_t)blocks, scales_by_16, f);
            return check_launch("scaled_operand_from_mxfp");
        }
        return fail(ERR_UNSUPPORTED, "element format not supported by the block-scaled GEMM");
    });
}

static int scaled_from_dense_entry(const void* x, const void* up, int64_t ld, int x_dtype, int exp_bits, int frac_bits, int64_t rows, int64_t K,
                                   uint8_t* out_codes, uint32_t* out_scales, void* stream, bool minifloat = false) {
    uint32_t rows_pad;
    if (int rc = scaled_operand_args(rows, K, exp_bits, frac_bits, rows_pad)) return rc;
    if (x_dtype != BF16) return fail(ERR_UNSUPPORTED, "a dense operand of the block-scaled GEMM must be bfloat16");
    if (!x || !out_codes || !out_scales) return fail(ERR_INVALID, "null pointer");
    if (ld < K || ld % 8 != 0) return fail(ERR_INVALID, "the row stride must be at least K and a multiple of 8 elements");
    if (!aligned(x, 16) || (up && !aligned(up, 16)) || !aligned(out_codes, 8) || !aligned(out_scales, 4))
        return fail(ERR_INVALID, "the dense inputs must be 16-byte aligned, out_codes 8-byte, out_scales 4-byte");
    hipStream_t s = static_cast<hipStream_t>(stream);
    return dispatch_fmt(exp_bits, frac_bits, 1, RN, [&](auto f) {
        if constexpr (decltype(f)::kStatic && decltype(f){}.E() != 5) {
            const int nmac = (int)(K / 128);
            const int64_t blocks = (rows + 31) / 32 * nmac;
            if (blocks > 0x7FFFFFFFll) return fail(ERR_UNSUPPORTED, "operand too large for one launch");
            const uint16_t *xp = static_cast<const uint16_t*>(x), *upp = static_cast<const uint16_t*>(up);
            if (minifloat)
                hipLaunchKernelGGL((scaled_from_dense_kernel<decltype(f), FROM_DENSE_MINIFLOAT>), dim3((unsigned)blocks), dim3(kThreads), 0, s, xp, upp,
                                   (size_t)ld, out_codes, out_scales, (int)rows, (int)K, nmac, rows_pad, f);
            else if (up)
                hipLaunchKernelGGL((scaled_from_dense_kernel<decltype(f), FROM_SWIGLU>), dim3((unsigned)blocks), dim3(kThreads), 0, s, xp, upp, (size_t)ld,
                                   out_codes, out_scales, (int)rows, (int)K, nmac, rows_pad, f);
            else
                hipLaunchKernelGGL((scaled_from_dense_kernel<decltype(f), FROM_DENSE>), dim3((unsigned)blocks), dim3(kThreads), 0, s, xp, upp, (size_t)ld,
                                   out_codes, out_scales, (int)rows, (int)K, nmac, rows_pad, f);
            return check_launch("scaled_operand_from_dense");
        }
        return fail(ERR_UNSUPPORTED, "element format not supported by the block-scaled GEMM");
    });
}

int mase_hip_scaled_operand_from_dense(const void* x, int x_dtype, int exp_bits, int frac_bits, int64_t rows, int64_t K, uint8_t* out_codes,
                                       uint32_t* out_scales, void* stream) {
    return scaled_from_dense_entry(x, nullptr, K, x_dtype, exp_bits, frac_bits, rows, K, out_codes, out_scales, stream);
}

int mase_hip_scaled_operand_from_dense_minifloat(const void* x, int x_dtype, int exp_bits, int frac_bits, int64_t rows, int64_t K,
                                                 uint8_t* out_codes, uint32_t* out_scales, void* stream) {
    return scaled_from_dense_entry(x, nullptr, K, x_dtype, exp_bits, frac_bits, rows, K, out_codes, out_scales, stream, true);
}

int mase_hip_scaled_operand_from_swiglu(const void* gate, const void* up, int dtype, int64_t row_stride, int exp_bits, int frac_bits, int64_t rows,
                                        int64_t K, uint8_t* out_codes, uint32_t* out_scales, void* stream) {
    if (!up) return fail(ERR_INVALID, "null pointer");
    return scaled_from_dense_entry(gate, up, row_stride, dtype, exp_bits, frac_bits, rows, K, out_codes, out_scales, stream);
}

}  // extern "C"
