// In-register compose of MXFP codes to bf16, shared by the GEMM kernels (which compose weights on their way to LDS) and the
// bf16 compose kernel of the casts.
#pragma once
#include "mase_device.h"

namespace mase {

typedef float floatx2_t __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
typedef _Float16 halfx2_t __attribute__((ext_vector_type(2)));

__device__ inline uint32_t cvt_pk_bf16(float a, float b) {
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(floatx2_t{a, b}, bf16x2_t));
}

// ---------------------------------------------------------------------------------------------
// In-register compose of MXFP codes to bf16.
//
// Fast route (every format with at most 4 exponent bits, almost every scale): gfx950's
// v_cvt_scalef32_pk_bf16_fp8 turns two E4M3 bytes and one power-of-two scale into two bf16, one
// instruction per pair, subnormal codes, subnormal results and overflow to inf included (checked
// against the reference's compose for every scale byte 0..254 and every code).  A code of a narrower
// format becomes an E4M3 byte by moving its sign to bit 7 and its magnitude bits to the top of the
// 7 magnitude bits' low end (exponent field in the low bits of E4M3's): that byte reads as
// value * 2^(bias - 7), for normal and subnormal codes alike, so the scale goes up by 7 - bias.
// The one difference in meaning: the hardware reads magnitude 0x7F as NaN where the reference's finite
// E4M3 has 480.  For E4M3 the magnitudes are therefore converted without their signs, the result is
// clamped (as a 16-bit integer, where NaN is above every finite pattern) to the pattern of
// 480 * 2^(scale - 127), the largest value the block can hold, and the signs are put back.
//
// Slow route, exact for every scale (a wave-uniform branch the callers take only when a scale in
// reach is at or above SLOW_FROM, i.e. the hardware's scale byte would reach 255, which it reads as
// NaN, or E4M3's clamp pattern would leave the normal bf16 range): the code's magnitude bits, placed
// so that its exponent field sits in the low bits of an fp16 exponent field, read as fp16 give
// value * 2^(bias - 15) for normal AND subnormal codes and 0 for the zero code; the fp16 -> fp32
// convert is exact; v_ldexp_f32 by (15 - bias + scale - 127) finishes with the single rounding the
// reference's fp32 multiply has, and the fp32 -> bf16 convert rounds to nearest even like the
// reference's cast.  Scale 255 means "times +inf" in the reference (0 -> NaN, anything else ->
// +-inf): patched on top.  E = 5 would fill the fp16 exponent field and has codes the hardware's
// E5M2 reads as inf / NaN, so E5M2 always takes the generic integer decode.
// ---------------------------------------------------------------------------------------------
template <class F>
struct Composer {
    static constexpr int E = F{}.E(), M = F{}.M();
    static constexpr int BIAS = (1 << (E - 1)) - 1;
    static constexpr bool HW = E <= 4;                       // hardware convert route
    // magnitude 0x7F: NaN to the hardware, 480 to the reference (prepared operands never hold it)
    static constexpr bool TOP_IS_NAN = E == 4 && M == 3 && !has_no_top_code<F>::value;
    static constexpr int SCALE_UP = 7 - BIAS;
    // first scale byte that needs the slow route (none for E5M2, whose only route handles every scale)
    static constexpr uint32_t SLOW_FROM = !HW ? 256u : TOP_IS_NAN ? 247u : (uint32_t)(255 - SCALE_UP);
    static constexpr uint32_t SIGN4 = (1u << (E + M)) * 0x01010101u, MAG4 = ((1u << (E + M)) - 1u) * 0x01010101u;
    // slow route: fp16 field placement
    static constexpr int PRE = 7 - E - M;      // left shift that moves the sign bit to bit 7 of each byte
    static constexpr int ASHR = 5 - E;         // then: exponent field from bits 14.. down to bits ..10 of each half
    static constexpr uint32_t KEEP = (0x8000u | (0x7FFFu >> ASHR)) * 0x00010001u;

    uint32_t scale;
    float hw_scale;   // 2^(scale + SCALE_UP - 127) as the convert's scale operand
    uint32_t top2;    // E4M3: bf16 pattern of 480 * 2^(scale - 127), in both halves
    __device__ inline explicit Composer(uint32_t scale_) : scale(scale_) {
        hw_scale = bits_f32((scale_ + (uint32_t)SCALE_UP) << 23);
        top2 = scale_ * 0x00800080u + 0x04700470u;
    }
    __device__ static inline bool is_slow(uint32_t scale_) { return HW && scale_ >= SLOW_FROM; }
    // does any of the four scale bytes of `s4` need the slow route?
    __device__ static inline bool any_slow4(uint32_t s4) {
        if (!HW) return false;
        // byte >= SLOW_FROM (> 128)  <=>  its bit 7 is set and its low 7 bits plus (256 - SLOW_FROM) carry into bit 7
        return ((((s4 & 0x7F7F7F7Fu) + (256u - SLOW_FROM) * 0x01010101u) & s4) & 0x80808080u) != 0u;
    }

    // four codes of a dword as E4M3 bytes
    __device__ static inline uint32_t embed4(uint32_t w) {
        if (E == 4 && M == 3) return w;
        if (E == 3 && M == 2) return (w + (w & SIGN4)) << 1;  // sign bit 5 -> 6 by the carry, then everything up by one
        return ((w & SIGN4) << (7 - E - M)) | ((w & MAG4) << (3 - M));
    }
    template <bool HI>
    __device__ inline uint32_t hw_pair(uint32_t w, uint32_t e4) const {  // e4 = embed4(w)
        typedef unsigned short ushort2_t __attribute__((ext_vector_type(2)));
        const uint32_t r = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(e4, hw_scale, HI));
        if (!TOP_IS_NAN) return r;
        // magnitude 0x7F comes back as 0xFFC0 whatever its sign; every other code as the right bf16, sign included.  As
        // unsigned 16-bit numbers 0xFFC0 is above every finite pattern of either sign and (sign | top) is the largest
        // finite one of its sign, so the minimum with (sign of the code | top) replaces exactly the NaNs.
        const uint32_t sg = __builtin_amdgcn_perm(0u, w, HI ? 0x030C020Cu : 0x010C000Cu);  // the pair's code bytes in the high byte of each half
        const uint32_t cand = (sg & 0x80008000u) | top2;
        return __builtin_bit_cast(uint32_t, __builtin_elementwise_min(__builtin_bit_cast(ushort2_t, r), __builtin_bit_cast(ushort2_t, cand)));
    }
    __device__ inline uint32_t bf16_pair_fp16(uint32_t x) const {  // x: each 16-bit half = (code << PRE) << 8
        typedef short shortx2 __attribute__((ext_vector_type(2)));
        const int n = (int)scale - 112 - BIAS;  // ldexp exponent: 15 - bias + scale - 127
        const shortx2 sh = __builtin_bit_cast(shortx2, x) >> (short)ASHR;   // v_pk_ashrrev_i16
        const halfx2_t h = __builtin_bit_cast(halfx2_t, __builtin_bit_cast(uint32_t, sh) & KEEP);
        return cvt_pk_bf16(ldexpf((float)h[0], n), ldexpf((float)h[1], n));
    }
    __device__ inline uint32_t bf16_pair_wide(uint32_t w, int p) const {
        const F f{};
        const float s_wide = scale_f32(scale);
        const float a = decode_f32((w >> (16 * p)) & 0xFFu, f) * s_wide, b = decode_f32((w >> (16 * p + 8)) & 0xFFu, f) * s_wide;
        return cvt_pk_bf16(a, b);
    }
    // codes 0,1 (pair_lo) / 2,3 (pair_hi) of a dword of 4 codes -> 2 bf16; any code; any scale below SLOW_FROM
    __device__ inline uint32_t pair_lo(uint32_t w) const {
        if (!HW) return bf16_pair_wide(w, 0);
        return hw_pair<false>(w, embed4(w));
    }
    __device__ inline uint32_t pair_hi(uint32_t w) const {
        if (!HW) return bf16_pair_wide(w, 1);
        return hw_pair<true>(w, embed4(w));
    }
    __device__ inline void pair2(uint32_t w, uint32_t& o0, uint32_t& o1) const {
        if (!HW) { o0 = bf16_pair_wide(w, 0); o1 = bf16_pair_wide(w, 1); return; }
        const uint32_t e4 = embed4(w);
        o0 = hw_pair<false>(w, e4);
        o1 = hw_pair<true>(w, e4);
    }
    // the same pairs on the slow route: any code, any scale (255 included)
    __device__ inline void pair2_slow(uint32_t w, uint32_t& o0, uint32_t& o1) const {
        if (!HW) { o0 = bf16_pair_wide(w, 0); o1 = bf16_pair_wide(w, 1); return; }
        o0 = bf16_pair_fp16(__builtin_amdgcn_perm(0u, w << PRE, 0x010C000Cu));  // top bits of every byte are zero: no spill between bytes
        o1 = bf16_pair_fp16(__builtin_amdgcn_perm(0u, w << PRE, 0x030C020Cu));
        if (scale == 255u) {
            // the ldexp gave 0 for zero codes where the reference has 0 * inf = NaN (non-zero codes already overflowed to +-inf)
            const uint32_t mag = (1u << (E + M)) - 1u;
#pragma unroll
            for (int b = 0; b < 4; ++b)
                if (((w >> (8 * b)) & mag) == 0u) {
                    uint32_t& d = (b >> 1) ? o1 : o0;
                    d = (b & 1) ? ((d & 0x0000FFFFu) | 0x7FC00000u) : ((d & 0xFFFF0000u) | 0x00007FC0u);
                }
        }
    }
    // 16 codes (one 128-bit word) of one block -> 16 bf16 (two 128-bit words), any code, any scale below SLOW_FROM
    __device__ inline void run16(const uint4& codes, uint4& lo, uint4& hi) const {
        const uint32_t w[4] = {codes.x, codes.y, codes.z, codes.w};
        uint32_t o[8];
#pragma unroll
        for (int j = 0; j < 4; ++j) pair2(w[j], o[2 * j], o[2 * j + 1]);
        lo = make_uint4(o[0], o[1], o[2], o[3]);
        hi = make_uint4(o[4], o[5], o[6], o[7]);
    }
    // SAFE = false is for callers that know no scale in reach needs the slow route (checked once per tile)
    template <bool SAFE>
    __device__ static inline void compose16(const uint4& codes, uint32_t scale_, uint4& lo, uint4& hi) {
        Composer(scale_).run16(codes, lo, hi);
        if (SAFE) fix_slow(scale_, codes, lo, hi);
    }
    // redo the lanes whose scale needs the slow route.  Rare: one wave-uniform branch per call.
    __device__ static inline void fix_slow(uint32_t scale_, const uint4& codes, uint4& lo, uint4& hi) {
        if (!HW) return;  // the generic route is exact for every scale
        if (__builtin_amdgcn_ballot_w64(is_slow(scale_)) == 0) return;
        if (!is_slow(scale_)) return;
        const Composer c(scale_);
        const uint32_t w[4] = {codes.x, codes.y, codes.z, codes.w};
        uint32_t o[8];
#pragma unroll
        for (int j = 0; j < 4; ++j) c.pair2_slow(w[j], o[2 * j], o[2 * j + 1]);
        lo = make_uint4(o[0], o[1], o[2], o[3]);
        hi = make_uint4(o[4], o[5], o[6], o[7]);
    }
};

}  // namespace mase
