// Device-side arithmetic shared by the cast kernels and the GEMM: minifloat encode/decode and
// the MXFP shared-exponent rules, bit-exact with the PyTorch "fake" path of the reference
// (src/mase_triton/minifloat/fake.py, src/mase_triton/mxfp/fake.py), written as integer
// operations on IEEE bit patterns so that the result does not depend on the GPU's denormal
// or rounding mode (the two float multiplies in decode rely on IEEE denormal handling, which
// is the HIP default on gfx950).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include <type_traits>

namespace mase {

enum DType : int { F32 = 0, F16 = 1, BF16 = 2 };
enum Round : int { RN = 0, RU = 1, RD = 2, RZ = 3 };

// ---------------------------------------------------------------------------------------
// Element formats.  SFmt is resolved at compile time (the five presets, rn, finite); DFmt
// carries the same four numbers at run time for every other (E, M, finite, round) combination.
// ---------------------------------------------------------------------------------------
template <int E_, int M_, bool FIN_ = true, int RM_ = RN>
struct SFmt {
    static constexpr bool kStatic = true;
    __host__ __device__ constexpr int E() const { return E_; }
    __host__ __device__ constexpr int M() const { return M_; }
    __host__ __device__ constexpr bool finite() const { return FIN_; }
    __host__ __device__ constexpr int rmode() const { return RM_; }
};

// E4M3 bytes as the operand-prepare kernels of the block-scaled GEMM leave them: every element format embedded into
// E4M3 with the same value, and no byte with the magnitude 0x7F (the one E4M3 code the hardware converts read as NaN)
struct PreparedE4M3 : SFmt<4, 3> {
    static constexpr bool kNoTopCode = true;
};
template <class F, class = void> struct has_no_top_code { static constexpr bool value = false; };
template <class F> struct has_no_top_code<F, std::enable_if_t<F::kNoTopCode>> { static constexpr bool value = true; };

struct DFmt {
    static constexpr bool kStatic = false;
    int e, m, fin, rm;
    __host__ __device__ int E() const { return e; }
    __host__ __device__ int M() const { return m; }
    __host__ __device__ bool finite() const { return fin != 0; }
    __host__ __device__ int rmode() const { return rm; }
};

template <class F> __host__ __device__ inline int fmt_bias(const F& f) { return (1 << (f.E() - 1)) - 1; }
template <class F> __host__ __device__ inline int fmt_emax_field(const F& f) {
    return f.finite() ? (1 << f.E()) - 1 : (1 << f.E()) - 2;
}
template <class F> __host__ __device__ inline int fmt_emax_unb(const F& f) { return fmt_emax_field(f) - fmt_bias(f); }
template <class F> __host__ __device__ inline uint32_t fmt_sign(const F& f) { return 1u << (f.E() + f.M()); }

// ---------------------------------------------------------------------------------------
// Scalar <-> fp32 bit pattern conversions for the three I/O dtypes.
// ---------------------------------------------------------------------------------------
__device__ inline uint32_t f32_bits(float v) { return __float_as_uint(v); }
__device__ inline float bits_f32(uint32_t u) { return __uint_as_float(u); }

__device__ inline uint32_t half_bits_to_f32_bits(uint32_t h) {
    // exact for every fp16 pattern, including subnormals, without relying on the fp16
    // denormal mode
    uint32_t s = (h & 0x8000u) << 16, e = (h >> 10) & 0x1Fu, m = h & 0x3FFu;
    if (e == 0) {
        if (m == 0) return s;
        int lz = __clz(m) - 21;  // m < 2^10: leading zeros within the 11-bit window
        m = (m << lz) & 0x3FFu;
        return s | ((uint32_t)(113 - lz) << 23) | (m << 13);
    }
    if (e == 31) return s | 0x7F800000u | (m << 13);
    return s | ((e + 112u) << 23) | (m << 13);
}

__device__ inline uint32_t f32_bits_to_bf16_bits(uint32_t u) {  // RNE; NaN stays NaN
    if ((u & 0x7FFFFFFFu) > 0x7F800000u) return 0x7FC0u | ((u >> 16) & 0x8000u);
    return (u + 0x7FFFu + ((u >> 16) & 1u)) >> 16;
}

__device__ inline uint32_t f32_bits_to_half_bits(uint32_t u) {  // IEEE RNE, integer only
    uint32_t s = (u >> 16) & 0x8000u, a = u & 0x7FFFFFFFu;
    if (a > 0x7F800000u) return s | 0x7E00u;
    if (a >= 0x47800000u) return s | 0x7C00u;
    if (a >= 0x38800000u) {
        uint32_t r = a - 0x38000000u;
        r = r + 0xFFFu + ((r >> 13) & 1u);
        return s | (r >> 13);
    }
    if (a < 0x33000000u) return s;
    uint32_t e = a >> 23, m = (a & 0x7FFFFFu) | 0x800000u;
    int sh = (int)(113 - e) + 13;
    uint32_t q = m >> sh, rem = m & ((1u << sh) - 1u), half = 1u << (sh - 1);
    q += (rem > half) || (rem == half && (q & 1u));
    return s | q;
}

// ---------------------------------------------------------------------------------------
// Mantissa rounding (minifloat/fake.py:41-56).  Every mode except rz first truncates the
// 23-bit mantissa to 15 bits and only then rounds to M bits.  Result is in [0, 2^M].
// ---------------------------------------------------------------------------------------
template <class F>
__device__ inline uint32_t round_mantissa(uint32_t f23, const F& f) {
    const int M = f.M();
    if (f.rmode() == RZ) return f23 >> (23 - M);
    const uint32_t f15 = f23 >> 8;
    const int sh = 15 - M;
    const uint32_t q = f15 >> sh;
    if (f.rmode() == RD) return q;
    const uint32_t r = f15 & ((1u << sh) - 1u);
    if (f.rmode() == RU) return q + (r != 0u);
    // round half to even: add (half - 1 + lsb) and truncate
    return (f15 + ((1u << (sh - 1)) - 1u) + (q & 1u)) >> sh;
}

// Code of a finite, fp32-normal value  (-1)^neg * 2^e * (1 + f23 / 2^23)   (fake.py:34-76).
// Note the deliberate OR at the end: a mantissa carry into an odd exponent field is lost.
template <class F>
__device__ inline uint32_t encode_normal(bool neg, int e, uint32_t f23, const F& f) {
    const int M = f.M(), bias = fmt_bias(f);
    uint32_t yf = round_mantissa(f23, f);
    int ye = e + bias;
    if (ye == 0 && yf != 0u) yf = (yf | (1u << M)) >> 1;
    if (e < -bias) { ye = 0; yf = 0u; }
    if (e > fmt_emax_unb(f)) { ye = fmt_emax_field(f); yf = (1u << M) - 1u; }
    uint32_t y = ((uint32_t)ye << M) | yf;
    return neg ? y + fmt_sign(f) : y;
}

// Code of the NaN/inf input with mantissa field f23 (frexp gives exponent 0, so e = -1; the
// NaN payload, quiet bit forced, goes through the mantissa rounding like any other).
template <class F>
__device__ inline uint32_t encode_nonfinite(bool neg_inf, bool is_nan, uint32_t f23, const F& f) {
    if (!f.finite()) {
        const uint32_t top = (uint32_t)fmt_emax_field(f) << f.M();
        if (is_nan) return top | ((1u << f.M()) - 1u);
        return neg_inf ? top + fmt_sign(f) : top;
    }
    if (is_nan) f23 |= 0x400000u;
    return encode_normal(neg_inf, -1, f23, f);
}

// Code of an arbitrary fp32 bit pattern (the minifloat path, fake.py:21-77).
template <class F>
__device__ inline uint32_t encode_f32_bits(uint32_t u, const F& f) {
    const uint32_t a = u & 0x7FFFFFFFu, ef = a >> 23;
    const bool sgn = (u >> 31) != 0u;
    if (ef == 0u) return (sgn && a != 0u) ? fmt_sign(f) : 0u;  // flushed; negative subnormal keeps the sign code
    if (ef == 255u) {
        const bool is_nan = a > 0x7F800000u;
        return encode_nonfinite(sgn && !is_nan, is_nan, a & 0x7FFFFFu, f);
    }
    return encode_normal(sgn, (int)ef - 127, a & 0x7FFFFFu, f);
}

// The same code for a compile-time format (finite, round to nearest even) and any input that is not inf / NaN, without
// branches.  With a15 = |u| >> 8 (exponent field above the 15 mantissa bits the reference keeps) and
//     t = a15 - ((127 - bias) << 15)            (clamped at 0: e < -bias gives code 0)
// t is (ye << 15) | f15, the exponent field in the target format above those 15 bits, and the rounding, the lost
// carry of the final OR, the subnormal binade ye == 0 and the saturation are functions of t.  Zero and subnormal
// inputs have a15 < 2^15 and fall to t = 0; they keep the sign code when negative and not -0.0 (fake.py:21-77).
template <class F>
__device__ inline uint32_t encode_f32_finite_rn(uint32_t u, const F& f) {
    static_assert(F::kStatic, "compile-time formats only");
    static_assert(F{}.finite() && F{}.rmode() == RN, "finite formats, round to nearest even");
    constexpr int E = F{}.E(), M = F{}.M(), SH = 15 - M, BIAS = (1 << (E - 1)) - 1;
    constexpr uint32_t TOP = (1u << (E + M)) - 1u, SIGN = 1u << (E + M);   // top exponent field 2^E - 1, mantissa all ones
    constexpr uint32_t OFFSET = (uint32_t)(127 - BIAS) << 15;
    const uint32_t a15 = (u >> 8) & 0x7FFFFFu;
    const uint32_t t = a15 > OFFSET ? a15 - OFFSET : 0u;
    const uint32_t q = t >> SH;                                               // (ye << M) | truncated mantissa
    const uint32_t v = (t + ((1u << (SH - 1)) - 1u) + (q & 1u)) >> SH;        // (ye << M) + rounded mantissa
    const uint32_t ef = q & ~((1u << M) - 1u);
    const uint32_t code_n = min(ef | (v - ef), TOP);   // a carry into an odd exponent field is lost; ye above the top field saturates
    const uint32_t code_s = ((min(v, 1u) << M) | v) >> 1;  // ye == 0: the mantissa under an explicit leading one
    const uint32_t mag = q < (1u << M) ? code_s : code_n;
    return mag | (u > 0x80000000u ? SIGN : 0u);
}

// ---------------------------------------------------------------------------------------
// Decode (minifloat/fake.py:97-123): 2^(xe - bias [+1 if subnormal]) * (xf / 2^M [+1]).
// ---------------------------------------------------------------------------------------
__device__ inline float pow2_f32(int e) {  // exp2 of an integer as fp32 evaluates it
    if (e > 127) return bits_f32(0x7F800000u);
    if (e >= -126) return bits_f32((uint32_t)(e + 127) << 23);
    if (e >= -149) return bits_f32(1u << (e + 149));
    return 0.0f;
}

template <class F>
__device__ inline float decode_f32(uint32_t code, const F& f) {
    const int E = f.E(), M = f.M();
    const uint32_t c = code & 0x7FFFu;
    const uint32_t xe = (c >> M) & ((1u << E) - 1u), xf = c & ((1u << M) - 1u);
    float y;
    if (F::kStatic && E <= 6) {
        // exponent field placed in the fp32 exponent field: value * 2^(bias - 127), exact
        // for subnormal codes too (they become fp32 subnormals); one multiply rescales
        y = bits_f32(((xe << M) | xf) << (23 - M)) * bits_f32((uint32_t)(254 - fmt_bias(f)) << 23);
    } else {
        const bool sub = xe == 0u;
        const float frac = (float)(xf + (sub ? 0u : (1u << M))) * bits_f32((uint32_t)(127 - M) << 23);
        y = (xe == 0u && xf == 0u) ? 0.0f : pow2_f32((int)xe - fmt_bias(f) + (sub ? 1 : 0)) * frac;
    }
    if (!f.finite() && xe == (1u << E) - 1u) y = xf == 0u ? bits_f32(0x7F800000u) : bits_f32(0x7FC00000u);
    return (code & fmt_sign(f)) ? -y : y;
}

// scale byte -> 2^(scale - 127) as fp32 (2^-127 is subnormal, 2^128 is +inf)
__device__ inline float scale_f32(uint32_t scale) {
    return bits_f32(scale == 0u ? 0x00400000u : scale << 23);
}

// ---------------------------------------------------------------------------------------
// MXFP shared exponent (mxfp/fake.py:44-50).
// ---------------------------------------------------------------------------------------
// floor(log2(a)) as fp32 evaluates it for a normal fp32 `a`: log2 is rounded to fp32 first, so
// the few largest floats below 2^k give exactly k.  For a correctly rounded log2 that band is
// floor(ln2 * 2^p) floats wide, p set by the float spacing around k.
__device__ inline int floor_log2_fp32(uint32_t a) {
    const int e = (int)(a >> 23) - 127, k = e + 1;
    const uint32_t f23 = a & 0x7FFFFFu;
    if (f23 < 0x800000u - 44u) return e;  // no band is wider than 44
    int idx;
    if (k == 0) idx = 0;
    else if (k > 0) idx = (k == 1) ? 0 : 32 - __clz(k - 1);  // ceil(log2 k)
    else idx = 32 - __clz(-k);                                 // floor(log2 -k) + 1
    // widths 0,0,1,2,5,11,22,44 packed one per byte
    const uint64_t widths = 0x2C160B0502010000ull;
    const uint32_t w = (uint32_t)(widths >> (8 * (idx > 7 ? 7 : idx))) & 0xFFu;
    return f23 >= 0x800000u - w ? k : e;
}

// Shared exponent se (unbiased, clamped) of a block whose largest |x| has bits amax.
// Returns 128 for blocks holding inf/NaN and for all-zero blocks (the reference's
// float->int32 cast of +-inf/NaN gives INT_MIN, which wraps and clamps to 128).
template <class F, bool HALF_PRECISION_INPUT>
__device__ inline int shared_exponent(uint32_t amax, const F& f) {
    if (amax >= 0x7F800000u || amax == 0u) return 128;
    const uint32_t ef = amax >> 23;
    int fl;
    if (ef == 0u) fl = -127;  // fp32-subnormal maximum: every element is flushed anyway
    else fl = HALF_PRECISION_INPUT ? (int)ef - 127 : floor_log2_fp32(amax);
    int se = fl - fmt_emax_unb(f);
    return se < -127 ? -127 : se;  // upper clamp (128) is unreachable for finite amax
}

// Code of one element x (fp32 bits u) of a block with shared exponent se: encode(x / 2^se),
// with the quotient formed exactly as an fp32 division would (mxfp/fake.py:52-57).
template <class F>
__device__ inline uint32_t encode_mxfp_element(uint32_t u, int se, const F& f) {
    const uint32_t a = u & 0x7FFFFFFFu, ef = a >> 23, f23 = a & 0x7FFFFFu;
    if (ef == 0u) return 0u;  // flushed input -> +0.0
    if (se == 128) {          // divisor is +inf
        if (ef != 255u) return 0u;  // finite / inf = +-0, and -0.0 < 0 is false
        return encode_nonfinite(false, true, f23, f);  // inf/inf and nan/inf are NaN
    }
    const bool neg = (u >> 31) != 0u;
    const int eq = (int)ef - 127 - se;
    if (eq >= -126) return encode_normal(neg, eq, f23, f);
    // fp32-subnormal quotient: flushed by the encoder, but a negative one keeps its sign
    // code unless the division already rounded it to zero
    const bool to_zero = eq < -150 || (eq == -150 && f23 == 0u);
    if (to_zero || !neg) return 0u;
    // the encoder sees either a subnormal (flushed) or, if rounding reached 2^-126, a value
    // below the range of every format with E <= 7: both give the sign-only code
    return fmt_sign(f);
}

}  // namespace mase
