/*
 * CPU checker for the MXFP / minifloat cast path.  TEST INFRASTRUCTURE ONLY.
 *
 * This file is a plain-C, integer-arithmetic restatement of the PyTorch "fake"
 * implementation of the reference (paths relative to the reference checkout):
 *
 *   orc_extract_minifloat   <- src/mase_triton/minifloat/fake.py:7-78
 *   orc_compose_minifloat   <- src/mase_triton/minifloat/fake.py:81-125
 *   orc_extract_mxfp        <- src/mase_triton/mxfp/fake.py:11-59
 *   orc_compose_mxfp        <- src/mase_triton/mxfp/fake.py:62-79
 *   orc_qdq_*               <- compose(extract(x)) as in
 *                              src/mase_triton/minifloat/functional/cast.py:72-90 and
 *                              src/mase_triton/mxfp/functional/cast.py:103-129
 *
 * It may be linked, loaded or run only by tests, by the smoke check and by the CPU-baseline
 * leg of the benchmark; the shipped GPU path never calls into it.
 *
 * Parity status: every function here is pinned against vectors written by the reference
 * itself (the .npz files under tests/golden) and against closed forms; see tests/test_oracle_golden.py.
 *
 * The reference computes with float tensor ops (frexp, log2, floor, exp2, division,
 * round-half-even).  Each is replaced by the integer operation that gives the same result
 * for every fp32 input on x86-64 PyTorch, including the cases where the reference's result
 * is an accident of the platform (float->int32 of inf/NaN = INT_MIN, int32 wrap-around,
 * inf/inf = NaN, frexp(inf|nan) exponent 0).
 */
#include <math.h>
#include <stdint.h>
#include <string.h>

enum { ORC_F32 = 0, ORC_F16 = 1, ORC_BF16 = 2 };
enum { ORC_RN = 0, ORC_RU = 1, ORC_RD = 2, ORC_RZ = 3 };

typedef struct {
    int E, M, finite, rmode;
    int bias, emax_field, emax_unb, fmax;
    uint32_t sign_code;
} fmt_t;

static fmt_t make_fmt(int E, int M, int finite, int rmode) {
    fmt_t f;
    f.E = E; f.M = M; f.finite = finite; f.rmode = rmode;
    f.bias = (1 << (E - 1)) - 1;                                /* fake.py:13 */
    f.emax_field = finite ? (1 << E) - 1 : (1 << E) - 2;        /* fake.py:15 */
    f.emax_unb = f.emax_field - f.bias;                         /* fake.py:16 */
    f.fmax = (1 << M) - 1;                                      /* fake.py:19 */
    f.sign_code = 1u << (E + M);                                /* fake.py:76 */
    return f;
}

/* ---------------------------------------------------------------- dtype helpers */
static uint32_t f16_to_f32_bits(uint16_t h) {
    uint32_t s = (uint32_t)(h & 0x8000u) << 16;
    uint32_t e = (h >> 10) & 0x1Fu, m = h & 0x3FFu;
    if (e == 0) {
        if (m == 0) return s;
        int sh = 0;
        while (!(m & 0x400u)) { m <<= 1; ++sh; }
        m &= 0x3FFu;
        return s | ((uint32_t)(127 - 15 - sh + 1) << 23) | (m << 13);
    }
    if (e == 31) return s | 0x7F800000u | (m << 13);
    return s | ((e + 112u) << 23) | (m << 13);
}

static uint32_t load_as_f32_bits(const void *x, int dtype, int64_t i) {
    switch (dtype) {
    case ORC_F32: return ((const uint32_t *)x)[i];
    case ORC_BF16: return (uint32_t)((const uint16_t *)x)[i] << 16;
    default: return f16_to_f32_bits(((const uint16_t *)x)[i]);
    }
}

static uint16_t f32_bits_to_bf16(uint32_t u) {      /* round-to-nearest-even, NaN -> 0x7FC0 */
    if ((u & 0x7FFFFFFFu) > 0x7F800000u) return 0x7FC0;
    return (uint16_t)((u + 0x7FFFu + ((u >> 16) & 1u)) >> 16);
}

static uint16_t f32_bits_to_f16(uint32_t u) {       /* IEEE round-to-nearest-even */
    uint32_t s = (u >> 16) & 0x8000u, a = u & 0x7FFFFFFFu;
    if (a > 0x7F800000u) return (uint16_t)(s | 0x7E00u);
    if (a >= 0x47800000u) return (uint16_t)(s | 0x7C00u);          /* >= 65536 -> inf   */
    if (a >= 0x38800000u) {                                          /* normal fp16       */
        uint32_t r = a - 0x38000000u;                                /* rebias 127 -> 15  */
        r = r + 0xFFFu + ((r >> 13) & 1u);
        return (uint16_t)(s | (r >> 13));                            /* carry may give inf */
    }
    if (a < 0x33000000u) return (uint16_t)s;                         /* < 2^-25 -> 0      */
    {
        uint32_t e = a >> 23, m = (a & 0x7FFFFFu) | 0x800000u;
        int sh = (int)(113 - e) + 13;                                /* 14..24            */
        uint32_t q = m >> sh, rem = m & ((1u << sh) - 1u), half = 1u << (sh - 1);
        if (rem > half || (rem == half && (q & 1u))) ++q;
        return (uint16_t)(s | q);
    }
}

static void store_from_f32(void *out, int dtype, int64_t i, float v) {
    uint32_t u;
    memcpy(&u, &v, 4);
    switch (dtype) {
    case ORC_F32: ((uint32_t *)out)[i] = u; break;
    case ORC_BF16: ((uint16_t *)out)[i] = f32_bits_to_bf16(u); break;
    default: ((uint16_t *)out)[i] = f32_bits_to_f16(u); break;
    }
}

/* ---------------------------------------------------------------- minifloat extract */
/* fake.py:41-56: mantissa -> frac_bits.  Every mode but "rz" first drops the low 8 bits. */
static uint32_t round_mantissa(uint32_t f23, const fmt_t *f) {
    if (f->rmode == ORC_RZ) return f23 >> (23 - f->M);
    uint32_t f15 = f23 >> 8;
    int sh = 15 - f->M;
    uint32_t q = f15 >> sh, r = f15 & ((1u << sh) - 1u), half = 1u << (sh - 1);
    switch (f->rmode) {
    case ORC_RU: return q + (r != 0);
    case ORC_RD: return q;
    default: return q + ((r > half) || (r == half && (q & 1u)));   /* torch.round = half-even */
    }
}

/* Code for one fp32 value given as bits (fake.py:21-77). */
static uint16_t encode_f32_bits(uint32_t u, const fmt_t *f) {
    uint32_t a = u & 0x7FFFFFFFu;
    int is_nan = a > 0x7F800000u, is_inf = a == 0x7F800000u;
    int neg = (u >> 31) && a != 0 && !is_nan;                        /* x < 0        :22 */
    uint32_t ef = a >> 23, f23 = a & 0x7FFFFFu;
    int ftz = ef == 0;                                               /*              :24 */
    int e;
    if (ef == 255) { e = -1; if (is_nan) f23 |= 0x400000u; }         /* frexp(inf|nan): exponent 0 -> -1 */
    else if (ftz) { e = -1; f23 = 0; }                               /* frexp(0) = (0,0) */
    else e = (int)ef - 127;
    int underflow = e < -f->bias, overflow = e > f->emax_unb;        /*           :35-36 */
    int32_t ye = e + f->bias;
    uint32_t yf = round_mantissa(f23, f);
    if (ye == 0 && yf != 0) yf = (yf | (1u << f->M)) >> 1;           /*           :58-60 */
    if (underflow) { yf = 0; ye = 0; }
    if (overflow) { yf = (uint32_t)f->fmax; ye = f->emax_field; }
    if (ftz) { yf = 0; ye = 0; }
    if (!f->finite) {                                                /*           :70-74 */
        if (is_inf) { yf = 0; ye = f->emax_field; }
        if (is_nan) { yf = (uint32_t)f->fmax; ye = f->emax_field; }
    }
    uint32_t y = ((uint32_t)ye << f->M) | yf;                        /* OR, not add  :75 */
    if (neg) y += f->sign_code;
    return (uint16_t)y;
}

void orc_extract_minifloat(const void *x, int x_dtype, uint16_t *codes, int64_t n,
                           int E, int M, int finite, int rmode) {
    fmt_t f = make_fmt(E, M, finite, rmode);
#pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < n; ++i)
        codes[i] = encode_f32_bits(load_as_f32_bits(x, x_dtype, i), &f);
}

/* ---------------------------------------------------------------- minifloat compose */
static float pow2f_like_torch(int e) {          /* torch.exp2(int32) evaluated in fp32 */
    if (e > 127) return INFINITY;
    if (e < -149) return 0.0f;
    return ldexpf(1.0f, e);
}

static float decode_to_f32(uint32_t code, const fmt_t *f) {          /* fake.py:97-123 */
    uint32_t sign = code & f->sign_code;
    uint32_t c = code & 0x7FFFu;
    uint32_t xe = (c >> f->M) & ((1u << f->E) - 1u), xf = c & ((1u << f->M) - 1u);
    int sub = xe == 0 && xf != 0, zero = xe == 0 && xf == 0;
    int ye = (int)xe - f->bias + (sub ? 1 : 0);
    float frac = (float)xf / (float)(1u << f->M);
    if (!sub) frac += 1.0f;
    float y = pow2f_like_torch(ye) * frac;
    if (!f->finite && xe == (1u << f->E) - 1u) y = xf == 0 ? INFINITY : NAN;
    if (zero) y = 0.0f;
    if (sign) y = -y;
    return y;
}

void orc_compose_minifloat(const uint16_t *codes, void *out, int out_dtype, int64_t n,
                           int E, int M, int finite) {
    fmt_t f = make_fmt(E, M, finite, ORC_RN);
#pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < n; ++i) store_from_f32(out, out_dtype, i, decode_to_f32(codes[i], &f));
}

void orc_qdq_minifloat(const void *x, int x_dtype, void *out, int out_dtype, int64_t n,
                       int E, int M, int finite, int rmode) {
    fmt_t f = make_fmt(E, M, finite, rmode);
#pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < n; ++i) {
        uint16_t c = encode_f32_bits(load_as_f32_bits(x, x_dtype, i), &f);
        store_from_f32(out, out_dtype, i, decode_to_f32(c, &f));
    }
}

/* ---------------------------------------------------------------- MXFP extract */
/* floor(log2(a)) as torch evaluates it in fp32 for a normal fp32 `a` (mxfp/fake.py:45).
 * log2 is rounded to fp32 before the floor, so the largest few floats below 2^k come out
 * as exactly k.  With a correctly rounded log2 the count is floor(ln2 * 2^p) where 2^p is
 * half the spacing of the floats next to k, in units of 2^-24. */
static int floor_log2_fp32(uint32_t a) {
    static const int band[8] = {0, 0, 1, 2, 5, 11, 22, 44};
    int e = (int)(a >> 23) - 127;
    uint32_t f23 = a & 0x7FFFFFu;
    int k = e + 1, idx;
    if (k == 0) idx = 0;
    else if (k > 0) { idx = 0; while ((1 << idx) < k) ++idx; }       /* ceil(log2 k)      */
    else { int m = -k; idx = 0; while ((2 << idx) <= m) ++idx; ++idx; } /* floor(log2 m)+1 */
    if (idx > 7) idx = 7;
    return (f23 >= 0x800000u - (uint32_t)band[idx]) ? k : e;
}

static void extract_block(const void *x, int x_dtype, int64_t base, int B, const fmt_t *f,
                          uint8_t *scale_out, uint8_t *el_out) {
    uint32_t amax = 0;
    int all_flushed = 1;
    for (int j = 0; j < B; ++j) {
        uint32_t a = load_as_f32_bits(x, x_dtype, base + j) & 0x7FFFFFFFu;
        if (a > amax) amax = a;                 /* NaN bit patterns sort above inf: max propagates */
        if (a >> 23) all_flushed = 0;
    }
    int special = amax >= 0x7F800000u || amax == 0;   /* log2 -> +-inf/NaN -> int32 INT_MIN */
    int se;
    if (special) se = 128;                             /* INT_MIN - emax wraps positive, clamps to 128 */
    else {
        int fl = (amax >> 23) ? floor_log2_fp32(amax) : -127 /* subnormal: anything <= -127 */;
        se = fl - f->emax_unb;                         /* mxfp/fake.py:46 */
        if (se < -127) se = -127;
        if (se > 128) se = 128;                        /* :47 */
    }
    *scale_out = all_flushed ? 0 : (uint8_t)(se + 127); /* :48-50 */

    for (int j = 0; j < B; ++j) {
        uint32_t u = load_as_f32_bits(x, x_dtype, base + j);
        uint32_t a = u & 0x7FFFFFFFu, ef = a >> 23, f23 = a & 0x7FFFFFu;
        uint32_t q;                                    /* bits of x / 2^se (:52-54) */
        if (ef == 0) q = 0;                            /* flushed input -> +0.0 */
        else if (se == 128) {                          /* divide by +inf */
            if (ef == 255) q = 0x7FC00000u | f23;      /* inf/inf, nan/inf: quiet NaN, sign dropped later */
            else q = u & 0x80000000u;                  /* finite/inf = +-0 */
        } else {
            int eq = (int)ef - 127 - se;
            if (ef == 255) q = u;                      /* cannot happen: special blocks have se=128 */
            else if (eq >= -126) q = (u & 0x80000000u) | ((uint32_t)(eq + 127) << 23) | f23;
            else {                                     /* quotient is an fp32 subnormal: RNE */
                int sh = -126 - eq;                    /* >= 1 */
                uint32_t m = f23 | 0x800000u, r;
                if (sh > 24) r = 0;
                else {
                    uint32_t keep = m >> sh, rem = m & ((1u << sh) - 1u), half = 1u << (sh - 1);
                    r = keep + ((rem > half) || (rem == half && (keep & 1u)));
                }
                q = (u & 0x80000000u) | r;             /* r may be 0x800000 = smallest normal */
            }
        }
        el_out[j] = (uint8_t)encode_f32_bits(q, f);    /* :55-57 */
    }
}

void orc_extract_mxfp(const void *x, int x_dtype, uint8_t *scales, uint8_t *elements,
                      int64_t n, int B, int E, int M, int finite, int rmode) {
    fmt_t f = make_fmt(E, M, finite, rmode);
    int64_t nb = n / B;
#pragma omp parallel for schedule(static)
    for (int64_t b = 0; b < nb; ++b)
        extract_block(x, x_dtype, b * B, B, &f, scales + b, elements + b * B);
}

/* ---------------------------------------------------------------- MXFP compose */
static float mxfp_value(uint8_t scale, uint8_t code, const fmt_t *f) {   /* mxfp/fake.py:71-77 */
    float s = pow2f_like_torch((int)scale - 127);
    return decode_to_f32(code, f) * s;
}

void orc_compose_mxfp(const uint8_t *scales, const uint8_t *elements, void *out, int out_dtype,
                      int64_t n, int B, int E, int M, int finite) {
    fmt_t f = make_fmt(E, M, finite, ORC_RN);
#pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < n; ++i)
        store_from_f32(out, out_dtype, i, mxfp_value(scales[i / B], elements[i], &f));
}

void orc_qdq_mxfp(const void *x, int x_dtype, void *out, int out_dtype, int64_t n, int B,
                  int E, int M, int finite, int rmode) {
    fmt_t f = make_fmt(E, M, finite, rmode);
    int64_t nb = n / B;
#pragma omp parallel for schedule(static)
    for (int64_t b = 0; b < nb; ++b) {
        uint8_t sc, el[1024];
        uint8_t *e = el;
        uint8_t heap_needed = B > 1024;
        if (heap_needed) continue;                     /* block sizes above 1024 are not used */
        extract_block(x, x_dtype, b * B, B, &f, &sc, e);
        for (int j = 0; j < B; ++j)
            store_from_f32(out, out_dtype, b * B + j, mxfp_value(sc, e[j], &f));
    }
}

/* ---------------------------------------------------------------- dequantize-then-matmul
 * y[m,n] = bf16( sum_k xq[m,k] * wq[n,k] ) with fp32 accumulation over dequantised operands,
 * the "separate" backend of src/mase_triton/mxfp/functional/linear.py:36-64 (torch's GEMM
 * accumulates bf16 products in fp32; summation order is unspecified there, so this result
 * is a reference only up to reassociation).  Inputs are dequantised fp32 arrays. */
void orc_matmul_nt_f32(const float *a, const float *b, float *c, int64_t Mrows, int64_t N,
                       int64_t K) {
#pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < Mrows; ++i)
        for (int64_t j = 0; j < N; ++j) {
            double acc = 0.0;
            for (int64_t k = 0; k < K; ++k) acc += (double)a[i * K + k] * (double)b[j * K + k];
            c[i * N + j] = (float)acc;
        }
}
