// silu(gate) * up on packed bf16 pairs, in registers: the arithmetic of the operand kernel that quantises the input of a
// SwiGLU block's down projection (cast_kernels.hip).  Also built into the test helper library on its own, so that a test
// can put every bf16 gate value through it.
#pragma once
#include "mxfp_compose.h"

namespace mase {

// SiLU g / (1 + exp(-g)) of a gate with |g| < 87.5, from the hardware's exp2 and reciprocal: 14 instruction slots
// (a wavefront's VALU instruction takes four cycles, the two transcendental ones sixteen) where the library's exp and
// IEEE division take about 45, and a kernel that streams two bf16 inputs per element has about 30 slots per element before
// arithmetic, not memory, bounds it.  Both instructions are accurate to an ulp; one Newton step on the quotient
// (residual g - q d in one fma) takes the reciprocal's error out again, the sign comes from g (the step turns -0 into
// +0).  The gate is bfloat16 and the result is rounded to bfloat16, so there are 65536 cases: measured over all of them,
// the rounded result is the library expression's (and the correctly rounded one) every time; without the Newton step one
// gate, 5.9375, whose SiLU lies 4e-7 below the midpoint of two bfloat16 values, rounds the other way
// (tests/test_gpu_scaled_gemm.py goes through all gates).
__device__ inline float silu_small(float g) {
    const float d = 1.0f + __builtin_amdgcn_exp2f(g * -1.44269504088896340736f);
    const float rc = __builtin_amdgcn_rcpf(d);
    const float q = g * rc;
    return __builtin_copysignf(__builtin_fmaf(__builtin_fmaf(-q, d, g), rc, q), g);
}

// bf16 bit pattern, sign dropped, from which a gate takes the plain expression instead: |g| >= 87.5, where exp(-g)
// reaches 2^126 for negative g and the reciprocal would be subnormal (flushed by the hardware), inf and NaN (positive
// gates that large would be right either way: the test looks at magnitudes only)
constexpr uint32_t SILU_PLAIN_FROM = 0x42AFu;

// does any of the eight gates of a 128-bit word need the plain expression?
__device__ inline bool swiglu_any_plain(const uint4& g) {
    typedef unsigned short ushort2_t __attribute__((ext_vector_type(2)));
    const uint32_t w[4] = {g.x, g.y, g.z, g.w};
    ushort2_t m = {0, 0};
#pragma unroll
    for (int j = 0; j < 4; ++j) m = __builtin_elementwise_max(m, __builtin_bit_cast(ushort2_t, w[j] & 0x7FFF7FFFu));
    return m[0] >= SILU_PLAIN_FROM || m[1] >= SILU_PLAIN_FROM;
}

// two gates g2 and two ups u2 (bf16 pairs) -> bf16 pair of silu(g) * u, rounded where two separate bf16 tensor
// operations round: the SiLU (evaluated in fp32) to bf16, then the product (fp32) to bf16.  PLAIN: the library expression,
// for words that hold a gate beyond SILU_PLAIN_FROM (the caller tests a whole word, wave-uniformly).
template <bool PLAIN>
__device__ inline uint32_t swiglu_pair(uint32_t g2, uint32_t u2) {
    const float g0 = bits_f32(g2 << 16), g1 = bits_f32(g2 & 0xFFFF0000u);
    const uint32_t s2 = PLAIN ? cvt_pk_bf16(g0 / (1.0f + expf(-g0)), g1 / (1.0f + expf(-g1))) : cvt_pk_bf16(silu_small(g0), silu_small(g1));
    return cvt_pk_bf16(bits_f32(s2 << 16) * bits_f32(u2 << 16), bits_f32(s2 & 0xFFFF0000u) * bits_f32(u2 & 0xFFFF0000u));
}

// eight elements at once; the rare plain route behind one wave-uniform branch
__device__ inline uint4 swiglu_x8(const uint4& g, const uint4& u) {
    uint4 h = make_uint4(swiglu_pair<false>(g.x, u.x), swiglu_pair<false>(g.y, u.y), swiglu_pair<false>(g.z, u.z), swiglu_pair<false>(g.w, u.w));
    const bool plain = swiglu_any_plain(g);
    if (__builtin_amdgcn_ballot_w64(plain) != 0 && plain)
        h = make_uint4(swiglu_pair<true>(g.x, u.x), swiglu_pair<true>(g.y, u.y), swiglu_pair<true>(g.z, u.z), swiglu_pair<true>(g.w, u.w));
    return h;
}

}  // namespace mase
