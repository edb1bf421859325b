// Fast formulation of NVFP4 round-to-nearest quantisation of one 1x16 block for gfx950.
//
// Bit-identical to the operation-by-operation form in fos_quantize_common.h, but built
// from cheaper exact steps:
//  * E4M3 scale encode = v_cvt_pk_fp8_f32 (same rounding as torch's float8_e4m3fn cast,
//    checked exhaustively on the device against the integer formulation);
//  * E2M1 rounding + nibble packing = v_cvt_scalef32_pk_fp4_f32 with scale 1 (round to
//    nearest even onto {0,.5,1,1.5,2,3,4,6}, sign kept, saturating at 6).  The reference
//    does not saturate (a magnitude in [7,9) becomes 8); that needs a block scale that is
//    sub-normal in E4M3, so blocks with such a scale take the operation-by-operation path;
//  * everything that depends only on the scale byte -- 1/(dec*s), and the dequantisation
//    factors of the selection error -- comes from a 128-entry table in LDS built once per
//    workgroup with the reference's own operations;
//  * bmax / 6 is a 3-instruction correctly rounded division by a constant (q0 = x*r,
//    q = fma(fma(-6,q0,x), r, q0); exhaustively equal to IEEE division for normal results);
//  * the candidate's dequantised value RN(RN(fq*s*amax)/1536): fq*s*amax is exact (2+4+8
//    significant bits), so it is RN(fq*g/1536) with g = s*amax.  For fq in {.5,1,2,4} that
//    is fq*RN(g/1536); for fq in {1.5,3,6} it is (fq/1.5)*(g/1024), exact.  Either way it is
//    (power of two) x (table value), so deq - x is ONE fma with the reference's rounding.
// The error terms d*d (or |d|) and their summation order are unchanged.
//
// A negative zero in the input must encode as +0 (the reference multiplies by sign(x),
// and sign(-0) = 0) while a small negative value that rounds to zero keeps its sign; the
// hardware convert keeps the sign in both cases, so when pass 1 saw a -0.0 anywhere the
// block values are first canonicalised with x + 0.
#pragma once

#include <type_traits>

#include "fos_quantize_common.h"

namespace fos {

typedef float float2_t __attribute__((ext_vector_type(2)));

// Compile-time loop: f(std::integral_constant<int, I>) for I = 0 .. N-1 (the convert
// builtins take their byte selector as an immediate).
template <int I, int N, class F>
FOS_DEVICE void static_for(F &&f) {
    if constexpr (I < N) {
        f(std::integral_constant<int, I>{});
        static_for<I + 1, N>(f);
    }
}

// Two floats -> two E2M1 nibbles (a low, b high) into byte SEL of `old`.
template <int SEL>
FOS_DEVICE uint32_t pack_fp4(uint32_t old, float a, float b) {
    return __builtin_amdgcn_cvt_scalef32_pk_fp4_f32(old, a, b, 1.0f, SEL);
}

// Byte SEL of `word` -> the two E2M1 values (low nibble in .x).
template <int SEL>
FOS_DEVICE float2_t unpack_fp4(uint32_t word) {
    return __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(word, 1.0f, SEL);
}

struct FastLutEntry {
    float inv;       // 1 / (dec * s)                       (0 for s == 0)
    float d1;        // RN((s * amax) / errdiv)             factor for fq in {.5, 1, 2, 4}
    uint32_t delta;  // bits((s * amax) / 1024) - bits(d1)  added for fq in {1.5, 3, 6}
    uint32_t pad;
};

// Entry for scale byte `s` (0..127); built with the reference's operations.
FOS_DEVICE FastLutEntry make_lut_entry(uint32_t s, const QuantConsts &k) {
    FastLutEntry e;
    const float sf = e4m3_decode(s);
    e.inv = s == 0 ? 0.0f : 1.0f / (k.dec * sf);
    const float g = sf * k.amax;
    e.d1 = g / k.errdiv;
    e.delta = f2u(g * 0x1p-10f) - f2u(e.d1);  // errdiv is 1536 = 1.5 * 2^10 on this path
    e.pad = 0;
    return e;
}

// x / y for a constant y with r = RN(1/y); equals IEEE division whenever the quotient is
// a normal number.
FOS_DEVICE float div_const(float x, float y, float r) {
    const float q0 = x * r;
    return __builtin_fmaf(__builtin_fmaf(-y, q0, x), r, q0);
}

// deq - x for one decoded candidate value fq (on the E2M1 grid).
FOS_DEVICE float candidate_residual(float fq, const FastLutEntry &e, float x) {
    const uint32_t fb = f2u(fq);
    const float p2 = u2f(fb & 0xffbfffffu);                    // 1.5 * 2^j -> 2^j
    const uint32_t three = (fb >> 22) & 1u;                    // fq in {1.5, 3, 6}
    const float mult = u2f(__umul24(three, e.delta) + f2u(e.d1));
    return __builtin_fmaf(p2, mult, -x);
}

// One 1x16 block on the fast path.  Returns false when the block must be redone by the
// operation-by-operation path (sub-normal block scale).  `rq` = RN(1 / qdiv).
template <int RULE, bool TWO_D>
FOS_DEVICE bool quantize_block_fast(const uint32_t *w, const QuantConsts &k, float enc, float rq, bool canon,
                                    const FastLutEntry *lut, uint32_t *codes, uint32_t &sbyte) {
    constexpr bool STATIC = (RULE == FOS_RULE_STATIC_6 || RULE == FOS_RULE_STATIC_4);
    float x[16];
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        x[2 * i] = u2f(w[i] << 16);
        x[2 * i + 1] = u2f(w[i] & 0xffff0000u);
    }
    if (canon) {
#pragma unroll
        for (int i = 0; i < 16; ++i) x[i] = x[i] + 0.0f;
    }
    float bmax = 0.0f;
#pragma unroll
    for (int i = 0; i < 16; i += 2) bmax = fmaxf(fmaxf(fabsf(x[i]), fabsf(x[i + 1])), bmax);
    if (TWO_D) bmax = row16_max(bmax);

    const float s_hp6 = div_const(bmax, k.qdiv, rq) * enc;
    const float s_hp4 = s_hp6 * 1.5f;
    const uint32_t pk = (uint32_t)__builtin_amdgcn_cvt_pk_fp8_f32(s_hp6, s_hp4, 0, false);
    const uint32_t s6 = pk & 0xffu, s4 = (pk >> 8) & 0xffu;
    if (s6 < 8u) {
        if (bmax == 0.0f) {  // an all-zero block: zero codes, zero scale
            codes[0] = 0;
            codes[1] = 0;
            sbyte = 0;
            return true;
        }
        return false;
    }

    const FastLutEntry A = lut[s6];
    if (STATIC) {
        uint32_t c0 = 0, c1 = 0;
        static_for<0, 4>([&](auto jc) {
            constexpr int j = decltype(jc)::value;
            c0 = pack_fp4<j>(c0, x[2 * j] * A.inv, x[2 * j + 1] * A.inv);
            c1 = pack_fp4<j>(c1, x[8 + 2 * j] * A.inv, x[9 + 2 * j] * A.inv);
        });
        codes[0] = c0;
        codes[1] = c1;
        sbyte = s6;
        return true;
    }

    const FastLutEntry B = lut[s4];
    uint32_t a0 = 0, a1 = 0, b0 = 0, b1 = 0;
    static_for<0, 4>([&](auto jc) {
        constexpr int j = decltype(jc)::value;
        a0 = pack_fp4<j>(a0, x[2 * j] * A.inv, x[2 * j + 1] * A.inv);
        a1 = pack_fp4<j>(a1, x[8 + 2 * j] * A.inv, x[9 + 2 * j] * A.inv);
        b0 = pack_fp4<j>(b0, x[2 * j] * B.inv, x[2 * j + 1] * B.inv);
        b1 = pack_fp4<j>(b1, x[8 + 2 * j] * B.inv, x[9 + 2 * j] * B.inv);
    });
    float eA[16], eB[16];
    static_for<0, 8>([&](auto jc) {
        constexpr int j = decltype(jc)::value;
        const float2_t fa = unpack_fp4<(j & 3)>(j < 4 ? a0 : a1);
        const float2_t fb = unpack_fp4<(j & 3)>(j < 4 ? b0 : b1);
        const float dA0 = candidate_residual(fa.x, A, x[2 * j]), dA1 = candidate_residual(fa.y, A, x[2 * j + 1]);
        const float dB0 = candidate_residual(fb.x, B, x[2 * j]), dB1 = candidate_residual(fb.y, B, x[2 * j + 1]);
        eA[2 * j] = RULE == FOS_RULE_MSE ? dA0 * dA0 : fabsf(dA0);
        eA[2 * j + 1] = RULE == FOS_RULE_MSE ? dA1 * dA1 : fabsf(dA1);
        eB[2 * j] = RULE == FOS_RULE_MSE ? dB0 * dB0 : fabsf(dB0);
        eB[2 * j + 1] = RULE == FOS_RULE_MSE ? dB1 * dB1 : fabsf(dB1);
    });
    const float errA = reduce_error<RULE, TWO_D>(eA);
    const float errB = reduce_error<RULE, TWO_D>(eB);
    const bool pickB = errB < errA;
    codes[0] = pickB ? b0 : a0;
    codes[1] = pickB ? b1 : a1;
    sbyte = pickB ? s4 : s6;
    return true;
}

}  // namespace fos
