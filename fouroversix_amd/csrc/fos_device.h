// Device-side helpers shared by the gfx950 quantize, dequantize and GEMM kernels.
//
// Everything here is fp32 with one IEEE rounding per written operation: the library is
// compiled with -ffp-contract=off, correctly rounded division, fp32 denormals enabled,
// and fused multiply-adds appear only where __builtin_fmaf is spelled out.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include <type_traits>

#define FOS_DEVICE __device__ __forceinline__

namespace fos {

FOS_DEVICE float u2f(uint32_t u) { return __uint_as_float(u); }
FOS_DEVICE uint32_t f2u(float f) { return __float_as_uint(f); }

// ---- E4M3 (float8_e4m3fn) block scales ---------------------------------------------

// Bits 0..6 of an E4M3 byte -> float.  The byte placed at bit 20 is a float whose
// exponent/mantissa fields are those of the E4M3 value with bias 127 instead of 7
// (a float denormal when the E4M3 value is sub-normal); 2^120 rebiases both cases exactly.
FOS_DEVICE float e4m3_decode(uint32_t b7) { return u2f(b7 << 20) * 0x1p120f; }

// Non-negative finite float -> E4M3 byte, round to nearest even; 2^-10 -> 0, 464 -> 448,
// anything larger rounds into the NaN pattern 0x7F (no saturation), as torch's cast does.
FOS_DEVICE uint32_t e4m3_encode(float f) {
    uint32_t u = f2u(f);
    if (u >= 0x43f00000u) return 0x7fu;
    if (u < 0x3c800000u) return (uint32_t)__builtin_rintf(f * 512.0f);
    u += 0x7ffffu + ((u >> 20) & 1u);
    return (u >> 20) - (120u << 3);
}

// ---- cross-lane moves inside a row of 16 lanes (DPP) --------------------------------

constexpr int kDppRowShl = 0x100;  // + n: lane i reads lane i + n
constexpr int kDppRowShr = 0x110;  // + n: lane i reads lane i - n
constexpr int kDppRowRor = 0x120;  // + n: lane i reads lane (i - n) mod 16

// Lanes whose source lies outside the row keep `old`.
template <int CTRL>
FOS_DEVICE float dpp_move(float old, float v) {
    return __int_as_float(__builtin_amdgcn_update_dpp(__float_as_int(old), __float_as_int(v),
                                                     CTRL, 0xf, 0xf, false));
}

// max over the 16 lanes of a DPP row, result in every lane.
FOS_DEVICE float row16_max(float v) {
    v = fmaxf(v, dpp_move<kDppRowRor + 8>(v, v));
    v = fmaxf(v, dpp_move<kDppRowRor + 4>(v, v));
    v = fmaxf(v, dpp_move<kDppRowRor + 2>(v, v));
    v = fmaxf(v, dpp_move<kDppRowRor + 1>(v, v));
    return v;
}

// ---- Philox4x32-10 ------------------------------------------------------------------

struct Philox4 { uint32_t v[4]; };

FOS_DEVICE Philox4 philox4x32_10(uint32_t c0, uint32_t c1, uint32_t c2, uint32_t c3,
                                 uint32_t k0, uint32_t k1) {
#pragma unroll
    for (int r = 0; r < 10; ++r) {
        uint32_t hi0 = __umulhi(0xD2511F53u, c0), lo0 = 0xD2511F53u * c0;
        uint32_t hi1 = __umulhi(0xCD9E8D57u, c2), lo1 = 0xCD9E8D57u * c2;
        uint32_t n0 = hi1 ^ c1 ^ k0, n2 = hi0 ^ c3 ^ k1;
        c0 = n0; c1 = lo1; c2 = n2; c3 = lo0;
        k0 += 0x9E3779B9u;
        k1 += 0xBB67AE85u;
    }
    return Philox4{{c0, c1, c2, c3}};
}

// Dither of element i (0..3) of a Philox word: (byte + 0.5) / 256 - 0.5, 256 equally likely
// values symmetric about zero (the INT4 candidate of IF4).
FOS_DEVICE float dither_from_byte(uint32_t w, int i) {
    return __builtin_fmaf((float)((w >> (8 * i)) & 0xffu), 0x1p-8f, -0.498046875f);
}

// ---- E2M1 converts --------------------------------------------------------------------

typedef float float2_t __attribute__((ext_vector_type(2)));

// Compile-time loop: f(std::integral_constant<int, I>) for I = 0 .. N-1 (the convert
// instructions take their byte selector as an immediate).
template <int I, int N, class F>
FOS_DEVICE void static_for(F &&f) {
    if constexpr (I < N) {
        f(std::integral_constant<int, I>{});
        static_for<I + 1, N>(f);
    }
}

// Two floats -> two E2M1 nibbles (a low, b high) into byte SEL of `old`: round to nearest
// even onto {0,.5,1,1.5,2,3,4,6}, sign kept, saturating at 6.
template <int SEL>
FOS_DEVICE uint32_t pack_fp4(uint32_t old, float a, float b) {
    return __builtin_amdgcn_cvt_scalef32_pk_fp4_f32(old, a, b, 1.0f, SEL);
}

// Byte SEL of `word` -> the two E2M1 values (low nibble in .x).
template <int SEL>
FOS_DEVICE float2_t unpack_fp4(uint32_t word) {
    return __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(word, 1.0f, SEL);
}

// Stochastic rounding of a pair of floats to E2M1 with V_CVT_SCALEF32_SR_PK_FP4_F32: the
// codes land in byte SEL of `acc` (v.x low nibble; other bytes kept).  The instruction
// adds 22 bits of `rword` -- bits 31..10 for v.x, bits 30..9 for v.y -- to the discarded
// mantissa bits, aligned to their top, and truncates: with the significand
// M = 1.m * 2^23 (0.m * 2^23 for a sub-normal float) and d discarded bits -- 22 for
// |x| >= 1, 22 - exponent below -- q = (M + (R << (d - 22))) >> d counts half-steps of the
// value's binade (of 1 below 1.0); the result saturates at 6 and keeps the sign, also on
// zero.  Measured on gfx950 against this statement (2^21 random and boundary inputs per
// slot, exact thresholds for single-bit and patterned random words).  The two slots'
// dithers are one bit apart, so a call yields one usable code: the caller gives each
// element a word of its own and masks the other slot out.  Written as inline assembly
// because the compiler's builtin does not tie the accumulator to the destination register;
// the s_nop is the wait state this convert needs before a VALU instruction may read its
// partially written destination (the compiler adds it for its own converts only).
template <int SEL>
FOS_DEVICE uint32_t sr_fp4_pair_into_byte(uint32_t acc, float2_t v, uint32_t rword) {
    if constexpr (SEL == 0) asm("v_cvt_scalef32_sr_pk_fp4_f32 %0, %1, %2, 1.0\n\ts_nop 0" : "+v"(acc) : "v"(v), "v"(rword));
    if constexpr (SEL == 1) asm("v_cvt_scalef32_sr_pk_fp4_f32 %0, %1, %2, 1.0 op_sel:[0,0,1,0]\n\ts_nop 0" : "+v"(acc) : "v"(v), "v"(rword));
    if constexpr (SEL == 2) asm("v_cvt_scalef32_sr_pk_fp4_f32 %0, %1, %2, 1.0 op_sel:[0,0,0,1]\n\ts_nop 0" : "+v"(acc) : "v"(v), "v"(rword));
    if constexpr (SEL == 3) asm("v_cvt_scalef32_sr_pk_fp4_f32 %0, %1, %2, 1.0 op_sel:[0,0,1,1]\n\ts_nop 0" : "+v"(acc) : "v"(v), "v"(rword));
    return acc;
}

// 16 scaled values -> 16 stochastically rounded E2M1 codes (element i in nibble i % 8 of
// c0 / c1).  Element i takes word i / 4 of the Philox output rotated so that byte i % 4
// leads; its dither is bits 31..10 (even i) or 30..9 (odd i) of that rotation.  Each pair
// is converted twice, once per element's word, and the valid nibbles are merged.
FOS_DEVICE void sr_pack16(const float *xs, const Philox4 &p, uint32_t &c0, uint32_t &c1) {
    uint32_t even[2] = {0u, 0u}, odd[2] = {0u, 0u};
    static_for<0, 8>([&](auto jc) {
        constexpr int pr = decltype(jc)::value, sel = pr & 3, half = pr >> 2;
        const float2_t v = {xs[2 * pr], xs[2 * pr + 1]};
        const uint32_t w = p.v[pr >> 1];
        // bytes 2 (pr % 2) and 2 (pr % 2) + 1 of the word lead for the even and the odd element
        const uint32_t r_even = __builtin_amdgcn_alignbit(w, w, (pr & 1) ? 24 : 8);
        const uint32_t r_odd = (pr & 1) ? w : __builtin_amdgcn_alignbit(w, w, 16);
        even[half] = sr_fp4_pair_into_byte<sel>(even[half], v, r_even);
        odd[half] = sr_fp4_pair_into_byte<sel>(odd[half], v, r_odd);
    });
    // low nibbles from `even`, high nibbles from `odd`
    c0 = (even[0] & 0x0f0f0f0fu) | (odd[0] & 0xf0f0f0f0u);
    c1 = (even[1] & 0x0f0f0f0fu) | (odd[1] & 0xf0f0f0f0u);
}

// The 16 values of two code words.
FOS_DEVICE void unpack16_fp4(uint32_t c0, uint32_t c1, float *v) {
    static_for<0, 8>([&](auto jc) {
        constexpr int j = decltype(jc)::value;
        const float2_t f = unpack_fp4<(j & 3)>(j < 4 ? c0 : c1);
        v[2 * j] = f.x;
        v[2 * j + 1] = f.y;
    });
}

}  // namespace fos
