// Device-side helpers shared by the gfx950 quantize, dequantize and GEMM kernels.
//
// Everything here is fp32 with one IEEE rounding per written operation: the library is
// compiled with -ffp-contract=off, correctly rounded division, fp32 denormals enabled,
// and fused multiply-adds appear only where __builtin_fmaf is spelled out.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

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
// values symmetric about zero.
FOS_DEVICE float dither_from_byte(uint32_t w, int i) {
    return __builtin_fmaf((float)((w >> (8 * i)) & 0xffu), 0x1p-8f, -0.498046875f);
}

}  // namespace fos
