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
// hardware convert keeps the sign in both cases, so the scaled value is formed as
// fma(x, inv, +0): the product of a non-zero x is unchanged and (-0) * inv + 0 is +0.
#pragma once

#include <type_traits>

#include "fos_quantize_common.h"

namespace fos {

struct FastLutEntry {
    float inv;       // 1 / (dec * s)                       (0 for s == 0)
    float d1;        // RN((s * amax) / errdiv)             factor for fq in {.5, 1, 2, 4}
    uint32_t delta;  // bits((s * amax) / 1024) - bits(d1)  added for fq in {1.5, 3, 6}
    float hh;        // weight of this scale's sum of squares in the shortcut: (d1 / 2^e)^2 with 2^e <= amax < 2^(e+1)
                     // (d1^2 itself leaves fp32's normal range for tensors whose maximum is far from 1); the
                     // product form of the MSE shortcut keeps d1 / 2^e here instead
};

// 2^-e for 2^e <= amax < 2^(e+1) (a normal amax)
FOS_DEVICE float amax_norm(float amax) {
    const uint32_t e = (f2u(amax) >> 23) & 0xffu;
    return u2f((254u - (e < 1u ? 1u : (e > 253u ? 253u : e))) << 23);
}

// Entry for scale byte `s` (0..127); built with the reference's operations.
template <bool PRODUCT_FORM = false>
FOS_DEVICE FastLutEntry make_lut_entry(uint32_t s, const QuantConsts &k) {
    FastLutEntry e;
    const float sf = e4m3_decode(s);
    e.inv = s == 0 ? 0.0f : 1.0f / (k.dec * sf);
    const float g = sf * k.amax;
    e.d1 = g / k.errdiv;
    e.delta = f2u((1.5f * g) / k.errdiv) - f2u(e.d1);  // 1.5 g is exact; with errdiv = 1536 this is g / 1024
    const float hn = e.d1 * amax_norm(k.amax);
    e.hh = PRODUCT_FORM ? hn : hn * hn;
    return e;
}

// Scaled value of one element: x * inv with the sign of a zero product dropped.
FOS_DEVICE float scaled(float x, float inv) { return __builtin_fmaf(x, inv, 0.0f); }

// x / y for a constant y with r = RN(1/y); equals IEEE division whenever the quotient is
// a normal number.
FOS_DEVICE float div_const(float x, float y, float r) {
    const float q0 = x * r;
    return __builtin_fmaf(__builtin_fmaf(-y, q0, x), r, q0);
}

// a * b + c on 24-bit unsigned a, b in one instruction (the compiler turns a multiplication by a
// one-bit value into a sign-extending bit-field extract, an AND and an addition: three)
FOS_DEVICE uint32_t mad_u24(uint32_t a, uint32_t b, uint32_t c) {
    uint32_t d;
    asm("v_mad_u32_u24 %0, %1, %2, %3" : "=v"(d) : "v"(a), "v"(b), "v"(c));
    return d;
}

// deq - x for one decoded candidate value fq (on the E2M1 grid).
FOS_DEVICE float candidate_residual(float fq, const FastLutEntry &e, float x) {
    const uint32_t fb = f2u(fq);
    const float p2 = u2f(fb & 0xffbfffffu);                    // 1.5 * 2^j -> 2^j
    const uint32_t three = (fb >> 22) & 1u;                    // fq in {1.5, 3, 6}
    const float mult = u2f(mad_u24(three, e.delta, f2u(e.d1)));
    return __builtin_fmaf(p2, mult, -x);
}

// ---------------------------------------------------------------------------------------
// 4/6-MSE with a certified shortcut
// ---------------------------------------------------------------------------------------
//
// The exact decision compares E_k = sum_i fl(fl(deq_i - x_i)^2), k in {6, 4}, which costs
// ~8 instructions per element and candidate.  In the block's scaled domain the same
// quantity is h_k^2 * S_k with S_k = sum_i (fq_i - x_i / h_k)^2 and h_k = s_k * amax / 1536,
// and S_k is 4 instructions per element (the scaled value x_i * inv_k is needed for the
// rounding anyway).  With u = 2^-24, |x_i / h_k| <= 6.5 and |fq_i - x_i / h_k| <= 1, a
// term-by-term bound of every rounding in both evaluations gives
//     |E_k - h_k^2 S~_k| <= h_k^2 * u * (330 sqrt(S_k) + 40 S_k)        (16 elements)
// (5 roundings from amax to x*inv: 33u absolute on the scaled value; 7u on the reference's
// residual; 16u relative on either sum; 256-element tiles multiply the two coefficients by
// 4 and 16).  The kernel uses 2^-14 ((1 + S) / 2 + S) for a block and 2^-14 (2 (1 + S) + 2 S) for a
// tile, both >= three times that (sqrt(S) <= (1 + S) / 2), as the tolerance: when the two intervals do not overlap the comparison E_4 < E_6 is
// decided by the shortcut, otherwise (a few blocks in 10^4 on real data; every block of a
// tensor whose candidates tie exactly) the exact evaluation runs.

// max / sum over the 16 lanes of a DPP row; every lane gets lane 0's result so that the
// whole row takes the same branch.
FOS_DEVICE float row16_sum_lane0(float v) {
    v = v + dpp_move<kDppRowRor + 8>(v, v);
    v = v + dpp_move<kDppRowRor + 4>(v, v);
    v = v + dpp_move<kDppRowRor + 2>(v, v);
    v = v + dpp_move<kDppRowRor + 1>(v, v);
    const int lane = threadIdx.x & 63;
    return __shfl(v, lane & 48);
}

// Certified comparison of two candidates' errors from their scaled-domain reductions (S already
// reduced over the tile when TWO_D): returns +1 when the second is surely smaller, -1 when it is
// surely not smaller (the first wins, also on a tie), 0 when the two tolerance intervals overlap.
// The weight w of a candidate is d1^2 (MSE) or d1 (MAE, abs-max); tolerance w (k0 + k1 S) each:
//  * MSE: as derived above;
//  * MAE, E = h sum |fq - x / h|: the 40u per element add up, 16 * 40u = 640u (256 * 40u for a
//    tile), and the two summations and the products round with <= 40u S (520u S): three times
//    that is below 2^-14 (2 + S / 8) resp. 2^-14 (32 + 2 S);
//  * abs-max, E = h max |fq - x / h|: 40u and one rounding of the product, three times that is
//    below 2^-17 whatever the block size.
template <int RULE, bool TWO_D>
FOS_DEVICE int shortcut_compare(float SA, float wA, float SB, float wB) {
    constexpr float k0 = RULE == FOS_RULE_MSE ? (TWO_D ? 4.0f : 1.0f) * 0.5f * 0x1p-14f
                         : RULE == FOS_RULE_MAE ? (TWO_D ? 32.0f : 2.0f) * 0x1p-14f
                                                : 0x1p-17f;
    constexpr float k1 = RULE == FOS_RULE_MSE ? (TWO_D ? 2.0f + 2.0f : 1.0f + 0.5f) * 0x1p-14f
                         : RULE == FOS_RULE_MAE ? (TWO_D ? 2.0f : 0.125f) * 0x1p-14f
                                                : 0.0f;
    // |EB - EA| against tA + tB (the differences and sums round within a few 2^-24 of
    // quantities that the tolerances exceed by 2^10)
    const float D = __builtin_fmaf(wB, SB, -(wA * SA));
    const float T = __builtin_fmaf(wA, __builtin_fmaf(k1, SA, k0), wB * __builtin_fmaf(k1, SB, k0));
    if (fabsf(D) > T) return D < 0.0f ? 1 : -1;
    return 0;
}

// One element pair's rounding residuals into the running reduction of a rule.
template <int RULE>
FOS_DEVICE void accumulate_scaled(float r0, float r1, float &S) {
    if (RULE == FOS_RULE_MSE) {
        S = __builtin_fmaf(r0, r0, S);
        S = __builtin_fmaf(r1, r1, S);
    } else if (RULE == FOS_RULE_MAE) {
        S = S + fabsf(r0);
        S = S + fabsf(r1);
    } else {
        S = fmaxf(fmaxf(fabsf(r0), fabsf(r1)), S);
    }
}

// Weight of a candidate's scaled-domain reduction in its error.
template <int RULE>
FOS_DEVICE float shortcut_weight(const FastLutEntry &e) {
    return RULE == FOS_RULE_MSE ? e.hh : e.d1;
}

// ---------------------------------------------------------------------------------------
// 4/6-MSE shortcut in product form (bf16 elements, 1x16 blocks)
// ---------------------------------------------------------------------------------------
//
// E_k = sum_i (h_k fq_i - x_i)^2 = h_k^2 F_k - 2 h_k G_k + sum_i x_i^2 with F_k = sum fq_i^2 and
// G_k = sum fq_i x_i, and the last term is the same for both candidates:
//     (E_4 - E_6) / 2 = h_4 q_4 - h_6 q_6,     q_k = (h_k / 2) F_k - G_k.
// F_k and G_k come from v_dot2_f32_bf16 on the codes converted to bf16 pairs and the block's
// packed elements AS LOADED (no unpacking, no scaled residuals): three instructions per element
// pair and candidate where the residual form needs five.  Both sums are exact: a non-zero fq_i
// needs a scaled magnitude above 1/4 and the block's largest is below 7, so the elements that
// contribute span fewer than five binades; with 8 significant bits each, every product fq_i x_i
// (fq_i = j / 2, j <= 12) is a multiple of 2^(e - 8) for the smallest such element's exponent e,
// and every partial sum of the 16 stays below 2^(e + 13): 21 bits.  F_k <= 16 * 36 in units of 1/4.
// What is left to bound:
//  * the reference's own roundings.  Its dequantised value is c_i * d1 or c_i * (d1 (+) delta),
//    within 2u (4u for a maximum with more than 8 significant bits) of h_k fq_i with h_k = d1;
//    its residual, square and summation add 1 + 1 + 9 roundings: with scaled residuals of at
//    most 1 (sum at most 16, sum of squares S at most 16)
//        |E_ref - E_k| <= h_k^2 u (200 sqrt(S) + 11 S) <= 976 u h_k^2,          u = 2^-24;
//  * three roundings here (q_k, h_k q_k, the difference): <= 3u (|h_6 q_6| + |h_4 q_4|) on the half difference.
// Tolerance on the half difference: 2^-14 (h_6^2 + h_4^2) + 2^-21 (|h_6 q_6| + |h_4 q_4|), i.e. 2048u per
// candidate against 976u and 8u against 3u.  One factor h_k of every product is taken relative to
// the tensor maximum's power of two (FastLutEntry::hh in its product form), so that nothing
// leaves fp32's normal range for the tensor maxima the shortcuts are used with (QuantConsts::shortcut_ok).
typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));

// Byte SEL of `word` -> the two E2M1 values as a bf16 pair (low nibble first).
template <int SEL>
FOS_DEVICE bf16x2_t unpack_fp4_bf16(uint32_t word) {
    return __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(word, 1.0f, SEL);
}

FOS_DEVICE float dot2_bf16(bf16x2_t a, bf16x2_t b, float c) { return __builtin_amdgcn_fdot2_f32_bf16(a, b, c, false); }

// +1: the second candidate's error is surely smaller; -1: surely not; 0: within the tolerance.
FOS_DEVICE int product_compare(float FA, float GA, const FastLutEntry &A, float FB, float GB, const FastLutEntry &B) {
    const float qA = __builtin_fmaf(0.5f * A.d1, FA, -GA), qB = __builtin_fmaf(0.5f * B.d1, FB, -GB);
    const float pA = A.hh * qA, pB = B.hh * qB;  // (hh: d1 over the maximum's power of two)
    const float D = pB - pA;
    const float T = __builtin_fmaf(0x1p-21f, fabsf(pA) + fabsf(pB), 0x1p-14f * __builtin_fmaf(A.hh, A.d1, B.hh * B.d1));
    if (fabsf(D) > T) return D < 0.0f ? 1 : -1;
    return 0;
}

// The two rare paths are real function calls (arguments and results by value, in
// registers) written as rolled loops over the eight column pairs (l, l + 8) -- the order
// in which torch.sum consumes a block -- so that their register needs and code size stay
// out of the hot loop.  Arrays indexed by the loop counter live in scratch memory.
struct Block16 {
    uint32_t w[8];
};
struct BlockOut {
    uint32_t c0, c1, s;
};

// F16: the block holds fp16 pairs instead of bf16 pairs (both convert to f32 exactly).
template <bool F16 = false>
FOS_DEVICE float block_element(const uint32_t *w, int idx) {
    const uint32_t word = w[idx >> 1];
    if (F16) return (float)__builtin_bit_cast(_Float16, (uint16_t)((idx & 1) ? word >> 16 : word));
    return (idx & 1) ? u2f(word & 0xffff0000u) : u2f(word << 16);
}

// Column sum of one value per lane down the 16 rows of a tile, even and odd rows apart
// (lane 14 ends with the even-row sum, lane 15 with the odd-row sum).
FOS_DEVICE float tile_column_chain(float e) {
    float t = e;
#pragma unroll
    for (int step = 0; step < 7; ++step) t = dpp_move<kDppRowShr + 2>(-0.0f, t) + e;
    return t;
}

// Running reduction of the selection error over the column pairs, in torch.sum's order.
template <int RULE, bool TWO_D>
FOS_DEVICE void accumulate_pair(float e_lo, float e_hi, int l, float &total) {
    if (RULE == FOS_RULE_ABS_MAX) {
        total = fmaxf(total, fmaxf(e_lo, e_hi));  // errors are >= 0 and total starts at 0
    } else if (!TWO_D) {
        const float pair = e_lo + e_hi;
        total = l == 0 ? pair : total + pair;
    } else {
        const float t_lo = tile_column_chain(e_lo), t_hi = tile_column_chain(e_hi);
        float a = t_lo + t_hi;
        a = a + dpp_move<kDppRowShl + 1>(0.0f, t_lo);
        a = a + dpp_move<kDppRowShl + 1>(0.0f, t_hi);
        total = l == 0 ? a : total + a;
    }
}

template <int RULE, bool TWO_D>
FOS_DEVICE float finish_error(float total) {
    if (!TWO_D) return total;
    if (RULE == FOS_RULE_ABS_MAX) return row16_max(total);
    const int lane = threadIdx.x & 63;
    return __shfl(total, (lane & 48) | 14);
}

FOS_DEVICE float e2m1_value(uint32_t code) {
    const uint32_t e = (code >> 1) & 3u, m = code & 1u;
    const float v = e == 0 ? 0.5f * (float)m : u2f((126u + e) << 23 | m << 22);
    return (code & 8u) ? -v : v;
}

// True when the two candidates of a block dequantise to identical values, element by
// element, so that the reference's two error sums are bit-equal and "6" wins the tie.
// With s4 = 1.5 * s6 exactly, fq6 * s6 == fq4 * s4 iff (fq6, fq4) is (0, 0), (1.5, 1),
// (3, 2) or (6, 4) with equal signs: in codes, both magnitudes 0, or code4 in {2, 4, 6} and
// code6 = code4 | 1.  That is the typical block with one dominant element: the outlier is
// exact under both scales and everything else rounds to zero.  Nibble-parallel on a word
// of 8 codes; `a` holds the "6" codes, `b` the "4" codes.
FOS_DEVICE uint32_t tie_violations(uint32_t a, uint32_t b) {
    const uint32_t d = a ^ b;
    const uint32_t u = (a | b) & 0x77777777u;
    const uint32_t nz = (u | (u >> 1) | (u >> 2)) & 0x11111111u;          // a magnitude is non-zero
    const uint32_t nzb = ((b >> 1) | (b >> 2)) & 0x11111111u;             // code4 in {2..7}
    return ((d & 0x77777777u) ^ nz)   // magnitudes differ exactly in bit 0 where non-zero, nowhere else
           | (d & (nz << 3))          // equal signs where non-zero
           | (~a & nz)                // the set bit 0 belongs to code6
           | (nzb ^ nz);              // code4 is not 0 or 1 where non-zero
}

// Exact selection of a block whose shortcut was inconclusive: the residuals of both
// candidates from their packed codes, with the reference's rounding and order.
template <int RULE, bool TWO_D>
__device__ __attribute__((noinline)) bool exact_pick_b(Block16 blk, uint32_t a0, uint32_t a1, uint32_t b0,
                                                       uint32_t b1, FastLutEntry A, FastLutEntry B) {
    uint32_t w[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) w[i] = blk.w[i];
    const uint64_t ca = ((uint64_t)a1 << 32) | a0, cb = ((uint64_t)b1 << 32) | b0;
    float totA = 0.0f, totB = 0.0f;
#pragma nounroll
    for (int l = 0; l < 8; ++l) {
        float e[2][2];
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            const int idx = l + 8 * h;
            const float x = block_element(w, idx);  // the sign of a zero does not reach |d| or d * d
            const float dA = candidate_residual(e2m1_value((uint32_t)(ca >> (4 * idx)) & 0xfu), A, x);
            const float dB = candidate_residual(e2m1_value((uint32_t)(cb >> (4 * idx)) & 0xfu), B, x);
            e[0][h] = RULE == FOS_RULE_MSE ? dA * dA : fabsf(dA);
            e[1][h] = RULE == FOS_RULE_MSE ? dB * dB : fabsf(dB);
        }
        accumulate_pair<RULE, TWO_D>(e[0][0], e[0][1], l, totA);
        accumulate_pair<RULE, TWO_D>(e[1][0], e[1][1], l, totB);
    }
    return finish_error<RULE, TWO_D>(totB) < finish_error<RULE, TWO_D>(totA);
}

// The same for a 1x16 block, unrolled in registers: no call and no scratch memory, so it can
// sit in the streaming loop (a call there makes the wavefront wait for every load it has in
// flight, and a few such waits were what the slowest wavefronts of a launch spent their time on).
template <int RULE>
FOS_DEVICE bool exact_pick_b_1d(const float *x, uint32_t a0, uint32_t a1, uint32_t b0, uint32_t b1, const FastLutEntry &A,
                                const FastLutEntry &B) {
    float eA[16], eB[16];
    static_for<0, 8>([&](auto jc) {
        constexpr int j = decltype(jc)::value;
        const float2_t fa = unpack_fp4<(j & 3)>(j < 4 ? a0 : a1);
        const float2_t fb = unpack_fp4<(j & 3)>(j < 4 ? b0 : b1);
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            const float dA = candidate_residual(fa[h], A, x[2 * j + h]);
            const float dB = candidate_residual(fb[h], B, x[2 * j + h]);
            eA[2 * j + h] = RULE == FOS_RULE_MSE ? dA * dA : fabsf(dA);
            eB[2 * j + h] = RULE == FOS_RULE_MSE ? dB * dB : fabsf(dB);
        }
    });
    return reduce_error<RULE, false>(eB) < reduce_error<RULE, false>(eA);
}

// The same, one undecided block at a time spread over the wavefront: lane (c, e) = (lane >> 4 & 1, lane & 15)
// evaluates element e of candidate c, and the 16 errors of a candidate meet in torch.sum's order through
// DPP moves inside its row of 16 lanes -- about 40 instructions per undecided block, where the per-lane
// form above costs the wavefront its 300 whenever a single lane is undecided (one wavefront step in
// twenty on N(0,1) data).  Every lane of the wavefront must call it (convergent control flow); `scratch`
// = 16 words of LDS private to the wavefront.  Returns the decision in the lanes that asked.
struct ExactRequest {
    bool wanted = false;
    uint32_t b0 = 0, b1 = 0, sB = 0;  // second candidate (the first is the provisional BlockOut)
};

template <int RULE, bool F16>
FOS_DEVICE bool exact_pick_b_spread(bool wanted, const Block16 &blk, uint32_t a0, uint32_t a1, uint32_t b0, uint32_t b1,
                                    const FastLutEntry &A, const FastLutEntry &B, uint32_t *scratch) {
    static_assert(RULE == FOS_RULE_MSE || RULE == FOS_RULE_MAE, "rules that sum their errors");
    const int lane = threadIdx.x & 63;
    const int e = lane & 15, c = (lane >> 4) & 1;
    bool pickB = false;
    uint64_t pending = __builtin_amdgcn_ballot_w64(wanted);
    while (pending != 0) {
        const int l = __builtin_ctzll(pending);
        pending &= pending - 1;
        if (lane == l) {
            uint4 *dst = reinterpret_cast<uint4 *>(scratch);
            dst[0] = make_uint4(blk.w[0], blk.w[1], blk.w[2], blk.w[3]);
            dst[1] = make_uint4(blk.w[4], blk.w[5], blk.w[6], blk.w[7]);
            dst[2] = make_uint4(a0, a1, b0, b1);
            dst[3] = make_uint4(f2u(A.d1), A.delta, f2u(B.d1), B.delta);
        }
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
        const uint32_t xw = scratch[e >> 1];
        float x;
        if (F16) x = (float)__builtin_bit_cast(_Float16, (uint16_t)((e & 1) ? xw >> 16 : xw));
        else x = (e & 1) ? u2f(xw & 0xffff0000u) : u2f(xw << 16);
        const uint32_t cw = scratch[8 + 2 * c + (e >> 3)];
        const float fq = unpack_fp4<0>(cw >> (4 * (e & 7))).x;
        FastLutEntry E;
        E.d1 = u2f(scratch[12 + 2 * c]);
        E.delta = scratch[13 + 2 * c];
        const float d = candidate_residual(fq, E, x);
        const float err = RULE == FOS_RULE_MSE ? d * d : fabsf(d);
        // p[i] = err[i] + err[i + 8] in lanes 0..7 of the row, then ((p0 + p1) + p2) + ... + p7 into lane 7
        const float pr = err + dpp_move<kDppRowShl + 8>(0.0f, err);
        float t = pr;
#pragma unroll
        for (int step = 0; step < 7; ++step) t = dpp_move<kDppRowShr + 1>(-0.0f, t) + pr;
        const float EA = __shfl(t, 7), EB = __shfl(t, 23);
        if (lane == l) pickB = EB < EA;
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
    }
    return pickB;
}

// exact_pick_b_1d from the packed block (for callers that no longer hold the unpacked elements).
template <int RULE, bool F16>
FOS_DEVICE bool exact_pick_b_1d_packed(const Block16 &blk, uint32_t a0, uint32_t a1, uint32_t b0, uint32_t b1, const FastLutEntry &A,
                                       const FastLutEntry &B) {
    float x[16];
#pragma unroll
    for (int i = 0; i < 16; ++i) x[i] = block_element<F16>(blk.w, i);
    return exact_pick_b_1d<RULE>(x, a0, a1, b0, b1, A, B);
}

// Operation-by-operation form (sub-normal block scales, out-of-range tensors): the
// arithmetic of quantize_block in fos_quantize_common.h, rolled.
template <int RULE, bool TWO_D, bool F16 = false>
__device__ __attribute__((noinline)) BlockOut generic_block(Block16 blk, QuantConsts k) {
    constexpr bool STATIC = (RULE == FOS_RULE_STATIC_6 || RULE == FOS_RULE_STATIC_4);
    uint32_t w[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) w[i] = blk.w[i];
    float bmax = 0.0f;
#pragma nounroll
    for (int i = 0; i < 16; ++i) bmax = fmaxf(bmax, fabsf(block_element<F16>(w, i)));
    if (TWO_D) bmax = row16_max(bmax);
    uint32_t sA, sB = 0;
    float sfA, invA, sfB = 0.0f, invB = 0.0f;
    block_scale(k, bmax, false, sA, sfA, invA);
    if (!STATIC) block_scale(k, bmax, true, sB, sfB, invB);
    uint64_t ca = 0, cb = 0;
    float totA = 0.0f, totB = 0.0f;
#pragma nounroll
    for (int l = 0; l < 8; ++l) {
        float e[2][2];
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            const int idx = l + 8 * h;
            const float x = block_element<F16>(w, idx);
            const float xsA = (sA != 0) ? x * invA : 0.0f;
            const float rA = e2m1_round(fabsf(xsA));
            const bool negA = xsA < 0.0f;
            ca |= (uint64_t)(e2m1_mag_code(rA) | (negA ? 8u : 0u)) << (4 * idx);
            if (!STATIC) {
                const float xsB = (sB != 0) ? x * invB : 0.0f;
                const float rB = e2m1_round(fabsf(xsB));
                const bool negB = xsB < 0.0f;
                cb |= (uint64_t)(e2m1_mag_code(rB) | (negB ? 8u : 0u)) << (4 * idx);
                const float deqA = (((negA ? -rA : rA) * sfA) * k.amax) / k.errdiv;
                const float deqB = (((negB ? -rB : rB) * sfB) * k.amax) / k.errdiv;
                e[0][h] = error_term<RULE>(deqA, x);
                e[1][h] = error_term<RULE>(deqB, x);
            }
        }
        if (!STATIC) {
            accumulate_pair<RULE, TWO_D>(e[0][0], e[0][1], l, totA);
            accumulate_pair<RULE, TWO_D>(e[1][0], e[1][1], l, totB);
        }
    }
    bool pickB = false;
    if (!STATIC) pickB = finish_error<RULE, TWO_D>(totB) < finish_error<RULE, TWO_D>(totA);
    const uint64_t c = pickB ? cb : ca;
    return BlockOut{(uint32_t)c, (uint32_t)(c >> 32), pickB ? sB : sA};
}

// Operation-by-operation form for the stochastic style (quantize_block, out of line).
template <int RULE, bool TWO_D>
__device__ __attribute__((noinline)) BlockOut generic_block_sr(Block16 blk, QuantConsts k, uint64_t seed, uint64_t offset,
                                                              uint64_t blkid) {
    uint32_t codes[2], sbyte;
    quantize_block<FOS_DTYPE_NVFP4, RULE, FOS_ROUND_STOCHASTIC, TWO_D>(blk.w, k, seed, offset, blkid, codes, sbyte);
    return BlockOut{codes[0], codes[1], sbyte};
}

// One 1x16 block, NVFP4, any rule, round to nearest or (SR) a stochastic style; falls
// back by itself.  `blkid` = row * (cols_p / 16) + block column keys the dither.
// F16: fp16 elements (1x16 blocks, round to nearest).  Nothing in the formulation depends on the element
// type beyond the conversion to f32: the scaled value is the reference's own x * inv, the division of
// the block maximum by 6 or 4 is correctly rounded for every fp16 numerator too (checked exhaustively),
// and fq * s * amax stays exact with the 11 significant bits of an fp16 maximum (2 + 4 + 11 <= 24).
// PRODUCT: the MSE shortcut in its product form (bf16 elements, 1x16 blocks, round to nearest; the table built
// with make_lut_entry<true>).
// SPREAD: a block whose shortcut is inconclusive is not evaluated here; it comes back as the first candidate
// with `req` filled in, for exact_pick_b_spread at a point where the whole wavefront is together.
template <int RULE, bool TWO_D, bool SR, bool F16 = false, bool PRODUCT = false, bool SPREAD = false>
FOS_DEVICE BlockOut quantize_block_nvfp4_fast(const Block16 &blk, const QuantConsts &k, float enc, float rq,
                                              bool in_range, const FastLutEntry *lut, uint64_t seed, uint64_t offset,
                                              uint64_t blkid, ExactRequest *req = nullptr) {
    static_assert(!SPREAD || (!TWO_D && (RULE == FOS_RULE_MSE || RULE == FOS_RULE_MAE)), "spread evaluation: 1x16 blocks, summing rules");
    static_assert(!F16 || (!TWO_D && !SR), "fp16 elements: 1x16 blocks, round to nearest");
    static_assert(!PRODUCT || (RULE == FOS_RULE_MSE && !TWO_D && !SR && !F16), "product form: MSE, 1x16, bf16, round to nearest");
    constexpr bool STATIC = (RULE == FOS_RULE_STATIC_6 || RULE == FOS_RULE_STATIC_4);
    // the certified shortcut: MSE, and MAE for 1x16 blocks.  (Abs-max has one too, but 3 % of the
    // blocks of N(0,1) data tie exactly under that rule -- the largest residual belongs to an
    // element that both candidates represent by the same value -- so nearly every wavefront step
    // ran the exact evaluation anyway and the shortcut only added to it: 55 us against 47.)
    constexpr bool SHORTCUT = RULE == FOS_RULE_MSE || (RULE == FOS_RULE_MAE && !TWO_D);
    if (in_range) {
        float x[16];
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            if (F16) {
                x[2 * i] = (float)__builtin_bit_cast(_Float16, (uint16_t)blk.w[i]);
                x[2 * i + 1] = (float)__builtin_bit_cast(_Float16, (uint16_t)(blk.w[i] >> 16));
            } else {
                x[2 * i] = u2f(blk.w[i] << 16);
                x[2 * i + 1] = u2f(blk.w[i] & 0xffff0000u);
            }
        }
        float bmax = 0.0f;
#pragma unroll
        for (int i = 0; i < 16; i += 2) bmax = fmaxf(fmaxf(fabsf(x[i]), fabsf(x[i + 1])), bmax);
        if (TWO_D) bmax = row16_max(bmax);

        // the 3-operation division is exact for the divisors 6 and 4 (every bf16 numerator);
        // the unbiased stochastic style rescales them, and f32(6 * 16 / 17) is not
        float bq;
        if (SR && k.qdiv != 6.0f && k.qdiv != 4.0f) bq = bmax / k.qdiv;
        else bq = div_const(bmax, k.qdiv, rq);
        const float s_hp6 = bq * enc;
        const float s_hp4 = s_hp6 * 1.5f;
        const uint32_t pk = (uint32_t)__builtin_amdgcn_cvt_pk_fp8_f32(s_hp6, s_hp4, 0, false);
        const uint32_t s6 = pk & 0xffu, s4 = (pk >> 8) & 0xffu;
        // The hardware convert saturates at 6 where the reference's unclamped rounding gives
        // 8 for a scaled magnitude in [7, 9): that needs a sub-normal scale byte that was
        // rounded down by more than 7/6 (only candidate "6" can get there).  A zero scale
        // byte of a non-zero block has no scaled domain at all.  Everything else -- normal
        // and sub-normal scales alike -- is exact on the fast path.
        // The stochastic style clamps to 6 in the reference as well, so only the zero scale
        // byte is left out there.
        const FastLutEntry A = lut[s6];
        if (SR ? s6 != 0u : (s6 >= 8u || (s6 != 0u && bmax * A.inv < 7.0f))) {
            if constexpr (SR) {
                // scaled values, hardware stochastic rounding (one Philox call per block);
                // the certified shortcut holds unchanged: its bound does not use how far a
                // rounded value may lie from the scaled one
                float xa[16];
#pragma unroll
                for (int i = 0; i < 16; ++i) xa[i] = scaled(x[i], A.inv);
                const Philox4 pA = block_philox(seed, offset, blkid);
                uint32_t a0, a1;
                sr_pack16(xa, pA, a0, a1);
                if (STATIC) return BlockOut{a0, a1, s6};
                const FastLutEntry B = lut[s4];
                float xb[16];
#pragma unroll
                for (int i = 0; i < 16; ++i) xb[i] = scaled(x[i], B.inv);
                const Philox4 pB = second_candidate_words(pA);
                uint32_t b0, b1;
                sr_pack16(xb, pB, b0, b1);
                bool pickB = false, certain = false;
                if (SHORTCUT) {
                    float SA = 0.0f, SB = 0.0f;
                    static_for<0, 8>([&](auto jc) {
                        constexpr int j = decltype(jc)::value;
                        const float2_t fa = unpack_fp4<(j & 3)>(j < 4 ? a0 : a1);
                        const float2_t fb = unpack_fp4<(j & 3)>(j < 4 ? b0 : b1);
                        accumulate_scaled<RULE>(fa.x - xa[2 * j], fa.y - xa[2 * j + 1], SA);
                        accumulate_scaled<RULE>(fb.x - xb[2 * j], fb.y - xb[2 * j + 1], SB);
                    });
                    if (TWO_D) {
                        SA = row16_sum_lane0(SA);
                        SB = row16_sum_lane0(SB);
                    }
                    const int cmp = k.shortcut_ok ? shortcut_compare<RULE, TWO_D>(SA, shortcut_weight<RULE>(A), SB, shortcut_weight<RULE>(B)) : 0;
                    certain = cmp != 0;
                    pickB = cmp > 0;
                }
                if (!certain) {
                    bool tie = SHORTCUT && e4m3_decode(s4) == 1.5f * e4m3_decode(s6) && (tie_violations(a0, b0) | tie_violations(a1, b1)) == 0;
                    if (SHORTCUT && TWO_D) tie = row16_max(tie ? 0.0f : 1.0f) == 0.0f;
                    if (tie) pickB = false;
                    else if (k.exact_ok) {
                        if constexpr (SPREAD) {
                            req->wanted = true;
                            req->b0 = b0;
                            req->b1 = b1;
                            req->sB = s4;
                        } else if constexpr (TWO_D) pickB = exact_pick_b<RULE, TWO_D>(blk, a0, a1, b0, b1, A, B);
                        else pickB = exact_pick_b_1d<RULE>(x, a0, a1, b0, b1, A, B);
                    } else return generic_block_sr<RULE, TWO_D>(blk, k, seed, offset, blkid);  // e.g. the unbiased style's divisor
                }
                return BlockOut{pickB ? b0 : a0, pickB ? b1 : a1, pickB ? s4 : s6};
            }
            if (STATIC) {
                uint32_t c0 = 0, c1 = 0;
                static_for<0, 4>([&](auto jc) {
                    constexpr int j = decltype(jc)::value;
                    c0 = pack_fp4<j>(c0, scaled(x[2 * j], A.inv), scaled(x[2 * j + 1], A.inv));
                    c1 = pack_fp4<j>(c1, scaled(x[8 + 2 * j], A.inv), scaled(x[9 + 2 * j], A.inv));
                });
                return BlockOut{c0, c1, s6};
            }
            const FastLutEntry B = lut[s4];
            uint32_t a0 = 0, a1 = 0, b0 = 0, b1 = 0;
            float SA = 0.0f, SB = 0.0f, GA = 0.0f, GB = 0.0f;  // (product form: SA / SB hold F)
            static_for<0, 8>([&](auto jc) {
                constexpr int j = decltype(jc)::value;
                const float xa0 = scaled(x[2 * j], A.inv), xa1 = scaled(x[2 * j + 1], A.inv);
                const float xb0 = scaled(x[2 * j], B.inv), xb1 = scaled(x[2 * j + 1], B.inv);
                if (j < 4) {
                    a0 = pack_fp4<(j & 3)>(a0, xa0, xa1);
                    b0 = pack_fp4<(j & 3)>(b0, xb0, xb1);
                } else {
                    a1 = pack_fp4<(j & 3)>(a1, xa0, xa1);
                    b1 = pack_fp4<(j & 3)>(b1, xb0, xb1);
                }
                if constexpr (!PRODUCT && SHORTCUT) {
                    const float2_t fa = unpack_fp4<(j & 3)>(j < 4 ? a0 : a1);
                    const float2_t fb = unpack_fp4<(j & 3)>(j < 4 ? b0 : b1);
                    accumulate_scaled<RULE>(fa.x - xa0, fa.y - xa1, SA);
                    accumulate_scaled<RULE>(fb.x - xb0, fb.y - xb1, SB);
                }
            });
            bool pickB = false, certain = false;
            if constexpr (PRODUCT) {
                // (from the finished code words: decoding byte j while the word is still being filled made the
                // compiler keep a copy of every intermediate word)
                static_for<0, 8>([&](auto jc) {
                    constexpr int j = decltype(jc)::value;
                    const bf16x2_t fa = unpack_fp4_bf16<(j & 3)>(j < 4 ? a0 : a1);
                    const bf16x2_t fb = unpack_fp4_bf16<(j & 3)>(j < 4 ? b0 : b1);
                    const bf16x2_t xw = __builtin_bit_cast(bf16x2_t, blk.w[j]);
                    GA = dot2_bf16(fa, xw, GA);
                    SA = dot2_bf16(fa, fa, SA);
                    GB = dot2_bf16(fb, xw, GB);
                    SB = dot2_bf16(fb, fb, SB);
                });
                const int cmp = k.shortcut_ok ? product_compare(SA, GA, A, SB, GB, B) : 0;
                certain = cmp != 0;
                pickB = cmp > 0;
            } else if (SHORTCUT) {
                if (TWO_D) {
                    SA = row16_sum_lane0(SA);
                    SB = row16_sum_lane0(SB);
                }
                const int cmp = k.shortcut_ok ? shortcut_compare<RULE, TWO_D>(SA, shortcut_weight<RULE>(A), SB, shortcut_weight<RULE>(B)) : 0;
                certain = cmp != 0;
                pickB = cmp > 0;
            }
            if (!certain) {
                // exact ties by construction first (cheap), the full evaluation otherwise (a rule
                // without a shortcut evaluates every block exactly, ties included: no pre-check)
                bool tie = SHORTCUT && e4m3_decode(s4) == 1.5f * e4m3_decode(s6) && (tie_violations(a0, b0) | tie_violations(a1, b1)) == 0;
                if (SHORTCUT && TWO_D) {
                    // every row of the tile must agree
                    tie = row16_max(tie ? 0.0f : 1.0f) == 0.0f;
                }
                if (tie) pickB = false;
                else if (k.exact_ok) {
                    if constexpr (SPREAD) {
                        req->wanted = true;
                        req->b0 = b0;
                        req->b1 = b1;
                        req->sB = s4;
                    } else if constexpr (TWO_D) pickB = exact_pick_b<RULE, TWO_D>(blk, a0, a1, b0, b1, A, B);
                    else pickB = exact_pick_b_1d<RULE>(x, a0, a1, b0, b1, A, B);
                } else return generic_block<RULE, TWO_D, F16>(blk, k);
            }
            return BlockOut{pickB ? b0 : a0, pickB ? b1 : a1, pickB ? s4 : s6};
        }
        if (bmax == 0.0f) return BlockOut{0, 0, 0};  // an all-zero block: zero codes, zero scale
    }
    if constexpr (SR) return generic_block_sr<RULE, TWO_D>(blk, k, seed, offset, blkid);
    else return generic_block<RULE, TWO_D, F16>(blk, k);
}

// ---------------------------------------------------------------------------------------
// IF4 (one scale; E2M1 candidate against INT4 candidate), 4/6-style MSE selection
// ---------------------------------------------------------------------------------------
//
// Both candidates share the scale, so in the block's scaled domain (h = s * amax / 2688)
// their errors are h^2 S_fp and h^2 S_int with S_fp = sum (fq - x/h)^2 and
// S_int = sum (0.857... q - x/h)^2, and the decision err_int < err_fp compares the two
// sums.  The rounding bound of the 4/6 shortcut carries over (the INT4 value goes
// through one more rounding, 12u instead of 6u on a scaled magnitude <= 6, inside the
// same threefold margin); undecided blocks take the operation-by-operation form.
template <int RULE, bool TWO_D>
__device__ __attribute__((noinline)) BlockOut generic_block_if4(Block16 blk, QuantConsts k) {
    uint32_t codes[2], sbyte;
    quantize_block<FOS_DTYPE_IF4, RULE, FOS_ROUND_NEAREST, TWO_D>(blk.w, k, 0, 0, 0, codes, sbyte);
    return BlockOut{codes[0], codes[1], sbyte};
}

template <bool TWO_D>
FOS_DEVICE BlockOut quantize_block_if4_mse(const Block16 &blk, const QuantConsts &k, float enc, float rq,
                                           bool in_range, const FastLutEntry *lut) {
    if (in_range) {
        float x[16];
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            x[2 * i] = u2f(blk.w[i] << 16);
            x[2 * i + 1] = u2f(blk.w[i] & 0xffff0000u);
        }
        float bmax = 0.0f;
#pragma unroll
        for (int i = 0; i < 16; i += 2) bmax = fmaxf(fmaxf(fabsf(x[i]), fabsf(x[i + 1])), bmax);
        if (TWO_D) bmax = row16_max(bmax);
        const float s_hp = div_const(bmax, k.qdiv, rq) * enc;
        const uint32_t s = (uint32_t)__builtin_amdgcn_cvt_pk_fp8_f32(s_hp, 0.0f, 0, false) & 0xffu;
        const FastLutEntry A = lut[s];
        // same exclusions as the NVFP4 path: the unclamped E2M1 value 8 and the zero scale byte
        if (s >= 8u || (s != 0u && bmax * A.inv < 7.0f)) {
            uint32_t a0 = 0, a1 = 0, b0 = 0, b1 = 0;
            float SA = 0.0f, SB = 0.0f;
            static_for<0, 8>([&](auto jc) {
                constexpr int j = decltype(jc)::value;
                const float x0 = scaled(x[2 * j], A.inv), x1 = scaled(x[2 * j + 1], A.inv);
                if (j < 4) a0 = pack_fp4<(j & 3)>(a0, x0, x1);
                else a1 = pack_fp4<(j & 3)>(a1, x0, x1);
                const float2_t fa = unpack_fp4<(j & 3)>(j < 4 ? a0 : a1);
                const float r0 = fa.x - x0, r1 = fa.y - x1;
                SA = __builtin_fmaf(r0, r0, SA);
                SA = __builtin_fmaf(r1, r1, SA);
                // INT4: rint(clamp(x * 7/6, -7, 7)); adding 1.5 * 2^23 rounds to nearest even and
                // leaves the two's-complement integer in the low mantissa bits
                const float t0 = __builtin_amdgcn_fmed3f(x0 * 1.16666666f, -7.0f, 7.0f) + 12582912.0f;
                const float t1 = __builtin_amdgcn_fmed3f(x1 * 1.16666666f, -7.0f, 7.0f) + 12582912.0f;
                const float q0 = t0 - 12582912.0f, q1 = t1 - 12582912.0f;
                const float d0 = __builtin_fmaf(q0, 0.8571428571f, -x0), d1 = __builtin_fmaf(q1, 0.8571428571f, -x1);
                SB = __builtin_fmaf(d0, d0, SB);
                SB = __builtin_fmaf(d1, d1, SB);
                const uint32_t byte = (f2u(t0) & 0xfu) | ((f2u(t1) & 0xfu) << 4);
                if (j < 4) b0 |= byte << (8 * (j & 3));
                else b1 |= byte << (8 * (j & 3));
            });
            if (TWO_D) {
                SA = row16_sum_lane0(SA);
                SB = row16_sum_lane0(SB);
            }
            const int cmp = k.shortcut_ok ? shortcut_compare<FOS_RULE_MSE, TWO_D>(SA, 1.0f, SB, 1.0f) : 0;  // same scale: compare the sums
            if (cmp > 0) return BlockOut{b0, b1, s | 0x80u};
            if (cmp < 0) return BlockOut{a0, a1, s};
            // undecided (uniform over the 16 lanes of a tile when TWO_D: both sums are tile sums)
        } else if (bmax == 0.0f) {
            return BlockOut{0, 0, 0};
        }
    }
    return generic_block_if4<FOS_RULE_MSE, TWO_D>(blk, k);
}

// The 16 dequantised values of a quantised NVFP4 block as bf16 pairs, with the operations
// of the reference's dequantize (src/fouroversix/quantize/backend.py:141-155):
// bf16(((value * scale) * amax) / c); value * scale is exact.  FASTDIV replaces the IEEE
// division by the exact 3-operation form (quotient normal or zero) and restores the sign
// of a zero quotient.
template <bool FASTDIV>
FOS_DEVICE void dequant_block_bf16(const BlockOut &o, float amax, float c, float rc, uint32_t *w) {
    typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
    const float sf = e4m3_decode(o.s & 0x7fu);
    static_for<0, 8>([&](auto jc) {
        constexpr int j = decltype(jc)::value;
        const float2_t v = unpack_fp4<(j & 3)>(j < 4 ? o.c0 : o.c1);
        float2_t q;
#pragma unroll
        for (int e = 0; e < 2; ++e) {
            const float f = (v[e] * sf) * amax;
            if (FASTDIV) q[e] = u2f((f2u(div_const(f, c, rc)) & 0x7fffffffu) | (f2u(f) & 0x80000000u));
            else q[e] = f / c;
        }
        w[j] = __builtin_bit_cast(uint32_t, __builtin_convertvector(q, bf16x2_t));
    });
}

// ... for either format and 16-bit output type, operation by operation as dequantize_kernel does it (the
// fp16 product value * scale is exact for E2M1 values and rounds for IF4's integer blocks, whose values are
// fp16(6/7 * integer)).  `o.s` carries the integer-block flag in bit 7.
template <bool IF4, bool OUT_F16, bool FASTDIV>
FOS_DEVICE void dequant_block_any(const BlockOut &o, float amax, float c, float rc, uint32_t *w) {
    typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
    typedef _Float16 f16x2_t __attribute__((ext_vector_type(2)));
    const float sf = e4m3_decode(o.s & 0x7fu);
    const bool int_block = IF4 && (o.s & 0x80u);
    const _Float16 s16 = (_Float16)sf;
    static_for<0, 8>([&](auto jc) {
        constexpr int j = decltype(jc)::value;
        const uint32_t word = j < 4 ? o.c0 : o.c1;
        float2_t f = unpack_fp4<(j & 3)>(word) * sf;
        if (int_block) {
#pragma unroll
            for (int e = 0; e < 2; ++e) {
                const int iv = ((int)(word << (28 - 8 * (j & 3) - 4 * e))) >> 28;  // the nibble, sign-extended
                f[e] = (float)((_Float16)((float)iv * (float)(6.0 / 7.0)) * s16);
            }
        }
        float2_t q;
#pragma unroll
        for (int e = 0; e < 2; ++e) {
            const float t = f[e] * amax;
            if (FASTDIV) q[e] = u2f((f2u(div_const(t, c, rc)) & 0x7fffffffu) | (f2u(t) & 0x80000000u));
            else q[e] = t / c;
        }
        if (OUT_F16) w[j] = __builtin_bit_cast(uint32_t, __builtin_convertvector(q, f16x2_t));
        else w[j] = __builtin_bit_cast(uint32_t, __builtin_convertvector(q, bf16x2_t));
    });
}

// The same through the per-scale table when fq * s * amax is exact (a maximum of <= 8 significant bits, no
// sub-normal results): RN(fq * g / c) with g = s * amax is fq * RN(g / c) for fq in {.5, 1, 2, 4} and
// (fq / 1.5) * RN(1.5 g / c) for fq in {1.5, 3, 6} (1.5 g is exact), i.e. (power of two) x (table value):
// three operations per element instead of eight.  `e` = the entry of the block's scale byte in a table
// built with divisor c.
FOS_DEVICE void dequant_block_bf16_lut(const BlockOut &o, const FastLutEntry &e, uint32_t *w) {
    typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
    static_for<0, 8>([&](auto jc) {
        constexpr int j = decltype(jc)::value;
        const float2_t v = unpack_fp4<(j & 3)>(j < 4 ? o.c0 : o.c1);
        float2_t q;
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            const uint32_t fb = f2u(v[h]);
            const float p2 = u2f(fb & 0xffbfffffu);  // 1.5 * 2^j -> 2^j (sign and zero kept)
            const uint32_t three = (fb >> 22) & 1u;
            q[h] = p2 * u2f(mad_u24(three, e.delta, f2u(e.d1)));
        }
        w[j] = __builtin_bit_cast(uint32_t, __builtin_convertvector(q, bf16x2_t));
    });
}

}  // namespace fos
