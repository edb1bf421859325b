// Shared pieces of the gfx950 quantize kernels: launch parameters, workgroup reductions and
// the operation-by-operation ("generic") quantisation of one 1x16 block, which restates
// the reference's PyTorch backend one IEEE fp32 rounding per reference operation
// (src/fouroversix/quantize/pytorch/reference.py:30-63, 184-552).
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "fos_device.h"
#include "fouroversix_hip.h"

namespace fos {


constexpr int kThreads = 256;
constexpr int kMaxPartials = 1024;  // pairs of 32-bit words in the workspace

struct QuantParams {
    const uint16_t *x;           // bf16 / fp16 elements, or (x_type == FOS_T_F32) really const float *
    int x_type = FOS_T_BF16;     // fp16 and fp32 inputs go through the element-wise kernel only
    int x_vec = 0;               // ... with 128-bit loads when base, row pitch and width allow (16-byte aligned rows, cols % 16 == 0)
    int64_t rows, cols, ld;      // logical input
    int64_t rows_p, cols_p;      // padded output extents
    uint8_t *codes;              // [rows_p, cols_p / 2]
    uint8_t *sf;                 // rows_p * cols_p / 16 bytes
    const uint32_t *partials;    // pass-1 results, pairs {max|x| as f32 bits, reserved}
    int n_partials;              // number of pairs; 0 = `partials` points at a caller-supplied f32 amax;
                                 // -1 = no pass 1 ran: pass 2 scans the (small, contiguous, aligned) input itself
    float *amax_out;             // written by workgroup 0 when not null
    uint64_t seed, offset;       // dither key of the stochastic styles ...
    const uint64_t *key = nullptr;  // ... or, when not null, where the kernels read {seed, offset} from (device memory)
    int sf_layout;
    int tiles_x;                 // workgroup tiles along the columns
    int tile_map = 0;            // TileMap: which tile the n-th unit of work is
    float c, qdiv, errdiv;       // f32(qmax*smax*adj), f32(qmax*adj), selection divisor
    uint16_t *pseudo_out;        // fused quantize -> dequantize: bf16 [rows, cols] output instead of codes / sf
    int64_t ldo;                 // its leading dimension
};

// Order in which the streaming kernels walk their tiles.  Workgroups are dealt to the eight
// XCDs (each with its own L2) round-robin, so unit n runs on XCD n % 8.
enum TileMap {
    kMapRowMajor = 0,  // unit n = tile n, row-major: an XCD sees every eighth tile of each tile row
    kMapBands = 1,     // XCD k walks the contiguous band of tiles [k n/8, (k+1) n/8) (needs n % 8 == 0)
    kMapColMajor = 2,  // unit n = tile n, column-major
    kMapBandsCol = 3,  // bands of the column-major order
    kMapSplitHalves = 4,  // (16x16-tile kernel, with the above) a workgroup's two 256-column halves lie 2048 columns apart
};

struct TileYX {
    uint32_t y, x;
};

// (returned by value: results handed back through references to members of a struct went
// through a stack slot, which gave the kernels a private segment)
FOS_DEVICE TileYX map_tile(uint32_t unit, uint32_t n_tiles, uint32_t tiles_x, int map) {
    if ((map & 1) && n_tiles % 8 == 0) unit = (unit & 7u) * (n_tiles >> 3) + (unit >> 3);
    TileYX t;
    if (map & 2) {
        const uint32_t tiles_y = n_tiles / tiles_x;
        t.x = unit / tiles_y;
        t.y = unit - t.x * tiles_y;
    } else {
        t.y = unit / tiles_x;
        t.x = unit - t.y * tiles_x;
    }
    return t;
}

// ---- workgroup reductions ------------------------------------------------------------

FOS_DEVICE uint32_t pk_max_u16(uint32_t a, uint32_t b) {
    typedef uint16_t u16x2 __attribute__((ext_vector_type(2)));
    u16x2 va = __builtin_bit_cast(u16x2, a), vb = __builtin_bit_cast(u16x2, b);
    u16x2 r = __builtin_elementwise_max(va, vb);
    return __builtin_bit_cast(uint32_t, r);
}

FOS_DEVICE uint32_t pk_min_i16(uint32_t a, uint32_t b) {
    typedef int16_t i16x2 __attribute__((ext_vector_type(2)));
    i16x2 va = __builtin_bit_cast(i16x2, a), vb = __builtin_bit_cast(i16x2, b);
    i16x2 r = __builtin_elementwise_min(va, vb);
    return __builtin_bit_cast(uint32_t, r);
}

FOS_DEVICE uint32_t wave_max_u32(uint32_t v) {
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) {
        uint32_t o = (uint32_t)__shfl_xor((int)v, off);
        v = v > o ? v : o;
    }
    return v;
}

// Max over the workgroup; valid in every thread.
FOS_DEVICE uint32_t block_max_u32(uint32_t v, uint32_t *smem /* >= 4 words */) {
    v = wave_max_u32(v);
    const int wave = threadIdx.x >> 6;
    if ((threadIdx.x & 63) == 0) smem[wave] = v;
    __syncthreads();
    uint32_t r = smem[0];
#pragma unroll
    for (int i = 1; i < kThreads / 64; ++i) r = r > smem[i] ? r : smem[i];
    __syncthreads();
    return r;
}

// Tensor-wide result of pass 1, valid in every thread: the bits of max|x|.  (The second word
// of each partial pair is reserved and ignored.)
FOS_DEVICE uint32_t reduce_partials(const QuantParams &p, uint32_t *smem) {
    if (p.n_partials == 0) return p.partials[0];
    if (p.n_partials < 0) {
        // small contiguous input: no pass 1 was launched and every workgroup scans the
        // whole tensor itself (rows * cols / 8 aligned 128-bit vectors, 128 KiB out of L2 at
        // most), which costs less than a launch and its dependency
        const uint4 *v4 = reinterpret_cast<const uint4 *>(p.x);
        const int n_vec = (int)((p.rows * p.cols) >> 3);
        uint32_t m = 0;
        constexpr int U = 16;  // loads in flight per thread: the scan is latency-bound
        for (int base = 0; base < n_vec; base += U * kThreads) {
            uint4 v[U];
#pragma unroll
            for (int u = 0; u < U; ++u) {
                const int i = base + u * kThreads + (int)threadIdx.x;
                v[u] = i < n_vec ? v4[i] : make_uint4(0u, 0u, 0u, 0u);
            }
#pragma unroll
            for (int u = 0; u < U; ++u) {
                m = pk_max_u16(m, v[u].x & 0x7fff7fffu);
                m = pk_max_u16(m, v[u].y & 0x7fff7fffu);
                m = pk_max_u16(m, v[u].z & 0x7fff7fffu);
                m = pk_max_u16(m, v[u].w & 0x7fff7fffu);
            }
        }
        const uint32_t mm = (m & 0xffffu) > (m >> 16) ? (m & 0xffffu) : (m >> 16);
        return block_max_u32(mm, smem) << 16;  // bf16 magnitude bits -> fp32 bits
    }
    uint32_t m = 0;
    for (int i = threadIdx.x; i < p.n_partials; i += kThreads) {
        const uint32_t v = p.partials[2 * i];
        m = m > v ? m : v;
    }
    return block_max_u32(m, smem);
}

// ---------------------------------------------------------------------------------------
// building blocks of one 1x16 block
// ---------------------------------------------------------------------------------------

struct QuantConsts {
    float amax, enc, dec, qdiv, errdiv;
    float rerr = 0.0f;      // RN(1 / errdiv)
    bool fast_div = false;  // errdiv is a constant with an exact 3-operation division and every quotient is normal or zero
    // The fast exact evaluation of a candidate's error (one fma per element from a per-scale
    // table) needs scale * amax to be exact in fp32 -- a tensor maximum with at most 8
    // significant bits, which every maximum of bf16 data has but a caller-supplied one need
    // not -- and the divisor 1536; without both, undecided blocks take the generic form.
    bool exact_ok = false;
    // The certified shortcuts of the adaptive rules model the reference's error sums with relative
    // rounding errors.  That holds while the reference's own fp32 arithmetic stays in the normal range:
    // its squared residuals are of the size of (amax / 1536 x block scale)^2 with block scales down to
    // 2^-9, so for a tensor of values around 2^-70 every squared error is flushed to zero or rounded as a
    // sub-normal (and every block ties), and sums of up to 256 squares of residuals up to amax / 4 overflow
    // from amax = 2^62 on.  The shortcuts are used for tensor maxima in [2^-40, 2^60]: at the lower end what
    // the reference loses to sub-normal squares (<= 256 x 2^-150) is 2^-12 of the smallest tolerance
    // (2^-15 h^2 with h >= 2^-59.6).  Beyond, every block takes the exact evaluation.
    bool shortcut_ok = false;
};

FOS_DEVICE bool shortcut_range(float amax) { return amax >= 0x1p-40f && amax <= 0x1p60f; }

// v / k.errdiv with IEEE rounding (the sign of a zero quotient may differ; callers subtract).
FOS_DEVICE float div_errdiv(float v, const QuantConsts &k) {
    if (k.fast_div) {
        const float q0 = v * k.rerr;
        return __builtin_fmaf(__builtin_fmaf(-k.errdiv, q0, v), k.rerr, q0);
    }
    return v / k.errdiv;
}

// compute_nv_scale_factors (reference.py:184-241) for one block maximum.
FOS_DEVICE void block_scale(const QuantConsts &k, float bmax, bool expand, uint32_t &s, float &sf, float &inv) {
    float s_hp = (k.amax == 0.0f) ? 0.0f : (bmax / k.qdiv) * k.enc;
    if (expand) s_hp = s_hp * 1.5f;
    s = e4m3_encode(s_hp);
    sf = e4m3_decode(s);
    inv = 1.0f / (k.dec * sf);
}

// E2M1 grid rounding of a magnitude, round to nearest (reference.py:30-51): no clamp (a
// magnitude in [7, 9) gives 8, which the nibble encoding below spills into bit 3 exactly
// as the reference's bit extraction does).  The stochastic styles round with the
// hardware convert (sr_pack16), which clamps to 6 as the reference's dithered branch does.
FOS_DEVICE float e2m1_round(float a) {
    float r1 = __builtin_rintf(a + a) * 0.5f;
    float r2 = __builtin_rintf(a);
    float r3 = 2.0f * __builtin_rintf(a * 0.5f);
    return a < 2.0f ? r1 : (a < 4.0f ? r2 : r3);
}

// Grid magnitude {0,.5,1,1.5,2,3,4,6,(8)} -> 3-bit code (8 for the overflow value).
FOS_DEVICE uint32_t e2m1_mag_code(float r) {
    float c = r < 2.0f ? (r + r) : (r < 4.0f ? r + 2.0f : r * 0.5f + 4.0f);
    return (uint32_t)c;
}

template <bool SR>
FOS_DEVICE float int4_round(float y, float u) {
    if (SR) {
        float t = fminf(fmaxf(fabsf(y) + u, -7.0f), 7.0f);
        float r = __builtin_rintf(t);
        r = (r == 0.0f) ? 0.0f : r;
        return y < 0.0f ? -r : (y > 0.0f ? r : 0.0f * r);
    }
    return __builtin_rintf(fminf(fmaxf(y, -7.0f), 7.0f));
}

// torch.sum order over the 16 values of a 1x16 block.
FOS_DEVICE float sum16(const float *e) {
    float t = e[0] + e[8];
#pragma unroll
    for (int l = 1; l < 8; ++l) t = t + (e[l] + e[l + 8]);
    return t;
}

// torch.sum order over a 16x16 tile flattened row-major, where this lane holds row
// (lane & 15) of the tile in e[0..15] and the 16 rows lie along one DPP row.
// Per column: even rows and odd rows are summed top to bottom (a chain of row_shr:2
// adds; -0.0 is what lanes 0 and 1 receive, so they keep their own value), then
// A[l] = ((E[l] + E[l+8]) + O[l]) + O[l+8] and the eight A[l] are summed left to right.
// The result is valid in lane 14 of each row and broadcast from there.
FOS_DEVICE float sum256_rows(const float *e) {
    float t[16];
#pragma unroll
    for (int c = 0; c < 16; ++c) t[c] = e[c];
#pragma unroll
    for (int step = 0; step < 7; ++step) {
#pragma unroll
        for (int c = 0; c < 16; ++c) t[c] = dpp_move<kDppRowShr + 2>(-0.0f, t[c]) + e[c];
    }
    float total = 0.0f;
#pragma unroll
    for (int l = 0; l < 8; ++l) {
        float a = t[l] + t[l + 8];
        a = a + dpp_move<kDppRowShl + 1>(0.0f, t[l]);
        a = a + dpp_move<kDppRowShl + 1>(0.0f, t[l + 8]);
        total = (l == 0) ? a : total + a;
    }
    const int lane = threadIdx.x & 63;
    return __shfl(total, (lane & 48) | 14);
}

template <int RULE, bool TWO_D>
FOS_DEVICE float reduce_error(const float *e) {
    if (RULE == FOS_RULE_ABS_MAX) {
        float m = e[0];
#pragma unroll
        for (int i = 1; i < 16; ++i) m = fmaxf(m, e[i]);
        return TWO_D ? row16_max(m) : m;
    }
    return TWO_D ? sum256_rows(e) : sum16(e);
}

template <int RULE>
FOS_DEVICE float error_term(float deq, float x) {
    float d = deq - x;
    return RULE == FOS_RULE_MSE ? d * d : fabsf(d);
}

// Random words for 1x16 block `blk`: ONE Philox4x32-10 call keyed (seed; blk, 0, offset)
// serves both candidates of the block.  The first candidate's element i reads word i / 4;
// the second candidate's element i reads what the first one's element i ^ 8 does (words
// exchanged pairwise), so within a candidate no two elements share a dither and the two
// dithers of one element are as independent as those of different elements.  (The
// reference's own native kernel rounds every element of the tensor and both candidates
// with one 32-bit word, src/fouroversix/csrc/include/utils.h:521,611,649-650.)
FOS_DEVICE Philox4 block_philox(uint64_t seed, uint64_t offset, uint64_t blk) {
    return philox4x32_10((uint32_t)blk, (uint32_t)(blk >> 32), 0u, (uint32_t)offset, (uint32_t)seed, (uint32_t)(seed >> 32));
}
FOS_DEVICE Philox4 second_candidate_words(const Philox4 &p) { return Philox4{{p.v[2], p.v[3], p.v[0], p.v[1]}}; }

// One 1x16 block (one row of a 16x16 tile when TWO_D): 8 input words -> 2 code words
// and the scale byte.  `blk` = row * (cols_p / 16) + block column keys the dither.
// The block arrives as 16 fp32 values (the reference converts its input with `.float()`,
// reference.py:577,593,596, so bf16, fp16 and fp32 inputs meet here).
template <int DT, int RULE, int ROUND, bool TWO_D>
FOS_DEVICE void quantize_block_f32(const float *x, const QuantConsts &k, uint64_t seed, uint64_t offset,
                                   uint64_t blk, uint32_t *codes, uint32_t &sbyte) {
    constexpr bool SR = ROUND != FOS_ROUND_NEAREST;
    constexpr bool STATIC = (RULE == FOS_RULE_STATIC_6 || RULE == FOS_RULE_STATIC_4);
    float bmax = 0.0f;
#pragma unroll
    for (int i = 0; i < 16; i += 2) bmax = fmaxf(fmaxf(fabsf(x[i]), fabsf(x[i + 1])), bmax);
    if (TWO_D) bmax = row16_max(bmax);

    uint32_t sA;
    float sfA, invA;
    block_scale(k, bmax, false, sA, sfA, invA);
    // x * inv + 0 drops the sign of a zero product, as the reference's sign(x) does
    auto scaled = [&](uint32_t s, float inv, float *xs) {
#pragma unroll
        for (int i = 0; i < 16; ++i) xs[i] = (s != 0) ? __builtin_fmaf(x[i], inv, 0.0f) : 0.0f;
    };
    Philox4 pA, pB;
    if (SR) pA = block_philox(seed, offset, blk);

    if (STATIC) {
        uint32_t c0 = 0, c1 = 0;
        if (SR) {
            float xs[16];
            scaled(sA, invA, xs);
            sr_pack16(xs, pA, c0, c1);
        } else {
#pragma unroll
            for (int i = 0; i < 16; ++i) {
                float xs = (sA != 0) ? x[i] * invA : 0.0f;
                float r = e2m1_round(fabsf(xs));
                uint32_t nib = e2m1_mag_code(r) | ((xs < 0.0f) ? 8u : 0u);
                if (i < 8) c0 |= nib << (4 * i);
                else c1 |= nib << (4 * (i - 8));
            }
        }
        codes[0] = c0;
        codes[1] = c1;
        sbyte = sA;
        return;
    }

    if (SR) pB = second_candidate_words(pA);
    float eA[16], eB[16];
    uint32_t a0 = 0, a1 = 0, b0 = 0, b1 = 0;

    if (DT == FOS_DTYPE_IF4) {
        // select_intfloat (reference.py:328-425): candidate A = E2M1, candidate B = INT4
        // on the same scale; B wins on a strictly smaller error.
        float xsS[16], fqS[16];
        if (SR) {
            scaled(sA, invA, xsS);
            sr_pack16(xsS, pA, a0, a1);
            unpack16_fp4(a0, a1, fqS);
        }
#pragma unroll
        for (int i = 0; i < 16; ++i) {
            float xs = (sA != 0) ? x[i] * invA : 0.0f;
            float fq;
            if (SR) {
                fq = fqS[i];
            } else {
                float r = e2m1_round(fabsf(xs));
                bool neg = xs < 0.0f;
                fq = neg ? -r : r;
                uint32_t nibA = e2m1_mag_code(r) | (neg ? 8u : 0u);
                if (i < 8) a0 |= nibA << (4 * i);
                else a1 |= nibA << (4 * (i - 8));
            }
            float q = int4_round<SR>(xs * 1.16666666f, SR ? dither_from_byte(pB.v[i >> 2], i & 3) : 0.0f);
            uint32_t nibB = (uint32_t)((int)q) & 0xfu;
            float deqA = div_errdiv((fq * sfA) * k.amax, k);
            float deqB = div_errdiv(((q * sfA) * k.amax) * 0.8571428571f, k);
            eA[i] = error_term<RULE>(deqA, x[i]);
            eB[i] = error_term<RULE>(deqB, x[i]);
            if (i < 8) b0 |= nibB << (4 * i);
            else b1 |= nibB << (4 * (i - 8));
        }
        float errA = reduce_error<RULE, TWO_D>(eA);
        float errB = reduce_error<RULE, TWO_D>(eB);
        bool pickB = errB < errA;
        codes[0] = pickB ? b0 : a0;
        codes[1] = pickB ? b1 : a1;
        sbyte = pickB ? (sA + 128u) : sA;
        return;
    }

    // 4/6 (reference.py:262-325, 519-552): candidate A scales the block maximum to 6,
    // candidate B to 4 (scale * 1.5); B wins on a strictly smaller error.
    uint32_t sB;
    float sfB, invB;
    block_scale(k, bmax, true, sB, sfB, invB);
    if (SR) {
        float xsA[16], xsB[16], fqA[16], fqB[16];
        scaled(sA, invA, xsA);
        scaled(sB, invB, xsB);
        sr_pack16(xsA, pA, a0, a1);
        sr_pack16(xsB, pB, b0, b1);
        unpack16_fp4(a0, a1, fqA);
        unpack16_fp4(b0, b1, fqB);
#pragma unroll
        for (int i = 0; i < 16; ++i) {
            eA[i] = error_term<RULE>(div_errdiv((fqA[i] * sfA) * k.amax, k), x[i]);
            eB[i] = error_term<RULE>(div_errdiv((fqB[i] * sfB) * k.amax, k), x[i]);
        }
    } else {
#pragma unroll
        for (int i = 0; i < 16; ++i) {
            float xsA = (sA != 0) ? x[i] * invA : 0.0f;
            float xsB = (sB != 0) ? x[i] * invB : 0.0f;
            float rA = e2m1_round(fabsf(xsA));
            float rB = e2m1_round(fabsf(xsB));
            bool negA = xsA < 0.0f, negB = xsB < 0.0f;
            uint32_t nibA = e2m1_mag_code(rA) | (negA ? 8u : 0u);
            uint32_t nibB = e2m1_mag_code(rB) | (negB ? 8u : 0u);
            float deqA = div_errdiv(((negA ? -rA : rA) * sfA) * k.amax, k);
            float deqB = div_errdiv(((negB ? -rB : rB) * sfB) * k.amax, k);
            eA[i] = error_term<RULE>(deqA, x[i]);
            eB[i] = error_term<RULE>(deqB, x[i]);
            if (i < 8) { a0 |= nibA << (4 * i); b0 |= nibB << (4 * i); }
            else { a1 |= nibA << (4 * (i - 8)); b1 |= nibB << (4 * (i - 8)); }
        }
    }
    float errA = reduce_error<RULE, TWO_D>(eA);
    float errB = reduce_error<RULE, TWO_D>(eB);
    bool pickB = errB < errA;
    codes[0] = pickB ? b0 : a0;
    codes[1] = pickB ? b1 : a1;
    sbyte = pickB ? sB : sA;
}

// The same for 8 words of bf16 pairs.
template <int DT, int RULE, int ROUND, bool TWO_D>
FOS_DEVICE void quantize_block(const uint32_t *w, const QuantConsts &k, uint64_t seed, uint64_t offset,
                               uint64_t blk, uint32_t *codes, uint32_t &sbyte) {
    float x[16];
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        x[2 * i] = u2f(w[i] << 16);
        x[2 * i + 1] = u2f(w[i] & 0xffff0000u);
    }
    quantize_block_f32<DT, RULE, ROUND, TWO_D>(x, k, seed, offset, blk, codes, sbyte);
}

// The 16 elements of block column cb of row r as fp32, 128-bit loads (QuantParams::x_vec).
FOS_DEVICE void load_block16(const QuantParams &p, int64_t r, int64_t c0, float *x) {
    if (p.x_type == FOS_T_F32) {
        const float4 *src = reinterpret_cast<const float4 *>(reinterpret_cast<const float *>(p.x) + r * p.ld + c0);
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const float4 v = src[i];
            x[4 * i] = v.x, x[4 * i + 1] = v.y, x[4 * i + 2] = v.z, x[4 * i + 3] = v.w;
        }
        return;
    }
    const uint4 *src = reinterpret_cast<const uint4 *>(p.x + r * p.ld + c0);
    const uint4 lo = src[0], hi = src[1];
    const uint32_t w[8] = {lo.x, lo.y, lo.z, lo.w, hi.x, hi.y, hi.z, hi.w};
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        if (p.x_type == FOS_T_F16) {
            x[2 * i] = (float)__builtin_bit_cast(_Float16, (uint16_t)(w[i] & 0xffffu));
            x[2 * i + 1] = (float)__builtin_bit_cast(_Float16, (uint16_t)(w[i] >> 16));
        } else {
            x[2 * i] = u2f(w[i] << 16);
            x[2 * i + 1] = u2f(w[i] & 0xffff0000u);
        }
    }
}

// Element (r, c) of the input as fp32 (exact for each of the three input types).
FOS_DEVICE float load_element(const QuantParams &p, int64_t r, int64_t c) {
    const int64_t i = r * p.ld + c;
    if (p.x_type == FOS_T_F32) return reinterpret_cast<const float *>(p.x)[i];
    const uint16_t h = p.x[i];
    if (p.x_type == FOS_T_F16) return (float)__builtin_bit_cast(_Float16, h);
    return u2f((uint32_t)h << 16);
}

// Offset of scale (r, c) inside the 128x4-tile layout (quantize/utils.py:88-96).
FOS_DEVICE int64_t tiled_sf_offset(int64_t r, int64_t c, int64_t sf_cols) {
    return ((r >> 7) * (sf_cols >> 2) + (c >> 2)) * 512 + (r & 31) * 16 + ((r & 127) >> 5) * 4 + (c & 3);
}


}  // namespace fos
