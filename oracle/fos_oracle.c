/*
 * fos_oracle.c -- TEST INFRASTRUCTURE, NOT PRODUCT CODE.
 *
 * Scalar CPU restatement of the reference's PyTorch quantize / dequantize / FP4-matmul
 * path, used only as the checker for the gfx950 kernels (tests, the smoke check and the
 * CPU-baseline leg of the benchmark).  Nothing under fouroversix_amd/ may call it.
 *
 * Reference files restated (paths relative to the reference tree):
 *   src/fouroversix/quantize/pytorch/reference.py
 *       fake_quantize_to_e2m1 :30-51, fake_quantize_to_int4 :54-63,
 *       quantize_bf16_to_unpacked_{int4,fp4} :78-108, pack_unpacked_fp4 :111-132,
 *       compute_nv_scale_factors :184-241, select_fouroversix :262-325,
 *       select_intfloat :328-425, generic/intfloat/fouroversix dispatch :428-552,
 *       quantize :555-679
 *   src/fouroversix/quantize/utils.py          to_blocked :88-96
 *   src/fouroversix/quantize/dequantize_utils.py  from_blocked :4-12, E2M1/IF4 decode :15-67
 *   src/fouroversix/quantize/backend.py        dequantize :89-160
 *   src/fouroversix/matmul/pytorch.py          quantized_matmul :33-52
 *   src/fouroversix/kernels/constants.py       IF4 expansion constants :4-5
 *
 * Parity pins (tests/test_oracle.py): E4M3 cast vs torch's own cast over a full sweep;
 * E2M1 rounding vs the reference's threshold table over every bf16 value; the 16- and
 * 256-element summation orders vs torch.sum; closed forms for zeros / ones / rand01;
 * golden vectors written by the reference itself (tests/golden); the dot products of the
 * reference's MAC test benches (if4_mac/tb/*.svh, transcribed to tests/golden/if4_mac.npz)
 * for code decode, E4M3 decode and IF4 integer blocks; Philox4x32-10 against the published
 * Random123 known answers; the reference's stochastic-rounding known answers for NVFP4
 * (137 / 122 / 158 / 139) and IF4 (110 / 122), which is what holds int4_sr and the IF4
 * stochastic branch.
 * Stochastic rounding is "parity unpinned" bit-wise by construction: the reference draws
 * from torch's global generator; here the dither comes from Philox4x32-10 keyed by
 * (seed, block, candidate) so that this file and the GPU kernel agree bit-for-bit, and
 * agreement with the reference is statistical (its own known-answer distances).
 *
 * Build: gcc -O2 -std=c11 -fPIC -shared -fopenmp -ffp-contract=off fos_oracle.c -lm
 * All arithmetic is IEEE binary32 with one rounding per operation (SSE2 scalar code,
 * contraction disabled), which is what torch's CPU kernels do for these ops.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#define FOS_NVFP4 0
#define FOS_IF4 1

#define RULE_STATIC6 0
#define RULE_STATIC4 1
#define RULE_MAE 2
#define RULE_MSE 3
#define RULE_ABSMAX 4

#define ROUND_NEAREST 0
#define ROUND_STOCHASTIC 1
#define ROUND_STOCHASTIC_UNBIASED 2

static inline float bits_to_f32(uint32_t u) { float f; memcpy(&f, &u, 4); return f; }
static inline uint32_t f32_to_bits(float f) { uint32_t u; memcpy(&u, &f, 4); return u; }
static inline float bf16_to_f32(uint16_t h) { return bits_to_f32((uint32_t)h << 16); }

/* float -> bf16, round to nearest even (torch's .bfloat16()). */
static inline uint16_t f32_to_bf16(float f) {
    uint32_t u = f32_to_bits(f);
    if ((u & 0x7fffffffu) > 0x7f800000u) return 0x7fc0;
    u += 0x7fffu + ((u >> 16) & 1u);
    return (uint16_t)(u >> 16);
}

/* float rounded to the nearest binary16 value (ties to even), returned as float. */
static float round_to_f16(float f) {
    float a = fabsf(f);
    if (!(a < 65520.0f)) return f < 0 ? -INFINITY : INFINITY;
    if (a < 6.103515625e-05f) { /* below 2^-14: fixed step 2^-24 */
        float r = rintf(a * 16777216.0f) * 5.9604644775390625e-08f;
        return copysignf(r, f);
    }
    uint32_t u = f32_to_bits(a);
    u += 0xfffu + ((u >> 13) & 1u);
    u &= ~0x1fffu;
    return copysignf(bits_to_f32(u), f);
}

/* ---- E4M3 (float8_e4m3fn) --------------------------------------------------------- */

/* torch's `.to(torch.float8_e4m3fn)`: round to nearest even, 2^-10 -> 0, 464 -> 448,
 * anything that rounds past 448 becomes the NaN pattern 0x7F (no saturation). */
uint8_t fos_oracle_e4m3_from_f32(float f) {
    uint32_t u = f32_to_bits(f);
    uint8_t sign = (uint8_t)((u >> 31) << 7);
    uint32_t a = u & 0x7fffffffu;
    if (a >= 0x43f00000u) return sign | 0x7f; /* >= 480, inf, nan */
    if (a < 0x3c800000u) {                    /* < 2^-6: subnormal grid, step 2^-9 */
        float r = rintf(bits_to_f32(a) * 512.0f);
        return sign | (uint8_t)r;
    }
    a += 0x7ffffu + ((a >> 20) & 1u);
    return sign | (uint8_t)((a >> 20) - (120u << 3));
}

float fos_oracle_e4m3_to_f32(uint8_t b) {
    int e = (b >> 3) & 15, m = b & 7;
    float v;
    if ((b & 0x7f) == 0x7f) v = NAN;
    else if (e == 0) v = ldexpf((float)m, -9);
    else v = ldexpf(1.0f + (float)m * 0.125f, e - 7);
    return (b & 0x80) ? -v : v;
}

/* ---- E2M1 ------------------------------------------------------------------------- */

static inline float sign_of(float x) { return (float)((x > 0.0f) - (x < 0.0f)); }

/* reference.py:30-51, nearest branch: three rint regimes, no clamp. */
float fos_oracle_e2m1_rtn(float xs) {
    float a = fabsf(xs), r;
    if (a < 2.0f) r = rintf(2.0f * a) / 2.0f;
    else if (a < 4.0f) r = rintf(a);
    else r = 2.0f * rintf(a / 2.0f);
    return sign_of(xs) * r;
}

/* Stochastic rounding of a scaled value to an E2M1 code (reference.py:39-44 adds
 * U[-0.5, 0.5) before the rint of the magnitude's regime and clamps to 6).  Restated in
 * the form the gfx950 convert V_CVT_SCALEF32_SR_PK_FP4_F32 implements, so that kernel and
 * oracle agree bit for bit: the top 22 bits of `rword` are added to the discarded bits
 * of the significand, aligned to their top, and the sum is truncated -- rounding up with
 * probability (discarded fraction) to within 2^-22; saturation at 6; the sign is kept,
 * also on a zero result.  M = 1.m * 2^23 (0.m * 2^23 for a sub-normal float), d = 22
 * discarded bits for |x| >= 1 and 22 - exponent below, q = (M + (R << (d - 22))) >> d
 * counts half-steps of the binade (of 1 below 1.0).  `R22` is the 22-bit dither. */
uint8_t fos_oracle_e2m1_sr_code(float xs, uint32_t R22) {
    uint32_t b;
    memcpy(&b, &xs, 4);
    uint32_t sign = b >> 31, exp = (b >> 23) & 0xffu, mant = b & 0x7fffffu;
    uint32_t code;
    if (exp == 255) {
        code = 7;
    } else {
        uint64_t M = exp ? (mant | 0x800000u) : mant;
        int e = exp ? (int)exp - 127 : -126;
        int d = e >= 0 ? 22 : 22 - e;
        uint64_t R = R22 & 0x3fffffu;
        uint64_t q = d >= 46 ? 0 : (M + (R << (d - 22))) >> d;
        if (e >= 0) {
            uint64_t c = 2 * (uint64_t)(e > 8 ? 8 : e) + q;
            code = c > 7 ? 7 : (uint32_t)c;
        } else {
            code = (uint32_t)q;
        }
    }
    return (uint8_t)(code | (sign << 3));
}

/* reference.py:54-63 */
static float int4_rtn(float y) {
    float c = y < -7.0f ? -7.0f : (y > 7.0f ? 7.0f : y);
    return rintf(c);
}
static float int4_sr(float y, float u) {
    float t = fabsf(y) + u;
    t = t < -7.0f ? -7.0f : (t > 7.0f ? 7.0f : t);
    float r = rintf(t);
    if (r == 0.0f) r = 0.0f;
    return sign_of(y) * r;
}

/* reference.py:82-108 applied to the bf16 image of a fake-quantized value: 4-bit code
 * s<<3 | (e-126)<<1 | m with 0.5 -> (0,1) and zero -> 0 (sign kept).  The value 8,
 * which only a degenerate sub-normal block scale can produce, spills into bit 3. */
static uint8_t e2m1_code_from_fq(float fq) {
    uint16_t b = f32_to_bf16(fq);
    int s = (b >> 15) & 1, e = (b >> 7) & 0xff, m = b & 0x7f;
    int is_zero = (e == 0) && (m == 0);
    m = (m >> 6) & 1;
    if (e == 126 && m == 0) m = 1;
    e = e - 126;
    if (is_zero) { e = 0; m = 0; }
    return (uint8_t)(((s << 3) | (e << 1) | m) & 0xff);
}

/* reference.py:78-79 */
static uint8_t int4_code_from_fq(float q) {
    float c = q < -7.0f ? -7.0f : (q > 7.0f ? 7.0f : q);
    return (uint8_t)((int8_t)c) & 0xf;
}

float fos_oracle_e2m1_decode(uint8_t code) {
    static const float mag[8] = {0.0f, 0.5f, 1.0f, 1.5f, 2.0f, 3.0f, 4.0f, 6.0f};
    float v = mag[code & 7];
    return (code & 8) ? -v : v;
}

/* ---- torch.sum(dim=-1) order on the CPU build the reference ran on ---------------- */

/* 16 floats: p[l] = v[l] + v[l+8], then left to right. */
float fos_oracle_sum16(const float *v) {
    float p[8];
    for (int l = 0; l < 8; ++l) p[l] = v[l] + v[l + 8];
    float t = p[0];
    for (int l = 1; l < 8; ++l) t = t + p[l];
    return t;
}

/* 256 floats seen as 32 vectors of 8: four interleaved accumulators (vectors k, k+4, ...),
 * combined ((P0+P1)+P2)+P3, then the 8 lanes left to right. */
float fos_oracle_sum256(const float *v) {
    float P[4][8];
    for (int k = 0; k < 4; ++k)
        for (int l = 0; l < 8; ++l) P[k][l] = v[8 * k + l];
    for (int j = 4; j < 32; ++j)
        for (int l = 0; l < 8; ++l) P[j & 3][l] = P[j & 3][l] + v[8 * j + l];
    float A[8];
    for (int l = 0; l < 8; ++l) A[l] = ((P[0][l] + P[1][l]) + P[2][l]) + P[3][l];
    float t = A[0];
    for (int l = 1; l < 8; ++l) t = t + A[l];
    return t;
}

/* ---- Philox4x32-10 dither ---------------------------------------------------------- */

static inline void philox_round(uint32_t c[4], const uint32_t k[2]) {
    uint64_t p0 = (uint64_t)0xD2511F53u * c[0];
    uint64_t p1 = (uint64_t)0xCD9E8D57u * c[2];
    uint32_t n0 = (uint32_t)(p1 >> 32) ^ c[1] ^ k[0];
    uint32_t n1 = (uint32_t)p1;
    uint32_t n2 = (uint32_t)(p0 >> 32) ^ c[3] ^ k[1];
    uint32_t n3 = (uint32_t)p0;
    c[0] = n0; c[1] = n1; c[2] = n2; c[3] = n3;
}

void fos_oracle_philox4x32_10(const uint32_t ctr[4], const uint32_t key[2], uint32_t out[4]) {
    uint32_t c[4] = {ctr[0], ctr[1], ctr[2], ctr[3]};
    uint32_t k[2] = {key[0], key[1]};
    for (int r = 0; r < 10; ++r) {
        philox_round(c, k);
        k[0] += 0x9E3779B9u;
        k[1] += 0xBB67AE85u;
    }
    memcpy(out, c, 16);
}

/* Random words for the 16 elements of 1x16 block `blk` (= row * blocks_per_row + block
 * column of the padded tensor): ONE Philox4x32-10 call with counter (blk_lo, blk_hi, 0,
 * offset_lo) and key (seed_lo, seed_hi) serves both candidates of the block; the second
 * candidate's element i takes what the first one's element i ^ 8 takes (`cand`), so no two
 * elements of a candidate share a dither.  (The reference's own native kernel rounds a
 * whole tensor and both candidates with one 32-bit word,
 * src/fouroversix/csrc/include/utils.h:521,611,649-650.)  Element i of the first candidate
 * belongs to byte i % 4 of word i / 4.  E2M1 rounding takes the word rotated so that this byte leads and
 * from it the 22 bits that the convert's slot reads -- 31..10 for even i, 30..9 for odd i
 * (rw[i]; the leading 7 or 8 bits are the element's own, the rest come from its three
 * neighbours at 1/256 of the weight); the INT4 candidate of IF4 takes
 * u = (byte + 0.5) / 256 - 0.5, 256 equally likely values symmetric about zero.  The
 * reference draws from torch's generator, so its stream cannot be matched bit for bit. */
static void dither16(uint64_t seed, uint64_t offset, uint64_t blk, int cand, float u[16], uint32_t rw[16]) {
    uint32_t key[2] = {(uint32_t)seed, (uint32_t)(seed >> 32)};
    uint32_t ctr[4] = {(uint32_t)blk, (uint32_t)(blk >> 32), 0u, (uint32_t)offset};
    uint32_t w[4];
    fos_oracle_philox4x32_10(ctr, key, w);
    for (int i = 0; i < 16; ++i) {
        uint32_t word = w[((i >> 2) + (cand ? 2 : 0)) & 3];
        int sh = (8 * ((i & 3) + 1)) & 31;
        u[i] = (float)((word >> (8 * (i & 3))) & 0xffu) * 0.00390625f - 0.498046875f;
        uint32_t rot = sh ? ((word >> sh) | (word << (32 - sh))) : word;
        rw[i] = (i & 1) ? (rot >> 9) & 0x3fffffu : rot >> 10;
    }
}

/* ---- quantize ---------------------------------------------------------------------- */

typedef struct {
    int dtype, rule, round_style, block2d;
    float amax;
    float c;      /* f32(qmax * smax * adj) */
    float qdiv;   /* f32(qmax * adj) */
    float enc;    /* c / amax */
    float dec;    /* 1 / (c / amax) */
    float errdiv; /* divisor of the selection-error dequantisation */
    uint64_t seed, offset;
    int64_t blocks_per_row;
} qctx;

/* compute_nv_scale_factors (reference.py:184-241) for one block. */
static void scale_block(const qctx *q, const float *x, int n, float bmax, int expand,
                        uint8_t *s_out, float *xs, float *inv_out) {
    float s_hp;
    if (q->amax == 0.0f) s_hp = 0.0f;
    else s_hp = (bmax / q->qdiv) * q->enc;
    if (expand) s_hp = s_hp * 1.5f;
    uint8_t s = fos_oracle_e4m3_from_f32(s_hp);
    float sf = fos_oracle_e4m3_to_f32(s);
    float inv = 1.0f / (q->dec * sf);
    for (int i = 0; i < n; ++i) xs[i] = (s != 0) ? x[i] * inv : 0.0f;
    *s_out = s;
    *inv_out = inv;
}

static float block_error(int rule, const float *deq, const float *x, int n) {
    float e[256];
    if (rule == RULE_ABSMAX) {
        float m = 0.0f;
        for (int i = 0; i < n; ++i) { float d = fabsf(deq[i] - x[i]); if (d > m || d != d) m = d; }
        return m;
    }
    for (int i = 0; i < n; ++i) {
        float d = deq[i] - x[i];
        e[i] = (rule == RULE_MAE) ? fabsf(d) : d * d;
    }
    return n == 16 ? fos_oracle_sum16(e) : fos_oracle_sum256(e);
}

/* Fill the dither for every element of an n-element block (n = 16, or 256 for a 16x16
 * tile whose r-th row is 1x16 block blk0 + r * blocks_per_row). */
static void block_dither(const qctx *q, uint64_t blk0, int n, int cand, float *u, uint32_t *rw) {
    for (int r = 0; r < n / 16; ++r)
        dither16(q->seed, q->offset, blk0 + (uint64_t)r * (uint64_t)q->blocks_per_row, cand, u + 16 * r, rw + 16 * r);
}

/* E2M1 candidate of one block with stochastic rounding: x * inv + 0 (one rounding; the
 * sign of a zero product is dropped, as the reference's sign(x) does), then the convert. */
static void e2m1_sr_block(const float *x, int n, uint8_t s, float inv, const uint32_t *rw, float *fq) {
    for (int i = 0; i < n; ++i) {
        float xs = (s != 0) ? fmaf(x[i], inv, 0.0f) : 0.0f;
        fq[i] = fos_oracle_e2m1_decode(fos_oracle_e2m1_sr_code(xs, rw[i]));
    }
}

/* One block (16 or 256 floats): writes fake-quantized values fq[n], whether they are
 * integer coded, and the scale byte. */
static void quantize_block(const qctx *q, const float *x, int n, uint64_t blk0,
                           float *fq, int *is_int, uint8_t *s_out, float *err2) {
    if (err2) err2[0] = err2[1] = 0.0f;
    float bmax = 0.0f;
    for (int i = 0; i < n; ++i) { float a = fabsf(x[i]); if (a > bmax) bmax = a; }
    float xs6[256], xs4[256], f6[256], f4[256], d6[256], d4[256], u[256], inv6, inv4;
    uint32_t rw[256];
    uint8_t s6, s4;
    int sr = q->round_style != ROUND_NEAREST;
    *is_int = 0;

    if (q->rule == RULE_STATIC6 || q->rule == RULE_STATIC4) {
        scale_block(q, x, n, bmax, 0, &s6, xs6, &inv6);
        if (sr) {
            block_dither(q, blk0, n, 0, u, rw);
            e2m1_sr_block(x, n, s6, inv6, rw, fq);
        } else {
            for (int i = 0; i < n; ++i) fq[i] = fos_oracle_e2m1_rtn(xs6[i]);
        }
        *s_out = s6;
        return;
    }

    if (q->dtype == FOS_IF4) { /* select_intfloat, reference.py:328-425 */
        scale_block(q, x, n, bmax, 0, &s6, xs6, &inv6);
        float sf = fos_oracle_e4m3_to_f32(s6);
        if (sr) {
            block_dither(q, blk0, n, 0, u, rw);
            e2m1_sr_block(x, n, s6, inv6, rw, f6);
            block_dither(q, blk0, n, 1, u, rw);
        } else {
            for (int i = 0; i < n; ++i) f6[i] = fos_oracle_e2m1_rtn(xs6[i]);
        }
        for (int i = 0; i < n; ++i) {
            float y = xs6[i] * 1.16666666f;
            f4[i] = sr ? int4_sr(y, u[i]) : int4_rtn(y);
        }
        for (int i = 0; i < n; ++i) {
            d6[i] = ((f6[i] * sf) * q->amax) / q->errdiv;
            d4[i] = (((f4[i] * sf) * q->amax) * 0.8571428571f) / q->errdiv;
        }
        float err_fp = block_error(q->rule, d6, x, n);
        float err_int = block_error(q->rule, d4, x, n);
        int pick_int = err_int < err_fp;
        if (err2) { err2[0] = err_fp; err2[1] = err_int; }
        memcpy(fq, pick_int ? f4 : f6, sizeof(float) * (size_t)n);
        *is_int = pick_int;
        *s_out = pick_int ? (uint8_t)(s6 + 128) : s6;
        return;
    }

    /* 4/6 adaptive, reference.py:519-552 and 262-325 */
    scale_block(q, x, n, bmax, 0, &s6, xs6, &inv6);
    scale_block(q, x, n, bmax, 1, &s4, xs4, &inv4);
    if (sr) {
        block_dither(q, blk0, n, 0, u, rw);
        e2m1_sr_block(x, n, s6, inv6, rw, f6);
        block_dither(q, blk0, n, 1, u, rw);
        e2m1_sr_block(x, n, s4, inv4, rw, f4);
    } else {
        for (int i = 0; i < n; ++i) f6[i] = fos_oracle_e2m1_rtn(xs6[i]);
        for (int i = 0; i < n; ++i) f4[i] = fos_oracle_e2m1_rtn(xs4[i]);
    }
    float sf6 = fos_oracle_e4m3_to_f32(s6), sf4 = fos_oracle_e4m3_to_f32(s4);
    for (int i = 0; i < n; ++i) {
        d6[i] = ((f6[i] * sf6) * q->amax) / q->errdiv;
        d4[i] = ((f4[i] * sf4) * q->amax) / q->errdiv;
    }
    float e4 = block_error(q->rule, d4, x, n);
    float e6 = block_error(q->rule, d6, x, n);
    int pick4 = e4 < e6;
    if (err2) { err2[0] = e6; err2[1] = e4; }
    memcpy(fq, pick4 ? f4 : f6, sizeof(float) * (size_t)n);
    *s_out = pick4 ? s4 : s6;
}

static double adj_of(int round_style) {
    return round_style == ROUND_STOCHASTIC_UNBIASED ? 16.0 / 17.0 : 1.0;
}

/*
 * Quantize a padded bf16 matrix x[M,N] (M % 128 == 0 only matters to the caller's scale
 * layout; here M % 16 == 0 if block2d, N % 16 == 0).
 *   codes : u8 [M, N/2], low nibble = even column
 *   sf    : u8 [M, N/16] row-major (one byte per 1x16 block; 2D tiles repeat theirs)
 *   amax  : f32 max|x|
 * Returns 0, or -1 on an unsupported combination.
 */
/* `amax_in` (may be NULL) is the reference function's x_amax argument (reference.py:557,
 * 573-578): the tensor scale to use instead of max|x|. */
/* fp16 bits -> fp32 (exact). */
static inline float f16_to_f32(uint16_t h) {
    const uint32_t e = (h >> 10) & 31u, m = h & 1023u;
    float v;
    if (e == 0) v = ldexpf((float)m, -24);
    else if (e == 31) v = m ? NAN : INFINITY;
    else v = ldexpf((float)(m | 1024u), (int)e - 25);
    return (h & 0x8000u) ? -v : v;
}

/* Element i of an input of type x_type (0 bf16, 1 fp16: 16-bit patterns; 2 fp32) as fp32:
 * the reference converts whatever it is given with `.float()` (reference.py:577,593,596). */
static inline float load_x(const void *x, int x_type, int64_t i) {
    if (x_type == 2) return ((const float *)x)[i];
    const uint16_t h = ((const uint16_t *)x)[i];
    return x_type == 1 ? f16_to_f32(h) : bf16_to_f32(h);
}

/* `errors` (may be NULL): f32 [M, N/16, 2], the two selection errors the adaptive rules
 * compared for each 1x16 block (first candidate "6" / E2M1, second "4" / INT4; a 16x16
 * tile repeats its pair on its 16 rows; zeros for the static rules) -- what the tests use to
 * find blocks whose candidates nearly tie. */
static int quantize_typed(const void *x, int x_type, int64_t M, int64_t N, int dtype, int rule,
                          int round_style, int block2d, uint64_t seed, uint64_t offset,
                          uint8_t *codes, uint8_t *sf, float *amax_out, const float *amax_in,
                          int nthreads, float *errors) {
    if (x_type < 0 || x_type > 2) return -1;
    if (N % 16 != 0 || (block2d && M % 16 != 0)) return -1;
    if (dtype != FOS_NVFP4 && dtype != FOS_IF4) return -1;
    if (dtype == FOS_IF4 && (rule == RULE_STATIC6 || rule == RULE_STATIC4)) return -1;
    if (rule < 0 || rule > 4) return -1;

    float amax = 0.0f;
    if (amax_in) {
        amax = *amax_in;
    } else {
        for (int64_t i = 0; i < M * N; ++i) {
            float a = fabsf(load_x(x, x_type, i));
            if (a > amax) amax = a;
        }
    }
    *amax_out = amax;

    qctx q;
    memset(&q, 0, sizeof q);
    q.dtype = dtype; q.rule = rule; q.round_style = round_style; q.block2d = block2d;
    q.amax = amax; q.seed = seed; q.offset = offset; q.blocks_per_row = N / 16;
    double adj = adj_of(round_style);
    /* (qmax, smax): static_6 (6,448), static_4 (4,448), adaptive nvfp4 (6,256), if4 (6,448) */
    double qmax = (rule == RULE_STATIC4) ? 4.0 : 6.0;
    double smax = (dtype == FOS_IF4 || rule == RULE_STATIC6 || rule == RULE_STATIC4) ? 448.0 : 256.0;
    q.c = (float)(qmax * smax * adj);
    q.qdiv = (float)(qmax * adj);
    q.enc = q.c / amax;
    q.dec = 1.0f / (q.c / amax);
    q.errdiv = (dtype == FOS_IF4) ? (float)(6.0 * 448.0 * adj) : (float)(6.0 * 256.0 * adj);

    int64_t bpr = N / 16;
    if (nthreads < 1) nthreads = 1;
    if (!block2d) {
#pragma omp parallel for num_threads(nthreads) schedule(static)
        for (int64_t r = 0; r < M; ++r) {
            float xb[16], fq[16];
            for (int64_t cb = 0; cb < bpr; ++cb) {
                for (int i = 0; i < 16; ++i) xb[i] = load_x(x, x_type, r * N + cb * 16 + i);
                int is_int; uint8_t s;
                quantize_block(&q, xb, 16, (uint64_t)(r * bpr + cb), fq, &is_int, &s,
                               errors ? errors + 2 * (r * bpr + cb) : NULL);
                sf[r * bpr + cb] = s;
                uint8_t *dst = codes + r * (N / 2) + cb * 8;
                for (int i = 0; i < 8; ++i) {
                    uint8_t lo = is_int ? int4_code_from_fq(fq[2 * i]) : e2m1_code_from_fq(fq[2 * i]);
                    uint8_t hi = is_int ? int4_code_from_fq(fq[2 * i + 1]) : e2m1_code_from_fq(fq[2 * i + 1]);
                    dst[i] = (uint8_t)((hi << 4) | lo);
                }
            }
        }
    } else {
#pragma omp parallel for num_threads(nthreads) schedule(static)
        for (int64_t rt = 0; rt < M / 16; ++rt) {
            float xb[256], fq[256];
            for (int64_t cb = 0; cb < bpr; ++cb) {
                for (int r = 0; r < 16; ++r)
                    for (int i = 0; i < 16; ++i)
                        xb[16 * r + i] = load_x(x, x_type, (rt * 16 + r) * N + cb * 16 + i);
                int is_int; uint8_t s;
                float e2[2];
                quantize_block(&q, xb, 256, (uint64_t)(rt * 16 * bpr + cb), fq, &is_int, &s, e2);
                for (int r = 0; r < 16; ++r) {
                    if (errors) {
                        errors[2 * ((rt * 16 + r) * bpr + cb)] = e2[0];
                        errors[2 * ((rt * 16 + r) * bpr + cb) + 1] = e2[1];
                    }
                    sf[(rt * 16 + r) * bpr + cb] = s;
                    uint8_t *dst = codes + (rt * 16 + r) * (N / 2) + cb * 8;
                    const float *f = fq + 16 * r;
                    for (int i = 0; i < 8; ++i) {
                        uint8_t lo = is_int ? int4_code_from_fq(f[2 * i]) : e2m1_code_from_fq(f[2 * i]);
                        uint8_t hi = is_int ? int4_code_from_fq(f[2 * i + 1]) : e2m1_code_from_fq(f[2 * i + 1]);
                        dst[i] = (uint8_t)((hi << 4) | lo);
                    }
                }
            }
        }
    }
    return 0;
}

int fos_oracle_quantize_typed(const void *x, int x_type, int64_t M, int64_t N, int dtype, int rule,
                              int round_style, int block2d, uint64_t seed, uint64_t offset,
                              uint8_t *codes, uint8_t *sf, float *amax_out, const float *amax_in,
                              int nthreads) {
    return quantize_typed(x, x_type, M, N, dtype, rule, round_style, block2d, seed, offset, codes, sf, amax_out,
                          amax_in, nthreads, NULL);
}

/* fos_oracle_quantize_typed that also reports the selection errors (see quantize_typed). */
int fos_oracle_quantize_errors(const void *x, int x_type, int64_t M, int64_t N, int dtype, int rule,
                               int round_style, int block2d, uint64_t seed, uint64_t offset,
                               uint8_t *codes, uint8_t *sf, float *amax_out, const float *amax_in,
                               int nthreads, float *errors) {
    return quantize_typed(x, x_type, M, N, dtype, rule, round_style, block2d, seed, offset, codes, sf, amax_out,
                          amax_in, nthreads, errors);
}

int fos_oracle_quantize_with_amax(const uint16_t *x, int64_t M, int64_t N, int dtype, int rule,
                                  int round_style, int block2d, uint64_t seed, uint64_t offset,
                                  uint8_t *codes, uint8_t *sf, float *amax_out, const float *amax_in,
                                  int nthreads) {
    return fos_oracle_quantize_typed(x, 0, M, N, dtype, rule, round_style, block2d, seed, offset, codes, sf, amax_out,
                                     amax_in, nthreads);
}

int fos_oracle_quantize(const uint16_t *x, int64_t M, int64_t N, int dtype, int rule,
                        int round_style, int block2d, uint64_t seed, uint64_t offset,
                        uint8_t *codes, uint8_t *sf, float *amax_out, int nthreads) {
    return fos_oracle_quantize_with_amax(x, M, N, dtype, rule, round_style, block2d, seed, offset, codes, sf,
                                         amax_out, NULL, nthreads);
}

/* ---- scale layout ------------------------------------------------------------------ */

/* Offset of scale (r, c) of an [rows, cols] grid in the 128x4-tile layout produced by
 * to_blocked (quantize/utils.py:88-96). */
int64_t fos_oracle_blocked_offset(int64_t r, int64_t c, int64_t cols) {
    return ((r / 128) * (cols / 4) + c / 4) * 512 + (r % 32) * 16 + ((r % 128) / 32) * 4 + c % 4;
}

void fos_oracle_to_blocked(const uint8_t *lin, int64_t rows, int64_t cols, uint8_t *blk) {
    for (int64_t r = 0; r < rows; ++r)
        for (int64_t c = 0; c < cols; ++c)
            blk[fos_oracle_blocked_offset(r, c, cols)] = lin[r * cols + c];
}

void fos_oracle_from_blocked(const uint8_t *blk, int64_t rows, int64_t cols, uint8_t *lin) {
    for (int64_t r = 0; r < rows; ++r)
        for (int64_t c = 0; c < cols; ++c)
            lin[r * cols + c] = blk[fos_oracle_blocked_offset(r, c, cols)];
}

/* ---- dequantize (quantize/backend.py:89-160, fp16 intermediate) -------------------- */

/* codes u8[M,N/2], sf row-major u8[M,N/16], out f32[M,N].  div = qmax*smax*adj of the
 * tensor's scale rule, as a double (it is rounded to f32 for the division, as torch
 * does for a Python-scalar divisor). */
/* `f32_intermediate`: value and block scale meet in fp32 instead of fp16
 * (dequantize(..., intermediate_dtype=torch.float32), quantize/backend.py:89-160). */
int fos_oracle_dequantize_ex(const uint8_t *codes, const uint8_t *sf, float amax, int dtype,
                             double div, int64_t M, int64_t N, float *out, int nthreads, int f32_intermediate) {
    if (N % 16 != 0) return -1;
    float fdiv = (float)div;
    float six_sevenths = (float)(6.0 / 7.0);
    if (nthreads < 1) nthreads = 1;
#pragma omp parallel for num_threads(nthreads) schedule(static)
    for (int64_t r = 0; r < M; ++r) {
        for (int64_t cb = 0; cb < N / 16; ++cb) {
            uint8_t sb = sf[r * (N / 16) + cb];
            int is_int = (dtype == FOS_IF4) && (sb & 0x80);
            float s = (dtype == FOS_IF4) ? fos_oracle_e4m3_to_f32(sb & 0x7f) : fos_oracle_e4m3_to_f32(sb);
            for (int i = 0; i < 16; ++i) {
                uint8_t byte = codes[r * (N / 2) + cb * 8 + i / 2];
                uint8_t code = (i & 1) ? (byte >> 4) : (byte & 0xf);
                float v;
                if (is_int) {
                    int iv = (int8_t)(code << 4) >> 4;
                    v = (float)iv * six_sevenths;
                    if (!f32_intermediate) v = round_to_f16(v);
                } else {
                    v = fos_oracle_e2m1_decode(code);
                }
                float prod = f32_intermediate ? v * s : round_to_f16(v * s);
                out[r * N + cb * 16 + i] = (prod * amax) / fdiv;
            }
        }
    }
    return 0;
}

int fos_oracle_dequantize(const uint8_t *codes, const uint8_t *sf, float amax, int dtype,
                          double div, int64_t M, int64_t N, float *out, int nthreads) {
    return fos_oracle_dequantize_ex(codes, sf, amax, dtype, div, M, N, out, nthreads, 0);
}

/* ---- matmul oracle (matmul/pytorch.py:42-52) --------------------------------------- */

/* out[M,N] (bf16 bits) = bf16(f32(sum_k a[m,k] * b[n,k])), accumulated in double. */
void fos_oracle_matmul_nt(const float *a, const float *b, int64_t M, int64_t N, int64_t K,
                          uint16_t *out_bf16, float *out_f32, int nthreads) {
    if (nthreads < 1) nthreads = 1;
#pragma omp parallel for num_threads(nthreads) schedule(static)
    for (int64_t m = 0; m < M; ++m) {
        for (int64_t n = 0; n < N; ++n) {
            const float *pa = a + m * K, *pb = b + n * K;
            double acc0 = 0.0, acc1 = 0.0, acc2 = 0.0, acc3 = 0.0;
            int64_t k = 0;
            for (; k + 4 <= K; k += 4) {
                acc0 += (double)pa[k] * pb[k];
                acc1 += (double)pa[k + 1] * pb[k + 1];
                acc2 += (double)pa[k + 2] * pb[k + 2];
                acc3 += (double)pa[k + 3] * pb[k + 3];
            }
            for (; k < K; ++k) acc0 += (double)pa[k] * pb[k];
            float f = (float)((acc0 + acc1) + (acc2 + acc3));
            if (out_f32) out_f32[m * N + n] = f;
            if (out_bf16) out_bf16[m * N + n] = f32_to_bf16(f);
        }
    }
}

/* CUTLASS-form product (matmul/cutlass/backend.py:86-98 + csrc/fp4_gemm.cu:143):
 * out = bf16(alpha * sum_k (vA*sA)(vB*sB)) straight from codes and row-major scales. */
void fos_oracle_gemm_nvfp4(const uint8_t *A, const uint8_t *B, const uint8_t *sfa,
                           const uint8_t *sfb, float alpha, int64_t M, int64_t N, int64_t K,
                           uint16_t *out_bf16, float *out_f32, int nthreads) {
    float *a = (float *)malloc(sizeof(float) * (size_t)(M * K));
    float *b = (float *)malloc(sizeof(float) * (size_t)(N * K));
    for (int64_t m = 0; m < M; ++m)
        for (int64_t k = 0; k < K; ++k) {
            uint8_t byte = A[m * (K / 2) + k / 2];
            uint8_t code = (k & 1) ? (byte >> 4) : (byte & 0xf);
            a[m * K + k] = fos_oracle_e2m1_decode(code) * fos_oracle_e4m3_to_f32(sfa[m * (K / 16) + k / 16]);
        }
    for (int64_t n = 0; n < N; ++n)
        for (int64_t k = 0; k < K; ++k) {
            uint8_t byte = B[n * (K / 2) + k / 2];
            uint8_t code = (k & 1) ? (byte >> 4) : (byte & 0xf);
            b[n * K + k] = fos_oracle_e2m1_decode(code) * fos_oracle_e4m3_to_f32(sfb[n * (K / 16) + k / 16]);
        }
    if (nthreads < 1) nthreads = 1;
#pragma omp parallel for num_threads(nthreads) schedule(static)
    for (int64_t m = 0; m < M; ++m) {
        for (int64_t n = 0; n < N; ++n) {
            const float *pa = a + m * K, *pb = b + n * K;
            double acc = 0.0;
            for (int64_t k = 0; k < K; ++k) acc += (double)pa[k] * pb[k];
            float f = alpha * (float)acc;
            if (out_f32) out_f32[m * N + n] = f;
            if (out_bf16) out_bf16[m * N + n] = f32_to_bf16(f);
        }
    }
    free(a);
    free(b);
}
