// gfx950 quantize path: tensor-wide max|x| (pass 1) and block-scaled 4-bit quantisation
// with E4M3 block scales (pass 2).
//
// Arithmetic follows the reference's PyTorch backend operation by operation
// (src/fouroversix/quantize/pytorch/reference.py:30-63, 184-552; one IEEE fp32 rounding
// per reference operation, torch.sum's summation order for the mse/mae decisions), so
// the packed codes and scale bytes are bit-identical to it for round-to-nearest.
//
// Work decomposition (pass 2): one lane owns one 1x16 block (32 contiguous input bytes,
// two 128-bit loads; 8 output bytes, one 64-bit store).  A wavefront covers 16 rows x 4
// blocks with the 16 rows of a 16x16 tile laid along one DPP row, so the 2-D tile
// reductions are DPP row operations.  A 256-thread workgroup covers 128 rows x (64*T)
// columns, i.e. T complete 128x4 scale tiles, which it assembles in LDS and writes as
// contiguous 512-byte runs.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "fos_device.h"
#include "fouroversix_hip.h"

namespace fos {

constexpr int kThreads = 256;
constexpr int kMaxPartials = 1024;

struct QuantParams {
    const uint16_t *x;
    int64_t rows, cols, ld;      // logical input
    int64_t rows_p, cols_p;      // padded output extents
    uint8_t *codes;              // [rows_p, cols_p / 2]
    uint8_t *sf;                 // rows_p * cols_p / 16 bytes
    const uint32_t *partials;    // per-workgroup maxima of pass 1 (f32 bit patterns >= 0)
    int n_partials;
    float *amax_out;             // written by workgroup 0 when not null
    uint64_t seed, offset;
    int sf_layout;
    int tiles_x;                 // workgroup tiles along the columns
    float c, qdiv, errdiv;       // f32(qmax*smax*adj), f32(qmax*adj), selection divisor
};

// ---------------------------------------------------------------------------------------
// pass 1: per-workgroup max |x| as an integer max over the magnitude bits
// ---------------------------------------------------------------------------------------

template <bool IS_BF16>
FOS_DEVICE uint32_t mag16_to_f32_bits(uint32_t m) {
    if (IS_BF16) return m << 16;
    _Float16 h = __builtin_bit_cast(_Float16, (uint16_t)m);
    return f2u((float)h);
}

FOS_DEVICE uint32_t pk_max_u16(uint32_t a, uint32_t b) {
    typedef uint16_t u16x2 __attribute__((ext_vector_type(2)));
    u16x2 va = __builtin_bit_cast(u16x2, a), vb = __builtin_bit_cast(u16x2, b);
    u16x2 r = __builtin_elementwise_max(va, vb);
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

// Contiguous, 16-byte aligned input viewed as n_vec 128-bit vectors.
template <bool IS_BF16>
__global__ __launch_bounds__(kThreads) void amax_flat_kernel(const uint4 *__restrict__ x, int64_t n_vec,
                                                             uint32_t *__restrict__ partials) {
    __shared__ uint32_t smem[4];
    const int64_t stride = (int64_t)gridDim.x * kThreads;
    int64_t i = (int64_t)blockIdx.x * kThreads + threadIdx.x;
    uint32_t m = 0;
    constexpr int U = 8;
    for (; i + (U - 1) * stride < n_vec; i += U * stride) {
        uint4 v[U];
#pragma unroll
        for (int u = 0; u < U; ++u) v[u] = x[i + u * stride];
#pragma unroll
        for (int u = 0; u < U; ++u) {
            m = pk_max_u16(m, v[u].x & 0x7fff7fffu);
            m = pk_max_u16(m, v[u].y & 0x7fff7fffu);
            m = pk_max_u16(m, v[u].z & 0x7fff7fffu);
            m = pk_max_u16(m, v[u].w & 0x7fff7fffu);
        }
    }
    for (; i < n_vec; i += stride) {
        uint4 v = x[i];
        m = pk_max_u16(m, v.x & 0x7fff7fffu);
        m = pk_max_u16(m, v.y & 0x7fff7fffu);
        m = pk_max_u16(m, v.z & 0x7fff7fffu);
        m = pk_max_u16(m, v.w & 0x7fff7fffu);
    }
    uint32_t mm = (m & 0xffffu) > (m >> 16) ? (m & 0xffffu) : (m >> 16);
    mm = block_max_u32(mm, smem);
    if (threadIdx.x == 0) partials[blockIdx.x] = mag16_to_f32_bits<IS_BF16>(mm);
}

// Any strides / alignment: one workgroup per row, strided over the rows.
template <bool IS_BF16>
__global__ __launch_bounds__(kThreads) void amax_rows_kernel(const uint16_t *__restrict__ x, int64_t rows,
                                                             int64_t cols, int64_t ld,
                                                             uint32_t *__restrict__ partials) {
    __shared__ uint32_t smem[4];
    uint32_t m = 0;
    for (int64_t r = blockIdx.x; r < rows; r += gridDim.x) {
        const uint16_t *row = x + r * ld;
        for (int64_t c = threadIdx.x; c < cols; c += kThreads) {
            uint32_t v = row[c] & 0x7fffu;
            m = m > v ? m : v;
        }
    }
    m = block_max_u32(m, smem);
    if (threadIdx.x == 0) partials[blockIdx.x] = mag16_to_f32_bits<IS_BF16>(m);
}

// partials -> one f32 (single workgroup)
__global__ __launch_bounds__(kThreads) void amax_finalize_kernel(const uint32_t *__restrict__ partials, int n,
                                                                 float *__restrict__ amax) {
    __shared__ uint32_t smem[4];
    uint32_t m = 0;
    for (int i = threadIdx.x; i < n; i += kThreads) m = m > partials[i] ? m : partials[i];
    m = block_max_u32(m, smem);
    if (threadIdx.x == 0) *amax = u2f(m);
}

// ---------------------------------------------------------------------------------------
// pass 2 building blocks
// ---------------------------------------------------------------------------------------

struct QuantConsts {
    float amax, enc, dec, qdiv, errdiv;
};

// compute_nv_scale_factors (reference.py:184-241) for one block maximum.
FOS_DEVICE void block_scale(const QuantConsts &k, float bmax, bool expand, uint32_t &s, float &sf, float &inv) {
    float s_hp = (k.amax == 0.0f) ? 0.0f : (bmax / k.qdiv) * k.enc;
    if (expand) s_hp = s_hp * 1.5f;
    s = e4m3_encode(s_hp);
    sf = e4m3_decode(s);
    inv = 1.0f / (k.dec * sf);
}

// E2M1 grid rounding of a magnitude (reference.py:30-51).  Round-to-nearest has no clamp
// (a magnitude in [7, 9) gives 8, which the nibble encoding below spills into bit 3
// exactly as the reference's bit extraction does); the dithered variant clamps to 6.
template <bool SR>
FOS_DEVICE float e2m1_round(float a, float u) {
    float r;
    if (SR) {
        float r1 = __builtin_rintf((a + a) + u) * 0.5f;
        float r2 = __builtin_rintf(a + u);
        float r3 = fminf(2.0f * __builtin_rintf(a * 0.5f + u), 6.0f);
        r = a < 2.0f ? r1 : (a < 4.0f ? r2 : r3);
        r = (r == 0.0f) ? 0.0f : r;
    } else {
        float r1 = __builtin_rintf(a + a) * 0.5f;
        float r2 = __builtin_rintf(a);
        float r3 = 2.0f * __builtin_rintf(a * 0.5f);
        r = a < 2.0f ? r1 : (a < 4.0f ? r2 : r3);
    }
    return r;
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

// Dither for the 16 elements of 1x16 block `blk`, candidate `cand`.
FOS_DEVICE void dither16(uint64_t seed, uint64_t offset, uint64_t blk, int cand, float *u) {
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        Philox4 p = philox4x32_10((uint32_t)blk, (uint32_t)(blk >> 32), (uint32_t)(4 * cand + j),
                                  (uint32_t)offset, (uint32_t)seed, (uint32_t)(seed >> 32));
#pragma unroll
        for (int i = 0; i < 4; ++i) u[4 * j + i] = dither_from_word(p.v[i]);
    }
}

// One 1x16 block (one row of a 16x16 tile when TWO_D): 8 input words -> 2 code words
// and the scale byte.  `blk` = row * (cols_p / 16) + block column keys the dither.
template <int DT, int RULE, int ROUND, bool TWO_D>
FOS_DEVICE void quantize_block(const uint32_t *w, const QuantConsts &k, uint64_t seed, uint64_t offset,
                               uint64_t blk, uint32_t *codes, uint32_t &sbyte) {
    constexpr bool SR = ROUND != FOS_ROUND_NEAREST;
    constexpr bool STATIC = (RULE == FOS_RULE_STATIC_6 || RULE == FOS_RULE_STATIC_4);
    float x[16];
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        x[2 * i] = u2f(w[i] << 16);
        x[2 * i + 1] = u2f(w[i] & 0xffff0000u);
    }
    float bmax = 0.0f;
#pragma unroll
    for (int i = 0; i < 16; i += 2) bmax = fmaxf(fmaxf(fabsf(x[i]), fabsf(x[i + 1])), bmax);
    if (TWO_D) bmax = row16_max(bmax);

    uint32_t sA;
    float sfA, invA;
    block_scale(k, bmax, false, sA, sfA, invA);
    float uA[16], uB[16];
    if (SR) dither16(seed, offset, blk, 0, uA);

    if (STATIC) {
        uint32_t c0 = 0, c1 = 0;
#pragma unroll
        for (int i = 0; i < 16; ++i) {
            float xs = (sA != 0) ? x[i] * invA : 0.0f;
            float r = e2m1_round<SR>(fabsf(xs), SR ? uA[i] : 0.0f);
            uint32_t nib = e2m1_mag_code(r) | ((xs < 0.0f) ? 8u : 0u);
            if (i < 8) c0 |= nib << (4 * i);
            else c1 |= nib << (4 * (i - 8));
        }
        codes[0] = c0;
        codes[1] = c1;
        sbyte = sA;
        return;
    }

    if (SR) dither16(seed, offset, blk, 1, uB);
    float eA[16], eB[16];
    uint32_t a0 = 0, a1 = 0, b0 = 0, b1 = 0;

    if (DT == FOS_DTYPE_IF4) {
        // select_intfloat (reference.py:328-425): candidate A = E2M1, candidate B = INT4
        // on the same scale; B wins on a strictly smaller error.
#pragma unroll
        for (int i = 0; i < 16; ++i) {
            float xs = (sA != 0) ? x[i] * invA : 0.0f;
            float r = e2m1_round<SR>(fabsf(xs), SR ? uA[i] : 0.0f);
            bool neg = xs < 0.0f;
            float fq = neg ? -r : r;
            uint32_t nibA = e2m1_mag_code(r) | (neg ? 8u : 0u);
            float q = int4_round<SR>(xs * 1.16666666f, SR ? uB[i] : 0.0f);
            uint32_t nibB = (uint32_t)((int)q) & 0xfu;
            float deqA = ((fq * sfA) * k.amax) / k.errdiv;
            float deqB = (((q * sfA) * k.amax) * 0.8571428571f) / k.errdiv;
            eA[i] = error_term<RULE>(deqA, x[i]);
            eB[i] = error_term<RULE>(deqB, x[i]);
            if (i < 8) { a0 |= nibA << (4 * i); b0 |= nibB << (4 * i); }
            else { a1 |= nibA << (4 * (i - 8)); b1 |= nibB << (4 * (i - 8)); }
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
#pragma unroll
    for (int i = 0; i < 16; ++i) {
        float xsA = (sA != 0) ? x[i] * invA : 0.0f;
        float xsB = (sB != 0) ? x[i] * invB : 0.0f;
        float rA = e2m1_round<SR>(fabsf(xsA), SR ? uA[i] : 0.0f);
        float rB = e2m1_round<SR>(fabsf(xsB), SR ? uB[i] : 0.0f);
        bool negA = xsA < 0.0f, negB = xsB < 0.0f;
        uint32_t nibA = e2m1_mag_code(rA) | (negA ? 8u : 0u);
        uint32_t nibB = e2m1_mag_code(rB) | (negB ? 8u : 0u);
        float deqA = (((negA ? -rA : rA) * sfA) * k.amax) / k.errdiv;
        float deqB = (((negB ? -rB : rB) * sfB) * k.amax) / k.errdiv;
        eA[i] = error_term<RULE>(deqA, x[i]);
        eB[i] = error_term<RULE>(deqB, x[i]);
        if (i < 8) { a0 |= nibA << (4 * i); b0 |= nibB << (4 * i); }
        else { a1 |= nibA << (4 * (i - 8)); b1 |= nibB << (4 * (i - 8)); }
    }
    float errA = reduce_error<RULE, TWO_D>(eA);
    float errB = reduce_error<RULE, TWO_D>(eB);
    bool pickB = errB < errA;
    codes[0] = pickB ? b0 : a0;
    codes[1] = pickB ? b1 : a1;
    sbyte = pickB ? sB : sA;
}

// Offset of scale (r, c) inside the 128x4-tile layout (quantize/utils.py:88-96).
FOS_DEVICE int64_t tiled_sf_offset(int64_t r, int64_t c, int64_t sf_cols) {
    return ((r >> 7) * (sf_cols >> 2) + (c >> 2)) * 512 + (r & 31) * 16 + ((r & 127) >> 5) * 4 + (c & 3);
}

// ---------------------------------------------------------------------------------------
// pass 2 kernel
// ---------------------------------------------------------------------------------------

// ALIGNED: x 16-byte aligned, ld % 8 == 0, cols % 16 == 0 -> 128-bit loads.
template <int DT, int RULE, int ROUND, bool TWO_D, int T, bool ALIGNED>
__global__ __launch_bounds__(kThreads) void quantize_kernel(const QuantParams p) {
    __shared__ uint32_t red[4];
    __shared__ uint32_t sf_tile[T * 128];  // T tiles of 512 scale bytes

    // tensor-wide maximum from the pass-1 partials
    uint32_t m = 0;
    for (int i = threadIdx.x; i < p.n_partials; i += kThreads) {
        uint32_t v = p.partials[i];
        m = m > v ? m : v;
    }
    m = block_max_u32(m, red);
    QuantConsts k;
    k.amax = u2f(m);
    k.enc = p.c / k.amax;
    k.dec = 1.0f / (p.c / k.amax);
    k.qdiv = p.qdiv;
    k.errdiv = p.errdiv;
    if (blockIdx.x == 0 && threadIdx.x == 0 && p.amax_out) *p.amax_out = k.amax;

    const int tile_x = blockIdx.x % p.tiles_x;
    const int64_t tile_y = blockIdx.x / p.tiles_x;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int64_t sf_cols = p.cols_p >> 4;
    const int64_t row_base = tile_y * 128 + wave * 16 + (lane & 15);
    const int64_t cb_base = (int64_t)tile_x * (4 * T) + (lane >> 4);

    constexpr int NB = 2 * T;  // blocks per lane: T column groups x 2 row halves
    uint32_t w[NB][8];
#pragma unroll
    for (int it = 0; it < NB; ++it) {
        const int64_t r = row_base + (it & 1) * 64;
        const int64_t cb = cb_base + (it >> 1) * 4;
        const int64_t c0 = cb * 16;
        if (ALIGNED) {
            if (r < p.rows && c0 < p.cols) {
                const uint4 *src = reinterpret_cast<const uint4 *>(p.x + r * p.ld + c0);
                uint4 lo = src[0], hi = src[1];
                w[it][0] = lo.x; w[it][1] = lo.y; w[it][2] = lo.z; w[it][3] = lo.w;
                w[it][4] = hi.x; w[it][5] = hi.y; w[it][6] = hi.z; w[it][7] = hi.w;
            } else {
#pragma unroll
                for (int i = 0; i < 8; ++i) w[it][i] = 0;
            }
        } else {
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                uint32_t lo = 0, hi = 0;
                if (r < p.rows) {
                    const uint16_t *src = p.x + r * p.ld;
                    if (c0 + 2 * i < p.cols) lo = src[c0 + 2 * i];
                    if (c0 + 2 * i + 1 < p.cols) hi = src[c0 + 2 * i + 1];
                }
                w[it][i] = lo | (hi << 16);
            }
        }
    }

#pragma unroll
    for (int it = 0; it < NB; ++it) {
        const int64_t r = row_base + (it & 1) * 64;
        const int64_t cb = cb_base + (it >> 1) * 4;
        if (cb >= sf_cols) continue;  // whole wave-row group lies past the padded width
        uint32_t codes[2], sbyte;
        quantize_block<DT, RULE, ROUND, TWO_D>(w[it], k, p.seed, p.offset,
                                               (uint64_t)(r * sf_cols + cb), codes, sbyte);
        *reinterpret_cast<uint2 *>(p.codes + r * (p.cols_p >> 1) + cb * 8) = make_uint2(codes[0], codes[1]);
        if (p.sf_layout == FOS_SF_TILED_128X4) {
            const int rr = (int)(r & 127);
            reinterpret_cast<uint8_t *>(sf_tile)[(it >> 1) * 512 + (rr & 31) * 16 + (rr >> 5) * 4 + (int)(cb & 3)] =
                (uint8_t)sbyte;
        } else {
            p.sf[r * sf_cols + cb] = (uint8_t)sbyte;
        }
    }

    if (p.sf_layout == FOS_SF_TILED_128X4) {
        __syncthreads();
        // T tiles x 128 words, contiguous in the output when the tiles are in range.
        for (int i = threadIdx.x; i < T * 128; i += kThreads) {
            const int t = i >> 7;
            const int64_t tile_c = (int64_t)tile_x * T + t;  // 4-block column group
            if (tile_c < (sf_cols >> 2)) {
                uint32_t *dst = reinterpret_cast<uint32_t *>(p.sf + (tile_y * (sf_cols >> 2) + tile_c) * 512);
                dst[i & 127] = sf_tile[i];
            }
        }
    }
}

}  // namespace fos

// ---------------------------------------------------------------------------------------
// host side
// ---------------------------------------------------------------------------------------

using namespace fos;

extern "C" int64_t fos_padded_rows(int64_t rows) { return (rows + 127) / 128 * 128; }
extern "C" int64_t fos_padded_cols(int64_t cols) { return (cols + 63) / 64 * 64; }

extern "C" size_t fos_quantize_workspace_bytes(int64_t, int64_t) { return kMaxPartials * sizeof(uint32_t); }

namespace {

// Launch pass 1; returns the number of partial maxima written to `partials`.
int launch_amax(const void *x, int64_t rows, int64_t cols, int64_t ld, bool aligned, uint32_t *partials, hipStream_t s) {
    int n_partials;
    if (ld == cols && aligned) {
        const int64_t n_vec = rows * cols / 8;
        int64_t want = (n_vec + kThreads * 8 - 1) / (kThreads * 8);
        n_partials = (int)(want > kMaxPartials ? kMaxPartials : (want < 1 ? 1 : want));
        hipLaunchKernelGGL((amax_flat_kernel<true>), dim3(n_partials), dim3(kThreads), 0, s, (const uint4 *)x, n_vec,
                           partials);
    } else {
        n_partials = (int)(rows < kMaxPartials ? rows : kMaxPartials);
        hipLaunchKernelGGL((amax_rows_kernel<true>), dim3(n_partials), dim3(kThreads), 0, s, (const uint16_t *)x, rows,
                           cols, ld, partials);
    }
    return n_partials;
}

template <int DT, int RULE, int ROUND, bool TWO_D, int T>
void launch_quantize_t(const QuantParams &p, bool aligned, dim3 grid, hipStream_t s) {
    if (aligned) {
        hipLaunchKernelGGL((quantize_kernel<DT, RULE, ROUND, TWO_D, T, true>), grid, dim3(kThreads), 0, s, p);
    } else if constexpr (T == 1) {
        hipLaunchKernelGGL((quantize_kernel<DT, RULE, ROUND, TWO_D, 1, false>), grid, dim3(kThreads), 0, s, p);
    }
}

template <int DT, int RULE, int ROUND, bool TWO_D>
void launch_quantize(QuantParams &p, bool aligned, hipStream_t s) {
    // Wide tiles (full 128-byte lines of packed output per row) once there are enough
    // workgroups to fill the chip; narrow tiles for small tensors.
    const int64_t tiles_y = p.rows_p / 128;
    const int64_t groups = p.cols_p / 64;
    if (aligned && groups % 4 == 0 && tiles_y * (groups / 4) >= 1024) {
        p.tiles_x = (int)(groups / 4);
        launch_quantize_t<DT, RULE, ROUND, TWO_D, 4>(p, aligned, dim3((unsigned)(tiles_y * p.tiles_x)), s);
    } else {
        p.tiles_x = (int)groups;
        launch_quantize_t<DT, RULE, ROUND, TWO_D, 1>(p, aligned, dim3((unsigned)(tiles_y * p.tiles_x)), s);
    }
}

template <int DT, int RULE, int ROUND>
void dispatch_2d(QuantParams &p, bool two_d, bool aligned, hipStream_t s) {
    if (two_d) launch_quantize<DT, RULE, ROUND, true>(p, aligned, s);
    else launch_quantize<DT, RULE, ROUND, false>(p, aligned, s);
}

template <int DT, int RULE>
void dispatch_round(QuantParams &p, int round_style, bool two_d, bool aligned, hipStream_t s) {
    if (round_style == FOS_ROUND_NEAREST) dispatch_2d<DT, RULE, FOS_ROUND_NEAREST>(p, two_d, aligned, s);
    else dispatch_2d<DT, RULE, FOS_ROUND_STOCHASTIC>(p, two_d, aligned, s);
}

}  // namespace

extern "C" int fos_amax(const void *x, int x_type, int64_t rows, int64_t cols, int64_t ld, float *amax,
                        void *workspace, size_t workspace_bytes, fos_stream_t stream) {
    if (!x || !amax) return FOS_E_NULL_POINTER;
    if (rows <= 0 || cols <= 0 || ld < cols) return FOS_E_BAD_SHAPE;
    if (x_type != FOS_T_BF16) return FOS_E_UNSUPPORTED;
    if (!workspace || workspace_bytes < fos_quantize_workspace_bytes(rows, cols)) return FOS_E_WORKSPACE;
    if (((uintptr_t)x & 1) || ((uintptr_t)workspace & 3) || ((uintptr_t)amax & 3)) return FOS_E_BAD_ALIGNMENT;
    hipStream_t s = (hipStream_t)stream;
    const bool aligned = (((uintptr_t)x & 15) == 0) && (ld % 8 == 0) && (cols % 16 == 0);
    uint32_t *partials = (uint32_t *)workspace;
    const int n = launch_amax(x, rows, cols, ld, aligned, partials, s);
    hipLaunchKernelGGL(amax_finalize_kernel, dim3(1), dim3(kThreads), 0, s, partials, n, amax);
    return hipGetLastError() == hipSuccess ? FOS_OK : FOS_E_LAUNCH;
}

extern "C" int fos_quantize(const void *x, int x_type, int64_t rows, int64_t cols, int64_t ld,
                            int dtype, int rule, int round_style, int block2d,
                            uint64_t seed, uint64_t offset, int sf_layout,
                            uint8_t *codes, uint8_t *sf, float *amax, int amax_is_input,
                            void *workspace, size_t workspace_bytes, fos_stream_t stream) {
    if (!x || !codes || !sf || !amax) return FOS_E_NULL_POINTER;
    if (rows <= 0 || cols <= 0 || ld < cols) return FOS_E_BAD_SHAPE;
    if (x_type != FOS_T_BF16) return FOS_E_UNSUPPORTED;
    if (dtype != FOS_DTYPE_NVFP4 && dtype != FOS_DTYPE_IF4) return FOS_E_UNSUPPORTED;
    if (rule < FOS_RULE_STATIC_6 || rule > FOS_RULE_ABS_MAX) return FOS_E_UNSUPPORTED;
    if (round_style < FOS_ROUND_NEAREST || round_style > FOS_ROUND_STOCHASTIC_UNBIASED) return FOS_E_UNSUPPORTED;
    if (dtype == FOS_DTYPE_IF4 && (rule == FOS_RULE_STATIC_6 || rule == FOS_RULE_STATIC_4)) return FOS_E_UNSUPPORTED;
    if (sf_layout != FOS_SF_LINEAR && sf_layout != FOS_SF_TILED_128X4) return FOS_E_UNSUPPORTED;
    if (!workspace || workspace_bytes < fos_quantize_workspace_bytes(rows, cols)) return FOS_E_WORKSPACE;
    if (((uintptr_t)x & 1) || ((uintptr_t)codes & 7) || ((uintptr_t)sf & 3) || ((uintptr_t)workspace & 3) ||
        ((uintptr_t)amax & 3))
        return FOS_E_BAD_ALIGNMENT;
    const int64_t rows_p = fos_padded_rows(rows), cols_p = fos_padded_cols(cols);
    if (rows_p * (cols_p / 64) > 0x7fffffffLL) return FOS_E_BAD_SHAPE;

    hipStream_t s = (hipStream_t)stream;
    uint32_t *partials = (uint32_t *)workspace;
    const bool aligned = (((uintptr_t)x & 15) == 0) && (ld % 8 == 0) && (cols % 16 == 0);

    QuantParams p;
    p.x = (const uint16_t *)x;
    p.rows = rows; p.cols = cols; p.ld = ld;
    p.rows_p = rows_p; p.cols_p = cols_p;
    p.codes = codes; p.sf = sf;
    p.seed = seed; p.offset = offset;
    p.sf_layout = sf_layout;

    if (amax_is_input) {
        p.partials = (const uint32_t *)amax;
        p.n_partials = 1;
        p.amax_out = nullptr;
    } else {
        p.partials = partials;
        p.n_partials = launch_amax(x, rows, cols, ld, aligned, partials, s);
        p.amax_out = amax;
    }

    // (qmax, smax): static_6 (6,448); static_4 (4,448); adaptive NVFP4 (6,256); IF4 (6,448).
    const double adj = round_style == FOS_ROUND_STOCHASTIC_UNBIASED ? 16.0 / 17.0 : 1.0;
    const double qmax = rule == FOS_RULE_STATIC_4 ? 4.0 : 6.0;
    const bool is_static = rule == FOS_RULE_STATIC_6 || rule == FOS_RULE_STATIC_4;
    const double smax = (dtype == FOS_DTYPE_IF4 || is_static) ? 448.0 : 256.0;
    p.c = (float)(qmax * smax * adj);
    p.qdiv = (float)(qmax * adj);
    p.errdiv = dtype == FOS_DTYPE_IF4 ? (float)(6.0 * 448.0 * adj) : (float)(6.0 * 256.0 * adj);

    const bool two_d = block2d != 0;
    if (dtype == FOS_DTYPE_IF4) {
        switch (rule) {
            case FOS_RULE_MAE: dispatch_round<FOS_DTYPE_IF4, FOS_RULE_MAE>(p, round_style, two_d, aligned, s); break;
            case FOS_RULE_MSE: dispatch_round<FOS_DTYPE_IF4, FOS_RULE_MSE>(p, round_style, two_d, aligned, s); break;
            default: dispatch_round<FOS_DTYPE_IF4, FOS_RULE_ABS_MAX>(p, round_style, two_d, aligned, s); break;
        }
    } else {
        switch (rule) {
            case FOS_RULE_STATIC_6:
            case FOS_RULE_STATIC_4:
                // the two static rules differ only in the host-computed constants
                dispatch_round<FOS_DTYPE_NVFP4, FOS_RULE_STATIC_6>(p, round_style, two_d, aligned, s);
                break;
            case FOS_RULE_MAE: dispatch_round<FOS_DTYPE_NVFP4, FOS_RULE_MAE>(p, round_style, two_d, aligned, s); break;
            case FOS_RULE_MSE: dispatch_round<FOS_DTYPE_NVFP4, FOS_RULE_MSE>(p, round_style, two_d, aligned, s); break;
            default: dispatch_round<FOS_DTYPE_NVFP4, FOS_RULE_ABS_MAX>(p, round_style, two_d, aligned, s); break;
        }
    }
    return hipGetLastError() == hipSuccess ? FOS_OK : FOS_E_LAUNCH;
}
