// gfx950 pre-transform of the training-side quantize options: y = x^T and / or the 16-point
// random Hadamard transform of every group of 16 consecutive elements of a row, together
// with the tensor maximum of y -- the steps the reference performs before it scales
// (src/fouroversix/quantize/pytorch/reference.py:567-578; sign vector and matrix
// src/fouroversix/quantize/utils.py:19-85; CUDA form src/fouroversix/csrc/include/
// hadamard_transform.h:16-37).  The result is a plain matrix of the input's type (bf16 or
// fp16) that fos_quantize then reads with `amax_is_input`, so the whole option costs one extra
// write and read of x.
//
// RHT arithmetic: the reference multiplies bf16 [.., 16] by the bf16 matrix
// diag(signs) * H16 / 4 with fp32 accumulation and one rounding to bf16.  All products are
// exact, so the sum is evaluated here as a fast Walsh-Hadamard butterfly in fp32 (64 adds
// instead of 256 multiply-adds) and scaled by 1/4 at the end; the two orders of summation
// agree unless the fp32 partial sums themselves round, i.e. unless a group spans more
// than ~12 binades, and then only when the last fp32 bit decides a bf16 rounding.  fp16 input:
// the reference casts the matrix to the input's type (`had.to(x.dtype)`: +-1/4 is exact) and the
// product is an fp16 matmul -- the same sum, rounded once to fp16.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "fos_buffer.h"
#include "fos_quantize_common.h"
#include "fouroversix_hip.h"

namespace fos {

struct TransformParams {
    const uint16_t *x;
    int64_t rows, cols, ld;  // input
    uint16_t *y;
    int64_t ldy;             // output [cols, rows] if transposed else [rows, cols]
    uint32_t *partials;      // pairs {max |y| as f32 bits, 1 if a -0.0 was written}
    int64_t n_units;         // tiles (transpose) or 16-element groups (rows)
    int tiles_x;
    int vec;                 // x is 16-byte aligned with ld % 8 == 0: whole groups are read as two 128-bit loads
};

// The 16 elements x[r][c0 .. c0 + 15] as packed pairs, zero beyond the last column.
FOS_DEVICE void load_group(const TransformParams &p, int64_t r, int64_t c0, uint32_t *w) {
    if (p.vec && c0 + 16 <= p.cols) {
        const uint4 *src = reinterpret_cast<const uint4 *>(p.x + r * p.ld + c0);
        const uint4 lo = src[0], hi = src[1];
        w[0] = lo.x; w[1] = lo.y; w[2] = lo.z; w[3] = lo.w;
        w[4] = hi.x; w[5] = hi.y; w[6] = hi.z; w[7] = hi.w;
        return;
    }
    const uint16_t *row = p.x + r * p.ld;
#pragma unroll
    for (int j = 0; j < 8; ++j) {
        const uint32_t a = c0 + 2 * j < p.cols ? row[c0 + 2 * j] : 0u, b = c0 + 2 * j + 1 < p.cols ? row[c0 + 2 * j + 1] : 0u;
        w[j] = a | (b << 16);
    }
}

typedef float float2_tt __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x2_tt __attribute__((ext_vector_type(2)));

// signs of the reference's fixed vector as a bit mask (bit i set: element i is negated)
constexpr uint32_t kRhtNegMask = (1u << 3) | (1u << 5) | (1u << 6) | (1u << 7) | (1u << 8) | (1u << 9) | (1u << 10) |
                                 (1u << 12) | (1u << 14) | (1u << 15);

// w[0..7]: 16 bf16 / fp16 (element 2j in the low half of w[j]) -> RHT -> 16 of the same type, same packing.
template <bool F16>
FOS_DEVICE void rht16(uint32_t *w) {
    float v[16];
#pragma unroll
    for (int j = 0; j < 8; ++j) {
        if (F16) {
            // the sign bit of the 16-bit pattern is flipped before the conversion
            const uint32_t flipped = w[j] ^ (((kRhtNegMask >> (2 * j)) & 1u) << 15) ^ (((kRhtNegMask >> (2 * j + 1)) & 1u) << 31);
            v[2 * j] = (float)__builtin_bit_cast(_Float16, (uint16_t)(flipped & 0xffffu));
            v[2 * j + 1] = (float)__builtin_bit_cast(_Float16, (uint16_t)(flipped >> 16));
        } else {
            v[2 * j] = u2f((w[j] << 16) ^ (((kRhtNegMask >> (2 * j)) & 1u) << 31));
            v[2 * j + 1] = u2f((w[j] & 0xffff0000u) ^ (((kRhtNegMask >> (2 * j + 1)) & 1u) << 31));
        }
    }
#pragma unroll
    for (int len = 1; len < 16; len <<= 1) {
#pragma unroll
        for (int i = 0; i < 16; ++i) {
            if ((i & len) == 0) {
                const float a = v[i], b = v[i + len];
                v[i] = a + b;
                v[i + len] = a - b;
            }
        }
    }
#pragma unroll
    for (int j = 0; j < 8; ++j) {
        // + 0.0f: a dot product accumulated from +0 never yields -0
        const float2_tt q = {v[2 * j] * 0.25f + 0.0f, v[2 * j + 1] * 0.25f + 0.0f};
        if (F16)
            w[j] = (uint32_t)__builtin_bit_cast(uint16_t, (_Float16)q.x) | ((uint32_t)__builtin_bit_cast(uint16_t, (_Float16)q.y) << 16);
        else
            w[j] = __builtin_bit_cast(uint32_t, __builtin_convertvector(q, bf16x2_tt));
    }
}

FOS_DEVICE void track(const uint32_t *w, uint32_t &m, uint32_t &z) {
#pragma unroll
    for (int j = 0; j < 8; ++j) {
        m = pk_max_u16(m, w[j] & 0x7fff7fffu);
        z = pk_min_i16(z, w[j]);
    }
}

// (magnitudes of either 16-bit type order like their bit patterns)
template <bool F16>
FOS_DEVICE void write_partials(uint32_t m, uint32_t z, uint32_t *partials) {
    __shared__ uint32_t smem[4];
    uint32_t mm = (m & 0xffffu) > (m >> 16) ? (m & 0xffffu) : (m >> 16);
    mm = block_max_u32(mm, smem);
    const uint32_t zz = block_max_u32(((z & 0xffffu) == 0x8000u || (z >> 16) == 0x8000u) ? 1u : 0u, smem);
    if (threadIdx.x == 0) {
        partials[2 * blockIdx.x] = F16 ? f2u((float)__builtin_bit_cast(_Float16, (uint16_t)mm)) : mm << 16;
        partials[2 * blockIdx.x + 1] = zz;
    }
}

// RHT without transposition: one thread per group of 16, grid-stride.  A lane's 32 output bytes would leave
// as two stores of 16, each instruction covering half of every line; where the wavefront's 64 groups are
// consecutive in one row (cols % 1024 == 0) they are exchanged through 2 KiB of LDS instead, so that lane l
// stores the 16-byte pieces l and 64 + l of the 2 KiB run: whole lines per instruction, stored non-temporally.
template <bool F16>
__global__ __launch_bounds__(kThreads) void rht_rows_kernel(const TransformParams p) {
    __shared__ __attribute__((aligned(16))) uint4 swap[kThreads / 64][128];
    const int64_t groups_per_row = (p.cols + 15) >> 4;  // a last, partial group is completed with zeros
    const bool runs = (groups_per_row & 63) == 0;        // (then n_units % 64 == 0 as well: whole wavefronts)
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    uint32_t m = 0, z = 0;
    for (int64_t g = (int64_t)blockIdx.x * kThreads + threadIdx.x; g < p.n_units; g += (int64_t)gridDim.x * kThreads) {
        const int64_t r = g / groups_per_row, cb = g - r * groups_per_row;
        uint32_t w[8];
        load_group(p, r, cb * 16, w);
        rht16<F16>(w);
        track(w, m, z);
        uint4 *dst = reinterpret_cast<uint4 *>(p.y + r * p.ldy + cb * 16);
        if (runs) {
            swap[wave][2 * lane] = make_uint4(w[0], w[1], w[2], w[3]);
            swap[wave][2 * lane + 1] = make_uint4(w[4], w[5], w[6], w[7]);
            // (LDS operations of one wavefront complete in order: its own writes are visible to its reads)
            __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
            __builtin_amdgcn_wave_barrier();
            __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
            const uint4 a = swap[wave][lane], b = swap[wave][64 + lane];
            __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
            __builtin_amdgcn_wave_barrier();
            uint4 *run = dst - 2 * lane;  // the wavefront's first group
            stream_store(run + lane, a);
            stream_store(run + 64 + lane, b);
        } else {
            dst[0] = make_uint4(w[0], w[1], w[2], w[3]);
            dst[1] = make_uint4(w[4], w[5], w[6], w[7]);
        }
    }
    write_partials<F16>(m, z, p.partials);
}

// Transposition (optionally followed by the RHT along the new rows) through an LDS tile of 64 rows x 128
// columns of x: rows of x come in as 256-byte runs (eight threads to a row), rows of y leave as 128-byte
// runs (four threads to a row of y, which holds 64 elements of this tile).  Groups of 16 that reach past
// the last row / column are completed with zeros (y is written in whole groups: its rows hold a multiple of
// 16 elements).
constexpr int kTR = 64, kTC = 128;  // tile rows / columns of x (64 x 64: 3 % slower; 64 x 256, 128 x 128, 128 x 256: 1-4 % slower)
template <bool RHT, bool F16>
__global__ __launch_bounds__(kThreads) void transpose_kernel(const TransformParams p) {
    constexpr int kPitchT = kTC + 2;  // halfs per LDS row: an odd number of dwords, so a column walk changes bank every row
    __shared__ uint16_t tile[kTR * kPitchT];
    const int t = threadIdx.x;
    uint32_t m = 0, z = 0;
    constexpr int kChunks = kTC / 16, kRowsPerPass = kThreads / kChunks;
    // this thread's two groups of 16 input elements of tile u (rows t / 8 and 32 + t / 8, columns 16 (t % 8) ...)
    auto fetch = [&](int64_t u, uint32_t (&w)[kTR / kRowsPerPass][8]) {
        const int64_t ty = u / p.tiles_x, tx = u - ty * p.tiles_x;
#pragma unroll
        for (int i = 0; i < kTR / kRowsPerPass; ++i) {
            const int64_t r = ty * kTR + t / kChunks + kRowsPerPass * i, c = tx * kTC + (t % kChunks) * 16;
#pragma unroll
            for (int j = 0; j < 8; ++j) w[i][j] = 0;
            if (r < p.rows && c < p.cols) load_group(p, r, c, w[i]);
        }
    };
    uint32_t next[kTR / kRowsPerPass][8];
    if ((int64_t)blockIdx.x < p.n_units) fetch(blockIdx.x, next);
    for (int64_t u = blockIdx.x; u < p.n_units; u += gridDim.x) {
        const int64_t ty = u / p.tiles_x, tx = u - ty * p.tiles_x;
        const int64_t r0 = ty * kTR, c0 = tx * kTC;
#pragma unroll
        for (int i = 0; i < kTR / kRowsPerPass; ++i) {
            const int row = t / kChunks + kRowsPerPass * i, chunk = t % kChunks;
            uint32_t *d = reinterpret_cast<uint32_t *>(tile + row * kPitchT + chunk * 16);
#pragma unroll
            for (int j = 0; j < 8; ++j) d[j] = next[i][j];
        }
        __syncthreads();
        // the next tile's loads are in flight while this one is turned round and written
        if (u + gridDim.x < p.n_units) fetch(u + gridDim.x, next);
        {
            // a thread turns one group of 16 rows of a column PAIR round: 16 dword reads (row stride 65 dwords:
            // the 64 lanes of a wavefront, 4 row groups x 16 column pairs, hit 64 different banks) give the two
            // output rows c0 + 2 cp and c0 + 2 cp + 1, output columns r0 + 16 rb ...
            static_assert(kTR == 64 && kTC == 128 && kThreads == 256, "one column pair and row group per thread");
            const int rb = t & 3, cp = t >> 2;
            const uint32_t *col = reinterpret_cast<const uint32_t *>(tile) + rb * 16 * (kPitchT / 2) + cp;
            uint32_t d[16];
#pragma unroll
            for (int k = 0; k < 16; ++k) d[k] = col[k * (kPitchT / 2)];
#pragma unroll
            for (int h = 0; h < 2; ++h) {
                const int c = 2 * cp + h;
                if (c0 + c < p.cols && r0 + rb * 16 < p.rows) {
                    uint32_t w[8];
#pragma unroll
                    for (int j = 0; j < 8; ++j)
                        w[j] = h ? __builtin_amdgcn_perm(d[2 * j + 1], d[2 * j], 0x07060302u)   // the two high halves
                                 : __builtin_amdgcn_perm(d[2 * j + 1], d[2 * j], 0x05040100u);  // the two low halves
                    if (RHT) rht16<F16>(w);
                    track(w, m, z);
                    // (exchanging the pieces through LDS so that every store instruction covers whole lines, as
                    // rht_rows_kernel does, is worth 1 us of 62 here)
                    uint4 *dst = reinterpret_cast<uint4 *>(p.y + (c0 + c) * p.ldy + r0 + rb * 16);
                    dst[0] = make_uint4(w[0], w[1], w[2], w[3]);
                    dst[1] = make_uint4(w[4], w[5], w[6], w[7]);
                }
            }
        }
        __syncthreads();
    }
    write_partials<F16>(m, z, p.partials);
}

// fp32 input (the reference converts with `.float()` and multiplies by the fp32 matrix: a library matmul whose
// summation order is not part of any interface, so the target is the product itself, to fp32 rounding).  One
// thread per output group of 16: the butterfly in fp32 (four levels of additions: within 4 units in the last
// place of the largest partial sum), fp32 out.  With transposition a wavefront's lanes take consecutive output
// rows, i.e. consecutive columns of x, so that each of its 16 loads reads a contiguous run of one row of x.
struct TransformParamsF32 {
    const float *x;
    int64_t rows, cols, ld;
    float *y;
    int64_t ldy;
    uint32_t *partials;
    int64_t out_rows, groups;  // output rows, groups of 16 per output row
};

template <bool TRANSPOSE, bool RHT>
__global__ __launch_bounds__(kThreads) void transform_f32_kernel(const TransformParamsF32 p) {
    __shared__ uint32_t smem[4];
    uint32_t m = 0;
    const int64_t n_units = p.out_rows * p.groups;
    for (int64_t u = (int64_t)blockIdx.x * kThreads + threadIdx.x; u < n_units; u += (int64_t)gridDim.x * kThreads) {
        // transposed: consecutive units walk down the output rows (a column of groups at a time)
        const int64_t r = TRANSPOSE ? u % p.out_rows : u / p.groups, g = TRANSPOSE ? u / p.out_rows : u % p.groups;
        float v[16];
#pragma unroll
        for (int i = 0; i < 16; ++i) {
            const int64_t c = g * 16 + i;  // column of y = (transposed) row of x
            float e = 0.0f;
            if (TRANSPOSE) { if (c < p.rows) e = p.x[c * p.ld + r]; }
            else if (c < p.cols) e = p.x[r * p.ld + c];
            v[i] = RHT && ((kRhtNegMask >> i) & 1u) ? -e : e;
        }
        if (RHT) {
#pragma unroll
            for (int len = 1; len < 16; len <<= 1) {
#pragma unroll
                for (int i = 0; i < 16; ++i) {
                    if ((i & len) == 0) {
                        const float a = v[i], b = v[i + len];
                        v[i] = a + b;
                        v[i + len] = a - b;
                    }
                }
            }
#pragma unroll
            for (int i = 0; i < 16; ++i) v[i] = v[i] * 0.25f + 0.0f;
        }
        float4 *dst = reinterpret_cast<float4 *>(p.y + r * p.ldy + g * 16);
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            dst[q] = make_float4(v[4 * q], v[4 * q + 1], v[4 * q + 2], v[4 * q + 3]);
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const uint32_t mag = f2u(v[4 * q + i]) & 0x7fffffffu;
                m = mag > m ? mag : m;
            }
        }
    }
    m = block_max_u32(m, smem);
    if (threadIdx.x == 0) {
        p.partials[2 * blockIdx.x] = m;
        p.partials[2 * blockIdx.x + 1] = 0u;
    }
}

__global__ __launch_bounds__(kThreads) void transform_amax_kernel(const uint32_t *__restrict__ partials, int n,
                                                                  float *__restrict__ amax) {
    __shared__ uint32_t smem[4];
    uint32_t m = 0;
    for (int i = threadIdx.x; i < n; i += kThreads) m = m > partials[2 * i] ? m : partials[2 * i];
    m = block_max_u32(m, smem);
    if (threadIdx.x == 0) *amax = u2f(m);
}

}  // namespace fos

namespace fos {
int transform_impl(const void *x, int x_type, int64_t rows, int64_t cols, int64_t ld, int transpose, int rht, void *y, int64_t ldy,
                   float *amax, int *n_partials, void *workspace, size_t workspace_bytes, fos_stream_t stream);
}
using namespace fos;

// Body of fos_transform.  `amax` null: the reduction kernel is left out and *n_partials tells how many
// {maximum, reserved} pairs the transform left in the workspace (for a pass 2 that reduces them itself).
int fos::transform_impl(const void *x, int x_type, int64_t rows, int64_t cols, int64_t ld,
                        int transpose, int rht, void *y, int64_t ldy, float *amax, int *n_partials,
                        void *workspace, size_t workspace_bytes, fos_stream_t stream) {
    if (!x || !y || (!amax && !n_partials)) return FOS_E_NULL_POINTER;
    if (rows <= 0 || cols <= 0 || ld < cols) return FOS_E_BAD_SHAPE;
    if ((x_type != FOS_T_BF16 && x_type != FOS_T_F16 && x_type != FOS_T_F32) || (!transpose && !rht)) return FOS_E_UNSUPPORTED;
    const bool f16 = x_type == FOS_T_F16;
    const int64_t out_cols = transpose ? rows : cols;
    // y is written in whole 16-element groups
    if (ldy < (out_cols + 15) / 16 * 16) return FOS_E_BAD_SHAPE;
    if (!workspace || workspace_bytes < fos_quantize_workspace_bytes(rows, cols)) return FOS_E_WORKSPACE;
    if (x_type == FOS_T_F32) {
        if (((uintptr_t)x & 3) || ((uintptr_t)y & 15) || (ldy % 4 != 0) || ((uintptr_t)workspace & 7) || ((uintptr_t)amax & 3))
            return FOS_E_BAD_ALIGNMENT;
        TransformParamsF32 q;
        q.x = static_cast<const float *>(x);
        q.rows = rows; q.cols = cols; q.ld = ld;
        q.y = static_cast<float *>(y);
        q.ldy = ldy;
        q.partials = static_cast<uint32_t *>(workspace);
        q.out_rows = transpose ? cols : rows;
        q.groups = (out_cols + 15) / 16;
        hipStream_t s32 = (hipStream_t)stream;
        int64_t grid32 = (q.out_rows * q.groups + kThreads - 1) / kThreads;
        if (grid32 > 1024) grid32 = 1024;  // pairs the workspace holds
        if (transpose && rht) hipLaunchKernelGGL((transform_f32_kernel<true, true>), dim3((unsigned)grid32), dim3(kThreads), 0, s32, q);
        else if (transpose) hipLaunchKernelGGL((transform_f32_kernel<true, false>), dim3((unsigned)grid32), dim3(kThreads), 0, s32, q);
        else hipLaunchKernelGGL((transform_f32_kernel<false, true>), dim3((unsigned)grid32), dim3(kThreads), 0, s32, q);
        if (n_partials) *n_partials = (int)grid32;
        if (amax) hipLaunchKernelGGL(transform_amax_kernel, dim3(1), dim3(kThreads), 0, s32, q.partials, (int)grid32, amax);
        return hipGetLastError() == hipSuccess ? FOS_OK : FOS_E_LAUNCH;
    }
    if (((uintptr_t)x & 1) || ((uintptr_t)y & 15) || (ldy % 8 != 0) || ((uintptr_t)workspace & 7) || ((uintptr_t)amax & 3))
        return FOS_E_BAD_ALIGNMENT;
    TransformParams p;
    p.x = static_cast<const uint16_t *>(x);
    p.rows = rows; p.cols = cols; p.ld = ld;
    p.y = static_cast<uint16_t *>(y);
    p.ldy = ldy;
    p.partials = static_cast<uint32_t *>(workspace);
    p.vec = (((uintptr_t)x & 15) == 0 && ld % 8 == 0) ? 1 : 0;
    hipStream_t s = (hipStream_t)stream;
    int64_t grid;
    constexpr int64_t kMaxGrid = 1024;  // pairs the workspace holds
    if (transpose) {
        p.tiles_x = (int)((cols + kTC - 1) / kTC);
        p.n_units = ((rows + kTR - 1) / kTR) * p.tiles_x;
        grid = p.n_units < kMaxGrid ? p.n_units : kMaxGrid;
        if (rht && f16) hipLaunchKernelGGL((transpose_kernel<true, true>), dim3((unsigned)grid), dim3(kThreads), 0, s, p);
        else if (rht) hipLaunchKernelGGL((transpose_kernel<true, false>), dim3((unsigned)grid), dim3(kThreads), 0, s, p);
        else if (f16) hipLaunchKernelGGL((transpose_kernel<false, true>), dim3((unsigned)grid), dim3(kThreads), 0, s, p);
        else hipLaunchKernelGGL((transpose_kernel<false, false>), dim3((unsigned)grid), dim3(kThreads), 0, s, p);
    } else {
        p.tiles_x = 0;
        p.n_units = rows * ((cols + 15) / 16);
        grid = (p.n_units + kThreads - 1) / kThreads;
        if (grid > kMaxGrid) grid = kMaxGrid;
        if (f16) hipLaunchKernelGGL(rht_rows_kernel<true>, dim3((unsigned)grid), dim3(kThreads), 0, s, p);
        else hipLaunchKernelGGL(rht_rows_kernel<false>, dim3((unsigned)grid), dim3(kThreads), 0, s, p);
    }
    if (n_partials) *n_partials = (int)grid;
    if (amax) hipLaunchKernelGGL(transform_amax_kernel, dim3(1), dim3(kThreads), 0, s, p.partials, (int)grid, amax);
    return hipGetLastError() == hipSuccess ? FOS_OK : FOS_E_LAUNCH;
}

extern "C" int fos_transform(const void *x, int x_type, int64_t rows, int64_t cols, int64_t ld,
                             int transpose, int rht, void *y, int64_t ldy, float *amax,
                             void *workspace, size_t workspace_bytes, fos_stream_t stream) {
    if (!amax) return FOS_E_NULL_POINTER;
    return transform_impl(x, x_type, rows, cols, ld, transpose, rht, y, ldy, amax, nullptr, workspace, workspace_bytes, stream);
}
