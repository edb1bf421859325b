// Pass-2 kernel of the gfx950 quantize path, shared by the translation units that
// instantiate it.
//
// Work decomposition: one lane owns one 1x16 block (32 contiguous input bytes, two 128-bit
// loads; 8 output bytes, one 64-bit store).  A wavefront covers 16 rows x 4 blocks with
// the 16 rows of a 16x16 tile laid along one DPP row, so the 2-D tile reductions are DPP
// row operations.  A 256-thread workgroup covers 128 rows x (64*T) columns, i.e. T
// complete 128x4 scale tiles, which it assembles in LDS and writes as contiguous
// 512-byte runs.
#pragma once

#include "fos_quantize_common.h"
#include "fos_quantize_fast.h"

namespace fos {

// FAST: NVFP4 round-to-nearest (or IF4 round-to-nearest with the MSE rule) through the fast
// block formulations, with the operation-by-operation form as the per-block fallback.  ALIGNED: x 16-byte aligned, ld % 8 == 0,
// cols % 16 == 0 -> 128-bit loads.
template <bool FAST, int DT, int RULE, int ROUND, bool TWO_D, int T, bool ALIGNED>
__global__ __launch_bounds__(kThreads) void quantize_kernel(const QuantParams p) {
    __shared__ uint32_t red[4];
    __shared__ uint32_t sf_tile[T * 128];  // T tiles of 512 scale bytes
    __shared__ __attribute__((aligned(16))) FastLutEntry lut[FAST ? 128 : 1];

    const uint32_t amax_bits = reduce_partials(p, red);
    QuantConsts k;
    k.amax = u2f(amax_bits);
    k.enc = p.c / k.amax;
    k.dec = 1.0f / (p.c / k.amax);
    k.qdiv = p.qdiv;
    k.errdiv = p.errdiv;
    k.exact_ok = k.errdiv == 1536.0f && (amax_bits & 0xffffu) == 0;
    k.shortcut_ok = shortcut_range(k.amax);
    if (blockIdx.x == 0 && threadIdx.x == 0 && p.amax_out) *p.amax_out = k.amax;
    // dither key: launch arguments, or read from device memory (a captured launch whose key the caller advances)
    uint64_t key_seed = p.seed, key_offset = p.offset;
    if (ROUND != FOS_ROUND_NEAREST && p.key) {
        key_seed = p.key[0];
        key_offset = p.key[1];
    }

    // The fast formulation assumes that no intermediate leaves the normal fp32 range,
    // which holds for 2^-100 <= amax <= 2^100; other tensors use the fallback throughout.
    const bool in_range = k.amax >= 0x1p-100f && k.amax <= 0x1p100f;
    const float enc_fast = in_range ? k.enc : 0.0f;
    const float rq = 1.0f / k.qdiv;
    k.rerr = 1.0f / k.errdiv;
    k.fast_div = in_range && (k.errdiv == 1536.0f || k.errdiv == 2688.0f);
    if (FAST) {
        if (threadIdx.x < 128) lut[threadIdx.x] = make_lut_entry(threadIdx.x, k);
        __syncthreads();
    }

    const int tile_x = blockIdx.x % p.tiles_x;
    const int64_t tile_y = blockIdx.x / p.tiles_x;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int64_t sf_cols = p.cols_p >> 4;
    const int64_t row_base = tile_y * 128 + wave * 16 + (lane & 15);
    const int64_t cb_base = (int64_t)tile_x * (4 * T) + (lane >> 4);

    constexpr int NB = 2 * T;  // blocks per lane: T column groups x 2 row halves
    // the element-wise form (any alignment) is also the one that reads fp16 and fp32 inputs
    constexpr bool TYPED = !FAST && !ALIGNED;
    uint32_t w[NB][8];
    float xf[TYPED ? NB : 1][16];
#pragma unroll
    for (int it = 0; it < NB; ++it) {
        const int64_t r = row_base + (it & 1) * 64;
        const int64_t cb = cb_base + (it >> 1) * 4;
        const int64_t c0 = cb * 16;
        if (TYPED) {
            if (p.x_vec && r < p.rows && c0 < p.cols) {
                load_block16(p, r, c0, xf[it]);
            } else {
#pragma unroll
                for (int i = 0; i < 16; ++i) xf[it][i] = (r < p.rows && c0 + i < p.cols) ? load_element(p, r, c0 + i) : 0.0f;
            }
        } else if (ALIGNED) {
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
        if (FAST) {
            Block16 blk;
#pragma unroll
            for (int i = 0; i < 8; ++i) blk.w[i] = w[it][i];
            BlockOut o;
            if constexpr (DT == FOS_DTYPE_IF4) o = quantize_block_if4_mse<TWO_D>(blk, k, enc_fast, rq, in_range, lut);
            else o = quantize_block_nvfp4_fast<RULE, TWO_D, false>(blk, k, enc_fast, rq, in_range, lut, 0, 0, 0);
            codes[0] = o.c0;
            codes[1] = o.c1;
            sbyte = o.s;
        } else if (TYPED)
            quantize_block_f32<DT, RULE, ROUND, TWO_D>(xf[it], k, key_seed, key_offset, (uint64_t)(r * sf_cols + cb), codes,
                                                       sbyte);
        else
            quantize_block<DT, RULE, ROUND, TWO_D>(w[it], k, key_seed, key_offset, (uint64_t)(r * sf_cols + cb), codes,
                                                   sbyte);
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

// Grid / tile-width choice and launch, for one (FAST, DT, RULE, ROUND, TWO_D).
template <bool FAST, int DT, int RULE, int ROUND, bool TWO_D>
void launch_quantize(QuantParams &p, bool aligned, hipStream_t s) {
    // Wide tiles (full 128-byte lines of packed output per row) once there are enough
    // workgroups to fill the chip; narrow tiles for small or unaligned tensors.
    const int64_t tiles_y = p.rows_p / 128;
    const int64_t groups = p.cols_p / 64;
    if constexpr (FAST && DT == FOS_DTYPE_NVFP4) {
        // aligned NVFP4 round-to-nearest inputs go to the persistent kernel instead
        p.tiles_x = (int)groups;
        hipLaunchKernelGGL((quantize_kernel<FAST, DT, RULE, ROUND, TWO_D, 1, false>),
                           dim3((unsigned)(tiles_y * p.tiles_x)), dim3(kThreads), 0, s, p);
        return;
    }
    if (aligned && groups % 4 == 0 && tiles_y * (groups / 4) >= 1024) {
        p.tiles_x = (int)(groups / 4);
        hipLaunchKernelGGL((quantize_kernel<FAST, DT, RULE, ROUND, TWO_D, 4, true>),
                           dim3((unsigned)(tiles_y * p.tiles_x)), dim3(kThreads), 0, s, p);
    } else if (aligned) {
        p.tiles_x = (int)groups;
        hipLaunchKernelGGL((quantize_kernel<FAST, DT, RULE, ROUND, TWO_D, 1, true>),
                           dim3((unsigned)(tiles_y * p.tiles_x)), dim3(kThreads), 0, s, p);
    } else {
        p.tiles_x = (int)groups;
        hipLaunchKernelGGL((quantize_kernel<FAST, DT, RULE, ROUND, TWO_D, 1, false>),
                           dim3((unsigned)(tiles_y * p.tiles_x)), dim3(kThreads), 0, s, p);
    }
}

// Defined in fos_quantize_fast.hip: NVFP4, any rule, round to nearest or (sr, aligned inputs
// only) a stochastic style.
void launch_quantize_nvfp4_fast(QuantParams &p, int rule, bool two_d, bool aligned, bool sr, hipStream_t s);
void launch_quantize_if4_mse_rows(QuantParams &p, hipStream_t s);
void launch_quantize_if4_mse_tiles(QuantParams &p, hipStream_t s);

// MXFP4 (fos_mxfp4.hip)
int launch_quantize_mxfp4(const void *x, int x_type, int64_t rows, int64_t cols, int64_t ld, int rule, int sf_layout, uint8_t *codes,
                          uint8_t *sf, float *amax, hipStream_t s);

}  // namespace fos
