// Pass 2 for NVFP4 with round-to-nearest or plain stochastic rounding, around the fast
// block formulation of fos_quantize_fast.h.  Two lane mappings:
//
//  * 1x16 blocks (quantize_nvfp4_rows_kernel): a wavefront covers 4 rows x 16 blocks,
//    i.e. 512 contiguous bytes per row.  Measured on MI355X, a wavefront that touches 16
//    rows x 128 bytes streams at ~4.1 TB/s while 4 rows x 512 bytes reaches ~6 TB/s, so the
//    row-contiguous mapping is what the HBM-bound path uses.  A 256-thread workgroup
//    covers 128 rows x 256 columns in eight steps of 16 rows (the next step's loads are
//    issued before the current step is processed), stages the 4 complete 128x4 scale
//    tiles in LDS and writes them as one contiguous 2 KiB run.
//  * 16x16 tiles (quantize_nvfp4_tile_kernel): the 16 rows of a tile must lie along one DPP
//    row for the tile reductions, so a wavefront covers 16 rows x 4 blocks; persistent
//    workgroups walk over 128 x 64 tiles with the next tile prefetched.
#include <cstdlib>

#include "fos_quantize_kernel.h"

namespace fos {

struct TileRegs {
    Block16 b[2];
};

FOS_DEVICE void load_tile(const QuantParams &p, uint32_t tile, int lane, int wave, TileRegs &t) {
    const int64_t tile_y = tile / (uint32_t)p.tiles_x, tile_x = tile - (uint32_t)tile_y * (uint32_t)p.tiles_x;
    const int64_t c0 = (tile_x * 4 + (lane >> 4)) * 16;
#pragma unroll
    for (int h = 0; h < 2; ++h) {
        const int64_t r = tile_y * 128 + h * 64 + wave * 16 + (lane & 15);
        if (r < p.rows && c0 < p.cols) {
            const uint4 *src = reinterpret_cast<const uint4 *>(p.x + r * p.ld + c0);
            const uint4 lo = src[0], hi = src[1];
            t.b[h].w[0] = lo.x; t.b[h].w[1] = lo.y; t.b[h].w[2] = lo.z; t.b[h].w[3] = lo.w;
            t.b[h].w[4] = hi.x; t.b[h].w[5] = hi.y; t.b[h].w[6] = hi.z; t.b[h].w[7] = hi.w;
        } else {
#pragma unroll
            for (int i = 0; i < 8; ++i) t.b[h].w[i] = 0;
        }
    }
}

template <int RULE, bool TWO_D, bool PSEUDO, bool SR>
__global__ __launch_bounds__(kThreads) __attribute__((amdgpu_waves_per_eu(4))) void quantize_nvfp4_tile_kernel(const QuantParams p) {
    __shared__ uint32_t red[4];
    __shared__ uint32_t sf_tile[2][128];
    __shared__ __attribute__((aligned(16))) FastLutEntry lut[128];

    uint32_t amax_bits;
    bool maybe_negzero;
    reduce_partials(p, red, amax_bits, maybe_negzero);
    QuantConsts k;
    k.amax = u2f(amax_bits);
    k.enc = p.c / k.amax;
    k.dec = 1.0f / (p.c / k.amax);
    k.qdiv = p.qdiv;
    k.errdiv = p.errdiv;
    k.exact_ok = k.errdiv == 1536.0f && (amax_bits & 0xffffu) == 0;
    if (blockIdx.x == 0 && threadIdx.x == 0 && p.amax_out) *p.amax_out = k.amax;
    const bool in_range = k.amax >= 0x1p-100f && k.amax <= 0x1p100f;
    const float enc_fast = in_range ? k.enc : 0.0f;
    const float rq = 1.0f / k.qdiv, rc = 1.0f / p.c;
    if (threadIdx.x < 128) lut[threadIdx.x] = make_lut_entry(threadIdx.x, k);
    __syncthreads();

    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int64_t sf_cols = p.cols_p >> 4;
    const uint32_t n_tiles = (uint32_t)(p.rows_p >> 7) * (uint32_t)p.tiles_x;
    const bool tiled = !PSEUDO && p.sf_layout == FOS_SF_TILED_128X4;

    auto process = [&](uint32_t tile, const TileRegs &t, uint32_t *stage) {
        const int64_t tile_y = tile / (uint32_t)p.tiles_x, tile_x = tile - (uint32_t)tile_y * (uint32_t)p.tiles_x;
        const int64_t cb = tile_x * 4 + (lane >> 4);
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            const int rr = h * 64 + wave * 16 + (lane & 15);
            const int64_t r = tile_y * 128 + rr;
            const BlockOut o = quantize_block_nvfp4_fast<RULE, TWO_D, SR>(t.b[h], k, enc_fast, rq, maybe_negzero, in_range, lut,
                                                                          p.seed, p.offset, (uint64_t)(r * sf_cols + cb));
            if (PSEUDO) {
                uint32_t w[8];
                if (in_range) dequant_block_bf16<true>(o, k.amax, p.c, rc, w);
                else dequant_block_bf16<false>(o, k.amax, p.c, rc, w);
                if (r < p.rows && cb * 16 < p.cols) {
                    uint4 *d = reinterpret_cast<uint4 *>(p.pseudo_out + r * p.ldo + cb * 16);
                    d[0] = make_uint4(w[0], w[1], w[2], w[3]);
                    d[1] = make_uint4(w[4], w[5], w[6], w[7]);
                }
                continue;
            }
            *reinterpret_cast<uint2 *>(p.codes + r * (p.cols_p >> 1) + cb * 8) = make_uint2(o.c0, o.c1);
            if (tiled) reinterpret_cast<uint8_t *>(stage)[(rr & 31) * 16 + (rr >> 5) * 4 + (lane >> 4)] = (uint8_t)o.s;
            else p.sf[r * sf_cols + cb] = (uint8_t)o.s;
        }
        if (tiled) {
            __syncthreads();
            if (threadIdx.x < 128)
                reinterpret_cast<uint32_t *>(p.sf + (tile_y * (sf_cols >> 2) + tile_x) * 512)[threadIdx.x] = stage[threadIdx.x];
        }
    };

    // two tiles per trip so that the prefetch registers alternate without copies
    TileRegs ta, tb;
    uint32_t tile = blockIdx.x;
    const uint32_t step = gridDim.x;
    if (tile < n_tiles) load_tile(p, tile, lane, wave, ta);
    while (tile < n_tiles) {
        if (tile + step < n_tiles) load_tile(p, tile + step, lane, wave, tb);
        process(tile, ta, sf_tile[0]);
        tile += step;
        if (tile >= n_tiles) break;
        if (tile + step < n_tiles) load_tile(p, tile + step, lane, wave, ta);
        process(tile, tb, sf_tile[1]);
        tile += step;
    }
}


// 1x16 blocks, row-contiguous mapping: lane -> block column (lane & 15) of row (lane >> 4)
// within the wavefront's 4 rows; workgroup tile 128 rows x 256 columns; workgroups stride
// over the tiles so that the per-workgroup setup (tensor maximum, scale table) is paid
// once for several tiles.  FULL: rows % 128 == 0 and cols % 256 == 0, no bounds checks.
template <int RULE, bool FULL, bool PSEUDO, bool SR>
__global__ __launch_bounds__(kThreads) __attribute__((amdgpu_waves_per_eu(4))) void quantize_nvfp4_rows_kernel(
    const QuantParams p) {
    __shared__ uint32_t red[4];
    __shared__ uint32_t sf_stage[2][4 * 128];  // 4 scale tiles of 512 bytes, double-buffered
    __shared__ __attribute__((aligned(16))) FastLutEntry lut[128];

    uint32_t amax_bits;
    bool maybe_negzero;
    reduce_partials(p, red, amax_bits, maybe_negzero);
    QuantConsts k;
    k.amax = u2f(amax_bits);
    k.enc = p.c / k.amax;
    k.dec = 1.0f / (p.c / k.amax);
    k.qdiv = p.qdiv;
    k.errdiv = p.errdiv;
    k.exact_ok = k.errdiv == 1536.0f && (amax_bits & 0xffffu) == 0;
    if (blockIdx.x == 0 && threadIdx.x == 0 && p.amax_out) *p.amax_out = k.amax;
    const bool in_range = k.amax >= 0x1p-100f && k.amax <= 0x1p100f;
    const float enc_fast = in_range ? k.enc : 0.0f;
    const float rq = 1.0f / k.qdiv, rc = 1.0f / p.c;
    if (threadIdx.x < 128) lut[threadIdx.x] = make_lut_entry(threadIdx.x, k);
    __syncthreads();

    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int64_t sf_cols = p.cols_p >> 4;
    const int lb = lane & 15;                // block column inside the tile
    const int rr0 = wave * 4 + (lane >> 4);  // row inside a 16-row step
    const bool tiled = !PSEUDO && p.sf_layout == FOS_SF_TILED_128X4;
    const int64_t row_pitch = p.ld, code_pitch = p.cols_p >> 1;
    const uint32_t n_tiles = (uint32_t)(p.rows_p >> 7) * (uint32_t)p.tiles_x;
    int buf = 0;

    for (uint32_t tile = blockIdx.x; tile < n_tiles; tile += gridDim.x, buf ^= 1) {
        const uint32_t tile_y = tile / (uint32_t)p.tiles_x, tile_x = tile - tile_y * (uint32_t)p.tiles_x;
        const int64_t cb = (int64_t)tile_x * 16 + lb;  // block column in the tensor
        const bool col_ok = FULL || cb < sf_cols;
        const int64_t row0 = (int64_t)tile_y * 128 + rr0;
        const uint16_t *src = p.x + row0 * row_pitch + cb * 16;
        uint8_t *dst = p.codes + row0 * code_pitch + cb * 8;
        uint8_t *stage = reinterpret_cast<uint8_t *>(sf_stage[buf]) + (lb >> 2) * 512 + (lb & 3);

        auto load = [&](int g, Block16 &b) {
            if (FULL || (col_ok && row0 + g * 16 < p.rows && cb * 16 < p.cols)) {
                const uint4 *q = reinterpret_cast<const uint4 *>(src + (int64_t)g * 16 * row_pitch);
                const uint4 lo = q[0], hi = q[1];
                b.w[0] = lo.x; b.w[1] = lo.y; b.w[2] = lo.z; b.w[3] = lo.w;
                b.w[4] = hi.x; b.w[5] = hi.y; b.w[6] = hi.z; b.w[7] = hi.w;
            } else {
#pragma unroll
                for (int i = 0; i < 8; ++i) b.w[i] = 0;
            }
        };

        Block16 blk[8];
        load(0, blk[0]);
        load(1, blk[1]);
#pragma unroll
        for (int g = 0; g < 8; ++g) {
            if (g + 2 < 8) load(g + 2, blk[g + 2]);
            if (col_ok) {
                const int rr = g * 16 + rr0;
                // a 16-row step that lies wholly in the row padding (decode-sized inputs: seven of
                // the eight steps) only writes its zero codes and scales
                const bool padding_step = !FULL && (int64_t)tile_y * 128 + g * 16 >= p.rows;
                BlockOut o{0u, 0u, 0u};
                if (!padding_step)
                    o = quantize_block_nvfp4_fast<RULE, false, SR>(blk[g], k, enc_fast, rq, maybe_negzero, in_range, lut, p.seed,
                                                                   p.offset, (uint64_t)((row0 + g * 16) * sf_cols + cb));
                if (PSEUDO) {
                    uint32_t w[8];
                    if (in_range) dequant_block_bf16<true>(o, k.amax, p.c, rc, w);
                    else dequant_block_bf16<false>(o, k.amax, p.c, rc, w);
                    if (FULL || (row0 + g * 16 < p.rows && cb * 16 < p.cols)) {
                        uint4 *d = reinterpret_cast<uint4 *>(p.pseudo_out + (row0 + g * 16) * p.ldo + cb * 16);
                        d[0] = make_uint4(w[0], w[1], w[2], w[3]);
                        d[1] = make_uint4(w[4], w[5], w[6], w[7]);
                    }
                    continue;
                }
                *reinterpret_cast<uint2 *>(dst + (int64_t)g * 16 * code_pitch) = make_uint2(o.c0, o.c1);
                if (tiled) stage[(rr & 31) * 16 + (rr >> 5) * 4] = (uint8_t)o.s;
                else p.sf[(row0 + g * 16) * sf_cols + cb] = (uint8_t)o.s;
            }
        }
        if (tiled) {
            __syncthreads();
            // 4 scale tiles x 512 bytes, contiguous in the output; 8 bytes per thread.  The
            // other staging buffer is in use by the next tile, so one barrier per tile does.
            const int t = threadIdx.x >> 6;
            const int64_t group = (int64_t)tile_x * 4 + t;
            if (FULL || group < (sf_cols >> 2)) {
                uint2 *out = reinterpret_cast<uint2 *>(p.sf + ((int64_t)tile_y * (sf_cols >> 2) + group) * 512);
                out[lane] = reinterpret_cast<const uint2 *>(sf_stage[buf])[threadIdx.x];
            }
        }
    }
}

template <int RULE, bool PSEUDO, bool SR>
static void by_dim(QuantParams &p, bool two_d, bool aligned, hipStream_t s) {
    if (!aligned) {
        if (PSEUDO || SR) return;  // rejected by the entry point / routed to the generic kernel
        if (two_d) launch_quantize<true, FOS_DTYPE_NVFP4, RULE, FOS_ROUND_NEAREST, true>(p, aligned, s);
        else launch_quantize<true, FOS_DTYPE_NVFP4, RULE, FOS_ROUND_NEAREST, false>(p, aligned, s);
        return;
    }
    if (!two_d) {
        p.tiles_x = (int)((p.cols_p + 255) / 256);
        const int64_t n = (p.rows_p / 128) * p.tiles_x;
        // five resident workgroups per compute unit (256 CUs, <= 102 VGPRs); more tiles than
        // that are walked by the same workgroups.  FOS_QUANT_GRID overrides for tuning runs.
        int64_t grid = 1280;
        if (const char *e = getenv("FOS_QUANT_GRID")) grid = atoll(e) > 0 ? atoll(e) : grid;
        if (grid > n) grid = n;
        const bool full = p.rows % 128 == 0 && p.cols % 256 == 0;
        if (full)
            hipLaunchKernelGGL((quantize_nvfp4_rows_kernel<RULE, true, PSEUDO, SR>), dim3((unsigned)grid), dim3(kThreads), 0, s, p);
        else
            hipLaunchKernelGGL((quantize_nvfp4_rows_kernel<RULE, false, PSEUDO, SR>), dim3((unsigned)grid), dim3(kThreads), 0, s, p);
        return;
    }
    p.tiles_x = (int)(p.cols_p / 64);
    const int64_t n_tiles = (p.rows_p / 128) * p.tiles_x;
    // Persistent grid: a few workgroups per compute unit (256 CUs), fewer when the tensor
    // is small.  FOS_QUANT_GRID overrides the count for tuning runs.
    int64_t grid = 256 * 6;
    if (const char *e = getenv("FOS_QUANT_GRID")) grid = atoll(e) > 0 ? atoll(e) : grid;
    if (grid > n_tiles) grid = n_tiles;
    hipLaunchKernelGGL((quantize_nvfp4_tile_kernel<RULE, true, PSEUDO, SR>), dim3((unsigned)grid), dim3(kThreads), 0, s, p);
}

template <bool PSEUDO, bool SR>
static void by_rule(QuantParams &p, int rule, bool two_d, bool aligned, hipStream_t s) {
    switch (rule) {
        case FOS_RULE_STATIC_6:
        case FOS_RULE_STATIC_4:
            // the two static rules differ only in the host-computed constants
            by_dim<FOS_RULE_STATIC_6, PSEUDO, SR>(p, two_d, aligned, s);
            break;
        case FOS_RULE_MAE: by_dim<FOS_RULE_MAE, PSEUDO, SR>(p, two_d, aligned, s); break;
        case FOS_RULE_MSE: by_dim<FOS_RULE_MSE, PSEUDO, SR>(p, two_d, aligned, s); break;
        default: by_dim<FOS_RULE_ABS_MAX, PSEUDO, SR>(p, two_d, aligned, s); break;
    }
}

// `sr`: a stochastic style on an aligned input.  The fast exact evaluation is tied to the
// selection divisor 1536; with the unbiased style's rescaled divisor an inconclusive
// shortcut falls back to the operation-by-operation form.
void launch_quantize_nvfp4_fast(QuantParams &p, int rule, bool two_d, bool aligned, bool sr, hipStream_t s) {
    if (sr) by_rule<false, true>(p, rule, two_d, aligned, s);
    else if (p.pseudo_out) by_rule<true, false>(p, rule, two_d, aligned, s);
    else by_rule<false, false>(p, rule, two_d, aligned, s);
}

}  // namespace fos
