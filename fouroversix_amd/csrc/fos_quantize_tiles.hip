// Pass 2 for NVFP4 with 16x16 scale tiles (block_scale_2d), round to nearest or a stochastic style, rules static_6 /
// static_4 and 4/6 with the MSE, MAE or abs-max rule, on the row-contiguous lane mapping of the 1x16 kernel: a wavefront
// touches 4 rows x 512 contiguous bytes per step.
//
// Workgroup tile: 128 rows x two windows of 256 columns.  Wavefront w covers window w >> 1 and
// the 16-row bands of parity w & 1: rows 32 q + 16 (w & 1) + 4 s + i for group q = 0..3, step
// s = 0..3 and i = lane >> 4; lane & 15 is the block column.  A lane therefore holds, per group,
// the four 1x16 blocks of rows i, 4 + i, 8 + i, 12 + i of ONE 16x16 tile, and the tile's other
// rows sit in the lanes 16, 32 and 48 further on: a tile reduction is an in-register reduction
// over the four blocks and two v_permlane{16,32}_swap steps, after which all four lanes hold the
// same bits and take the same decision.  The scales of rows r, r + 32, r + 64, r + 96 share a
// 16-byte unit of the 128x4 layout, so after its four groups a wavefront owns whole units: it
// builds them with quad permutes and writes 256 contiguous bytes per scale tile -- no LDS, no
// workgroup barrier.  Input, codes and the pseudo-quantize output go through buffer
// instructions as in the 1x16 kernel (wave-uniform descriptor per tile, fixed per-lane offset,
// uniform offset per step; a ragged tile reads zeros past the tensor's last row / column).
// A tile whose certified shortcut is inconclusive, whose scale byte is zero or sub-normal in a
// way the hardware convert cannot follow, or a tensor whose maximum is outside the fast range
// takes the operation-by-operation form, one tile at a time spread over the whole wavefront
// (slow_tile in the kernel; slow_tile_sr for the stochastic styles, whose dither is keyed per row of a tile).
#include "fos_buffer.h"
#include "fos_quantize_kernel.h"
#include "fos_tuning.h"

namespace fos {

namespace {

// v of the lanes 16 / 32 apart: `even` = the value held by DPP rows 0 and 2 (seen from rows
// {0,1} and {2,3}), `odd` = rows 1 and 3; `lo` = rows 0 and 1 (seen from {0,2} and {1,3}), `hi`
// = rows 2 and 3.
FOS_DEVICE void rows_pairs(uint32_t v, uint32_t &even, uint32_t &odd) {
    const u32x2 r = __builtin_amdgcn_permlane16_swap(v, v, false, false);
    even = r.x, odd = r.y;
}
FOS_DEVICE void rows_halves(uint32_t v, uint32_t &lo, uint32_t &hi) {
    const u32x2 r = __builtin_amdgcn_permlane32_swap(v, v, false, false);
    lo = r.x, hi = r.y;
}

// Reductions over the four lanes lane & 15, + 16, + 32, + 48; the same bits in all four.
FOS_DEVICE float tile_max(float v) {
    uint32_t a, b;
    rows_pairs(f2u(v), a, b);
    v = fmaxf(u2f(a), u2f(b));
    rows_halves(f2u(v), a, b);
    return fmaxf(u2f(a), u2f(b));
}
FOS_DEVICE float tile_sum(float v) {
    uint32_t a, b;
    rows_pairs(f2u(v), a, b);
    v = u2f(a) + u2f(b);
    rows_halves(f2u(v), a, b);
    return u2f(a) + u2f(b);
}
FOS_DEVICE uint32_t tile_or(uint32_t v) {
    uint32_t a, b;
    rows_pairs(v, a, b);
    v = a | b;
    rows_halves(v, a, b);
    return a | b;
}

// Both candidates of one block in the scaled domain: codes, and (adaptive rules) the rule's
// reduction of the rounding residuals added to SA / SB.
template <int RULE>
FOS_DEVICE void block_candidates(const Block16 &blk, float invA, float invB, uint32_t &a0, uint32_t &a1, uint32_t &b0,
                                 uint32_t &b1, float &SA, float &SB) {
    a0 = a1 = b0 = b1 = 0;
    static_for<0, 8>([&](auto jc) {
        constexpr int j = decltype(jc)::value;
        const float x0 = u2f(blk.w[j] << 16), x1 = u2f(blk.w[j] & 0xffff0000u);
        const float xa0 = scaled(x0, invA), xa1 = scaled(x1, invA);
        if (j < 4) a0 = pack_fp4<(j & 3)>(a0, xa0, xa1);
        else a1 = pack_fp4<(j & 3)>(a1, xa0, xa1);
        if (RULE != FOS_RULE_STATIC_6) {
            const float xb0 = scaled(x0, invB), xb1 = scaled(x1, invB);
            if (j < 4) b0 = pack_fp4<(j & 3)>(b0, xb0, xb1);
            else b1 = pack_fp4<(j & 3)>(b1, xb0, xb1);
            const float2_t fa = unpack_fp4<(j & 3)>(j < 4 ? a0 : a1);
            const float2_t fb = unpack_fp4<(j & 3)>(j < 4 ? b0 : b1);
            accumulate_scaled<RULE>(fa.x - xa0, fa.y - xa1, SA);
            accumulate_scaled<RULE>(fb.x - xb0, fb.y - xb1, SB);
        }
    });
}

// ... with a stochastic style: the hardware's dithered convert on the scaled values, one Philox call per block
// keyed by `blkid` = row * (cols_p / 16) + block column (the second candidate reads the words exchanged pairwise),
// as in the 1x16 path.
template <int RULE>
FOS_DEVICE void block_candidates_sr(const Block16 &blk, float invA, float invB, uint64_t seed, uint64_t offset, uint64_t blkid,
                                    uint32_t &a0, uint32_t &a1, uint32_t &b0, uint32_t &b1, float &SA, float &SB) {
    float xs[16];
#pragma unroll
    for (int j = 0; j < 8; ++j) {
        xs[2 * j] = scaled(u2f(blk.w[j] << 16), invA);
        xs[2 * j + 1] = scaled(u2f(blk.w[j] & 0xffff0000u), invA);
    }
    const Philox4 pA = block_philox(seed, offset, blkid);
    sr_pack16(xs, pA, a0, a1);
    b0 = b1 = 0;
    if (RULE != FOS_RULE_STATIC_6) {
        static_for<0, 8>([&](auto jc) {
            constexpr int j = decltype(jc)::value;
            const float2_t fa = unpack_fp4<(j & 3)>(j < 4 ? a0 : a1);
            accumulate_scaled<RULE>(fa.x - xs[2 * j], fa.y - xs[2 * j + 1], SA);
        });
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            xs[2 * j] = scaled(u2f(blk.w[j] << 16), invB);
            xs[2 * j + 1] = scaled(u2f(blk.w[j] & 0xffff0000u), invB);
        }
        sr_pack16(xs, second_candidate_words(pA), b0, b1);
        static_for<0, 8>([&](auto jc) {
            constexpr int j = decltype(jc)::value;
            const float2_t fb = unpack_fp4<(j & 3)>(j < 4 ? b0 : b1);
            accumulate_scaled<RULE>(fb.x - xs[2 * j], fb.y - xs[2 * j + 1], SB);
        });
    }
}

// IF4: the E2M1 candidate ("a") and the INT4 candidate ("b") of one block on their common scale,
// with the sums of squared residuals in the scaled domain (quantize_block_if4_mse, for a tile).
FOS_DEVICE void block_candidates_if4(const Block16 &blk, float inv, uint32_t &a0, uint32_t &a1, uint32_t &b0, uint32_t &b1,
                                     float &SA, float &SB) {
    a0 = a1 = b0 = b1 = 0;
    static_for<0, 8>([&](auto jc) {
        constexpr int j = decltype(jc)::value;
        const float x0 = scaled(u2f(blk.w[j] << 16), inv), x1 = scaled(u2f(blk.w[j] & 0xffff0000u), inv);
        if (j < 4) a0 = pack_fp4<(j & 3)>(a0, x0, x1);
        else a1 = pack_fp4<(j & 3)>(a1, x0, x1);
        const float2_t fa = unpack_fp4<(j & 3)>(j < 4 ? a0 : a1);
        accumulate_scaled<FOS_RULE_MSE>(fa.x - x0, fa.y - x1, SA);
        // INT4: rint(clamp(x * 7/6, -7, 7)); adding 1.5 * 2^23 rounds to nearest even and leaves the
        // two's-complement integer in the low mantissa bits
        const float t0 = __builtin_amdgcn_fmed3f(x0 * 1.16666666f, -7.0f, 7.0f) + 12582912.0f;
        const float t1 = __builtin_amdgcn_fmed3f(x1 * 1.16666666f, -7.0f, 7.0f) + 12582912.0f;
        const float q0 = t0 - 12582912.0f, q1 = t1 - 12582912.0f;
        accumulate_scaled<FOS_RULE_MSE>(__builtin_fmaf(q0, 0.8571428571f, -x0), __builtin_fmaf(q1, 0.8571428571f, -x1), SB);
        const uint32_t byte = (f2u(t0) & 0xfu) | ((f2u(t1) & 0xfu) << 4);
        if (j < 4) b0 |= byte << (8 * (j & 3));
        else b1 |= byte << (8 * (j & 3));
    });
}

struct TilesPos {
    uint64_t x_base, codes_base, out_base;  // first input element / code byte / output element of the wavefront's share
    uint32_t x_bytes;    // extent of the input descriptor
    uint32_t x_off;      // this lane's offset into it (beyond the descriptor for a lane past the last column)
    int32_t row0;        // first row of the wavefront's share of the tile (rows_p < 2^31: checked by the host)
    int32_t cb;          // this lane's block column in the tensor
    int64_t unit_base;   // offset of scale unit 16 (w & 1) of the wavefront's first scale tile
};

template <int q>
FOS_DEVICE uint32_t quad_bytes(uint32_t l0, uint32_t l1, uint32_t l2, uint32_t l3) {
    // byte q of the four lanes of a quad, in lane order
    const uint32_t p01 = __builtin_amdgcn_perm(l1, l0, 0x0c0c0000u | ((4u + q) << 8) | q);
    const uint32_t p23 = __builtin_amdgcn_perm(l3, l2, 0x0c0c0000u | ((4u + q) << 8) | q);
    return __builtin_amdgcn_perm(p23, p01, 0x05040100u);
}

// IF4: the IF4 format with its MSE rule (both candidates on one scale; the chosen one is flagged in
// bit 7 of the scale byte) instead of NVFP4.
// SR: a stochastic rounding style (NVFP4); its two sets of scaled values and the Philox state take the
// registers of three wavefronts per SIMD.
template <int RULE, bool FULL, bool PSEUDO, bool IF4 = false, bool SR = false>
__global__ __launch_bounds__(kThreads) __attribute__((amdgpu_waves_per_eu(SR ? 3 : 4, SR ? 3 : 8))) void quantize_nvfp4_tiles_kernel(
    const QuantParams p) {
    static_assert(!(SR && IF4), "stochastic styles: NVFP4");
    constexpr bool STATIC = RULE == FOS_RULE_STATIC_6;
    constexpr bool ADAPTIVE = !STATIC;            // 4/6 with the MSE, MAE or abs-max rule
    constexpr bool MAXRULE = RULE == FOS_RULE_ABS_MAX;  // the error is the largest term, not the sum
    __shared__ uint32_t red[4];
    __shared__ __attribute__((aligned(16))) FastLutEntry lut[128];

    const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);  // (scalar: what derives from it stays in scalar registers)
    const int par = wave & 1, half = wave >> 1;
    const int lb = lane & 15, li = lane >> 4;
    const int64_t sf_cols = p.cols_p >> 4;
    const int32_t rows32 = (int32_t)p.rows, cols16 = (int32_t)(p.cols >> 4);  // (cols % 16 == 0 on this path)
    const bool tiled = !PSEUDO && p.sf_layout == FOS_SF_TILED_128X4;
    const int64_t code_pitch = p.cols_p >> 1;
    const uint32_t n_tiles = (uint32_t)(p.rows_p >> 7) * (uint32_t)p.tiles_x;
    // byte offsets inside the wavefront's share (the host checked that a tile spans less than
    // 2^31 bytes); step s of group q starts 32 q + 4 s rows below the first
    const uint32_t x_lane = (uint32_t)(li * p.ld + lb * 16) * 2u, x_row = (uint32_t)p.ld * 2u;
    const uint32_t c_lane = (uint32_t)(li * code_pitch + lb * 8), c_row = (uint32_t)code_pitch;
    const uint32_t o_lane = PSEUDO ? (uint32_t)(li * p.ldo + lb * 16) * 2u : 0u, o_row = PSEUDO ? (uint32_t)p.ldo * 2u : 0u;

    auto open_tile = [&](uint32_t tile, bool valid) {
        TilesPos t;
        const TileYX yx = map_tile(tile, n_tiles, (uint32_t)p.tiles_x, p.tile_map);
        const uint32_t tile_y = yx.y, tile_x = yx.x;
        t.row0 = (int32_t)(tile_y * 128u) + 16 * par;
        // The two 256-column windows of a workgroup lie eight windows apart inside each complete run
        // of sixteen (kMapSplitHalves; side by side otherwise and in what is left of a row): with
        // row-major units an XCD then reads every eighth 512-byte window of a row, the pattern of the
        // 1x16 kernel.  Measured at 8192 x 8192, 4/6-MSE: 37.8 us against 45.9 with the windows side
        // by side and 39.2 with one band of tiles per XCD.
        int64_t col0 = (int64_t)tile_x * 512 + 256 * half;
        if ((p.tile_map & kMapSplitHalves) && tile_x < 8u * (uint32_t)(p.cols_p >> 12))
            col0 = (int64_t)((tile_x >> 3) * 16 + (tile_x & 7u) + 8u * half) * 256;
        t.cb = (int32_t)(col0 >> 4) + lb;
        uint32_t x_bytes = valid ? 0xffffffffu : 0u;
        if (!FULL && valid) {
            const int64_t left = ((p.rows - t.row0) * p.ld - col0) * 2;  // (64-bit: p.rows is)
            x_bytes = left <= 0 ? 0u : (left > 0x7fffffffLL ? 0x7fffffffu : (uint32_t)left);
        }
        t.x_bytes = __builtin_amdgcn_readfirstlane(x_bytes);
        t.x_base = uniform64((uint64_t)(p.x + (int64_t)t.row0 * p.ld + col0));
        t.codes_base = PSEUDO ? 0 : uniform64((uint64_t)(p.codes + (int64_t)t.row0 * code_pitch + col0 / 2));
        t.out_base = PSEUDO ? uniform64((uint64_t)(p.pseudo_out + (int64_t)t.row0 * p.ldo + col0)) : 0;
        t.x_off = (FULL || t.cb < cols16) ? x_lane : 0x80000000u;
        t.unit_base = ((int64_t)tile_y * (sf_cols >> 2) + (col0 >> 6)) * 512 + 256 * par;
        return t;
    };
    // block `rstep` rows below the first row of the wavefront's share
    auto load = [&](const TilesPos &t, uint32_t rstep, Block16 &b) {
        const BufferRsrc rx = make_rsrc(reinterpret_cast<const void *>(uniform64(t.x_base)), __builtin_amdgcn_readfirstlane(t.x_bytes));
        const uint32_t step = __builtin_amdgcn_readfirstlane(rstep * x_row);
        u32x4 lo, hi;
        if (FULL) {
            lo = __builtin_amdgcn_raw_buffer_load_b128(rx, t.x_off, step, 0);
            hi = __builtin_amdgcn_raw_buffer_load_b128(rx, t.x_off + 16u, step, 0);
        } else {
            // the range check covers the per-lane offset only: keep the step inside it
            lo = __builtin_amdgcn_raw_buffer_load_b128(rx, t.x_off + step, 0, 0);
            hi = __builtin_amdgcn_raw_buffer_load_b128(rx, t.x_off + step + 16u, 0, 0);
        }
        b.w[0] = lo.x; b.w[1] = lo.y; b.w[2] = lo.z; b.w[3] = lo.w;
        b.w[4] = hi.x; b.w[5] = hi.y; b.w[6] = hi.z; b.w[7] = hi.w;
    };

    // pass-1 results first, the first group's loads (which do not depend on them) right behind:
    // loads return in order, so the setup below does not wait for the group
    uint32_t pm[4] = {0u, 0u, 0u, 0u};
    if (p.n_partials == 0) {
        pm[0] = p.partials[0];
    } else if (p.n_partials > 0) {
#pragma unroll
        for (int u = 0; u < kMaxPartials / kThreads; ++u)
            if ((int)threadIdx.x + u * kThreads < p.n_partials) pm[u] = p.partials[2 * (threadIdx.x + u * kThreads)];
    }
    uint32_t tile = blockIdx.x;
    TilesPos cur = open_tile(tile, tile < n_tiles);
    // One register set holds a group; each block's registers are refilled with the next group's as
    // soon as the block has been consumed.  (More loads in flight do not help: with a second set,
    // or with three wavefronts per SIMD and deeper queues, the launch took as long or longer --
    // wavefronts whose first loads were served late then finished late.)
    Block16 blk[4];
#pragma unroll
    for (int s = 0; s < 4; ++s) load(cur, 4 * s, blk[s]);

    uint32_t amax_bits;
    if (p.n_partials == 0) amax_bits = pm[0];
    else if (p.n_partials > 0) amax_bits = block_max_u32(max(max(pm[0], pm[1]), max(pm[2], pm[3])), red);
    else amax_bits = reduce_partials(p, red);  // small input: scan it here
    // wave-uniform constants, moved to scalar registers once computed
    auto sgpr = [](float v) { return u2f(__builtin_amdgcn_readfirstlane(f2u(v))); };
    QuantConsts k;
    k.amax = sgpr(u2f(amax_bits));
    k.enc = sgpr(p.c / k.amax);
    k.dec = sgpr(1.0f / (p.c / k.amax));
    k.qdiv = p.qdiv;
    k.errdiv = p.errdiv;
    if (blockIdx.x == 0 && threadIdx.x == 0 && p.amax_out) *p.amax_out = k.amax;
    const bool in_range = k.amax >= 0x1p-100f && k.amax <= 0x1p100f;
    const float enc_fast = in_range ? k.enc : 0.0f;
    const float rq = sgpr(1.0f / k.qdiv), rc = sgpr(1.0f / p.c);
    k.rerr = sgpr(1.0f / k.errdiv);
    k.fast_div = in_range && k.errdiv == 1536.0f;
    k.shortcut_ok = shortcut_range(k.amax);
    // dither key: launch arguments, or read from device memory (a captured launch whose key the caller advances)
    uint64_t key_seed = p.seed, key_offset = p.offset;
    if (SR && p.key) {
        key_seed = uniform64(p.key[0]);
        key_offset = uniform64(p.key[1]);
    }
    // pseudo-quantize: the table also serves the dequantization (divisor c: the selection's for the adaptive
    // rules; the static rules make no selection, so their table is built with c)
    constexpr bool kStaticRule = RULE == FOS_RULE_STATIC_6 || RULE == FOS_RULE_STATIC_4;
    QuantConsts kt = k;
    if (PSEUDO && kStaticRule) kt.errdiv = p.c;
    // (the 3-operation division is exact for these divisors only; the unbiased stochastic style rescales them)
    const bool fast_c = p.c == 1536.0f || p.c == 1792.0f || p.c == 2688.0f;
    const bool deq_lut = PSEUDO && in_range && fast_c && (amax_bits & 0xffffu) == 0 && kt.errdiv == p.c;
    if (threadIdx.x < 128) lut[threadIdx.x] = make_lut_entry(threadIdx.x, kt);
    __syncthreads();

    // one quantised block (row `rstep` rows below the share's first, + li) to memory
    auto emit = [&](const TilesPos &t, uint32_t rstep, uint32_t c0, uint32_t c1, uint32_t sbyte, bool pred) {
        const int32_t row = t.row0 + (int32_t)rstep + li;
        if (PSEUDO) {
            uint32_t w[8];
            const BlockOut o{c0, c1, sbyte};
            if (deq_lut) dequant_block_bf16_lut(o, lut[sbyte & 0x7fu], w);
            else if (in_range && fast_c) dequant_block_bf16<true>(o, k.amax, p.c, rc, w);
            else dequant_block_bf16<false>(o, k.amax, p.c, rc, w);
            if (pred && (FULL || (row < rows32 && t.cb < cols16))) {
                const u32x4 d0 = {w[0], w[1], w[2], w[3]}, d1 = {w[4], w[5], w[6], w[7]};
                // (a 128-bit buffer store with a scalar offset register reads its data late: the step
                // goes into the per-lane offset)
                const uint32_t o_off = o_lane + rstep * o_row;
                const BufferRsrc rout = make_rsrc(reinterpret_cast<const void *>(uniform64(t.out_base)), 0xffffffffu);
                // (plain stores: the two halves of a line come from two instructions and meet in L2)
                __builtin_amdgcn_raw_buffer_store_b128(d0, rout, o_off, 0, 0);
                __builtin_amdgcn_raw_buffer_store_b128(d1, rout, o_off + 16u, 0, 0);
            }
            return;
        }
        if (pred && (FULL || t.cb < (int32_t)sf_cols)) {  // inside the padded width
            const u32x2 c01 = {c0, c1};
            const BufferRsrc rcodes = make_rsrc(reinterpret_cast<const void *>(uniform64(t.codes_base)), 0xffffffffu);
            __builtin_amdgcn_raw_buffer_store_b64(c01, rcodes, c_lane, __builtin_amdgcn_readfirstlane(rstep * c_row), kStreamStore);
            if (!tiled) {
                const BufferRsrc rsf = make_rsrc(reinterpret_cast<const void *>(uniform64((uint64_t)(p.sf + (int64_t)t.row0 * sf_cols))), 0xffffffffu);
                __builtin_amdgcn_raw_buffer_store_b8((uint8_t)sbyte, rsf, (uint32_t)((rstep + li) * (uint32_t)sf_cols + (uint32_t)t.cb), 0, 0);
            }
        }
    };

    // Operation-by-operation form of ONE tile, block column `tl` of group q of the wavefront's
    // share, computed by the whole wavefront: the tile's 256 elements are spread over all 64 lanes
    // (read again, from L2 most likely), so that a rare undecided tile costs a few hundred
    // instructions instead of stalling its wavefront -- the launch ends with its slowest wavefront.
    // Errors: lane = (column c = lane & 15, row parity (lane >> 4) & 1, candidate lane >> 5) walks
    // its 8 rows top to bottom, which is torch.sum's order over a tile flattened row-major (per
    // column the even and the odd rows are summed top to bottom, A[l] = ((E[l] + E[l+8]) + O[l]) +
    // O[l+8], and the eight A[l] are summed left to right).  Codes: lane = (row lane >> 2, four
    // columns 4 (lane & 3) ...).  Writes the tile's outputs; returns the scale byte.
    auto slow_tile = [&](const TilesPos &t, uint32_t q, uint32_t tl) -> uint32_t {
        const BufferRsrc rx = make_rsrc(reinterpret_cast<const void *>(uniform64(t.x_base)), __builtin_amdgcn_readfirstlane(t.x_bytes));
        // the tile's first element, in bytes from the share's; a tile in the column padding reads zeros
        const int32_t cb_tile = __builtin_amdgcn_readfirstlane(t.cb - lb) + (int32_t)tl;
        const uint32_t gbase = (FULL || cb_tile < cols16) ? 32u * q * x_row + tl * 32u : 0x80000000u;
        const uint32_t c = lane & 15, rp = (lane >> 4) & 1;
        const bool cand_b = lane >= 32;
        float x[8];
#pragma unroll
        for (int m = 0; m < 8; ++m)
            x[m] = u2f((uint32_t)__builtin_amdgcn_raw_buffer_load_b16(rx, gbase + (rp + 2 * m) * x_row + c * 2u, 0, 0) << 16);
        float bmax = 0.0f;
#pragma unroll
        for (int m = 0; m < 8; ++m) bmax = fmaxf(bmax, fabsf(x[m]));
#pragma unroll
        for (int off = 32; off >= 1; off >>= 1) bmax = fmaxf(bmax, __shfl_xor(bmax, off));
        uint32_t sX;
        float sfX, invX;
        block_scale(k, bmax, !STATIC && !IF4 && cand_b, sX, sfX, invX);
        bool pickB = false;
        if (!STATIC) {
            float chain = 0.0f;
#pragma unroll
            for (int m = 0; m < 8; ++m) {
                const float xs = (sX != 0) ? x[m] * invX : 0.0f;
                const float r = e2m1_round(fabsf(xs));
                float deq = div_errdiv(((xs < 0.0f ? -r : r) * sfX) * k.amax, k);
                if (IF4) {
                    // (select_intfloat, reference.py:328-425: the INT4 candidate on the same scale)
                    const float qi = int4_round<false>(xs * 1.16666666f, 0.0f);
                    const float deq_i = div_errdiv(((qi * sfX) * k.amax) * 0.8571428571f, k);
                    deq = cand_b ? deq_i : deq;
                }
                const float e = error_term<RULE>(deq, x[m]);
                chain = m == 0 ? e : (MAXRULE ? fmaxf(chain, e) : chain + e);
            }
            float tot_a, tot_b;
            if (MAXRULE) {
                // the largest term of each candidate's 32 lanes
#pragma unroll
                for (int off = 16; off >= 1; off >>= 1) chain = fmaxf(chain, __shfl_xor(chain, off));
                tot_a = u2f(__builtin_amdgcn_readlane(f2u(chain), 0));
                tot_b = u2f(__builtin_amdgcn_readlane(f2u(chain), 32));
            } else {
                // lanes 0..7 of DPP rows 0 (candidate "6") and 2 (candidate "4"): E[l] own, E[l+8] eight lanes
                // on, O[l] and O[l+8] in the next DPP row
                const float chain8 = dpp_move<kDppRowShl + 8>(0.0f, chain);
                uint32_t ev, od, ev8, od8;
                rows_pairs(f2u(chain), ev, od);
                rows_pairs(f2u(chain8), ev8, od8);
                const float a = ((chain + chain8) + u2f(od)) + u2f(od8);
                float tot = a;
#pragma unroll
                for (int step = 0; step < 7; ++step) tot = dpp_move<kDppRowShr + 1>(-0.0f, tot) + a;  // lane 7: ((a0 + a1) + ...) + a7
                tot_a = u2f(__builtin_amdgcn_readlane(f2u(tot), 7));
                tot_b = u2f(__builtin_amdgcn_readlane(f2u(tot), 39));
            }
            pickB = tot_b < tot_a;
        }
        const uint32_t src_lane = pickB ? 32 : 0;
        const uint32_t sP = __builtin_amdgcn_readlane(sX, src_lane);
        const float invP = u2f(__builtin_amdgcn_readlane(f2u(invX), src_lane));
        const uint32_t s_out = IF4 && pickB ? sP + 128u : sP;  // what goes into the scale byte
        // codes: lane = (row, four columns)
        const uint32_t r = lane >> 2, cq = lane & 3;
        const u32x2 w = __builtin_amdgcn_raw_buffer_load_b64(rx, gbase + r * x_row + cq * 8u, 0, 0);
        uint32_t nibs = 0;
        float v[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const uint32_t word = i < 2 ? w.x : w.y;
            const float xe = (i & 1) ? u2f(word & 0xffff0000u) : u2f(word << 16);
            const float xs = (sP != 0) ? xe * invP : 0.0f;
            uint32_t nib = e2m1_mag_code(e2m1_round(fabsf(xs))) | (xs < 0.0f ? 8u : 0u);
            if (IF4 && pickB) nib = (uint32_t)((int)int4_round<false>(xs * 1.16666666f, 0.0f)) & 0xfu;
            nibs |= nib << (4 * i);
            v[i] = e2m1_value(nib & 0xfu);
        }
        const uint32_t rstep = 32u * q + r;
        const int32_t row = t.row0 + (int32_t)rstep;
        if (PSEUDO) {
            typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
            const float sfP = e4m3_decode(sP);
            uint32_t d[2];
#pragma unroll
            for (int h = 0; h < 2; ++h) {
                float2_t qv;
                qv.x = ((v[2 * h] * sfP) * k.amax) / p.c;
                qv.y = ((v[2 * h + 1] * sfP) * k.amax) / p.c;
                d[h] = __builtin_bit_cast(uint32_t, __builtin_convertvector(qv, bf16x2_t));
            }
            if (FULL || (row < rows32 && cb_tile < cols16)) {
                const u32x2 dd = {d[0], d[1]};
                const BufferRsrc rout = make_rsrc(reinterpret_cast<const void *>(uniform64(t.out_base)), 0xffffffffu);
                __builtin_amdgcn_raw_buffer_store_b64(dd, rout, rstep * o_row + tl * 32u + cq * 8u, 0, 0);
            }
            return sP;
        }
        const BufferRsrc rcodes = make_rsrc(reinterpret_cast<const void *>(uniform64(t.codes_base)), 0xffffffffu);
        __builtin_amdgcn_raw_buffer_store_b16((uint16_t)nibs, rcodes, rstep * c_row + tl * 8u + cq * 2u, 0, 0);
        if (!tiled && cq == 0) {
            const BufferRsrc rsf = make_rsrc(reinterpret_cast<const void *>(uniform64((uint64_t)(p.sf + (int64_t)t.row0 * sf_cols))), 0xffffffffu);
            __builtin_amdgcn_raw_buffer_store_b8((uint8_t)s_out, rsf, rstep * (uint32_t)sf_cols + (uint32_t)cb_tile, 0, 0);
        }
        return s_out;
    };

    // The same for the stochastic styles: lane & 15 = row of the tile, which the lane quantizes as one block of
    // the tile with the operation-by-operation block function (its tile reductions run along the 16 lanes of a
    // DPP row; the four DPP rows compute the same tile and the first one writes).  The dither is keyed per
    // row of the tile, as everywhere.
    auto slow_tile_sr = [&](const TilesPos &t, uint32_t q, uint32_t tl) -> uint32_t {
        const BufferRsrc rx = make_rsrc(reinterpret_cast<const void *>(uniform64(t.x_base)), __builtin_amdgcn_readfirstlane(t.x_bytes));
        const int32_t cb_tile = __builtin_amdgcn_readfirstlane(t.cb - lb) + (int32_t)tl;
        const uint32_t gbase = (FULL || cb_tile < cols16) ? 32u * q * x_row + tl * 32u : 0x80000000u;
        const uint32_t r = lane & 15;
        const u32x4 lo = __builtin_amdgcn_raw_buffer_load_b128(rx, gbase + r * x_row, 0, 0);
        const u32x4 hi = __builtin_amdgcn_raw_buffer_load_b128(rx, gbase + r * x_row + 16u, 0, 0);
        const uint32_t w[8] = {lo.x, lo.y, lo.z, lo.w, hi.x, hi.y, hi.z, hi.w};
        float x[16];
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            x[2 * j] = u2f(w[j] << 16);
            x[2 * j + 1] = u2f(w[j] & 0xffff0000u);
        }
        const uint32_t rstep = 32u * q + r;
        const int32_t row = t.row0 + (int32_t)rstep;
        uint32_t codes[2], sbyte;
        quantize_block_f32<FOS_DTYPE_NVFP4, RULE, FOS_ROUND_STOCHASTIC, true>(x, k, key_seed, key_offset,
                                                                              (uint64_t)((int64_t)row * sf_cols + cb_tile), codes, sbyte);
        if (PSEUDO) {
            uint32_t d[8];
            dequant_block_bf16<false>(BlockOut{codes[0], codes[1], sbyte}, k.amax, p.c, rc, d);
            if (lane < 16 && (FULL || (row < rows32 && cb_tile < cols16))) {
                const u32x4 d0 = {d[0], d[1], d[2], d[3]}, d1 = {d[4], d[5], d[6], d[7]};
                const BufferRsrc rout = make_rsrc(reinterpret_cast<const void *>(uniform64(t.out_base)), 0xffffffffu);
                __builtin_amdgcn_raw_buffer_store_b128(d0, rout, rstep * o_row + tl * 32u, 0, 0);
                __builtin_amdgcn_raw_buffer_store_b128(d1, rout, rstep * o_row + tl * 32u + 16u, 0, 0);
            }
            return sbyte;
        }
        if (lane < 16) {
            const u32x2 c01 = {codes[0], codes[1]};
            const BufferRsrc rcodes = make_rsrc(reinterpret_cast<const void *>(uniform64(t.codes_base)), 0xffffffffu);
            __builtin_amdgcn_raw_buffer_store_b64(c01, rcodes, rstep * c_row + tl * 8u, 0, 0);
            if (!tiled) {
                const BufferRsrc rsf = make_rsrc(reinterpret_cast<const void *>(uniform64((uint64_t)(p.sf + (int64_t)t.row0 * sf_cols))), 0xffffffffu);
                __builtin_amdgcn_raw_buffer_store_b8((uint8_t)sbyte, rsf, rstep * (uint32_t)sf_cols + (uint32_t)cb_tile, 0, 0);
            }
        }
        return sbyte;
    };

    // one group: four blocks per lane in, codes (or dequantised values) out; returns the scale byte
    auto process = [&](const TilesPos &t, uint32_t q, const TilesPos &nt, uint32_t nq) -> uint32_t {
        const int32_t grow = t.row0 + 32 * (int32_t)q;  // first row of the group (wave-uniform)
        uint32_t oc[4][2] = {{0, 0}, {0, 0}, {0, 0}, {0, 0}}, os = 0;
        bool need_slow = false;
        // a group that lies wholly in the row padding only writes zero codes and scales
        const bool padding = !FULL && grow >= rows32;
        if (in_range && !padding) {
            // max|x|: the high element of a word is compared with its neighbour's bits still
            // below it, which the final truncation removes (truncation is monotonic)
            float bmax = 0.0f;
#pragma unroll
            for (int s = 0; s < 4; ++s)
#pragma unroll
                for (int j = 0; j < 8; ++j)
                    bmax = fmaxf(fmaxf(fabsf(u2f(blk[s].w[j] << 16)), fabsf(u2f(blk[s].w[j]))), bmax);
            bmax = tile_max(u2f(f2u(bmax) & 0xffff0000u));
            // (the 3-operation division is exact for the divisors 6 and 4; the unbiased stochastic style rescales them)
            float bq;
            if (SR && k.qdiv != 6.0f && k.qdiv != 4.0f) bq = bmax / k.qdiv;
            else bq = div_const(bmax, k.qdiv, rq);
            const float s_hp6 = bq * enc_fast;
            const float s_hp4 = s_hp6 * 1.5f;
            const uint32_t pk = (uint32_t)__builtin_amdgcn_cvt_pk_fp8_f32(s_hp6, s_hp4, 0, false);
            const uint32_t s6 = pk & 0xffu, s4 = (pk >> 8) & 0xffu;
            const FastLutEntry A = lut[s6];
            FastLutEntry B = A;
            if (ADAPTIVE && !IF4) B = lut[s4];
            // the hardware convert saturates at 6 where the reference's unclamped rounding gives 8:
            // that needs a sub-normal scale byte rounded down by more than 7/6; a zero scale byte
            // of a non-zero tile has no scaled domain.  (The stochastic styles clamp to 6 in the
            // reference as well: only the zero scale byte is left out there.)
            const bool fast_ok = SR ? s6 != 0u : (s6 >= 8u || (s6 != 0u && bmax * A.inv < 7.0f));
            uint32_t cB[4][2];
            float SA = 0.0f, SB = 0.0f;
#pragma unroll
            for (int s = 0; s < 4; ++s) {
                if constexpr (IF4) block_candidates_if4(blk[s], A.inv, oc[s][0], oc[s][1], cB[s][0], cB[s][1], SA, SB);
                else if constexpr (SR)
                    block_candidates_sr<RULE>(blk[s], A.inv, B.inv, key_seed, key_offset, (uint64_t)((int64_t)(grow + 4 * s + li) * sf_cols + t.cb),
                                              oc[s][0], oc[s][1], cB[s][0], cB[s][1], SA, SB);
                else block_candidates<RULE>(blk[s], A.inv, B.inv, oc[s][0], oc[s][1], cB[s][0], cB[s][1], SA, SB);
                load(nt, 32 * nq + 4 * s, blk[s]);
            }
            int cmp = -1;
            if (ADAPTIVE) {
                SA = MAXRULE ? tile_max(SA) : tile_sum(SA);
                SB = MAXRULE ? tile_max(SB) : tile_sum(SB);
                // (IF4: one scale, so the two sums compare as they are)
                if (!k.shortcut_ok) cmp = 0;
                else if (IF4) cmp = shortcut_compare<FOS_RULE_MSE, true>(SA, 1.0f, SB, 1.0f);
                else cmp = shortcut_compare<RULE, true>(SA, shortcut_weight<RULE>(A), SB, shortcut_weight<RULE>(B));
            }
            // an all-zero tile came out as zero codes under the zero scale byte
            need_slow = !(bmax == 0.0f || (fast_ok && cmp != 0));
            if (ADAPTIVE && !IF4 && __builtin_amdgcn_ballot_w64(need_slow) != 0) {
                // candidates that dequantise to the same values element by element tie: "6" wins
                uint32_t viol = 1u;
                if (fast_ok && e4m3_decode(s4) == 1.5f * e4m3_decode(s6)) {
                    viol = 0u;
#pragma unroll
                    for (int s = 0; s < 4; ++s) viol |= tie_violations(oc[s][0], cB[s][0]) | tie_violations(oc[s][1], cB[s][1]);
                }
                viol = tile_or(viol);
                if (need_slow && viol == 0u) {
                    cmp = -1;
                    need_slow = false;
                }
            }
            const bool pickB = ADAPTIVE && cmp > 0;
            os = IF4 ? (pickB ? s6 + 128u : s6) : (pickB ? s4 : s6);
            if (ADAPTIVE) {
#pragma unroll
                for (int s = 0; s < 4; ++s) {
                    oc[s][0] = pickB ? cB[s][0] : oc[s][0];
                    oc[s][1] = pickB ? cB[s][1] : oc[s][1];
                }
            }
        } else {
#pragma unroll
            for (int s = 0; s < 4; ++s) load(nt, 32 * nq + 4 * s, blk[s]);
            need_slow = !padding && (FULL || t.cb < (int32_t)sf_cols);  // (not beyond the padded width)
        }
#pragma unroll
        for (int s = 0; s < 4; ++s) emit(t, 32 * q + 4 * s, oc[s][0], oc[s][1], os, !need_slow);
        // (the four lanes of a tile are flagged together)
        uint64_t pending = __builtin_amdgcn_ballot_w64(need_slow);
        while (pending != 0) {
            const uint32_t tl = (uint32_t)__builtin_ctzll(pending) & 15u;
            uint32_t sP;
            if constexpr (SR) sP = slow_tile_sr(t, q, tl);
            else sP = slow_tile(t, q, tl);
            if ((uint32_t)lb == tl) os = sP;
            pending &= ~(0x0001000100010001ull << tl);
        }
        return os;
    };

    while (tile < n_tiles) {
        const uint32_t next = tile + gridDim.x;
        const bool has_next = next < n_tiles;
        const TilesPos nxt = open_tile(has_next ? next : tile, has_next);  // without a next tile: loads of nothing
        uint32_t sw = 0;  // the lane's scale bytes of the four groups
#pragma nounroll
        for (uint32_t q = 0; q < 4; ++q) {
            sw |= process(cur, q, q == 3 ? nxt : cur, q == 3 ? 0u : q + 1) << (8 * q);
        }
        if (tiled) {
            // 16-byte unit of rows r, r + 32, r + 64, r + 96 and block columns 4 g .. 4 g + 3: word q =
            // group q's bytes of the four lanes of the quad; the 16 rows of the band share it
            const uint32_t l0 = (uint32_t)__builtin_amdgcn_mov_dpp((int)sw, 0x00, 0xf, 0xf, true);
            const uint32_t l1 = (uint32_t)__builtin_amdgcn_mov_dpp((int)sw, 0x55, 0xf, 0xf, true);
            const uint32_t l2 = (uint32_t)__builtin_amdgcn_mov_dpp((int)sw, 0xaa, 0xf, 0xf, true);
            const uint32_t l3 = (uint32_t)__builtin_amdgcn_mov_dpp((int)sw, 0xff, 0xf, 0xf, true);
            const uint4 unit = make_uint4(quad_bytes<0>(l0, l1, l2, l3), quad_bytes<1>(l0, l1, l2, l3),
                                          quad_bytes<2>(l0, l1, l2, l3), quad_bytes<3>(l0, l1, l2, l3));
            if (FULL || cur.cb < (int32_t)sf_cols)
                *reinterpret_cast<uint4 *>(p.sf + cur.unit_base + (lb >> 2) * 512 + (4 * (lb & 3) + li) * 16) = unit;
        }
        cur = nxt;
        tile = next;
    }
}

}  // namespace

template <int RULE, bool PSEUDO, bool SR>
void launch_quantize_nvfp4_tiles(QuantParams &p, hipStream_t s) {
    p.tiles_x = (int)((p.cols_p + 511) / 512);
    const int64_t n = (p.rows_p / 128) * p.tiles_x;
    // three workgroups per compute unit (256 CUs; four would fit), walking the tiles between them:
    // measured best at 8192 x 8192 (43.9 us against 45.9 with 1024).  FOS_QUANT_GRID overrides for
    // tuning runs.
    int64_t grid = 768;
    if (const int forced = tuning().quant_grid) grid = forced > 0 ? forced : grid;
    if (grid > n) grid = n;
    p.tile_map = kMapSplitHalves;
    if (const int forced = tuning().quant_map) p.tile_map = forced - 1;
    const bool full = p.rows % 128 == 0 && p.cols % 512 == 0;
    if (full)
        hipLaunchKernelGGL((quantize_nvfp4_tiles_kernel<RULE, true, PSEUDO, false, SR>), dim3((unsigned)grid), dim3(kThreads), 0, s, p);
    else
        hipLaunchKernelGGL((quantize_nvfp4_tiles_kernel<RULE, false, PSEUDO, false, SR>), dim3((unsigned)grid), dim3(kThreads), 0, s, p);
}

// IF4 with the MSE rule, round to nearest, 16x16 tiles, aligned input.
void launch_quantize_if4_mse_tiles(QuantParams &p, hipStream_t s) {
    p.tiles_x = (int)((p.cols_p + 511) / 512);
    const int64_t n = (p.rows_p / 128) * p.tiles_x;
    int64_t grid = 768;
    if (const int forced = tuning().quant_grid) grid = forced > 0 ? forced : grid;
    if (grid > n) grid = n;
    p.tile_map = kMapSplitHalves;
    if (const int forced = tuning().quant_map) p.tile_map = forced - 1;
    if (p.rows % 128 == 0 && p.cols % 512 == 0)
        hipLaunchKernelGGL((quantize_nvfp4_tiles_kernel<FOS_RULE_MSE, true, false, true>), dim3((unsigned)grid), dim3(kThreads), 0, s, p);
    else
        hipLaunchKernelGGL((quantize_nvfp4_tiles_kernel<FOS_RULE_MSE, false, false, true>), dim3((unsigned)grid), dim3(kThreads), 0, s, p);
}

template void launch_quantize_nvfp4_tiles<FOS_RULE_STATIC_6, false, false>(QuantParams &, hipStream_t);
template void launch_quantize_nvfp4_tiles<FOS_RULE_STATIC_6, true, false>(QuantParams &, hipStream_t);
template void launch_quantize_nvfp4_tiles<FOS_RULE_STATIC_6, false, true>(QuantParams &, hipStream_t);
template void launch_quantize_nvfp4_tiles<FOS_RULE_STATIC_6, true, true>(QuantParams &, hipStream_t);
template void launch_quantize_nvfp4_tiles<FOS_RULE_MSE, false, false>(QuantParams &, hipStream_t);
template void launch_quantize_nvfp4_tiles<FOS_RULE_MSE, true, false>(QuantParams &, hipStream_t);
template void launch_quantize_nvfp4_tiles<FOS_RULE_MSE, false, true>(QuantParams &, hipStream_t);
template void launch_quantize_nvfp4_tiles<FOS_RULE_MSE, true, true>(QuantParams &, hipStream_t);
template void launch_quantize_nvfp4_tiles<FOS_RULE_MAE, false, false>(QuantParams &, hipStream_t);
template void launch_quantize_nvfp4_tiles<FOS_RULE_MAE, true, false>(QuantParams &, hipStream_t);
template void launch_quantize_nvfp4_tiles<FOS_RULE_MAE, false, true>(QuantParams &, hipStream_t);
template void launch_quantize_nvfp4_tiles<FOS_RULE_MAE, true, true>(QuantParams &, hipStream_t);
template void launch_quantize_nvfp4_tiles<FOS_RULE_ABS_MAX, false, false>(QuantParams &, hipStream_t);
template void launch_quantize_nvfp4_tiles<FOS_RULE_ABS_MAX, true, false>(QuantParams &, hipStream_t);
template void launch_quantize_nvfp4_tiles<FOS_RULE_ABS_MAX, false, true>(QuantParams &, hipStream_t);
template void launch_quantize_nvfp4_tiles<FOS_RULE_ABS_MAX, true, true>(QuantParams &, hipStream_t);

}  // namespace fos
