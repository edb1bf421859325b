// Pass 2 for NVFP4 with round-to-nearest or a stochastic rounding style and 1x16 blocks, around the fast
// block formulation of fos_quantize_fast.h (quantize_nvfp4_rows_kernel): a wavefront covers 4 rows x 16
// blocks, i.e. 512 contiguous bytes per row.  Measured on MI355X, a wavefront that touches 16
// rows x 128 bytes streams at ~4.1 TB/s while 4 rows x 512 bytes reaches ~6 TB/s, so the
// row-contiguous mapping is what the HBM-bound path uses.  A 256-thread workgroup
// covers 128 rows x 256 columns in eight steps of 16 rows (the next step's loads are
// issued before the current step is processed), stages the 4 complete 128x4 scale
// tiles in LDS and writes them as one contiguous 2 KiB run.  16x16 tiles have the same mapping in
// fos_quantize_tiles.hip; the dispatch by rule, block shape and style is at the end of this file.
#include <cstdlib>

#include "fos_buffer.h"
#include "fos_quantize_kernel.h"
#include "fos_tuning.h"

namespace fos {

// 1x16 blocks, row-contiguous mapping.  Workgroup tile: 128 rows x 256 columns, walked in
// eight steps; in a step a wavefront covers 4 rows x 16 blocks (lane -> block column lane & 15
// of row lane >> 4), i.e. 512 contiguous bytes per row.  Wavefront w owns rows
// 32 q + 8 w + 4 h + i (q = 0..3, h = 0..1: step g = 2 q + h; i = lane >> 4) of the tile: in the
// 128x4 scale layout the scales of rows r, r + 32, r + 64, r + 96 share a 16-byte unit, so these
// 32 rows' scales are 128 contiguous bytes of each of the tile's four scale tiles, which the
// wavefront assembles in its own 512 bytes of LDS and writes itself -- the loop has no
// workgroup barrier.  Workgroups stride over the tiles (the setup -- tensor maximum, scale
// table -- is paid once) and the loads run three steps ahead, across tile boundaries.
// Input, codes and the pseudo-quantize output go through buffer instructions: a
// wave-uniform descriptor per tile, a per-lane 32-bit offset that is the same for every
// tile, and a uniform offset per step, so the loop holds no 64-bit address arithmetic.  A
// ragged tile's descriptor ends with the tensor's last row and lanes past the last column
// get an offset beyond it: both read zeros, which is the padding the reference adds.
// FULL: rows % 128 == 0 and cols % 256 == 0, no bounds checks.
struct RowsTile {
    uint64_t x_base, codes_base, out_base;  // addresses of the tile's first input element / code byte / output element
    uint32_t x_bytes;    // extent of the input descriptor
    uint32_t x_off;      // this lane's offset into it (beyond the descriptor for a lane past the last column)
    int64_t row_base;    // first row of the tile
    int64_t cb;          // this lane's block column in the tensor
    uint32_t tile_y, tile_x;
};

// IF4: the IF4 format with its MSE rule (E2M1 candidate against INT4 candidate on one scale,
// quantize_block_if4_mse) instead of NVFP4.
// F16: fp16 elements instead of bf16 (NVFP4, round to nearest, codes out).
template <int RULE, bool FULL, bool PSEUDO, bool SR, bool IF4 = false, bool F16 = false>
// (the stochastic instantiations hold two sets of scaled values and the Philox state: with 128
// registers they spilled -- 30 MB of scratch traffic per launch at 8192 x 8192 -- and the launch
// grid of three workgroups per compute unit leaves 168; the IF4 instantiation spilled as well)
__global__ __launch_bounds__(kThreads) __attribute__((amdgpu_waves_per_eu((SR || IF4) ? 3 : 4, (SR || IF4) ? 3 : 8))) void quantize_nvfp4_rows_kernel(
    const QuantParams p) {
    __shared__ uint32_t red[4];
    // per wavefront: 4 scale tiles x 128 bytes (pseudo-quantize: the 2 KiB of a step's output instead)
    __shared__ __attribute__((aligned(16))) uint32_t sf_stage[4][PSEUDO ? 512 : 128];
    __shared__ __attribute__((aligned(16))) FastLutEntry lut[128];
    // undecided blocks are evaluated exactly one at a time, spread over the wavefront (whole tiles only: every
    // lane takes part); per wavefront 16 words of staging
    constexpr bool kSpread = FULL && !IF4 && (RULE == FOS_RULE_MSE || RULE == FOS_RULE_MAE);
    __shared__ __attribute__((aligned(16))) uint32_t exact_stage[4][kSpread ? 16 : 4];

    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int64_t sf_cols = p.cols_p >> 4;
    const int lb = lane & 15;               // block column inside the tile
    const int rl = wave * 8 + (lane >> 4);  // this lane's row in step 0
    const bool tiled = !PSEUDO && p.sf_layout == FOS_SF_TILED_128X4;
    const int64_t code_pitch = p.cols_p >> 1;
    const uint32_t n_tiles = (uint32_t)(p.rows_p >> 7) * (uint32_t)p.tiles_x;
    // byte offsets inside a tile (the host checked that a tile spans less than 2^31 bytes);
    // step g starts 32 (g >> 1) + 4 (g & 1) rows below step 0
    const uint32_t x_lane = (uint32_t)(rl * p.ld + lb * 16) * 2u, x_row = (uint32_t)p.ld * 2u;
    const uint32_t c_lane = (uint32_t)(rl * code_pitch + lb * 8), c_row = (uint32_t)code_pitch;
    const uint32_t o_lane = PSEUDO ? (uint32_t)(rl * p.ldo + lb * 16) * 2u : 0u, o_row = PSEUDO ? (uint32_t)p.ldo * 2u : 0u;
    auto step_row = [](int g) { return 32 * (g >> 1) + 4 * (g & 1); };
    // scale byte of (q, h, i; block column lb) in the wavefront's staging area: 128 bytes per
    // scale tile lb >> 2, unit 4 h + i, byte 4 q + (lb & 3)
    uint8_t *stage = reinterpret_cast<uint8_t *>(sf_stage[wave]) + (lb >> 2) * 128 + (lane >> 4) * 16 + (lb & 3);

    auto open_tile = [&](uint32_t tile, bool valid) {
        RowsTile t;
        const TileYX yx = map_tile(tile, n_tiles, (uint32_t)p.tiles_x, p.tile_map);
        t.tile_y = yx.y;
        t.tile_x = yx.x;
        t.row_base = (int64_t)t.tile_y * 128;
        const int64_t col_base = (int64_t)t.tile_x * 256;
        t.cb = (int64_t)t.tile_x * 16 + lb;
        // input: everything from the tile's first element to the end of the tensor's last row
        uint32_t x_bytes = valid ? 0xffffffffu : 0u;
        if (!FULL && valid) {
            const int64_t left = ((p.rows - t.row_base) * p.ld - col_base) * 2;
            x_bytes = left <= 0 ? 0u : (left > 0x7fffffffLL ? 0x7fffffffu : (uint32_t)left);
        }
        t.x_bytes = __builtin_amdgcn_readfirstlane(x_bytes);
        t.x_base = uniform64((uint64_t)(p.x + t.row_base * p.ld + col_base));
        t.codes_base = PSEUDO ? 0 : uniform64((uint64_t)(p.codes + t.row_base * code_pitch + col_base / 2));
        t.out_base = PSEUDO ? uniform64((uint64_t)(p.pseudo_out + t.row_base * p.ldo + col_base)) : 0;
        t.x_off = (FULL || t.cb * 16 < p.cols) ? x_lane : 0x80000000u;
        return t;
    };
    auto load = [&](const RowsTile &t, int g, Block16 &b) __attribute__((always_inline)) {
        const BufferRsrc rx = make_rsrc(reinterpret_cast<const void *>(uniform64(t.x_base)), __builtin_amdgcn_readfirstlane(t.x_bytes));
        u32x4 lo, hi;
        if (FULL) {
            lo = __builtin_amdgcn_raw_buffer_load_b128(rx, t.x_off, step_row(g) * x_row, 0);
            hi = __builtin_amdgcn_raw_buffer_load_b128(rx, t.x_off + 16u, step_row(g) * x_row, 0);
        } else {
            // the range check covers the per-lane offset only: keep the step inside it
            lo = __builtin_amdgcn_raw_buffer_load_b128(rx, t.x_off + step_row(g) * x_row, 0, 0);
            hi = __builtin_amdgcn_raw_buffer_load_b128(rx, t.x_off + step_row(g) * x_row + 16u, 0, 0);
        }
        b.w[0] = lo.x; b.w[1] = lo.y; b.w[2] = lo.z; b.w[3] = lo.w;
        b.w[4] = hi.x; b.w[5] = hi.y; b.w[6] = hi.z; b.w[7] = hi.w;
    };
    // pass-1 results first, the first input loads (which do not depend on them) right behind: loads
    // return in order, so the setup below does not wait for the input
    uint32_t pm[4] = {0u, 0u, 0u, 0u};
    if (p.n_partials == 0) {
        pm[0] = p.partials[0];
    } else if (p.n_partials > 0) {
#pragma unroll
        for (int u = 0; u < kMaxPartials / kThreads; ++u)
            if ((int)threadIdx.x + u * kThreads < p.n_partials) pm[u] = p.partials[2 * (threadIdx.x + u * kThreads)];
    }
    uint32_t tile = blockIdx.x;
    RowsTile cur = open_tile(tile, tile < n_tiles);
    Block16 ring[4];
    load(cur, 0, ring[0]);
    load(cur, 1, ring[1]);
    load(cur, 2, ring[2]);

    // setup: tensor maximum, constants, per-scale table
    uint32_t amax_bits;
    if (p.n_partials == 0) amax_bits = pm[0];
    else if (p.n_partials > 0) amax_bits = block_max_u32(max(max(pm[0], pm[1]), max(pm[2], pm[3])), red);
    else amax_bits = reduce_partials(p, red);  // small input: scan it here
    QuantConsts k;
    k.amax = u2f(amax_bits);
    k.enc = p.c / k.amax;
    k.dec = 1.0f / (p.c / k.amax);
    k.qdiv = p.qdiv;
    k.errdiv = p.errdiv;
    // (the exact evaluation needs fq * s * amax exact: a maximum of the element type's significant bits)
    k.exact_ok = k.errdiv == 1536.0f && (amax_bits & (F16 ? 0x1fffu : 0xffffu)) == 0;
    k.shortcut_ok = shortcut_range(k.amax);
    if (blockIdx.x == 0 && threadIdx.x == 0 && p.amax_out) *p.amax_out = k.amax;
    // dither key: launch arguments, or read from device memory (a captured launch whose key the caller advances)
    uint64_t key_seed = p.seed, key_offset = p.offset;
    if (SR && p.key) {
        key_seed = uniform64(p.key[0]);
        key_offset = uniform64(p.key[1]);
    }
    const bool in_range = k.amax >= 0x1p-100f && k.amax <= 0x1p100f;
    const float enc_fast = in_range ? k.enc : 0.0f;
    const float rq = 1.0f / k.qdiv, rc = 1.0f / p.c;
    // pseudo-quantize: the table also serves the dequantization, whose divisor c is the selection's for the
    // adaptive rules; the static rules make no selection, so their table is built with c
    constexpr bool kStaticRule = RULE == FOS_RULE_STATIC_6 || RULE == FOS_RULE_STATIC_4;
    QuantConsts kt = k;
    if (PSEUDO && kStaticRule) kt.errdiv = p.c;
    // (the 3-operation division is exact for these divisors only; the unbiased stochastic style rescales them)
    const bool fast_c = p.c == 1536.0f || p.c == 1792.0f || p.c == 2688.0f;
    const bool deq_lut = PSEUDO && in_range && fast_c && (amax_bits & 0xffffu) == 0 && kt.errdiv == p.c;
    // the MSE decision in its product form (bf16 elements, round to nearest)
    constexpr bool kProduct = RULE == FOS_RULE_MSE && !SR && !IF4 && !F16;
    if (threadIdx.x < 128) lut[threadIdx.x] = make_lut_entry<kProduct>(threadIdx.x, kt);
    __syncthreads();

    auto process = [&](const RowsTile &t, int g, const Block16 &b) __attribute__((always_inline)) {
        if (!FULL && t.cb >= sf_cols) return;  // past the padded width
        const int64_t row = t.row_base + step_row(g) + rl;
        // a step that lies wholly in the row padding (decode-sized inputs: most steps) only
        // writes its zero codes and scales
        const bool padding_step = !FULL && t.row_base + step_row(g) + wave * 8 >= p.rows;
        BlockOut o{0u, 0u, 0u};
        if (!padding_step) {
            if constexpr (IF4) o = quantize_block_if4_mse<false>(b, k, enc_fast, rq, in_range, lut);
            else if constexpr (kSpread) {
                ExactRequest req;
                o = quantize_block_nvfp4_fast<RULE, false, SR, F16, kProduct, true>(b, k, enc_fast, rq, in_range, lut, key_seed, key_offset,
                                                                                    (uint64_t)(row * sf_cols + t.cb), &req);
                const uint64_t asking = __builtin_amdgcn_ballot_w64(req.wanted);
                if (asking != 0) {
                    // a few lanes (what data brings: one wavefront step in ten has one): one block at a time across the
                    // wavefront; many lanes (a tensor outside the shortcuts' range: all of them): every lane its own
                    bool pick_second = false;
                    if (__builtin_popcountll(asking) <= 6)
                        pick_second = exact_pick_b_spread<RULE, F16>(req.wanted, b, o.c0, o.c1, req.b0, req.b1, lut[o.s & 0x7fu],
                                                                     lut[req.sB & 0x7fu], exact_stage[wave]);
                    else if (req.wanted)
                        pick_second = exact_pick_b_1d_packed<RULE, F16>(b, o.c0, o.c1, req.b0, req.b1, lut[o.s & 0x7fu], lut[req.sB & 0x7fu]);
                    if (req.wanted && pick_second) o = BlockOut{req.b0, req.b1, req.sB};
                }
            } else o = quantize_block_nvfp4_fast<RULE, false, SR, F16, kProduct>(b, k, enc_fast, rq, in_range, lut, key_seed, key_offset,
                                                                                 (uint64_t)(row * sf_cols + t.cb));
        }
        if (PSEUDO) {
            uint32_t w[8];
            if constexpr (IF4 || F16) {
                if (in_range && fast_c) dequant_block_any<IF4, F16, true>(o, k.amax, p.c, rc, w);
                else dequant_block_any<IF4, F16, false>(o, k.amax, p.c, rc, w);
            } else {
                if (deq_lut) dequant_block_bf16_lut(o, lut[o.s & 0x7fu], w);
                else if (in_range && fast_c) dequant_block_bf16<true>(o, k.amax, p.c, rc, w);
                else dequant_block_bf16<false>(o, k.amax, p.c, rc, w);
            }
            const BufferRsrc rout = make_rsrc(reinterpret_cast<const void *>(uniform64(t.out_base)), 0xffffffffu);
            if constexpr (FULL) {
                // A lane's 32 bytes would leave as two stores of 16, each instruction covering half of every
                // line.  The wavefront's 4 rows x 512 bytes go through its staging area instead (free in a
                // pseudo-quantize launch, which writes no scales): lane l then stores the 16-byte pieces l and
                // 64 + l of those 2 KiB, whole lines per instruction, non-temporally.
                uint4 *swap = reinterpret_cast<uint4 *>(sf_stage[wave]);
                swap[2 * lane] = make_uint4(w[0], w[1], w[2], w[3]);
                swap[2 * lane + 1] = make_uint4(w[4], w[5], w[6], w[7]);
                __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
                __builtin_amdgcn_wave_barrier();
                __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
                const uint4 a = swap[lane], b = swap[64 + lane];
                __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
                __builtin_amdgcn_wave_barrier();
                const u32x4 d0 = {a.x, a.y, a.z, a.w}, d1 = {b.x, b.y, b.z, b.w};
                // piece l: row l >> 5 of the step, bytes 16 (l & 31) ...; piece 64 + l: two rows further down
                const uint32_t o_off = (uint32_t)(wave * 8 + step_row(g) + (lane >> 5)) * o_row + (uint32_t)(lane & 31) * 16u;
                __builtin_amdgcn_raw_buffer_store_b128(d0, rout, o_off, 0, kStreamStore);
                __builtin_amdgcn_raw_buffer_store_b128(d1, rout, o_off + 2u * o_row, 0, kStreamStore);
            } else if (row < p.rows && t.cb * 16 < p.cols) {
                const u32x4 d0 = {w[0], w[1], w[2], w[3]}, d1 = {w[4], w[5], w[6], w[7]};
                // (a 128-bit buffer store with a scalar offset register reads its data late: a VALU
                // write to the data registers right behind it reached memory in tests, so the step goes
                // into the per-lane offset)
                const uint32_t o_off = o_lane + step_row(g) * o_row;
                // (plain stores: the two halves of a line come from two instructions and meet in L2)
                __builtin_amdgcn_raw_buffer_store_b128(d0, rout, o_off, 0, 0);
                __builtin_amdgcn_raw_buffer_store_b128(d1, rout, o_off + 16u, 0, 0);
            }
            return;
        }
        const u32x2 c01 = {o.c0, o.c1};
        const BufferRsrc rcodes = make_rsrc(reinterpret_cast<const void *>(uniform64(t.codes_base)), 0xffffffffu);
        __builtin_amdgcn_raw_buffer_store_b64(c01, rcodes, c_lane, step_row(g) * c_row, kStreamStore);
        if (tiled) stage[(g & 1) * 64 + (g >> 1) * 4] = (uint8_t)o.s;
        else p.sf[row * sf_cols + t.cb] = (uint8_t)o.s;
    };

    __builtin_amdgcn_s_setprio(3);
    while (tile < n_tiles) {
        const uint32_t next = tile + gridDim.x;
        const bool has_next = next < n_tiles;
        const RowsTile nxt = open_tile(has_next ? next : tile, has_next);  // without a next tile: loads of nothing
        auto step = [&](int g) __attribute__((always_inline)) {
            // in its last tile a wavefront gives way, step by step, to those that are further behind
            if (!has_next && (g & 1) == 0) {
                if (g == 0) __builtin_amdgcn_s_setprio(3);
                if (g == 2) __builtin_amdgcn_s_setprio(2);
                if (g == 4) __builtin_amdgcn_s_setprio(1);
                if (g == 6) __builtin_amdgcn_s_setprio(0);
            }
            if (g + 3 < 8) load(cur, g + 3, ring[(g + 3) & 3]);
            else load(nxt, g + 3 - 8, ring[(g + 3) & 3]);
            process(cur, g, ring[g & 3]);
        };
        if constexpr (PSEUDO && SR) {
            // (the largest instantiations: beyond the size up to which the unroll pragma is honoured, and a loop
            // that stays a loop indexes the ring of input registers at run time; unrolled by construction)
            static_for<0, 8>(step);
        } else {
#pragma unroll
            for (int g = 0; g < 8; ++g) step(g);
        }
        if (tiled) {
            // the wavefront's own 4 x 128 bytes: written above by its lanes, read back here in
            // output order (LDS operations of one wavefront complete in order)
            __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
            __builtin_amdgcn_wave_barrier();
            __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
            const int64_t group = (int64_t)cur.tile_x * 4 + (lane >> 4);
            const uint2 v = reinterpret_cast<const uint2 *>(sf_stage[wave])[lane];
            if (FULL || group < (sf_cols >> 2))
                *reinterpret_cast<uint2 *>(p.sf + ((int64_t)cur.tile_y * (sf_cols >> 2) + group) * 512 + wave * 128 + (lane & 15) * 8) = v;
            __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
            __builtin_amdgcn_wave_barrier();
        }
        cur = nxt;
        tile = next;
    }
}

// 16x16 tiles on the row-contiguous mapping (fos_quantize_tiles.hip): every rule and rounding style.
template <int RULE, bool PSEUDO, bool SR>
void launch_quantize_nvfp4_tiles(QuantParams &p, hipStream_t s);

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
        // three workgroups per compute unit (256 CUs), each walking several tiles: measured at
        // 8192 x 8192 with the 4/6-MSE rule, 768 workgroups take 31.6 us where 1024 take 33.2 and the
        // 1280 that fit (<= 102 VGPRs) 35.5 -- the setup is paid fewer times and the wavefronts stay
        // in their streaming loop longer.  FOS_QUANT_GRID overrides for tuning runs.
        int64_t grid = 768;
        if (const int forced = tuning().quant_grid) grid = forced > 0 ? forced : grid;
        if (grid > n) grid = n;
        p.tile_map = kMapRowMajor;
        if (const int forced = tuning().quant_map) p.tile_map = forced - 1;
        const bool full = p.rows % 128 == 0 && p.cols % 256 == 0;
        if constexpr (!SR) {
            if (p.x_type == FOS_T_F16) {
                if (full)
                    hipLaunchKernelGGL((quantize_nvfp4_rows_kernel<RULE, true, PSEUDO, false, false, true>), dim3((unsigned)grid), dim3(kThreads), 0, s, p);
                else
                    hipLaunchKernelGGL((quantize_nvfp4_rows_kernel<RULE, false, PSEUDO, false, false, true>), dim3((unsigned)grid), dim3(kThreads), 0, s, p);
                return;
            }
        }
        if (full)
            hipLaunchKernelGGL((quantize_nvfp4_rows_kernel<RULE, true, PSEUDO, SR>), dim3((unsigned)grid), dim3(kThreads), 0, s, p);
        else
            hipLaunchKernelGGL((quantize_nvfp4_rows_kernel<RULE, false, PSEUDO, SR>), dim3((unsigned)grid), dim3(kThreads), 0, s, p);
        return;
    }
    launch_quantize_nvfp4_tiles<RULE, PSEUDO, SR>(p, s);
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

// IF4 with the MSE rule, round to nearest, 1x16 blocks, aligned input: the streaming kernel.
void launch_quantize_if4_mse_rows(QuantParams &p, hipStream_t s) {
    p.tiles_x = (int)((p.cols_p + 255) / 256);
    const int64_t n = (p.rows_p / 128) * p.tiles_x;
    int64_t grid = 768;
    if (const int forced = tuning().quant_grid) grid = forced > 0 ? forced : grid;
    if (grid > n) grid = n;
    p.tile_map = kMapRowMajor;
    if (const int forced = tuning().quant_map) p.tile_map = forced - 1;
    const bool full = p.rows % 128 == 0 && p.cols % 256 == 0;
    if (p.pseudo_out) {
        if (full) hipLaunchKernelGGL((quantize_nvfp4_rows_kernel<FOS_RULE_MSE, true, true, false, true>), dim3((unsigned)grid), dim3(kThreads), 0, s, p);
        else hipLaunchKernelGGL((quantize_nvfp4_rows_kernel<FOS_RULE_MSE, false, true, false, true>), dim3((unsigned)grid), dim3(kThreads), 0, s, p);
    } else if (full) {
        hipLaunchKernelGGL((quantize_nvfp4_rows_kernel<FOS_RULE_MSE, true, false, false, true>), dim3((unsigned)grid), dim3(kThreads), 0, s, p);
    } else {
        hipLaunchKernelGGL((quantize_nvfp4_rows_kernel<FOS_RULE_MSE, false, false, false, true>), dim3((unsigned)grid), dim3(kThreads), 0, s, p);
    }
}

// `sr`: a stochastic style on an aligned input.  The fast exact evaluation is tied to the
// selection divisor 1536; with the unbiased style's rescaled divisor an inconclusive
// shortcut falls back to the operation-by-operation form.
void launch_quantize_nvfp4_fast(QuantParams &p, int rule, bool two_d, bool aligned, bool sr, hipStream_t s) {
    if (sr && p.pseudo_out) by_rule<true, true>(p, rule, two_d, aligned, s);
    else if (sr) by_rule<false, true>(p, rule, two_d, aligned, s);
    else if (p.pseudo_out) by_rule<true, false>(p, rule, two_d, aligned, s);
    else by_rule<false, false>(p, rule, two_d, aligned, s);
}

}  // namespace fos
