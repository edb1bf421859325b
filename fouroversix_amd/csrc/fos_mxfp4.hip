// gfx950 MXFP4: E2M1 codes with one E8M0 (power-of-two) scale per 1x32 block, no tensor
// scale (OCP microscaling).  Three kernels:
//
//  * quantize: one streaming pass (there is no tensor maximum to find first) with the
//    arithmetic of quantize_to_mxfp4 + fake_quantize_to_e2m1
//    (src/fouroversix/quantize/pytorch/reference.py:30-51, 149-181): scale = the block
//    maximum over qmax rounded UP to a power of two, values divided by it (exact) and
//    rounded to the E2M1 grid, half to even.
//  * dequantize: the mx branch of QuantizeBackendBase.dequantize
//    (src/fouroversix/quantize/backend.py:89-160): value and scale meet in fp16.
//  * GEMM: this is the one format the matrix cores take natively --
//    v_mfma_scale_f32_32x32x64_f8f6f4 multiplies packed FP4 operands and applies one E8M0
//    scale per row and 32-wide K block, exactly the MX block -- so packed codes go
//    global -> LDS -> MFMA without any conversion, at four times the fp16 MFMA rate.
//    Stands in for gemm_mxfp4mxfp4_accum_fp32_out_bf16_tnt
//    (src/fouroversix/csrc/bindings.cpp:26-35, src/fouroversix/matmul/cutlass/backend.py:79-110).
#include <hip/hip_runtime.h>
#include <stdint.h>

#include <cstdlib>

#include "fos_buffer.h"
#include "fos_quantize_fast.h"
#include "fos_tuning.h"
#include "fouroversix_hip.h"

namespace fos {

// ---------------------------------------------------------------------------------------
// quantize
// ---------------------------------------------------------------------------------------

struct MxQuantParams {
    const uint16_t *x;
    int64_t rows, cols, ld;
    int64_t rows_p, cols_p;  // rows to 128, cols to 128
    uint8_t *codes;          // [rows_p, cols_p / 2]
    uint8_t *sf;             // rows_p * cols_p / 32 E8M0 bytes
    float qmax;              // 6 or 4
    int sf_layout;
    int tiles_x;
    int vector_loads;        // x 16-byte aligned, ld % 8 == 0
    float *amax;             // written with 1: the format has no tensor scale
};

// One lane owns 8 consecutive elements (one 128-bit load), four neighbouring lanes own a
// 1x32 block: every load instruction of a wavefront covers 1 KiB of one row (whole cache
// lines), the block maximum is two quad permutes, and the codes leave as one 32-bit word
// per lane (256 contiguous bytes per wavefront and row).
FOS_DEVICE uint32_t quad_max_u32(uint32_t v) {
    const uint32_t a = (uint32_t)__builtin_amdgcn_mov_dpp((int)v, 0xB1, 0xf, 0xf, true);  // quad_perm [1,0,3,2]
    v = v > a ? v : a;
    const uint32_t b = (uint32_t)__builtin_amdgcn_mov_dpp((int)v, 0x4E, 0xf, 0xf, true);  // quad_perm [2,3,0,1]
    return v > b ? v : b;
}

// 8 elements (4 words of 2 bf16) of a block -> their code word and the block's scale byte.
FOS_DEVICE void quantize_octet_mxfp4(const uint4 &x, float qmax, uint32_t &codes, uint32_t &e) {
    const uint32_t w[4] = {x.x, x.y, x.z, x.w};
    uint32_t m = 0;
#pragma unroll
    for (int i = 0; i < 4; ++i) m = pk_max_u16(m, w[i] & 0x7fff7fffu);
    uint32_t mm = (m & 0xffffu) > (m >> 16) ? (m & 0xffffu) : (m >> 16);
    mm = quad_max_u32(mm);
    const float s_hp = u2f(mm << 16) / qmax;
    const uint32_t u = f2u(s_hp);
    e = (u >> 23) & 0xffu;
    if (u & 0x7fffffu) e = (e + 1u) & 0xffu;  // round up to the next power of two
    // 1 / 2^(e - 127); e == 0 marks an all-zero block (values become 0), 255 is inf / NaN
    const float inv = e == 0u || e == 255u ? 0.0f : (e == 254u ? u2f(0x00400000u) : u2f((254u - e) << 23));
    uint32_t c = 0;
    static_for<0, 4>([&](auto jc) {
        constexpr int j = decltype(jc)::value;
        // + 0: the reference multiplies by sign(x) with sign(-0.0) = 0, so a negative zero
        // (also one produced by underflow) must not keep its sign; a negative value that
        // rounds to zero does
        const float lo = __builtin_fmaf(u2f(w[j] << 16), inv, 0.0f);
        const float hi = __builtin_fmaf(u2f(w[j] & 0xffff0000u), inv, 0.0f);
        c = pack_fp4<j>(c, lo, hi);
    });
    codes = c;
}

// Workgroup tile 128 rows x 512 columns (16 blocks per row): a wavefront covers one row of
// the tile per load instruction (512 elements = 1 KiB), four rows per step; 8 wavefronts,
// four steps of 32 rows; the four complete 128x4 scale tiles are staged in LDS and leave as
// one contiguous 2 KiB run.
// FULL: the tensor is whole tiles and 16-byte aligned, so every load is an unconditional
// 128-bit load (loads under a branch make the compiler wait for all of them at once).
constexpr int kMxQuantThreads = 512;
template <bool FULL>
__global__ __launch_bounds__(kMxQuantThreads) void quantize_mxfp4_kernel(const MxQuantParams p) {
    __shared__ uint32_t sf_stage[4 * 128];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int lb = lane >> 2;  // block column inside the tile
    const int64_t sf_cols = p.cols_p >> 5;
    const int64_t tile_y = blockIdx.x / p.tiles_x, tile_x = blockIdx.x - tile_y * p.tiles_x;
    const int64_t cb = tile_x * 16 + lb;
    const int64_t c0 = tile_x * 512 + lane * 8;  // first column of this lane's 8 elements
    const bool col_ok = FULL || cb < sf_cols;
    const bool tiled = p.sf_layout == FOS_SF_TILED_128X4;
    if (blockIdx.x == 0 && threadIdx.x == 0) *p.amax = 1.0f;  // the reference reports amax = 1 (reference.py:573-578)

    auto load = [&](int64_t r, uint4 &v) {
        if (FULL || (r < p.rows && c0 + 8 <= p.cols && p.vector_loads)) {
            v = *reinterpret_cast<const uint4 *>(p.x + r * p.ld + c0);
        } else {
            uint32_t w[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                uint32_t lo = 0, hi = 0;
                if (r < p.rows && c0 + 2 * i < p.cols) lo = p.x[r * p.ld + c0 + 2 * i];
                if (r < p.rows && c0 + 2 * i + 1 < p.cols) hi = p.x[r * p.ld + c0 + 2 * i + 1];
                w[i] = lo | (hi << 16);
            }
            v = make_uint4(w[0], w[1], w[2], w[3]);
        }
    };

    // rows of step g: tile_y * 128 + g * 32 + wave * 4 + j; three steps (12 loads) in flight
    constexpr int kSteps = 4;
    uint4 x[3][4];
    const int64_t row_w = tile_y * 128 + wave * 4;
#pragma unroll
    for (int j = 0; j < 4; ++j) load(row_w + j, x[0][j]);
#pragma unroll
    for (int j = 0; j < 4; ++j) load(row_w + 32 + j, x[1][j]);
#pragma unroll
    for (int g = 0; g < kSteps; ++g) {
        if (g + 2 < kSteps) {
#pragma unroll
            for (int j = 0; j < 4; ++j) load(row_w + (g + 2) * 32 + j, x[(g + 2) % 3][j]);
        }
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            uint32_t codes, e;
            quantize_octet_mxfp4(x[g % 3][j], p.qmax, codes, e);  // all lanes: the quad permutes need their neighbours
            if (!col_ok) continue;
            const int rr = g * 32 + wave * 4 + j;
            const int64_t r = tile_y * 128 + rr;
            stream_store(reinterpret_cast<uint32_t *>(p.codes + r * (p.cols_p >> 1) + (c0 >> 1)), codes);
            if ((lane & 3) == 0) {
                if (tiled) reinterpret_cast<uint8_t *>(sf_stage)[(lb >> 2) * 512 + (rr & 31) * 16 + (rr >> 5) * 4 + (lb & 3)] = (uint8_t)e;
                else p.sf[r * sf_cols + cb] = (uint8_t)e;
            }
        }
    }
    if (tiled) {
        __syncthreads();
        const int t = threadIdx.x >> 6;  // wavefronts 0-3: one scale tile each, 512 bytes, 8 per lane
        const int64_t group = tile_x * 4 + t;
        if (t < 4 && (FULL || group < (sf_cols >> 2))) {
            uint2 *out = reinterpret_cast<uint2 *>(p.sf + (tile_y * (sf_cols >> 2) + group) * 512);
            out[lane] = reinterpret_cast<const uint2 *>(sf_stage)[threadIdx.x];
        }
    }
}

// Streaming form for 16-byte aligned rows with cols % 16 == 0: the lane mapping and launch shape of the NVFP4
// 1x16 kernel (fos_quantize_fast.hip).  A lane owns 16 consecutive elements (two 128-bit buffer loads, one
// 64-bit non-temporal store of codes), two neighbouring lanes own a 1x32 block (its maximum is one quad
// permute).  A wavefront covers 4 rows x 512 contiguous bytes per step; a 256-thread workgroup walks a
// 128 x 256 tile in eight steps with the loads three steps ahead, across tile boundaries; 768 workgroups stride
// over the tiles, die b % 8 taking the 512-byte windows b % 8, b % 8 + 8, ... of every row.  Wavefront w owns
// rows 32 q + 8 w + 4 h + i (step 2 q + h, i = lane >> 4): in the 128x4 scale layout the scales of rows r,
// r + 32, r + 64, r + 96 share a 16-byte unit, so its 32 rows' scales are 128 contiguous bytes of each of the
// tile's two scale tiles, assembled in 256 bytes of LDS and written by the wavefront itself (no workgroup
// barrier).  A ragged tile's descriptor ends with the tensor's last row and lanes past the last column get an
// offset beyond it: both read zeros, which is the padding the reference adds.
struct MxRowsTile {
    uint64_t x_base, codes_base;
    uint32_t x_bytes, x_off;
    int64_t row_base, cb;  // first row of the tile; this lane's 16-element column group in the tensor
    uint32_t tile_y, tile_x;
};

// F16: fp16 elements instead of bf16 (magnitudes of either type order like their bit patterns; both convert
// to f32 exactly).
template <bool FULL, bool F16 = false>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(4))) void quantize_mxfp4_rows_kernel(const MxQuantParams p) {
    __shared__ __attribute__((aligned(16))) uint32_t sf_stage[4][64];  // per wavefront: 2 scale tiles x 128 bytes
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int64_t sf_cols = p.cols_p >> 5;
    const int lb = lane & 15;               // 16-element column group inside the tile
    const int rl = wave * 8 + (lane >> 4);  // this lane's row in step 0
    const bool tiled = p.sf_layout == FOS_SF_TILED_128X4;
    const int64_t code_pitch = p.cols_p >> 1;
    const uint32_t n_tiles = (uint32_t)(p.rows_p >> 7) * (uint32_t)p.tiles_x;
    const uint32_t x_lane = (uint32_t)(rl * p.ld + lb * 16) * 2u, x_row = (uint32_t)p.ld * 2u;
    const uint32_t c_lane = (uint32_t)(rl * code_pitch + lb * 8), c_row = (uint32_t)code_pitch;
    auto step_row = [](int g) { return 32 * (g >> 1) + 4 * (g & 1); };
    // scale byte of (q, h, i; block column b = lb >> 1) in the wavefront's staging area: 128 bytes per scale
    // tile b >> 2, unit 4 h + i, byte 4 q + (b & 3)
    uint8_t *stage = reinterpret_cast<uint8_t *>(sf_stage[wave]) + (lb >> 3) * 128 + (lane >> 4) * 16 + ((lb >> 1) & 3);
    if (blockIdx.x == 0 && threadIdx.x == 0) *p.amax = 1.0f;  // the reference reports amax = 1 (reference.py:573-578)

    auto open_tile = [&](uint32_t tile, bool valid) {
        MxRowsTile t;
        t.tile_y = tile / (uint32_t)p.tiles_x;
        t.tile_x = tile - t.tile_y * (uint32_t)p.tiles_x;
        t.row_base = (int64_t)t.tile_y * 128;
        const int64_t col_base = (int64_t)t.tile_x * 256;
        t.cb = (int64_t)t.tile_x * 16 + lb;
        uint32_t x_bytes = valid ? 0xffffffffu : 0u;
        if (!FULL && valid) {
            const int64_t left = ((p.rows - t.row_base) * p.ld - col_base) * 2;
            x_bytes = left <= 0 ? 0u : (left > 0x7fffffffLL ? 0x7fffffffu : (uint32_t)left);
        }
        t.x_bytes = __builtin_amdgcn_readfirstlane(x_bytes);
        t.x_base = uniform64((uint64_t)(p.x + t.row_base * p.ld + col_base));
        t.codes_base = uniform64((uint64_t)(p.codes + t.row_base * code_pitch + col_base / 2));
        t.x_off = (FULL || t.cb * 16 < p.cols) ? x_lane : 0x80000000u;
        return t;
    };
    auto load = [&](const MxRowsTile &t, int g, uint32_t (&w)[8]) {
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
        w[0] = lo.x; w[1] = lo.y; w[2] = lo.z; w[3] = lo.w;
        w[4] = hi.x; w[5] = hi.y; w[6] = hi.z; w[7] = hi.w;
    };
    auto process = [&](const MxRowsTile &t, int g, const uint32_t (&w)[8]) {
        // block maximum: 16 elements of this lane, then the neighbour's (all lanes: the permute needs both)
        uint32_t m = 0;
#pragma unroll
        for (int i = 0; i < 8; ++i) m = pk_max_u16(m, w[i] & 0x7fff7fffu);
        uint32_t mm = (m & 0xffffu) > (m >> 16) ? (m & 0xffffu) : (m >> 16);
        const uint32_t other = (uint32_t)__builtin_amdgcn_mov_dpp((int)mm, 0xB1, 0xf, 0xf, true);  // quad_perm [1,0,3,2]
        mm = mm > other ? mm : other;
        if (!FULL && t.cb >= (p.cols_p >> 4)) return;  // past the padded width
        const float bmax = F16 ? (float)__builtin_bit_cast(_Float16, (uint16_t)mm) : u2f(mm << 16);
        const float s_hp = bmax / p.qmax;
        const uint32_t u = f2u(s_hp);
        uint32_t e = (u >> 23) & 0xffu;
        if (u & 0x7fffffu) e = (e + 1u) & 0xffu;  // round up to the next power of two
        // 1 / 2^(e - 127); e == 0 marks an all-zero block (values become 0), 255 is inf / NaN
        const float inv = e == 0u || e == 255u ? 0.0f : (e == 254u ? u2f(0x00400000u) : u2f((254u - e) << 23));
        auto lo_of = [](uint32_t word) { return F16 ? (float)__builtin_bit_cast(_Float16, (uint16_t)word) : u2f(word << 16); };
        auto hi_of = [](uint32_t word) { return F16 ? (float)__builtin_bit_cast(_Float16, (uint16_t)(word >> 16)) : u2f(word & 0xffff0000u); };
        uint32_t c0 = 0, c1 = 0;
        static_for<0, 4>([&](auto jc) {
            constexpr int j = decltype(jc)::value;
            // + 0: a negative zero (also one produced by underflow) must not keep its sign; a negative value
            // that rounds to zero does (the reference multiplies by sign(x), and sign(-0.0) = 0)
            c0 = pack_fp4<j>(c0, __builtin_fmaf(lo_of(w[j]), inv, 0.0f), __builtin_fmaf(hi_of(w[j]), inv, 0.0f));
            c1 = pack_fp4<j>(c1, __builtin_fmaf(lo_of(w[4 + j]), inv, 0.0f), __builtin_fmaf(hi_of(w[4 + j]), inv, 0.0f));
        });
        const u32x2 c01 = {c0, c1};
        const BufferRsrc rcodes = make_rsrc(reinterpret_cast<const void *>(uniform64(t.codes_base)), 0xffffffffu);
        __builtin_amdgcn_raw_buffer_store_b64(c01, rcodes, c_lane, step_row(g) * c_row, kStreamStore);
        if ((lane & 1) == 0) {
            if (tiled) stage[(g & 1) * 64 + (g >> 1) * 4] = (uint8_t)e;
            else p.sf[(t.row_base + step_row(g) + rl) * sf_cols + (t.cb >> 1)] = (uint8_t)e;
        }
    };

    uint32_t tile = blockIdx.x;
    MxRowsTile cur = open_tile(tile, tile < n_tiles);
    uint32_t ring[4][8];
    load(cur, 0, ring[0]);
    load(cur, 1, ring[1]);
    load(cur, 2, ring[2]);
    while (tile < n_tiles) {
        const uint32_t next = tile + gridDim.x;
        const bool has_next = next < n_tiles;
        const MxRowsTile nxt = open_tile(has_next ? next : tile, has_next);  // without a next tile: loads of nothing
#pragma unroll
        for (int g = 0; g < 8; ++g) {
            if (g + 3 < 8) load(cur, g + 3, ring[(g + 3) & 3]);
            else load(nxt, g + 3 - 8, ring[(g + 3) & 3]);
            process(cur, g, ring[g & 3]);
        }
        if (tiled) {
            // the wavefront's own 2 x 128 bytes: written above by its lanes, read back here in output order
            // (LDS operations of one wavefront complete in order)
            __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
            __builtin_amdgcn_wave_barrier();
            __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
            const int64_t group = (int64_t)cur.tile_x * 2 + (lane >> 4);
            if (lane < 32 && (FULL || group < (sf_cols >> 2))) {
                const uint2 v = reinterpret_cast<const uint2 *>(sf_stage[wave])[lane];
                *reinterpret_cast<uint2 *>(p.sf + ((int64_t)cur.tile_y * (sf_cols >> 2) + group) * 512 + wave * 128 + (lane & 15) * 8) = v;
            }
            __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
            __builtin_amdgcn_wave_barrier();
        }
        cur = nxt;
        tile = next;
    }
}

// fp32 inputs, and fp16 ones that the streaming kernel does not take: the tile shape and scale staging of
// quantize_mxfp4_kernel with elements read one by one and converted to f32 (exact for both types), which is
// where the reference's arithmetic starts (`.float()`, reference.py:149-181).
template <bool F32>
__global__ __launch_bounds__(kMxQuantThreads) void quantize_mxfp4_typed_kernel(const MxQuantParams p) {
    __shared__ uint32_t sf_stage[4 * 128];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int lb = lane >> 2;  // block column inside the tile
    const int64_t sf_cols = p.cols_p >> 5;
    const int64_t tile_y = blockIdx.x / p.tiles_x, tile_x = blockIdx.x - tile_y * p.tiles_x;
    const int64_t cb = tile_x * 16 + lb;
    const int64_t c0 = tile_x * 512 + lane * 8;  // first column of this lane's 8 elements
    const bool col_ok = cb < sf_cols;
    const bool tiled = p.sf_layout == FOS_SF_TILED_128X4;
    if (blockIdx.x == 0 && threadIdx.x == 0) *p.amax = 1.0f;
    for (int g = 0; g < 4; ++g) {
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int rr = g * 32 + wave * 4 + j;
            const int64_t r = tile_y * 128 + rr;
            float v[8];
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                v[i] = 0.0f;
                if (r < p.rows && c0 + i < p.cols) {
                    if (F32) v[i] = reinterpret_cast<const float *>(p.x)[r * p.ld + c0 + i];
                    else v[i] = (float)__builtin_bit_cast(_Float16, p.x[r * p.ld + c0 + i]);
                }
            }
            // block maximum over the four lanes of the block (all lanes: the permutes need their neighbours)
            float bmax = 0.0f;
#pragma unroll
            for (int i = 0; i < 8; ++i) bmax = fmaxf(bmax, fabsf(v[i]));
            bmax = u2f(quad_max_u32(f2u(bmax)));  // non-negative floats order like their bit patterns
            const float s_hp = bmax / p.qmax;
            const uint32_t u = f2u(s_hp);
            uint32_t e = (u >> 23) & 0xffu;
            if (u & 0x7fffffu) e = (e + 1u) & 0xffu;
            const float inv = e == 0u || e == 255u ? 0.0f : (e == 254u ? u2f(0x00400000u) : u2f((254u - e) << 23));
            uint32_t codes = 0;
            static_for<0, 4>([&](auto jc) {
                constexpr int q = decltype(jc)::value;
                codes = pack_fp4<q>(codes, __builtin_fmaf(v[2 * q], inv, 0.0f), __builtin_fmaf(v[2 * q + 1], inv, 0.0f));
            });
            if (!col_ok) continue;
            *reinterpret_cast<uint32_t *>(p.codes + r * (p.cols_p >> 1) + (c0 >> 1)) = codes;
            if ((lane & 3) == 0) {
                if (tiled) reinterpret_cast<uint8_t *>(sf_stage)[(lb >> 2) * 512 + (rr & 31) * 16 + (rr >> 5) * 4 + (lb & 3)] = (uint8_t)e;
                else p.sf[r * sf_cols + cb] = (uint8_t)e;
            }
        }
    }
    if (tiled) {
        __syncthreads();
        const int t = threadIdx.x >> 6;  // wavefronts 0-3: one scale tile each, 512 bytes, 8 per lane
        const int64_t group = tile_x * 4 + t;
        if (t < 4 && group < (sf_cols >> 2)) {
            uint2 *out = reinterpret_cast<uint2 *>(p.sf + (tile_y * (sf_cols >> 2) + group) * 512);
            out[lane] = reinterpret_cast<const uint2 *>(sf_stage)[threadIdx.x];
        }
    }
}

int launch_quantize_mxfp4(const void *x, int x_type, int64_t rows, int64_t cols, int64_t ld, int rule, int sf_layout, uint8_t *codes,
                          uint8_t *sf, float *amax, hipStream_t s) {
    MxQuantParams p;
    p.x = static_cast<const uint16_t *>(x);
    p.rows = rows; p.cols = cols; p.ld = ld;
    p.rows_p = (rows + 127) / 128 * 128;
    p.cols_p = (cols + 127) / 128 * 128;
    p.codes = codes; p.sf = sf;
    p.qmax = rule == FOS_RULE_STATIC_4 ? 4.0f : 6.0f;
    p.sf_layout = sf_layout;
    p.tiles_x = (int)((p.cols_p + 511) / 512);
    p.vector_loads = (((uintptr_t)x & 15) == 0) && (ld % 8 == 0);
    const int64_t grid = (p.rows_p / 128) * p.tiles_x;
    if (grid > 0x7fffffffLL) return FOS_E_BAD_SHAPE;
    p.amax = amax;
    const bool streams = x_type != FOS_T_F32 && p.vector_loads && cols % 16 == 0 && ld < (int64_t{1} << 23) &&
                         (tuning().mx_quant != 1 || x_type == FOS_T_F16);
    if (!streams && x_type != FOS_T_BF16) {
        if (x_type == FOS_T_F32) hipLaunchKernelGGL(quantize_mxfp4_typed_kernel<true>, dim3((unsigned)grid), dim3(kMxQuantThreads), 0, s, p);
        else hipLaunchKernelGGL(quantize_mxfp4_typed_kernel<false>, dim3((unsigned)grid), dim3(kMxQuantThreads), 0, s, p);
        return hipGetLastError() == hipSuccess ? FOS_OK : FOS_E_LAUNCH;
    }
    if (streams) {
        // the streaming form (32-bit byte offsets inside a 128-row tile: rows of less than 16 MiB)
        p.tiles_x = (int)((p.cols_p + 255) / 256);
        const int64_t n = (p.rows_p / 128) * p.tiles_x;
        int64_t launch = 768;
        if (const int forced = tuning().quant_grid) launch = forced > 0 ? forced : launch;
        if (launch > n) launch = n;
        const bool full = rows % 128 == 0 && cols % 256 == 0;
        if (x_type == FOS_T_F16) {
            if (full) hipLaunchKernelGGL((quantize_mxfp4_rows_kernel<true, true>), dim3((unsigned)launch), dim3(256), 0, s, p);
            else hipLaunchKernelGGL((quantize_mxfp4_rows_kernel<false, true>), dim3((unsigned)launch), dim3(256), 0, s, p);
        } else {
            if (full) hipLaunchKernelGGL((quantize_mxfp4_rows_kernel<true, false>), dim3((unsigned)launch), dim3(256), 0, s, p);
            else hipLaunchKernelGGL((quantize_mxfp4_rows_kernel<false, false>), dim3((unsigned)launch), dim3(256), 0, s, p);
        }
        return hipGetLastError() == hipSuccess ? FOS_OK : FOS_E_LAUNCH;
    }
    if (p.vector_loads && rows % 128 == 0 && cols % 512 == 0)
        hipLaunchKernelGGL(quantize_mxfp4_kernel<true>, dim3((unsigned)grid), dim3(kMxQuantThreads), 0, s, p);
    else
        hipLaunchKernelGGL(quantize_mxfp4_kernel<false>, dim3((unsigned)grid), dim3(kMxQuantThreads), 0, s, p);
    return hipGetLastError() == hipSuccess ? FOS_OK : FOS_E_LAUNCH;
}

// ---------------------------------------------------------------------------------------
// dequantize
// ---------------------------------------------------------------------------------------

struct MxDequantParams {
    const uint8_t *codes, *sf;
    void *out;
    int64_t rows, cols, rows_p, cols_p, ldo;
    int sf_layout;
    int vector_stores;
    int f32_product;  // value * scale in fp32 (exact) instead of fp16
};

typedef _Float16 mx_half2_t __attribute__((ext_vector_type(2)));

// One thread per 8 consecutive elements (a quarter of a 1x32 block; a wavefront reads 256
// contiguous bytes of codes and writes 1 KiB per store instruction).  value (fp16) *
// fp16(2^(e - 127)), product in fp16: scales outside fp16's range turn into 0 / inf there,
// as in the reference.
template <int OUT>
__global__ __launch_bounds__(256) void dequantize_mxfp4_kernel(const MxDequantParams p) {
    const int64_t sf_cols = p.cols_p >> 5;
    const int64_t opr = (p.cols + 7) >> 3;  // octets per row
    const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (idx >= p.rows * opr) return;
    const int64_t r = idx / opr, oc = idx - r * opr, cb = oc >> 2;
    const uint32_t q = *reinterpret_cast<const uint32_t *>(p.codes + r * (p.cols_p >> 1) + oc * 4);
    const int64_t sofs = p.sf_layout == FOS_SF_TILED_128X4
                             ? ((r >> 7) * (sf_cols >> 2) + (cb >> 2)) * 512 + (r & 31) * 16 + ((r & 127) >> 5) * 4 + (cb & 3)
                             : r * sf_cols + cb;
    const uint32_t e = p.sf[sofs];
    const float s32 = e == 0u ? u2f(0x00400000u) : u2f(e << 23);  // 2^(e - 127); e = 255 is a NaN, as in E8M0
    const _Float16 s16 = (_Float16)s32;
    const mx_half2_t s2 = {s16, s16};
    float f[8];
    static_for<0, 4>([&](auto jc) {
        constexpr int j = decltype(jc)::value;
        if (p.f32_product) {
            const float2_t v = unpack_fp4<j>(q);
            f[2 * j] = v.x * s32;
            f[2 * j + 1] = v.y * s32;
        } else {
            const mx_half2_t v = __builtin_amdgcn_cvt_scalef32_pk_f16_fp4(q, 1.0f, j) * s2;
            f[2 * j] = (float)v.x;
            f[2 * j + 1] = (float)v.y;
        }
    });
    const int64_t c0 = oc * 8;
    const bool whole = p.vector_stores && c0 + 8 <= p.cols;
    if (OUT == FOS_T_F32) {
        float *o = reinterpret_cast<float *>(p.out) + r * p.ldo + c0;
        if (whole) {
            reinterpret_cast<float4 *>(o)[0] = make_float4(f[0], f[1], f[2], f[3]);
            reinterpret_cast<float4 *>(o)[1] = make_float4(f[4], f[5], f[6], f[7]);
        } else {
#pragma unroll
            for (int i = 0; i < 8; ++i)
                if (c0 + i < p.cols) o[i] = f[i];
        }
        return;
    }
    uint32_t w[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const float2_t v = {f[2 * j], f[2 * j + 1]};
        if (OUT == FOS_T_F16) {
            w[j] = __builtin_bit_cast(uint32_t, __builtin_convertvector(v, mx_half2_t));
        } else {
            typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
            w[j] = __builtin_bit_cast(uint32_t, __builtin_convertvector(v, bf16x2_t));
        }
    }
    uint16_t *o = reinterpret_cast<uint16_t *>(p.out) + r * p.ldo + c0;
    if (whole) {
        stream_store(reinterpret_cast<uint4 *>(o), make_uint4(w[0], w[1], w[2], w[3]));
    } else {
#pragma unroll
        for (int i = 0; i < 8; ++i)
            if (c0 + i < p.cols) o[i] = (uint16_t)(w[i >> 1] >> (16 * (i & 1)));
    }
}

int launch_dequantize_mxfp4(const uint8_t *codes, const uint8_t *sf, int sf_layout, int64_t rows, int64_t cols,
                            int64_t rows_p, int64_t cols_p, void *out, int out_type, int64_t ldo, int f32_product,
                            hipStream_t s) {
    if (cols_p % 32 != 0 || (sf_layout == FOS_SF_TILED_128X4 && cols_p % 128 != 0)) return FOS_E_BAD_SHAPE;
    if ((uintptr_t)codes & 3) return FOS_E_BAD_ALIGNMENT;
    MxDequantParams p;
    p.codes = codes; p.sf = sf; p.out = out;
    p.rows = rows; p.cols = cols; p.rows_p = rows_p; p.cols_p = cols_p; p.ldo = ldo;
    p.sf_layout = sf_layout;
    p.f32_product = f32_product;
    const int64_t esize = out_type == FOS_T_F32 ? 4 : 2;
    p.vector_stores = ((uintptr_t)out & 15) == 0 && (ldo * esize) % 16 == 0;
    const int64_t n_octets = rows * ((cols + 7) / 8);
    if ((n_octets + 255) / 256 > 0x7fffffffLL) return FOS_E_BAD_SHAPE;
    dim3 grid((unsigned)((n_octets + 255) / 256));
    if (out_type == FOS_T_F32) hipLaunchKernelGGL(dequantize_mxfp4_kernel<FOS_T_F32>, grid, dim3(256), 0, s, p);
    else if (out_type == FOS_T_F16) hipLaunchKernelGGL(dequantize_mxfp4_kernel<FOS_T_F16>, grid, dim3(256), 0, s, p);
    else hipLaunchKernelGGL(dequantize_mxfp4_kernel<FOS_T_BF16>, grid, dim3(256), 0, s, p);
    return hipGetLastError() == hipSuccess ? FOS_OK : FOS_E_LAUNCH;
}

// ---------------------------------------------------------------------------------------
// GEMM on the scaled FP4 matrix instruction
// ---------------------------------------------------------------------------------------
//
// D[M, N] = alpha * sum_k (A[m,k] 2^(sfA[m,k/32]-127)) (B[n,k] 2^(sfB[n,k/32]-127)).
// Operand layout of v_mfma_scale_f32_32x32x64_f8f6f4 with FP4 inputs (probed on the
// device): lane (r = lane & 31, h = lane >> 5) supplies the 32 codes k = 32 h .. 32 h + 31 of
// row r (16 bytes, low nibble = even k) and, in one byte of a scale register, that row's
// E8M0 scale for its K block; accumulator register 4 g + e of lane l is
// C[8 g + 4 (l >> 5) + e][l & 31] with rows taken from the first operand.  B (rows n) is
// fed as the first operand so that a lane's consecutive registers are consecutive n.
//
// Tile 256 x 256 x 128 (BK = 128 codes = 64 bytes per row = one scale chunk), 8 wavefronts
// of 128 x 64, LDS pitch 80 bytes (conflict-free 128-bit accesses), two stages; the
// pipeline is the one of the NVFP4 kernel minus the dequantisation: registers hold step
// k+2 in flight, step k+1 goes to LDS in halves while step k is multiplied.  Scales bypass
// LDS: the 128x4 tiled layout holds the four scale bytes of a 128-wide K chunk of rows r,
// r+32, r+64, r+96 next to each other, so a wavefront's lanes fetch one 32-bit word per
// row tile and chunk straight from global memory.

typedef int mx_v8i __attribute__((ext_vector_type(8)));
typedef float mx_v16f __attribute__((ext_vector_type(16)));
typedef __amdgpu_buffer_rsrc_t MxRsrc;

struct MxGemmParams {
    const uint8_t *A, *B, *sfA, *sfB;
    const float *alpha;
    void *D;
    int64_t M, N, K, ldd;
    int tiles_m, tiles_n;
};

constexpr int kMxBK = 128;    // codes per K step
constexpr int kMxPitch = 80;  // LDS bytes per row (64 + 16)

FOS_DEVICE MxRsrc mx_rsrc(const void *base, uint32_t bytes) {
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<void *>(base), 0, (int)bytes, 0x00020000);
}

// N consecutive 32-bit words (N = 1, 2, 4) with one buffer load.
template <int N>
FOS_DEVICE void mx_load_words(uint32_t (&dst)[N], MxRsrc r, int voffset, int soffset) {
    static_assert(N == 1 || N == 2 || N == 4, "one load instruction");
    if constexpr (N == 1) {
        dst[0] = __builtin_amdgcn_raw_buffer_load_b32(r, voffset, soffset, 0);
    } else if constexpr (N == 2) {
        const auto v = __builtin_bit_cast(uint2, __builtin_amdgcn_raw_buffer_load_b64(r, voffset, soffset, 0));
        dst[0] = v.x, dst[1] = v.y;
    } else {
        const auto v = __builtin_bit_cast(uint4, __builtin_amdgcn_raw_buffer_load_b128(r, voffset, soffset, 0));
        dst[0] = v.x, dst[1] = v.y, dst[2] = v.z, dst[3] = v.w;
    }
}

FOS_DEVICE mx_v8i frag_of(const uint4 &q) {
    mx_v8i v = {(int)q.x, (int)q.y, (int)q.z, (int)q.w, 0, 0, 0, 0};  // FP4 operands use the first four registers
    return v;
}

FOS_DEVICE void mx_tile_of(int bid, int tiles_m, int tiles_n, int &tm, int &tn) {
    // workgroups with equal bid % 8 share an XCD: give each XCD a compact run of tiles,
    // ordered in column bands of 8 tile rows
    const int total = tiles_m * tiles_n;
    const int per_xcd = (total + 7) / 8;
    int t = (bid & 7) * per_xcd + (bid >> 3);
    if (t >= total || (total & 7) != 0) t = bid;
    constexpr int kBand = 8;
    const int band = t / (kBand * tiles_n), in_band = t - band * kBand * tiles_n;
    const int rows = (tiles_m - band * kBand) < kBand ? (tiles_m - band * kBand) : kBand;
    tm = band * kBand + in_band % rows;
    tn = in_band / rows;
}

// Epilogue of the tile kernels.  acc[i][j][4 g + e] is D[m][n] with m = 32 i + r and
// n = 32 j + 8 g + 4 h + e (r = lane & 31, h = lane >> 5) of the wavefront's block: stored from
// the registers, an instruction would touch 32 rows with 16 bytes each (1.6 bytes written to
// memory per byte of output).  Each wavefront turns a 32-row tile round in its own piece of
// the operand staging, which is idle by now (the caller has waited for every wavefront), and
// stores whole rows of its block, 16 bytes per lane.
template <int WM, int WN, bool OUT_BF16>
FOS_DEVICE void mx_store_rows(const mx_v16f (&acc)[WM][WN], uint8_t *lds, int wave, int lane, float alpha, uint16_t *D,
                              int64_t ldd, int64_t m_base, int64_t n_base) {
    constexpr int kRowBytes = WN * 64, kEpiPitch = kRowBytes + 16;
    constexpr int kLanesPerRow = kRowBytes / 16, kRowsPerPass = 64 / kLanesPerRow;
    const int r = lane & 31, h = lane >> 5;
    uint8_t *epi = lds + wave * 32 * kEpiPitch;
#pragma unroll
    for (int i = 0; i < WM; ++i) {
#pragma unroll
        for (int j = 0; j < WN; ++j) {
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                uint32_t w[2];
#pragma unroll
                for (int e = 0; e < 2; ++e) {
                    const float2_t v = {alpha * acc[i][j][4 * g + 2 * e], alpha * acc[i][j][4 * g + 2 * e + 1]};
                    if (OUT_BF16) {
                        typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
                        w[e] = __builtin_bit_cast(uint32_t, __builtin_convertvector(v, bf16x2_t));
                    } else {
                        w[e] = __builtin_bit_cast(uint32_t, __builtin_convertvector(v, mx_half2_t));
                    }
                }
                *reinterpret_cast<uint2 *>(epi + r * kEpiPitch + (j * 32 + 8 * g + 4 * h) * 2) = make_uint2(w[0], w[1]);
            }
        }
        // (LDS operations of one wavefront complete in order: its own writes are visible to its reads)
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
#pragma unroll
        for (int t = 0; t < 32 / kRowsPerPass; ++t) {
            const int row = t * kRowsPerPass + lane / kLanesPerRow, c16 = lane % kLanesPerRow;
            const uint4 v = *reinterpret_cast<const uint4 *>(epi + row * kEpiPitch + c16 * 16);
            *reinterpret_cast<uint4 *>(D + (m_base + i * 32 + row) * ldd + n_base + c16 * 8) = v;
        }
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
    }
}

template <int WAVES_M, int WAVES_N, int WM, int WN, bool OUT_BF16>
__global__ __launch_bounds__(64 * WAVES_M *WAVES_N) void gemm_mxfp4_kernel(const MxGemmParams p) {
    constexpr int kThreadsG = 64 * WAVES_M * WAVES_N;
    constexpr int BM = WAVES_M * WM * 32, BN = WAVES_N * WN * 32;
    constexpr int kRowsPerPass = kThreadsG / 4;  // 4 lanes cover the 64 bytes of a row
    constexpr int PA = BM / kRowsPerPass, PB = BN / kRowsPerPass;
    static_assert(PA % 2 == 0 && PB % 2 == 0 && WM * 32 <= 128 && WN * 32 <= 128, "tile shape: staged in two halves");
    extern __shared__ __attribute__((aligned(16))) uint8_t mx_lds[];
    uint8_t *lds_a[2] = {mx_lds, mx_lds + (BM + BN) * kMxPitch};
    uint8_t *lds_b[2] = {mx_lds + BM * kMxPitch, mx_lds + (BM + BN) * kMxPitch + BM * kMxPitch};

    const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int r = lane & 31, h = lane >> 5;
    int tile_m, tile_n;
    mx_tile_of(blockIdx.x, p.tiles_m, p.tiles_n, tile_m, tile_n);
    const int64_t m0 = (int64_t)tile_m * BM, n0 = (int64_t)tile_n * BN;
    const int64_t kbytes = p.K >> 1;
    const int64_t ksteps = p.K / kMxBK;  // = 128-wide K chunks = scale groups per band

    const MxRsrc ra = mx_rsrc(p.A + m0 * kbytes, (uint32_t)(BM * kbytes));
    const MxRsrc rb = mx_rsrc(p.B + n0 * kbytes, (uint32_t)(BN * kbytes));
    const int ld_row = tid >> 2, ld_col = (tid & 3) * 16;
    const uint32_t q_off = (uint32_t)(ld_row * kbytes + ld_col);
    const uint32_t lds_off = (uint32_t)(ld_row * kMxPitch + ld_col);

    // scales of this wavefront's rows, straight from global memory
    const int wm = wave / WAVES_N, wn = wave % WAVES_N;
    const int64_t a_row0 = m0 + wm * WM * 32, b_row0 = n0 + wn * WN * 32;
    const MxRsrc rsa = mx_rsrc(p.sfA + (a_row0 >> 7) * ksteps * 512, (uint32_t)(ksteps * 512));
    const MxRsrc rsb = mx_rsrc(p.sfB + (b_row0 >> 7) * ksteps * 512, (uint32_t)(ksteps * 512));
    const uint32_t sa_off = (uint32_t)(r * 16 + ((a_row0 & 127) >> 5) * 4);
    const uint32_t sb_off = (uint32_t)(r * 16 + ((b_row0 & 127) >> 5) * 4);

    struct Staged {
        uint4 a[PA], b[PB];
    };
    struct Scales {
        uint32_t a[WM], b[WN];  // scale bytes of the step's four K blocks, per row tile
    };
    auto fetch = [&](int64_t ks, Staged &s) {
        // per-pass and per-step displacements ride in the scalar offset: one address register
        const int kq = (int)(ks * (kMxBK / 2));
#pragma unroll
        for (int i = 0; i < PA; ++i)
            s.a[i] = __builtin_bit_cast(uint4, __builtin_amdgcn_raw_buffer_load_b128(ra, (int)q_off, kq + (int)(i * kRowsPerPass * kbytes), 0));
#pragma unroll
        for (int i = 0; i < PB; ++i)
            s.b[i] = __builtin_bit_cast(uint4, __builtin_amdgcn_raw_buffer_load_b128(rb, (int)q_off, kq + (int)(i * kRowsPerPass * kbytes), 0));
    };
    // raw scale words of step ks (bytes = the four K blocks of the chunk)
    // (the words of a wavefront's row tiles are adjacent in the 16-byte unit of row r: one
    // load per operand instead of one per row tile)
    auto fetch_scales = [&](int64_t ks, Scales &s) {
        const int ksf = (int)(ks * 512);
        mx_load_words<WM>(s.a, rsa, (int)sa_off, ksf);
        mx_load_words<WN>(s.b, rsb, (int)sb_off, ksf);
    };
    // half q of the staged registers -> LDS stage `buf`
    auto stage_part = [&](const Staged &s, int buf, int q) {
#pragma unroll
        for (int i = q * (PA / 2); i < (q + 1) * (PA / 2); ++i)
            *reinterpret_cast<uint4 *>(lds_a[buf] + lds_off + i * kRowsPerPass * kMxPitch) = s.a[i];
#pragma unroll
        for (int i = q * (PB / 2); i < (q + 1) * (PB / 2); ++i)
            *reinterpret_cast<uint4 *>(lds_b[buf] + lds_off + i * kRowsPerPass * kMxPitch) = s.b[i];
    };

    mx_v16f acc[WM][WN];
#pragma unroll
    for (int i = 0; i < WM; ++i)
#pragma unroll
        for (int j = 0; j < WN; ++j)
#pragma unroll
            for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.0f;

    auto read_frags = [&](int buf, int kk, uint4 *fa, uint4 *fb) {
        const int kofs = kk * 32 + h * 16;
#pragma unroll
        for (int i = 0; i < WM; ++i) fa[i] = *reinterpret_cast<const uint4 *>(lds_a[buf] + (wm * WM * 32 + i * 32 + r) * kMxPitch + kofs);
#pragma unroll
        for (int j = 0; j < WN; ++j) fb[j] = *reinterpret_cast<const uint4 *>(lds_b[buf] + (wn * WN * 32 + j * 32 + r) * kMxPitch + kofs);
    };

    Staged st[2];
    Scales sc[2];
    uint4 fa[2][WM], fb[2][WN];
    fetch(0, st[0]);
    fetch_scales(0, sc[0]);
    stage_part(st[0], 0, 0);
    stage_part(st[0], 0, 1);
    if (ksteps > 1) fetch(1, st[1]);
    __syncthreads();
    read_frags(0, 0, fa[0], fb[0]);

    // One K step: multiply out of stage `buf` (fragments of slice 0 are in registers) while
    // step ks+1 (`nxt`) goes to the other stage; the barrier sits between the last staging
    // write and the last slice's MFMAs, and the next step's first fragments are read right
    // after it.  Branch-free; the last step is its own instantiation.
    auto kstep = [&](auto have_next_c, int64_t ks, int buf, Staged &cur_regs, Staged &nxt, const Scales &s_cur, Scales &s_nxt) {
        constexpr bool have_next = decltype(have_next_c)::value;
        // lanes of the upper half use the next byte: after the shift, byte 0 / byte 2 of every
        // lane's register are the scales of the K blocks it feeds in slice 0 / slice 1.  Done
        // here, a step after the load was issued, so that nothing waits on a fresh load.
        Scales sh;
#pragma unroll
        for (int i = 0; i < WM; ++i) sh.a[i] = s_cur.a[i] >> (8 * h);
#pragma unroll
        for (int j = 0; j < WN; ++j) sh.b[j] = s_cur.b[j] >> (8 * h);
        if (have_next) {
            fetch_scales(ks + 1, s_nxt);
            fetch(ks + 2 < ksteps ? ks + 2 : ksteps - 1, cur_regs);
        }
#pragma unroll
        for (int kk = 0; kk < 2; ++kk) {
            if (kk == 0) read_frags(buf, 1, fa[1], fb[1]);
            if (have_next) {
                stage_part(nxt, buf ^ 1, kk);
                if (kk == 1) {
                    __syncthreads();
                    read_frags(buf ^ 1, 0, fa[0], fb[0]);
                    __builtin_amdgcn_sched_barrier(0);
                }
            }
#pragma unroll
            for (int i = 0; i < WM; ++i)
#pragma unroll
                for (int j = 0; j < WN; ++j) {
                    if (kk == 1)
                        acc[i][j] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(
                            frag_of(fb[1][j]), frag_of(fa[1][i]), acc[i][j], 4, 4, 2, (int)sh.b[j], 2, (int)sh.a[i]);
                    else
                        acc[i][j] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(
                            frag_of(fb[0][j]), frag_of(fa[0][i]), acc[i][j], 4, 4, 0, (int)sh.b[j], 0, (int)sh.a[i]);
                }
            __builtin_amdgcn_sched_barrier(0);
        }
    };

    using yes = std::integral_constant<bool, true>;
    using no = std::integral_constant<bool, false>;
    int64_t ks = 0;
    for (; ks + 2 < ksteps; ks += 2) {
        kstep(yes{}, ks, 0, st[0], st[1], sc[0], sc[1]);
        kstep(yes{}, ks + 1, 1, st[1], st[0], sc[1], sc[0]);
    }
    if (ks + 2 == ksteps) {
        kstep(yes{}, ks, 0, st[0], st[1], sc[0], sc[1]);
        kstep(no{}, ks + 1, 1, st[1], st[0], sc[1], sc[0]);
    } else {
        kstep(no{}, ks, 0, st[0], st[1], sc[0], sc[1]);
    }

    static_assert(2 * (BM + BN) * kMxPitch >= WAVES_M * WAVES_N * 32 * (WN * 64 + 16), "epilogue staging fits the operand buffers");
    __syncthreads();  // every wavefront is done reading the operand buffers
    mx_store_rows<WM, WN, OUT_BF16>(acc, mx_lds, wave, lane, *p.alpha, reinterpret_cast<uint16_t *>(p.D), p.ldd, a_row0, b_row0);
}

template <int WAVES_M, int WAVES_N, int WM, int WN>
static int launch_gemm_mxfp4(MxGemmParams &p, int out_type, hipStream_t s) {
    constexpr int BM = WAVES_M * WM * 32, BN = WAVES_N * WN * 32;
    constexpr size_t lds_bytes = 2 * (size_t)(BM + BN) * kMxPitch;
    p.tiles_m = (int)(p.M / BM);
    p.tiles_n = (int)(p.N / BN);
    auto kernel = out_type == FOS_T_BF16 ? gemm_mxfp4_kernel<WAVES_M, WAVES_N, WM, WN, true>
                                         : gemm_mxfp4_kernel<WAVES_M, WAVES_N, WM, WN, false>;
    if (lds_bytes > 64 * 1024 &&
        hipFuncSetAttribute((const void *)kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_bytes) != hipSuccess)
        return FOS_E_LAUNCH;
    hipLaunchKernelGGL(kernel, dim3((unsigned)(p.tiles_m * p.tiles_n)), dim3(64 * WAVES_M * WAVES_N), lds_bytes, s, p);
    return hipGetLastError() == hipSuccess ? FOS_OK : FOS_E_LAUNCH;
}

// ---------------------------------------------------------------------------------------
// The same 256 x 256 x 128 tile with the operands loaded from global memory straight into
// LDS (buffer_load ... lds: lane i of a wavefront fills the i-th 16-byte unit of a 1 KiB
// run), so no registers stage them and four LDS stages keep three K steps in flight -- the
// register-staged kernel above has one step of latency cover, and a step then lasts as long
// as a load takes whatever the matrix pipe could do.
//
// A stage holds 256 rows x 64 bytes of each operand without padding and the four 512-byte
// scale tiles of the step (fetched the same way, 4 bytes per lane); the 16-byte unit c of
// row rho sits at unit c ^ ((rho >> 2) & 3).  A 128-bit LDS read serves 16 lanes per cycle
// from 64 banks, i.e. the 16 rows a quarter-wave reads must differ in address bits 7:4:
// those are 4 (rho & 3) + (c ^ ((rho >> 2) & 3)), all 16 values.  (With (rho >> 1) & 3, which
// serves 8 lanes from 32 banks, the counters showed every fragment read taking twice as
// long.)  The load of lane i therefore fetches unit (i & 3) ^ ((i >> 4) & 3) of row i >> 2 of
// its 16-row run.
constexpr int kDmaStages = 4;
constexpr int kDmaOperandBytes = 256 * 64;
constexpr int kDmaStageBytes = 2 * kDmaOperandBytes + 2048;  // + the step's scales: A tiles 0, 1, B tiles 0, 1
typedef __attribute__((address_space(3))) void *MxLdsPtr;
typedef int mx_v4i __attribute__((ext_vector_type(4)));

// Buffer descriptor as four plain words (for inline assembly): base, stride 0, size in
// bytes, raw 32-bit offsets with range checking -- the words mx_rsrc() makes.
FOS_DEVICE mx_v4i mx_raw_rsrc(const void *base, uint32_t bytes) {
    const uint64_t a = (uint64_t)(uintptr_t)base;
    mx_v4i v = {(int)(uint32_t)a, (int)(uint32_t)((a >> 32) & 0xffffu), (int)bytes, 0x00020000};
    return v;
}

// s_waitcnt vmcnt(n) alone (gfx9 encoding: vmcnt in bits 3:0 and 15:14, the other counters at their maxima)
#define MX_WAIT_VMCNT(n) __builtin_amdgcn_s_waitcnt(((n) & 15) | (((n) >> 4) << 14) | (7 << 4) | (15 << 8))

template <bool OUT_BF16>
__global__ __launch_bounds__(512) void gemm_mxfp4_dma_kernel(const MxGemmParams p) {
    constexpr int WAVES_N = 4, WM = 4, WN = 2, BM = 256, BN = 256;
    extern __shared__ __attribute__((aligned(16))) uint8_t mx_lds[];

    const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int r = lane & 31, h = lane >> 5;
    int tile_m, tile_n;
    mx_tile_of(blockIdx.x, p.tiles_m, p.tiles_n, tile_m, tile_n);
    const int64_t m0 = (int64_t)tile_m * BM, n0 = (int64_t)tile_n * BN;
    const int64_t kbytes = p.K >> 1;
    const int64_t ksteps = p.K / kMxBK;

    // The loads into LDS are written as inline assembly: the compiler orders a wait for ALL
    // loads in flight before any LDS read that follows such a load it knows about, which would
    // undo the pipelining.  Every global load of the loop is of this kind (the scales too), so
    // the compiler places no vector-memory waits of its own there and the one wait per step
    // is placed by hand in kstep().
    const mx_v4i ra = mx_raw_rsrc(p.A + m0 * kbytes, (uint32_t)(BM * kbytes));
    const mx_v4i rb = mx_raw_rsrc(p.B + n0 * kbytes, (uint32_t)(BN * kbytes));
    // wavefront w loads rows 32 w ... 32 w + 31 of both operands, 16 rows per instruction
    const int ld_row = lane >> 2;
    const uint32_t ld_off = (uint32_t)((wave * 32 + ld_row) * kbytes + (((lane & 3) ^ ((ld_row >> 2) & 3)) * 16));
    const int ld_half = (int)(16 * kbytes);
    // ... and 256 of the step's 2 KiB of scales (a 512-byte tile per 128 rows and K step):
    // waves 0-3 those of A (row tile w >> 1, half w & 1), waves 4-7 those of B
    const uint8_t *sf_src = (wave < 4 ? p.sfA + (m0 >> 7) * ksteps * 512 : p.sfB + (n0 >> 7) * ksteps * 512) + ((wave >> 1) & 1) * ksteps * 512;
    const mx_v4i rs = mx_raw_rsrc(sf_src, (uint32_t)(ksteps * 512));
    const uint32_t sf_off = (uint32_t)((wave & 1) * 256 + lane * 4);
    const uint32_t lds_base = (uint32_t)(uintptr_t)(MxLdsPtr)mx_lds;
    auto issue = [&](int64_t ks, int stage) {
        const int kq = (int)(ks * (kMxBK / 2)), ksf = (int)(ks * 512);
        const uint32_t base = lds_base + (uint32_t)(stage * kDmaStageBytes);
        const uint32_t run = base + (uint32_t)(wave * 2048), sf_run = base + (uint32_t)(2 * kDmaOperandBytes + wave * 256);
        // m0 = LDS address of the run a wavefront fills (lane i: unit i); one wait state
        // between a write of m0 and its use.  (m0 is reserved: the compiler never keeps a
        // value in it across other code, it writes it right before each use of its own.)
#pragma unroll
        for (int t = 0; t < 2; ++t) {
            asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tbuffer_load_dwordx4 %1, %2, %3 offen lds"
                         :
                         : "s"(run + t * 1024), "v"(ld_off), "s"(ra), "s"(kq + t * ld_half)
                         : "memory");
            asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tbuffer_load_dwordx4 %1, %2, %3 offen lds"
                         :
                         : "s"(run + kDmaOperandBytes + t * 1024), "v"(ld_off), "s"(rb), "s"(kq + t * ld_half)
                         : "memory");
        }
        asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tbuffer_load_dword %1, %2, %3 offen lds"
                     :
                     : "s"(sf_run), "v"(sf_off), "s"(rs), "s"(ksf)
                     : "memory");
    };
    constexpr int kLoadsPerStep = 5;

    const int wm = wave / WAVES_N, wn = wave % WAVES_N;
    mx_v16f acc[WM][WN];
#pragma unroll
    for (int i = 0; i < WM; ++i)
#pragma unroll
        for (int j = 0; j < WN; ++j)
#pragma unroll
            for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.0f;

    const uint32_t fa_off = (uint32_t)((wm * WM * 32 + r) * 64), fb_off = (uint32_t)(kDmaOperandBytes + (wn * WN * 32 + r) * 64);
    const int swz = (r >> 2) & 3;
    auto read_frags = [&](int stage, int kk, uint4 *fa, uint4 *fb) {
        const uint8_t *base = mx_lds + stage * kDmaStageBytes + (((kk * 2 + h) ^ swz) * 16);
#pragma unroll
        for (int i = 0; i < WM; ++i) fa[i] = *reinterpret_cast<const uint4 *>(base + fa_off + i * 32 * 64);
#pragma unroll
        for (int j = 0; j < WN; ++j) fb[j] = *reinterpret_cast<const uint4 *>(base + fb_off + j * 32 * 64);
    };
    // scale words of this wavefront's row tiles: the 16-byte unit of row r holds those of rows
    // r, r + 32, r + 64, r + 96 of a 128-row tile (A: all four; B: two of them)
    const uint32_t sa_off = (uint32_t)(2 * kDmaOperandBytes + wm * 512 + r * 16);
    const uint32_t sb_off = (uint32_t)(2 * kDmaOperandBytes + 1024 + (wn >> 1) * 512 + r * 16 + (wn & 1) * 8);

    // steps 0 .. 2 in flight (past the end: the last step once more, into stages nobody reads)
#pragma unroll
    for (int s = 0; s < kDmaStages - 1; ++s) issue(s < ksteps ? s : ksteps - 1, s);

    // One K step.  On entry the loads of step ks are the oldest in flight; behind them are
    // those of steps ks + 1 and ks + 2.  After the barrier every wavefront has its share of
    // step ks in LDS and has read the last fragments of step ks - 1, whose stage the loads of
    // step ks + 3 may overwrite.  (Moving the barrier between the two slices, with the next
    // step's first fragments read behind it, measured slower -- 341 against 320 us at 8192^3:
    // it asks for a step's operands half a step earlier, and their arrival is what a step
    // waits for.)
    for (int64_t ks = 0; ks < ksteps; ++ks) {
        const int stage = (int)(ks & (kDmaStages - 1));
        MX_WAIT_VMCNT(2 * kLoadsPerStep);
        __syncthreads();
        issue(ks + 3 < ksteps ? ks + 3 : ksteps - 1, (stage + 3) & (kDmaStages - 1));
        const uint8_t *st = mx_lds + stage * kDmaStageBytes;
        const uint4 wa = *reinterpret_cast<const uint4 *>(st + sa_off);
        const uint2 wb = *reinterpret_cast<const uint2 *>(st + sb_off);
        // lanes of the upper half use the next byte: after the shift, byte 0 / byte 2 of every
        // lane's register are the scales of the K blocks it feeds in slice 0 / slice 1
        const uint32_t sha[WM] = {wa.x >> (8 * h), wa.y >> (8 * h), wa.z >> (8 * h), wa.w >> (8 * h)};
        const uint32_t shb[WN] = {wb.x >> (8 * h), wb.y >> (8 * h)};
        uint4 fa[2][WM], fb[2][WN];
        read_frags(stage, 0, fa[0], fb[0]);
        read_frags(stage, 1, fa[1], fb[1]);
#pragma unroll
        for (int kk = 0; kk < 2; ++kk) {
#pragma unroll
            for (int i = 0; i < WM; ++i)
#pragma unroll
                for (int j = 0; j < WN; ++j) {
                    if (kk == 1)
                        acc[i][j] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(
                            frag_of(fb[1][j]), frag_of(fa[1][i]), acc[i][j], 4, 4, 2, (int)shb[j], 2, (int)sha[i]);
                    else
                        acc[i][j] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(
                            frag_of(fb[0][j]), frag_of(fa[0][i]), acc[i][j], 4, 4, 0, (int)shb[j], 0, (int)sha[i]);
                }
        }
        // issue order: the scale words and the first slice's fragments, then the second slice's six
        // fragment reads one at a time between the first MFMAs -- with all twelve reads ahead
        // of the first MFMA a step began with a longer wait (8192^3: 271 -> 263 us,
        // 2048 x 14336 x 4096: 70.8 -> 68.0 us in alternating series)
        __builtin_amdgcn_sched_group_barrier(0x100, 8, 0);
#pragma unroll
        for (int i = 0; i < 6; ++i) {
            __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
            __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
        }
        __builtin_amdgcn_sched_group_barrier(0x008, 10, 0);
    }
    // loads still in flight write LDS: drain them before the stages are used again
    MX_WAIT_VMCNT(0);
    __syncthreads();  // ... those of every wavefront, and all fragment reads are done

    mx_store_rows<WM, WN, OUT_BF16>(acc, mx_lds, wave, lane, *p.alpha, reinterpret_cast<uint16_t *>(p.D), p.ldd,
                                     m0 + wm * WM * 32, n0 + wn * WN * 32);
}

static int launch_gemm_mxfp4_dma(MxGemmParams &p, int out_type, hipStream_t s) {
    constexpr size_t lds_bytes = (size_t)kDmaStages * kDmaStageBytes;
    p.tiles_m = (int)(p.M / 256);
    p.tiles_n = (int)(p.N / 256);
    auto kernel = out_type == FOS_T_BF16 ? gemm_mxfp4_dma_kernel<true> : gemm_mxfp4_dma_kernel<false>;
    if (hipFuncSetAttribute((const void *)kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_bytes) != hipSuccess)
        return FOS_E_LAUNCH;
    hipLaunchKernelGGL(kernel, dim3((unsigned)(p.tiles_m * p.tiles_n)), dim3(512), lds_bytes, s, p);
    return hipGetLastError() == hipSuccess ? FOS_OK : FOS_E_LAUNCH;
}

}  // namespace fos

using namespace fos;

extern "C" int fos_gemm_mxfp4(const uint8_t *A, const uint8_t *B, const uint8_t *sfA, const uint8_t *sfB,
                              const float *alpha, int64_t M, int64_t N, int64_t K,
                              void *D, int out_type, int64_t ldd, fos_stream_t stream) {
    if (!A || !B || !sfA || !sfB || !alpha || !D) return FOS_E_NULL_POINTER;
    if (M <= 0 || N <= 0 || K <= 0 || M % 128 != 0 || N % 128 != 0 || K % 128 != 0 || ldd < N) return FOS_E_BAD_SHAPE;
    if (out_type != FOS_T_BF16 && out_type != FOS_T_F16) return FOS_E_UNSUPPORTED;
    if (((uintptr_t)A & 15) || ((uintptr_t)B & 15) || ((uintptr_t)sfA & 15) || ((uintptr_t)sfB & 15) ||
        ((uintptr_t)D & 15) || (ldd % 8 != 0) || ((uintptr_t)alpha & 3))
        return FOS_E_BAD_ALIGNMENT;
    if ((M / 128) * (N / 128) > 0x7fffffffLL || K > (1LL << 22)) return FOS_E_BAD_SHAPE;  // a 256-row panel of packed codes stays below 2^31 bytes (32-bit buffer offsets)
    MxGemmParams p;
    p.A = A; p.B = B; p.sfA = sfA; p.sfB = sfB; p.alpha = alpha; p.D = D;
    p.M = M; p.N = N; p.K = K; p.ldd = ldd;
    hipStream_t s = (hipStream_t)stream;
    bool big = (M % 256 == 0) && (N % 256 == 0) && (M / 256) * (N / 256) >= 256;
    int forced = 0;
    forced = fos::tuning().mx_tile;  // tuning / tests: 128 small tile, 256 register-staged big tile
    big = big && forced != 128;
    if (big && forced != 256) return launch_gemm_mxfp4_dma(p, out_type, s);
    if (big) return launch_gemm_mxfp4<2, 4, 4, 2>(p, out_type, s);
    return launch_gemm_mxfp4<2, 2, 2, 2>(p, out_type, s);
}
