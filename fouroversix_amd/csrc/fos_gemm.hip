// gfx950 NVFP4 x NVFP4 GEMM:  D[M,N] = alpha * sum_k (A[m,k] sA[m,k/16]) (B[n,k] sB[n,k/16]).
//
// The contraction runs on the fp16 MFMA pipe.  E2M1 codes and E4M3 block scales are
// loaded from HBM in their packed form, turned into fp16(value * scale) in registers
// (the product has at most 6 significant bits and lies in [2^-10, 2688], so it is exact
// in fp16 -- the same intermediate the reference's dequantize uses,
// src/fouroversix/quantize/backend.py:89-160), staged in LDS as fp16 and fed to
// v_mfma_f32_32x32x16_f16 with FP32 accumulation; alpha is applied in the epilogue from
// device memory (src/fouroversix/csrc/fp4_gemm.cu:143).
//
// Pipeline per workgroup (tile BM x BN x 64, BM = threads / 2): every thread owns 32 codes of
// one A row per K step.  Registers hold the packed data of step k+2 (in flight from HBM) while
// step k+1 is dequantised into one LDS buffer and step k is multiplied out of the other, so
// there is one barrier per K step and the VALU work of the dequantisation issues in the shadow
// of the MFMAs.  Only A goes through LDS: with both operands there, LDS traffic (fragment
// reads plus staging writes) took as many cycles per K step as the MFMAs themselves -- a build
// without the B fragment reads ran 13 % faster -- so each wavefront loads the packed rows of its
// own B columns and turns them into MFMA operands in registers.  Within a K step the
// contraction index is permuted the same way for both operands: the 16-wide slice kk of lane
// half h covers k = 32 h + 8 kk ... + 7, so that a lane's B codes are 16 contiguous bytes.
// The wavefronts of a workgroup sit side by side along N, each with all BM rows and 32
// columns (256 x 256 tile: 8 wavefronts of 256 x 32; 128 x 128 tile: 4 of 128 x 32), so every
// code of either operand is converted once per workgroup.  With two rows of wavefronts (128 x 64
// and 64 x 64 per wavefront) the two wavefronts that share B columns both converted them: the
// arrangement here reads twice the A fragments from LDS per MFMA and still measured faster,
// 8192^3 811 -> 790 us, 4096^3 107.5 -> 105.0 us in alternating series on one box, and
// 3072 x 4096 x 4096 131 -> 105 us, 1152 x 4096 x 4096 71 -> 56 us on the 128 x 128 tile (a
// 256 x 128 tile of 8 wavefronts of 128 x 32 in two rows lost to it wherever 256 x 256 tiles
// are too few to fill the chip), with bit-identical outputs.  The 128 x 128 tile serves
// shapes that are not multiples of 256 or too small to fill the chip otherwise, and a 128 x 256
// tile (the template with BM = 128 and eight wavefronts: every thread stages a quarter row of A) those
// that it covers with one workgroup per compute unit.
// Workgroups are numbered so that the tiles resident on one XCD (blockIdx % 8) form a
// compact block of the output, which keeps their A/B panels in that XCD's L2.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include <cstdlib>
#include <type_traits>

#include "fos_device.h"
#include "fos_tuning.h"
#include "fouroversix_hip.h"

namespace fos {

typedef _Float16 half2_t __attribute__((ext_vector_type(2)));
typedef _Float16 half8_t __attribute__((ext_vector_type(8)));
typedef float float16_t __attribute__((ext_vector_type(16)));
typedef float float4_t __attribute__((ext_vector_type(4)));

struct GemmParams {
    const uint8_t *A, *B;      // [M, K/2], [N, K/2]
    const uint8_t *sfA, *sfB;  // 128x4-tiled E4M3 bytes
    const float *alpha;        // output scale on the device, or null: (amax_a * amax_b) * inv_den
    const float *amax_a, *amax_b;
    float inv_den;
    void *D;
    const void *bias;          // optional: N values of the output type, added to the rounded product and rounded again
    float *d_amax;             // optional: max|D| as stored is folded into d_amax[0] (unsigned atomic max on the bits)
    int64_t M, N, K, ldd;
    int tiles_m, tiles_n;
    // split-K: workgroup (tile, blockIdx.y) contracts K steps [y * ksteps_per_split, ...) and
    // writes its FP32 partial tile to partials[y][M][N]; splits == 1 writes D directly
    float *partials;
    int splits, ksteps_per_split;
};

// Output scale: read from the device, or formed from the two tensor maxima with the
// arithmetic of gemm_alpha_kernel (product, then times the fp32 reciprocal of the divisor).
FOS_DEVICE float load_alpha(const GemmParams &p) {
    return p.alpha ? *p.alpha : (*p.amax_a * *p.amax_b) * p.inv_den;
}

// One value of the result as stored: alpha * acc rounded to the output type (16 bits returned).
template <bool OUT_BF16>
FOS_DEVICE uint32_t round_out(float v) {
    if (OUT_BF16) {
        uint32_t u = f2u(v);
        u += 0x7fffu + ((u >> 16) & 1u);
        return u >> 16;
    }
    // (v is a product already rounded to fp32 -- the reference's epilogue multiplies in fp32, then converts -- and
    // must stay one: left to itself the compiler folds the multiplication into the conversion, v_fma_mixlo_f16,
    // which rounds the exact product once and differs from the two roundings in one output in 10^5)
    asm("" : "+v"(v));
    return (uint32_t)__builtin_bit_cast(uint16_t, (_Float16)v);
}
template <bool OUT_BF16>
FOS_DEVICE float widen_out(uint32_t bits) {
    if (OUT_BF16) return u2f(bits << 16);
    return (float)__builtin_bit_cast(_Float16, (uint16_t)bits);
}

// Four consecutive outputs (columns n .. n + 3, n % 4 == 0) from their scaled accumulators: rounded to the output
// type, and with a bias rounded, added to bias[n ..] in fp32 and rounded again -- the two roundings of the
// reference's `out + bias` on the GEMM's result (src/fouroversix/model/modules/linear.py:83-92).  The magnitude
// bits of what goes into the last rounding are folded into `umax` as unsigned integers, which order finite
// values, infinity and NaN (largest) alike: a NaN in the output ends up as the recorded maximum, as it does
// in the reference's x.abs().max().
template <bool OUT_BF16>
FOS_DEVICE uint32_t finish_output(float f, bool with_bias, uint32_t bias16, uint32_t &umax) {
    if (with_bias) f = widen_out<OUT_BF16>(round_out<OUT_BF16>(f)) + widen_out<OUT_BF16>(bias16);
    const uint32_t mag = f2u(f) & 0x7fffffffu;
    umax = mag > umax ? mag : umax;
    return round_out<OUT_BF16>(f);
}
template <bool OUT_BF16>
FOS_DEVICE uint2 pack_outputs(const float *v, const void *bias, int64_t n, uint32_t &umax) {
    uint2 bw = make_uint2(0u, 0u);
    if (bias) bw = *reinterpret_cast<const uint2 *>(static_cast<const uint16_t *>(bias) + n);
    const uint32_t o0 = finish_output<OUT_BF16>(v[0], bias != nullptr, bw.x & 0xffffu, umax);
    const uint32_t o1 = finish_output<OUT_BF16>(v[1], bias != nullptr, bw.x >> 16, umax);
    const uint32_t o2 = finish_output<OUT_BF16>(v[2], bias != nullptr, bw.y & 0xffffu, umax);
    const uint32_t o3 = finish_output<OUT_BF16>(v[3], bias != nullptr, bw.y >> 16, umax);
    return make_uint2(o0 | (o1 << 16), o2 | (o3 << 16));
}
// ... two consecutive outputs (n % 2 == 0)
template <bool OUT_BF16>
FOS_DEVICE uint32_t pack_outputs2(float v0, float v1, const void *bias, int64_t n, uint32_t &umax) {
    uint32_t bw = 0u;
    if (bias) bw = *reinterpret_cast<const uint32_t *>(static_cast<const uint16_t *>(bias) + n);
    const uint32_t o0 = finish_output<OUT_BF16>(v0, bias != nullptr, bw & 0xffffu, umax);
    const uint32_t o1 = finish_output<OUT_BF16>(v1, bias != nullptr, bw >> 16, umax);
    return o0 | (o1 << 16);
}

// max|D| for the caller that quantizes D next: `umax` holds the magnitude bits of the largest value this
// lane stored, before its rounding to the output type (0 for a lane that stored nothing).  Rounding is
// monotonic, so the rounded maximum is the maximum of the rounded values.  At most one vector atomic per
// wavefront on the unsigned image of the value (non-negative floats order like their bits, NaN above all);
// every lane of the wavefront must call it.
template <bool OUT_BF16>
FOS_DEVICE void fold_amax(float *d_amax, uint32_t umax) {
    uint32_t r;
    if (umax > 0x7f800000u) r = 0x7fc00000u;
    else r = f2u(widen_out<OUT_BF16>(round_out<OUT_BF16>(u2f(umax))));
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) {
        const uint32_t other = (uint32_t)__shfl_xor((int)r, off);
        r = other > r ? other : r;
    }
    // (the atomics of a launch all go to one address and are served one after the other: a
    // wavefront first looks whether its value would change anything -- only the first few do)
    if ((threadIdx.x & 63) == 0) {
        unsigned int *word = reinterpret_cast<unsigned int *>(d_amax);
        if (r > __hip_atomic_load(word, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT)) atomicMax(word, r);
    }
}

// The two E4M3 bytes in the low 16 bits of `w` -> fp16 pair {s0, s1} (one hardware
// convert; exact, sub-normals included -- checked against the OCP decode of all 256 bytes).
FOS_DEVICE half2_t e4m3x2_to_half2(uint32_t w) {
    return __builtin_amdgcn_cvt_scalef32_pk_f16_fp8(w, 1.0f, false);
}

// 8 packed codes (one 32-bit word) times a block scale -> 8 fp16 in k order.
FOS_DEVICE half8_t dequant8(uint32_t word, half2_t s) {
    half2_t p0 = __builtin_amdgcn_cvt_scalef32_pk_f16_fp4(word, 1.0f, 0) * s;
    half2_t p1 = __builtin_amdgcn_cvt_scalef32_pk_f16_fp4(word, 1.0f, 1) * s;
    half2_t p2 = __builtin_amdgcn_cvt_scalef32_pk_f16_fp4(word, 1.0f, 2) * s;
    half2_t p3 = __builtin_amdgcn_cvt_scalef32_pk_f16_fp4(word, 1.0f, 3) * s;
    half8_t r = {p0.x, p0.y, p1.x, p1.y, p2.x, p2.y, p3.x, p3.y};
    return r;
}

constexpr int BK = 64;
constexpr int kPitch = BK + 8;  // halfs per LDS row (144 bytes: conflict-free 128-bit accesses)

// Buffer resource (V#) over [base, base + bytes): raw 32-bit offsets, no swizzle.
typedef __amdgpu_buffer_rsrc_t BufferRsrc;
typedef uint32_t uint4_t __attribute__((ext_vector_type(4)));
FOS_DEVICE BufferRsrc make_rsrc(const void *base, uint32_t bytes) {
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<void *>(base), 0, (int)bytes, 0x00020000);
}

// Packed operands of one K step as a thread holds them: the half row of A that it turns into
// fp16 in LDS for the whole workgroup, and, per 32-row tile of its wavefront's B columns, the
// 32 codes and 4 scale bytes it multiplies itself.
template <int WN>
struct Staged {
    uint4 qa;      // 32 codes of one A row
    uint32_t sa;   // the 4 scale bytes of that row's K step
    uint4 qb[WN];  // B row of tile j: codes 32 h ... 32 h + 31 of the step (h = lane >> 5)
    uint32_t sb[WN];
};

// Output tile of workgroup `bid`: workgroups with equal bid % 8 share an XCD; give each
// XCD a contiguous run of tiles, ordered in column bands of 8 tile rows.
FOS_DEVICE void tile_of(int bid, int tiles_m, int tiles_n, int &tm, int &tn) {
    const int total = tiles_m * tiles_n;
    const int per_xcd = (total + 7) / 8;
    int t = (bid & 7) * per_xcd + (bid >> 3);
    if (t >= total || (total & 7) != 0) t = bid;  // ragged counts: plain order
    constexpr int kBand = 8;
    const int band = t / (kBand * tiles_n), in_band = t - band * kBand * tiles_n;
    const int rows = (tiles_m - band * kBand) < kBand ? (tiles_m - band * kBand) : kBand;
    tm = band * kBand + in_band % rows;
    tn = in_band / rows;
}

// WAVES_M x WAVES_N wavefronts, each WM x WN MFMA tiles of 32 x 32.  The MFMA "A" operand
// is fed from the B matrix (rows n) and the "B" operand from the A matrix (rows m), so
// that a lane's four consecutive accumulator registers are four consecutive n of one
// output row and can be stored as 8 bytes.
enum { kOutF16 = 0, kOutBF16 = 1, kOutPartial = 2 };

// QUARTER (4 * BM == threads): every thread stages a quarter row of A (16 codes) instead of the first 2 * BM threads
// half a row each, so that all wavefronts carry the same conversion work.
template <int WAVES_M, int WAVES_N, int WM, int WN, int OUT, bool QUARTER = false>
__global__ __launch_bounds__(64 * WAVES_M *WAVES_N) void gemm_nvfp4_kernel(const GemmParams p) {
    constexpr bool OUT_BF16 = OUT == kOutBF16;
    constexpr int kThreadsG = 64 * WAVES_M * WAVES_N;
    constexpr int BM = WAVES_M * WM * 32, BN = WAVES_N * WN * 32;
    static_assert(2 * BM <= kThreadsG, "one thread per half row of A (wavefronts beyond the first 2 * BM threads stage nothing)");
    static_assert(!QUARTER || 4 * BM == kThreadsG, "quarter rows: four threads per row of A");
    constexpr bool kAllStage = QUARTER || 2 * BM == kThreadsG;
    extern __shared__ __attribute__((aligned(16))) _Float16 lds[];
    _Float16 *lds_a[2] = {lds, lds + BM * kPitch};

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    int tile_m, tile_n;
    tile_of(blockIdx.x, p.tiles_m, p.tiles_n, tile_m, tile_n);
    const int64_t m0 = (int64_t)tile_m * BM, n0 = (int64_t)tile_n * BN;
    const int64_t kbytes = p.K >> 1;     // packed bytes per row
    const int64_t sf_groups = p.K >> 6;  // 4-block groups per row

    // global -> register staging: 32 codes (16 bytes) of one row of each operand, through
    // buffer loads (wave-uniform base + per-thread 32-bit offset + scalar K offset), which
    // keeps 64-bit address arithmetic out of the loop
    // (QUARTER: ld_half counts quarter rows, 0..3)
    const int ld_row = QUARTER ? tid >> 2 : tid >> 1, ld_half = QUARTER ? tid & 3 : tid & 1;
    const bool stager = __builtin_amdgcn_readfirstlane(tid) < 2 * BM;  // wavefront-uniform
    const BufferRsrc ra = make_rsrc(p.A + m0 * kbytes, (uint32_t)(BM * kbytes));
    const BufferRsrc rb = make_rsrc(p.B + n0 * kbytes, (uint32_t)(BN * kbytes));
    const BufferRsrc rsa = make_rsrc(p.sfA + (m0 >> 7) * sf_groups * 512, (uint32_t)((BM >> 7) * sf_groups * 512));
    const BufferRsrc rsb = make_rsrc(p.sfB + (n0 >> 7) * sf_groups * 512, (uint32_t)((BN >> 7) * sf_groups * 512));
    const uint32_t q_off = (uint32_t)(ld_row * kbytes + ld_half * (QUARTER ? 8 : 16));
    const uint32_t s_off = (uint32_t)((ld_row >> 7) * sf_groups * 512 + (ld_row & 31) * 16 + ((ld_row & 127) >> 5) * 4);
    // this lane's B rows: row (lane & 31) of tile j of the wavefront's columns, K half lane >> 5
    const int wm = wave / WAVES_N, wn = wave % WAVES_N;
    const int lh = lane >> 5;
    uint32_t qb_off[WN], sb_off[WN];
#pragma unroll
    for (int j = 0; j < WN; ++j) {
        const int row = wn * WN * 32 + j * 32 + (lane & 31);
        qb_off[j] = (uint32_t)(row * kbytes + lh * 16);
        sb_off[j] = (uint32_t)((row >> 7) * sf_groups * 512 + (row & 31) * 16 + ((row & 127) >> 5) * 4);
    }
    // this workgroup's share of the K steps (all of them unless the launch splits K)
    const int64_t ks0 = OUT == kOutPartial ? (int64_t)blockIdx.y * p.ksteps_per_split : 0;
    const int64_t ksteps_all = p.K / BK;
    const int64_t ksteps =
        OUT == kOutPartial ? (ksteps_all - ks0 < p.ksteps_per_split ? ksteps_all - ks0 : p.ksteps_per_split) : ksteps_all;

    typedef Staged<WN> StagedT;
    auto fetch = [&](int64_t ks, StagedT &s) {
        const uint32_t kq = (uint32_t)(ks0 + ks) * 32u, ksf = (uint32_t)(ks0 + ks) * 512u;
        if constexpr (QUARTER) {
            const uint2 w = __builtin_bit_cast(uint2, __builtin_amdgcn_raw_buffer_load_b64(ra, (int)q_off, (int)kq, 0));
            s.qa.x = w.x;
            s.qa.y = w.y;
            s.sa = __builtin_amdgcn_raw_buffer_load_b32(rsa, (int)s_off, (int)ksf, 0);
        } else if (kAllStage || stager) {
            s.qa = __builtin_bit_cast(uint4, __builtin_amdgcn_raw_buffer_load_b128(ra, (int)q_off, (int)kq, 0));
            s.sa = __builtin_amdgcn_raw_buffer_load_b32(rsa, (int)s_off, (int)ksf, 0);
        }
#pragma unroll
        for (int j = 0; j < WN; ++j) {
            s.qb[j] = __builtin_bit_cast(uint4, __builtin_amdgcn_raw_buffer_load_b128(rb, (int)qb_off[j], (int)kq, 0));
            s.sb[j] = __builtin_amdgcn_raw_buffer_load_b32(rsb, (int)sb_off[j], (int)ksf, 0);
        }
    };
    // quarter q (0..3) of the staged A data -> 8 halfs in LDS buffer `buf`
    auto stage_quarter = [&](const StagedT &s, int buf, int q) {
        if constexpr (QUARTER) {
            // the thread's 16 codes are one block: its two words go out in the first and the third slice of a step
            if (q & 1) return;
            const uint32_t wq = q == 0 ? s.qa.x : s.qa.y;
            const half2_t s2 = e4m3x2_to_half2(s.sa >> (8 * ld_half));
            const half2_t sq = __builtin_shufflevector(s2, s2, 0, 0);
            half8_t *dq = reinterpret_cast<half8_t *>(lds_a[buf] + ld_row * kPitch + ld_half * 16);
            dq[q >> 1] = dequant8(wq, sq);
            return;
        }
        if (!kAllStage && !stager) return;
        const uint32_t wa = q == 0 ? s.qa.x : q == 1 ? s.qa.y : q == 2 ? s.qa.z : s.qa.w;
        // this thread's two block scales: bytes 2*ld_half, 2*ld_half + 1
        const half2_t sa2 = e4m3x2_to_half2(s.sa >> (16 * ld_half));
        const half2_t sa = (q >> 1) ? __builtin_shufflevector(sa2, sa2, 1, 1) : __builtin_shufflevector(sa2, sa2, 0, 0);
        half8_t *da = reinterpret_cast<half8_t *>(lds_a[buf] + ld_row * kPitch + ld_half * 32);
        da[q] = dequant8(wa, sa);
    };
    // MFMA operands of slice kk from this lane's packed B rows: word kk of its 16 bytes, blocks
    // 2 h + (kk >> 1) of the step
    auto b_frags = [&](const StagedT &s, int kk, half8_t *fb) {
#pragma unroll
        for (int j = 0; j < WN; ++j) {
            const uint32_t wb = kk == 0 ? s.qb[j].x : kk == 1 ? s.qb[j].y : kk == 2 ? s.qb[j].z : s.qb[j].w;
            const half2_t sb2 = e4m3x2_to_half2(s.sb[j] >> (16 * lh));
            const half2_t sb = (kk >> 1) ? __builtin_shufflevector(sb2, sb2, 1, 1) : __builtin_shufflevector(sb2, sb2, 0, 0);
            fb[j] = dequant8(wb, sb);
        }
    };

    float16_t acc[WM][WN];
#pragma unroll
    for (int i = 0; i < WM; ++i)
#pragma unroll
        for (int j = 0; j < WN; ++j)
#pragma unroll
            for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.0f;

    auto read_frags = [&](int buf, int kk, half8_t *fa) {
        const int kofs = lh * 32 + kk * 8;
#pragma unroll
        for (int i = 0; i < WM; ++i)
            fa[i] = *reinterpret_cast<const half8_t *>(lds_a[buf] + (wm * WM * 32 + i * 32 + (lane & 31)) * kPitch + kofs);
    };

    StagedT st[2];
    StagedT bcur;                  // the step being multiplied: its B rows (st[] is refilled two steps ahead)
    half8_t fa[2][WM], fb[2][WN];  // MFMA fragments of the current and the next 16-wide K slice
    fetch(0, st[0]);
#pragma unroll
    for (int q = 0; q < 4; ++q) stage_quarter(st[0], 0, q);
    b_frags(st[0], 0, fb[0]);
    bcur = st[0];
    if (ksteps > 1) fetch(1, st[1]);
    __syncthreads();
    read_frags(0, 0, fa[0]);

    // Body of one K step: multiply out of buffer `buf` while staging `nxt` (step ks+1) into
    // the other buffer.  Inside a 16-wide K slice the order is: issue the LDS reads of the
    // NEXT slice, dequantise + write a quarter of the next step, then the MFMAs of the
    // current slice, whose fragments are already in registers.  The step's barrier sits
    // between the last quarter's writes and the last slice's MFMAs, and the first slice of
    // the next step is read right after it, so the matrix pipe has work on both sides of
    // the barrier and no LDS latency is exposed at the step boundary.
    // The body is branch-free (the last step, which has nothing to stage, is a separate
    // instantiation; the prefetch index is clamped instead of guarded): waits are then
    // placed per register instead of conservatively at control-flow joins.
    auto kstep = [&](auto have_next_c, int64_t ks, int buf, StagedT &cur_regs, StagedT &nxt) {
        constexpr bool have_next = decltype(have_next_c)::value;
        // `cur_regs` (step ks): its A part went into LDS during the previous step and its B part
        // was copied to `bcur` (before the first step, and at the end of the previous one); refill
        // them now, two steps ahead of their use, so HBM / L2 latency has a whole K step to hide in
        if (have_next) fetch(ks + 2 < ksteps ? ks + 2 : ksteps - 1, cur_regs);
#pragma unroll
        for (int kk = 0; kk < BK / 16; ++kk) {
            if (kk + 1 < BK / 16) {
                read_frags(buf, kk + 1, fa[(kk + 1) & 1]);
                b_frags(bcur, kk + 1, fb[(kk + 1) & 1]);
            }
            if (have_next) stage_quarter(nxt, buf ^ 1, kk);
            const bool at_barrier = have_next && kk + 1 == BK / 16;
            auto mfmas = [&](int i_begin, int i_end) {
#pragma unroll
                for (int i = i_begin; i < i_end; ++i)
#pragma unroll
                    for (int j = 0; j < WN; ++j)
                        acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(fb[kk & 1][j], fa[kk & 1][i], acc[i][j], 0, 0, 0);
            };
            if (at_barrier) {
                // half of the last slice's MFMAs go above the barrier, where they overlap the
                // last quarter's dequantisation, and half below it, where they cover the LDS
                // latency of the next step's first fragments (the scheduler must not move
                // them across: either side would leave the matrix pipe idle)
                mfmas(0, WM / 2);
                __builtin_amdgcn_sched_barrier(0);
                __syncthreads();
                read_frags(buf ^ 1, 0, fa[0]);
                __builtin_amdgcn_sched_barrier(0);
                mfmas(WM / 2, WM);
                // the next step's B rows become the current ones (fb[0] is free: slice 3 used fb[1])
                bcur = nxt;
                b_frags(bcur, 0, fb[0]);
            } else {
                mfmas(0, WM);
                // issue order inside the slice: one MFMA, one LDS read of the next slice's
                // fragments, a few of the conversion instructions, and so on -- left to itself the
                // scheduler bunches the reads ahead of the MFMAs (8192^3: 830 -> 815 us,
                // 16384 x 1024 x 4096: 114.7 -> 110.8 us in alternating series)
#pragma unroll
                for (int i = 0; i < WM * WN; ++i) {
                    __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);  // MFMA
                    if (i < WM) __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);  // LDS read
                    __builtin_amdgcn_sched_group_barrier(0x002, 4, 0);  // VALU
                }
            }
            // slices are scheduled one at a time: a wider window only raises register pressure
            __builtin_amdgcn_sched_barrier(0);
        }
    };

    using yes = std::integral_constant<bool, true>;
    using no = std::integral_constant<bool, false>;
    // Steps go in pairs (the two LDS buffers and register sets alternate by name).  The
    // last pair stages the clamped prefetch -- the final step's data once more -- into the
    // buffer nobody reads again, which is cheaper than a separate copy of the loop body
    // for the end of the K range; an odd step count leaves one step without staging.
    int64_t ks = 0;
    for (; ks + 2 <= ksteps; ks += 2) {
        kstep(yes{}, ks, 0, st[0], st[1]);
        kstep(yes{}, ks + 1, 1, st[1], st[0]);
    }
    if (ks < ksteps) kstep(no{}, ks, 0, st[0], st[1]);

    // epilogue: acc[i][j][4*g + e] is D[m][n] with m = wm*WM*32 + i*32 + (lane & 31),
    // n = wn*WN*32 + j*32 + 8*g + 4*(lane >> 5) + e
    if (OUT == kOutPartial) {
        float *P = p.partials + (int64_t)blockIdx.y * p.M * p.N;
#pragma unroll
        for (int i = 0; i < WM; ++i) {
            const int64_t m = m0 + wm * WM * 32 + i * 32 + (lane & 31);
#pragma unroll
            for (int j = 0; j < WN; ++j)
#pragma unroll
                for (int g = 0; g < 4; ++g) {
                    const int64_t n = n0 + wn * WN * 32 + j * 32 + 8 * g + 4 * (lane >> 5);
                    *reinterpret_cast<float4 *>(P + m * p.N + n) =
                        make_float4(acc[i][j][4 * g], acc[i][j][4 * g + 1], acc[i][j][4 * g + 2], acc[i][j][4 * g + 3]);
                }
        }
        return;
    }
    const float alpha = load_alpha(p);
    uint16_t *D = reinterpret_cast<uint16_t *>(p.D);
    // A lane holds 4 consecutive n of row m = lane & 31: written as they are, a store
    // instruction touches 32 rows with 16 bytes each, and the counters showed 2.2 bytes
    // written to memory per byte of output.  Each wavefront therefore turns its 32-row tiles
    // round in LDS (free after the last K step: 32 rows x WN * 64 bytes + 16 bytes of padding
    // per wavefront) and stores whole rows: 16 bytes per lane, WN * 4 lanes per row.
    constexpr int kRowBytes = WN * 64, kEpiPitch = kRowBytes + 16;
    static_assert(2 * BM * kPitch * (int)sizeof(_Float16) >= WAVES_M * WAVES_N * 32 * kEpiPitch, "epilogue staging fits the A buffers");
    __syncthreads();  // every wavefront is done reading the A buffers
    uint8_t *epi = reinterpret_cast<uint8_t *>(lds) + wave * 32 * kEpiPitch;
    constexpr int kLanesPerRow = kRowBytes / 16, kRowsPerPass = 64 / kLanesPerRow;
    uint32_t umax = 0u;
#pragma unroll
    for (int i = 0; i < WM; ++i) {
#pragma unroll
        for (int j = 0; j < WN; ++j) {
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                const float v[4] = {alpha * acc[i][j][4 * g], alpha * acc[i][j][4 * g + 1], alpha * acc[i][j][4 * g + 2],
                                    alpha * acc[i][j][4 * g + 3]};
                const int nl = j * 32 + 8 * g + 4 * (lane >> 5);  // column inside the wavefront's strip
                *reinterpret_cast<uint2 *>(epi + (lane & 31) * kEpiPitch + nl * 2) =
                    pack_outputs<OUT_BF16>(v, p.bias, n0 + wn * WN * 32 + nl, umax);
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
            const int64_t m = m0 + wm * WM * 32 + i * 32 + row;
            *reinterpret_cast<uint4 *>(D + m * p.ldd + n0 + wn * WN * 32 + c16 * 8) = v;
        }
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
    }
    if (p.d_amax) fold_amax<OUT_BF16>(p.d_amax, umax);
}

// ---------------------------------------------------------------------------------------
// M <= 128 ("skinny": decode-sized batches, one 128-row band of A).  The weight matrix B is
// streamed once from HBM; a workgroup owns 32 rows of B and the first 32 * MT rows of A,
// and its 8 wavefronts split the K steps of 256 between them (wave w takes steps w, w + 8,
// ...), so no data is shared between wavefronts and the main loop has no barrier.
//
// The 32 rows are n128 + 32 q + r0 + i (q = 0..3, i = 0..7; tile row rho = 8 q + i): the tiled
// scale layout keeps rows r, r + 32, r + 64, r + 96 in one 16-byte unit, so the scales of
// these rows are 128 contiguous bytes per K group, where 32 consecutive rows would use 4
// bytes of each of 32 units.
//
// Per step a lane (r = lane & 31, h = lane >> 5) multiplies the 128 codes
// k = 256 step + 128 h ... of B tile row r with the same codes of A rows r + 32 i.
// The MFMA contraction index is thereby permuted (slice x pairs codes 8x..8x+7 of both
// lane halves); A and B use the same permutation, so the sum is unchanged.
//  * A codes are re-read by every workgroup, so their path through the vector cache
//    matters: a wavefront loads its A step with 8 lanes per 128-byte row segment (whole
//    cache lines) and transposes it through a private LDS region into the per-row
//    fragment order (LDS operations of one wavefront execute in order: no barrier).
//  * B codes take the same route for M <= 64; a lane loading its own 64 bytes would
//    touch every line with four instructions, and with a few thousand lines in flight per
//    CU the vector cache refetches them.  For M = 128 the A regions leave no room and B
//    goes straight from global memory to the lane that multiplies it.
//  * Scales: the 128x4 tiled layout puts the four blocks of a 64-wide K group of rows r,
//    r + 32, r + 64, r + 96 next to each other, so one 128-bit load per group fetches the
//    scales of the A rows of a lane (fewer words for fewer row tiles); B takes one 32-bit
//    word per group.
// The 8 partial accumulators are tree-reduced through LDS at the end (fixed order).
constexpr int kSkinnyRotation = 5;  // K steps between the starting points of neighbouring workgroups (odd: 8 in a row are in flight)
constexpr int kSkinnyPitch = 144;  // LDS bytes per A row (128 + 16: conflict-free 128-bit accesses)

// N consecutive 32-bit words (N = 1, 2, 4) with one buffer load.
template <int N>
FOS_DEVICE void load_words(uint32_t (&dst)[N], BufferRsrc r, int voffset, int soffset) {
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

template <int MT, int WN>
struct SkinnyRegs {
    uint32_t sb[WN][2]; // the 8 block scales of each B row (two groups)
    uint32_t sa[2][MT]; // block scales of the A rows: [group][i] = row r + 32 i
};

// Wavefronts of a workgroup: 8 with one 32-row tile of B each; 4 with two (WN = 2), and then two
// workgroups per compute unit.
constexpr int skinny_waves(int WN) { return WN == 2 ? 4 : 8; }

template <int MT, int WN, int OUT>
__global__ __launch_bounds__(64 * skinny_waves(WN), (WN == 2 && MT == 2) ? 2 : 1) void gemm_nvfp4_skinny_kernel(const GemmParams p) {
    constexpr int kWaves = skinny_waves(WN), kAcc = MT * WN * 16;
    // B through LDS as well (whole cache lines per load instruction, see above) where the
    // second staging region fits next to A's
    constexpr bool kBViaLds = MT <= 2 || WN == 2;
    constexpr int kRegionA = MT * 32 * kSkinnyPitch;
    constexpr int kRegion = kRegionA + (kBViaLds ? WN * 32 * kSkinnyPitch : 0);
    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
    // the wave index steers loops and scalar buffer offsets: make its uniformity known
    const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), r = lane & 31, h = lane >> 5;
    uint8_t *region = smem + wave * kRegion;
    // tile t holds rows n128 + 32 q + r0 + 8 t + i (q = 0..3, i = 0..7): their scales are whole
    // cache lines of the tiled layout (four rows 32 apart share a 16-byte unit); tile row rho = 8 q + i
    static_assert(WN == 1 || (WN == 2 && MT <= 2), "32 or 64 of the 128 rows of a band per workgroup");
    constexpr int kPerBand = 4 / WN;
    const int64_t n128 = (int64_t)(blockIdx.x / kPerBand) * 128;
    const int r0 = (int)(blockIdx.x % kPerBand) * 8 * WN;
    // a launch with gridDim.z > 1 gives every 32 MT rows of A workgroups of their own
    const int m_base = (int)blockIdx.z * 32 * MT;
    const int64_t kbytes = p.K >> 1, sf_groups = p.K >> 6;
    const int64_t steps_all = p.K >> 8;
    const int64_t s_begin = OUT == kOutPartial ? (int64_t)blockIdx.y * p.ksteps_per_split : 0;
    const int64_t s_end = OUT == kOutPartial ? (s_begin + p.ksteps_per_split < steps_all ? s_begin + p.ksteps_per_split : steps_all)
                                             : steps_all;

    // Workgroups start at different K offsets and wrap around: started together at K = 0 they
    // would all ask the same few memory channels for the same columns of their rows at the
    // same time (rows are K / 2 bytes apart, typically a power of two).  The order of
    // accumulation of a column block thereby depends on its index, and on nothing else.
    const int64_t nsteps = s_end - s_begin;
    const int64_t rot_wg = nsteps > 0 ? ((int64_t)blockIdx.x * kSkinnyRotation) % nsteps : 0;
    auto phys = [&](int64_t j) -> int64_t {  // j-th step of this workgroup -> K step
        const int64_t q = j + rot_wg;
        return s_begin + (q >= nsteps ? q - nsteps : q);
    };

    // rows of A past M read as zero codes (buffer range check), so A needs only M rows
    const BufferRsrc ra = make_rsrc(p.A, (uint32_t)(p.M * kbytes));
    const BufferRsrc rb = make_rsrc(p.B + n128 * kbytes, (uint32_t)(128 * kbytes));
    const BufferRsrc rsa = make_rsrc(p.sfA, (uint32_t)(sf_groups * 512));
    const BufferRsrc rsb = make_rsrc(p.sfB + (n128 >> 7) * sf_groups * 512, (uint32_t)(sf_groups * 512));
    const uint32_t a_off = (uint32_t)((lane >> 3) * kbytes + (lane & 7) * 16);  // row 8 j + lane / 8, 16-byte column lane % 8
    const uint32_t a_row0 = (uint32_t)(m_base * kbytes);
    const uint32_t b_off = (uint32_t)((32 * (r >> 3) + r0 + (r & 7)) * kbytes + h * 64);
    const uint32_t sa_off = (uint32_t)(h * 1024 + r * 16 + (m_base >> 5) * 4);
    const uint32_t sb_off = (uint32_t)(h * 1024 + (r0 + (r & 7)) * 16 + (r >> 3) * 4);
    const uint32_t lds_w = (uint32_t)((lane >> 3) * kSkinnyPitch + (lane & 7) * 16);
    const uint32_t lds_r = (uint32_t)(r * kSkinnyPitch + h * 64);

    // Loads are issued unconditionally, so that the wait counts in the loop below are exact
    // (a load under a branch makes the compiler wait for everything in flight, the prefetches
    // just issued included): a step past the end reads through a descriptor of size zero,
    // which returns zeros without touching memory.
    const BufferRsrc r_none = make_rsrc(p.A, 0);
    uint4 a_stage[MT * 4];  // one A step in flight from global memory
    auto fetch_a = [&](int64_t j) {
        const bool ok = j < nsteps;
        const BufferRsrc r = ok ? ra : r_none;
        const int kq = ok ? (int)(phys(j) * 128) : 0;
#pragma unroll
        for (int i = 0; i < MT * 4; ++i)
            a_stage[i] = __builtin_bit_cast(uint4, __builtin_amdgcn_raw_buffer_load_b128(r, (int)(a_row0 + a_off + i * 8 * kbytes), kq, 0));
    };
    // 128 codes of each B row; two register sets (loaded two steps ahead), one with two tiles
    constexpr int kBSets = (WN == 2 || MT == 2) ? 1 : 2;  // (the 4 x 1 form multiplies straight from these registers: two sets)
    typedef uint4 BCodes[WN][4];
    BCodes bst[kBSets];
    auto fetch_b_codes = [&](int64_t j, BCodes &b) {
        const bool ok = j < nsteps;
        const BufferRsrc r = ok ? rb : r_none;
        const int kq = ok ? (int)(phys(j) * 128) : 0;
#pragma unroll
        for (int t = 0; t < WN; ++t)
#pragma unroll
            for (int q = 0; q < 4; ++q)
                b[t][q] = __builtin_bit_cast(
                    uint4, kBViaLds ? __builtin_amdgcn_raw_buffer_load_b128(r, (int)(a_off + (q * 32 + r0 + 8 * t) * kbytes), kq, 0)
                                    : __builtin_amdgcn_raw_buffer_load_b128(r, (int)(b_off + 8 * t * kbytes + q * 16), kq, 0));
    };
    auto fetch_scales = [&](int64_t j, SkinnyRegs<MT, WN> &s) {
        const bool ok = j < nsteps;
        const BufferRsrc r_a = ok ? rsa : r_none, r_b = ok ? rsb : r_none;
        const int ksf = ok ? (int)(phys(j) * 2048) : 0;
#pragma unroll
        for (int t = 0; t < WN; ++t)
#pragma unroll
            for (int u = 0; u < 2; ++u) s.sb[t][u] = __builtin_amdgcn_raw_buffer_load_b32(r_b, (int)(sb_off + t * 128 + u * 512), ksf, 0);
#pragma unroll
        for (int u = 0; u < 2; ++u)
            load_words<MT>(s.sa[u], r_a, (int)(sa_off + u * 512), ksf);
    };

    float16_t acc[MT][WN];
#pragma unroll
    for (int i = 0; i < MT; ++i)
#pragma unroll
        for (int t = 0; t < WN; ++t)
#pragma unroll
            for (int e = 0; e < 16; ++e) acc[i][t][e] = 0.0f;

    auto word_of = [](const uint4 &v, int j) -> uint32_t { return j == 0 ? v.x : j == 1 ? v.y : j == 2 ? v.z : v.w; };
    // scale of code word x (0..15) of a lane: block x >> 1 = byte (x >> 1) & 3 of group word x >> 3
    auto scale_of = [](uint32_t w, int x) -> half2_t {
        const half2_t s2 = e4m3x2_to_half2((x & 4) ? w >> 16 : w);
        return ((x >> 1) & 1) ? __builtin_shufflevector(s2, s2, 1, 1) : __builtin_shufflevector(s2, s2, 0, 0);
    };
    auto read_frags = [&](int q, uint4 *fr) {
#pragma unroll
        for (int i = 0; i < MT; ++i) fr[i] = *reinterpret_cast<const uint4 *>(region + lds_r + i * 32 * kSkinnyPitch + q * 16);
    };
    auto read_frags_b = [&](int q, uint4 *fr) {
#pragma unroll
        for (int t = 0; t < WN; ++t)
            fr[t] = *reinterpret_cast<const uint4 *>(region + kRegionA + lds_r + t * 32 * kSkinnyPitch + q * 16);
    };
    // one step: the staged codes go through LDS, the loads that refill the staging registers
    // are issued (A for the wavefront's next step first: it is needed first and loads return
    // in order; then, where B is staged too, the codes of this register set's step after
    // next: the scales stay in use and follow after the multiplication), then 16 K slices
    // are multiplied
    auto compute = [&](SkinnyRegs<MT, WN> &s, BCodes &b, int64_t next_step, int64_t refill_step) {
#pragma unroll
        for (int j = 0; j < MT * 4; ++j) *reinterpret_cast<uint4 *>(region + lds_w + j * 8 * kSkinnyPitch) = a_stage[j];
        if (kBViaLds) {
#pragma unroll
            for (int t = 0; t < WN; ++t)
#pragma unroll
                for (int q = 0; q < 4; ++q)
                    *reinterpret_cast<uint4 *>(region + kRegionA + lds_w + (t * 32 + q * 8) * kSkinnyPitch) = b[t][q];
        }
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        uint4 fr[2][MT], frb[2][WN];
        read_frags(0, fr[0]);
        if (kBViaLds) read_frags_b(0, frb[0]);
        // the refills go out here, ahead of the arithmetic: the scheduler may not sink them
        if constexpr (kBViaLds) {
            __builtin_amdgcn_sched_barrier(0);
            fetch_a(next_step);
            fetch_b_codes(refill_step, b);
            __builtin_amdgcn_sched_barrier(0);
        } else {
            if (next_step < nsteps) fetch_a(next_step);
        }
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            if (q + 1 < 4) {
                read_frags(q + 1, fr[(q + 1) & 1]);
                if (kBViaLds) read_frags_b(q + 1, frb[(q + 1) & 1]);
            }
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const int x = q * 4 + j;
                half8_t fb[WN], fa[MT];
#pragma unroll
                for (int t = 0; t < WN; ++t)
                    fb[t] = dequant8(word_of(kBViaLds ? frb[q & 1][t] : b[t][q], j), scale_of(s.sb[t][x >> 3], x));
#pragma unroll
                for (int i = 0; i < MT; ++i) fa[i] = dequant8(word_of(fr[q & 1][i], j), scale_of(s.sa[x >> 3][i], x));
#pragma unroll
                for (int i = 0; i < MT; ++i)
#pragma unroll
                    for (int t = 0; t < WN; ++t)
                        acc[i][t] = __builtin_amdgcn_mfma_f32_32x32x16_f16(fb[t], fa[i], acc[i][t], 0, 0, 0);
            }
        }
        // the next step's LDS writes must not pass this step's reads
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
        __builtin_amdgcn_wave_barrier();
    };

    // read now, used in the epilogue: short launches would otherwise end on this latency
    const float alpha = OUT == kOutPartial ? 0.0f : load_alpha(p);

    SkinnyRegs<MT, WN> st[2];
    int64_t step = wave;  // counts this workgroup's steps, see phys()
    if constexpr (kBViaLds) {
        // a register set of codes is refilled for the step kBSets steps after the one it held
        constexpr int kAhead = (kBSets - 1) * kWaves;
        fetch_a(step);
        fetch_b_codes(step, bst[0]);
        fetch_scales(step, st[0]);
        if (kBSets == 2) fetch_b_codes(step + kWaves, bst[kBSets - 1]);
        fetch_scales(step + kWaves, st[1]);
        for (; step + kWaves < nsteps; step += 2 * kWaves) {
            compute(st[0], bst[0], step + kWaves, step + kWaves + kAhead);
            fetch_scales(step + 2 * kWaves, st[0]);
            compute(st[1], bst[kBSets - 1], step + 2 * kWaves, step + 2 * kWaves + kAhead);
            fetch_scales(step + 3 * kWaves, st[1]);
        }
        if (step < nsteps) compute(st[0], bst[0], nsteps, nsteps);  // odd count: the last step, nothing left to fetch
    } else {
        // 256 registers are in use here: the loads stay under branches, which costs the exact
        // wait counts but keeps the accumulators out of scratch memory
        auto fetch_b = [&](int64_t j, int set) {
            fetch_b_codes(j, bst[set]);
            fetch_scales(j, st[set]);
        };
        if (step < nsteps) {
            fetch_a(step);
            fetch_b(step, 0);
        }
        if (step + kWaves < nsteps) fetch_b(step + kWaves, 1);
        for (; step < nsteps; step += 2 * kWaves) {
            compute(st[0], bst[0], step + kWaves, 0);
            if (step + 2 * kWaves < nsteps) fetch_b(step + 2 * kWaves, 0);
            if (step + kWaves < nsteps) {
                compute(st[1], bst[kBSets - 1], step + 2 * kWaves, 0);
                if (step + 3 * kWaves < nsteps) fetch_b(step + 3 * kWaves, 1);
            }
        }
    }

    // Reduction of the wavefronts' accumulators, scattered: every wavefront writes all of its
    // registers to its LDS slot, then wavefront w sums registers [w R, (w + 1) R) of all slots in
    // slot order (fixed, hence deterministic) and stores that share of the output, so the
    // conversion and the stores are spread over the workgroup as well.  Register f = (i WN + t) 16 + e
    // of a lane sits at float (slot (kAcc / 4) + f / 4) 256 + 4 lane + f % 4: 128-bit accesses,
    // consecutive lanes 16 bytes apart.  The slots overlay the staging regions, so every wavefront
    // must have left the main loop.
    constexpr int R = kAcc / kWaves;  // 2 (MT = 1), 4, 8, 16 or 32
    static_assert(R == 2 || R % 4 == 0, "whole groups of four columns, or half of one");
    __syncthreads();
    float *red = reinterpret_cast<float *>(smem);
#pragma unroll
    for (int i = 0; i < MT; ++i)
#pragma unroll
        for (int t = 0; t < WN; ++t)
#pragma unroll
            for (int g = 0; g < 4; ++g)
                *reinterpret_cast<float4 *>(red + ((wave * (kAcc / 4) + (i * WN + t) * 4 + g) * 64 + lane) * 4) =
                    make_float4(acc[i][t][4 * g], acc[i][t][4 * g + 1], acc[i][t][4 * g + 2], acc[i][t][4 * g + 3]);
    __syncthreads();
    float mine[R];
#pragma unroll
    for (int k = 0; k < R; ++k) mine[k] = 0.0f;
#pragma unroll
    for (int v = 0; v < kWaves; ++v) {
        const float *slot = red + (v * (kAcc / 4) * 64 + lane) * 4 + (R == 2 ? (wave >> 1) * 256 + (wave & 1) * 2 : wave * (R / 4) * 256);
        if constexpr (R == 2) {
            const float2 x = *reinterpret_cast<const float2 *>(slot);
            mine[0] += x.x, mine[1] += x.y;
        } else {
#pragma unroll
            for (int c = 0; c < R / 4; ++c) {
                const float4 x = *reinterpret_cast<const float4 *>(slot + c * 256);
                mine[4 * c] += x.x, mine[4 * c + 1] += x.y, mine[4 * c + 2] += x.z, mine[4 * c + 3] += x.w;
            }
        }
    }

    // Register f is D[m][n], m = m_base + 32 i + r, n = n128 + 32 g + r0 + 8 t + 4 h + e % 4 (tile row 8 g + 4 h + e % 4),
    // g = (f % 16) / 4; rows m >= M are padding of the band and are not written.  This wavefront's
    // registers are groups of four columns c4 = w R / 4 ... (or, for R = 2, half of group w / 2).
    constexpr int kGroups = R == 2 ? 1 : R / 4;
    float *P = OUT == kOutPartial ? p.partials + (int64_t)blockIdx.y * p.M * p.N : nullptr;
    uint16_t *D = reinterpret_cast<uint16_t *>(p.D);
    uint32_t umax = 0u;
#pragma unroll
    for (int c = 0; c < kGroups; ++c) {
        const int c4 = R == 2 ? (wave >> 1) : wave * (R / 4) + c;  // group of four columns: c4 = (i WN + t) 4 + g
        const int g = c4 & 3, t = (c4 >> 2) % WN, i = (c4 >> 2) / WN;
        const int m = m_base + 32 * i + r;
        if (m >= p.M) continue;
        const int64_t n = n128 + 32 * g + r0 + 8 * t + 4 * h + (R == 2 ? (wave & 1) * 2 : 0);
        if constexpr (R == 2) {
            if (OUT == kOutPartial) {
                *reinterpret_cast<float2 *>(P + (int64_t)m * p.N + n) = make_float2(mine[0], mine[1]);
            } else {
                *reinterpret_cast<uint32_t *>(D + (int64_t)m * p.ldd + n) =
                    pack_outputs2<OUT == kOutBF16>(alpha * mine[0], alpha * mine[1], p.bias, n, umax);
            }
        } else {
            if (OUT == kOutPartial) {
                *reinterpret_cast<float4 *>(P + (int64_t)m * p.N + n) = make_float4(mine[4 * c], mine[4 * c + 1], mine[4 * c + 2], mine[4 * c + 3]);
            } else {
                const float v[4] = {alpha * mine[4 * c], alpha * mine[4 * c + 1], alpha * mine[4 * c + 2], alpha * mine[4 * c + 3]};
                *reinterpret_cast<uint2 *>(D + (int64_t)m * p.ldd + n) = pack_outputs<OUT == kOutBF16>(v, p.bias, n, umax);
            }
        }
    }
    if (OUT != kOutPartial && p.d_amax) fold_amax<OUT == kOutBF16>(p.d_amax, umax);
}

// ---------------------------------------------------------------------------------------
// M <= 16 (decode batches).  Same decomposition as the weight-streaming kernel above (32 rows
// of B per workgroup, 8 wavefronts share the K steps of 256, staggered start, tree reduction),
// built on the 16 x 16 x 32 MFMA: a 32 x 32 tile would spend half of its rows, and half of
// the activation conversions, on padding.
//
// A workgroup owns the rows n128 + 32 q + r0 + i (q = 0..3, i = 0..7) of one 128-row band,
// r0 = 8 (blockIdx.x % 4): in the tiled scale layout the four rows r, r + 32, r + 64, r + 96
// share a 16-byte unit, so the scales of these 32 rows are 128 contiguous bytes per K group
// -- whole cache lines, one 64-bit load per lane -- where 32 consecutive rows would use 4
// bytes of each of 32 units.
//
// Lane l = (c = l & 15, g = l >> 4).  Per step it holds the 64 codes k = 256 step + 64 g ...
// of B rows n128 + 32 (2 (c >> 3) + b) + r0 + (c & 7), b = 0, 1, and of A row c: 32 contiguous
// bytes each, whose four blocks are exactly one scale group (one 32-bit word of the tiled
// layout).  MFMA slice s = 0..7 multiplies 32-bit word s of every lane, i.e. the contraction
// index is permuted (slice s pairs codes 8 s ... 8 s + 7 of all four lane groups), identically
// for both operands.  Operands go from global memory to registers to the MFMA: no LDS in the
// loop.  acc[b][e] is D[m = c][n = n128 + 32 (2 (g >> 1) + b) + r0 + 4 (g & 1) + e].
//
// NB = 1 halves the workgroup to 16 rows (n128 + 32 q + r0 + i, i = 0..3, r0 = 4 (blockIdx.x % 8);
// lane row c: q = c >> 2, i = c & 3): twice the workgroups for narrow outputs (N <= 4096), which
// would otherwise split K and pay a reduction kernel.  acc[0][e] is then D[c][n128 + 32 g + r0 + e].
template <int NB>
struct DecodeRegs {
    uint4 b[NB][2];   // 64 codes of NB rows of B
    uint4 a[2];       // 64 codes of the A row
    uint32_t sb[NB];  // their scale groups (NB = 2: adjacent words of one 16-byte unit)
    uint32_t sa;
};

template <int NB, int OUT>
__global__ __launch_bounds__(512) void gemm_nvfp4_decode_kernel(const GemmParams p) {
    constexpr int kWaves = 8, kDepth = 3;
    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
    const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), c = lane & 15, g = lane >> 4;
    const int64_t n128 = (int64_t)(blockIdx.x >> (NB == 2 ? 2 : 3)) * 128;
    const int r0 = NB == 2 ? (int)(blockIdx.x & 3) * 8 : (int)(blockIdx.x & 7) * 4;
    const int64_t kbytes = p.K >> 1, sf_groups = p.K >> 6;
    const int64_t steps_all = p.K >> 8;
    const int64_t s_begin = OUT == kOutPartial ? (int64_t)blockIdx.y * p.ksteps_per_split : 0;
    const int64_t s_end = OUT == kOutPartial ? (s_begin + p.ksteps_per_split < steps_all ? s_begin + p.ksteps_per_split : steps_all)
                                             : steps_all;
    // staggered start, as in the weight-streaming kernel
    const int64_t nsteps = s_end - s_begin;
    const int64_t rot_wg = nsteps > 0 ? ((int64_t)blockIdx.x * kSkinnyRotation) % nsteps : 0;
    auto phys = [&](int64_t j) -> int64_t {
        const int64_t q = j + rot_wg;
        return s_begin + (q >= nsteps ? q - nsteps : q);
    };

    // rows of A past M read as zero codes (buffer range check); loads past the last step go
    // through the empty descriptor, so that none of them sits under a branch
    const BufferRsrc ra = make_rsrc(p.A, (uint32_t)(p.M * kbytes));
    const BufferRsrc rb = make_rsrc(p.B + n128 * kbytes, (uint32_t)(128 * kbytes));
    const BufferRsrc rsa = make_rsrc(p.sfA, (uint32_t)(sf_groups * 512));
    const BufferRsrc rsb = make_rsrc(p.sfB + (n128 >> 7) * sf_groups * 512, (uint32_t)(sf_groups * 512));
    const BufferRsrc r_none = make_rsrc(p.A, 0);
    const uint32_t qa_off = (uint32_t)(c * kbytes + g * 32);
    const uint32_t qb_off = NB == 2 ? (uint32_t)((64 * (c >> 3) + r0 + (c & 7)) * kbytes + g * 32)  // b = 1: 32 rows further
                                    : (uint32_t)((32 * (c >> 2) + r0 + (c & 3)) * kbytes + g * 32);
    const uint32_t sa_off = (uint32_t)(g * 512 + c * 16);
    const uint32_t sb_off = NB == 2 ? (uint32_t)(g * 512 + (r0 + (c & 7)) * 16 + (c >> 3) * 8)
                                    : (uint32_t)(g * 512 + (r0 + (c & 3)) * 16 + (c >> 2) * 4);

    auto fetch = [&](int64_t j, DecodeRegs<NB> &s) {
        const bool ok = j < nsteps;
        const BufferRsrc qa = ok ? ra : r_none, qb = ok ? rb : r_none, fa = ok ? rsa : r_none, fb = ok ? rsb : r_none;
        const int kq = ok ? (int)(phys(j) * 128) : 0, ksf = ok ? (int)(phys(j) * 2048) : 0;
#pragma unroll
        for (int b = 0; b < NB; ++b)
#pragma unroll
            for (int u = 0; u < 2; ++u)
                s.b[b][u] = __builtin_bit_cast(uint4, __builtin_amdgcn_raw_buffer_load_b128(qb, (int)(qb_off + b * 32 * kbytes + u * 16), kq, 0));
#pragma unroll
        for (int u = 0; u < 2; ++u)
            s.a[u] = __builtin_bit_cast(uint4, __builtin_amdgcn_raw_buffer_load_b128(qa, (int)(qa_off + u * 16), kq, 0));
        load_words<NB>(s.sb, fb, (int)sb_off, ksf);
        s.sa = __builtin_amdgcn_raw_buffer_load_b32(fa, (int)sa_off, ksf, 0);
    };

    float4_t acc[NB];
#pragma unroll
    for (int b = 0; b < NB; ++b) acc[b] = float4_t{0.0f, 0.0f, 0.0f, 0.0f};
    auto word_of = [](const uint4 &v, int j) -> uint32_t { return j == 0 ? v.x : j == 1 ? v.y : j == 2 ? v.z : v.w; };
    // scale of code word x (0..7) of a lane: block x >> 1 = byte x >> 1 of the group word
    auto scale_of = [](uint32_t w, int x) -> half2_t {
        const half2_t s2 = e4m3x2_to_half2((x & 4) ? w >> 16 : w);
        return ((x >> 1) & 1) ? __builtin_shufflevector(s2, s2, 1, 1) : __builtin_shufflevector(s2, s2, 0, 0);
    };
    auto compute = [&](const DecodeRegs<NB> &s) {
#pragma unroll
        for (int x = 0; x < 8; ++x) {
            const half8_t fa = dequant8(word_of(s.a[x >> 2], x & 3), scale_of(s.sa, x));
#pragma unroll
            for (int b = 0; b < NB; ++b) {
                const half8_t fb = dequant8(word_of(s.b[b][x >> 2], x & 3), scale_of(s.sb[b], x));
                acc[b] = __builtin_amdgcn_mfma_f32_16x16x32_f16(fb, fa, acc[b], 0, 0, 0);
            }
        }
    };

    // read now, used in the epilogue: short launches would otherwise end on this latency
    const float alpha = OUT == kOutPartial ? 0.0f : load_alpha(p);

    DecodeRegs<NB> st[kDepth];
    int64_t step = wave;  // counts this workgroup's steps, see phys()
#pragma unroll
    for (int d = 0; d < kDepth; ++d) fetch(step + d * kWaves, st[d]);
    for (; step + (kDepth - 1) * kWaves < nsteps; step += kDepth * kWaves) {
#pragma unroll
        for (int d = 0; d < kDepth; ++d) {
            compute(st[d]);
            // the refill goes out here: the scheduler may not collect the loads at the loop's end
            __builtin_amdgcn_sched_barrier(0);
            fetch(step + (d + kDepth) * kWaves, st[d]);
            __builtin_amdgcn_sched_barrier(0);
        }
    }
#pragma unroll
    for (int d = 0; d + 1 < kDepth; ++d)
        if (step + d * kWaves < nsteps) compute(st[d]);  // the last, incomplete round

    // tree reduction of the 8 wavefronts' accumulators (fixed order, hence deterministic)
    float *red = reinterpret_cast<float *>(smem);
#pragma unroll
    for (int stride = kWaves / 2; stride >= 1; stride >>= 1) {
        if (wave >= stride && wave < 2 * stride) {
            float *slot = red + (wave - stride) * (4 * NB * 64);
#pragma unroll
            for (int b = 0; b < NB; ++b)
#pragma unroll
                for (int e = 0; e < 4; ++e) slot[(b * 4 + e) * 64 + lane] = acc[b][e];
        }
        __syncthreads();
        if (wave < stride) {
            const float *slot = red + wave * (4 * NB * 64);
#pragma unroll
            for (int b = 0; b < NB; ++b)
#pragma unroll
                for (int e = 0; e < 4; ++e) acc[b][e] += slot[(b * 4 + e) * 64 + lane];
        }
        __syncthreads();
    }
    if (wave != 0) return;
    const bool row_ok = c < p.M;  // rows beyond M are padding of the band and are not written

    const int64_t n_out = NB == 2 ? n128 + 64 * (g >> 1) + r0 + 4 * (g & 1)  // column of acc[0][0]; acc[1] is 32 further
                                  : n128 + 32 * g + r0;
    if (OUT == kOutPartial) {
        float *P = p.partials + (int64_t)blockIdx.y * p.M * p.N;
        if (row_ok) {
#pragma unroll
            for (int b = 0; b < NB; ++b)
                *reinterpret_cast<float4 *>(P + (int64_t)c * p.N + n_out + 32 * b) = make_float4(acc[b][0], acc[b][1], acc[b][2], acc[b][3]);
        }
        return;
    }
    uint16_t *D = reinterpret_cast<uint16_t *>(p.D);
    uint32_t umax = 0u;
#pragma unroll
    for (int b = 0; b < NB; ++b) {
        const float v[4] = {alpha * acc[b][0], alpha * acc[b][1], alpha * acc[b][2], alpha * acc[b][3]};
        uint32_t um = 0u;
        const uint2 o = pack_outputs<OUT == kOutBF16>(v, p.bias, n_out + 32 * b, um);
        if (row_ok) {
            umax = um > umax ? um : umax;
            *reinterpret_cast<uint2 *>(D + (int64_t)c * p.ldd + n_out + 32 * b) = o;
        }
    }
    if (p.d_amax) fold_amax<OUT == kOutBF16>(p.d_amax, umax);
}

// D = alpha * (sum of the split-K partial tiles, in split order), 4 consecutive n per thread.
template <bool OUT_BF16>
__global__ __launch_bounds__(256) void gemm_reduce_kernel(const GemmParams p) {
    const int64_t quads = p.M * (p.N >> 2);
    const int64_t t_raw = (int64_t)blockIdx.x * 256 + threadIdx.x;
    const bool mine = t_raw < quads;
    const int64_t t = mine ? t_raw : 0;  // (idle lanes redo quad 0 and store nothing: every lane reaches fold_amax)
    const int64_t m = t / (p.N >> 2), n = (t - m * (p.N >> 2)) << 2;
    const float4 *P = reinterpret_cast<const float4 *>(p.partials + m * p.N + n);
    const int64_t stride = (p.M * p.N) >> 2;
    float4 s = P[0];
    for (int y = 1; y < p.splits; ++y) {
        const float4 v = P[y * stride];
        s.x += v.x; s.y += v.y; s.z += v.z; s.w += v.w;
    }
    const float alpha = load_alpha(p);
    const float v[4] = {alpha * s.x, alpha * s.y, alpha * s.z, alpha * s.w};
    uint32_t um = 0u;
    const uint2 o = pack_outputs<OUT_BF16>(v, p.bias, n, um);
    if (mine) *reinterpret_cast<uint2 *>(reinterpret_cast<uint16_t *>(p.D) + m * p.ldd + n) = o;
    if (p.d_amax) fold_amax<OUT_BF16>(p.d_amax, mine ? um : 0u);
}

template <int WAVES_M, int WAVES_N, int WM, int WN, bool QUARTER = false>
static int launch_gemm(GemmParams &p, int out_type, hipStream_t s) {
    constexpr int BM = WAVES_M * WM * 32, BN = WAVES_N * WN * 32;
    constexpr int kThreadsG = 64 * WAVES_M * WAVES_N;
    constexpr size_t lds_bytes = 2 * (size_t)BM * kPitch * sizeof(_Float16);  // two buffers of A
    p.tiles_m = (int)(p.M / BM);
    p.tiles_n = (int)(p.N / BN);
    dim3 grid((unsigned)(p.tiles_m * p.tiles_n), (unsigned)p.splits);
    auto kbf = gemm_nvfp4_kernel<WAVES_M, WAVES_N, WM, WN, kOutBF16, QUARTER>;
    auto kh = gemm_nvfp4_kernel<WAVES_M, WAVES_N, WM, WN, kOutF16, QUARTER>;
    auto kp = gemm_nvfp4_kernel<WAVES_M, WAVES_N, WM, WN, kOutPartial, QUARTER>;
    auto kernel = p.splits > 1 ? kp : out_type == FOS_T_BF16 ? kbf : kh;
    if (lds_bytes > 64 * 1024) {
        // more than the default dynamic LDS limit: opt in (idempotent, no device state besides the function attribute)
        if (hipFuncSetAttribute((const void *)kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_bytes) != hipSuccess)
            return FOS_E_LAUNCH;
    }
    hipLaunchKernelGGL(kernel, grid, dim3(kThreadsG), lds_bytes, s, p);
    if (hipGetLastError() != hipSuccess) return FOS_E_LAUNCH;
    if (p.splits > 1) {
        const int64_t quads = p.M * (p.N >> 2);
        dim3 rgrid((unsigned)((quads + 255) / 256));
        if (out_type == FOS_T_BF16) hipLaunchKernelGGL(gemm_reduce_kernel<true>, rgrid, dim3(256), 0, s, p);
        else hipLaunchKernelGGL(gemm_reduce_kernel<false>, rgrid, dim3(256), 0, s, p);
    }
    return hipGetLastError() == hipSuccess ? FOS_OK : FOS_E_LAUNCH;
}

template <int MT, int WN>
static int launch_skinny(GemmParams &p, int out_type, hipStream_t s, int row_groups = 1) {
    constexpr int kWaves = skinny_waves(WN);
    constexpr size_t stage_bytes = (size_t)kWaves * (MT * 32 + (MT <= 2 || WN == 2 ? WN * 32 : 0)) * kSkinnyPitch,
                     red_bytes = (size_t)kWaves * (MT * WN * 16) * 64 * sizeof(float);
    constexpr size_t lds_bytes = stage_bytes > red_bytes ? stage_bytes : red_bytes;
    dim3 grid((unsigned)(p.N / (32 * WN)), (unsigned)p.splits, (unsigned)row_groups);
    auto kernel = p.splits > 1 ? gemm_nvfp4_skinny_kernel<MT, WN, kOutPartial>
                  : out_type == FOS_T_BF16 ? gemm_nvfp4_skinny_kernel<MT, WN, kOutBF16> : gemm_nvfp4_skinny_kernel<MT, WN, kOutF16>;
    if (lds_bytes > 64 * 1024 &&
        hipFuncSetAttribute((const void *)kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_bytes) != hipSuccess)
        return FOS_E_LAUNCH;
    hipLaunchKernelGGL(kernel, grid, dim3(64 * kWaves), lds_bytes, s, p);
    if (hipGetLastError() != hipSuccess) return FOS_E_LAUNCH;
    if (p.splits > 1) {
        const int64_t quads = p.M * (p.N >> 2);
        dim3 rgrid((unsigned)((quads + 255) / 256));
        if (out_type == FOS_T_BF16) hipLaunchKernelGGL(gemm_reduce_kernel<true>, rgrid, dim3(256), 0, s, p);
        else hipLaunchKernelGGL(gemm_reduce_kernel<false>, rgrid, dim3(256), 0, s, p);
    }
    return hipGetLastError() == hipSuccess ? FOS_OK : FOS_E_LAUNCH;
}

template <int NB>
static int launch_decode(GemmParams &p, int out_type, hipStream_t s) {
    constexpr size_t lds_bytes = (size_t)4 * (4 * NB) * 64 * sizeof(float);
    dim3 grid((unsigned)(p.N / (16 * NB)), (unsigned)p.splits);
    auto kernel = p.splits > 1 ? gemm_nvfp4_decode_kernel<NB, kOutPartial>
                  : out_type == FOS_T_BF16 ? gemm_nvfp4_decode_kernel<NB, kOutBF16> : gemm_nvfp4_decode_kernel<NB, kOutF16>;
    hipLaunchKernelGGL(kernel, grid, dim3(512), lds_bytes, s, p);
    if (hipGetLastError() != hipSuccess) return FOS_E_LAUNCH;
    if (p.splits > 1) {
        const int64_t quads = p.M * (p.N >> 2);
        dim3 rgrid((unsigned)((quads + 255) / 256));
        if (out_type == FOS_T_BF16) hipLaunchKernelGGL(gemm_reduce_kernel<true>, rgrid, dim3(256), 0, s, p);
        else hipLaunchKernelGGL(gemm_reduce_kernel<false>, rgrid, dim3(256), 0, s, p);
    }
    return hipGetLastError() == hipSuccess ? FOS_OK : FOS_E_LAUNCH;
}

// Which kernel runs a shape, and how K is split across workgroups (splits > 1 needs the
// caller's workspace for splits * M * N FP32 partials).
enum { kPlanBig, kPlanWide, kPlanSmall, kPlanSkinny };
struct GemmPlan {
    int kind, splits, ksteps_per_split;
    int narrow;  // M <= 16: workgroups of 16 instead of 32 rows of B
    int wide;    // M > 32: workgroups of 64 rows of B and 64 rows of A, four wavefronts with two by two tiles each
};
constexpr int kTargetWorkgroups = 256;
static GemmPlan plan_gemm(int64_t M, int64_t N, int64_t K) {
    GemmPlan g;
    g.narrow = g.wide = 0;
    const int tile = tuning().gemm_tile;  // tuning / tests: 128 = small tile, 129 = 128 x 256 tile and 256 = 256 x 256 tile wherever M and N allow, 1 = no weight-streaming kernel
    int64_t steps, tiles;
    if (M <= 128 && K % 256 == 0 && (tile == 0 || tile == 16 || tile == 32 || tile == 64)) {
        // one 128-row band: weight streaming, steps of 256 along K shared by 8 wavefronts
        g.kind = kPlanSkinny;
        steps = K / 256;
        tiles = N / 32;
        if (M <= 16 && tiles <= kTargetWorkgroups / 2 && (tile == 16 || (tile == 0 && steps >= 16))) {
            // narrow outputs on the 16-row kernel: 16 rows of B per workgroup give twice the
            // workgroups, instead of a split of K and its reduction kernel
            g.narrow = 1;
            tiles = N / 16;
        }
        if (M > 32 && (tile == 64 || (tile == 0 && (M > 64 || tiles > kTargetWorkgroups)))) {
            // 64 rows of B per workgroup of four wavefronts, two workgroups per compute unit, and
            // workgroups of their own for rows 64 ... of A: half the reads of A per multiplication.
            // At M <= 64 it pays once the 32-row workgroups no longer run all at once (N = 14336,
            // K = 4096: 22.4 -> 13.9 us at M = 64; N = 8192: 11.3 against 14.3 us)
            g.wide = 1;
            tiles = (N / 64) * (M > 64 ? 2 : 1);
        }
    } else if ((M % 256 == 0) && (N % 256 == 0) && ((M / 256) * (N / 256) >= 256 || tile == 256) && tile != 128) {
        // 256 x 256 tiles once they give each of the 256 compute units a workgroup
        g.kind = kPlanBig;
        g.splits = 1;
        g.ksteps_per_split = (int)(K / BK);
        return g;
    } else if (tile != 128 && M % 128 == 0 && N % 256 == 0 && M >= 128 &&
               (tile == 129 || ((M / 128) * (N / 256) > 128 && (M / 128) * (N / 256) <= 256))) {
        // 128 x 256 tiles (eight wavefronts of 128 x 32; every thread stages a quarter row of A) where they give
        // every compute unit at most one workgroup and more than half of them one: A is converted
        // once per 256 columns instead of once per 128.  Against the 128 x 128 tile, alternating
        // runs: 2048 x 4096 x 4096 71.9 -> 69.3 us, 2048 x 4096 x 14336 242.5 -> 228 us,
        // 1792 x 4096 x 4096 67.0 -> 64.6 us; with 1.5 workgroups per compute unit
        // (3072 x 4096 x 4096) 109 -> 123 us, with half a one (1024 x 4096 x 4096) 41.7 -> 51.8 us.
        g.kind = kPlanWide;
        g.splits = 1;
        g.ksteps_per_split = (int)(K / BK);
        return g;
    } else {
        g.kind = kPlanSmall;
        steps = K / BK;
        tiles = ((M + 127) / 128) * (N / 128);
    }
    // split so that about kTargetWorkgroups workgroups run, each with a useful share of K
    // (at M <= 32 a split must leave two steps per wavefront: 16 x 4096 x 4096 takes 6.4 us
    // unsplit and 7.1 us in two halves plus their reduction)
    // (with row groups, M > 64: 128 x 4096 x 4096 takes 12.3 us unsplit, 13.4 us in two halves)
    const int64_t min_steps = g.kind == kPlanSkinny ? (M <= 32 || (g.wide && M > 64) ? 16 : 8) : 4;
    // (the weight-streaming kernel also splits in two when its workgroups would cover exactly
    // half of the compute units: measured 18.8 -> 15.1 us at M = 16, N = 4096, K = 14336)
    const int64_t enough = g.kind == kPlanSkinny ? kTargetWorkgroups / 2 + 1 : kTargetWorkgroups / 2;
    int64_t want = tiles >= enough ? 1 : (kTargetWorkgroups + tiles - 1) / tiles;
    if (want > steps / min_steps) want = steps / min_steps;
    if (const int forced_splits = tuning().gemm_splitk) want = forced_splits;  // tuning / tests
    if (want > steps) want = steps;
    if (want > 32) want = 32;
    if (want < 1) want = 1;
    g.ksteps_per_split = (int)((steps + want - 1) / want);
    g.splits = (int)((steps + g.ksteps_per_split - 1) / g.ksteps_per_split);
    return g;
}

}  // namespace fos

using namespace fos;

namespace fos {
// tensor / python-scalar on a GPU is, in torch, a multiplication by the reciprocal, which is
// formed once on the host in double precision and rounded to fp32 (measured against
// torch on the device); the reference's alpha is formed that way
__global__ void gemm_alpha_kernel(const float *amax_a, const float *amax_b, float inv_den, float *alpha) {
    *alpha = (*amax_a * *amax_b) * inv_den;
}
}  // namespace fos

extern "C" int fos_gemm_alpha(const float *amax_a, const float *amax_b, double denominator, float *alpha,
                              fos_stream_t stream) {
    if (!amax_a || !amax_b || !alpha) return FOS_E_NULL_POINTER;
    hipLaunchKernelGGL(gemm_alpha_kernel, dim3(1), dim3(1), 0, (hipStream_t)stream, amax_a, amax_b, (float)(1.0 / denominator), alpha);
    return hipGetLastError() == hipSuccess ? FOS_OK : FOS_E_LAUNCH;
}

extern "C" size_t fos_gemm_workspace_bytes(int64_t M, int64_t N, int64_t K) {
    if (M <= 0 || N <= 0 || K <= 0 || (M > 128 && M % 128 != 0) || (M < 128 && K % 256 != 0) || N % 128 != 0 || K % 64 != 0)
        return 0;
    const GemmPlan g = plan_gemm(M, N, K);
    return g.splits > 1 ? (size_t)g.splits * (size_t)M * (size_t)N * sizeof(float) : 0;
}

static int gemm_nvfp4_impl(const uint8_t *A, const uint8_t *B, const uint8_t *sfA, const uint8_t *sfB,
                           const float *alpha, const float *amax_a, const float *amax_b, double denominator,
                           int64_t M, int64_t N, int64_t K, void *D, int out_type, int64_t ldd, const void *bias, float *d_amax,
                           void *workspace, size_t workspace_bytes, fos_stream_t stream) {
    if (!A || !B || !sfA || !sfB || !D) return FOS_E_NULL_POINTER;
    if (((uintptr_t)d_amax & 3) || ((uintptr_t)bias & 7)) return FOS_E_BAD_ALIGNMENT;
    if (!alpha && (!amax_a || !amax_b)) return FOS_E_NULL_POINTER;
    if (!alpha && (((uintptr_t)amax_a & 3) || ((uintptr_t)amax_b & 3))) return FOS_E_BAD_ALIGNMENT;
    if (M <= 0 || N <= 0 || K <= 0 || (M > 128 && M % 128 != 0) || N % 128 != 0 || K % 64 != 0 || ldd < N) return FOS_E_BAD_SHAPE;
    if (M < 128 && K % 256 != 0) return FOS_E_BAD_SHAPE;  // partial bands only through the weight-streaming kernel
    if (out_type != FOS_T_BF16 && out_type != FOS_T_F16) return FOS_E_UNSUPPORTED;
    if (((uintptr_t)A & 15) || ((uintptr_t)B & 15) || ((uintptr_t)sfA & 15) || ((uintptr_t)sfB & 15) ||
        ((uintptr_t)D & 7) || (ldd % 4 != 0) || ((uintptr_t)alpha & 3))
        return FOS_E_BAD_ALIGNMENT;
    if ((M / 128) * (N / 128) > 0x7fffffffLL || K > (1LL << 22)) return FOS_E_BAD_SHAPE;  // a 256-row panel of packed codes stays below 2^31 bytes (32-bit buffer offsets)
    GemmParams p;
    p.A = A; p.B = B; p.sfA = sfA; p.sfB = sfB; p.alpha = alpha; p.D = D; p.bias = bias; p.d_amax = d_amax;
    p.amax_a = amax_a; p.amax_b = amax_b; p.inv_den = alpha ? 0.0f : (float)(1.0 / denominator);
    p.M = M; p.N = N; p.K = K; p.ldd = ldd;
    hipStream_t s = (hipStream_t)stream;
    GemmPlan g = plan_gemm(M, N, K);
    if (M < 128 && g.kind != kPlanSkinny) return FOS_E_BAD_SHAPE;
    // the tile kernels store whole rows of their output tiles, 16 bytes per lane
    if (g.kind != kPlanSkinny && (((uintptr_t)D & 15) || (ldd % 8 != 0))) return FOS_E_BAD_ALIGNMENT;  // partial bands only through the weight-streaming kernel
    if (g.splits > 1 && !(workspace && !((uintptr_t)workspace & 15) &&
                          workspace_bytes >= (size_t)g.splits * (size_t)M * (size_t)N * sizeof(float))) {
        // no (or too small a) workspace: run unsplit
        g.splits = 1;
        g.ksteps_per_split = (int)(K / (g.kind == kPlanSkinny ? 256 : BK));
    }
    p.partials = g.splits > 1 ? static_cast<float *>(workspace) : nullptr;
    p.splits = g.splits;
    p.ksteps_per_split = g.ksteps_per_split;
    switch (g.kind) {
        case kPlanBig: return launch_gemm<1, 8, 8, 1>(p, out_type, s);
        // (quarter rows of A per thread: with half rows the first four wavefronts carried all of A's conversion; alternating
        // series on one box, 2048 x 4096 x 4096 66.6-72.0 against 67.6-75.7 us, 1792 x 4096 x 4096 62.0-68.3 against 63.6-71.7)
        case kPlanWide: return launch_gemm<1, 8, 4, 1, true>(p, out_type, s);
        case kPlanSkinny:
            // the 16-row kernel pays off from two K steps per wavefront on (measured at N = 14336:
            // K = 2048 7.6 us against 6.3 us with 32-row tiles, K = 4096 10.6 against 12.3);
            // FOS_GEMM_TILE = 16 / 32 forces / forbids it (tuning, tests)
            if (M <= 16) {
                const int forced = tuning().gemm_tile;
                if (forced == 16 || (forced != 32 && g.ksteps_per_split >= 16))
                    return g.narrow ? launch_decode<1>(p, out_type, s) : launch_decode<2>(p, out_type, s);
            }
            if (M <= 32) return launch_skinny<1, 1>(p, out_type, s);
            if (M <= 64) return g.wide ? launch_skinny<2, 2>(p, out_type, s) : launch_skinny<2, 1>(p, out_type, s);
            return g.wide ? launch_skinny<2, 2>(p, out_type, s, 2) : launch_skinny<4, 1>(p, out_type, s);
        default: return launch_gemm<1, 4, 4, 1>(p, out_type, s);
    }
}

extern "C" int fos_gemm_nvfp4(const uint8_t *A, const uint8_t *B, const uint8_t *sfA, const uint8_t *sfB,
                              const float *alpha, int64_t M, int64_t N, int64_t K,
                              void *D, int out_type, int64_t ldd,
                              void *workspace, size_t workspace_bytes, fos_stream_t stream) {
    if (!alpha) return FOS_E_NULL_POINTER;
    return gemm_nvfp4_impl(A, B, sfA, sfB, alpha, nullptr, nullptr, 1.0, M, N, K, D, out_type, ldd, nullptr, nullptr, workspace,
                           workspace_bytes, stream);
}

extern "C" int fos_gemm_nvfp4_amax(const uint8_t *A, const uint8_t *B, const uint8_t *sfA, const uint8_t *sfB,
                                   const float *amax_a, const float *amax_b, double denominator,
                                   int64_t M, int64_t N, int64_t K, void *D, int out_type, int64_t ldd,
                                   void *workspace, size_t workspace_bytes, fos_stream_t stream) {
    if (!amax_a || !amax_b) return FOS_E_NULL_POINTER;
    if (!(denominator > 0.0)) return FOS_E_BAD_SHAPE;
    return gemm_nvfp4_impl(A, B, sfA, sfB, nullptr, amax_a, amax_b, denominator, M, N, K, D, out_type, ldd, nullptr, nullptr, workspace,
                           workspace_bytes, stream);
}

extern "C" int fos_gemm_nvfp4_amax_out(const uint8_t *A, const uint8_t *B, const uint8_t *sfA, const uint8_t *sfB,
                                       const float *amax_a, const float *amax_b, double denominator,
                                       int64_t M, int64_t N, int64_t K, void *D, int out_type, int64_t ldd, float *d_amax,
                                       void *workspace, size_t workspace_bytes, fos_stream_t stream) {
    if (!amax_a || !amax_b || !d_amax) return FOS_E_NULL_POINTER;
    if (!(denominator > 0.0)) return FOS_E_BAD_SHAPE;
    return gemm_nvfp4_impl(A, B, sfA, sfB, nullptr, amax_a, amax_b, denominator, M, N, K, D, out_type, ldd, nullptr, d_amax, workspace,
                           workspace_bytes, stream);
}

extern "C" int fos_gemm_nvfp4_linear(const uint8_t *A, const uint8_t *B, const uint8_t *sfA, const uint8_t *sfB,
                                     const float *amax_a, const float *amax_b, double denominator,
                                     int64_t M, int64_t N, int64_t K, void *D, int out_type, int64_t ldd, const void *bias,
                                     float *d_amax, void *workspace, size_t workspace_bytes, fos_stream_t stream) {
    if (!amax_a || !amax_b) return FOS_E_NULL_POINTER;
    if (!(denominator > 0.0)) return FOS_E_BAD_SHAPE;
    return gemm_nvfp4_impl(A, B, sfA, sfB, nullptr, amax_a, amax_b, denominator, M, N, K, D, out_type, ldd, bias, d_amax, workspace,
                           workspace_bytes, stream);
}
