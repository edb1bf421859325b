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
// Pipeline per workgroup (tile BM x BN x 64, BM = BN = threads / 2): every thread owns 32
// codes of one A row and of one B row per K step.  Registers hold the packed data of step
// k+2 (in flight from HBM) while step k+1 is dequantised into one LDS buffer and step k is
// multiplied out of the other, so there is one barrier per K step and the VALU work of the
// dequantisation issues in the shadow of the MFMAs.  The big tile (256 x 256, 8
// wavefronts of 128 x 64) keeps LDS reads at ~75 % of their bandwidth; a 128 x 128 tile
// serves shapes that are not multiples of 256 or too small to fill the chip otherwise.
// Workgroups are numbered so that the tiles resident on one XCD (blockIdx % 8) form a
// compact block of the output, which keeps their A/B panels in that XCD's L2.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include <cstdlib>
#include <type_traits>

#include "fos_device.h"
#include "fouroversix_hip.h"

namespace fos {

typedef _Float16 half2_t __attribute__((ext_vector_type(2)));
typedef _Float16 half8_t __attribute__((ext_vector_type(8)));
typedef float float16_t __attribute__((ext_vector_type(16)));

struct GemmParams {
    const uint8_t *A, *B;      // [M, K/2], [N, K/2]
    const uint8_t *sfA, *sfB;  // 128x4-tiled E4M3 bytes
    const float *alpha;
    void *D;
    int64_t M, N, K, ldd;
    int tiles_m, tiles_n;
};

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

// Packed operands of one K step as a thread holds them.
struct Staged {
    uint4 qa, qb;     // 32 codes of one A row / one B row
    uint32_t sa, sb;  // the 4 scale bytes of that row's K step
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
template <int WAVES_M, int WAVES_N, int WM, int WN, bool OUT_BF16>
__global__ __launch_bounds__(64 * WAVES_M *WAVES_N) void gemm_nvfp4_kernel(const GemmParams p) {
    constexpr int kThreadsG = 64 * WAVES_M * WAVES_N;
    constexpr int BM = WAVES_M * WM * 32, BN = WAVES_N * WN * 32;
    static_assert(BM == kThreadsG / 2 && BN == kThreadsG / 2, "one thread per half row of each operand");
    extern __shared__ __attribute__((aligned(16))) _Float16 lds[];
    _Float16 *lds_a[2] = {lds, lds + (BM + BN) * kPitch};
    _Float16 *lds_b[2] = {lds + BM * kPitch, lds + (BM + BN) * kPitch + BM * kPitch};

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    int tile_m, tile_n;
    tile_of(blockIdx.x, p.tiles_m, p.tiles_n, tile_m, tile_n);
    const int64_t m0 = (int64_t)tile_m * BM, n0 = (int64_t)tile_n * BN;
    const int64_t kbytes = p.K >> 1;     // packed bytes per row
    const int64_t sf_groups = p.K >> 6;  // 4-block groups per row

    // global -> register staging: 32 codes (16 bytes) of one row of each operand, through
    // buffer loads (wave-uniform base + per-thread 32-bit offset + scalar K offset), which
    // keeps 64-bit address arithmetic out of the loop
    const int ld_row = tid >> 1, ld_half = tid & 1;
    const BufferRsrc ra = make_rsrc(p.A + m0 * kbytes, (uint32_t)(BM * kbytes));
    const BufferRsrc rb = make_rsrc(p.B + n0 * kbytes, (uint32_t)(BN * kbytes));
    const BufferRsrc rsa = make_rsrc(p.sfA + (m0 >> 7) * sf_groups * 512, (uint32_t)((BM >> 7) * sf_groups * 512));
    const BufferRsrc rsb = make_rsrc(p.sfB + (n0 >> 7) * sf_groups * 512, (uint32_t)((BN >> 7) * sf_groups * 512));
    const uint32_t q_off = (uint32_t)(ld_row * kbytes + ld_half * 16);
    const uint32_t s_off = (uint32_t)((ld_row >> 7) * sf_groups * 512 + (ld_row & 31) * 16 + ((ld_row & 127) >> 5) * 4);
    const int64_t ksteps = p.K / BK;

    auto fetch = [&](int64_t ks, Staged &s) {
        const uint32_t kq = (uint32_t)ks * 32u, ksf = (uint32_t)ks * 512u;
        s.qa = __builtin_bit_cast(uint4, __builtin_amdgcn_raw_buffer_load_b128(ra, (int)q_off, (int)kq, 0));
        s.qb = __builtin_bit_cast(uint4, __builtin_amdgcn_raw_buffer_load_b128(rb, (int)q_off, (int)kq, 0));
        s.sa = __builtin_amdgcn_raw_buffer_load_b32(rsa, (int)s_off, (int)ksf, 0);
        s.sb = __builtin_amdgcn_raw_buffer_load_b32(rsb, (int)s_off, (int)ksf, 0);
    };
    // quarter q (0..3) of the staged data -> 8 halfs of each operand in LDS buffer `buf`
    auto stage_quarter = [&](const Staged &s, int buf, int q) {
        const uint32_t wa = q == 0 ? s.qa.x : q == 1 ? s.qa.y : q == 2 ? s.qa.z : s.qa.w;
        const uint32_t wb = q == 0 ? s.qb.x : q == 1 ? s.qb.y : q == 2 ? s.qb.z : s.qb.w;
        // this thread's two block scales of each operand: bytes 2*ld_half, 2*ld_half + 1
        const half2_t sa2 = e4m3x2_to_half2(s.sa >> (16 * ld_half)), sb2 = e4m3x2_to_half2(s.sb >> (16 * ld_half));
        const half2_t sa = (q >> 1) ? __builtin_shufflevector(sa2, sa2, 1, 1) : __builtin_shufflevector(sa2, sa2, 0, 0);
        const half2_t sb = (q >> 1) ? __builtin_shufflevector(sb2, sb2, 1, 1) : __builtin_shufflevector(sb2, sb2, 0, 0);
        half8_t *da = reinterpret_cast<half8_t *>(lds_a[buf] + ld_row * kPitch + ld_half * 32);
        half8_t *db = reinterpret_cast<half8_t *>(lds_b[buf] + ld_row * kPitch + ld_half * 32);
        da[q] = dequant8(wa, sa);
        db[q] = dequant8(wb, sb);
    };

    const int wm = wave / WAVES_N, wn = wave % WAVES_N;
    float16_t acc[WM][WN];
#pragma unroll
    for (int i = 0; i < WM; ++i)
#pragma unroll
        for (int j = 0; j < WN; ++j)
#pragma unroll
            for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.0f;

    auto read_frags = [&](int buf, int kk, half8_t *fa, half8_t *fb) {
        const int kofs = kk * 16 + (lane >> 5) * 8;
#pragma unroll
        for (int i = 0; i < WM; ++i)
            fa[i] = *reinterpret_cast<const half8_t *>(lds_a[buf] + (wm * WM * 32 + i * 32 + (lane & 31)) * kPitch + kofs);
#pragma unroll
        for (int j = 0; j < WN; ++j)
            fb[j] = *reinterpret_cast<const half8_t *>(lds_b[buf] + (wn * WN * 32 + j * 32 + (lane & 31)) * kPitch + kofs);
    };

    Staged st[2];
    half8_t fa[2][WM], fb[2][WN];  // MFMA fragments of the current and the next 16-wide K slice
    fetch(0, st[0]);
#pragma unroll
    for (int q = 0; q < 4; ++q) stage_quarter(st[0], 0, q);
    if (ksteps > 1) fetch(1, st[1]);
    __syncthreads();
    read_frags(0, 0, fa[0], fb[0]);

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
    auto kstep = [&](auto have_next_c, int64_t ks, int buf, Staged &cur_regs, Staged &nxt) {
        constexpr bool have_next = decltype(have_next_c)::value;
        // `cur_regs` (step ks) went into LDS during the previous step: refill them now,
        // two steps ahead of their use, so HBM / L2 latency has a whole K step to hide in
        if (have_next) fetch(ks + 2 < ksteps ? ks + 2 : ksteps - 1, cur_regs);
#pragma unroll
        for (int kk = 0; kk < BK / 16; ++kk) {
            if (kk + 1 < BK / 16) read_frags(buf, kk + 1, fa[(kk + 1) & 1], fb[(kk + 1) & 1]);
            if (have_next) {
                stage_quarter(nxt, buf ^ 1, kk);
                if (kk + 1 == BK / 16) {
                    __syncthreads();
                    read_frags(buf ^ 1, 0, fa[0], fb[0]);
                    // keep this slice's MFMAs below the barrier (the scheduler would
                    // otherwise hoist them and leave the matrix pipe idle behind it)
                    __builtin_amdgcn_sched_barrier(0);
                }
            }
#pragma unroll
            for (int i = 0; i < WM; ++i)
#pragma unroll
                for (int j = 0; j < WN; ++j)
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(fb[kk & 1][j], fa[kk & 1][i], acc[i][j], 0, 0, 0);
            // slices are scheduled one at a time: a wider window only raises register pressure
            __builtin_amdgcn_sched_barrier(0);
        }
    };

    using yes = std::integral_constant<bool, true>;
    using no = std::integral_constant<bool, false>;
    int64_t ks = 0;
    for (; ks + 2 < ksteps; ks += 2) {
        kstep(yes{}, ks, 0, st[0], st[1]);
        kstep(yes{}, ks + 1, 1, st[1], st[0]);
    }
    if (ks + 2 == ksteps) {
        kstep(yes{}, ks, 0, st[0], st[1]);
        kstep(no{}, ks + 1, 1, st[1], st[0]);
    } else {
        kstep(no{}, ks, 0, st[0], st[1]);
    }

    // epilogue: acc[i][j][4*g + e] is D[m][n] with m = wm*WM*32 + i*32 + (lane & 31),
    // n = wn*WN*32 + j*32 + 8*g + 4*(lane >> 5) + e
    const float alpha = *p.alpha;
    uint16_t *D = reinterpret_cast<uint16_t *>(p.D);
#pragma unroll
    for (int i = 0; i < WM; ++i) {
        const int64_t m = m0 + wm * WM * 32 + i * 32 + (lane & 31);
#pragma unroll
        for (int j = 0; j < WN; ++j) {
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                const int64_t n = n0 + wn * WN * 32 + j * 32 + 8 * g + 4 * (lane >> 5);
                uint16_t o[4];
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    float v = alpha * acc[i][j][4 * g + e];
                    if (OUT_BF16) {
                        uint32_t u = f2u(v);
                        u += 0x7fffu + ((u >> 16) & 1u);
                        o[e] = (uint16_t)(u >> 16);
                    } else {
                        o[e] = __builtin_bit_cast(uint16_t, (_Float16)v);
                    }
                }
                uint2 pk = make_uint2(o[0] | ((uint32_t)o[1] << 16), o[2] | ((uint32_t)o[3] << 16));
                *reinterpret_cast<uint2 *>(D + m * p.ldd + n) = pk;
            }
        }
    }
}

template <int WAVES_M, int WAVES_N, int WM, int WN>
static int launch_gemm(GemmParams &p, int out_type, hipStream_t s) {
    constexpr int BM = WAVES_M * WM * 32, BN = WAVES_N * WN * 32;
    constexpr int kThreadsG = 64 * WAVES_M * WAVES_N;
    constexpr size_t lds_bytes = 2 * (size_t)(BM + BN) * kPitch * sizeof(_Float16);
    p.tiles_m = (int)(p.M / BM);
    p.tiles_n = (int)(p.N / BN);
    dim3 grid((unsigned)(p.tiles_m * p.tiles_n));
    auto kbf = gemm_nvfp4_kernel<WAVES_M, WAVES_N, WM, WN, true>;
    auto kh = gemm_nvfp4_kernel<WAVES_M, WAVES_N, WM, WN, false>;
    if (lds_bytes > 64 * 1024) {
        // more than the default dynamic LDS limit: opt in (idempotent, no device state besides the function attribute)
        if (hipFuncSetAttribute((const void *)(out_type == FOS_T_BF16 ? kbf : kh), hipFuncAttributeMaxDynamicSharedMemorySize,
                                (int)lds_bytes) != hipSuccess)
            return FOS_E_LAUNCH;
    }
    if (out_type == FOS_T_BF16) hipLaunchKernelGGL(kbf, grid, dim3(kThreadsG), lds_bytes, s, p);
    else hipLaunchKernelGGL(kh, grid, dim3(kThreadsG), lds_bytes, s, p);
    return hipGetLastError() == hipSuccess ? FOS_OK : FOS_E_LAUNCH;
}

}  // namespace fos

using namespace fos;

extern "C" int fos_gemm_nvfp4(const uint8_t *A, const uint8_t *B, const uint8_t *sfA, const uint8_t *sfB,
                              const float *alpha, int64_t M, int64_t N, int64_t K,
                              void *D, int out_type, int64_t ldd, fos_stream_t stream) {
    if (!A || !B || !sfA || !sfB || !alpha || !D) return FOS_E_NULL_POINTER;
    if (M <= 0 || N <= 0 || K <= 0 || M % 128 != 0 || N % 128 != 0 || K % 64 != 0 || ldd < N) return FOS_E_BAD_SHAPE;
    if (out_type != FOS_T_BF16 && out_type != FOS_T_F16) return FOS_E_UNSUPPORTED;
    if (((uintptr_t)A & 15) || ((uintptr_t)B & 15) || ((uintptr_t)sfA & 3) || ((uintptr_t)sfB & 3) ||
        ((uintptr_t)D & 7) || (ldd % 4 != 0) || ((uintptr_t)alpha & 3))
        return FOS_E_BAD_ALIGNMENT;
    if ((M / 128) * (N / 128) > 0x7fffffffLL) return FOS_E_BAD_SHAPE;
    GemmParams p;
    p.A = A; p.B = B; p.sfA = sfA; p.sfB = sfB; p.alpha = alpha; p.D = D;
    p.M = M; p.N = N; p.K = K; p.ldd = ldd;
    hipStream_t s = (hipStream_t)stream;
    // 256 x 256 tiles when they divide the problem and give every compute unit work;
    // FOS_GEMM_TILE=128 forces the small tile (tuning / tests).
    bool big = (M % 256 == 0) && (N % 256 == 0) && (M / 256) * (N / 256) >= 128;
    if (const char *e = getenv("FOS_GEMM_TILE")) big = big && atoi(e) != 128;
    if (big) return launch_gemm<2, 4, 4, 2>(p, out_type, s);
    return launch_gemm<2, 2, 2, 2>(p, out_type, s);
}
