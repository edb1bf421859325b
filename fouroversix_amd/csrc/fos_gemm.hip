// gfx950 NVFP4 x NVFP4 GEMM:  D[M,N] = alpha * sum_k (A[m,k] sA[m,k/16]) (B[n,k] sB[n,k/16]).
//
// The contraction runs on the fp16 MFMA pipe.  E2M1 codes and E4M3 block scales are
// loaded from HBM in their packed form, turned into fp16(value * scale) in registers
// (the product has at most 6 significant bits and lies in [2^-10, 2688], so it is exact
// in fp16 -- the same intermediate the reference's dequantize uses,
// src/fouroversix/quantize/backend.py:89-160), staged in LDS as fp16 and fed to
// v_mfma_f32_32x32x16_f16 with FP32 accumulation; alpha is applied in the epilogue from
// device memory (src/fouroversix/csrc/fp4_gemm.cu:143).
#include <hip/hip_runtime.h>
#include <stdint.h>

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
    int tiles_n;
};

// E4M3 byte (bits 0..6) -> fp16 pair {s, s}.  The byte at bit 7 of a half is the E4M3
// value with exponent bias 15 instead of 7; 2^8 rebiases it (sub-normals included).
FOS_DEVICE half2_t e4m3_to_half2(uint32_t b) {
    uint32_t h = (b & 0x7fu) << 7;
    half2_t v = __builtin_bit_cast(half2_t, h | (h << 16));
    const half2_t k = {(_Float16)256.0f, (_Float16)256.0f};
    return v * k;
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

constexpr int BM = 128, BN = 128, BK = 64;
constexpr int kGemmThreads = 256;
constexpr int kPitch = BK + 8;  // halfs per LDS row (144 bytes: conflict-free 128-bit reads)

// Tile 128 x 128 x 64, 4 wavefronts in a 2 x 2 arrangement, each 64 x 64 as 2 x 2 MFMA
// 32x32x16 tiles.  The MFMA "A" operand is fed from the B matrix (rows n) and the "B"
// operand from the A matrix (rows m), so that a lane's four consecutive accumulator
// registers are four consecutive n of one output row and can be stored as 8 bytes.
template <bool OUT_BF16>
__global__ __launch_bounds__(kGemmThreads) void gemm_nvfp4_kernel(const GemmParams p) {
    __shared__ __attribute__((aligned(16))) _Float16 lds_a[BM * kPitch];
    __shared__ __attribute__((aligned(16))) _Float16 lds_b[BN * kPitch];

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int tile_n = blockIdx.x % p.tiles_n;
    const int64_t tile_m = blockIdx.x / p.tiles_n;
    const int64_t m0 = tile_m * BM, n0 = (int64_t)tile_n * BN;
    const int64_t kbytes = p.K >> 1;      // packed bytes per row
    const int64_t sf_groups = p.K >> 6;   // 4-block groups per row

    // global -> register staging: thread handles 32 codes (16 bytes) of one row of each operand
    const int ld_row = tid >> 1, ld_half = tid & 1;
    const uint8_t *a_ptr = p.A + (m0 + ld_row) * kbytes + ld_half * 16;
    const uint8_t *b_ptr = p.B + (n0 + ld_row) * kbytes + ld_half * 16;
    const int sf_in_tile = (ld_row & 31) * 16 + (ld_row >> 5) * 4;
    const uint8_t *sfa_ptr = p.sfA + tile_m * sf_groups * 512 + sf_in_tile;
    const uint8_t *sfb_ptr = p.sfB + (int64_t)tile_n * sf_groups * 512 + sf_in_tile;

    const int wm = wave >> 1, wn = wave & 1;  // wave position in the 2 x 2 arrangement
    float16_t acc[2][2];
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
            for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.0f;

    uint4 qa = *reinterpret_cast<const uint4 *>(a_ptr);
    uint4 qb = *reinterpret_cast<const uint4 *>(b_ptr);
    uint32_t sa = *reinterpret_cast<const uint32_t *>(sfa_ptr);
    uint32_t sb = *reinterpret_cast<const uint32_t *>(sfb_ptr);

    const int64_t ksteps = p.K / BK;
    for (int64_t ks = 0; ks < ksteps; ++ks) {
        // dequantize the staged registers into LDS
        {
            half2_t s0 = e4m3_to_half2(sa >> (16 * ld_half));
            half2_t s1 = e4m3_to_half2(sa >> (16 * ld_half + 8));
            half8_t *dst = reinterpret_cast<half8_t *>(lds_a + ld_row * kPitch + ld_half * 32);
            dst[0] = dequant8(qa.x, s0);
            dst[1] = dequant8(qa.y, s0);
            dst[2] = dequant8(qa.z, s1);
            dst[3] = dequant8(qa.w, s1);
            half2_t t0 = e4m3_to_half2(sb >> (16 * ld_half));
            half2_t t1 = e4m3_to_half2(sb >> (16 * ld_half + 8));
            half8_t *dstb = reinterpret_cast<half8_t *>(lds_b + ld_row * kPitch + ld_half * 32);
            dstb[0] = dequant8(qb.x, t0);
            dstb[1] = dequant8(qb.y, t0);
            dstb[2] = dequant8(qb.z, t1);
            dstb[3] = dequant8(qb.w, t1);
        }
        __syncthreads();
        // prefetch the next K step while this one is multiplied
        if (ks + 1 < ksteps) {
            qa = *reinterpret_cast<const uint4 *>(a_ptr + (ks + 1) * 32);
            qb = *reinterpret_cast<const uint4 *>(b_ptr + (ks + 1) * 32);
            sa = *reinterpret_cast<const uint32_t *>(sfa_ptr + (ks + 1) * 512);
            sb = *reinterpret_cast<const uint32_t *>(sfb_ptr + (ks + 1) * 512);
        }
#pragma unroll
        for (int kk = 0; kk < BK / 16; ++kk) {
            half8_t fa[2], fb[2];
            const int kofs = kk * 16 + (lane >> 5) * 8;
#pragma unroll
            for (int i = 0; i < 2; ++i)
                fa[i] = *reinterpret_cast<const half8_t *>(lds_a + (wm * 64 + i * 32 + (lane & 31)) * kPitch + kofs);
#pragma unroll
            for (int j = 0; j < 2; ++j)
                fb[j] = *reinterpret_cast<const half8_t *>(lds_b + (wn * 64 + j * 32 + (lane & 31)) * kPitch + kofs);
#pragma unroll
            for (int i = 0; i < 2; ++i)
#pragma unroll
                for (int j = 0; j < 2; ++j)
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(fb[j], fa[i], acc[i][j], 0, 0, 0);
        }
        __syncthreads();
    }

    // epilogue: acc[i][j][4*g + e] is D[m][n] with m = wm*64 + i*32 + (lane & 31),
    // n = wn*64 + j*32 + 8*g + 4*(lane >> 5) + e
    const float alpha = *p.alpha;
    uint16_t *D = reinterpret_cast<uint16_t *>(p.D);
#pragma unroll
    for (int i = 0; i < 2; ++i) {
        const int64_t m = m0 + wm * 64 + i * 32 + (lane & 31);
#pragma unroll
        for (int j = 0; j < 2; ++j) {
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                const int64_t n = n0 + wn * 64 + j * 32 + 8 * g + 4 * (lane >> 5);
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
    if ((M / BM) * (N / BN) > 0x7fffffffLL) return FOS_E_BAD_SHAPE;
    GemmParams p;
    p.A = A; p.B = B; p.sfA = sfA; p.sfB = sfB; p.alpha = alpha; p.D = D;
    p.M = M; p.N = N; p.K = K; p.ldd = ldd;
    p.tiles_n = (int)(N / BN);
    dim3 grid((unsigned)((M / BM) * (N / BN)));
    hipStream_t s = (hipStream_t)stream;
    if (out_type == FOS_T_BF16)
        hipLaunchKernelGGL((gemm_nvfp4_kernel<true>), grid, dim3(kGemmThreads), 0, s, p);
    else
        hipLaunchKernelGGL((gemm_nvfp4_kernel<false>), grid, dim3(kGemmThreads), 0, s, p);
    return hipGetLastError() == hipSuccess ? FOS_OK : FOS_E_LAUNCH;
}
