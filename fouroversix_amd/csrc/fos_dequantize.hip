// gfx950 dequantize: packed 4-bit codes + E4M3 block scales + FP32 tensor scale -> bf16 /
// fp16 / fp32, with the arithmetic of QuantizeBackendBase.dequantize
// (src/fouroversix/quantize/backend.py:89-160): value and scale meet in fp16, the result
// is widened to fp32, multiplied by amax and divided by f32(qmax * smax * adjustment).
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "fos_device.h"
#include "fouroversix_hip.h"

namespace fos {

struct DequantParams {
    const uint8_t *codes, *sf;
    const float *amax;
    void *out;
    int64_t rows, cols, rows_p, cols_p, ldo;
    float divisor;
    int sf_layout;
};

FOS_DEVICE float e2m1_value(uint32_t code) {
    // magnitudes 0, .5, 1, 1.5, 2, 3, 4, 6: (e, m) = (code >> 1 & 3, code & 1)
    const uint32_t e = (code >> 1) & 3u, m = code & 1u;
    float v = e == 0 ? 0.5f * (float)m : u2f((126u + e) << 23 | m << 22);
    return (code & 8u) ? -v : v;
}

template <int DT, int OUT>
__global__ __launch_bounds__(256) void dequantize_kernel(const DequantParams p) {
    const int64_t sf_cols = p.cols_p >> 4;
    const int64_t blk = (int64_t)blockIdx.x * 256 + threadIdx.x;
    const int64_t n_blocks = p.rows * ((p.cols + 15) >> 4);
    if (blk >= n_blocks) return;
    const int64_t bpr = (p.cols + 15) >> 4;
    const int64_t r = blk / bpr, cb = blk % bpr;
    const uint2 q = *reinterpret_cast<const uint2 *>(p.codes + r * (p.cols_p >> 1) + cb * 8);
    const int64_t sofs = p.sf_layout == FOS_SF_TILED_128X4
                             ? ((r >> 7) * (sf_cols >> 2) + (cb >> 2)) * 512 + (r & 31) * 16 + ((r & 127) >> 5) * 4 + (cb & 3)
                             : r * sf_cols + cb;
    const uint32_t sb = p.sf[sofs];
    const bool is_int = DT == FOS_DTYPE_IF4 && (sb & 0x80u);
    const _Float16 s16 = (_Float16)e4m3_decode(sb & 0x7fu);
    const float amax = *p.amax;
    const float six_sevenths = (float)(6.0 / 7.0);
#pragma unroll
    for (int i = 0; i < 16; ++i) {
        const int64_t c = cb * 16 + i;
        if (c >= p.cols) break;
        const uint32_t word = i < 8 ? q.x : q.y;
        const uint32_t code = (word >> (4 * (i & 7))) & 0xfu;
        _Float16 v16;
        if (is_int) {
            const int iv = ((int)(code << 28)) >> 28;
            v16 = (_Float16)((float)iv * six_sevenths);
        } else {
            v16 = (_Float16)e2m1_value(code);
        }
        const _Float16 r16 = v16 * s16;
        const float f = ((float)r16 * amax) / p.divisor;
        if (OUT == FOS_T_F32) {
            reinterpret_cast<float *>(p.out)[r * p.ldo + c] = f;
        } else if (OUT == FOS_T_F16) {
            reinterpret_cast<_Float16 *>(p.out)[r * p.ldo + c] = (_Float16)f;
        } else {
            uint32_t u = f2u(f);
            u += 0x7fffu + ((u >> 16) & 1u);
            reinterpret_cast<uint16_t *>(p.out)[r * p.ldo + c] = (uint16_t)(u >> 16);
        }
    }
}

}  // namespace fos

using namespace fos;

namespace {
template <int DT>
void launch_dequant(const DequantParams &p, int out_type, dim3 grid, hipStream_t s) {
    if (out_type == FOS_T_F32) hipLaunchKernelGGL((dequantize_kernel<DT, FOS_T_F32>), grid, dim3(256), 0, s, p);
    else if (out_type == FOS_T_F16) hipLaunchKernelGGL((dequantize_kernel<DT, FOS_T_F16>), grid, dim3(256), 0, s, p);
    else hipLaunchKernelGGL((dequantize_kernel<DT, FOS_T_BF16>), grid, dim3(256), 0, s, p);
}
}  // namespace

extern "C" int fos_dequantize(const uint8_t *codes, const uint8_t *sf, const float *amax,
                              int dtype, int sf_layout, double divisor,
                              int64_t rows, int64_t cols, int64_t rows_p, int64_t cols_p,
                              void *out, int out_type, int64_t ldo, fos_stream_t stream) {
    if (!codes || !sf || !amax || !out) return FOS_E_NULL_POINTER;
    if (rows <= 0 || cols <= 0 || rows > rows_p || cols > cols_p || cols_p % 16 != 0 || ldo < cols) return FOS_E_BAD_SHAPE;
    if (sf_layout == FOS_SF_TILED_128X4 && (rows_p % 128 != 0 || cols_p % 64 != 0)) return FOS_E_BAD_SHAPE;
    if (dtype != FOS_DTYPE_NVFP4 && dtype != FOS_DTYPE_IF4) return FOS_E_UNSUPPORTED;
    if (sf_layout != FOS_SF_LINEAR && sf_layout != FOS_SF_TILED_128X4) return FOS_E_UNSUPPORTED;
    if (out_type != FOS_T_BF16 && out_type != FOS_T_F16 && out_type != FOS_T_F32) return FOS_E_UNSUPPORTED;
    if (((uintptr_t)codes & 7) || ((uintptr_t)amax & 3)) return FOS_E_BAD_ALIGNMENT;
    DequantParams p;
    p.codes = codes; p.sf = sf; p.amax = amax; p.out = out;
    p.rows = rows; p.cols = cols; p.rows_p = rows_p; p.cols_p = cols_p; p.ldo = ldo;
    p.divisor = (float)divisor;
    p.sf_layout = sf_layout;
    const int64_t n_blocks = rows * ((cols + 15) / 16);
    if ((n_blocks + 255) / 256 > 0x7fffffffLL) return FOS_E_BAD_SHAPE;
    dim3 grid((unsigned)((n_blocks + 255) / 256));
    hipStream_t s = (hipStream_t)stream;
    if (dtype == FOS_DTYPE_IF4) launch_dequant<FOS_DTYPE_IF4>(p, out_type, grid, s);
    else launch_dequant<FOS_DTYPE_NVFP4>(p, out_type, grid, s);
    return hipGetLastError() == hipSuccess ? FOS_OK : FOS_E_LAUNCH;
}
