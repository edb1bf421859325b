// gfx950 dequantize: packed 4-bit codes + E4M3 block scales + FP32 tensor scale -> bf16 /
// fp16 / fp32, with the arithmetic of QuantizeBackendBase.dequantize
// (src/fouroversix/quantize/backend.py:89-160): value and scale meet in fp16, the result
// is widened to fp32, multiplied by amax and divided by f32(qmax * smax * adjustment).
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "fos_buffer.h"
#include "fos_quantize_fast.h"
#include "fouroversix_hip.h"

namespace fos {

struct DequantParams {
    const uint8_t *codes, *sf;
    const float *amax;
    void *out;
    int64_t rows, cols, rows_p, cols_p, ldo;
    float divisor;
    int sf_layout;
    int fast_div;       // divisor is 1536, 1792 or 2688 (exact 3-operation division)
    int vector_stores;  // out and ldo allow 16-byte stores of whole blocks
    int f32_product;    // value * scale formed in fp32 instead of fp16 (differs for IF4's integer blocks)
    int wave_lines;     // fp32 output: whole wavefronts inside a row (cols % 512 == 0) and 16-byte stores allowed
};

// One thread per 8 consecutive elements, i.e. half a 1x16 block (consecutive threads =
// consecutive octets of a row: a wavefront reads 256 contiguous bytes of codes and writes
// 1 KiB per store instruction); blockIdx.y walks the rows.  `p.fast_div`: the divisor is one
// of the constants for which the 3-operation division is exact; it is used when amax is far
// enough from the ends of the float range for every quotient to be normal or zero.
// When, besides, amax has at most 8 significant bits (the maximum of a bf16 tensor), value *
// scale * amax is exact and its quotient is (power of two) x RN(g / c) or x RN(1.5 g / c) with
// g = scale * amax (see dequant_block_bf16_lut): the two quotients are formed once per thread
// and an element costs four operations instead of eight.
template <int DT, int OUT>
__global__ __launch_bounds__(256) void dequantize_kernel(const DequantParams p) {
    const int64_t sf_cols = p.cols_p >> 4;
    const uint32_t opr = (uint32_t)((p.cols + 7) >> 3);  // octets per row
    // (32-bit column quantities: the row parts of every address are wavefront-uniform and stay on
    // the scalar unit, a thread adds a 32-bit offset)
    const uint32_t oc = blockIdx.x * 256u + threadIdx.x, cb = oc >> 1;
    if (oc >= opr) return;
    const uint32_t sf_col_off = p.sf_layout == FOS_SF_TILED_128X4 ? (cb >> 2) * 512u + (cb & 3u) : cb;
    const float amax = *p.amax;
    const bool fast = p.fast_div && amax >= 0x1p-100f && amax <= 0x1p100f;
    const bool table = fast && (f2u(amax) & 0xffffu) == 0;
    const float rc = 1.0f / p.divisor;
    __shared__ float4 swap[OUT == FOS_T_F32 ? 4 : 1][OUT == FOS_T_F32 ? 128 : 1];
    for (int64_t r = blockIdx.y; r < p.rows; r += gridDim.y) {
        const uint8_t *row_codes = p.codes + r * (p.cols_p >> 1);
        const uint8_t *row_sf = p.sf + (p.sf_layout == FOS_SF_TILED_128X4
                                            ? (r >> 7) * (sf_cols >> 2) * 512 + (r & 31) * 16 + ((r & 127) >> 5) * 4
                                            : r * sf_cols);
        const uint32_t q = *reinterpret_cast<const uint32_t *>(row_codes + oc * 4u);
        const uint32_t sb = row_sf[sf_col_off];
        const float sf = e4m3_decode(sb & 0x7fu);

        float f[8];
        const bool int_block = DT == FOS_DTYPE_IF4 && (sb & 0x80u);
        if (table && !int_block && (sb & 0x7fu) != 0x7fu) {
            const float g = sf * amax;  // exact: 4 + 8 significant bits
            const float d1 = div_const(g, p.divisor, rc), d15 = div_const(1.5f * g, p.divisor, rc);
            const uint32_t delta = f2u(d15) - f2u(d1);
            static_for<0, 4>([&](auto jc) {
                constexpr int j = decltype(jc)::value;
                const float2_t v = unpack_fp4<j>(q);
#pragma unroll
                for (int h = 0; h < 2; ++h) {
                    const uint32_t fb = f2u(v[h]);
                    f[2 * j + h] = u2f(fb & 0xffbfffffu) * u2f(mad_u24((fb >> 22) & 1u, delta, f2u(d1)));
                }
            });
        } else {
            // value * scale, as the fp16 product of the reference (exact for E2M1 values)
            if (int_block) {
                const _Float16 s16 = (_Float16)sf;
                const float six_sevenths = (float)(6.0 / 7.0);
#pragma unroll
                for (int i = 0; i < 8; ++i) {
                    const uint32_t code = (q >> (4 * i)) & 0xfu;
                    const int iv = ((int)(code << 28)) >> 28;
                    f[i] = p.f32_product ? ((float)iv * six_sevenths) * sf : (float)((_Float16)((float)iv * six_sevenths) * s16);
                }
            } else {
                static_for<0, 4>([&](auto jc) {
                    constexpr int j = decltype(jc)::value;
                    const float2_t v = unpack_fp4<j>(q);
                    f[2 * j] = v.x * sf;
                    f[2 * j + 1] = v.y * sf;
                });
            }
            if (fast) {
#pragma unroll
                for (int i = 0; i < 8; ++i) {
                    const float t = f[i] * amax;
                    f[i] = u2f((f2u(div_const(t, p.divisor, rc)) & 0x7fffffffu) | (f2u(t) & 0x80000000u));
                }
            } else {
#pragma unroll
                for (int i = 0; i < 8; ++i) f[i] = (f[i] * amax) / p.divisor;
            }
        }

        const uint32_t c0 = oc * 8u;
        const bool whole = p.vector_stores && c0 + 8 <= p.cols;
        if (OUT == FOS_T_F32) {
            float *o = reinterpret_cast<float *>(p.out) + r * p.ldo + c0;
            if (p.wave_lines) {
                // a lane's 32 bytes as two stores 16 bytes apart would leave every instruction
                // writing half of each line it touches: the wavefront turns its 2 KiB round in LDS
                // and stores two contiguous KiB
                const int lane = threadIdx.x & 63;
                float4 *mine = swap[threadIdx.x >> 6];
                mine[2 * lane] = make_float4(f[0], f[1], f[2], f[3]);
                mine[2 * lane + 1] = make_float4(f[4], f[5], f[6], f[7]);
                __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
                __builtin_amdgcn_wave_barrier();
                __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
                const float4 lo = mine[lane], hi = mine[64 + lane];
                uint4 *ow = reinterpret_cast<uint4 *>(o - 8 * lane);  // the wavefront's first element
                stream_store(ow + lane, __builtin_bit_cast(uint4, lo));
                stream_store(ow + 64 + lane, __builtin_bit_cast(uint4, hi));
                __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
                __builtin_amdgcn_wave_barrier();
            } else if (whole) {
                reinterpret_cast<float4 *>(o)[0] = make_float4(f[0], f[1], f[2], f[3]);
                reinterpret_cast<float4 *>(o)[1] = make_float4(f[4], f[5], f[6], f[7]);
            } else {
#pragma unroll
                for (int i = 0; i < 8; ++i)
                    if (c0 + i < p.cols) o[i] = f[i];
            }
            continue;
        }
        uint32_t w[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const float2_t v = {f[2 * j], f[2 * j + 1]};
            if (OUT == FOS_T_F16) {
                typedef _Float16 half2_t __attribute__((ext_vector_type(2)));
                w[j] = __builtin_bit_cast(uint32_t, __builtin_convertvector(v, half2_t));
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
}

}  // namespace fos

namespace fos {
// MXFP4 (fos_mxfp4.hip)
int launch_dequantize_mxfp4(const uint8_t *codes, const uint8_t *sf, int sf_layout, int64_t rows, int64_t cols,
                            int64_t rows_p, int64_t cols_p, void *out, int out_type, int64_t ldo, int f32_product,
                            hipStream_t s);
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
                              void *out, int out_type, int64_t ldo, int intermediate_type, fos_stream_t stream) {
    if (!codes || !sf || !out || (!amax && dtype != FOS_DTYPE_MXFP4)) return FOS_E_NULL_POINTER;
    if (intermediate_type != FOS_T_F16 && intermediate_type != FOS_T_F32) return FOS_E_UNSUPPORTED;
    const int f32_product = intermediate_type == FOS_T_F32;
    if (dtype == FOS_DTYPE_MXFP4) {
        if (rows <= 0 || cols <= 0 || rows > rows_p || cols > cols_p || ldo < cols) return FOS_E_BAD_SHAPE;
        if (sf_layout == FOS_SF_TILED_128X4 && rows_p % 128 != 0) return FOS_E_BAD_SHAPE;
        if (sf_layout != FOS_SF_LINEAR && sf_layout != FOS_SF_TILED_128X4) return FOS_E_UNSUPPORTED;
        if (out_type != FOS_T_BF16 && out_type != FOS_T_F16 && out_type != FOS_T_F32) return FOS_E_UNSUPPORTED;
        return launch_dequantize_mxfp4(codes, sf, sf_layout, rows, cols, rows_p, cols_p, out, out_type, ldo, f32_product,
                                       (hipStream_t)stream);
    }
    if (rows <= 0 || cols <= 0 || rows > rows_p || cols > cols_p || cols_p % 16 != 0 || ldo < cols) return FOS_E_BAD_SHAPE;
    if (sf_layout == FOS_SF_TILED_128X4 && (rows_p % 128 != 0 || cols_p % 64 != 0)) return FOS_E_BAD_SHAPE;
    if (dtype != FOS_DTYPE_NVFP4 && dtype != FOS_DTYPE_IF4) return FOS_E_UNSUPPORTED;
    if (sf_layout != FOS_SF_LINEAR && sf_layout != FOS_SF_TILED_128X4) return FOS_E_UNSUPPORTED;
    if (out_type != FOS_T_BF16 && out_type != FOS_T_F16 && out_type != FOS_T_F32) return FOS_E_UNSUPPORTED;
    if (((uintptr_t)codes & 3) || ((uintptr_t)amax & 3)) return FOS_E_BAD_ALIGNMENT;
    DequantParams p;
    p.codes = codes; p.sf = sf; p.amax = amax; p.out = out;
    p.rows = rows; p.cols = cols; p.rows_p = rows_p; p.cols_p = cols_p; p.ldo = ldo;
    p.divisor = (float)divisor;
    p.sf_layout = sf_layout;
    p.f32_product = f32_product;
    p.fast_div = p.divisor == 1536.0f || p.divisor == 1792.0f || p.divisor == 2688.0f;
    const int64_t esize = out_type == FOS_T_F32 ? 4 : 2;
    p.vector_stores = ((uintptr_t)out & 15) == 0 && (ldo * esize) % 16 == 0;
    p.wave_lines = out_type == FOS_T_F32 && p.vector_stores && cols % 512 == 0;
    const int64_t opr = (cols + 7) / 8;
    if (cols_p > 0x7fffffffLL) return FOS_E_BAD_SHAPE;  // 32-bit column offsets in the kernel
    dim3 grid((unsigned)((opr + 255) / 256), (unsigned)(rows < 65535 ? rows : 65535));
    hipStream_t s = (hipStream_t)stream;
    if (dtype == FOS_DTYPE_IF4) launch_dequant<FOS_DTYPE_IF4>(p, out_type, grid, s);
    else launch_dequant<FOS_DTYPE_NVFP4>(p, out_type, grid, s);
    return hipGetLastError() == hipSuccess ? FOS_OK : FOS_E_LAUNCH;
}
