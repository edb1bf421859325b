// gfx950 quantize path: tensor-wide max|x| (pass 1) and block-scaled 4-bit quantisation
// with E4M3 block scales (pass 2).
//
// Arithmetic follows the reference's PyTorch backend operation by operation
// (src/fouroversix/quantize/pytorch/reference.py:30-63, 184-552; one IEEE fp32 rounding
// per reference operation, torch.sum's summation order for the mse/mae decisions), so
// the packed codes and scale bytes are bit-identical to it for round-to-nearest.
//
// This file holds pass 1, the C entry points, and the pass-2 instantiations that use only
// the operation-by-operation form (IF4, stochastic rounding); NVFP4 round-to-nearest is
// instantiated in fos_quantize_fast.hip.
#include <atomic>
#include <type_traits>
#include <cstdlib>

#include "fos_quantize_kernel.h"
#include "fos_tuning.h"

namespace fos {

// Pass-1 partials of fos_quantize_static: the one buffer the quantizer needs besides its
// inputs and outputs, held by every GPU the library runs on until the process ends.  In
// host code this name is only a handle for hipGetSymbolAddress, never a device address.
constexpr size_t kStaticScratchBytes = 2 * kMaxPartials * sizeof(uint32_t);
static __device__ __align__(256) uint32_t scratch[2 * kMaxPartials];

// ---------------------------------------------------------------------------------------
// pass 1: per-workgroup max |x| as an integer max over the magnitude bits (the second
// word of each partial pair is reserved and written as zero)
// ---------------------------------------------------------------------------------------

template <bool IS_BF16>
FOS_DEVICE uint32_t mag16_to_f32_bits(uint32_t m) {
    if (IS_BF16) return m << 16;
    _Float16 h = __builtin_bit_cast(_Float16, (uint16_t)m);
    return f2u((float)h);
}

// Contiguous, 16-byte aligned input viewed as n_vec 128-bit vectors.
template <bool IS_BF16>
__global__ __launch_bounds__(kThreads) void amax_flat_kernel(const uint4 *__restrict__ x, int64_t n_vec,
                                                             uint32_t *__restrict__ partials) {
    __shared__ uint32_t smem[4];
    const int64_t stride = (int64_t)gridDim.x * kThreads;
    const int64_t first = (int64_t)blockIdx.x * kThreads + threadIdx.x;
    uint32_t m = 0;
    constexpr int U = 8;
    auto fold = [&](const uint4 &v) {
        m = pk_max_u16(m, v.x & 0x7fff7fffu);
        m = pk_max_u16(m, v.y & 0x7fff7fffu);
        m = pk_max_u16(m, v.z & 0x7fff7fffu);
        m = pk_max_u16(m, v.w & 0x7fff7fffu);
    };
    const int64_t n_full = n_vec / (U * stride);  // trips in which every thread has its U vectors
    // the ragged end of the tensor ...
    for (int64_t i = n_full * U * stride + first; i < n_vec; i += stride) fold(x[i]);
    // ... and the full trips
    for (int64_t k = 0; k < n_full; ++k) {
        const int64_t i = k * U * stride + first;
        uint4 v[U];
#pragma unroll
        for (int u = 0; u < U; ++u) v[u] = x[i + u * stride];
#pragma unroll
        for (int u = 0; u < U; ++u) fold(v[u]);
    }
    uint32_t mm = (m & 0xffffu) > (m >> 16) ? (m & 0xffffu) : (m >> 16);
    mm = block_max_u32(mm, smem);
    if (threadIdx.x == 0) {
        partials[2 * blockIdx.x] = mag16_to_f32_bits<IS_BF16>(mm);
        partials[2 * blockIdx.x + 1] = 0u;
    }
}

// bf16 / fp16 input with cols % 2048 == 0, read so that pass 2 finds in L2 what this pass read last (clean lines
// survive the kernel boundary).  The streaming pass-2 kernels give workgroup b the 128 x 256 units b,
// b + grid, ... in row-major order, and the compute die (XCD) that takes workgroup b of a launch is b % 8:
// with a multiple of 8 units to a row, die j quantizes the 512-byte windows j, j + 8, ... of every row,
// starting with the top rows.  Here die j reads exactly those windows, bottom rows first, so the top rows are
// what its L2 holds when pass 2 starts.  At any time the grid reads one contiguous range of whole rows (16
// rows per workgroup and step at 8192 columns, 512 rows in all).  At 8192 x 8192 the scan itself takes
// 0.3 us longer than the flat one and the pass 2 behind it 1-2.5 us less.
template <bool IS_BF16>
__global__ __launch_bounds__(kThreads) void amax_units_kernel(const uint16_t *__restrict__ x, int64_t ld, uint32_t win_per_die,
                                                              uint32_t n_winrows, uint32_t n_steps,
                                                              uint32_t *__restrict__ partials) {
    __shared__ uint32_t smem[4];
    const uint32_t t = threadIdx.x;
    const uint32_t die = blockIdx.x & 7u, slot = blockIdx.x >> 3;  // 32 workgroups to a die
    uint32_t m = 0;
    // a step of a workgroup = 64 window-rows (512 bytes each) = 8 loads of 16 bytes per thread; window-row q
    // of a die is window q % win_per_die of row q / win_per_die.  Only the step at the bottom of the tensor
    // can run past the end: it repeats the final window-row there.
    auto scan = [&](uint32_t step, auto ragged) {
        const uint32_t q0 = ((n_steps - 1 - step) * 32 + slot) * 64 + (t >> 5);
        uint4 v[8];
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            uint32_t q = q0 + j * 8;
            if (ragged) q = q < n_winrows ? q : n_winrows - 1;
            const uint32_t row = q / win_per_die, win = q - row * win_per_die;
            v[j] = *reinterpret_cast<const uint4 *>(x + (int64_t)row * ld + (die + 8 * win) * 256 + (t & 31) * 8);
        }
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            m = pk_max_u16(m, v[j].x & 0x7fff7fffu);
            m = pk_max_u16(m, v[j].y & 0x7fff7fffu);
            m = pk_max_u16(m, v[j].z & 0x7fff7fffu);
            m = pk_max_u16(m, v[j].w & 0x7fff7fffu);
        }
    };
    scan(0, std::true_type{});
    for (uint32_t step = 1; step < n_steps; ++step) scan(step, std::false_type{});
    uint32_t mm = (m & 0xffffu) > (m >> 16) ? (m & 0xffffu) : (m >> 16);
    mm = block_max_u32(mm, smem);
    if (threadIdx.x == 0) {
        partials[2 * blockIdx.x] = mag16_to_f32_bits<IS_BF16>(mm);
        partials[2 * blockIdx.x + 1] = 0u;
    }
}

// Any strides / alignment: one workgroup per row, strided over the rows.
template <bool IS_BF16>
__global__ __launch_bounds__(kThreads) void amax_rows_kernel(const uint16_t *__restrict__ x, int64_t rows,
                                                             int64_t cols, int64_t ld,
                                                             uint32_t *__restrict__ partials) {
    __shared__ uint32_t smem[4];
    uint32_t m = 0;
    for (int64_t r = blockIdx.x; r < rows; r += gridDim.x) {
        const uint16_t *row = x + r * ld;
        for (int64_t c = threadIdx.x; c < cols; c += kThreads) {
            const uint32_t v = row[c] & 0x7fffu;
            m = m > v ? m : v;
        }
    }
    m = block_max_u32(m, smem);
    if (threadIdx.x == 0) {
        partials[2 * blockIdx.x] = mag16_to_f32_bits<IS_BF16>(m);
        partials[2 * blockIdx.x + 1] = 0u;
    }
}

// fp32 input, contiguous and 16-byte aligned, viewed as n_vec 128-bit vectors.
__global__ __launch_bounds__(kThreads) void amax_flat_f32_kernel(const uint4 *__restrict__ x, int64_t n_vec,
                                                                 uint32_t *__restrict__ partials) {
    __shared__ uint32_t smem[4];
    const int64_t stride = (int64_t)gridDim.x * kThreads;
    uint32_t m = 0;
    auto take = [&](uint32_t u) {
        const uint32_t v = u & 0x7fffffffu;
        m = m > v ? m : v;
    };
    constexpr int U = 8;
    int64_t i = (int64_t)blockIdx.x * kThreads + threadIdx.x;
    for (; i + (U - 1) * stride < n_vec; i += U * stride) {
        uint4 v[U];
#pragma unroll
        for (int u = 0; u < U; ++u) v[u] = x[i + u * stride];
#pragma unroll
        for (int u = 0; u < U; ++u) take(v[u].x), take(v[u].y), take(v[u].z), take(v[u].w);
    }
    for (; i < n_vec; i += stride) {
        const uint4 v = x[i];
        take(v.x), take(v.y), take(v.z), take(v.w);
    }
    m = block_max_u32(m, smem);
    if (threadIdx.x == 0) {
        partials[2 * blockIdx.x] = m;
        partials[2 * blockIdx.x + 1] = 0u;
    }
}

// fp32 input, any strides: one workgroup per row, strided over the rows.
__global__ __launch_bounds__(kThreads) void amax_rows_f32_kernel(const uint32_t *__restrict__ x, int64_t rows,
                                                                 int64_t cols, int64_t ld,
                                                                 uint32_t *__restrict__ partials) {
    __shared__ uint32_t smem[4];
    uint32_t m = 0;
    for (int64_t r = blockIdx.x; r < rows; r += gridDim.x) {
        const uint32_t *row = x + r * ld;
        for (int64_t c = threadIdx.x; c < cols; c += kThreads) {
            const uint32_t v = row[c] & 0x7fffffffu;  // magnitudes order like their bit patterns
            m = m > v ? m : v;
        }
    }
    m = block_max_u32(m, smem);
    if (threadIdx.x == 0) {
        partials[2 * blockIdx.x] = m;
        partials[2 * blockIdx.x + 1] = 0u;
    }
}

// partials -> one f32 (single workgroup)
__global__ __launch_bounds__(kThreads) void amax_finalize_kernel(const uint32_t *__restrict__ partials, int n,
                                                                 float *__restrict__ amax) {
    __shared__ uint32_t smem[4];
    uint32_t m = 0;
    for (int i = threadIdx.x; i < n; i += kThreads) m = m > partials[2 * i] ? m : partials[2 * i];
    m = block_max_u32(m, smem);
    if (threadIdx.x == 0) *amax = u2f(m);
}

}  // namespace fos

// ---------------------------------------------------------------------------------------
// host side
// ---------------------------------------------------------------------------------------

using namespace fos;

extern "C" int64_t fos_padded_rows(int64_t rows) { return (rows + 127) / 128 * 128; }
extern "C" int64_t fos_padded_cols(int64_t cols) { return (cols + 63) / 64 * 64; }
extern "C" int64_t fos_padded_cols_for(int dtype, int64_t cols) {
    const int64_t mult = dtype == FOS_DTYPE_MXFP4 ? 128 : 64;  // four blocks of 32 / of 16
    return (cols + mult - 1) / mult * mult;
}

extern "C" size_t fos_quantize_workspace_bytes(int64_t, int64_t) { return 2 * kMaxPartials * sizeof(uint32_t); }

namespace {

// Launch pass 1; returns the number of partial maxima written to `partials`.
int launch_amax(const void *x, int x_type, int64_t rows, int64_t cols, int64_t ld, bool aligned, uint32_t *partials,
                hipStream_t s) {
    int n_partials;
    // bf16 / fp16: the scan that leaves the first units of a streaming pass 2 in L2 (tensors of 16 MiB and
    // more; window-rows per die = rows * cols / 2048, a step of the grid takes 32 * 64 of them)
    const int64_t n_winrows = cols % 2048 == 0 ? rows * (cols / 2048) : 0;
    if (x_type != FOS_T_F32 && ((uintptr_t)x & 15) == 0 && ld % 8 == 0 && n_winrows >= 4096 && n_winrows < (int64_t{1} << 31) &&
        tuning().amax_units >= 0) {
        const uint32_t win = (uint32_t)(cols / 2048), steps = (uint32_t)((n_winrows + 2047) / 2048);
        if (x_type == FOS_T_BF16)
            hipLaunchKernelGGL((amax_units_kernel<true>), dim3(256), dim3(kThreads), 0, s, (const uint16_t *)x, ld, win,
                               (uint32_t)n_winrows, steps, partials);
        else
            hipLaunchKernelGGL((amax_units_kernel<false>), dim3(256), dim3(kThreads), 0, s, (const uint16_t *)x, ld, win,
                               (uint32_t)n_winrows, steps, partials);
        return 256;
    }
    if (x_type != FOS_T_BF16 && ld == cols && ((uintptr_t)x & 15) == 0 && (rows * cols) % 8 == 0) {
        // contiguous: the flat scans (fp16 shares the bf16 one, magnitudes order like bit patterns)
        const int64_t n_vec = rows * cols / (x_type == FOS_T_F32 ? 4 : 8);
        const int64_t want = (n_vec + kThreads * 8 - 1) / (kThreads * 8);
        n_partials = (int)(want > 256 ? 256 : (want < 1 ? 1 : want));
        if (x_type == FOS_T_F32)
            hipLaunchKernelGGL(amax_flat_f32_kernel, dim3(n_partials), dim3(kThreads), 0, s, (const uint4 *)x, n_vec, partials);
        else
            hipLaunchKernelGGL((amax_flat_kernel<false>), dim3(n_partials), dim3(kThreads), 0, s, (const uint4 *)x, n_vec,
                               partials);
        return n_partials;
    }
    if (x_type != FOS_T_BF16) {
        n_partials = (int)(rows < kMaxPartials ? rows : kMaxPartials);
        if (x_type == FOS_T_F32)
            hipLaunchKernelGGL(amax_rows_f32_kernel, dim3(n_partials), dim3(kThreads), 0, s, (const uint32_t *)x, rows, cols, ld,
                               partials);
        else
            hipLaunchKernelGGL((amax_rows_kernel<false>), dim3(n_partials), dim3(kThreads), 0, s, (const uint16_t *)x, rows,
                               cols, ld, partials);
        return n_partials;
    }
    if (ld == cols && aligned) {
        const int64_t n_vec = rows * cols / 8;
        // each thread keeps 8 independent 128-bit loads in flight
        int64_t want = (n_vec + kThreads * 8 - 1) / (kThreads * 8);
        // one workgroup per compute unit reads fastest (128 MiB, inputs rotating through 512 MiB:
        // 21.6 us with 256 workgroups, 22.6 with 512, 26.9 with 1024 for the bare loads)
        int64_t cap = 256;
        if (const int forced = tuning().amax_grid) cap = forced > 0 && forced <= kMaxPartials ? forced : cap;
        n_partials = (int)(want > cap ? cap : (want < 1 ? 1 : want));
        hipLaunchKernelGGL((amax_flat_kernel<true>), dim3(n_partials), dim3(kThreads), 0, s, (const uint4 *)x, n_vec,
                           partials);
    } else {
        n_partials = (int)(rows < kMaxPartials ? rows : kMaxPartials);
        hipLaunchKernelGGL((amax_rows_kernel<true>), dim3(n_partials), dim3(kThreads), 0, s, (const uint16_t *)x, rows,
                           cols, ld, partials);
    }
    return n_partials;
}

template <int DT, int RULE, int ROUND>
void dispatch_2d(QuantParams &p, bool two_d, bool aligned, hipStream_t s) {
    if (two_d) launch_quantize<false, DT, RULE, ROUND, true>(p, aligned, s);
    else launch_quantize<false, DT, RULE, ROUND, false>(p, aligned, s);
}

// fp16 / fp32 inputs: the element-wise kernel, whatever the alignment
template <int DT, int RULE, int ROUND>
void launch_typed(QuantParams &p, bool two_d, hipStream_t s) {
    p.tiles_x = (int)(p.cols_p / 64);
    const dim3 grid((unsigned)((p.rows_p / 128) * p.tiles_x));
    if (two_d) hipLaunchKernelGGL((quantize_kernel<false, DT, RULE, ROUND, true, 1, false>), grid, dim3(kThreads), 0, s, p);
    else hipLaunchKernelGGL((quantize_kernel<false, DT, RULE, ROUND, false, 1, false>), grid, dim3(kThreads), 0, s, p);
}

template <int DT, int RULE>
void dispatch_round(QuantParams &p, int round_style, bool two_d, bool aligned, hipStream_t s) {
    if (p.x_type != FOS_T_BF16 && !(aligned && p.x_type == FOS_T_F16)) {
        if (round_style == FOS_ROUND_NEAREST) launch_typed<DT, RULE, FOS_ROUND_NEAREST>(p, two_d, s);
        else launch_typed<DT, RULE, FOS_ROUND_STOCHASTIC>(p, two_d, s);
        return;
    }
    if (round_style == FOS_ROUND_NEAREST) {
        // NVFP4 round-to-nearest lives in fos_quantize_fast.hip
        if constexpr (DT == FOS_DTYPE_NVFP4) {
            launch_quantize_nvfp4_fast(p, RULE, two_d, aligned, false, s);
        } else if constexpr (RULE == FOS_RULE_MSE) {
            // IF4 with the MSE rule: fast block formulation, on the streaming kernel for aligned 1x16
            // inputs and inside the generic kernel's mapping otherwise
            if (two_d && aligned && !p.pseudo_out) launch_quantize_if4_mse_tiles(p, s);
            else if (two_d) launch_quantize<true, DT, RULE, FOS_ROUND_NEAREST, true>(p, aligned, s);
            else if (aligned) launch_quantize_if4_mse_rows(p, s);
            else launch_quantize<true, DT, RULE, FOS_ROUND_NEAREST, false>(p, aligned, s);
        } else {
            dispatch_2d<DT, RULE, FOS_ROUND_NEAREST>(p, two_d, aligned, s);
        }
    } else {
        // ... and so does stochastic rounding of aligned inputs (the unbiased style differs
        // in the host-computed constants only; the MSE rule decides through its certified
        // shortcut there and the other adaptive rules stay with the generic kernel)
        if constexpr (DT == FOS_DTYPE_NVFP4) {
            constexpr bool kShortcut = RULE == FOS_RULE_MSE || RULE == FOS_RULE_STATIC_6 || RULE == FOS_RULE_STATIC_4;
            if (aligned && (round_style == FOS_ROUND_STOCHASTIC || kShortcut)) {
                launch_quantize_nvfp4_fast(p, RULE, two_d, aligned, true, s);
                return;
            }
        }
        dispatch_2d<DT, RULE, FOS_ROUND_STOCHASTIC>(p, two_d, aligned, s);
    }
}

}  // namespace

extern "C" int fos_amax(const void *x, int x_type, int64_t rows, int64_t cols, int64_t ld, float *amax,
                        void *workspace, size_t workspace_bytes, fos_stream_t stream) {
    if (!x || !amax) return FOS_E_NULL_POINTER;
    if (rows <= 0 || cols <= 0 || ld < cols) return FOS_E_BAD_SHAPE;
    if (x_type != FOS_T_BF16 && x_type != FOS_T_F16 && x_type != FOS_T_F32) return FOS_E_UNSUPPORTED;
    if (!workspace || workspace_bytes < fos_quantize_workspace_bytes(rows, cols)) return FOS_E_WORKSPACE;
    if (((uintptr_t)x & (x_type == FOS_T_F32 ? 3 : 1)) || ((uintptr_t)workspace & 3) || ((uintptr_t)amax & 3)) return FOS_E_BAD_ALIGNMENT;
    hipStream_t s = (hipStream_t)stream;
    const bool aligned = (((uintptr_t)x & 15) == 0) && (ld % 8 == 0) && (cols % 16 == 0);
    uint32_t *partials = (uint32_t *)workspace;
    const int n = launch_amax(x, x_type, rows, cols, ld, aligned, partials, s);
    hipLaunchKernelGGL(amax_finalize_kernel, dim3(1), dim3(kThreads), 0, s, partials, n, amax);
    return hipGetLastError() == hipSuccess ? FOS_OK : FOS_E_LAUNCH;
}

// Inputs up to this many elements (32 KiB) are quantized in one launch, in which every workgroup
// scans the whole tensor for its maximum.  The scan runs at what one compute unit reads from
// L2, so it stops paying early: per call inside a HIP graph, one launch against two, 1 x 4096
// 5.0 against 6.5 us, 16 x 1024 6.2 against 6.9, 16 x 2048 7.35 against 7.3, 16 x 4096 10.1 against 7.3.
constexpr int64_t kFusedAmaxElements = 16384;
// Outside a stream capture the host is the slower side at these sizes (a launch costs it about
// 3 us; through the Python frontend 16 x 4096 takes 16 us per call in one launch and 19 in two,
// more than either form on the GPU), so eager calls keep the single launch up to 128 KiB.
constexpr int64_t kFusedAmaxElementsEager = 65536;

static bool stream_is_capturing(hipStream_t s) {
    hipStreamCaptureStatus status = hipStreamCaptureStatusNone;
    if (hipStreamIsCapturing(s, &status) != hipSuccess) {
        (void)hipGetLastError();  // the query's own failure must not read as a failed launch later
        return true;
    }
    return status != hipStreamCaptureStatusNone;
}

// Which combinations the fused quantize -> dequantize kernels cover (alignment aside): NVFP4 with round to
// nearest (bf16 with either block shape, fp16 with 1x16 blocks), NVFP4 with a stochastic style on bf16
// (the unbiased style with the rules whose decision the streaming kernels make), IF4 with the MSE
// rule on bf16, round to nearest, 1x16 blocks.
extern "C" int fos_pseudo_quantize_is_fused(int x_type, int dtype, int rule, int round_style, int block2d) {
    const bool rtn = round_style == FOS_ROUND_NEAREST;
    if (dtype == FOS_DTYPE_NVFP4 && rtn) return x_type == FOS_T_BF16 || (x_type == FOS_T_F16 && !block2d);
    if (x_type != FOS_T_BF16) return 0;
    if (dtype == FOS_DTYPE_IF4) return rtn && rule == FOS_RULE_MSE && !block2d;
    if (dtype != FOS_DTYPE_NVFP4) return 0;
    if (round_style == FOS_ROUND_STOCHASTIC) return 1;
    return round_style == FOS_ROUND_STOCHASTIC_UNBIASED &&
           (rule == FOS_RULE_MSE || rule == FOS_RULE_STATIC_6 || rule == FOS_RULE_STATIC_4);
}

// Shared body of fos_quantize and fos_pseudo_quantize (pseudo_out != null: bf16 round trip
// instead of codes / scales).
static int quantize_impl(const void *x, int x_type, int64_t rows, int64_t cols, int64_t ld,
                         int dtype, int rule, int round_style, int block2d,
                         uint64_t seed, uint64_t offset, int sf_layout,
                         uint8_t *codes, uint8_t *sf, float *amax, int amax_is_input,
                         void *workspace, size_t workspace_bytes, fos_stream_t stream,
                         uint16_t *pseudo_out, int64_t ldo, const uint64_t *key = nullptr, int ready_partials = 0) {
    if (!x || !amax || (!pseudo_out && (!codes || !sf))) return FOS_E_NULL_POINTER;
    if ((uintptr_t)key & 7) return FOS_E_BAD_ALIGNMENT;
    if (dtype == FOS_DTYPE_MXFP4) {
        // one streaming kernel; no tensor maximum, no workspace
        if (rows <= 0 || cols <= 0 || ld < cols) return FOS_E_BAD_SHAPE;
        if ((x_type != FOS_T_BF16 && x_type != FOS_T_F16 && x_type != FOS_T_F32) || pseudo_out || block2d ||
            round_style != FOS_ROUND_NEAREST || amax_is_input || (rule != FOS_RULE_STATIC_6 && rule != FOS_RULE_STATIC_4))
            return FOS_E_UNSUPPORTED;
        if (sf_layout != FOS_SF_LINEAR && sf_layout != FOS_SF_TILED_128X4) return FOS_E_UNSUPPORTED;
        if (((uintptr_t)x & (x_type == FOS_T_F32 ? 3 : 1)) || ((uintptr_t)codes & 15) || ((uintptr_t)sf & 7) || ((uintptr_t)amax & 3))
            return FOS_E_BAD_ALIGNMENT;
        return launch_quantize_mxfp4(x, x_type, rows, cols, ld, rule, sf_layout, codes, sf, amax, (hipStream_t)stream);
    }
    if (rows <= 0 || cols <= 0 || ld < cols) return FOS_E_BAD_SHAPE;
    if (x_type != FOS_T_BF16 && x_type != FOS_T_F16 && x_type != FOS_T_F32) return FOS_E_UNSUPPORTED;
    if (pseudo_out && !fos_pseudo_quantize_is_fused(x_type, dtype, rule, round_style, block2d)) return FOS_E_UNSUPPORTED;
    if (dtype != FOS_DTYPE_NVFP4 && dtype != FOS_DTYPE_IF4) return FOS_E_UNSUPPORTED;
    if (rule < FOS_RULE_STATIC_6 || rule > FOS_RULE_ABS_MAX) return FOS_E_UNSUPPORTED;
    if (round_style < FOS_ROUND_NEAREST || round_style > FOS_ROUND_STOCHASTIC_UNBIASED) return FOS_E_UNSUPPORTED;
    if (dtype == FOS_DTYPE_IF4 && (rule == FOS_RULE_STATIC_6 || rule == FOS_RULE_STATIC_4)) return FOS_E_UNSUPPORTED;
    if (sf_layout != FOS_SF_LINEAR && sf_layout != FOS_SF_TILED_128X4) return FOS_E_UNSUPPORTED;
    if (!workspace || workspace_bytes < fos_quantize_workspace_bytes(rows, cols)) return FOS_E_WORKSPACE;
    if (((uintptr_t)x & (x_type == FOS_T_F32 ? 3 : 1)) || ((uintptr_t)codes & 7) || ((uintptr_t)sf & 3) ||
        ((uintptr_t)workspace & 3) || ((uintptr_t)amax & 3))
        return FOS_E_BAD_ALIGNMENT;
    const int64_t rows_p = fos_padded_rows(rows), cols_p = fos_padded_cols(cols);
    if (rows_p * (cols_p / 64) > 0x7fffffffLL) return FOS_E_BAD_SHAPE;

    hipStream_t s = (hipStream_t)stream;
    uint32_t *partials = (uint32_t *)workspace;
    // (fp32 inputs, and fp16 ones outside the case below, take the element-wise kernel: they are treated as
    // unaligned throughout)
    // The streaming kernels address a 128-row tile with 32-bit byte offsets: a row pitch of 2^23
    // elements or more (16 MiB rows) takes the element-wise kernel like an unaligned input.
    constexpr int64_t kMaxPitch = int64_t{1} << 23;
    // fp16 input has a streaming form for NVFP4 codes with 1x16 blocks and round to nearest
    const bool f16_streams = x_type == FOS_T_F16 && dtype == FOS_DTYPE_NVFP4 && round_style == FOS_ROUND_NEAREST && !block2d;
    const bool aligned = (x_type == FOS_T_BF16 || f16_streams) && (((uintptr_t)x & 15) == 0) && (ld % 8 == 0) && (cols % 16 == 0) && ld < kMaxPitch;
    if (pseudo_out) {
        // only the streaming kernels have the fused epilogue
        if (!aligned) return FOS_E_UNSUPPORTED;
        if (ldo < cols || ldo >= kMaxPitch) return FOS_E_BAD_SHAPE;
        if (((uintptr_t)pseudo_out & 15) || (ldo % 8 != 0)) return FOS_E_BAD_ALIGNMENT;
    }

    QuantParams p;
    p.pseudo_out = pseudo_out;
    p.ldo = ldo;
    p.x = (const uint16_t *)x;
    p.x_type = x_type;
    {
        const int64_t esize = x_type == FOS_T_F32 ? 4 : 2;
        p.x_vec = x_type != FOS_T_BF16 && ((uintptr_t)x & 15) == 0 && (ld * esize) % 16 == 0 && cols % 16 == 0;
    }
    p.rows = rows; p.cols = cols; p.ld = ld;
    p.rows_p = rows_p; p.cols_p = cols_p;
    p.codes = codes; p.sf = sf;
    p.seed = seed; p.offset = offset;
    p.key = key;
    p.sf_layout = sf_layout;

    if (ready_partials > 0) {
        // the producer of x (fos_transform) has left its per-workgroup maxima in the workspace
        p.partials = partials;
        p.n_partials = ready_partials;
        p.amax_out = amax;
    } else if (amax_is_input) {
        p.partials = (const uint32_t *)amax;
        p.n_partials = 0;
        p.amax_out = nullptr;
    } else if (aligned && x_type == FOS_T_BF16 && ld == cols &&
               (rows * cols <= kFusedAmaxElements || (rows * cols <= kFusedAmaxElementsEager && !stream_is_capturing(s)))) {
        // decode-sized input: one launch, every workgroup of pass 2 finds the maximum itself
        p.partials = partials;
        p.n_partials = -1;
        p.amax_out = amax;
    } else {
        p.partials = partials;
        p.n_partials = launch_amax(x, x_type, rows, cols, ld, aligned, partials, s);
        p.amax_out = amax;
    }

    if (tuning().quant_passes == 1) return hipGetLastError() == hipSuccess ? FOS_OK : FOS_E_LAUNCH;  // timing runs: pass 1 alone

    // (qmax, smax): static_6 (6,448); static_4 (4,448); adaptive NVFP4 (6,256); IF4 (6,448).
    const double adj = round_style == FOS_ROUND_STOCHASTIC_UNBIASED ? 16.0 / 17.0 : 1.0;
    const double qmax = rule == FOS_RULE_STATIC_4 ? 4.0 : 6.0;
    const bool is_static = rule == FOS_RULE_STATIC_6 || rule == FOS_RULE_STATIC_4;
    const double smax = (dtype == FOS_DTYPE_IF4 || is_static) ? 448.0 : 256.0;
    p.c = (float)(qmax * smax * adj);
    p.qdiv = (float)(qmax * adj);
    p.errdiv = dtype == FOS_DTYPE_IF4 ? (float)(6.0 * 448.0 * adj) : (float)(6.0 * 256.0 * adj);

    const bool two_d = block2d != 0;
    if (dtype == FOS_DTYPE_IF4) {
        switch (rule) {
            case FOS_RULE_MAE: dispatch_round<FOS_DTYPE_IF4, FOS_RULE_MAE>(p, round_style, two_d, aligned, s); break;
            case FOS_RULE_MSE: dispatch_round<FOS_DTYPE_IF4, FOS_RULE_MSE>(p, round_style, two_d, aligned, s); break;
            default: dispatch_round<FOS_DTYPE_IF4, FOS_RULE_ABS_MAX>(p, round_style, two_d, aligned, s); break;
        }
    } else {
        switch (rule) {
            case FOS_RULE_STATIC_6:
            case FOS_RULE_STATIC_4:
                // the two static rules differ only in the host-computed constants
                dispatch_round<FOS_DTYPE_NVFP4, FOS_RULE_STATIC_6>(p, round_style, two_d, aligned, s);
                break;
            case FOS_RULE_MAE: dispatch_round<FOS_DTYPE_NVFP4, FOS_RULE_MAE>(p, round_style, two_d, aligned, s); break;
            case FOS_RULE_MSE: dispatch_round<FOS_DTYPE_NVFP4, FOS_RULE_MSE>(p, round_style, two_d, aligned, s); break;
            default: dispatch_round<FOS_DTYPE_NVFP4, FOS_RULE_ABS_MAX>(p, round_style, two_d, aligned, s); break;
        }
    }
    return hipGetLastError() == hipSuccess ? FOS_OK : FOS_E_LAUNCH;
}

extern "C" int fos_quantize(const void *x, int x_type, int64_t rows, int64_t cols, int64_t ld,
                            int dtype, int rule, int round_style, int block2d,
                            uint64_t seed, uint64_t offset, int sf_layout,
                            uint8_t *codes, uint8_t *sf, float *amax, int amax_is_input,
                            void *workspace, size_t workspace_bytes, fos_stream_t stream) {
    return quantize_impl(x, x_type, rows, cols, ld, dtype, rule, round_style, block2d, seed, offset, sf_layout, codes, sf,
                         amax, amax_is_input, workspace, workspace_bytes, stream, nullptr, 0);
}

extern "C" int fos_quantize_devkey(const void *x, int x_type, int64_t rows, int64_t cols, int64_t ld,
                                   int dtype, int rule, int round_style, int block2d,
                                   const uint64_t *key, int sf_layout,
                                   uint8_t *codes, uint8_t *sf, float *amax, int amax_is_input,
                                   void *workspace, size_t workspace_bytes, fos_stream_t stream) {
    if (!key) return FOS_E_NULL_POINTER;
    if (dtype == FOS_DTYPE_MXFP4) return FOS_E_UNSUPPORTED;  // (no stochastic style there)
    return quantize_impl(x, x_type, rows, cols, ld, dtype, rule, round_style, block2d, 0, 0, sf_layout, codes, sf,
                         amax, amax_is_input, workspace, workspace_bytes, stream, nullptr, 0, key);
}

namespace fos {
int transform_impl(const void *x, int x_type, int64_t rows, int64_t cols, int64_t ld, int transpose, int rht, void *y, int64_t ldy,
                   float *amax, int *n_partials, void *workspace, size_t workspace_bytes, fos_stream_t stream);
}

extern "C" int fos_transform_quantize(const void *x, int x_type, int64_t rows, int64_t cols, int64_t ld,
                                      int transpose, int rht, void *y, int64_t ldy,
                                      int dtype, int rule, int round_style, int block2d,
                                      uint64_t seed, uint64_t offset, int sf_layout,
                                      uint8_t *codes, uint8_t *sf, float *amax,
                                      void *workspace, size_t workspace_bytes, fos_stream_t stream) {
    if (!amax || !codes || !sf) return FOS_E_NULL_POINTER;
    if (dtype != FOS_DTYPE_NVFP4 && dtype != FOS_DTYPE_IF4) return FOS_E_UNSUPPORTED;  // (MXFP4 has no tensor maximum to hand over)
    int n = 0;
    const int rc = fos::transform_impl(x, x_type, rows, cols, ld, transpose, rht, y, ldy, nullptr, &n, workspace, workspace_bytes, stream);
    if (rc != FOS_OK) return rc;
    const int64_t out_rows = transpose ? cols : rows, out_cols = transpose ? rows : cols;
    // with rht a ragged last group of 16 holds values in all its places: the padded width is what gets quantized
    const int64_t q_cols = rht ? (out_cols + 15) / 16 * 16 : out_cols;
    return quantize_impl(y, x_type, out_rows, q_cols, ldy, dtype, rule, round_style, block2d, seed, offset, sf_layout, codes, sf,
                         amax, 0, workspace, workspace_bytes, stream, nullptr, 0, nullptr, n);
}

extern "C" int fos_pseudo_quantize(const void *x, int x_type, int64_t rows, int64_t cols, int64_t ld,
                                   int dtype, int rule, int round_style, int block2d,
                                   void *out, int64_t ldo, float *amax, int amax_is_input,
                                   void *workspace, size_t workspace_bytes, fos_stream_t stream) {
    if (!out) return FOS_E_NULL_POINTER;
    return quantize_impl(x, x_type, rows, cols, ld, dtype, rule, round_style, block2d, 0, 0, FOS_SF_LINEAR, nullptr, nullptr,
                         amax, amax_is_input, workspace, workspace_bytes, stream, static_cast<uint16_t *>(out), ldo);
}

extern "C" int fos_pseudo_quantize_keyed(const void *x, int x_type, int64_t rows, int64_t cols, int64_t ld,
                                         int dtype, int rule, int round_style, int block2d, uint64_t seed, uint64_t offset,
                                         void *out, int64_t ldo, float *amax, int amax_is_input,
                                         void *workspace, size_t workspace_bytes, fos_stream_t stream) {
    if (!out) return FOS_E_NULL_POINTER;
    return quantize_impl(x, x_type, rows, cols, ld, dtype, rule, round_style, block2d, seed, offset, FOS_SF_LINEAR, nullptr, nullptr,
                         amax, amax_is_input, workspace, workspace_bytes, stream, static_cast<uint16_t *>(out), ldo);
}

// Device address of `scratch` on the current device, looked up once per device.
namespace {
constexpr int kMaxDevices = 64;
std::atomic<void *> g_scratch_ptr[kMaxDevices];
}  // namespace

extern "C" int fos_quantize_static(const void *x, int x_type, int64_t rows, int64_t cols, int64_t ld,
                                   int dtype, int rule, int round_style, int block2d,
                                   uint64_t seed, uint64_t offset, int sf_layout,
                                   uint8_t *codes, uint8_t *sf, float *amax, int amax_is_input,
                                   fos_stream_t stream) {
    if (rows <= 0 || cols <= 0) return FOS_E_BAD_SHAPE;
    if (fos_quantize_workspace_bytes(rows, cols) > kStaticScratchBytes) return FOS_E_WORKSPACE;  // beyond the built-in scratch
    int dev = -1;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return FOS_E_LAUNCH;
    void *ptr = g_scratch_ptr[dev].load(std::memory_order_acquire);
    if (!ptr) {
        // every GPU holds its own copy of the array at its own address
        if (hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch)) != hipSuccess || !ptr) return FOS_E_LAUNCH;
        g_scratch_ptr[dev].store(ptr, std::memory_order_release);
    }
    return quantize_impl(x, x_type, rows, cols, ld, dtype, rule, round_style, block2d, seed, offset, sf_layout, codes, sf,
                         amax, amax_is_input, ptr, kStaticScratchBytes, stream, nullptr, 0);
}
