// PyTorch binding of the gfx950 library: the `fouroversix::*` operators of the reference
// (src/fouroversix/csrc/bindings.cpp:26-35) registered for the GPU dispatch key, each a thin wrapper that
// checks its arguments, allocates the outputs and makes one call through the C ABI
// (include/fouroversix_hip.h) on torch's current stream.  The same functions are exported to Python
// directly (module `fouroversix_amd._C`) for the frontends' own calls: at decode sizes the dispatcher's
// boxing costs as much as the kernels take.
//
// Operator names and schemas are the reference's; `quantize_ex`, `pseudo_quantize`, `transform`,
// `dequantize`, `gemm_nvfp4_amax` and `gemm_alpha` are additions that carry what the reference's native
// ops do not have (formats, dither key, scale layout, in-kernel output scale, recorded output maximum).
#include <ATen/ATen.h>
#include <ATen/hip/impl/HIPGuardImplMasqueradingAsCUDA.h>
#include <ATen/hip/impl/HIPStreamMasqueradingAsCUDA.h>
#include <c10/hip/HIPGraphsC10Utils.h>
#include <torch/extension.h>
#include <torch/library.h>

#include <mutex>
#include <tuple>
#include <unordered_map>

#include "fouroversix_hip.h"

namespace {

using at::Tensor;
// (PyTorch on ROCm names its GPU device type "cuda": the guard and stream types that go with it)
using DeviceGuard = c10::hip::HIPGuardMasqueradingAsCUDA;

constexpr int64_t kMxfp4 = FOS_DTYPE_MXFP4;

void check(int code, const char *what) {
    TORCH_CHECK(code == FOS_OK, what, ": ", fos_error_string(code), " (code ", code, ")");
}

int type_id(at::ScalarType t, const char *what) {
    switch (t) {
        case at::kBFloat16: return FOS_T_BF16;
        case at::kHalf: return FOS_T_F16;
        case at::kFloat: return FOS_T_F32;
        default: TORCH_CHECK(false, what, " must be bfloat16, float16 or float32, got ", t);
    }
    return -1;
}

void require_gpu(const Tensor &t, const char *name) {
    TORCH_CHECK_VALUE(t.is_cuda(), name, " must live on the GPU (got ", t.device(), "); this library has no CPU path");
}

fos_stream_t current_stream(const Tensor &t) { return c10::hip::getCurrentHIPStreamMasqueradingAsCUDA(t.get_device()).stream(); }

std::pair<int64_t, int64_t> padded(int64_t rows, int64_t cols, int64_t dtype) {
    return {fos_padded_rows(rows), fos_padded_cols_for((int)dtype, cols)};
}

// Pass-1 workspace (8 KiB), one per (device, stream): calls on one stream are ordered, so they can share
// it; calls on different streams must not.  While a stream is being captured into a graph the workspace
// comes from the allocator instead (the graph's private pool keeps it for the graph's lifetime; a cached
// one would be shared by every graph captured on that stream and pinned after they are gone).
Tensor quantize_workspace(const Tensor &like, fos_stream_t stream) {
    static const int64_t bytes = (int64_t)fos_quantize_workspace_bytes(1, 1);
    const auto opts = like.options().dtype(at::kByte);
    if (c10::hip::currentStreamCaptureStatusMayInitCtx() != c10::hip::CaptureStatus::None) return at::empty({bytes}, opts);
    static std::mutex mutex;
    static std::unordered_map<uint64_t, Tensor> cache;
    const uint64_t key = ((uint64_t)(uintptr_t)stream << 8) ^ (uint64_t)like.get_device();
    std::lock_guard<std::mutex> lock(mutex);
    auto it = cache.find(key);
    if (it == cache.end()) it = cache.emplace(key, at::empty({bytes}, opts)).first;
    return it->second;
}

Tensor amax_buffer(const c10::optional<Tensor> &amax, const Tensor &x) {
    if (amax.has_value()) return amax->reshape({1}).to(x.device(), at::kFloat).contiguous();
    return at::empty({1}, x.options().dtype(at::kFloat));
}

// quantize_ex(x, dtype, selection_rule, round_style, is_2d, seed, offset, sf_layout, amax?, key?) -> (values, scale_factors, amax)
// key: int64[2] on x's device holding {seed, offset}, read by the kernels when they run (seed / offset are then ignored)
std::tuple<Tensor, Tensor, Tensor> quantize_ex(const Tensor &x, int64_t dtype, int64_t rule, int64_t round_style, bool is_2d,
                                               int64_t seed, int64_t offset, int64_t sf_layout, const c10::optional<Tensor> &amax,
                                               const c10::optional<Tensor> &key) {
    TORCH_CHECK(x.dim() == 2, "quantize: x must be 2-D");
    const int xt = type_id(x.scalar_type(), "quantize: x");
    TORCH_CHECK(x.stride(-1) == 1, "quantize: x must be contiguous on the last dim");
    require_gpu(x, "x");
    const int64_t rows = x.size(0), cols = x.size(1);
    const auto [rows_p, cols_p] = padded(rows, cols, dtype);
    const auto bytes = x.options().dtype(at::kByte);
    Tensor values = at::empty({rows_p, cols_p / 2}, bytes);
    Tensor sf = dtype == kMxfp4 ? at::empty({rows_p * cols_p / 32}, x.options().dtype(at::kFloat8_e8m0fnu))
                                : at::empty({rows_p * cols_p / 16}, x.options().dtype(at::kFloat8_e4m3fn));
    if (rows == 0 || cols == 0) {
        values.zero_();
        sf.view(at::kByte).zero_();
        return {values, sf, at::full({1}, dtype == kMxfp4 ? 1.0 : 0.0, x.options().dtype(at::kFloat))};
    }
    Tensor amax_buf = amax_buffer(amax, x);
    const DeviceGuard guard(x.device());
    const fos_stream_t stream = current_stream(x);
    Tensor ws = quantize_workspace(x, stream);
    if (key.has_value()) {
        TORCH_CHECK(key->scalar_type() == at::kLong && key->numel() == 2 && key->is_contiguous() && key->device() == x.device(),
                    "quantize: key must be a contiguous int64[2] tensor on x's device");
        check(fos_quantize_devkey(x.data_ptr(), xt, rows, cols, x.stride(0), (int)dtype, (int)rule, (int)round_style, is_2d ? 1 : 0,
                                  reinterpret_cast<const uint64_t *>(key->data_ptr<int64_t>()), (int)sf_layout, values.data_ptr<uint8_t>(),
                                  static_cast<uint8_t *>(sf.data_ptr()), amax_buf.data_ptr<float>(), amax.has_value() ? 1 : 0,
                                  ws.data_ptr(), (size_t)ws.numel(), stream),
              "fouroversix::quantize");
        return {values, sf, amax_buf};
    }
    check(fos_quantize(x.data_ptr(), xt, rows, cols, x.stride(0), (int)dtype, (int)rule, (int)round_style, is_2d ? 1 : 0,
                       (uint64_t)seed, (uint64_t)offset, (int)sf_layout, values.data_ptr<uint8_t>(),
                       static_cast<uint8_t *>(sf.data_ptr()), amax_buf.data_ptr<float>(), amax.has_value() ? 1 : 0,
                       ws.data_ptr(), (size_t)ws.numel(), stream),
          "fouroversix::quantize");
    return {values, sf, amax_buf};
}

// True when the library has a fused quantize -> dequantize kernel for this call.
bool pseudo_quantize_is_fused(const Tensor &x, int64_t dtype, int64_t rule, int64_t round_style, bool is_2d) {
    if (x.dim() != 2 || (x.scalar_type() != at::kBFloat16 && x.scalar_type() != at::kHalf)) return false;
    return fos_pseudo_quantize_is_fused(x.scalar_type() == at::kHalf ? FOS_T_F16 : FOS_T_BF16, (int)dtype, (int)rule, (int)round_style,
                                        is_2d ? 1 : 0) &&
           x.numel() > 0 && x.stride(-1) == 1 && x.size(1) % 16 == 0 && x.stride(0) % 8 == 0 &&
           x.stride(0) < (int64_t(1) << 23)  // (the streaming kernels' 32-bit tile offsets)
           && reinterpret_cast<uintptr_t>(x.data_ptr()) % 16 == 0;
}

Tensor pseudo_quantize(const Tensor &x, int64_t dtype, int64_t rule, int64_t round_style, bool is_2d, const c10::optional<Tensor> &amax,
                       int64_t seed, int64_t offset) {
    TORCH_CHECK(pseudo_quantize_is_fused(x, dtype, rule, round_style, is_2d),
                "pseudo_quantize: no fused kernel for these arguments (quantize, then dequantize)");
    require_gpu(x, "x");
    const int64_t rows = x.size(0), cols = x.size(1);
    Tensor out = at::empty({rows, cols}, x.options());
    Tensor amax_buf = amax_buffer(amax, x);
    const DeviceGuard guard(x.device());
    const fos_stream_t stream = current_stream(x);
    Tensor ws = quantize_workspace(x, stream);
    check(fos_pseudo_quantize_keyed(x.data_ptr(), x.scalar_type() == at::kHalf ? FOS_T_F16 : FOS_T_BF16, rows, cols, x.stride(0), (int)dtype,
                                    (int)rule, (int)round_style, is_2d ? 1 : 0, (uint64_t)seed, (uint64_t)offset, out.data_ptr(), cols,
                                    amax_buf.data_ptr<float>(), amax.has_value() ? 1 : 0, ws.data_ptr(), (size_t)ws.numel(), stream),
          "fouroversix::pseudo_quantize");
    return out;
}

// (y, amax): y = RHT(x^T) as the reference forms it before scaling, amax = max|y|
std::tuple<Tensor, Tensor> transform(const Tensor &x_in, bool transpose, bool rht) {
    TORCH_CHECK(x_in.dim() == 2 && (x_in.scalar_type() == at::kBFloat16 || x_in.scalar_type() == at::kHalf || x_in.scalar_type() == at::kFloat),
                "transform: x must be a 2-D bfloat16, float16 or float32 tensor");
    require_gpu(x_in, "x");
    const Tensor x = x_in.stride(-1) == 1 ? x_in : x_in.contiguous();
    const int64_t rows = x.size(0), cols = x.size(1);
    const int64_t out_rows = transpose ? cols : rows, out_cols = transpose ? rows : cols;
    // y is written in whole groups of 16 (zeros complete a ragged last group; with rht that group then holds
    // values in all 16 places, so the padded width is what gets quantized)
    const int64_t width = (out_cols + 15) / 16 * 16;
    Tensor y = at::empty({out_rows, width}, x.options());
    Tensor amax = at::empty({1}, x.options().dtype(at::kFloat));
    const DeviceGuard guard(x.device());
    const fos_stream_t stream = current_stream(x);
    Tensor ws = quantize_workspace(x, stream);
    check(fos_transform(x.data_ptr(), type_id(x.scalar_type(), "transform: x"), rows, cols, x.stride(0), transpose ? 1 : 0, rht ? 1 : 0,
                        y.data_ptr(), y.stride(0), amax.data_ptr<float>(), ws.data_ptr(), (size_t)ws.numel(), stream),
          "fouroversix::transform");
    if (!rht && width != out_cols) y = y.slice(1, 0, out_cols);
    return {y, amax};
}

// transform, then quantize_ex of its result, in one call into the library (one small kernel and one dispatch less):
// (values, scale_factors, amax) of the transformed tensor
std::tuple<Tensor, Tensor, Tensor> transform_quantize(const Tensor &x_in, bool transpose, bool rht, int64_t dtype, int64_t rule,
                                                      int64_t round_style, bool is_2d, int64_t seed, int64_t offset, int64_t sf_layout) {
    TORCH_CHECK(x_in.dim() == 2 && (x_in.scalar_type() == at::kBFloat16 || x_in.scalar_type() == at::kHalf || x_in.scalar_type() == at::kFloat),
                "transform_quantize: x must be a 2-D bfloat16, float16 or float32 tensor");
    TORCH_CHECK(x_in.numel() > 0 && (transpose || rht), "transform_quantize: a non-empty tensor and at least one of transpose / rht");
    require_gpu(x_in, "x");
    const Tensor x = x_in.stride(-1) == 1 ? x_in : x_in.contiguous();
    const int64_t rows = x.size(0), cols = x.size(1);
    const int64_t out_rows = transpose ? cols : rows, out_cols = transpose ? rows : cols;
    const int64_t width = (out_cols + 15) / 16 * 16;
    Tensor y = at::empty({out_rows, width}, x.options());
    const auto [rows_p, cols_p] = padded(out_rows, rht ? width : out_cols, dtype);
    const auto bytes = x.options().dtype(at::kByte);
    Tensor values = at::empty({rows_p, cols_p / 2}, bytes);
    Tensor sf = at::empty({rows_p * cols_p / 16}, x.options().dtype(at::kFloat8_e4m3fn));
    Tensor amax = at::empty({1}, x.options().dtype(at::kFloat));
    const DeviceGuard guard(x.device());
    const fos_stream_t stream = current_stream(x);
    Tensor ws = quantize_workspace(x, stream);
    check(fos_transform_quantize(x.data_ptr(), type_id(x.scalar_type(), "transform_quantize: x"), rows, cols, x.stride(0), transpose ? 1 : 0,
                                 rht ? 1 : 0, y.data_ptr(), y.stride(0), (int)dtype, (int)rule, (int)round_style, is_2d ? 1 : 0,
                                 (uint64_t)seed, (uint64_t)offset, (int)sf_layout, values.data_ptr<uint8_t>(),
                                 static_cast<uint8_t *>(sf.data_ptr()), amax.data_ptr<float>(), ws.data_ptr(), (size_t)ws.numel(), stream),
          "fouroversix::transform_quantize");
    return {values, sf, amax};
}

// The reference's schema (csrc/bindings.cpp:28): NVFP4 only; `rbits` seeds the stochastic style.
std::tuple<Tensor, Tensor, Tensor> quantize_ref(const Tensor &x, bool is_nvfp4, bool is_rtn, bool is_rht, bool is_2d, bool is_transpose,
                                                int64_t selection_rule, int64_t rbits) {
    TORCH_CHECK(is_nvfp4, "quantize: only the NVFP4 format is implemented by this op (use quantize_ex for IF4)");
    TORCH_CHECK(selection_rule >= 0 && selection_rule <= 4, "Invalid selection_rule: ", selection_rule);
    // the reference's native op takes fp16 and bf16 (csrc/quantize/fp4_quant.cu:134-136)
    TORCH_CHECK(x.scalar_type() == at::kHalf || x.scalar_type() == at::kBFloat16, "quantize: x must be bfloat16 or float16, got ",
                x.scalar_type());
    const int64_t seed = rbits < 0 ? 0 : rbits;
    if (is_rht || is_transpose)
        return transform_quantize(x, is_transpose, is_rht, FOS_DTYPE_NVFP4, selection_rule, is_rtn ? 0 : 1, is_2d, seed, 0, FOS_SF_TILED_128X4);
    return quantize_ex(x, FOS_DTYPE_NVFP4, selection_rule, is_rtn ? 0 : 1, is_2d, seed, 0, FOS_SF_TILED_128X4, c10::nullopt, c10::nullopt);
}

// Operand checks of the reference's GEMM op (csrc/include/element_traits.hpp:122-170, csrc/fp4_gemm.cu:105-107).
void check_gemm_operands(const Tensor &a, const Tensor &b, const Tensor &a_sf, const Tensor &b_sf, const Tensor *scales[], int n_scales,
                         const char *scale_names[]) {
    const Tensor *all[4] = {&a, &b, &a_sf, &b_sf};
    const char *names[4] = {"A", "B", "A_sf", "B_sf"};
    for (int i = 0; i < 4 + n_scales; ++i) {
        const Tensor &t = i < 4 ? *all[i] : *scales[i - 4];
        const char *name = i < 4 ? names[i] : scale_names[i - 4];
        require_gpu(t, name);
        TORCH_CHECK(t.is_contiguous(), "gemm: ", name, " must be contiguous");
        TORCH_CHECK(t.device() == a.device(), "gemm: all operands must be on the same GPU");
    }
    TORCH_CHECK(a.scalar_type() == at::kByte && b.scalar_type() == at::kByte, "A and B must be uint8");
    TORCH_CHECK(a.dim() == 2 && b.dim() == 2, "A and B must be 2D");
    TORCH_CHECK(a_sf.scalar_type() == at::kFloat8_e4m3fn && b_sf.scalar_type() == at::kFloat8_e4m3fn, "A_sf and B_sf must be Float8_e4m3fn");
    const int64_t m = a.size(0), ka = a.size(1) * 2, n = b.size(0), kb = b.size(1) * 2;
    TORCH_CHECK(ka >= 16 && kb >= 16, "K-dim must be >= 16");
    TORCH_CHECK(ka == kb, "Inner dims mismatch: ", ka, " vs ", kb);
    // A may be the first m < 128 rows of a quantized tensor whose scales cover the whole padded 128-row band
    // (small batches: the kernel then skips the padding rows)
    TORCH_CHECK(a_sf.numel() * 16 == (m >= 128 ? m : 128) * ka, "A_sf size mismatch");
    TORCH_CHECK(m >= 128 || ka % 256 == 0, "A with fewer than 128 rows needs K to be a multiple of 256");
    TORCH_CHECK(b_sf.numel() * 16 == n * kb, "B_sf size mismatch");
}

// One GEMM launch.  alpha, or (amax_a, amax_b, denominator) for the output scale formed in the kernel;
// with the latter, d_amax (device f32[1], zero or an earlier maximum) receives max|out|.
Tensor gemm_launch(const Tensor &a, const Tensor &b, const Tensor &a_sf, const Tensor &b_sf, const Tensor *alpha, const Tensor *amax_a,
                   const Tensor *amax_b, double denominator, at::ScalarType out_dtype, const Tensor *d_amax, const Tensor *bias = nullptr) {
    const int64_t m = a.size(0), n = b.size(0), k = a.size(1) * 2;
    Tensor out = at::empty({m, n}, a.options().dtype(out_dtype));
    const size_t ws_bytes = fos_gemm_workspace_bytes(m, n, k);
    const DeviceGuard guard(a.device());
    // split-K partial tiles of small-M shapes; from torch's caching allocator, which keeps the block tied to the current stream
    Tensor ws;
    if (ws_bytes) ws = at::empty({(int64_t)ws_bytes}, a.options().dtype(at::kByte));
    void *wsp = ws_bytes ? ws.data_ptr() : nullptr;
    const int out_type = out_dtype == at::kBFloat16 ? FOS_T_BF16 : FOS_T_F16;
    const fos_stream_t stream = current_stream(a);
    const uint8_t *A = a.data_ptr<uint8_t>(), *B = b.data_ptr<uint8_t>();
    const uint8_t *sA = static_cast<const uint8_t *>(a_sf.data_ptr()), *sB = static_cast<const uint8_t *>(b_sf.data_ptr());
    int rc;
    if (alpha) {
        rc = fos_gemm_nvfp4(A, B, sA, sB, alpha->data_ptr<float>(), m, n, k, out.data_ptr(), out_type, n, wsp, ws_bytes, stream);
    } else if (d_amax || bias) {
        if (d_amax) require_gpu(*d_amax, "d_amax");
        if (bias) {
            require_gpu(*bias, "bias");
            TORCH_CHECK(bias->scalar_type() == out_dtype && bias->dim() == 1 && bias->size(0) == n && bias->is_contiguous(),
                        "gemm: bias must be a contiguous [N] tensor of the output type");
        }
        rc = fos_gemm_nvfp4_linear(A, B, sA, sB, amax_a->data_ptr<float>(), amax_b->data_ptr<float>(), denominator, m, n, k,
                                   out.data_ptr(), out_type, n, bias ? bias->data_ptr() : nullptr,
                                   d_amax ? d_amax->data_ptr<float>() : nullptr, wsp, ws_bytes, stream);
    } else {
        rc = fos_gemm_nvfp4_amax(A, B, sA, sB, amax_a->data_ptr<float>(), amax_b->data_ptr<float>(), denominator, m, n, k,
                                 out.data_ptr(), out_type, n, wsp, ws_bytes, stream);
    }
    check(rc, "fouroversix::gemm_nvfp4nvfp4_accum_fp32");
    return out;
}

Tensor gemm_nvfp4(const Tensor &a, const Tensor &b, const Tensor &a_sf, const Tensor &b_sf, const Tensor &alpha, at::ScalarType out_dtype) {
    const Tensor *scales[1] = {&alpha};
    const char *names[1] = {"alpha"};
    check_gemm_operands(a, b, a_sf, b_sf, scales, 1, names);
    return gemm_launch(a, b, a_sf, b_sf, &alpha, nullptr, nullptr, 1.0, out_dtype, nullptr);
}
Tensor gemm_nvfp4_bf16(const Tensor &a, const Tensor &b, const Tensor &a_sf, const Tensor &b_sf, const Tensor &alpha) {
    return gemm_nvfp4(a, b, a_sf, b_sf, alpha, at::kBFloat16);
}
Tensor gemm_nvfp4_fp16(const Tensor &a, const Tensor &b, const Tensor &a_sf, const Tensor &b_sf, const Tensor &alpha) {
    return gemm_nvfp4(a, b, a_sf, b_sf, alpha, at::kHalf);
}

// The NVFP4 GEMM with the output scale (amax_a * amax_b) * f32(1 / denominator) formed in the kernel: one launch
// less than alpha + GEMM, same result.  `checked`: the operands are the members of two QuantizedTensors on
// one GPU (the frontend has looked): only the shapes are compared.
// `bias` ([N], output type): added to the rounded product and rounded again, as `out + bias` would.
Tensor gemm_nvfp4_amax(const Tensor &a, const Tensor &b, const Tensor &a_sf, const Tensor &b_sf, const Tensor &amax_a, const Tensor &amax_b,
                       double denominator, at::ScalarType out_dtype, const c10::optional<Tensor> &d_amax, bool checked,
                       const c10::optional<Tensor> &bias) {
    if (checked) {
        TORCH_CHECK(a.size(1) == b.size(1), "Inner dims mismatch: ", a.size(1) * 2, " vs ", b.size(1) * 2);
    } else {
        const Tensor *scales[2] = {&amax_a, &amax_b};
        const char *names[2] = {"amax_a", "amax_b"};
        check_gemm_operands(a, b, a_sf, b_sf, scales, 2, names);
    }
    return gemm_launch(a, b, a_sf, b_sf, nullptr, &amax_a, &amax_b, denominator, out_dtype, d_amax.has_value() ? &*d_amax : nullptr,
                       bias.has_value() ? &*bias : nullptr);
}

// alpha[0] = (amax_a * amax_b) * f32(1 / denominator) on the device
void gemm_alpha(const Tensor &amax_a, const Tensor &amax_b, double denominator, Tensor alpha) {
    const DeviceGuard guard(alpha.device());
    check(fos_gemm_alpha(amax_a.data_ptr<float>(), amax_b.data_ptr<float>(), denominator, alpha.data_ptr<float>(), current_stream(alpha)),
          "fouroversix::gemm_alpha");
}

// MXFP4 x MXFP4 GEMM on the scaled FP4 matrix instruction; checks as the NVFP4 op with blocks of 32, E8M0 scales.
Tensor gemm_mxfp4_typed(const Tensor &a, const Tensor &b, const Tensor &a_sf, const Tensor &b_sf, const Tensor &alpha, at::ScalarType out_dtype) {
    const Tensor *all[5] = {&a, &b, &a_sf, &b_sf, &alpha};
    const char *names[5] = {"A", "B", "A_sf", "B_sf", "alpha"};
    for (int i = 0; i < 5; ++i) {
        require_gpu(*all[i], names[i]);
        TORCH_CHECK(all[i]->is_contiguous(), "gemm: ", names[i], " must be contiguous");
        TORCH_CHECK(all[i]->device() == a.device(), "gemm: all operands must be on the same GPU");
    }
    TORCH_CHECK(a.scalar_type() == at::kByte && b.scalar_type() == at::kByte && a.dim() == 2 && b.dim() == 2, "A and B must be 2D uint8");
    TORCH_CHECK(a_sf.scalar_type() == at::kFloat8_e8m0fnu && b_sf.scalar_type() == at::kFloat8_e8m0fnu, "A_sf and B_sf must be Float8_e8m0fnu");
    const int64_t m = a.size(0), ka = a.size(1) * 2, n = b.size(0), kb = b.size(1) * 2;
    TORCH_CHECK(ka == kb, "Inner dims mismatch: ", ka, " vs ", kb);
    TORCH_CHECK(a_sf.numel() * 32 == m * ka && b_sf.numel() * 32 == n * kb, "scale factor size mismatch");
    Tensor out = at::empty({m, n}, a.options().dtype(out_dtype));
    const DeviceGuard guard(a.device());
    check(fos_gemm_mxfp4(a.data_ptr<uint8_t>(), b.data_ptr<uint8_t>(), static_cast<const uint8_t *>(a_sf.data_ptr()),
                         static_cast<const uint8_t *>(b_sf.data_ptr()), alpha.data_ptr<float>(), m, n, ka, out.data_ptr(),
                         out_dtype == at::kBFloat16 ? FOS_T_BF16 : FOS_T_F16, n, current_stream(a)),
          "fouroversix::gemm_mxfp4mxfp4_accum_fp32");
    return out;
}
Tensor gemm_mxfp4_bf16(const Tensor &a, const Tensor &b, const Tensor &a_sf, const Tensor &b_sf, const Tensor &alpha) {
    return gemm_mxfp4_typed(a, b, a_sf, b_sf, alpha, at::kBFloat16);
}

Tensor dequantize(const Tensor &values, const Tensor &scale_factors, const Tensor &amax, int64_t dtype, int64_t sf_layout, double divisor,
                  int64_t rows, int64_t cols, at::ScalarType out_dtype, bool f32_intermediate) {
    require_gpu(values, "values");
    const int64_t rows_p = values.size(0), cols_p = values.size(1) * 2;
    Tensor out = at::empty({rows, cols}, values.options().dtype(out_dtype));
    if (rows == 0 || cols == 0) return out;
    const Tensor amax32 = amax.reshape({1}).to(values.device(), at::kFloat);
    const Tensor v = values.contiguous(), s = scale_factors.contiguous();
    const DeviceGuard guard(values.device());
    check(fos_dequantize(v.data_ptr<uint8_t>(), static_cast<const uint8_t *>(s.data_ptr()), amax32.data_ptr<float>(), (int)dtype,
                         (int)sf_layout, divisor, rows, cols, rows_p, cols_p, out.data_ptr(), type_id(out_dtype, "dequantize: out_dtype"),
                         cols, f32_intermediate ? FOS_T_F32 : FOS_T_F16, current_stream(values)),
          "fouroversix::dequantize");
    return out;
}

}  // namespace

TORCH_LIBRARY(fouroversix, m) {
    m.def(
        "quantize(Tensor x, bool is_nvfp4, bool is_rtn, bool is_rht, bool is_2d, bool is_transpose, "
        "int selection_rule, int rbits) -> (Tensor, Tensor, Tensor)");
    m.def(
        "quantize_ex(Tensor x, int dtype, int selection_rule, int round_style, bool is_2d, int seed, int offset, "
        "int sf_layout, Tensor? amax, Tensor? key=None) -> (Tensor, Tensor, Tensor)");
    m.def("pseudo_quantize(Tensor x, int dtype, int selection_rule, int round_style, bool is_2d, Tensor? amax, int seed=0, int offset=0) -> Tensor");
    m.def("transform(Tensor x, bool transpose, bool rht) -> (Tensor, Tensor)");
    m.def(
        "transform_quantize(Tensor x, bool transpose, bool rht, int dtype, int selection_rule, int round_style, bool is_2d, "
        "int seed, int offset, int sf_layout) -> (Tensor, Tensor, Tensor)");
    m.def("gemm_nvfp4nvfp4_accum_fp32_out_bf16_tnt(Tensor A, Tensor B, Tensor A_sf, Tensor B_sf, Tensor alpha) -> Tensor");
    m.def("gemm_nvfp4nvfp4_accum_fp32_out_fp16_tnt(Tensor A, Tensor B, Tensor A_sf, Tensor B_sf, Tensor alpha) -> Tensor");
    m.def("gemm_mxfp4mxfp4_accum_fp32_out_bf16_tnt(Tensor A, Tensor B, Tensor A_sf, Tensor B_sf, Tensor alpha) -> Tensor");
    m.def(
        "gemm_nvfp4_amax(Tensor A, Tensor B, Tensor A_sf, Tensor B_sf, Tensor amax_a, Tensor amax_b, float denominator, "
        "ScalarType out_dtype, Tensor(a!)? d_amax, bool checked=False, Tensor? bias=None) -> Tensor");
    m.def(
        "dequantize(Tensor values, Tensor scale_factors, Tensor amax, int dtype, int sf_layout, float divisor, "
        "int rows, int cols, ScalarType out_dtype, bool f32_intermediate=False) -> Tensor");
}

TORCH_LIBRARY_IMPL(fouroversix, CUDA, m) {
    m.impl("quantize", &quantize_ref);
    m.impl("quantize_ex", &quantize_ex);
    m.impl("pseudo_quantize", &pseudo_quantize);
    m.impl("transform", &transform);
    m.impl("transform_quantize", &transform_quantize);
    m.impl("gemm_nvfp4nvfp4_accum_fp32_out_bf16_tnt", &gemm_nvfp4_bf16);
    m.impl("gemm_nvfp4nvfp4_accum_fp32_out_fp16_tnt", &gemm_nvfp4_fp16);
    m.impl("gemm_mxfp4mxfp4_accum_fp32_out_bf16_tnt", &gemm_mxfp4_bf16);
    m.impl("gemm_nvfp4_amax", &gemm_nvfp4_amax);
    m.impl("dequantize", &dequantize);
}

PYBIND11_MODULE(TORCH_EXTENSION_NAME, m) {
    m.doc() = "direct entry points of the fouroversix:: operators (same functions, no dispatcher)";
    m.def("quantize_ex", &quantize_ex);
    m.def("pseudo_quantize", &pseudo_quantize);
    m.def("pseudo_quantize_is_fused", &pseudo_quantize_is_fused);
    m.def("transform", &transform);
    m.def("transform_quantize", &transform_quantize);
    m.def("gemm_nvfp4", &gemm_nvfp4);
    m.def("gemm_nvfp4_amax", &gemm_nvfp4_amax);
    m.def("gemm_alpha", &gemm_alpha);
    m.def("gemm_mxfp4", &gemm_mxfp4_typed);
    m.def("dequantize", &dequantize);
}
