"""``torch.ops.fouroversix.*`` operators backed by the gfx950 library.

The operator names and schemas are the reference's
(``src/fouroversix/csrc/bindings.cpp:26-35``), with the fake (meta) shapes of
``src/fouroversix/quantize/cuda/ops.py:28-47`` and
``src/fouroversix/matmul/cutlass/ops.py:82-92``, so code that calls the ops directly, or
traces them, keeps working.  ``quantize_ex`` / ``dequantize`` are additions carrying the
options the reference's native op does not have (format, dither key, output layout).
Each implementation allocates the outputs and makes one call through the C ABI on the
current stream.
"""

from __future__ import annotations

import contextlib

import torch

from fouroversix_amd import _native as nat

_LIB = torch.library.Library("fouroversix", "DEF")
_LIB.define(
    "quantize(Tensor x, bool is_nvfp4, bool is_rtn, bool is_rht, bool is_2d, bool is_transpose, "
    "int selection_rule, int rbits) -> (Tensor, Tensor, Tensor)"
)
_LIB.define(
    "quantize_ex(Tensor x, int dtype, int selection_rule, int round_style, bool is_2d, int seed, int offset, "
    "int sf_layout, Tensor? amax) -> (Tensor, Tensor, Tensor)"
)
_LIB.define(
    "pseudo_quantize(Tensor x, int dtype, int selection_rule, int round_style, bool is_2d, Tensor? amax) -> Tensor"
)
_LIB.define("gemm_nvfp4nvfp4_accum_fp32_out_bf16_tnt(Tensor A, Tensor B, Tensor A_sf, Tensor B_sf, Tensor alpha) -> Tensor")
_LIB.define("gemm_nvfp4nvfp4_accum_fp32_out_fp16_tnt(Tensor A, Tensor B, Tensor A_sf, Tensor B_sf, Tensor alpha) -> Tensor")
_LIB.define("gemm_mxfp4mxfp4_accum_fp32_out_bf16_tnt(Tensor A, Tensor B, Tensor A_sf, Tensor B_sf, Tensor alpha) -> Tensor")
_LIB.define(
    "dequantize(Tensor values, Tensor scale_factors, Tensor amax, int dtype, int sf_layout, float divisor, "
    "int rows, int cols, ScalarType out_dtype, bool f32_intermediate=False) -> Tensor"
)


MXFP4 = 2  # format id at the native boundary (blocks of 32, E8M0 scales)


def _padded(rows: int, cols: int, dtype: int = 0) -> tuple[int, int]:
    col_multiple = 128 if dtype == MXFP4 else 64  # four blocks
    return -(-rows // 128) * 128, -(-cols // col_multiple) * col_multiple


# Pass-1 workspace (8 KiB), one per (device, stream): calls on one stream are ordered, so
# they can share it; calls on different streams must not.  While a stream is being captured
# into a graph the workspace comes from the allocator instead (the graph's private pool keeps
# it for the graph's lifetime; a cached one would be shared by every graph captured on that
# stream and pinned after they are gone).
_WORKSPACES: dict[tuple[int, int], torch.Tensor] = {}
_WS_BYTES = 0


def _workspace(dev: torch.device, stream: int) -> torch.Tensor:
    global _WS_BYTES
    if _WS_BYTES == 0:
        _WS_BYTES = int(nat.lib().fos_quantize_workspace_bytes(1, 1))
    if torch.cuda.is_current_stream_capturing():
        return torch.empty(_WS_BYTES, dtype=torch.uint8, device=dev)
    key = (dev.index if dev.index is not None else torch.cuda.current_device(), stream)
    ws = _WORKSPACES.get(key)
    if ws is None:
        ws = torch.empty(_WS_BYTES, dtype=torch.uint8, device=dev)
        _WORKSPACES[key] = ws
    return ws


_SAME_DEVICE = contextlib.nullcontext()


def _on_device(dev: torch.device):
    """`with torch.cuda.device(dev)` only when `dev` is not already current."""
    if dev.index is None or dev.index == torch.cuda.current_device():
        return _SAME_DEVICE
    return torch.cuda.device(dev)


# split-K workspace size per GEMM shape (the library plans the shape once for the size and once
# for the launch; the size never changes)
_GEMM_WS_BYTES: dict[tuple[int, int, int], int] = {}


def _quantize_impl(x, dtype, selection_rule, round_style, is_2d, seed, offset, sf_layout, amax):
    if x.dim() != 2:
        raise RuntimeError("quantize: x must be 2-D")
    if x.dtype not in nat.TORCH_TO_T:
        raise RuntimeError(f"quantize: x must be bfloat16, float16 or float32, got {x.dtype}")
    if x.stride(-1) != 1:
        raise RuntimeError("quantize: x must be contiguous on the last dim")
    nat.require_gpu_tensor(x, "x")
    rows, cols = x.shape
    rows_p, cols_p = _padded(rows, cols, dtype)
    dev = x.device
    values = torch.empty(rows_p, cols_p // 2, dtype=torch.uint8, device=dev)
    if dtype == MXFP4:
        sf = torch.empty(rows_p * cols_p // 32, dtype=torch.float8_e8m0fnu, device=dev)
    else:
        sf = torch.empty(rows_p * cols_p // 16, dtype=torch.float8_e4m3fn, device=dev)
    if rows == 0 or cols == 0:
        values.zero_()
        sf.view(torch.uint8).zero_()
        return values, sf, torch.full((1,), 1.0 if dtype == MXFP4 else 0.0, dtype=torch.float32, device=dev)
    L = nat.lib()
    amax_is_input = amax is not None
    amax_buf = (
        amax.reshape(1).to(device=dev, dtype=torch.float32).contiguous()
        if amax_is_input
        else torch.empty(1, dtype=torch.float32, device=dev)
    )
    with _on_device(dev):
        stream = nat.current_stream(dev)
        workspace = _workspace(dev, stream)
        rc = L.fos_quantize(
            x.data_ptr(), nat.TORCH_TO_T[x.dtype], rows, cols, x.stride(0), dtype, selection_rule, round_style, int(is_2d),
            seed & 0xFFFFFFFFFFFFFFFF, offset & 0xFFFFFFFFFFFFFFFF, sf_layout,
            values.data_ptr(), sf.data_ptr(), amax_buf.data_ptr(), int(amax_is_input),
            workspace.data_ptr(), workspace.numel(), stream,
        )
    nat.check(rc, "fouroversix::quantize")
    return values, sf, amax_buf


def pseudo_quantize_is_fused(x: torch.Tensor, dtype: int, round_style: int) -> bool:
    """True when the library has a fused quantize->dequantize kernel for this call."""
    return (
        dtype == 0
        and round_style == 0
        and x.dim() == 2
        and x.dtype == torch.bfloat16
        and x.numel() > 0
        and x.stride(-1) == 1
        and x.shape[1] % 16 == 0
        and x.stride(0) % 8 == 0
        and x.stride(0) < (1 << 23)  # (the streaming kernels' 32-bit tile offsets)
        and x.data_ptr() % 16 == 0
    )


def _pseudo_quantize_impl(x, dtype, selection_rule, round_style, is_2d, amax):
    if not pseudo_quantize_is_fused(x, dtype, round_style):
        raise RuntimeError("pseudo_quantize: no fused kernel for these arguments (quantize, then dequantize)")
    nat.require_gpu_tensor(x, "x")
    rows, cols = x.shape
    dev = x.device
    out = torch.empty(rows, cols, dtype=torch.bfloat16, device=dev)
    amax_is_input = amax is not None
    amax_buf = (
        amax.reshape(1).to(device=dev, dtype=torch.float32).contiguous()
        if amax_is_input
        else torch.empty(1, dtype=torch.float32, device=dev)
    )
    with _on_device(dev):
        stream = nat.current_stream(dev)
        workspace = _workspace(dev, stream)
        rc = nat.lib().fos_pseudo_quantize(
            x.data_ptr(), nat.T_BF16, rows, cols, x.stride(0), dtype, selection_rule, round_style, int(is_2d),
            out.data_ptr(), cols, amax_buf.data_ptr(), int(amax_is_input),
            workspace.data_ptr(), workspace.numel(), stream,
        )
    nat.check(rc, "fouroversix::pseudo_quantize")
    return out


def transform_unsupported_reason(x: torch.Tensor, transpose: bool, rht: bool) -> str | None:
    """Why the transpose / random-Hadamard pre-transform cannot run on ``x``, or None."""
    return None if x.dim() == 2 else "transpose / rht need a 2-D tensor"


def _transform_impl(x, transpose, rht):
    """``(y, amax)``: y = RHT(x^T) as the reference forms it before scaling, amax = max|y|."""
    if x.dim() != 2 or x.dtype not in (torch.bfloat16, torch.float16):
        raise RuntimeError("transform: x must be a 2-D bfloat16 or float16 tensor")
    nat.require_gpu_tensor(x, "x")
    reason = transform_unsupported_reason(x, transpose, rht)
    if reason is not None:
        raise RuntimeError(f"transform: {reason}")
    if x.stride(-1) != 1:
        x = x.contiguous()
    rows, cols = x.shape
    dev = x.device
    out_rows, out_cols = (cols, rows) if transpose else (rows, cols)
    # y is written in whole groups of 16 (zeros complete a ragged last group; with rht that group
    # then holds values in all 16 places, so the padded width is what gets quantized)
    width = -(-out_cols // 16) * 16
    y = torch.empty((out_rows, width), dtype=x.dtype, device=dev)
    amax = torch.empty(1, dtype=torch.float32, device=dev)
    with _on_device(dev):
        stream = nat.current_stream(dev)
        workspace = _workspace(dev, stream)
        rc = nat.lib().fos_transform(
            x.data_ptr(), nat.TORCH_TO_T[x.dtype], rows, cols, x.stride(0), int(transpose), int(rht),
            y.data_ptr(), y.stride(0), amax.data_ptr(), workspace.data_ptr(), workspace.numel(), stream,
        )
    nat.check(rc, "fouroversix::transform")
    return (y if rht or width == out_cols else y[:, :out_cols]), amax


def _quantize_ref_schema(x, is_nvfp4, is_rtn, is_rht, is_2d, is_transpose, selection_rule, rbits):
    if not is_nvfp4:
        raise RuntimeError("quantize: only the NVFP4 format is implemented by this op (use quantize_ex for IF4)")
    if not 0 <= selection_rule <= 4:
        raise RuntimeError(f"Invalid selection_rule: {selection_rule}")
    # the reference's native op takes fp16 and bf16 (csrc/quantize/fp4_quant.cu:134-136)
    if x.dtype not in (torch.float16, torch.bfloat16):
        raise RuntimeError(f"quantize: x must be bfloat16 or float16, got {x.dtype}")
    seed = 0 if rbits < 0 else rbits
    amax = None
    if is_rht or is_transpose:
        x, amax = _transform_impl(x, is_transpose, is_rht)
    return _quantize_impl(x, 0, selection_rule, 0 if is_rtn else 1, is_2d, seed, 0, nat.SF_TILED, amax)


def _gemm_impl(a, b, a_sf, b_sf, alpha, out_dtype, amax=None, d_amax=None, checked=False):
    """``amax`` = (amax_a, amax_b, denominator) forms the output scale inside the kernel
    (``alpha`` is then ignored and may be None); with it, ``d_amax`` (device f32[1], zero or an
    earlier maximum) receives max|out|.  ``checked``: the operands are the members of two
    QuantizedTensors on one GPU (the frontend has looked): only the shapes are compared."""
    if checked:
        m, ka, n = a.shape[0], a.shape[1] * 2, b.shape[0]
        if b.shape[1] * 2 != ka:
            raise RuntimeError(f"Inner dims mismatch: {ka} vs {b.shape[1] * 2}")
        return _gemm_launch(a, b, a_sf, b_sf, alpha, out_dtype, amax, d_amax, m, n, ka)
    scale_tensors = (("alpha", alpha),) if amax is None else (("amax_a", amax[0]), ("amax_b", amax[1]))
    for name, t in (("A", a), ("B", b), ("A_sf", a_sf), ("B_sf", b_sf), *scale_tensors):
        nat.require_gpu_tensor(t, name)
        if not t.is_contiguous():
            raise RuntimeError(f"gemm: {name} must be contiguous")
        if t.device != a.device:
            raise RuntimeError("gemm: all operands must be on the same GPU")
    if a.dtype != torch.uint8 or b.dtype != torch.uint8:
        raise RuntimeError("A and B must be uint8")
    if a.dim() != 2 or b.dim() != 2:
        raise RuntimeError("A and B must be 2D")
    if a_sf.dtype != torch.float8_e4m3fn or b_sf.dtype != torch.float8_e4m3fn:
        raise RuntimeError("A_sf and B_sf must be Float8_e4m3fn")
    m, ka = a.shape[0], a.shape[1] * 2
    n, kb = b.shape[0], b.shape[1] * 2
    if ka < 16 or kb < 16:
        raise RuntimeError("K-dim must be >= 16")
    if ka != kb:
        raise RuntimeError(f"Inner dims mismatch: {ka} vs {kb}")
    # A may be the first m < 128 rows of a quantized tensor whose scales cover the whole
    # padded 128-row band (small batches: the kernel then skips the padding rows)
    if a_sf.numel() * 16 != (m if m >= 128 else 128) * ka:
        raise RuntimeError("A_sf size mismatch")
    if m < 128 and ka % 256 != 0:
        raise RuntimeError("A with fewer than 128 rows needs K to be a multiple of 256")
    if b_sf.numel() * 16 != n * kb:
        raise RuntimeError("B_sf size mismatch")
    return _gemm_launch(a, b, a_sf, b_sf, alpha, out_dtype, amax, d_amax, m, n, ka)


def _gemm_launch(a, b, a_sf, b_sf, alpha, out_dtype, amax, d_amax, m, n, ka):
    out = torch.empty(m, n, dtype=out_dtype, device=a.device)
    L = nat.lib()
    ws_bytes = _GEMM_WS_BYTES.get((m, n, ka))
    if ws_bytes is None:
        ws_bytes = _GEMM_WS_BYTES[(m, n, ka)] = int(L.fos_gemm_workspace_bytes(m, n, ka))
    with _on_device(a.device):
        # split-K partial tiles of small-M shapes; from torch's caching allocator, which
        # keeps the block tied to the current stream
        ws = torch.empty(ws_bytes, dtype=torch.uint8, device=a.device) if ws_bytes else None
        tail = (m, n, ka, out.data_ptr(), nat.TORCH_TO_T[out_dtype], n,
                ws.data_ptr() if ws is not None else None, ws_bytes, nat.current_stream(a.device))
        if amax is None:
            rc = L.fos_gemm_nvfp4(a.data_ptr(), b.data_ptr(), a_sf.data_ptr(), b_sf.data_ptr(), alpha.data_ptr(), *tail)
        elif d_amax is not None:
            nat.require_gpu_tensor(d_amax, "d_amax")
            rc = L.fos_gemm_nvfp4_amax_out(a.data_ptr(), b.data_ptr(), a_sf.data_ptr(), b_sf.data_ptr(),
                                           amax[0].data_ptr(), amax[1].data_ptr(), float(amax[2]), *tail[:6], d_amax.data_ptr(), *tail[6:])
        else:
            rc = L.fos_gemm_nvfp4_amax(a.data_ptr(), b.data_ptr(), a_sf.data_ptr(), b_sf.data_ptr(),
                                       amax[0].data_ptr(), amax[1].data_ptr(), float(amax[2]), *tail)
    nat.check(rc, "fouroversix::gemm_nvfp4nvfp4_accum_fp32")
    return out


def gemm_alpha_into(amax_a, amax_b, denominator, alpha):
    """alpha[0] = (amax_a * amax_b) * f32(1 / denominator) on the device, torch's GPU arithmetic for
    ``(amax_a * amax_b) / denominator``."""
    with _on_device(alpha.device):
        rc = nat.lib().fos_gemm_alpha(amax_a.data_ptr(), amax_b.data_ptr(), float(denominator), alpha.data_ptr(),
                                      nat.current_stream(alpha.device))
    nat.check(rc, "fouroversix::gemm_alpha")


def _gemm_mxfp4_impl(a, b, a_sf, b_sf, alpha, out_dtype=torch.bfloat16):
    """MXFP4 x MXFP4 GEMM on the scaled FP4 matrix instruction; checks as the NVFP4 op
    (reference csrc/include/element_traits.hpp:122-170 with blocks of 32, E8M0 scales)."""
    for name, t in (("A", a), ("B", b), ("A_sf", a_sf), ("B_sf", b_sf), ("alpha", alpha)):
        nat.require_gpu_tensor(t, name)
        if not t.is_contiguous():
            raise RuntimeError(f"gemm: {name} must be contiguous")
        if t.device != a.device:
            raise RuntimeError("gemm: all operands must be on the same GPU")
    if a.dtype != torch.uint8 or b.dtype != torch.uint8 or a.dim() != 2 or b.dim() != 2:
        raise RuntimeError("A and B must be 2D uint8")
    if a_sf.dtype != torch.float8_e8m0fnu or b_sf.dtype != torch.float8_e8m0fnu:
        raise RuntimeError("A_sf and B_sf must be Float8_e8m0fnu")
    m, ka = a.shape[0], a.shape[1] * 2
    n, kb = b.shape[0], b.shape[1] * 2
    if ka != kb:
        raise RuntimeError(f"Inner dims mismatch: {ka} vs {kb}")
    if a_sf.numel() * 32 != m * ka or b_sf.numel() * 32 != n * kb:
        raise RuntimeError("scale factor size mismatch")
    out = torch.empty(m, n, dtype=out_dtype, device=a.device)
    with _on_device(a.device):
        rc = nat.lib().fos_gemm_mxfp4(
            a.data_ptr(), b.data_ptr(), a_sf.data_ptr(), b_sf.data_ptr(), alpha.data_ptr(),
            m, n, ka, out.data_ptr(), nat.TORCH_TO_T[out_dtype], n, nat.current_stream(a.device),
        )
    nat.check(rc, "fouroversix::gemm_mxfp4mxfp4_accum_fp32")
    return out


def _dequantize_impl(values, scale_factors, amax, dtype, sf_layout, divisor, rows, cols, out_dtype, f32_intermediate=False):
    nat.require_gpu_tensor(values, "values")
    rows_p, cols_p = values.shape[0], values.shape[1] * 2
    out = torch.empty(rows, cols, dtype=out_dtype, device=values.device)
    if rows == 0 or cols == 0:
        return out
    amax32 = amax.reshape(1).to(device=values.device, dtype=torch.float32)
    with _on_device(values.device):
        rc = nat.lib().fos_dequantize(
            values.contiguous().data_ptr(), scale_factors.contiguous().data_ptr(), amax32.data_ptr(),
            dtype, sf_layout, divisor, rows, cols, rows_p, cols_p,
            out.data_ptr(), nat.TORCH_TO_T[out_dtype], cols, nat.T_F32 if f32_intermediate else nat.T_F16,
            nat.current_stream(values.device),
        )
    nat.check(rc, "fouroversix::dequantize")
    return out


_LIB.impl("quantize", _quantize_ref_schema, "CUDA")
_LIB.impl("quantize_ex", _quantize_impl, "CUDA")
_LIB.impl("pseudo_quantize", _pseudo_quantize_impl, "CUDA")
_LIB.impl(
    "gemm_nvfp4nvfp4_accum_fp32_out_bf16_tnt",
    lambda a, b, a_sf, b_sf, alpha: _gemm_impl(a, b, a_sf, b_sf, alpha, torch.bfloat16),
    "CUDA",
)
_LIB.impl(
    "gemm_nvfp4nvfp4_accum_fp32_out_fp16_tnt",
    lambda a, b, a_sf, b_sf, alpha: _gemm_impl(a, b, a_sf, b_sf, alpha, torch.float16),
    "CUDA",
)
_LIB.impl("gemm_mxfp4mxfp4_accum_fp32_out_bf16_tnt", _gemm_mxfp4_impl, "CUDA")
_LIB.impl("dequantize", _dequantize_impl, "CUDA")


def _fake_quantize_shapes(x, dtype=0):
    rows_p, cols_p = _padded(x.shape[0], x.shape[1], dtype)
    block, sf_dtype = (32, torch.float8_e8m0fnu) if dtype == MXFP4 else (16, torch.float8_e4m3fn)
    return (
        torch.empty(rows_p, cols_p // 2, dtype=torch.uint8, device=x.device),
        torch.empty(rows_p * cols_p // block, dtype=sf_dtype, device=x.device),
        torch.empty(1, dtype=torch.float32, device=x.device),
    )


@torch.library.register_fake("fouroversix::quantize")
def _(x, is_nvfp4, is_rtn, is_rht, is_2d, is_transpose, selection_rule, rbits):
    return _fake_quantize_shapes(x)


@torch.library.register_fake("fouroversix::quantize_ex")
def _(x, dtype, selection_rule, round_style, is_2d, seed, offset, sf_layout, amax):
    return _fake_quantize_shapes(x, dtype)


@torch.library.register_fake("fouroversix::pseudo_quantize")
def _(x, dtype, selection_rule, round_style, is_2d, amax):
    return torch.empty_like(x, memory_format=torch.contiguous_format)


@torch.library.register_fake("fouroversix::gemm_nvfp4nvfp4_accum_fp32_out_bf16_tnt")
def _(a, b, a_sf, b_sf, alpha):
    return torch.empty(a.shape[0], b.shape[0], dtype=torch.bfloat16, device=a.device)


@torch.library.register_fake("fouroversix::gemm_nvfp4nvfp4_accum_fp32_out_fp16_tnt")
def _(a, b, a_sf, b_sf, alpha):
    return torch.empty(a.shape[0], b.shape[0], dtype=torch.float16, device=a.device)


@torch.library.register_fake("fouroversix::gemm_mxfp4mxfp4_accum_fp32_out_bf16_tnt")
def _(a, b, a_sf, b_sf, alpha):
    return torch.empty(a.shape[0], b.shape[0], dtype=torch.bfloat16, device=a.device)


@torch.library.register_fake("fouroversix::dequantize")
def _(values, scale_factors, amax, dtype, sf_layout, divisor, rows, cols, out_dtype, f32_intermediate=False):
    return torch.empty(rows, cols, dtype=out_dtype, device=values.device)


def quantize(x, is_nvfp4, is_rtn, is_rht, is_2d, is_transpose, selection_rule, rbits):
    """Same call as the reference's ``fouroversix.quantize.cuda.ops.quantize``."""
    return torch.ops.fouroversix.quantize.default(
        x, is_nvfp4, is_rtn, is_rht, is_2d, is_transpose, selection_rule, rbits
    )


def quantize_ex(x, dtype, selection_rule, round_style, is_2d, seed, offset, sf_layout, amax=None):
    """Extended quantize.  Real tensors go straight to the implementation (the dispatcher
    costs more host time than a small quantize takes on the GPU); fake / meta tensors and
    tracing go through the registered operator."""
    if type(x) is torch.Tensor and x.device.type == "cuda" and not torch.compiler.is_compiling():
        return _quantize_impl(x, dtype, selection_rule, round_style, is_2d, seed, offset, sf_layout, amax)
    return torch.ops.fouroversix.quantize_ex.default(
        x, dtype, selection_rule, round_style, is_2d, seed, offset, sf_layout, amax
    )


def transform(x, transpose, rht):
    """Pre-transform of the ``transpose`` / ``rht`` quantize options: ``(y, amax)``."""
    return _transform_impl(x, transpose, rht)


def pseudo_quantize(x, dtype, selection_rule, round_style, is_2d, amax=None):
    """Fused quantize -> dequantize (bf16 in, bf16 out); see ``pseudo_quantize_is_fused``."""
    if type(x) is torch.Tensor and x.device.type == "cuda" and not torch.compiler.is_compiling():
        return _pseudo_quantize_impl(x, dtype, selection_rule, round_style, is_2d, amax)
    return torch.ops.fouroversix.pseudo_quantize.default(x, dtype, selection_rule, round_style, is_2d, amax)


def _direct(t: torch.Tensor) -> bool:
    return type(t) is torch.Tensor and t.device.type == "cuda" and not torch.compiler.is_compiling()


def gemm_nvfp4nvfp4_accum_fp32_out_bf16_tnt(a, b, a_sf, b_sf, alpha):
    if _direct(a):
        return _gemm_impl(a, b, a_sf, b_sf, alpha, torch.bfloat16)
    return torch.ops.fouroversix.gemm_nvfp4nvfp4_accum_fp32_out_bf16_tnt.default(a, b, a_sf, b_sf, alpha)


def gemm_nvfp4nvfp4_accum_fp32_out_fp16_tnt(a, b, a_sf, b_sf, alpha):
    if _direct(a):
        return _gemm_impl(a, b, a_sf, b_sf, alpha, torch.float16)
    return torch.ops.fouroversix.gemm_nvfp4nvfp4_accum_fp32_out_fp16_tnt.default(a, b, a_sf, b_sf, alpha)


def gemm_nvfp4_from_amax(a, b, a_sf, b_sf, amax_a, amax_b, denominator, out_dtype, d_amax=None, checked=False):
    """The NVFP4 GEMM with the output scale ``(amax_a * amax_b) * f32(1 / denominator)`` formed
    in the kernel (``fos_gemm_nvfp4_amax``): one launch less than alpha + GEMM, same result.
    ``d_amax`` (device f32[1] holding 0) additionally receives max|out|."""
    return _gemm_impl(a, b, a_sf, b_sf, None, out_dtype, amax=(amax_a, amax_b, denominator), d_amax=d_amax, checked=checked)


def gemm_mxfp4mxfp4_accum_fp32_out_bf16_tnt(a, b, a_sf, b_sf, alpha, out_dtype=torch.bfloat16):
    """Same call as the reference's ``matmul/cutlass/ops.py:6-20`` (fp16 output as an extension)."""
    if _direct(a):
        return _gemm_mxfp4_impl(a, b, a_sf, b_sf, alpha, out_dtype)
    return torch.ops.fouroversix.gemm_mxfp4mxfp4_accum_fp32_out_bf16_tnt.default(a, b, a_sf, b_sf, alpha)


def dequantize(values, scale_factors, amax, dtype, sf_layout, divisor, rows, cols, out_dtype, f32_intermediate=False):
    return torch.ops.fouroversix.dequantize.default(
        values, scale_factors, amax, dtype, sf_layout, divisor, rows, cols, out_dtype, f32_intermediate
    )
