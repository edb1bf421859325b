"""``torch.ops.fouroversix.*`` operators backed by the gfx950 library.

The operators are registered by the compiled extension ``fouroversix_amd._C``
(``csrc/torch_ops.cpp``): names and schemas are the reference's
(``src/fouroversix/csrc/bindings.cpp:26-35``), each implementation checks its arguments,
allocates the outputs and makes one call through the C ABI on the current stream.  This module
adds the fake (meta) shapes of ``src/fouroversix/quantize/cuda/ops.py:28-47`` and
``src/fouroversix/matmul/cutlass/ops.py:82-92``, so that code which calls the ops directly, or
traces them, keeps working, and the Python entry points the frontends use: real GPU tensors go
straight to the extension's functions (the dispatcher's boxing costs as much as a decode-sized
kernel takes), fake / meta tensors and tracing through the registered operators.
``quantize_ex`` / ``dequantize`` / ``transform`` / ``gemm_nvfp4_amax`` are additions carrying the
options the reference's native ops do not have (format, dither key, output layout, recorded maximum).
"""

from __future__ import annotations

import os

import torch

from fouroversix_amd import _native as nat

_EXT_PATH = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "_C.so")
if not os.path.exists(_EXT_PATH):
    msg = (
        f"{_EXT_PATH} not found: the PyTorch binding has not been built "
        "(run `python fouroversix_amd/build.py`); there is no fallback path"
    )
    raise nat.NativeLibraryError(msg)
nat.lib()  # (the binding links against the C-ABI library next to it: fail with its message if that is missing)
from fouroversix_amd import _C  # noqa: E402  (registers the fouroversix:: operators)

MXFP4 = 2  # format id at the native boundary (blocks of 32, E8M0 scales)


def _padded(rows: int, cols: int, dtype: int = 0) -> tuple[int, int]:
    col_multiple = 128 if dtype == MXFP4 else 64  # four blocks
    return -(-rows // 128) * 128, -(-cols // col_multiple) * col_multiple


def _direct(t: torch.Tensor) -> bool:
    return type(t) is torch.Tensor and t.device.type == "cuda" and not torch.compiler.is_compiling()


def pseudo_quantize_is_fused(x: torch.Tensor, dtype: int, selection_rule: int, round_style: int, is_2d: bool) -> bool:
    """True when the library has a fused quantize->dequantize kernel for this call."""
    return _C.pseudo_quantize_is_fused(x, dtype, selection_rule, round_style, is_2d)


def transform_unsupported_reason(x: torch.Tensor, transpose: bool, rht: bool) -> str | None:
    """Why the transpose / random-Hadamard pre-transform cannot run on ``x``, or None."""
    return None if x.dim() == 2 else "transpose / rht need a 2-D tensor"


def quantize(x, is_nvfp4, is_rtn, is_rht, is_2d, is_transpose, selection_rule, rbits):
    """Same call as the reference's ``fouroversix.quantize.cuda.ops.quantize``."""
    return torch.ops.fouroversix.quantize.default(
        x, is_nvfp4, is_rtn, is_rht, is_2d, is_transpose, selection_rule, rbits
    )


def quantize_ex(x, dtype, selection_rule, round_style, is_2d, seed, offset, sf_layout, amax=None, key=None):
    """Extended quantize: ``(values, scale_factors, amax)``.  ``key``: int64[2] device tensor {seed, offset}
    that the kernels read when they run, in place of the two integers (for launches recorded into a graph)."""
    seed, offset = seed & 0x7FFFFFFFFFFFFFFF, offset & 0x7FFFFFFFFFFFFFFF
    if _direct(x):
        return _C.quantize_ex(x, dtype, selection_rule, round_style, is_2d, seed, offset, sf_layout, amax, key)
    return torch.ops.fouroversix.quantize_ex.default(
        x, dtype, selection_rule, round_style, is_2d, seed, offset, sf_layout, amax, key
    )


def transform(x, transpose, rht):
    """Pre-transform of the ``transpose`` / ``rht`` quantize options: ``(y, amax)``."""
    if _direct(x):
        return _C.transform(x, transpose, rht)
    return torch.ops.fouroversix.transform.default(x, transpose, rht)


def transform_quantize(x, transpose, rht, dtype, selection_rule, round_style, is_2d, seed, offset, sf_layout):
    """``transform`` and ``quantize_ex`` of its result in one call into the library: ``(values, scale_factors,
    amax)`` of the transformed tensor (NVFP4 / IF4)."""
    seed, offset = seed & 0x7FFFFFFFFFFFFFFF, offset & 0x7FFFFFFFFFFFFFFF
    if _direct(x):
        return _C.transform_quantize(x, transpose, rht, dtype, selection_rule, round_style, is_2d, seed, offset, sf_layout)
    return torch.ops.fouroversix.transform_quantize.default(
        x, transpose, rht, dtype, selection_rule, round_style, is_2d, seed, offset, sf_layout
    )


def pseudo_quantize(x, dtype, selection_rule, round_style, is_2d, amax=None, seed=0, offset=0):
    """Fused quantize -> dequantize (out has x's type); see ``pseudo_quantize_is_fused``.  ``seed`` /
    ``offset`` key the dither of the stochastic styles, as in ``quantize_ex``."""
    seed, offset = seed & 0x7FFFFFFFFFFFFFFF, offset & 0x7FFFFFFFFFFFFFFF
    if _direct(x):
        return _C.pseudo_quantize(x, dtype, selection_rule, round_style, is_2d, amax, seed, offset)
    return torch.ops.fouroversix.pseudo_quantize.default(x, dtype, selection_rule, round_style, is_2d, amax, seed, offset)


def gemm_nvfp4nvfp4_accum_fp32_out_bf16_tnt(a, b, a_sf, b_sf, alpha):
    if _direct(a):
        return _C.gemm_nvfp4(a, b, a_sf, b_sf, alpha, torch.bfloat16)
    return torch.ops.fouroversix.gemm_nvfp4nvfp4_accum_fp32_out_bf16_tnt.default(a, b, a_sf, b_sf, alpha)


def gemm_nvfp4nvfp4_accum_fp32_out_fp16_tnt(a, b, a_sf, b_sf, alpha):
    if _direct(a):
        return _C.gemm_nvfp4(a, b, a_sf, b_sf, alpha, torch.float16)
    return torch.ops.fouroversix.gemm_nvfp4nvfp4_accum_fp32_out_fp16_tnt.default(a, b, a_sf, b_sf, alpha)


def gemm_nvfp4_from_amax(a, b, a_sf, b_sf, amax_a, amax_b, denominator, out_dtype, d_amax=None, checked=False, bias=None):
    """The NVFP4 GEMM with the output scale ``(amax_a * amax_b) * f32(1 / denominator)`` formed
    in the kernel (``fos_gemm_nvfp4_amax``): one launch less than alpha + GEMM, same result.
    ``d_amax`` (device f32[1] holding 0) additionally receives max|out|.  ``checked``: the operands are
    the members of two QuantizedTensors on one GPU (the frontend has looked): only the shapes are compared.
    ``bias`` ([N], output type) is added to the rounded product and the sum rounded again, as ``out + bias``."""
    return _C.gemm_nvfp4_amax(a, b, a_sf, b_sf, amax_a, amax_b, denominator, out_dtype, d_amax, checked, bias)


def gemm_alpha_into(amax_a, amax_b, denominator, alpha):
    """alpha[0] = (amax_a * amax_b) * f32(1 / denominator) on the device, torch's GPU arithmetic for
    ``(amax_a * amax_b) / denominator``."""
    _C.gemm_alpha(amax_a, amax_b, float(denominator), alpha)


def gemm_mxfp4mxfp4_accum_fp32_out_bf16_tnt(a, b, a_sf, b_sf, alpha, out_dtype=torch.bfloat16):
    """Same call as the reference's ``matmul/cutlass/ops.py:6-20`` (fp16 output as an extension)."""
    if _direct(a):
        return _C.gemm_mxfp4(a, b, a_sf, b_sf, alpha, out_dtype)
    return torch.ops.fouroversix.gemm_mxfp4mxfp4_accum_fp32_out_bf16_tnt.default(a, b, a_sf, b_sf, alpha)


def dequantize(values, scale_factors, amax, dtype, sf_layout, divisor, rows, cols, out_dtype, f32_intermediate=False):
    if _direct(values):
        return _C.dequantize(values, scale_factors, amax, dtype, sf_layout, divisor, rows, cols, out_dtype, f32_intermediate)
    return torch.ops.fouroversix.dequantize.default(
        values, scale_factors, amax, dtype, sf_layout, divisor, rows, cols, out_dtype, f32_intermediate
    )


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
def _(x, dtype, selection_rule, round_style, is_2d, seed, offset, sf_layout, amax, key=None):
    return _fake_quantize_shapes(x, dtype)


@torch.library.register_fake("fouroversix::pseudo_quantize")
def _(x, dtype, selection_rule, round_style, is_2d, amax, seed=0, offset=0):
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


@torch.library.register_fake("fouroversix::transform")
def _(x, transpose, rht):
    rows, cols = (x.shape[1], x.shape[0]) if transpose else (x.shape[0], x.shape[1])
    width = -(-cols // 16) * 16 if rht else cols
    return torch.empty(rows, width, dtype=x.dtype, device=x.device), torch.empty(1, dtype=torch.float32, device=x.device)


@torch.library.register_fake("fouroversix::transform_quantize")
def _(x, transpose, rht, dtype, selection_rule, round_style, is_2d, seed, offset, sf_layout):
    rows, cols = (x.shape[1], x.shape[0]) if transpose else (x.shape[0], x.shape[1])
    width = -(-cols // 16) * 16 if rht else cols
    return _fake_quantize_shapes(torch.empty(rows, width, dtype=x.dtype, device=x.device), dtype)


@torch.library.register_fake("fouroversix::gemm_nvfp4_amax")
def _(a, b, a_sf, b_sf, amax_a, amax_b, denominator, out_dtype, d_amax, checked=False, bias=None):
    return torch.empty(a.shape[0], b.shape[0], dtype=out_dtype, device=a.device)
