"""``quantized_matmul``: the reference's frontend
(``src/fouroversix/matmul/frontend.py:18-132``) over the gfx950 FP4 GEMM.

``input @ other.T`` with both operands block-scaled 4-bit.  Operands given in high
precision are quantized first with ``input_config`` / ``other_config``.  The GEMM is the
native-op form of the reference (``src/fouroversix/matmul/cutlass/backend.py:56-155``):
``alpha = amaxA * amaxB / (qA * sA * qB * sB * adjA * adjB)`` stays on the device and the
padded result is cropped to ``(M, N)``.
"""

from __future__ import annotations

from typing import Any

import torch

from fouroversix_amd import _native as nat
from fouroversix_amd.quantize import QuantizationConfig, QuantizedTensor, quantize
from fouroversix_amd.quantize import ops
from fouroversix_amd.quantize.frontend import attach_known_amax, dequantize, dequantize_divisor
from fouroversix_amd.utils import NATIVE_FORMAT_IDS, DataType, MatmulBackend


def is_supported(input: QuantizedTensor, other: QuantizedTensor, *, out_dtype: DataType) -> bool:
    """Mirror of ``MatmulBackendBase.is_supported`` + the native backend's conditions."""
    if input.original_shape[1] != other.original_shape[1]:
        msg = (
            "The first input must be in row-major layout, the second input must be"
            "in column-major layout, and both inputs must have the same inner "
            "dimension"
        )
        raise ValueError(msg)
    return (
        input.dtype == other.dtype
        and input.dtype in (DataType.nvfp4, DataType.mxfp4)
        and input.device.type == "cuda"
        and out_dtype in (DataType.bfloat16, DataType.float16)
        and input.scale_factors_are_in_blackwell_layout
        and other.scale_factors_are_in_blackwell_layout
    )


def _dequantize_form_applies(input: QuantizedTensor, other: QuantizedTensor, out_dtype: DataType) -> bool:
    """Both operands are formats the dequantize kernel reads, on one GPU."""
    return (
        input.dtype.value in NATIVE_FORMAT_IDS
        and other.dtype.value in NATIVE_FORMAT_IDS
        and input.values.is_cuda
        and other.values.device == input.values.device
        and out_dtype in (DataType.bfloat16, DataType.float16, DataType.float32)
    )


def _members_fit(q: QuantizedTensor, values: torch.Tensor) -> bool:
    """The cheap form of the op's argument checks for the members of a QuantizedTensor: packed
    codes and E4M3 scales of the padded shape (or its first rows), contiguous, on the GPU."""
    rows_p, cols_p = q.padded_shape
    sf = q.scale_factors
    return (
        values.dtype == torch.uint8
        and values.dim() == 2
        and values.shape[1] * 2 == cols_p
        and (values.shape[0] == rows_p or (values.shape[0] < 128 == rows_p and cols_p % 256 == 0))
        and values.is_contiguous()
        and sf.dtype == torch.float8_e4m3fn
        and sf.numel() * 16 == rows_p * cols_p
        and sf.is_contiguous()
        and sf.device == values.device
    )


# What the NVFP4 GEMM needs to know about an operand, looked up once per QuantizedTensor and kept on it
# while its three tensors are the same objects (a layer's weights are the same object in every call):
# (values, scale_factors, amax, usable, kernel_values, divisor, device, inner).  `usable`: NVFP4 in the
# tiled scale layout whose members pass the op's checks, with an f32 maximum on the same GPU;
# `kernel_values`: the codes the kernel reads (the real rows only for a small batch).
_GEMM_RECORD = "_fos_gemm_record"


def _gemm_record(q: QuantizedTensor) -> tuple:
    values, sf, amax = q.values, q.scale_factors, q.amax
    rec = q.__dict__.get(_GEMM_RECORD)
    if (
        rec is not None
        and rec[0] is values
        and rec[1] is sf
        and rec[2] is amax
        and rec[8] is q.scale_rule
        and rec[9] is q.round_style
        and rec[10] == q.original_shape
        and rec[11] == q.padded_shape
    ):
        return rec
    kernel_values = values
    m_orig = q.original_shape[0]
    if m_orig < 128 and values.dim() == 2 and values.shape[0] == 128 and values.shape[1] % 128 == 0:
        kernel_values = values[:m_orig]  # small batch: only the real rows, so the kernel skips the padding
    usable = (
        q.dtype == DataType.nvfp4
        and q.scale_factors_are_in_blackwell_layout
        and type(values) is torch.Tensor
        and values.is_cuda
        and amax is not None
        and amax.dtype == torch.float32
        and amax.device == values.device
        and _members_fit(q, kernel_values)
    )
    rec = (values, sf, amax, usable, kernel_values, dequantize_divisor(q) if usable else 0.0, values.device,
           q.original_shape[1], q.scale_rule, q.round_style, q.original_shape, q.padded_shape)
    q.__dict__[_GEMM_RECORD] = rec
    return rec


_UNIT_ALPHA: dict = {}


def _unit_alpha(device: torch.device) -> torch.Tensor:
    """A device f32[1] holding 1.0, made once per device (never written afterwards)."""
    if torch.compiler.is_compiling():
        return torch.ones(1, dtype=torch.float32, device=device)
    one = _UNIT_ALPHA.get(device)
    if one is None:
        one = _UNIT_ALPHA[device] = torch.ones(1, dtype=torch.float32, device=device)
    return one


# Words that receive max|output| of a GEMM (emit_amax): the kernel folds into the word with an unsigned
# atomic max, so it has to start at zero.  Outside a graph capture the words come from a zero-filled
# block per (device, stream), one fresh word per call (a fill kernel per call would cost a decode-sized
# GEMM a third of its time; the block's one fill is ordered before its words' uses by the stream); a
# captured call gets a word of its own with its own fill, which replays with it.
_AMAX_WORDS = 4096
_AMAX_POOL: dict = {}


def _fresh_amax_word(device: torch.device) -> torch.Tensor:
    if torch.cuda.is_current_stream_capturing():
        return torch.zeros(1, dtype=torch.float32, device=device)
    key = (device, nat.current_stream(device))
    slot = _AMAX_POOL.get(key)
    if slot is None or slot[1] == _AMAX_WORDS:
        slot = _AMAX_POOL[key] = [torch.zeros(_AMAX_WORDS, dtype=torch.float32, device=device), 0]
    word = slot[0][slot[1] : slot[1] + 1]
    slot[1] += 1
    return word


def gemm_alpha(input: QuantizedTensor, other: QuantizedTensor) -> torch.Tensor:
    """``(amaxA * amaxB) / (qA sA qB sB adjA adjB)`` as a device f32[1] (reference
    matmul/cutlass/backend.py:86-98); one small kernel when both maxima are f32 GPU tensors."""
    den = dequantize_divisor(input) * dequantize_divisor(other)
    a, b = input.amax, other.amax
    if a.dtype == torch.float32 and b.dtype == torch.float32 and a.is_cuda and b.device == a.device:
        alpha = torch.empty(1, dtype=torch.float32, device=a.device)
        ops.gemm_alpha_into(a, b, den, alpha)
        return alpha
    return ((a * b) / den).to(torch.float32).reshape(1)


def quantized_matmul(
    input: torch.Tensor | QuantizedTensor,
    other: torch.Tensor | QuantizedTensor,
    *,
    backend: MatmulBackend | None = None,
    input_config: QuantizationConfig | None = None,
    other_config: QuantizationConfig | None = None,
    out_dtype: DataType = DataType.bfloat16,
    **kwargs: dict[str, Any],
) -> torch.Tensor:
    """FP4 matrix product ``input @ other.T`` -> ``[M, N]`` tensor of ``out_dtype``.

    ``emit_amax=True`` (no counterpart in the reference) lets the NVFP4 GEMM record max|out| while
    it stores it and attaches it to the result (``known_amax``), so that a following
    ``quantize(out)`` skips its own reduction pass over the tensor.  ``bias=`` (a ``[N]`` tensor, no
    counterpart either) returns ``out + bias``: the NVFP4 GEMM adds it in its epilogue with the two
    roundings of that expression, and the recorded maximum is then that of the sum.  The tag is dropped
    only by writes that torch counts (see ``attach_known_amax``)."""
    emit_amax = bool(kwargs.pop("emit_amax", False))
    bias = kwargs.pop("bias", None)
    del kwargs
    if isinstance(input, torch.Tensor):
        input = quantize(input, input_config)
    if isinstance(other, torch.Tensor):
        other = quantize(other, other_config)
    if isinstance(out_dtype, str):
        out_dtype = DataType(out_dtype)

    # two NVFP4 operands on one GPU: straight to the kernel, which forms alpha from the two maxima itself
    # (same arithmetic as gemm_alpha, one launch less)
    ra, rb = _gemm_record(input), _gemm_record(other)
    if (
        ra[3]
        and rb[3]
        and ra[6] == rb[6]
        and ra[7] == rb[7]
        and (out_dtype is DataType.bfloat16 or out_dtype is DataType.float16)
        and not torch.compiler.is_compiling()
    ):
        torch_dtype = torch.bfloat16 if out_dtype is DataType.bfloat16 else torch.float16
        fused_bias = (
            bias is not None
            and bias.dtype == torch_dtype
            and bias.dim() == 1
            and bias.shape[0] == rb[0].shape[0]  # (no row padding of the weight between the bias and the product)
            and bias.device == ra[6]
            and bias.is_contiguous()
            and bias.data_ptr() % 8 == 0
        )
        d_amax = _fresh_amax_word(ra[6]) if emit_amax and (bias is None or fused_bias) else None
        out = ops.gemm_nvfp4_from_amax(
            ra[4], rb[0], ra[1], rb[1], ra[2], rb[2], ra[5] * rb[5], torch_dtype, d_amax, True,
            bias.detach() if fused_bias else None,
        )
        m, n = input.original_shape[0], other.original_shape[0]
        if out.shape[0] != m or out.shape[1] != n:
            out = out[:m, :n]  # (the padding is zeros: same maximum)
        if d_amax is not None:
            attach_known_amax(out, d_amax)
        if bias is not None and not fused_bias:
            out = out + bias
        return out

    if not is_supported(input, other, out_dtype=out_dtype):
        if _dequantize_form_applies(input, other, out_dtype):
            # formats without a native GEMM (IF4; mixed formats): the reference's PyTorch backend,
            # ``matmul(dequantize(a, f32), dequantize(b, f32).T)`` rounded to the output type
            # (src/fouroversix/matmul/pytorch.py:33-52) -- the dequantize kernel plus a library GEMM
            out = torch.matmul(
                dequantize(input, dtype=torch.float32), dequantize(other, dtype=torch.float32).T
            ).to(out_dtype.torch_dtype)
            out_shape = (input.original_shape[0], other.original_shape[0])
            out = out if tuple(out.shape) == out_shape else out[: out_shape[0], : out_shape[1]]
            return out if bias is None else out + bias
        if backend is None:
            msg = "No backend found that supports the given parameters"
        else:
            msg = f"Backend {backend} does not support the given parameters"
        raise ValueError(msg)

    out_shape = (input.original_shape[0], other.original_shape[0])
    if input.dtype == DataType.mxfp4:
        # no tensor scale: alpha = 1 (src/fouroversix/matmul/cutlass/backend.py:79-85)
        alpha = _unit_alpha(input.values.device)
        out = ops.gemm_mxfp4mxfp4_accum_fp32_out_bf16_tnt(
            input.values, other.values, input.scale_factors, other.scale_factors, alpha,
            torch.bfloat16 if out_dtype == DataType.bfloat16 else torch.float16,
        )
        out = out if tuple(out.shape) == out_shape else out[: out_shape[0], : out_shape[1]]
        return out if bias is None else out + bias

    a_values = input.values
    m_orig = input.original_shape[0]
    if m_orig < 128 and a_values.shape[0] == 128 and a_values.shape[1] % 128 == 0:
        # small batch: hand over only the real rows, so the kernel skips the padding
        a_values = a_values[:m_orig]
    # (torch.compile, or maxima that are not f32 tensors on the GPU: alpha from its own small kernel or from
    # torch arithmetic; emit_amax has no effect here and the next quantize finds the maximum itself)
    alpha = gemm_alpha(input, other)
    gemm = (
        ops.gemm_nvfp4nvfp4_accum_fp32_out_bf16_tnt
        if out_dtype == DataType.bfloat16
        else ops.gemm_nvfp4nvfp4_accum_fp32_out_fp16_tnt
    )
    out = gemm(a_values, other.values, input.scale_factors, other.scale_factors, alpha)
    out_shape = (input.original_shape[0], other.original_shape[0])
    if tuple(out.shape) != out_shape:
        out = out[: out_shape[0], : out_shape[1]]
    return out if bias is None else out + bias
