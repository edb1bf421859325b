"""``quantize`` / ``dequantize``: the reference's frontends
(``src/fouroversix/quantize/frontend.py:19-157``) over the gfx950 kernels.

There is one implementation, so the reference's backend auto-selection collapses to a
support check with the same outcome for the caller: a ``ValueError`` when nothing can
quantize the given tensor/config.  The result follows the reference's PyTorch backend
(``src/fouroversix/quantize/pytorch/backend.py:39-121``): values padded to (128, 64)
multiples, NVFP4 scales in the 128x4-tile layout, IF4 scales row-major, 0-dim fp32 amax.
"""

from __future__ import annotations

import functools
import warnings

import torch

from fouroversix_amd import _native as nat
from fouroversix_amd.utils import NATIVE_FORMAT_IDS, DataType, QuantizeBackend, ScaleType

from . import ops
from .config import QuantizationConfig
from .quantized_tensor import QuantizedTensor

_LINEAR_SCALE_FORMATS = {DataType.if4, DataType.nvint4}
_DEFAULT_CONFIG = QuantizationConfig()


def unsupported_reason(x: torch.Tensor, config: QuantizationConfig) -> str | None:
    """Why this (tensor, config) cannot be quantized, or None if it can."""
    if x.ndim != 2:
        return "input must be 2-D"
    if config.scale_rule not in config.dtype.supported_scale_rules:
        return f"scale rule {config.scale_rule.value} is not defined for {config.dtype.value}"
    if config.dtype.value not in NATIVE_FORMAT_IDS:
        return f"format {config.dtype.value} has no gfx950 kernel"
    if x.device.type != "cuda":
        return f"input must live on the GPU, got {x.device}"
    if x.dtype not in (torch.bfloat16, torch.float16, torch.float32):
        return f"input must be bfloat16, float16 or float32, got {x.dtype}"
    if config.dtype == DataType.mxfp4 and (config.block_scale_2d or config.round_style.is_stochastic):
        return "mxfp4 has kernels for 1x32 blocks with round-to-nearest only"
    if config.rht or config.transpose:
        return ops.transform_unsupported_reason(x, config.transpose, config.rht)
    return None


def can_quantize(x: torch.Tensor, config: QuantizationConfig) -> bool:
    return unsupported_reason(x, config) is None


def _quantize_meta(x: torch.Tensor, config: QuantizationConfig) -> QuantizedTensor | torch.Tensor:
    """Shapes only, for tensors on the meta device (model construction before weights are
    loaded): zero-filled meta tensors of the padded sizes, as the reference's PyTorch backend
    returns (``src/fouroversix/quantize/pytorch/backend.py:57-97``)."""
    if config.pseudo_quantize:
        return torch.empty_like(x)
    shape = (x.shape[1], x.shape[0]) if config.transpose else tuple(x.shape)
    block = config.dtype.block_size
    rows_p, cols_p = -(-shape[0] // 128) * 128, -(-shape[1] // (4 * block)) * (4 * block)
    sf_dtype = config.dtype.scale_type.torch_dtype
    if sf_dtype == torch.float8_e8m0fnu:
        sf_dtype = torch.uint8
    linear = config.dtype in _LINEAR_SCALE_FORMATS
    return QuantizedTensor(
        torch.zeros(rows_p, cols_p // config.dtype.quantized_value_type.packing_factor, dtype=torch.uint8, device=x.device),
        torch.zeros(rows_p * cols_p // block, dtype=sf_dtype, device=x.device),
        torch.zeros(1, dtype=torch.float32, device=x.device),
        config.dtype,
        tuple(shape),
        config.scale_rule,
        config.round_style,
        scale_factors_are_in_blackwell_layout=not linear,
    )


# max|x| that a producer already has (the FP4 GEMM can record it while storing its output): kept
# as an attribute of the tensor object together with the tensor's version counter, so that an
# in-place write, or any operation that returns a new tensor, drops it.  Only writes that torch
# counts are seen: a write through ``x.data``, through a raw pointer (this library's own C entry
# points, an ``out=`` kernel of another extension) leaves the counter, and with it the tag, as it was.
# Tensors made under ``torch.inference_mode()`` have no version counter: they are never tagged and
# ``quantize`` finds their maximum itself.
_KNOWN_AMAX = "_fos_known_amax"


def _version_or_none(x: torch.Tensor) -> int | None:
    if x.is_inference():
        return None
    try:
        return x._version
    except RuntimeError:  # tensors that do not track a version counter
        return None


def attach_known_amax(x: torch.Tensor, amax: torch.Tensor) -> torch.Tensor:
    """Record ``amax`` (device f32[1] = max|x|) on ``x`` for a later ``quantize(x)``; without effect
    on tensors that have no version counter (inference tensors)."""
    version = _version_or_none(x)
    if version is not None:
        # (address and shape as well: a tag copied along with the object's attributes onto other storage is not believed)
        setattr(x, _KNOWN_AMAX, (amax, version, x.data_ptr(), x.shape))
    return x


def known_amax(x: torch.Tensor) -> torch.Tensor | None:
    """The maximum recorded by ``attach_known_amax`` if ``x`` has not been written since."""
    tag = getattr(x, _KNOWN_AMAX, None)
    if tag is None or tag[0].device != x.device or tag[1] != _version_or_none(x) or tag[2] != x.data_ptr() or tag[3] != x.shape:
        return None
    return tag[0]


def quantize(
    x: torch.Tensor,
    config: QuantizationConfig | None = None,
) -> QuantizedTensor | torch.Tensor:
    """Quantize a 2-D bf16, fp16 or fp32 GPU tensor to a block-scaled 4-bit format.

    With no config: NVFP4, 1x16 blocks, round-to-nearest, 4/6 selection by block MSE.
    ``config.kwargs`` may carry ``seed`` / ``offset`` (ints) keying the dither of the
    stochastic rounding styles (default: drawn from torch's global generator), or ``key``
    (an int64[2] tensor {seed, offset} on x's device, read when the kernels run: a call
    recorded into a graph rounds with whatever the tensor holds at each replay), and
    ``amax`` (a tensor) to skip the tensor-wide maximum pass.
    """
    if config is None:
        config = _DEFAULT_CONFIG  # (read only)

    if x.device.type == "meta" and x.dim() == 2:
        return _quantize_meta(x, config)

    reason = unsupported_reason(x, config)
    if reason is not None:
        if config.backend is None:
            msg = f"No backend found that supports the given parameters ({reason})"
        else:
            msg = f"Backend {config.backend} does not support the given parameters ({reason})"
        raise ValueError(msg)

    key = config.kwargs.get("key") if config.round_style.is_stochastic else None
    if key is not None:
        seed = 0  # (the kernels read {seed, offset} from the tensor when they run)
    elif config.round_style.is_stochastic and "seed" not in config.kwargs:
        if x.is_cuda and torch.cuda.is_current_stream_capturing():
            # the seed is a launch argument: a graph replays the one drawn now, every time
            warnings.warn(
                "stochastic rounding captured into a graph without kwargs['key'] (an int64[2] device tensor holding seed "
                "and offset, which the captured code can advance): every replay will round with the same random bits",
                stacklevel=2,
            )
        seed = int(torch.randint(0, 2**62, (1,)).item())
    else:
        seed = int(config.kwargs.get("seed", config.kwargs.get("rbits", 0)))
        seed = max(seed, 0)
    offset = int(config.kwargs.get("offset", 0))

    if config.transpose or config.rht:
        # x.T and / or the random Hadamard transform first (reference
        # quantize/pytorch/reference.py:567-571), as one pass that also yields the tensor
        # maximum; the rest is the plain path on the transformed tensor
        if "amax" in config.kwargs:
            msg = "kwargs['amax'] cannot be combined with transpose / rht (the maximum is that of the transformed tensor)"
            raise ValueError(msg)
        # the logical shape is that of x (transposed); a ragged width that the Hadamard transform
        # filled up to a multiple of 16 keeps its codes in the padding, as in the reference
        # (src/fouroversix/quantize/pytorch/backend.py:57-79,110-121)
        logical_shape = (x.shape[1], x.shape[0]) if config.transpose else tuple(x.shape)
        if not config.pseudo_quantize and key is None and config.dtype != DataType.mxfp4:
            # both steps in one call into the library (pass 2 reduces the transform's partial maxima itself)
            linear = config.dtype in _LINEAR_SCALE_FORMATS
            values, scale_factors, amax = ops.transform_quantize(
                x,
                config.transpose,
                config.rht,
                NATIVE_FORMAT_IDS[config.dtype.value],
                config.scale_rule.cuda_id,
                config.round_style.native_id,
                config.block_scale_2d,
                seed,
                offset,
                nat.SF_LINEAR if linear else nat.SF_TILED,
            )
            return QuantizedTensor.from_kernel(
                values,
                scale_factors,
                amax.reshape(()),
                config.dtype,
                logical_shape,
                config.scale_rule,
                config.round_style,
                (values.shape[0], values.shape[1] * config.dtype.quantized_value_type.packing_factor),
                not linear,
            )
        y, amax = ops.transform(x, config.transpose, config.rht)
        plain = QuantizationConfig(
            **{
                **config.__dict__,
                "transpose": False,
                "rht": False,
                "kwargs": {**config.kwargs, "amax": amax, "seed": seed, "offset": offset},
            }
        )
        q = quantize(y, plain)
        if isinstance(q, QuantizedTensor):
            q.original_shape = logical_shape
        return q

    if config.pseudo_quantize:
        # one fused kernel where the library has it, else the two-step round trip
        # (QuantizeBackendBase.pseudo_quantize, src/fouroversix/quantize/backend.py:213-234)
        fmt, style = NATIVE_FORMAT_IDS[config.dtype.value], config.round_style.native_id
        if key is None and ops.pseudo_quantize_is_fused(x, fmt, config.scale_rule.cuda_id, style, config.block_scale_2d):
            return ops.pseudo_quantize(
                x, fmt, config.scale_rule.cuda_id, style, config.block_scale_2d, config.kwargs.get("amax", known_amax(x)), seed, offset
            )
        plain = QuantizationConfig(
            **{**config.__dict__, "pseudo_quantize": False, "kwargs": {**config.kwargs, "seed": seed, "offset": offset}}
        )
        return dequantize(quantize(x, plain), dtype=x.dtype)

    linear = config.dtype in _LINEAR_SCALE_FORMATS

    x_rows = x if x.stride(-1) == 1 else x.contiguous()
    values, scale_factors, amax = ops.quantize_ex(
        x_rows,
        NATIVE_FORMAT_IDS[config.dtype.value],
        config.scale_rule.cuda_id,
        config.round_style.native_id,
        config.block_scale_2d,
        seed,
        offset,
        nat.SF_LINEAR if linear else nat.SF_TILED,
        None if config.dtype == DataType.mxfp4 else config.kwargs.get("amax", known_amax(x)),  # mxfp4 has no tensor scale
        key,
    )
    return QuantizedTensor.from_kernel(
        values,
        scale_factors,
        amax.reshape(()),
        config.dtype,
        (x.shape[0], x.shape[1]),
        config.scale_rule,
        config.round_style,
        (values.shape[0], values.shape[1] * config.dtype.quantized_value_type.packing_factor),  # as the kernel padded it
        not linear,
    )


@functools.lru_cache(maxsize=None)
def _divisor(dtype: DataType, scale_rule, round_style) -> float:
    return (
        dtype.quantized_value_type.get_maximum_value(scale_rule)
        * dtype.scale_type.get_maximum_value(scale_rule)
        * round_style.adjustment_factor
    )


def dequantize_divisor(tensor: QuantizedTensor) -> float:
    """qmax * smax * adjustment of the tensor's scale rule and rounding style."""
    return _divisor(tensor.dtype, tensor.scale_rule, tensor.round_style)


def dequantize(
    tensor: QuantizedTensor,
    dtype: torch.dtype = torch.bfloat16,
    *,
    backend: QuantizeBackend | None = None,
    intermediate_dtype: torch.dtype = torch.float16,
) -> torch.Tensor:
    """High-precision tensor of ``tensor.original_shape`` from a quantized tensor.

    Value and block scale are multiplied in ``intermediate_dtype`` (fp16 or fp32; exact
    either way for NVFP4, different for IF4's integer blocks and for MXFP4 scales outside
    fp16's range), widened to fp32,
    scaled by ``amax / (qmax * smax * adjustment)`` and cast to ``dtype``.
    """
    del backend
    if tensor.dtype.value not in NATIVE_FORMAT_IDS:
        msg = f"No backend can dequantize {tensor.dtype.value}"
        raise ValueError(msg)
    if tensor.amax is None and tensor.dtype.scale_type != ScaleType.mx:
        msg = "dequantize needs the tensor-wide amax"
        raise ValueError(msg)
    if intermediate_dtype not in (torch.float16, torch.float32):
        msg = "intermediate_dtype must be float16 or float32"
        raise ValueError(msg)
    if dtype not in nat.TORCH_TO_T:
        msg = f"unsupported output dtype {dtype}"
        raise ValueError(msg)
    rows, cols = tensor.original_shape
    amax = tensor.amax if tensor.amax is not None else torch.ones(1, dtype=torch.float32, device=tensor.values.device)
    return ops.dequantize(
        tensor.values,
        tensor.scale_factors,
        amax,
        NATIVE_FORMAT_IDS[tensor.dtype.value],
        nat.SF_TILED if tensor.scale_factors_are_in_blackwell_layout else nat.SF_LINEAR,
        1.0 if tensor.dtype.scale_type == ScaleType.mx else float(dequantize_divisor(tensor)),
        rows,
        cols,
        dtype,
        intermediate_dtype == torch.float32,
    )
