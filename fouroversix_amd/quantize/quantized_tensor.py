"""``QuantizedTensor``: the container ``quantize`` returns and the GEMM consumes.

Same constructor order, attributes and padding rules as the reference's
``src/fouroversix/quantize/quantized_tensor.py:10-144``: values are padded to rows % 128
== 0 and cols % 64 == 0; 1-D scale tensors are taken to be in their final layout, 2-D
ones are padded (0 for nvfp4, 1 otherwise) and tiled when the tiled layout is claimed.
"""

from __future__ import annotations

import torch
import torch.nn.functional as F

from fouroversix_amd.utils import DataType, RoundStyle, ScaleRule

from .layout import to_blocked

ROW_MULTIPLE = 128
BLOCKS_PER_COL_GROUP = 4


def padded_shape_for(shape: tuple[int, int], dtype: DataType) -> tuple[int, int]:
    col_multiple = BLOCKS_PER_COL_GROUP * dtype.block_size
    return (-(-shape[0] // ROW_MULTIPLE) * ROW_MULTIPLE, -(-shape[1] // col_multiple) * col_multiple)


class QuantizedTensor:
    """Packed values + block scales + tensor scale of one quantized matrix."""

    values: torch.Tensor
    scale_factors: torch.Tensor
    amax: torch.Tensor
    dtype: DataType
    original_shape: tuple[int, int]
    scale_rule: ScaleRule
    round_style: RoundStyle
    padded_shape: tuple[int, int]
    scale_factors_are_in_blackwell_layout: bool

    def __init__(
        self,
        values: torch.Tensor,
        scale_factors: torch.Tensor,
        amax: torch.Tensor,
        dtype: DataType,
        original_shape: tuple[int, int],
        scale_rule: ScaleRule,
        round_style: RoundStyle,
        padded_shape: tuple[int, int] | None = None,
        *,
        scale_factors_are_in_blackwell_layout: bool = True,
    ) -> None:
        self.dtype = DataType(dtype) if isinstance(dtype, str) else dtype
        self.original_shape = tuple(int(v) for v in original_shape)
        self.scale_rule = ScaleRule(scale_rule) if isinstance(scale_rule, str) else scale_rule
        self.round_style = RoundStyle(round_style) if isinstance(round_style, str) else round_style
        self.scale_factors_are_in_blackwell_layout = scale_factors_are_in_blackwell_layout

        if padded_shape is not None:
            self.padded_shape = tuple(int(v) for v in padded_shape)
        else:
            self.padded_shape = padded_shape_for(self.original_shape, self.dtype)
            rows_p, cols_p = self.padded_shape
            pack = self.dtype.quantized_value_type.packing_factor
            n_values = rows_p * cols_p // pack
            n_scales = rows_p * cols_p // self.dtype.block_size

            if values.numel() != n_values:
                values = F.pad(values, (0, cols_p // pack - values.shape[1], 0, rows_p - values.shape[0]))

            if scale_factors.ndim > 1 and scale_factors.numel() != n_scales:
                # pad value 0 for nvfp4, 1.0 otherwise; one-byte float dtypes are padded
                # through their byte image (E4M3 1.0 = 0x38, E8M0 1.0 = 0x7F)
                sf_cols = cols_p // self.dtype.block_size
                pad = (0, sf_cols - scale_factors.shape[1], 0, rows_p - scale_factors.shape[0])
                if scale_factors.element_size() == 1 and scale_factors.dtype != torch.uint8:
                    one = 0x7F if scale_factors.dtype == torch.float8_e8m0fnu else 0x38
                    fill = 0 if self.dtype == DataType.nvfp4 else one
                    sf_dtype = scale_factors.dtype
                    scale_factors = F.pad(scale_factors.view(torch.uint8), pad, value=fill).view(sf_dtype)
                else:
                    scale_factors = F.pad(scale_factors, pad, value=0 if self.dtype == DataType.nvfp4 else 1)
                if self.scale_factors_are_in_blackwell_layout:
                    scale_factors = to_blocked(scale_factors)

            if values.numel() != n_values:
                msg = f"Expected {n_values} e2m1 values, got {values.numel()}"
                raise ValueError(msg)
            if scale_factors.numel() != n_scales:
                msg = f"Expected {n_scales} scale factors, got {scale_factors.numel()}"
                raise ValueError(msg)

        self.values = values
        self.scale_factors = scale_factors
        self.amax = amax

    @classmethod
    def from_kernel(cls, values, scale_factors, amax, dtype, original_shape, scale_rule, round_style, padded_shape,
                    tiled: bool) -> "QuantizedTensor":
        """What ``quantize`` builds from the kernel's outputs: members of the final sizes and enum-typed
        attributes, stored as they are (the constructor's conversions and padding have nothing to do)."""
        q = object.__new__(cls)
        q.dtype = dtype
        q.original_shape = original_shape
        q.scale_rule = scale_rule
        q.round_style = round_style
        q.scale_factors_are_in_blackwell_layout = tiled
        q.padded_shape = padded_shape
        q.values = values
        q.scale_factors = scale_factors
        q.amax = amax
        return q

    @property
    def device(self) -> torch.device:
        return self.values.device

    def __repr__(self) -> str:
        return (
            f"QuantizedTensor(dtype={self.dtype.value}, original_shape={self.original_shape}, "
            f"padded_shape={self.padded_shape}, scale_rule={self.scale_rule.value}, "
            f"round_style={self.round_style.value}, device={self.device})"
        )
