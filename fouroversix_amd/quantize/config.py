"""``QuantizationConfig``: field-for-field the reference's dataclass
(``src/fouroversix/quantize/config.py:7-58``), including the str -> enum coercion."""

from __future__ import annotations

from dataclasses import dataclass, field
from typing import Any

from fouroversix_amd.utils import DataType, QuantizeBackend, RoundStyle, ScaleRule

_ENUM_FIELDS = {
    "backend": QuantizeBackend,
    "dtype": DataType,
    "round_style": RoundStyle,
    "scale_rule": ScaleRule,
}


@dataclass
class QuantizationConfig:
    """How to quantize one tensor.

    backend         kept for source compatibility; there is one implementation
    block_scale_2d  one scale (and one 4-vs-6 decision) per 16x16 tile instead of 1x16
    dtype           target format (``nvfp4`` or ``if4`` have kernels)
    kwargs          extra backend arguments: ``seed`` / ``offset`` of the dither stream
    pseudo_quantize return the quantize -> dequantize round trip as a high-precision tensor
    rht             random Hadamard transform of every 16 consecutive row elements before quantizing
    round_style     nearest / stochastic / stochastic_unbiased
    scale_rule      static_6, static_4, or the adaptive mse / mae / abs_max
    transpose       quantize the transposed input
    """

    backend: QuantizeBackend | None = None
    block_scale_2d: bool = False
    dtype: DataType = DataType.nvfp4
    kwargs: dict[str, Any] = field(default_factory=dict)
    pseudo_quantize: bool = False
    rht: bool = False
    round_style: RoundStyle = RoundStyle.nearest
    scale_rule: ScaleRule = ScaleRule.mse
    transpose: bool = False

    def __post_init__(self) -> None:
        for name, enum_cls in _ENUM_FIELDS.items():
            value = getattr(self, name)
            if isinstance(value, str) and not isinstance(value, enum_cls):
                setattr(self, name, enum_cls(value))
