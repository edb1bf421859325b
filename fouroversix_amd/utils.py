"""Enumerations and per-format tables of the quantize / FP4-matmul path.

Mirrors the public names and values of the reference's ``src/fouroversix/utils.py``
(``DataType`` :13-189, ``MatmulBackend`` :192-203, ``QuantizeBackend`` :206-220,
``RoundStyle`` :223-247, ``ScaleRule`` :250-285, ``ScaleType`` :288-320,
``QuantizedValueType`` :323-383) so that configs written for the reference keep
working.  The per-format facts live in one table (``_FORMATS``) instead of one dict
per property.  Only ``nvfp4`` and ``if4`` have gfx950 kernels; the other members
exist so that configs naming them are parsed and then rejected by ``can_quantize``.
"""

from __future__ import annotations

from enum import Enum
from typing import NamedTuple

import torch


class QuantizedValueType(str, Enum):
    """Element encodings a block-scaled format can hold."""

    fp3 = "fp3"
    fp4 = "fp4"
    fp6_e2m3 = "fp6_e2m3"
    fp6_e3m2 = "fp6_e3m2"
    if3 = "if3"
    if4 = "if4"
    if6_e2m3 = "if6_e2m3"
    if6_e3m2 = "if6_e3m2"
    int3 = "int3"
    int4 = "int4"
    int6 = "int6"

    def get_maximum_value(self, scale_rule: "ScaleRule") -> float:
        """Largest magnitude a block is scaled to (4 under ``static_4``)."""
        if scale_rule == ScaleRule.static_4:
            return 4
        return _VALUE_MAX[self]

    @property
    def packing_factor(self) -> int:
        """Elements per stored byte (2 for the 4-bit encodings, else 1)."""
        return 2 if self in _FOUR_BIT else 1


_VALUE_MAX = {
    QuantizedValueType.fp3: 4,
    QuantizedValueType.fp4: 6,
    QuantizedValueType.fp6_e2m3: 7.5,
    QuantizedValueType.fp6_e3m2: 28,
    QuantizedValueType.if3: 4,
    QuantizedValueType.if4: 6,
    QuantizedValueType.if6_e2m3: 7.5,
    QuantizedValueType.if6_e3m2: 28,
    QuantizedValueType.int3: 3,
    QuantizedValueType.int4: 7,
    QuantizedValueType.int6: 31,
}
_FOUR_BIT = {QuantizedValueType.fp4, QuantizedValueType.if4, QuantizedValueType.int4}


class ScaleType(str, Enum):
    """Block-scale encodings: ``mx`` = E8M0, ``nv`` = E4M3, ``nv_if`` = E4M3 whose
    sign bit marks integer-coded blocks."""

    mx = "mx"
    nv = "nv"
    nv_if = "nv_if"

    def get_maximum_value(self, scale_rule: "ScaleRule") -> int | None:
        """Largest block scale: 448, or 256 for the adaptive 4/6 rules on ``nv``."""
        if self == ScaleType.mx:
            return None
        if self == ScaleType.nv and not scale_rule.is_static:
            return 256
        return 448

    @property
    def torch_dtype(self) -> torch.dtype:
        return torch.float8_e8m0fnu if self == ScaleType.mx else torch.float8_e4m3fn


class ScaleRule(str, Enum):
    """How a block picks between scaling its maximum to 6 or to 4."""

    abs_max = "abs_max"
    mae = "mae"
    mse = "mse"
    static_4 = "static_4"
    static_6 = "static_6"

    @property
    def cuda_id(self) -> int:
        """Integer id of the rule at the native boundary (0 static_6, 1 static_4,
        2 mae, 3 mse, 4 abs_max)."""
        return _RULE_IDS[self]

    @property
    def is_static(self) -> bool:
        return self in (ScaleRule.static_4, ScaleRule.static_6)


_RULE_IDS = {
    ScaleRule.static_6: 0,
    ScaleRule.static_4: 1,
    ScaleRule.mae: 2,
    ScaleRule.mse: 3,
    ScaleRule.abs_max: 4,
}


class RoundStyle(str, Enum):
    """Round-to-nearest-even, or dithered rounding (optionally with the 16/17
    range shrink that makes it unbiased at the top of the range)."""

    nearest = "nearest"
    stochastic = "stochastic"
    stochastic_unbiased = "stochastic_unbiased"

    @property
    def adjustment_factor(self) -> float:
        return 16 / 17 if self == RoundStyle.stochastic_unbiased else 1

    @property
    def is_stochastic(self) -> bool:
        return self != RoundStyle.nearest

    @property
    def native_id(self) -> int:
        """Integer id at the native boundary (0 nearest, 1 stochastic, 2 unbiased)."""
        return ("nearest", "stochastic", "stochastic_unbiased").index(self.value)


class QuantizeBackend(str, Enum):
    """Accepted for source compatibility; every member resolves to the one gfx950
    implementation."""

    cuda = "cuda"
    pytorch = "pytorch"
    transformer_engine = "transformer_engine"
    triton = "triton"
    hip = "hip"


class MatmulBackend(str, Enum):
    """Accepted for source compatibility; every member resolves to the one gfx950
    implementation."""

    cutlass = "cutlass"
    triton = "triton"
    pytorch = "pytorch"
    hip = "hip"


class _Format(NamedTuple):
    block: int
    value: QuantizedValueType
    scale: ScaleType
    rules: str  # "all" | "static" | "adaptive" | "static_6"


_V, _S = QuantizedValueType, ScaleType
_FORMATS: dict[str, _Format] = {
    "mxfp3": _Format(32, _V.fp3, _S.mx, "static"),
    "mxfp3_bs8": _Format(8, _V.fp3, _S.mx, "static"),
    "mxfp4": _Format(32, _V.fp4, _S.mx, "static"),
    "mxfp4_bs8": _Format(8, _V.fp4, _S.mx, "static"),
    "mxfp6_e2m3": _Format(32, _V.fp6_e2m3, _S.mx, "static"),
    "mxfp6_e3m2": _Format(32, _V.fp6_e3m2, _S.mx, "static"),
    "nvfp3": _Format(16, _V.fp3, _S.nv, "static_6"),
    "nvfp3_bs8": _Format(8, _V.fp3, _S.nv, "static_6"),
    "nvfp4": _Format(16, _V.fp4, _S.nv, "all"),
    "nvfp4_bs8": _Format(8, _V.fp4, _S.nv, "all"),
    "nvfp6_e2m3": _Format(16, _V.fp6_e2m3, _S.nv, "static_6"),
    "nvfp6_e3m2": _Format(16, _V.fp6_e3m2, _S.nv, "static_6"),
    "nvint3": _Format(16, _V.int3, _S.nv, "static_6"),
    "nvint3_bs8": _Format(8, _V.int3, _S.nv, "static_6"),
    "nvint4": _Format(16, _V.int4, _S.nv, "static_6"),
    "nvint4_bs8": _Format(8, _V.int4, _S.nv, "static_6"),
    "nvint6": _Format(16, _V.int6, _S.nv, "static_6"),
    "if3": _Format(16, _V.if3, _S.nv_if, "adaptive"),
    "if3_bs8": _Format(8, _V.if3, _S.nv_if, "adaptive"),
    "if4": _Format(16, _V.if4, _S.nv_if, "adaptive"),
    "if4_bs8": _Format(8, _V.if4, _S.nv_if, "adaptive"),
    "if6_e2m3": _Format(16, _V.if6_e2m3, _S.nv_if, "adaptive"),
    "if6_e3m2": _Format(16, _V.if6_e3m2, _S.nv_if, "adaptive"),
}
_HIGH_PRECISION = {
    "bfloat16": torch.bfloat16,
    "float16": torch.float16,
    "float32": torch.float32,
}


def _make_datatype() -> type:
    names = list(_HIGH_PRECISION) + list(_FORMATS)
    return Enum("DataType", {n: n for n in names}, type=str, module=__name__)


DataType = _make_datatype()
DataType.__doc__ = "High-precision dtypes and block-scaled quantized formats."


def _fmt(self: "DataType") -> _Format | None:
    return _FORMATS.get(self.value)


def _block_size(self: "DataType") -> int | None:
    f = _fmt(self)
    return f.block if f else None


def _value_type(self: "DataType") -> QuantizedValueType | None:
    f = _fmt(self)
    return f.value if f else None


def _scale_type(self: "DataType") -> ScaleType | None:
    f = _fmt(self)
    return f.scale if f else None


_RULES_CACHE: dict = {}


def _rules(self: "DataType") -> frozenset[ScaleRule]:
    cached = _RULES_CACHE.get(self)
    if cached is not None:
        return cached
    f = _fmt(self)
    if f is None:
        rules = frozenset()
    elif f.rules == "all":
        rules = frozenset(ScaleRule)
    elif f.rules == "static":
        rules = frozenset(r for r in ScaleRule if r.is_static)
    elif f.rules == "adaptive":
        rules = frozenset(r for r in ScaleRule if not r.is_static)
    else:
        rules = frozenset({ScaleRule.static_6})
    _RULES_CACHE[self] = rules
    return rules


def _torch_dtype(self: "DataType") -> torch.dtype | None:
    return _HIGH_PRECISION.get(self.value)


DataType.block_size = property(_block_size)
DataType.quantized_value_type = property(_value_type)
DataType.scale_type = property(_scale_type)
DataType.supported_scale_rules = property(_rules)
DataType.torch_dtype = property(_torch_dtype)

# Formats that have a gfx950 kernel, with their id at the native boundary.
NATIVE_FORMAT_IDS = {"nvfp4": 0, "if4": 1, "mxfp4": 2}
