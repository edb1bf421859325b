"""Module / model quantization configs with the reference's fields and defaults
(``src/fouroversix/model/config.py:16-272``).  Only the forward-pass fields act here;
the gradient / Quartet-II fields are carried so that existing configs still parse."""

from __future__ import annotations

import hashlib
import json
from dataclasses import dataclass, field, fields
from typing import Any

from fouroversix_amd.quantize import QuantizationConfig
from fouroversix_amd.utils import DataType, MatmulBackend, QuantizeBackend, RoundStyle, ScaleRule

_ENUMS = {
    "activation_dtype": DataType,
    "activation_round_style": RoundStyle,
    "activation_scale_rule": ScaleRule,
    "dtype": DataType,
    "gradient_dtype": DataType,
    "gradient_round_style": RoundStyle,
    "gradient_scale_rule": ScaleRule,
    "matmul_backend": MatmulBackend,
    "output_dtype": DataType,
    "quantize_backend": QuantizeBackend,
    "quartet_ii_dtype": DataType,
    "scale_rule": ScaleRule,
    "weight_dtype": DataType,
    "weight_round_style": RoundStyle,
    "weight_scale_rule": ScaleRule,
}


@dataclass
class ModuleQuantizationConfig:
    """Quantization settings of one module.  ``None`` dtypes / scale rules fall back to
    ``dtype`` / ``scale_rule``."""

    activation_dtype: DataType | None = None
    activation_round_style: RoundStyle = RoundStyle.nearest
    activation_scale_rule: ScaleRule | None = None
    disable_dgrad_quantization: bool = False
    disable_fprop_quantization: bool = False
    disable_wgrad_quantization: bool = False
    dtype: DataType = DataType.nvfp4
    emit_output_amax: bool = True  # (not in the reference) the forward GEMM records max|output| for the next layer's quantize
    gradient_dtype: DataType | None = None
    gradient_round_style: RoundStyle = RoundStyle.stochastic
    gradient_scale_rule: ScaleRule | None = None
    keep_master_weights: bool = False
    matmul_backend: MatmulBackend | None = None
    output_dtype: DataType = DataType.bfloat16
    pseudo_quantize: bool = False
    quantize_backend: QuantizeBackend | None = None
    quartet_ii_dtype: DataType | None = None
    quartet_ii_rerotate_had: bool = False
    scale_rule: ScaleRule = ScaleRule.mse
    weight_dtype: DataType | None = None
    weight_round_style: RoundStyle = RoundStyle.nearest
    weight_scale_2d: bool = False
    weight_scale_rule: ScaleRule | None = None
    wgrad_nvint4: bool = False

    def __post_init__(self) -> None:
        for f in fields(self):
            enum_cls = _ENUMS.get(f.name)
            value = getattr(self, f.name)
            if enum_cls is not None and isinstance(value, str) and not isinstance(value, enum_cls):
                setattr(self, f.name, enum_cls(value))
        for prefix in ("activation", "gradient", "weight"):
            if getattr(self, f"{prefix}_dtype") is None:
                setattr(self, f"{prefix}_dtype", self.dtype)
            if getattr(self, f"{prefix}_scale_rule") is None:
                setattr(self, f"{prefix}_scale_rule", self.scale_rule)

    def _config(self, prefix: str, extra: dict[str, Any], overrides: dict[str, Any]) -> QuantizationConfig:
        return QuantizationConfig(
            **{
                "backend": self.quantize_backend,
                "dtype": getattr(self, f"{prefix}_dtype"),
                "pseudo_quantize": self.pseudo_quantize,
                "round_style": getattr(self, f"{prefix}_round_style"),
                "scale_rule": getattr(self, f"{prefix}_scale_rule"),
                **extra,
                **overrides,
            },
        )

    def get_activation_config(self, **kwargs: Any) -> QuantizationConfig:
        return self._config("activation", {}, kwargs)

    def get_gradient_config(self, **kwargs: Any) -> QuantizationConfig:
        return self._config("gradient", {}, kwargs)

    def get_weight_config(self, **kwargs: Any) -> QuantizationConfig:
        return self._config("weight", {"block_scale_2d": self.weight_scale_2d}, kwargs)


@dataclass
class ModelQuantizationConfig(ModuleQuantizationConfig):
    """Model-wide settings plus per-module overrides and a skip list."""

    module_config_overrides: dict[str, ModuleQuantizationConfig] = field(default_factory=dict)
    modules_to_not_convert: list[str] = field(default_factory=lambda: ["lm_head"])

    def __post_init__(self) -> None:
        super().__post_init__()
        if self.module_config_overrides is not None:
            for name, cfg in list(self.module_config_overrides.items()):
                if isinstance(cfg, dict):
                    self.module_config_overrides[name] = ModuleQuantizationConfig(**cfg)

    def get_module_config(self, module_name: str) -> ModuleQuantizationConfig:
        if self.module_config_overrides is None:
            return self
        return self.module_config_overrides.get(module_name, self)

    def __hash__(self) -> str:
        return hashlib.sha256(json.dumps(self.__dict__, sort_keys=True).encode()).hexdigest()
