"""``quantize_model`` and the high-precision -> quantized module registry
(reference ``src/fouroversix/model/quantize.py:13-127``)."""

from __future__ import annotations

from typing import TYPE_CHECKING, Any, ClassVar

import torch.nn as nn

if TYPE_CHECKING:
    from collections.abc import Callable

from .config import ModelQuantizationConfig


class QuantizedModule:
    """Registry mapping a high-precision module class to its quantized replacement."""

    _registry: ClassVar[dict[type[nn.Module], type[nn.Module]]] = {}
    _should_replace_existing_modules_in_model: ClassVar[dict[type[nn.Module], bool]] = {}

    @classmethod
    def is_quantized_module_type(cls, module_type: type[nn.Module]) -> bool:
        return module_type in cls._registry.values()

    @classmethod
    def get_cls(cls, high_precision_cls: type[nn.Module]) -> type[nn.Module] | None:
        return cls._registry.get(high_precision_cls)

    @classmethod
    def should_replace_existing_modules_in_model(cls, module_type: type[nn.Module]) -> bool:
        return cls._should_replace_existing_modules_in_model.get(module_type, False)

    @classmethod
    def register(
        cls,
        high_precision_cls: type[nn.Module],
        *,
        replace_existing_modules_in_registry: bool = False,
        replace_existing_modules_in_model: bool = True,
    ) -> Callable[[type[nn.Module]], type[nn.Module]]:
        """Class decorator registering ``wrapped_cls`` as the replacement of
        ``high_precision_cls``.  Registering a class (or a subclass of a registered
        class) twice is an error unless ``replace_existing_modules_in_registry``."""
        if high_precision_cls in cls._registry and not replace_existing_modules_in_registry:
            msg = f"High-precision module {high_precision_cls} is already registered."
            raise ValueError(msg)

        shadowed = [
            known
            for known in cls._registry
            if high_precision_cls is not None and issubclass(high_precision_cls, known)
        ]
        if shadowed and not replace_existing_modules_in_registry:
            msg = (
                f"High-precision module {high_precision_cls} is a subclass of "
                f"{shadowed[0]}, which is already registered."
            )
            raise TypeError(msg)
        for known in shadowed:
            del cls._registry[known]

        def wrap(wrapped_cls: type[nn.Module]) -> type[nn.Module]:
            cls._registry[high_precision_cls] = wrapped_cls
            cls._should_replace_existing_modules_in_model[high_precision_cls] = replace_existing_modules_in_model
            return wrapped_cls

        return wrap


def quantize_model(
    model: nn.Module,
    config: ModelQuantizationConfig | None = None,
    **kwargs: Any,
) -> None:
    """Replace, in place, every registered module of ``model`` (except the skip list)
    by its quantized counterpart.  ``kwargs`` go to the replacement's constructor."""
    if config is None:
        config = ModelQuantizationConfig()
    for name, module in list(model.named_modules()):
        if name == "" or name in config.modules_to_not_convert or not isinstance(module, nn.Module):
            continue
        replacement = QuantizedModule.get_cls(type(module))
        if replacement is None or not QuantizedModule.should_replace_existing_modules_in_model(type(module)):
            continue
        model.set_submodule(name, replacement(module, config.get_module_config(name), **kwargs))
