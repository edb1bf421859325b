"""``import fouroversix`` for code written against the reference package: the same public
names (reference ``src/fouroversix/__init__.py:22-40``), served by ``fouroversix_amd`` --
the gfx950 implementation of the quantize + FP4-matmul path.  Sub-packages ``quantize``,
``matmul``, ``model`` and ``utils`` resolve to their ``fouroversix_amd`` counterparts."""

import sys as _sys

import fouroversix_amd as _impl
from fouroversix_amd import *  # noqa: F401,F403
from fouroversix_amd import __all__ as _names
from fouroversix_amd import matmul, model, quantize_model, utils  # noqa: F401
from fouroversix_amd import quantize as _quantize_pkg

__all__ = list(_names)
__version__ = _impl.__version__

# `fouroversix.quantize` is both the function (as in the reference) and, for
# `from fouroversix.quantize import QuantizationConfig`, the sub-package
for _name in ("quantize", "matmul", "model", "utils"):
    _sys.modules[f"{__name__}.{_name}"] = _sys.modules[f"fouroversix_amd.{_name}"]
for _name in list(_sys.modules):
    if _name.startswith("fouroversix_amd.") and _name.count(".") >= 2:
        _sys.modules["fouroversix." + _name[len("fouroversix_amd."):]] = _sys.modules[_name]
del _name
