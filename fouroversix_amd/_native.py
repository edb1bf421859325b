"""ctypes binding of ``libfouroversix_hip.so`` (the C ABI declared in
``include/fouroversix_hip.h``).

The library is the only implementation: there is no CPU or eager fallback.  Loading
fails loudly when the shared object is missing; build it with
``python fouroversix_amd/build.py``.
"""

from __future__ import annotations

import ctypes
import os

import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libfouroversix_hip.so")

T_BF16, T_F16, T_F32 = 0, 1, 2
SF_LINEAR, SF_TILED = 0, 1
TORCH_TO_T = {torch.bfloat16: T_BF16, torch.float16: T_F16, torch.float32: T_F32}

EXPORTS = (
    "fos_version",
    "fos_error_string",
    "fos_tuning_reload",
    "fos_padded_rows",
    "fos_padded_cols",
    "fos_quantize_workspace_bytes",
    "fos_amax",
    "fos_quantize",
    "fos_quantize_static",
    "fos_quantize_devkey",
    "fos_pseudo_quantize",
    "fos_pseudo_quantize_keyed",
    "fos_pseudo_quantize_is_fused",
    "fos_transform",
    "fos_transform_quantize",
    "fos_gemm_nvfp4",
    "fos_gemm_nvfp4_amax",
    "fos_gemm_nvfp4_amax_out",
    "fos_gemm_nvfp4_linear",
    "fos_gemm_mxfp4",
    "fos_gemm_alpha",
    "fos_padded_cols_for",
    "fos_gemm_workspace_bytes",
    "fos_dequantize",
)

_lib = None


class NativeLibraryError(RuntimeError):
    """The HIP library is missing or a call into it failed."""


def lib() -> ctypes.CDLL:
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        msg = (
            f"{LIB_PATH} not found: the gfx950 library has not been built "
            "(run `python fouroversix_amd/build.py`); there is no fallback path"
        )
        raise NativeLibraryError(msg)
    L = ctypes.CDLL(LIB_PATH)
    c = ctypes
    vp, i64, u64, i32, sz, dbl = c.c_void_p, c.c_int64, c.c_uint64, c.c_int, c.c_size_t, c.c_double
    L.fos_version.argtypes = []
    L.fos_version.restype = i32
    L.fos_error_string.argtypes = [i32]
    L.fos_error_string.restype = c.c_char_p
    L.fos_tuning_reload.argtypes = []
    L.fos_tuning_reload.restype = None
    L.fos_padded_rows.argtypes = [i64]
    L.fos_padded_rows.restype = i64
    L.fos_padded_cols.argtypes = [i64]
    L.fos_padded_cols.restype = i64
    L.fos_quantize_workspace_bytes.argtypes = [i64, i64]
    L.fos_quantize_workspace_bytes.restype = sz
    L.fos_amax.argtypes = [vp, i32, i64, i64, i64, vp, vp, sz, vp]
    L.fos_amax.restype = i32
    L.fos_quantize.argtypes = [vp, i32, i64, i64, i64, i32, i32, i32, i32, u64, u64, i32,
                               vp, vp, vp, i32, vp, sz, vp]
    L.fos_quantize.restype = i32
    L.fos_quantize_static.argtypes = [vp, i32, i64, i64, i64, i32, i32, i32, i32, u64, u64, i32, vp, vp, vp, i32, vp]
    L.fos_quantize_static.restype = i32
    L.fos_quantize_devkey.argtypes = [vp, i32, i64, i64, i64, i32, i32, i32, i32, vp, i32, vp, vp, vp, i32, vp, sz, vp]
    L.fos_quantize_devkey.restype = i32
    L.fos_pseudo_quantize.argtypes = [vp, i32, i64, i64, i64, i32, i32, i32, i32, vp, i64, vp, i32, vp, sz, vp]
    L.fos_pseudo_quantize.restype = i32
    L.fos_pseudo_quantize_keyed.argtypes = [vp, i32, i64, i64, i64, i32, i32, i32, i32, u64, u64, vp, i64, vp, i32, vp, sz, vp]
    L.fos_pseudo_quantize_keyed.restype = i32
    L.fos_pseudo_quantize_is_fused.argtypes = [i32, i32, i32, i32, i32]
    L.fos_pseudo_quantize_is_fused.restype = i32
    L.fos_transform.argtypes = [vp, i32, i64, i64, i64, i32, i32, vp, i64, vp, vp, sz, vp]
    L.fos_transform.restype = i32
    L.fos_transform_quantize.argtypes = [vp, i32, i64, i64, i64, i32, i32, vp, i64, i32, i32, i32, i32, u64, u64, i32, vp, vp, vp, vp, sz, vp]
    L.fos_transform_quantize.restype = i32
    L.fos_gemm_nvfp4.argtypes = [vp, vp, vp, vp, vp, i64, i64, i64, vp, i32, i64, vp, ctypes.c_size_t, vp]
    L.fos_gemm_nvfp4.restype = i32
    L.fos_gemm_nvfp4_amax.argtypes = [vp, vp, vp, vp, vp, vp, dbl, i64, i64, i64, vp, i32, i64, vp, ctypes.c_size_t, vp]
    L.fos_gemm_nvfp4_amax.restype = i32
    L.fos_gemm_nvfp4_amax_out.argtypes = [vp, vp, vp, vp, vp, vp, dbl, i64, i64, i64, vp, i32, i64, vp, vp, ctypes.c_size_t, vp]
    L.fos_gemm_nvfp4_amax_out.restype = i32
    L.fos_gemm_nvfp4_linear.argtypes = [vp, vp, vp, vp, vp, vp, dbl, i64, i64, i64, vp, i32, i64, vp, vp, vp, ctypes.c_size_t, vp]
    L.fos_gemm_nvfp4_linear.restype = i32
    L.fos_gemm_alpha.argtypes = [vp, vp, dbl, vp, vp]
    L.fos_gemm_alpha.restype = i32
    L.fos_gemm_mxfp4.argtypes = [vp, vp, vp, vp, vp, i64, i64, i64, vp, i32, i64, vp]
    L.fos_gemm_mxfp4.restype = i32
    L.fos_padded_cols_for.argtypes = [i32, i64]
    L.fos_padded_cols_for.restype = i64
    L.fos_gemm_workspace_bytes.argtypes = [i64, i64, i64]
    L.fos_gemm_workspace_bytes.restype = ctypes.c_size_t
    L.fos_dequantize.argtypes = [vp, vp, vp, i32, i32, dbl, i64, i64, i64, i64, vp, i32, i64, i32, vp]
    L.fos_dequantize.restype = i32
    _lib = L
    return L


def check(code: int, what: str) -> None:
    if code != 0:
        text = lib().fos_error_string(code).decode()
        raise RuntimeError(f"{what}: {text} (code {code})")


def current_stream(device: torch.device) -> int:
    """Handle of torch's current stream on ``device`` (the raw query: building a
    ``torch.cuda.Stream`` object for it costs several microseconds per call)."""
    index = device.index
    return torch._C._cuda_getCurrentRawStream(torch.cuda.current_device() if index is None else index)


def require_gpu_tensor(t: torch.Tensor, name: str) -> None:
    if t.device.type != "cuda":
        msg = f"{name} must live on the GPU (got {t.device}); this library has no CPU path"
        raise ValueError(msg)
