"""Scale-factor layouts: row-major ``[rows, cols/16]`` and the 128x4-tile layout the FP4
GEMM consumes (reference ``to_blocked`` ``src/fouroversix/quantize/utils.py:88-96`` and
``from_blocked`` ``src/fouroversix/quantize/dequantize_utils.py:4-12``).

Scale (r, c) of an [R, C] grid lives at
``((r // 128) * (C // 4) + c // 4) * 512 + (r % 32) * 16 + ((r % 128) // 32) * 4 + c % 4``.
These helpers are index permutations on whatever device the tensor is on; the kernels
write and read the tiled layout directly.
"""

from __future__ import annotations

import torch


def tiled_offsets(rows: int, cols: int, device: torch.device | str = "cpu") -> torch.Tensor:
    """int64 [rows, cols]: flat offset of every scale in the tiled layout."""
    r = torch.arange(rows, device=device).unsqueeze(1)
    c = torch.arange(cols, device=device).unsqueeze(0)
    return ((r // 128) * (cols // 4) + c // 4) * 512 + (r % 32) * 16 + ((r % 128) // 32) * 4 + c % 4


def to_blocked(a: torch.Tensor) -> torch.Tensor:
    """Row-major [R, C] (R % 128 == 0, C % 4 == 0) -> flat tiled layout."""
    rows, cols = a.shape
    if rows % 128 or cols % 4:
        msg = f"to_blocked needs rows % 128 == 0 and cols % 4 == 0, got {tuple(a.shape)}"
        raise ValueError(msg)
    raw = a.contiguous().view(torch.uint8) if a.element_size() == 1 else a.contiguous()
    out = torch.empty(rows * cols, dtype=raw.dtype, device=a.device)
    out[tiled_offsets(rows, cols, a.device).reshape(-1)] = raw.reshape(-1)
    return out.view(a.dtype) if a.element_size() == 1 else out


def from_blocked(a: torch.Tensor, orig_shape: tuple[int, int]) -> torch.Tensor:
    """Flat tiled layout -> row-major ``orig_shape`` = (rows, cols)."""
    rows, cols = orig_shape
    raw = a.contiguous().view(torch.uint8) if a.element_size() == 1 else a.contiguous()
    out = raw.reshape(-1)[tiled_offsets(rows, cols, a.device)]
    return out.view(a.dtype) if a.element_size() == 1 else out
