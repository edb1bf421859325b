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


# ---- random Hadamard transform matrix ------------------------------------------------------

# The fixed sign vector of the reference's wgrad transform (src/fouroversix/quantize/utils.py:19-30).
_RHT_SIGNS = (1, 1, 1, -1, 1, -1, -1, -1, -1, -1, -1, 1, -1, 1, -1, -1)


def get_rht_matrix(*, with_random_sign_mask: bool = True, device: torch.device | str | int = "cuda") -> torch.Tensor:
    """bf16 [16, 16]: ``diag(signs) @ H16 / 4`` with the Sylvester-ordered Hadamard matrix
    ``H16[i, j] = (-1) ** popcount(i & j)`` -- the matrix ``x.reshape(-1, 16) @ M`` applies
    (reference ``get_rht_matrix``, ``src/fouroversix/quantize/utils.py:68-85``; the kernels
    apply the same transform as a butterfly, this is for callers that want the matrix)."""
    idx = torch.arange(16)
    parity = torch.tensor([[bin(int(i) & int(j)).count("1") & 1 for j in idx] for i in idx])
    had = (1.0 - 2.0 * parity.float()) * 0.25
    signs = torch.tensor(_RHT_SIGNS, dtype=torch.float32) if with_random_sign_mask else torch.ones(16)
    return (signs.unsqueeze(1) * had).to(device=device, dtype=torch.bfloat16)
