"""Dispatch of bfloat16 products with few rows to the hand-written skinny kernel."""

from __future__ import annotations

import ctypes
from typing import Optional

import torch

from .kernels import _check, _fn, _ptr, _stream, dtype_code

__all__ = ["try_linear", "MAX_ROWS"]

MAX_ROWS = 64
_c_int, _c_ptr = ctypes.c_int, ctypes.c_void_p


def prefers_skinny(m: int, n: int, k: int) -> bool:
    """Where the skinny kernel beats the library's product on MI355X (measured at the 7B decoder's
    shapes): always up to 4 rows; with more rows the rows of x, which every wave reads again from
    L2, weigh more, and the library wins on the large matrices."""
    size = n * k
    if m <= 4:
        return True
    if m <= 8:
        return size <= 72_000_000
    if m <= 16:
        return size <= 20_000_000
    if m <= 32:
        return size <= 13_000_000 or k >= 4 * n
    return False


def try_linear(x: torch.Tensor, weight: torch.Tensor, bias: Optional[torch.Tensor],
               out_dtype: Optional[torch.dtype]) -> Optional[torch.Tensor]:
    """``x @ weight.T (+ bias)`` through the skinny kernel, or None if the shape is not one it takes
    (more than 64 rows, an inner size that is not a multiple of 8, rows that are not 16-byte aligned)."""
    m, k = x.shape
    n = weight.shape[0]
    if not prefers_skinny(m, n, k):
        return None
    if m > MAX_ROWS or k % 8 or x.stride(1) != 1 or weight.stride(1) != 1 or x.stride(0) % 8 or weight.stride(0) % 8:
        return None
    if x.data_ptr() % 16 or weight.data_ptr() % 16:
        return None
    if bias is not None and (bias.dtype != torch.float32 or not bias.is_contiguous() or bias.shape != (n,)):
        return None
    odt = out_dtype or x.dtype
    out = torch.empty((m, n), dtype=odt, device=x.device)
    fn = _fn("gemm_skinny", "qvl_gemm_skinny",
             [_c_ptr, _c_int, _c_ptr, _c_int, _c_ptr, _c_ptr, _c_int, _c_int, _c_int, _c_int, _c_int, _c_ptr])
    _check(fn(_ptr(x), x.stride(0), _ptr(weight), weight.stride(0), _ptr(bias), _ptr(out), out.stride(0), m, n, k,
              dtype_code(odt), _stream()), "linear (skinny)")
    return out
