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
    """Where the streaming skinny kernel (rows of x read again from L2 by every wave) beats the
    library's product on MI355X, measured at the 7B decoder's shapes: always up to 4 rows; with
    more rows the rows of x weigh more, and the library wins on the large matrices."""
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


RESIDENT_ROWS = 16       # up to here the rows of x stay in registers
RESIDENT_K = 4096        # inner size one block of the resident kernel covers
_cu_count = {}


def _compute_units(device) -> int:
    key = torch.device(device).index or 0
    if key not in _cu_count:
        _cu_count[key] = torch.cuda.get_device_properties(key).multi_processor_count
    return _cu_count[key]


def try_linear(x: torch.Tensor, weight: torch.Tensor, bias: Optional[torch.Tensor],
               out_dtype: Optional[torch.dtype], allow_slabs: bool = False) -> Optional[torch.Tensor]:
    """``x @ weight.T (+ bias)`` through a skinny kernel, or None if the shape is not one they take
    (too many rows, an inner size that is not a multiple of 8, rows that are not 16-byte aligned).

    Up to 16 rows the resident kernel runs.  An inner size above 4096 makes it write partial sums
    in slabs ``[S, M, N]`` (float32), which the caller must have asked for with ``allow_slabs`` and
    whose consumer adds them up in slab order (the residual add + norm kernel does)."""
    m, k = x.shape
    n = weight.shape[0]
    aligned = (k % 8 == 0 and x.stride(1) == 1 and weight.stride(1) == 1 and x.stride(0) % 8 == 0
               and weight.stride(0) % 8 == 0 and x.data_ptr() % 16 == 0 and weight.data_ptr() % 16 == 0)
    bias_ok = bias is None or (bias.dtype == torch.float32 and bias.is_contiguous() and bias.shape == (n,))
    odt = out_dtype or x.dtype
    slabs = (k + RESIDENT_K - 1) // RESIDENT_K
    if (m <= RESIDENT_ROWS and aligned and bias_ok
            and (slabs == 1 or (allow_slabs and odt == torch.float32))):
        shape = (m, n) if slabs == 1 else (slabs, m, n)
        out = torch.empty(shape, dtype=odt, device=x.device)
        fn = _fn("gemm_skinny", "qvl_gemm_resident",
                 [_c_ptr, _c_int, _c_ptr, _c_int, _c_ptr, _c_ptr, _c_int, ctypes.c_longlong, _c_int, _c_int, _c_int,
                  _c_int, _c_int, _c_ptr])
        _check(fn(_ptr(x), x.stride(0), _ptr(weight), weight.stride(0), _ptr(bias), _ptr(out), n, m * n, m, n, k,
                  dtype_code(odt), _compute_units(x.device), _stream()), "linear (skinny, resident)")
        return out
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
