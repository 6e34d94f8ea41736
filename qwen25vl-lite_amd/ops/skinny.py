"""Dispatch of bfloat16 products with few rows to the hand-written kernels.

Up to 32 rows: the resident kernel (``csrc/gemm_resident.hip``), which can also fold the RMSNorm
before the product, the residual add after it, or the SwiGLU activation into itself; with 17 to 32
rows it needs an inner size that fits one pass of a block.
17 to 32 rows beyond that: the streaming kernel (``csrc/gemm_skinny.hip``) where it beats the library.
"""

from __future__ import annotations

import ctypes
from typing import Optional

import torch

from .kernels import _check, _fn, _ptr, _stream, dtype_code

__all__ = ["resident_product", "takes_resident", "qkv_rope_product", "takes_qkv_rope", "try_streaming", "RESIDENT_ROWS", "resident_norm_k", "resident_two_tile_k", "folds_norm", "MAX_ROWS",
           "STORE", "RESIDUAL", "SWIGLU"]

MAX_ROWS = 32            # the streaming kernel's limit in use
RESIDENT_ROWS = 32       # up to here the resident kernel runs (one column tile of 16 rows, or two)
_pass_k = None
_two_tile_k = None
STORE, RESIDUAL, SWIGLU = 0, 1, 2
_c_int, _c_float, _c_ptr = ctypes.c_int, ctypes.c_float, ctypes.c_void_p
_cu_count = {}


def _compute_units(device) -> int:
    key = torch.device(device).index or 0
    if key not in _cu_count:
        _cu_count[key] = torch.cuda.get_device_properties(key).multi_processor_count
    return _cu_count[key]


def _rows_aligned(t: torch.Tensor, elems: int) -> bool:
    return t.stride(1) == 1 and t.stride(0) % elems == 0 and t.data_ptr() % 16 == 0


def resident_norm_k() -> int:
    """The longest row whose norm the resident kernel folds in: the whole row must fit one pass of
    the block (the kernel's own constant)."""
    global _pass_k
    if _pass_k is None:
        _pass_k = int(_fn("gemm_resident", "qvl_gemm_resident_pass_k", [])())
    return _pass_k


def resident_two_tile_k() -> int:
    """The longest inner size with which the resident kernel takes 17 to 32 rows (their second
    half waits in LDS; the kernel's own constant)."""
    global _two_tile_k
    if _two_tile_k is None:
        _two_tile_k = int(_fn("gemm_resident", "qvl_gemm_resident_two_tile_k", [])())
    return _two_tile_k


def folds_norm(m: int, k: int) -> bool:
    """Whether the resident kernel forms the norm of ``m`` rows of width ``k`` by itself."""
    return m <= RESIDENT_ROWS and k <= (resident_norm_k() if m <= 16 else resident_two_tile_k())


def takes_resident(m: int, k: int, weight: torch.Tensor, *, norm: bool = False) -> bool:
    """Whether the resident kernel takes a product of ``m`` rows with this weight, and is the
    better choice for it.  A K that fits one pass of the block always is (the rows stay in
    registers for all of the block's tiles).  With a longer K the rows are read again for every
    pass of every tile, which only pays while each compute unit has a single tile (at most
    16 weight rows each): beyond that the library's product streams such a matrix faster
    (measured at the 72B decoder's shapes, K of 8192 and 29568)."""
    if m > RESIDENT_ROWS or k % 8 or weight.dtype != torch.bfloat16 or not _rows_aligned(weight, 8):
        return False
    if k <= (resident_norm_k() if m <= 16 else resident_two_tile_k()):
        return True
    return not norm and weight.shape[0] <= 16 * _compute_units(weight.device)


def resident_product(weight: torch.Tensor, *, x: Optional[torch.Tensor] = None, h: Optional[torch.Tensor] = None,
                     norm_weight: Optional[torch.Tensor] = None, eps: float = 0.0,
                     bias: Optional[torch.Tensor] = None, epilogue: int = STORE,
                     out: Optional[torch.Tensor] = None, out_dtype: torch.dtype = torch.float32) -> torch.Tensor:
    """``X @ weight.T`` for at most 32 rows.  ``X`` is ``x`` (bfloat16), or ``rmsnorm(h) * norm_weight``
    formed inside the kernel from the float32 rows ``h``.  ``epilogue``: ``STORE`` writes the product
    (plus ``bias``) to a new tensor of ``out_dtype``; ``RESIDUAL`` adds it to ``out`` (float32) in
    place; ``SWIGLU`` takes ``weight``'s rows as groups of 8 gate, 8 up rows and returns
    ``silu(gate) * up`` as bfloat16 ``[M, N/2]``."""
    src = x if x is not None else h
    m, k = src.shape
    n = weight.shape[0]
    if not takes_resident(m, k, weight, norm=h is not None) or weight.shape[1] != k:
        raise ValueError("the resident kernel does not take this product")
    if x is not None and (x.dtype != torch.bfloat16 or not _rows_aligned(x, 8)):
        raise ValueError("x must be bfloat16 with 16-byte aligned rows")
    if h is not None and (h.dtype != torch.float32 or not _rows_aligned(h, 4) or norm_weight is None
                          or norm_weight.dtype != torch.float32 or norm_weight.shape != (k,)):
        raise ValueError("h must be float32 rows with a float32 norm weight of their width")
    if bias is not None and (bias.dtype != torch.float32 or not bias.is_contiguous() or bias.shape != (n,)):
        raise ValueError("bias must be float32 [N]")
    if epilogue == RESIDUAL:
        if out is None or out.dtype != torch.float32 or out.shape != (m, n) or out.stride(1) != 1:
            raise ValueError("the residual must be float32 [M, N]")
        odt = torch.float32
    elif epilogue == SWIGLU:
        if n % 16:
            raise ValueError("gate | up rows must come in groups of 8 + 8")
        out, odt = torch.empty((m, n // 2), dtype=torch.bfloat16, device=src.device), torch.bfloat16
    else:
        out, odt = torch.empty((m, n), dtype=out_dtype, device=src.device), out_dtype
    fn = _fn("gemm_resident", "qvl_gemm_resident",
             [_c_ptr, _c_int, _c_ptr, _c_int, _c_ptr, _c_float, _c_ptr, _c_int, _c_ptr, _c_ptr, _c_int, _c_int, _c_int,
              _c_int, _c_int, _c_int, _c_int, _c_ptr])
    _check(fn(_ptr(x), x.stride(0) if x is not None else 0, _ptr(h), h.stride(0) if h is not None else 0,
              _ptr(norm_weight), float(eps), _ptr(weight), weight.stride(0), _ptr(bias), _ptr(out), out.stride(0),
              m, n, k, dtype_code(odt), epilogue, _compute_units(src.device), _stream()), "linear (resident)")
    return out


def takes_qkv_rope(m: int, k: int, weight: torch.Tensor, head_dim: int, rot_half: int, cache_dtype, *,
                   norm: bool = False) -> bool:
    """Whether the resident kernel can rotate and store the stacked projection by itself: bfloat16,
    a head size in steps of 16 and a rotation over the whole head."""
    return (takes_resident(m, k, weight, norm=norm) and head_dim % 16 == 0 and 2 * rot_half == head_dim
            and cache_dtype in (None, torch.bfloat16))


def qkv_rope_product(weight: torch.Tensor, cs: torch.Tensor, *, x: Optional[torch.Tensor] = None,
                     h: Optional[torch.Tensor] = None, norm_weight: Optional[torch.Tensor] = None, eps: float = 0.0,
                     bias: Optional[torch.Tensor] = None, slots: Optional[torch.Tensor] = None,
                     k_cache: Optional[torch.Tensor] = None, v_cache: Optional[torch.Tensor] = None,
                     num_q_heads: int, num_kv_heads: int, head_dim: int, page_size: int) -> torch.Tensor:
    """The stacked query | key | value projection of at most 32 tokens with the rotation and the
    cache write inside the product's kernel: returns the rotated queries ``[M, nq hd]`` (bfloat16);
    rotated keys and values are in their page slots.  ``cs`` is :func:`kernels.rope_table` of the
    step's tokens.  With ``num_kv_heads == 0`` the weight holds query rows only."""
    src = x if x is not None else h
    m, k = src.shape
    nq, nkv, hd = int(num_q_heads), int(num_kv_heads), int(head_dim)
    if weight.shape != ((nq + 2 * nkv) * hd, k) or not takes_qkv_rope(m, k, weight, hd, cs.shape[1], None,
                                                                        norm=h is not None):
        raise ValueError("the resident kernel does not take this projection")
    if x is not None and (x.dtype != torch.bfloat16 or not _rows_aligned(x, 8)):
        raise ValueError("x must be bfloat16 with 16-byte aligned rows")
    if h is not None and (h.dtype != torch.float32 or not _rows_aligned(h, 4) or norm_weight is None
                          or norm_weight.dtype != torch.float32 or norm_weight.shape != (k,)):
        raise ValueError("h must be float32 rows with a float32 norm weight of their width")
    if bias is not None and (bias.dtype != torch.float32 or not bias.is_contiguous() or bias.shape != (weight.shape[0],)):
        raise ValueError("bias must be float32 [(nq + 2 nkv) hd]")
    if cs.dtype != torch.float32 or cs.shape != (m, hd // 2, 2) or not cs.is_contiguous():
        raise ValueError("cs must be float32 [M, hd/2, 2]")
    if nkv:
        if (slots is None or slots.dtype != torch.int32 or slots.shape != (m,) or not slots.is_contiguous()
                or k_cache is None or v_cache is None or k_cache.dtype != torch.bfloat16
                or v_cache.dtype != torch.bfloat16 or not k_cache.is_contiguous() or not v_cache.is_contiguous()
                or tuple(k_cache.shape[1:]) != (nkv, page_size, hd) or tuple(v_cache.shape[1:]) != (nkv, hd, page_size)
                or v_cache.shape[0] != k_cache.shape[0]):
            raise ValueError("slots int32 [M] and bfloat16 caches [pages, nkv, ps, hd] / [pages, nkv, hd, ps] are needed")
    q_out = torch.empty((m, nq * hd), dtype=torch.bfloat16, device=src.device)
    fn = _fn("gemm_resident", "qvl_gemm_resident_rope",
             [_c_ptr, _c_int, _c_ptr, _c_int, _c_ptr, _c_float, _c_ptr, _c_int, _c_ptr, _c_int, _c_int, _c_ptr, _c_ptr,
              _c_ptr, _c_ptr, _c_ptr, _c_int, _c_int, _c_int, _c_int, _c_int, _c_ptr])
    _check(fn(_ptr(x), x.stride(0) if x is not None else 0, _ptr(h), h.stride(0) if h is not None else 0,
              _ptr(norm_weight), float(eps), _ptr(weight), weight.stride(0), _ptr(bias), m, k, _ptr(cs),
              _ptr(slots if nkv else None), _ptr(q_out), _ptr(k_cache if nkv else None),
              _ptr(v_cache if nkv else None), nq, nkv, hd, int(page_size), _compute_units(src.device), _stream()),
           "linear (resident, rotation and cache write)")
    return q_out


def prefers_streaming(m: int, n: int, k: int) -> bool:
    """Where the streaming kernel (rows of x read again from L2 by every wave) beats the library's
    product on MI355X, measured at the 7B decoder's shapes with 17 to 32 rows: the small square
    matrix and the one with a long inner size."""
    return 16 < m <= MAX_ROWS and (n * k <= 13_000_000 or k >= 4 * n)


def try_streaming(x: torch.Tensor, weight: torch.Tensor, bias: Optional[torch.Tensor],
                  out_dtype: Optional[torch.dtype]) -> Optional[torch.Tensor]:
    """``x @ weight.T (+ bias)`` through the streaming kernel, or None if it is not the better choice
    or does not take the shape."""
    m, k = x.shape
    n = weight.shape[0]
    if not prefers_streaming(m, n, k) or k % 8 or not _rows_aligned(x, 8) or not _rows_aligned(weight, 8):
        return None
    if bias is not None and (bias.dtype != torch.float32 or not bias.is_contiguous() or bias.shape != (n,)):
        return None
    odt = out_dtype or x.dtype
    out = torch.empty((m, n), dtype=odt, device=x.device)
    fn = _fn("gemm_skinny", "qvl_gemm_skinny",
             [_c_ptr, _c_int, _c_ptr, _c_int, _c_ptr, _c_ptr, _c_int, _c_int, _c_int, _c_int, _c_int, _c_ptr])
    _check(fn(_ptr(x), x.stride(0), _ptr(weight), weight.stride(0), _ptr(bias), _ptr(out), out.stride(0), m, n, k,
              dtype_code(odt), _stream()), "linear (streaming)")
    return out
