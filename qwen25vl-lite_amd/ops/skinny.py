"""Dispatch of bfloat16 products with few rows to the hand-written kernels.

Up to 64 rows: the resident kernel (``csrc/gemm_resident.hip``), which can also fold the RMSNorm
before the product, the residual add after it, the SwiGLU activation, or the rotation and cache
write into itself.  One block carries up to 32 rows; more rows (or 17 to 32 with a long inner
size) are spread over teams of blocks that walk the same weight tiles on one XCD.
"""

from __future__ import annotations

import ctypes
from typing import Optional

import torch

from .kernels import _check, _fn, _ptr, _stream, dtype_code

__all__ = ["resident_product", "takes_resident", "qkv_rope_product", "takes_qkv_rope", "RESIDENT_ROWS", "resident_norm_k", "resident_two_tile_k", "folds_norm", "ONE_BLOCK_ROWS", "split_product", "takes_split", "prefers_split", "SPLIT_ROWS",
           "STORE", "RESIDUAL", "SWIGLU"]

RESIDENT_ROWS = 64       # up to here the resident kernel runs
ONE_TILE_ROWS = 16       # the rows of one column tile of the matrix instruction
ONE_BLOCK_ROWS = 32      # up to here one block carries all rows: beyond, teams of blocks share the weight's
                         # tiles, which pays for the fused q | k | v projection only
_MAX_WEIGHT_BYTES = 0xffffff00   # qvl_gemm_resident_max_weight_bytes() + 1
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


NARROW_K = 2048   # up to this inner size the resident kernel's build with 128 columns a wave runs


def _build_for(k: int):
    """The build of the resident kernel for an inner size: with 256 columns a wave, half of a
    block's 16 waves have no columns of an inner size of 2,048 and the other half carry all loads
    (the 3B decoder's gate | up product: 24.4 us against 17.7 with 128 columns a wave)."""
    return {"RK": 4} if k <= NARROW_K else None


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


def folds_norm(m: int, k: int, device=None) -> bool:
    """Whether the resident kernel forms the norm of ``m`` rows of width ``k`` by itself (the
    kernel's own rule: the rows must stay in their blocks for all of the weight's tiles)."""
    if m > RESIDENT_ROWS or k % 8:
        return False
    fn = _fn("gemm_resident", "qvl_gemm_resident_folds_norm", [_c_int, _c_int, _c_int], _build_for(k))
    return bool(fn(int(m), int(k), _compute_units(device if device is not None else torch.cuda.current_device())))


def takes_resident(m: int, k: int, weight: torch.Tensor, *, norm: bool = False) -> bool:
    """Whether the resident kernel takes a product of ``m`` rows with this weight, and is the
    better choice for it.  A K that fits one pass of the block always is (the rows stay in
    registers for all of the block's tiles; with 33 to 64 rows in those of a team of blocks).  Up to 32 rows with a longer K are read again for every pass of every tile,
    which only pays while each compute unit has a single tile (at most 16 weight rows each):
    beyond that the library's product streams such a matrix faster (measured at the 72B
    decoder's shapes, K of 8192 and 29568)."""
    if m > RESIDENT_ROWS or k % 8 or weight.dtype != torch.bfloat16 or not _rows_aligned(weight, 8):
        return False
    if ((weight.shape[0] - 1) * weight.stride(0) + k) * 2 >= _MAX_WEIGHT_BYTES:
        return False     # the kernel reaches its operands through 32-bit byte offsets
    if norm:
        return folds_norm(m, k, weight.device)
    if k <= NARROW_K:
        return True      # one pass in either build, with any number of rows (and no question to the other build)
    if m > 32:
        return k <= resident_norm_k()    # teams keep their rows for one pass; in several passes they lose to the library
    if k <= (resident_norm_k() if m <= 16 else resident_two_tile_k()):
        return True
    return weight.shape[0] <= 16 * _compute_units(weight.device)


def resident_product(weight: torch.Tensor, *, x: Optional[torch.Tensor] = None, h: Optional[torch.Tensor] = None,
                     norm_weight: Optional[torch.Tensor] = None, eps: float = 0.0,
                     bias: Optional[torch.Tensor] = None, epilogue: int = STORE,
                     out: Optional[torch.Tensor] = None, out_dtype: torch.dtype = torch.float32) -> torch.Tensor:
    """``X @ weight.T`` for at most 64 rows (``h`` for at most 32).  ``X`` is ``x`` (bfloat16), or ``rmsnorm(h) * norm_weight``
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
              _c_int, _c_int, _c_int, _c_int, _c_ptr], _build_for(k))
    _check(fn(_ptr(x), x.stride(0) if x is not None else 0, _ptr(h), h.stride(0) if h is not None else 0,
              _ptr(norm_weight), float(eps), _ptr(weight), weight.stride(0), _ptr(bias), _ptr(out), out.stride(0),
              m, n, k, dtype_code(odt), epilogue, _compute_units(src.device), _stream()),
           "linear (resident)")
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
    """The stacked query | key | value projection of at most 64 tokens with the rotation and the
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
              _c_ptr, _c_ptr, _c_ptr, _c_int, _c_int, _c_int, _c_int, _c_int, _c_ptr], _build_for(k))
    _check(fn(_ptr(x), x.stride(0) if x is not None else 0, _ptr(h), h.stride(0) if h is not None else 0,
              _ptr(norm_weight), float(eps), _ptr(weight), weight.stride(0), _ptr(bias), m, k, _ptr(cs),
              _ptr(slots if nkv else None), _ptr(q_out), _ptr(k_cache if nkv else None),
              _ptr(v_cache if nkv else None), nq, nkv, hd, int(page_size), _compute_units(src.device), _stream()),
           "linear (resident, rotation and cache write)")
    return q_out


SPLIT_ROWS = 64   # the most rows the split kernel is built for


def takes_split(m: int, k: int, weight: torch.Tensor) -> bool:
    """Whether the split kernel (``csrc/gemm_split.hip``) takes a product of ``m`` rows with this
    weight: up to 64 bfloat16 rows, whose partial sums over chunks of the inner size come back as
    slabs."""
    if not (1 <= m <= SPLIT_ROWS and k % 8 == 0 and weight.dtype == torch.bfloat16 and _rows_aligned(weight, 8)):
        return False
    n = weight.shape[0]
    if ((n - 1) * weight.stride(0) + k) * 2 >= _MAX_WEIGHT_BYTES:
        return False
    cus = _compute_units(weight.device)
    return int(_fn("gemm_split", "qvl_gemm_split_chunks", [_c_int, _c_int, _c_int, _c_int])(m, n, k, cus)) > 0


def prefers_split(m: int, k: int, weight: torch.Tensor) -> bool:
    """Where the split kernel is the fastest way to a product that is added to the residual
    (measured on MI355X at the 3B, 7B and 72B decoders' output and down projections): up to 16 rows
    when the inner size is too long for a block of the resident kernel to keep its rows for one
    pass over the weight (the down projection at 8 rows: 26.9 us against 37.3, which pays for the
    norm kernel that then adds the slabs, 5.7 us, where the resident kernel adds in place and the
    next product forms the norm itself); with more rows always (the output projection at 32 rows:
    9.9 us and a norm kernel of 6 against 14.3 in place and 8 more for the norm inside the gate | up
    product; at 64 rows 14.4 us against the library's 13.9 to 17.6, the down projection 36.2
    against 46.6)."""
    if not takes_split(m, k, weight):
        return False
    return m > ONE_TILE_ROWS or (k > NARROW_K and k > resident_norm_k())


def split_product(weight: torch.Tensor, x: torch.Tensor) -> torch.Tensor:
    """Partial sums of ``x @ weight.T`` over chunks of the inner size: float32 ``[chunks, M, N]``,
    whose sum over the first axis (taken in order by whoever reads them: the norm that follows) is
    the product.  ``x`` is bfloat16 ``[M, K]``."""
    m = x.shape[0]
    n, k = weight.shape
    if not takes_split(m, k, weight) or x.shape[1] != k:
        raise ValueError("the split kernel does not take this product")
    if x.dtype != torch.bfloat16 or not _rows_aligned(x, 8):
        raise ValueError("x must be bfloat16 with 16-byte aligned rows")
    cus = _compute_units(x.device)
    chunks = int(_fn("gemm_split", "qvl_gemm_split_chunks", [_c_int, _c_int, _c_int, _c_int])(m, n, k, cus))
    out = torch.empty((chunks, m, n), dtype=torch.float32, device=x.device)
    fn = _fn("gemm_split", "qvl_gemm_split",
             [_c_ptr, _c_int, _c_ptr, _c_int, _c_ptr, _c_int, _c_int, _c_int, _c_int, _c_ptr])
    _check(fn(_ptr(x), x.stride(0), _ptr(weight), weight.stride(0), _ptr(out), m, n, k, cus, _stream()),
           "linear (split)")
    return out
