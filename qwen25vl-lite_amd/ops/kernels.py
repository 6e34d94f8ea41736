"""Python entry points of the HIP kernels.

Every function takes device tensors, checks on the host that their shapes, dtypes and
layouts are what the kernel and its grid assume, and launches on the current HIP stream.
There is no CPU path and no library stand-in: a tensor that is not on the GPU is refused.
"""

from __future__ import annotations

import ctypes
from typing import Dict, Optional, Sequence, Tuple

import torch

from .library import load_library

__all__ = ["rope_table", "copy_pages", 
    "KernelError", "embed_gather", "add_rmsnorm", "rope_kv_write", "paged_attention_generic", "swiglu",
    "gemm_f32", "dtype_code",
]

_c_int, _c_float, _c_ptr = ctypes.c_int, ctypes.c_float, ctypes.c_void_p

_ERRORS = {1: "shape", 2: "dtype", 3: "launch", 4: "size limit"}


class KernelError(RuntimeError):
    """A kernel refused its arguments or failed to launch."""


_functions: Dict[Tuple[str, str, Tuple], ctypes._CFuncPtr] = {}


def _fn(stem: str, name: str, argtypes, defines=None):
    key = (stem, name, tuple(sorted((defines or {}).items())))
    fn = _functions.get(key)
    if fn is None:
        fn = getattr(load_library(stem, defines), name)
        fn.argtypes = list(argtypes)
        fn.restype = _c_int
        _functions[key] = fn
    return fn


def _check(code: int, what: str) -> None:
    if code:
        raise KernelError(f"{what}: the kernel refused its arguments ({_ERRORS.get(code, code)})")


def dtype_code(dtype: torch.dtype) -> int:
    if dtype == torch.float32:
        return 0
    if dtype == torch.bfloat16:
        return 1
    raise KernelError(f"dtype {dtype} is not built (float32 and bfloat16 are)")


def _dev(*tensors: Optional[torch.Tensor]) -> None:
    for t in tensors:
        if t is not None and not t.is_cuda:
            raise KernelError("this operation has no CPU path: its tensors must be on the GPU")


def _ptr(t: Optional[torch.Tensor]):
    return None if t is None else t.data_ptr()


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)


def _stream():
    """The current HIP stream's handle (the short way where this PyTorch has it: the call is made
    once per kernel launch)."""
    if _raw_stream is not None:
        return _raw_stream(torch.cuda.current_device())
    return torch.cuda.current_stream().cuda_stream


def _need(cond: bool, msg: str) -> None:
    if not cond:
        raise KernelError(msg)


# --------------------------------------------------------------------------------------------
def embed_gather(ids: torch.Tensor, table: torch.Tensor, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """``out[n] = float32(table[ids[n]])`` — the residual stream starts in float32."""
    _dev(ids, table, out)
    _need(ids.dtype == torch.int32 and ids.dim() == 1 and ids.is_contiguous(), "ids must be contiguous int32 [N]")
    _need(table.dim() == 2 and table.is_contiguous(), "table must be contiguous [V, H]")
    n, (v, h) = ids.shape[0], table.shape
    if out is None:
        out = torch.empty((n, h), dtype=torch.float32, device=table.device)
    _need(out.dtype == torch.float32 and out.shape == (n, h) and out.is_contiguous(), "out must be float32 [N, H]")
    fn = _fn("elementwise", "qvl_embed_gather", [_c_ptr, _c_ptr, _c_ptr, _c_int, _c_int, _c_int, _c_int, _c_ptr])
    _check(fn(_ptr(ids), _ptr(table), _ptr(out), n, h, v, dtype_code(table.dtype), _stream()), "embed_gather")
    return out


def add_rmsnorm(h: torch.Tensor, delta: Optional[torch.Tensor], weight: torch.Tensor, eps: float,
                out_dtype: torch.dtype, rows: Optional[torch.Tensor] = None,
                out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """``h += delta`` (float32 sum) and return ``rmsnorm(h) * weight`` in ``out_dtype``.

    With ``rows`` (int32 row indices) only those rows are normalised and ``h`` is not written.
    ``delta`` may be float32 ``[slabs, N, H]``: partial sums of a product that was cut along its
    inner size, added in slab order.
    """
    _dev(h, delta, weight, rows, out)
    _need(h.dtype == torch.float32 and h.dim() == 2 and h.is_contiguous(), "h must be contiguous float32 [N, H]")
    n, width = h.shape
    _need(weight.dtype == torch.float32 and weight.shape == (width,) and weight.is_contiguous(),
          "norm weight must be float32 [H]")
    nslabs, slab_stride = 1, 0
    if delta is not None and delta.dim() == 3:
        _need(delta.dtype == torch.float32 and tuple(delta.shape[1:]) == tuple(h.shape) and delta.is_contiguous()
              and width % 4 == 0, "slabs of delta must be contiguous float32 [slabs, N, H] with H in steps of 4")
        nslabs, slab_stride = delta.shape[0], n * width
    elif delta is not None:
        _need(delta.shape == h.shape and delta.is_contiguous(), "delta must match h's shape")
    m = n
    if rows is not None:
        _need(rows.dtype == torch.int32 and rows.dim() == 1 and rows.is_contiguous(), "rows must be int32 [M]")
        m = rows.shape[0]
    if out is None:
        out = torch.empty((m, width), dtype=out_dtype, device=h.device)
    _need(out.shape == (m, width) and out.dtype == out_dtype and out.is_contiguous(), "out must be [M, H]")
    fn = _fn("elementwise", "qvl_add_rmsnorm",
             [_c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_int, _c_int, _c_float, _c_int, _c_int, _c_int,
              ctypes.c_longlong, _c_ptr])
    _check(fn(_ptr(h), _ptr(delta), _ptr(weight), _ptr(out), _ptr(rows), m, width, float(eps),
              dtype_code(delta.dtype if delta is not None else out_dtype), dtype_code(out_dtype), nslabs, slab_stride,
              _stream()), "add_rmsnorm")
    return out


def rope_kv_write(x: torch.Tensor, bias: Optional[torch.Tensor], positions: torch.Tensor, inv_freq: torch.Tensor,
                  freq_row: torch.Tensor, slots: Optional[torch.Tensor], k_cache: Optional[torch.Tensor],
                  v_cache: Optional[torch.Tensor], num_q_heads: int, num_kv_heads: int, head_dim: int,
                  page_size: int, out_dtype: Optional[torch.dtype] = None,
                  q_out: Optional[torch.Tensor] = None, cs: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Rotate queries and keys, write keys and values into their page slots, return queries.

    ``x`` may be float32 while queries and the cache are bfloat16 (``out_dtype``): the bias is
    added and the rotation done in float32 and each value is rounded once.

    ``x`` is ``[N, (nq + 2 nkv) hd]``: query heads, key heads, value heads; or float32
    ``[slabs, N, (nq + 2 nkv) hd]``, partial sums of a projection cut along its inner size, which are
    added in slab order before the bias (bfloat16 outputs, ``cs`` given and widths in steps of 4
    only).  ``positions`` is
    int32 ``[rows, N]``; ``freq_row[f]`` names the row that frequency ``f`` uses (-1: none).
    ``k_cache`` is one layer's ``[pages, nkv, page_size, hd]``, ``v_cache`` its
    ``[pages, nkv, hd, page_size]``.  With ``num_kv_heads == 0`` only queries are rotated.
    ``cs`` is :func:`rope_table` of the same positions and tables, if the caller has it: the
    kernel then reads the cosines and sines instead of computing them for every head.
    """
    _dev(x, bias, positions, inv_freq, freq_row, slots, k_cache, v_cache, q_out)
    nq, nkv, hd = int(num_q_heads), int(num_kv_heads), int(head_dim)
    cols = (nq + 2 * nkv) * hd
    nslabs, slab_stride = 1, 0
    if x.dim() == 3:
        _need(x.dtype == torch.float32 and x.is_contiguous() and cs is not None,
              "slabs of x must be contiguous float32 and come with the table of cosines and sines")
        nslabs, slab_stride = x.shape[0], x.stride(0)
        x = x[0]
    n = x.shape[0]
    _need(x.dim() == 2 and x.shape[1] == cols and x.stride(1) == 1, "x must be [N, (nq + 2 nkv) hd]")
    odt = out_dtype or x.dtype
    rot_half = inv_freq.shape[0]
    _need(inv_freq.dtype == torch.float32 and inv_freq.is_contiguous() and 2 * rot_half <= hd,
          "inv_freq must be float32 [rot/2] with rot <= head_dim")
    _need(freq_row.dtype == torch.int32 and freq_row.shape == (rot_half,) and freq_row.is_contiguous(),
          "freq_row must be int32 [rot/2]")
    _need(positions.dtype == torch.int32 and positions.dim() == 2 and positions.shape[1] >= n
          and positions.stride(1) == 1, "positions must be int32 [rows, N]")
    if bias is not None:
        _need(bias.dtype == torch.float32 and bias.shape == (cols,) and bias.is_contiguous(),
              "bias must be float32 [(nq + 2 nkv) hd]")
    if nkv:
        _need(slots is not None and slots.dtype == torch.int32 and slots.shape == (n,) and slots.is_contiguous(),
              "slots must be int32 [N]")
        _need(k_cache is not None and v_cache is not None and k_cache.dtype == odt and v_cache.dtype == odt,
              "the cache must have the activation dtype")
        _need(k_cache.is_contiguous() and k_cache.dim() == 4 and tuple(k_cache.shape[1:]) == (nkv, page_size, hd),
              "k_cache must be [pages, nkv, page_size, hd]")
        _need(v_cache.is_contiguous() and v_cache.dim() == 4 and tuple(v_cache.shape[1:]) == (nkv, hd, page_size)
              and v_cache.shape[0] == k_cache.shape[0], "v_cache must be [pages, nkv, hd, page_size]")
    if q_out is None:
        q_out = torch.empty((n, nq * hd), dtype=odt, device=x.device)
    _need(q_out.shape == (n, nq * hd) and q_out.dtype == odt and q_out.is_contiguous(), "q_out must be [N, nq hd]")
    if cs is not None:
        _dev(cs)
        _need(cs.dtype == torch.float32 and cs.is_contiguous() and cs.dim() == 3 and cs.shape[0] >= n
              and tuple(cs.shape[1:]) == (rot_half, 2), "cs must be float32 [N, rot/2, 2]")
    fn = _fn("elementwise", "qvl_rope_kv_write",
             [_c_ptr, _c_int, _c_ptr, _c_ptr, _c_int, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr,
              _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, ctypes.c_longlong, _c_ptr])
    _check(fn(_ptr(x), x.stride(0), _ptr(bias), _ptr(positions), positions.stride(0), _ptr(inv_freq),
              _ptr(freq_row), _ptr(cs), _ptr(slots), _ptr(q_out), _ptr(k_cache), _ptr(v_cache), n, nq, nkv, hd, rot_half,
              int(page_size), dtype_code(x.dtype), dtype_code(odt), int(nslabs), int(slab_stride), _stream()),
           "rope_kv_write")
    return q_out


def rope_table(positions: torch.Tensor, inv_freq: torch.Tensor, freq_row: torch.Tensor, n: int) -> torch.Tensor:
    """Cosine and sine of every token's rotation angle: float32 ``[n, rot/2, 2]`` with
    ``(cos, sin)(positions[freq_row[f], i] * inv_freq[f])``, or ``(1, 0)`` where ``freq_row[f] < 0``."""
    _dev(positions, inv_freq, freq_row)
    rot_half = inv_freq.shape[0]
    _need(inv_freq.dtype == torch.float32 and inv_freq.is_contiguous(), "inv_freq must be float32 [rot/2]")
    _need(freq_row.dtype == torch.int32 and freq_row.shape == (rot_half,) and freq_row.is_contiguous(),
          "freq_row must be int32 [rot/2]")
    _need(positions.dtype == torch.int32 and positions.dim() == 2 and positions.shape[1] >= n
          and positions.stride(1) == 1, "positions must be int32 [rows, N]")
    out = torch.empty((n, rot_half, 2), dtype=torch.float32, device=positions.device)
    fn = _fn("elementwise", "qvl_rope_table", [_c_ptr, _c_int, _c_ptr, _c_ptr, _c_ptr, _c_int, _c_int, _c_ptr])
    _check(fn(_ptr(positions), positions.stride(0), _ptr(inv_freq), _ptr(freq_row), _ptr(out), int(n), rot_half,
              _stream()), "rope_table")
    return out


def copy_pages(cache: torch.Tensor, src: Sequence[int], dst: Sequence[int]) -> None:
    """Copy page ``src[i]`` to page ``dst[i]`` in every layer of ``cache [layers, pages, ...]``
    (the pages must not overlap between the two lists)."""
    _dev(cache)
    _need(cache.dim() >= 3 and cache.is_contiguous(), "cache must be contiguous [layers, pages, ...]")
    _need(len(src) == len(dst), "as many source as destination pages are needed")
    if not src:
        return
    pages = cache.shape[1]
    _need(all(0 <= int(p) < pages for p in list(src) + list(dst)), "a page id is outside the cache")
    _need(not set(map(int, src)) & set(map(int, dst)), "a page is both copied from and copied to")
    page_bytes = cache[0, 0].numel() * cache.element_size()
    idx = torch.tensor([list(map(int, src)), list(map(int, dst))], dtype=torch.int32, device=cache.device)
    fn = _fn("elementwise", "qvl_copy_pages",
             [_c_ptr, ctypes.c_longlong, _c_int, _c_ptr, _c_ptr, _c_int, _c_int, _c_ptr])
    _check(fn(_ptr(cache), pages * page_bytes, page_bytes, _ptr(idx[0]), _ptr(idx[1]), len(src), cache.shape[0],
              _stream()), "copy_pages")


def paged_attention_generic(q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor,
                            block_table: torch.Tensor, token_req: torch.Tensor, token_seqpos: torch.Tensor,
                            num_q_heads: int, window: Optional[int], scale: float,
                            out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Attention of every token over its request's pages; any head size, float32 arithmetic.

    ``q`` is ``[N, nq hd]``; token ``n`` belongs to row ``token_req[n]`` of ``block_table`` and
    sits at sequence index ``token_seqpos[n]``; it sees keys ``max(0, p - window + 1) .. p``.
    """
    _dev(q, k_cache, v_cache, block_table, token_req, token_seqpos, out)
    n = q.shape[0]
    nq = int(num_q_heads)
    _need(k_cache.dim() == 4 and k_cache.is_contiguous() and v_cache.is_contiguous(), "cache must be contiguous")
    pages, nkv, ps, hd = k_cache.shape
    _need(tuple(v_cache.shape) == (pages, nkv, hd, ps), "v_cache must be [pages, nkv, hd, page_size]")
    _need(q.shape == (n, nq * hd) and q.is_contiguous() and q.dtype == k_cache.dtype == v_cache.dtype,
          "q must be [N, nq hd] in the cache's dtype")
    _need(block_table.dtype == torch.int32 and block_table.dim() == 2 and block_table.is_contiguous(),
          "block_table must be int32 [R, width]")
    for t in (token_req, token_seqpos):
        _need(t.dtype == torch.int32 and t.shape == (n,) and t.is_contiguous(), "token maps must be int32 [N]")
    if out is None:
        out = torch.empty_like(q)
    _need(out.shape == q.shape and out.dtype == q.dtype and out.is_contiguous(), "out must match q")
    fn = _fn("attention_generic", "qvl_attn_generic",
             [_c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_int, _c_ptr, _c_ptr, _c_ptr, _c_int, _c_int, _c_int, _c_int,
              _c_int, _c_int, _c_float, _c_int, _c_ptr])
    _check(fn(_ptr(q), _ptr(k_cache), _ptr(v_cache), _ptr(block_table), block_table.shape[1], _ptr(token_req),
              _ptr(token_seqpos), _ptr(out), n, nq, nkv, hd, ps, int(window or 0), float(scale),
              dtype_code(q.dtype), _stream()), "paged_attention_generic")
    return out


def swiglu(x: torch.Tensor, out: Optional[torch.Tensor] = None, grouped: bool = False) -> torch.Tensor:
    """``silu(gate) * up`` for ``x`` of ``[N, 2 I]``: gate in the first ``I`` columns and up in the
    rest, or, ``grouped``, in alternating groups of 8 gate and 8 up columns."""
    _dev(x, out)
    _need(x.dim() == 2 and x.shape[1] % 2 == 0 and x.is_contiguous(), "x must be contiguous [N, 2 I]")
    n, inter = x.shape[0], x.shape[1] // 2
    if out is None:
        out = torch.empty((n, inter), dtype=x.dtype, device=x.device)
    _need(out.shape == (n, inter) and out.dtype == x.dtype and out.is_contiguous(), "out must be [N, I]")
    _need(not grouped or inter % 8 == 0, "grouped columns need a width in steps of 8")
    fn = _fn("elementwise", "qvl_swiglu", [_c_ptr, _c_ptr, _c_int, _c_int, _c_int, _c_int, _c_ptr])
    _check(fn(_ptr(x), _ptr(out), n, inter, dtype_code(x.dtype), int(grouped), _stream()), "swiglu")
    return out


def gemm_f32(x: torch.Tensor, weight: torch.Tensor, bias: Optional[torch.Tensor] = None,
             out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """True float32 ``x @ weight.T (+ bias)``; ``weight`` is ``[N, K]`` as a Linear stores it."""
    _dev(x, weight, bias, out)
    _need(x.dtype == torch.float32 and weight.dtype == torch.float32, "gemm_f32 takes float32 operands")
    _need(x.dim() == 2 and weight.dim() == 2 and x.shape[1] == weight.shape[1], "x [M, K] and weight [N, K]")
    _need(x.stride(1) == 1 and weight.stride(1) == 1, "rows of x and weight must be contiguous")
    m, k = x.shape
    n = weight.shape[0]
    if bias is not None:
        _need(bias.dtype == torch.float32 and bias.shape == (n,) and bias.is_contiguous(), "bias must be float32 [N]")
    if out is None:
        out = torch.empty((m, n), dtype=torch.float32, device=x.device)
    _need(out.shape == (m, n) and out.dtype == torch.float32 and out.stride(1) == 1, "out must be float32 [M, N]")
    fn = _fn("gemm_f32", "qvl_gemm_f32",
             [_c_ptr, _c_int, _c_ptr, _c_int, _c_ptr, _c_ptr, _c_int, _c_int, _c_int, _c_int, _c_ptr])
    _check(fn(_ptr(x), x.stride(0), _ptr(weight), weight.stride(0), _ptr(bias), _ptr(out), out.stride(0), m, n, k,
              _stream()), "gemm_f32")
    return out
