"""Dispatch to the matrix-core attention kernel (bfloat16, head sizes in steps of 16).

The kernel is compiled per head size (``-DHD=...``) at its first use.  A step's tokens are cut
into tiles of 16 columns, a column being a (token, query head of one key/value group) pair; the
tile list depends on the batch and on the group size only and is built once per step.
"""

from __future__ import annotations

import collections
import ctypes
from typing import Optional, Tuple

import numpy as np
import torch

from .kernels import _check, _fn, _need, _ptr, _stream

__all__ = ["try_attention", "supports", "tiles_for", "plan_splits"]

_c_int, _c_float, _c_ptr = ctypes.c_int, ctypes.c_float, ctypes.c_void_p
_MAX_HD = 256
# Thresholds that follow the device: counts per compute unit (measured on 256 of them); the names below
# them hold a number instead of None where a caller (a test) fixes the count itself.
TARGET_PER_CU = 2          # from this many (tile, head) pairs a compute unit on, a wave per tile fills the device
FILL_PER_CU = 1            # with fewer cooperative blocks than this, contexts are split among blocks
WIDE_WALKS_PER_CU = 3      # the kind of the kernel whose waves carry three column tiles: from this many walks on
WIDE_BLOCKS_PER_CU = 586   # ... that have this many 32-key blocks to walk between them (150,000 on 256 units)
TARGET_BLOCKS = None
FILL_BLOCKS = None
MIN_KEYS_PER_SPLIT = 256   # keys a split has at least
SPLIT_FROM_KEYS = 768      # shorter contexts are walked by one block: merging splits (stores, a counter and loads that go
                           # through to memory) costs a decode step about 4.5 us, a block's walk 12.7 us per 1,000 keys
                           # (one compute unit by itself fetches its keys and values at about 40 GB/s); measured at batch 1 and 8:
                           # 527 keys 11.5 us whole, 11.9 in two splits; 1,024 keys 17.8 whole, 12.0 in four
MERGE_COUNTERS = 1 << 16   # (tile, kv head) pairs whose splits one launch can merge by itself
ALONE_KEYS = 4096          # decoded tokens beside prompt portions get a launch of their own from this context on
WIDE_CT = 3
_cu_count = {}


def _compute_units(device=None) -> int:
    key = torch.device(device).index if device is not None and torch.device(device).index is not None else torch.cuda.current_device()
    if key not in _cu_count:
        _cu_count[key] = torch.cuda.get_device_properties(key).multi_processor_count
    return _cu_count[key]


def _target_blocks(device=None) -> int:
    return TARGET_BLOCKS if TARGET_BLOCKS is not None else TARGET_PER_CU * _compute_units(device)


def _fill_blocks(device=None) -> int:
    return FILL_BLOCKS if FILL_BLOCKS is not None else FILL_PER_CU * _compute_units(device)


def supports(head_dim: int, dtype: torch.dtype) -> bool:
    return dtype == torch.bfloat16 and head_dim % 16 == 0 and 16 <= head_dim <= _MAX_HD




def block_tiles(head_dim: int, wide: bool = False) -> int:
    """Column tiles of one entry of the block list (BLK_WAVES * BLK_CT in the source)."""
    return int(_fn("attention_mfma", "qvl_attn_mfma_block_tiles", [], block_defines(head_dim, wide))())


def block_defines(head_dim: int, wide: bool) -> dict:
    """The library of the kernel for many tiles: compiled per head size, and for head sizes up to 128
    in a second kind whose waves carry three column tiles instead of two.  That kind reads its operands
    from LDS once for three tiles (a third less LDS traffic and bookkeeping per product) at the price
    of longer walks and no second group of waves: 6 % faster from about 8,192 prompt tokens on at the
    7B decoder's heads, slower below."""
    return {"HD": head_dim, "BLK_CT": WIDE_CT} if wide and head_dim <= 128 else {"HD": head_dim}


def tiles_for(cu_q, group: int, tile_ct: int = 1, ctx_len=None) -> Tuple[np.ndarray, np.ndarray]:
    """``(tile_req, tile_ct)``: for request r with q tokens, ceil(q * group / (16 * tile_ct)) entries.
    With ``ctx_len`` the entries are listed by the last key they see, latest first: the longest
    walks start first and the short ones fill the compute units as they become free."""
    q = np.diff(np.asarray(cu_q, dtype=np.int64))
    cols = 16 * tile_ct
    counts = (q * group + cols - 1) // cols
    req = np.repeat(np.arange(len(q), dtype=np.int32), counts)
    starts = np.cumsum(counts) - counts
    ct = (np.arange(int(counts.sum()), dtype=np.int64) - np.repeat(starts, counts)).astype(np.int32)
    if ctx_len is not None and len(req):
        last_token = np.minimum(((ct.astype(np.int64) + 1) * cols - 1) // group, q[req] - 1)
        last_key = np.asarray(ctx_len, dtype=np.int64)[req] - q[req] + last_token
        order = np.argsort(-last_key, kind="stable")
        req, ct = req[order], ct[order]
    return req, ct


def plan_splits(num_tiles: int, nkv: int, max_ctx: int, device=None) -> Tuple[str, int, int]:
    """``(kernel, nsplit, keys_per_split)``.  ``"tile"``: many tiles, as in prefill: a block owns
    several tiles per wave and shares the keys through LDS.  ``"coop"``: the waves of a block share a tile (few tiles, as in decode); its keys are
    split among ``nsplit`` blocks when the context is long and the blocks are few."""
    blocks = num_tiles * nkv
    if blocks >= _target_blocks(device):
        return "tile", 1, 0
    want = (_fill_blocks(device) + blocks - 1) // blocks
    nsplit = max(1, min(want, max_ctx // MIN_KEYS_PER_SPLIT)) if max_ctx >= SPLIT_FROM_KEYS else 1
    if nsplit == 1:
        return "coop", 1, 0
    # splits begin at a multiple of 32 at or below the first key a tile sees: up to 31 keys more
    per = ((max_ctx + 31 + nsplit - 1) // nsplit + 31) // 32 * 32
    return "coop", (max_ctx + 31 + per - 1) // per, per


_queues = {}
_merge_counters = {}
taken = collections.Counter()   # launches by kind of kernel (a captured launch counts once): what a measurement reports


def _counters(device: torch.device) -> torch.Tensor:
    """Per device: the counters by which the blocks of a split attention find out which of them
    finishes last and merges.  As with the work queues, a launch finds them at zero and leaves
    them at zero, and launches on one device must follow each other on one stream."""
    key = torch.device(device).index or 0
    if key not in _merge_counters:
        _merge_counters[key] = torch.zeros(MERGE_COUNTERS, dtype=torch.int32, device=device)
    return _merge_counters[key]


def _work_queue(device: torch.device):
    """Per device: the counters of the block kernel's work queues and how many workgroups fill
    the device.  A launch finds the counters at zero and leaves them at zero; launches on one
    device share them, so they must follow each other on one stream (the engine has one).  A launch
    that reports an error has them cleared."""
    key = torch.device(device).index or 0
    if key not in _queues:
        cus = torch.cuda.get_device_properties(device).multi_processor_count
        _queues[key] = (torch.zeros(16, dtype=torch.int32, device=device), cus)
    return _queues[key]


def _step_tiles(step, group: int, tile_ct: int, device, by_length: bool = False, only=None):
    """The step's entries on the device; ``only``: a tuple of 0/1 per request, entries of the others left out."""
    cache = step.derived
    key = ("tiles", group, tile_ct, by_length, only)
    if key not in cache:
        req, ct = tiles_for(step.cu_q_host, group, tile_ct, step.ctx_len_host if by_length else None)
        if only is not None:
            keep = np.asarray(only, dtype=bool)[req]
            req, ct = req[keep], ct[keep]
        both = torch.from_numpy(np.concatenate([req, ct])).to(device, non_blocking=True)
        cache[key] = (both[:len(req)], both[len(req):], len(req))
    return cache[key]


def _walk_blocks(step, group: int, tile_ct: int, only=None) -> int:
    """About how many 32-key blocks the step's entries of ``tile_ct`` column tiles walk, for one key/value head."""
    q = np.diff(np.asarray(step.cu_q_host, dtype=np.int64))
    ctx = np.asarray(step.ctx_len_host, dtype=np.int64)
    if only is not None:
        q = q * np.asarray(only, dtype=np.int64)
    entries = (q * group + 16 * tile_ct - 1) // (16 * tile_ct)
    return int((entries * np.maximum(1, (ctx - q // 2 + 31) // 32)).sum())


def long_single_tiles(step, group: int, nkv: int, device=None):
    """In a step that has prompt portions too: the requests whose tokens make one tile only
    (decoded tokens) if they are few and their contexts long, as a tuple of 0/1 per request, else
    None.  Planned together with the portions, each of them gets one workgroup (or one block) that
    walks its whole context, and that walk is what the step then waits for; in a launch of their
    own their contexts are split among blocks (measured at the 7B decoder's heads: 8 decoded tokens
    at 8,192 keys beside a portion of 256 take 87 us together, 32 and 13 apart).  Below
    ``ALONE_KEYS`` the two launches, one after the other, cost more than the walks they shorten."""
    q = np.diff(np.asarray(step.cu_q_host, dtype=np.int64))
    single = (q > 0) & (q * group <= 16)
    if not single.any() or single.all():
        return None
    longest = int(np.asarray(step.ctx_len_host, dtype=np.int64)[single].max())
    if longest < ALONE_KEYS or int(single.sum()) * nkv >= _fill_blocks(device):
        return None
    return tuple(int(x) for x in single)


def block_groups(walks: int, places: int, head_dim: int) -> int:
    """Wave groups per workgroup for a step of ``walks`` (entry, head) pairs on a device that holds
    ``places`` plain workgroups at a time.  Two groups (head sizes up to 128) halve a walk's time at
    a tenth less throughput (measured at 2,048 to 8,192 tokens): they pay when all walks start at
    once and the longest decides, not when places are taken several times over."""
    most = int(_fn("attention_mfma", "qvl_attn_mfma_block_max_groups", [], {"HD": head_dim})())
    return 2 if most >= 2 and walks <= places else 1


def try_attention(q, k_cache, v_cache, block_table, step, num_q_heads: int, window: Optional[int],
                  scale: float, force_groups: Optional[int] = None, force_wide: Optional[bool] = None) -> Optional[torch.Tensor]:
    """The attention through the matrix-core kernel, or None if it does not take this shape.
    Calls on one device must not overlap (one stream): the kernel for prompt portions keeps its
    work-queue counters in memory that all calls on the device share.
    ``force_groups``, ``force_wide`` (tests): the workgroup kind of the kernel for prompt portions and
    whether its waves carry three column tiles, else chosen by :func:`block_groups` and the number of walks."""
    pages, nkv, ps, hd = k_cache.shape
    if not supports(hd, q.dtype) or ps % 16:
        return None
    n, nq = q.shape[0], int(num_q_heads)
    _need(q.is_cuda and q.shape == (n, nq * hd) and q.is_contiguous(), "q must be contiguous [N, nq hd] on the GPU")
    _need(k_cache.dtype == v_cache.dtype == torch.bfloat16 and k_cache.is_contiguous() and v_cache.is_contiguous()
          and tuple(v_cache.shape) == (pages, nkv, hd, ps), "cache must be bfloat16 [pages, nkv, ps, hd] / [.., hd, ps]")
    _need(block_table.dtype == torch.int32 and block_table.dim() == 2 and block_table.is_contiguous()
          and block_table.shape[0] == step.num_reqs, "block_table must be int32 [R, width]")
    _need(nq % nkv == 0, "query heads must be a multiple of key/value heads")
    tile_req, tile_ct, num_tiles = _step_tiles(step, nq // nkv, 1, q.device)
    out = torch.empty_like(q)
    defines = {"HD": hd}
    kind, nsplit, per = plan_splits(num_tiles, nkv, step.max_ctx_len, q.device)

    def many_tiles(only):
        tile_req, tile_ct, num_tiles = _step_tiles(step, nq // nkv, block_tiles(hd), q.device, by_length=True, only=only)
        wide = force_wide
        if wide is None:   # many and long walks: measured at the 7B decoder's heads, the wide kind wins from one prompt of about 8,192 tokens on
            cus = _compute_units(q.device)
            wide = (hd <= 128 and num_tiles * nkv >= WIDE_WALKS_PER_CU * cus
                    and _walk_blocks(step, nq // nkv, block_tiles(hd), only) * nkv >= WIDE_BLOCKS_PER_CU * cus)
        defines = block_defines(hd, wide)
        if wide:
            tile_req, tile_ct, num_tiles = _step_tiles(step, nq // nkv, block_tiles(hd, True), q.device, by_length=True, only=only)
        fn = _fn("attention_mfma", "qvl_attn_mfma_block",
                 [_c_ptr] * 4 + [_c_int] + [_c_ptr] * 4 + [_c_int, _c_ptr] + [_c_int] * 4
                 + [_c_float, _c_ptr, _c_int, _c_int, _c_ptr], defines)
        queue, cus = _work_queue(q.device)
        per_cu = int(_fn("attention_mfma", "qvl_attn_mfma_block_per_cu", [], defines)())
        most = int(_fn("attention_mfma", "qvl_attn_mfma_block_max_groups", [], defines)())
        groups = block_groups(num_tiles * nkv, cus * per_cu, hd) if force_groups is None else force_groups
        groups = min(groups, most) if force_groups is None else groups
        code = fn(_ptr(q), _ptr(k_cache), _ptr(v_cache), _ptr(block_table), block_table.shape[1], _ptr(step.cu_q),
                  _ptr(step.ctx_len), _ptr(tile_req), _ptr(tile_ct), num_tiles, _ptr(out), nq, nkv, ps, int(window or 0),
                  float(scale), _ptr(queue), cus * (per_cu if groups == 1 else 1), groups, _stream())
        if code:
            # whatever a launch that went wrong did to the counters, the next one starts from zero
            queue.zero_()
        _check(code, "paged_attention (matrix cores)")
        taken[f"many tiles, {WIDE_CT if wide else 2} column tiles a wave, {groups} wave group{'s' if groups > 1 else ''}"] += 1

    def shared_tiles(only, nsplit, per):
        tile_req, tile_ct, num_tiles = _step_tiles(step, nq // nkv, 1, q.device, only=only)
        cu_q = step.cu_q
        if only is None and step.max_q_len == 1 and num_tiles == step.num_reqs == len(step.cu_q_host) - 1 == step.cu_q_host[-1]:
            # decoded tokens only: request i brings token i and has tile i, and the kernel is told so
            # instead of reading it (two dependent reads less before its first key is asked for)
            tile_req = tile_ct = cu_q = None
        scratch = None
        if nsplit > 1:
            floats = _fn("attention_mfma", "qvl_attn_mfma_scratch_floats", [_c_int] * 3, defines)
            floats.restype = ctypes.c_longlong
            scratch = torch.empty(int(floats(num_tiles, nkv, nsplit)), dtype=torch.float32, device=q.device)
        if nsplit > 1 and num_tiles * nkv <= MERGE_COUNTERS:
            # the block of each (tile, head) that finishes last merges the splits: one launch
            counters = _counters(q.device)
            fn = _fn("attention_mfma", "qvl_attn_mfma_coop_merged",
                     [_c_ptr] * 4 + [_c_int] + [_c_ptr] * 4 + [_c_int, _c_ptr, _c_ptr, _c_ptr] + [_c_int] * 4
                     + [_c_float, _c_int, _c_int, _c_ptr], defines)
            code = fn(_ptr(q), _ptr(k_cache), _ptr(v_cache), _ptr(block_table), block_table.shape[1], _ptr(cu_q),
                      _ptr(step.ctx_len), _ptr(tile_req), _ptr(tile_ct), num_tiles, _ptr(out), _ptr(scratch),
                      _ptr(counters), nq, nkv, ps, int(window or 0), float(scale), nsplit, per, _stream())
            if code:
                counters.zero_()
            _check(code, "paged_attention (matrix cores, shared tiles, merged)")
            taken["shared tiles, keys split among blocks, merged in the launch"] += 1
            return
        fn = _fn("attention_mfma", "qvl_attn_mfma_coop",
                 [_c_ptr] * 4 + [_c_int] + [_c_ptr] * 4 + [_c_int, _c_ptr, _c_ptr] + [_c_int] * 4
                 + [_c_float, _c_int, _c_int, _c_ptr], defines)
        _check(fn(_ptr(q), _ptr(k_cache), _ptr(v_cache), _ptr(block_table), block_table.shape[1], _ptr(cu_q),
                  _ptr(step.ctx_len), _ptr(tile_req), _ptr(tile_ct), num_tiles, _ptr(out), _ptr(scratch), nq, nkv, ps,
                  int(window or 0), float(scale), nsplit, per, _stream()),
               "paged_attention (matrix cores, shared tiles)")
        taken["shared tiles" + (", keys split among blocks, merged by a second launch" if nsplit > 1 else "")] += 1

    single = long_single_tiles(step, nq // nkv, nkv, q.device) if force_groups is None else None
    if single is not None:   # the few decoded tokens with long contexts by themselves, the rest planned anew
        longest = max(c for c, s in zip(step.ctx_len_host, single) if s)
        _, nsplit1, per1 = plan_splits(sum(single), nkv, longest, q.device)   # fewer blocks than fill the device: the kernel that splits
        shared_tiles(single, nsplit1, per1)
        rest = tuple(1 - s for s in single)
        kind, nsplit, per = plan_splits(_step_tiles(step, nq // nkv, 1, q.device, only=rest)[2], nkv,
                                        max(c for c, s in zip(step.ctx_len_host, rest) if s), q.device)
        if kind == "tile":
            many_tiles(rest)
        else:
            shared_tiles(rest, nsplit, per)
    elif kind == "tile":
        many_tiles(None)
    else:
        shared_tiles(None, nsplit, per)
    return out
