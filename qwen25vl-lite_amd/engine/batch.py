"""Building one step's batch: from (request, its next tokens) to the flat device arrays.

A step takes any mix of prompt portions and single decoded tokens.  Each entry contributes a
contiguous run of tokens; the arrays say, per token, its id, its position rows, its request
and its index in the sequence, and per cache group where its keys and values go; per request,
where its run starts, how long its context is after the step, its pages and its state slot.
All integer arrays of a step travel to the device in one copy.
"""

from __future__ import annotations

from dataclasses import dataclass, field
from typing import List, Optional, Sequence

import numpy as np
import torch

from ..cache.manager import CacheManager
from ..parts.base import GroupStep, StepContext

__all__ = ["StepEntry", "build_step"]


@dataclass
class StepEntry:
    """A request's part in a step: ``tokens`` follow the ``start`` tokens already in the cache.

    ``positions`` gives the position rows of these tokens (``[rows][len(tokens)]``); None means
    text positions, ``start + i + rope_delta`` on every row (reference rope.py:238-247).
    ``want`` lists the places among ``tokens`` whose logits are asked for.
    """

    req_id: object
    tokens: Sequence[int]
    start: int
    want: Sequence[int] = ()
    positions: Optional[Sequence[Sequence[int]]] = None
    rope_delta: int = 0


def _align(n: int, a: int = 4) -> int:
    return (n + a - 1) // a * a


def build_step(entries: Sequence[StepEntry], cache: CacheManager, position_rows: int, dtype: torch.dtype,
               device: torch.device, vocab_size: Optional[int] = None) -> StepContext:
    """Lay out the batch (pages must have been reserved) and copy it to the device."""
    if not entries:
        raise ValueError("a step needs at least one entry")
    n_total = sum(len(e.tokens) for e in entries)
    r = len(entries)
    ngroups = len(cache.groups)
    ps = cache.page_size

    token_ids = np.empty(n_total, np.int32)
    positions = np.empty((position_rows, n_total), np.int32)
    token_req = np.empty(n_total, np.int32)
    token_seqpos = np.empty(n_total, np.int32)
    cu_q = np.zeros(r + 1, np.int32)
    ctx_len = np.empty(r, np.int32)
    req_slots = np.empty(r, np.int32)
    slot_maps = [np.empty(n_total, np.int32) for _ in range(ngroups)]
    logit_rows: List[int] = []
    seen = set()
    width = 1
    for e in entries:
        for g in range(ngroups):
            width = max(width, len(cache.table(e.req_id, g)))
    tables = [np.full((r, width), -1, np.int32) for _ in range(ngroups)]

    at = 0
    for i, e in enumerate(entries):
        n = len(e.tokens)
        if n == 0:
            raise ValueError(f"request {e.req_id!r} brings no tokens to the step")
        if e.req_id in seen:
            raise ValueError(f"request {e.req_id!r} appears twice in one step")
        seen.add(e.req_id)
        if cache.num_tokens(e.req_id) != e.start:
            raise ValueError(f"request {e.req_id!r}: the cache holds {cache.num_tokens(e.req_id)} tokens, "
                             f"the step continues from {e.start}")
        ids = np.asarray(e.tokens, dtype=np.int64)
        if vocab_size is not None and (ids.min() < 0 or ids.max() >= vocab_size):
            raise ValueError(f"request {e.req_id!r}: token id outside [0, {vocab_size})")
        token_ids[at:at + n] = ids
        seq = np.arange(e.start, e.start + n, dtype=np.int32)
        token_seqpos[at:at + n] = seq
        token_req[at:at + n] = i
        if e.positions is None:
            positions[:, at:at + n] = seq + np.int32(e.rope_delta)
        else:
            pos = np.asarray(e.positions, dtype=np.int64)
            if pos.shape != (position_rows, n):
                raise ValueError(f"request {e.req_id!r}: positions must be [{position_rows}, {n}], got {pos.shape}")
            positions[:, at:at + n] = pos
        cu_q[i + 1] = at + n
        ctx_len[i] = e.start + n
        req_slots[i] = cache.slot_of(e.req_id)
        for g in range(ngroups):
            slot_maps[g][at:at + n] = cache.slot_mapping(e.req_id, g, e.start, e.start + n)
            t = cache.table(e.req_id, g)
            tables[g][i, :len(t)] = t
        for w in e.want:
            if not 0 <= int(w) < n:
                raise ValueError(f"request {e.req_id!r}: wanted place {w} is outside its {n} tokens")
            logit_rows.append(at + int(w))
        at += n

    pieces = [token_ids, positions.reshape(-1), token_req, token_seqpos, cu_q, ctx_len, req_slots,
              np.asarray(logit_rows, np.int32)]
    for g in range(ngroups):
        pieces += [slot_maps[g], tables[g].reshape(-1)]
    offsets, total = [], 0
    for p in pieces:
        offsets.append(total)
        total += _align(p.size)
    host = torch.empty(max(total, 1), dtype=torch.int32, pin_memory=(device.type == "cuda"))
    hv = host.numpy()
    for off, p in zip(offsets, pieces):
        hv[off:off + p.size] = p
    dev = host.to(device, non_blocking=True)

    def view(k: int, shape=None):
        t = dev[offsets[k]:offsets[k] + pieces[k].size]
        return t if shape is None else t.view(shape)

    groups = [GroupStep(slot_mapping=view(8 + 2 * g), block_table=view(9 + 2 * g, (r, width)), page_size=ps)
              for g in range(ngroups)]
    return StepContext(
        num_tokens=n_total, num_reqs=r,
        token_ids=view(0), positions=view(1, (position_rows, n_total)), token_req=view(2), token_seqpos=view(3),
        cu_q=view(4), ctx_len=view(5), req_slots=view(6), groups=groups, logit_rows=view(7),
        cu_q_host=cu_q.tolist(), ctx_len_host=ctx_len.tolist(), req_slots_host=req_slots.tolist(),
        max_q_len=int(np.max(cu_q[1:] - cu_q[:-1])), max_ctx_len=int(ctx_len.max()), dtype=dtype,
    )
