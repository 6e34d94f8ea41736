"""Decode steps replayed from HIP graphs.

A decode step of a 7B model is a few hundred short kernels; launched one by one from Python
the host, not the GPU, sets the step time (the reference measured the same on its hardware,
reference src/qwen25vl_lite/graphs.py:3-7, and also answers with graph capture).  A step in
which every request brings exactly one token has a fixed shape, so it is captured once per
(batch bucket, context bucket) and replayed: per step the host fills one pinned buffer with the
step's integers (token ids, positions, page slots, block tables, context lengths), copies it to
a fixed device buffer in one transfer, and launches the graph.

Batch sizes are rounded up to 1, 2, 3, 4, 6, 8, 12, 16, ... so that a server whose batch shrinks
and grows request by request captures a dozen graphs, not one per size.  The rows added are
padding: token 0 at position 0 with a context of one key, no page slot to write to (slot -1), a
block table that names page 0 for that key (whatever it holds is finite) and the spare state
row; their logits are computed and dropped.

The context bucket (the next power of two above the longest context) only fixes how many waves
the attention kernel splits a request's keys over; the true lengths travel in the buffer.

Lifetime.  A captured graph must never be destroyed while another capture is under way: its
destructor synchronizes the device, which a capture refuses, and an error thrown from a
destructor ends the process.  So nothing here refers back to the runner that owns it (a graph
holds the model, the cache and the slots, none of which know the runner): an engine that is
dropped frees its graphs at once, by reference count, not whenever the cycle collector next
runs.  A capture starts with a collection (garbage of the caller's own may hold graphs) and
keeps the collector off until it ends, and :meth:`DecodeGraphs.close` drops every graph after a
device synchronization for callers that want it done at a place of their choosing.
"""

from __future__ import annotations

import gc
from typing import Dict, List, Optional, Sequence, Tuple

import numpy as np
import torch

from ..parts.base import GroupStep, StepContext
from .batch import StepEntry

__all__ = ["DecodeGraphs"]


def _batch_bucket(n: int, most: int) -> int:
    """The smallest of 1, 2, 3, 4, 6, 8, 12, 16, 24, ... that holds n rows (at most ``most``)."""
    b = 1
    while True:
        for cand in (b, b + b // 2):
            if cand >= n:
                return min(cand, max(most, n))
        b *= 2


def _bucket(n: int, floor: int = 256) -> int:
    b = floor
    while b < n:
        b *= 2
    return b


class _Graph:
    """One captured step shape: its buffers, its StepContext of fixed views, its graph."""

    def __init__(self, parts: "_RunnerParts", batch: int, ctx_bucket: int):
        self.parts = parts
        self.batch = batch
        cache = parts.cache
        self.ngroups = len(cache.groups)
        self.rows = parts.model.spec.position_rows
        self.width = parts.max_blocks_per_seq
        self.ps = cache.page_size
        b, w = batch, self.width
        sizes = [("token_ids", b), ("positions", self.rows * b), ("token_req", b), ("token_seqpos", b),
                 ("cu_q", b + 1), ("ctx_len", b), ("req_slots", b), ("logit_rows", b)]
        for g in range(self.ngroups):
            sizes += [(f"slots{g}", b), (f"table{g}", b * w)]
        self.offsets: Dict[str, Tuple[int, int]] = {}
        total = 0
        for name, n in sizes:
            self.offsets[name] = (total, n)
            total += (n + 3) // 4 * 4
        self.host = torch.zeros(total, dtype=torch.int32, pin_memory=True)
        self.hv = self.host.numpy()
        self.dev = torch.zeros(total, dtype=torch.int32, device=parts.device)
        self.copied = torch.cuda.Event()
        self.copied.record()
        h, d = self.h, self._d
        h("token_req")[:] = np.arange(b)
        h("cu_q")[:] = np.arange(b + 1)
        h("logit_rows")[:] = np.arange(b)
        for g in range(self.ngroups):
            h(f"table{g}")[:] = -1
        self.tables = [h(f"table{g}", (b, w)) for g in range(self.ngroups)]
        self.row_req: List[object] = [None] * b
        self.row_len = [[0] * b for _ in range(self.ngroups)]
        self.step = StepContext(
            num_tokens=b, num_reqs=b, token_ids=d("token_ids"), positions=d("positions", (self.rows, b)),
            token_req=d("token_req"), token_seqpos=d("token_seqpos"), cu_q=d("cu_q"), ctx_len=d("ctx_len"),
            req_slots=d("req_slots"),
            groups=[GroupStep(d(f"slots{g}"), d(f"table{g}", (b, w)), self.ps) for g in range(self.ngroups)],
            logit_rows=d("logit_rows"), cu_q_host=list(range(b + 1)), ctx_len_host=[ctx_bucket] * b,
            req_slots_host=[0] * b, max_q_len=1, max_ctx_len=ctx_bucket, dtype=parts.dtype)
        self.graph = None
        self.logits = None

    def h(self, name, shape=None):
        """The named array of the pinned host buffer."""
        o, n = self.offsets[name]
        v = self.hv[o:o + n]
        return v if shape is None else v.reshape(shape)

    def _d(self, name, shape=None):
        o, n = self.offsets[name]
        v = self.dev[o:o + n]
        return v if shape is None else v.view(shape)

    def fill(self, entries: Sequence[StepEntry]) -> None:
        cache, ps, h = self.parts.cache, self.ps, self.h
        n, b = len(entries), self.batch
        self.copied.synchronize()          # the previous transfer has read the pinned buffer
        # where each request stands and the offset of its positions come from its slot's record,
        # gathered by slot index
        records = cache.records
        at = np.fromiter((cache.requests[e.req_id].slot for e in entries), np.int64, n)
        starts = np.zeros(b, np.int32)     # rows from n on are padding: position 0, one key, no slot
        deltas = np.zeros(b, np.int32)
        starts[:n] = records.num_tokens[at]
        deltas[:n] = records.rope_delta[at]
        tokens = h("token_ids")
        tokens[:n] = np.fromiter((e.tokens[0] for e in entries), np.int32, n)
        tokens[n:] = 0
        h("token_seqpos")[:] = starts
        h("positions", (self.rows, b))[:] = starts + deltas
        h("ctx_len")[:] = starts + 1
        slots_of = h("req_slots")
        slots_of[:n] = at
        slots_of[n:] = self.parts.pad_state_slot
        for g in range(self.ngroups):
            table_np, lens, slots = self.tables[g], self.row_len[g], h(f"slots{g}")
            for i, e in enumerate(entries):
                t = cache.table(e.req_id, g)
                if self.row_req[i] is not cache.requests[e.req_id]:   # another request, or this one admitted anew
                    table_np[i, :] = -1
                    lens[i] = 0
                if len(t) > lens[i]:
                    # pages only ever join at the end; entries a window has given back are never read
                    table_np[i, lens[i]:len(t)] = t[lens[i]:]
                    lens[i] = len(t)
                slots[i] = t[e.start // ps] * ps + e.start % ps
            for i in range(n, b):
                if self.row_req[i] is not None or table_np[i, 0] != 0:
                    table_np[i, :] = -1
                    table_np[i, 0] = 0
                    lens[i] = 0
                slots[i] = -1
        for i, e in enumerate(entries):
            self.row_req[i] = cache.requests[e.req_id]
        for i in range(n, b):
            self.row_req[i] = None

    def run(self, entries: Sequence[StepEntry], device_tokens: Optional[torch.Tensor] = None) -> torch.Tensor:
        parts = self.parts
        self.fill(entries)
        self.dev.copy_(self.host, non_blocking=True)
        self.copied.record()
        if device_tokens is not None:
            # the entries' token ids are still on the device (sampled by the step before, whose ids
            # the host has not seen): they go into the step's input without a detour
            self.step.token_ids[:len(entries)].copy_(device_tokens)
        if self.graph is None:
            # twice eagerly (libraries pick kernels and workspaces, per-step tile lists are made),
            # then once more under capture.  Keys and values go to the step's own cache slots and
            # the logits to their buffer, so running the step again with the same inputs changes
            # nothing there.  Per-request state of a mixer is another matter: every pass advances
            # it.  The rows are copied aside first and put back after each eager pass, so that the
            # replay below is the only pass that counts.
            kept = [None if s is None else s.clone() for s in parts.states]
            for _ in range(2):
                self.step.per_pass.clear()
                parts.model.forward(self.step, parts.slots)
                for s, k in zip(parts.states, kept):
                    if s is not None:
                        s.copy_(k)
            torch.cuda.synchronize()
            self.step.per_pass.clear()    # what a pass computes from the step's values is computed in the graph
            self.graph, self.logits = _capture(lambda: parts.model.forward(self.step, parts.slots))
        self.graph.replay()
        return self.logits[:len(entries)]


def _capture(work):
    """Capture ``work()`` into a graph; returns ``(graph, what work returned)``.

    Garbage that holds an older graph is collected before the capture begins and the cycle
    collector stays off until it has ended: no graph's destructor may run in between."""
    gc.collect()
    was_on = gc.isenabled()
    gc.disable()
    try:
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            out = work()
    finally:
        if was_on:
            gc.enable()
    return graph, out


class _RunnerParts:
    """What a graph needs of the runner it belongs to, without the runner itself (which owns
    the graphs: a reference back would make a cycle that only the collector could free)."""

    def __init__(self, runner):
        self.model = runner.model
        self.cache = runner.cache
        self.slots = runner.slots
        self.states = runner.states
        self.device = runner.device
        self.dtype = runner.dtype
        self.pad_state_slot = runner.pad_state_slot
        self.max_blocks_per_seq = runner.ecfg.max_blocks_per_seq
        self.max_num_seqs = runner.ecfg.max_num_seqs


class DecodeGraphs:
    """The graphs of a runner, keyed by (batch bucket, context bucket)."""

    def __init__(self, runner, max_graphs: int = 32):
        self.parts = _RunnerParts(runner)
        self.max_graphs = max_graphs
        self.graphs: Dict[Tuple[int, int], _Graph] = {}

    def close(self) -> None:
        """Drop every captured graph, after the device has finished what it was given."""
        if self.graphs:
            if torch.cuda.is_available():
                torch.cuda.synchronize()
            self.graphs.clear()

    @staticmethod
    def takes(entries: Sequence[StepEntry]) -> bool:
        return all(len(e.tokens) == 1 and e.positions is None and list(e.want) == [0] for e in entries)

    def run(self, entries: Sequence[StepEntry], device_tokens: Optional[torch.Tensor] = None) -> torch.Tensor:
        ctx = max(e.start for e in entries) + 1
        key = (_batch_bucket(len(entries), self.parts.max_num_seqs), _bucket(ctx))
        g = self.graphs.get(key)
        if g is None:
            if len(self.graphs) >= self.max_graphs:
                # the oldest graph goes, here and now (nothing else refers to it), outside any capture
                torch.cuda.synchronize()
                del self.graphs[next(iter(self.graphs))]
            g = self.graphs[key] = _Graph(self.parts, *key)
        return g.run(entries, device_tokens)
