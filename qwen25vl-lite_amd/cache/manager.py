"""The cache manager: pages for keys and values, a block table per request and group,
and slots for per-request state of fixed size.

Layers with the same need (key/value heads, head size, window) form a *group*.  Each group
has a page pool of its own and each live request a block table per group: entry ``i`` is the
page that holds tokens ``i * page_size ...`` of the request, or -1 once a windowed group has
given that page back.  Pages are given back when a request ends, when it is preempted, and,
in a windowed group, as soon as no later token can see any key of the page; they are handed
out again to whoever asks next.

Beside the pages every live request holds one *slot*, an index below ``max_num_seqs``.  A
mixer with state of fixed size keeps it in row ``slot`` of its state tensor; the runner
clears the row when the slot is taken.  Row ``slot`` of :class:`SlotRecords` (``records``) is the
request's fixed-size record: its cached length, its rope delta and its sampler's state, filled at
admission and gathered by slot index when a step is built and sampled.

All of this is host bookkeeping; the tensors live in :class:`KVStorage`.
"""

from __future__ import annotations

from dataclasses import dataclass, field
from typing import Dict, List, Optional, Sequence, Tuple

from ..parts.base import CacheNeed
from .pages import OutOfPages, PagePool
from .prefix import RadixPrefixCache
from .slots import SlotRecords

__all__ = ["CacheGroupSpec", "CacheManager", "RequestPages", "OutOfPages", "OutOfSlots"]


class OutOfSlots(RuntimeError):
    """More requests are live than there are state slots."""


@dataclass(frozen=True)
class CacheGroupSpec:
    need: CacheNeed
    num_layers: int


@dataclass
class RequestPages:
    slot: int
    tables: List[List[int]]                 # per group; -1 = given back
    num_tokens: int = 0                     # tokens whose keys are in the cache
    prefix_nodes: List[int] = field(default_factory=list)
    fresh: bool = True                      # the slot's state rows still need clearing


class CacheManager:
    def __init__(self, groups: Sequence[CacheGroupSpec], num_pages: int, page_size: int, max_num_seqs: int,
                 enable_prefix_cache: bool = True, max_prefix_nodes: int = 4096):
        if page_size <= 0:
            raise ValueError("page_size must be positive")
        self.groups = list(groups)
        self.page_size = int(page_size)
        self.max_num_seqs = int(max_num_seqs)
        self.pools = [PagePool(num_pages) for _ in self.groups]
        self._free_slots = list(range(self.max_num_seqs - 1, -1, -1))
        self.records = SlotRecords(self.max_num_seqs)
        self.requests: Dict[object, RequestPages] = {}
        # A shared prefix is only valid where every group still holds all of its pages.
        self.prefix_cache: Optional[RadixPrefixCache] = None
        if enable_prefix_cache and self.groups and all(g.need.window is None for g in self.groups):
            self.prefix_cache = RadixPrefixCache(self.pools, self.page_size, max_prefix_nodes)

    # ------------------------------------------------------------------ requests and slots
    def admit(self, req_id, params=None, rope_delta: int = 0, generated: int = 0) -> int:
        """Give the request a slot and fill the slot's record: ``params`` are its sampling settings
        (None: it is not sampled), ``rope_delta`` the offset of its text positions, ``generated`` the
        tokens it has generated already (a request admitted again after it gave way)."""
        if req_id in self.requests:
            raise ValueError(f"request {req_id!r} is already live")
        if not self._free_slots:
            raise OutOfSlots(f"all {self.max_num_seqs} request slots are taken")
        slot = self._free_slots.pop()
        self.requests[req_id] = RequestPages(slot=slot, tables=[[] for _ in self.groups])
        self.records.assign(slot, params, rope_delta, generated)
        return slot

    def slot_of(self, req_id) -> int:
        return self.requests[req_id].slot

    def take_fresh(self, req_id) -> bool:
        """True once per admission: the caller clears the slot's state rows."""
        rp = self.requests[req_id]
        fresh, rp.fresh = rp.fresh, False
        return fresh

    def num_tokens(self, req_id) -> int:
        return self.requests[req_id].num_tokens

    def release(self, req_id) -> None:
        """The request is over (finished or preempted): everything it holds goes back."""
        rp = self.requests.pop(req_id)
        for g, table in enumerate(rp.tables):
            self.pools[g].free([p for p in table if p >= 0])
        if rp.prefix_nodes and self.prefix_cache is not None:
            self.prefix_cache.release(rp.prefix_nodes)
        self.records.clear(rp.slot)
        self._free_slots.append(rp.slot)

    # ------------------------------------------------------------------ pages
    def _first_needed_page(self, group: int, start: int) -> int:
        """The first page a query at sequence index ``start`` can still see."""
        window = self.groups[group].need.window
        if window is None:
            return 0
        return max(0, start - window + 1) // self.page_size

    def pages_missing(self, req_id, upto: int) -> List[int]:
        """Pages each group would have to hand out so that tokens ``[0, upto)`` have a place."""
        rp = self.requests[req_id]
        want = (upto + self.page_size - 1) // self.page_size
        return [max(0, want - len(t)) for t in rp.tables]

    def can_reserve(self, req_id, upto: int) -> bool:
        return all(m <= pool.num_free for m, pool in zip(self.pages_missing(req_id, upto), self.pools))

    def reserve(self, req_id, upto: int) -> None:
        """Make room for tokens ``[num_tokens, upto)`` in every group, or raise
        :class:`OutOfPages` and change nothing.  Cached prefixes nobody uses are evicted
        first if that helps."""
        rp = self.requests[req_id]
        if all(upto <= len(t) * self.page_size for t in rp.tables):
            return                       # the usual case of a decoded token: its page is there
        missing = self.pages_missing(req_id, upto)
        if self.prefix_cache is not None and any(m > pool.num_free for m, pool in zip(missing, self.pools)):
            self.prefix_cache.evict(max(missing))
        for m, pool in zip(missing, self.pools):
            if m > pool.num_free:
                raise OutOfPages(f"{m} pages wanted, {pool.num_free} free")
        for g, m in enumerate(missing):
            rp.tables[g].extend(self.pools[g].allocate(m))

    def commit(self, req_id, num_tokens: int) -> None:
        """Tokens ``[0, num_tokens)`` are now in the cache.  A windowed group gives back the
        pages no later token can see: the next query sits at index ``num_tokens`` and sees keys
        from ``num_tokens - window + 1`` on."""
        rp = self.requests[req_id]
        if num_tokens < rp.num_tokens:
            raise ValueError("a request's cached length cannot shrink")
        rp.num_tokens = num_tokens
        self.records.num_tokens[rp.slot] = num_tokens
        for g, table in enumerate(rp.tables):
            first = min(self._first_needed_page(g, num_tokens), len(table))
            gone = [p for p in table[:first] if p >= 0]
            if gone:
                self.pools[g].free(gone)
                for i in range(first):
                    table[i] = -1

    def table(self, req_id, group: int) -> List[int]:
        return self.requests[req_id].tables[group]

    def slot_mapping(self, req_id, group: int, start: int, end: int) -> List[int]:
        """Where tokens ``[start, end)`` go: ``table[p // page_size] * page_size + p % page_size``
        (reference cache.py:624-629)."""
        table = self.requests[req_id].tables[group]
        ps = self.page_size
        out = []
        for p in range(start, end):
            page = table[p // ps]
            if page < 0:
                raise RuntimeError(f"token {p} of request {req_id!r} maps to a page that was given back")
            out.append(page * ps + p % ps)
        return out

    # ------------------------------------------------------------------ forking
    def fork(self, src_id, dst_id) -> List[Tuple[int, int, int]]:
        """A new request ``dst_id`` that continues from where ``src_id`` stands (several
        continuations of one prompt).  Pages that are full are shared (one more holder each); the
        page still being filled gets a copy of its own, because both requests will write to it.
        Returns the copies the caller has to make on the device, as ``(group, from page, to page)``.
        Raises :class:`OutOfPages` / :class:`OutOfSlots` and changes nothing if there is no room."""
        src = self.requests[src_id]
        full = src.num_tokens // self.page_size
        partial = src.num_tokens % self.page_size != 0
        if partial:
            if self.prefix_cache is not None and any(pool.num_free < 1 for pool in self.pools):
                self.prefix_cache.evict(1)
            for pool in self.pools:
                if pool.num_free < 1:
                    raise OutOfPages("no page free for the copy of the page being filled")
        self.admit(dst_id)
        dst = self.requests[dst_id]
        self.records.copy(src.slot, dst.slot)
        copies: List[Tuple[int, int, int]] = []
        for g, table in enumerate(src.tables):
            shared = list(table[:full])
            self.pools[g].fork([p for p in shared if p >= 0])
            if partial:
                fresh = self.pools[g].allocate(1)[0]
                copies.append((g, table[full], fresh))
                shared.append(fresh)
            dst.tables[g] = shared
        dst.num_tokens = src.num_tokens
        if src.prefix_nodes and self.prefix_cache is not None:
            self.prefix_cache.add_users(src.prefix_nodes)
            dst.prefix_nodes = list(src.prefix_nodes)
        return copies

    # ------------------------------------------------------------------ shared prefixes
    def adopt_prefix(self, req_id, tokens: Sequence[int], extra_keys: Optional[Sequence] = None) -> int:
        """Reuse cached pages for the longest known prefix, keeping at least one token to
        compute (reference engine.py:590-614).  Returns the number of tokens adopted."""
        rp = self.requests[req_id]
        if self.prefix_cache is None or rp.num_tokens or any(rp.tables):
            return 0
        matched, nodes, pages = self.prefix_cache.match(tokens, extra_keys, max_tokens=len(tokens) - 1)
        if not matched:
            return 0
        for g, pool in enumerate(self.pools):
            pool.fork(pages[g])
            rp.tables[g] = list(pages[g])
        rp.prefix_nodes = nodes
        rp.num_tokens = matched
        self.records.num_tokens[rp.slot] = matched
        return matched

    def register_prefix(self, req_id, tokens: Sequence[int], extra_keys: Optional[Sequence] = None) -> int:
        """Offer the request's full pages of ``tokens`` to the prefix cache
        (reference engine.py:616-625)."""
        if self.prefix_cache is None:
            return 0
        rp = self.requests[req_id]
        n = min(len(tokens), rp.num_tokens) // self.page_size
        if n <= 0:
            return 0
        return self.prefix_cache.insert(tokens, [t[:n] for t in rp.tables], extra_keys)

    # ------------------------------------------------------------------ accounting
    def free_pages(self) -> List[int]:
        return [p.num_free for p in self.pools]

    def pages_in_use(self) -> List[int]:
        return [p.in_use() for p in self.pools]

    def check(self) -> None:
        """No page lost, held twice without a count, or freed twice; no slot lost."""
        for g, pool in enumerate(self.pools):
            holders: Dict[int, int] = {}
            for rp in self.requests.values():
                for p in rp.tables[g]:
                    if p >= 0:
                        holders[p] = holders.get(p, 0) + 1
            if self.prefix_cache is not None:
                for p, c in self.prefix_cache.held_pages(g).items():
                    holders[p] = holders.get(p, 0) + c
            pool.check(holders)
        slots = sorted(self._free_slots + [rp.slot for rp in self.requests.values()])
        if slots != list(range(self.max_num_seqs)):
            raise AssertionError(f"slots lost or held twice: {slots}")
