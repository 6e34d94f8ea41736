"""Prefix cache: a tree over whole pages of tokens
(reference src/qwen25vl_lite/cache.py:94-274).

A node stands for one full page of a prompt and holds the page ids (one per cache group)
whose keys and values were computed for exactly that token prefix.  The cache holds one
reference to each of its pages, taken when the node is made and dropped when it is evicted;
a node's ``users`` counts the live requests that adopted it and decides only whether it may
be evicted.  A trailing partial page is never cached: what it will hold depends on tokens
that follow.  Besides the reference's limit on the number of nodes, nodes are also evicted
when the pools run short (oldest unused leaves first), before any request is preempted.
"""

from __future__ import annotations

from dataclasses import dataclass, field
from typing import Dict, List, Optional, Sequence, Tuple

from .pages import PagePool

__all__ = ["RadixPrefixCache"]


@dataclass
class _Node:
    key: Tuple
    pages: Tuple[int, ...]            # one page id per cache group
    parent: int
    children: Dict[Tuple, int] = field(default_factory=dict)
    last_used: int = 0
    users: int = 0


class RadixPrefixCache:
    ROOT = -1

    def __init__(self, pools: Sequence[PagePool], page_size: int, max_nodes: int = 4096):
        self.pools = list(pools)
        self.page_size = int(page_size)
        self.max_nodes = int(max_nodes)
        self.nodes: Dict[int, _Node] = {self.ROOT: _Node(key=(), pages=(), parent=self.ROOT)}
        self._next_id = 0
        self._clock = 0
        self.hits = 0
        self.misses = 0

    def __len__(self) -> int:
        return len(self.nodes) - 1

    def _tick(self) -> int:
        self._clock += 1
        return self._clock

    def _key(self, tokens: Sequence[int], i: int, extra_keys: Optional[Sequence]) -> Tuple:
        page = tuple(int(t) for t in tokens[i * self.page_size:(i + 1) * self.page_size])
        extra = extra_keys[i] if extra_keys is not None and i < len(extra_keys) else None
        return page if extra is None else (("extra", extra),) + page

    def match(self, tokens: Sequence[int], extra_keys: Optional[Sequence] = None,
              max_tokens: Optional[int] = None) -> Tuple[int, List[int], List[List[int]]]:
        """Longest cached prefix of whole pages, at most ``max_tokens`` long.

        Returns ``(matched_tokens, node_ids, pages_per_group)`` and counts the caller as a user
        of the matched nodes (give them back with :meth:`release`).
        """
        limit = len(tokens) if max_tokens is None else min(len(tokens), max_tokens)
        node_id = self.ROOT
        path: List[int] = []
        i = 0
        while (i + 1) * self.page_size <= limit:
            nxt = self.nodes[node_id].children.get(self._key(tokens, i, extra_keys))
            if nxt is None:
                break
            path.append(nxt)
            node_id = nxt
            i += 1
        now = self._tick()
        for nid in path:
            self.nodes[nid].users += 1
            self.nodes[nid].last_used = now
        if path:
            self.hits += 1
        else:
            self.misses += 1
        pages = [[self.nodes[nid].pages[g] for nid in path] for g in range(len(self.pools))]
        return len(path) * self.page_size, path, pages

    def add_users(self, node_ids: Sequence[int]) -> None:
        """One more request uses these nodes (a fork of a request that adopted them)."""
        for nid in node_ids:
            self.nodes[nid].users += 1

    def release(self, node_ids: Sequence[int]) -> None:
        """A request that adopted these nodes is done with them."""
        for nid in node_ids:
            node = self.nodes.get(nid)
            if node is not None and node.users > 0:
                node.users -= 1

    def insert(self, tokens: Sequence[int], pages_per_group: Sequence[Sequence[int]],
               extra_keys: Optional[Sequence] = None) -> int:
        """Register the first ``n`` whole pages of ``tokens`` (``n`` = pages given per group).
        Returns the number of new nodes.  The registering request does not become a user."""
        if len(pages_per_group) != len(self.pools):
            raise ValueError("one page list per cache group is needed")
        n = len(pages_per_group[0]) if pages_per_group else 0
        if any(len(p) != n for p in pages_per_group):
            raise ValueError("the groups' page lists differ in length")
        if len(tokens) < n * self.page_size:
            raise ValueError("fewer tokens than pages supplied")
        node_id = self.ROOT
        made = 0
        now = self._tick()
        for i in range(n):
            key = self._key(tokens, i, extra_keys)
            node = self.nodes[node_id]
            child = node.children.get(key)
            if child is None:
                pages = tuple(int(pages_per_group[g][i]) for g in range(len(self.pools)))
                for g, pool in enumerate(self.pools):
                    pool.fork([pages[g]])
                child = self._next_id
                self._next_id += 1
                self.nodes[child] = _Node(key=key, pages=pages, parent=node_id, last_used=now)
                node.children[key] = child
                made += 1
            else:
                self.nodes[child].last_used = now
            node_id = child
        self._evict_over_budget()
        return made

    # ------------------------------------------------------------------ eviction
    def _drop(self, nid: int) -> int:
        """Remove a node and all below it; returns the pages given back per group (count)."""
        parent = self.nodes[self.nodes[nid].parent]
        parent.children.pop(self.nodes[nid].key, None)
        stack, dropped = [nid], 0
        while stack:
            cur = self.nodes.pop(stack.pop())
            stack.extend(cur.children.values())
            for g, pool in enumerate(self.pools):
                pool.free([cur.pages[g]])
            dropped += 1
        return dropped

    def _evictable_leaves(self) -> List[int]:
        return sorted((nid for nid, n in self.nodes.items()
                       if nid != self.ROOT and not n.children and n.users == 0),
                      key=lambda nid: self.nodes[nid].last_used)

    def _evict_over_budget(self) -> None:
        while len(self) > self.max_nodes:
            leaves = self._evictable_leaves()
            if not leaves:
                return
            self._drop(leaves[0])

    def evict(self, pages_wanted: int) -> int:
        """Evict unused leaves, oldest first, until every pool has ``pages_wanted`` free pages or
        no leaf is left whose eviction would free a page.  A leaf whose pages a running request
        still holds (the one that registered it) stays: dropping it would give nothing back and
        only lose the entry.  Returns the number of nodes evicted."""
        evicted = 0
        while any(pool.num_free < pages_wanted for pool in self.pools):
            leaves = [nid for nid in self._evictable_leaves()
                      if any(pool.refcount(self.nodes[nid].pages[g]) == 1 for g, pool in enumerate(self.pools))]
            if not leaves:
                break
            evicted += self._drop(leaves[0])
        return evicted

    def clear(self) -> int:
        """Forget every entry that no running request uses (leaves first, so whole unused branches
        go); their pages return to the pools unless a request still holds them.  Returns the number
        of nodes dropped."""
        dropped = 0
        while True:
            leaves = self._evictable_leaves()
            if not leaves:
                return dropped
            for nid in leaves:
                dropped += self._drop(nid)

    def held_pages(self, group: int) -> Dict[int, int]:
        out: Dict[int, int] = {}
        for nid, node in self.nodes.items():
            if nid != self.ROOT:
                out[node.pages[group]] = out.get(node.pages[group], 0) + 1
        return out

    def stats(self) -> Dict[str, float]:
        total = self.hits + self.misses
        return {"hits": self.hits, "misses": self.misses, "hit_rate": self.hits / total if total else 0.0,
                "nodes": len(self)}
