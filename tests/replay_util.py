"""Helpers that build replay traces and gather the logits they produce."""

from __future__ import annotations

import random
from typing import Dict, List, Sequence, Tuple

import torch


def round64(n: int) -> int:
    return (n + 63) // 64 * 64


def random_tokens(n: int, vocab: int, seed: int) -> List[int]:
    g = torch.Generator().manual_seed(seed)
    return torch.randint(0, vocab, (n,), generator=g).tolist()


def whole_trace(requests: Dict[str, List[int]]) -> List[dict]:
    """Each request alone, in one step, every place wanted."""
    return [{"step": i, "entries": [{"id": rid, "tokens": toks, "want": list(range(len(toks)))}], "end": [rid]}
            for i, (rid, toks) in enumerate(requests.items())]


def tail_trace(requests: Dict[str, List[int]], tail: int = 32) -> List[dict]:
    """All but the last `tail` tokens in one step, then one token a step."""
    steps, n = [], 0
    for rid, toks in requests.items():
        head = max(1, len(toks) - tail)
        steps.append({"step": n, "entries": [{"id": rid, "tokens": toks[:head], "want": list(range(head))}],
                      "end": []})
        n += 1
        for p in range(head, len(toks)):
            steps.append({"step": n, "entries": [{"id": rid, "tokens": [toks[p]], "want": [0]}],
                          "end": [rid] if p == len(toks) - 1 else []})
            n += 1
        if head == len(toks):
            steps[-1]["end"] = [rid]
    return steps


def portion_trace(requests: Dict[str, List[int]], sizes: Sequence[int] = (7, 2, 13, 5, 2, 31, 3, 16, 2, 9)) -> List[dict]:
    """Portions of changing size, down to two tokens, not aligned to pages."""
    steps, n = [], 0
    for rid, toks in requests.items():
        at, k = 0, 0
        while at < len(toks):
            size = min(sizes[k % len(sizes)], len(toks) - at)
            k += 1
            steps.append({"step": n, "entries": [{"id": rid, "tokens": toks[at:at + size],
                                                  "want": list(range(size))}],
                          "end": [rid] if at + size == len(toks) else []})
            at += size
            n += 1
    return steps


def mixed_trace(requests: Dict[str, List[int]], seed: int = 0, max_live: int = 4,
                prompt_frac: float = 0.6) -> Tuple[List[dict], int]:
    """Up to `max_live` requests at a time: the first part of each (its "prompt") arrives in
    portions of random size, the rest one token a step, portions of some beside single tokens of
    others; a request may sit out a step.  Returns the steps and the most tokens live requests
    hold at any time (each rounded up to 64), which is what the page pool is made for."""
    rng = random.Random(seed)
    waiting = list(requests.items())
    live: Dict[str, dict] = {}
    steps, n, peak = [], 0, 0
    while waiting or live:
        while waiting and len(live) < max_live:
            rid, toks = waiting.pop(0)
            live[rid] = {"toks": toks, "at": 0, "prompt": max(1, int(len(toks) * prompt_frac))}
        entries, end = [], []
        for rid, st in list(live.items()):
            if len(live) > 1 and rng.random() < 0.15:
                continue  # sits this step out
            left_prompt = st["prompt"] - st["at"]
            if left_prompt > 0:
                size = min(left_prompt, rng.choice([2, 3, 5, 8, 13, 21, 40]))
                if left_prompt - size == 1:
                    size += 1
            else:
                size = 1
            size = min(size, len(st["toks"]) - st["at"])
            entries.append({"id": rid, "tokens": st["toks"][st["at"]:st["at"] + size], "want": list(range(size))})
            st["at"] += size
            if st["at"] == len(st["toks"]):
                end.append(rid)
        if not entries:
            continue
        rng.shuffle(entries)
        peak = max(peak, sum(round64(st["at"]) for st in live.values()))
        steps.append({"step": n, "entries": entries, "end": end})
        n += 1
        for rid in end:
            del live[rid]
    return steps, peak


def run_steps(replayer, steps: List[dict], holders: Dict[Tuple[int, int], set] = None,
              at: Dict[str, int] = None) -> Dict[Tuple[str, int], torch.Tensor]:
    """Replay and return {(request, index in its sequence): logits row} on the host.  ``holders``,
    if given, collects for every (cache group, page) the requests that held it at some time.
    ``at`` (request -> tokens fed so far) lets a caller replay a trace in several calls."""
    at = {} if at is None else at
    out: Dict[Tuple[str, int], torch.Tensor] = {}
    cache = replayer.runner.cache
    for rec in steps:
        if holders is not None:
            # pages are handed out when the step runs and given back when a request ends: look before the ends
            ends, rec = rec.get("end", []), dict(rec, end=[])
        logits = replayer.step(rec)
        if holders is not None:
            for e in rec["entries"]:
                for g in range(len(cache.groups)):
                    for page in cache.table(e["id"], g):
                        if page >= 0:
                            holders.setdefault((g, int(page)), set()).add(e["id"])
            if ends:
                replayer.step({"entries": [], "end": ends})
        rows = logits.float().cpu() if logits is not None else None
        k = 0
        for e in rec["entries"]:
            base = at.get(e["id"], 0)
            for w in e.get("want", []):
                out[(e["id"], base + w)] = rows[k]
                k += 1
            at[e["id"]] = base + len(e["tokens"])
        assert rows is None or k == rows.shape[0]
    return out
