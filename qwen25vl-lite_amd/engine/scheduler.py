"""The scheduler: admits requests, cuts prompts into portions under a token budget, decodes,
finishes and frees (reference src/qwen25vl_lite/engine.py:489-937).

Each step builds ONE batch for the step function: first the single next tokens of requests
that are decoding, then further portions of prompts already admitted, then portions of newly
admitted prompts, all under ``max_num_batched_tokens`` (decoded tokens count).  The reference
runs a prompt portion per request and a separate batched decode instead (engine.py:741-808).

A request is a list of tokens (prompt, then what it generated) of which a prefix is in the
cache.  Whatever is not yet in the cache is run next; when a portion reaches the end of the
list, the logits of its last place are sampled and the token appended.  Decoding is the case
of one token left.

When pages run out, unused cached prefixes are evicted first; then the running request of
lowest priority, newest first, is preempted (reference engine.py:700-720): it gives every page
back, returns to the front of the waiting queue and is later prefilled again, prompt and the
tokens it had generated, from which it continues (only "recompute" is built; the reference's
own recompute forgets the generated tokens' keys, engine.py:713-718).  A request that cannot
get pages while it is the only one running can never finish: that raises.
"""

from __future__ import annotations

import time
from collections import deque
from dataclasses import dataclass, field
from typing import Deque, Dict, List, Optional, Sequence, Tuple

from ..cache import OutOfPages
from ..config.engine_config import EngineConfig
from ..sampling.params import SamplingParams
from .batch import StepEntry

__all__ = ["LLMEngine", "RequestOutput", "EngineStats", "Sequence_"]


@dataclass
class RequestOutput:
    """What the caller gets back for a finished request (reference engine.py:96-112)."""

    seq_id: int
    prompt_token_ids: List[int]
    output_token_ids: List[int]
    finish_reason: str
    metrics: Dict[str, float] = field(default_factory=dict)

    @property
    def num_prompt_tokens(self) -> int:
        return len(self.prompt_token_ids)

    @property
    def num_output_tokens(self) -> int:
        return len(self.output_token_ids)


@dataclass
class EngineStats:
    """Counters (reference engine.py:122-137, without the vision and swap counters)."""

    steps: int = 0
    prefill_chunks: int = 0
    decode_tokens: int = 0
    batched_tokens: int = 0
    preemptions: int = 0
    prefix_cache_hits: int = 0
    prefix_cache_tokens_saved: int = 0


@dataclass(eq=False)
class Sequence_:
    """A request in flight (reference cache.py:584-629).  Two requests are the same only if they
    are the same object (membership tests in the queues compare identities, not fields)."""

    seq_id: int
    prompt_token_ids: List[int]
    params: SamplingParams
    priority: int = 0
    output_token_ids: List[int] = field(default_factory=list)
    num_computed_tokens: int = 0
    cached_tokens: int = 0
    prompt_positions: Optional[List[List[int]]] = None   # [rows][prompt length], None = text
    rope_delta: int = 0
    slot: int = -1                                       # its slot while it is running (see cache.SlotRecords)
    prefix_keys: Optional[List] = None
    arrival: float = field(default_factory=time.time)
    first_token_at: Optional[float] = None
    status: str = "waiting"

    @property
    def tokens(self) -> List[int]:
        return self.prompt_token_ids + self.output_token_ids

    @property
    def num_tokens(self) -> int:
        return len(self.prompt_token_ids) + len(self.output_token_ids)

    @property
    def remaining(self) -> int:
        return self.num_tokens - self.num_computed_tokens


class LLMEngine:
    """Iteration-level scheduler above a runner (``runner.cache``, ``runner.execute``,
    ``runner.sample``, ``runner.vocab_size``, ``runner.eos_token_id``)."""

    def __init__(self, runner, engine_cfg: Optional[EngineConfig] = None):
        self.runner = runner
        self.ecfg = engine_cfg or runner.ecfg
        self.waiting: Deque[Sequence_] = deque()
        self.running: List[Sequence_] = []
        self.stats_ = EngineStats()
        self._next_id = 0
        self._finished_total = 0
        self._ahead: Optional[Tuple[List[Tuple[Sequence_, int]], List[StepEntry], object]] = None
        self.position_rows = getattr(runner, "position_rows", 3)

    # ------------------------------------------------------------------ requests
    def add_request(self, prompt_token_ids: Sequence[int], sampling_params: Optional[SamplingParams] = None, *,
                    position_ids: Optional[Sequence[Sequence[int]]] = None, rope_delta: Optional[int] = None,
                    priority: int = 0) -> int:
        """Register a request and return its id (reference engine.py:507-588).

        ``position_ids`` gives explicit position rows ``[rows][len(prompt)]`` (the reference
        derives them from image grids, engine.py:554-562); the tokens generated after the prompt
        sit at ``index + rope_delta`` on every row, ``rope_delta`` defaulting to
        ``max(position) + 1 - len(prompt)`` (reference rope.py:233)."""
        params = sampling_params or SamplingParams()
        params.validate()
        if params.stop:
            # reference engine.py:518-525
            raise ValueError("string stop sequences need a tokenizer, which the engine does not have; "
                             "use stop_token_ids")
        ids = [int(t) for t in prompt_token_ids]
        if not ids:
            raise ValueError("prompt is empty")
        if len(ids) > self.ecfg.max_model_len:
            raise ValueError(f"prompt of {len(ids)} tokens exceeds max_model_len {self.ecfg.max_model_len}")
        vocab = self.runner.vocab_size
        if min(ids) < 0 or max(ids) >= vocab:
            raise ValueError(f"prompt holds a token id outside [0, {vocab})")
        if not self.ecfg.enable_chunked_prefill and len(ids) > self.ecfg.max_num_batched_tokens:
            raise ValueError(f"prompt of {len(ids)} tokens cannot run in one step of "
                             f"{self.ecfg.max_num_batched_tokens} tokens and chunked prefill is off")
        seq = Sequence_(seq_id=self._next_id, prompt_token_ids=ids, params=params, priority=int(priority))
        if position_ids is not None:
            rows = [[int(p) for p in row] for row in position_ids]
            if len(rows) != self.position_rows or any(len(r) != len(ids) for r in rows):
                raise ValueError(f"position_ids must be [{self.position_rows}][{len(ids)}]")
            seq.prompt_positions = rows
            seq.rope_delta = int(rope_delta) if rope_delta is not None else max(max(r) for r in rows) + 1 - len(ids)
            ps = self.ecfg.block_size
            seq.prefix_keys = [tuple(tuple(r[i * ps:(i + 1) * ps]) for r in rows) for i in range(len(ids) // ps)]
        elif rope_delta is not None:
            seq.rope_delta = int(rope_delta)
            if seq.rope_delta:  # shifted text positions: not the keys an unshifted prompt computed
                seq.prefix_keys = [("delta", seq.rope_delta)] * (len(ids) // self.ecfg.block_size)
        self._next_id += 1
        self.waiting.append(seq)
        return seq.seq_id

    def has_work(self) -> bool:
        return bool(self.waiting or self.running)

    # ------------------------------------------------------------------ scheduling
    def _victim(self) -> Optional[Sequence_]:
        if not self.running:
            return None
        return min(self.running, key=lambda s: (s.priority, -s.seq_id))

    def _preempt(self, victim: Sequence_) -> None:
        self.running.remove(victim)
        self.runner.cache.release(victim.seq_id)
        victim.slot = -1
        victim.num_computed_tokens = 0
        victim.cached_tokens = 0
        victim.status = "waiting"
        self.waiting.appendleft(victim)
        self.stats_.preemptions += 1

    def _reserve(self, seq: Sequence_, upto: int, plan: List[Tuple[Sequence_, int]]) -> bool:
        """Get pages for ``seq`` up to ``upto`` tokens, preempting others if needed.  False if
        ``seq`` itself had to give way."""
        cache = self.runner.cache
        while True:
            try:
                cache.reserve(seq.seq_id, upto)
                return True
            except OutOfPages:
                victim = self._victim()
                if victim is None or (victim is seq and len(self.running) == 1):
                    raise OutOfPages(
                        f"request {seq.seq_id} needs pages for {upto} tokens but the pool cannot hold them even "
                        f"with every other request preempted ({cache.free_pages()} pages free)") from None
                self._preempt(victim)
                plan[:] = [(s, n) for s, n in plan if s is not victim]
                if victim is seq:
                    return False

    def _portion(self, seq: Sequence_, budget: int) -> int:
        """How many of the request's next tokens run this step.  Without chunked prefill it is all
        or nothing (reference engine.py:649-654), unless they could never fit a step at all (a
        preempted request that has grown past the budget)."""
        whole_fits_some_step = seq.remaining <= self.ecfg.max_num_batched_tokens
        if self.ecfg.enable_chunked_prefill or seq.remaining <= budget or not whole_fits_some_step:
            return min(seq.remaining, budget)
        return 0

    def _schedule(self) -> List[Tuple[Sequence_, int]]:
        """Decide this step's batch: ``[(sequence, number of its next tokens)]``."""
        budget = self.ecfg.max_num_batched_tokens
        plan: List[Tuple[Sequence_, int]] = []
        # 1. decoding requests (one token left), then 2. prompts already admitted
        for decoding in (True, False):
            for seq in list(self.running):
                # a request earlier in this loop may have preempted this one
                if seq.status != "running" or (seq.remaining == 1) != decoding or budget <= 0:
                    continue
                n = self._portion(seq, budget)
                if n <= 0:
                    continue
                if self._reserve(seq, seq.num_computed_tokens + n, plan):
                    plan.append((seq, n))
                    budget -= n
        # 3. new requests, in arrival order, never past the head of the queue.  A newcomer never
        # preempts: it waits until pages are free (cached prefixes nobody uses go first).
        cache = self.runner.cache
        while self.waiting and len(self.running) < self.ecfg.max_num_seqs and budget > 0:
            seq = self.waiting[0]
            n = self._portion(seq, budget)
            if n <= 0:
                break
            # the slot's record: sampling settings, rope delta, tokens generated before a preemption
            seq.slot = cache.admit(seq.seq_id, seq.params, seq.rope_delta, len(seq.output_token_ids))
            adopted = 0
            if self.ecfg.enable_prefix_cache:
                adopted = cache.adopt_prefix(seq.seq_id, seq.tokens, seq.prefix_keys)
                n = min(n, seq.num_tokens - adopted)
            try:
                cache.reserve(seq.seq_id, adopted + n)
            except OutOfPages:
                cache.release(seq.seq_id)
                seq.slot = -1
                if not self.running:
                    raise OutOfPages(f"request {seq.seq_id} cannot get pages for its first {adopted + n} tokens "
                                     "although nothing else is running") from None
                break
            if adopted:
                seq.num_computed_tokens = seq.cached_tokens = adopted
                self.stats_.prefix_cache_hits += 1
                self.stats_.prefix_cache_tokens_saved += adopted
            self.waiting.popleft()
            seq.status = "running"
            self.running.append(seq)
            plan.append((seq, n))
            budget -= n
        return plan

    def _entry(self, seq: Sequence_, n: int) -> StepEntry:
        start = seq.num_computed_tokens
        p_len = len(seq.prompt_token_ids)
        if start >= p_len:
            tokens = seq.output_token_ids[start - p_len:start - p_len + n]
        else:
            tokens = seq.tokens[start:start + n]
        positions = None
        if seq.prompt_positions is not None and start < len(seq.prompt_token_ids):
            p_len = len(seq.prompt_token_ids)
            positions = []
            for row in seq.prompt_positions:
                part = row[start:min(start + n, p_len)]
                part += [i + seq.rope_delta for i in range(p_len, start + n)]
                positions.append(part)
        want = [n - 1] if start + n == seq.num_tokens else []
        return StepEntry(req_id=seq.seq_id, tokens=tokens, start=start, want=want, positions=positions,
                         rope_delta=seq.rope_delta)

    # ------------------------------------------------------------------ stepping
    def step(self) -> List[RequestOutput]:
        """One scheduling iteration; returns the requests that finished in it."""
        done: List[RequestOutput] = []
        ahead, self._ahead = self._ahead, None
        if ahead is not None and not any(seq.status == "running" for seq, _ in ahead[0]):
            ahead = None                       # everyone in the step queued ahead has finished since
        if ahead is not None:
            plan, entries, logits = ahead      # queued by the step before (see _queue_ahead)
            self.stats_.steps += 1
        else:
            plan = self._schedule()
            self.stats_.steps += 1
            if not plan:
                return done
            entries = [self._entry(seq, n) for seq, n in plan]
            logits = self.runner.execute(entries)
        sampled: List[Sequence_] = []
        rows: List[int] = []
        for row, ((seq, n), entry) in enumerate(zip(plan, entries)):
            if seq.status != "running":
                continue   # it finished after this step was queued ahead: its row is computed for nothing
            rows.append(row)
            was_prompt = seq.num_computed_tokens < len(seq.prompt_token_ids)
            seq.num_computed_tokens += n
            self.stats_.batched_tokens += n
            if n == 1 and not was_prompt:
                self.stats_.decode_tokens += 1
            else:
                self.stats_.prefill_chunks += 1
            if was_prompt and seq.num_computed_tokens >= len(seq.prompt_token_ids) and self.ecfg.enable_prefix_cache:
                self.runner.cache.register_prefix(seq.seq_id, seq.prompt_token_ids, seq.prefix_keys)
            if entry.want:
                sampled.append(seq)
        if sampled:
            if ahead is not None and len(rows) < len(plan):
                logits = logits[rows]          # every entry of a step queued ahead wants one row
            prev = [s.output_token_ids for s in sampled]
            by_slot = hasattr(self.runner, "sample_slots_begin")   # settings and sampler state from the slot records
            if by_slot:
                pending = self.runner.sample_slots_begin(logits, [s.slot for s in sampled], prev)
            else:
                args = ([s.params for s in sampled], prev, [len(p) for p in prev])
            if self._may_look_ahead(plan, sampled):
                if not by_slot:
                    pending = self.runner.sample_begin(logits, *args)
                self._queue_ahead(sampled, pending)
                tokens = pending.result()
            elif by_slot:
                tokens = pending.result()
            else:
                tokens = self.runner.sample(logits, *args)
            for seq, token in zip(sampled, tokens):
                self._accept(seq, int(token), done)
        self._finished_total += len(done)
        return done

    # ------------------------------------------------------------------ looking one step ahead
    def _may_look_ahead(self, plan: List[Tuple[Sequence_, int]], sampled: List[Sequence_]) -> bool:
        """Whether the step after this one can be queued before this one's tokens are known: it is a
        decode step of exactly the requests sampled now (nobody waits for admission, nobody is left
        out or still in its prompt), and no request's sampling reads the tokens it generated."""
        if not (self.ecfg.hip_graph and self.ecfg.decode_lookahead and hasattr(self.runner, "sample_begin")):
            return False
        if self.waiting or len(sampled) != len(self.running):
            return False
        return all(s.params.repetition_penalty == 1.0 and s.params.presence_penalty == 0.0
                   and s.params.frequency_penalty == 0.0 for s in sampled)

    def _queue_ahead(self, sampled: List[Sequence_], pending) -> None:
        """Queue the next decode step on the GPU.  Its token ids are the ones being sampled, taken
        on the device.  Requests that are known to end with this token (length) are left out; one
        that ends on a stop token is found out only afterwards: its row of the queued step is then
        computed for nothing and ignored, and what it writes lands in pages that are free again,
        before any later step's own writes to them.  Nothing else differs from scheduling the
        step afterwards: rows do not depend on each other."""
        keep = [i for i, s in enumerate(sampled)
                if len(s.output_token_ids) + 1 < s.params.max_tokens and s.num_tokens + 1 < self.ecfg.max_model_len]
        if not keep or len(keep) > self.ecfg.max_num_batched_tokens:
            return
        cache = self.runner.cache
        seqs = [sampled[i] for i in keep]
        entries = [StepEntry(req_id=s.seq_id, tokens=[0], start=s.num_computed_tokens, want=[0], positions=None,
                             rope_delta=s.rope_delta) for s in seqs]
        if not self.runner.decodes_from_graph(entries):
            return
        try:
            for s in seqs:
                cache.reserve(s.seq_id, s.num_computed_tokens + 1)
        except OutOfPages:
            return      # the scheduler decides who gives way, with the tokens known
        ids = pending.device_ids
        if len(keep) < len(sampled):
            ids = ids[keep]
        logits = self.runner.execute(entries, device_tokens=ids)
        self._ahead = ([(s, 1) for s in seqs], entries, logits)

    def _accept(self, seq: Sequence_, token: int, done: List[RequestOutput]) -> None:
        """Append a sampled token and finish the request if it must (reference engine.py:831-872)."""
        params = seq.params
        seq.output_token_ids.append(token)
        self.runner.cache.records.generated[seq.slot] += 1     # the sampler's state moves on with the token
        if seq.first_token_at is None:
            seq.first_token_at = time.time()
        reason: Optional[str] = None
        eos = self.runner.eos_token_id
        if eos is not None and token == eos and not params.ignore_eos:
            reason = "stop"
        elif token in set(params.stop_token_ids or ()):
            reason = "stop"
        elif len(seq.output_token_ids) >= params.max_tokens:
            reason = "length"
        elif seq.num_tokens >= self.ecfg.max_model_len:
            reason = "length"
        if reason is None:
            return
        seq.status = "finished"
        self.runner.cache.release(seq.seq_id)
        seq.slot = -1
        self.running.remove(seq)
        now = time.time()
        done.append(RequestOutput(
            seq_id=seq.seq_id,
            prompt_token_ids=list(seq.prompt_token_ids),
            output_token_ids=list(seq.output_token_ids),
            finish_reason=reason,
            metrics={
                "cached_tokens": float(seq.cached_tokens),
                "prompt_tokens": float(len(seq.prompt_token_ids)),
                "completion_tokens": float(len(seq.output_token_ids)),
                "ttft_s": max(0.0, (seq.first_token_at or now) - seq.arrival),
                "elapsed_s": now - seq.arrival,
            }))

    # ------------------------------------------------------------------ driver
    def run_until_complete(self, max_steps: int = 100_000, max_stall: int = 64) -> List[RequestOutput]:
        """Drive the engine until every request has finished; raise if the scheduler spins
        without computing anything (reference engine.py:878-914).  Returns the requests that finished
        during this call (the engine keeps no list of them: a caller that drives :meth:`step` itself
        gets each step's own)."""
        steps = stall = 0
        finished: List[RequestOutput] = []
        last = self._progress()
        while self.has_work() and steps < max_steps:
            finished.extend(self.step())
            steps += 1
            now = self._progress()
            if now == last:
                stall += 1
                if stall >= max_stall:
                    raise RuntimeError(f"scheduler made no progress for {max_stall} steps "
                                       f"(waiting={len(self.waiting)} running={len(self.running)})")
            else:
                stall, last = 0, now
        if self.has_work():
            raise RuntimeError(f"engine did not finish within {max_steps} steps")
        return finished

    def _progress(self) -> tuple:
        return (len(self.waiting), len(self.running), self._finished_total, self.stats_.batched_tokens,
                self.stats_.preemptions)

    def stats(self) -> Dict[str, float]:
        """A flat dictionary of counters (reference engine.py:916-937)."""
        out = {k: float(v) for k, v in vars(self.stats_).items()}
        cache = self.runner.cache
        out.update({
            "waiting": float(len(self.waiting)),
            "running": float(len(self.running)),
            "kv_blocks_used": float(max(cache.pages_in_use(), default=0)),
            "kv_blocks_total": float(self.ecfg.num_blocks),
        })
        if cache.prefix_cache is not None:
            out["prefix_hit_rate"] = cache.prefix_cache.stats()["hit_rate"]
        return out
