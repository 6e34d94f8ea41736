"""The scheduler's decisions, with a runner that computes nothing (no GPU).

The fake runner keeps the real cache manager, checks every batch the scheduler hands it
against the cache, and answers with logits that make token ``(last token + 1) % vocab`` the
argmax, so that what a request generates tells which tokens it was fed.
"""

import pytest
import torch

from qwen25vl_lite_amd.cache import CacheGroupSpec, CacheManager, OutOfPages
from qwen25vl_lite_amd.config import EngineConfig
from qwen25vl_lite_amd.engine.scheduler import LLMEngine
from qwen25vl_lite_amd.parts import CacheNeed
from qwen25vl_lite_amd.sampling import SamplingParams

VOCAB = 50


class FakeRunner:
    position_rows = 3

    def __init__(self, ecfg, windows=(None,), eos=None):
        self.ecfg = ecfg
        self.vocab_size = VOCAB
        self.eos_token_id = eos
        groups = [CacheGroupSpec(CacheNeed(1, 8, w), 1) for w in windows]
        self.cache = CacheManager(groups, ecfg.num_blocks, ecfg.block_size, ecfg.max_num_seqs,
                                  enable_prefix_cache=ecfg.enable_prefix_cache)
        self.batches = []
        self.ahead_steps = 0

    def decodes_from_graph(self, entries):
        return bool(self.ecfg.hip_graph) and all(len(e.tokens) == 1 and e.positions is None and list(e.want) == [0]
                                                 for e in entries)

    def sample_begin(self, logits, params, prev_ids, steps):
        ids = self.sample(logits, params, prev_ids, steps)

        class Pending:
            device_ids = torch.tensor(ids, dtype=torch.int32)

            @staticmethod
            def result():
                return ids
        return Pending

    def execute(self, entries, device_tokens=None):
        if device_tokens is not None:
            # a step queued ahead: its token ids are still "on the device"
            assert self.decodes_from_graph(entries) and len(device_tokens) == len(entries)
            self.ahead_steps += 1
            entries = [type(e)(req_id=e.req_id, tokens=[int(t)], start=e.start, want=e.want, positions=e.positions,
                               rope_delta=e.rope_delta) for e, t in zip(entries, device_tokens)]
        rows = []
        total = 0
        seen = set()
        for e in entries:
            assert e.req_id not in seen
            seen.add(e.req_id)
            assert self.cache.num_tokens(e.req_id) == e.start, "a portion must continue where the cache ends"
            self.cache.reserve(e.req_id, e.start + len(e.tokens))
            for g in range(len(self.cache.groups)):
                self.cache.slot_mapping(e.req_id, g, e.start, e.start + len(e.tokens))  # every token has a place
            total += len(e.tokens)
            for w in e.want:
                row = torch.zeros(VOCAB)
                row[(e.tokens[w] + 1) % VOCAB] = 5.0
                rows.append(row)
        assert total <= self.ecfg.max_num_batched_tokens
        assert len(entries) <= self.ecfg.max_num_seqs
        self.batches.append([(e.req_id, e.start, len(e.tokens), list(e.want), e.positions) for e in entries])
        for e in entries:
            self.cache.commit(e.req_id, e.start + len(e.tokens))
        self.cache.check()
        return torch.stack(rows) if rows else torch.zeros(0, VOCAB)

    def sample(self, logits, params, prev_ids, steps):
        assert all(len(p) == s for p, s in zip(prev_ids, steps))
        return [int(torch.argmax(row)) for row in logits]


def _engine(**kw):
    windows = kw.pop("windows", (None,))
    eos = kw.pop("eos", None)
    base = dict(num_blocks=64, block_size=16, max_num_seqs=4, max_num_batched_tokens=64, max_model_len=512,
                dtype="float32")
    base.update(kw)
    ecfg = EngineConfig(**base)
    runner = FakeRunner(ecfg, windows, eos)
    return LLMEngine(runner, ecfg), runner


def _expected(prompt, n):
    out, last = [], prompt[-1]
    for _ in range(n):
        last = (last + 1) % VOCAB
        out.append(last)
    return out


def test_greedy_generation_and_finish():
    eng, runner = _engine()
    sid = eng.add_request([3, 4, 5], SamplingParams(max_tokens=8, ignore_eos=True))
    outs = eng.run_until_complete()
    assert [o.seq_id for o in outs] == [sid]
    assert outs[0].output_token_ids == _expected([3, 4, 5], 8) and outs[0].finish_reason == "length"
    assert outs[0].metrics["prompt_tokens"] == 3 and outs[0].metrics["completion_tokens"] == 8
    # the prompt in one portion, then one token a step
    assert [b[0][2] for b in runner.batches] == [3] + [1] * 7
    assert runner.cache.pages_in_use() == [0] and not eng.has_work()


def test_long_prompt_is_cut_under_the_budget():
    # reference tests/test_engine.py:211-217: 64 tokens, 16 a step -> at least 4 portions
    eng, runner = _engine(max_num_batched_tokens=16, enable_prefix_cache=False)
    prompt = [(7 + i) % VOCAB for i in range(64)]
    eng.add_request(prompt, SamplingParams(max_tokens=2, ignore_eos=True))
    outs = eng.run_until_complete()
    assert [b[0][2] for b in runner.batches[:4]] == [16] * 4
    assert [b[0][3] for b in runner.batches[:4]] == [[], [], [], [15]], "only the last portion wants logits"
    assert outs[0].output_token_ids == _expected(prompt, 2)
    assert eng.stats()["prefill_chunks"] == 4


def test_decode_tokens_come_first_and_count_against_the_budget():
    eng, runner = _engine(max_num_batched_tokens=20, enable_prefix_cache=False)
    a = eng.add_request([1] * 10, SamplingParams(max_tokens=6, ignore_eos=True))
    eng.step()                       # a's prompt
    b = eng.add_request([2] * 50, SamplingParams(max_tokens=2, ignore_eos=True))
    eng.step()
    batch = runner.batches[-1]
    assert [(rid, n) for rid, _, n, _, _ in batch] == [(a, 1), (b, 19)], "decoded token first, then 19 of the prompt"
    eng.step()
    assert [(rid, n) for rid, _, n, _, _ in runner.batches[-1]] == [(a, 1), (b, 19)]
    outs = eng.run_until_complete()
    assert sorted(o.seq_id for o in outs) == [a, b]


def test_admission_respects_max_num_seqs_and_order():
    eng, runner = _engine(max_num_seqs=2, enable_prefix_cache=False)
    ids = [eng.add_request([i + 1] * 5, SamplingParams(max_tokens=3, ignore_eos=True)) for i in range(4)]
    eng.step()
    assert [rid for rid, *_ in runner.batches[-1]] == ids[:2]
    outs = eng.run_until_complete()
    assert sorted(o.seq_id for o in outs) == ids
    first_seen = {}
    for i, batch in enumerate(runner.batches):
        for rid, *_ in batch:
            first_seen.setdefault(rid, i)
    assert first_seen[ids[2]] <= first_seen[ids[3]] and first_seen[ids[2]] > first_seen[ids[1]]
    assert all(len(b) <= 2 for b in runner.batches)


def test_stop_reasons():
    eng, _ = _engine(eos=7)
    a = eng.add_request([5], SamplingParams(max_tokens=10))                      # 6, 7 -> eos
    b = eng.add_request([5], SamplingParams(max_tokens=10, ignore_eos=True, stop_token_ids=[9]))
    c = eng.add_request([5], SamplingParams(max_tokens=3, ignore_eos=True))
    outs = {o.seq_id: o for o in eng.run_until_complete()}
    assert (outs[a].output_token_ids, outs[a].finish_reason) == ([6, 7], "stop")
    assert (outs[b].output_token_ids, outs[b].finish_reason) == ([6, 7, 8, 9], "stop")
    assert (outs[c].output_token_ids, outs[c].finish_reason) == ([6, 7, 8], "length")
    eng2, _ = _engine(max_model_len=6)
    d = eng2.add_request([1, 2, 3, 4], SamplingParams(max_tokens=50, ignore_eos=True))
    out = eng2.run_until_complete()[0]
    assert out.finish_reason == "length" and len(out.output_token_ids) == 2   # 4 + 2 = max_model_len


def test_rejects():
    # reference tests/test_engine.py:220-223, 253-260
    eng, _ = _engine(max_model_len=8)
    with pytest.raises(ValueError):
        eng.add_request([], SamplingParams())
    with pytest.raises(ValueError):
        eng.add_request([1] * 9, SamplingParams())
    with pytest.raises(ValueError):
        eng.add_request([1], SamplingParams(stop=["x"]))
    with pytest.raises(ValueError):
        eng.add_request([VOCAB], SamplingParams())
    with pytest.raises(ValueError):
        eng.add_request([1], SamplingParams(top_p=0.0))
    with pytest.raises(ValueError):
        eng.add_request([1, 2], SamplingParams(), position_ids=[[0, 1]])


def test_pages_run_out_newest_is_preempted_and_recomputed():
    # after reference tests/test_engine.py:120-147 (few pages, 4 requests of 32 tokens); here two
    # prompts fit (4 of 5 pages) but both need a third page to decode
    eng, runner = _engine(num_blocks=5, enable_prefix_cache=False)
    prompts = [[(11 * i + j) % VOCAB for j in range(32)] for i in range(4)]
    ids = [eng.add_request(p, SamplingParams(max_tokens=12, ignore_eos=True)) for p in prompts]
    outs = {o.seq_id: o for o in eng.run_until_complete()}
    assert sorted(outs) == ids and all(o.finish_reason == "length" for o in outs.values())
    assert eng.stats()["preemptions"] > 0
    for sid, p in zip(ids, prompts):
        assert outs[sid].output_token_ids == _expected(p, 12), "a recomputed request continues where it was"
    assert runner.cache.pages_in_use() == [0]
    # a preempted request is prefilled again from the start, its generated tokens included
    restarts = [(rid, n) for b in runner.batches for rid, start, n, _, _ in b if start == 0]
    assert any(n > 32 for _, n in restarts)


def test_a_request_that_can_never_fit_raises():
    eng, _ = _engine(num_blocks=2, enable_prefix_cache=False)
    eng.add_request([1] * 40, SamplingParams(max_tokens=4))
    with pytest.raises(OutOfPages):
        eng.run_until_complete()
    eng, _ = _engine(num_blocks=2, enable_prefix_cache=False)
    eng.add_request([1] * 30, SamplingParams(max_tokens=8, ignore_eos=True))
    with pytest.raises(OutOfPages):
        eng.run_until_complete()     # grows past two pages while it is the only request


def test_priority_decides_the_victim():
    eng, runner = _engine(num_blocks=4, enable_prefix_cache=False)
    low = eng.add_request([1] * 30, SamplingParams(max_tokens=6, ignore_eos=True), priority=0)
    high = eng.add_request([2] * 30, SamplingParams(max_tokens=6, ignore_eos=True), priority=5)
    outs = eng.run_until_complete()
    # both need a third page at the same step; the low-priority one gives way although it is older
    assert [o.seq_id for o in outs] == [high, low]
    assert eng.stats()["preemptions"] >= 1


def test_shared_prefix_is_reused():
    # reference tests/test_engine.py:57-106
    eng, runner = _engine()
    shared = [(3 * i) % VOCAB for i in range(40)]
    a = eng.add_request(shared + [1, 2], SamplingParams(max_tokens=2, ignore_eos=True))
    eng.run_until_complete()
    b = eng.add_request(shared + [9, 9, 9], SamplingParams(max_tokens=2, ignore_eos=True))
    out = [o for o in eng.run_until_complete() if o.seq_id == b][0]
    assert out.metrics["cached_tokens"] == 32
    first = [x for batch in runner.batches for x in batch if x[0] == b][0]
    assert (first[1], first[2]) == (32, 11), "only what the cache lacks is computed"
    assert out.output_token_ids == _expected([9], 2)
    assert eng.stats()["prefix_cache_tokens_saved"] == 32
    # a fully cached prompt still computes its last token
    c = eng.add_request(shared[:32], SamplingParams(max_tokens=1, ignore_eos=True))
    eng.run_until_complete()
    first = [x for batch in runner.batches for x in batch if x[0] == c][0]
    assert first[1] == 16 and first[2] == 16


def test_explicit_positions_and_delta():
    eng, runner = _engine(enable_prefix_cache=False, max_num_batched_tokens=4)
    rows = [[0, 1, 1, 1, 2], [0, 1, 1, 2, 2], [0, 1, 2, 1, 2]]
    eng.add_request([5, 6, 7, 8, 9], SamplingParams(max_tokens=3, ignore_eos=True), position_ids=rows)
    eng.run_until_complete()
    flat = [x for batch in runner.batches for x in batch]
    assert flat[0][4] == [r[:4] for r in rows]
    assert flat[1][4] == [r[4:] for r in rows]
    assert flat[2][4] is None and flat[3][4] is None   # text after the prompt: index + delta
    seq_delta = 3 - 5                                  # max position + 1 - prompt length (reference rope.py:233)
    eng2, r2 = _engine(enable_prefix_cache=False)
    eng2.add_request([5, 6, 7, 8, 9], SamplingParams(max_tokens=2, ignore_eos=True), position_ids=rows)
    eng2.step()
    assert eng2.running[0].rope_delta == seq_delta


def test_windowed_model_runs_through_the_scheduler():
    eng, runner = _engine(windows=(None, 8), num_blocks=8, max_num_batched_tokens=12)
    assert runner.cache.prefix_cache is None
    ids = [eng.add_request([(i + j) % VOCAB for j in range(30)], SamplingParams(max_tokens=20, ignore_eos=True))
           for i in range(2)]
    outs = eng.run_until_complete()
    assert sorted(o.seq_id for o in outs) == ids and runner.cache.pages_in_use() == [0, 0]


def test_stall_guard():
    eng, runner = _engine()
    eng.add_request([1, 2], SamplingParams(max_tokens=2, ignore_eos=True))
    eng._schedule = lambda: []          # a scheduler that never runs anything
    with pytest.raises(RuntimeError):
        eng.run_until_complete(max_stall=5)


# ---------------------------------------------------------------------------------------------
# The decode step queued ahead (with decode graphs): whatever happens meanwhile, tokens and finish
# reasons are those of an engine that schedules every step with the tokens known.

def _both_ways(requests, arrivals=(), **kw):
    """Run the same requests with and without the look-ahead; ``arrivals`` are ``(after step,
    prompt, params)`` added while the engine runs.  Returns ``(outputs by id, engine, runner)`` of
    each way."""
    ways = []
    for ahead in (False, True):
        eng, runner = _engine(hip_graph=True, decode_lookahead=ahead, **kw)
        for prompt, params in requests:
            eng.add_request(prompt, params)
        late = sorted(arrivals, key=lambda a: a[0])
        outs, steps = {}, 0
        while eng.has_work() or late:
            while late and late[0][0] <= steps:
                _, prompt, params = late.pop(0)
                eng.add_request(prompt, params)
            for o in eng.step():
                outs[o.seq_id] = (o.output_token_ids, o.finish_reason)
            steps += 1
            assert steps < 2000
        runner.cache.check()
        if runner.cache.prefix_cache is not None:
            runner.cache.prefix_cache.clear()      # what the remembered prompts hold
            runner.cache.check()
        assert all(n == 0 for n in runner.cache.pages_in_use()), "every page has come back"
        assert eng._ahead is None
        ways.append((outs, eng, runner))
    assert ways[0][2].ahead_steps == 0
    return ways


def test_ahead_stop_token_found_one_step_late():
    # request 0 stops on token 9 after four tokens, request 1 on the end-of-sequence token, request 2 by
    # length: the first two are found out after the next step has been queued with a row for them
    reqs = [([5], SamplingParams(max_tokens=20, ignore_eos=True, stop_token_ids=[9])),
            ([20], SamplingParams(max_tokens=20)),
            ([30], SamplingParams(max_tokens=12, ignore_eos=True))]
    (plain, _, _), (ahead, eng, runner) = _both_ways(reqs, eos=27, enable_prefix_cache=False)
    assert ahead == plain
    assert ahead[0] == ([6, 7, 8, 9], "stop") and ahead[1][1] == "stop" and ahead[2][1] == "length"
    assert runner.ahead_steps >= 8, "the look-ahead ran"
    # a row computed for nothing is not counted as a decoded token
    assert eng.stats()["decode_tokens"] == sum(len(t) for t, _ in ahead.values()) - 3


def test_ahead_with_an_arrival_while_a_step_is_queued():
    reqs = [([5, 6, 7], SamplingParams(max_tokens=10, ignore_eos=True))]
    late = [(4, [40, 41], SamplingParams(max_tokens=5, ignore_eos=True)),
            (5, [11] * 20, SamplingParams(max_tokens=3, ignore_eos=True))]
    (plain, _, _), (ahead, _, runner) = _both_ways(reqs, late, enable_prefix_cache=False)
    assert ahead == plain and len(ahead) == 3
    assert runner.ahead_steps > 0


def test_ahead_when_everyone_in_the_queued_step_has_finished():
    # both stop on the same step through a stop token: the queued step holds only dead rows
    reqs = [([5], SamplingParams(max_tokens=20, ignore_eos=True, stop_token_ids=[8])),
            ([15], SamplingParams(max_tokens=20, ignore_eos=True, stop_token_ids=[18]))]
    late = [(6, [1, 2], SamplingParams(max_tokens=2, ignore_eos=True))]
    (plain, _, _), (ahead, eng, runner) = _both_ways(reqs, late, enable_prefix_cache=False)
    assert ahead == plain and ahead[0] == ([6, 7, 8], "stop") and ahead[1] == ([16, 17, 18], "stop")
    assert runner.ahead_steps > 0


def test_ahead_when_pages_run_out_while_queueing():
    # five pages: both requests need a third page for the same step; the first gets the last free page
    # inside the look-ahead, the second does not: the queued step is given up and the scheduler,
    # with the tokens known, preempts as it would have
    reqs = [([(3 * j) % VOCAB for j in range(31)], SamplingParams(max_tokens=8, ignore_eos=True)),
            ([(5 * j) % VOCAB for j in range(31)], SamplingParams(max_tokens=8, ignore_eos=True))]
    (plain, e0, _), (ahead, e1, runner) = _both_ways(reqs, num_blocks=5, enable_prefix_cache=False)
    assert ahead == plain
    assert e0.stats()["preemptions"] >= 1 and e1.stats()["preemptions"] >= 1
    for (prompt, _), (tokens, reason) in zip(reqs, (ahead[0], ahead[1])):
        assert tokens == _expected(prompt, 8) and reason == "length"


def test_ahead_with_the_prefix_cache():
    shared = [(7 * i) % VOCAB for i in range(40)]
    reqs = [(shared + [1], SamplingParams(max_tokens=6, ignore_eos=True)),
            (shared + [2, 3], SamplingParams(max_tokens=4, ignore_eos=True, stop_token_ids=[5]))]
    late = [(9, shared + [9], SamplingParams(max_tokens=5, ignore_eos=True)),
            (12, shared[:32], SamplingParams(max_tokens=3, ignore_eos=True))]
    (plain, e0, _), (ahead, e1, runner) = _both_ways(reqs, late, max_num_seqs=2)
    assert ahead == plain and runner.ahead_steps > 0
    assert e1.stats()["prefix_cache_tokens_saved"] == e0.stats()["prefix_cache_tokens_saved"] > 0


def test_ahead_is_left_alone_by_penalties_and_by_waiting_requests():
    reqs = [([5], SamplingParams(max_tokens=6, ignore_eos=True, repetition_penalty=1.3))]
    (plain, _, _), (ahead, _, runner) = _both_ways(reqs, enable_prefix_cache=False)
    assert ahead == plain and runner.ahead_steps == 0, "a sampler that reads the generated tokens waits for them"
    reqs = [([i + 1], SamplingParams(max_tokens=6, ignore_eos=True)) for i in range(3)]
    (plain, _, _), (ahead, _, runner) = _both_ways(reqs, max_num_seqs=2, enable_prefix_cache=False)
    assert ahead == plain


def test_finished_outputs_are_handed_over_once():
    eng, _ = _engine()
    eng.add_request([1, 2], SamplingParams(max_tokens=2, ignore_eos=True))
    assert len(eng.run_until_complete()) == 1
    eng.add_request([3, 4], SamplingParams(max_tokens=2, ignore_eos=True))
    outs = eng.run_until_complete()
    assert len(outs) == 1 and outs[0].prompt_token_ids == [3, 4]


def test_the_slot_record_follows_its_request():
    """Every live request's slot holds its fixed-size record: cached length, rope delta, sampler
    settings and the number of tokens it has generated (what the seed rule draws from).  The record
    is filled at admission, moves on with every step, survives a preemption (the request is admitted
    again with what it had generated) and is cleared when the slot is given back."""
    eng, runner = _engine(num_blocks=6, block_size=16, max_num_seqs=3, max_num_batched_tokens=64,
                          enable_prefix_cache=False)
    rec = runner.cache.records
    a = eng.add_request(list(range(1, 31)), SamplingParams(temperature=0.7, top_k=5, seed=11, max_tokens=40, ignore_eos=True))
    b = eng.add_request(list(range(2, 22)), SamplingParams(max_tokens=40, repetition_penalty=1.3, ignore_eos=True),
                        rope_delta=4)
    seqs = {s.seq_id: s for s in eng.waiting}
    preempted = False
    for _ in range(400):
        eng.step()
        preempted = preempted or eng.stats_.preemptions > 0
        for s in eng.running:
            slot = runner.cache.slot_of(s.seq_id)
            assert s.slot == slot
            assert rec.num_tokens[slot] == s.num_computed_tokens == runner.cache.num_tokens(s.seq_id)
            assert rec.generated[slot] == len(s.output_token_ids)
            assert rec.rope_delta[slot] == s.rope_delta
            assert rec.seed[slot] == (-1 if s.params.seed is None else s.params.seed)
            assert rec.temperature[slot] == pytest.approx(s.params.temperature) and rec.top_k[slot] == s.params.top_k
            assert rec.repetition[slot] == pytest.approx(s.params.repetition_penalty)
        free = set(range(3)) - {runner.cache.slot_of(s.seq_id) for s in eng.running}
        for slot in free:      # a slot nobody holds has the record of a plain greedy request
            assert rec.num_tokens[slot] == rec.generated[slot] == rec.rope_delta[slot] == 0 and rec.seed[slot] == -1
            assert rec.temperature[slot] == 0 and rec.repetition[slot] == 1 and rec.top_k[slot] == -1
        if not eng.has_work():
            break
    assert preempted, "the pool is small enough that one of the two had to give way and come back"
    assert seqs[a].status == seqs[b].status == "finished" and not eng.has_work()
    assert rec.plain_greedy(__import__("numpy").arange(3))
