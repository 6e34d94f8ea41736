"""Generation through the entry points, the sampler kernel, and the trace_run program."""

import json
import os
import subprocess
import sys

import pytest
import torch

from plain_model import plain_filtered_probs, plain_model_logits, plain_penalties
from replay_util import random_tokens

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _plain_greedy(model_dir, prompt, n):
    ids, out = list(prompt), []
    for _ in range(n):
        nxt = int(torch.argmax(plain_model_logits(model_dir, ids)[-1]))
        out.append(nxt)
        ids.append(nxt)
    return out


@pytest.mark.parametrize("name, dtype", [("A", "float32"), ("B_sharp", "float32"), ("C_sharp", "float32")])
def test_greedy_generation_through_llm(model_dirs, name, dtype):
    # reference tests/test_engine.py:36-54 (prompt 3..12, 8 tokens), and batched = alone (test_chunked_prefill.py:155-190)
    from qwen25vl_lite_amd import LLM, SamplingParams

    d = model_dirs[name]
    vocab = {"A": 256, "B": 509, "C": 300}[name[0]]
    prompts = [list(range(3, 13)), random_tokens(6, vocab, 1), random_tokens(3, vocab, 2), random_tokens(45, vocab, 3)]
    llm = LLM(d, dtype=dtype, num_blocks=32, block_size=16, max_num_seqs=3, max_num_batched_tokens=24)
    outs = llm.generate(prompts, SamplingParams(temperature=0.0, max_tokens=8, ignore_eos=True))
    for prompt, out in zip(prompts, outs):
        assert out.prompt_token_ids == prompt and out.finish_reason == "length"
        assert out.output_token_ids == _plain_greedy(d, prompt, 8)
    assert llm.runner.cache.pages_in_use()[0] == (len(llm.runner.cache.prefix_cache)
                                                  if llm.runner.cache.prefix_cache else 0)
    llm.runner.cache.check()


def test_long_decode_and_preemption(model_dirs):
    """Decoding well past several pages, with so few pages that requests are preempted and
    prefilled again: the tokens are still the plain implementation's."""
    from qwen25vl_lite_amd import LLM, SamplingParams

    d = model_dirs["B_sharp"]
    prompts = [random_tokens(20, 509, 10 + i) for i in range(3)]
    llm = LLM(d, dtype="float32", num_blocks=10, block_size=16, max_num_seqs=3, max_num_batched_tokens=32,
              enable_prefix_cache=False)
    outs = llm.generate(prompts, SamplingParams(temperature=0.0, max_tokens=70, ignore_eos=True))
    assert llm.engine.stats()["preemptions"] > 0
    for prompt, out in zip(prompts, outs):
        assert out.output_token_ids == _plain_greedy(d, prompt, 70)
    assert llm.runner.cache.pages_in_use() == [0, 0]


def test_a_dropped_engine_frees_its_graphs_at_once(model_dirs):
    """Captured graphs go when their engine goes, by reference count (the collector is off here):
    a graph that lingered until a collection could be destroyed inside a later capture, which ends
    the process.  A second and third engine then capture their own graphs."""
    import gc
    import weakref

    from qwen25vl_lite_amd import LLM, SamplingParams

    d = model_dirs["A"]
    params = SamplingParams(temperature=0.0, max_tokens=6, ignore_eos=True)
    first = None
    for _ in range(3):
        gc.collect()
        gc.disable()
        try:
            llm = LLM(d, dtype="float32", num_blocks=16, block_size=16, max_num_seqs=2, hip_graph=True,
                      enable_prefix_cache=False)
            out = llm.generate([[1, 2, 3]], params)[0].output_token_ids
            graphs = list(llm.runner.graphs.graphs.values())
            assert graphs and all(g.graph is not None for g in graphs)
            watched = [weakref.ref(g) for g in graphs] + [weakref.ref(g.graph) for g in graphs]
            del graphs
            torch.cuda.synchronize()
            del llm
            assert all(w() is None for w in watched), "a captured graph outlived its engine"
        finally:
            gc.enable()
        first = first or out
        assert out == first
    with LLM(d, dtype="float32", num_blocks=16, block_size=16, max_num_seqs=2, hip_graph=True) as llm:
        assert llm.generate([[1, 2, 3]], params)[0].output_token_ids == first
        held = llm.runner.graphs
        assert held.graphs
    assert held.graphs == {}, "leaving the with block gives the graphs back"


@pytest.mark.parametrize("name", ["B_sharp", "C_sharp"])
def test_very_long_decode(model_dirs, name):
    """Three hundred tokens decoded from a short prompt, from HIP graphs: a dozen and a half pages,
    the window of the windowed layers passed many times over (their pages come back while the
    request runs), several context buckets.  float32: the plain implementation's tokens."""
    from qwen25vl_lite_amd import LLM, SamplingParams

    d = model_dirs[name]
    vocab = {"B": 509, "C": 300}[name[0]]
    prompt = random_tokens(7, vocab, 77)
    llm = LLM(d, dtype="float32", num_blocks=24, block_size=16, max_num_seqs=2, hip_graph=True,
              enable_prefix_cache=False)
    out = llm.generate([prompt], SamplingParams(temperature=0.0, max_tokens=300, ignore_eos=True))[0]
    assert out.output_token_ids == _plain_greedy(d, prompt, 300)
    assert len(llm.runner.graphs.graphs) >= 2
    assert llm.runner.cache.pages_in_use() == [0] * len(llm.runner.cache.groups)


@pytest.mark.parametrize("name, dtype, block_size", [("B_sharp", "float32", 16), ("C_sharp", "bfloat16", 16),
                                                     ("A", "bfloat16", 16), ("B_sharp", "float32", 48),
                                                     ("C_sharp", "bfloat16", 32)])
def test_decode_from_hip_graphs_gives_the_same_tokens(model_dirs, name, dtype, block_size):
    """Decode steps replayed from HIP graphs, many replays with eager prefill steps, admissions and
    finishes in between (batch size and context bucket change): every token equals the eager run's."""
    from qwen25vl_lite_amd import LLM, SamplingParams

    d = model_dirs[name]
    vocab = {"A": 256, "B": 509, "C": 300}[name[0]]
    prompts = [random_tokens(n, vocab, 50 + n) for n in (5, 250, 31, 70, 12)]
    params = [SamplingParams(temperature=0.0, max_tokens=m, ignore_eos=True) for m in (40, 30, 60, 9, 25)]
    common = dict(dtype=dtype, num_blocks=64, block_size=block_size, max_num_seqs=3, max_num_batched_tokens=64,
                  enable_prefix_cache=False)
    eager = LLM(d, **common).generate(prompts, params)
    llm = LLM(d, hip_graph=True, **common)
    assert llm.runner.graphs is not None
    graphed = llm.generate(prompts, params)
    assert len(llm.runner.graphs.graphs) >= 3
    for a, b in zip(eager, graphed):
        assert a.output_token_ids == b.output_token_ids
    if dtype == "float32":
        for prompt, out, p in zip(prompts, graphed, params):
            assert out.output_token_ids == _plain_greedy(d, prompt, p.max_tokens)


@pytest.mark.parametrize("name, dtype", [("B_sharp", "float32"), ("C_sharp", "bfloat16")])
def test_decode_graphs_with_padding_rows(model_dirs, name, dtype):
    """Batch sizes between the captured ones (7 and 5 requests run in graphs of 8 and 6 rows): the
    padding rows change nothing for the real ones, and the windowed layers' pages still come back."""
    from qwen25vl_lite_amd import LLM, SamplingParams

    d = model_dirs[name]
    vocab = {"B": 509, "C": 300}[name[0]]
    prompts = [random_tokens(n, vocab, 70 + n) for n in (9, 40, 3, 66, 21, 14, 50)]
    params = [SamplingParams(temperature=0.0, max_tokens=m, ignore_eos=True) for m in (30, 12, 44, 20, 52, 36, 25)]
    common = dict(dtype=dtype, num_blocks=96, block_size=16, max_num_seqs=8, max_num_batched_tokens=256,
                  enable_prefix_cache=False)
    eager = LLM(d, **common).generate(prompts, params)
    llm = LLM(d, hip_graph=True, **common)
    graphed = llm.generate(prompts, params)
    sizes = sorted({k[0] for k in llm.runner.graphs.graphs})
    assert 8 in sizes and 6 in sizes and 7 not in sizes and 5 not in sizes, sizes
    for a, b in zip(eager, graphed):
        assert a.output_token_ids == b.output_token_ids
    assert llm.runner.cache.pages_in_use() == [0] * len(llm.runner.cache.groups)


@pytest.mark.parametrize("name, dtype", [("B_sharp", "float32"), ("C", "bfloat16")])
def test_decode_step_queued_ahead_changes_nothing(model_dirs, name, dtype):
    """With decode graphs the scheduler queues the next decode step before it has seen the running
    step's tokens.  Requests that stop on a token (found out one step late), on their length
    (known beforehand), that sample with a seed, that arrive while others decode, and one whose
    penalties switch the lookahead off while it runs: tokens and finish reasons are those of the
    engine that schedules every step afterwards (requests that arrive while a step is queued are
    admitted one step later), and every page comes back."""
    from qwen25vl_lite_amd import LLM, SamplingParams

    d = model_dirs[name]
    vocab = {"B": 509, "C": 300}[name[0]]
    prompts = [random_tokens(n, vocab, 900 + n) for n in (12, 5, 30, 9, 17, 3)]
    def run(lookahead, stops):
        llm = LLM(d, dtype=dtype, num_blocks=64, block_size=16, max_num_seqs=6, max_num_batched_tokens=64,
                  enable_prefix_cache=False, hip_graph=True, decode_lookahead=lookahead)
        runner, engine = llm.runner, llm.engine
        params = [SamplingParams(temperature=0.0, max_tokens=40, ignore_eos=True, stop_token_ids=stops[0]),
                  SamplingParams(temperature=0.8, top_k=20, seed=5, max_tokens=23, ignore_eos=True),
                  SamplingParams(temperature=0.0, max_tokens=31, ignore_eos=True, stop_token_ids=stops[2]),
                  SamplingParams(temperature=0.0, max_tokens=8, ignore_eos=True),
                  SamplingParams(temperature=0.0, max_tokens=6, ignore_eos=True, repetition_penalty=1.3),
                  SamplingParams(temperature=1.1, top_p=0.9, seed=11, max_tokens=19, ignore_eos=True)]
        for p, sp in zip(prompts[:3], params[:3]):
            engine.add_request(p, sp)
        steps = queued = 0
        finished = []
        while engine.has_work():
            finished += engine.step()
            steps += 1
            queued += engine._ahead is not None
            if steps == 6:            # three more arrive while the first three decode
                for p, sp in zip(prompts[3:], params[3:]):
                    engine.add_request(p, sp)
        outs = sorted(finished, key=lambda o: o.seq_id)
        assert runner.cache.pages_in_use() == [0] * len(runner.cache.groups)
        runner.cache.check()
        return [(o.output_token_ids, o.finish_reason) for o in outs], steps, queued

    free, _, _ = run(False, [(), (), ()])
    # stop tokens that the requests really produce, in the middle of their outputs
    stops = [(free[0][0][14],), (), (free[2][0][6],)]
    plain, plain_steps, none_queued = run(False, stops)
    ahead, ahead_steps, queued = run(True, stops)
    assert none_queued == 0 and queued > 10, queued
    assert plain[0][1] == "stop" and plain[2][1] == "stop" and len(plain[0][0]) <= 15
    assert ahead == plain
    assert ahead_steps in (plain_steps, plain_steps + 1)   # the arrivals wait for the step that was queued already
    if dtype == "float32":
        assert plain[3][0] == _plain_greedy(d, prompts[3], 8)


@pytest.mark.parametrize("name, hip_graph, count", [("C_sharp", False, 21), ("B_sharp", True, 21), ("A_sharp", True, 52),
                                                    ("C_sharp", False, 45)])
def test_twenty_odd_requests_decode_together(model_dirs, name, hip_graph, count):
    """Between 17 and 32 decoded tokens a step the bfloat16 products run with two column tiles of
    rows (norm, rotation with cache write, activation and residual folded in as with fewer), and
    between 33 and 64 with teams of blocks for the fused q | k | v projection and the kernel that
    cuts the inner size for the output and down projections: 21, 45 or 52
    requests of different lengths, some ending early so that the batch shrinks through 48, 32, 24, 16 and
    12 rows.  float32 gives the plain implementation's tokens.  bfloat16 gives them up to the first
    place where the plain logits' two best lie closer than the bound on bfloat16 logits (2e-2, as
    in the replay tests): there the token the engine picked lies within that bound of the best, and
    what follows it is another sequence."""
    from qwen25vl_lite_amd import LLM, SamplingParams

    d = model_dirs[name]
    vocab = {"A": 256, "B": 509, "C": 300}[name[0]]
    prompts = [random_tokens(3 + (5 * i) % 23, vocab, 300 + i) for i in range(count)]
    params = [SamplingParams(temperature=0.0, max_tokens=4 + (7 * i) % 19, ignore_eos=True) for i in range(count)]
    common = dict(num_blocks=256, block_size=16, max_num_seqs=64, max_num_batched_tokens=1024,
                  enable_prefix_cache=False, hip_graph=hip_graph)
    exact = LLM(d, dtype="float32", **common).generate(prompts, params)
    llm = LLM(d, dtype="bfloat16", **common)
    outs = llm.generate(prompts, params)
    if hip_graph:
        assert (24 if count < 32 else 48) in {k[0] for k in llm.runner.graphs.graphs}
    whole = 0
    for prompt, out, ex, p in zip(prompts, outs, exact, params):
        want = _plain_greedy(d, prompt, p.max_tokens)
        assert ex.output_token_ids == want
        got = out.output_token_ids
        if got == want:
            whole += 1
            continue
        j = next(k for k in range(len(want)) if got[k] != want[k])
        row = plain_model_logits(d, list(prompt) + want[:j])[-1]
        assert float(row.max() - row[got[j]]) < 2e-2, (j, torch.topk(row, 3), got[j])
    assert whole >= count * 2 // 3          # ties are the exception
    assert llm.runner.cache.pages_in_use() == [0] * len(llm.runner.cache.groups)


@pytest.mark.parametrize("name, seed", [("A_sharp", 0), ("A_sharp", 1), ("C_sharp", 2)])
def test_everything_at_once(model_dirs, name, seed):
    """A server's day in small: requests of random lengths, some sharing a prefix, more of them than
    request slots, so few pages that some are preempted and computed again, decode steps from HIP
    graphs with padding rows, the prefix cache on (model A) or a windowed group giving pages back
    (model C).  In float32 every request's tokens are the plain implementation's, and all pages
    come back."""
    import random
    from qwen25vl_lite_amd import LLM, SamplingParams

    d = model_dirs[name]
    vocab = {"A": 256, "C": 300}[name[0]]
    rng = random.Random(seed)
    shared = random_tokens(40, vocab, 500 + seed)
    prompts, params = [], []
    for i in range(9):
        n = 8 if i == 0 else rng.randint(2, 60)
        body = random_tokens(n, vocab, 600 + 10 * seed + i)
        # the first request holds the shared prefix for as long as it runs; two later ones find it
        prompts.append(shared + body if i in (0, 6, 7) else body)
        params.append(SamplingParams(temperature=0.0, max_tokens=45 if i == 0 else rng.randint(3, 40),
                                     ignore_eos=True))
    llm = LLM(d, dtype="float32", num_blocks=18, block_size=16, max_num_seqs=5, max_num_batched_tokens=48,
              hip_graph=True, enable_prefix_cache=True)
    outs = llm.generate(prompts, params)
    stats = llm.engine.stats()
    assert stats["preemptions"] > 0, stats
    assert len(llm.runner.graphs.graphs) >= 2
    if name[0] == "A":
        assert stats["prefix_cache_hits"] > 0, stats
    for prompt, p, out in zip(prompts, params, outs):
        assert out.output_token_ids == _plain_greedy(d, prompt, p.max_tokens), (len(prompt), p.max_tokens)
    llm.runner.cache.check()
    cached = len(llm.runner.cache.prefix_cache) if llm.runner.cache.prefix_cache else 0
    assert llm.runner.cache.pages_in_use()[0] == cached


@pytest.mark.parametrize("name, seed, pool, seqs", [("A", 3, 12, 5), ("C", 6, 14, 4)])
def test_look_ahead_under_preemption_stops_arrivals_and_the_prefix_cache(model_dirs, name, seed, pool, seqs):
    """The decode step queued ahead, in a server's day: requests arriving over a dozen steps, a shared
    prefix and the prefix cache (model A) or a windowed group (model C), stop tokens frequent enough
    to end some requests early (found out one step late), seeded sampling beside greedy, a request
    with a penalty, and so few pages that requests are preempted and computed again.  Tokens and
    finish reasons are those of the engine without the look-ahead; greedy requests give the plain
    implementation's tokens; all pages come back."""
    import random
    from qwen25vl_lite_amd import LLM, SamplingParams

    d = model_dirs[name]
    vocab = {"A": 256, "C": 300}[name]
    rng = random.Random(1000 + seed)
    n = 10
    shared = random_tokens(36, vocab, 4000 + seed)
    prompts = [random_tokens(rng.randint(2, 50), vocab, 5000 + 50 * seed + i) for i in range(n)]
    for i in (0, 4, 7):
        prompts[i] = shared + prompts[i][:12]
    params = []
    for i in range(n):
        kind = rng.random()
        params.append(SamplingParams(temperature=0.0 if kind < 0.6 else 0.9, top_k=0 if kind < 0.8 else 30,
                                     seed=rng.randint(0, 99), max_tokens=rng.randint(25, 60), ignore_eos=True,
                                     repetition_penalty=1.2 if i == 5 else 1.0))
    arrive = sorted(rng.randint(0, 12) for _ in range(n))
    arrive[0] = 0

    def run(look):
        llm = LLM(d, dtype="float32", num_blocks=pool, block_size=16, max_num_seqs=seqs, max_num_batched_tokens=48,
                  enable_prefix_cache=True, hip_graph=True, decode_lookahead=look)
        eng, step, nxt, queued, outs = llm.engine, 0, 0, 0, []
        while nxt < n or eng.has_work():
            while nxt < n and arrive[nxt] <= step:
                eng.add_request(prompts[nxt], params[nxt])
                nxt += 1
            if eng.has_work():
                outs += eng.step()
                queued += eng._ahead is not None
            step += 1
            assert step < 5000
        cache = llm.runner.cache
        cache.check()
        cached = len(cache.prefix_cache) if cache.prefix_cache else 0
        assert cache.pages_in_use()[0] == cached and all(u == 0 for u in cache.pages_in_use()[1:])
        return sorted(((o.seq_id, o.output_token_ids, o.finish_reason) for o in outs)), queued, eng.stats()

    free, _, _ = run(False)
    for sid, tokens, _ in free:        # every other request stops on a token it really produces, half way
        if sid % 2 and len(tokens) >= 4:
            params[sid].stop_token_ids = (tokens[len(tokens) // 2],)
    plain, none_queued, stats0 = run(False)
    ahead, queued, stats1 = run(True)
    assert none_queued == 0 and queued > 10, queued
    assert stats0["preemptions"] > 0 and stats1["preemptions"] > 0, (stats0, stats1)
    assert any(reason == "stop" for _, _, reason in ahead)
    if name == "A":
        assert stats1["prefix_cache_hits"] > 0
    assert ahead == plain
    for sid, tokens, reason in ahead:
        p = params[sid]
        if p.temperature == 0.0 and p.repetition_penalty == 1.0:
            want = _plain_greedy(d, prompts[sid], len(tokens))
            assert tokens == want, sid


@pytest.mark.parametrize("name", ["B_sharp", "C_sharp"])
def test_forked_request_continues_on_its_own_pages(model_dirs, name):
    """A request forked in the middle of a page (reference cache.py:537-545 copies blocks for
    this): the two continuations share the full pages, each writes to its own copy of the page
    being filled, and each one's logits are those of its own whole sequence."""
    from qwen25vl_lite_amd import LLM
    from qwen25vl_lite_amd.engine.batch import StepEntry

    d = model_dirs[name]
    vocab = {"B": 509, "C": 300}[name[0]]
    runner = LLM(d, dtype="float32", num_blocks=12, block_size=16, max_num_seqs=3, enable_prefix_cache=False).runner
    prompt = random_tokens(53, vocab, 31)
    tails = {"a": random_tokens(20, vocab, 32), "b": random_tokens(20, vocab, 33)}
    runner.admit("a")
    runner.execute([StepEntry("a", prompt, 0, [])])
    runner.fork("a", "b")
    got = {"a": [], "b": []}
    for i in range(20):
        logits = runner.execute([StepEntry(r, [tails[r][i]], 53 + i, [0]) for r in ("b", "a")])
        got["b"].append(logits[0].cpu())
        got["a"].append(logits[1].cpu())
    for r in ("a", "b"):
        want = plain_model_logits(d, prompt + tails[r])[53:]
        assert torch.allclose(torch.stack(got[r]), want, atol=1e-4, rtol=1e-3), r
    runner.cache.check()
    runner.release("a")
    runner.release("b")
    assert runner.cache.pages_in_use() == [0] * len(runner.cache.groups)


def test_prefix_reuse_gives_the_same_tokens(model_dirs):
    # reference tests/test_chunked_prefill.py:193-227, tests/test_engine.py:57-106
    from qwen25vl_lite_amd import LLM, SamplingParams

    d = model_dirs["A_sharp"]
    shared = random_tokens(40, 256, 77)
    llm = LLM(d, dtype="float32", num_blocks=32, block_size=16, max_num_seqs=2)
    params = SamplingParams(temperature=0.0, max_tokens=6, ignore_eos=True)
    first = llm.generate([shared + [1, 2, 3]], params)[0]
    second = llm.generate([shared + [9, 8]], params)[0]
    assert second.metrics["cached_tokens"] == 32 and first.metrics["cached_tokens"] == 0
    assert second.output_token_ids == _plain_greedy(d, shared + [9, 8], 6)
    assert first.output_token_ids == _plain_greedy(d, shared + [1, 2, 3], 6)


def test_temperature_sampling_is_seeded_and_batch_independent(model_dirs):
    from qwen25vl_lite_amd import LLM, SamplingParams

    d = model_dirs["B"]
    prompts = [random_tokens(n, 509, 30 + n) for n in (1, 9, 40)]
    params = SamplingParams(temperature=0.7, max_tokens=12, seed=1, ignore_eos=True)
    llm = LLM(d, dtype="float32", num_blocks=32, block_size=16, max_num_seqs=4, max_num_batched_tokens=7)
    together = [o.output_token_ids for o in llm.generate(prompts, params)]
    alone = [llm.generate([p], params)[0].output_token_ids for p in prompts]
    assert together == alone
    other = llm.generate([prompts[2]], SamplingParams(temperature=0.7, max_tokens=12, seed=2, ignore_eos=True))[0]
    assert other.output_token_ids != together[2]


def _plain_draw(logits, prev, p, u):
    pen = plain_penalties(logits, prev, p.repetition_penalty, p.presence_penalty, p.frequency_penalty)
    if p.temperature <= 0:
        return int(torch.argmax(pen))
    probs = plain_filtered_probs(pen, p.temperature, p.top_k, p.top_p, p.min_p)
    cdf = torch.cumsum(probs.double(), 0)
    return int(torch.searchsorted(cdf, torch.tensor(u * float(cdf[-1]), dtype=torch.float64), right=True).clamp(max=len(probs) - 1))


def test_sampler_kernel_against_plain():
    from qwen25vl_lite_amd.sampling import SamplingParams
    from qwen25vl_lite_amd.sampling.sampler import sample_rows

    g = torch.Generator().manual_seed(0)
    vocab = 1531
    cases = [
        SamplingParams(temperature=0.0),
        SamplingParams(temperature=0.0, repetition_penalty=1.7, presence_penalty=0.4, frequency_penalty=0.3),
        SamplingParams(temperature=1.0),
        SamplingParams(temperature=0.7, top_k=5),
        SamplingParams(temperature=1.3, top_p=0.6),
        SamplingParams(temperature=0.9, min_p=0.1),
        SamplingParams(temperature=0.8, top_k=40, top_p=0.9, min_p=0.02, repetition_penalty=1.2),
        SamplingParams(temperature=1.0, top_k=1),
    ]
    for trial in range(6):
        logits = torch.randn(len(cases), vocab, generator=g) * 3
        prev = [torch.randint(0, vocab, (trial * 7,), generator=g).tolist() for _ in cases]
        us = torch.rand(len(cases), generator=g).tolist()
        got = sample_rows(logits.cuda(), cases, prev, [len(p) for p in prev], uniforms=us)
        for i, p in enumerate(cases):
            want = _plain_draw(logits[i], prev[i], p, us[i])
            if got[i] != want:
                # a draw that lands within rounding of a boundary of the distribution function
                probs = plain_filtered_probs(plain_penalties(logits[i], prev[i], p.repetition_penalty,
                                                             p.presence_penalty, p.frequency_penalty),
                                             max(p.temperature, 1e-6), p.top_k, p.top_p, p.min_p).double()
                cdf = torch.cumsum(probs, 0) / probs.sum()
                assert probs[got[i]] > 0 and min(abs(cdf[got[i]] - us[i]), abs(cdf[got[i]] - probs[got[i]] - us[i])) < 1e-5, \
                    (trial, i, got[i], want)
    # greedy rows: the lowest index among equal maxima, wherever in the row they lie (the row is
    # scanned in pieces), for a vocabulary that is no multiple of anything
    vocab = 152064 + 7
    rows = torch.randn(4, vocab, generator=g)
    top = rows.max() + 1
    spots = [[5, 70000, 152070], [152070], [4752, 4753, 9504], [0, 152070]]
    for r, where in enumerate(spots):
        rows[r, where] = top
    greedy = [SamplingParams(temperature=0.0)] * 3 + [SamplingParams(temperature=0.0, presence_penalty=0.5)]
    got = sample_rows(rows.cuda(), greedy, [[], [], [], [0]], [0, 0, 0, 1])
    assert got == [5, 152070, 4752, 152070]        # the last row's token 0 is pushed down by its penalty

    # the distribution itself: many draws of one row follow the filtered probabilities
    p = SamplingParams(temperature=1.0, top_k=4)
    row = torch.tensor([2.0, 1.0, 0.5, 0.0, -1.0, -3.0])
    n = 4000
    us = ((torch.arange(n) + 0.5) / n).tolist()
    draws = sample_rows(row.repeat(n, 1).cuda(), [p] * n, [[]] * n, [0] * n, uniforms=us)
    freq = torch.bincount(torch.tensor(draws), minlength=6).double() / n
    assert torch.allclose(freq, plain_filtered_probs(row, 1.0, top_k=4).double(), atol=2e-3)


def test_trace_run_program(model_dirs, tmp_path):
    """bin/trace_run as a user calls it: JSON steps on standard input, `done <step>` lines,
    <step>.f32 files of little-endian float32 [wanted, vocab]."""
    d = model_dirs["A"]
    toks = random_tokens(21, 256, 4)
    steps = [
        {"step": 0, "entries": [{"id": "a", "tokens": toks[:9], "want": [0, 8]}], "end": []},
        {"step": 1, "entries": [{"id": "a", "tokens": toks[9:20], "want": []}], "end": []},
        {"step": 2, "entries": [{"id": "a", "tokens": toks[20:], "want": [0]},
                                {"id": "b", "tokens": toks[:3], "want": [2]}], "end": ["a", "b"]},
    ]
    out = tmp_path / "out"
    proc = subprocess.run(
        [sys.executable, os.path.join(ROOT, "bin", "trace_run"), "--model", d, "--dtype", "float32", "--out", str(out),
         "--max-tokens", "128"],
        input="".join(json.dumps(s) + "\n" for s in steps), capture_output=True, text=True, timeout=110)
    assert proc.returncode == 0, proc.stderr[-2000:]
    assert proc.stdout.split() == ["done", "0", "done", "1", "done", "2"]
    assert sorted(os.listdir(out)) == ["0.f32", "2.f32"]
    ref = plain_model_logits(d, toks)
    import numpy as np
    s0 = torch.from_numpy(np.fromfile(out / "0.f32", dtype="<f4").reshape(2, 256))
    s2 = torch.from_numpy(np.fromfile(out / "2.f32", dtype="<f4").reshape(2, 256))
    assert torch.allclose(s0, ref[[0, 8]], atol=1e-4, rtol=1e-3)
    assert torch.allclose(s2[0], ref[20], atol=1e-4, rtol=1e-3) and torch.allclose(s2[1], ref[2], atol=1e-4, rtol=1e-3)


def test_generate_and_bench_commands(model_dirs):
    """`qwen25vl-lite generate` as a user calls it (reference cli.py:267-278): two prompts separated
    by ';', decode steps from a captured graph with the next step queued ahead; it prints each
    request's list of output ids, which are the plain implementation's.  Without prompt ids it
    exits with 2 (reference cli.py:271-274).  `bench` runs its one prompt and prints its rates."""
    import ast
    d = model_dirs["B_sharp"]
    prompts = [[7, 300, 41, 2, 99], [5, 6]]
    cli = [sys.executable, os.path.join(ROOT, "bin", "qwen25vl-lite")]
    common = ["--model", d, "--dtype", "float32", "--num-blocks", "32", "--max-num-seqs", "2", "--max-model-len", "256"]
    proc = subprocess.run(cli + ["generate", *common, "--cuda-graph", "--decode-lookahead", "--max-tokens", "9",
                                 "--ignore-eos", "--prompt-token-ids", ";".join(",".join(map(str, p)) for p in prompts)],
                          capture_output=True, text=True, timeout=110)
    assert proc.returncode == 0, proc.stderr[-2000:]
    printed = [ast.literal_eval(line) for line in proc.stdout.strip().splitlines()]
    assert printed == [_plain_greedy(d, p, 9) for p in prompts]
    proc = subprocess.run(cli + ["generate", *common], capture_output=True, text=True, timeout=110)
    assert proc.returncode == 2 and "--prompt-token-ids" in proc.stderr
    proc = subprocess.run(cli + ["bench", *common, "--prompt-tokens", "40", "--max-tokens", "6"],
                          capture_output=True, text=True, timeout=110)
    assert proc.returncode == 0, proc.stderr[-2000:]
    assert "prefill 40 tokens + decode 6 tokens" in proc.stdout and "tok/s" in proc.stdout


def test_smoke_entry():
    sys.path.insert(0, ROOT)
    import __graft_entry__
    __graft_entry__.smoke()
