"""The benchmark's own context length through the real choice of attention kernels.

One request of 8,300 tokens at the 7B decoder's head geometry (narrow width, two layers, peaked
attention) is fed as portions of 4,096, decoded token by token, and stepped beside a portion of
a second request.  No limit of the dispatch is lowered and no kind of kernel is forced: the test
watches which kinds the dispatch takes by itself and holds every wanted row to the plain
implementation (page edges and long contexts as in reference tests/test_paged_attn_kernel.py:82-112).
"""

import pytest
import torch

from plain_model import as_bfloat16, plain_model_logits
from replay_util import random_tokens, round64, run_steps

pytestmark = pytest.mark.gpu

LONG, SHORT = 8300, 300


def _trace(long_toks, short_toks):
    steps = []

    def add(entries, end=()):
        steps.append({"step": len(steps), "entries": entries, "end": list(end)})

    def portion(rid, toks, lo, hi):
        n = hi - lo
        return {"id": rid, "tokens": toks[lo:hi], "want": sorted({0, 1, n // 2, n - 2, n - 1} & set(range(n)))}

    add([portion("long", long_toks, 0, 4096)])
    add([portion("long", long_toks, 4096, 8192)])          # late in a long prompt: many long walks
    add([portion("long", long_toks, 8192, 8280)])
    at = 8280
    for _ in range(4):                                       # single tokens over more than 8,192 keys
        add([portion("long", long_toks, at, at + 1)])
        at += 1
    # a decoded token with a long context beside a portion of another request
    add([portion("long", long_toks, at, at + 1), portion("short", short_toks, 0, 256)])
    at += 1
    add([portion("short", short_toks, 256, SHORT - 4), portion("long", long_toks, at, at + 1)])
    at += 1
    for i in range(4):                                       # both decode, one context short, one long
        last = i == 3
        add([portion("short", short_toks, SHORT - 4 + i, SHORT - 3 + i), portion("long", long_toks, at, at + 1)],
            end=["short"] if last else [])
        at += 1
    while at < LONG:
        add([portion("long", long_toks, at, at + 1)], end=["long"] if at == LONG - 1 else [])
        at += 1
    return steps


@pytest.fixture(scope="module")
def sharp_d(model_dirs):
    return model_dirs["D_sharp"]


@pytest.fixture(scope="module")
def tokens():
    return random_tokens(LONG, 300, 77), random_tokens(SHORT, 300, 78)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_context_of_the_benchmark_through_the_real_dispatch(sharp_d, tokens, dtype, monkeypatch):
    from qwen25vl_lite_amd.engine.replay import Replayer
    from qwen25vl_lite_amd.ops import attention_mfma
    long_toks, short_toks = tokens
    store = as_bfloat16 if dtype == "bfloat16" else (lambda x: x)
    ref = {"long": plain_model_logits(sharp_d, long_toks, store=store),
           "short": plain_model_logits(sharp_d, short_toks, store=store)}
    # what the dispatch decides, step by step
    seen = []
    real_fn = attention_mfma._fn

    def spy_fn(stem, name, argtypes, defines=None):
        fn = real_fn(stem, name, argtypes, defines)
        if name not in ("qvl_attn_mfma_block", "qvl_attn_mfma_coop", "qvl_attn_mfma_coop_merged"):
            return fn

        def launch(*args):
            # the kernel for few tiles is told into how many ranges the keys are split (the argument
            # before the keys per split and the stream)
            split = {} if name.endswith("block") else {"nsplit": args[-3], "keys": args[-2]}
            seen.append(("qvl_attn_mfma_coop" if "coop" in name else name, dict(defines or {}, **split)))
            return fn(*args)
        return launch

    monkeypatch.setattr(attention_mfma, "_fn", spy_fn)
    rp = Replayer(sharp_d, dtype, round64(LONG) + round64(SHORT))
    steps = _trace(long_toks, short_toks)
    per_step, got, at = [], {}, {}
    for rec in steps:
        seen.clear()
        got.update(run_steps(rp, [rec], at=at))
        per_step.append(list(seen))
    worst = 0.0
    for (rid, pos), row in got.items():
        want = ref[rid][pos]
        if dtype == "float32":
            ok, err = torch.allclose(row, want, atol=1e-4, rtol=1e-3), (row - want).abs().max().item()
        else:
            err = ((row - want).abs().max() / want.abs().max()).item()
            ok = err < 2e-2
        worst = max(worst, err)
        assert ok, f"request {rid} position {pos}: error {err:.3e}"
    print(dtype, "worst error", worst, "rows", len(got))
    assert rp.runner.cache.pages_in_use() == [0] * len(rp.runner.cache.groups)
    if dtype != "bfloat16":
        return
    layers = 2

    def calls(i, name):
        return [d for n, d in per_step[i] if n == name]

    def splits(i):
        return sorted(d["nsplit"] for d in calls(i, "qvl_attn_mfma_coop"))

    # the first portion: plain workgroups; the second, late in the prompt: the kind with three column tiles a wave
    assert len(calls(0, "qvl_attn_mfma_block")) == layers and all("BLK_CT" not in d for d in calls(0, "qvl_attn_mfma_block"))
    assert len(calls(1, "qvl_attn_mfma_block")) == layers and all(d.get("BLK_CT") == 3 for d in calls(1, "qvl_attn_mfma_block"))
    # single tokens over 8,280 keys: the keys split among blocks at the real limit of keys per split
    per = attention_mfma.MIN_KEYS_PER_SPLIT
    assert per <= 1024 and attention_mfma.ALONE_KEYS == 4096 and attention_mfma.SPLIT_FROM_KEYS <= 4096

    def cut(ctx):
        """As many splits as the limit of keys per split allows (the blocks are few): their length in
        whole blocks of 32 keys, and how many of that length cover the context."""
        most = ctx // per
        keys = ((ctx + 31 + most - 1) // most + 31) // 32 * 32
        return (ctx + 31 + keys - 1) // keys, keys

    many = cut(8284)[0]
    assert many >= 8 and all(cut(c)[0] == many for c in range(8281, 8300))
    for i in range(3, 7):
        assert calls(i, "qvl_attn_mfma_block") == [] and splits(i) == [many] * layers
        assert all(per <= d["keys"] < per + 64 for d in calls(i, "qvl_attn_mfma_coop"))
    # a decoded token with a long context beside a portion: a launch of its own for it, split, and one for the portion
    for i in (7, 8):
        assert calls(i, "qvl_attn_mfma_block") == [] and len(splits(i)) == 2 * layers
        assert all(n <= 4 for n in splits(i)[:layers]) and splits(i)[layers:] == [many] * layers
    # both decode: one launch, split by the longer context
    assert calls(9, "qvl_attn_mfma_block") == [] and len(splits(9)) == layers and all(n == many for n in splits(9))
