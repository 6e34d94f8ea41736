"""Captured decode graphs die with the runner that owns them, by reference count.

A graph destroyed while another capture is under way ends the process (its destructor
synchronizes the device, which a capture refuses).  So a dropped engine must not wait for the
cycle collector: nothing the graphs hold may refer back to the runner.  These tests keep the
collector off and watch the objects go.
"""

import gc
import types
import weakref

import pytest
import torch

from qwen25vl_lite_amd.engine import graph as graph_mod
from qwen25vl_lite_amd.engine.graph import DecodeGraphs


class _Token:
    """Stands for a captured graph: something whose death can be watched."""


def _stub_runner():
    runner = types.SimpleNamespace(
        model=types.SimpleNamespace(spec=types.SimpleNamespace(position_rows=3)),
        cache=types.SimpleNamespace(groups=[], page_size=16), slots=[], device=torch.device("cpu"),
        dtype=torch.float32, pad_state_slot=4, states=[],
        ecfg=types.SimpleNamespace(max_blocks_per_seq=8, max_num_seqs=4))
    runner.graphs = DecodeGraphs(runner)
    return runner


def test_dropping_the_runner_frees_its_graphs_without_a_collection():
    gc.collect()
    gc.disable()
    try:
        runner = _stub_runner()
        token = _Token()
        runner.graphs.graphs[(1, 256)] = token
        gone_token, gone_graphs = weakref.ref(token), weakref.ref(runner.graphs)
        del token
        assert gone_token() is not None
        del runner
        assert gone_graphs() is None and gone_token() is None, "something refers back to the runner"
    finally:
        gc.enable()


def test_nothing_a_graph_set_holds_refers_to_the_runner():
    runner = _stub_runner()
    seen, todo = set(), [runner.graphs]
    while todo:
        obj = todo.pop()
        if id(obj) in seen:
            continue
        seen.add(id(obj))
        assert obj is not runner
        todo.extend(r for r in gc.get_referents(obj) if not isinstance(r, (type, types.ModuleType, types.FunctionType)))


def test_close_drops_the_graphs():
    runner = _stub_runner()
    token = _Token()
    runner.graphs.graphs[(1, 256)] = token
    gone = weakref.ref(token)
    del token
    runner.graphs.close()
    assert gone() is None and runner.graphs.graphs == {}


def test_capture_collects_first_and_keeps_the_collector_off(monkeypatch):
    """Garbage that holds an older graph goes before the capture begins; inside it the collector
    is off; afterwards it is as it was."""
    events = []

    class FakeGraph:
        pass

    class FakeCapture:
        def __init__(self, g):
            pass

        def __enter__(self):
            events.append(("begin", gc.isenabled(), cyc_alive()))

        def __exit__(self, *a):
            events.append(("end", gc.isenabled()))

    monkeypatch.setattr(graph_mod.torch.cuda, "CUDAGraph", FakeGraph)
    monkeypatch.setattr(graph_mod.torch.cuda, "graph", FakeCapture)

    class Cyc:
        pass

    a, b = Cyc(), Cyc()
    a.other, b.other = b, a
    ref = weakref.ref(a)
    cyc_alive = lambda: ref() is not None
    del a, b
    assert gc.isenabled()
    graph, out = graph_mod._capture(lambda: events.append(("work", gc.isenabled())) or 7)
    assert isinstance(graph, FakeGraph) and out == 7
    assert events == [("begin", False, False), ("work", False), ("end", False)]
    assert gc.isenabled()
    with pytest.raises(ZeroDivisionError):
        graph_mod._capture(lambda: 1 // 0)
    assert gc.isenabled(), "the collector comes back on after a failed capture too"
