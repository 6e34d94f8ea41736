"""Each part alone, and parts defined here (a mixer with state of its own, a routed feed-forward,
another position encoding) registered, built and stepped without touching the framework."""

import math

import pytest
import torch

from plain_model import plain_attention, plain_inv_freq, plain_rmsnorm

pytestmark = pytest.mark.gpu


def _spec_model(layers, hidden, vocab, dtype=torch.float32, run=None, seed=0):
    from qwen25vl_lite_amd.models import DecoderModel, LayerSpec, ModelSpec, RunEntry
    from qwen25vl_lite_amd.parts import PartSpec
    from qwen25vl_lite_amd.weights import fill_random

    norm = PartSpec("rms_norm", {"size": hidden, "eps": 1e-6})
    specs = []
    for i, (mixer, ffn) in enumerate(layers):
        block = PartSpec("pre_norm", {"norm1": norm, "mixer": mixer, "norm2": norm, "ffn": ffn,
                                      "names": {"norm1": "ln1", "mixer": "mix", "norm2": "ln2", "ffn": "ff"}})
        specs.append(LayerSpec(block, f"blocks.{i}."))
    spec = ModelSpec(hidden_size=hidden, vocab_size=vocab, layers=specs,
                     run=run or [RunEntry(i) for i in range(len(layers))], final_norm=norm,
                     tie_word_embeddings=True, position_rows=3, embed_name="tok.weight", final_norm_prefix="ln_f.")
    model = DecoderModel(spec, dtype, "cuda:0")
    fill_random(model, seed, std=0.3)
    return model


def _runner(model, pages=32, seqs=4):
    from qwen25vl_lite_amd.config import EngineConfig
    from qwen25vl_lite_amd.engine import ModelRunner
    ecfg = EngineConfig(num_blocks=pages, block_size=16, max_num_seqs=seqs, max_num_batched_tokens=512,
                        max_model_len=pages * 16, enable_prefix_cache=False, dtype=model.dtype)
    return ModelRunner(model, ecfg)


def _run(runner, rid, tokens, cuts):
    from qwen25vl_lite_amd.engine import StepEntry
    runner.admit(rid)
    rows, at = [], 0
    for c in cuts:
        part = tokens[at:at + c]
        rows.append(runner.execute([StepEntry(rid, part, at, want=list(range(len(part))))]).cpu())
        at += len(part)
    assert at == len(tokens)
    runner.release(rid)
    return torch.cat(rows)


def _attn_spec(hidden, nq, nkv, hd, position, window=None, scale=None):
    from qwen25vl_lite_amd.parts import PartSpec
    return PartSpec("paged_attention", {"hidden_size": hidden, "num_heads": nq, "num_kv_heads": nkv, "head_dim": hd,
                                        "qkv_bias": False, "window": window, "scale": scale, "position": position})


def test_norm_part_alone():
    from qwen25vl_lite_amd.parts import PartSpec, ResidualStream, build_part
    torch.manual_seed(0)
    part = build_part("norm", PartSpec("rms_norm", {"size": 70, "eps": 1e-3}), torch.float32, torch.device("cuda:0"))
    assert {k: v.shape for k, v in part.param_specs().items()} == {"weight": (70,)}
    w = torch.randn(70)
    part.load({"weight": w.cuda()})
    h, d = torch.randn(4, 70), torch.randn(4, 70)
    stream = ResidualStream(h.cuda(), d.cuda())
    out = part.forward(stream)
    assert stream.pending is None and torch.allclose(stream.h.cpu(), h + d, atol=1e-6)
    assert torch.allclose(out.cpu(), plain_rmsnorm(h + d, w, 1e-3), atol=1e-5)


def test_position_parts_alone():
    from qwen25vl_lite_amd.parts import PartSpec, build_part
    dev = torch.device("cuda:0")
    mrope = build_part("position", PartSpec("mrope", {"theta": 1e4, "sections": (2, 3, 3)}), torch.float32, dev)
    inv, rows = mrope.rotary_tables(16)
    assert rows.tolist() == [0, 0, 1, 1, 1, 2, 2, 2] and torch.equal(inv.cpu(), plain_inv_freq(16, 1e4))
    with pytest.raises(ValueError):
        mrope.rotary_tables(32)        # sections must cover half the head (reference rope.py:89-93)
    rope = build_part("position", PartSpec("rope", {"theta": 1e4, "rotary_dim": 8}), torch.float32, dev)
    inv, rows = rope.rotary_tables(16)
    assert rows.tolist() == [0] * 4 and torch.equal(inv.cpu(), plain_inv_freq(8, 1e4))


def test_feed_forward_part_alone():
    from qwen25vl_lite_amd.parts import PartSpec, build_part
    torch.manual_seed(1)
    part = build_part("ffn", PartSpec("swiglu", {"hidden_size": 40, "intermediate_size": 72}), torch.float32,
                      torch.device("cuda:0"))
    g, u, d = torch.randn(72, 40), torch.randn(72, 40), torch.randn(40, 72)
    part.load({"gate_proj.weight": g.cuda(), "up_proj.weight": u.cuda(), "down_proj.weight": d.cuda()})
    x = torch.randn(5, 40)
    want = (torch.nn.functional.silu(x @ g.T) * (x @ u.T)) @ d.T
    assert torch.allclose(part.forward(x.cuda(), None).cpu(), want, atol=1e-4)
    assert torch.equal(part.named_weights()["up_proj.weight"].cpu(), u)


def test_attention_part_without_rotation_is_plain_attention():
    """One layer whose position encoding rotates nothing (rotary_dim 0) and a custom scale: the
    mixer reduces to causal attention over the projections, computed here with the library."""
    from qwen25vl_lite_amd.parts import PartSpec
    hidden, nq, nkv, hd = 48, 4, 2, 12
    pos = PartSpec("rope", {"theta": 1e4, "rotary_dim": 0})
    ffn = PartSpec("swiglu", {"hidden_size": hidden, "intermediate_size": 16})
    model = _spec_model([(_attn_spec(hidden, nq, nkv, hd, pos, scale=0.37), ffn)], hidden, 50)
    mixer = model.blocks[0].mixer
    w = {k: v.float().cpu() for k, v in mixer.named_weights().items()}
    torch.manual_seed(2)
    t = 37
    x = torch.randn(t, hidden)
    from qwen25vl_lite_amd.engine import StepEntry
    from qwen25vl_lite_amd.engine.batch import build_step
    runner = _runner(model)
    runner.admit("a")
    runner.cache.reserve("a", t)
    step = build_step([StepEntry("a", [0] * t, 0)], runner.cache, 3, torch.float32, model.device)
    out = mixer.forward(x.cuda(), step, runner.slots[0]).cpu()
    q = (x @ w["q_proj.weight"].T).view(t, nq, hd).transpose(0, 1)
    k = (x @ w["k_proj.weight"].T).view(t, nkv, hd).transpose(0, 1)
    v = (x @ w["v_proj.weight"].T).view(t, nkv, hd).transpose(0, 1)
    lib = torch.nn.functional.scaled_dot_product_attention(
        q[None], k.repeat_interleave(2, 0)[None], v.repeat_interleave(2, 0)[None], is_causal=True, scale=0.37)[0]
    want = lib.transpose(0, 1).reshape(t, nq * hd) @ w["o_proj.weight"].T
    assert torch.allclose(out, want, atol=1e-4)


def test_a_layer_named_twice_and_a_layer_reading_anothers_cache():
    """Run list [0, 1, 0, 2->cache of entry 1]: layer 0 runs twice with caches of its own, the last
    entry has no key/value projections and attends over what entry 1 wrote.  Cutting the sequence
    differently must not change a logit."""
    from qwen25vl_lite_amd.models import RunEntry
    from qwen25vl_lite_amd.parts import PartSpec
    hidden = 32
    pos = PartSpec("mrope", {"theta": 100.0, "sections": (1, 2, 1)})
    ffn = PartSpec("swiglu", {"hidden_size": hidden, "intermediate_size": 40})
    full = _attn_spec(hidden, 4, 2, 8, pos)
    shared = PartSpec("paged_attention", dict(full.params, kv_shared=True))
    model = _spec_model([(full, ffn), (full, ffn), (shared, ffn)], hidden, 60,
                        run=[RunEntry(0), RunEntry(1), RunEntry(0), RunEntry(2, cache_from=1)])
    assert model.cache_groups()[0].num_layers == 3 and "blocks.2.mix.k_proj.weight" not in model.expected_tensors()
    runner = _runner(model)
    toks = torch.randint(0, 60, (45,), generator=torch.Generator().manual_seed(3)).tolist()
    whole = _run(runner, "w", toks, [45])
    cut = _run(runner, "c", toks, [7, 2, 20, 1, 1, 14])
    assert torch.allclose(whole, cut, atol=1e-5)
    assert not torch.allclose(whole[1:], whole[:-1], atol=1e-3)


# ---------------------------------------------------------------------------------------------
# parts defined in the test
# ---------------------------------------------------------------------------------------------
def _register_toys():
    from qwen25vl_lite_amd.parts import (FeedForward, Mixer, ParamSpec, PositionEncoding, StateNeed, known_parts,
                                         register_part)
    if "toy_decay" in known_parts("mixer"):
        return

    class DecayMixer(Mixer):
        """y_t = s_t,  s_t = a * s_{t-1} + B x_t  with a state s of its own per request."""

        def __init__(self, params, dtype, device):
            super().__init__(dtype, device)
            self.hidden, self.width = params["hidden_size"], params["state_size"]

        def state_need(self):
            return StateNeed((self.width,), torch.float32)

        def param_specs(self):
            return {"a": ParamSpec((self.width,), "vector"), "B.weight": ParamSpec((self.width, self.hidden)),
                    "C.weight": ParamSpec((self.hidden, self.width))}

        def load(self, tensors):
            self.a, self.B, self.C = torch.sigmoid(tensors["a"]), tensors["B.weight"].float(), tensors["C.weight"].float()

        def forward(self, x, step, slot):
            u = x.float() @ self.B.T
            out = torch.empty_like(u)
            for r, slot_id in enumerate(step.req_slots_host):
                s = slot.state[slot_id]
                for n in range(step.cu_q_host[r], step.cu_q_host[r + 1]):
                    s = self.a * s + u[n]
                    out[n] = s
                slot.state[slot_id] = s
            return (out @ self.C.T).to(torch.float32)

    class RoutedFeedForward(FeedForward):
        """Two experts of one matrix each; a token goes to the expert its router logit favours."""

        def __init__(self, params, dtype, device):
            super().__init__(dtype, device)
            self.hidden = params["hidden_size"]

        def param_specs(self):
            return {"router.weight": ParamSpec((2, self.hidden)), "experts.0.weight": ParamSpec((self.hidden, self.hidden)),
                    "experts.1.weight": ParamSpec((self.hidden, self.hidden))}

        def load(self, tensors):
            self.t = {k: v.float() for k, v in tensors.items()}

        def forward(self, x, step):
            xf = x.float()
            pick = (xf @ self.t["router.weight"].T).argmax(-1)
            y0, y1 = xf @ self.t["experts.0.weight"].T, xf @ self.t["experts.1.weight"].T
            return torch.where(pick[:, None] == 0, y0, y1)

    class HalfSpeedRoPE(PositionEncoding):
        """1-D rotation on row 2 of the positions with halved frequencies, first half of the head only."""
        num_rows = 3

        def __init__(self, params, dtype, device):
            super().__init__(dtype, device)
            self.theta = params["theta"]
            self.tables = {}

        def rotary_tables(self, head_dim):
            if head_dim not in self.tables:      # made once: a captured step must not copy from the host
                rot = head_dim // 2
                inv = 0.5 * plain_inv_freq(rot, self.theta)
                self.tables[head_dim] = (inv.to(self.device),
                                         torch.full((rot // 2,), 2, dtype=torch.int32, device=self.device))
            return self.tables[head_dim]

    class GraphDecayMixer(DecayMixer):
        """The same mixer with a decode path that may be captured: the requests' state rows are
        found through the step's device tensor, not through a host loop."""
        graph_safe = True

        def forward(self, x, step, slot):
            if step.max_q_len != 1:
                return super().forward(x, step, slot)
            rows = step.req_slots.long()
            s = self.a * slot.state.index_select(0, rows) + x.float() @ self.B.T
            slot.state.index_copy_(0, rows, s)
            return (s @ self.C.T).to(torch.float32)

    class GraphRoutedFeedForward(RoutedFeedForward):
        graph_safe = True

    register_part("mixer", "toy_decay", DecayMixer)
    register_part("mixer", "toy_decay_graph", GraphDecayMixer)
    register_part("ffn", "toy_routed", RoutedFeedForward)
    register_part("ffn", "toy_routed_graph", GraphRoutedFeedForward)
    register_part("position", "toy_half_speed", HalfSpeedRoPE)


def _plain_toy_model(model, toks, pos_row2):
    """The toy model of `test_toy_parts...` computed whole, in plain float32 on the CPU."""
    w = {}
    for part, names in model.part_groups():
        pass
    hidden = model.spec.hidden_size
    emb = model.embed.float().cpu()
    h = emb[torch.tensor(toks)]
    t = len(toks)
    for block in model.blocks:
        x = plain_rmsnorm(h, block.norm1.weight.cpu(), 1e-6)
        m = block.mixer
        if hasattr(m, "B"):
            a, B, C = m.a.cpu(), m.B.cpu(), m.C.cpu()
            s, ys = torch.zeros(B.shape[0]), []
            for n in range(t):
                s = a * s + B @ x[n]
                ys.append(s)
            y = torch.stack(ys) @ C.T
        else:
            nw = {k: v.float().cpu() for k, v in m.named_weights().items()}
            q = (x @ nw["q_proj.weight"].T).view(t, m.nq, m.hd).transpose(0, 1)
            k = (x @ nw["k_proj.weight"].T).view(t, m.nkv, m.hd).transpose(0, 1)
            v = (x @ nw["v_proj.weight"].T).view(t, m.nkv, m.hd).transpose(0, 1)
            rot = m.hd // 2
            inv = 0.5 * plain_inv_freq(rot, 50.0)
            ang = pos_row2.float()[:, None] * inv[None]
            cos, sin = ang.cos(), ang.sin()

            def rotate(z):
                z = z.clone()
                a1, a2 = z[..., :rot // 2].clone(), z[..., rot // 2:rot].clone()
                z[..., :rot // 2] = a1 * cos - a2 * sin
                z[..., rot // 2:rot] = a2 * cos + a1 * sin
                return z

            o = plain_attention(rotate(q), rotate(k), v, m.hd ** -0.5, m.window)
            y = o.transpose(0, 1).reshape(t, m.nq * m.hd) @ nw["o_proj.weight"].T
        h = h + y
        x2 = plain_rmsnorm(h, block.norm2.weight.cpu(), 1e-6)
        f = block.ffn
        if hasattr(f, "t"):
            tt = {k: v.cpu() for k, v in f.t.items()}
            pick = (x2 @ tt["router.weight"].T).argmax(-1)
            y2 = torch.where(pick[:, None] == 0, x2 @ tt["experts.0.weight"].T, x2 @ tt["experts.1.weight"].T)
        else:
            nw = {k: v.float().cpu() for k, v in f.named_weights().items()}
            y2 = (torch.nn.functional.silu(x2 @ nw["gate_proj.weight"].T) * (x2 @ nw["up_proj.weight"].T)) @ nw["down_proj.weight"].T
        h = h + y2
    return plain_rmsnorm(h, model.final_norm.weight.cpu(), 1e-6) @ emb.T


def test_toy_parts_register_build_and_step():
    """A mixer with a state of its own, a routed feed-forward and another position encoding, all
    defined above, in one model with a windowed attention layer: whole, cut into portions, and two
    requests interleaved (so that each one's state must live in its own slot)."""
    from qwen25vl_lite_amd.engine import StepEntry
    from qwen25vl_lite_amd.parts import PartSpec
    _register_toys()
    hidden = 24
    toy_pos = PartSpec("toy_half_speed", {"theta": 50.0})
    decay = PartSpec("toy_decay", {"hidden_size": hidden, "state_size": 10})
    routed = PartSpec("toy_routed", {"hidden_size": hidden})
    swiglu = PartSpec("swiglu", {"hidden_size": hidden, "intermediate_size": 40})
    layers = [(decay, routed), (_attn_spec(hidden, 3, 1, 8, toy_pos, window=9), swiglu), (decay, swiglu)]
    model = _spec_model(layers, hidden, 40, seed=5)
    assert [s is not None for s in model.entry_state] == [True, False, True]
    assert "blocks.0.mix.B.weight" in model.expected_tensors() and "blocks.0.ff.router.weight" in model.expected_tensors()
    runner = _runner(model, pages=8)
    g = torch.Generator().manual_seed(9)
    ta = torch.randint(0, 40, (30,), generator=g).tolist()
    tb = torch.randint(0, 40, (21,), generator=g).tolist()
    want_a = _plain_toy_model(model, ta, torch.arange(30))
    want_b = _plain_toy_model(model, tb, torch.arange(21))
    assert torch.allclose(_run(runner, "a", ta, [30]), want_a, atol=2e-4)
    assert torch.allclose(_run(runner, "a2", ta, [4, 2, 11, 1, 1, 1, 10]), want_a, atol=2e-4)
    # interleaved: portions of a beside single tokens of b, in the same steps
    runner.admit("a")
    runner.admit("b")
    got_a, got_b, ia, ib = [], [], 0, 0
    while ia < len(ta) or ib < len(tb):
        entries = []
        if ia < len(ta):
            n = min(5, len(ta) - ia)
            entries.append(StepEntry("a", ta[ia:ia + n], ia, want=list(range(n))))
        if ib < len(tb):
            entries.append(StepEntry("b", tb[ib:ib + 1], ib, want=[0]))
        out = runner.execute(entries).cpu()
        if ia < len(ta):
            got_a.append(out[:n]); out = out[n:]; ia += n
        if ib < len(tb):
            got_b.append(out); ib += 1
    assert torch.allclose(torch.cat(got_a), want_a, atol=2e-4) and torch.allclose(torch.cat(got_b), want_b, atol=2e-4)
    # a slot that is taken again starts from a cleared state
    runner.release("a"); runner.release("b")
    assert torch.allclose(_run(runner, "again", tb, [21]), want_b, atol=2e-4)


# ---------------------------------------------------------------------------------------------
# a whole toy architecture, from a model folder, with nothing but registrations
# ---------------------------------------------------------------------------------------------
TOY_CONFIG = {
    "architectures": ["ToyDecayLM"], "width": 24, "tokens": 40, "state": 10, "inner": 40, "heads": 3, "groups": 1,
    "head": 8, "reach": 9, "base": 50.0, "stop_id": 39,
    # which mixer and feed-forward each layer has; no key of the Qwen decoder appears anywhere
    "plan": [["decay", "routed"], ["attention", "swiglu"], ["decay", "swiglu"]],
}


def _register_toy_architecture(name="ToyDecayLM", graph=""):
    """``graph="_graph"``: the same architecture from the toy parts that may be captured."""
    from qwen25vl_lite_amd.config import known_architectures, register_architecture
    from qwen25vl_lite_amd.models import LayerSpec, ModelSpec, RunEntry
    from qwen25vl_lite_amd.parts import PartSpec
    _register_toys()
    if name in known_architectures():
        return

    def build_spec(cfg):
        hidden = cfg.width
        norm = PartSpec("rms_norm", {"size": hidden, "eps": 1e-6})
        pos = PartSpec("toy_half_speed", {"theta": cfg.base})
        mixers = {"decay": PartSpec("toy_decay" + graph, {"hidden_size": hidden, "state_size": cfg.state}),
                  "attention": _attn_spec(hidden, cfg.heads, cfg.groups, cfg.head, pos, window=cfg.reach)}
        ffns = {"routed": PartSpec("toy_routed" + graph, {"hidden_size": hidden}),
                "swiglu": PartSpec("swiglu", {"hidden_size": hidden, "intermediate_size": cfg.inner})}
        layers = []
        for i, (mixer, ffn) in enumerate(cfg.plan):
            block = PartSpec("pre_norm", {"norm1": norm, "mixer": mixers[mixer], "norm2": norm, "ffn": ffns[ffn],
                                          "names": {"norm1": "ln1", "mixer": "mix", "norm2": "ln2", "ffn": "ff"}})
            layers.append(LayerSpec(block, f"blocks.{i}."))
        return ModelSpec(hidden_size=hidden, vocab_size=cfg.tokens, layers=layers,
                         run=[RunEntry(i) for i in range(len(layers))], final_norm=norm, tie_word_embeddings=True,
                         position_rows=3, embed_name="tok.weight", final_norm_prefix="ln_f.",
                         store_name=lambda name: "toy." + name,
                         map_name=lambda name: name[4:] if name.startswith("toy.") else name,
                         eos_token_id=cfg.stop_id)

    register_architecture(name, build_spec)      # no reader of its own: the raw keys are its configuration


def test_toy_architecture_from_a_model_folder(tmp_path):
    """A model folder whose config.json names an architecture registered here, with keys of its
    own (none of the Qwen decoder's), a mixer with per-request state, a routed feed-forward and its
    own position encoding: written with random weights, loaded through ``LLM``, replayed through
    ``Replayer``, generated from greedily, with nothing but ``register_part`` and
    ``register_architecture`` calls.  The prefix cache switches itself off (a cached prefix could
    not bring the mixer's state back)."""
    import json
    from qwen25vl_lite_amd import LLM, SamplingParams, write_random_model
    from qwen25vl_lite_amd.config import load_config
    from qwen25vl_lite_amd.engine.replay import Replayer
    from qwen25vl_lite_amd.weights import SafetensorsFile
    _register_toy_architecture()
    d = str(tmp_path / "toy")
    write_random_model(load_config(TOY_CONFIG), d, seed=11, std=0.3, dtype=torch.float32)
    with open(f"{d}/config.json") as fh:
        assert json.load(fh) == TOY_CONFIG
    with SafetensorsFile(f"{d}/model.safetensors") as f:
        assert "toy.blocks.0.mix.B.weight" in f.keys() and "toy.tok.weight" in f.keys()
    llm = LLM(d, dtype="float32", num_blocks=16, block_size=16, max_num_seqs=3, max_num_batched_tokens=16,
              enable_prefix_cache=True)
    assert llm.runner.cache.prefix_cache is None, "a model with per-request state must not reuse cached prefixes"
    assert llm.runner.eos_token_id == 39
    g = torch.Generator().manual_seed(4)
    prompts = [torch.randint(0, 39, (n,), generator=g).tolist() for n in (5, 23, 12)]
    # the second shares the first's opening tokens: with a prefix cache it would skip them
    prompts[1][:5] = prompts[0]
    outs = llm.generate(prompts, SamplingParams(temperature=0.0, max_tokens=7, ignore_eos=True))
    for prompt, out in zip(prompts, outs):
        ids, want = list(prompt), []
        for _ in range(7):
            nxt = int(torch.argmax(_plain_toy_model(llm.model, ids, torch.arange(len(ids)))[-1]))
            want.append(nxt)
            ids.append(nxt)
        assert out.output_token_ids == want
    assert llm.engine.stats()["prefix_cache_hits"] == 0
    # the same folder through the replay tool's class: whole, then cut
    rp = Replayer(d, "float32", 64)
    toks = prompts[1]
    whole = rp.step({"step": 0, "entries": [{"id": "w", "tokens": toks, "want": list(range(len(toks)))}], "end": ["w"]})
    want = _plain_toy_model(llm.model, toks, torch.arange(len(toks)))
    assert torch.allclose(whole.cpu(), want, atol=2e-4)
    rows = []
    for i, (a, b) in enumerate(((0, 9), (9, 11), (11, 23))):
        rows.append(rp.step({"step": i + 1, "entries": [{"id": "c", "tokens": toks[a:b], "want": list(range(b - a))}]}))
    assert torch.allclose(torch.cat(rows).cpu(), want, atol=2e-4)


def test_a_stateful_mixer_under_decode_graphs(tmp_path):
    """A mixer that keeps per-request state and says it may be captured: decode steps then run from
    HIP graphs.  A new graph is warmed up by running its first step several times, each of which
    advances the state; the engine must put the state rows back, or the tokens after the first
    capture differ from the eager run's and the plain toy's.  Two batch sizes are captured (three
    requests, then two once the shortest has ended)."""
    from qwen25vl_lite_amd import LLM, SamplingParams, write_random_model
    from qwen25vl_lite_amd.config import load_config
    _register_toy_architecture("ToyDecayGraphLM", "_graph")
    d = str(tmp_path / "toy_graph")
    write_random_model(load_config(dict(TOY_CONFIG, architectures=["ToyDecayGraphLM"])), d, seed=11, std=0.3,
                       dtype=torch.float32)
    g = torch.Generator().manual_seed(6)
    prompts = [torch.randint(0, 39, (n,), generator=g).tolist() for n in (5, 23, 12)]
    params = [SamplingParams(temperature=0.0, max_tokens=n, ignore_eos=True) for n in (9, 4, 9)]
    options = dict(dtype="float32", num_blocks=16, block_size=16, max_num_seqs=3, max_num_batched_tokens=64)
    with LLM(d, hip_graph=True, **options) as llm:
        assert llm.model.graph_safe and llm.runner.graphs is not None
        outs = llm.generate(prompts, params)
        assert len(llm.runner.graphs.graphs) >= 2, "decode steps of two batch sizes ran from graphs"
        model = llm.model
        for prompt, sp, out in zip(prompts, params, outs):
            ids, want = list(prompt), []
            for _ in range(sp.max_tokens):
                nxt = int(torch.argmax(_plain_toy_model(model, ids, torch.arange(len(ids)))[-1]))
                want.append(nxt)
                ids.append(nxt)
            assert out.output_token_ids == want
    eager = LLM(d, hip_graph=False, **options)
    assert [o.output_token_ids for o in eager.generate(prompts, params)] == [o.output_token_ids for o in outs]


def test_a_block_with_two_mixers_gets_a_slot_for_each():
    """A block defined here runs an attention mixer and a state mixer side by side on the same
    normalised input.  The model gives each its own place: pages for one, a state row for the
    other, found under the mixer's sub-part name.  Whole, cut and interleaved runs agree, and
    both mixers contribute."""
    from qwen25vl_lite_amd.engine import StepEntry
    from qwen25vl_lite_amd.models import DecoderModel, LayerSpec, ModelSpec, RunEntry
    from qwen25vl_lite_amd.parts import Block, PartSpec, build_part, known_parts, register_part
    from qwen25vl_lite_amd.weights import fill_random
    _register_toys()

    class SideBySide(Block):
        def __init__(self, params, dtype, device):
            super().__init__(dtype, device)
            self.norm1 = build_part("norm", params["norm"], dtype, device)
            self.attn = build_part("mixer", params["attn"], dtype, device)
            self.decay = build_part("mixer", params["decay"], dtype, device)
            self.norm2 = build_part("norm", params["norm"], dtype, device)
            self.ffn = build_part("ffn", params["ffn"], dtype, device)

        def sub_parts(self):
            return {"ln1": self.norm1, "attn": self.attn, "decay": self.decay, "ln2": self.norm2, "ff": self.ffn}

        def forward(self, stream, step, slot):
            x = self.norm1.forward(stream)
            a = self.attn.forward(x, step, slot.by_part["attn"])
            b = self.decay.forward(x, step, slot.by_part["decay"])
            stream.pending = a.float() + b
            y = self.norm2.forward(stream)
            stream.pending = self.ffn.forward(y, step)
            return stream

    if "toy_side_by_side" not in known_parts("block"):
        register_part("block", "toy_side_by_side", SideBySide)
    hidden = 24
    norm = PartSpec("rms_norm", {"size": hidden, "eps": 1e-6})
    pos = PartSpec("rope", {"theta": 100.0, "rotary_dim": 8})
    block = PartSpec("toy_side_by_side", {
        "norm": norm, "attn": _attn_spec(hidden, 3, 1, 8, pos), "ffn": PartSpec("toy_routed", {"hidden_size": hidden}),
        "decay": PartSpec("toy_decay", {"hidden_size": hidden, "state_size": 6})})
    spec = ModelSpec(hidden_size=hidden, vocab_size=40, layers=[LayerSpec(block, "b0."), LayerSpec(block, "b1.")],
                     run=[RunEntry(0), RunEntry(1)], final_norm=norm, tie_word_embeddings=True, position_rows=3,
                     embed_name="tok.weight", final_norm_prefix="ln_f.")
    model = DecoderModel(spec, torch.float32, "cuda:0")
    fill_random(model, 8, std=0.3)
    assert model.entry_places == [{"attn": 0, "decay": 1}, {"attn": 2, "decay": 3}]
    assert [s is not None for s in model.entry_state] == [False, True, False, True]
    assert model.cache_groups()[0].num_layers == 2
    runner = _runner(model, pages=8)
    slot = runner.slots[1]
    assert slot.by_part["attn"].k_cache is not None and slot.by_part["attn"].state is None
    assert slot.by_part["decay"].k_cache is None and slot.by_part["decay"].state.shape == (5, 6)
    g = torch.Generator().manual_seed(2)
    ta = torch.randint(0, 40, (26,), generator=g).tolist()
    tb = torch.randint(0, 40, (9,), generator=g).tolist()
    whole_a, whole_b = _run(runner, "a", ta, [26]), _run(runner, "b", tb, [9])
    assert torch.allclose(_run(runner, "a2", ta, [3, 2, 17, 1, 1, 2]), whole_a, atol=1e-5)
    runner.admit("a"); runner.admit("b")
    got_a, got_b = [], []
    for i in range(9):                       # portions of a beside single tokens of b
        n = 3 if i < 8 else 2
        out = runner.execute([StepEntry("b", tb[i:i + 1], i, want=[0]),
                              StepEntry("a", ta[3 * i:3 * i + n], 3 * i, want=list(range(n)))]).cpu()
        got_b.append(out[:1]); got_a.append(out[1:])
    assert torch.allclose(torch.cat(got_a), whole_a, atol=1e-5) and torch.allclose(torch.cat(got_b), whole_b, atol=1e-5)
    runner.release("a"); runner.release("b")
    # each mixer matters: without its output projection the logits change
    for name in ("b0.attn.o_proj.weight", "b1.decay.C.weight"):
        part, local, _ = model.params[name]
        kept = (part.w_out if local == "o_proj.weight" else part.C).clone()
        (part.w_out if local == "o_proj.weight" else part.C).zero_()
        assert not torch.allclose(_run(runner, "z", ta, [26]), whole_a, atol=1e-3)
        (part.w_out if local == "o_proj.weight" else part.C).copy_(kept)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_toy_ends_of_the_model(dtype):
    """The two ends are parts as well: an embedding that scales its rows and a head with a bias and
    a soft cap, defined here, registered, named in a spec, given random weights and stepped through
    the runner; the head is tied to the toy embedding's table.  One toy layer sits between them."""
    from qwen25vl_lite_amd.models import DecoderModel, LayerSpec, ModelSpec, RunEntry
    from qwen25vl_lite_amd.ops import kernels
    from qwen25vl_lite_amd.ops.linear import linear
    from qwen25vl_lite_amd.parts import Embedding, Head, ParamSpec, PartSpec, known_parts, register_part
    from qwen25vl_lite_amd.weights import fill_random

    class ScaledTable(Embedding):
        graph_safe = True

        def __init__(self, params, dtype, device):
            super().__init__(dtype, device)
            self.vocab, self.hidden, self.scale = params["vocab_size"], params["hidden_size"], float(params["scale"])

        def param_specs(self):
            return {"weight": ParamSpec((self.vocab, self.hidden), "table")}

        def load(self, tensors):
            self.table = tensors["weight"]

        def forward(self, token_ids, step):
            return kernels.embed_gather(token_ids, self.table) * self.scale

    class CappedHead(Head):
        graph_safe = True

        def __init__(self, params, dtype, device):
            super().__init__(dtype, device)
            self.vocab, self.hidden, self.cap = params["vocab_size"], params["hidden_size"], float(params["cap"])

        def param_specs(self):
            return {"weight": ParamSpec((self.vocab, self.hidden)), "bias": ParamSpec((self.vocab,), "vector")}

        def load(self, tensors):
            self.bias = tensors["bias"]
            self.weight = tensors.get("weight", getattr(self, "weight", None))

        def tie(self, embedding):
            self.weight = embedding.table

        def forward(self, x, step):
            return self.cap * torch.tanh((linear(x, self.weight, out_dtype=torch.float32) + self.bias) / self.cap)

    if "toy_scaled" not in known_parts("embedding"):
        register_part("embedding", "toy_scaled", ScaledTable)
        register_part("head", "toy_capped", CappedHead)
    hidden, vocab, scale, cap = 64, 97, 8.0, 3.0
    sizes = {"vocab_size": vocab, "hidden_size": hidden}
    norm = PartSpec("rms_norm", {"size": hidden, "eps": 1e-5})
    spec = ModelSpec(hidden_size=hidden, vocab_size=vocab, layers=[], run=[], final_norm=norm, tie_word_embeddings=True,
                     embed_name="tok.weight", head_name="out.weight", final_norm_prefix="ln_f.",
                     embed=PartSpec("toy_scaled", dict(sizes, scale=scale)), head=PartSpec("toy_capped", dict(sizes, cap=cap)))
    model = DecoderModel(spec, dtype, "cuda:0")
    assert sorted(model.expected_tensors()) == ["ln_f.weight", "out.bias", "out.weight", "tok.weight"]
    fill_random(model, 5, std=0.3)
    assert model.head_part.weight is model.embedding.table          # tied: no tensor of its own was drawn
    runner = _runner(model)
    tokens = [5, 96, 0, 41, 41, 7]
    got = _run(runner, "a", tokens, [4, 1, 1])
    table, g, b = model.embed.float().cpu(), model.final_norm.weight.float().cpu(), model.head_part.bias.float().cpu()
    h = table[tokens] * scale
    x = plain_rmsnorm(h, g, 1e-5)
    if dtype == torch.bfloat16:
        x = x.bfloat16().float()
    want = cap * torch.tanh((x @ table.T + b) / cap)
    tol = dict(atol=1e-4, rtol=1e-4) if dtype == torch.float32 else dict(atol=3e-2, rtol=3e-2)
    assert torch.allclose(got, want, **tol), (got - want).abs().max()
