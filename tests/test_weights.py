"""The safetensors loader's errors and the random-weights mode (no GPU: the loader's checks run
before anything is copied, and a model on the `meta` device has no storage)."""

import json
import os

import pytest
import torch

from conftest import TINY_A, TINY_B
from qwen25vl_lite_amd import Qwen25VLConfig, WeightsError, build_model, load_weights, write_random_model
from qwen25vl_lite_amd.models.qwen25vl_text import map_checkpoint_name
from qwen25vl_lite_amd.weights import SafetensorsFile, random_tensors, write_safetensors


def _folder(tmp_path, raw, seed=0, **kw):
    d = str(tmp_path / "m")
    write_random_model(Qwen25VLConfig.from_dict(raw), d, seed, **kw)
    return d


def _rewrite(d, edit):
    path = os.path.join(d, "model.safetensors")
    with SafetensorsFile(path) as f:
        tensors = {k: f.tensor(k).clone() for k in f.keys()}
    edit(tensors)
    write_safetensors(path, tensors)


def test_name_mapping_takes_both_layouts_and_skips_vision():
    # reference model.py:52-73
    assert map_checkpoint_name("model.language_model.layers.0.mlp.up_proj.weight") == "layers.0.mlp.up_proj.weight"
    assert map_checkpoint_name("model.layers.0.mlp.up_proj.weight") == "layers.0.mlp.up_proj.weight"
    assert map_checkpoint_name("model.embed_tokens.weight") == "embed_tokens.weight"
    assert map_checkpoint_name("model.language_model.norm.weight") == "norm.weight"
    assert map_checkpoint_name("lm_head.weight") == "lm_head.weight"
    assert map_checkpoint_name("visual.blocks.0.attn.qkv.weight") is None
    assert map_checkpoint_name("model.visual.merger.mlp.0.weight") is None


def test_random_model_folder_is_complete_and_seeded(tmp_path):
    d = _folder(tmp_path, TINY_B, seed=3)
    assert sorted(os.listdir(d)) == ["config.json", "model.safetensors"]
    cfg = Qwen25VLConfig.from_pretrained(d)
    model = build_model(cfg, device="meta")
    with SafetensorsFile(os.path.join(d, "model.safetensors")) as f:
        stored = {map_checkpoint_name(k): (f.shape(k), f.dtype(k)) for k in f.keys()}
        norm = f.tensor("model.language_model.norm.weight").float()
        w = f.tensor("model.language_model.layers.1.mlp.up_proj.weight").float()
    assert set(stored) == set(model.expected_tensors())
    assert all(dt == torch.bfloat16 for _, dt in stored.values())
    assert abs(norm.mean().item() - 1.0) < 0.02 and abs(w.mean().item()) < 1e-3 and abs(w.std().item() - 0.02) < 2e-3
    # a tensor's values depend on (seed, name) only
    a = dict(random_tensors(model, 3))
    b = dict(random_tensors(model, 3))
    c = dict(random_tensors(model, 4))
    assert torch.equal(a["layers.0.self_attn.q_proj.bias"], b["layers.0.self_attn.q_proj.bias"])
    assert not torch.equal(a["layers.0.self_attn.q_proj.bias"], c["layers.0.self_attn.q_proj.bias"])


def test_tied_model_stores_no_head(tmp_path):
    d = _folder(tmp_path, TINY_A)
    with SafetensorsFile(os.path.join(d, "model.safetensors")) as f:
        assert "lm_head.weight" not in f.keys()


def test_one_error_lists_missing_unexpected_and_wrong_shapes(tmp_path):
    d = _folder(tmp_path, TINY_B)

    def edit(t):
        del t["model.language_model.layers.1.self_attn.k_proj.bias"]
        del t["lm_head.weight"]
        t["model.language_model.layers.9.mlp.up_proj.weight"] = torch.zeros(2, 2)
        t["model.language_model.layers.0.mlp.gate_proj.weight"] = torch.zeros(352, 143)
        t["visual.patch_embed.proj.weight"] = torch.zeros(3)  # vision tower: skipped, not an error

    _rewrite(d, edit)
    model = build_model(Qwen25VLConfig.from_pretrained(d), device="meta")
    with pytest.raises(WeightsError) as err:
        load_weights(d, model)
    e = err.value
    assert e.missing == ["layers.1.self_attn.k_proj.bias", "lm_head.weight"]
    assert e.unexpected == ["model.language_model.layers.9.mlp.up_proj.weight"]
    assert [(n, got, want) for n, got, want in e.wrong_shape] == [
        ("model.language_model.layers.0.mlp.gate_proj.weight", (352, 143), (352, 144))]
    text = str(e)
    for fragment in ("missing (2)", "unexpected (1)", "wrong shape (1)", "(352, 143)", "layers.9"):
        assert fragment in text


def test_missing_files(tmp_path):
    cfg = Qwen25VLConfig.from_dict(TINY_A)
    (tmp_path / "config.json").write_text(json.dumps(cfg.to_dict()))
    with pytest.raises(FileNotFoundError):
        load_weights(str(tmp_path), build_model(cfg, device="meta"))


def test_safetensors_reader_rejects_garbage(tmp_path):
    p = tmp_path / "x.safetensors"
    p.write_bytes(b"\x00" * 4)
    with pytest.raises(ValueError):
        SafetensorsFile(str(p))
    p.write_bytes((10 ** 9).to_bytes(8, "little") + b"{}")
    with pytest.raises(ValueError):
        SafetensorsFile(str(p))


def test_safetensors_roundtrip_against_the_library(tmp_path):
    from safetensors.torch import load_file, save_file

    tensors = {"a": torch.randn(3, 5).bfloat16(), "b": torch.arange(7, dtype=torch.int32), "c": torch.randn(2, 2, 2)}
    ours = str(tmp_path / "ours.safetensors")
    write_safetensors(ours, tensors)
    theirs = load_file(ours)
    save_file(tensors, str(tmp_path / "theirs.safetensors"))
    with SafetensorsFile(str(tmp_path / "theirs.safetensors")) as f:
        for k, v in tensors.items():
            assert torch.equal(theirs[k], v) and torch.equal(f.tensor(k), v) and f.dtype(k) == v.dtype


def test_a_folder_of_two_shards_with_an_index(tmp_path):
    """Checkpoints of real size come as several files named by ``model.safetensors.index.json``
    (reference model.py:312-348).  The same tensors in two shards (and a vision tensor that is
    skipped) load to the very values of the single file; a tensor that no shard holds is
    reported as missing."""
    d = _folder(tmp_path, TINY_B, seed=5)
    cfg = Qwen25VLConfig.from_pretrained(d)
    single = build_model(cfg, torch.bfloat16, "cpu")
    assert load_weights(d, single)["loaded"] == len(single.expected_tensors())
    path = os.path.join(d, "model.safetensors")
    with SafetensorsFile(path) as f:
        tensors = {k: f.tensor(k).clone() for k in f.keys()}
    names = sorted(tensors)
    first, second = names[::2], names[1::2]
    write_safetensors(os.path.join(d, "model-00001-of-00002.safetensors"), {k: tensors[k] for k in first})
    write_safetensors(os.path.join(d, "model-00002-of-00002.safetensors"),
                      {**{k: tensors[k] for k in second}, "visual.patch_embed.proj.weight": torch.zeros(3, 2)})
    weight_map = {k: "model-00001-of-00002.safetensors" for k in first}
    weight_map.update({k: "model-00002-of-00002.safetensors" for k in second})
    with open(os.path.join(d, "model.safetensors.index.json"), "w") as fh:
        json.dump({"metadata": {}, "weight_map": weight_map}, fh)
    os.remove(path)
    sharded = build_model(cfg, torch.bfloat16, "cpu")
    counts = load_weights(d, sharded)
    assert counts["loaded"] == len(sharded.expected_tensors()) and counts["skipped"] == 1
    assert torch.equal(sharded.embed, single.embed) and torch.equal(sharded.head, single.head)
    for a, b in zip(sharded.blocks, single.blocks):
        for name, t in a.mixer.named_weights().items():
            assert torch.equal(t, b.mixer.named_weights()[name]), name
        for name, t in a.ffn.named_weights().items():
            assert torch.equal(t, b.ffn.named_weights()[name]), name
        assert torch.equal(a.norm1.weight, b.norm1.weight) and torch.equal(a.norm2.weight, b.norm2.weight)
    # a shard that lost a tensor: one error that names it
    lost = second[0]
    write_safetensors(os.path.join(d, "model-00002-of-00002.safetensors"), {k: tensors[k] for k in second[1:]})
    with pytest.raises(WeightsError) as err:
        load_weights(d, build_model(cfg, torch.bfloat16, "cpu"))
    assert err.value.missing == [map_checkpoint_name(lost)]
