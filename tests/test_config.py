"""Configuration parsing and the architecture registry (no GPU)."""

import json
import os

import pytest

from conftest import TINY_A, TINY_B, TINY_C
from qwen25vl_lite_amd import ConfigError, Qwen25VLConfig, build_model, known_architectures, register_architecture
from qwen25vl_lite_amd.config import EngineConfig, resolve_architecture

SEVEN_B = {  # sizes of the Qwen2.5-VL-7B text decoder
    "architectures": ["Qwen2_5_VLForConditionalGeneration"], "tie_word_embeddings": False,
    "hidden_size": 3584, "intermediate_size": 18944, "num_hidden_layers": 28, "num_attention_heads": 28,
    "num_key_value_heads": 4, "vocab_size": 152064, "rope_theta": 1e6, "rms_norm_eps": 1e-6,
    "sliding_window": 32768, "use_sliding_window": False,
    "rope_scaling": {"type": "mrope", "mrope_section": [16, 24, 24]},
}


def test_text_config_in_text_config_block():
    cfg = Qwen25VLConfig.from_dict(TINY_A)
    t = cfg.text_config
    assert (t.hidden_size, t.num_hidden_layers, t.num_attention_heads, t.num_key_value_heads) == (64, 2, 4, 2)
    assert t.head_dim == 16 and t.mrope_section == (2, 3, 3) and t.rope_theta == 10000.0
    assert t.tie_word_embeddings is True
    assert t.layer_types == ("full_attention",) * 2 and t.layer_window(0) is None
    assert cfg.architecture == "Qwen2_5_VLForConditionalGeneration"


def test_top_level_fields_without_text_config():
    t = Qwen25VLConfig.from_dict(TINY_C).text_config
    assert t.hidden_size == 200 and t.head_dim == 48 and t.num_key_value_groups == 5
    assert t.layer_types == ("full_attention", "sliding_attention")
    assert t.layer_window(1) == 40 and t.layer_window(0) is None
    assert t.tie_word_embeddings is False and t.rms_norm_eps == 2e-6


def test_window_rule_and_explicit_layer_types():
    t = Qwen25VLConfig.from_dict(TINY_B).text_config
    assert t.layer_types == ("full_attention", "sliding_attention", "sliding_attention")
    raw = json.loads(json.dumps(TINY_B))
    raw["text_config"]["layer_types"] = ["sliding_attention", "full_attention", "full_attention"]
    t = Qwen25VLConfig.from_dict(raw).text_config
    assert t.layer_window(0) == 16 and t.layer_window(2) is None
    # the released 7B configuration carries sliding_window but switches it off
    assert set(Qwen25VLConfig.from_dict(SEVEN_B).text_config.layer_types) == {"full_attention"}


def test_rope_keys_from_rope_parameters_and_precedence():
    raw = json.loads(json.dumps(TINY_A))
    del raw["rope_scaling"]
    raw["rope_parameters"] = {"mrope_section": [3, 3, 2], "rope_theta": 5.0}
    t = Qwen25VLConfig.from_dict(raw).text_config
    assert t.mrope_section == (3, 3, 2)
    assert t.rope_theta == 10000.0  # the decoder's own key wins over the block (reference config.py:165-177)


@pytest.mark.parametrize("mutate, fragment", [
    (lambda r: r["text_config"].pop("hidden_size"), "hidden_size"),
    (lambda r: r["text_config"].pop("vocab_size"), "vocab_size"),
    (lambda r: r["text_config"].update(num_key_value_heads=3), "multiple"),
    (lambda r: r["rope_scaling"].update(mrope_section=[2, 3, 4]), "mrope_section"),
    (lambda r: r.pop("rope_scaling"), "mrope_section"),
    (lambda r: r["text_config"].update(hidden_act="gelu"), "hidden_act"),
    (lambda r: r["text_config"].update(layer_types=["full_attention"]), "layer_types"),
    (lambda r: r["text_config"].update(use_sliding_window=True, sliding_window=None, max_window_layers=0),
     "sliding_window"),
])
def test_bad_configs_are_refused(mutate, fragment):
    raw = json.loads(json.dumps(TINY_A))
    mutate(raw)
    with pytest.raises(ConfigError) as err:
        Qwen25VLConfig.from_dict(raw)
    assert fragment in str(err.value)


def test_num_params_and_kv_bytes():
    t = Qwen25VLConfig.from_dict(SEVEN_B).text_config
    assert t.num_params() == 7_615_616_512
    assert t.kv_bytes_per_token(2) == 57_344
    three_b = dict(SEVEN_B, hidden_size=2048, intermediate_size=11008, num_hidden_layers=36, num_attention_heads=16,
                   num_key_value_heads=2, vocab_size=151936, tie_word_embeddings=True)
    t3 = Qwen25VLConfig.from_dict(three_b).text_config
    assert t3.num_params() == 3_085_938_688
    assert t3.kv_bytes_per_token(2) == 36_864  # reference tests/test_components.py:84-89


def test_from_pretrained_and_roundtrip(tmp_path):
    with pytest.raises(FileNotFoundError):
        Qwen25VLConfig.from_pretrained(str(tmp_path))
    cfg = Qwen25VLConfig.from_dict(TINY_B)
    (tmp_path / "config.json").write_text(json.dumps(cfg.to_dict()))
    again = Qwen25VLConfig.from_pretrained(str(tmp_path))
    assert again.text_config == cfg.text_config
    assert Qwen25VLConfig.from_pretrained(os.path.join(str(tmp_path), "config.json")).text_config == cfg.text_config


def test_registry():
    assert "Qwen2_5_VLForConditionalGeneration" in known_architectures()
    with pytest.raises(KeyError) as err:
        resolve_architecture("NoSuchModel")
    assert "Qwen2_5_VLForConditionalGeneration" in str(err.value)
    with pytest.raises(ValueError):
        register_architecture("Qwen2_5_VLForConditionalGeneration", lambda c: None)
    raw = dict(TINY_C, architectures=["NoSuchModel"])
    with pytest.raises(KeyError):
        build_model(Qwen25VLConfig.from_dict(raw), device="meta")


def test_model_structure_from_config():
    model = build_model(Qwen25VLConfig.from_dict(TINY_B), device="meta")
    groups = model.cache_groups()
    # layer 0 sees everything, layers 1 and 2 share a window: two groups with pages of their own
    assert [(g.need.window, g.num_layers) for g in groups] == [(None, 1), (16, 2)]
    names = model.expected_tensors()
    assert names["layers.2.self_attn.k_proj.weight"].shape == (48, 144)
    assert names["layers.0.mlp.down_proj.weight"].shape == (144, 352)
    assert names["lm_head.weight"].shape == (509, 144) and names["norm.weight"].role == "vector"


def test_layer_schedule_repeats_and_shares_cache():
    raw = json.loads(json.dumps(TINY_A))
    raw["text_config"]["num_hidden_layers"] = 3
    raw["text_config"]["layer_schedule"] = [0, 1, 0, {"layer": 2, "cache_from": 1}]
    model = build_model(Qwen25VLConfig.from_dict(raw), device="meta")
    assert model.entry_cache_layer == [0, 1, 2, 1] and model.entry_writes == [True, True, True, False]
    assert model.cache_groups()[0].num_layers == 3
    names = model.expected_tensors()
    assert "layers.2.self_attn.q_proj.weight" in names and "layers.2.self_attn.k_proj.weight" not in names


def test_engine_config_validation():
    EngineConfig(dtype="bfloat16")
    for bad in (dict(block_size=0), dict(block_size=24), dict(max_num_seqs=0), dict(preemption="swap"),
                dict(dtype="float16"), dict(max_num_batched_tokens=0)):
        with pytest.raises(ValueError):
            EngineConfig(**bad)


def test_command_line_is_reachable_as_a_module(tmp_path):
    """``python -m qwen25vl_lite_amd`` is the command line; make-random writes a model folder."""
    import json
    import subprocess
    import sys

    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    cfg = tmp_path / "config.json"
    cfg.write_text(json.dumps(TINY_A))
    out = tmp_path / "m"
    res = subprocess.run([sys.executable, "-m", "qwen25vl_lite_amd", "make-random", "--config", str(cfg),
                          "--out", str(out), "--seed", "3"], cwd=root, capture_output=True, text=True, timeout=120)
    assert res.returncode == 0, res.stderr
    assert (out / "config.json").exists() and (out / "model.safetensors").exists()
