"""Shared fixtures: tiny configurations, model folders with random weights, the GPU marker."""

import os
import sys

import pytest
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)
if os.path.dirname(os.path.abspath(__file__)) not in sys.path:
    sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs an MI355X (run on the GPU box with -m gpu)")


def pytest_collection_modifyitems(config, items):
    if torch.cuda.is_available():
        return
    skip = pytest.mark.skip(reason="no GPU here")
    for item in items:
        if "gpu" in item.keywords:
            item.add_marker(skip)


# Tiny configurations that differ in every size and option.
TINY_A = {
    "architectures": ["Qwen2_5_VLForConditionalGeneration"],
    "model_type": "qwen2_5_vl",
    "tie_word_embeddings": True,
    "rope_scaling": {"type": "mrope", "mrope_section": [2, 3, 3]},
    "text_config": {
        "hidden_size": 64, "intermediate_size": 128, "num_hidden_layers": 2, "num_attention_heads": 4,
        "num_key_value_heads": 2, "vocab_size": 256, "rope_theta": 10000.0, "rms_norm_eps": 1e-6,
        "use_sliding_window": False, "sliding_window": 32768,
    },
}

TINY_B = {
    "architectures": ["Qwen2_5_VLForConditionalGeneration"],
    "model_type": "qwen2_5_vl",
    "tie_word_embeddings": False,
    "text_config": {
        "hidden_size": 144, "intermediate_size": 352, "num_hidden_layers": 3, "num_attention_heads": 6,
        "num_key_value_heads": 2, "vocab_size": 509, "rope_theta": 1000000.0, "rms_norm_eps": 1e-5,
        "use_sliding_window": True, "sliding_window": 16, "max_window_layers": 1,
        "rope_scaling": {"type": "mrope", "mrope_section": [4, 4, 4]},
    },
}

# Head size in steps of 16 (the matrix-core attention path), one key/value head, five query
# heads per group, an explicit head_dim that is not hidden_size / heads, a longer window.
TINY_C = {
    "architectures": ["Qwen2_5_VLForConditionalGeneration"],
    "tie_word_embeddings": False,
    "hidden_size": 200, "intermediate_size": 296, "num_hidden_layers": 2, "num_attention_heads": 5,
    "num_key_value_heads": 1, "head_dim": 48, "vocab_size": 300, "rope_theta": 500000.0, "rms_norm_eps": 2e-6,
    "use_sliding_window": True, "sliding_window": 40, "max_window_layers": 1,
    "rope_scaling": {"type": "mrope", "mrope_section": [10, 6, 8]},
}

# The 7B decoder's head geometry (28 query heads on 4 key/value heads of 128 channels, its rotation
# sections) at a narrow width: the attention of a long context at the sizes the dispatch rules
# were measured for, cheap enough for the plain implementation.
TINY_D = {
    "architectures": ["Qwen2_5_VLForConditionalGeneration"],
    "tie_word_embeddings": True,
    "hidden_size": 256, "intermediate_size": 520, "num_hidden_layers": 2, "num_attention_heads": 28,
    "num_key_value_heads": 4, "head_dim": 128, "vocab_size": 300, "rope_theta": 1000000.0, "rms_norm_eps": 1e-6,
    "use_sliding_window": False, "sliding_window": 32768,
    "rope_scaling": {"type": "mrope", "mrope_section": [16, 24, 24]},
}

TINY = {"A": (TINY_A, 0), "B": (TINY_B, 1), "C": (TINY_C, 2), "D": (TINY_D, 3)}


@pytest.fixture(scope="session")
def model_dirs(tmp_path_factory):
    """Model folders (config.json, model.safetensors) of the tiny configurations, weights stored
    in bfloat16 so that the float32 and the bfloat16 runs read the same values."""
    from qwen25vl_lite_amd import Qwen25VLConfig, write_random_model

    from qwen25vl_lite_amd.weights import SafetensorsFile, write_safetensors

    out = {}
    for name, (raw, seed) in TINY.items():
        d = str(tmp_path_factory.mktemp(f"tiny_{name}"))
        write_random_model(Qwen25VLConfig.from_dict(raw), d, seed, dtype=torch.bfloat16)
        out[name] = d
        # The same model with query and key projections scaled up: N(0, 0.02) weights give nearly
        # uniform attention, which would hide a wrong key, window edge or page; these make the
        # softmax peaked so that such faults show in the logits.
        sharp = str(tmp_path_factory.mktemp(f"tiny_{name}_sharp"))
        with SafetensorsFile(os.path.join(d, "model.safetensors")) as f:
            tensors = {k: f.tensor(k).clone() for k in f.keys()}
        for k in tensors:
            if ".q_proj." in k or ".k_proj." in k:
                tensors[k] = (tensors[k].float() * 7.0).to(torch.bfloat16)
        write_safetensors(os.path.join(sharp, "model.safetensors"), tensors)
        with open(os.path.join(d, "config.json")) as src, open(os.path.join(sharp, "config.json"), "w") as dst:
            dst.write(src.read())
        out[name + "_sharp"] = sharp
    return out
