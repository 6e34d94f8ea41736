"""The engine at the layer sizes of the 7B text decoder (two layers of them): the shapes the
decode kernels are tuned for, a vocabulary and widths that are no power of two, 7 query heads per
key/value head, head size 128."""

import pytest
import torch

from plain_model import as_bfloat16, plain_forward, plain_read_config, plain_read_weights
from replay_util import mixed_trace, random_tokens, round64, run_steps, tail_trace, whole_trace

pytestmark = pytest.mark.gpu

WIDE = {
    "architectures": ["Qwen2_5_VLForConditionalGeneration"], "model_type": "qwen2_5_vl", "tie_word_embeddings": False,
    "hidden_size": 3584, "intermediate_size": 18944, "num_hidden_layers": 2, "num_attention_heads": 28,
    "num_key_value_heads": 4, "vocab_size": 152064, "rope_theta": 1000000.0, "rms_norm_eps": 1e-6,
    "sliding_window": 32768, "use_sliding_window": False,
    "rope_scaling": {"type": "mrope", "mrope_section": [16, 24, 24]},
}
LENGTHS = [70, 45, 9]


@pytest.fixture(scope="module")
def wide(tmp_path_factory):
    from qwen25vl_lite_amd import Qwen25VLConfig, write_random_model
    d = str(tmp_path_factory.mktemp("wide"))
    write_random_model(Qwen25VLConfig.from_dict(WIDE), d, seed=5, dtype=torch.bfloat16)
    requests = {f"w{i}": random_tokens(n, WIDE["vocab_size"], 900 + i) for i, n in enumerate(LENGTHS)}
    cfg, weights = plain_read_config(d), plain_read_weights(d)
    ref = {"float32": {rid: plain_forward(cfg, weights, toks, None, lambda x: x) for rid, toks in requests.items()},
           "bfloat16": {rid: plain_forward(cfg, weights, toks, None, as_bfloat16) for rid, toks in requests.items()}}
    del weights
    return d, requests, ref


def _worst(got, ref, dtype, what):
    worst = 0.0
    for (rid, pos), row in got.items():
        want = ref[rid][pos]
        if dtype == "float32":
            assert torch.allclose(row, want, atol=1e-4, rtol=1e-3), f"{what}: {rid} position {pos}: " \
                f"{(row - want).abs().max().item():.3e}"
            worst = max(worst, (row - want).abs().max().item())
        else:
            err = ((row - want).abs().max() / want.abs().max()).item()
            assert err < 2e-2, f"{what}: {rid} position {pos}: error {err:.3e}"
            worst = max(worst, err)
    return worst


@pytest.mark.parametrize("dtype", ["bfloat16", "float32"])
def test_wide_layers_whole_decoded_and_mixed(wide, dtype):
    from qwen25vl_lite_amd.engine.replay import Replayer
    d, requests, ref = wide
    total = sum(LENGTHS)
    rp = Replayer(d, dtype, round64(max(LENGTHS)))
    got = run_steps(rp, whole_trace(requests))
    assert len(got) == total
    print(dtype, "whole", _worst(got, ref[dtype], dtype, "whole"))
    got = run_steps(rp, tail_trace(requests))        # the last 32 tokens one by one: the decode kernels
    assert len(got) == total
    print(dtype, "tail", _worst(got, ref[dtype], dtype, "tail"))
    steps, peak = mixed_trace(requests, seed=3, max_live=3)
    rp = Replayer(d, dtype, peak)
    got = run_steps(rp, steps)                       # portions beside decoded tokens, two or three rows of them
    assert len(got) == total
    print(dtype, "mixed", _worst(got, ref[dtype], dtype, "mixed"))
    assert rp.runner.cache.pages_in_use() == [0] * len(rp.runner.cache.groups)
