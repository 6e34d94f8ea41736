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


# All 28 layers of the 7B decoder at a narrow width: what depth does to bfloat16.  Random weights give
# small, flat logits, and 28 layers of bfloat16 roundings move them by a few hundredths of the largest
# one whoever does the rounding, so a fixed bound against float32 arithmetic says little here.  The
# statement that holds at any depth: the engine's bfloat16 logits are no further from float32
# arithmetic than those of the plain implementation with bfloat16 storage, and they name float32's
# token about as often.
DEEP = {
    "architectures": ["Qwen2_5_VLForConditionalGeneration"], "model_type": "qwen2_5_vl", "tie_word_embeddings": False,
    "hidden_size": 320, "intermediate_size": 864, "num_hidden_layers": 28, "num_attention_heads": 5,
    "num_key_value_heads": 1, "vocab_size": 1531, "rope_theta": 1000000.0, "rms_norm_eps": 1e-6,
    "sliding_window": 32768, "use_sliding_window": False,
    "rope_scaling": {"type": "mrope", "mrope_section": [8, 12, 12]},
}
DEEP_LENGTHS = [90, 41]


def test_full_depth_bfloat16_is_as_close_to_float32_as_plain_bfloat16(tmp_path):
    from qwen25vl_lite_amd import Qwen25VLConfig, write_random_model
    from qwen25vl_lite_amd.engine.replay import Replayer
    d = str(tmp_path / "deep")
    write_random_model(Qwen25VLConfig.from_dict(DEEP), d, seed=11, dtype=torch.bfloat16)
    requests = {f"d{i}": random_tokens(n, DEEP["vocab_size"], 40 + i) for i, n in enumerate(DEEP_LENGTHS)}
    cfg, weights = plain_read_config(d), plain_read_weights(d)
    exact = {rid: plain_forward(cfg, weights, toks, None, lambda x: x) for rid, toks in requests.items()}
    stored = {rid: plain_forward(cfg, weights, toks, None, as_bfloat16) for rid, toks in requests.items()}

    def distance(rows):   # per position: largest difference from float32 arithmetic over the largest logit; and whether the token agrees
        errs, same = [], 0
        for (rid, pos), row in rows.items():
            want = exact[rid][pos]
            errs.append(((row - want).abs().max() / want.abs().max()).item())
            same += int(row.argmax().item() == want.argmax().item())
        return max(errs), sum(errs) / len(errs), same

    plain = distance({(rid, pos): stored[rid][pos] for rid, toks in requests.items() for pos in range(len(toks))})
    total = sum(DEEP_LENGTHS)
    rp = Replayer(d, "float32", round64(max(DEEP_LENGTHS)))
    f32 = distance(run_steps(rp, tail_trace(requests)))
    assert f32[0] < 1e-4 and f32[2] >= total - 1, f"float32 engine against the plain implementation: {f32}"
    for name, steps_of in (("whole", whole_trace), ("tail", tail_trace)):
        rp = Replayer(d, "bfloat16", round64(max(DEEP_LENGTHS)))
        got = run_steps(rp, steps_of(requests))
        assert len(got) == total
        engine = distance(got)
        print(f"28 layers, bfloat16, {name}: engine worst {engine[0]:.3e} mean {engine[1]:.3e} same token {engine[2]}/{total}; "
              f"plain with bfloat16 storage worst {plain[0]:.3e} mean {plain[1]:.3e} same token {plain[2]}/{total}")
        assert engine[1] <= 1.25 * plain[1], f"{name}: mean distance {engine[1]:.3e} against the plain implementation's {plain[1]:.3e}"
        assert engine[0] <= 1.5 * plain[0], f"{name}: worst distance {engine[0]:.3e} against the plain implementation's {plain[0]:.3e}"
        assert engine[2] >= plain[2] - total // 10, f"{name}: {engine[2]} tokens agree with float32, the plain implementation's {plain[2]}"
