"""The benchmark's own model at its full depth: the Qwen2.5-VL-7B text decoder's sizes, all 28
layers, random weights, against the plain implementation (which runs on the host's CPU with the
weights in float32: about 30 GB of host memory, under a minute).

float32: the reference's own criterion for logits, and bit-identical logits however the tokens
are cut.  bfloat16: no fixed bound against float32 arithmetic is claimed at this depth (random
weights give small, flat logits, and 28 layers of bfloat16 storage move them by a few per cent of
the largest); what is held is that the engine is no further from float32 arithmetic than the
plain implementation is when it stores its activations in bfloat16, and names float32's token as
often.  The figures are printed (run with -s); `profiles/accuracy_7b_full_depth.txt` keeps a copy.
"""

import pytest
import torch

import bench
from plain_model import as_bfloat16, plain_forward, plain_read_config, plain_read_weights
from replay_util import mixed_trace, random_tokens, run_steps, tail_trace, whole_trace

pytestmark = pytest.mark.gpu


def test_all_28_layers_at_7b_sizes(tmp_path):
    from qwen25vl_lite_amd import Qwen25VLConfig, write_random_model
    from qwen25vl_lite_amd.engine.replay import Replayer
    d = str(tmp_path / "full7b")
    cfg = Qwen25VLConfig.from_dict(bench.decoder_config())
    assert cfg.text_config.num_hidden_layers == 28 and cfg.text_config.hidden_size == 3584
    write_random_model(cfg, d, seed=11, dtype=torch.bfloat16)
    requests = {"a": random_tokens(48, 152064, 1), "b": random_tokens(20, 152064, 2)}
    pc, pw = plain_read_config(d), plain_read_weights(d)
    truth = {rid: plain_forward(pc, pw, toks, None) for rid, toks in requests.items()}
    plain16 = {rid: plain_forward(pc, pw, toks, None, as_bfloat16) for rid, toks in requests.items()}
    del pw
    traces = (("whole", whole_trace(requests)), ("last 16 one by one", tail_trace(requests, 16)),
              ("mixed", mixed_trace(requests, seed=1, max_live=2)[0]))

    def worst(got, ref):   # worst error of a row, of the largest logit of that row
        return max(((row - ref[rid][pos]).abs().max() / ref[rid][pos].abs().max()).item() for (rid, pos), row in got.items())

    def names_the_same(got, ref):
        return sum(int(row.argmax() == ref[rid][pos].argmax()) for (rid, pos), row in got.items())

    rp = Replayer(d, "float32", 128)
    first = None
    for what, steps in traces:
        got = run_steps(rp, steps)
        assert len(got) == 68
        err = max((row - truth[rid][pos]).abs().max().item() for (rid, pos), row in got.items())
        print(f"float32, {what}: worst error {err:.3e} ({worst(got, truth):.3e} of the largest logit)")
        for (rid, pos), row in got.items():
            assert torch.allclose(row, truth[rid][pos], atol=1e-3, rtol=1e-3), (what, rid, pos)
        if first is None:
            first = got
        else:   # however the tokens are cut and batched: the very same bits
            assert all(torch.equal(row, first[key]) for key, row in got.items()), what
    del rp
    torch.cuda.empty_cache()

    flat16 = {(rid, pos): plain16[rid][pos] for rid in requests for pos in range(len(requests[rid]))}
    plain_err, plain_same = worst(flat16, truth), names_the_same(flat16, truth)
    print(f"plain implementation with bfloat16 storage against float32 arithmetic: worst {plain_err:.3e} of the "
          f"largest logit, names float32's token in {plain_same} of 68 places")
    rp = Replayer(d, "bfloat16", 128)
    for what, steps in traces:
        got = run_steps(rp, steps)
        assert len(got) == 68
        err, same = worst(got, truth), names_the_same(got, truth)
        print(f"bfloat16, {what}: {err:.3e} of the largest logit from float32 arithmetic, "
              f"{worst(got, plain16):.3e} from the plain implementation with bfloat16 storage; names float32's "
              f"token in {same} of 68 places")
        assert err < 1.3 * plain_err + 5e-3, what
        assert same >= plain_same - 3, what
