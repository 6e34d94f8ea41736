"""Command line: ``generate``, ``bench``, ``replay`` and ``make-random``.

``generate`` and ``bench`` take the reference's options with the reference's meanings
(reference src/qwen25vl_lite/cli.py:634-713): ``--model --device --dtype``, the engine options
``--num-blocks --block-size --max-num-seqs --max-num-batched-tokens --max-model-len
--no-prefix-cache --no-chunked-prefill --preemption``, and for generate ``--prompt-token-ids
"1,2,3" --temperature --top-p --max-tokens``.  Options of parts that are not built here
(quantised weights and cache, vision tiers, pruning, graph capture flags, backend pinning) do
not exist.  Added: ``--top-k --seed --ignore-eos``, several prompts separated by ``;``, and
``--random-weights SEED`` to run a configuration without stored weights.
"""

from __future__ import annotations

import argparse
import json
import sys
import time
from typing import List, Optional

__all__ = ["main", "build_parser"]


def _llm(args):
    from .config import load_config
    from .engine.llm import LLM

    if "cuda" not in args.device:
        raise SystemExit("this engine runs on the GPU only: --device must be cuda or cuda:N")
    device = args.device if ":" in args.device else args.device + ":0"
    options = dict(
        num_blocks=args.num_blocks, block_size=args.block_size, max_num_seqs=args.max_num_seqs,
        max_num_batched_tokens=args.max_num_batched_tokens, max_model_len=args.max_model_len,
        enable_prefix_cache=not args.no_prefix_cache, enable_chunked_prefill=not args.no_chunked_prefill,
        preemption=args.preemption, hip_graph=args.cuda_graph, decode_lookahead=args.decode_lookahead)
    t0 = time.time()
    if args.random_weights is not None:
        llm = LLM(load_config(args.model), args.dtype, random_seed=args.random_weights,
                  device=device, **options)
    else:
        llm = LLM(args.model, args.dtype, device=device, **options)
    print(f"loaded {len(llm.model.expected_tensors())} tensors in {time.time() - t0:.1f}s", file=sys.stderr)
    return llm


def cmd_generate(args) -> int:
    from .sampling.params import SamplingParams

    if not args.prompt_token_ids:
        # reference cli.py:271-274
        print("--prompt-token-ids is required (this CLI does not bundle a tokenizer)", file=sys.stderr)
        return 2
    prompts = _read_prompts(args.prompt_token_ids)
    llm = _llm(args)
    params = SamplingParams(temperature=args.temperature, top_p=args.top_p, top_k=args.top_k,
                            max_tokens=args.max_tokens, seed=args.seed, ignore_eos=args.ignore_eos)
    outs = llm.generate(prompts, params)
    for out in outs:
        print(out.output_token_ids)
    return 0


def _read_prompts(arg: str):
    """``"1,2,3"``, several prompts separated by ``;``, or the path of a JSON file that holds a
    list of token ids or a list of such lists."""
    import json
    import os

    if os.path.isfile(arg):
        with open(arg) as f:
            data = json.load(f)
        if data and not isinstance(data[0], list):
            data = [data]
        return [[int(t) for t in prompt] for prompt in data]
    return [[int(t) for t in part.split(",") if t.strip()] for part in arg.split(";")]


def cmd_bench(args) -> int:
    """One prompt of ``--prompt-tokens`` ids, greedy, ``--max-tokens`` generated
    (reference cli.py:246-264)."""
    from .sampling.params import SamplingParams

    llm = _llm(args)
    vocab = llm.model.spec.vocab_size
    prompt = [(1000 + i) % vocab for i in range(args.prompt_tokens)]
    params = SamplingParams(temperature=0.0, max_tokens=args.max_tokens, ignore_eos=True)
    t0 = time.time()
    out = llm.generate([prompt], params)[0]
    elapsed = time.time() - t0
    n_out = len(out.output_token_ids)
    print(f"prefill {args.prompt_tokens} tokens + decode {n_out} tokens in {elapsed:.2f}s")
    print(f"  ttft {out.metrics['ttft_s'] * 1e3:.1f} ms; decode throughput: "
          f"{(n_out - 1) / max(1e-9, elapsed - out.metrics['ttft_s']):.1f} tok/s")
    print(f"  stats: {llm.engine.stats()}")
    return 0


def cmd_replay(args) -> int:
    from .engine.replay import main as replay_main

    return replay_main(["--model", args.model, "--dtype", args.dtype, "--out", args.out,
                        "--max-tokens", str(args.max_tokens), "--block-size", str(args.block_size)])


def cmd_make_random(args) -> int:
    from .config import dtype_from_name, load_config
    from .weights import write_random_model

    cfg = load_config(args.config)
    write_random_model(cfg, args.out, args.seed, std=args.std, dtype=dtype_from_name(args.dtype))
    print(f"wrote {args.out}/config.json and model.safetensors (seed {args.seed})")
    return 0


def build_parser() -> argparse.ArgumentParser:
    parser = argparse.ArgumentParser(prog="qwen25vl-lite", description=__doc__,
                                     formatter_class=argparse.RawDescriptionHelpFormatter)
    sub = parser.add_subparsers(dest="command", required=True)

    def add_model_opts(p):
        p.add_argument("--model", required=True, help="folder with config.json and model.safetensors")
        p.add_argument("--device", default="cuda", help="cuda, cuda:0 ... (there is no CPU path)")
        p.add_argument("--dtype", default="float32", choices=["float32", "bfloat16"])
        p.add_argument("--random-weights", type=int, default=None, metavar="SEED",
                       help="ignore stored weights and draw random ones from this seed")

    def add_engine_opts(p):
        p.add_argument("--num-blocks", type=int, default=2048)
        p.add_argument("--block-size", type=int, default=16)
        p.add_argument("--max-num-seqs", type=int, default=8)
        p.add_argument("--max-num-batched-tokens", type=int, default=4096)
        p.add_argument("--max-model-len", type=int, default=32768)
        p.add_argument("--no-prefix-cache", action="store_true")
        p.add_argument("--no-chunked-prefill", action="store_true")
        p.add_argument("--preemption", default="recompute", choices=["recompute"])
        p.add_argument("--decode-lookahead", action="store_true",
                       help="with --cuda-graph: queue the next decode step before the running one's tokens "
                            "have reached the host")
        p.add_argument("--cuda-graph", action="store_true",
                       help="replay decode steps from a captured graph (a HIP graph here; the option keeps "
                            "the reference's name): a decode step is launch-bound, this removes the host's "
                            "dispatch cost")

    p = sub.add_parser("generate", help="one-shot generation from token ids")
    add_model_opts(p)
    add_engine_opts(p)
    p.add_argument("--prompt-token-ids", default=None, help='"1,2,3"; several prompts separated by ";"; or a JSON file with a list of lists')
    p.add_argument("--temperature", type=float, default=0.0)
    p.add_argument("--top-p", type=float, default=1.0)
    p.add_argument("--top-k", type=int, default=-1)
    p.add_argument("--max-tokens", type=int, default=64)
    p.add_argument("--seed", type=int, default=None)
    p.add_argument("--ignore-eos", action="store_true")
    p.set_defaults(func=cmd_generate)

    p = sub.add_parser("bench", help="run a short benchmark")
    add_model_opts(p)
    add_engine_opts(p)
    p.add_argument("--prompt-tokens", type=int, default=512)
    p.add_argument("--max-tokens", type=int, default=64)
    p.set_defaults(func=cmd_bench)

    p = sub.add_parser("replay", help="replay a trace of steps from standard input and write logits")
    p.add_argument("--model", required=True)
    p.add_argument("--dtype", required=True, choices=["float32", "bfloat16"])
    p.add_argument("--out", required=True)
    p.add_argument("--max-tokens", type=int, required=True)
    p.add_argument("--block-size", type=int, default=16)
    p.set_defaults(func=cmd_replay)

    p = sub.add_parser("make-random", help="write a model folder with random weights")
    p.add_argument("--config", required=True, help="config.json (or a folder that holds one)")
    p.add_argument("--out", required=True)
    p.add_argument("--seed", type=int, default=0)
    p.add_argument("--std", type=float, default=0.02)
    p.add_argument("--dtype", default="bfloat16", choices=["float32", "bfloat16"])
    p.set_defaults(func=cmd_make_random)
    return parser


def main(argv: Optional[List[str]] = None) -> int:
    args = build_parser().parse_args(argv)
    return int(args.func(args))


if __name__ == "__main__":
    raise SystemExit(main())
