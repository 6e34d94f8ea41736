"""Trace replay: feed given token ids through the model step by step and write logits.

It samples nothing and schedules nothing; it drives the same model, step function, cache and
kernels that generation uses.  The reference's nearest thing is the manual driving of its
runner in its tests (reference tests/test_chunked_prefill.py:44-68, 130-146).

Steps arrive as JSON lines::

    {"step": 0, "entries": [{"id": "a", "tokens": [5, 17, 3], "want": [0, 2]}], "end": []}

An entry may also carry ``"positions": [[t...], [h...], [w...]]`` for its tokens and
``"rope_delta"``, which shifts the text positions of its later tokens.  For a step in which
logits are wanted, ``<out>/<step>.f32`` holds them as little-endian float32 ``[wanted, vocab]``.
"""

from __future__ import annotations

import argparse
import json
import os
import sys
from typing import Dict, IO, Optional

import torch

from ..config import EngineConfig, dtype_from_name, load_config
from ..models import build_model
from ..weights import load_weights
from .batch import StepEntry
from .runner import ModelRunner

__all__ = ["Replayer", "main"]

ROUND_TO = 64  # a request's token count is rounded up to a multiple of this when sizing the pool


class Replayer:
    def __init__(self, model_dir: str, dtype: str, max_tokens: int, block_size: int = 16, max_live: int = 8):
        cfg = load_config(model_dir)
        run_dtype = dtype_from_name(dtype)
        model = build_model(cfg, run_dtype, "cuda:0")
        load_weights(model_dir, model)
        max_tokens = max(ROUND_TO, (int(max_tokens) + ROUND_TO - 1) // ROUND_TO * ROUND_TO)
        # Pages for max_tokens tokens; a page size that does not divide the rounding unit can leave
        # each live request one page short of that, so it gets one more per request.
        num_blocks = (max_tokens + block_size - 1) // block_size + (max_live if ROUND_TO % block_size else 0)
        ecfg = EngineConfig(
            num_blocks=num_blocks, block_size=block_size, max_num_seqs=max_live,
            max_num_batched_tokens=max_tokens, max_model_len=max_tokens, enable_prefix_cache=False,
            dtype=run_dtype, device="cuda:0")
        self.runner = ModelRunner(model, ecfg)
        self.rope_delta: Dict[object, int] = {}

    def step(self, record: dict) -> Optional[torch.Tensor]:
        cache = self.runner.cache
        entries = []
        for e in record.get("entries", []):
            rid = e["id"]
            if rid not in cache.requests:
                self.runner.admit(rid)
                self.rope_delta[rid] = 0
            if "rope_delta" in e:
                self.rope_delta[rid] = int(e["rope_delta"])
                cache.records.rope_delta[cache.slot_of(rid)] = self.rope_delta[rid]
            entries.append(StepEntry(req_id=rid, tokens=list(e["tokens"]), start=cache.num_tokens(rid),
                                     want=list(e.get("want", [])), positions=e.get("positions"),
                                     rope_delta=self.rope_delta[rid]))
        logits = None
        if entries:
            logits = self.runner.execute(entries)
        for rid in record.get("end", []):
            if rid in cache.requests:
                self.runner.release(rid)
                self.rope_delta.pop(rid, None)
        return logits

    def run(self, lines: IO[str], out_dir: str, done: IO[str]) -> None:
        os.makedirs(out_dir, exist_ok=True)
        for line in lines:
            line = line.strip()
            if not line:
                continue
            record = json.loads(line)
            logits = self.step(record)
            if logits is not None and logits.shape[0] > 0:
                host = logits.to(torch.float32).cpu().contiguous()
                host.numpy().astype("<f4", copy=False).tofile(os.path.join(out_dir, f"{record['step']}.f32"))
            else:
                torch.cuda.synchronize()
            done.write(f"done {record['step']}\n")
            done.flush()


def main(argv=None) -> int:
    parser = argparse.ArgumentParser(prog="trace_run", description="replay a trace of steps and write logits")
    parser.add_argument("--model", required=True, help="folder with config.json and model.safetensors")
    parser.add_argument("--dtype", required=True, choices=["bfloat16", "float32"])
    parser.add_argument("--out", required=True, help="folder for <step>.f32")
    parser.add_argument("--max-tokens", type=int, required=True,
                        help="most tokens live requests hold at any time (each rounded up to a multiple of 64)")
    parser.add_argument("--block-size", type=int, default=16)
    args = parser.parse_args(argv)
    replayer = Replayer(args.model, args.dtype, args.max_tokens, args.block_size)
    replayer.run(sys.stdin, args.out, sys.stdout)
    return 0
