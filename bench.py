"""Decode and prefill throughput of the engine on one MI355X.

    python bench.py --gpus 1 --steps K --warmup W

The model has the layer sizes of the Qwen2.5-VL-7B text decoder
with random weights N(0, 0.02) in bfloat16; token ids are seeded uniform random integers.  A
"step" is one decode step of the scheduler: every live request gets its next token through the
engine's own path (batch building, the step function over the paged cache, sampling on the
device, the copy of the sampled ids to the host).  The default batch is 8 requests with
512-token prompts.  The same run also measures decoding at batch 1 and 64 and a 2,048-token
prefill, and prints one JSON line.
"""

from __future__ import annotations

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0          # MI355X published HBM3E bandwidth
MFMA_PEAK = {"bf16": 2.5e15, "fp32": 157.3e12}


SIZES = {   # layer sizes of the Qwen2.5-VL 3B, 7B and 72B text decoders
    "3b": dict(hidden_size=2048, intermediate_size=11008, num_hidden_layers=36, num_attention_heads=16,
               num_key_value_heads=2, vocab_size=151936, tie_word_embeddings=True),
    "7b": dict(hidden_size=3584, intermediate_size=18944, num_hidden_layers=28, num_attention_heads=28,
               num_key_value_heads=4, vocab_size=152064, tie_word_embeddings=False),
    "72b": dict(hidden_size=8192, intermediate_size=29568, num_hidden_layers=80, num_attention_heads=64,
                num_key_value_heads=8, vocab_size=152064, tie_word_embeddings=False),
}


def decoder_config(layers=None, size="7b"):
    """The 7B text decoder (or another of SIZES) as a config.json dictionary."""
    raw = {
        "architectures": ["Qwen2_5_VLForConditionalGeneration"], "model_type": "qwen2_5_vl",
        "rope_theta": 1000000.0, "rms_norm_eps": 1e-6, "sliding_window": 32768, "use_sliding_window": False,
        "max_position_embeddings": 8192, "rope_scaling": {"type": "mrope", "mrope_section": [16, 24, 24]},
    }
    raw.update(SIZES[size])
    if layers:
        raw["num_hidden_layers"] = int(layers)
    return raw


def step_bytes(t, batch, ctx, bytes_per_value=2):
    """Bytes a decode step has to read: every weight it uses once (all layers and the head; of the
    embedding only the rows looked up) and the keys and values of the live requests."""
    h, hd, inter = t.hidden_size, t.head_dim, t.intermediate_size
    nh, nkv = t.num_attention_heads, t.num_key_value_heads
    per_layer = h * (nh + 2 * nkv) * hd + nh * hd * h + 3 * h * inter
    weights = (per_layer * t.num_hidden_layers + t.vocab_size * h) * bytes_per_value
    kv = batch * ctx * t.kv_bytes_per_token(bytes_per_value)
    return weights + kv


def prefill_flops(t, tokens):
    h, hd, inter = t.hidden_size, t.head_dim, t.intermediate_size
    nh, nkv = t.num_attention_heads, t.num_key_value_heads
    per_layer = h * (nh + 2 * nkv) * hd + nh * hd * h + 3 * h * inter
    linear = 2.0 * tokens * per_layer * t.num_hidden_layers
    attention = 4.0 * nh * hd * (tokens * (tokens + 1) / 2) * t.num_hidden_layers   # causal: QK^T and PV
    head = 2.0 * t.vocab_size * h                                                   # one row
    return linear + attention + head


def measure_attention(torch, size, lengths, page=16, reps=10):
    """The causal attention of one prompt of each length, through the kernel that prompt portions take
    (qwen25vl-lite_amd/csrc/attention_mfma.hip): mean time of ``reps`` calls and the rate of its
    4 * heads * head_dim * T (T + 1) / 2 flops."""
    from qwen25vl_lite_amd.ops import attention_mfma
    from qwen25vl_lite_amd.parts import StepContext

    nq, nkv = size["num_attention_heads"], size["num_key_value_heads"]
    hd = size["hidden_size"] // nq
    out = {"heads": nq, "kv_heads": nkv, "head_dim": hd, "page_size": page}
    for T in lengths:
        pages = (T + page - 1) // page
        torch.manual_seed(0)
        q = torch.randn(T, nq * hd, device="cuda").bfloat16()
        kc = torch.randn(pages, nkv, page, hd, device="cuda").bfloat16()
        vc = torch.randn(pages, nkv, hd, page, device="cuda").bfloat16()
        table = torch.randperm(pages, device="cuda").int().view(1, pages)
        none = torch.zeros(0, dtype=torch.int32, device="cuda")
        ar = torch.arange(T, dtype=torch.int32, device="cuda")
        step = StepContext(num_tokens=T, num_reqs=1, token_ids=none, positions=none, token_req=torch.zeros_like(ar),
                           token_seqpos=ar, cu_q=torch.tensor([0, T], dtype=torch.int32, device="cuda"),
                           ctx_len=torch.tensor([T], dtype=torch.int32, device="cuda"), req_slots=none, groups=[],
                           logit_rows=none, cu_q_host=[0, T], ctx_len_host=[T], max_q_len=T, max_ctx_len=T,
                           dtype=torch.bfloat16)
        for _ in range(3):
            attention_mfma.try_attention(q, kc, vc, table, step, nq, None, hd ** -0.5)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(reps):
            attention_mfma.try_attention(q, kc, vc, table, step, nq, None, hd ** -0.5)
        torch.cuda.synchronize()
        sec = (time.perf_counter() - t0) / reps
        out[f"tokens_{T}"] = {"us": round(sec * 1e6, 1), "tflops": round(4.0 * nq * hd * T * (T + 1) / 2 / sec / 1e12, 1)}
    return out


def measure_peaks(torch):
    """Plain read and copy rates, the matrix instruction's rate on registers and the cost of an empty
    launch, each the best of several repeats (kernels in qwen25vl-lite_amd/csrc/peaks.hip)."""
    import ctypes

    from qwen25vl_lite_amd.ops.kernels import _check, _fn, _stream

    c_int, c_ptr, c_ll = ctypes.c_int, ctypes.c_void_p, ctypes.c_longlong
    read = _fn("peaks", "qvl_peak_read", [c_ptr, c_ll, c_ptr, c_int, c_ptr])
    copy = _fn("peaks", "qvl_peak_copy", [c_ptr, c_ptr, c_ll, c_int, c_ptr])
    mfma = _fn("peaks", "qvl_peak_mfma", [c_ptr, c_int, c_int, c_int, c_ptr, c_ptr])
    empty = _fn("peaks", "qvl_peak_empty", [c_int, c_ptr])
    cus = torch.cuda.get_device_properties(0).multi_processor_count

    def best_ms(fn, reps=7):
        fn()
        torch.cuda.synchronize()
        best = 1e9
        for _ in range(reps):
            a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            a.record()
            fn()
            b.record()
            torch.cuda.synchronize()
            best = min(best, a.elapsed_time(b))
        return best

    out = {"device": torch.cuda.get_device_name(0), "compute_units": cus}
    flag = torch.zeros(64, dtype=torch.int32, device="cuda")
    for mib in (256, 1024, 4096):      # below and above the 256 MiB memory-side cache
        nbytes = mib << 20
        src = torch.empty(nbytes, dtype=torch.uint8, device="cuda").fill_(1)
        dst = torch.empty_like(src)
        ms = best_ms(lambda: _check(read(src.data_ptr(), nbytes // 16, flag.data_ptr(), cus * 8, _stream()), "read"))
        out[f"read_{mib}MiB_TBps"] = round(nbytes / ms / 1e9, 3)
        ms = best_ms(lambda: _check(copy(src.data_ptr(), dst.data_ptr(), nbytes // 16, cus * 8, _stream()), "copy"))
        out[f"copy_{mib}MiB_read_plus_write_TBps"] = round(2 * nbytes / ms / 1e9, 3)
        ms = best_ms(lambda: dst.copy_(src))
        out[f"device_to_device_copy_{mib}MiB_read_plus_write_TBps"] = round(2 * nbytes / ms / 1e9, 3)
        del src, dst
    # What the L2 caches deliver: every block reads the same 2 MiB (every XCD's L2 holds all of it) 64 times over.
    small = torch.empty(2 << 20, dtype=torch.uint8, device="cuda").fill_(1)
    reps = 8
    read_l2 = _fn("peaks", "qvl_peak_read_again", [c_ptr, c_ll, c_int, c_ptr, c_int, c_ptr])
    ms = best_ms(lambda: _check(read_l2(small.data_ptr(), small.numel() // 16, reps, flag.data_ptr(), cus * 8, _stream()), "read"))
    out["read_2MiB_by_every_block_from_L2_TBps"] = round(cus * 8 * small.numel() * reps / ms / 1e9, 3)
    # v_mfma_f32_16x16x32_bf16 back to back on registers, eight independent chains a wave.  Blocks of
    # 1,024 threads (four waves on every SIMD, which stay there together), two such blocks a compute
    # unit: the rate, the clock the shader really ran at (its own cycle counter against the constant
    # 100 MHz clock, read around one wave's loop) and the cycles between two of a wave's instructions.
    # A slow clock would show in the second figure, an instruction that cannot be issued faster in the third.
    iters, blocks = 4096, cus * 8
    clocks = torch.zeros(2 * blocks, dtype=torch.int64, device="cuda")
    for label, threads, per_cu in (("", 1024, 2), ("_one_block_of_8_waves_a_cu", 512, 1), ("_blocks_of_4_waves", 256, 8)):
        n = cus * per_cu
        launch = lambda: _check(mfma(flag.data_ptr(), iters, n, threads, clocks.data_ptr(), _stream()), "mfma")
        for _ in range(3):      # the clock settles under load
            launch()
        ms = best_ms(launch, reps=5)
        c = clocks.view(blocks, 2)[:n].double()
        cycles, wall_s = c[:, 0].median().item(), c[:, 1].median().item() / 100e6
        out[f"mfma_16x16x32_bf16{label}_PFLOPs"] = round(n * (threads // 64) * iters * 8 * 2.0 * 16 * 16 * 32 / ms / 1e12, 3)
        out[f"mfma_16x16x32_bf16{label}_shader_clock_GHz"] = round(cycles / wall_s / 1e9, 3)
        out[f"mfma_16x16x32_bf16{label}_cycles_between_a_waves_instructions"] = round(cycles / (iters * 8), 2)
    # an empty kernel many times in a row, from the host and from a graph
    n = 200
    ms = best_ms(lambda: _check(empty(n, _stream()), "empty"))
    out["empty_launch_from_host_us"] = round(ms * 1e3 / n, 2)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        _check(empty(n, _stream()), "empty")
    ms = best_ms(graph.replay)
    out["empty_launch_in_graph_us"] = round(ms * 1e3 / n, 2)
    return out


def main(argv=None) -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=128)
    ap.add_argument("--warmup", type=int, default=8)
    ap.add_argument("--batch", type=int, default=8)
    ap.add_argument("--prompt-tokens", type=int, default=512)
    ap.add_argument("--layers", type=int, default=None, help="fewer layers than the configuration has")
    ap.add_argument("--size", default="7b", choices=sorted(SIZES), help="layer sizes (default: the 7B decoder)")
    ap.add_argument("--dtype", default="bfloat16", choices=["bfloat16", "float32"])
    ap.add_argument("--no-points", action="store_true", help="skip batch 1 / 64 and the prefill")
    ap.add_argument("--prefill-only", action="store_true", help="only the 2,048-token prefill (for profiles)")
    ap.add_argument("--serving", action="store_true",
                    help="instead: continuous batching of 64 requests (prompts "
                         "of 64 to 2048 tokens, 32 to 512 generated, a quarter sharing a 1024-token prefix)")
    ap.add_argument("--peaks", action="store_true",
                    help="instead: what the device does at best (plain reads and copies, matrix instructions on "
                         "registers, an empty launch), for the fractions above to be read against")
    ap.add_argument("--attention", type=int, nargs="+", metavar="TOKENS",
                    help="instead: the prefill attention alone (one request of that many tokens in one step, the "
                         "chosen size's heads, bfloat16, pages in shuffled order), microseconds and TFLOP/s for each length")
    ap.add_argument("--no-graph", action="store_true", help="do not replay decode steps from a HIP graph")
    ap.add_argument("--no-lookahead", action="store_true",
                    help="do not queue the next decode step before the running one's tokens are known")
    ap.add_argument("--no-tune", action="store_true", help="do not let TunableOp choose the library's kernels")
    args = ap.parse_args(argv)
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        print(f"bench.py measures one GPU: this engine does not run on {args.gpus} GPUs (run with --gpus 1)")
        return 2

    import torch

    if args.peaks:
        print(json.dumps(measure_peaks(torch)))
        return 0

    if args.attention:
        print(json.dumps(measure_attention(torch, SIZES[args.size], args.attention)))
        return 0

    from qwen25vl_lite_amd import EngineConfig, LLMEngine, ModelRunner, Qwen25VLConfig, SamplingParams, build_model
    from qwen25vl_lite_amd.config import dtype_from_name
    from qwen25vl_lite_amd.weights import fill_random

    cfg = Qwen25VLConfig.from_dict(decoder_config(args.layers, args.size))
    t = cfg.text_config
    dtype = dtype_from_name(args.dtype)
    model = build_model(cfg, dtype, "cuda:0")
    fill_random(model, seed=0)
    torch.cuda.synchronize()

    page = 16
    max_ctx = 8192
    gen = torch.Generator().manual_seed(0)

    def make_engine(max_seqs, tokens_per_seq, budget):
        ecfg = EngineConfig(num_blocks=max_seqs * ((tokens_per_seq + page - 1) // page + 1), block_size=page,
                            max_num_seqs=max_seqs, max_num_batched_tokens=budget, max_model_len=max_ctx,
                            enable_prefix_cache=False, dtype=dtype, device="cuda:0", hip_graph=not args.no_graph,
                            decode_lookahead=not args.no_lookahead, tune_library_products=not args.no_tune)
        runner = ModelRunner(model, ecfg)
        return LLMEngine(runner, ecfg), runner

    def prompt(n):
        return torch.randint(0, t.vocab_size, (n,), generator=gen).tolist()

    def decode_rate(batch, steps, warmup):
        budget = max(4096, batch)
        # requests admitted first already decode while later prompts are still prefilled
        early = (batch * args.prompt_tokens + budget - 1) // budget + 2
        total = args.prompt_tokens + warmup + steps + early + 2
        engine, runner = make_engine(batch, total, budget)
        params = SamplingParams(temperature=0.0, max_tokens=warmup + steps + early + 1, ignore_eos=True)
        for _ in range(batch):
            engine.add_request(prompt(args.prompt_tokens), params)
        while any(s.remaining > 1 for s in engine.running) or engine.waiting:
            engine.step()                      # prefill
        for _ in range(warmup):
            engine.step()
        torch.cuda.synchronize()
        before = engine.stats_.decode_tokens
        t0 = time.perf_counter()
        for _ in range(steps):
            engine.step()
        torch.cuda.synchronize()
        dt = time.perf_counter() - t0
        tokens = engine.stats_.decode_tokens - before
        assert tokens == batch * steps, (tokens, batch, steps)
        ctx_mid = args.prompt_tokens + warmup + steps // 2
        runner.close()                         # the captured graphs go now, not when a collector runs
        del engine, runner
        torch.cuda.empty_cache()
        return tokens / dt, dt / steps * 1e3, ctx_mid

    def prefill_rate(tokens, reps=3):
        engine, runner = make_engine(2, tokens + 8, tokens)
        params = SamplingParams(temperature=0.0, max_tokens=1, ignore_eos=True)
        times = []
        for i in range(reps + 1):
            engine.add_request(prompt(tokens), params)
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            done = engine.step()               # the whole prompt in one step, then its first token is sampled
            torch.cuda.synchronize()
            assert len(done) == 1
            if i:
                times.append(time.perf_counter() - t0)
        runner.close()                         # the captured graphs go now, not when a collector runs
        del engine, runner
        torch.cuda.empty_cache()
        return min(times)

    if args.serving:
        import random
        rng = random.Random(0)
        shared = prompt(1024)
        reqs = []
        for i in range(64):
            n, out = rng.randint(64, 2048), rng.randint(32, 512)
            toks = (shared + prompt(max(0, n - 1024)))[:max(n, 1025)] if i % 4 == 0 else prompt(n)
            reqs.append((toks, out))
        need_pages = sum((len(tk) + out + page - 1) // page + 1 for tk, out in reqs)
        ecfg = EngineConfig(num_blocks=need_pages, block_size=page, max_num_seqs=64, max_num_batched_tokens=4096,
                            max_model_len=max_ctx, enable_prefix_cache=True, dtype=dtype, device="cuda:0",
                            hip_graph=not args.no_graph, decode_lookahead=not args.no_lookahead,
                            tune_library_products=not args.no_tune)

        runner = ModelRunner(model, ecfg)        # one runner, as a server has: its decode graphs stay

        def serve():
            if runner.cache.prefix_cache is not None:
                runner.cache.prefix_cache.clear()  # every run starts without remembered prompts
            engine = LLMEngine(runner, ecfg)
            for tk, out in reqs:
                engine.add_request(tk, SamplingParams(temperature=0.0, max_tokens=out, ignore_eos=True))
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            outs = engine.run_until_complete()
            torch.cuda.synchronize()
            return time.perf_counter() - t0, outs, engine.stats()

        from qwen25vl_lite_amd.ops import attention_mfma
        serve()                                   # library tuning, kernel builds, graph captures
        attention_mfma.taken.clear()
        sec, outs, stats = serve()
        generated = sum(len(o.output_token_ids) for o in outs)
        prompt_tokens = sum(len(tk) for tk, _ in reqs)
        print(json.dumps({
            "metric": f"continuous batching, generated tok/s (Qwen2.5-VL-{args.size.upper()} text decoder sizes, "
                      f"{args.dtype}, 64 requests)",
            "value": round(generated / sec, 1), "unit": "tokens/s", "seconds": round(sec, 3),
            "generated_tokens": generated, "prompt_tokens": prompt_tokens, "steps": int(stats["steps"]),
            "prefix_cache_hits": int(stats["prefix_cache_hits"]),
            "prefix_cache_tokens_saved": int(stats["prefix_cache_tokens_saved"]),
            "preemptions": int(stats["preemptions"]), "data": "synthetic",
            "attention_kernels": dict(attention_mfma.taken)}))
        return 0
    if args.prefill_only:
        sec = prefill_rate(2048)
        print(json.dumps({"prefill": {"value": round(2048 / sec, 1), "tokens": 2048, "ms": round(sec * 1e3, 3)}}))
        return 0
    # The prefill is measured first: of the workloads here it is the one bound by the matrix cores,
    # whose clocks give way once the device has been kept busy for a while (after the decode runs of
    # this program's default length the same prefill takes a few per cent longer).
    from qwen25vl_lite_amd.ops import attention_mfma
    prefill_sec = None if args.no_points else prefill_rate(2048)
    kinds = {"prefill_2048": dict(attention_mfma.taken)}
    attention_mfma.taken.clear()
    value, ms_per_step, ctx_mid = decode_rate(args.batch, args.steps, args.warmup)
    kinds["prompts_and_decode"] = dict(attention_mfma.taken)   # launches by kind; a captured decode step counts once
    need = step_bytes(t, args.batch, ctx_mid, 2 if args.dtype == "bfloat16" else 4)
    achieved = need / (ms_per_step * 1e-3) / 1e9
    peak_key = "bf16" if args.dtype == "bfloat16" else "fp32"
    line = {
        "metric": f"decode tok/s (Qwen2.5-VL-{args.size.upper()} text decoder, {args.dtype}, batch {args.batch}, "
                  f"{args.prompt_tokens}-token prompts)",
        "value": round(value, 2), "unit": "tokens/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 4), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16" if args.dtype == "bfloat16" else "fp32", "data": "synthetic",
        "config": {
            "model": f"Qwen2.5-VL-{args.size.upper()} text decoder (random weights)", "layers": t.num_hidden_layers,
            "layers_of_config": SIZES[args.size]["num_hidden_layers"], "hidden_size": t.hidden_size, "heads": t.num_attention_heads,
            "kv_heads": t.num_key_value_heads, "head_dim": t.head_dim, "intermediate_size": t.intermediate_size,
            "vocab_size": t.vocab_size, "global_batch": args.batch, "seq_len": args.prompt_tokens,
            "context_mid": ctx_mid, "max_context": max_ctx, "page_size": page, "parallelism": "single GPU",
            "hip_graph": not args.no_graph, "decode_lookahead": not (args.no_graph or args.no_lookahead),
            "tuned_library_products": not args.no_tune,
        },
        "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": round(achieved / HBM_PEAK_GBS, 4)},
    }
    if not args.no_points:
        points = {}
        for b, steps in ((1, min(args.steps, 64)), (64, min(args.steps, 64))):
            rate, _, _ = decode_rate(b, steps, min(args.warmup, 4))
            points[f"decode_b{b}"] = round(rate, 2)
        line["points"] = points
        tokens, sec = 2048, prefill_sec
        flops = prefill_flops(t, tokens)
        line["prefill"] = {"value": round(tokens / sec, 1), "tokens": tokens, "ms": round(sec * 1e3, 3),
                           "frac": round(flops / sec / MFMA_PEAK[peak_key], 4)}
    line["attention_kernels"] = kinds
    print(json.dumps(line))
    return 0


if __name__ == "__main__":
    raise SystemExit(main())
