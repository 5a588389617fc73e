"""Command line in the manner of the reference's demos.

Options that the demos have keep their names and meanings (demo/llama.cpp:94-110,
demo/prefix_caching_benchmark.cpp:592): ``--model``, ``--dtype``, ``--temperature`` (default 0:
greedy), ``--top-k``, ``--top-p``, ``--rep-penalty``, ``--seed``, ``--max-tokens``.  ``--model`` is a
model folder here (the demos map a preset name to fixed paths), ``--dtype`` is fp32 or bf16 (the
demos offer fp32 or int8).  What the demos fix at compile time (demo/batched_infer_multi_prompts.cpp:18-25)
are options: ``--max-batch-size``, ``--max-sequences``, ``--prefill-chunk-size``, ``--block-size``,
``--num-cache-blocks``; ``--max-decode-run`` is this engine's own.  Prompts are token ids (``--prompt-ids``) or random ids of given lengths
(``--prompt-len``): text goes through a tokenizer, which is outside this engine.
"""
from __future__ import annotations

import argparse
import json
import sys
import tempfile
import time
from typing import List

_DTYPES = {"fp32": "float32", "float32": "float32", "bf16": "bfloat16", "bfloat16": "bfloat16"}


def build_parser() -> argparse.ArgumentParser:
    ap = argparse.ArgumentParser(prog="nanoinfer", description="generate tokens with the MI355X engine")
    ap.add_argument("--model", help="model folder (config.json + model.safetensors)")
    ap.add_argument("--random-config", help="a config.json to make a random-weights model from (instead of --model)")
    ap.add_argument("--random-seed", type=int, default=0, help="seed of the random weights")
    ap.add_argument("--save-random-model", help="folder to keep the random model in (default: a temporary one)")
    ap.add_argument("--dtype", default="bf16", choices=sorted(_DTYPES), help="compute type")
    ap.add_argument("--temperature", type=float, default=0.0, help="0 = greedy (default)")
    ap.add_argument("--top-k", type=int, default=-1)
    ap.add_argument("--top-p", type=float, default=1.0)
    ap.add_argument("--rep-penalty", type=float, default=1.0)
    ap.add_argument("--seed", type=int, default=-1, help="sampling seed; -1: drawn by the engine")
    ap.add_argument("--max-tokens", type=int, default=128, help="new tokens per request")
    ap.add_argument("--prompt-ids", action="append", default=[],
                    help="a prompt as comma-separated token ids; may be given several times")
    ap.add_argument("--prompt-len", action="append", type=int, default=[],
                    help="a prompt of this many random token ids; may be given several times")
    ap.add_argument("--prompt-seed", type=int, default=0, help="seed of the random prompts")
    ap.add_argument("--ignore-eos", action="store_true", help="generate --max-tokens tokens whatever is sampled")
    ap.add_argument("--max-batch-size", type=int, default=8)
    ap.add_argument("--max-sequences", type=int, default=16)
    ap.add_argument("--prefill-chunk-size", type=int, default=2048)
    ap.add_argument("--max-num-batched-tokens", type=int, default=2048)
    ap.add_argument("--block-size", type=int, default=16)
    ap.add_argument("--num-cache-blocks", type=int, default=1024)
    ap.add_argument("--kv-cache-gb", type=float, default=None,
                    help="size the page pool by device memory (GiB for all key and value pools) instead of --num-cache-blocks")
    ap.add_argument("--max-model-len", type=int, default=None)
    ap.add_argument("--max-decode-run", type=int, default=8,
                    help="decode steps run back to back on one scheduling decision (requests without a repetition penalty)")
    ap.add_argument("--one-weight-copy", action="store_true",
                    help="keep every layer matrix once on the device (no re-tiled copy for decode steps: less memory, slower decoding)")
    ap.add_argument("--json", action="store_true", help="print the generated ids as one JSON line per request")
    return ap


def main(argv: List[str] = None) -> int:
    args = build_parser().parse_args(argv)
    if bool(args.model) == bool(args.random_config):
        print("give exactly one of --model and --random-config", file=sys.stderr)
        return 2
    import random

    from .engine.llm import Engine
    from .engine.scheduler import EngineConfig
    from .sampling.params import SamplingParams
    from .weights.loader import make_random_model

    model_dir = args.model
    if args.random_config:
        with open(args.random_config) as fh:
            raw = json.load(fh)
        model_dir = args.save_random_model or tempfile.mkdtemp(prefix="nanoinfer-random-")
        make_random_model(model_dir, raw, args.random_seed, dtype=_DTYPES[args.dtype])
        print(f"random model written to {model_dir}", file=sys.stderr)
    cfg = EngineConfig(max_batch_size=args.max_batch_size, max_sequences=args.max_sequences,
                       prefill_chunk_size=args.prefill_chunk_size, block_size=args.block_size,
                       num_cache_blocks=args.num_cache_blocks, max_num_batched_tokens=args.max_num_batched_tokens,
                       max_model_len=args.max_model_len, max_decode_run=args.max_decode_run, dtype=_DTYPES[args.dtype],
                       kv_cache_bytes=None if args.kv_cache_gb is None else int(args.kv_cache_gb * (1 << 30)),
                       one_weight_copy=args.one_weight_copy)
    print(f"Model: {model_dir}  dtype: {args.dtype}", file=sys.stderr)
    t0 = time.perf_counter()
    engine = Engine(model_dir, cfg, ignore_eos=args.ignore_eos)
    print(f"Loaded in {time.perf_counter() - t0:.2f} s", file=sys.stderr)
    mem = engine.runner.memory_report()
    print(f"Device memory: weights {mem['weights'] / 2**30:.3f} GiB ({mem['weights'] / max(mem['checkpoint'], 1):.2f} x the "
          f"checkpoint's {mem['checkpoint'] / 2**30:.3f} GiB), key/value pools {mem['kv_pools'] / 2**30:.3f} GiB", file=sys.stderr)

    prompts = [[int(t) for t in p.split(",") if t.strip()] for p in args.prompt_ids]
    rng = random.Random(args.prompt_seed)
    for n in args.prompt_len:
        prompts.append([rng.randrange(engine.runner.vocab_size) for _ in range(n)])
    if not prompts:
        prompts.append([rng.randrange(engine.runner.vocab_size) for _ in range(16)])
    params = SamplingParams(args.temperature, args.top_k, args.top_p, args.rep_penalty, args.seed)

    import torch

    ids = [engine.add_request(p, args.max_tokens, params) for p in prompts]
    torch.cuda.synchronize()
    t_start = time.perf_counter()
    prefill_s = decode_s = 0.0
    prefill_tokens = decode_tokens = steps = 0
    while engine.has_work():
        t1 = time.perf_counter()
        engine.step()
        torch.cuda.synchronize()
        dt = time.perf_counter() - t1
        n = engine.scheduler.last_scheduled_tokens
        steps += 1
        # a step counts as prefill time in proportion to its prompt tokens
        prompt_share = engine.last_prompt_tokens / n if n else 0.0
        prefill_s += dt * prompt_share
        decode_s += dt * (1.0 - prompt_share)
        prefill_tokens += engine.last_prompt_tokens
        decode_tokens += n - engine.last_prompt_tokens
    elapsed = time.perf_counter() - t_start
    generated = 0
    for rid in ids:
        r = engine.get_request(rid)
        generated += len(r.generated)
        if args.json:
            print(json.dumps({"id": rid, "prompt_len": len(r.prompt), "tokens": r.generated,
                              "finish_reason": r.finish_reason}))
        else:
            print(f"[request {rid}] prompt {len(r.prompt)} tokens -> {len(r.generated)} new ({r.finish_reason}): "
                  + " ".join(str(t) for t in r.generated))
    print("\n======================================")
    if prefill_s > 0:
        print(f"Prefill:  {prefill_tokens} tokens, {prefill_s * 1e3:.2f} ms ({prefill_tokens / prefill_s:.1f} tok/s)")
    if decode_s > 0:
        print(f"Decode:   {decode_tokens} tokens, {decode_s * 1e3:.2f} ms ({decode_tokens / decode_s:.1f} tok/s)")
    print(f"Total:    {prefill_tokens + decode_tokens} tokens run, {generated} generated, {engine.num_steps} steps "
          f"on {steps} scheduling decisions, {elapsed * 1e3:.2f} ms")
    st = engine.scheduler.stats()
    print(f"Scheduler - Finished: {st['num_finished']}  Running: {st['num_running']}  Waiting: {st['num_waiting']}  "
          f"Preemptions: {st['num_preemptions']}")
    return 0


if __name__ == "__main__":
    sys.exit(main())
