"""Decode and prefill throughput of the engine on one MI355X, Llama 3.2 1B shape, random weights.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--dtype bf16|fp32] [--shape 1b|3b|8b] [--layers L]
    python bench.py --workload serving [--shape 3b] [--dtype fp32]

A step is one decode step of a batch of 8 requests whose prompts of 2,048 random tokens are in
the cache (context limit 4,096): the step function runs the 8 new tokens as one batch, the
argmax kernels pick the next ones, and they come back to the host, as in greedy generation.  ``value``
is decoded tokens per second.  The same line carries the prefill of one 2,048-token prompt in
portions of 512 (``prefill``; ``--prefill-chunk`` changes the cut), in one portion, the engine's
default (``prefill_one_portion``, and ``prefill_one_portion_eager`` with every kernel launched from
the host instead of a recorded step; a longer ``--prompt-len`` goes in portions of 2,048 there), the decode step's fraction of the HBM roofline, and in
``points`` decode at batch 1 and 64 (``rooflines`` holds the roofline fraction of every point by
its name).  The default line (1B shape, bfloat16) adds further points, each timed over 96 steps:
decode at batch 8 and 64 from contexts of 8,192 and 32,768 tokens; prompts of 8,192 and 32,768
tokens (``prefill_8k``, ``prefill_32k``, in portions of 2,048); the same model in true float32
(``decode_b8_fp32``, ``decode_b8_ctx8k_fp32``, ``prefill_fp32``: the reference's own precision);
requests that draw instead of taking the largest logit (``decode_b8_temperature``,
``decode_b8_top_k_top_p``); the
3B shape in bfloat16 at batch 1, 8 and 64; requests through the scheduler (``serving_1b_bf16``,
``serving_1b_bf16_128req_half_pool`` with half the pages its 128 requests need, and
``serving_3b_fp32``: 64 concurrent requests of the 3B shape in float32, prompts uniform in
[128, 2048], 256 new tokens each); and the 8B shape at its full 32 layers in float32
(``prefill_8b_fp32`` of 2,048 tokens in portions of 512, ``decode_b1/b8/b64_8b_fp32``) and in
bfloat16.  A further point that fails is named in ``errors`` and costs the line nothing else.
Peaks are MI355X's published ones: HBM
8 TB/s, dense bf16 MFMA 2.5 PFLOP/s, fp32 157.3 TFLOP/s.  The reference publishes no numbers for
this model, so ``vs_baseline`` is null.  ``--workload serving`` measures requests through the
scheduler instead and prints a line of its own.
"""
from __future__ import annotations

import argparse
import json
import os
import random
import sys
import tempfile
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

LLAMA_1B = {
    "architectures": ["LlamaForCausalLM"], "model_type": "llama",
    "hidden_size": 2048, "num_hidden_layers": 16, "num_attention_heads": 32, "num_key_value_heads": 8,
    "head_dim": 64, "intermediate_size": 8192, "vocab_size": 128256, "rms_norm_eps": 1e-5,
    "rope_theta": 500000.0,
    "rope_scaling": {"rope_type": "llama3", "factor": 32.0, "low_freq_factor": 1.0, "high_freq_factor": 4.0,
                     "original_max_position_embeddings": 8192},
    "max_position_embeddings": 131072, "tie_word_embeddings": True, "hidden_act": "silu",
    "bos_token_id": 128000, "eos_token_id": 128001,
}
FULL_LAYERS = 16


def _family(hidden, layers, heads, kv_heads, head_dim, inter, factor, tied):
    cfg = dict(LLAMA_1B, hidden_size=hidden, num_hidden_layers=layers, num_attention_heads=heads,
               num_key_value_heads=kv_heads, head_dim=head_dim, intermediate_size=inter, tie_word_embeddings=tied)
    cfg["rope_scaling"] = dict(LLAMA_1B["rope_scaling"], factor=factor)
    return cfg


# other sizes of the family, for --shape (the default and the result line's contract is the 1B shape)
SHAPES = {"1b": ("llama-3.2-1b-shape", "Llama 3.2 1B", LLAMA_1B),
          "3b": ("llama-3.2-3b-shape", "Llama 3.2 3B", _family(3072, 28, 24, 8, 128, 8192, 32.0, True)),
          "8b": ("llama-3.1-8b-shape", "Llama 3.1 8B", _family(4096, 32, 32, 8, 128, 14336, 8.0, False))}
PROMPT_LEN = 2048
CONTEXT_LEN = 4096
PREFILL_CHUNK = 512       # portions of the prefill measurement, as the benchmark configuration names them
ENGINE_CHUNK = 2048       # the engine's own default: a portion as long as the step's token budget
DECODE_RUN = 8            # the engine's own default of max_decode_run
BLOCK_SIZE = 16
HBM_PEAK = 8.0e12
FLOP_PEAK = {"bf16": 2.5e15, "fp32": 157.3e12}


def log(msg: str) -> None:
    print(f"[bench] {msg}", file=sys.stderr, flush=True)


def decode_bytes(cfg: dict, batch: int, mean_context: float, elem: int) -> float:
    """Bytes a decode step has to read: every matrix once (the tied head is the embedding
    matrix), the norm weights, and the keys and values of the live requests."""
    d, L, H, KVH, hd = cfg["hidden_size"], cfg["num_hidden_layers"], cfg["num_attention_heads"], \
        cfg["num_key_value_heads"], cfg["head_dim"]
    I, V = cfg["intermediate_size"], cfg["vocab_size"]
    per_layer = (H * hd * d + 2 * KVH * hd * d + d * H * hd + 3 * I * d) * elem + 2 * d * 4
    weights = L * per_layer + V * d * elem + d * 4
    kv = batch * mean_context * L * 2 * KVH * hd * elem
    return weights + kv


def prefill_flops(cfg: dict, tokens: int) -> float:
    """Matrix products of every layer on every token, causal attention, and the head on one row."""
    d, L, H, KVH, hd = cfg["hidden_size"], cfg["num_hidden_layers"], cfg["num_attention_heads"], \
        cfg["num_key_value_heads"], cfg["head_dim"]
    I, V = cfg["intermediate_size"], cfg["vocab_size"]
    linear = 2.0 * tokens * L * (H * hd * d + 2 * KVH * hd * d + d * H * hd + 3 * I * d)
    attention = L * H * 4.0 * hd * (tokens * (tokens + 1) / 2.0)
    return linear + attention + 2.0 * V * d


def config_record(cfg: dict, layers: int, batch: int, mean_ctx: float, prefill_chunk: int, decode_run: int,
                  model: str = "llama-3.2-1b-shape", full_layers: int = FULL_LAYERS) -> dict:
    """Every size of the measured configuration, flat (nothing nested, at most 20 keys)."""
    return {
        "model": model, "layers": layers, "layers_full_model": full_layers,
        "hidden_size": cfg["hidden_size"], "heads": cfg["num_attention_heads"],
        "kv_heads": cfg["num_key_value_heads"], "head_dim": cfg["head_dim"],
        "intermediate_size": cfg["intermediate_size"], "vocab_size": cfg["vocab_size"],
        "tied_embeddings": bool(cfg["tie_word_embeddings"]), "global_batch": batch, "prompt_len": PROMPT_LEN,
        "seq_len": CONTEXT_LEN, "decode_context_mean": round(mean_ctx, 1), "kv_block_size": BLOCK_SIZE,
        "prefill_chunk": prefill_chunk, "decode_run": decode_run, "parallelism": "single-gpu",
    }


LONG_CONTEXTS = (8192, 32768)   # further decode points at batch 8
POINT_STEPS = 96               # timed steps of every point beside the headline (whatever --steps says):
POINT_WARMUP = 16              # enough for batch 64 to repeat within a few per cent


class Rig:
    """A random model of the given sizes in a runner, and the two measurements over it."""

    def __init__(self, cfg: dict, dtype: str, pool_tokens: int, max_requests: int, decode_run: int):
        import torch

        import nanoinfer_amd  # noqa: F401
        from nanoinfer_amd.engine.runner import ModelRunner
        from nanoinfer_amd.weights.loader import make_random_model

        self.cfg, self.decode_run = cfg, decode_run
        self.rng = random.Random(0)
        name = {"bf16": "bfloat16", "fp32": "float32"}[dtype]
        with tempfile.TemporaryDirectory(prefix="nanoinfer-bench-") as folder:
            t0 = time.perf_counter()
            make_random_model(folder, cfg, seed=0, dtype=name)
            log(f"random model ({cfg['num_hidden_layers']} layers of {cfg['hidden_size']}, {dtype}) written in "
                f"{time.perf_counter() - t0:.1f} s")
            t0 = time.perf_counter()
            self.runner = ModelRunner(folder, dtype=name, page_size=BLOCK_SIZE, max_tokens=pool_tokens,
                                      max_requests=max_requests)
            log(f"model loaded in {time.perf_counter() - t0:.1f} s")
        self.torch = torch

    def close(self) -> None:
        self.runner = None
        import gc
        gc.collect()
        self.torch.cuda.empty_cache()

    def prompt(self, n: int):
        V = self.cfg["vocab_size"]
        return [self.rng.randrange(V) for _ in range(n)]

    def prefill(self, length: int, chunk: int, recorded: bool = True) -> float:
        """Seconds for one prompt of ``length`` tokens in portions of ``chunk``, up to its first
        token on the host; the best of the second and third of three prompts.  ``recorded`` False:
        every kernel launched from the host, as a portion's shape runs when it comes the first time."""
        from nanoinfer_amd import kernels as K
        from nanoinfer_amd.engine.runner import StepEntry

        runner, torch = self.runner, self.torch
        graphs, runner.use_graphs = runner.use_graphs, runner.use_graphs and recorded
        times = []
        try:
            for rep in range(3):
                toks = self.prompt(length)
                torch.cuda.synchronize()
                t = time.perf_counter()
                for s in range(0, length, chunk):
                    part = toks[s:s + chunk]
                    last = s + chunk >= length
                    logits = runner.step([StepEntry("p", part, [len(part) - 1] if last else [])])
                K.argmax(logits).tolist()
                torch.cuda.synchronize()
                times.append(time.perf_counter() - t)
                runner.release("p")
        finally:
            runner.use_graphs = graphs
        return min(times[1:])

    def decode(self, batch: int, context: int, steps: int, warmup: int, sampling=None):
        """(seconds a step, mean context) of ``steps`` decode steps of ``batch`` requests whose
        prompts of ``context`` tokens are in the cache, as the engine decodes greedy requests: runs
        of steps on one scheduling decision, the tokens passing from step to step on the device.
        ``sampling`` (a ``SamplingParams`` without a repetition penalty): every request draws with
        these options instead, as the engine runs such requests: the draw is part of the recorded step."""
        from nanoinfer_amd import kernels as K
        from nanoinfer_amd.engine.runner import StepEntry

        runner, torch = self.runner, self.torch
        ids = [f"d{i}" for i in range(batch)]
        tokens = []
        for i in ids:   # fill the cache: one request at a time, in portions of the engine's token budget
            toks = self.prompt(context)
            for s in range(0, context, ENGINE_CHUNK):
                part = toks[s:s + ENGINE_CHUNK]
                logits = runner.step([StepEntry(i, part, [len(part) - 1] if s + ENGINE_CHUNK >= context else [])])
            tokens.append(K.argmax(logits).tolist()[0])
        log(f"batch {batch}: prompts of {context} tokens are in the cache")

        generated = [[] for _ in ids]
        sampler = None
        if sampling is not None:
            from nanoinfer_amd.sampling.sampler import Sampler
            sampler = Sampler(runner.device)

        def run(toks, n):
            while n > 0:
                k = min(self.decode_run, n)
                entries = [StepEntry(i, [t], [0]) for i, t in zip(ids, toks)]
                if sampler is None:
                    toks = runner.decode_run(entries, k)[-1]
                else:
                    rows = runner.decode_run(entries, k, draw=sampler.draw_tables([sampling] * batch, generated, k))
                    for row in rows:
                        for g, t in zip(generated, row):
                            g.append(t)
                    toks = rows[-1]
                n -= k
            return toks

        tokens = run(tokens, warmup)
        torch.cuda.synchronize()
        first_ctx = runner.computed_tokens(ids[0])
        t = time.perf_counter()
        tokens = run(tokens, steps)
        torch.cuda.synchronize()
        dt = time.perf_counter() - t
        for i in ids:
            runner.release(i)
        return dt / steps, first_ctx + (steps + 1) / 2.0


def percentile(values, q: float) -> float:
    values = sorted(values)
    if not values:
        return 0.0
    return values[min(len(values) - 1, int(q * len(values)))]


def serving_measure(args) -> dict:
    """Requests through the engine's own scheduler, as a user's program drives it
    (``Engine.add_request`` / ``Engine.step``): ``args.requests`` requests arrive at once, prompts of
    uniform random length in [``min_prompt``, ``max_prompt``] (seeded), ``new_tokens`` new tokens each,
    greedy, continuous batching with prompt portions beside decode tokens.  The report follows the
    reference's demo (demo/batched_infer_multi_prompts.cpp:356-362: prefill and decode tokens a
    second) and adds the step times, the share of the HBM roofline of the decode steps, and the
    host's share of the wall time (wall minus the spans between the GPU events around every
    step's launches).  Returns the result line as a dict."""
    import gc

    import torch

    import nanoinfer_amd  # noqa: F401
    from nanoinfer_amd.engine.llm import Engine
    from nanoinfer_amd.engine.scheduler import EngineConfig
    from nanoinfer_amd.sampling.params import SamplingParams
    from nanoinfer_amd.weights.loader import make_random_model

    torch.cuda.set_device(0)
    model_name, shown_name, full = SHAPES[args.shape]
    cfg = dict(full)
    layers = args.layers or full["num_hidden_layers"]
    cfg["num_hidden_layers"] = layers
    dtype = {"bf16": "bfloat16", "fp32": "float32"}[args.dtype]
    elem = 2 if args.dtype == "bf16" else 4
    rng = random.Random(0)
    n_req, new_tokens = args.requests, args.new_tokens
    lengths = [rng.randint(args.min_prompt, args.max_prompt) for _ in range(n_req)]
    prompts = [[rng.randrange(cfg["vocab_size"]) for _ in range(n)] for n in lengths]
    pages = sum(-(-(n + new_tokens) // BLOCK_SIZE) for n in lengths) + n_req
    if args.pool_share < 1.0:
        pages = max(int(pages * args.pool_share), -(-(max(lengths) + new_tokens) // BLOCK_SIZE) + 1)
    with tempfile.TemporaryDirectory(prefix="nanoinfer-bench-") as folder:
        t0 = time.perf_counter()
        make_random_model(folder, cfg, seed=0, dtype=dtype)
        log(f"random model written in {time.perf_counter() - t0:.1f} s")
        t0 = time.perf_counter()
        engine = Engine(folder, EngineConfig(max_batch_size=n_req, max_sequences=n_req, block_size=BLOCK_SIZE,
                                             num_cache_blocks=pages, prefill_chunk_size=args.prefill_chunk or ENGINE_CHUNK,
                                             max_num_batched_tokens=args.token_budget, max_decode_run=args.decode_run,
                                             dtype=dtype), ignore_eos=True)
        log(f"model loaded in {time.perf_counter() - t0:.1f} s")
    runner = engine.runner

    def one_pass(measure: bool):
        for p in prompts:
            engine.add_request(p, new_tokens, SamplingParams.greedy())
        runner.timeline = [] if measure else None
        rows = []           # per scheduling decision: wall s, gpu s, model steps, prompt tokens, decode tokens, bytes
        torch.cuda.synchronize()
        t_begin = time.perf_counter()
        while engine.has_work():
            live = [(r.num_computed, r) for r in engine.scheduler.running]
            steps_before = engine.num_steps
            t1 = time.perf_counter()
            engine.step()
            wall = time.perf_counter() - t1
            n = engine.scheduler.last_scheduled_tokens
            prompt_tokens = engine.last_prompt_tokens
            model_steps = engine.num_steps - steps_before
            gpu = 0.0
            if measure:
                torch.cuda.synchronize()
                gpu = sum(a.elapsed_time(b) for a, b in runner.timeline) * 1e-3
                runner.timeline.clear()
            # keys a decode-only decision reads: a request with c tokens in the cache reads c + 1 + k in step k
            kv_tokens = 0 if prompt_tokens else sum(model_steps * (c + 1) + model_steps * (model_steps - 1) // 2
                                                    for c, _ in live)
            rows.append((wall, gpu, model_steps, prompt_tokens, n - prompt_tokens, kv_tokens))
        torch.cuda.synchronize()
        total = time.perf_counter() - t_begin
        engine.scheduler.clear_finished()
        return rows, total

    log("first pass (records the decode shapes) ...")
    one_pass(False)
    log("measured pass ...")
    rows, total = one_pass(True)
    preempted_before = engine.scheduler.num_preemptions
    plain_rows, plain_total = one_pass(False)      # without events and their synchronisation: the figure that counts
    preempted = engine.scheduler.num_preemptions - preempted_before

    generated = n_req * new_tokens
    prefill_s = sum(w * (p / (p + d)) for w, _, _, p, d, _ in plain_rows if p + d)
    decode_s = sum(w * (d / (p + d)) for w, _, _, p, d, _ in plain_rows if p + d)
    prompt_total = sum(lengths)
    decode_rows = [r for r in rows if r[3] == 0 and r[4] > 0]
    per_step = [r[0] / r[2] for r in decode_rows for _ in range(r[2])]
    weights = decode_bytes(cfg, 0, 0, elem)
    kv_per_token = cfg["num_hidden_layers"] * 2 * cfg["num_key_value_heads"] * cfg["head_dim"] * elem
    decode_time = sum(r[0] for r in decode_rows)
    decode_read = sum(weights * r[2] + kv_per_token * r[5] for r in decode_rows)
    wall_sum = sum(r[0] for r in rows)
    gpu_sum = sum(r[1] for r in rows)
    host_share_decode = 1.0 - sum(r[1] for r in decode_rows) / decode_time if decode_time else 0.0
    result = {
        "metric": f"serving: generated tok/s, {n_req} concurrent requests ({shown_name} shape, continuous batching)",
        "value": round(generated / plain_total, 1), "unit": "tokens/s", "n_gpus": 1,
        "steps": sum(r[2] for r in plain_rows), "warmup": 1,
        "ms_per_step": round(1e3 * (sum(per_step) / len(per_step) if per_step else 0.0), 4),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": args.dtype,
        "data": "synthetic: random weights (seed 0), uniform random token ids, prompt lengths uniform (seed 0)",
        "config": {"model": model_name, "layers": layers, "layers_full_model": full["num_hidden_layers"],
                   "hidden_size": cfg["hidden_size"], "heads": cfg["num_attention_heads"],
                   "kv_heads": cfg["num_key_value_heads"], "head_dim": cfg["head_dim"],
                   "intermediate_size": cfg["intermediate_size"], "vocab_size": cfg["vocab_size"],
                   "requests": n_req, "prompt_len_min": args.min_prompt, "prompt_len_max": args.max_prompt,
                   "new_tokens": new_tokens, "kv_block_size": BLOCK_SIZE, "cache_pages": pages,
                   "token_budget": args.token_budget, "decode_run": args.decode_run, "parallelism": "single-gpu"},
        "total_ms": round(plain_total * 1e3, 1),
        "prefill": {"value": round(prompt_total / prefill_s, 1) if prefill_s else None, "tokens": prompt_total,
                    "ms": round(prefill_s * 1e3, 2)},
        "decode": {"value": round((generated - n_req) / decode_s, 1) if decode_s else None, "tokens": generated - n_req,
                   "ms": round(decode_s * 1e3, 2)},
        "decode_step_ms": {"mean": round(1e3 * sum(per_step) / max(len(per_step), 1), 4),
                           "p50": round(1e3 * percentile(per_step, 0.5), 4), "p99": round(1e3 * percentile(per_step, 0.99), 4)},
        "roofline": {"bound": "hbm", "achieved": round(decode_read / decode_time / 1e9, 1) if decode_time else None,
                     "peak": HBM_PEAK / 1e9, "unit": "GB/s",
                     "frac": round(decode_read / decode_time / HBM_PEAK, 4) if decode_time else None},
        "host_share": {"all_steps": round(1.0 - gpu_sum / wall_sum, 4) if wall_sum else None,
                       "decode_steps": round(host_share_decode, 4),
                       "measured_pass_ms": round(total * 1e3, 1)},
        "preemptions": preempted,          # of the pass that ``value`` is from
    }
    del engine, runner
    gc.collect()
    torch.cuda.empty_cache()
    return result


def serving(args) -> int:
    """``--workload serving``: a result line of its own for :func:`serving_measure`."""
    print(json.dumps(serving_measure(args)))
    return 0


def serving_brief(full: dict) -> dict:
    """The figures of a serving result that go onto the default line, flat."""
    return {"value": full["value"], "total_ms": full["total_ms"], "requests": full["config"]["requests"],
            "new_tokens": full["config"]["new_tokens"], "prefill_tok_s": full["prefill"]["value"],
            "decode_tok_s": full["decode"]["value"], "decode_step_ms": full["decode_step_ms"]["mean"],
            "decode_step_p99_ms": full["decode_step_ms"]["p99"], "roofline_frac": full["roofline"]["frac"],
            "host_share": full["host_share"]["all_steps"], "preemptions": full["preemptions"],
            "cache_pages": full["config"]["cache_pages"]}


def main() -> int:
    global PROMPT_LEN, CONTEXT_LEN
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--dtype", default="bf16", choices=["bf16", "fp32"])
    ap.add_argument("--batch", type=int, default=8)
    ap.add_argument("--shape", default="1b", choices=sorted(SHAPES), help="layer sizes of the family member to measure (default: 1b)")
    ap.add_argument("--layers", type=int, default=None, help="fewer layers than the model has (named in config)")
    ap.add_argument("--prefill-chunk", type=int, default=None,
                    help="tokens of a prompt portion in the prefill measurement (default 512); serving: the engine's "
                         "prefill_chunk_size (default: the token budget)")
    ap.add_argument("--decode-run", type=int, default=DECODE_RUN,
                    help="decode steps on one scheduling decision (the engine's max_decode_run; 1: the host reads every token before the next step)")
    ap.add_argument("--prompt-len", type=int, default=PROMPT_LEN,
                    help="tokens of every prompt (the measured prefill, and the context that decoding starts from); "
                         "the pool holds 2,048 more for every request")
    ap.add_argument("--no-points", action="store_true", help="skip decode at batch 1 and 64 and the further points")
    ap.add_argument("--no-further", action="store_true",
                    help="skip the points beyond the contract's: contexts of 8k and 32k, float32, the 3B shape")
    ap.add_argument("--workload", default="steps", choices=["steps", "serving"],
                    help="steps: the decode step and prefill of the result line's contract (default); "
                         "serving: concurrent requests through the engine's scheduler, a line of its own")
    ap.add_argument("--requests", type=int, default=64, help="serving: concurrent requests")
    ap.add_argument("--new-tokens", type=int, default=256, help="serving: tokens generated per request")
    ap.add_argument("--min-prompt", type=int, default=128, help="serving: shortest prompt")
    ap.add_argument("--max-prompt", type=int, default=2048, help="serving: longest prompt")
    ap.add_argument("--token-budget", type=int, default=2048, help="serving: tokens of one step (max_num_batched_tokens)")
    ap.add_argument("--pool-share", type=float, default=1.0,
                    help="serving: pages of the pool as a share of what all requests need at their ends "
                         "(below 1 requests wait or are preempted)")
    ap.add_argument("--phase", default="all", choices=["all", "decode", "prefill"],
                    help="run one phase only (for profiling; prints no result line)")
    args = ap.parse_args()
    if args.prompt_len < 1 or args.prompt_len + 2048 > LLAMA_1B["max_position_embeddings"]:
        print(f"--prompt-len must lie between 1 and {LLAMA_1B['max_position_embeddings'] - 2048}")
        return 2
    PROMPT_LEN, CONTEXT_LEN = args.prompt_len, args.prompt_len + 2048
    if args.gpus != 1:
        print(f"bench.py measures one GPU only: this engine runs on a single MI355X, --gpus {args.gpus} is not supported")
        return 2
    if args.workload == "serving":
        return serving(args)
    args.prefill_chunk = args.prefill_chunk or PREFILL_CHUNK

    import torch

    torch.cuda.set_device(0)
    model_name, shown_name, full = SHAPES[args.shape]
    cfg = dict(full)
    if args.layers is None:
        args.layers = full["num_hidden_layers"]
    cfg["num_hidden_layers"] = args.layers
    elem = 2 if args.dtype == "bf16" else 4
    extras = not args.no_points and args.phase == "all"
    # the further points (longer contexts, float32, the 3B shape) belong to the default line only
    further = extras and args.shape == "1b" and args.dtype == "bf16" and args.layers == full["num_hidden_layers"] \
        and args.prompt_len == 2048 and not args.no_further

    max_batch = max(args.batch, 64) if extras else args.batch
    pool = max_batch * CONTEXT_LEN
    if further:
        pool = max(pool, 64 * (LONG_CONTEXTS[-1] + 512))
    rig = Rig(cfg, args.dtype, pool, max_batch, args.decode_run)

    if args.phase == "prefill":
        log(f"prefill of {PROMPT_LEN} in portions of {args.prefill_chunk}: "
            f"{rig.prefill(PROMPT_LEN, args.prefill_chunk) * 1e3:.2f} ms")
        return 0
    if args.phase == "decode":
        step_s, _ = rig.decode(args.batch, PROMPT_LEN, args.steps, args.warmup)
        log(f"decode batch {args.batch}: {step_s * 1e3:.3f} ms a step")
        return 0
    flops = prefill_flops(cfg, PROMPT_LEN)

    def prefill_record(seconds: float, dtype: str = args.dtype, fl: float = flops) -> dict:
        return {"value": round(PROMPT_LEN / seconds, 1), "tokens": PROMPT_LEN, "ms": round(seconds * 1e3, 3),
                "frac": round(fl / seconds / FLOP_PEAK[dtype], 4)}

    log("prefill ...")
    prefill_s = rig.prefill(PROMPT_LEN, args.prefill_chunk)
    log(f"prefill of {PROMPT_LEN} in portions of {args.prefill_chunk}: {prefill_s * 1e3:.2f} ms")
    how = "in one portion" if PROMPT_LEN <= ENGINE_CHUNK else f"in portions of {ENGINE_CHUNK}"      # the engine's default cut
    whole_s = rig.prefill(PROMPT_LEN, ENGINE_CHUNK)
    log(f"prefill of {PROMPT_LEN} {how}: {whole_s * 1e3:.2f} ms")
    eager_s = rig.prefill(PROMPT_LEN, ENGINE_CHUNK, recorded=False)
    log(f"prefill of {PROMPT_LEN} {how}, launched kernel by kernel: {eager_s * 1e3:.2f} ms")
    step_s, mean_ctx = rig.decode(args.batch, PROMPT_LEN, args.steps, args.warmup)
    log(f"decode batch {args.batch}: {step_s * 1e3:.3f} ms a step")
    points = {}
    more = {}
    errors = []

    def attempt(what: str, fn) -> None:
        """A further point must not cost the line its contract: what fails is named in ``errors``."""
        try:
            fn()
        except Exception as e:      # noqa: BLE001
            log(f"{what} failed: {type(e).__name__}: {e}")
            errors.append(f"{what}: {type(e).__name__}: {str(e)[:200]}")

    def decode_point(r, c, name: str, batch: int, context: int, el: int, label: str) -> None:
        sec, ctx = r.decode(batch, context, POINT_STEPS, POINT_WARMUP)
        points[name] = round(batch / sec, 1)
        more.setdefault("rooflines", {})[name] = round(decode_bytes(c, batch, ctx, el) / sec / HBM_PEAK, 4)
        log(f"{label}: decode batch {batch} at context {context}: {sec * 1e3:.3f} ms a step")

    if extras:
        for b in (1, 64):
            decode_point(rig, cfg, f"decode_b{b}", b, PROMPT_LEN, elem, f"{args.shape} {args.dtype}")

        def sampled():
            # requests that draw instead of taking the largest logit (the draw is part of the recorded step)
            from nanoinfer_amd.sampling.params import SamplingParams
            for name, params in (("decode_b8_temperature", SamplingParams(temperature=0.8, seed=1)),
                                 ("decode_b8_top_k_top_p", SamplingParams(temperature=0.8, top_k=50, top_p=0.9, seed=1))):
                sec, _ = rig.decode(args.batch, PROMPT_LEN, POINT_STEPS, POINT_WARMUP, sampling=params)
                points[name.replace("b8", f"b{args.batch}")] = round(args.batch / sec, 1)
                log(f"{name}: {sec * 1e3:.3f} ms a step")
        attempt("sampled decoding", sampled)
    if further:
        def long_contexts():
            for n in LONG_CONTEXTS:
                sec, ctx = rig.decode(8, n, POINT_STEPS, POINT_WARMUP)
                points[f"decode_b8_ctx{n // 1024}k"] = round(8 / sec, 1)
                more[f"roofline_ctx{n // 1024}k"] = round(decode_bytes(cfg, 8, ctx, elem) / sec / HBM_PEAK, 4)
                log(f"decode batch 8 at context {n}: {sec * 1e3:.3f} ms a step")
            for n in LONG_CONTEXTS:
                decode_point(rig, cfg, f"decode_b64_ctx{n // 1024}k", 64, n, elem, "1B bf16")
            for n in LONG_CONTEXTS:      # long prompts, where the attention is the larger part, in portions of the token budget
                sec = rig.prefill(n, ENGINE_CHUNK)
                more[f"prefill_{n // 1024}k"] = {"value": round(n / sec, 1), "tokens": n, "ms": round(sec * 1e3, 3),
                                                "frac": round(prefill_flops(cfg, n) / sec / FLOP_PEAK[args.dtype], 4)}
                log(f"prefill of {n} in portions of {ENGINE_CHUNK}: {sec * 1e3:.2f} ms")
        attempt("long contexts", long_contexts)
        rig.close()

        def float32_1b():
            # the reference's own precision: the same model in true float32
            rig32 = Rig(cfg, "fp32", 8 * (LONG_CONTEXTS[0] + 2048), 8, args.decode_run)
            try:
                sec = rig32.prefill(PROMPT_LEN, args.prefill_chunk)
                more["prefill_fp32"] = prefill_record(sec, "fp32")
                more["prefill_fp32_one_portion"] = prefill_record(rig32.prefill(PROMPT_LEN, ENGINE_CHUNK), "fp32")
                log(f"float32: prefill of {PROMPT_LEN} in portions of {args.prefill_chunk}: {sec * 1e3:.2f} ms")
                sec, ctx = rig32.decode(8, PROMPT_LEN, POINT_STEPS, POINT_WARMUP)
                points["decode_b8_fp32"] = round(8 / sec, 1)
                more["roofline_fp32"] = round(decode_bytes(cfg, 8, ctx, 4) / sec / HBM_PEAK, 4)
                log(f"float32: decode batch 8: {sec * 1e3:.3f} ms a step")
                decode_point(rig32, cfg, "decode_b8_ctx8k_fp32", 8, LONG_CONTEXTS[0], 4, "1B fp32")
            finally:
                rig32.close()
        attempt("float32", float32_1b)

        def shape_3b():
            # the next size of the family
            cfg3 = dict(SHAPES["3b"][2])
            rig3 = Rig(cfg3, "bf16", 64 * CONTEXT_LEN, 64, args.decode_run)
            try:
                sec = rig3.prefill(PROMPT_LEN, ENGINE_CHUNK)
                more["prefill_3b_one_portion"] = prefill_record(sec, "bf16", prefill_flops(cfg3, PROMPT_LEN))
                sec, ctx = rig3.decode(8, PROMPT_LEN, POINT_STEPS, POINT_WARMUP)
                points["decode_b8_3b"] = round(8 / sec, 1)
                more["roofline_3b"] = round(decode_bytes(cfg3, 8, ctx, 2) / sec / HBM_PEAK, 4)
                log(f"3B shape: decode batch 8: {sec * 1e3:.3f} ms a step")
                for b in (1, 64):
                    decode_point(rig3, cfg3, f"decode_b{b}_3b", b, PROMPT_LEN, 2, "3B bf16")
            finally:
                rig3.close()
        attempt("3B shape", shape_3b)

        def serving_points():
            # through the scheduler (the benchmark configuration of the 3B shape: float32, 64 concurrent requests,
            # prompts uniform in [128, 2048], 256 new tokens each), and the 1B shape in bfloat16 beside it
            import copy
            for key, shape, dt, n_req, share in (("serving_1b_bf16", "1b", "bf16", 64, 1.0),
                                                 ("serving_1b_bf16_128req_half_pool", "1b", "bf16", 128, 0.5),
                                                 ("serving_3b_fp32", "3b", "fp32", 64, 1.0)):
                a = copy.copy(args)
                a.shape, a.dtype, a.layers, a.prefill_chunk, a.requests, a.pool_share = shape, dt, None, None, n_req, share
                full_line = serving_measure(a)
                more[key] = serving_brief(full_line)
                log(f"{key}: {full_line['value']} generated tok/s, decode steps of {full_line['decode_step_ms']['mean']} ms "
                    f"at {full_line['roofline']['frac']} of the roofline, {full_line['preemptions']} preemptions")
        attempt("serving", serving_points)

        def shape_8b(dt: str, el: int, prefill_too: bool):
            # the 8B shape at full depth (in float32: 32 GB of weights)
            cfg8 = dict(SHAPES["8b"][2])
            rig8 = Rig(cfg8, dt, 64 * CONTEXT_LEN, 64, args.decode_run)
            try:
                if prefill_too:
                    sec = rig8.prefill(PROMPT_LEN, PREFILL_CHUNK)
                    more[f"prefill_8b_{dt}"] = prefill_record(sec, dt, prefill_flops(cfg8, PROMPT_LEN))
                    log(f"8B shape, {dt}: prefill of {PROMPT_LEN} in portions of {PREFILL_CHUNK}: {sec * 1e3:.2f} ms")
                for b in (1, 8, 64):
                    decode_point(rig8, cfg8, f"decode_b{b}_8b_{dt}", b, PROMPT_LEN, el, f"8B {dt}")
            finally:
                rig8.close()
        attempt("8B shape, float32", lambda: shape_8b("fp32", 4, True))
        attempt("8B shape, bfloat16", lambda: shape_8b("bf16", 2, False))

    achieved = decode_bytes(cfg, args.batch, mean_ctx, elem) / step_s
    result = {
        "metric": f"decode tok/s at batch {args.batch} ({shown_name} shape, prompts of {PROMPT_LEN} tokens, "
                  f"decode context ~{round(mean_ctx)}, pool for {CONTEXT_LEN})",
        "value": round(args.batch / step_s, 1),
        "unit": "tokens/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(step_s * 1e3, 4),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": args.dtype,
        "data": "synthetic: random weights (seed 0), uniform random token ids",
        "config": config_record(cfg, args.layers, args.batch, mean_ctx, args.prefill_chunk, args.decode_run,
                                model_name, full["num_hidden_layers"]),
        "prefill": prefill_record(prefill_s),
        "prefill_one_portion": prefill_record(whole_s),
        "prefill_one_portion_eager": prefill_record(eager_s),
        "roofline": {"bound": "hbm", "achieved": round(achieved / 1e9, 1), "peak": HBM_PEAK / 1e9, "unit": "GB/s",
                     "frac": round(achieved / HBM_PEAK, 4)},
        "points": points,
    }
    result.update(more)
    if errors:
        result["errors"] = errors
    print(json.dumps(result))
    return 0


if __name__ == "__main__":
    sys.exit(main())
