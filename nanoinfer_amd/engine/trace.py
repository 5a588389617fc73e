"""Trace replay: the program behind ``bin/trace_run``.

It reads steps (JSON lines) from standard input, drives :class:`ModelRunner` with them, and
writes the float32 logits of the wanted places.  It samples nothing and has no model, cache or
loader of its own.  The nearest thing in the reference is its single-prompt demo, which feeds a
``ForwardBatch`` straight into the model with an identity block table (demo/llama.cpp:77-87,
179-236); here the cache manager allocates and frees for real, so pages are used again.
"""
from __future__ import annotations

import argparse
import json
import os
import sys
from typing import List


def parse_args(argv: List[str]):
    ap = argparse.ArgumentParser(prog="trace_run", description="replay token traces through the engine, write logits")
    ap.add_argument("--model", required=True, help="folder with config.json and model.safetensors")
    ap.add_argument("--dtype", required=True, choices=["bfloat16", "float32"],
                    help="bfloat16: the kernels and precisions of serving; float32: everything in true 32-bit")
    ap.add_argument("--out", required=True, help="folder for <step>.f32 files")
    ap.add_argument("--max-tokens", type=int, required=True,
                    help="most tokens live requests hold at any time; the page pool is made for this many")
    ap.add_argument("--page-size", type=int, default=16, help="tokens per cache page (default 16)")
    ap.add_argument("--max-requests", type=int, default=16, help="most requests live at a time (default 16)")
    return ap.parse_args(argv)


def main(argv: List[str] = None) -> int:
    args = parse_args(sys.argv[1:] if argv is None else argv)
    os.makedirs(args.out, exist_ok=True)
    print("[trace_run] loading the framework ...", file=sys.stderr, flush=True)
    from .runner import ModelRunner, StepEntry

    runner = ModelRunner(args.model, dtype=args.dtype, page_size=args.page_size, max_tokens=args.max_tokens,
                         max_requests=args.max_requests)
    print(f"[trace_run] model ready: {runner.arch.name}, {args.dtype}, "
          f"{runner.cache.num_pages} pages of {runner.page_size}", file=sys.stderr, flush=True)
    import torch

    for line in sys.stdin:
        line = line.strip()
        if not line:
            continue
        rec = json.loads(line)
        step = rec["step"]
        entries = [StepEntry(e["id"], e["tokens"], e.get("want", [])) for e in rec.get("entries", [])]
        logits = runner.step(entries, end=rec.get("end", []))
        if logits is not None:
            host = logits.to("cpu", torch.float32).contiguous().numpy()
            tmp = os.path.join(args.out, f".{step}.f32.tmp")
            host.astype("<f4", copy=False).tofile(tmp)
            os.replace(tmp, os.path.join(args.out, f"{step}.f32"))
        else:
            torch.cuda.synchronize()
        print(f"done {step}", flush=True)
    return 0
