"""Trace replay: feed given token ids through the model step by step and write logits.

Nothing is sampled and nothing is scheduled: every line of the trace is one call of the
engine's own step function, on the engine's own model, cache and kernels.

A trace is a sequence of JSON objects, one per step::

    {"step": 0, "entries": [{"id": "a", "tokens": [5, 17, 3], "want": [0, 2]}], "end": []}

``entries``: per request its next tokens and the places among them whose logits are wanted;
``end``: requests that are finished after the step (their pages and row are given back).
For a step with wanted places the logits ``[wanted, vocab]`` are written to ``<out>/<step>.f32``
as little-endian float32 in the order of the entries and of ``want``.
"""
from __future__ import annotations

import json
import os
import sys

import numpy as np

from .runner import ModelRunner, StepEntry


def replay_step(runner: ModelRunner, record: dict, out_dir: str | None, taps: dict | None = None):
    """Run one trace record; returns the logits array (or None).  ``taps`` receives intermediates."""
    entries = [StepEntry(str(e["id"]), [int(t) for t in e["tokens"]], [int(w) for w in e.get("want", [])])
               for e in record.get("entries", [])]
    logits = None
    if entries:
        result = runner.step(entries, taps=taps)
        if result.shape[0]:
            logits = result.cpu().numpy().astype("<f4", copy=False)
            if out_dir is not None:
                logits.tofile(os.path.join(out_dir, f"{record['step']}.f32"))
    for request_id in record.get("end", []):
        runner.release(str(request_id))
    return logits


def replay_stream(runner: ModelRunner, lines, out_dir: str, report=sys.stdout) -> int:
    """Replay records from an iterable of JSON lines; prints ``done <step>`` after each."""
    os.makedirs(out_dir, exist_ok=True)
    steps = 0
    for line in lines:
        line = line.strip()
        if not line:
            continue
        record = json.loads(line)
        replay_step(runner, record, out_dir)
        print(f"done {record['step']}", file=report, flush=True)
        steps += 1
    return steps


def main(argv=None) -> int:
    import argparse
    parser = argparse.ArgumentParser(prog="trace_run", description=__doc__.split("\n\n")[0])
    parser.add_argument("--model", required=True, help="folder with config.json and model.safetensors")
    parser.add_argument("--dtype", required=True, choices=["bfloat16", "float32"])
    parser.add_argument("--out", required=True, help="folder for the <step>.f32 files")
    parser.add_argument("--max-tokens", type=int, required=True,
                        help="most tokens live requests hold at any time (each rounded up to a page multiple)")
    parser.add_argument("--page-size", type=int, default=64, help="tokens per cache page (a divisor of 64)")
    parser.add_argument("--max-requests", type=int, default=8, help="most requests live at a time")
    args = parser.parse_args(argv)
    if args.page_size <= 0 or 64 % args.page_size:
        parser.error("--page-size must divide 64")
    print(f"[trace_run] loading {args.model} ({args.dtype})", file=sys.stderr, flush=True)
    runner = ModelRunner.from_folder(
        args.model, dtype=args.dtype, device="cuda", kv_page_size=args.page_size,
        num_kvcache_tokens=-(-args.max_tokens // 64) * 64, max_num_seqs=args.max_requests)
    print("[trace_run] ready", file=sys.stderr, flush=True)
    replay_stream(runner, sys.stdin, args.out)
    return 0
