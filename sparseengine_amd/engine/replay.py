"""Trace replay: feed given token ids through the model step by step and write logits.

Nothing is sampled and nothing is scheduled: every line of the trace is one call of the
engine's own step function, on the engine's own model, cache and kernels.

A trace is a sequence of JSON objects, one per step::

    {"step": 0, "entries": [{"id": "a", "tokens": [5, 17, 3], "want": [0, 2]}], "end": []}

``entries``: per request its next tokens and the places among them whose logits are wanted;
``end``: requests that are finished after the step (their pages and row are given back).
For a step with wanted places the logits ``[wanted, vocab]`` are written to ``<out>/<step>.f32``
as little-endian float32 in the order of the entries and of ``want``.  Beside them
``<out>/pages.jsonl`` gets one line per step with the page ids that every request of the step held
in every cache group when the step ran (``{"step": 0, "pages": {"a": {"0": [3, 7]}}}``): a page id
that turns up under two requests in different steps is a page that was used again.  With
``--taps`` a step's intermediates (the residual stream after every layer, the routed experts) go to
``<out>/<step>.taps.safetensors``.
"""
from __future__ import annotations

import json
import os
import sys

from .runner import ModelRunner, StepEntry, kernels_for_program


def pages_held(runner: ModelRunner, request_ids) -> dict[str, dict[str, list[int]]]:
    """request -> cache group index -> the page ids it holds now, in the order of its tokens."""
    cache = runner.cache
    out = {}
    for request_id in request_ids:
        if cache.has_row(request_id):
            row = cache.row_of(request_id)
            out[str(request_id)] = {str(g.index): [int(p) for p in g.table[row] if p >= 0] for g in cache.groups}
    return out


def replay_step(runner: ModelRunner, record: dict, out_dir: str | None, taps: dict | None = None,
                pages_log=None):
    """Run one trace record; returns the logits array (or None).  ``taps`` receives intermediates;
    ``pages_log`` (a text stream) the page ids the step's requests held while it ran."""
    entries = [StepEntry(str(e["id"]), [int(t) for t in e["tokens"]], [int(w) for w in e.get("want", [])])
               for e in record.get("entries", [])]
    logits = None
    if entries:
        result = runner.step(entries, taps=taps)
        if result.shape[0]:
            logits = result.cpu().numpy().astype("<f4", copy=False)
            if out_dir is not None:
                logits.tofile(os.path.join(out_dir, f"{record['step']}.f32"))
    if pages_log is not None:
        pages_log.write(json.dumps({"step": record["step"], "pages": pages_held(runner, [e.request_id for e in entries])}) + "\n")
        pages_log.flush()
    for request_id in record.get("end", []):
        runner.release(str(request_id))
    return logits


def _write_taps(taps: dict, path: str) -> None:
    from safetensors.torch import save_file
    tensors = {}
    for position, hidden in enumerate(taps.get("layer_out", [])):
        tensors[f"layer_out.{position}"] = hidden.float().cpu().contiguous()
    for layer, (ids, weights) in enumerate(taps.get("router", [])):
        tensors[f"router.{layer}.ids"] = ids.cpu().contiguous()
        tensors[f"router.{layer}.weights"] = weights.float().cpu().contiguous()
    save_file(tensors, path)


def replay_stream(runner: ModelRunner, lines, out_dir: str, report=sys.stdout, with_taps: bool = False) -> int:
    """Replay records from an iterable of JSON lines; prints ``done <step>`` after each."""
    os.makedirs(out_dir, exist_ok=True)
    steps = 0
    with open(os.path.join(out_dir, "pages.jsonl"), "w") as pages_log:
        for line in lines:
            line = line.strip()
            if not line:
                continue
            record = json.loads(line)
            taps = {} if with_taps else None
            replay_step(runner, record, out_dir, taps=taps, pages_log=pages_log)
            if taps:
                _write_taps(taps, os.path.join(out_dir, f"{record['step']}.taps.safetensors"))
            print(f"done {record['step']}", file=report, flush=True)
            steps += 1
    return steps


def pool_tokens(max_tokens: int, page_size: int, max_requests: int) -> int:
    """Tokens of cache for ``--max-tokens`` (the live requests' lengths, each rounded up to a multiple of
    64, added up).  Pages that divide 64 hold exactly that; with other page sizes (48, 128) a request's
    last page may reach beyond its multiple of 64, by less than a page per live request."""
    rounded = -(-max_tokens // 64) * 64
    if 64 % page_size == 0:
        return rounded
    return (-(-rounded // page_size) + max_requests) * page_size


def main(argv=None) -> int:
    import argparse
    parser = argparse.ArgumentParser(prog="trace_run", description=__doc__.split("\n\n")[0])
    parser.add_argument("--model", required=True, help="folder with config.json and model.safetensors")
    parser.add_argument("--dtype", required=True, choices=["bfloat16", "float32"])
    parser.add_argument("--out", required=True, help="folder for the <step>.f32 files")
    parser.add_argument("--max-tokens", type=int, required=True,
                        help="most tokens live requests hold at any time (each rounded up to a page multiple)")
    parser.add_argument("--page-size", type=int, default=64,
                        help="tokens per cache page: any size the engine takes (a multiple of 8)")
    parser.add_argument("--max-requests", type=int, default=8, help="most requests live at a time")
    parser.add_argument("--taps", action="store_true", help="also write every step's intermediates")
    parser.add_argument("--device", default="cuda", choices=["cuda", "cpu"],
                        help="cpu runs only with a stand-in for the HIP kernels named in SPARSEENGINE_AMD_KERNELS (tests)")
    args = parser.parse_args(argv)
    try:
        kernels, device = kernels_for_program(args.device)
    except ValueError as exc:
        parser.error(str(exc))
    if args.page_size <= 0 or args.page_size % 8:
        parser.error("--page-size must be a positive multiple of 8")
    print(f"[trace_run] loading {args.model} ({args.dtype})", file=sys.stderr, flush=True)
    runner = ModelRunner.from_folder(
        args.model, dtype=args.dtype, device=device, kernels=kernels, kv_page_size=args.page_size,
        num_kvcache_tokens=pool_tokens(args.max_tokens, args.page_size, args.max_requests),
        max_num_seqs=args.max_requests)
    print("[trace_run] ready", file=sys.stderr, flush=True)
    replay_stream(runner, sys.stdin, args.out, with_taps=args.taps)
    return 0
