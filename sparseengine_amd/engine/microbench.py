"""Throughput of the whole engine (scheduler, step function, sampler) for given prompt lengths and
batch sizes: ``python -m sparseengine_amd bench``.

The reference's counterpart is benchmark/microbench.py:968-1070; its option names are kept where the
option exists here (``--model_path --lengths --batch_sizes --output_len --temperature --top_p
--hyper_params --max_model_len_override --output_jsonl``).  One case = ``batch`` random prompts of
``length`` tokens, each generating ``output_len`` tokens with ``ignore_eos``; steps that bring prompt
tokens count as prefill, the others as decode, as ``LLM.step`` reports them
(engine/llm_engine.py:1976-2055).
"""
from __future__ import annotations

import argparse
import json
import random
import sys
import time


def _json_arg(text: str) -> dict:
    if text.startswith("@"):
        with open(text[1:]) as fh:
            text = fh.read()
    value = json.loads(text)
    if not isinstance(value, dict):
        raise ValueError("--hyper_params must be a JSON object")
    return value


def run_case(llm, length: int, batch: int, output_len: int, temperature: float, top_p: float, seed: int,
             sync=None) -> dict:
    """Feed ``batch`` random prompts and step until all have finished; returns the case's figures."""
    from ..sampling.params import SamplingParams
    rng = random.Random(seed)
    params = SamplingParams(temperature=temperature, top_p=top_p, max_tokens=output_len, ignore_eos=True)
    for _ in range(batch):
        llm.add_request([rng.randrange(llm.vocab_size) for _ in range(length)], params)
    sync = sync or (lambda: None)
    prefill_tokens = decode_tokens = prefill_steps = decode_steps = 0
    prefill_s = decode_s = 0.0
    first_token_s = None
    completions = 0
    sync()
    started = time.perf_counter()
    while not llm.is_finished():
        t0 = time.perf_counter()
        finished, count = llm.step()
        sync()
        dt = time.perf_counter() - t0
        if count > 0:
            prefill_tokens, prefill_steps, prefill_s = prefill_tokens + count, prefill_steps + 1, prefill_s + dt
        elif count < 0:
            if first_token_s is None:
                first_token_s = t0 - started
            decode_tokens, decode_steps, decode_s = decode_tokens - count, decode_steps + 1, decode_s + dt
        completions += len(finished)
    total_s = time.perf_counter() - started
    return {
        "length": length, "batch_size": batch, "output_len": output_len, "completed": completions,
        "prefill_tokens": prefill_tokens, "prefill_steps": prefill_steps, "prefill_s": round(prefill_s, 6),
        "prefill_tok_s": round(prefill_tokens / prefill_s, 1) if prefill_s else None,
        "decode_tokens": decode_tokens, "decode_steps": decode_steps, "decode_s": round(decode_s, 6),
        "decode_tok_s": round(decode_tokens / decode_s, 1) if decode_s else None,
        "ms_per_decode_step": round(decode_s / decode_steps * 1e3, 3) if decode_steps else None,
        "time_to_first_decode_s": round(first_token_s, 6) if first_token_s is not None else None,
        "total_s": round(total_s, 6),
    }


def build_parser() -> argparse.ArgumentParser:
    parser = argparse.ArgumentParser(prog="python -m sparseengine_amd bench", description=__doc__,
                                     formatter_class=argparse.RawDescriptionHelpFormatter)
    parser.add_argument("--model_path", "--model", dest="model_path", required=True,
                        help="model folder (config.json; weights unless tiny_random is set in --hyper_params)")
    parser.add_argument("--lengths", default="1024,2048", help="prompt lengths, comma separated")
    parser.add_argument("--batch_sizes", default="1,8", help="requests per case, comma separated")
    parser.add_argument("--output_len", type=int, default=64, help="generated tokens per request")
    parser.add_argument("--temperature", type=float, default=0.0)
    parser.add_argument("--top_p", type=float, default=1.0)
    parser.add_argument("--max_model_len_override", type=int, default=None,
                        help="max_model_len; default: longest length + output_len + 100")
    parser.add_argument("--hyper_params", default="{}", help="keyword arguments of LLM(...) as JSON or @file")
    parser.add_argument("--seed", type=int, default=0)
    parser.add_argument("--device", default="cuda", choices=["cuda", "cpu"],
                        help="cpu runs only with a stand-in for the HIP kernels named in SPARSEENGINE_AMD_KERNELS (tests)")
    parser.add_argument("--output_jsonl", default=None, help="write one JSON row per case here as well")
    return parser


def main(argv=None, llm_factory=None) -> int:
    args = build_parser().parse_args(argv)
    lengths = [int(x) for x in args.lengths.split(",") if x]
    batches = [int(x) for x in args.batch_sizes.split(",") if x]
    if not lengths or not batches or min(lengths) <= 0 or min(batches) <= 0 or args.output_len <= 0:
        raise SystemExit("bench: --lengths, --batch_sizes and --output_len must be positive")
    kwargs = _json_arg(args.hyper_params)
    kwargs.setdefault("max_model_len", args.max_model_len_override or max(lengths) + args.output_len + 100)
    kwargs.setdefault("max_num_seqs_in_batch", max(batches))
    if llm_factory is None:
        from .llm import LLM
        from .runner import kernels_for_program
        kernels, device = kernels_for_program(args.device)
        if kernels is not None:
            kwargs.update(_kernels=kernels, _device=device)
        llm_factory = LLM
    llm = llm_factory(args.model_path, **kwargs)
    sync = None
    try:
        import torch
        if torch.cuda.is_available():
            sync = torch.cuda.synchronize
    except ImportError:
        pass
    out = open(args.output_jsonl, "w") if args.output_jsonl else None
    try:
        run_case(llm, min(lengths), 1, 2, 0.0, 1.0, args.seed, sync)      # warm-up: libraries, buffers
        for length in lengths:
            for batch in batches:
                row = run_case(llm, length, batch, args.output_len, args.temperature, args.top_p, args.seed, sync)
                line = json.dumps(row)
                print(line, flush=True)
                if out:
                    out.write(line + "\n")
                    out.flush()
    finally:
        if out:
            out.close()
        llm.exit()
    return 0


if __name__ == "__main__":
    sys.exit(main())
