"""Command line: ``python -m sparseengine_amd <command>``.

  generate   run prompts through ``LLM.generate`` (every ``Config`` field is ``--kebab-name``,
             every ``SamplingParams`` field too)
  random     write a model folder (config.json, model.safetensors) from a configuration and a seed
  replay     the trace replay tool (same as bin/trace_run)
  bench      throughput of the whole engine for given prompt lengths and batch sizes (the reference's
             benchmark/microbench.py options: --model_path --lengths --batch_sizes --output_len ...)

The reference has no generation command line (its console scripts are the server's,
pyproject.toml:66-69); option names here are the names of its ``Config`` and ``SamplingParams``.
"""
from __future__ import annotations

import argparse
import dataclasses
import json
import sys
import typing


def _add_dataclass_options(parser, cls, skip=(), prefix_if_taken: str = ""):
    """One option per field.  A name another dataclass has taken already gets ``prefix_if_taken``
    (``eos_token_ids`` is a field of ``Config`` and of ``SamplingParams``: the request-level one is
    ``--sampling-eos-token-ids``)."""
    hints = typing.get_type_hints(cls)
    taken = {action.dest for action in parser._actions}
    for f in dataclasses.fields(cls):
        if not f.init or f.name in skip:
            continue
        dest = f.name if f.name not in taken else prefix_if_taken + f.name
        flag = "--" + dest.replace("_", "-")
        kind = hints.get(f.name, str)
        if kind is bool:
            parser.add_argument(flag, dest=dest, action=argparse.BooleanOptionalAction, default=None)
        else:
            parser.add_argument(flag, dest=dest, default=None, help=f"({kind})")


def _coerce(value: str):
    try:
        return json.loads(value)
    except (ValueError, TypeError):
        return value


def _collect(args, cls, skip=(), prefix: str = ""):
    out = {}
    for f in dataclasses.fields(cls):
        if not f.init or f.name in skip:
            continue
        value = getattr(args, prefix + f.name, None) if hasattr(args, prefix + f.name) else getattr(args, f.name, None)
        if value is not None:
            out[f.name] = _coerce(value) if isinstance(value, str) else value
    return out


def build_parser() -> argparse.ArgumentParser:
    from .config.runtime import Config
    from .sampling.params import SamplingParams
    parser = argparse.ArgumentParser(prog="python -m sparseengine_amd", description=__doc__,
                                     formatter_class=argparse.RawDescriptionHelpFormatter)
    sub = parser.add_subparsers(dest="command", required=True)

    gen = sub.add_parser("generate", help="generate completions")
    gen.add_argument("--model", required=True, help="folder with config.json (and weights unless --tiny-random)")
    gen.add_argument("--prompt", action="append", default=[], help="text prompt (needs tokenizer.json); repeatable")
    gen.add_argument("--prompt-ids", action="append", default=[],
                     help="prompt as JSON list of token ids, or a file with one JSON list per line; repeatable")
    gen.add_argument("--device", default="cuda", choices=["cuda", "cpu"],
                     help="cpu runs only with a stand-in for the HIP kernels named in SPARSEENGINE_AMD_KERNELS (tests)")
    _add_dataclass_options(gen, Config, skip=("model",))
    _add_dataclass_options(gen, SamplingParams, prefix_if_taken="sampling_")

    rnd = sub.add_parser("random", help="write a random-weights model folder")
    rnd.add_argument("--config", required=True, help="config.json file (or JSON text) of the architecture")
    rnd.add_argument("--out", required=True)
    rnd.add_argument("--seed", type=int, default=0)
    rnd.add_argument("--std", type=float, default=0.02)
    rnd.add_argument("--norm-std", type=float, default=0.1)
    rnd.add_argument("--bias-std", type=float, default=0.1)

    rep = sub.add_parser("replay", help="trace replay (see bin/trace_run)", add_help=False)
    rep.add_argument("rest", nargs=argparse.REMAINDER)
    ben = sub.add_parser("bench", help="engine throughput by prompt length and batch size", add_help=False)
    ben.add_argument("rest", nargs=argparse.REMAINDER)
    return parser


def main(argv=None) -> int:
    from .config.runtime import Config
    from .sampling.params import SamplingParams
    argv = sys.argv[1:] if argv is None else list(argv)
    if argv and argv[0] == "replay":       # its options are its own (they begin with dashes, which the
        from .engine.replay import main as replay_main      # sub-command parser would claim)
        return replay_main(argv[1:])
    if argv and argv[0] == "bench":
        from .engine.microbench import main as bench_main
        return bench_main(argv[1:])
    parser = build_parser()
    args = parser.parse_args(argv)
    if args.command == "random":
        import os
        from .weights.random_weights import write_model_folder
        text = open(args.config).read() if os.path.isfile(args.config) else args.config
        write_model_folder(args.out, json.loads(text), args.seed,
                           dict(std=args.std, norm_std=args.norm_std, bias_std=args.bias_std))
        print(args.out)
        return 0

    import os
    from .engine.llm import LLM
    prompts = list(args.prompt)
    for item in args.prompt_ids:
        if os.path.isfile(item):
            with open(item) as fh:
                prompts += [json.loads(line) for line in fh if line.strip()]
        else:
            prompts.append(json.loads(item))
    if not prompts:
        parser.error("give at least one --prompt or --prompt-ids")
    from .engine.runner import kernels_for_program
    try:
        kernels, device = kernels_for_program(args.device)
    except ValueError as exc:
        parser.error(str(exc))
    seam = {} if kernels is None else {"_kernels": kernels, "_device": device}
    llm = LLM(args.model, **_collect(args, Config, skip=("model",)), **seam)
    params = SamplingParams(**_collect(args, SamplingParams, prefix="sampling_"))
    for prompt, out in zip(prompts, llm.generate(prompts, params, use_tqdm=False)):
        print(json.dumps({"prompt": prompt, **out}))
    return 0


if __name__ == "__main__":
    sys.exit(main())
