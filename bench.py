"""Decode and prefill throughput at MiniMax-M2 layer sizes on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W]

Model: the sizes of MiniMax M2 (hidden 3072, 48 query / 8 kv heads of 128, rotary 64, 256 experts
top-8 of width 1536, vocabulary 200064) cut to 16 of its 62 layers, random weights, bfloat16.
A "step" is one decode step of a batch of 8 requests whose prompts were 2048 random token ids
(sampling greedily, token ids read back each step).  One JSON line is printed: ``value`` is decoded
tokens per second at batch 8; ``prefill`` is a 2048-token prompt in one step with its tokens spread evenly
over all experts (``frac``: its flops against the matrix peak, ``hbm_frac``: the bytes it has to read against
8 TB/s, ``experts_touched``: the experts per layer that its tokens take); ``points`` holds decode at batch 1 and
64 and the prefill of eight 2048-token prompts in one step; ``roofline`` prices the batch-8 decode
step against 8 TB/s and ``point_rooflines`` the other decode points the same way (every weight the
step uses once - the experts it touched are counted from the step's own routing - and the cache of
the live requests).  With random weights the router itself sends the tokens of a prompt to a few dozen experts
past the first layer, which makes a prompt cheaper than real weights would: ``prefill_natural_routing`` is that
step (``experts_touched``: the mean number of experts per layer that its tokens chose); in ``prefill`` every token
is sent to eight experts drawn evenly from all 256 instead (the routing is replaced after the router has run, so
the router's own work is still in the time).  ``roofline.measured_peak`` is what a kernel of this engine that does nothing but read 8 GiB
reaches on this box at the start of the run (``memory`` holds that and the rate of a copy), and ``measured_frac`` /
``point_rooflines_measured`` price the same steps against it.  ``kernels`` holds, for the prefill
and for every decode point, one further step with events around each call of the kernels object: the time of
experts, attention, the dense products and the head, with the bytes (decode) or flops (prefill) each has to do
per second.  ``--prompt-len C --no-prefill --fake-context`` gives decode steps at other context lengths.

    python bench.py --workload long_context | serving

runs a whole workload through the engine's entry point (``LLM``: scheduler, cache manager, step
function, sampler) instead and prints one JSON line of its own: ``long_context`` is 4 requests of
131072 random token ids, prefilled in portions of 8192 tokens, then decode steps at batch 4 (8 layers);
``serving`` is 32 requests with prompts of 512 to 16384 tokens in portions of 512 tokens beside the
decoded tokens of the others, 512 output tokens each (24 layers, 217 GiB).
"""
from __future__ import annotations

import argparse
import json
import sys
import time

HBM_PEAK = 8.0e12            # bytes / s
MFMA_PEAK = {"bf16": 2.5e15, "fp32": 157.3e12}

MODEL = dict(
    architectures=["MiniMaxM2ForCausalLM"], model_type="minimax_m2", hidden_size=3072,
    num_attention_heads=48, num_key_value_heads=8, head_dim=128, rotary_dim=64, rope_theta=5000000.0,
    num_local_experts=256, num_experts_per_tok=8, intermediate_size=1536, vocab_size=200064,
    rms_norm_eps=1e-6, use_qk_norm=True, max_position_embeddings=204800, tie_word_embeddings=False)
FULL_MODEL_LAYERS = 62
PROMPT_LEN = 2048
CONTEXT_LEN = 8192


def main() -> int:
    global PROMPT_LEN, CONTEXT_LEN
    parser = argparse.ArgumentParser()
    parser.add_argument("--gpus", type=int, default=1)
    parser.add_argument("--steps", type=int, default=64)
    parser.add_argument("--warmup", type=int, default=8)
    parser.add_argument("--layers", type=int, default=16)
    parser.add_argument("--batch", type=int, default=8)
    parser.add_argument("--dtype", default="bfloat16", choices=["bfloat16", "float32"])
    parser.add_argument("--points", default="1,64", help="further decode batch sizes, comma separated")
    parser.add_argument("--kv-requests", type=int, default=64, help="requests of full context the cache is sized for")
    parser.add_argument("--prompt-len", type=int, default=PROMPT_LEN,
                        help="tokens a request holds when its decoding starts (with --no-prefill --fake-context: decode "
                             "steps at other context lengths; the cache is sized for --kv-requests of this plus 6144)")
    parser.add_argument("--no-prefill", action="store_true", help="skip the prefill measurement (for profiling decode)")
    parser.add_argument("--no-decode", action="store_true", help="skip the decode measurements (for profiling prefill)")
    parser.add_argument("--prefill-prompts", type=int, default=8,
                        help="also time this many 2048-token prompts in one step (points.prefill_Nx2048); 1: skip")
    parser.add_argument("--prefill-routing", default="both", choices=["both", "natural", "uniform"],
                        help="profiling aid: which of the two prefill measurements to run (a reported line needs both)")
    parser.add_argument("--workload", default="step", choices=["step", "long_context", "serving"],
                        help="step: the decode / prefill steps described above; the others: a whole workload "
                             "through the engine's entry point")
    parser.add_argument("--output-len", type=int, default=None, help="decoded tokens per request of a workload")
    parser.add_argument("--kv-page-size", type=int, default=None,
                        help="tokens per cache page of a workload (default: the engine's; 16 makes block tables of 8192 "
                             "pages for the long-context workload)")
    parser.add_argument("--fake-context", action="store_true",
                        help="profiling aid, never used for reported numbers: reserve the prompts' cache pages "
                             "without computing them, so that a kernel trace holds decode steps only")
    args = parser.parse_args()
    if args.gpus != 1:
        print(f"bench.py measures one GPU; --gpus {args.gpus} is not supported by this engine")
        return 2

    if args.workload != "step":
        return run_workload(args)
    PROMPT_LEN, CONTEXT_LEN = args.prompt_len, max(CONTEXT_LEN, args.prompt_len + 6144)

    import torch

    import sparseengine_amd  # noqa: F401
    from sparseengine_amd.engine.runner import ModelRunner, StepEntry
    from sparseengine_amd.sampling.params import SamplingParams
    from sparseengine_amd.sampling.sampler import Sampler

    cfg = dict(MODEL, num_hidden_layers=args.layers)
    from sparseengine_amd.kernels.hip_ops import HipKernels
    memory = HipKernels().measure_memory(gib=8.0)       # before the model is there: what this box's memory delivers
    torch.cuda.empty_cache()
    measured_peak = memory["read_GBps"] * 1e9
    print(f"[bench] memory: a kernel that only reads 8 GiB {memory['read_GBps']:.0f} GB/s, a copy "
          f"{memory['copy_GBps']:.0f} GB/s (read + written)", file=sys.stderr, flush=True)
    t0 = time.time()
    runner = ModelRunner.from_random(
        cfg, seed=0, options=dict(std=0.02, norm_std=0.1, bias_std=0.01), on_device=True, dtype=args.dtype,
        kv_page_size=64, num_kvcache_tokens=args.kv_requests * CONTEXT_LEN,
        max_num_seqs=max([64, args.batch] + [int(x) for x in args.points.split(",") if x]),
        max_model_len=CONTEXT_LEN)
    torch.cuda.synchronize()
    print(f"[bench] model built in {time.time() - t0:.1f} s, "
          f"{torch.cuda.memory_allocated() / 2**30:.1f} GiB allocated", file=sys.stderr, flush=True)
    sampler = Sampler(runner.kernels, runner.device, 0)
    greedy = SamplingParams(temperature=0.0, max_tokens=1 << 20, ignore_eos=True)
    gen = torch.Generator().manual_seed(0)

    def prompt():
        return torch.randint(0, cfg["vocab_size"], (PROMPT_LEN,), generator=gen).tolist()

    def sync():
        torch.cuda.synchronize()

    def prefill(ids, n_at_once=4):
        """Prompts of the requests ``ids``, a few whole prompts per step; returns their first tokens."""
        first = {}
        for i in range(0, len(ids), n_at_once):
            chunk = ids[i:i + n_at_once]
            logits = runner.step([StepEntry(r, prompt(), [PROMPT_LEN - 1]) for r in chunk])
            tokens = sampler.sample(logits, [(greedy, [], [])] * len(chunk), [(0, 0)] * len(chunk))
            first.update(dict(zip(chunk, tokens)))
        return first

    def decode(batch, steps, warmup, tag):
        ids = [f"{tag}{i}" for i in range(batch)]
        if args.fake_context:
            runner.cache.append([(runner.admit(r), PROMPT_LEN) for r in ids])
            last = dict(zip(ids, torch.randint(0, cfg["vocab_size"], (batch,), generator=gen).tolist()))
        else:
            last = prefill(ids)
        rows = [(greedy, [], [])] * batch
        seeds = [(0, 0)] * batch

        def one():
            logits = runner.step([StepEntry(r, [last[r]], [0]) for r in ids])
            for r, t in zip(ids, sampler.sample(logits, rows, seeds)):
                last[r] = t
            if args.fake_context:       # an empty cache gives every request the same token: draw them
                last.update(zip(ids, torch.randint(0, cfg["vocab_size"], (batch,), generator=gen).tolist()))
        for _ in range(warmup):
            one()
        sync()
        start = time.perf_counter()
        for _ in range(steps):
            one()
        sync()
        seconds = time.perf_counter() - start
        taps = {}
        runner.step([StepEntry(r, [last[r]], []) for r in ids], taps=taps)       # untimed: which experts a step touches
        distinct = [int(torch.unique(i).numel()) for i, _ in taps["router"]]
        context = PROMPT_LEN + warmup + steps / 2
        calls = time_calls(runner.kernels, lambda: runner.step([StepEntry(r, [last[r]], [0]) for r in ids]))
        for r in ids:
            runner.release(r)
        return seconds / steps, distinct, context, calls

    itemsize = 2 if args.dtype == "bfloat16" else 4
    h, H, Hkv, D, E, K, I, V, L = (cfg["hidden_size"], cfg["num_attention_heads"], cfg["num_key_value_heads"],
                                   cfg["head_dim"], cfg["num_local_experts"], cfg["num_experts_per_tok"],
                                   cfg["intermediate_size"], cfg["vocab_size"], args.layers)
    dense_layer = ((H + 2 * Hkv) * D * h + h * H * D) * itemsize + E * h * 4
    expert_bytes = 3 * I * h * itemsize
    kv_token_layer = 2 * Hkv * D * itemsize

    def decode_bytes(batch, distinct, context):
        return (L * dense_layer + sum(distinct) * expert_bytes + V * h * itemsize
                + batch * context * kv_token_layer * L)

    def decode_calls(batch, distinct, context, calls):
        """The calls a decode step's time goes to: milliseconds per step and the bytes each has to read per second."""
        needs = {"moe_experts": sum(distinct) * expert_bytes, "paged_attention": batch * context * kv_token_layer * L,
                 f"linear_{(H + 2 * Hkv) * D}": L * (H + 2 * Hkv) * D * h * itemsize, f"linear_{h}": L * h * H * D * itemsize,
                 f"linear_{V}": V * h * itemsize}
        label = {"moe_experts": "experts", "paged_attention": "attention", f"linear_{(H + 2 * Hkv) * D}": "qkv",
                 f"linear_{h}": "o", f"linear_{V}": "head"}
        out = {label[k]: {"ms": round(calls[k], 3), "GB/s": round(needs[k] / calls[k] / 1e6, 1)} for k in needs if calls.get(k)}
        out["rest"] = {"ms": round(sum(v for k, v in calls.items() if k not in needs), 3)}
        return out

    # ---- prefill of one 2048-token prompt
    natural = not args.no_prefill and args.prefill_routing != "uniform"
    times = [] if natural else [0.0, 1.0]
    for i in range(4 if natural else 0):
        sync()
        t = time.perf_counter()
        runner.step([StepEntry(f"p{i}", prompt(), [PROMPT_LEN - 1])])
        sync()
        times.append(time.perf_counter() - t)
        runner.release(f"p{i}")
    prefill_s = min(times[1:])
    T = PROMPT_LEN
    kernels = {}      # per call of the kernels object, from one step with events around each
    prefill_bytes = touched = None
    uniform_s = uniform_bytes = None
    if natural:     # untimed: the experts the prompt touches, layer by layer, are what it has to read
        taps = {}
        runner.step([StepEntry("p_taps", prompt(), [PROMPT_LEN - 1])], taps=taps)
        runner.release("p_taps")
        touched = [int(torch.unique(i).numel()) for i, _ in taps["router"]]
        prefill_bytes = L * dense_layer + sum(touched) * expert_bytes + V * h * itemsize
        del taps
        calls = time_calls(runner.kernels, lambda: runner.step([StepEntry("p_calls", prompt(), [PROMPT_LEN - 1])]))
        runner.release("p_calls")
        work = {"moe_experts": ("experts", 2 * T * K * 3 * I * h * L), "paged_attention": ("attention", 4 * H * D * T * (T + 1) / 2 * L),
                f"linear_{(H + 2 * Hkv) * D}": ("qkv", 2 * T * h * (H + 2 * Hkv) * D * L), f"linear_{h}": ("o", 2 * T * H * D * h * L)}
        kernels[f"prefill_{T}_natural_routing"] = {name: {"ms": round(calls[k], 3), "TFLOP/s": round(flops / calls[k] / 1e9, 1)}
                                                   for k, (name, flops) in work.items() if calls.get(k)}
        kernels[f"prefill_{T}_natural_routing"]["rest"] = {"ms": round(sum(v for k, v in calls.items() if k not in work), 3)}
    if not args.no_prefill and args.prefill_routing != "natural":
        # the same step with even expert load: eight distinct experts per token, drawn uniformly
        dev_gen = torch.Generator(device="cuda").manual_seed(1)
        even = [torch.rand(T, E, generator=dev_gen, device="cuda").topk(K, dim=-1).indices.to(torch.int32).contiguous()
                for _ in range(L)]
        uniform_times = []
        for i in range(3):
            sync()
            t = time.perf_counter()
            runner.step([StepEntry(f"u{i}", prompt(), [PROMPT_LEN - 1])], forced_routing=even)
            sync()
            uniform_times.append(time.perf_counter() - t)
            runner.release(f"u{i}")
        uniform_s = min(uniform_times[1:])
        uniform_bytes = L * dense_layer + L * min(E, T * K) * expert_bytes + V * h * itemsize
        calls = time_calls(runner.kernels, lambda: runner.step([StepEntry("u_calls", prompt(), [PROMPT_LEN - 1])],
                                                               forced_routing=even))
        runner.release("u_calls")
        work = {"moe_experts": ("experts", 2 * T * K * 3 * I * h * L), "paged_attention": ("attention", 4 * H * D * T * (T + 1) / 2 * L),
                f"linear_{(H + 2 * Hkv) * D}": ("qkv", 2 * T * h * (H + 2 * Hkv) * D * L), f"linear_{h}": ("o", 2 * T * H * D * h * L)}
        kernels[f"prefill_{T}"] = {name: {"ms": round(calls[k], 3), "TFLOP/s": round(flops / calls[k] / 1e9, 1)}
                                   for k, (name, flops) in work.items() if calls.get(k)}
        if calls.get("moe_experts"):      # every expert table is read once: the experts' share is a matter of memory
            kernels[f"prefill_{T}"]["experts"]["GB/s"] = round(L * min(E, T * K) * expert_bytes / calls["moe_experts"] / 1e6, 1)
        kernels[f"prefill_{T}"]["rest"] = {"ms": round(sum(v for k, v in calls.items() if k not in work), 3)}
        del even
    prefill_flops = L * (2 * T * h * (H + 2 * Hkv) * D + 2 * T * H * D * h + 2 * T * h * E + 2 * T * K * 3 * I * h
                         + 4 * H * D * T * (T + 1) / 2) + 2 * V * h
    peak = MFMA_PEAK["bf16" if args.dtype == "bfloat16" else "fp32"]
    print(f"[bench] prefill {T} tokens: {prefill_s * 1e3:.1f} ms", file=sys.stderr, flush=True)

    many_prompts = None
    if args.prefill_prompts > 1 and natural:      # several prompts in one step: hundreds of rows per expert
        n, best = args.prefill_prompts, float("inf")
        for i in range(3):
            ids = [f"m{i}_{j}" for j in range(n)]
            entries = [StepEntry(r, prompt(), [PROMPT_LEN - 1]) for r in ids]
            sync()
            t = time.perf_counter()
            runner.step(entries)
            sync()
            best = min(best, time.perf_counter() - t)
            for r in ids:
                runner.release(r)
        many_prompts = (f"prefill_{n}x{T}", round(n * T / best, 1))
        print(f"[bench] prefill {n} x {T} tokens in one step: {best * 1e3:.1f} ms, {n * T / best:.0f} tokens/s",
              file=sys.stderr, flush=True)

    # ---- decode
    if args.no_decode:
        return 0
    step_s, distinct, context, calls = decode(args.batch, args.steps, args.warmup, "d")
    kernels[f"decode_b{args.batch}"] = decode_calls(args.batch, distinct, context, calls)
    print(f"[bench] decode batch {args.batch}: {step_s * 1e3:.2f} ms/step, {sum(distinct) / len(distinct):.0f} experts touched "
          f"per layer, {decode_bytes(args.batch, distinct, context) / step_s / 1e9:.0f} GB/s", file=sys.stderr, flush=True)
    points, point_rooflines, point_rooflines_measured = {}, {}, {}
    for b in [int(x) for x in args.points.split(",") if x]:
        s, d, c, calls = decode(b, max(8, args.steps // 2), max(2, args.warmup // 2), f"b{b}_")
        kernels[f"decode_b{b}"] = decode_calls(b, d, c, calls)
        points[f"decode_b{b}"] = round(b / s, 1)
        point_rooflines[f"decode_b{b}"] = round(decode_bytes(b, d, c) / s / HBM_PEAK, 4)
        point_rooflines_measured[f"decode_b{b}"] = round(decode_bytes(b, d, c) / s / measured_peak, 4)
        print(f"[bench] decode batch {b}: {s * 1e3:.2f} ms/step, {sum(d) / len(d):.0f} experts touched per layer, "
              f"{decode_bytes(b, d, c) / s / 1e9:.0f} GB/s", file=sys.stderr, flush=True)

    if many_prompts:
        points[many_prompts[0]] = many_prompts[1]
    achieved = decode_bytes(args.batch, distinct, context) / step_s
    natural_record = None if not natural else {
        "value": round(T / prefill_s, 1), "tokens": T, "ms": round(prefill_s * 1e3, 3), "routing": "the model's own (random weights)",
        "frac": round(prefill_flops / prefill_s / peak, 5),
        # a 2048-token step reads every expert it touches for a few dozen rows each: memory bound too
        "hbm_frac": round(prefill_bytes / prefill_s / HBM_PEAK, 4),
        "hbm_measured_frac": round(prefill_bytes / prefill_s / measured_peak, 4),
        "flops": prefill_flops, "bytes": prefill_bytes, "experts_touched": round(sum(touched) / len(touched), 1)}
    uniform_record = None if uniform_s is None else {
        "value": round(T / uniform_s, 1), "tokens": T, "ms": round(uniform_s * 1e3, 3), "routing": "even over all experts",
        "frac": round(prefill_flops / uniform_s / peak, 5), "hbm_frac": round(uniform_bytes / uniform_s / HBM_PEAK, 4),
        "hbm_measured_frac": round(uniform_bytes / uniform_s / measured_peak, 4),
        "flops": prefill_flops, "bytes": uniform_bytes, "experts_touched": min(E, T * K)}
    line = {
        "metric": f"decode tok/s @ batch {args.batch} (MiniMax-M2 sizes, {L} layers, 1 GPU)", "value": round(args.batch / step_s, 1),
        "unit": "tokens/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(step_s * 1e3, 3), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16" if args.dtype == "bfloat16" else "fp32", "data": "synthetic: random token ids, random weights",
        "config": {"model": "MiniMax-M2 layer sizes", "num_layers": L, "model_layers": FULL_MODEL_LAYERS,
                   "global_batch": args.batch, "seq_len": CONTEXT_LEN, "prompt_len": PROMPT_LEN, "hidden_size": h,
                   "num_attention_heads": H, "num_key_value_heads": Hkv, "head_dim": D, "rotary_dim": cfg["rotary_dim"],
                   "num_local_experts": E, "num_experts_per_tok": K, "intermediate_size": I, "vocab_size": V,
                   "kv_page_size": 64, "kv_cache_tokens": args.kv_requests * CONTEXT_LEN,
                   "max_position_embeddings": cfg["max_position_embeddings"], "parallelism": "single GPU"},
        # The 2048-token prompt with its tokens spread evenly over all experts, as a trained router spreads them: every
        # expert table is read.  With this model's random weights the router sends a prompt's tokens to a few dozen
        # experts per layer, which is the cheaper step reported beside it.
        "prefill": uniform_record if uniform_record is not None else natural_record,
        "prefill_natural_routing": natural_record,
        "roofline": {"bound": "hbm", "achieved": round(achieved / 1e9, 1), "peak": HBM_PEAK / 1e9, "unit": "GB/s",
                     "frac": round(achieved / HBM_PEAK, 4), "measured_peak": round(measured_peak / 1e9, 1),
                     "measured_frac": round(achieved / measured_peak, 4)},
        # a kernel that only reads / a kernel that copies 8 GiB, timed at the start of this run
        "memory": memory,
        "points": points,
        "point_rooflines": point_rooflines,
        "point_rooflines_measured": point_rooflines_measured,
        # per call of the kernels object, from one step with events around each: what the step's time goes to
        "kernels": kernels,
    }
    print(json.dumps(line), flush=True)
    return 0


def time_calls(kernels, run) -> dict:
    """Milliseconds per entry point of the kernels object over one call of ``run`` (an untimed step of its own):
    a pair of events around every outermost call.  Dense products are told apart by their number of weight rows.
    The events cost a microsecond or two each, so the figures serve for the calls that a step's time goes to."""
    import torch

    names = ("embedding", "rms_norm", "qk_norm_rope_store", "paged_attention", "route", "moe_experts", "linear")
    spans, depth = [], [0]

    def wrap(name, fn):
        def call(*a, **k):
            if depth[0]:
                return fn(*a, **k)
            label = f"linear_{a[1].shape[0]}" if name == "linear" else name
            first, last = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            depth[0] += 1
            first.record()
            try:
                return fn(*a, **k)
            finally:
                last.record()
                depth[0] -= 1
                spans.append((label, first, last))
        return call

    for name in names:
        setattr(kernels, name, wrap(name, getattr(kernels, name)))
    try:
        run()
    finally:
        for name in names:
            delattr(kernels, name)       # the class's method shows again
    torch.cuda.synchronize()
    total = {}
    for label, first, last in spans:
        total[label] = total.get(label, 0.0) + first.elapsed_time(last)
    return total


def run_workload(args) -> int:
    """A whole workload through ``LLM``: the model is MiniMax-M2's layer sizes with random weights made on
    the device (``tiny_random``), the model folder holds nothing but its config.json."""
    import os
    import random
    import tempfile

    import torch

    from sparseengine_amd import LLM, SamplingParams
    from sparseengine_amd.engine.microbench import run_case

    long_context = args.workload == "long_context"
    layers = 8 if long_context else 24
    folder = tempfile.mkdtemp(prefix="bench_model_")
    with open(os.path.join(folder, "config.json"), "w") as fh:
        json.dump(dict(MODEL, num_hidden_layers=layers, max_position_embeddings=196608), fh)
    sync = torch.cuda.synchronize
    page = {"kv_page_size": args.kv_page_size} if args.kv_page_size else {}
    from sparseengine_amd.kernels.hip_ops import HipKernels
    memory = HipKernels().measure_memory(gib=8.0)       # before the model is there: what this box's memory delivers
    torch.cuda.empty_cache()
    print(f"[bench] memory: a kernel that only reads 8 GiB {memory['read_GBps']:.0f} GB/s, a copy "
          f"{memory['copy_GBps']:.0f} GB/s (read + written)", file=sys.stderr, flush=True)
    t0 = time.time()
    if long_context:
        length, batch, output_len = 131072, 4, args.output_len or 1024
        llm = LLM(folder, tiny_random=True, dtype=args.dtype, num_kvcache_slots=batch * (length + 4096),
                  engine_prefill_chunk_size=8192, max_num_batched_tokens=8192, max_num_seqs_in_batch=batch, **page)
        print(f"[bench] engine built in {time.time() - t0:.1f} s, {torch.cuda.memory_allocated() / 2**30:.1f} GiB "
              f"allocated", file=sys.stderr, flush=True)
        case = run_case(llm, length, batch, output_len, 0.0, 1.0, 0, sync=sync)
        line = {"metric": "4 requests of 131072 tokens through the engine (MiniMax-M2 sizes, 8 layers, 1 GPU)",
                "value": case["prefill_tok_s"], "unit": "prompt tokens/s", "n_gpus": 1, "dtype": args.dtype,
                "data": "synthetic: random token ids, random weights",
                "config": {"num_layers": layers, "requests": batch, "prompt_len": length, "portion": 8192,
                           "output_len": output_len, "kv_page_size": llm.config.kv_page_size},
                "prefill_s": case["prefill_s"], "prefill_steps": case["prefill_steps"],
                "decode_tok_s": case["decode_tok_s"], "ms_per_decode_step": case["ms_per_decode_step"],
                "decode_steps": case["decode_steps"], "total_s": case["total_s"]}
    else:
        requests, output_len = 32, args.output_len or 512
        llm = LLM(folder, tiny_random=True, dtype=args.dtype, num_kvcache_slots=requests * 17408, max_model_len=17408,
                  max_num_seqs_in_batch=requests, max_num_batched_tokens=512 + requests, engine_prefill_chunk_size=512,
                  decode_reservation_tokens=1024, **page)
        for name, tensor in llm.runner.params.items():      # bias N(0, 0.01): routing spreads over all experts
            if name.endswith("router_bias"):
                tensor.mul_(0.1)
        print(f"[bench] engine built in {time.time() - t0:.1f} s, {torch.cuda.memory_allocated() / 2**30:.1f} GiB "
              f"allocated", file=sys.stderr, flush=True)
        rng = random.Random(0)
        prompts = [[rng.randrange(MODEL["vocab_size"]) for _ in range(rng.randrange(512, 16384))] for _ in range(requests)]
        sampling = SamplingParams(temperature=0.0, max_tokens=output_len, ignore_eos=True)
        for prompt in prompts:
            llm.add_request(prompt, sampling)
        # a step's time by what it holds: portions of prompts beside decoded tokens, or decoded tokens alone
        mixed_ms, decode_ms, output_tokens = [], [], 0
        # What a step with a prompt portion has to read: the dense weights once, the tables of the experts its
        # tokens chose (counted in every sixteenth such step, which is then left out of the times: the router's
        # choices are copied out layer by layer) and the cache of every request that is running after it (the
        # portion's own request and the decoding ones).
        itemsize = 2 if args.dtype == "bfloat16" else 4
        h, H, Hkv, D, E, I, V = (MODEL["hidden_size"], MODEL["num_attention_heads"], MODEL["num_key_value_heads"],
                                 MODEL["head_dim"], MODEL["num_local_experts"], MODEL["intermediate_size"], MODEL["vocab_size"])
        dense_once = layers * (((H + 2 * Hkv) * D * h + h * H * D) * itemsize + E * h * 4) + V * h * itemsize
        expert_bytes = 3 * I * h * itemsize
        kv_token = 2 * Hkv * D * itemsize * layers
        run_step, taps_of_step = llm.runner.step, [None]
        llm.runner.step = lambda entries, **kw: run_step(entries, taps=taps_of_step[0], **kw)
        mixed_steps, chosen = [], []           # (seconds, tokens of context), experts chosen per layer in the counted steps
        sync()
        start = time.perf_counter()
        steps_done = 0
        while not llm.is_finished():
            counted = steps_done % 16 == 8
            taps_of_step[0] = {} if counted else None
            t1 = time.perf_counter()
            finished, count = llm.step()
            sync()
            took = time.perf_counter() - t1
            steps_done += 1
            if counted and count > 0:
                chosen.append(sum(int(torch.unique(ids).numel()) for ids, _ in taps_of_step[0]["router"]) / layers)
            elif not counted:
                (mixed_ms if count > 0 else decode_ms).append(took * 1e3)
                if count > 0:
                    mixed_steps.append((took, sum(s.num_computed_tokens for s in llm.scheduler.running)))
            output_tokens += sum(len(f[1]) for f in finished)
        seconds = time.perf_counter() - start
        prompt_tokens = sum(len(p) for p in prompts)
        experts_read = sum(chosen) / len(chosen) if chosen else float(E)
        weights_once = dense_once + layers * experts_read * expert_bytes
        mixed_rates = sorted((weights_once + context * kv_token) / took / 1e9 for took, context in mixed_steps)
        typical = mixed_rates[len(mixed_rates) // 2] if mixed_rates else 0.0

        def spread(ms):
            ms = sorted(ms)
            at = lambda f: round(ms[min(len(ms) - 1, int(f * len(ms)))], 3)
            return {"steps": len(ms), "mean": round(sum(ms) / len(ms), 3), "p50": at(0.5), "p90": at(0.9),
                    "p99": at(0.99), "max": round(ms[-1], 3)} if ms else {"steps": 0}
        line = {"metric": "32 requests, prompts of 512 to 16384 tokens in 512-token portions beside decodes "
                          "(MiniMax-M2 sizes, 24 layers, 1 GPU)",
                "value": round((prompt_tokens + output_tokens) / seconds, 1), "unit": "tokens/s (prompt + output)",
                "n_gpus": 1, "dtype": args.dtype, "data": "synthetic: random token ids, random weights",
                "config": {"num_layers": layers, "requests": requests, "portion": 512, "output_len": output_len},
                "prompt_tokens": prompt_tokens, "output_tokens": output_tokens, "total_s": round(seconds, 3),
                "step_ms_with_prompt_portions": spread(mixed_ms), "step_ms_decode_only": spread(decode_ms),
                # the median step with a prompt portion: the bytes it has to read over its time
                "mixed_step_roofline": {"bound": "hbm", "achieved": round(typical, 1), "peak": 8000.0, "unit": "GB/s",
                                        "frac": round(typical / 8000.0, 4), "measured_peak": round(memory["read_GBps"], 1),
                                        "measured_frac": round(typical / memory["read_GBps"], 4),
                                        "weights_GB": round(weights_once / 1e9, 2),
                                        "experts_read_per_layer": round(experts_read, 1), "steps_counted": len(chosen)},
                "memory": {k: round(v, 1) for k, v in memory.items()},
                "preemptions": llm.scheduler.total_preemptions}
    print(json.dumps(line), flush=True)
    return 0


if __name__ == "__main__":
    sys.exit(main())
