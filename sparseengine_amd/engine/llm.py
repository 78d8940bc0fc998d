"""The Python entry point: ``LLM(model, **config).generate(prompts, sampling_params)``.

Surface and meanings follow the reference (engine/llm_engine.py:232-348,1119-1133,1754-1762,
1976-2055): keyword arguments are exactly the fields of ``Config`` (an unknown one raises),
prompts are strings or lists of token ids, ``generate`` returns ``[{"text", "token_ids"}]`` in
the order of submission, ``step`` returns the finished requests and the signed token count of
the step (positive: prompt tokens, negative: decoded tokens).
"""
from __future__ import annotations

import os
import sys
import time

import torch

from ..config.method_registry import resolve_method
from ..config.runtime import Config
from ..sampling.params import SamplingParams
from ..sampling.sampler import Sampler
from .runner import ModelRunner, StepEntry
from .scheduler import MemoryOracle, Scheduler
from .sequence import Sequence


class CacheOracle(MemoryOracle):
    """The scheduler's view of the cache manager, in tokens of cache (whole pages of the tightest group)."""

    def __init__(self, cache, method=None):
        self.cache = cache
        self.method = method

    def free_tokens(self):
        return min((g.pool.free_count * g.page_size for g in self.cache.groups), default=1 << 40)

    def total_tokens(self):
        return min((g.pool.num_pages * g.page_size for g in self.cache.groups), default=1 << 40)

    def free_rows(self):
        return self.cache.num_free_rows

    def _cost(self, pages: dict[int, int], row, new_tokens) -> int:
        if self.method is not None:       # what the sparse method keeps for itself on top
            for group, extra in self.method.extra_pages(row, new_tokens).items():
                pages[group] = pages.get(group, 0) + extra
        sizes = {g.index: g.page_size for g in self.cache.groups}
        return max((n * sizes[group] for group, n in pages.items()), default=0)

    def cost_of_new(self, tokens):
        return self._cost(self.cache.pages_for_tokens(tokens), None, tokens)

    def cost_to_append(self, seq_id, new_tokens):
        if new_tokens <= 0:
            return 0
        if not self.cache.has_row(seq_id):
            return self.cost_of_new(new_tokens)
        row = self.cache.row_of(seq_id)
        return self._cost(self.cache.pages_needed(row, new_tokens), row, new_tokens)

    def tokens_that_fit(self, seq_id, room):
        length = int(self.cache.row_len[self.cache.row_of(seq_id)]) if self.cache.has_row(seq_id) else 0
        # per group: what is left of the row's last page, and the whole pages that the room holds
        return min(((-length) % g.page_size + max(0, room) // g.page_size * g.page_size for g in self.cache.groups),
                   default=1 << 40)

    def admit(self, seq_id):
        self.cache.admit(seq_id)

    def holds(self, seq_id):
        return self.cache.has_row(seq_id)

    def release(self, seq_id):
        self.cache.free(seq_id)


class StepTimes:
    """Wall time of the sections of ``LLM.step`` (``enable_profiler``): the device is waited for at each
    section's end, so that a section is charged with the work it started.  The reference's profiler
    (utils/profiler.py:14-105) keeps named sections and prints their totals; so does ``report``."""

    def __init__(self, enabled: bool, device):
        self.enabled, self.device = enabled, device
        self.seconds: dict[str, float] = {}
        self.calls: dict[str, int] = {}
        self._mark = 0.0

    def start(self) -> None:
        if self.enabled:
            self._mark = time.perf_counter()

    def section(self, name: str) -> None:
        """Close the section that began at the last ``start`` or ``section`` call."""
        if not self.enabled:
            return
        if getattr(self.device, "type", str(self.device)) == "cuda":
            torch.cuda.synchronize()
        now = time.perf_counter()
        self.seconds[name] = self.seconds.get(name, 0.0) + now - self._mark
        self.calls[name] = self.calls.get(name, 0) + 1
        self._mark = now

    def report(self) -> str:
        total = sum(self.seconds.values()) or 1.0
        return "\n".join(f"{name:10s} {1e3 * sec:10.1f} ms {100 * sec / total:5.1f} %  {self.calls[name]} calls"
                         for name, sec in sorted(self.seconds.items(), key=lambda kv: -kv[1]))


class ThroughputLog:
    """A line on stderr every ``interval`` seconds with the tokens per second since the last one
    (``throughput_log_interval_s``; 0 switches it off).  The reference logs from a thread of its own
    (engine/llm_engine.py:90-230); here the step that crosses the interval writes the line."""

    def __init__(self, interval: float, stream=None):
        self.interval, self.stream = float(interval), stream
        self.prefill = self.decode = self.steps = 0
        self.since = time.perf_counter()

    def record(self, signed_tokens: int, running: int, waiting: int) -> None:
        if self.interval <= 0:
            return
        if signed_tokens > 0:
            self.prefill += signed_tokens
        else:
            self.decode -= signed_tokens
        self.steps += 1
        now = time.perf_counter()
        if now - self.since < self.interval:
            return
        dt = now - self.since
        print(f"[throughput] prefill {self.prefill / dt:.0f} tok/s, decode {self.decode / dt:.0f} tok/s, "
              f"{self.steps} steps, {running} running, {waiting} waiting", file=self.stream or sys.stderr, flush=True)
        self.prefill = self.decode = self.steps = 0
        self.since = now


class LLM:
    def __init__(self, model: str, **kwargs):
        kernels = kwargs.pop("_kernels", None)           # test seam: the kernel twins on the CPU
        device = kwargs.pop("_device", "cuda")
        self.config = config = Config.from_kwargs(model, **kwargs)
        binding = resolve_method(config.sparse_method)
        self.method = binding.runtime_factory()
        cache_tokens = config.num_kvcache_slots
        common = dict(dtype=config.dtype, device=device, kv_page_size=config.kv_page_size,
                      max_num_seqs=config.max_num_seqs_in_gpu, max_model_len=config.max_model_len,
                      mlp_chunk_size=config.mlp_chunk_size, kernels=kernels, method=self.method,
                      cache_manager_cls=binding.cache_manager(),
                      validate_runtime_invariants=config.validate_runtime_invariants)
        if config.tiny_random:
            self.runner = ModelRunner.from_random(config.raw_model_config, seed=config.tiny_random_seed,
                                                  on_device=config.tiny_random_on_device,
                                                  num_kvcache_tokens=cache_tokens,
                                                  gpu_memory_utilization=config.gpu_memory_utilization, **common)
        else:
            self.runner = ModelRunner.from_folder(model, num_kvcache_tokens=cache_tokens,
                                                  gpu_memory_utilization=config.gpu_memory_utilization, **common)
        self.oracle = CacheOracle(self.runner.cache, self.method)
        self.scheduler = Scheduler(
            self.oracle, max_num_batched_tokens=config.max_num_batched_tokens,
            max_num_seqs_in_batch=config.max_num_seqs_in_batch, max_decoding_seqs=config.max_decoding_seqs,
            engine_prefill_chunk_size=config.engine_prefill_chunk_size,
            decode_reservation_tokens=config.decode_reservation_tokens, eos=config.eos,
            eos_token_ids=config.eos_token_ids)
        self.sampler = Sampler(self.runner.kernels, self.runner.device, config.sampler_seed)
        self.tokenizer = self._load_tokenizer(model)
        self.vocab_size = self.runner.spec.vocab_size
        self.last_step_seconds = 0.0
        self.step_times = StepTimes(config.enable_profiler, self.runner.device)
        self.throughput_log = ThroughputLog(config.throughput_log_interval_s)

    @staticmethod
    def _load_tokenizer(folder: str):
        path = os.path.join(folder, "tokenizer.json")
        if not os.path.isfile(path):
            return None
        from tokenizers import Tokenizer
        return Tokenizer.from_file(path)

    # ------------------------------------------------------------------ requests
    def _tokenize(self, prompt) -> list[int]:
        if isinstance(prompt, str):
            if self.tokenizer is None:
                raise ValueError("the model folder has no tokenizer.json; pass prompts as lists of token ids")
            ids = self.tokenizer.encode(prompt).ids
        else:
            ids = [int(t) for t in prompt]
        if not ids:
            raise ValueError("an empty prompt cannot be generated from")
        return ids

    def add_request(self, prompt, sampling_params: SamplingParams) -> int:
        ids = self._tokenize(prompt)
        bad = [t for t in ids if not 0 <= t < self.vocab_size]
        if bad:
            raise ValueError(f"prompt token {bad[0]} is outside the vocabulary [0, {self.vocab_size})")
        longest = len(ids) + sampling_params.max_tokens
        if longest > self.config.max_model_len:
            raise ValueError(
                f"this request may grow to {longest} tokens ({len(ids)} of prompt, max_tokens = "
                f"{sampling_params.max_tokens}), more than max_model_len = {self.config.max_model_len} allows")
        sampling_params.validate_for_vocab(self.vocab_size)
        seq = Sequence(ids, sampling_params)
        self.scheduler.add(seq)
        return seq.seq_id

    def abort_request(self, seq_id: int) -> bool:
        return bool(self.scheduler.abort([seq_id]))

    def is_finished(self) -> bool:
        return self.scheduler.is_finished()

    # ------------------------------------------------------------------ one engine step
    def step(self):
        """Schedule, run, sample, account.  Returns (finished, signed token count) where finished is
        a list of (seq_id, completion token ids, token logprobs, top logprobs)."""
        started = time.perf_counter()
        times = self.step_times
        times.start()
        schedule = self.scheduler.schedule()
        times.section("schedule")
        if not schedule.items:
            return [], 0
        entries = [StepEntry(i.seq.seq_id, i.seq.next_tokens(i.num_tokens), [i.num_tokens - 1] if i.wants_logits else [])
                   for i in schedule.items]
        try:
            logits = self.runner.step(entries)
            times.section("model")
            wanting = [i.seq for i in schedule.items if i.wants_logits]
            sampled, logprobs = {}, {}
            if wanting:
                rows = [(s.sampling_params, s.prompt_token_ids, s.completion_token_ids, s.sampler_notes) for s in wanting]
                logits = self.sampler.apply_penalties(logits, rows)
                tokens = self.sampler.sample(logits, rows, [(s.seed, s.num_completion_tokens) for s in wanting])
                chosen, tops = self.sampler.logprobs(logits, tokens, [s.sampling_params.logprobs for s in wanting])
                for s, t, c, top in zip(wanting, tokens, chosen, tops):
                    sampled[s.seq_id] = t
                    logprobs[s.seq_id] = (c, top)
            times.section("sample")
        except Exception:
            self.scheduler.fail_step(schedule)
            raise
        prefill, decode = schedule.num_prefill_tokens, schedule.num_decode_tokens
        finished = self.scheduler.postprocess(schedule, sampled, logprobs)
        if self.config.validate_runtime_invariants:
            self.runner.cache.check_invariants()
        times.section("account")
        self.last_step_seconds = time.perf_counter() - started
        outputs = [(s.seq_id, s.completion_token_ids, s.token_logprobs, s.top_logprobs) for s in finished]
        signed = prefill if prefill else -decode
        self.throughput_log.record(signed, len(self.scheduler.running), len(self.scheduler.waiting))
        return outputs, signed

    # ------------------------------------------------------------------ the blocking call
    def generate(self, prompts, sampling_params, use_tqdm: bool = True) -> list[dict]:
        if isinstance(sampling_params, list) and len(sampling_params) != len(prompts):
            raise ValueError(f"{len(prompts)} prompts came with a list of {len(sampling_params)} sampling_params: "
                             "give one for all prompts, or one per prompt")
        if not isinstance(sampling_params, list):
            sampling_params = [sampling_params] * len(prompts)
        order = [self.add_request(p, sp) for p, sp in zip(prompts, sampling_params)]
        outputs = {}
        prefill_rate = decode_rate = 0.0
        while not self.is_finished():
            t0 = time.perf_counter()
            finished, count = self.step()
            dt = max(time.perf_counter() - t0, 1e-9)
            if count > 0:
                prefill_rate = count / dt
            elif count < 0:
                decode_rate = -count / dt
            for seq_id, token_ids, _, _ in finished:
                outputs[seq_id] = token_ids
            if use_tqdm and finished:
                print(f"\rGenerating {len(outputs)}/{len(prompts)}  prefill {int(prefill_rate)} tok/s  "
                      f"decode {int(decode_rate)} tok/s", end="", file=sys.stderr, flush=True)
        if use_tqdm:
            print(file=sys.stderr)
        results = []
        for seq_id in order:
            ids = outputs[seq_id]
            text = self.tokenizer.decode(ids, skip_special_tokens=True) if self.tokenizer is not None else ""
            results.append({"text": text, "token_ids": ids})
        return results

    def exit(self) -> None:
        self.runner = None
        if torch.cuda.is_available():
            torch.cuda.empty_cache()
