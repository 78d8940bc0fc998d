"""Continuous batching above the step function.

Every step takes the decoding requests first (one token each), then fills what is left of the
token budget with portions of prompts in arrival order (the ``all_chunked`` policy); the last
portion of a prompt asks for logits.  The reference schedules prefill steps and decode steps
apart (engine/scheduler.py:534-1079); admission, budgets, finishing and preemption follow it:

* a new prompt is admitted only if its whole length plus a decode window fits beside what the
  running requests are still promised (scheduler.py:735-858, cache_manager/decode_reservation.py);
  otherwise it waits (is deferred), in order;
* when a decode cannot get a page, the youngest running request is preempted: its pages are
  freed and it goes back to the head of the queue; when it is admitted again its prompt AND the
  tokens it had generated are fed again in portions, and generation continues from there
  (scheduler.py:336-424; sequence.py:262-347).  Sampling noise is a function of the request and
  the position, so the continuation is the same;
* a single running request that cannot get a page, or a prompt that cannot fit an empty cache,
  is an error (scheduler.py:360-382).
"""
from __future__ import annotations

from collections import deque
from dataclasses import dataclass, field

from ..sampling.params import resolve_eos_token_ids
from .sequence import Sequence, SequenceStatus


class MemoryOracle:
    """What the scheduler asks of the cache.  Every count is in tokens of cache, taken in whole pages: the
    cache's groups may have pages of different sizes, so pages are no common unit; an answer is that of the
    group for which it is tightest (what is free: the least; what something costs: the most), which makes
    the sum of several costs an upper bound for every group."""

    def free_tokens(self) -> int: raise NotImplementedError
    def total_tokens(self) -> int: raise NotImplementedError
    def free_rows(self) -> int: raise NotImplementedError
    def cost_of_new(self, tokens: int) -> int: raise NotImplementedError              # a request of so many tokens, from nothing
    def cost_to_append(self, seq_id, new_tokens: int) -> int: raise NotImplementedError
    def tokens_that_fit(self, seq_id, room: int) -> int: raise NotImplementedError     # new tokens of the request that `room` holds
    def admit(self, seq_id) -> None: raise NotImplementedError
    def holds(self, seq_id) -> bool: raise NotImplementedError
    def release(self, seq_id) -> None: raise NotImplementedError


@dataclass
class ScheduledItem:
    seq: Sequence
    num_tokens: int
    wants_logits: bool


@dataclass
class Schedule:
    items: list[ScheduledItem] = field(default_factory=list)
    preempted: list[Sequence] = field(default_factory=list)

    @property
    def num_prefill_tokens(self) -> int:
        return sum(i.num_tokens for i in self.items if not (i.num_tokens == 1 and i.seq.num_completion_tokens))

    @property
    def num_decode_tokens(self) -> int:
        return sum(1 for i in self.items if i.num_tokens == 1 and i.seq.num_completion_tokens)


class Scheduler:
    def __init__(self, oracle: MemoryOracle, *, max_num_batched_tokens: int, max_num_seqs_in_batch: int,
                 max_decoding_seqs: int, engine_prefill_chunk_size: int, decode_reservation_tokens: int,
                 eos: int = -1, eos_token_ids=()):
        self.oracle = oracle
        self.max_num_batched_tokens = int(max_num_batched_tokens)
        self.max_num_seqs_in_batch = int(max_num_seqs_in_batch)
        self.max_decoding_seqs = int(max_decoding_seqs)
        self.chunk = int(engine_prefill_chunk_size)
        self.decode_reservation_tokens = int(decode_reservation_tokens)
        self.eos, self.eos_token_ids = eos, tuple(eos_token_ids)
        self.waiting: deque[Sequence] = deque()
        self.running: list[Sequence] = []          # in order of admission
        self.total_preemptions = 0
        self.total_recomputed_tokens = 0

    # ------------------------------------------------------------------ queue ownership
    def add(self, seq: Sequence) -> None:
        seq.status = SequenceStatus.WAITING
        self.waiting.append(seq)

    def is_finished(self) -> bool:
        return not self.waiting and not self.running

    def abort(self, seq_ids) -> list[Sequence]:
        """Remove the requests from both queues and give back what they hold."""
        seq_ids = set(seq_ids)
        gone = [s for s in list(self.waiting) + self.running if s.seq_id in seq_ids]
        self.waiting = deque(s for s in self.waiting if s.seq_id not in seq_ids)
        self.running = [s for s in self.running if s.seq_id not in seq_ids]
        for s in gone:
            if self.oracle.holds(s.seq_id):
                self.oracle.release(s.seq_id)
            s.status = SequenceStatus.FINISHED
        return gone

    # ------------------------------------------------------------------ promises
    def _window(self, seq: Sequence) -> int:
        return max(0, min(self.decode_reservation_tokens, seq.tokens_left_to_generate()))

    def _promised(self, seq: Sequence) -> int:
        """Cache a running request may still take: the rest of its known tokens + its decode window."""
        return self.oracle.cost_to_append(seq.seq_id, seq.num_remaining_tokens + self._window(seq))

    def _preempt(self, victim: Sequence, schedule: Schedule) -> None:
        self.running.remove(victim)
        self.oracle.release(victim.seq_id)
        self.total_recomputed_tokens += victim.num_computed_tokens
        victim.num_computed_tokens = 0
        victim.num_preemptions += 1
        victim.status = SequenceStatus.WAITING
        self.waiting.appendleft(victim)
        self.total_preemptions += 1
        schedule.preempted.append(victim)

    # ------------------------------------------------------------------ one step's batch
    def schedule(self) -> Schedule:
        schedule = Schedule()
        oracle = self.oracle
        budget = self.max_num_batched_tokens
        taken = 0                                  # cache this step's items will take

        def room() -> int:
            return oracle.free_tokens() - taken

        # 1. every decoding request feeds its last token
        decoders = [s for s in self.running if s.num_remaining_tokens == 1][:min(self.max_decoding_seqs, self.max_num_seqs_in_batch)]
        for seq in decoders:
            if seq not in self.running:            # preempted a moment ago
                continue
            need = oracle.cost_to_append(seq.seq_id, 1)
            while need > room():
                scheduled = {i.seq.seq_id for i in schedule.items}
                victims = [s for s in self.running if s.seq_id not in scheduled and s is not seq]
                if victims:
                    self._preempt(victims[-1], schedule)      # the youngest that is not in this step
                    continue
                if schedule.items:
                    self._preempt(seq, schedule)              # the others of this step go on without it
                    break
                raise RuntimeError(
                    "KV cache is too small for the only running request to go on: "
                    f"seq_id={seq.seq_id} tokens={seq.num_tokens} free cache tokens={oracle.free_tokens()} "
                    f"of {oracle.total_tokens()}; recomputing it would end in the same place")
            if seq not in self.running:
                continue
            taken += need
            budget -= 1
            schedule.items.append(ScheduledItem(seq, 1, True))

        # 2. portions of prompts that are under way, oldest first
        def add_portion(seq: Sequence) -> bool:
            nonlocal taken, budget
            n = min(seq.num_remaining_tokens, self.chunk, budget)
            n = min(n, oracle.tokens_that_fit(seq.seq_id, room()))
            if n <= 0:
                return False
            taken += oracle.cost_to_append(seq.seq_id, n)
            budget -= n
            schedule.items.append(ScheduledItem(seq, n, n == seq.num_remaining_tokens))
            return True

        for seq in [s for s in self.running if s.num_remaining_tokens > 1]:
            if budget <= 0 or len(schedule.items) >= self.max_num_seqs_in_batch:
                break
            if schedule.preempted and seq in schedule.preempted:
                continue
            add_portion(seq)

        # 3. new prompts, in order, while their whole need fits beside what is promised
        while (self.waiting and budget > 0 and len(schedule.items) < self.max_num_seqs_in_batch
               and not schedule.preempted):
            seq = self.waiting[0]
            if len(self.running) >= self.max_decoding_seqs or oracle.free_rows() <= 0:
                break
            need = oracle.cost_of_new(seq.num_tokens + self._window(seq))
            if need > oracle.total_tokens():
                if not self.running:
                    raise ValueError(
                        f"request {seq.seq_id} needs cache for {need} tokens ({seq.num_tokens} tokens and its "
                        f"decode window, in whole pages); the cache holds {oracle.total_tokens()}")
                break
            promised = sum(self._promised(s) for s in self.running)
            if need + promised > oracle.free_tokens():
                break                                            # deferred: stays at the head
            self.waiting.popleft()
            oracle.admit(seq.seq_id)
            seq.status = SequenceStatus.RUNNING
            self.running.append(seq)
            if not add_portion(seq):
                break

        if not schedule.items and not schedule.preempted and not self.is_finished():
            raise RuntimeError(
                f"nothing can run: {len(self.waiting)} waiting, {len(self.running)} running, "
                f"{oracle.free_tokens()} of {oracle.total_tokens()} cache tokens free")
        return schedule

    # ------------------------------------------------------------------ after the step
    def postprocess(self, schedule: Schedule, sampled: dict[int, int], logprobs: dict | None = None) -> list[Sequence]:
        """Account the step; ``sampled``: seq_id -> token for items that wanted logits.
        Returns the requests that finished (their pages are already given back)."""
        finished = []
        logprobs = logprobs or {}
        for item in schedule.items:
            seq = item.seq
            seq.num_computed_tokens += item.num_tokens
            if not item.wants_logits:
                continue
            forced = seq.sampling_params.benchmark_forced_token_ids
            token = forced[seq.num_completion_tokens] if forced is not None else sampled[seq.seq_id]
            seq.append_token(token, *logprobs.get(seq.seq_id, (None, None)))
            eos = resolve_eos_token_ids(seq.sampling_params.eos_token_ids, self.eos_token_ids, fallback=self.eos)
            if ((not seq.sampling_params.ignore_eos and token in eos)
                    or seq.num_completion_tokens >= seq.sampling_params.max_tokens):
                seq.status = SequenceStatus.FINISHED
                self.running.remove(seq)
                self.oracle.release(seq.seq_id)
                finished.append(seq)
        return finished

    def fail_step(self, schedule: Schedule) -> None:
        """A step raised: give back what its requests hold and queue them again from the start
        (reference engine/llm_engine.py:1826-1857)."""
        for item in reversed(schedule.items):
            seq = item.seq
            if seq in self.running:
                self.running.remove(seq)
            if self.oracle.holds(seq.seq_id):
                self.oracle.release(seq.seq_id)
            seq.num_computed_tokens = 0
            seq.status = SequenceStatus.WAITING
            self.waiting.appendleft(seq)
