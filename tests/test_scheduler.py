"""The scheduler's decisions against a fake cache and a fake step: admission and deferral, the
token budget, portions, finishing, and what happens when pages run out."""
import pytest

from sparseengine_amd.engine.scheduler import MemoryOracle, Scheduler
from sparseengine_amd.engine.sequence import Sequence, SequenceStatus
from sparseengine_amd.sampling.params import SamplingParams


class FakeCache(MemoryOracle):
    """Pages of ``page`` tokens, one pool; counts what each request holds."""

    def __init__(self, pages, rows=8, page=16):
        self.pages, self.rows, self.page = pages, rows, page
        self.held = {}                      # seq_id -> tokens appended

    def used(self):
        return sum(-(-n // self.page) for n in self.held.values())

    # the scheduler's unit is tokens of cache in whole pages
    def free_tokens(self): return (self.pages - self.used()) * self.page
    def total_tokens(self): return self.pages * self.page
    def free_rows(self): return self.rows - len(self.held)
    def cost_of_new(self, tokens): return -(-tokens // self.page) * self.page
    def cost_to_append(self, seq_id, n):
        have = self.held.get(seq_id, 0)
        return (-(-(have + n) // self.page) - -(-have // self.page)) * self.page
    def tokens_that_fit(self, seq_id, room):
        return (-self.held.get(seq_id, 0)) % self.page + max(0, room) // self.page * self.page
    def admit(self, seq_id): self.held[seq_id] = 0
    def holds(self, seq_id): return seq_id in self.held
    def release(self, seq_id): del self.held[seq_id]


def make(cache, **kw):
    opts = dict(max_num_batched_tokens=64, max_num_seqs_in_batch=8, max_decoding_seqs=8,
                engine_prefill_chunk_size=64, decode_reservation_tokens=0, eos=-1)
    opts.update(kw)
    return Scheduler(cache, **opts)


def seq(n, max_tokens=4, **kw):
    return Sequence(list(range(1, n + 1)), SamplingParams(temperature=0.0, max_tokens=max_tokens, **kw))


def run_step(sched, cache, token=lambda s: 7):
    """The engine's step with a fake model: appends to the fake cache, 'samples' a token."""
    schedule = sched.schedule()
    for item in schedule.items:
        assert cache.cost_to_append(item.seq.seq_id, item.num_tokens) <= cache.free_tokens()
        cache.held[item.seq.seq_id] += item.num_tokens
    sampled = {i.seq.seq_id: token(i.seq) for i in schedule.items if i.wants_logits}
    return schedule, sched.postprocess(schedule, sampled)


def test_prompts_are_cut_into_portions_under_the_budget():
    cache = FakeCache(pages=100)
    sched = make(cache, max_num_batched_tokens=48, engine_prefill_chunk_size=32)
    a, b = seq(70), seq(20)
    sched.add(a); sched.add(b)
    s1, _ = run_step(sched, cache)
    assert [(i.seq.seq_id, i.num_tokens, i.wants_logits) for i in s1.items] == [(a.seq_id, 32, False), (b.seq_id, 16, False)]
    s2, _ = run_step(sched, cache)          # the older prompt first, the budget caps the second
    assert [(i.seq.seq_id, i.num_tokens, i.wants_logits) for i in s2.items] == [(a.seq_id, 32, False), (b.seq_id, 4, True)]
    s3, _ = run_step(sched, cache)          # b decodes (first in the batch), a finishes its prompt
    assert [(i.seq.seq_id, i.num_tokens, i.wants_logits) for i in s3.items] == [(b.seq_id, 1, True), (a.seq_id, 6, True)]
    assert a.completion_token_ids == [7] and b.completion_token_ids == [7, 7]
    assert s3.num_decode_tokens == 1 and s3.num_prefill_tokens == 6


def test_finish_by_max_tokens_and_by_eos_frees_at_once():
    cache = FakeCache(pages=10)
    sched = make(cache, eos=99)
    a, b, c = seq(5, max_tokens=2), seq(5, max_tokens=50), seq(5, max_tokens=50, ignore_eos=True)
    for s in (a, b, c):
        sched.add(s)
    tokens = {a.seq_id: [1, 2], b.seq_id: [1, 99], c.seq_id: [99, 99, 5]}
    done = []
    for _ in range(2):
        _, finished = run_step(sched, cache, token=lambda s: tokens[s.seq_id][s.num_completion_tokens])
        done += finished
    assert {s.seq_id for s in done} == {a.seq_id, b.seq_id}
    assert a.status is SequenceStatus.FINISHED and b.completion_token_ids == [1, 99]
    assert not cache.holds(a.seq_id) and not cache.holds(b.seq_id) and cache.holds(c.seq_id)
    assert c.completion_token_ids == [99, 99] and not sched.is_finished()
    custom = seq(3, max_tokens=9, eos_token_ids=[5])
    sched.add(custom)
    run_step(sched, cache, token=lambda s: 5)
    assert custom.status is SequenceStatus.FINISHED       # the request's own end tokens win over the configured one


def test_a_prompt_waits_until_its_whole_need_fits():
    cache = FakeCache(pages=6)                             # 96 tokens
    sched = make(cache, decode_reservation_tokens=16)
    a, b = seq(60, max_tokens=30), seq(40, max_tokens=30)
    sched.add(a); sched.add(b)
    s1, _ = run_step(sched, cache)
    assert [i.seq.seq_id for i in s1.items] == [a.seq_id]  # b needs 3 + 1 pages; a is promised 4 + 1
    assert list(sched.waiting) == [b]
    for _ in range(40):
        if a.status is SequenceStatus.FINISHED:
            break
        run_step(sched, cache)
    assert a.status is SequenceStatus.FINISHED and b.num_preemptions == 0     # b waited; nobody was thrown out
    while not sched.is_finished():
        run_step(sched, cache)
    assert len(b.completion_token_ids) == 30 and cache.used() == 0


def test_too_large_a_prompt_is_an_error_not_a_hang():
    cache = FakeCache(pages=2)
    sched = make(cache)
    sched.add(seq(60))
    with pytest.raises(ValueError, match="pages"):
        sched.schedule()


def test_running_out_of_pages_preempts_the_youngest_and_recomputes_it():
    cache = FakeCache(pages=6)                             # 96 tokens, no decode window promised
    sched = make(cache)
    a, b = seq(30, max_tokens=40), seq(30, max_tokens=40)
    sched.add(a); sched.add(b)
    history = []
    for _ in range(200):
        if sched.is_finished():
            break
        schedule, _ = run_step(sched, cache, token=lambda s: 100 + s.num_completion_tokens)
        history.append(schedule)
    assert sched.is_finished() and cache.used() == 0
    assert sched.total_preemptions >= 1
    first = next(s for s in history if s.preempted)
    assert first.preempted == [b]                          # the younger request goes, the older goes on
    assert a.num_preemptions == 0 and b.num_preemptions >= 1
    # both produced the tokens an undisturbed run produces: tokens depend on (request, index) only
    assert a.completion_token_ids == [100 + i for i in range(40)] == b.completion_token_ids
    # after the preemption b fed prompt AND generated tokens again, in portions, before decoding on
    replays = [i for s in history[history.index(first):] for i in s.items if i.seq is b and i.num_tokens > 1]
    assert replays and sum(i.num_tokens for i in replays) > 30


def test_the_only_request_that_cannot_go_on_is_an_error():
    cache = FakeCache(pages=2)
    sched = make(cache)
    sched.add(seq(30, max_tokens=40))
    with pytest.raises(RuntimeError, match="too small"):
        for _ in range(10):
            run_step(sched, cache)


def test_limits_on_requests_per_step_and_abort():
    cache = FakeCache(pages=100, rows=3)
    sched = make(cache, max_num_seqs_in_batch=2, max_decoding_seqs=2)
    seqs = [seq(4, max_tokens=3) for _ in range(4)]
    for s in seqs:
        sched.add(s)
    s1, _ = run_step(sched, cache)
    assert len(s1.items) == 2 and len(sched.waiting) == 2    # two rows of decoders at most
    gone = sched.abort([seqs[0].seq_id, seqs[3].seq_id])
    assert {s.seq_id for s in gone} == {seqs[0].seq_id, seqs[3].seq_id}
    assert not cache.holds(seqs[0].seq_id) and list(sched.waiting) == [seqs[2]]
    while not sched.is_finished():
        run_step(sched, cache)
    assert [len(s.completion_token_ids) for s in seqs] == [1, 3, 3, 0]


def test_a_failed_step_puts_its_requests_back():
    cache = FakeCache(pages=10)
    sched = make(cache)
    a = seq(10)
    sched.add(a)
    schedule = sched.schedule()
    cache.held[a.seq_id] += 10
    sched.fail_step(schedule)
    assert list(sched.waiting) == [a] and not sched.running and cache.used() == 0 and a.num_computed_tokens == 0


def test_forced_tokens_replace_the_sampled_ones():
    cache = FakeCache(pages=10)
    sched = make(cache)
    forced = Sequence([1, 2, 3], SamplingParams(max_tokens=3, ignore_eos=True, benchmark_forced_token_ids=(4, 5, 6)))
    sched.add(forced)
    while not sched.is_finished():
        run_step(sched, cache)
    assert forced.completion_token_ids == [4, 5, 6]
    with pytest.raises(ValueError, match="ignore_eos"):
        SamplingParams(max_tokens=1, benchmark_forced_token_ids=(1,))
