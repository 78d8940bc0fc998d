"""The engine's host side (batches, cache, step function, replay, scheduler, entry point) on the
CPU: the kernel twins stand in for the HIP kernels, everything else is the product's own code.
The kernels themselves are tested on the GPU."""
import json
import os

import numpy as np
import pytest
import torch

from sparseengine_amd import LLM, SamplingParams
from sparseengine_amd.engine.replay import replay_step, replay_stream
from sparseengine_amd.engine.runner import ModelRunner, StepEntry
from sparseengine_amd.cache.page_pool import OutOfPages
from sparseengine_amd.kernels.attention_work import build_attention_work
from tests import traces
from tests.helpers import CONFIGS, make_folder, random_tokens
from tests.plain.minimax_m2 import PlainMiniMaxM2
from tests.twin_kernels import TwinKernels

LENGTHS = {"A": [5, 17, 31, 100, 64, 129], "B": [1, 9, 40, 100, 200]}


@pytest.fixture(scope="module", params=["A_loud", "B_loud"])
def model(request, tmp_path_factory):
    key = request.param
    folder = make_folder(tmp_path_factory.mktemp("cpu_models"), key)
    vocab = CONFIGS[key][0]["vocab_size"]
    requests = {f"r{i}": random_tokens(n, vocab, 100 + i) for i, n in enumerate(LENGTHS[key[0]])}
    plain = PlainMiniMaxM2(folder)
    return folder, requests, {rid: plain.logits(t).numpy() for rid, t in requests.items()}, plain


def runner_for(folder, tokens, page_size=16, rows=4, dtype="float32"):
    return ModelRunner.from_folder(folder, dtype=dtype, device="cpu", kv_page_size=page_size,
                                   num_kvcache_tokens=-(-tokens // 64) * 64, max_num_seqs=rows, kernels=TwinKernels())


def replay(folder, records, tokens, page_size=16):
    runner = runner_for(folder, tokens, page_size)
    out = {}
    for rec in records:
        logits = replay_step(runner, rec, None)
        if logits is not None:
            out[rec["step"]] = logits
        runner.cache.check_invariants()
    assert all(g.pool.free_count == g.pool.num_pages for g in runner.cache.groups) and runner.cache.num_free_rows == 4
    return traces.gather(records, out)


@pytest.mark.parametrize("mode", ["whole", "tail", "portions", "mixed"])
def test_every_way_of_cutting_gives_the_plain_logits(model, mode):
    folder, requests, expected, _ = model
    if mode == "whole":
        records, peak = traces.whole(requests), 256
    elif mode == "tail":
        records, peak = traces.prefill_then_decode(requests, tail=32), 256
    elif mode == "portions":
        records, peak = traces.changing_portions(requests, seed=1), 256
    else:
        records, peak = traces.mixed(requests, seed=0)
        assert peak < sum(-(-len(t) // 64) * 64 for t in requests.values())      # pages must be used again
    got = replay(folder, records, peak)
    for rid, ref in expected.items():
        assert np.abs(got[rid] - ref).max() < 2e-5 * max(1.0, np.abs(ref).max()), rid


def test_step_refuses_what_does_not_fit_and_changes_nothing(model):
    folder, requests, _, _ = model
    runner = runner_for(folder, 64)
    toks = requests["r3"]
    with pytest.raises(OutOfPages):
        runner.step([StepEntry("big", toks[:100], [])])
    assert not runner.cache.has_row("big") and runner.cache.num_free_rows == 4
    runner.step([StepEntry("ok", toks[:60], [])])
    with pytest.raises(OutOfPages):
        runner.step([StepEntry("ok", toks[60:70], []), StepEntry("other", toks[:3], [])])
    assert int(runner.cache.row_len[runner.cache.row_of("ok")]) == 60 and not runner.cache.has_row("other")
    with pytest.raises(ValueError, match="vocabulary"):
        runner.step([StepEntry("ok", [10 ** 6], [])])
    runner.cache.check_invariants()


def test_trace_stream_writes_files_and_done_lines(model, tmp_path):
    folder, requests, expected, _ = model
    records, peak = traces.mixed(requests, seed=5)
    runner = runner_for(folder, peak)

    class Report(list):
        def write(self, text): self.append(text)
        def flush(self): pass
    report = Report()
    steps = replay_stream(runner, (json.dumps(r) for r in records), str(tmp_path / "out"), report=report)
    assert steps == len(records)
    assert [l.strip() for l in "".join(report).splitlines()] == [f"done {r['step']}" for r in records]
    vocab = next(iter(expected.values())).shape[1]
    logits = {r["step"]: np.fromfile(tmp_path / "out" / f"{r['step']}.f32", dtype="<f4").reshape(-1, vocab)
              for r in records if any(e["want"] for e in r["entries"])}
    got = traces.gather(records, logits)
    for rid, ref in expected.items():
        assert np.abs(got[rid] - ref).max() < 2e-5 * max(1.0, np.abs(ref).max())


def llm(folder, **kw):
    opts = dict(dtype="float32", num_kvcache_slots=512, kv_page_size=16, max_num_seqs_in_batch=4,
                validate_runtime_invariants=True, _kernels=TwinKernels(), _device="cpu")
    opts.update(kw)
    return LLM(folder, **opts)


def test_generate_is_the_plain_greedy_decoding(model):
    folder, requests, _, plain = model
    prompts = [t[:n] for t, n in zip(requests.values(), (5, 17, 31))]
    engine = llm(folder)
    outs = engine.generate(prompts, SamplingParams(temperature=0.0, max_tokens=8, ignore_eos=True), use_tqdm=False)
    assert [o["token_ids"] for o in outs] == [plain.greedy(p, 8) for p in prompts]
    assert all(o["text"] == "" for o in outs)                       # no tokenizer in a random folder
    with pytest.raises(ValueError, match="more than max_model_len"):
        engine.add_request(prompts[0], SamplingParams(max_tokens=10 ** 6))
    with pytest.raises(ValueError, match="unknown configuration keys"):
        LLM(folder, not_an_option=1)
    with pytest.raises(ValueError, match="tokenizer"):
        engine.add_request("text", SamplingParams(max_tokens=1))


def test_portions_beside_decodes_and_pressure_change_no_token(model):
    folder, requests, _, plain = model
    prompts = [t[:n] for t, n in zip(requests.values(), (5, 17, 31, 60))]
    params = SamplingParams(temperature=0.0, max_tokens=20, ignore_eos=True)
    expected = [plain.greedy(p, 20) for p in prompts]
    chunked = llm(folder, max_num_batched_tokens=16)                 # 16-token portions beside decodes
    assert [o["token_ids"] for o in chunked.generate(prompts, params, use_tqdm=False)] == expected
    tight = llm(folder, num_kvcache_slots=128, decode_reservation_tokens=0)   # 8 pages: somebody must be thrown out
    assert [o["token_ids"] for o in tight.generate(prompts, params, use_tqdm=False)] == expected
    assert tight.scheduler.total_preemptions >= 1
    assert all(g.pool.free_count == g.pool.num_pages for g in tight.runner.cache.groups)


def test_sampling_does_not_depend_on_the_batch(model):
    folder, requests, _, _ = model
    prompts = [t[:n] for t, n in zip(requests.values(), (5, 17, 31))]
    engine = llm(folder)
    sp = SamplingParams(temperature=0.8, top_k=50, top_p=0.9, max_tokens=12, ignore_eos=True, seed=5)
    alone = engine.generate([prompts[1]], sp, use_tqdm=False)[0]["token_ids"]
    others = [SamplingParams(temperature=1.3, max_tokens=9, ignore_eos=True, seed=1), sp,
              SamplingParams(temperature=0.0, max_tokens=5, ignore_eos=True)]
    together = engine.generate(prompts, others, use_tqdm=False)[1]["token_ids"]
    assert alone == together and len(set(alone)) > 3
    again = llm(folder, sampler_seed=1).generate([prompts[1]], sp, use_tqdm=False)[0]["token_ids"]
    assert again != alone                                            # another sampler seed, another draw


def test_penalties_logprobs_and_eos(model):
    folder, requests, _, plain = model
    prompt = list(requests.values())[2][:20]
    engine = llm(folder)
    base = engine.generate([prompt], SamplingParams(temperature=0.0, max_tokens=6, ignore_eos=True, logprobs=3), use_tqdm=False)
    first = base[0]["token_ids"][0]
    stopped = engine.generate([prompt], SamplingParams(temperature=0.0, max_tokens=6, eos_token_ids=[first]), use_tqdm=False)
    assert stopped[0]["token_ids"] == [first]
    # penalties, token for token against the plain logits with the reference's rule applied by hand
    # (layers/sampler.py:11-64: logits of prompt and generated tokens divided by the repetition
    # penalty if positive, else multiplied; the presence penalty subtracted from generated tokens)
    pen = engine.generate([prompt], SamplingParams(temperature=0.0, max_tokens=12, ignore_eos=True, presence_penalty=2.0,
                                                   repetition_penalty=1.5), use_tqdm=False)[0]["token_ids"]
    tokens, generated = list(prompt), []
    for _ in range(12):
        logits = plain.logits(tokens)[-1].clone()
        seen = torch.tensor(sorted(set(tokens)))
        logits[seen] = torch.where(logits[seen] > 0, logits[seen] / 1.5, logits[seen] * 1.5)
        if generated:
            logits[torch.tensor(sorted(set(generated)))] -= 2.0
        generated.append(int(logits.argmax()))
        tokens.append(generated[-1])
    assert pen == generated
    free = engine.generate([prompt], SamplingParams(temperature=0.0, max_tokens=12, ignore_eos=True), use_tqdm=False)[0]["token_ids"]
    assert pen != free, "the penalties changed nothing: the prompt does not exercise them"
    engine.add_request(prompt, SamplingParams(temperature=0.0, max_tokens=2, ignore_eos=True, logprobs=2))
    finished = []
    while not engine.is_finished():
        out, count = engine.step()
        finished += out
    (_, tokens, logprobs, tops), = finished
    ref = torch.log_softmax(plain.logits(prompt)[-1], -1)
    assert logprobs[0] == pytest.approx(float(ref[tokens[0]]), abs=1e-4)
    assert set(tops[0]) == set(torch.topk(ref, 2).indices.tolist())


def test_penalties_of_several_rows_at_once():
    """Rows with different penalties in one call, tokens named twice, a row without any: against the rule applied
    row by row (reference layers/sampler.py:11-64); a prompt's distinct tokens are kept with the request."""
    from sparseengine_amd.sampling.sampler import Sampler
    torch.manual_seed(0)
    vocab = 50
    logits = torch.randn(4, vocab)
    rows = [(SamplingParams(repetition_penalty=1.5), [3, 3, 7, 49], [7, 8, 8], {}),
            (SamplingParams(presence_penalty=2.0), [1, 2], [5, 5, 0], {}),
            (SamplingParams(), [4], [4, 4], {}),
            (SamplingParams(repetition_penalty=0.5, presence_penalty=-1.0), [9], [], {})]
    expect = logits.clone()
    for r, (p, prompt, completion, _) in enumerate(rows):
        if p.repetition_penalty != 1.0:
            for t in set(prompt) | set(completion):
                expect[r, t] = expect[r, t] / p.repetition_penalty if expect[r, t] > 0 else expect[r, t] * p.repetition_penalty
        for t in set(completion):
            expect[r, t] -= p.presence_penalty
    sampler = Sampler(None, "cpu")
    before = logits.clone()
    for _ in range(2):      # the second call finds the prompts' tokens where the first left them
        torch.testing.assert_close(sampler.apply_penalties(logits, rows), expect)
    assert torch.equal(logits, before), "the caller's logits are not touched"
    assert rows[0][3]["prompt_tokens"].tolist() == [3, 7, 49] and not rows[1][3]


def test_attention_work_lists_cover_every_row_and_key_once():
    for q_len, ctx, group, kvh, window in [([1], [2049], 6, 8, 0), ([1] * 64, [2200 - i for i in range(64)], 6, 8, 0),
                                            ([37, 23, 1], [37, 150, 301], 2, 2, 0), ([2048], [2048], 6, 8, 0),
                                            ([1, 1], [5000, 300], 4, 1, 128), ([3], [70], 16, 1, 0)]:
        work = build_attention_work(q_len, ctx, group, kvh, window)
        units = work.units
        for item, (ql, c) in enumerate(zip(q_len, ctx)):
            mine = units[units[:, 0] == item]
            tiles = -(-ql * group // 16)
            assert sorted(set(mine[:, 1].tolist())) == list(range(tiles))
            for tile in range(tiles):
                ranges = sorted((b, e) for _, t, b, e, *_ in mine.tolist() if t == tile)
                assert ranges[-1][1] == c and all(b % 32 == 0 for b, _ in ranges)
                assert all(a[1] == b[0] for a, b in zip(ranges, ranges[1:]))        # no gap, no overlap
                first = ranges[0][0]
                assert first == 0 or (window and first <= max(0, c - ql - window + 1))
        split = units[units[:, 4] >= 0]
        assert sorted(split[:, 4].tolist()) == list(range(work.num_slots))
        starts = [sum(q_len[:i]) for i in range(len(q_len))]
        for u in units.tolist():              # every unit carries its item's place, length and context
            assert u[5:] == [starts[u[0]], q_len[u[0]], ctx[u[0]]]
        for item, tile, first_slot, n, q_start, ql in work.tasks.tolist():
            slots = sorted(u[4] for u in units.tolist() if u[0] == item and u[1] == tile)
            assert slots == list(range(first_slot, first_slot + n)) and n <= 256
            assert (q_start, ql) == (starts[item], q_len[item])


def _check_ranges(ranges, ctx, first_allowed=0):
    """Key ranges of one tile (or run of tiles): joined up, multiples of 32 at the seams, ending at ctx."""
    ranges = sorted(ranges)
    assert ranges[0][0] <= first_allowed and ranges[-1][1] == ctx
    assert all(a[1] == b[0] and a[1] % 32 == 0 for a, b in zip(ranges, ranges[1:]))


def test_block_work_lists_for_many_rows_cover_every_tile_once_longest_first():
    """Items with many rows take blocks of consecutive tiles, items with few rows (a decoded token
    beside a prompt portion) keep one wavefront per tile; both split their keys when their class
    alone would not fill the chip, and every tile with split keys has one merge task."""
    from sparseengine_amd.kernels.attention_work import TILES_PER_BLOCK
    for q_len, ctx, group, kvh, window in [([2048], [2048], 6, 8, 0), ([900, 411, 1], [900, 1300, 301], 6, 8, 0),
                                            ([1500, 600], [1500, 900], 2, 8, 70),
                                            ([1, 2048, 1, 3], [70000, 2048, 9, 500], 6, 8, 0),
                                            ([100], [100000], 6, 8, 0), ([512] + [1] * 32, [8192] + [4096] * 32, 6, 8, 0),
                                            ([40, 1], [5000, 5000], 6, 1, 256)]:
        work = build_attention_work(q_len, ctx, group, kvh, window, head_dim=128)
        slots_seen = []
        for item, (ql, c) in enumerate(zip(q_len, ctx)):
            tiles = -(-ql * group // 16)
            lowest = max(0, c - ql - window + 1) if window else 0
            mine = work.block_units[work.block_units[:, 0] == item]
            alone = work.units[work.units[:, 0] == item]
            tasks = [t for t in work.tasks.tolist() if t[0] == item]
            if tiles >= TILES_PER_BLOCK // 2:
                assert len(alone) == 0
                assert sorted(set(mine[:, 1].tolist())) == list(range(0, tiles, TILES_PER_BLOCK))
                assert (mine[:, 5:9] == [sum(q_len[:item]), ql, c, mine[0, 8]]).all()
                splits = int(mine[0, 8])
                for first in range(0, tiles, TILES_PER_BLOCK):
                    runs = mine[mine[:, 1] == first]
                    assert len(runs) == splits
                    _check_ranges([(b, e) for b, e in runs[:, 2:4].tolist()], c, lowest)
                    if splits == 1:
                        assert runs[0, 4] == -1
                    else:       # slot of the run's first tile; the other tiles follow at a stride of `splits`
                        for t in range(first, min(first + TILES_PER_BLOCK, tiles)):
                            slots_seen += [int(sl) + (t - first) * splits for sl in runs[:, 4]]
            else:
                assert len(mine) == 0 and sorted(set(alone[:, 1].tolist())) == list(range(tiles))
                assert (alone[:, 5:] == [sum(q_len[:item]), ql, c]).all()
                splits = len(alone) // tiles
                for tile in range(tiles):
                    _check_ranges([(b, e) for _, t, b, e, *_ in alone.tolist() if t == tile], c, lowest)
                slots_seen += [int(sl) for sl in alone[:, 4] if sl >= 0]
            if splits > 1:
                assert sorted(t[1] for t in tasks) == list(range(tiles)) and all(t[3] == splits for t in tasks)
                assert all(t[2] == tasks[0][2] + (t[1] - tasks[0][1]) * splits for t in tasks)
                assert all(t[4:] == [sum(q_len[:item]), ql] for t in tasks)
            else:
                assert not tasks
        assert sorted(slots_seen) == list(range(work.num_slots))        # every partial slot written exactly once
        lengths = []
        for item, first, begin, end, *_ in work.block_units.tolist():
            last_row = min((first + TILES_PER_BLOCK) * 16, q_len[item] * group) - 1
            stop = min(ctx[item] - q_len[item] + last_row // group + 1, end)
            start = begin
            if window:
                start = max(begin, ctx[item] - q_len[item] + first * 16 // group - window + 1)
            lengths.append(max(stop - start, 0))
        assert lengths == sorted(lengths, reverse=True)
    # a long single token beside a prompt gets many more ranges than its short neighbours
    work = build_attention_work([1, 2048, 1], [70000, 2048, 2048], 6, 8, 0, head_dim=128)
    assert (work.units[:, 0] == 0).sum() >= 20 * (work.units[:, 0] == 2).sum()
    # a portion on a long prefix is cut into ranges of at least 2048 keys, about three rounds of blocks; the keys of a
    # portion that is most of what it reads (a whole prompt, a prompt's second half) are not cut at all
    ranges = lambda q, c: int(build_attention_work([q], [c], 6, 8, 0, head_dim=128).block_units[0, 8])
    assert ranges(512, 16384) == 8 and ranges(512, 32768) == 8 and ranges(2048, 8192) == 2
    assert ranges(2048, 2048) == 1 and ranges(1024, 1024) == 1 and ranges(2048, 4096) == 1 and ranges(3000, 3000) == 1
    # a head size the block kernel does not take, and a step of single tokens, keep the per-wavefront list
    assert len(build_attention_work([2048], [2048], 6, 8, 0, head_dim=160).block_units) == 0
    assert len(build_attention_work([1] * 8, [300] * 8, 6, 8, 0, head_dim=128).block_units) == 0


def test_work_lists_refuse_items_with_more_new_tokens_than_context():
    from sparseengine_amd.kernels.attention_work import build_attention_work_numpy
    for builder in (build_attention_work, build_attention_work_numpy):
        for q_len, ctx_len in (([2], [1]), ([1, 0], [5, 5]), ([3, 9], [3, 8])):
            with pytest.raises(ValueError, match="new token"):
                builder(q_len, ctx_len, 6, 8, 0, head_dim=128)
        builder([3, 8], [3, 8], 6, 8, 0, head_dim=128)


def test_compiled_work_list_builder_gives_the_same_lists():
    """csrc/host_work.hip against the numpy builder, list for list, on random steps."""
    import numpy as np
    from sparseengine_amd.kernels import attention_work as aw
    if aw._native_library() is None:
        pytest.skip("the compiled builder cannot be built here")
    rng = np.random.default_rng(0)
    for _ in range(400):
        items = int(rng.integers(1, 12))
        q = [int(rng.choice([1, 1, 1, 2, 7, 40, 300, 2048])) for _ in range(items)]
        c = [n + int(rng.integers(0, 70000)) * int(rng.integers(0, 2)) + int(rng.integers(0, 300)) for n in q]
        group, kvh = int(rng.choice([1, 2, 6, 16, 20])), int(rng.choice([1, 2, 8]))
        window, head_dim = int(rng.choice([0, 0, 64, 1000])), int(rng.choice([0, 64, 128, 160]))
        target = int(rng.choice([1024, 256]))
        a = aw.build_attention_work(q, c, group, kvh, window, target, head_dim)
        b = aw.build_attention_work_numpy(q, c, group, kvh, window, target, head_dim)
        assert a.num_slots == b.num_slots
        assert np.array_equal(a.units, b.units) and np.array_equal(a.tasks, b.tasks)
        assert np.array_equal(a.block_units, b.block_units)


def test_text_prompts_go_through_the_folders_tokenizer(model, tmp_path):
    """A tokenizer.json in the model folder: strings in, text out, same tokens as the ids would give."""
    import shutil
    from tokenizers import Tokenizer
    from tokenizers.models import WordLevel
    from tokenizers.pre_tokenizers import Whitespace
    folder, _, _, plain = model
    copy = str(tmp_path / "with_tokenizer")
    shutil.copytree(folder, copy)
    vocab = {f"w{i}": i for i in range(plain.cfg.vocab_size)}
    tok = Tokenizer(WordLevel(vocab, unk_token="w0"))
    tok.pre_tokenizer = Whitespace()
    tok.save(os.path.join(copy, "tokenizer.json"))
    engine = llm(copy)
    ids = [7, 300, 41, 41, 9]
    text = " ".join(f"w{i}" for i in ids)
    out, = engine.generate([text], SamplingParams(temperature=0.0, max_tokens=6, ignore_eos=True), use_tqdm=False)
    assert out["token_ids"] == plain.greedy(ids, 6)
    assert out["text"].split() == [f"w{i}" for i in out["token_ids"]]


def test_step_times_and_throughput_lines(model):
    """``enable_profiler`` and ``throughput_log_interval_s`` do what their names say."""
    import io
    folder, requests, _, _ = model
    engine = llm(folder, enable_profiler=True, throughput_log_interval_s=1e-9)
    engine.throughput_log.stream = lines = io.StringIO()
    prompts = [t[:9] for t in list(requests.values())[:2]]
    engine.generate(prompts, SamplingParams(temperature=0.0, max_tokens=4, ignore_eos=True), use_tqdm=False)
    assert set(engine.step_times.seconds) == {"schedule", "model", "sample", "account"}
    assert engine.step_times.calls["model"] == engine.step_times.calls["sample"] >= 4
    assert "model" in engine.step_times.report()
    logged = [l for l in lines.getvalue().splitlines() if l.startswith("[throughput]")]
    assert len(logged) == engine.step_times.calls["model"] and "decode" in logged[-1]
    quiet = llm(folder)
    quiet.generate(prompts[:1], SamplingParams(temperature=0.0, max_tokens=2, ignore_eos=True), use_tqdm=False)
    assert not quiet.step_times.seconds


def test_engine_bench_counts_every_token_once(model, tmp_path, capsys):
    """The bench sub-command: each case feeds batch x length prompt tokens; a request decodes
    output_len - 1 tokens (its first completion token comes from the prompt's last step), of which
    those that ride in a step beside prompt portions are counted with that step, as prefill."""
    from sparseengine_amd.engine import microbench
    folder = model[0]
    out = tmp_path / "rows.jsonl"
    rc = microbench.main(["--model_path", str(folder), "--lengths", "9,20", "--batch_sizes", "1,3", "--output_len", "5",
                          "--hyper_params", json.dumps({"max_num_batched_tokens": 16}), "--output_jsonl", str(out)],
                         llm_factory=lambda path, **kw: llm(path, **kw))
    assert rc == 0
    rows = [json.loads(line) for line in out.read_text().splitlines()]
    assert [json.loads(line) for line in capsys.readouterr().out.splitlines()] == rows
    assert [(r["length"], r["batch_size"]) for r in rows] == [(9, 1), (9, 3), (20, 1), (20, 3)]
    for r in rows:
        assert r["completed"] == r["batch_size"] and r["output_len"] == 5
        assert r["prefill_tokens"] == r["batch_size"] * r["length"]
        assert 0 < r["decode_tokens"] <= r["batch_size"] * 4
        if r["batch_size"] == 1:
            assert r["decode_tokens"] == 4 and r["decode_steps"] == 4
        assert r["decode_tok_s"] > 0 and r["prefill_tok_s"] > 0 and r["total_s"] >= r["prefill_s"] + r["decode_s"] - 1e-3
    with pytest.raises(SystemExit):
        microbench.main(["--model_path", str(folder), "--lengths", "0"], llm_factory=lambda path, **kw: llm(path, **kw))


# ------------------------------------------------------------------ what another architecture needs, without a GPU
def test_toy_architecture_on_the_cpu(tmp_path):
    """The toy architecture of the tests (a mixer with state of its own, a windowed cache group, a
    layer that runs twice, a shared cache, its own feed-forward and rotation) registers, builds and
    steps on the kernel twins: float32 logits equal its plain implementation under a mixed trace."""
    from tests import backends
    from tests.test_gpu_engine import run_toy_architecture
    with backends.use("twin"):
        run_toy_architecture(tmp_path, "float32", [70, 9, 33, 100, 1, 64])


def test_an_architecture_with_state_only_and_no_cache_pages(tmp_path):
    """Every layer keeps state of fixed size and none keeps keys and values: no cache group, no page
    pool, no block table; item boundaries come from the step itself (``ForwardBatch.item_q_start``)."""
    from sparseengine_amd.weights.random_weights import write_model_folder
    from tests import toy_arch
    config = dict(toy_arch.TOY_CONFIG, max_position_embeddings=256, layers=[
        dict(mixer="decay", state_size=12, decay=0.8, ffn="dense", intermediate=40),
        dict(mixer="decay", state_size=5, decay=0.5, ffn="sign", intermediate=24)],
        schedule=[dict(layer=0), dict(layer=1), dict(layer=0)])
    folder = write_model_folder(str(tmp_path / "state_only"), config, 4, {"std": 0.15})
    plain = toy_arch.PlainToy(folder)
    requests = {f"r{i}": random_tokens(n, 300, 70 + i) for i, n in enumerate([40, 3, 65, 1, 17])}
    records, peak = traces.mixed(requests, seed=2)
    runner = ModelRunner.from_folder(folder, dtype="float32", device="cpu", kv_page_size=16, num_kvcache_tokens=64,
                                     max_num_seqs=4, kernels=TwinKernels())
    assert runner.cache.groups == [] and sorted(runner.cache.state_positions) == [0, 1, 2]
    out = {}
    for rec in records:
        logits = replay_step(runner, rec, None)
        if logits is not None:
            out[rec["step"]] = logits
        runner.cache.check_invariants()
    got = traces.gather(records, out)
    for rid, toks in requests.items():
        ref = plain.logits(toks).numpy()
        assert np.abs(got[rid] - ref).max() < 2e-5 * max(1.0, np.abs(ref).max()), rid
    assert runner.cache.num_free_rows == 4
    # and through the entry point: the scheduler has no pages to count, only rows
    engine = LLM(folder, dtype="float32", num_kvcache_slots=64, kv_page_size=16, max_num_seqs_in_batch=2,
                 _kernels=TwinKernels(), _device="cpu")
    prompts = [requests["r0"][:9], requests["r2"][:20], requests["r4"]]
    outs = engine.generate(prompts, SamplingParams(temperature=0.0, max_tokens=5, ignore_eos=True), use_tqdm=False)
    for prompt, o in zip(prompts, outs):
        toks = list(prompt)
        for t in o["token_ids"]:
            assert t == int(plain.logits(toks)[-1].argmax())
            toks.append(t)


def test_a_second_sparse_method_gets_every_hook(model):
    """A method registered from outside the package is resolved by name, bound to the cache and
    called once per step (prepare, finish), once per cache-keeping layer (select, after attention)
    and asked for its own pages; handing back the view it was given changes no token."""
    from sparseengine_amd.config import method_registry
    folder, requests, _, plain = model
    calls = []

    class Counting(method_registry.MethodRuntime):
        name = "counting"

        def bind(self, cache):
            super().bind(cache)
            calls.append(("bind", len(cache.groups)))

        def prepare_step(self, fb):
            calls.append(("prepare", fb.num_tokens))

        def select(self, position, meta):
            calls.append(("select", position))
            return meta

        def after_attention(self, position, fb):
            calls.append(("after", position))

        def finish_step(self, fb):
            calls.append(("finish", fb.num_tokens))

        def extra_pages(self, row, new_tokens):
            calls.append(("extra", new_tokens))
            return {0: 0}

    from sparseengine_amd.cache.manager import CacheManager

    class CountingCache(CacheManager):
        """The method's own cache manager: the paged one, counting what it is asked."""
        appended = 0

        def append(self, items):
            CountingCache.appended += sum(n for _, n in items)
            return super().append(items)

    method_registry.register_method("counting", Counting, "all_chunked", cache_manager_cls=CountingCache)
    try:
        assert method_registry.resolve_method("counting").cache_manager() is CountingCache
        assert method_registry.resolve_method("vanilla").cache_manager() is CacheManager
        engine = llm(folder, sparse_method="counting")
        assert type(engine.runner.cache) is CountingCache and engine.oracle.cache is engine.runner.cache
        assert type(llm(folder).runner.cache) is CacheManager
        prompt = list(requests.values())[1][:17]
        out = engine.generate([prompt], SamplingParams(temperature=0.0, max_tokens=3, ignore_eos=True), use_tqdm=False)
        assert out[0]["token_ids"] == plain.greedy(prompt, 3)
        layers = len(engine.runner.spec.schedule)
        steps = [c for c in calls if c[0] == "prepare"]
        assert calls[0] == ("bind", 1) and len(steps) == 3 and steps[0] == ("prepare", len(prompt)) and steps[1] == ("prepare", 1)
        assert [c for c in calls if c[0] == "finish"] == [("finish", n) for _, n in steps]
        assert [c[1] for c in calls if c[0] == "select"] == list(range(layers)) * 3
        assert [c[1] for c in calls if c[0] == "after"] == list(range(layers)) * 3
        assert any(c[0] == "extra" for c in calls)
        assert CountingCache.appended == len(prompt) + 2          # the prompt, then two fed-back tokens
        with pytest.raises(ValueError, match="counting"):
            llm(folder, sparse_method="counting", prefill_schedule_policy="something_else")
    finally:
        method_registry._METHODS.pop("counting", None)


def test_block_table_entries_are_checked_before_a_launch(model):
    """``validate_runtime_invariants``: before attention launches, every block-table entry the launch will
    read must name a page of the pool.  Entries a window has given back (-1) lie before what is read and
    pass; an entry inside the read range that is -1 or beyond the pool stops the step on the host, with
    the item and the entry named."""
    from types import SimpleNamespace
    from sparseengine_amd.engine.batch import BlockTableError, check_block_table
    table = np.array([[3, 5, 9, -1], [-1, -1, 2, 7]], dtype=np.int32)
    meta = SimpleNamespace(block_table_host=table, page_size=16, item_q_len=np.array([4, 1]), item_ctx_len=np.array([40, 60]))
    with pytest.raises(BlockTableError, match=r"item 1 .* entry 0 = -1"):
        check_block_table(meta, 0, 10)                             # no window: item 1 reads its pages 0..3
    check_block_table(meta, 24, 10)                                # window 24: item 1 reads keys 36..59, pages 2..3
    with pytest.raises(BlockTableError, match=r"item 0 .* entry 2 = 9"):
        check_block_table(meta, 0, 9)                              # page 9 of a pool of 9
    meta.item_ctx_len = np.array([50, 60])
    with pytest.raises(BlockTableError, match=r"item 0 .* entry 3 = -1"):
        check_block_table(meta, 24, 10)                            # item 0 now reaches into its fourth page
    meta.item_ctx_len = np.array([40, 70])
    with pytest.raises(BlockTableError, match="4 columns"):
        check_block_table(meta, 24, 10)
    # in the engine: on for a whole generation, and a table corrupted behind the cache manager's back is caught
    folder, requests, _, _ = model
    engine = llm(folder, validate_runtime_invariants=True)
    prompt = list(requests.values())[3][:40]
    engine.generate([prompt], SamplingParams(temperature=0.0, max_tokens=3, ignore_eos=True), use_tqdm=False)
    runner = engine.runner
    assert runner.validate_runtime_invariants
    runner.step([StepEntry("x", prompt[:20], [])])
    runner.cache.groups[0].table[runner.cache.row_of("x"), 0] = -1
    with pytest.raises(BlockTableError, match="entry 0 = -1"):
        runner.step([StepEntry("x", prompt[20:22], [1])])


def test_replay_writes_the_pages_each_request_held(model, tmp_path):
    """``pages.jsonl``: per step the page ids of the step's requests; under a pool of exactly the
    peak need, pages of finished requests turn up again under later ones."""
    folder, requests, _, _ = model
    records, peak = traces.mixed(requests, seed=5)
    runner = runner_for(folder, peak)
    replay_stream(runner, (json.dumps(r) for r in records), str(tmp_path / "out"), report=open(os.devnull, "w"),
                  with_taps=True)
    lines = [json.loads(line) for line in open(tmp_path / "out" / "pages.jsonl")]
    assert [l["step"] for l in lines] == [r["step"] for r in records]
    owners: dict[int, set] = {}
    fed: dict[str, int] = {}
    for rec, line in zip(records, lines):
        assert sorted(line["pages"]) == sorted(e["id"] for e in rec["entries"])
        held_now = [p for groups in line["pages"].values() for p in groups["0"]]
        assert len(held_now) == len(set(held_now)), "a page under two requests in one step"
        for e in rec["entries"]:
            fed[e["id"]] = fed.get(e["id"], 0) + len(e["tokens"])
            assert len(line["pages"][e["id"]]["0"]) == -(-fed[e["id"]] // 16)
            for page in line["pages"][e["id"]]["0"]:
                owners.setdefault(page, set()).add(e["id"])
    assert any(len(ids) > 1 for ids in owners.values()), "no page was used again"
    from safetensors.torch import load_file
    taps = load_file(str(tmp_path / "out" / f"{records[0]['step']}.taps.safetensors"))
    tokens = sum(len(e["tokens"]) for e in records[0]["entries"])
    assert taps["layer_out.0"].shape[0] == tokens and taps["router.0.ids"].shape[0] == tokens


def test_trace_run_program_on_the_cpu(model, tmp_path):
    """``bin/trace_run`` itself, as a user calls it, with the kernel twins named through the test
    seam: stdin in, logits files, ``done`` lines and the page log out; without the seam ``--device
    cpu`` is refused (the engine's own kernels are the GPU's)."""
    import subprocess
    import sys
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    folder, requests, expected, _ = model
    records, peak = traces.mixed(dict(list(requests.items())[:3]), seed=3)
    cmd = [sys.executable, os.path.join(root, "bin", "trace_run"), "--model", folder, "--dtype", "float32", "--out",
           str(tmp_path / "out"), "--max-tokens", str(peak), "--page-size", "16", "--device", "cpu"]
    env = {k: v for k, v in os.environ.items() if k != "SPARSEENGINE_AMD_KERNELS"}
    refused = subprocess.run(cmd, input="", capture_output=True, text=True, env=env)
    assert refused.returncode != 0 and "SPARSEENGINE_AMD_KERNELS" in refused.stderr
    env.update(SPARSEENGINE_AMD_KERNELS="tests.twin_kernels:TwinKernels", PYTHONPATH=root)
    proc = subprocess.run(cmd, input="".join(json.dumps(r) + "\n" for r in records), capture_output=True, text=True,
                          env=env, timeout=600)
    assert proc.returncode == 0, proc.stderr[-2000:]
    assert [l for l in proc.stdout.splitlines() if l.startswith("done")] == [f"done {r['step']}" for r in records]
    vocab = next(iter(expected.values())).shape[1]
    logits = {r["step"]: np.fromfile(tmp_path / "out" / f"{r['step']}.f32", dtype="<f4").reshape(-1, vocab) for r in records}
    got = traces.gather(records, logits)
    for rid in got:
        assert np.abs(got[rid] - expected[rid]).max() < 2e-5 * max(1.0, np.abs(expected[rid]).max())
    assert len(open(tmp_path / "out" / "pages.jsonl").readlines()) == len(records)
    # the variable without --device cpu is refused: it never replaces the GPU's kernels quietly
    on_gpu = [a for a in cmd if a not in ("--device", "cpu")]
    refused = subprocess.run(on_gpu, input="", capture_output=True, text=True, env=env)
    assert refused.returncode != 0 and "SPARSEENGINE_AMD_KERNELS is set" in refused.stderr
    # every page size the engine takes, also one that does not divide 64 and one above it
    for page_size in (48, 128):
        out = tmp_path / f"out{page_size}"
        other = [str(out) if a == str(tmp_path / "out") else a for a in cmd]
        other[other.index("--page-size") + 1] = str(page_size)
        proc = subprocess.run(other, input="".join(json.dumps(r) + "\n" for r in records), capture_output=True,
                              text=True, env=env, timeout=600)
        assert proc.returncode == 0, proc.stderr[-2000:]
        for r in records:
            assert np.abs(np.fromfile(out / f"{r['step']}.f32", dtype="<f4").reshape(-1, vocab) - logits[r["step"]]).max() < 2e-5
