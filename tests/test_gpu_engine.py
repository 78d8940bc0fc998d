"""The engine on the GPU beyond replay: long decoding, the first tokens of a sequence, greedy
generation through the entry point, weights kept in 32-bit under a bfloat16 engine, each part
alone, and a toy architecture (defined in the tests) with a recurrent mixer, a windowed cache
group, a dense feed-forward, a layer that runs twice and a shared cache."""
import os

import numpy as np
import pytest
import torch
from safetensors.torch import load_file, save_file

from tests import backends, traces
from tests.helpers import CONFIGS, make_folder, random_tokens
from tests.plain import minimax_m2 as P
from tests.plain.minimax_m2 import PlainMiniMaxM2

pytestmark = pytest.mark.gpu


from tests.test_gpu_replay import assert_close_to_plain, bound      # noqa: E402  (float32 bound; bfloat16: rounding noise only)


def runner_for(folder, dtype, tokens=1024, page_size=16, rows=4):
    from sparseengine_amd.engine.runner import ModelRunner
    return ModelRunner.from_folder(folder, dtype=dtype, kv_page_size=page_size,
                                   num_kvcache_tokens=-(-tokens // 64) * 64, max_num_seqs=rows,
                                   **backends.ACTIVE.runner_kwargs())


def replay_with_routing(runner, records):
    from sparseengine_amd.engine.replay import replay_step
    out, routing = {}, {}
    for rec in records:
        taps = {}
        logits = replay_step(runner, rec, None, taps=taps)
        if logits is not None:
            out[rec["step"]] = logits
        cursor = 0
        for e in rec["entries"]:
            n = len(e["tokens"])
            layers = routing.setdefault(e["id"], [[] for _ in taps.get("router", [])])
            for layer, (ids, _) in enumerate(taps.get("router", [])):
                layers[layer].append(ids[cursor:cursor + n].cpu())
            cursor += n
    return traces.gather(records, out), {r: [torch.cat(c).long() for c in layers] for r, layers in routing.items()}


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("key", ["B_loud", "A_loud", "C_loud"])
def test_long_decoding_token_by_token(tmp_path, key, dtype):
    """A short prompt and then hundreds of single-token steps across many pages."""
    folder = make_folder(tmp_path, key)
    raw = CONFIGS[key][0]
    n = raw["max_position_embeddings"] - 6
    if backends.ACTIVE.slow:      # a few pages instead of the whole context
        n = 70
    tokens = random_tokens(n, raw["vocab_size"], 77)
    records = traces.prefill_then_decode({"long": tokens}, tail=n - 3)
    runner = runner_for(folder, dtype, tokens=n + 64)
    got, routing = replay_with_routing(runner, records)
    plain = PlainMiniMaxM2(folder)
    ref = plain.logits(tokens, forced_routing=routing["long"] if dtype == "bfloat16" else None).numpy()
    assert_close_to_plain(dtype, got["long"], ref, f"{key}, {n} tokens one by one", layers=raw["num_hidden_layers"])


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_first_tokens_of_a_sequence(tmp_path, dtype):
    """Positions 0, 1, 2: one key, no prefix, an almost empty page; alone and three requests at once."""
    folder = make_folder(tmp_path, "B_loud")
    plain = PlainMiniMaxM2(folder)
    from sparseengine_amd.engine.runner import StepEntry
    runner = runner_for(folder, dtype)
    seqs = {f"s{i}": random_tokens(3, 1000, 200 + i) for i in range(3)}
    taps = {}
    logits = runner.step([StepEntry(r, t[:1], [0]) for r, t in seqs.items()], taps=taps).cpu().numpy()
    for i, (r, t) in enumerate(seqs.items()):
        forced = [ids[i:i + 1].cpu().long() for ids, _ in taps["router"]] if dtype == "bfloat16" else None
        ref = plain.logits(t[:1], forced_routing=forced).numpy()
        assert_close_to_plain(dtype, logits[i:i + 1], ref, f"first token of {r}", layers=3)
    taps = {}
    logits = runner.step([StepEntry(r, t[1:3], [0, 1]) for r, t in seqs.items()], taps=taps).cpu().numpy()
    if dtype == "float32":
        for i, (r, t) in enumerate(seqs.items()):
            ref = plain.logits(t).numpy()
            assert np.abs(logits[2 * i:2 * i + 2] - ref[1:3]).max() <= bound(dtype, ref)


@pytest.mark.parametrize("key", ["A_loud", "C_loud"])     # the general kernels; the matrix-core kernels in bfloat16
def test_greedy_generation_through_the_entry_point(tmp_path, key):
    from sparseengine_amd import LLM, SamplingParams
    folder = make_folder(tmp_path, key)
    plain = PlainMiniMaxM2(folder)
    prompts = [random_tokens(n, CONFIGS[key][0]["vocab_size"], 300 + n) for n in (5, 17, 31, 90)]
    params = SamplingParams(temperature=0.0, max_tokens=24, ignore_eos=True)
    expected = [plain.greedy(p, 24) for p in prompts]
    llm = LLM(folder, dtype="float32", num_kvcache_slots=1024, kv_page_size=16, max_num_seqs_in_batch=4,
              validate_runtime_invariants=True, **backends.ACTIVE.llm_kwargs())
    assert [o["token_ids"] for o in llm.generate(prompts, params, use_tqdm=False)] == expected
    # portions of 16 tokens beside decodes, and a cache so small that a request is thrown out and recomputed
    tight = LLM(folder, dtype="float32", num_kvcache_slots=192, kv_page_size=16, max_num_seqs_in_batch=4,
                max_num_batched_tokens=16, decode_reservation_tokens=0, validate_runtime_invariants=True,
                **backends.ACTIVE.llm_kwargs())
    assert [o["token_ids"] for o in tight.generate(prompts, params, use_tqdm=False)] == expected
    assert tight.scheduler.total_preemptions >= 1
    # bfloat16: every generated token is, for the plain logits of its own context, as good as the best
    # one up to bfloat16 rounding.  Rounding may tip a near-tie of the router, which moves logits by
    # more than rounding does: the plain implementation runs with the experts the engine chose (the
    # replay tests check that those are top-k choices up to a small slack).
    half = LLM(folder, dtype="bfloat16", num_kvcache_slots=1024, kv_page_size=16, max_num_seqs_in_batch=4,
               **backends.ACTIVE.llm_kwargs())
    run_step, fed = half.runner.step, {}

    def step_and_note_routing(entries, taps=None):
        taps = {}
        logits = run_step(entries, taps=taps)
        cursor = 0
        for e in entries:
            n = len(e.tokens)
            layers = fed.setdefault(e.request_id, [[] for _ in taps["router"]])
            for layer, (ids, _) in enumerate(taps["router"]):
                layers[layer].append(ids[cursor:cursor + n].cpu())
            cursor += n
        return logits
    half.runner.step = step_and_note_routing
    outs = half.generate(prompts, params, use_tqdm=False)
    by_request = [fed[k] for k in sorted(fed)]              # sequence ids grow in the order of the prompts
    assert len(by_request) == len(prompts) and half.scheduler.total_preemptions == 0
    for prompt, out, layers in zip(prompts, outs, by_request):
        ids = out["token_ids"]
        routing = [torch.cat(chunks).long() for chunks in layers]
        assert routing[0].shape[0] == len(prompt) + len(ids) - 1     # every token but the last was fed once
        logits = plain.logits(prompt + ids[:-1], forced_routing=routing)[len(prompt) - 1:]
        chosen = logits.gather(1, torch.tensor(ids)[:, None])[:, 0]
        assert (logits.max(-1).values - chosen).max() <= 2 * 0.04 * float(logits.abs().max())
    # temperature sampling: the same seed gives the same tokens, alone and in a batch
    sp = SamplingParams(temperature=0.8, top_k=40, top_p=0.95, max_tokens=12, ignore_eos=True, seed=9)
    alone = llm.generate([prompts[1]], sp, use_tqdm=False)[0]["token_ids"]
    mixed = llm.generate(prompts[:3], [params, sp, SamplingParams(temperature=1.2, max_tokens=7, ignore_eos=True)],
                         use_tqdm=False)[1]["token_ids"]
    assert alone == mixed


def test_random_workloads_through_the_entry_point(tmp_path):
    """Seeded random workloads (numbers and lengths of requests, completion lengths, page sizes, cache
    sizes from ample to barely enough, token budgets down to eight) in float32: every request gets
    exactly the plain implementation's greedy tokens, whatever was cut, batched, deferred or thrown
    out and computed again on the way."""
    import random
    from sparseengine_amd import LLM, SamplingParams
    rng = random.Random(11)
    key = "B_loud"
    folder = make_folder(tmp_path, key)
    raw = CONFIGS[key][0]
    plain = PlainMiniMaxM2(folder)
    known = {}
    preemptions = 0
    for scenario in range(5):
        n = rng.randint(2, 8)
        prompts = [random_tokens(rng.choice([1, 3, 17, 40, 90, 150]), raw["vocab_size"], rng.randrange(10 ** 6)) for _ in range(n)]
        params = [SamplingParams(temperature=0.0, max_tokens=rng.choice([1, 5, 20, 40]), ignore_eos=True) for _ in range(n)]
        page = rng.choice([8, 16, 32])
        need = max(len(p) + sp.max_tokens for p, sp in zip(prompts, params))
        slots = max(-(-need // page) * page + page, rng.choice([160, 192, 256, 512]))
        in_batch = rng.choice([2, 4, 8])
        llm = LLM(folder, dtype="float32", num_kvcache_slots=slots, kv_page_size=page, max_num_seqs_in_batch=in_batch,
                  max_num_batched_tokens=max(in_batch, rng.choice([8, 16, 64, 512])),
                  decode_reservation_tokens=rng.choice([0, 16, 64]), validate_runtime_invariants=True,
                  **backends.ACTIVE.llm_kwargs())
        outs = llm.generate(prompts, params, use_tqdm=False)
        for p, sp, o in zip(prompts, params, outs):
            ref = known.setdefault((tuple(p), sp.max_tokens), plain.greedy(p, sp.max_tokens))
            assert o["token_ids"] == ref, f"scenario {scenario}: prompt of {len(p)}, {sp.max_tokens} new tokens"
        preemptions += llm.scheduler.total_preemptions
    assert preemptions >= 1, "no scenario ran out of pages: the seed no longer covers preemption"


@pytest.fixture
def command_line_backend(monkeypatch):
    """The command line builds its engine itself; on the emulated backend the kernels' stand-in is
    named through the environment, as for any other program."""
    if backends.ACTIVE.name == "emu":
        monkeypatch.setenv("SPARSEENGINE_AMD_KERNELS", "tests.emu.kernels:EmuKernels")
        return ["--device", "cpu"]
    return []


def test_command_line_generates_what_the_entry_point_generates(tmp_path, capsys, command_line_backend):
    import json
    from sparseengine_amd import LLM, SamplingParams
    from sparseengine_amd.__main__ import main
    folder = make_folder(tmp_path, "B_loud")
    prompts = [random_tokens(n, 1000, 40 + n) for n in (7, 23)]
    llm = LLM(folder, dtype="float32", num_kvcache_slots=512, kv_page_size=16, **backends.ACTIVE.llm_kwargs())
    expected = llm.generate(prompts, SamplingParams(temperature=0.7, top_k=20, max_tokens=9, ignore_eos=True, seed=5),
                            use_tqdm=False)
    del llm
    ids_file = tmp_path / "prompts.jsonl"
    ids_file.write_text(json.dumps(prompts[1]) + "\n")
    capsys.readouterr()
    assert main(["generate", "--model", folder, "--prompt-ids", json.dumps(prompts[0]), "--prompt-ids", str(ids_file),
                 "--dtype", "float32", "--num-kvcache-slots", "512", "--kv-page-size", "16", "--temperature", "0.7",
                 "--top-k", "20", "--max-tokens", "9", "--ignore-eos", "--seed", "5", *command_line_backend]) == 0
    lines = [json.loads(line) for line in capsys.readouterr().out.splitlines() if line.startswith("{")]
    assert [line["prompt"] for line in lines] == prompts
    assert [line["token_ids"] for line in lines] == [e["token_ids"] for e in expected]


def test_command_line_bench_runs_every_case_on_the_gpu(tmp_path, capsys, command_line_backend):
    import json
    from sparseengine_amd.__main__ import main
    folder = make_folder(tmp_path, "A_loud")
    capsys.readouterr()
    assert main(["bench", "--model_path", folder, "--lengths", "40,130", "--batch_sizes", "1,4", "--output_len", "6",
                 "--hyper_params", json.dumps({"kv_page_size": 16, "num_kvcache_slots": 2048,
                                               "max_num_batched_tokens": 96}), *command_line_backend]) == 0
    rows = [json.loads(line) for line in capsys.readouterr().out.splitlines() if line.startswith("{")]
    assert [(r["length"], r["batch_size"]) for r in rows] == [(40, 1), (40, 4), (130, 1), (130, 4)]
    for r in rows:
        assert r["completed"] == r["batch_size"] and r["prefill_tokens"] == r["batch_size"] * r["length"]
        # the counts and rates of a row are those of its case: every prompt token fed once, the first
        # generated token comes with the prompt's last portion, the five others from decode steps
        # (a step that holds a prompt portion beside decoded tokens counts as a prompt step, as in the reference)
        assert 5 <= r["decode_tokens"] <= 5 * r["batch_size"] and r["decode_steps"] >= 5
        assert r["batch_size"] > 1 or r["decode_tokens"] == 5
        assert r["prefill_steps"] >= -(-r["prefill_tokens"] // 96)          # the token budget of 96 cuts the prompts
        assert r["decode_tok_s"] == pytest.approx(r["decode_tokens"] / r["decode_s"], rel=1e-3, abs=0.06)     # rounded to 0.1
        assert r["prefill_tok_s"] == pytest.approx(r["prefill_tokens"] / r["prefill_s"], rel=1e-3, abs=0.06)
        assert r["ms_per_decode_step"] == pytest.approx(r["decode_s"] / r["decode_steps"] * 1e3, rel=1e-2)
        assert 0 < r["time_to_first_decode_s"] <= r["total_s"] and r["prefill_s"] + r["decode_s"] <= r["total_s"] * 1.001


def test_weights_stored_in_32_bit_stay_so_under_bfloat16(tmp_path):
    folder = make_folder(tmp_path, "A_loud")
    path = os.path.join(folder, "model.safetensors")
    tensors = {k: v.float() for k, v in load_file(path).items()}         # the whole checkpoint in float32
    save_file(tensors, path)
    runner = runner_for(folder, "bfloat16")
    assert all(p.dtype == torch.float32 for p in runner.params.values())
    tokens = random_tokens(60, 512, 8)
    records = traces.changing_portions({"r": tokens}, seed=3)
    got, routing = replay_with_routing(runner, records)
    ref = PlainMiniMaxM2(folder).logits(tokens, forced_routing=routing["r"]).numpy()
    assert_close_to_plain("bfloat16", got["r"], ref, "weights kept in float32")


# ------------------------------------------------------------------ each part alone
class Harness:
    """A cache, a batch builder and a hand-made batch for one part."""

    def __init__(self, dtype, requests=None, pages=32, page_size=16):
        from sparseengine_amd.cache.manager import CacheManager
        from sparseengine_amd.engine.batch import BatchBuilder
        self.dtype = dtype
        self.cache = CacheManager(requests or {}, max_rows=4, max_model_len=512, page_size=page_size, num_pages=pages,
                                  dtype=dtype, device=backends.ACTIVE.device)
        self.builder = BatchBuilder(backends.ACTIVE.kernels(), self.cache, dtype, backends.ACTIVE.device, vocab_size=1 << 20)

    def batch(self, lengths):
        from sparseengine_amd.engine.batch import StepItem
        items = []
        for rid, n in lengths:
            if not self.cache.has_row(rid):
                self.cache.admit(rid)
            items.append(StepItem(self.cache.row_of(rid), [0] * n, []))
        return self.builder.build(items)


def materialize(part, dtype, seed, scale=0.1):
    g = torch.Generator().manual_seed(seed)
    params = {}
    for name, decl in part.all_param_decls().items():
        value = torch.randn(decl.shape, generator=g) * scale
        if "norm" in name:
            value = 1 + value
        params[name] = value.to(torch.float32 if decl.policy == "float32" else dtype).to(backends.ACTIVE.device)
    part.bind_all(params)
    return {k: v.float().cpu().clone() for k, v in params.items()}


def assert_part_close(dtype, got, ref):
    """float32: float rounding.  bfloat16: the bound of the logits tests, 4 % of the largest value."""
    if dtype == torch.float32:
        torch.testing.assert_close(got, ref, rtol=1e-4, atol=1e-4)
    else:
        assert float((got - ref).abs().max()) <= 0.04 * float(ref.abs().max())


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_norm_part(dtype):
    from sparseengine_amd.config.specs import NormSpec
    from sparseengine_amd.parts import NORMS
    norm = NORMS.build(NormSpec(eps=1e-3), hidden_size=200)
    w = materialize(norm, dtype, 1)
    h = Harness(dtype)
    fb = h.batch([("a", 7)])
    x = torch.randn(7, 200).to(dtype).to(backends.ACTIVE.device)
    r = torch.randn(7, 200).to(dtype).to(backends.ACTIVE.device)
    x0, r0 = x.float().cpu().clone(), r.float().cpu().clone()      # on a CPU backend .cpu() copies nothing
    norm.forward(fb, x, residual=r)
    y, merged = P.add_rms_norm(x0, r0, w["weight"], 1e-3)
    assert_part_close(dtype, x.float().cpu().clone(), y)
    assert_part_close(dtype, r.float().cpu().clone(), merged)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("head_dim,rotary,theta,scaling", [(128, 64, 5e6, None), (48, 48, 1e4, None),
                                                           (64, 32, 1e4, (("factor", 4.0), ("rope_type", "linear")))])
def test_position_part(dtype, head_dim, rotary, theta, scaling):
    """The rotary part alone: its table through the kernel that applies it (no norm, no cache write), at the
    positions of the reference's vector (tests/test_flashinfer_rope.py:12-30).  The dims beyond the rotary ones
    come back bit for bit, position 0 changes nothing, and positions divided by a linear scaling factor turn
    by the angles of the plain implementation at the divided positions."""
    from sparseengine_amd.config.specs import RotarySpec
    from sparseengine_amd.parts import POSITIONS
    part = POSITIONS.build(RotarySpec(rotary_dim=rotary, theta=theta, max_position=2048, scaling=scaling), head_dim=head_dim)
    part.limit_positions(1100)
    part.prepare(backends.ACTIVE.device)
    assert part.table.shape == (1100, rotary) and part.table.dtype == torch.float32
    heads, kv_heads = 3, 2
    positions = torch.tensor([0, 1, 17, 127, 1023], dtype=torch.int32)
    T = positions.numel()
    qkv = torch.randn(T, (heads + 2 * kv_heads) * head_dim, generator=torch.Generator().manual_seed(5)).to(dtype)
    given = qkv.float().clone()
    on_device = qkv.to(backends.ACTIVE.device)
    backends.ACTIVE.kernels().qk_norm_rope_store(on_device, positions.to(backends.ACTIVE.device), part.table, None, None, 1e-6,
                                                 heads, kv_heads, head_dim, part.rotary_dim, None, None, 0, pairing=part.pairing)
    got = on_device.float().cpu().clone()
    factor = dict(scaling)["factor"] if scaling else 1.0
    cos, sin = P.rope_angles(positions.float() / factor, rotary, theta)
    width = (heads + kv_heads) * head_dim
    ref = P.partial_rope(given[:, :width].reshape(T, heads + kv_heads, head_dim), cos, sin, rotary).reshape(T, width)
    assert_part_close(dtype, got[:, :width], ref)
    assert torch.equal(got[:, width:], given[:, width:]), "values are not rotated"
    assert torch.equal(got[0], given[0]), "position 0 is the identity"
    if rotary < head_dim:
        kept = got[:, :width].reshape(T, -1, head_dim)[..., rotary:]
        assert torch.equal(kept, given[:, :width].reshape(T, -1, head_dim)[..., rotary:]), "dims beyond the rotary ones pass through"


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("heads,kv_heads,head_dim,rotary,norm,window", [(6, 2, 32, 16, "flat", None), (5, 5, 48, 48, "none", 10),
                                                                        (8, 1, 64, 0, "flat", None)])
def test_attention_part_in_two_portions(dtype, heads, kv_heads, head_dim, rotary, norm, window):
    from sparseengine_amd.config.specs import AttentionSpec, NoPositionSpec, RotarySpec
    from sparseengine_amd.parts import MIXERS
    position = RotarySpec(rotary_dim=rotary, theta=1e4, max_position=512) if rotary else NoPositionSpec()
    spec = AttentionSpec(num_heads=heads, num_kv_heads=kv_heads, head_dim=head_dim, scale=head_dim ** -0.5,
                         qk_norm=norm, qk_norm_eps=1e-5, window=window, position=position)
    mixer = MIXERS.build(spec, hidden_size=72)
    w = materialize(mixer, dtype, 2, scale=0.2)
    h = Harness(dtype, {0: mixer.cache_request()})
    T, cut = 45, 29
    x = torch.randn(T, 72).to(dtype)
    out = torch.cat([mixer.forward(h.batch([("a", cut)]), x[:cut].to(backends.ACTIVE.device), 0).float().cpu().clone(),
                     mixer.forward(h.batch([("a", T - cut)]), x[cut:].to(backends.ACTIVE.device), 0).float().cpu().clone()])
    xf = x.float()
    qkv = xf @ w["qkv"].T
    q, k, v = qkv[:, :heads * head_dim], qkv[:, heads * head_dim:(heads + kv_heads) * head_dim], qkv[:, (heads + kv_heads) * head_dim:]
    if norm == "flat":
        q, k = P.flat_qk_norm(q, w["q_norm"], 1e-5), P.flat_qk_norm(k, w["k_norm"], 1e-5)
    q, k, v = q.reshape(T, heads, head_dim), k.reshape(T, kv_heads, head_dim), v.reshape(T, kv_heads, head_dim)
    if rotary:
        cos, sin = P.rope_angles(torch.arange(T), rotary, 1e4)
        q, k = P.partial_rope(q, cos, sin, rotary), P.partial_rope(k, cos, sin, rotary)
    ref = P.causal_gqa_attention(q, k, v, head_dim ** -0.5, window=window).reshape(T, -1) @ w["o"].T
    assert_part_close(dtype, out, ref)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("hidden,experts,top_k,inter,scoring,bias", [(96, 5, 5, 40, "sigmoid", True), (256, 12, 3, 128, "softmax", False)])
def test_feed_forward_parts(dtype, hidden, experts, top_k, inter, scoring, bias):
    from sparseengine_amd.config.specs import DenseMLPSpec, MoESpec
    from sparseengine_amd.parts import FEED_FORWARDS
    moe = FEED_FORWARDS.build(MoESpec(num_experts=experts, top_k=top_k, intermediate_size=inter, scoring=scoring,
                                      selection_bias=bias, norm_topk_prob=bias, routed_scaling_factor=1.0 if bias else 2.0),
                              hidden_size=hidden, chunk_tokens=16)       # 37 tokens: three chunks, invisible
    w = materialize(moe, dtype, 3, scale=0.15)
    h = Harness(dtype)
    x = torch.randn(37, hidden).to(dtype)
    fb = h.batch([("a", 37)])
    fb.taps = {}
    out = moe.forward(fb, x.to(backends.ACTIVE.device)).float().cpu().clone()
    ids = torch.cat([i for i, _ in fb.taps["router"]]).long().cpu()
    xf = x.float()
    scores = torch.sigmoid(xf @ w["router"].T) if scoring == "sigmoid" else torch.softmax(xf @ w["router"].T, -1)
    wts = scores.gather(1, ids)
    wts = wts / wts.sum(-1, keepdim=True) if bias else wts * 2.0
    ref = P.swiglu_experts(xf, w["w13"][:, :inter], w["w13"][:, inter:], w["w2"], ids, wts)
    assert_part_close(dtype, out, ref)
    if dtype == torch.float32:       # the choice itself: top-k of score (+ bias)
        sel = scores + w["router_bias"] if bias else scores
        assert torch.equal(ids.sort(-1).values, torch.topk(sel, top_k).indices.sort(-1).values)
    mlp = FEED_FORWARDS.build(DenseMLPSpec(intermediate_size=inter), hidden_size=hidden)
    w = materialize(mlp, dtype, 4, scale=0.15)
    out = mlp.forward(h.batch([("b", 37)]), x.to(backends.ACTIVE.device)).float().cpu().clone()
    gu = xf @ w["gate_up"].T
    assert_part_close(dtype, out, (torch.nn.functional.silu(gu[:, :inter]) * gu[:, inter:]) @ w["down"].T)


# ------------------------------------------------------------------ the toy architecture
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_toy_architecture_registers_builds_and_steps(tmp_path, dtype):
    run_toy_architecture(tmp_path, dtype, [70, 9, 33, 150, 1, 64])


def run_toy_architecture(tmp_path, dtype, lengths):
    from sparseengine_amd.weights.random_weights import write_model_folder
    from tests.toy_arch import TOY_CONFIG, PlainToy
    folder = write_model_folder(str(tmp_path / "toy"), TOY_CONFIG, 3, {"std": 0.15})
    plain = PlainToy(folder)
    requests = {f"r{i}": random_tokens(n, 300, 50 + i) for i, n in enumerate(lengths)}
    expected = {r: plain.logits(t).numpy() for r, t in requests.items()}
    records, peak = traces.mixed(requests, seed=1)
    runner = runner_for(folder, dtype, tokens=peak)
    # three groups of cache pages: two kv heads (a layer that runs twice and the position after them), the window, one kv head
    assert [(g.request.window, g.positions) for g in runner.cache.groups] == [(None, [0, 3, 6]), (24, [2]), (None, [5])]
    assert list(runner.cache.state_positions) == [1]
    from sparseengine_amd.engine.replay import replay_step
    out, chosen = {}, {rid: {"router": [[], []], "sign": [[]]} for rid in requests}
    for rec in records:
        taps = {}
        logits = replay_step(runner, rec, None, taps=taps)
        if logits is not None:
            out[rec["step"]] = logits
        cursor = 0
        for e in rec["entries"]:      # what the routed layers chose for every token, per request
            n = len(e["tokens"])
            for layer, (ids, _) in enumerate(taps["router"]):
                chosen[e["id"]]["router"][layer].append(ids[cursor:cursor + n].cpu().long())
            chosen[e["id"]]["sign"][0].append(taps["toy_sign"][0][cursor:cursor + n].cpu())
            cursor += n
        runner.cache.check_invariants()
    got = traces.gather(records, out)
    for rid, ref in expected.items():
        if dtype == "bfloat16":   # a near-tie of a routed layer may tip in bfloat16: the plain run takes the engine's choices
            forced = {kind: [torch.cat(chunks) for chunks in layers] for kind, layers in chosen[rid].items()}
            ref = plain.logits(requests[rid], forced=forced).numpy()
        assert_close_to_plain(dtype, got[rid], ref, f"toy architecture, request {rid}", layers=len(TOY_CONFIG["schedule"]))
    assert all(g.pool.free_count == g.pool.num_pages for g in runner.cache.groups)
    windowed = runner.cache.groups[1]
    assert windowed.window == 24 and windowed.page_size == 8 and runner.cache.groups[0].page_size == 16   # pages of its own size
