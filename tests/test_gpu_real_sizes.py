"""The bfloat16 engine against its own float32 path at MiniMax-M2 layer sizes (hidden 3072, 48 query
and 8 kv heads of 128, rotary 64, 256 experts of width 1536 with top-8), one layer, a vocabulary cut
to 2048: the only place where the matrix-core expert kernels at K = 3072 / 1536, the 128-wide
attention kernels and the skinny products meet a reference inside the engine.

Both engines hold the same weights (drawn by name on the device and rounded to bfloat16 before either
engine stores them).  The float32 engine is first checked against the plain implementation, then
serves as the reference of the bfloat16 engine in every replay mode, with the bfloat16 engine's
expert choices forced on it (a near-tie among 256 experts tips in bfloat16, which moves a logit by
far more than rounding does; the choices themselves are checked to be top-8 up to a small slack).
The bound.  A bfloat16 rounding is off by 2^-9 / sqrt(3) = 0.11 % of the value (rms); sixteen
roundings lie between the embedding and a logit of one layer (norms, projections, the five of the
attention inputs and outputs, the stored residual, four in the experts, the slot sum, the head), so
a logit should be off by about 0.45 % of the logits' spread (rms) at a position with few keys.
Measured on MI355X: 0.41 % at the first positions, growing to 1.0 % at position 700 (attention
averages more and more rounded keys and values), the same at every position of equal context,
Gaussian (largest error of 1.4 million logits: 5.1 times the rms).  What a fault looks like is
different: a wrong key, page or expert moves the logits of some positions by their whole spread.
So the test asks for (1) an rms error of at most 1.5 % of the spread at every single position,
(2) no single logit further off than 6.5 times the request's rms error (a Gaussian tail over a
million samples ends at 5.2) and (3) 1 % of the logit's own size on top, for its own rounding.
(The reference compares its model with a float oracle at rtol 1e-2 / atol 2e-2 on a tiny model,
tests/test_minimax_m2_model.py:95; the suite's general bfloat16 bound, 4 % of the largest logit,
is about 20 % of the spread.)
"""
import numpy as np
import pytest
import torch

from tests import backends, traces
from tests.helpers import random_tokens
from tests.plain.minimax_m2 import PlainMiniMaxM2

pytestmark = pytest.mark.gpu

REAL = dict(
    architectures=["MiniMaxM2ForCausalLM"], model_type="minimax_m2", num_hidden_layers=2, hidden_size=3072,
    num_attention_heads=48, num_key_value_heads=8, head_dim=128, rotary_dim=64, rope_theta=5000000.0,
    num_local_experts=256, num_experts_per_tok=8, intermediate_size=1536, vocab_size=2048, rms_norm_eps=1e-6,
    use_qk_norm=True, max_position_embeddings=1024, tie_word_embeddings=False)
OPTIONS = dict(std=0.02, norm_std=0.1, bias_std=0.02)
SEED = 21
ROUTING_SLACK = 0.02


def engine(dtype, tokens):
    from sparseengine_amd.engine.runner import ModelRunner
    return ModelRunner.from_random(REAL, seed=SEED, options=OPTIONS, on_device=True, dtype=dtype, kv_page_size=64,
                                   num_kvcache_tokens=tokens, max_num_seqs=4, max_model_len=1024)


def plain_model():
    """The plain implementation on the same tensors (by checkpoint name), on the device."""
    from sparseengine_amd.config.registry import resolve_architecture
    from sparseengine_amd.parts import build_model
    from sparseengine_amd.weights import random_weights
    arch = resolve_architecture(REAL)
    cfg = arch.parse_config(REAL)
    decls = build_model(arch.build_spec(cfg)).all_param_decls()
    tensors = {src.name: value for src, value in
               random_weights.checkpoint_tensors(arch, cfg, decls, SEED, OPTIONS, device=torch.device("cuda"))}
    return PlainMiniMaxM2.from_tensors(REAL, tensors)


def replay(runner, records, forced=None):
    """Logits per step, and per step the experts every routed layer chose."""
    from sparseengine_amd.engine.replay import replay_step
    out, chosen = {}, {}
    for rec in records:
        taps = {}
        entries = [e for e in rec["entries"]]
        if forced is None:
            logits = replay_step(runner, rec, None, taps=taps)
        else:       # the same step with given choices
            from sparseengine_amd.engine.runner import StepEntry
            step = [StepEntry(str(e["id"]), list(e["tokens"]), list(e.get("want", []))) for e in entries]
            result = runner.step(step, taps=taps, forced_routing=forced[rec["step"]])
            logits = result.cpu().numpy() if result.shape[0] else None
            for rid in rec.get("end", []):
                runner.release(str(rid))
        if logits is not None:
            out[rec["step"]] = logits
        chosen[rec["step"]] = [ids.clone() for ids, _ in taps["router"]]
    return out, chosen


def choices_by_request(records, chosen, requests):
    """Per request and layer the experts chosen for each of its positions, from the per-step records."""
    layers = len(next(iter(chosen.values())))
    out = {rid: [[] for _ in range(layers)] for rid in requests}
    for rec in records:
        cursor = 0
        for e in rec["entries"]:
            n = len(e["tokens"])
            for layer in range(layers):
                out[e["id"]][layer].append(chosen[rec["step"]][layer][cursor:cursor + n])
            cursor += n
    return {rid: [torch.cat(parts).long() for parts in layers] for rid, layers in out.items()}


def plain_with_choices(plain, tokens, choices, slack, what):
    """The plain logits with the given experts, after checking that every choice is a top-k of the plain
    selection scores up to ``slack`` (rounding may tip a near-tie among 256 experts; nothing else may)."""
    log = {}
    ref = plain.logits(tokens, forced_routing=choices, routing_log=log).cpu().numpy()
    for layer, ids in enumerate(choices):
        scores = log[layer]
        kth = torch.topk(scores, ids.shape[1], dim=-1).values[:, -1:]
        assert (scores.gather(1, ids) >= kth - slack).all(), f"{what}, layer {layer}: an expert below the top-{ids.shape[1]} was chosen"
    return ref


def assert_float32_meets_plain(got, ref, what):
    err = np.abs(got - ref).max(-1)
    bound = 2e-5 * max(1.0, float(np.abs(ref).max()))
    assert err.max() <= bound, f"float32 engine against plain, {what}: error {err.max():.3g} at position {int(err.argmax())}, bound {bound:.3g}"


def test_bfloat16_against_float32_at_real_layer_sizes():
    if backends.ACTIVE.name != "hip":
        pytest.skip("sizes of the full model: GPU only")
    torch.manual_seed(0)
    requests = {"a": random_tokens(5, 2048, 1), "b": random_tokens(130, 2048, 2), "c": random_tokens(700, 2048, 3)}
    full = engine("float32", 1024)
    plain = plain_model()
    # the float32 engine against the plain implementation, every request whole, with its own routing:
    # both are float32, so a choice may differ from the plain one only where two scores agree to rounding
    whole = traces.whole(requests)
    logits32, chosen32 = replay(full, whole)
    got32 = traces.gather(whole, logits32)
    own = choices_by_request(whole, chosen32, requests)
    for rid, tokens in requests.items():
        assert_float32_meets_plain(got32[rid], plain_with_choices(plain, tokens, own[rid], 2e-5, f"float32, request {rid}"),
                                   f"request {rid} whole")

    half = engine("bfloat16", 1024)
    assert all(layer.ffn._tiled is True for layer in half.model.layers)
    mixed, _ = traces.mixed(requests, seed=4)
    modes = {"whole": whole, "tail": traces.prefill_then_decode(requests, tail=32),
             "portions": traces.changing_portions(requests, seed=5), "mixed": mixed}
    for mode, records in modes.items():
        logits16, chosen = replay(half, records)
        reference, _ = replay(full, records, forced=chosen)
        got, ref = traces.gather(records, logits16), traces.gather(records, reference)
        theirs = choices_by_request(records, chosen, requests)
        for rid in requests:
            # the float32 engine, cut and batched this way and with the bfloat16 engine's choices, against the
            # plain implementation with the same choices (each a top-8 of the plain scores up to the slack)
            assert_float32_meets_plain(
                ref[rid], plain_with_choices(plain, requests[rid], theirs[rid], ROUTING_SLACK, f"{mode}, request {rid}"),
                f"{mode}, request {rid}")
            scale = float(ref[rid].std())
            err = np.abs(got[rid] - ref[rid])
            per_position = np.sqrt((err ** 2).mean(-1)) / scale
            assert per_position.max() <= 0.015, (
                f"{mode}, request {rid}: rms error {per_position.max():.4f} of the spread at position "
                f"{int(per_position.argmax())} (median over positions {float(np.median(per_position)):.4f})")
            rms = float(np.sqrt((err ** 2).mean()))
            allowed = 6.5 * rms + 1e-2 * np.abs(ref[rid])
            worst = np.unravel_index(int((err - allowed).argmax()), err.shape)
            assert (err <= allowed).all(), (
                f"{mode}, request {rid}: position {worst[0]}, token {worst[1]}: bfloat16 {got[rid][worst]:.4f}, "
                f"float32 {ref[rid][worst]:.4f}, rms error of the request {rms:.4f}, spread of the logits {scale:.3f}")
    assert half.cache.num_free_rows == 4 and full.cache.num_free_rows == 4
