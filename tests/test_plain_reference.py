"""Pins of the plain implementation beside the reference's text: vectors the reference's own tests
hold, special cases that reduce to a library routine, and invariants.  Each is chosen so that a
plausible mistake (a wrong sign or pairing, a norm in the wrong place) fails it."""
import math

import pytest
import torch
import torch.nn.functional as F

from tests.helpers import CONFIGS, make_folder, random_tokens
from tests.plain import minimax_m2 as plain


def test_rms_norm_is_the_library_routine_and_fused_form_adds_first():
    torch.manual_seed(37)
    x, r = torch.randn(7, 96), torch.randn(7, 96)
    w = 1 + 0.2 * torch.randn(96)
    torch.testing.assert_close(plain.rms_norm(x, w, 1e-5), F.rms_norm(x, (96,), w, 1e-5))
    # eps is added to the mean of squares (not to the rms, not outside the root)
    tiny = torch.full((1, 4), 1e-4)
    torch.testing.assert_close(plain.rms_norm(tiny, torch.ones(4), 1e-6), tiny / math.sqrt(1e-8 + 1e-6))
    # reference oracle tests/test_minimax_m2_model.py:59-71: the norm of the sum, and the sum itself
    y, merged = plain.add_rms_norm(x, r, w, 1e-5)
    torch.testing.assert_close(merged, x + r)
    torch.testing.assert_close(y, F.rms_norm(x + r, (96,), w, 1e-5))
    # scale equivariance for eps -> 0 and unit output rms for unit weight
    torch.testing.assert_close(plain.rms_norm(3 * x, w, 0.0), plain.rms_norm(x, w, 0.0))
    out = plain.rms_norm(x, torch.ones(96), 0.0)
    torch.testing.assert_close(out.square().mean(-1), torch.ones(7))


def test_flat_qk_norm_is_one_statistic_over_all_heads():
    torch.manual_seed(1)
    heads, dim = 4, 16
    x = torch.randn(5, heads * dim)
    x[:, :dim] *= 10          # heads of very different scale
    w = 1 + 0.1 * torch.randn(heads * dim)
    flat = plain.flat_qk_norm(x, w, 1e-6)
    torch.testing.assert_close(flat, F.rms_norm(x, (heads * dim,), w, 1e-6))
    per_head = (F.rms_norm(x.view(5, heads, dim), (dim,), None, 1e-6).reshape(5, -1)) * w
    assert not torch.allclose(flat, per_head, atol=1e-2)     # tests/test_minimax_m2_model.py:376-377,414


def rope(x, positions, rotary_dim, theta):
    cos, sin = plain.rope_angles(positions, rotary_dim, theta)
    return plain.partial_rope(x, cos, sin, rotary_dim)


def test_partial_rope_vector_of_the_reference():
    """tests/test_flashinfer_rope.py:12-63, case minimax-m2.7: 6 q heads, head 128, rotary 64,
    base 5e6, positions [0, 1, 17, 127, 1023]; pass-through dims bit-equal."""
    torch.manual_seed(0)
    positions = torch.tensor([0, 1, 17, 127, 1023])
    q = torch.randn(5, 6, 128)
    out = rope(q, positions, 64, 5e6)
    assert torch.equal(out[..., 64:], q[..., 64:])
    assert torch.equal(out[0], q[0])                                  # position 0 is the identity
    # pairs are (d, d + R/2) inside the first R dims: the rotation keeps each pair's norm
    pair_norm = lambda t: t[..., :32].square() + t[..., 32:64].square()
    torch.testing.assert_close(pair_norm(out), pair_norm(q))
    # the angle of dim d at position p is p * base^(-2d/R), with R (not the head size) below
    d, p = 3, 17
    angle = p * 5e6 ** (-2 * d / 64)
    x1, x2 = q[2, 0, d].item(), q[2, 0, d + 32].item()
    assert out[2, 0, d].item() == pytest.approx(x1 * math.cos(angle) - x2 * math.sin(angle), abs=1e-5)
    assert out[2, 0, d + 32].item() == pytest.approx(x2 * math.cos(angle) + x1 * math.sin(angle), abs=1e-5)
    # full rotary is the same function with R = D
    full = rope(q[..., :64].contiguous(), positions, 64, 5e6)
    torch.testing.assert_close(full, out[..., :64])


def test_rope_scores_depend_on_distance_only():
    torch.manual_seed(3)
    q, k = torch.randn(1, 1, 32), torch.randn(1, 1, 32)
    def score(pq, pk):
        return (rope(q, torch.tensor([pq]), 16, 1e4) * rope(k, torch.tensor([pk]), 16, 1e4)).sum()
    assert score(40, 33).item() == pytest.approx(score(140, 133).item(), abs=1e-4)
    assert score(40, 33).item() != pytest.approx(score(40, 30).item(), abs=1e-4)


def test_attention_is_the_library_routine():
    torch.manual_seed(5)
    T, H, Hkv, D = 13, 6, 2, 16
    q, k, v = torch.randn(T, H, D), torch.randn(T, Hkv, D), torch.randn(T, Hkv, D)
    out = plain.causal_gqa_attention(q, k, v, D ** -0.5)
    ref = F.scaled_dot_product_attention(q.transpose(0, 1)[None], k.transpose(0, 1)[None], v.transpose(0, 1)[None],
                                         is_causal=True, enable_gqa=True)[0].transpose(0, 1)
    torch.testing.assert_close(out, ref)
    torch.testing.assert_close(out[0], v[0].repeat_interleave(H // Hkv, 0))      # one key: the output is its value
    # query head i reads kv head i // group (not i % kv_heads)
    v2 = v.clone(); v2[:, 1] += 100
    out2 = plain.causal_gqa_attention(q, k, v2, D ** -0.5)
    torch.testing.assert_close(out2[:, :3], out[:, :3])
    assert (out2[:, 3:] - out[:, 3:]).abs().min() > 50
    # a window of w keeps keys p-w+1 .. p
    w = plain.causal_gqa_attention(q, k, v, D ** -0.5, window=4)
    tail = plain.causal_gqa_attention(q[9:], k[9:], v[9:], D ** -0.5)
    torch.testing.assert_close(w[12], tail[3])


def test_router_is_topk_of_biased_sigmoid_with_unbiased_weights():
    # oracle tests/test_minimax_m2_router.py:16-25; bias vector :110-122
    logits = torch.linspace(-4, 4, 256)[None]
    bias = torch.zeros(256); bias[:8] = 2
    weights, ids = plain.biased_sigmoid_router(logits, bias, 8)
    assert set(ids[0].tolist()) == set(range(8))
    s = torch.sigmoid(logits[0, ids[0]])
    torch.testing.assert_close(weights[0], s / s.sum())
    torch.manual_seed(27)
    logits = torch.randn(64, 256) * 3
    weights, ids = plain.biased_sigmoid_router(logits, torch.zeros(256), 8)
    assert torch.equal(ids.sort(-1).values, torch.topk(logits, 8).indices.sort(-1).values)   # b = 0: top-k of logits
    torch.testing.assert_close(weights.sum(-1), torch.ones(64))


def test_experts_reduce_to_a_plain_swiglu_and_to_a_mean():
    torch.manual_seed(7)
    T, h, I, E = 9, 32, 24, 4
    x = torch.randn(T, h)
    w1, w3, w2 = torch.randn(E, I, h) * 0.2, torch.randn(E, I, h) * 0.2, torch.randn(E, h, I) * 0.2
    one = plain.swiglu_experts(x, w1[:1], w3[:1], w2[:1], torch.zeros(T, 1, dtype=torch.long), torch.ones(T, 1))
    torch.testing.assert_close(one, (F.silu(x @ w1[0].T) * (x @ w3[0].T)) @ w2[0].T)       # w1 gate, w3 up, w2 down
    ids = torch.arange(E).expand(T, E)
    mean = plain.swiglu_experts(x, w1, w3, w2, ids, torch.full((T, E), 1 / E))
    each = torch.stack([(F.silu(x @ w1[e].T) * (x @ w3[e].T)) @ w2[e].T for e in range(E)])
    torch.testing.assert_close(mean, each.mean(0), atol=1e-5, rtol=1e-5)
    perm = torch.tensor([2, 0, 3, 1])                                                     # renaming experts changes nothing
    ids2 = torch.stack([torch.randperm(E)[:2] for _ in range(T)])
    wts = torch.rand(T, 2)
    a = plain.swiglu_experts(x, w1, w3, w2, ids2, wts)
    inverse = torch.argsort(perm)
    b = plain.swiglu_experts(x, w1[perm], w3[perm], w2[perm], inverse[ids2], wts)
    torch.testing.assert_close(a, b)


@pytest.fixture(scope="module")
def model_a(tmp_path_factory):
    return plain.PlainMiniMaxM2(make_folder(tmp_path_factory.mktemp("plain"), "A_loud"))


def test_residual_wiring(model_a):
    """With the output projections zeroed, mixer and experts add nothing: logits = head(norm(embed))."""
    m = plain.PlainMiniMaxM2.__new__(plain.PlainMiniMaxM2)
    m.cfg, m.dtype, m.w = model_a.cfg, model_a.dtype, dict(model_a.w)
    for name in m.w:
        if name.endswith("o_proj.weight") or name.endswith(".w2.weight"):
            m.w[name] = torch.zeros_like(m.w[name])
    toks = random_tokens(11, 512, 3)
    emb = m.w["model.embed_tokens.weight"][toks]
    expect = plain.rms_norm(emb, m.w["model.norm.weight"], m.cfg.rms_norm_eps) @ m.w["lm_head.weight"].T
    torch.testing.assert_close(m.logits(toks), expect)


def test_causality_and_position_shift(model_a):
    toks = random_tokens(20, 512, 4)
    full = model_a.logits(toks)
    torch.testing.assert_close(model_a.logits(toks[:12]), full[:12], atol=1e-5, rtol=1e-5)   # later tokens change nothing
    shifted = model_a.logits(toks, start_position=57)        # only distances count
    torch.testing.assert_close(shifted, full, atol=2e-4, rtol=2e-4)
    changed = list(toks); changed[5] = (changed[5] + 1) % 512
    other = model_a.logits(changed)
    torch.testing.assert_close(other[:5], full[:5])
    assert (other[5:] - full[5:]).abs().max() > 1e-3


def test_float64_agrees(model_a, tmp_path):
    m64 = plain.PlainMiniMaxM2(make_folder(tmp_path, "A_loud"), dtype=torch.float64)
    toks = random_tokens(25, 512, 5)
    assert (m64.logits(toks).float() - model_a.logits(toks)).abs().max() < 5e-5
