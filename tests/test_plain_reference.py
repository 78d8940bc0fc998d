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


def one_layer_model(tmp_path, zero=()):
    """Configuration A cut to one layer, loud weights; tensors whose names end in one of ``zero`` are zeroed."""
    from sparseengine_amd.weights.random_weights import write_model_folder
    raw, options, seed = CONFIGS["A_loud"]
    folder = write_model_folder(str(tmp_path / "one_layer"), dict(raw, num_hidden_layers=1), seed, options)
    m = plain.PlainMiniMaxM2(folder)
    for name in m.w:
        if name.endswith(tuple(zero)):
            m.w[name] = torch.zeros_like(m.w[name])
    return m


def test_qk_norm_comes_before_the_rotation(tmp_path):
    """The reference's own statement of the order (tests/test_minimax_m2_model.py:357-417): the rotated
    dims of what attention receives are the rotation of the *normed* row, the other dims are the
    normed row bit for bit.  With a norm weight that differs from dim to dim the other order
    (rotate, then norm) gives other numbers; the test says by how much."""
    m = one_layer_model(tmp_path)
    c, p = m.cfg, "model.layers.0.self_attn."
    H, Hkv, D, R = c.num_attention_heads, c.num_key_value_heads, c.head_dim, c.rotary_dim
    assert H * D == c.hidden_size          # so that an identity projection makes q the input row itself
    eye = torch.eye(c.hidden_size)
    m.w[p + "q_proj.weight"], m.w[p + "k_proj.weight"], m.w[p + "v_proj.weight"] = eye, eye[:Hkv * D], eye[Hkv * D:2 * Hkv * D]
    torch.manual_seed(3)
    m.w[p + "q_norm.weight"] = torch.linspace(0.2, 3.0, H * D)[torch.randperm(H * D)]      # strongly non-uniform
    m.w[p + "k_norm.weight"] = torch.linspace(3.0, 0.2, Hkv * D)
    u = torch.randn(3, c.hidden_size)
    u[:, :D] *= 0.1
    u[:, D:2 * D] *= 10.0
    positions = torch.tensor([0, 1, 17])
    q, k, v = m.attention_inputs(0, u, positions)
    normed_q = F.rms_norm(u, (H * D,), m.w[p + "q_norm.weight"], c.rms_norm_eps).view(3, H, D)
    normed_k = F.rms_norm(u[:, :Hkv * D], (Hkv * D,), m.w[p + "k_norm.weight"], c.rms_norm_eps).view(3, Hkv, D)
    assert torch.equal(v, u[:, Hkv * D:2 * Hkv * D].view(3, Hkv, D))                      # values: neither normed nor turned
    # the angle written out: p * theta^(-2d/R), pairs (d, d + R/2)
    d = torch.arange(R // 2, dtype=torch.float64)
    angle = positions.double()[:, None] * c.rope_theta ** (-2 * d / R)
    cos, sin = angle.cos().float()[:, None, :], angle.sin().float()[:, None, :]
    for got, normed in ((q, normed_q), (k, normed_k)):
        assert torch.equal(got[..., R:], normed[..., R:])                                 # pass-through dims: the normed row itself
        lo, hi = normed[..., :R // 2], normed[..., R // 2:R]
        torch.testing.assert_close(got[..., :R // 2], lo * cos - hi * sin, atol=1e-5, rtol=1e-5)
        torch.testing.assert_close(got[..., R // 2:R], hi * cos + lo * sin, atol=1e-5, rtol=1e-5)
    # the other order: rotate the raw row, then norm it
    raw_cos, raw_sin = plain.rope_angles(positions, R, c.rope_theta)
    swapped = plain.flat_qk_norm(plain.partial_rope(u.view(3, H, D), raw_cos, raw_sin, R).reshape(3, -1),
                                 m.w[p + "q_norm.weight"], c.rms_norm_eps).view(3, H, D)
    assert torch.equal(swapped[0], q[0])                                                   # position 0 turns nothing
    assert (swapped[1:, :, :R] - q[1:, :, :R]).abs().max() > 0.1


def hand_written_layer(m, toks, attention=True, experts=True):
    """One pre-norm layer and the head with library norms, written out: ``r = e (+ a)``;
    ``y = norm_f(r (+ moe(norm_post(r))))`` (models/minimax_m2.py:381-397, models/qwen3.py:291-325)."""
    c, w = m.cfg, m.w
    n = lambda z, name: F.rms_norm(z, (c.hidden_size,), w[name], c.rms_norm_eps)
    e = w["model.embed_tokens.weight"][toks]
    positions = torch.arange(len(toks))
    r = e
    if attention:
        r = e + m.attention(0, n(e, "model.layers.0.input_layernorm.weight"), positions)
    out = r
    if experts:
        out = r + m.moe(0, n(r, "model.layers.0.post_attention_layernorm.weight"))
    return n(out, "model.norm.weight") @ w["lm_head.weight"].T


def test_the_residual_inside_a_layer(tmp_path):
    """What only one of the two zeroed projections shows: the mixer's result is added to the residual
    before the second norm, that norm reads the sum (not the mixer's result alone: with the output
    projection zeroed that would norm a zero row and the experts would add nothing), and the final norm
    reads the experts' result plus that same sum."""
    toks = random_tokens(9, 512, 6)
    only_attention = one_layer_model(tmp_path, zero=(".w2.weight",))
    torch.testing.assert_close(only_attention.logits(toks), hand_written_layer(only_attention, toks, experts=False))
    only_experts = one_layer_model(tmp_path, zero=("o_proj.weight",))
    expect = hand_written_layer(only_experts, toks, attention=False)
    torch.testing.assert_close(only_experts.logits(toks), expect)
    bare = one_layer_model(tmp_path, zero=("o_proj.weight", ".w2.weight"))
    assert (expect - bare.logits(toks)).abs().max() > 1e-2          # the experts did add something
    both = one_layer_model(tmp_path)
    full = hand_written_layer(both, toks)
    torch.testing.assert_close(both.logits(toks), full)
    # the second norm reading the mixer's result alone would give other logits
    c, w = both.cfg, both.w
    e = w["model.embed_tokens.weight"][toks]
    a = both.attention(0, F.rms_norm(e, (c.hidden_size,), w["model.layers.0.input_layernorm.weight"], c.rms_norm_eps),
                       torch.arange(len(toks)))
    wrong = F.rms_norm(e + a + both.moe(0, F.rms_norm(a, (c.hidden_size,), w["model.layers.0.post_attention_layernorm.weight"],
                                                       c.rms_norm_eps)),
                       (c.hidden_size,), w["model.norm.weight"], c.rms_norm_eps) @ w["lm_head.weight"].T
    assert (wrong - full).abs().max() > 1e-2
