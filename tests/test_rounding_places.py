"""Where bfloat16 rounds, pinned by vectors made for it.

The reference computes norms, the SwiGLU product and the QK norm in float and rounds to the activations'
type at stated places (kernels/triton/rmsnorm.py:38-66: the norm of the *unrounded* sum, one rounding of
the result; layers/layernorm.py:210 and kernels/triton/column_parallel_rmsnorm.py:94-102: ``(x * inv_rms)``
rounded, then times the weight in the activations' type; kernels/triton/moe.py:726-733 and
kernels/triton/silu_and_mul.py:40-58: gate and up rounded, silu in float on the rounded gate, rounded, then
the product).  Random inputs cannot tell these places from their neighbours: moving one changes a value by
one unit in the last place now and then.  Each test here builds an input on which the stated order and a
plausible other order give *different bfloat16 values* (the test asserts that they do), and asks the
kernel for the stated one, exactly.  The same tests run the tensor-library twins on the CPU and the HIP
kernels on the GPU.
"""
import math

import pytest
import torch

from tests import backends

BF16 = torch.bfloat16


def r(x):
    """Round to bfloat16 and widen again."""
    return x.to(BF16).float()


def kernels_and_device(on_gpu: bool):
    if not on_gpu:
        from tests.twin_kernels import TwinKernels
        return TwinKernels(), "cpu"
    return backends.ACTIVE.kernels(), backends.ACTIVE.device


BACKENDS = [pytest.param(False, id="twin"), pytest.param(True, id="hip", marks=pytest.mark.gpu)]


def silu(z):
    return z / (1 + torch.exp(-z))


@pytest.mark.parametrize("on_gpu", BACKENDS)
@pytest.mark.parametrize("kernel", [None, "stream", "mid", "direct", "tall"])
def test_gate_and_up_are_rounded_before_the_activation(on_gpu, kernel):
    """Two intermediate columns whose gates are 1 and 1 + 3/1024: both round to 1 in bfloat16, so with the
    reference's places their activations are the same value and a down projection with weights +1 and -1
    gives exactly 0; the activation of the unrounded gates rounds to two different values (0.73046875 and
    0.734375), and the output would be their difference."""
    if kernel is not None and not on_gpu:
        pytest.skip("the twin has one expert path")
    g_exact = torch.tensor([1.0, 1.0 + 3 / 1024])
    stated = r(silu(r(g_exact)))
    other = r(silu(g_exact))
    assert stated[0] == stated[1] and other[0] != other[1]                       # the vector tells the two orders apart
    hip, dev = kernels_and_device(on_gpu)
    hidden, inter = 256, 128
    x = torch.zeros(1, hidden)
    x[0, 0], x[0, 1] = 1.0, 3 / 1024                                              # both exact in bfloat16
    w13 = torch.zeros(1, 2 * inter, hidden)
    w13[0, 0, 0] = 1.0                                                            # gate 0 = 1
    w13[0, 1, 0] = w13[0, 1, 1] = 1.0                                             # gate 1 = 1 + 3/1024 (exact in the float sum)
    w13[0, inter, 0] = w13[0, inter + 1, 0] = 1.0                                 # up = 1 for both
    w2 = torch.zeros(1, hidden, inter)
    w2[0, 0, 0], w2[0, 0, 1] = 1.0, -1.0                                          # output 0 = column 0 - column 1
    w2[0, 1, 0] = 1.0                                                             # output 1 = column 0
    ids = torch.zeros(1, 1, dtype=torch.int32)
    weights = torch.ones(1, 1)
    args = [t.to(BF16).to(dev) for t in (x, w13, w2)] + [ids.to(dev), weights.to(dev)]
    out = torch.full((1, hidden), float("nan"), dtype=BF16, device=dev)
    if on_gpu:
        from sparseengine_amd.kernels.hip_ops import MoeWorkspace
        ws = MoeWorkspace(1, 1, 1, hidden, inter, BF16, dev)
        hip.moe_experts(*args, out, ws, kernel=kernel, tile_rows={"mid": 64, "direct": 64, "tall": 64}.get(kernel))
    else:
        hip.moe_experts(*args, out)
    assert float(out[0, 0]) == 0.0
    assert float(out[0, 1]) == float(stated[0])
    assert float(out[0, 2:].abs().max()) == 0.0


def find_qk_row(width: int):
    """A row and a weight for which ``r(r(x * inv_rms) * w)`` and ``r(x * inv_rms * w)`` differ at element 0."""
    g = torch.Generator().manual_seed(5)
    for _ in range(2000):
        x = r(torch.randn(width, generator=g))
        w = r(1 + 0.5 * torch.randn(width, generator=g))
        inv = torch.rsqrt(x.square().sum() / width + 1e-6)
        stated = r(r(x * inv) * w)
        other = r(x * inv * w)
        differ = torch.nonzero(stated != other).flatten()
        if differ.numel():
            return x, w, stated, other, int(differ[0])
    raise AssertionError("no telling row found")


@pytest.mark.parametrize("on_gpu", BACKENDS)
def test_the_flat_qk_norm_rounds_before_its_weight(on_gpu):
    """``(x * inv_rms)`` is rounded to the activations' type and then multiplied by the weight in that type
    (two roundings), not multiplied in float and rounded once."""
    heads, kv_heads, head_dim = 2, 1, 32
    x, w, stated, other, at = find_qk_row(heads * head_dim)
    assert stated[at] != other[at]
    hip, dev = kernels_and_device(on_gpu)
    qkv = torch.zeros(1, (heads + 2 * kv_heads) * head_dim)
    qkv[0, :heads * head_dim] = x
    qkv[0, heads * head_dim:(heads + kv_heads) * head_dim] = 1.0
    qkv = qkv.to(BF16).to(dev)
    positions = torch.zeros(1, dtype=torch.int32, device=dev)
    hip.qk_norm_rope_store(qkv, positions, None, w.to(BF16).to(dev), torch.ones(kv_heads * head_dim, dtype=BF16, device=dev),
                           1e-6, heads, kv_heads, head_dim, 0)
    got = qkv[0, :heads * head_dim].float().cpu()
    assert torch.equal(got, stated), f"element {at}: {float(got[at])}, stated order {float(stated[at])}, single rounding {float(other[at])}"


def find_norm_rows(width: int):
    """x, residual, weight for which the norm of the unrounded sum (one rounding at the end) differs from the
    norm of the rounded sum, and from ``r(x * inv_rms)`` times the weight."""
    g = torch.Generator().manual_seed(9)
    for _ in range(4000):
        x, res = r(torch.randn(width, generator=g)), r(torch.randn(width, generator=g))
        w = r(1 + 0.5 * torch.randn(width, generator=g))
        merged = x + res                                                      # float
        stated = r(merged * torch.rsqrt(merged.square().mean() + 1e-5) * w)
        rounded_first = r(merged)
        of_rounded = r(rounded_first * torch.rsqrt(rounded_first.square().mean() + 1e-5) * w)
        two_roundings = r(r(merged * torch.rsqrt(merged.square().mean() + 1e-5)) * w)
        if (stated != of_rounded).any() and (stated != two_roundings).any():
            return x, res, w, stated, r(merged)
    raise AssertionError("no telling rows found")


@pytest.mark.parametrize("on_gpu", BACKENDS)
def test_the_fused_norm_reads_the_unrounded_sum_and_rounds_once(on_gpu):
    """``r = x + residual`` in float; the new residual is its rounding, the norm is taken of the *unrounded*
    sum, the weight is multiplied in float and the result rounded once."""
    width = 64
    x, res, w, stated, new_residual = find_norm_rows(width)
    hip, dev = kernels_and_device(on_gpu)
    xd, rd = x.to(BF16)[None].to(dev).contiguous(), res.to(BF16)[None].to(dev).contiguous()
    out = torch.empty_like(xd)
    hip.rms_norm(xd, w.to(BF16).to(dev), 1e-5, out, residual=rd)
    assert torch.equal(rd[0].float().cpu(), new_residual)
    assert torch.equal(out[0].float().cpu(), stated)
    # the same sum as a token's two slots that the norm adds up itself: slots are added in float and that sum is
    # rounded to the activations' type first (it stands for a tensor that the feed-forward would have stored)
    if getattr(hip, "slot_sum_deferral_tokens", 0):
        slots = torch.stack([x, torch.zeros_like(x)]).to(BF16).to(dev).contiguous()
        rd2 = res.to(BF16)[None].to(dev).contiguous()
        out2 = torch.empty_like(xd)
        hip.rms_norm(slots, w.to(BF16).to(dev), 1e-5, out2, residual=rd2, slots=2)
        assert torch.equal(out2, out) and torch.equal(rd2, rd)


def test_the_vectors_are_what_they_claim():
    """The arithmetic behind the first test, written out (no kernel): the gates' roundings and the two
    activations' roundings."""
    assert float(r(torch.tensor(1 + 3 / 1024))) == 1.0
    assert math.isclose(float(silu(torch.tensor(1.0))), 0.7310586, rel_tol=1e-6)
    assert float(r(silu(torch.tensor(1.0)))) == 0.73046875 and float(r(silu(torch.tensor(1 + 3 / 1024)))) == 0.734375


@pytest.mark.parametrize("on_gpu", BACKENDS)
@pytest.mark.parametrize("dtype_path", ["matrix_core", "general"])
def test_probabilities_are_rounded_before_the_value_product(on_gpu, dtype_path):
    """``p = exp(score - max)`` is rounded to the activations' type for ``p . V``, while the sum that divides
    the result keeps the unrounded values (kernels/triton/context_flashattention_nopad.py:119,
    gqa_flash_decoding_stage1.py:97).  Two keys whose scores are 0 and -1/1024: the second probability,
    exp(-1/1024) = 0.99902, rounds to 1; with values +1 and -1 the stated order gives exactly 0, the
    unrounded product gives 0.000244."""
    from types import SimpleNamespace
    import numpy as np
    from sparseengine_amd.cache import layout
    p2 = math.exp(-1 / 1024)
    assert float(r(torch.tensor(p2))) == 1.0 and float(r(torch.tensor((1 - p2) / (1 + p2)))) != 0.0
    hip, dev = kernels_and_device(on_gpu)
    if dtype_path == "general" and not on_gpu:
        pytest.skip("the twin has one attention path")
    heads, kv_heads, head_dim, page = 2, 1, 64, 16
    q = torch.zeros(1, heads, head_dim)
    q[0, :, 0] = 1.0
    keys = torch.zeros(2, kv_heads, head_dim)
    keys[1, 0, 0] = -(head_dim ** 0.5) / 1024              # score of key 1: -1/1024 after the scale
    values = torch.zeros(2, kv_heads, head_dim)
    values[0, 0, 0], values[1, 0, 0] = 1.0, -1.0           # dim 0: +1 and -1
    values[0, 0, 1] = 1.0                                   # dim 1: the first key alone
    cache = torch.zeros(3, 2, kv_heads, page, head_dim, dtype=BF16)
    pages, offsets = torch.tensor([2, 2]), torch.tensor([0, 1])
    layout.write_keys(cache, pages, offsets, keys.to(BF16))
    layout.write_values(cache, pages, offsets, values.to(BF16))
    table = torch.tensor([[2]], dtype=torch.int32)
    meta = SimpleNamespace(block_table=table.to(dev), token_row=torch.zeros(1, dtype=torch.int32, device=dev),
                           positions=torch.ones(1, dtype=torch.int32, device=dev), work={})
    if dtype_path == "matrix_core":       # with the items' lengths the bfloat16 call takes the matrix-core kernels
        meta.item_q_len, meta.item_ctx_len = np.asarray([1]), np.asarray([2])
        meta.item_meta = torch.tensor([[0], [1], [2]], dtype=torch.int32, device=dev)
    out = torch.full((1, heads * head_dim), float("nan"), dtype=BF16, device=dev)
    hip.paged_attention(q.to(BF16).to(dev), cache.to(dev), meta, out, head_dim ** -0.5, 0)
    got = out.float().cpu().view(heads, head_dim)
    assert float(got[:, 0].abs().max()) == 0.0
    assert torch.equal(got[:, 1], r(torch.tensor(1 / (1 + p2))).expand(heads))
    assert float(got[:, 2:].abs().max()) == 0.0
