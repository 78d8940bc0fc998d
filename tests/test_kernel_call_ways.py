"""The hot kernel calls have a short way through their checks; it must pass the entry points what the long way passes.

No kernel runs here: the table of entry points is replaced by a recorder, the tensors live on the CPU.  Every case
is called twice, with the short ways on and off, and the two records (entry point, every argument) are compared."""
import pytest
import torch

from sparseengine_amd.kernels import hip_ops

BF16 = torch.bfloat16


class Recorder:
    def __init__(self, status=None):
        self.calls, self.status = [], status or {}       # entry point -> the status it returns (default 0)

    def get(self, library, name):
        def entry(*args):
            self.calls.append((library, name, args))
            return self.status.get(name, 0)
        return entry


@pytest.fixture
def ways(monkeypatch):
    """Run ``call()`` with the short ways on and off; returns both records."""
    kernels = hip_ops.HipKernels.__new__(hip_ops.HipKernels)
    kernels._attention_partials = kernels._sample_partials = None
    monkeypatch.setattr(hip_ops, "_stream", lambda: 77)

    def both(call, status=None):
        records = []
        for short in (True, False):
            recorder = Recorder(status)
            monkeypatch.setattr(hip_ops, "_fn", recorder)
            monkeypatch.setattr(hip_ops, "_SHORT_WAYS", short)
            result = call(kernels)
            records.append((recorder.calls, result))
        return records
    return both


def same(records):
    (short_calls, short_result), (long_calls, long_result) = records
    assert short_calls and short_calls == long_calls
    return short_result, long_result


@pytest.mark.parametrize("dtype,wdtype", [(BF16, BF16), (BF16, torch.float32), (torch.float32, torch.float32)])
@pytest.mark.parametrize("with_residual", [True, False])
def test_rms_norm(ways, dtype, wdtype, with_residual):
    x, out = torch.zeros(3, 64, dtype=dtype), torch.zeros(3, 64, dtype=dtype)
    res = torch.zeros(3, 64, dtype=dtype) if with_residual else None
    w = torch.ones(64, dtype=wdtype)
    same(ways(lambda k: k.rms_norm(x, w, 1e-5, out, residual=res)))
    same(ways(lambda k: k.rms_norm(x, w, 1e-5, x, residual=res, write_residual=False)))
    wide = torch.zeros(3, 72, dtype=dtype)
    same(ways(lambda k: k.rms_norm(wide[:, :64], w, 1e-5, out, residual=res)))          # a view with a row stride


def test_rms_norm_of_slots(ways):
    slots, out, res, w = torch.zeros(12, 64, dtype=BF16), torch.zeros(3, 64, dtype=BF16), torch.zeros(3, 64, dtype=BF16), torch.ones(64, dtype=BF16)
    same(ways(lambda k: k.rms_norm(slots, w, 1e-5, out, residual=res, slots=4)))
    # the fused kernel refuses (status -1): both ways go on to the sum and the plain norm
    records = ways(lambda k: k.rms_norm(slots, w, 1e-5, out, residual=res, slots=4), status={"se_rms_norm_slots": -1})
    names = [[name for _, name, _ in calls] for calls, _ in records]
    assert names[1] == ["se_rms_norm_slots", "se_moe_sum", "se_rms_norm"] and names[0] == ["se_rms_norm_slots"] + names[1]


def test_rms_norm_mistakes_are_named_either_way(ways):
    x, w = torch.zeros(3, 64, dtype=BF16), torch.ones(32, dtype=BF16)
    for short in (True, False):
        with pytest.raises(ValueError, match="weight shape"):
            ways(lambda k: k.rms_norm(x, w, 1e-5, x))


def test_linear_on_a_prepared_matrix(ways):
    x, w, out = torch.zeros(4, 256, dtype=BF16), torch.zeros(48, 256, dtype=BF16), torch.zeros(4, 48, dtype=BF16)
    prepared = torch.zeros(48, 256, dtype=BF16)
    short, long = same(ways(lambda k: k.linear(x, w, out, prepared=prepared)))
    assert short is out and long is out
    with pytest.raises(ValueError, match="prepared copy"):
        ways(lambda k: k.linear(x, w, out, prepared=torch.zeros(32, 256, dtype=BF16)))


@pytest.mark.parametrize("wdtype", [BF16, torch.float32])
def test_qk_norm_rope_store(ways, wdtype):
    heads, kv_heads, head_dim, rotary, page = 4, 2, 32, 16, 8
    qkv = torch.zeros(5, (heads + 2 * kv_heads) * head_dim, dtype=BF16)
    positions, slots = torch.arange(5, dtype=torch.int32), torch.arange(5, dtype=torch.int32)
    table = torch.zeros(64, rotary)
    qw, kw = torch.ones(heads * head_dim, dtype=wdtype), torch.ones(kv_heads * head_dim, dtype=wdtype)
    cache = torch.zeros(3, 2, kv_heads, page, head_dim, dtype=BF16)
    for pairing in ("neox", "interleaved"):
        same(ways(lambda k: k.qk_norm_rope_store(qkv, positions, table, qw, kw, 1e-6, heads, kv_heads, head_dim, rotary,
                                                 cache, slots, page, pairing=pairing)))
    with pytest.raises(ValueError, match="cache layout"):
        ways(lambda k: k.qk_norm_rope_store(qkv, positions, table, qw, kw, 1e-6, heads, kv_heads, head_dim, rotary,
                                            cache, slots, 16))


@pytest.mark.parametrize("sum_slots", [True, False])
def test_expert_products_of_a_decode_step(ways, sum_slots):
    tokens, top_k, experts, hidden, inter = 2, 2, 8, 128, 128
    x, out = torch.zeros(tokens, hidden, dtype=BF16), torch.zeros(tokens, hidden, dtype=BF16)
    w13, w2 = torch.zeros(experts, 2 * inter, hidden, dtype=BF16), torch.zeros(experts, hidden, inter, dtype=BF16)
    ids = torch.zeros(tokens, top_k, dtype=torch.int32)
    weights = torch.ones(tokens, top_k)
    ws = hip_ops.MoeWorkspace(tokens, top_k, experts, hidden, inter, BF16, "cpu")

    def call(k):
        ws.grouped = (ids.data_ptr(), tokens, top_k, experts, 16, 4)       # what the router's launch leaves
        result = k.moe_experts(x, w13, w2, ids, weights, out, ws, tiled=True, sum_slots=sum_slots)
        assert ws.grouped is None
        return None if result is None else (result.data_ptr(), tuple(result.shape))
    short, long = same(ways(call))
    assert short == long
