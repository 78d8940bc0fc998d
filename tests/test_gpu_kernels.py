"""Each HIP kernel alone against its plain twin, at sizes other than the engine's."""
from types import SimpleNamespace

import pytest
import torch

from sparseengine_amd.cache import layout
from tests import backends
from tests.twin_kernels import TwinKernels

pytestmark = pytest.mark.gpu

DTYPES = [torch.float32, torch.bfloat16]
DEV = "cuda"      # where the tensors of a test live: the backend's device (set before every test)


@pytest.fixture(autouse=True)
def _device():
    global DEV
    DEV = backends.ACTIVE.device


@pytest.fixture
def hip():
    return backends.ACTIVE.kernels()


@pytest.fixture(scope="module")
def twin():
    return TwinKernels()


def emulator_skips(work: float, limit: float = 3e8):
    """The emulated backend runs a kernel's threads one after the other: cases whose size says
    nothing new about indexing are left to the GPU."""
    if backends.ACTIVE.slow and work > limit:
        pytest.skip("too large for the emulated backend")


def tol(dtype):
    return dict(rtol=2e-5, atol=2e-5) if dtype == torch.float32 else dict(rtol=1.6e-2, atol=1.6e-2)


def randn(*shape, dtype, scale=1.0, seed=0):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(*shape, generator=g) * scale).to(dtype).to(DEV)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("tokens,hidden,vocab", [(1, 64, 50), (37, 3072, 1000), (5, 200, 77)])
def test_embedding(hip, dtype, tokens, hidden, vocab):
    table = randn(vocab, hidden, dtype=dtype)
    ids = torch.randint(0, vocab, (tokens,), dtype=torch.int32).to(DEV)
    out = torch.empty(tokens, hidden, dtype=dtype, device=DEV)
    hip.embedding(ids, table, out)
    assert torch.equal(out, table[ids.long()])


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("wdtype", [None, torch.float32])
@pytest.mark.parametrize("tokens,hidden", [(1, 64), (7, 3072), (33, 200), (3, 6144), (2, 15360)])
def test_rms_norm_plain_and_fused(hip, twin, dtype, wdtype, tokens, hidden):
    wdtype = wdtype or dtype
    x = randn(tokens, hidden, dtype=dtype, seed=1)
    res = randn(tokens, hidden, dtype=dtype, seed=2)
    w = (1 + 0.2 * torch.randn(hidden)).to(wdtype).to(DEV)
    # plain
    out_h, out_t = torch.empty_like(x), torch.empty_like(x)
    hip.rms_norm(x, w, 1e-5, out_h)
    twin.rms_norm(x, w, 1e-5, out_t)
    torch.testing.assert_close(out_h, out_t, **tol(dtype))
    torch.testing.assert_close(out_h.float(), torch.nn.functional.rms_norm(x.float(), (hidden,), w.float(), 1e-5), **tol(dtype))
    # fused add, in place: the residual is the rounded sum, bit for bit
    xh, rh, xt, rt = x.clone(), res.clone(), x.clone(), res.clone()
    hip.rms_norm(xh, w, 1e-5, xh, residual=rh)
    twin.rms_norm(xt, w, 1e-5, xt, residual=rt)
    assert torch.equal(rh, (x.float() + res.float()).to(dtype))
    torch.testing.assert_close(xh, xt, **tol(dtype))
    # row selection leaves the residual alone
    rows = torch.tensor([tokens - 1, 0], dtype=torch.int32).to(DEV)
    oh = torch.empty(2, hidden, dtype=dtype, device=DEV)
    ot = torch.empty_like(oh)
    r_before = res.clone()
    hip.rms_norm(x, w, 1e-5, oh, residual=res, rows=rows)
    twin.rms_norm(x, w, 1e-5, ot, residual=res, rows=rows)
    torch.testing.assert_close(oh, ot, **tol(dtype))
    assert torch.equal(res, r_before)


def test_rms_norm_refuses_wide_rows(hip):
    from sparseengine_amd.kernels.hip_ops import KernelShapeError
    x = torch.zeros(1, 16384, device=DEV)
    with pytest.raises(KernelShapeError):
        hip.rms_norm(x, torch.ones(16384, device=DEV), 1e-6, torch.empty_like(x))


def rope_table(max_pos, rotary_dim, theta):
    inv = 1.0 / (theta ** (torch.arange(0, rotary_dim, 2, dtype=torch.float32) / rotary_dim))
    f = torch.arange(max_pos, dtype=torch.float32)[:, None] * inv[None]
    return torch.cat((f.cos(), f.sin()), -1).to(DEV)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("heads,kv_heads,head_dim,rotary,norm,page", [
    (4, 2, 16, 8, True, 16), (6, 3, 32, 32, False, 16), (48, 8, 128, 64, True, 64),
    (5, 5, 48, 16, True, 32), (6, 1, 128, 64, True, 16), (3, 1, 80, 0, False, 16)])
def test_qk_norm_rope_store(hip, twin, dtype, heads, kv_heads, head_dim, rotary, norm, page, pairing="neox",
                            per_head=False):
    tokens, pages = 9, 7
    width = (heads + 2 * kv_heads) * head_dim
    qkv = randn(tokens, width, dtype=dtype, seed=3)
    positions = torch.tensor([0, 1, 17, 127, 1023, 5, 6, 7, 300], dtype=torch.int32).to(DEV)
    table = rope_table(2048, rotary, 5e6) if rotary else torch.zeros(1, 1, device=DEV)
    qw = (1 + 0.1 * torch.randn(head_dim if per_head else heads * head_dim)).to(dtype).to(DEV) if norm else None
    kw = (1 + 0.1 * torch.randn(head_dim if per_head else kv_heads * head_dim)).to(dtype).to(DEV) if norm else None
    slots = torch.tensor([3 * page + 1, 0, page - 1, 5 * page, -1, 2 * page + 3, 2 * page + 4, 6 * page + page - 1, page],
                         dtype=torch.int32).to(DEV)
    cache_h = torch.zeros(pages, 2, kv_heads, page, head_dim, dtype=dtype, device=DEV)
    cache_t = cache_h.clone()
    a, b = qkv.clone(), qkv.clone()
    hip.qk_norm_rope_store(a, positions, table, qw, kw, 1e-6, heads, kv_heads, head_dim, rotary, cache_h, slots, page,
                           pairing=pairing, per_head_norm=per_head)
    twin.qk_norm_rope_store(b, positions, table, qw, kw, 1e-6, heads, kv_heads, head_dim, rotary, cache_t, slots, page,
                            pairing=pairing, per_head_norm=per_head)
    torch.testing.assert_close(a, b, **tol(dtype))
    if per_head and norm and not rotary:
        # every head by its own statistic: the library's norm over the last dim of [tokens, heads, head_dim]
        q_in = qkv[:, :heads * head_dim].view(tokens, heads, head_dim).float()
        ref = torch.nn.functional.rms_norm(q_in, (head_dim,), qw.float(), 1e-6)
        torch.testing.assert_close(a[:, :heads * head_dim].view(tokens, heads, head_dim).float(), ref, **tol(dtype))
    if pairing == "interleaved" and not norm and rotary:
        # neighbours as complex numbers: the rotation is a multiplication by exp(i * angle) (a library routine)
        q_in = qkv[:, :heads * head_dim].view(tokens, heads, head_dim)[..., :rotary].float()
        angle = torch.atan2(table[positions.long(), rotary // 2:], table[positions.long(), :rotary // 2])      # [T, R/2]
        turned = torch.view_as_real(torch.view_as_complex(q_in.reshape(tokens, heads, rotary // 2, 2).contiguous())
                                    * torch.polar(torch.ones_like(angle), angle)[:, None, :]).reshape(tokens, heads, rotary)
        torch.testing.assert_close(a[:, :heads * head_dim].view(tokens, heads, head_dim)[..., :rotary].float(), turned, **tol(dtype))
    torch.testing.assert_close(cache_h, cache_t, **tol(dtype))
    # v is never touched; without a norm the dims beyond the rotary part are bit-equal to the input
    assert torch.equal(a[:, (heads + kv_heads) * head_dim:], qkv[:, (heads + kv_heads) * head_dim:])
    if not norm:
        q_in = qkv[:, :heads * head_dim].view(tokens, heads, head_dim)
        assert torch.equal(a[:, :heads * head_dim].view(tokens, heads, head_dim)[..., rotary:], q_in[..., rotary:])
    # the cache holds exactly what the step's k and v rows hold
    kq = a[:, heads * head_dim:(heads + kv_heads) * head_dim].view(tokens, kv_heads, head_dim)
    for t in range(tokens):
        s = int(slots[t])
        if s >= 0:
            at = (torch.tensor([s // page]).to(DEV), torch.tensor([s % page]).to(DEV))
            assert torch.equal(layout.read_keys(cache_h, *at)[0], kq[t])
            assert torch.equal(layout.read_values(cache_h, *at)[0], a[t, (heads + kv_heads) * head_dim:].view(kv_heads, head_dim))


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("pairing", ["neox", "interleaved"])
@pytest.mark.parametrize("heads,kv_heads,head_dim,rotary,page", [(4, 2, 16, 8, 16), (6, 3, 32, 32, 16), (5, 5, 48, 0, 32),
                                                                 (48, 8, 128, 64, 64)])
def test_qk_norm_of_every_head_by_itself(hip, twin, dtype, pairing, heads, kv_heads, head_dim, rotary, page):
    """The other QK norm (one statistic per token and head, weights of one head's size), through the same checks
    as the flat one: against the twin, against the library's norm where nothing rotates, into the cache."""
    if pairing == "interleaved" and not rotary:
        pytest.skip("nothing turns")
    test_qk_norm_rope_store(hip, twin, dtype, heads, kv_heads, head_dim, rotary, True, page, pairing=pairing, per_head=True)
    # and it is not the flat norm: a row whose heads differ in size by a factor of a hundred
    qkv = randn(2, (heads + 2 * kv_heads) * head_dim, dtype=dtype, seed=8)
    qkv[:, :head_dim] *= 100
    positions, table = torch.zeros(2, dtype=torch.int32, device=DEV), torch.zeros(1, 1, device=DEV)
    w = torch.ones(head_dim, dtype=dtype, device=DEV)
    hip.qk_norm_rope_store(qkv, positions, table, w, w, 1e-6, heads, kv_heads, head_dim, 0, per_head_norm=True)
    per_head_rms = qkv[:, :heads * head_dim].view(2, heads, head_dim).float().square().mean(-1).sqrt()
    torch.testing.assert_close(per_head_rms, torch.ones_like(per_head_rms), rtol=2e-2, atol=2e-2)
    with pytest.raises(ValueError, match="weight shapes"):
        hip.qk_norm_rope_store(qkv, positions, table, torch.ones(heads * head_dim, dtype=dtype, device=DEV),
                               torch.ones(kv_heads * head_dim, dtype=dtype, device=DEV), 1e-6, heads, kv_heads, head_dim, 0,
                               per_head_norm=True)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("heads,kv_heads,head_dim,rotary,norm,page", [
    (4, 2, 16, 8, True, 16), (6, 3, 32, 32, False, 16), (48, 8, 128, 64, False, 64), (5, 5, 48, 16, True, 32)])
def test_rotation_of_neighbouring_dims(hip, twin, dtype, heads, kv_heads, head_dim, rotary, norm, page):
    """The other pairing of a rotary encoding: dims (2 j, 2 j + 1) turn together."""
    test_qk_norm_rope_store(hip, twin, dtype, heads, kv_heads, head_dim, rotary, norm, page, pairing="interleaved")


def make_paged(dtype, kv_heads, head_dim, page, lens, seed=0, extra_pages=3, window=0, q_lens=None):
    """Random k/v for requests of the given lengths scattered over shuffled pages, as the cache
    manager leaves them: with a window, the pages that lie wholly before the window of a request's
    first new token (``q_lens`` new tokens each) have been given back, so their table entries are -1;
    pages that no table names, the given-back ones among them, and the slots past a request's last
    key hold not-a-number.  A kernel that looks up a page it must not, or reads a slot it must not,
    shows it in its output (and faults under the emulated backend, whose tables end at a guard page)."""
    g = torch.Generator().manual_seed(seed)
    need = [(n + page - 1) // page for n in lens]
    total = sum(need) + extra_pages
    perm = torch.randperm(total, generator=g).tolist()
    cache = torch.randn(total, 2, kv_heads, page, head_dim, generator=g).to(dtype)
    table = torch.full((len(lens), max(need) + 1), -1, dtype=torch.int32)
    named = torch.zeros(total, dtype=torch.bool)
    for r, n in enumerate(need):
        first_live = 0
        if window and q_lens is not None:
            first_live = max(0, lens[r] - q_lens[r] - window + 1) // page       # cache/manager.py: _plan
        for j in range(n):
            p = perm.pop()
            if j >= first_live:
                table[r, j] = p
                named[p] = True
        last, used = int(table[r, n - 1]), lens[r] - (n - 1) * page
        if used < page:
            beyond = torch.arange(used, page)
            layout.keys_view(cache)[last, :, beyond] = float("nan")
            layout.values_view(cache)[last, :, beyond // 8, beyond % 8] = float("nan")
    cache[~named] = float("nan")
    return cache.to(DEV), table.to(DEV)


def make_meta(table, ctx_lens, q_lens):
    """What the batch builder hands to the attention kernels for items of these lengths."""
    import numpy as np
    token_row, positions = [], []
    for r, (n, ql) in enumerate(zip(ctx_lens, q_lens)):
        token_row += [r] * ql
        positions += list(range(n - ql, n))
    q_start = np.concatenate(([0], np.cumsum(q_lens)[:-1])).astype(np.int32)
    item_meta = torch.tensor(np.stack([q_start, np.asarray(q_lens), np.asarray(ctx_lens)]), dtype=torch.int32).to(DEV)
    return SimpleNamespace(block_table=table, token_row=torch.tensor(token_row, dtype=torch.int32).to(DEV),
                           positions=torch.tensor(positions, dtype=torch.int32).to(DEV), item_meta=item_meta,
                           item_q_len=np.asarray(q_lens), item_ctx_len=np.asarray(ctx_lens), work={})


def dense_attention(q, cache, table, row, pos, scale, window, page):
    """Reference through the library routine: gather the request's keys, call SDPA for one query."""
    first = max(0, pos - window + 1) if window else 0
    n = torch.arange(first, pos + 1, device=DEV)
    pages = table[row, n // page].long()
    k = layout.read_keys(cache, pages, n % page).float().transpose(0, 1)   # [Hkv, n, D]
    v = layout.read_values(cache, pages, n % page).float().transpose(0, 1)
    H, D = q.shape
    group = H // k.shape[0]
    k = k.repeat_interleave(group, 0)
    v = v.repeat_interleave(group, 0)
    o = torch.nn.functional.scaled_dot_product_attention(q.float()[:, None, :], k, v, scale=scale)
    return o[:, 0, :].reshape(-1)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("heads,kv_heads,head_dim,page,window", [
    (4, 2, 16, 16, 0), (6, 3, 32, 16, 0), (48, 8, 128, 64, 0), (12, 2, 64, 32, 0),
    (5, 1, 48, 16, 0), (8, 8, 80, 16, 0), (4, 2, 16, 16, 20), (6, 1, 128, 64, 100), (6, 3, 32, 8, 0),
    (12, 4, 96, 16, 0), (4, 1, 256, 32, 50), (14, 2, 160, 16, 0)])
def test_paged_attention_mixed_batch(hip, twin, dtype, heads, kv_heads, head_dim, page, window):
    # three requests: a whole prompt, a portion on top of a cached prefix, a single decoded token
    lens = [37, 150, 301]
    q_lens = [37, 23, 1]
    cache, table = make_paged(dtype, kv_heads, head_dim, page, lens, seed=heads, window=window, q_lens=q_lens)
    token_row, positions = [], []
    for r, (n, ql) in enumerate(zip(lens, q_lens)):
        token_row += [r] * ql
        positions += list(range(n - ql, n))
    T = len(token_row)
    meta = make_meta(table, lens, q_lens)
    qkv = randn(T, (heads + 2 * kv_heads) * head_dim, dtype=dtype, seed=9)
    q = qkv[:, :heads * head_dim].view(T, heads, head_dim)
    scale = head_dim ** -0.5
    out_h = torch.empty(T, heads * head_dim, dtype=dtype, device=DEV)
    out_t = torch.empty_like(out_h)
    hip.paged_attention(q, cache, meta, out_h, scale, window)
    twin.paged_attention(q, cache, meta, out_t, scale, window)
    torch.testing.assert_close(out_h, out_t, **tol(dtype))
    for t in (0, 36, 37, 59, 60):
        ref = dense_attention(q[t], cache, table, token_row[t], positions[t], scale, window, page)
        torch.testing.assert_close(out_h[t].float(), ref, **tol(dtype))


@pytest.mark.parametrize("dtype", DTYPES)
def test_paged_attention_finds_one_far_key(hip, dtype):
    """One key far back in a long context is made to dominate: the output must be its value."""
    heads, kv_heads, head_dim, page = 8, 2, 64, 16
    n = 1000
    cache, table = make_paged(dtype, kv_heads, head_dim, page, [n], seed=5)
    q = randn(1, heads, head_dim, dtype=dtype, seed=6)
    for target in (0, 15, 16, 513, 998, 999):
        c = cache.clone()
        pg, off = int(table[0, target // page]), target % page
        for h in range(heads):
            kvh = h // (heads // kv_heads)
        # key of the target = 40 * direction of the first query head of each group
        for kvh in range(kv_heads):
            qh = q[0, kvh * (heads // kv_heads)].float()
            layout.keys_view(c)[pg, kvh, off] = (qh / qh.norm() * 60).to(dtype).view(-1, 8)
        meta = make_meta(table, [n], [1])
        out = torch.empty(1, heads * head_dim, dtype=dtype, device=DEV)
        hip.paged_attention(q, c, meta, out, 1.0, 0)
        for kvh in range(kv_heads):
            head = kvh * (heads // kv_heads)
            got = out[0, head * head_dim:(head + 1) * head_dim].float()
            value = layout.values_view(c)[pg, kvh, off // 8, off % 8].float()
            torch.testing.assert_close(got, value, rtol=2e-2, atol=2e-2)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("tokens,experts,k", [(1, 256, 3072), (8, 256, 3072), (16, 7, 200), (13, 30, 1032), (40, 16, 64)])
def test_router_logits_are_float_products(hip, dtype, tokens, experts, k):
    """Few tokens take the small kernel (activations widened on the fly), more the library."""
    x = randn(tokens, k, dtype=dtype, seed=3)
    w = randn(experts, k, dtype=torch.float32, scale=k ** -0.5, seed=4)
    out = torch.empty(tokens, experts, dtype=torch.float32, device=DEV)
    hip.router_logits(x, w, out)
    ref = (x.double() @ w.double().T).float()
    torch.testing.assert_close(out, ref, rtol=1e-5, atol=1e-5)
    # a view with a row stride (the engine hands over slices of larger buffers)
    wide = randn(tokens, k + 8, dtype=dtype, seed=5)
    hip.router_logits(wide[:, :k], w, out)
    torch.testing.assert_close(out, (wide[:, :k].double() @ w.double().T).float(), rtol=1e-5, atol=1e-5)


def test_router_matches_library_topk(hip, twin):
    torch.manual_seed(27)
    for tokens, experts, k in [(4096, 256, 8), (33, 8, 2), (17, 16, 4), (5, 100, 7), (3, 1, 1), (9, 1000, 16)]:
        logits = (torch.randn(tokens, experts) * 3).to(DEV)
        bias = (torch.randn(experts) * 0.1).to(DEV)
        ids = torch.empty(tokens, k, dtype=torch.int32, device=DEV)
        w = torch.empty(tokens, k, device=DEV)
        hip.router_topk(logits, bias, k, ids, w)
        s = torch.sigmoid(logits)
        ref_ids = torch.topk(s + bias, k, dim=-1).indices
        assert torch.equal(ids.long().sort(-1).values, ref_ids.sort(-1).values)
        ref_w = s.gather(1, ids.long())
        ref_w = ref_w / ref_w.sum(-1, keepdim=True)
        torch.testing.assert_close(w, ref_w, rtol=1e-5, atol=1e-6)
        ids_t = torch.empty_like(ids); w_t = torch.empty_like(w)
        twin.router_topk(logits, bias, k, ids_t, w_t)
        assert torch.equal(ids, ids_t)


@pytest.mark.parametrize("tokens,experts,k", [(1, 256, 8), (8, 256, 8), (16, 256, 8), (5, 7, 3), (16, 1000, 16), (3, 1, 1)])
def test_router_with_grouping_in_one_launch(hip, tokens, experts, k):
    """Few tokens: routing and grouping in one launch give what the two launches give."""
    from sparseengine_amd.kernels.hip_ops import MoeWorkspace
    torch.manual_seed(tokens + experts)
    logits = (torch.randn(tokens, experts) * 3).to(DEV)
    bias = (torch.randn(experts) * 0.1).to(DEV)
    ids_a = torch.empty(tokens, k, dtype=torch.int32, device=DEV); w_a = torch.empty(tokens, k, device=DEV)
    ids_b = torch.empty_like(ids_a); w_b = torch.empty_like(w_a)
    ws_a = MoeWorkspace(tokens, k, experts, 128, 128, torch.bfloat16, DEV)
    ws_b = MoeWorkspace(tokens, k, experts, 128, 128, torch.bfloat16, DEV)
    hip.router_topk(logits, bias, k, ids_a, w_a)
    tiles_a = hip.moe_align(ids_a, experts, ws_a, 16)
    hip.router_topk(logits, bias, k, ids_b, w_b, workspace=ws_b)
    assert ws_b.grouped is not None and ws_b.grouped[5] == tiles_a
    assert torch.equal(ids_a, ids_b) and torch.equal(w_a, w_b)
    assert torch.equal(ws_a.counters, ws_b.counters)
    n_tiles, n_sorted = ws_a.counters.tolist()[:2]
    assert torch.equal(ws_a.tile_expert[:n_tiles], ws_b.tile_expert[:n_tiles])
    # the order inside an expert's run is free: compare the runs as sets
    sa, sb = ws_a.sorted[:n_sorted].view(n_tiles, 16), ws_b.sorted[:n_sorted].view(n_tiles, 16)
    assert torch.equal(sa.sort(-1).values, sb.sort(-1).values)
    # and the expert products consume it: same result as with a grouping of their own
    hidden, inter = 128, 128
    x = randn(tokens, hidden, dtype=torch.bfloat16, seed=1)
    w13 = randn(experts, 2 * inter, hidden, dtype=torch.bfloat16, scale=0.1, seed=2)
    w2 = randn(experts, hidden, inter, dtype=torch.bfloat16, scale=0.1, seed=3)
    out_a, out_b = torch.empty_like(x), torch.empty_like(x)
    hip.moe_experts(x, w13, w2, ids_a, w_a, out_a, ws_a)
    assert ws_b.grouped is not None
    hip.moe_experts(x, w13, w2, ids_b, w_b, out_b, ws_b)
    assert ws_b.grouped is None
    assert torch.equal(out_a, out_b)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("tokens,experts,k,hidden", [(1, 256, 8, 3072), (2, 256, 8, 3072), (3, 64, 6, 512), (8, 256, 8, 3072),
                                                      (16, 256, 8, 1024), (5, 7, 3, 200), (13, 1000, 16, 264), (3, 1, 1, 8)])
def test_whole_router(hip, dtype, tokens, experts, k, hidden):
    """``route`` gives what logits, routing and grouping give one by one, call after call on one workspace."""
    from sparseengine_amd.kernels.hip_ops import MoeWorkspace
    w = randn(experts, hidden, dtype=torch.float32, scale=3 * hidden ** -0.5, seed=40 + tokens)
    bias = randn(experts, dtype=torch.float32, scale=0.1, seed=41)
    ws_a = MoeWorkspace(16, k, experts, 128, 128, torch.bfloat16, DEV)
    ws_b = MoeWorkspace(16, k, experts, 128, 128, torch.bfloat16, DEV)
    for call in range(3):
        wide = randn(tokens, hidden + 8, dtype=dtype, seed=50 + call)
        x = wide[:, :hidden] if call == 1 else wide[:, :hidden].contiguous()     # also a view with a row stride
        logits_a = torch.empty(tokens, experts, dtype=torch.float32, device=DEV)
        logits_b = torch.full_like(logits_a, float("nan"))
        ids_a = torch.empty(tokens, k, dtype=torch.int32, device=DEV); w_a = torch.empty(tokens, k, device=DEV)
        ids_b = torch.full_like(ids_a, -1); w_b = torch.full_like(w_a, float("nan"))
        hip.router_logits(x, w, logits_a)
        hip.router_topk(logits_a, bias, k, ids_a, w_a)
        tiles_a = hip.moe_align(ids_a, experts, ws_a, 16)
        hip.route(x, w, bias, k, logits_b, ids_b, w_b, workspace=ws_b)
        assert ws_b.grouped is not None and ws_b.grouped[5] == tiles_a
        torch.testing.assert_close(logits_b, (x.double() @ w.double().T).float(), rtol=1e-5, atol=1e-5)
        assert torch.equal(logits_a, logits_b) and torch.equal(ids_a, ids_b) and torch.equal(w_a, w_b)
        assert torch.equal(ws_a.counters, ws_b.counters)
        n_tiles, n_sorted = ws_a.counters.tolist()[:2]
        assert torch.equal(ws_a.tile_expert[:n_tiles], ws_b.tile_expert[:n_tiles])
        sa, sb = ws_a.sorted[:n_sorted].view(n_tiles, 16), ws_b.sorted[:n_sorted].view(n_tiles, 16)
        assert torch.equal(sa.sort(-1).values, sb.sort(-1).values)


def test_router_ties_nonfinite_and_bias(hip, twin):
    # tie order and non-finite rows as in the reference's tests/test_minimax_m2_router.py:68-122
    logits = torch.zeros(4, 256).to(DEV)
    logits[1, :9] = 1
    logits[2, 120:129] = 1
    logits[3] = (torch.arange(256).to(DEV) // 8).float()
    bias = torch.zeros(256).to(DEV)
    ids = torch.empty(4, 8, dtype=torch.int32, device=DEV); w = torch.empty(4, 8, device=DEV)
    hip.router_topk(logits, bias, 8, ids, w)
    assert ids[0].tolist() == list(range(8))
    assert ids[1].tolist() == list(range(8))
    assert ids[2].tolist() == list(range(120, 128))
    s3 = torch.sigmoid(logits[3])   # saturates to 1.0 from index 136 on: the ties go to the lowest indices
    assert ids[3].tolist() == torch.nonzero(s3 == s3.max()).flatten()[:8].tolist()
    torch.testing.assert_close(w, torch.full_like(w, 0.125))
    logits = torch.zeros(6, 256).to(DEV)
    logits[0, 3] = float("nan"); logits[1, 7] = float("inf"); logits[2, 9] = -float("inf")
    logits[3] = 100; logits[4] = -100
    bias2 = bias.clone(); bias2[5] = float("nan")
    hip.router_topk(logits[:5], bias, 8, ids := torch.empty(5, 8, dtype=torch.int32, device=DEV),
                    w := torch.empty(5, 8, device=DEV))
    assert 3 in ids[0].tolist() and torch.isnan(w[0]).all()
    assert 7 in ids[1].tolist() and 9 not in ids[2].tolist()
    assert ids[3].tolist() == list(range(8)) and ids[4].tolist() == list(range(8))
    hip.router_topk(logits[5:], bias2, 8, ids6 := torch.empty(1, 8, dtype=torch.int32, device=DEV),
                    w6 := torch.empty(1, 8, device=DEV))
    assert ids6[0].tolist() == [5, 0, 1, 2, 3, 4, 6, 7]
    # a bias of +2 on experts 0..7 selects exactly them and leaves the weights unbiased
    logits = torch.linspace(-4, 4, 256)[None].to(DEV)
    bias3 = torch.zeros(256).to(DEV); bias3[:8] = 2
    hip.router_topk(logits, bias3, 8, ids6, w6)
    assert sorted(ids6[0].tolist()) == list(range(8))
    s = torch.sigmoid(logits[0, :8])
    torch.testing.assert_close(w6[0].sort().values, (s / s.sum()).sort().values)
    # softmax scoring, no renormalisation, scaling
    logits = torch.randn(7, 40).to(DEV)
    ids7 = torch.empty(7, 3, dtype=torch.int32, device=DEV); w7 = torch.empty(7, 3, device=DEV)
    hip.router_topk(logits, None, 3, ids7, w7, scoring="softmax", normalize=False, scaling=2.5)
    ref = torch.topk(torch.softmax(logits, -1), 3)
    assert torch.equal(ids7.long().sort(-1).values, ref.indices.sort(-1).values)
    torch.testing.assert_close(w7.sort(-1).values, (ref.values * 2.5).sort(-1).values)


def test_moe_align_groups_every_assignment_once(hip):
    from sparseengine_amd.kernels.hip_ops import MoeWorkspace
    for tokens, k, experts in [(1, 8, 256), (2048, 8, 256), (33, 2, 8), (100, 4, 16), (7, 1, 1)]:
        ids = torch.stack([torch.randperm(experts)[:k] for _ in range(tokens)]).to(torch.int32).to(DEV)
        ws = MoeWorkspace(tokens, k, experts, 16, 16, torch.float32, DEV)
        for rows in (16, 32, 64):
            ws.sorted.fill_(-7); ws.tile_expert.fill_(-7)
            hip.moe_align(ids, experts, ws, rows)
            n_tiles, n_sorted = ws.counters.tolist()[:2]
            assert n_sorted == n_tiles * rows
            sorted_ids = ws.sorted[:n_sorted].cpu()
            real = sorted_ids[sorted_ids < tokens * k]
            assert sorted(real.tolist()) == list(range(tokens * k))
            flat = ids.flatten().cpu()
            te = ws.tile_expert[:n_tiles].cpu()
            assert (te[1:] >= te[:-1]).all()
            for t in range(n_tiles):
                chunk = sorted_ids[t * rows:(t + 1) * rows]
                chunk = chunk[chunk < tokens * k]
                assert chunk.numel() > 0 and (flat[chunk.long()] == te[t]).all()


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("tokens,hidden,inter,experts,k", [
    (1, 64, 32, 8, 2), (45, 96, 48, 16, 4), (130, 200, 72, 5, 5), (9, 256, 128, 1, 1), (64, 384, 160, 32, 8),
    # sizes the matrix-core kernels take (hidden and width multiples of 128), tiles of 16, 32 and 64 rows
    (1, 256, 128, 8, 2), (3, 384, 256, 16, 4), (70, 256, 128, 4, 2), (200, 512, 384, 6, 3), (33, 3072, 1536, 16, 8),
    (2048, 256, 128, 64, 8),
    # hundreds of rows per expert: tiles of 128 rows x 256 weight rows
    (2048, 256, 128, 8, 8), (1000, 512, 384, 6, 3), (777, 768, 256, 3, 1)])
def test_moe_experts(hip, twin, dtype, tokens, hidden, inter, experts, k, activation="silu"):
    emulator_skips(tokens * k * hidden * inter, 1.2e9)
    from sparseengine_amd.kernels.hip_ops import MoeWorkspace
    x = randn(tokens, hidden, dtype=dtype, seed=11)
    w13 = randn(experts, 2 * inter, hidden, dtype=dtype, scale=hidden ** -0.5, seed=12)
    w2 = randn(experts, hidden, inter, dtype=dtype, scale=inter ** -0.5, seed=13)
    ids = torch.stack([torch.randperm(experts)[:k] for _ in range(tokens)]).to(torch.int32).to(DEV)
    weights = torch.rand(tokens, k).to(DEV)
    weights = weights / weights.sum(-1, keepdim=True)
    ws = MoeWorkspace(tokens, k, experts, hidden, inter, dtype, DEV)
    out_h = torch.empty_like(x); out_t = torch.empty_like(x)
    hip.moe_experts(x, w13, w2, ids, weights, out_h, ws, activation=activation)
    twin.moe_experts(x, w13, w2, ids, weights, out_t, activation=activation)
    torch.testing.assert_close(out_h, out_t, **tol(dtype))
    if dtype == torch.bfloat16 and hidden % 256 == 0 and inter % 128 == 0 and tokens <= 200:
        # every kernel and tile on a step that would not choose it (mostly padding): same result
        for kernel, rows in (("direct", 128), ("direct", 64), ("tall", 64), ("stream", 16), ("stream", 32), ("mid", 64),
                             ("mid", 96), ("auto", None)):
            out_w = torch.empty_like(x)
            hip.moe_experts(x, w13, w2, ids, weights, out_w, ws, kernel=kernel, tile_rows=rows, activation=activation)
            torch.testing.assert_close(out_w, out_t, **tol(dtype))
    if experts == 1:   # one expert, k = 1: a plain gated feed-forward through library routines
        xf = x.float()
        act = torch.nn.functional.silu if activation == "silu" else (lambda g: torch.nn.functional.gelu(g, approximate="tanh"))
        ref = (act(xf @ w13[0, :inter].float().T) * (xf @ w13[0, inter:].float().T)) @ w2[0].float().T
        torch.testing.assert_close(out_h.float(), ref, **tol(dtype))


@pytest.mark.parametrize("counts", [[1, 16, 17, 47, 48, 49, 64, 65, 96, 111, 112, 113, 128, 129, 270, 0],
                                    [128, 0, 0, 3], [200, 130, 80, 33, 2, 700]])
def test_wide_tiles_leave_out_row_blocks_of_padding(hip, twin, counts):
    """The wide expert kernel skips the row blocks of a tile that hold no row: experts with every
    number of rows around the edges of the 16-row blocks of a 128-row tile, one slot per token so that
    the counts are exact.  Against the twin, in both tile heights."""
    from sparseengine_amd.kernels.hip_ops import MoeWorkspace
    hidden, inter, experts, tokens = 256, 128, len(counts), sum(counts)
    emulator_skips(tokens * hidden * inter, 1.2e8)
    dtype = torch.bfloat16
    x = randn(tokens, hidden, dtype=dtype, seed=21)
    w13 = randn(experts, 2 * inter, hidden, dtype=dtype, scale=hidden ** -0.5, seed=22)
    w2 = randn(experts, hidden, inter, dtype=dtype, scale=inter ** -0.5, seed=23)
    order = torch.randperm(tokens, generator=torch.Generator().manual_seed(24))
    ids = torch.repeat_interleave(torch.arange(experts), torch.tensor(counts))[order].view(tokens, 1).to(torch.int32).to(DEV)
    weights = (0.5 + torch.rand(tokens, 1, generator=torch.Generator().manual_seed(25))).to(DEV)
    ws = MoeWorkspace(tokens, 1, experts, hidden, inter, dtype, DEV)
    out_t = torch.empty_like(x)
    twin.moe_experts(x, w13, w2, ids, weights, out_t)
    for kernel, rows in (("direct", 128), ("direct", 64), ("mid", 64), ("mid", 96)):
        out_h = torch.full_like(x, float("nan"))
        hip.moe_experts(x, w13, w2, ids, weights, out_h, ws, kernel=kernel, tile_rows=rows)
        torch.testing.assert_close(out_h, out_t, **tol(dtype))


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("tokens,hidden,inter,experts,k", [(45, 96, 48, 16, 4), (9, 256, 128, 1, 1), (70, 256, 128, 4, 2),
                                                      (300, 512, 384, 6, 3)])
def test_experts_with_the_other_activation(hip, twin, dtype, tokens, hidden, inter, experts, k):
    """gelu (tanh form) on the gate, in the general kernel and in every matrix-core kernel."""
    test_moe_experts(hip, twin, dtype, tokens, hidden, inter, experts, k, activation="gelu_tanh")
    x = randn(13, 2 * 72, dtype=dtype, seed=4)
    a = torch.empty(13, 72, dtype=dtype, device=DEV); b = torch.empty_like(a)
    hip.silu_mul(x, a, activation="gelu_tanh"); twin.silu_mul(x, b, activation="gelu_tanh")
    torch.testing.assert_close(a, b, **tol(dtype))
    torch.testing.assert_close(a.float(), torch.nn.functional.gelu(x[:, :72].float(), approximate="tanh") * x[:, 72:].float(), **tol(dtype))
    with pytest.raises(ValueError, match="relu"):
        hip.silu_mul(x, a, activation="relu")


@pytest.mark.parametrize("dtype", DTYPES)
def test_silu_mul(hip, twin, dtype):
    x = randn(13, 2 * 72, dtype=dtype, seed=4)
    a = torch.empty(13, 72, dtype=dtype, device=DEV); b = torch.empty_like(a)
    hip.silu_mul(x, a); twin.silu_mul(x, b)
    torch.testing.assert_close(a, b, **tol(dtype))
    torch.testing.assert_close(a.float(), torch.nn.functional.silu(x[:, :72].float()) * x[:, 72:].float(), **tol(dtype))


def test_sampling(hip, twin):
    torch.manual_seed(3)
    rows, vocab = 6, 1000
    logits = (torch.randn(rows, vocab) * 2).to(DEV)
    out = torch.empty(rows, dtype=torch.int32, device=DEV)
    # greedy, top_k = 1 and a tiny top_p all give the arg-max (reference tests/test_sampler.py:39-58)
    hip.sample(logits, None, None, None, None, out)
    assert torch.equal(out.long(), logits.argmax(-1))
    temp = torch.full((rows,), 0.7).to(DEV)
    seeds = torch.arange(rows, dtype=torch.int64).to(DEV) * 7919 + 1
    hip.sample(logits, temp, torch.ones(rows, dtype=torch.int32).to(DEV), None, seeds, out)
    assert torch.equal(out.long(), logits.argmax(-1))
    hip.sample(logits, temp, None, torch.full((rows,), 0.01).to(DEV), seeds, out)
    assert torch.equal(out.long(), logits.argmax(-1))
    # mixed rows against the twin: same noise, same choice
    temp = torch.tensor([0.0, 0.8, 1.0, 0.7, 1.3, 0.5]).to(DEV)
    top_k = torch.tensor([0, 0, 5, 0, 50, 3], dtype=torch.int32).to(DEV)
    top_p = torch.tensor([1.0, 1.0, 1.0, 0.6, 0.9, 0.5]).to(DEV)
    ref = torch.empty_like(out)
    hip.sample(logits, temp, top_k, top_p, seeds, out)
    twin.sample(logits, temp, top_k, top_p, seeds, ref)
    assert torch.equal(out, ref)
    # without filters the many-block path is taken: same noise, same choice as the one-block kernel
    big = (torch.randn(5, 20011) * 2).to(DEV)
    t5 = torch.tensor([0.0, 0.7, 1.0, 1.5, 0.3]).to(DEV)
    s5 = seeds[:5].contiguous()
    fast = torch.empty(5, dtype=torch.int32, device=DEV); slow = torch.empty_like(fast)
    hip.sample(big, t5, None, None, s5, fast)
    hip.sample(big, t5, torch.zeros(5, dtype=torch.int32).to(DEV), None, s5, slow)
    assert torch.equal(fast, slow) and int(fast[0]) == int(big[0].argmax())
    # filters over a vocabulary of several chunks, with many equal logits in some rows (whole groups of equal
    # values stay or go), a top_k beyond the vocabulary and a nucleus that is one token
    coarse = big.clone()
    coarse[2:] = (coarse[2:] * 2).round() / 2
    t5 = torch.tensor([0.0, 0.7, 1.0, 1.5, 0.3]).to(DEV)
    k5 = torch.tensor([3, 40, 1000, 0, 30000], dtype=torch.int32).to(DEV)
    p5 = torch.tensor([0.5, 0.9, 0.95, 0.3, 1e-4]).to(DEV)
    ref5 = torch.empty_like(fast)
    for rows_k, rows_p in ((k5, p5), (k5, None), (None, p5)):
        hip.sample(coarse, t5, rows_k, rows_p, s5, fast)
        twin.sample(coarse, t5, rows_k, rows_p, s5, ref5)
        assert torch.equal(fast, ref5), (fast.tolist(), ref5.tolist())
    assert int(fast[4]) == int(coarse[4].argmax())
    # a row's draw does not depend on the rest of the batch
    one = torch.empty(1, dtype=torch.int32, device=DEV)
    for r in range(rows):
        hip.sample(logits[r:r + 1], temp[r:r + 1], top_k[r:r + 1], top_p[r:r + 1], seeds[r:r + 1], one)
        assert int(one) == int(out[r])


@pytest.mark.parametrize("vocab,slope,draws", [(5000, 0.1, 128), (5000, 0.06, 256), (20011, 0.01, 8192)])
def test_sampling_keeps_exactly_the_tokens_of_the_filters(hip, vocab, slope, draws):
    """The kept set itself, to the single token: logits fall off evenly over tokens scattered through the
    vocabulary (several chunks), so that top_p = 0.5 keeps a few dozen of them, each likely enough to be drawn
    several times; the tokens drawn over many seeds are then exactly the set that float64 arithmetic keeps.
    The same for top_k."""
    emulator_skips(draws * vocab, 2e6)
    g = torch.Generator().manual_seed(11)
    order = torch.randperm(vocab, generator=g)
    ranked = 2000 if vocab > 10000 else 400
    row = torch.full((vocab,), -50.0)
    row[order[:ranked]] = -slope * torch.arange(ranked, dtype=torch.float32)
    logits = row[None].repeat(draws, 1).to(DEV)
    seeds = (torch.arange(draws, dtype=torch.int64) * 0x9E3779B1 + 99).to(DEV)
    out = torch.empty(draws, dtype=torch.int32, device=DEV)
    ones = torch.ones(draws).to(DEV)
    prob = torch.softmax(row.double(), 0)[order]            # in descending order
    before = torch.cumsum(prob, 0) - prob
    nucleus = int((before <= 0.5).sum())
    assert 6 <= nucleus <= 80
    hip.sample(logits, ones, None, torch.full((draws,), 0.5).to(DEV), seeds, out)
    assert set(out.tolist()) == set(order[:nucleus].tolist())
    k = nucleus - 3
    hip.sample(logits, ones, torch.full((draws,), k, dtype=torch.int32).to(DEV), None, seeds, out)
    assert set(out.tolist()) == set(order[:k].tolist())
    # both: the nucleus is taken among the survivors of top-k
    inside = prob[:k] / prob[:k].sum()
    both = int(((torch.cumsum(inside, 0) - inside) <= 0.5).sum())
    hip.sample(logits, ones, torch.full((draws,), k, dtype=torch.int32).to(DEV), torch.full((draws,), 0.5).to(DEV), seeds, out)
    assert set(out.tolist()) == set(order[:both].tolist()) and both < nucleus


def test_sampling_distribution(hip):
    emulator_skips(float("inf"))
    # 32768 draws at temperature 0.7 stay within 0.015 of softmax(l / 0.7) (reference tests/test_sampler.py:351-367)
    torch.manual_seed(5)
    vocab, draws = 12, 32768
    row = torch.randn(vocab) * 1.5
    logits = row[None].repeat(draws, 1).to(DEV)
    temp = torch.full((draws,), 0.7).to(DEV)
    seeds = (torch.arange(draws, dtype=torch.int64) * 0x9E3779B1 + 12345).to(DEV)
    out = torch.empty(draws, dtype=torch.int32, device=DEV)
    hip.sample(logits, temp, None, None, seeds, out)
    freq = torch.bincount(out.long().cpu(), minlength=vocab).float() / draws
    assert (freq - torch.softmax(row / 0.7, -1)).abs().max() < 0.015
    # top-k then top-p: the nucleus is taken over the survivors of top-k (tests/test_sampler.py:332-349)
    logits = torch.tensor([[3.0, 2.0, 1.0, 0.0, -1.0]]).repeat(draws, 1).to(DEV)
    hip.sample(logits, torch.ones(draws).to(DEV), torch.full((draws,), 3, dtype=torch.int32).to(DEV),
               torch.full((draws,), 0.7).to(DEV), seeds, out)
    freq = torch.bincount(out.long().cpu(), minlength=5).float() / draws
    p3 = torch.softmax(torch.tensor([3.0, 2.0, 1.0]), -1)   # 0.665, 0.245, 0.090: nucleus 0.7 keeps two
    expect = torch.tensor([p3[0], p3[1], 0, 0, 0]) / (p3[0] + p3[1])
    assert (freq - expect).abs().max() < 0.015


@pytest.mark.parametrize("batch,ctx,q_len", [(1, 2049, 1), (3, 700, 1), (64, 300, 1), (2, 1500, 130), (1, 4100, 1)])
def test_paged_attention_split_keys(hip, twin, batch, ctx, q_len):
    """Few rows and long contexts: the key ranges are split over many wavefronts and merged."""
    emulator_skips(batch * ctx * q_len * 48 * 128, 6e8)
    heads, kv_heads, head_dim, page = 48, 8, 128, 64
    dtype = torch.bfloat16
    lens = [ctx - 3 * i for i in range(batch)]
    cache, table = make_paged(dtype, kv_heads, head_dim, page, lens, seed=batch)
    meta = make_meta(table, lens, [q_len] * batch)
    T = batch * q_len
    q = randn(T, heads, head_dim, dtype=dtype, seed=2)
    out_h = torch.empty(T, heads * head_dim, dtype=dtype, device=DEV)
    hip.paged_attention(q, cache, meta, out_h, head_dim ** -0.5, 0)
    assert meta.work[(heads // kv_heads, 0)].num_tasks > 0 or batch * q_len >= 64, "expected split units"
    for t in sorted({0, T // 2, T - 1}):
        row, pos = int(meta.token_row[t]), int(meta.positions[t])
        ref = dense_attention(q[t], cache, table, row, pos, head_dim ** -0.5, 0, page)
        torch.testing.assert_close(out_h[t].float(), ref, rtol=1.6e-2, atol=1.6e-2)


@pytest.mark.parametrize("heads,kv_heads,head_dim,page,window,lens,q_lens", [
    (48, 8, 128, 64, 0, [900, 1300, 301], [900, 411, 1]),        # a whole prompt, a portion on a prefix, a decoded token
    (32, 16, 96, 16, 0, [800, 500], [800, 300]),
    (16, 8, 64, 32, 70, [1500, 900], [1500, 600]),               # window shorter than the portions
    (8, 8, 32, 8, 0, [4200], [4200]),
    (48, 8, 128, 64, 0, [2048 + 17], [2048 + 17]),
    (12, 2, 128, 16, 300, [5000, 3000], [4100, 2001]),
    (16, 8, 64, 24, 0, [1500, 900], [1500, 700]),                # pages that are no multiple of a step of 32 keys
    (24, 8, 96, 40, 333, [1500, 100, 90], [1400, 100, 1]),
    (48, 8, 128, 64, 0, [9000, 2100, 77], [1, 2100, 5]),          # a decoded token with a long context beside a prompt
    (48, 8, 128, 64, 0, [20000], [100]),                          # few blocks, long context: their keys are split
    (12, 2, 64, 16, 900, [6000, 5000], [300, 77]),                # the same with a window
    (8, 8, 32, 8, 0, [17000], [4100]),                           # more pages than the kernel keeps ids of at once
    (4, 2, 32, 16, 0, [2300], [40]),                             # one row block per kv head: three ranges of keys
    (12, 2, 64, 16, 1500, [2600, 2500], [30, 77])])              # the same within a window
def test_paged_attention_prompt_portions(hip, twin, heads, kv_heads, head_dim, page, window, lens, q_lens):
    """Steps with many rows: blocks share each step's keys and values through shared memory."""
    emulator_skips(sum(q * (min(n, window + q) if window else n) for q, n in zip(q_lens, lens)) * heads * head_dim, 2.5e9)
    dtype = torch.bfloat16
    # pages the window has passed are given back (-1 in the table); whatever no request holds is not-a-number
    cache, table = make_paged(dtype, kv_heads, head_dim, page, lens, seed=heads + head_dim, window=window, q_lens=q_lens)
    meta = make_meta(table, lens, q_lens)
    T = sum(q_lens)
    q = randn(T, heads, head_dim, dtype=dtype, seed=3)
    scale = head_dim ** -0.5
    out_h = torch.empty(T, heads * head_dim, dtype=dtype, device=DEV)
    out_t = torch.empty_like(out_h)
    hip.paged_attention(q, cache, meta, out_h, scale, window)
    work = meta.work[(heads // kv_heads, window)]
    assert work.num_block_units > 0, "expected the shared-memory kernel"
    few_rows = [-(-n * (heads // kv_heads) // 16) < 4 for n in q_lens]
    assert (work.num_units > 0) == any(few_rows), "few rows: one wavefront per tile"
    twin.paged_attention(q, cache, meta, out_t, scale, window)
    torch.testing.assert_close(out_h, out_t, **tol(dtype))
    for t in sorted({0, 1, 15, 16, q_lens[0] - 1, min(q_lens[0], T - 1), T // 2, T - 1}):
        row, pos = int(meta.token_row[t]), int(meta.positions[t])
        ref = dense_attention(q[t], cache, table, row, pos, scale, window, page)
        torch.testing.assert_close(out_h[t].float(), ref, **tol(dtype))


@pytest.mark.parametrize("heads,kv_heads,head_dim,page,window,ctx,q_len", [
    (8, 2, 64, 16, 0, 700, 300), (6, 1, 128, 64, 0, 1500, 200), (8, 4, 32, 8, 500, 900, 260)])
def test_prompt_attention_with_maxima_that_keep_rising(hip, twin, heads, kv_heads, head_dim, page, window, ctx, q_len):
    """The shared-memory kernel runs the steps that need no mask in a loop of its own and leaves it when
    a step would raise a row's maximum beyond its slack.  Here the maxima rise again and again deep
    inside that range: every query has a large component along one direction, and keys every 97
    positions lie along it, each longer than the one before (scores about 6, 12, 18, ... above the
    rest), so a row's answer is nearly the value of the last such key it can see."""
    emulator_skips(q_len * ctx * heads * head_dim, 2.5e9)
    dtype = torch.bfloat16
    cache, table = make_paged(dtype, kv_heads, head_dim, page, [ctx], seed=7, window=window, q_lens=[q_len])
    direction = torch.ones(head_dim) / head_dim ** 0.5
    marks = list(range(40, ctx, 97))
    for i, pos in enumerate(marks):
        entry = int(table[0, pos // page])
        if entry >= 0:
            key = (direction * (i + 1) * 6.0 * head_dim ** 0.5 / 8.0).to(dtype).to(DEV)
            layout.write_keys(cache, torch.tensor([entry]).to(DEV), torch.tensor([pos % page]).to(DEV),
                              key.expand(1, kv_heads, head_dim).contiguous())
    meta = make_meta(table, [ctx], [q_len])
    q = (randn(q_len, heads, head_dim, dtype=torch.float32, seed=9) + 8.0 * direction.to(DEV)).to(dtype)
    scale = head_dim ** -0.5
    out_h = torch.empty(q_len, heads * head_dim, dtype=dtype, device=DEV)
    out_t = torch.empty_like(out_h)
    hip.paged_attention(q, cache, meta, out_h, scale, window)
    assert meta.work[(heads // kv_heads, window)].num_block_units > 0, "expected the shared-memory kernel"
    twin.paged_attention(q, cache, meta, out_t, scale, window)
    torch.testing.assert_close(out_h, out_t, **tol(dtype))
    for t in (0, q_len // 2, q_len - 1):
        ref = dense_attention(q[t], cache, table, 0, ctx - q_len + t, scale, window, page)
        torch.testing.assert_close(out_h[t].float(), ref, **tol(dtype))
        seen = [m for m in marks if m <= ctx - q_len + t]
        weight = torch.softmax(torch.stack([(q[t, 0].float() * layout.read_keys(
            cache, torch.tensor([int(table[0, m // page])]).to(DEV), torch.tensor([m % page]).to(DEV))[0, 0].float()).sum() * scale
            for m in seen[-2:]]), 0)
        assert weight[-1] > 0.9, "the last marked key must dominate, or the test shows nothing"


@pytest.mark.parametrize("heads,kv_heads,head_dim,page,window,ctx,q_len", [
    (4, 2, 16, 16, 20, 150, 1), (4, 2, 16, 16, 20, 150, 60),           # the general kernel
    (6, 1, 128, 64, 100, 301, 1), (12, 2, 64, 8, 33, 500, 3),          # one wavefront per tile
    (16, 8, 64, 32, 70, 600, 300), (12, 4, 96, 24, 50, 400, 200)])     # blocks; pages that are no multiple of 32 keys
def test_attention_at_the_windows_edge(hip, heads, kv_heads, head_dim, page, window, ctx, q_len):
    """One key is made to dominate every query (all queries have a large component along one direction, the key
    lies along it, its score about 30 above the rest).  For the row whose window begins with that key the answer
    is the key's value; when the key lies one place further back, just outside that row's window, the row must
    not see it at all.  With random keys alone one key more or less moves the answer by less than the bound."""
    dtype = torch.bfloat16 if head_dim >= 32 else torch.float32
    cache0, table = make_paged(dtype, kv_heads, head_dim, page, [ctx], seed=3, window=window, q_lens=[q_len])
    direction = torch.ones(head_dim) / head_dim ** 0.5
    meta = make_meta(table, [ctx], [q_len])
    q = (randn(q_len, heads, head_dim, dtype=torch.float32, seed=4) + 8.0 * direction.to(DEV)).to(dtype)
    scale = head_dim ** -0.5
    t = q_len // 2
    pos = ctx - q_len + t
    for outside in (0, 1):
        key_pos = pos - window + 1 - outside
        entry = int(table[0, key_pos // page])
        assert entry >= 0, "the marked key lies in a page the request still holds"
        cache = cache0.clone()
        where = (torch.tensor([entry]).to(DEV), torch.tensor([key_pos % page]).to(DEV))
        layout.write_keys(cache, *where, (direction * 30.0 * head_dim ** 0.5 / 8.0).to(dtype).to(DEV).expand(1, kv_heads, head_dim).contiguous())
        out = torch.empty(q_len, heads * head_dim, dtype=dtype, device=DEV)
        hip.paged_attention(q, cache, meta, out, scale, window)
        got = out[t].float().reshape(heads, head_dim)
        value = layout.read_values(cache, *where)[0].float().repeat_interleave(heads // kv_heads, 0)
        ref = dense_attention(q[t], cache, table, 0, pos, scale, window, page).reshape(heads, head_dim)
        torch.testing.assert_close(got, ref, **tol(dtype))
        if outside:
            assert float((got - value).abs().max()) > 0.5, "a key outside the window has been seen"
        else:
            torch.testing.assert_close(got, value, rtol=2e-2, atol=2e-2)
        if t + 1 < q_len:       # the next row's window has passed the key in both cases
            after = dense_attention(q[t + 1], cache, table, 0, pos + 1, scale, window, page)
            torch.testing.assert_close(out[t + 1].float(), after, **tol(dtype))


def test_prompt_attention_repeats_bit_for_bit(hip):
    """The same step twice: the same bits (no atomics, no order that depends on timing; a wait that is too
    weak for the loads into shared memory would show as a difference now and then)."""
    emulator_skips(1e12)
    heads, kv_heads, head_dim, page = 48, 8, 128, 64
    lens, q_lens = [6000, 2500], [1500, 2500]
    cache, table = make_paged(torch.bfloat16, kv_heads, head_dim, page, lens, seed=5)
    meta = make_meta(table, lens, q_lens)
    q = randn(sum(q_lens), heads, head_dim, dtype=torch.bfloat16, seed=6)
    outs = []
    for _ in range(6):
        out = torch.full((sum(q_lens), heads * head_dim), float("nan"), dtype=torch.bfloat16, device=DEV)
        hip.paged_attention(q, cache, meta, out, head_dim ** -0.5, 0)
        outs.append(out)
    assert not torch.isnan(outs[0].float()).any()
    for out in outs[1:]:
        assert torch.equal(out, outs[0])


@pytest.mark.parametrize("rows,n,k", [(1, 8192, 3072), (8, 3072, 6144), (16, 256, 128), (17, 48, 256), (33, 1024, 384),
                                      (64, 200064, 3072), (5, 50, 128), (3, 64, 96),
                                      (7, 64, 768), (16, 48, 1536), (2, 32, 3072), (20, 64, 768)])   # stages of six steps, K over 4, 8, 16 wavefronts
def test_skinny_linear(hip, rows, n, k):
    """Few rows against a large matrix: the streaming kernel where its sizes fit, the library otherwise."""
    emulator_skips(rows * n * k, 4e8)
    x = randn(rows, k, dtype=torch.bfloat16, seed=1)
    w = randn(n, k, dtype=torch.bfloat16, scale=k ** -0.5, seed=2)
    out = torch.empty(rows, n, dtype=torch.bfloat16, device=DEV)
    hip.linear(x, w, out)
    ref = x.float() @ w.float().T
    torch.testing.assert_close(out.float(), ref, rtol=1.6e-2, atol=1.6e-2)
    # the same product on a tiled copy of the matrix: every dot product runs in the same order of k, so up
    # to the row count that both layouts leave to the streaming kernel the results are the same bits
    prepared = hip.prepare_dense_weight(w)
    if k % 128 or n % 16:
        assert prepared is None
        return
    assert prepared.shape == w.shape and not torch.equal(prepared, w)
    tiled_out = torch.full_like(out, float("nan"))
    hip.linear(x, w, tiled_out, prepared=prepared)
    torch.testing.assert_close(tiled_out.float(), ref, rtol=1.6e-2, atol=1.6e-2)
    if rows <= hip.SKINNY_ROWS:
        assert torch.equal(tiled_out, out)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("tokens,slots,hidden", [(1, 8, 3072), (5, 2, 256), (33, 8, 768), (7, 3, 200), (4, 11, 512), (3, 4, 20)])
def test_norm_adds_up_slots_as_it_reads(hip, dtype, tokens, slots, hidden):
    """``rms_norm(slots=k)`` is the slot sum followed by the norm, bit for bit: with a residual (which
    it replaces by the sum), without one, and for chosen rows; in sizes the fused kernel takes and in
    sizes that fall back to the two kernels."""
    from sparseengine_amd.kernels.hip_ops import _fn, _ptr, _code, _stream
    y = randn(tokens * slots, hidden, dtype=dtype, seed=60)
    w = randn(hidden, dtype=dtype, seed=61)
    res = randn(tokens, hidden, dtype=dtype, seed=62)
    summed = torch.empty(tokens, hidden, dtype=dtype, device=DEV)
    assert _fn.get("moe", "se_moe_sum")(_ptr(y), _ptr(summed), tokens, slots, hidden, _code(dtype), _stream()) == 0
    ref_sum = y.view(tokens, slots, hidden).float()
    acc = torch.zeros(tokens, hidden, device=DEV)
    for k in range(slots):
        acc += ref_sum[:, k]
    assert torch.equal(summed, acc.to(dtype))
    # with a residual
    res_a, res_b = res.clone(), res.clone()
    out_a = torch.empty_like(summed); out_b = torch.empty_like(summed)
    hip.rms_norm(summed, w, 1e-5, out_a, residual=res_a)
    hip.rms_norm(y, w, 1e-5, out_b, residual=res_b, slots=slots)
    assert torch.equal(out_a, out_b) and torch.equal(res_a, res_b)
    # without
    hip.rms_norm(summed, w, 1e-5, out_a)
    hip.rms_norm(y, w, 1e-5, out_b, slots=slots)
    assert torch.equal(out_a, out_b)
    # chosen rows: the residual is read, not written
    rows = torch.tensor([tokens - 1, 0, tokens // 2], dtype=torch.int32, device=DEV)
    pick_a = torch.empty(3, hidden, dtype=dtype, device=DEV); pick_b = torch.empty_like(pick_a)
    res_c = res.clone()
    hip.rms_norm(summed, w, 1e-5, pick_a, residual=res, rows=rows)
    hip.rms_norm(y, w, 1e-5, pick_b, residual=res_c, rows=rows, slots=slots)
    assert torch.equal(pick_a, pick_b) and torch.equal(res, res_c)


def test_rounding_to_bfloat16_is_to_nearest_even(hip):
    """The kernels round float results to bfloat16 with the chip's conversion instruction: it has to
    give what the tensor library gives, ties (to even), overflow to infinity and infinities included.
    Products of two bfloat16 numbers are exact in float and have up to 16 significant bits, so a
    product with one non-zero term shows the rounding of the result alone."""
    g = torch.Generator().manual_seed(9)
    rows, n, k = 16, 512, 128
    a = torch.randn(rows, generator=g).bfloat16()
    b = torch.randn(n, generator=g).bfloat16()
    # ties: (1 + 2^-7) * (1 + 2^-1) = 1.5 + 2^-7 + 2^-8 lies halfway between two bfloat16 numbers, and so
    # do their neighbours; huge products overflow; an infinite factor stays infinite
    a[:6] = torch.tensor([1 + 2 ** -7, 1 + 3 * 2 ** -7, -(1 + 2 ** -7), 3e38, float("inf"), 2 ** -120]).bfloat16()
    b[:6] = torch.tensor([1.5, 1.5, 1.5, 3.0, 1.0, 2 ** -20]).bfloat16()
    x = torch.zeros(rows, k, dtype=torch.bfloat16); x[:, 0] = a
    w = torch.zeros(n, k, dtype=torch.bfloat16); w[:, 0] = b
    out = torch.empty(rows, n, dtype=torch.bfloat16, device=DEV)
    hip.linear(x.to(DEV), w.to(DEV), out)
    ref = (a.float()[:, None] * b.float()[None, :]).bfloat16()
    finite = torch.isfinite(ref.float())
    assert torch.equal(out.cpu()[finite].view(torch.int16), ref[finite].view(torch.int16))
    assert torch.equal(torch.isinf(out.cpu().float()), torch.isinf(ref.float()))
    assert torch.equal(torch.isnan(out.cpu().float()), torch.isnan(ref.float()))      # inf * 0 terms


@pytest.mark.parametrize("dtype", DTYPES)
def test_cache_pages_beyond_four_gigabytes(hip, twin, dtype):
    """A layer's cache tensor larger than 2^32 bytes and 2^31 elements: the write and both
    attention kernels must address its last pages with 64-bit offsets (a 32-bit offset would wrap
    into the first pages, which stay zero here)."""
    emulator_skips(float("inf"))
    heads, kv_heads, head_dim, page, rotary = 48, 8, 128, 64, 64
    pages = 17000
    assert pages * 2 * kv_heads * page * head_dim > 2 ** 31
    cache = torch.zeros(pages, 2, kv_heads, page, head_dim, dtype=dtype, device=DEV)
    lens, q_lens = [700, 130], [200, 1]
    need = [-(-n // page) for n in lens]
    ids = [list(range(16990, 16990 - need[0], -1)), list(range(16900, 16900 + need[1]))]
    table = torch.full((2, max(need) + 1), -1, dtype=torch.int32)
    for r, row in enumerate(ids):
        table[r, :len(row)] = torch.tensor(row, dtype=torch.int32)
    table = table.to(DEV)
    T = sum(lens)
    width = (heads + 2 * kv_heads) * head_dim
    qkv = randn(T, width, dtype=dtype, seed=11)
    positions = torch.cat([torch.arange(n) for n in lens]).to(torch.int32).to(DEV)
    slots = torch.cat([torch.tensor([ids[r][p // page] * page + p % page for p in range(n)]) for r, n in enumerate(lens)])
    used = sorted(set(sum(ids, [])))
    remap = {p: i for i, p in enumerate(used)}
    small_slots = torch.tensor([remap[int(s) // page] * page + int(s) % page for s in slots], dtype=torch.int32).to(DEV)
    slots = slots.to(torch.int32).to(DEV)
    cos_sin = rope_table(2048, rotary, 5e6)
    qw = (1 + 0.1 * torch.randn(heads * head_dim)).to(dtype).to(DEV)
    kw = (1 + 0.1 * torch.randn(kv_heads * head_dim)).to(dtype).to(DEV)
    small = torch.zeros(len(used), 2, kv_heads, page, head_dim, dtype=dtype, device=DEV)
    a, b = qkv.clone(), qkv.clone()
    hip.qk_norm_rope_store(a, positions, cos_sin, qw, kw, 1e-6, heads, kv_heads, head_dim, rotary, cache, slots, page)
    twin.qk_norm_rope_store(b, positions, cos_sin, qw, kw, 1e-6, heads, kv_heads, head_dim, rotary, small, small_slots, page)
    torch.testing.assert_close(cache[torch.tensor(used).to(DEV)], small, **tol(dtype))
    assert float(cache[:16384].abs().max()) == 0.0                 # nothing wrapped into the low pages
    # attention over these pages: a prompt portion (blocks of tiles in bfloat16) and a decoded token
    rows = torch.cat([torch.arange(lens[0] - q_lens[0], lens[0]), torch.tensor([T - 1])]).to(DEV)
    q = a[rows, :heads * head_dim].reshape(-1, heads, head_dim).contiguous()
    meta = make_meta(table, lens, q_lens)
    out = torch.empty(q.shape[0], heads * head_dim, dtype=dtype, device=DEV)
    hip.paged_attention(q, cache, meta, out, head_dim ** -0.5, 0)
    for t in (0, 77, 199, 200):
        row, pos = int(meta.token_row[t]), int(meta.positions[t])
        ref = dense_attention(q[t], cache, table, row, pos, head_dim ** -0.5, 0, page)
        torch.testing.assert_close(out[t].float(), ref, rtol=1.6e-2, atol=1.6e-2)
    del cache
    if DEV == "cuda":
        torch.cuda.empty_cache()


@pytest.mark.parametrize("tokens", [3, 40, 600])
def test_expert_weights_beyond_two_to_the_31_elements(hip, twin, tokens):
    """MiniMax-M2's expert tables hold 2.4e9 and 1.2e9 elements; the last experts lie beyond a
    32-bit element offset (and, in bytes, beyond 2^32).  Only those are chosen here, in the
    streaming, the tall and the wide kernel."""
    emulator_skips(float("inf"))
    from sparseengine_amd.kernels.hip_ops import MoeWorkspace
    dtype, experts, hidden, inter, k = torch.bfloat16, 256, 3072, 1536, 2
    assert (experts - 3) * 2 * inter * hidden > 2 ** 31
    w13 = torch.zeros(experts, 2 * inter, hidden, dtype=dtype, device=DEV)
    w2 = torch.zeros(experts, hidden, inter, dtype=dtype, device=DEV)
    g = torch.Generator(device=DEV).manual_seed(5)
    for e in (experts - 3, experts - 2, experts - 1):
        w13[e] = (torch.randn(2 * inter, hidden, generator=g, device=DEV) * hidden ** -0.5).to(dtype)
        w2[e] = (torch.randn(hidden, inter, generator=g, device=DEV) * inter ** -0.5).to(dtype)
    x = randn(tokens, hidden, dtype=dtype, seed=21)
    ids = torch.stack([experts - 3 + torch.randperm(3)[:k] for _ in range(tokens)]).to(torch.int32).to(DEV)
    weights = torch.rand(tokens, k).to(DEV)
    weights = weights / weights.sum(-1, keepdim=True)
    ws = MoeWorkspace(tokens, k, experts, hidden, inter, dtype, DEV)
    out_h = torch.empty_like(x)
    hip.moe_experts(x, w13, w2, ids, weights, out_h, ws)
    # the twin on the three used experts alone
    out_t = torch.empty_like(x)
    twin.moe_experts(x, w13[experts - 3:].clone(), w2[experts - 3:].clone(), ids - (experts - 3), weights, out_t)
    assert float(out_t.abs().max()) > 0.1
    torch.testing.assert_close(out_h, out_t, **tol(dtype))
    del w13, w2
    if DEV == "cuda":
        torch.cuda.empty_cache()


def test_expert_tables_arranged_in_place_are_the_tiled_copy(hip, twin):
    """What the model does once (``arrange_expert_weights``, in place) and what a call with row-major
    tables does on the fly (``tile_expert_weights``) are the same layout, element for element; a call
    on arranged tables gives the twin's result."""
    from sparseengine_amd.kernels.hip_ops import MoeWorkspace
    dtype, tokens, hidden, inter, experts, k = torch.bfloat16, 37, 256, 128, 19, 3
    w13 = randn(experts, 2 * inter, hidden, dtype=dtype, scale=hidden ** -0.5, seed=1)
    w2 = randn(experts, hidden, inter, dtype=dtype, scale=inter ** -0.5, seed=2)
    # the layout, spelled out: element (n, k) of an expert lies at tile (n // 16, k // 32), place [(k % 32) // 8][n % 16][k % 8]
    tiled = hip.tile_expert_weights(w13)
    e, n, kk = 5, 37 + 16 * 3, 100
    tile = (n // 16) * (hidden // 32) + kk // 32
    place = tile * 512 + ((kk % 32) // 8 * 16 + n % 16) * 8 + kk % 8
    assert tiled[e].reshape(-1)[place] == w13[e, n, kk]
    a13, a2 = w13.clone(), w2.clone()
    assert hip.arrange_expert_weights(a13, a2) is True
    assert torch.equal(a13, tiled) and torch.equal(a2, hip.tile_expert_weights(w2))
    assert hip.arrange_expert_weights(w13.float(), w2.float()) is False          # float tables stay in rows
    odd = randn(2, 2 * 72, 200, dtype=dtype, seed=3)
    assert hip.arrange_expert_weights(odd, randn(2, 200, 72, dtype=dtype, seed=4)) is False   # sizes of the general kernel
    x = randn(tokens, hidden, dtype=dtype, seed=11)
    ids = torch.stack([torch.randperm(experts)[:k] for _ in range(tokens)]).to(torch.int32).to(DEV)
    weights = torch.rand(tokens, k).to(DEV)
    ws = MoeWorkspace(tokens, k, experts, hidden, inter, dtype, DEV)
    out_h, out_t = torch.empty_like(x), torch.empty_like(x)
    hip.moe_experts(x, a13, a2, ids, weights, out_h, ws, tiled=True)
    twin.moe_experts(x, w13, w2, ids, weights, out_t)
    torch.testing.assert_close(out_h, out_t, **tol(dtype))


def test_attention_on_random_shapes(hip):
    """Seeded random shapes (heads and groups, head sizes up to 256, page sizes that do not divide 32,
    windows, items from one decoded token to a long prompt) through the matrix-core kernels, each
    checked at a few rows against the library routine on the gathered keys."""
    import random
    rng = random.Random(3)
    dtype = torch.bfloat16
    for case in range(24):
        kv_heads = rng.choice([1, 2, 3, 8])
        heads = kv_heads * rng.choice([1, 2, 4, 6, 7])
        head_dim = rng.choice([32, 64, 96, 128, 160, 256])
        page = rng.choice([8, 16, 24, 40, 64])
        window = rng.choice([0, 0, 0, 17, 100, 333])
        lens, q_lens = [], []
        for _ in range(rng.randint(1, 5)):
            n = rng.choice([1, 2, 31, 32, 33, 64, 100, 255, 256, 500, 1000, 2500])
            lens.append(n)
            q_lens.append(max(1, min(n, rng.choice([1, 1, 2, 16, 65, n]))))
        cache, table = make_paged(dtype, kv_heads, head_dim, page, lens, seed=case, window=window, q_lens=q_lens)
        meta = make_meta(table, lens, q_lens)
        T = sum(q_lens)
        q = randn(T, heads, head_dim, dtype=dtype, seed=case + 1)
        out = torch.full((T, heads * head_dim), float("nan"), dtype=dtype, device=DEV)
        scale = head_dim ** -0.5
        hip.paged_attention(q, cache, meta, out, scale, window)
        what = f"case {case}: heads {heads}/{kv_heads}, head_dim {head_dim}, page {page}, window {window}, lens {lens}, new {q_lens}"
        assert torch.isfinite(out.float()).all(), what
        for t in sorted({0, T // 3, T // 2, T - 1}):
            row, pos = int(meta.token_row[t]), int(meta.positions[t])
            ref = dense_attention(q[t], cache, table, row, pos, scale, window, page)
            torch.testing.assert_close(out[t].float(), ref, rtol=1.6e-2, atol=1.6e-2, msg=lambda m: f"{what}, token {t}: {m}")


def test_experts_on_random_shapes_and_lumpy_routing(hip, twin):
    """Seeded random sizes and token counts with routing that prefers a few experts, through the
    kernel the host would choose and through every other one."""
    import random
    from sparseengine_amd.kernels.hip_ops import MoeWorkspace
    rng = random.Random(4)
    dtype = torch.bfloat16
    for case in range(16):
        experts = rng.choice([3, 4, 8, 16, 64])
        k = rng.randint(1, min(8, experts))
        hidden, inter = rng.choice([256, 512, 768]), rng.choice([128, 256, 384])
        tokens = rng.choice([1, 2, 7, 16, 17, 33, 64, 100, 255, 256, 257, 500, 1000, 2100])
        g = torch.Generator().manual_seed(case)
        x = torch.randn(tokens, hidden, generator=g).to(dtype).to(DEV)
        w13 = (torch.randn(experts, 2 * inter, hidden, generator=g) * hidden ** -0.5).to(dtype).to(DEV)
        w2 = (torch.randn(experts, hidden, inter, generator=g) * inter ** -0.5).to(dtype).to(DEV)
        liking = torch.rand(experts, generator=g) ** 3 + 1e-3
        ids = torch.stack([torch.multinomial(liking, k, generator=g) for _ in range(tokens)]).to(torch.int32).to(DEV)
        weights = torch.rand(tokens, k, generator=g).to(DEV)
        weights = weights / weights.sum(-1, keepdim=True)
        ws = MoeWorkspace(tokens, k, experts, hidden, inter, dtype, DEV)
        ref = torch.empty_like(x)
        twin.moe_experts(x, w13, w2, ids, weights, ref)
        a13, a2 = w13.clone(), w2.clone()
        assert hip.arrange_expert_weights(a13, a2)
        for kernel, rows in ((None, None), ("stream", 16), ("tall", 64), ("direct", 64), ("direct", 128), ("mid", 64),
                             ("mid", 96), ("auto", None)):
            out = torch.full_like(x, float("nan"))
            hip.moe_experts(x, a13, a2, ids, weights, out, ws, kernel=kernel, tile_rows=rows, tiled=True)
            torch.testing.assert_close(out, ref, **tol(dtype), msg=lambda m: (
                f"case {case}: {tokens} tokens, {experts} experts, top {k}, hidden {hidden}, width {inter}, kernel {kernel}: {m}"))


def test_the_device_chooses_the_expert_kernel_by_the_spread_of_the_rows(hip, twin):
    """"auto": the grouping kernel counts the experts that got rows and the tiles of 96 rows they fill, and chooses
    those tiles (the mid kernel's code) if reading a table per tile is less than what the wide kernel has to do
    (a table per expert, or its arithmetic), else tiles of 128.  The same tokens spread evenly and crowded onto
    two experts: the choice differs, the results are the twin's both times."""
    from sparseengine_amd.kernels.hip_ops import MoeWorkspace
    tokens, hidden, inter, experts, k = 400, 256, 128, 16, 2
    emulator_skips(tokens * k * hidden * inter, 1.2e8)
    dtype = torch.bfloat16
    x = randn(tokens, hidden, dtype=dtype, seed=31)
    w13 = randn(experts, 2 * inter, hidden, dtype=dtype, scale=hidden ** -0.5, seed=32)
    w2 = randn(experts, hidden, inter, dtype=dtype, scale=inter ** -0.5, seed=33)
    weights = torch.full((tokens, k), 0.5).to(DEV)
    ws = MoeWorkspace(tokens, k, experts, hidden, inter, dtype, DEV)
    g = torch.Generator().manual_seed(34)
    even = torch.stack([torch.randperm(experts, generator=g)[:k] for _ in range(tokens)]).to(torch.int32).to(DEV)   # 50 rows each
    crowded = torch.tensor([[3, 11]] * tokens, dtype=torch.int32).to(DEV)                                            # 400 rows each
    for ids, choice, tile_rows in ((even, 0, 96), (crowded, 1, 128)):
        ref = torch.empty_like(x)
        twin.moe_experts(x, w13, w2, ids, weights, ref)
        out = torch.full_like(x, float("nan"))
        hip.moe_experts(x, w13, w2, ids, weights, out, ws, kernel="auto")
        torch.testing.assert_close(out, ref, **tol(dtype))
        counters = ws.counters.tolist()
        assert counters[2] == choice
        rows = torch.bincount(ids.flatten().long().cpu(), minlength=experts)
        assert counters[0] == int(((rows + tile_rows - 1) // tile_rows).sum()) and counters[1] == counters[0] * tile_rows


def test_memory_probe_reads_and_copies_every_byte(hip):
    """The kernels the benchmarks price memory with: the read kernel's per-block words fold to the exclusive-or
    of the whole buffer (so every 16 bytes were read exactly once), also with a tail that does not fill a
    block's share; the copy kernel copies every byte."""
    if backends.ACTIVE.name != "hip":
        pytest.skip("a timing aid of the benchmarks: GPU only")
    for words in (1, 256 * 8 * 3 + 5, 1 << 20):
        src = torch.randint(-2 ** 31, 2 ** 31 - 1, (words * 4,), dtype=torch.int64).to(torch.int32).to(DEV)
        sink = torch.zeros(7 if words < 100 else 333, dtype=torch.int32, device=DEV)
        hip.stream_read(src, sink)
        import numpy as np
        assert (int(np.bitwise_xor.reduce(sink.cpu().numpy().view("uint32")))
                == int(np.bitwise_xor.reduce(src.cpu().numpy().view("uint32"))))
        dst = torch.zeros_like(src)
        hip.stream_copy(src, dst)
        assert torch.equal(src, dst)
    with pytest.raises(ValueError):
        hip.stream_read(torch.zeros(3, dtype=torch.int32, device=DEV))
