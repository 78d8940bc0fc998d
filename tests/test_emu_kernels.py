"""The kernel sources themselves on the CPU: ``tests/emu`` builds ``sparseengine_amd/csrc`` for the
host and runs every thread of every block, with each tensor argument next to an inaccessible page.

The test bodies are those of ``tests/test_gpu_kernels.py`` (against the twins and the library
routines), at sizes the emulator gets through in seconds; what is checked here and not on the GPU:
an access outside a tensor (before it or after it) ends the run with the kernel, block and thread
named; results do not depend on the order in which a block's threads run nor on when loads that go
straight into shared memory land.  ``SPARSEENGINE_AMD_TEST_BACKEND=emu pytest -m gpu`` runs all
of the GPU tests this way (an hour on eight cores).
"""
import pytest
import torch

import tests.test_gpu_kernels as G
from tests import backends
from tests.twin_kernels import TwinKernels

pytestmark = pytest.mark.skipif(not backends.EmulatedBackend().available(), reason="no host compiler for the emulated kernels")
BF16, F32 = torch.bfloat16, torch.float32


@pytest.fixture(params=["after", "before"])
def guard(request):
    return request.param


@pytest.fixture
def twin():
    return TwinKernels()


class Emulated:
    """Context: the emulated backend, with the GPU tests' module pointed at the CPU."""

    def __init__(self, **settings):
        self.backend = backends.EmulatedBackend(**settings)

    def __enter__(self):
        self.context = backends.use(self.backend)
        self.context.__enter__()
        G.DEV = "cpu"
        return self.backend.kernels()

    def __exit__(self, *exc):
        G.DEV = backends.ACTIVE.device
        return self.context.__exit__(*exc)


def test_embedding_norm_rotation_and_cache_write(guard, twin):
    with Emulated(guard=guard) as hip:
        for dtype in (F32, BF16):
            G.test_embedding(hip, dtype, 5, 200, 77)
            G.test_rms_norm_plain_and_fused(hip, twin, dtype, None, 7, 3072)
            G.test_rms_norm_plain_and_fused(hip, twin, dtype, F32, 33, 200)
            for shape in [(4, 2, 16, 8, True, 16), (6, 3, 32, 32, False, 16), (5, 5, 48, 16, True, 32),
                          (3, 1, 80, 0, False, 16), (48, 8, 128, 64, True, 64)]:
                G.test_qk_norm_rope_store(hip, twin, dtype, *shape)
            for shape in [(4, 2, 16, 8, True, 16), (6, 3, 32, 32, False, 16)]:
                G.test_rotation_of_neighbouring_dims(hip, twin, dtype, *shape)


@pytest.mark.parametrize("heads,kv_heads,head_dim,page,window", [
    (4, 2, 16, 16, 0), (6, 3, 32, 16, 0), (12, 2, 64, 32, 0), (4, 2, 16, 16, 20), (6, 1, 128, 64, 100), (6, 3, 32, 8, 0),
    (4, 1, 256, 32, 50), (6, 2, 32, 16, 24)])
def test_attention_mixed_batch(guard, twin, heads, kv_heads, head_dim, page, window):
    """A whole prompt, a portion on a cached prefix and a decoded token in one step.  With a window
    the pages it has passed are given back (-1 in the table, not-a-number in the page): no look-up
    may touch them.  head_dim 16 takes the general kernel, the others the matrix-core kernels."""
    with Emulated(guard=guard) as hip:
        for dtype in ((F32, BF16) if head_dim <= 32 else (BF16,)):
            G.test_paged_attention_mixed_batch(hip, twin, dtype, heads, kv_heads, head_dim, page, window)


def test_attention_split_keys_and_one_far_key(guard, twin):
    with Emulated(guard=guard) as hip:
        G.test_paged_attention_split_keys(hip, twin, 3, 700, 1)
        G.test_paged_attention_finds_one_far_key(hip, BF16)


@pytest.mark.parametrize("shape", [
    (16, 8, 64, 32, 70, [300, 200], [300, 150]),        # a window shorter than the portions
    (8, 8, 32, 8, 0, [420], [420]),
    (16, 8, 64, 24, 0, [300, 200], [300, 100]),         # pages that are no multiple of a step of 32 keys
    (24, 8, 96, 40, 33, [250, 100, 90], [240, 100, 1]),
    (12, 2, 64, 16, 90, [600, 500], [30, 77]),          # few blocks and a window
    (4, 2, 32, 16, 0, [2300], [40]),                    # one row block per kv head: three ranges of keys and a merge
    (12, 2, 64, 16, 1500, [2600, 2500], [30, 77])])     # the same within a window
def test_attention_prompt_portions(guard, twin, shape):
    with Emulated(guard=guard) as hip:
        G.test_paged_attention_prompt_portions(hip, twin, *shape)


def test_prompt_attention_with_maxima_that_keep_rising(guard, twin):
    with Emulated(guard=guard) as hip:
        G.test_prompt_attention_with_maxima_that_keep_rising(hip, twin, 8, 2, 64, 16, 0, 700, 300)
        G.test_prompt_attention_with_maxima_that_keep_rising(hip, twin, 8, 4, 32, 8, 500, 900, 260)


def test_attention_at_the_windows_edge(guard):
    with Emulated(guard=guard) as hip:
        for shape in [(4, 2, 16, 16, 20, 150, 60), (6, 1, 128, 64, 100, 301, 1), (12, 4, 96, 24, 50, 400, 200)]:
            G.test_attention_at_the_windows_edge(hip, *shape)


def test_router(guard, twin):
    with Emulated(guard=guard) as hip:
        for dtype in (F32, BF16):
            for shape in [(1, 256, 3072), (16, 7, 200), (13, 30, 1032)]:
                G.test_router_logits_are_float_products(hip, dtype, *shape)
            for shape in [(1, 256, 8, 3072), (3, 64, 6, 512), (5, 7, 3, 200), (3, 1, 1, 8)]:
                G.test_whole_router(hip, dtype, *shape)
        G.test_router_ties_nonfinite_and_bias(hip, twin)
        for shape in [(1, 256, 8), (8, 256, 8), (5, 7, 3), (3, 1, 1)]:
            G.test_router_with_grouping_in_one_launch(hip, *shape)


@pytest.mark.parametrize("tokens,hidden,inter,experts,k", [
    (1, 64, 32, 8, 2), (45, 96, 48, 16, 4), (130, 200, 72, 5, 5), (9, 256, 128, 1, 1),      # the general kernel
    (1, 256, 128, 8, 2), (3, 384, 256, 16, 4), (70, 256, 128, 4, 2)])                        # the matrix-core kernels
def test_experts(guard, twin, tokens, hidden, inter, experts, k):
    """bfloat16 at sizes in steps of 128 / 256 runs every matrix-core kernel and tile (the body of
    the GPU test forces each of them in turn)."""
    with Emulated(guard=guard) as hip:
        for dtype in (F32, BF16):
            G.test_moe_experts(hip, twin, dtype, tokens, hidden, inter, experts, k)


def test_wide_tiles_leave_out_row_blocks_of_padding(guard, twin):
    with Emulated(guard=guard) as hip:
        G.test_wide_tiles_leave_out_row_blocks_of_padding(hip, twin, [1, 16, 17, 47, 48, 49, 64, 65, 96, 111, 112, 113, 128, 129, 0])
        G.test_wide_tiles_leave_out_row_blocks_of_padding(hip, twin, [128, 0, 0, 3])


def test_experts_with_the_other_activation(guard, twin):
    with Emulated(guard=guard) as hip:
        G.test_experts_with_the_other_activation(hip, twin, F32, 45, 96, 48, 16, 4)
        G.test_experts_with_the_other_activation(hip, twin, BF16, 70, 256, 128, 4, 2)


def test_slot_sum_dense_products_and_sampling(guard, twin):
    with Emulated(guard=guard) as hip:
        for dtype in (F32, BF16):
            G.test_silu_mul(hip, twin, dtype)
        for shape in [(16, 256, 128), (17, 48, 256), (33, 1024, 384), (5, 50, 128), (3, 64, 96), (1, 512, 1024), (7, 64, 768), (16, 48, 1536),
                      (2, 32, 3072)]:
            G.test_skinny_linear(hip, *shape)
        G.test_rounding_to_bfloat16_is_to_nearest_even(hip)
        G.test_expert_tables_arranged_in_place_are_the_tiled_copy(hip, twin)
        G.test_sampling(hip, twin)
        if guard == "after":
            G.test_sampling_keeps_exactly_the_tokens_of_the_filters(hip, 5000, 0.1, 128)
        for dtype in (F32, BF16):
            for shape in [(1, 8, 3072), (5, 2, 256), (7, 3, 200), (3, 4, 20)]:
                G.test_norm_adds_up_slots_as_it_reads(hip, dtype, *shape)


def _outputs(hip, twin):
    """Kernels whose threads hand data to each other, on fixed inputs: their raw outputs."""
    from sparseengine_amd.kernels.hip_ops import MoeWorkspace
    out = {}
    heads, kv_heads, head_dim, page = 12, 2, 64, 16
    lens, q_lens = [300, 130, 77], [300, 40, 1]
    cache, table = G.make_paged(BF16, kv_heads, head_dim, page, lens, seed=1)
    meta = G.make_meta(table, lens, q_lens)
    q = G.randn(sum(q_lens), heads, head_dim, dtype=BF16, seed=2)
    att = torch.empty(sum(q_lens), heads * head_dim, dtype=BF16)
    hip.paged_attention(q, cache, meta, att, head_dim ** -0.5, 0)
    out["attention"] = att
    tokens, hidden, inter, experts, k = 150, 256, 128, 4, 2
    x = G.randn(tokens, hidden, dtype=BF16, seed=3)
    w13 = G.randn(experts, 2 * inter, hidden, dtype=BF16, scale=hidden ** -0.5, seed=4)
    w2 = G.randn(experts, hidden, inter, dtype=BF16, scale=inter ** -0.5, seed=5)
    ids = torch.stack([torch.randperm(experts, generator=torch.Generator().manual_seed(t))[:k] for t in range(tokens)]).int()
    weights = torch.full((tokens, k), 0.5)
    ws = MoeWorkspace(tokens, k, experts, hidden, inter, BF16, "cpu")
    for kernel, rows in (("stream", 16), ("tall", 64), ("direct", 128), ("mid", 64), ("mid", 96)):
        y = torch.empty_like(x)
        hip.moe_experts(x, w13, w2, ids, weights, y, ws, kernel=kernel, tile_rows=rows)
        out[f"{kernel}{rows}"] = y
    logits = G.randn(5, 40, dtype=F32, seed=6)
    ids5 = torch.empty(5, 3, dtype=torch.int32)
    w5 = torch.empty(5, 3)
    hip.router_topk(logits, None, 3, ids5, w5, workspace=MoeWorkspace(5, 3, 40, 128, 128, BF16, "cpu"))
    out["router"] = torch.cat([ids5.float(), w5], 1)
    return out


def test_results_do_not_depend_on_the_order_of_threads_or_on_when_loads_land(twin):
    """Between two synchronisation points the hardware runs a block's threads in any order, and a
    load that goes straight into shared memory may land at once or only when it is waited for.
    Bit-equal outputs under ascending, descending and shuffled orders and under both extremes of
    landing: a missing barrier or a wait that is too weak would show as a difference."""
    with Emulated(guard="after") as hip:
        base = _outputs(hip, twin)
    for settings in (dict(schedule="descending"), dict(schedule="shuffled", seed=7), dict(lds="at_issue"),
                     dict(schedule="shuffled", seed=11, lds="at_issue")):
        with Emulated(guard="after", **settings) as hip:
            other = _outputs(hip, twin)
        for name, value in base.items():
            assert torch.equal(value, other[name]), f"{name} differs under {settings}"


def test_an_access_outside_a_tensor_ends_the_run_with_its_name(tmp_path):
    """The tool itself: a kernel that reads past its input is stopped and named (in a child process)."""
    import subprocess
    import sys
    script = tmp_path / "overrun.py"
    script.write_text(
        "import torch\n"
        "from tests.emu.kernels import EmuKernels, emulated\n"
        "with emulated(guard='after'):\n"
        "    ids = torch.zeros(4, dtype=torch.int32)\n"
        "    table = torch.zeros(3, 64)\n"
        "    ids[2] = 3      # one row past the table: the host checks shapes, not values\n"
        "    EmuKernels().embedding(ids, table, torch.empty(4, 64))\n")
    proc = subprocess.run([sys.executable, str(script)], capture_output=True, text=True, cwd=G.__file__.rsplit("/tests/", 1)[0],
                          env={**__import__("os").environ, "PYTHONPATH": G.__file__.rsplit("/tests/", 1)[0]})
    assert proc.returncode == 97, proc.stderr[-2000:]
    assert "embedding_kernel" in proc.stderr and "past the end of argument 1 of se_embedding" in proc.stderr
