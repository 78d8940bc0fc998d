"""The engine on the CPU through the kernel sources themselves (``tests/emu``): model, cache, step
function and every kernel a step runs, with each tensor argument of each kernel call next to an
inaccessible page.  A short version of ``tests/test_gpu_replay.py`` / ``tests/test_gpu_engine.py``
(whose whole bodies run this way under ``SPARSEENGINE_AMD_TEST_BACKEND=emu pytest -m gpu``):
bfloat16 at sizes that take the matrix-core kernels, float32 through the general kernels, the toy
architecture with its windowed cache group, ``bin/trace_run`` as a program.
"""
import json
import os
import subprocess
import sys

import numpy as np
import pytest

import tests.test_gpu_replay as R
from tests import backends, traces
from tests.helpers import CONFIGS, make_folder, random_tokens
from tests.plain.minimax_m2 import PlainMiniMaxM2

pytestmark = pytest.mark.skipif(not backends.EmulatedBackend().available(), reason="no host compiler for the emulated kernels")
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def model_for(tmp_path, key, lengths):
    folder = make_folder(tmp_path, key)
    vocab = CONFIGS[key][0]["vocab_size"]
    requests = {f"r{i}": random_tokens(n, vocab, 100 + i) for i, n in enumerate(lengths)}
    plain = PlainMiniMaxM2(folder)
    return folder, requests, {rid: plain.logits(t).numpy() for rid, t in requests.items()}, plain


@pytest.mark.parametrize("key,dtype,guard,lengths", [
    ("C_loud", "bfloat16", "before", [3, 40, 70, 1, 33]),      # matrix-core attention, tiled expert tables, skinny products
    ("A_loud", "float32", "after", [5, 17, 64, 1, 48]),        # the general kernels
    ("B_loud", "bfloat16", "after", [1, 9, 65, 16])])          # matrix-core attention beside the general expert kernel
def test_mixed_requests_on_the_emulated_kernels(tmp_path, key, dtype, guard, lengths):
    model = model_for(tmp_path, key, lengths)
    records, peak = traces.mixed(model[1], seed=0)
    with backends.use(backends.EmulatedBackend(guard=guard)):
        logits, routing = R.run_records(model[0], dtype, records, peak, 16)
    R.compare(dtype, traces.gather(records, logits), model, routing)


def test_portions_and_single_tokens_on_the_emulated_kernels(tmp_path):
    model = model_for(tmp_path, "C_loud", [70, 33])
    for records in (traces.changing_portions(model[1], seed=16), traces.prefill_then_decode(model[1], tail=6)):
        with backends.use(backends.EmulatedBackend(guard="after")):
            logits, routing = R.run_records(model[0], "bfloat16", records, 128, 16)
        R.compare("bfloat16", traces.gather(records, logits), model, routing)


def test_toy_architecture_on_the_emulated_kernels(tmp_path):
    """Its windowed group gives pages back (window 24, pages of 16): with the inaccessible page
    *before* every tensor, a look-up of a page that was given back (id -1) ends the run."""
    from tests.test_gpu_engine import run_toy_architecture
    with backends.use(backends.EmulatedBackend(guard="before")):
        run_toy_architecture(tmp_path, "bfloat16", [50, 9, 1, 44])


def test_trace_run_program_on_the_emulated_kernels(tmp_path):
    model = model_for(tmp_path, "C_loud", [3, 40, 20])
    folder, requests, expected, _ = model
    records, peak = traces.mixed(requests, seed=3)
    env = dict(os.environ, SPARSEENGINE_AMD_KERNELS="tests.emu.kernels:EmulatedProgramKernels", PYTHONPATH=ROOT)
    proc = subprocess.run(
        [sys.executable, os.path.join(ROOT, "bin", "trace_run"), "--model", folder, "--dtype", "float32", "--out",
         str(tmp_path / "out"), "--max-tokens", str(peak), "--page-size", "16", "--device", "cpu"],
        input="".join(json.dumps(r) + "\n" for r in records), capture_output=True, text=True, timeout=900, env=env)
    assert proc.returncode == 0, proc.stderr[-2000:]
    vocab = next(iter(expected.values())).shape[1]
    logits = {r["step"]: np.fromfile(tmp_path / "out" / f"{r['step']}.f32", dtype="<f4").reshape(-1, vocab) for r in records}
    got = traces.gather(records, logits)
    for rid, ref in expected.items():
        assert np.abs(got[rid] - ref).max() <= R.bound("float32", ref), rid


@pytest.mark.parametrize("key,dtype", [("C_loud", "bfloat16"), ("A_loud", "float32")])
def test_the_slot_sum_left_to_the_next_norm_changes_no_bit(tmp_path, key, dtype):
    """In steps of few tokens the feed-forward hands its per-slot results on and the norm that reads them
    adds them up (one launch fewer per layer); otherwise the sum is a kernel of its own.  Same bits."""
    from sparseengine_amd.engine.replay import replay_step
    from sparseengine_amd.engine.runner import ModelRunner
    from sparseengine_amd.parts.base import SlotSum
    folder, requests, _, _ = model_for(tmp_path, key, [40, 3, 17])
    records, peak = traces.mixed(requests, seed=1)
    seen = []
    with backends.use(backends.EmulatedBackend(guard="after")):
        outs = []
        for deferral_tokens in (64, 0):
            options = backends.ACTIVE.runner_kwargs()
            options["kernels"].slot_sum_deferral_tokens = deferral_tokens
            runner = ModelRunner.from_folder(folder, dtype=dtype, kv_page_size=16, num_kvcache_tokens=peak, max_num_seqs=4,
                                             **options)
            norm = runner.model.final_norm
            rows = norm.forward_rows
            norm.forward_rows = lambda fb, x, *a, _rows=rows: (seen.append(isinstance(x, SlotSum)), _rows(fb, x, *a))[1]
            outs.append([replay_step(runner, rec, None, taps={}) for rec in records])
    assert seen[0] is True and seen[-1] is False          # the first run deferred the sum, the second did not
    for a, b in zip(*outs):
        assert (a is None and b is None) or np.array_equal(a, b)
