"""What a decode step launches, layer by layer.

A decode step of few tokens is bound by its launches as much as by its bytes (about eleven kernels a layer, each with
a start-up of its own), so their number and order are pinned here: the engine's own step function runs on the CPU
with the table of entry points replaced by a recorder (no kernel runs, the results are whatever the buffers held),
at sizes that take the matrix-core paths the full-size model takes."""
import pytest
import torch

from sparseengine_amd.engine.runner import ModelRunner, StepEntry
from sparseengine_amd.kernels import hip_ops

CONFIG = dict(
    architectures=["MiniMaxM2ForCausalLM"], model_type="minimax_m2", hidden_size=256, intermediate_size=128,
    num_hidden_layers=3, num_attention_heads=4, num_key_value_heads=2, head_dim=64, rotary_dim=32, vocab_size=1024,
    num_local_experts=32, num_experts_per_tok=4, rms_norm_eps=1e-6, rope_theta=10000.0, max_position_embeddings=4096,
    use_qk_norm=True, qk_norm_type="per_layer", scoring_func="sigmoid", use_routing_bias=True, hidden_act="silu",
    tie_word_embeddings=False, torch_dtype="bfloat16")

LAYER = ["se_skinny_gemm_mfma",          # q, k, v of the step's tokens in one product
         "se_qk_norm_rope_store",        # QK norm, rotation, cache write
         "se_paged_attention_mfma",      # attention over the cache (with the merge of its key ranges: two kernels)
         "se_skinny_gemm_mfma",          # output projection
         "se_rms_norm",                  # residual add + norm before the experts
         "se_router_logits",
         "se_router_topk_align",         # routing and grouping by expert
         "se_grouped_gemm_mfma",         # gate and up, activation, product
         "se_grouped_gemm_mfma"]         # down, times the routing weight (the sum over slots is left to the next norm)


class Recorder:
    def __init__(self):
        self.names = []

    def get(self, library, name):
        def entry(*args):
            self.names.append(name)
            return 0
        return entry


@pytest.mark.parametrize("batch", [1, 8])
def test_a_decode_step_is_these_launches(monkeypatch, batch):
    recorder = Recorder()
    monkeypatch.setattr(hip_ops, "_fn", recorder)
    monkeypatch.setattr(hip_ops, "_stream", lambda: 0)
    kernels = hip_ops.HipKernels.__new__(hip_ops.HipKernels)
    kernels._attention_partials = kernels._sample_partials = None
    runner = ModelRunner.from_random(CONFIG, seed=0, options=dict(std=0.02), dtype="bfloat16", kv_page_size=64,
                                     num_kvcache_tokens=16 * 1024, max_num_seqs=16, max_model_len=1024, device="cpu",
                                     kernels=kernels)
    ids = [f"r{i}" for i in range(batch)]
    runner.cache.append([(runner.admit(r), 300) for r in ids])           # contexts of 300 tokens, as if prefilled
    runner.step([StepEntry(r, [7], [0]) for r in ids])                   # buffers and workspaces are made here
    recorder.names.clear()
    logits = runner.step([StepEntry(r, [7], [0]) for r in ids])
    assert logits.shape == (batch, CONFIG["vocab_size"])
    layers = CONFIG["num_hidden_layers"]
    expected = (["se_embedding", "se_rms_norm"] + LAYER                                        # the first layer norms the embedding
                + (["se_rms_norm_slots"] + LAYER) * (layers - 1)                               # the others add up the experts' slots as they norm
                + ["se_rms_norm_slots", "se_skinny_gemm_mfma"])                                # final norm of the wanted rows, vocabulary head
    assert recorder.names == expected
    assert len(LAYER) + 1 == 10                                                                # ten calls, eleven kernels a layer
