"""Tiny MiniMax-M2 configurations of the tests and helpers to build model folders from them."""
from __future__ import annotations

import torch

# Two configurations that differ in every size and option.
TINY_A = dict(  # seed 0
    architectures=["MiniMaxM2ForCausalLM"], model_type="minimax_m2",
    num_hidden_layers=2, hidden_size=64, num_attention_heads=4, num_key_value_heads=2, head_dim=16,
    rotary_dim=8, rope_theta=10000.0, num_local_experts=8, num_experts_per_tok=2, intermediate_size=32,
    vocab_size=512, rms_norm_eps=1e-6, use_qk_norm=True, max_position_embeddings=256,
    tie_word_embeddings=False, hidden_act="silu", scoring_func="sigmoid", use_routing_bias=True,
    qk_norm_type="per_layer")
TINY_A_OPTIONS = dict(std=0.02, norm_std=0.1, bias_std=0.1)

TINY_B = dict(  # seed 1
    architectures=["MiniMaxM2ForCausalLM"], model_type="minimax_m2",
    num_hidden_layers=3, hidden_size=96, num_attention_heads=6, num_key_value_heads=3, head_dim=32,
    rotary_dim=32, rope_parameters={"rope_theta": 5000000.0, "rope_type": "default"}, num_local_experts=16,
    num_experts_per_tok=4, intermediate_size=48, vocab_size=1000, rms_norm_eps=1e-5, use_qk_norm=False,
    max_position_embeddings=512, tie_word_embeddings=False)
TINY_B_OPTIONS = dict(std=0.02, norm_std=0.0, bias_std=0.0)

# Sizes that the matrix-core kernels take (hidden and expert widths in steps of 128 / 256, head size in
# steps of 32, a vocabulary in steps of 16): the engine then runs the kernels that the full-size model
# runs: tiled expert tables, all three expert kernels, both attention kernels, the skinny products.
TINY_C = dict(  # seed 2
    architectures=["MiniMaxM2ForCausalLM"], model_type="minimax_m2",
    num_hidden_layers=2, hidden_size=256, num_attention_heads=6, num_key_value_heads=2, head_dim=64,
    rotary_dim=32, rope_theta=1000000.0, num_local_experts=8, num_experts_per_tok=2, intermediate_size=128,
    vocab_size=320, rms_norm_eps=1e-6, use_qk_norm=True, max_position_embeddings=1024,
    tie_word_embeddings=False, hidden_act="silu", scoring_func="sigmoid", use_routing_bias=True,
    qk_norm_type="per_layer")

# Weights this small give nearly uniform attention and routing; a larger spread makes scores,
# routing and logits depend visibly on every part.
LOUD_OPTIONS = dict(std=0.08, norm_std=0.3, bias_std=0.3)

CONFIGS = {"A": (TINY_A, TINY_A_OPTIONS, 0), "B": (TINY_B, TINY_B_OPTIONS, 1),
           "A_loud": (TINY_A, LOUD_OPTIONS, 10), "B_loud": (TINY_B, LOUD_OPTIONS, 11),
           "C_loud": (TINY_C, dict(std=0.05, norm_std=0.3, bias_std=0.3), 12)}


def make_folder(tmp_path, key: str) -> str:
    from sparseengine_amd.weights.random_weights import write_model_folder
    raw, options, seed = CONFIGS[key]
    return write_model_folder(str(tmp_path / f"model_{key}"), raw, seed, options)


def random_tokens(n: int, vocab: int, seed: int) -> list[int]:
    g = torch.Generator().manual_seed(seed)
    return torch.randint(0, vocab, (n,), generator=g).tolist()
