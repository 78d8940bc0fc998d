"""MiniMax M2 (``MiniMaxM2ForCausalLM``): its config.json keys, its layers as parts, its
checkpoint tensor names.

Every layer: RMSNorm -> full causal GQA attention with a flat QK RMSNorm and partial NeoX
rotation -> RMSNorm -> routed SwiGLU experts with a sigmoid router whose correction bias only
selects (reference models/minimax_m2.py:140-414; fixed semantics models/checkpoint.py:222-243;
official values tests/test_minimax_m2_config.py:25-52).  The reference runs this model with FP8
weights only; here the unquantised tensors are loaded, and ``use_qk_norm=false`` is allowed.
"""
from __future__ import annotations

import math
from dataclasses import asdict, dataclass, field

import torch

from ..config.registry import Architecture, WeightSource, register_architecture
from ..config.specs import (AttentionSpec, LayerSpec, ModelSpec, MoESpec, NormSpec, RotarySpec,
                            default_schedule)

ARCHITECTURE = "MiniMaxM2ForCausalLM"
_REQUIRED = ("vocab_size", "hidden_size", "intermediate_size", "num_hidden_layers", "num_attention_heads",
             "num_key_value_heads", "head_dim", "rotary_dim", "num_local_experts", "num_experts_per_tok",
             "rms_norm_eps", "max_position_embeddings")


@dataclass(frozen=True)
class MiniMaxM2Config:
    vocab_size: int
    hidden_size: int
    intermediate_size: int              # per expert
    num_hidden_layers: int
    num_attention_heads: int
    num_key_value_heads: int
    head_dim: int                        # read directly, not hidden_size / heads
    rotary_dim: int
    num_local_experts: int
    num_experts_per_tok: int
    rms_norm_eps: float
    max_position_embeddings: int
    rope_theta: float = 10000.0          # rope_parameters.rope_theta, else rope_theta (models/rope.py:37-43)
    rope_scaling: tuple | None = None    # sorted items of rope_parameters / rope_scaling when not "default"
    use_qk_norm: bool = True
    qk_norm_type: str = "per_layer"
    scoring_func: str = "sigmoid"
    use_routing_bias: bool = True
    hidden_act: str = "silu"
    tie_word_embeddings: bool = False
    routed_scaling_factor: float = 1.0
    shared_intermediate_size: int = 0
    extra: dict = field(default_factory=dict, compare=False)   # keys carried through untouched

    @classmethod
    def from_dict(cls, raw: dict) -> "MiniMaxM2Config":
        missing = [k for k in _REQUIRED if k not in raw]
        if missing:
            raise ValueError(f"MiniMax M2 config.json lacks the keys {missing}")
        rope = dict(raw.get("rope_parameters") or raw.get("rope_scaling") or {})
        theta = float(rope.get("rope_theta", raw.get("rope_theta", 10000.0)))
        rope_type = str(rope.get("rope_type", rope.get("type", "default"))).lower()
        scaling = None
        if rope_type != "default":
            rope.pop("type", None)
            rope["rope_type"] = rope_type
            scaling = tuple(sorted((k, tuple(v) if isinstance(v, list) else v) for k, v in rope.items()))
        known = set(cls.__dataclass_fields__) - {"extra", "rope_scaling"}
        cfg = cls(**{k: raw[k] for k in known if k in raw and k != "rope_theta"}, rope_theta=theta,
                  rope_scaling=scaling,
                  extra={k: v for k, v in raw.items() if k not in known and k not in ("rope_parameters", "rope_scaling")})
        cfg.validate()
        return cfg

    def validate(self) -> None:
        problems = []
        if self.hidden_act != "silu":
            problems.append(f"hidden_act must be 'silu', got {self.hidden_act!r}")
        if self.scoring_func != "sigmoid":
            problems.append(f"scoring_func must be 'sigmoid', got {self.scoring_func!r}")
        if self.use_qk_norm and self.qk_norm_type != "per_layer":
            problems.append(f"qk_norm_type must be 'per_layer', got {self.qk_norm_type!r}")
        if not self.use_routing_bias:
            problems.append("use_routing_bias must be true")
        if self.tie_word_embeddings:
            problems.append("tie_word_embeddings must be false")
        if float(self.routed_scaling_factor) != 1.0:
            problems.append("routed_scaling_factor must be 1.0")
        if self.shared_intermediate_size:
            problems.append("a shared expert (shared_intermediate_size > 0) is not part of this model")
        if self.num_key_value_heads <= 0 or self.num_attention_heads % self.num_key_value_heads:
            problems.append(f"{self.num_attention_heads} heads do not divide into {self.num_key_value_heads} kv heads")
        if not 1 <= self.num_experts_per_tok <= self.num_local_experts:
            problems.append(f"num_experts_per_tok must be in [1, {self.num_local_experts}]")
        if self.rotary_dim % 2 or not 0 < self.rotary_dim <= self.head_dim:
            problems.append(f"rotary_dim must be even and in (0, head_dim], got {self.rotary_dim}")
        if self.head_dim % 16:
            problems.append(f"head_dim must be a multiple of 16, got {self.head_dim}")
        if self.max_position_embeddings <= 0:
            problems.append("max_position_embeddings must be positive")
        if not (math.isfinite(self.rope_theta) and self.rope_theta > 0):
            problems.append(f"rope_theta must be finite and positive, got {self.rope_theta}")
        if self.rope_scaling and dict(self.rope_scaling)["rope_type"] not in ("linear", "llama3", "yarn"):
            problems.append(f"rope_type {dict(self.rope_scaling)['rope_type']!r} is not supported "
                            "(default, linear, llama3, yarn)")
        if "quantization_config" in self.extra and self.extra["quantization_config"]:
            problems.append("quantised checkpoints (quantization_config) are not supported")
        if problems:
            raise ValueError("MiniMax M2 configuration rejected: " + "; ".join(problems))

    def to_dict(self) -> dict:
        out = {k: v for k, v in asdict(self).items() if k not in ("extra", "rope_scaling")}
        if self.rope_scaling:
            out["rope_parameters"] = {**dict(self.rope_scaling), "rope_theta": self.rope_theta}
        out.update(self.extra)
        out["architectures"] = [ARCHITECTURE]
        out["model_type"] = "minimax_m2"
        return out


def build_spec(cfg: MiniMaxM2Config) -> ModelSpec:
    rotary = RotarySpec(rotary_dim=cfg.rotary_dim, theta=cfg.rope_theta,
                        max_position=cfg.max_position_embeddings, scaling=cfg.rope_scaling)
    attention = AttentionSpec(num_heads=cfg.num_attention_heads, num_kv_heads=cfg.num_key_value_heads,
                              head_dim=cfg.head_dim, scale=cfg.head_dim ** -0.5,
                              qk_norm="flat" if cfg.use_qk_norm else "none", qk_norm_eps=cfg.rms_norm_eps,
                              window=None, position=rotary)
    experts = MoESpec(num_experts=cfg.num_local_experts, top_k=cfg.num_experts_per_tok,
                      intermediate_size=cfg.intermediate_size, scoring="sigmoid", selection_bias=True,
                      norm_topk_prob=True, routed_scaling_factor=1.0, activation="silu")
    norm = NormSpec(eps=cfg.rms_norm_eps)
    layer = LayerSpec(mixer=attention, feed_forward=experts, norm=norm, block="prenorm")
    return ModelSpec(architecture=ARCHITECTURE, hidden_size=cfg.hidden_size, vocab_size=cfg.vocab_size,
                     layers=(layer,) * cfg.num_hidden_layers, schedule=default_schedule(cfg.num_hidden_layers),
                     final_norm=norm, max_position=cfg.max_position_embeddings, tie_word_embeddings=False)


def weight_sources(cfg: MiniMaxM2Config) -> list[WeightSource]:
    """Checkpoint names (reference models/minimax_m2.py:292-316,370-379,419-423,513-530): q, k, v
    stack into ``qkv``; w1 (gate) and w3 (up) stack into ``w13``; w2 is the down projection."""
    q = cfg.num_attention_heads * cfg.head_dim
    kv = cfg.num_key_value_heads * cfg.head_dim
    inter = cfg.intermediate_size
    out = [WeightSource("model.embed_tokens.weight", "embed.weight"),
           WeightSource("model.norm.weight", "final_norm.weight"),
           WeightSource("lm_head.weight", "head.weight")]
    for i in range(cfg.num_hidden_layers):
        src, dst = f"model.layers.{i}.", f"layers.{i}."
        out += [
            WeightSource(src + "input_layernorm.weight", dst + "norm_mixer.weight"),
            WeightSource(src + "post_attention_layernorm.weight", dst + "norm_ffn.weight"),
            WeightSource(src + "self_attn.q_proj.weight", dst + "mixer.qkv", (slice(0, q),)),
            WeightSource(src + "self_attn.k_proj.weight", dst + "mixer.qkv", (slice(q, q + kv),)),
            WeightSource(src + "self_attn.v_proj.weight", dst + "mixer.qkv", (slice(q + kv, q + 2 * kv),)),
            WeightSource(src + "self_attn.o_proj.weight", dst + "mixer.o"),
            WeightSource(src + "block_sparse_moe.gate.weight", dst + "ffn.router"),
            WeightSource(src + "block_sparse_moe.e_score_correction_bias", dst + "ffn.router_bias"),
        ]
        if cfg.use_qk_norm:
            out += [WeightSource(src + "self_attn.q_norm.weight", dst + "mixer.q_norm"),
                    WeightSource(src + "self_attn.k_norm.weight", dst + "mixer.k_norm")]
        for e in range(cfg.num_local_experts):
            esrc = f"{src}block_sparse_moe.experts.{e}."
            out += [WeightSource(esrc + "w1.weight", dst + "ffn.w13", (e, slice(0, inter))),
                    WeightSource(esrc + "w3.weight", dst + "ffn.w13", (e, slice(inter, 2 * inter))),
                    WeightSource(esrc + "w2.weight", dst + "ffn.w2", (e,))]
    return out


def ignored_tensor(name: str) -> bool:
    """Multi-token-prediction modules ship with the checkpoint and are not part of the decoder."""
    return ".mtp" in name or name.startswith("mtp.") or name.startswith("model.mtp")


def stored_dtype(name: str) -> str:
    """Router table and correction bias are 32-bit in the checkpoint (the reference declares them
    float32, models/minimax_m2.py:146-151); everything else is bfloat16."""
    if name.endswith("block_sparse_moe.gate.weight") or name.endswith("e_score_correction_bias"):
        return "float32"
    return "bfloat16"


def random_tensor(cfg, name: str, shape, generator: torch.Generator, options: dict) -> torch.Tensor:
    """Weights N(0, std); norm weights 1 + N(0, norm_std); correction bias N(0, bias_std)."""
    noise = torch.randn(tuple(shape), generator=generator, dtype=torch.float32, device=generator.device)
    if name.endswith("layernorm.weight") or name.endswith("norm.weight"):
        return 1.0 + noise * float(options.get("norm_std", 0.1))
    if name.endswith("e_score_correction_bias"):
        return noise * float(options.get("bias_std", 0.1))
    return noise * float(options.get("std", 0.02))


register_architecture(Architecture(
    name=ARCHITECTURE, model_types=("minimax_m2", "minimax"), parse_config=MiniMaxM2Config.from_dict,
    build_spec=build_spec, weight_sources=weight_sources, ignored_tensor=ignored_tensor,
    random_tensor=random_tensor, stored_dtype=stored_dtype, config_to_dict=MiniMaxM2Config.to_dict))
