"""Plain MiniMax-M2 forward pass: whole sequences, no cache, no batching.

Every function is one part of the architecture written directly from the
formulas of the reference (CURRENTF/SparseEngine, paths relative to
``src/sparseengine``).  It runs on the CPU in float32 (float64 on request for
everything but the rotation angles, which the reference defines in float32),
shares no code with ``sparseengine_amd`` and reads the model folder by itself.
"""
from __future__ import annotations

import json
import math
import os
from dataclasses import dataclass

import torch
from safetensors import safe_open


# --------------------------------------------------------------------------- #
# parts
# --------------------------------------------------------------------------- #
def rms_norm(x: torch.Tensor, weight: torch.Tensor, eps: float) -> torch.Tensor:
    """``x * rsqrt(mean(x^2) + eps) * w``; eps is added to the mean, weight is plain.

    layers/layernorm.py:151-159, kernels/triton/rmsnorm.py:57-66,
    oracle tests/test_minimax_m2_model.py:45-57.
    """
    variance = x.square().mean(dim=-1, keepdim=True)
    return x * torch.rsqrt(variance + eps) * weight


def add_rms_norm(x, residual, weight, eps):
    """Fused residual form: ``r = x + residual; y = norm(r)``; returns ``(y, r)``.

    kernels/triton/rmsnorm.py:44-56, models/minimax_m2.py:387-395.
    """
    merged = x + residual
    return rms_norm(merged, weight, eps), merged


def flat_qk_norm(x: torch.Tensor, weight: torch.Tensor, eps: float) -> torch.Tensor:
    """RMS norm over the whole projected row (all heads together), one weight
    vector of the full width.  layers/layernorm.py:204-215, models/minimax_m2.py:307-316,344.
    """
    inv_rms = torch.rsqrt(x.square().sum(dim=-1, keepdim=True) / x.shape[-1] + eps)
    return x * inv_rms * weight


def rope_angles(positions: torch.Tensor, rotary_dim: int, theta: float):
    """cos/sin of ``p * theta^(-2d/R)``, ``d in [0, R/2)``; float32 as the reference
    builds its table.  layers/rotary_embedding.py:20-22,217-222.
    """
    exponent = torch.arange(0, rotary_dim, 2, dtype=torch.float32, device=positions.device) / rotary_dim
    inv_freq = 1.0 / (theta ** exponent)
    freqs = positions.to(torch.float32)[:, None] * inv_freq[None, :]
    return freqs.cos(), freqs.sin()


def partial_rope(x: torch.Tensor, cos: torch.Tensor, sin: torch.Tensor, rotary_dim: int):
    """NeoX split-half rotation of dims ``[0, R)`` of each head, pairs ``(d, d+R/2)``;
    dims ``[R, D)`` pass through.  ``x`` is ``[T, heads, D]``.

    layers/rotary_embedding.py:104-112 (rotation), :129-167 (partial).
    """
    rotated = x[..., :rotary_dim]
    x1, x2 = rotated[..., : rotary_dim // 2], rotated[..., rotary_dim // 2:]
    c = cos[:, None, :].to(x.dtype)
    s = sin[:, None, :].to(x.dtype)
    y1 = x1 * c - x2 * s
    y2 = x2 * c + x1 * s
    return torch.cat((y1, y2, x[..., rotary_dim:]), dim=-1)


def causal_gqa_attention(q, k, v, scale: float, window: int | None = None):
    """Full causal attention of one sequence.  ``q [T,H,D]``, ``k,v [T,Hkv,D]``;
    query head ``i`` reads kv head ``i // (H/Hkv)``; scores scaled by ``scale``,
    softmax over keys ``n <= p`` (and ``n > p - window`` if a window is given).

    models/minimax_m2.py:324-332, kernels/triton/context_flashattention_nopad.py:92-127,
    kernels/triton/gqa_flash_decoding_stage1.py:69-120.
    """
    T, H, D = q.shape
    Hkv = k.shape[1]
    group = H // Hkv
    out = torch.empty_like(q)
    pos = torch.arange(T, device=q.device)
    allowed = pos[None, :] <= pos[:, None]
    if window is not None:
        allowed &= pos[None, :] > pos[:, None] - window
    for head in range(H):
        kv_head = head // group
        scores = (q[:, head, :] @ k[:, kv_head, :].T) * scale
        scores = scores.masked_fill(~allowed, float("-inf"))
        probs = torch.softmax(scores, dim=-1)
        out[:, head, :] = probs @ v[:, kv_head, :]
    return out


def biased_sigmoid_router(logits: torch.Tensor, bias: torch.Tensor, top_k: int):
    """``s = sigmoid(g)``; experts chosen by ``top_k(s + bias)``; weights are the
    unbiased ``s`` of the chosen experts, renormalised to sum 1 (no epsilon).

    kernels/triton/minimax_m2_router.py:50-63, kernels/triton/moe_biased_sigmoid.py:202-238,
    oracle tests/test_minimax_m2_router.py:16-25.
    """
    scores = torch.sigmoid(logits)
    _, ids = torch.topk(scores + bias, top_k, dim=-1, sorted=False)
    weights = scores.gather(1, ids)
    weights = weights / weights.sum(dim=-1, keepdim=True)
    return weights, ids


def swiglu_experts(x, w1, w3, w2, ids, weights):
    """``y_t = sum_k w_tk * W2_e( silu(W1_e x_t) * (W3_e x_t) )`` with ``e = ids[t,k]``.
    ``w1, w3: [E, I, h]`` (gate, up), ``w2: [E, h, I]`` (down).

    models/minimax_m2.py:175-176 (w1 gate, w3 up, w2 down), oracle tests/test_triton_moe.py:75-98.
    """
    out = torch.zeros_like(x)
    for expert in range(w1.shape[0]):
        token_idx, slot = torch.where(ids == expert)
        if token_idx.numel() == 0:
            continue
        xe = x[token_idx]
        gate = xe @ w1[expert].T
        up = xe @ w3[expert].T
        ye = (torch.nn.functional.silu(gate) * up) @ w2[expert].T
        out.index_add_(0, token_idx, ye * weights[token_idx, slot, None])
    return out


# --------------------------------------------------------------------------- #
# the model
# --------------------------------------------------------------------------- #
@dataclass
class PlainConfig:
    """The config.json keys the model code reads (models/minimax_m2.py:140-160,272-323,
    tests/test_minimax_m2_config.py:25-52)."""
    vocab_size: int
    hidden_size: int
    intermediate_size: int
    num_hidden_layers: int
    num_attention_heads: int
    num_key_value_heads: int
    head_dim: int
    rotary_dim: int
    num_local_experts: int
    num_experts_per_tok: int
    rms_norm_eps: float
    rope_theta: float
    use_qk_norm: bool

    @classmethod
    def from_folder(cls, folder: str) -> "PlainConfig":
        with open(os.path.join(folder, "config.json")) as fh:
            return cls.from_dict(json.load(fh))

    @classmethod
    def from_dict(cls, raw: dict) -> "PlainConfig":
        rope_parameters = raw.get("rope_parameters") or {}
        theta = rope_parameters.get("rope_theta", raw.get("rope_theta", 10000.0))  # models/rope.py:37-43
        return cls(
            vocab_size=raw["vocab_size"], hidden_size=raw["hidden_size"],
            intermediate_size=raw["intermediate_size"], num_hidden_layers=raw["num_hidden_layers"],
            num_attention_heads=raw["num_attention_heads"], num_key_value_heads=raw["num_key_value_heads"],
            head_dim=raw["head_dim"], rotary_dim=raw["rotary_dim"],
            num_local_experts=raw["num_local_experts"], num_experts_per_tok=raw["num_experts_per_tok"],
            rms_norm_eps=raw["rms_norm_eps"], rope_theta=float(theta),
            use_qk_norm=bool(raw.get("use_qk_norm", True)),
        )


class PlainMiniMaxM2:
    """Whole-prompt forward pass from a model folder (config.json + *.safetensors)."""

    def __init__(self, folder: str, dtype: torch.dtype = torch.float32):
        self.cfg = PlainConfig.from_folder(folder)
        self.dtype = dtype
        self.w: dict[str, torch.Tensor] = {}
        for name in sorted(os.listdir(folder)):
            if not name.endswith(".safetensors"):
                continue
            with safe_open(os.path.join(folder, name), framework="pt") as fh:
                for key in fh.keys():
                    self.w[key] = fh.get_tensor(key).to(dtype)

    @classmethod
    def from_tensors(cls, raw_config: dict, tensors: dict[str, torch.Tensor], dtype: torch.dtype = torch.float32):
        """The same model from checkpoint tensors by name that are in memory already (a model too
        large to pass through a file); they may live on another device, where the forward pass then runs."""
        self = cls.__new__(cls)
        self.cfg = PlainConfig.from_dict(raw_config)
        self.dtype = dtype
        self.w = {name: t.to(dtype) for name, t in tensors.items()}
        return self

    # one decoder layer: models/minimax_m2.py:334-397
    def attention_inputs(self, layer: int, u: torch.Tensor, positions: torch.Tensor):
        c, p = self.cfg, f"model.layers.{layer}.self_attn."
        q = u @ self.w[p + "q_proj.weight"].T
        k = u @ self.w[p + "k_proj.weight"].T
        v = u @ self.w[p + "v_proj.weight"].T
        if c.use_qk_norm:
            q = flat_qk_norm(q, self.w[p + "q_norm.weight"], c.rms_norm_eps)
            k = flat_qk_norm(k, self.w[p + "k_norm.weight"], c.rms_norm_eps)
        T = u.shape[0]
        q = q.view(T, c.num_attention_heads, c.head_dim)
        k = k.view(T, c.num_key_value_heads, c.head_dim)
        v = v.view(T, c.num_key_value_heads, c.head_dim)
        cos, sin = rope_angles(positions, c.rotary_dim, c.rope_theta)
        return partial_rope(q, cos, sin, c.rotary_dim), partial_rope(k, cos, sin, c.rotary_dim), v

    def attention(self, layer: int, u: torch.Tensor, positions: torch.Tensor):
        c = self.cfg
        q, k, v = self.attention_inputs(layer, u, positions)
        o = causal_gqa_attention(q, k, v, c.head_dim ** -0.5)
        return o.reshape(u.shape[0], -1) @ self.w[f"model.layers.{layer}.self_attn.o_proj.weight"].T

    def router(self, layer: int, m: torch.Tensor, forced_ids=None, log=None):
        """``forced_ids`` ([T, K], from another run) replaces the selection but not the weights:
        used to compare a reduced-precision run whose near-ties fall the other way.  ``log[layer]``
        receives the selection scores ``sigmoid(g) + bias`` so that such a choice can be checked."""
        c, p = self.cfg, f"model.layers.{layer}.block_sparse_moe."
        logits = m @ self.w[p + "gate.weight"].T
        bias = self.w[p + "e_score_correction_bias"]
        if log is not None:
            log[layer] = torch.sigmoid(logits) + bias
        if forced_ids is None:
            return biased_sigmoid_router(logits, bias, c.num_experts_per_tok)
        ids = torch.as_tensor(forced_ids, dtype=torch.long, device=logits.device)
        weights = torch.sigmoid(logits).gather(1, ids)
        return weights / weights.sum(dim=-1, keepdim=True), ids

    def moe(self, layer: int, m: torch.Tensor, forced_ids=None, log=None):
        c, p = self.cfg, f"model.layers.{layer}.block_sparse_moe.experts."
        weights, ids = self.router(layer, m, forced_ids, log)
        stack = lambda proj: torch.stack([self.w[f"{p}{e}.{proj}.weight"] for e in range(c.num_local_experts)])
        return swiglu_experts(m, stack("w1"), stack("w3"), stack("w2"), ids, weights)

    def hidden_states(self, token_ids, start_position: int = 0, taps: dict | None = None,
                      forced_routing=None, routing_log=None):
        """Final-normed hidden state of every token.  Residual wiring:
        models/minimax_m2.py:381-397, models/qwen3.py:291-325."""
        c = self.cfg
        device = self.w["model.embed_tokens.weight"].device      # the CPU, unless the tensors were handed over elsewhere
        ids = torch.as_tensor(token_ids, dtype=torch.long, device=device)
        positions = torch.arange(start_position, start_position + ids.numel(), device=device)
        x = self.w["model.embed_tokens.weight"][ids]
        residual = None
        for layer in range(c.num_hidden_layers):
            p = f"model.layers.{layer}."
            if residual is None:
                residual, u = x, rms_norm(x, self.w[p + "input_layernorm.weight"], c.rms_norm_eps)
            else:
                u, residual = add_rms_norm(x, residual, self.w[p + "input_layernorm.weight"], c.rms_norm_eps)
            a = self.attention(layer, u, positions)
            m, residual = add_rms_norm(a, residual, self.w[p + "post_attention_layernorm.weight"], c.rms_norm_eps)
            x = self.moe(layer, m, None if forced_routing is None else forced_routing[layer], routing_log)
            if taps is not None:
                taps[layer] = x + residual
        y, _ = add_rms_norm(x, residual, self.w["model.norm.weight"], c.rms_norm_eps)
        return y

    def logits(self, token_ids, start_position: int = 0, forced_routing=None, routing_log=None) -> torch.Tensor:
        """``[len, vocab]`` logits of a whole sequence (layers/embed_head.py:75-84: plain
        linear, no scale, no soft-cap)."""
        hidden = self.hidden_states(token_ids, start_position, forced_routing=forced_routing,
                                    routing_log=routing_log)
        return hidden @ self.w["lm_head.weight"].T

    def greedy(self, prompt, max_tokens: int) -> list[int]:
        tokens = list(prompt)
        out = []
        for _ in range(max_tokens):
            nxt = int(self.logits(tokens)[-1].argmax())
            out.append(nxt)
            tokens.append(nxt)
        return out
