"""A toy architecture defined wholly in the tests, to show that parts, cache groups, state slots
and the run order are general: layers differ in mixer (full attention, windowed attention, a
recurrent mixer with state of its own), in feed-forward (dense, routed experts, a feed-forward
with a routing rule of its own), in position encoding (rotary, a rotation with its own table, one that
is no rotation and applies itself), in the model's two ends (an embedding multiplier, a logit scale), in norm (the engine's, one with another statistic) and in how a layer is arranged (mixer
then feed-forward, or the two side by side), the schedule runs a layer twice and lets one position read another position's cache.  Nothing in ``sparseengine_amd``
knows about it: it registers itself through the public registries.  It is no model of anyone's.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import ClassVar

import torch

from sparseengine_amd.config.registry import Architecture, WeightSource, register_architecture
from sparseengine_amd.config.specs import (AttentionSpec, DenseMLPSpec, LayerSpec, ModelSpec, MoESpec, NoPositionSpec,
                                           NormSpec, RotarySpec, ScheduleEntry)
from sparseengine_amd.parts import (BLOCKS, FEED_FORWARDS, MIXERS, NORMS, POSITIONS, ParamDecl, Part, StateRequest,
                                     DecoderModel, FusedRotation, build_model)
from tests.plain import minimax_m2 as P


# ------------------------------------------------------------------ a mixer with state of its own
@dataclass(frozen=True)
class DecayMixerSpec:
    kind: ClassVar[str] = "toy_decay"
    state_size: int = 8
    decay: float = 0.9


class DecayMixer(Part):
    """``s_t = decay * s_{t-1} + W_in x_t``; ``y_t = W_out s_t``; the state is float32 and per request."""

    def __init__(self, spec: DecayMixerSpec, hidden_size: int):
        self.spec, self.hidden_size = spec, hidden_size

    def param_decls(self):
        return {"w_in": ParamDecl((self.spec.state_size, self.hidden_size)),
                "w_out": ParamDecl((self.hidden_size, self.spec.state_size))}

    def cache_request(self):
        return StateRequest((("s", (self.spec.state_size,), torch.float32),))

    def forward(self, fb, x, cache_position, write_cache=True):
        state = fb.state_view(cache_position)["s"]
        w_in, w_out = self.params["w_in"].float(), self.params["w_out"].float()
        out = torch.empty_like(x)
        for row, start, n in zip(fb.item_rows_host.tolist(), fb.item_q_start.tolist(), fb.item_q_len.tolist()):
            s = state[row].clone()
            for t in range(start, start + n):          # a portion's tokens, in order
                s = self.spec.decay * s + w_in @ x[t].float()
                out[t] = (w_out @ s).to(x.dtype)
            if write_cache:
                state[row] = s
        return out


MIXERS.register("toy_decay", lambda spec, hidden_size: DecayMixer(spec, hidden_size))


# ------------------------------------------------------------------ a feed-forward with its own routing
@dataclass(frozen=True)
class SignRoutedSpec:
    kind: ClassVar[str] = "toy_sign_routed"
    intermediate_size: int = 16


class SignRoutedFFN(Part):
    """Two small MLPs; a token goes to the one named by the sign of ``x . probe`` (hard top-1)."""

    def __init__(self, spec: SignRoutedSpec, hidden_size: int):
        self.spec, self.hidden_size = spec, hidden_size

    def param_decls(self):
        i, h = self.spec.intermediate_size, self.hidden_size
        return {"probe": ParamDecl((h,), "float32"), "up": ParamDecl((2, i, h)), "down": ParamDecl((2, h, i))}

    def forward(self, fb, x):
        p = self.params
        choice = (x.float() @ p["probe"].float() > 0).long()                   # [T]
        if fb.taps is not None:
            fb.taps.setdefault("toy_sign", []).append(choice.clone())
        up, down = p["up"].float()[choice], p["down"].float()[choice]          # [T, i, h], [T, h, i]
        hidden = torch.nn.functional.silu(torch.einsum("tih,th->ti", up, x.float()))
        return torch.einsum("thi,ti->th", down, hidden).to(x.dtype)


FEED_FORWARDS.register("toy_sign_routed", lambda spec, hidden_size, chunk_tokens=0: SignRoutedFFN(spec, hidden_size))


# ------------------------------------------------------------------ a position encoding with its own table
@dataclass(frozen=True)
class LinearRotarySpec:
    kind: ClassVar[str] = "toy_linear_rotary"
    rotary_dim: int = 8
    slope: float = 0.05
    max_position: int = 1024


class LinearRotary(Part):
    """NeoX-paired rotation whose angle of pair d at position p is ``p * slope * (d + 1)``."""

    def __init__(self, spec: LinearRotarySpec, head_dim: int):
        self.spec, self.rotary_dim, self.table = spec, spec.rotary_dim, None

    def prepare(self, device) -> None:
        angles = linear_rotary_angles(torch.arange(self.spec.max_position), self.spec.rotary_dim, self.spec.slope)
        self.table = torch.cat((angles.cos(), angles.sin()), dim=-1).contiguous().to(device)

    def fused_rotation(self):
        return FusedRotation(self.table, self.rotary_dim, "neox")


def linear_rotary_angles(positions, rotary_dim: int, slope: float):
    return positions.float()[:, None] * (slope * torch.arange(1, rotary_dim // 2 + 1, dtype=torch.float32))[None, :]


POSITIONS.register("toy_linear_rotary", lambda spec, head_dim: LinearRotary(spec, head_dim))


# ------------------------------------------------------------------ a position encoding that is no rotation by a table
@dataclass(frozen=True)
class DecayGainSpec:
    kind: ClassVar[str] = "toy_decay_gain"
    rate: float = 0.02


class DecayGain(Part):
    """Queries grow and keys shrink with their position: dim ``d`` of every head is multiplied by
    ``exp(+-rate * p * (d % 4))``, so that a score depends on the distance of query and key alone.  It is no
    rotation and has no table: it applies itself (``fused_rotation`` is None), between the mixer's QK norm and
    its cache write."""

    def __init__(self, spec: DecayGainSpec, head_dim: int):
        self.spec, self.head_dim = spec, head_dim

    def prepare(self, device) -> None:
        self.step = (self.spec.rate * (torch.arange(self.head_dim) % 4).float()).to(device)

    def fused_rotation(self):
        return None

    def apply(self, fb, q, k, positions) -> None:
        q_gain, k_gain = decay_gains(positions, self.step)
        q.copy_((q.float() * q_gain[:, None, :]).to(q.dtype))
        k.copy_((k.float() * k_gain[:, None, :]).to(k.dtype))


def decay_gains(positions, step):
    exponent = positions.float()[:, None] * step[None, :]
    return torch.exp(exponent), torch.exp(-exponent)


POSITIONS.register("toy_decay_gain", lambda spec, head_dim: DecayGain(spec, head_dim))


# ------------------------------------------------------------------ a norm of another kind
@dataclass(frozen=True)
class MeanAbsNormSpec:
    """``y = z / (mean |z| + eps) * w``: the statistic is the mean magnitude, not the mean square."""
    kind: ClassVar[str] = "toy_mean_abs"
    eps: float = 1e-5


class MeanAbsNorm(Part):
    """The interface of a norm: ``forward(fb, x, out, residual)`` adds ``x`` into the residual first (the
    rounded sum becomes the residual, the unrounded sum is normed), ``forward_rows`` does it for chosen
    rows and writes nothing but ``out``.  Statistic and sum in float, like the engine's own."""

    def __init__(self, spec: MeanAbsNormSpec, hidden_size: int):
        self.eps, self.hidden_size = float(spec.eps), int(hidden_size)

    def param_decls(self):
        return {"weight": ParamDecl((self.hidden_size,))}

    def _norm(self, z):
        return z / (z.abs().mean(-1, keepdim=True) + self.eps) * self.params["weight"].float()

    def forward(self, fb, x, out=None, residual=None):
        out = x if out is None else out
        z = x.float()
        if residual is not None:
            z = z + residual.float()
            residual.copy_(z)
        out.copy_(self._norm(z))
        return out

    def forward_rows(self, fb, x, residual, rows, out):
        z = x[rows.long()].float()
        if residual is not None:
            z = z + residual[rows.long()].float()
        out.copy_(self._norm(z))
        return out


NORMS.register("toy_mean_abs", lambda spec, hidden_size: MeanAbsNorm(spec, hidden_size))


def mean_abs_norm(z, weight, eps):
    return z / (z.abs().mean(-1, keepdim=True) + eps) * weight


# ------------------------------------------------------------------ another arrangement of a layer
class SideBySideBlock(Part):
    """Mixer and feed-forward read the same normed stream and their results are added (one norm per layer),
    where the engine's own arrangement runs them one after the other with a norm each.  The pair
    ``(x, residual)`` it hands on means what it means everywhere: the stream is their sum, and the next
    norm adds them."""

    def __init__(self, spec: LayerSpec, hidden_size: int, chunk_tokens: int = 16384):
        self.norm = NORMS.build(spec.norm, hidden_size=hidden_size)
        self.mixer = MIXERS.build(spec.mixer, hidden_size=hidden_size)
        self.ffn = FEED_FORWARDS.build(spec.feed_forward, hidden_size=hidden_size, chunk_tokens=chunk_tokens)

    def children(self):
        return {"norm": self.norm, "mixer": self.mixer, "ffn": self.ffn}

    def cache_request(self):
        request = getattr(self.mixer, "cache_request", None)
        return request() if request else None

    def forward(self, fb, x, residual, cache_position: int, write_cache: bool):
        if residual is None:
            residual = fb.buffer("block.residual", x.shape)
            residual.copy_(x)
            u = self.norm.forward(fb, x)
        else:
            u = self.norm.forward(fb, x, residual=residual)
        mixed = self.mixer.forward(fb, u, cache_position, write_cache)
        both = fb.buffer("toy.side_by_side", mixed.shape)
        both.copy_(mixed)
        both += self.ffn.forward(fb, u)
        return both, residual


BLOCKS.register("toy_side_by_side", lambda spec, hidden_size, chunk_tokens=16384: SideBySideBlock(spec, hidden_size, chunk_tokens))


def neighbour_rope(x, cos, sin, rotary_dim: int):
    """Plain rotation of dims ``(2 j, 2 j + 1)`` of each head by angle ``j``; ``x [T, heads, D]``."""
    out = x.clone()
    even, odd = x[..., 0:rotary_dim:2], x[..., 1:rotary_dim:2]
    out[..., 0:rotary_dim:2] = even * cos[:, None, :] - odd * sin[:, None, :]
    out[..., 1:rotary_dim:2] = odd * cos[:, None, :] + even * sin[:, None, :]
    return out


# ------------------------------------------------------------------ the architecture
def parse(raw: dict) -> dict:
    return raw


def _layer_spec(cfg, layer) -> LayerSpec:
    h = cfg["hidden_size"]
    if layer["mixer"] == "decay":
        mixer = DecayMixerSpec(state_size=layer["state_size"], decay=layer["decay"])
    else:
        if layer.get("decay_gain"):
            rotary = DecayGainSpec(rate=layer["decay_gain"])
        elif layer.get("linear_rotary"):
            rotary = LinearRotarySpec(rotary_dim=layer["rotary_dim"], slope=layer["linear_rotary"],
                                      max_position=cfg["max_position_embeddings"])
        elif layer["rotary_dim"]:
            rotary = RotarySpec(rotary_dim=layer["rotary_dim"], theta=cfg["rope_theta"],
                                max_position=cfg["max_position_embeddings"], pairing=layer.get("pairing", "neox"))
        else:
            rotary = NoPositionSpec()
        mixer = AttentionSpec(num_heads=layer["heads"], num_kv_heads=layer["kv_heads"], head_dim=layer["head_dim"],
                              scale=layer["head_dim"] ** -0.5,
                              qk_norm={None: "none", False: "none", True: "flat"}.get(layer.get("qk_norm"), layer.get("qk_norm")),
                              qk_norm_eps=cfg["eps"], window=layer.get("window"), position=rotary,
                              kv_page_size=layer.get("page_size"))
    if layer["ffn"] == "dense":
        ffn = DenseMLPSpec(intermediate_size=layer["intermediate"], activation=layer.get("activation", "silu"))
    elif layer["ffn"] == "sign":
        ffn = SignRoutedSpec(intermediate_size=layer["intermediate"])
    else:
        ffn = MoESpec(num_experts=layer["experts"], top_k=layer["top_k"], intermediate_size=layer["intermediate"],
                      scoring=layer.get("scoring", "sigmoid"), selection_bias=layer.get("bias", True),
                      norm_topk_prob=layer.get("normalize", True), routed_scaling_factor=layer.get("scaling", 1.0),
                      activation=layer.get("activation", "silu"))
    norm = MeanAbsNormSpec(eps=cfg["eps"]) if layer.get("norm") == "mean_abs" else NormSpec(eps=cfg["eps"])
    return LayerSpec(mixer=mixer, feed_forward=ffn, norm=norm, block=layer.get("block", "prenorm"))


def build_spec(cfg) -> ModelSpec:
    layers = tuple(_layer_spec(cfg, layer) for layer in cfg["layers"])
    schedule = tuple(ScheduleEntry(e["layer"], e.get("cache_from")) for e in cfg["schedule"])
    return ModelSpec(architecture="ToyForCausalLM", hidden_size=cfg["hidden_size"], vocab_size=cfg["vocab_size"],
                     layers=layers, schedule=schedule, final_norm=NormSpec(eps=cfg["eps"]),
                     max_position=cfg["max_position_embeddings"],
                     constants=(("embedding_multiplier", float(cfg.get("embedding_multiplier", 1.0))),
                                ("logit_scale", float(cfg.get("logit_scale", 1.0)))))


class ToyModel(DecoderModel):
    """The generic decoder with other ends: the embedding is multiplied by a constant and the logits are
    scaled (named by ``Architecture.model_factory``; the run of the schedule is the framework's)."""

    def embed_tokens(self, fb):
        return super().embed_tokens(fb).mul_(dict(self.spec.constants)["embedding_multiplier"])

    def logits_of(self, fb, last):
        return super().logits_of(fb, last).float() * dict(self.spec.constants)["logit_scale"]


def weight_sources(cfg):
    """Checkpoint names are the parameter paths with a ``toy.`` prefix, tensor for tensor."""
    return [WeightSource("toy." + path, path) for path in ToyModel(build_spec(cfg)).all_param_decls()]


def random_tensor(cfg, name, shape, generator, options):
    noise = torch.randn(tuple(shape), generator=generator, dtype=torch.float32, device=generator.device)
    if "norm" in name and name.endswith("weight"):
        return 1.0 + 0.2 * noise
    if name.endswith("router_bias"):
        return 0.3 * noise
    if name.endswith("probe"):
        return noise
    return noise * float(options.get("std", 0.1))


TOY = register_architecture(Architecture(
    name="ToyForCausalLM", model_types=("toy",), parse_config=parse, build_spec=build_spec,
    weight_sources=weight_sources, ignored_tensor=lambda name: False, random_tensor=random_tensor,
    stored_dtype=lambda name: "float32" if name.endswith(("router", "router_bias", "probe")) else "bfloat16",
    config_to_dict=lambda cfg: dict(cfg), model_factory=lambda spec, chunk_tokens=16384: ToyModel(spec, chunk_tokens)))

TOY_CONFIG = dict(
    architectures=["ToyForCausalLM"], model_type="toy", hidden_size=64, vocab_size=300, eps=1e-5, rope_theta=10000.0,
    max_position_embeddings=1024, embedding_multiplier=1.5, logit_scale=0.5,
    layers=[
        dict(mixer="attention", heads=4, kv_heads=2, head_dim=32, rotary_dim=16, pairing="interleaved", qk_norm=True,
             ffn="dense", intermediate=96),
        dict(mixer="decay", state_size=12, decay=0.8, ffn="moe", experts=6, top_k=2, intermediate=40, scoring="softmax",
             bias=False, normalize=False, scaling=1.5),
        # a window of 24 keys on pages of 8 tokens (the other groups take the engine's page size)
        # (its QK norm has one statistic per head and weights of one head's size)
        dict(mixer="attention", heads=6, kv_heads=2, head_dim=32, rotary_dim=32, window=24, page_size=8, qk_norm="per_head",
             ffn="moe", experts=4, top_k=3, intermediate=24, activation="gelu_tanh"),
        dict(mixer="attention", heads=2, kv_heads=2, head_dim=32, rotary_dim=0, decay_gain=0.004, qk_norm=True, ffn="dense",
             intermediate=48, activation="gelu_tanh", norm="mean_abs"),
        # (layer 0 turns neighbouring dims together, the others dims half a rotary width apart)
        dict(mixer="attention", heads=4, kv_heads=2, head_dim=32, rotary_dim=8, linear_rotary=0.05, ffn="sign",
             intermediate=20),
        # mixer and feed-forward side by side behind one norm of the other kind
        dict(mixer="attention", heads=2, kv_heads=1, head_dim=32, rotary_dim=0, decay_gain=0.003, qk_norm="per_head", ffn="dense",
             intermediate=32, norm="mean_abs", block="toy_side_by_side"),
    ],
    # layer 0 runs twice (two caches); position 4 reads the cache of position 0 (same geometry)
    schedule=[dict(layer=0), dict(layer=1), dict(layer=2), dict(layer=0), dict(layer=3, cache_from=0), dict(layer=5),
              dict(layer=4)])


# ------------------------------------------------------------------ its plain implementation
def per_head_qk_norm(x: torch.Tensor, weight: torch.Tensor, eps: float, head_dim: int) -> torch.Tensor:
    """RMS norm of every head by itself, one weight vector of a head's size for all heads
    (the reference's dense attention, models/qwen3.py:116-118,151-153: ``RMSNorm(head_dim)`` on ``[T, heads, D]``)."""
    heads = x.view(x.shape[0], -1, head_dim)
    return (heads * torch.rsqrt(heads.square().mean(-1, keepdim=True) + eps) * weight).reshape(x.shape)


class PlainToy:
    def __init__(self, folder: str):
        import json, os
        from safetensors.torch import load_file
        self.cfg = json.load(open(os.path.join(folder, "config.json")))
        self.w = {k[4:]: v.float() for k, v in load_file(os.path.join(folder, "model.safetensors")).items()}

    def logits(self, tokens, forced=None):
        """``forced``: {"router": [ids [T, k] per routed layer in run order], "sign": [choice [T] per
        sign-routed layer]}: the choices of a run in reduced precision, whose near-ties may tip."""
        cfg, w = self.cfg, self.w
        forced = forced or {}
        routers, signs = iter(forced.get("router", [])), iter(forced.get("sign", []))
        T = len(tokens)
        pos = torch.arange(T)
        x = w["embed.weight"][torch.as_tensor(tokens)] * cfg.get("embedding_multiplier", 1.0)
        residual = None
        kv_of = {}
        for position, entry in enumerate(cfg["schedule"]):
            i, layer = entry["layer"], cfg["layers"][entry["layer"]]
            p = f"layers.{i}."
            side_by_side = layer.get("block") == "toy_side_by_side"
            norm = (lambda z, wt: mean_abs_norm(z, wt, cfg["eps"])) if layer.get("norm") == "mean_abs" else \
                (lambda z, wt: P.rms_norm(z, wt, cfg["eps"]))
            first_norm = w[p + ("norm.weight" if side_by_side else "norm_mixer.weight")]
            residual = x if residual is None else x + residual
            u = norm(residual, first_norm)
            if layer["mixer"] == "decay":
                s = torch.zeros(layer["state_size"])
                a = torch.empty_like(u)
                for t in range(T):
                    s = layer["decay"] * s + w[p + "mixer.w_in"] @ u[t]
                    a[t] = w[p + "mixer.w_out"] @ s
            else:
                H, Hkv, D, R = layer["heads"], layer["kv_heads"], layer["head_dim"], layer["rotary_dim"]
                qkv = u @ w[p + "mixer.qkv"].T
                q, k, v = qkv[:, :H * D], qkv[:, H * D:(H + Hkv) * D], qkv[:, (H + Hkv) * D:]
                if layer.get("qk_norm") == "per_head":       # every head of a token by its own root mean square
                    q = per_head_qk_norm(q, w[p + "mixer.q_norm"], cfg["eps"], D)
                    k = per_head_qk_norm(k, w[p + "mixer.k_norm"], cfg["eps"], D)
                elif layer.get("qk_norm"):
                    q = P.flat_qk_norm(q, w[p + "mixer.q_norm"], cfg["eps"])
                    k = P.flat_qk_norm(k, w[p + "mixer.k_norm"], cfg["eps"])
                q, k, v = q.reshape(T, H, D), k.reshape(T, Hkv, D), v.reshape(T, Hkv, D)
                if layer.get("decay_gain"):
                    q_gain, k_gain = decay_gains(pos, layer["decay_gain"] * (torch.arange(D) % 4).float())
                    q, k = q * q_gain[:, None, :], k * k_gain[:, None, :]
                elif layer.get("linear_rotary"):
                    angles = linear_rotary_angles(pos, R, layer["linear_rotary"])
                    q, k = P.partial_rope(q, angles.cos(), angles.sin(), R), P.partial_rope(k, angles.cos(), angles.sin(), R)
                elif R and layer.get("pairing") == "interleaved":
                    cos, sin = P.rope_angles(pos, R, cfg["rope_theta"])
                    q, k = neighbour_rope(q, cos, sin, R), neighbour_rope(k, cos, sin, R)
                elif R:
                    cos, sin = P.rope_angles(pos, R, cfg["rope_theta"])
                    q, k = P.partial_rope(q, cos, sin, R), P.partial_rope(k, cos, sin, R)
                if entry.get("cache_from") is not None:
                    k, v = kv_of[entry["cache_from"]]            # reads another position's keys and values
                else:
                    kv_of[position] = (k, v)
                a = P.causal_gqa_attention(q, k, v, D ** -0.5, window=layer.get("window")).reshape(T, -1) @ w[p + "mixer.o"].T
            if side_by_side:
                m = u                          # the feed-forward reads what the mixer read
            else:
                residual = a + residual
                m = norm(residual, w[p + "norm_ffn.weight"])
            I = layer["intermediate"]
            gelu = layer.get("activation") == "gelu_tanh"
            if layer["ffn"] == "dense":
                gu = m @ w[p + "ffn.gate_up"].T
                gate = torch.nn.functional.gelu(gu[:, :I], approximate="tanh") if gelu else torch.nn.functional.silu(gu[:, :I])
                x = (gate * gu[:, I:]) @ w[p + "ffn.down"].T
            elif layer["ffn"] == "sign":
                choice = next(signs, None)
                if choice is None:
                    choice = (m @ w[p + "ffn.probe"] > 0).long()
                x = torch.stack([w[p + "ffn.down"][int(c)] @ torch.nn.functional.silu(w[p + "ffn.up"][int(c)] @ t)
                                 for t, c in zip(m, choice)])
            else:
                logits = m @ w[p + "ffn.router"].T
                scores = torch.softmax(logits, -1) if layer.get("scoring") == "softmax" else torch.sigmoid(logits)
                sel = scores + w[p + "ffn.router_bias"] if layer.get("bias", True) else scores
                ids = next(routers, None)
                if ids is None:
                    ids = torch.topk(sel, layer["top_k"], dim=-1).indices
                wts = scores.gather(1, ids)
                if layer.get("normalize", True):
                    wts = wts / wts.sum(-1, keepdim=True)
                wts = wts * layer.get("scaling", 1.0)
                if gelu:      # the routed sum spelled out: the plain helper knows silu only
                    x = torch.zeros_like(m)
                    for t in range(T):
                        for e, wt in zip(ids[t].tolist(), wts[t]):
                            gate = torch.nn.functional.gelu(w[p + "ffn.w13"][e, :I] @ m[t], approximate="tanh")
                            x[t] += wt * (w[p + "ffn.w2"][e] @ (gate * (w[p + "ffn.w13"][e, I:] @ m[t])))
                else:
                    x = P.swiglu_experts(m, w[p + "ffn.w13"][:, :I], w[p + "ffn.w13"][:, I:], w[p + "ffn.w2"], ids, wts)
            if side_by_side:
                x = a + x
        y, _ = P.add_rms_norm(x, residual, w["final_norm.weight"], cfg["eps"])
        return (y @ w["head.weight"].T) * cfg.get("logit_scale", 1.0)
