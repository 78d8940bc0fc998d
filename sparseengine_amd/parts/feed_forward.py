"""Feed-forward parts: routed SwiGLU experts and a dense gated MLP.

Routed experts, as the reference computes them (models/minimax_m2.py:140-172,212-269;
kernels/triton/moe_biased_sigmoid.py:202-238; kernels/triton/moe.py:1311-1440): router logits
in float32 from float32 weights; score = sigmoid (or softmax); experts picked by score + bias,
weights are the unbiased scores of the picked experts, renormalised; each (token, slot) runs
``W2_e(silu(W1_e x) * W3_e x)`` times its weight; the slots of a token are summed in float.
"""
from __future__ import annotations

import torch

from ..config.specs import DenseMLPSpec, MoESpec
from .base import FEED_FORWARDS, ParamDecl, Part, SlotSum
from .linear import linear, prepare


ACTIVATIONS = ("silu", "gelu_tanh")      # what the kernels' epilogues can apply to a gate


def forced_experts(fb):
    """Measurement and test seam, kept in this one place: ``fb.forced_routing`` holds, by schedule position
    (a list, or a dict that names some positions), the experts ``[T, top_k]`` that every token of the step
    is to take at that position's routed feed-forward; ``fb.schedule_position`` is the position that runs.
    Nothing in the product sets it."""
    given = getattr(fb, "forced_routing", None)
    if given is None:
        return None
    position = getattr(fb, "schedule_position", 0)
    if isinstance(given, dict):
        return given.get(position)
    return given[position] if position < len(given) else None


class RoutedExperts(Part):
    kernel_libraries = ("moe", "moe_mfma")

    def __init__(self, spec: MoESpec, hidden_size: int, chunk_tokens: int = 16384):
        if not 1 <= spec.top_k <= spec.num_experts:
            raise ValueError(f"top_k must be in [1, num_experts={spec.num_experts}], got {spec.top_k}")
        if spec.activation not in ACTIVATIONS:
            raise NotImplementedError(f"expert activation {spec.activation!r} is not supported ({', '.join(ACTIVATIONS)})")
        if spec.scoring not in ("sigmoid", "softmax"):
            raise NotImplementedError(f"router scoring {spec.scoring!r} is not supported (sigmoid, softmax)")
        self.spec = spec
        self.hidden_size = int(hidden_size)
        self.chunk_tokens = int(chunk_tokens)
        self._workspace = None
        self._tiled = False

    def param_decls(self):
        s = self.spec
        decls = {"router": ParamDecl((s.num_experts, self.hidden_size), "float32"),
                 "w13": ParamDecl((s.num_experts, 2 * s.intermediate_size, self.hidden_size)),
                 "w2": ParamDecl((s.num_experts, self.hidden_size, s.intermediate_size))}
        if s.selection_bias:
            decls["router_bias"] = ParamDecl((s.num_experts,), "float32")
        return decls

    def finalize(self, kernels) -> None:
        """The matrix-core expert kernels read the tables in tiles laid out for their operand loads;
        kernels that have such a layout put the tables into it here, once."""
        arrange = getattr(kernels, "arrange_expert_weights", None)
        if arrange is not None:
            self._tiled = bool(arrange(self.params["w13"], self.params["w2"]))

    def _workspace_for(self, fb, tokens: int, dtype):
        """The scratch tensors of the expert pipeline: the kernels object makes them (their shape is its
        kernels' business); they are kept with the step's other scratch and made anew when they do not fit."""
        s = self.spec
        ws = fb.scratch.tensors.get("moe.workspace")
        if ws is None or not ws.fits(tokens, s.top_k, s.num_experts, self.hidden_size, s.intermediate_size, dtype):
            ws = fb.kernels.make_moe_workspace(max(tokens, 1), s.top_k, s.num_experts, self.hidden_size,
                                               s.intermediate_size, dtype, fb.device)
            fb.scratch.tensors["moe.workspace"] = ws
        return ws

    can_defer_slot_sum = True

    def forward(self, fb, x, defer_slot_sum: bool = False):
        """``defer_slot_sum``: the reader accepts a ``SlotSum``; it gets one when the step is a single
        chunk of no more tokens than the kernels object says the hand-over pays for
        (``slot_sum_deferral_tokens``: 0 or absent, never)."""
        s, p, T = self.spec, self.params, x.shape[0]
        out = fb.buffer("ffn.out", (T, self.hidden_size))
        forced = forced_experts(fb)
        if (defer_slot_sum and T <= int(getattr(fb.kernels, "slot_sum_deferral_tokens", 0))
                and p["w13"].dtype == x.dtype):
            return SlotSum(self._forward_chunk(fb, x, out, forced, sum_slots=False), s.top_k)
        for start in range(0, T, self.chunk_tokens):
            stop = min(T, start + self.chunk_tokens)
            self._forward_chunk(fb, x[start:stop], out[start:stop], None if forced is None else forced[start:stop])
        return out

    def _force(self, logits, forced, ids, weights):
        """Measurement and test seam (``forced_experts``): the router's choice is replaced, the weights
        are the chosen experts' own scores as the router would have weighted them.  A run in reduced
        precision can so be compared with one in float32 expert for expert, and a benchmark can
        spread its tokens evenly over the experts; nothing in the product sets it."""
        s = self.spec
        scores = torch.sigmoid(logits) if s.scoring == "sigmoid" else torch.softmax(logits, dim=-1)
        ids.copy_(forced)
        chosen = scores.gather(1, forced.long())
        if s.norm_topk_prob:
            chosen = chosen / chosen.sum(-1, keepdim=True)
        weights.copy_(chosen * s.routed_scaling_factor)

    def _forward_chunk(self, fb, x, out, forced=None, sum_slots: bool = True):
        s, p, T = self.spec, self.params, x.shape[0]
        logits = fb.buffer("moe.logits", (T, s.num_experts), torch.float32)
        ids = fb.buffer("moe.ids", (T, s.top_k), torch.int32)
        weights = fb.buffer("moe.weights", (T, s.top_k), torch.float32)
        w13, w2 = p["w13"], p["w2"]
        ws = self._workspace_for(fb, T, w13.dtype)
        fb.kernels.route(x, p["router"], p.get("router_bias"), s.top_k, logits, ids, weights, scoring=s.scoring,
                         normalize=s.norm_topk_prob, scaling=s.routed_scaling_factor, workspace=ws)
        if forced is not None:
            self._force(logits, forced, ids, weights)
            ws.grouped = None          # whatever the router's launch grouped were its own choices
        if fb.taps is not None:
            fb.taps.setdefault("router", []).append((ids.clone(), weights.clone()))
        if not sum_slots:
            return fb.kernels.moe_experts(x, w13, w2, ids, weights, out, ws, tiled=self._tiled, sum_slots=False,
                                          activation=s.activation)
        if w13.dtype == x.dtype:
            fb.kernels.moe_experts(x, w13, w2, ids, weights, out, ws, tiled=self._tiled, activation=s.activation)
        else:   # expert weights kept in float32 under a bfloat16 engine
            x32 = x.float()
            out32 = torch.empty_like(x32)
            fb.kernels.moe_experts(x32, w13, w2, ids, weights, out32, ws, activation=s.activation)
            out.copy_(out32)


class DenseMLP(Part):
    """``down(act(gate x) * up x)``; ``gate_up`` holds the gate rows, then the up rows."""
    kernel_libraries = ("moe",)

    def __init__(self, spec: DenseMLPSpec, hidden_size: int, chunk_tokens: int = 16384):
        if spec.activation not in ACTIVATIONS:
            raise NotImplementedError(f"activation {spec.activation!r} is not supported ({', '.join(ACTIVATIONS)})")
        self.spec = spec
        self.hidden_size = int(hidden_size)
        self._prepared = {"gate_up": None, "down": None}

    def finalize(self, kernels) -> None:
        self._prepared = {name: prepare(kernels, self.params[name]) for name in ("gate_up", "down")}

    def param_decls(self):
        i = self.spec.intermediate_size
        return {"gate_up": ParamDecl((2 * i, self.hidden_size)), "down": ParamDecl((self.hidden_size, i))}

    def forward(self, fb, x):
        T, i = x.shape[0], self.spec.intermediate_size
        gate_up = linear(x, self.params["gate_up"], out=fb.buffer("mlp.gate_up", (T, 2 * i)), kernels=fb.kernels,
                         prepared=self._prepared["gate_up"])
        act = fb.buffer("mlp.act", (T, i))
        fb.kernels.silu_mul(gate_up, act, activation=self.spec.activation)
        return linear(act, self.params["down"], out=fb.buffer("ffn.out", (T, self.hidden_size)), kernels=fb.kernels,
                      prepared=self._prepared["down"])


FEED_FORWARDS.register("moe", lambda spec, hidden_size, chunk_tokens=16384: RoutedExperts(spec, hidden_size, chunk_tokens))
FEED_FORWARDS.register("dense_mlp", lambda spec, hidden_size, chunk_tokens=16384: DenseMLP(spec, hidden_size, chunk_tokens))
