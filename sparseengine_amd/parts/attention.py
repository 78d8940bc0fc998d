"""Causal grouped-query attention over the paged cache.

Order inside the mixer, as in the reference (models/minimax_m2.py:334-359): merged q/k/v
projection -> QK RMSNorm (optional: flat, over the whole q row and the whole k row, which is MiniMax M2's; or
per head with weights of one head's size, models/qwen3.py:116-118,151-153) -> rotation of
the leading rotary dims of every head -> k (normed, rotated) and v written to this step's slots
-> attention of the step's queries over everything the request has cached, its own tokens
included -> output projection.  Norm, rotation and the cache write are one kernel when the position
part is a rotation by a table (``fused_rotation()`` hands the kernel its arguments); a position part
that is something else returns None there and has ``apply(fb, q, k, positions)``, which changes
``q [T, heads, D]`` and ``k [T, kv_heads, D]`` in place between the norm and the cache write.
"""
from __future__ import annotations

from ..config.specs import AttentionSpec
from .base import MIXERS, POSITIONS, PagedKVRequest, ParamDecl, Part
from .linear import linear, prepare


class GQAAttention(Part):
    kernel_libraries = ("rope_kv", "attention_generic", "attention_mfma", "host_work")

    def __init__(self, spec: AttentionSpec, hidden_size: int):
        if spec.num_kv_heads <= 0 or spec.num_heads % spec.num_kv_heads:
            raise ValueError(f"{spec.num_heads} query heads do not divide into {spec.num_kv_heads} kv heads")
        if spec.head_dim % 16:
            raise ValueError(f"head_dim must be a multiple of 16, got {spec.head_dim}")
        if spec.qk_norm not in ("none", "flat", "per_head"):
            raise ValueError(f"qk_norm {spec.qk_norm!r} is unknown (none, flat, per_head)")
        self.spec = spec
        self.hidden_size = int(hidden_size)
        self.q_width = spec.num_heads * spec.head_dim
        self.kv_width = spec.num_kv_heads * spec.head_dim
        self.position = POSITIONS.build(spec.position, head_dim=spec.head_dim)
        self._prepared = {"qkv": None, "o": None}

    def param_decls(self):
        decls = {"qkv": ParamDecl((self.q_width + 2 * self.kv_width, self.hidden_size)),
                 "o": ParamDecl((self.hidden_size, self.q_width))}
        if self.spec.qk_norm == "flat":
            decls["q_norm"] = ParamDecl((self.q_width,))
            decls["k_norm"] = ParamDecl((self.kv_width,))
        elif self.spec.qk_norm == "per_head":
            decls["q_norm"] = ParamDecl((self.spec.head_dim,))
            decls["k_norm"] = ParamDecl((self.spec.head_dim,))
        return decls

    def limit_positions(self, positions: int) -> None:
        limit = getattr(self.position, "limit_positions", None)     # a position part of the tests may not have it
        if limit is not None:
            limit(positions)

    def bind(self, params):
        super().bind(params)
        self.position.prepare(params["qkv"].device)

    def finalize(self, kernels) -> None:
        self._prepared = {name: prepare(kernels, self.params[name]) for name in ("qkv", "o")}

    def work_key(self):
        """(query heads per kv head, window): what the attention kernel's work list depends on."""
        return self.spec.num_heads // self.spec.num_kv_heads, int(self.spec.window or 0)

    def cache_request(self):
        return PagedKVRequest(self.spec.num_kv_heads, self.spec.head_dim, self.spec.window, self.spec.kv_page_size)

    def forward(self, fb, x, cache_position: int, write_cache: bool = True):
        s, p, T = self.spec, self.params, x.shape[0]
        cache, meta = fb.kv_view(cache_position)
        qkv = linear(x, p["qkv"], out=fb.buffer("attn.qkv", (T, self.q_width + 2 * self.kv_width)), kernels=fb.kernels,
                     prepared=self._prepared["qkv"])
        q = qkv[:, :self.q_width].view(T, s.num_heads, s.head_dim)
        rotation = self.position.fused_rotation()
        store = (cache, meta.slots) if write_cache else (None, None)
        per_head = s.qk_norm == "per_head"
        if rotation is not None:      # a rotation by a table: norm, rotation and cache write in one launch
            fb.kernels.qk_norm_rope_store(
                qkv, meta.positions, rotation.table, p.get("q_norm"), p.get("k_norm"), s.qk_norm_eps,
                s.num_heads, s.num_kv_heads, s.head_dim, rotation.rotary_dim, *store, meta.page_size,
                pairing=rotation.pairing, per_head_norm=per_head)
        else:                         # the position part applies itself, between the norm and the cache write
            if "q_norm" in p:
                fb.kernels.qk_norm_rope_store(qkv, meta.positions, None, p["q_norm"], p["k_norm"], s.qk_norm_eps,
                                              s.num_heads, s.num_kv_heads, s.head_dim, 0, None, None, meta.page_size,
                                              per_head_norm=per_head)
            k = qkv[:, self.q_width:self.q_width + self.kv_width].view(T, s.num_kv_heads, s.head_dim)
            self.position.apply(fb, q, k, meta.positions)
            if write_cache:
                fb.kernels.qk_norm_rope_store(qkv, meta.positions, None, None, None, s.qk_norm_eps, s.num_heads,
                                              s.num_kv_heads, s.head_dim, 0, *store, meta.page_size)
        attended = fb.buffer("attn.out", (T, self.q_width))
        method = getattr(fb, "method", None)
        visible = meta if method is None else method.select(cache_position, meta)     # what this layer may read
        if getattr(fb, "check_tables", False):
            fb.check_block_table(visible, s.window or 0, cache.shape[0], f"schedule position {cache_position}")
        fb.kernels.paged_attention(q, cache, visible, attended, s.scale, s.window or 0)
        if method is not None:
            method.after_attention(cache_position, fb)
        if fb.taps is not None:
            fb.taps.setdefault("attention_inputs", []).append(qkv.clone())
        return linear(attended, p["o"], out=fb.buffer("attn.proj", (T, self.hidden_size)), kernels=fb.kernels,
                      prepared=self._prepared["o"])


MIXERS.register("gqa_attention", lambda spec, hidden_size: GQAAttention(spec, hidden_size))
