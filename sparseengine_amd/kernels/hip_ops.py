"""Python face of the HIP kernels: shape checks on the host, then one ctypes call per kernel.

All tensors live on the GPU; every call goes to the current stream and allocates nothing
unless it says so.  A wrong shape or dtype raises ``ValueError`` before anything is launched;
a size a kernel does not take raises ``KernelShapeError`` naming the limit.
"""
from __future__ import annotations

import ctypes
from ctypes import c_float, c_int, c_int64, c_void_p

import torch

from . import library

_DTYPE_CODE = {torch.float32: 0, torch.bfloat16: 1}


class KernelShapeError(ValueError):
    pass


def _code(dtype: torch.dtype) -> int:
    try:
        return _DTYPE_CODE[dtype]
    except KeyError:
        raise ValueError(f"kernels take float32 or bfloat16 storage, got {dtype}") from None


def _ptr(t: torch.Tensor | None):
    return None if t is None else t.data_ptr()


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)


def _stream():
    """Handle of the current device's current stream.  A decode step makes a few hundred launches;
    the tensor library's public accessor builds a stream object for each call and costs as much
    as a small kernel runs, its raw accessor does not."""
    if _raw_stream is not None:
        return _raw_stream(torch.cuda.current_device())
    return torch.cuda.current_stream().cuda_stream


def _check(status: int, what: str, takes: str = ""):
    if status == 0:
        return
    if status == -1:
        raise KernelShapeError(f"{what}: the kernel refuses these sizes" + (f" (it takes {takes})" if takes else ""))
    raise RuntimeError(f"{what}: kernel launch failed (status {status})")


def _require(cond: bool, message: str):
    if not cond:
        raise ValueError(message)


def _i32(t: torch.Tensor, name: str):
    _require(t.dtype == torch.int32 and t.is_contiguous(), f"{name} must be contiguous int32")


_SIGNATURES = {
    "norm": {
        "se_embedding": [c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_void_p],
        "se_rms_norm": [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_float,
                        c_int64, c_int64, c_int64, c_int, c_int, c_int, c_int, c_void_p],
        "se_rms_norm_slots": [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_float,
                              c_int64, c_int64, c_int64, c_int, c_int, c_int, c_int, c_int, c_void_p],
    },
    "rope_kv": {
        "se_qk_norm_rope_store": [c_void_p, c_int64, c_void_p, c_void_p, c_void_p, c_void_p, c_float,
                                  c_int, c_int, c_int, c_int, c_int, c_void_p, c_void_p, c_int,
                                  c_int, c_int, c_int, c_int, c_int, c_int, c_void_p],
    },
    "attention_generic": {
        "se_paged_attention_generic": [c_void_p, c_int64, c_void_p, c_void_p, c_int, c_void_p,
                                       c_void_p, c_void_p, c_int64, c_int, c_int, c_int, c_int,
                                       c_int, c_float, c_int, c_int, c_void_p],
    },
    "attention_mfma": {
        # q, q_stride, cache, block_table, bt_stride, units, num_units, tasks, num_tasks, out, out_stride,
        # part_o, part_ml, heads, kv_heads, head_dim, page_size, scale, window, stream
        "se_paged_attention_mfma": [c_void_p, c_int64, c_void_p, c_void_p, c_int, c_void_p, c_int, c_void_p,
                                    c_int, c_void_p, c_int64, c_void_p, c_void_p, c_int, c_int, c_int, c_int,
                                    c_float, c_int, c_void_p],
        # q, q_stride, cache, block_table, bt_stride, units, num_units, out, out_stride, part_o, part_ml,
        # heads, kv_heads, head_dim, page_size, scale, window, tiles_per_block, stream
        "se_paged_attention_tiled": [c_void_p, c_int64, c_void_p, c_void_p, c_int, c_void_p, c_int, c_void_p,
                                     c_int64, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_float, c_int,
                                     c_int, c_void_p],
    },
    "moe": {
        "se_router_topk": [c_void_p, c_int64, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int,
                           c_int, c_int, c_float, c_void_p],
        "se_router_logits": [c_void_p, c_int64, c_void_p, c_void_p, c_int64, c_int, c_int, c_int, c_int,
                             c_void_p],
        "se_router_topk_align": [c_void_p, c_int64, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int,
                                 c_int, c_float, c_int, c_void_p, c_void_p, c_void_p, c_void_p],
        "se_moe_align": [c_void_p, c_int, c_int, c_int, c_void_p, c_void_p, c_void_p, c_void_p],
        "se_moe_align_choice": [c_void_p, c_int, c_int, c_int, c_int, c_int, c_int, c_void_p, c_void_p, c_void_p, c_void_p],
        "se_grouped_gemm_generic": [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p,
                                    c_void_p, c_int, c_int, c_int, c_int, c_int, c_int, c_int, c_int,
                                    c_void_p],
        "se_moe_sum": [c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_void_p],
        "se_silu_mul": [c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_void_p],
    },
    "moe_mfma": {
        "se_grouped_gemm_mfma": [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p,
                                 c_int, c_int, c_int, c_int, c_int, c_int, c_int, c_int, c_int, c_void_p],
        "se_skinny_gemm_mfma": [c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_void_p],
        "se_grouped_gemm_tall": [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p,
                                 c_int, c_int, c_int, c_int, c_int, c_int, c_int, c_int, c_void_p],
        "se_grouped_gemm_wide": [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p,
                                 c_int, c_int, c_int, c_int, c_int, c_int, c_int, c_int, c_void_p],
        "se_grouped_gemm_mid": [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p,
                                c_int, c_int, c_int, c_int, c_int, c_int, c_int, c_int, c_void_p],
        "se_grouped_gemm_choice": [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p,
                                   c_int, c_int, c_int, c_int, c_int, c_int, c_int, c_void_p],
    },
    "memory_probe": {
        "se_stream_read": [c_void_p, c_int64, c_void_p, c_int, c_void_p],
        "se_stream_copy": [c_void_p, c_void_p, c_int64, c_int, c_void_p],
    },
    "sampling": {
        "se_sample": [c_void_p, c_int64, c_int, c_int, c_void_p, c_void_p, c_void_p, c_void_p,
                      c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p],
        "se_sample_unfiltered": [c_void_p, c_int64, c_int, c_int, c_void_p, c_void_p, c_void_p, c_void_p,
                                 c_void_p, c_void_p],
    },
}


class _Functions:
    """Lazy table of bound entry points; a library is loaded (and built) at its first use."""

    def __init__(self):
        self._cache = {}

    def get(self, lib_name: str, fn_name: str):
        key = (lib_name, fn_name)
        fn = self._cache.get(key)
        if fn is None:
            lib = library.load(lib_name)
            fn = getattr(lib, fn_name)
            fn.argtypes = _SIGNATURES[lib_name][fn_name]
            fn.restype = c_int
            self._cache[key] = fn
        return fn


_fn = _Functions()

# The calls a decode step makes hundreds of times take a short way through their checks (one expression each); a call
# that fails one of them, and every other kind of call, takes the long way, which names what is wrong.  The tests
# switch the short ways off to see that both pass the same arguments to the same entry points.
_SHORT_WAYS = True


def moe_tile_bounds(assignments: int, experts: int, tile_rows: int) -> tuple[int, int]:
    """(capacity of the sorted list, largest possible number of tiles) for an alignment."""
    touched = min(experts, assignments)
    return assignments + touched * (tile_rows - 1), assignments // tile_rows + touched


class MoeWorkspace:
    """Scratch tensors of the expert pipeline, sized for a largest number of tokens."""

    TILE_ROWS = (16, 32, 64, 96, 128)      # alignments the expert kernels may ask for

    def __init__(self, max_tokens: int, top_k: int, experts: int, hidden: int, intermediate: int,
                 dtype: torch.dtype, device):
        assignments = max_tokens * top_k
        bounds = [moe_tile_bounds(assignments, experts, rows) for rows in self.TILE_ROWS]
        capacity, max_tiles = max(b[0] for b in bounds), max(b[1] for b in bounds)
        self.max_tokens, self.top_k, self.experts = max_tokens, top_k, experts
        self.hidden, self.intermediate, self.dtype = hidden, intermediate, dtype
        self.sorted = torch.empty(capacity, dtype=torch.int32, device=device)
        self.tile_expert = torch.empty(max_tiles, dtype=torch.int32, device=device)
        self.counters = torch.zeros(4, dtype=torch.int32, device=device)     # tiles, sorted entries, the device's choice
        self.grouped = None      # set by router_topk when its launch has grouped the assignments already
        # rows by assignment, or (the direct kernel) by sorted position, padding included
        self.act = torch.empty(capacity, intermediate, dtype=dtype, device=device)
        self.slot_out = torch.empty(assignments, hidden, dtype=dtype, device=device)

    def fits(self, tokens, top_k, experts, hidden, intermediate, dtype) -> bool:
        return (tokens <= self.max_tokens and top_k == self.top_k and experts == self.experts
                and hidden == self.hidden and intermediate == self.intermediate and dtype == self.dtype)


class HipKernels:
    """The kernel interface of the engine, served by the gfx950 libraries."""

    libraries = ("norm", "rope_kv", "attention_generic", "attention_mfma", "moe", "moe_mfma", "sampling",
                 "host_work", "memory_probe")

    def __init__(self):
        if not torch.cuda.is_available():
            raise library.KernelLibraryError(
                "the HIP kernels need a GPU: torch.cuda.is_available() is False")
        self._attention_partials = None      # (float32 O partials, float32 max/sum partials)
        self._sample_partials = None         # (float32 values, int32 indices) of the partial arg-max

    # ------------------------------------------------------------------ embedding / norms
    def embedding(self, ids: torch.Tensor, table: torch.Tensor, out: torch.Tensor):
        _i32(ids, "ids")
        tokens, hidden = out.shape
        _require(ids.numel() == tokens and table.shape[1] == hidden and table.is_contiguous()
                 and out.is_contiguous(), "embedding: shape mismatch")
        _require(table.dtype == out.dtype or table.dtype == torch.float32, "embedding: table dtype")
        _check(_fn.get("norm", "se_embedding")(_ptr(ids), _ptr(table), _ptr(out), tokens, hidden,
                                               _code(out.dtype), _code(table.dtype), _stream()), "embedding")

    # rms_norm(slots=...) and moe_experts(sum_slots=False): the sum over a token's expert slots can be
    # left to the norm that reads the feed-forward's result (one launch and one pass over memory fewer
    # per layer); parts ask this flag before they hand a SlotSum on.
    # Up to this many tokens in a step.  Measured on MI355X at hidden 3072 with eight slots: the norm that
    # adds the slots up saves a launch in a decode step (batch 8: 5.96 -> 5.93 ms) and loses against the two
    # kernels from a few hundred tokens on (a 2048-token step: 17.6 -> 18.2 ms).
    slot_sum_deferral_tokens = 64

    make_moe_workspace = MoeWorkspace

    def rms_norm(self, x, weight, eps: float, out, residual=None, rows=None, write_residual=True, slots: int = 1):
        """``out = norm(x (+ residual)) * weight``; with ``residual`` the rounded sum replaces it
        (unless ``write_residual`` is False).  ``rows`` (int32) selects input rows: ``out[j]`` is
        the norm of row ``rows[j]``.  ``out`` may be ``x``.  ``slots`` > 1: input row ``r`` is the
        sum of rows ``r * slots ...`` of ``x`` (``[rows * slots, hidden]``, contiguous), added up in
        float in slot order and rounded to the storage type first: the sum over a token's expert
        slots done while the norm reads, bit for bit what a separate sum would give."""
        # The two calls every layer of every step makes (a few hundred launches a step: what the host spends per
        # launch is what a short step waits for) go through their checks in one expression; a call that fails one,
        # and every other kind of call, takes the long way below, which names what is wrong.
        if _SHORT_WAYS and rows is None:
            shape = out.shape
            hidden = shape[-1]
            if (len(shape) == 2 and out.stride(1) == 1 and out.dtype == x.dtype and hidden <= 15360
                    and weight.shape == shape[1:] and weight.is_contiguous()
                    and (residual is None or (residual.shape == shape and residual.dtype == x.dtype
                                              and residual.stride(1) == 1))):
                aligned = not ((x.data_ptr() | out.data_ptr() | weight.data_ptr()
                                | (0 if residual is None else residual.data_ptr())) & 15)
                res_stride = 0 if residual is None else residual.stride(0)
                if slots == 1:
                    if x.shape == shape and x.stride(1) == 1:
                        _check(_fn.get("norm", "se_rms_norm")(
                            _ptr(x), _ptr(residual), _ptr(weight), _ptr(out), None, shape[0], hidden, float(eps),
                            x.stride(0), res_stride, out.stride(0), int(bool(write_residual)), _code(x.dtype),
                            _code(weight.dtype), int(aligned), _stream()), "rms_norm")
                        return
                elif (x.dim() == 2 and x.shape[0] == shape[0] * slots and x.shape[1] == hidden and x.is_contiguous()
                      and out.data_ptr() != x.data_ptr()):
                    status = _fn.get("norm", "se_rms_norm_slots")(
                        _ptr(x), _ptr(residual), _ptr(weight), _ptr(out), None, shape[0], hidden, float(eps),
                        x.stride(0), res_stride, out.stride(0), int(bool(write_residual)), _code(x.dtype),
                        _code(weight.dtype), int(aligned), int(slots), _stream())
                    if status == 0:
                        return
                    if status != -1:
                        _check(status, "rms_norm (slot rows)")
        hidden = x.shape[-1]
        n_out = out.shape[0]
        if slots > 1:
            _require(x.dim() == 2 and x.is_contiguous() and x.shape[0] % slots == 0 and out.dim() == 2
                     and out.data_ptr() != x.data_ptr() and out.dtype == x.dtype, "rms_norm: slot rows")
            n_in = x.shape[0] // slots
            if residual is not None:
                _require(residual.shape == (n_in, hidden) and residual.dtype == x.dtype and residual.stride(1) == 1,
                         "rms_norm: residual shape/dtype")
            if rows is not None:
                _i32(rows, "rows")
                _require(rows.numel() == n_out, "rms_norm: rows/out mismatch")
                write_residual = False
            else:
                _require(n_out == n_in, "rms_norm: out rows")
            aligned = all(t is None or t.data_ptr() % 16 == 0 for t in (x, residual, weight, out))
            status = _fn.get("norm", "se_rms_norm_slots")(
                _ptr(x), _ptr(residual), _ptr(weight), _ptr(out), _ptr(rows), n_out, hidden, float(eps),
                x.stride(0), residual.stride(0) if residual is not None else 0, out.stride(0),
                int(bool(write_residual)), _code(x.dtype), _code(weight.dtype), int(aligned), int(slots),
                _stream()) if hidden <= 15360 else -1
            if status == 0:
                return
            if status != -1:      # only "these sizes are not taken" leads on to the two kernels below
                _check(status, "rms_norm (slot rows)")
            # sizes the fused kernel does not take: the sum first, then the norm of its result
            summed = torch.empty(n_in, hidden, dtype=x.dtype, device=x.device)
            _check(_fn.get("moe", "se_moe_sum")(_ptr(x), _ptr(summed), n_in, int(slots), hidden, _code(x.dtype),
                                                _stream()), "slot sum")
            x, slots = summed, 1
        _require(x.dim() == 2 and out.dim() == 2 and out.shape[1] == hidden, "rms_norm: x/out shapes")
        _require(x.stride(1) == 1 and out.stride(1) == 1, "rms_norm: rows must be dense")
        _require(weight.shape == (hidden,) and weight.is_contiguous(), "rms_norm: weight shape")
        _require(out.dtype == x.dtype, "rms_norm: out dtype")
        if residual is not None:
            _require(residual.shape == x.shape and residual.dtype == x.dtype and residual.stride(1) == 1,
                     "rms_norm: residual shape/dtype")
        if rows is not None:
            _i32(rows, "rows")
            _require(rows.numel() == n_out, "rms_norm: rows/out mismatch")
            write_residual = False
        else:
            _require(n_out == x.shape[0], "rms_norm: out rows")
        if hidden > 15360:
            raise KernelShapeError(f"rms_norm: hidden size {hidden} is above the kernel's limit 15360")
        _check(_fn.get("norm", "se_rms_norm")(
            _ptr(x), _ptr(residual), _ptr(weight), _ptr(out), _ptr(rows), n_out, hidden, float(eps),
            x.stride(0), residual.stride(0) if residual is not None else 0, out.stride(0),
            int(bool(write_residual)), _code(x.dtype), _code(weight.dtype),
            int(all(t is None or t.data_ptr() % 16 == 0 for t in (x, residual, weight, out))), _stream()),
            "rms_norm")

    # ------------------------------------------------------------------ attention inputs
    ROTARY_PAIRINGS = {"neox": 0, "interleaved": 1}

    def qk_norm_rope_store(self, qkv, positions, cos_sin, q_weight, k_weight, eps, heads, kv_heads,
                           head_dim, rotary_dim, cache=None, slots=None, page_size=0, pairing="neox",
                           per_head_norm: bool = False):
        """In place on ``qkv [T, (heads + 2 kv_heads) * head_dim]``: QK norm (if weights are given: flat, one
        statistic per token over all heads, weights ``[heads * head_dim]`` and ``[kv_heads * head_dim]``; or
        ``per_head_norm``, one statistic per token and head, weights ``[head_dim]``), partial rotation by
        ``cos_sin [max_pos, rotary_dim]`` (cos half, sin half; ``pairing`` "neox" turns dims ``(d, d + rotary_dim / 2)`` together, "interleaved" dims ``(2 j, 2 j + 1)``), and
        the write of k and v to ``cache [pages, 2, kv_heads, page_size, head_dim]`` at ``slots`` (the
        last two sizes are a page's geometry; the order of its elements is cache/layout.py's)."""
        tokens = qkv.shape[0]
        width = (heads + 2 * kv_heads) * head_dim
        int32 = torch.int32
        # the call of every layer (norm weights, a rotation table, the cache write) in one expression; a call that
        # fails a check, and every other kind of call, takes the long way below, which names what is wrong
        if (_SHORT_WAYS and not per_head_norm and q_weight is not None and cache is not None and rotary_dim
                and pairing in self.ROTARY_PAIRINGS
                and qkv.dim() == 2 and qkv.shape[1] == width and qkv.stride(1) == 1
                and positions.dtype == int32 and positions.is_contiguous() and positions.numel() == tokens
                and rotary_dim % 2 == 0 and 0 < rotary_dim <= head_dim
                and cos_sin.dtype == torch.float32 and cos_sin.is_contiguous() and cos_sin.shape[1] == rotary_dim
                and q_weight.shape == (heads * head_dim,) and k_weight.shape == (kv_heads * head_dim,)
                and q_weight.dtype == k_weight.dtype and q_weight.is_contiguous() and k_weight.is_contiguous()
                and slots.dtype == int32 and slots.is_contiguous() and slots.numel() == tokens
                and cache.dtype == qkv.dtype and cache.is_contiguous() and cache.dim() == 5
                and tuple(cache.shape[1:]) == (2, kv_heads, page_size, head_dim)
                and page_size % 8 == 0 and head_dim % 8 == 0):
            aligned = not ((qkv.data_ptr() | q_weight.data_ptr() | k_weight.data_ptr() | cache.data_ptr()
                            | cos_sin.data_ptr()) & 15)
            _check(_fn.get("rope_kv", "se_qk_norm_rope_store")(
                _ptr(qkv), qkv.stride(0), _ptr(positions), _ptr(cos_sin), _ptr(q_weight), _ptr(k_weight), float(eps),
                tokens, heads, kv_heads, head_dim, rotary_dim, _ptr(cache), _ptr(slots), page_size, 1,
                _code(qkv.dtype), _code(q_weight.dtype), int(aligned), self.ROTARY_PAIRINGS[pairing], 0, _stream()),
                "qk_norm_rope_store")
            return
        _require(qkv.dim() == 2 and qkv.shape[1] == width and qkv.stride(1) == 1, "qkv shape")
        _i32(positions, "positions")
        _require(positions.numel() == tokens, "positions length")
        _require(rotary_dim % 2 == 0 and 0 <= rotary_dim <= head_dim, "rotary_dim must be even and <= head_dim")
        if rotary_dim:
            _require(cos_sin.dtype == torch.float32 and cos_sin.is_contiguous()
                     and cos_sin.shape[1] == rotary_dim, "cos_sin table shape/dtype")
        if q_weight is not None:
            widths = ((head_dim,), (head_dim,)) if per_head_norm else ((heads * head_dim,), (kv_heads * head_dim,))
            _require(k_weight is not None and (tuple(q_weight.shape), tuple(k_weight.shape)) == widths
                     and q_weight.dtype == k_weight.dtype and q_weight.is_contiguous() and k_weight.is_contiguous(),
                     "qk norm weight shapes")
        if pairing not in self.ROTARY_PAIRINGS:
            raise ValueError(f"rotary pairing {pairing!r} is unknown ({', '.join(self.ROTARY_PAIRINGS)})")
        write_kv = cache is not None
        if write_kv:
            _i32(slots, "slots")
            _require(slots.numel() == tokens, "slots length")
            _require(cache.dtype == qkv.dtype and cache.is_contiguous() and cache.dim() == 5
                     and tuple(cache.shape[1:]) == (2, kv_heads, page_size, head_dim), "cache layout")
            if page_size % 8 or head_dim % 8:
                raise KernelShapeError(f"cache pages take page_size {page_size} and head_dim {head_dim} in steps of 8")
        wd = _code(q_weight.dtype) if q_weight is not None else _code(qkv.dtype)
        _check(_fn.get("rope_kv", "se_qk_norm_rope_store")(
            _ptr(qkv), qkv.stride(0), _ptr(positions), _ptr(cos_sin) if rotary_dim else None,
            _ptr(q_weight), _ptr(k_weight), float(eps), tokens, heads, kv_heads, head_dim, rotary_dim,
            _ptr(cache), _ptr(slots), page_size, int(write_kv), _code(qkv.dtype), wd,
            int(all(t is None or t.data_ptr() % 16 == 0 for t in (qkv, q_weight, k_weight, cache, cos_sin))),
            self.ROTARY_PAIRINGS[pairing], int(bool(per_head_norm and q_weight is not None)), _stream()),
            "qk_norm_rope_store")

    def paged_attention(self, q, cache, meta, out, scale: float, window: int = 0):
        """Causal attention of every token of the step against its request's pages.

        ``q``: ``[T, heads, head_dim]`` view (token stride free, heads dense); ``cache``:
        ``[pages, 2, kv_heads, page_size, head_dim]``; ``meta``: an object with ``block_table``
        (int32 ``[items, max_pages]``), ``token_row`` and ``positions`` (int32 ``[T]``) and, for the
        matrix-core kernels, the items' lengths on the host (``item_q_len``, ``item_ctx_len``) and
        optionally prepared work lists (``work``);
        ``out``: ``[T, heads * head_dim]``."""
        tokens, heads, head_dim = q.shape
        kv_heads, page_size = cache.shape[2], cache.shape[3]
        _require(q.stride(2) == 1 and q.stride(1) == head_dim, "q heads must be dense")
        _require(cache.dim() == 5 and cache.shape[1] == 2 and cache.shape[4] == head_dim
                 and cache.is_contiguous() and cache.dtype == q.dtype, "cache layout")
        _require(out.shape == (tokens, heads * head_dim) and out.stride(1) == 1 and out.dtype == q.dtype,
                 "attention out shape")
        _i32(meta.token_row, "token_row"); _i32(meta.positions, "positions")
        _require(meta.block_table.dtype == torch.int32 and meta.block_table.dim() == 2
                 and meta.block_table.stride(1) == 1, "block_table layout")
        _require(meta.token_row.numel() == tokens and meta.positions.numel() == tokens, "meta length")
        if heads % kv_heads:
            raise KernelShapeError(f"attention: {heads} heads do not divide into {kv_heads} kv heads")
        if page_size % 8:
            raise KernelShapeError(f"attention: page_size {page_size} must be a multiple of 8")
        window = int(window or 0)
        if (q.dtype == torch.bfloat16 and head_dim % 32 == 0 and head_dim <= 256
                and getattr(meta, "item_q_len", None) is not None):      # the step's items are known
            return self._paged_attention_mfma(q, cache, meta, out, scale, window)
        if head_dim % 8 or head_dim > 512:
            raise KernelShapeError(f"attention: head_dim {head_dim} must be a multiple of 8, at most 512")
        _check(_fn.get("attention_generic", "se_paged_attention_generic")(
            _ptr(q), q.stride(0), _ptr(cache), _ptr(meta.block_table), meta.block_table.stride(0),
            _ptr(meta.token_row), _ptr(meta.positions), _ptr(out), out.stride(0), tokens, heads,
            kv_heads, head_dim, page_size, float(scale), window, _code(q.dtype), _stream()),
            "paged_attention")

    def _paged_attention_mfma(self, q, cache, meta, out, scale, window):
        """Matrix-core path: work units (row tile x key range) from the step's item lengths."""
        tokens, heads, head_dim = q.shape
        kv_heads, page_size = cache.shape[2], cache.shape[3]
        group = heads // kv_heads
        work = None if getattr(meta, "work", None) is None else meta.work.get((group, window))
        if work is None:                      # not prepared by the batch builder: build it here
            from .attention_work import DeviceAttentionWork, build_attention_work
            host = build_attention_work(meta.item_q_len, meta.item_ctx_len, group, kv_heads, window,
                                        head_dim=head_dim)
            work = DeviceAttentionWork(
                torch.from_numpy(host.units).to(q.device), host.units.shape[0],
                torch.from_numpy(host.tasks).to(q.device), host.tasks.shape[0], host.num_slots,
                torch.from_numpy(host.block_units).to(q.device), host.block_units.shape[0], host.tiles_per_block)
            if getattr(meta, "work", None) is not None:
                meta.work[(group, window)] = work
        part_o = part_ml = None
        if work.num_slots:                    # key ranges leave partial results for the merge
            need = work.num_slots * kv_heads * 16
            if self._attention_partials is None or self._attention_partials[0].numel() < need * head_dim:
                self._attention_partials = (torch.empty(need * head_dim, dtype=torch.float32, device=q.device),
                                            torch.empty(need * 2, dtype=torch.float32, device=q.device))
            part_o, part_ml = self._attention_partials
            if part_ml.numel() < need * 2:
                part_ml = torch.empty(need * 2, dtype=torch.float32, device=q.device)
                self._attention_partials = (part_o, part_ml)
        if work.num_block_units:              # prompt portions: keys and values shared by a block
            _check(_fn.get("attention_mfma", "se_paged_attention_tiled")(
                _ptr(q), q.stride(0), _ptr(cache), _ptr(meta.block_table), meta.block_table.stride(0),
                _ptr(work.block_units), work.num_block_units, _ptr(out), out.stride(0), _ptr(part_o),
                _ptr(part_ml), heads, kv_heads, head_dim, page_size, float(scale), window,
                work.tiles_per_block, _stream()), "paged_attention (blocks)",
                "head_dim a multiple of 32 up to 128, page_size a multiple of 8")
        if work.num_units or work.num_tasks:  # one wavefront per tile and key range; then all merges
            _check(_fn.get("attention_mfma", "se_paged_attention_mfma")(
                _ptr(q), q.stride(0), _ptr(cache), _ptr(meta.block_table), meta.block_table.stride(0),
                _ptr(work.units) if work.num_units else None, work.num_units,
                _ptr(work.tasks) if work.num_tasks else None, work.num_tasks, _ptr(out), out.stride(0),
                _ptr(part_o), _ptr(part_ml), heads, kv_heads, head_dim, page_size, float(scale), window,
                _stream()), "paged_attention (wavefronts)",
                "head_dim a multiple of 32 up to 256, page_size a multiple of 8")

    # ------------------------------------------------------------------ mixture of experts
    ROUTER_KERNEL_TOKENS = 16   # up to this many tokens the router's product is one small kernel

    def router_logits(self, x, weight, out):
        """``out[T, experts] = x @ weight.T`` in float32 from float32 weights.  Few tokens take a
        kernel that widens the activations as it reads them; more go to the BLAS library."""
        tokens, k = x.shape
        experts = weight.shape[0]
        _require(weight.dtype == torch.float32 and weight.is_contiguous() and weight.shape[1] == k,
                 "router weight must be float32 [experts, hidden]")
        _require(out.dtype == torch.float32 and out.shape == (tokens, experts) and out.stride(1) == 1,
                 "router logits must be float32 [tokens, experts]")
        if (tokens <= self.ROUTER_KERNEL_TOKENS and k % 8 == 0 and x.stride(1) == 1 and x.stride(0) % 8 == 0
                and x.dtype in (torch.bfloat16, torch.float32)):
            _check(_fn.get("moe", "se_router_logits")(
                _ptr(x), x.stride(0), _ptr(weight), _ptr(out), out.stride(0), tokens, experts, k,
                _code(x.dtype), _stream()), "router_logits")
            return out
        return torch.mm(x.float(), weight.t(), out=out)

    FUSED_ROUTER_TOKENS = 16   # up to this many tokens one launch routes and groups the assignments

    def router_topk(self, logits, bias, top_k: int, ids, weights, scoring="sigmoid", normalize=True,
                    scaling: float = 1.0, workspace=None):
        """Scores, the chosen experts and their weights.  With a ``workspace`` (the one the expert
        products of the same step will use) and few tokens, the same launch also groups the
        assignments by expert in tiles of 16; ``moe_experts`` then skips that step."""
        tokens, experts = logits.shape
        _require(logits.dtype == torch.float32 and logits.stride(1) == 1, "router logits must be float32")
        if bias is not None:
            _require(bias.dtype == torch.float32 and bias.shape == (experts,) and bias.is_contiguous(),
                     "router bias must be float32 [experts]")
        _i32(ids, "ids")
        _require(ids.shape == (tokens, top_k) and weights.shape == (tokens, top_k)
                 and weights.dtype == torch.float32 and weights.is_contiguous(), "router outputs")
        if scoring not in ("sigmoid", "softmax"):
            raise ValueError(f"router scoring '{scoring}' is unknown (sigmoid, softmax)")
        if experts > 1024:
            raise KernelShapeError(f"router: {experts} experts are above the kernel's limit 1024")
        _require(1 <= top_k <= experts, "1 <= top_k <= experts")
        if workspace is not None:
            workspace.grouped = None
            capacity, max_tiles = moe_tile_bounds(tokens * top_k, experts, 16)
            if (tokens <= self.FUSED_ROUTER_TOKENS and workspace.sorted.numel() >= capacity
                    and workspace.tile_expert.numel() >= max_tiles):
                _check(_fn.get("moe", "se_router_topk_align")(
                    _ptr(logits), logits.stride(0), _ptr(bias), _ptr(ids), _ptr(weights), tokens, experts,
                    top_k, int(scoring == "softmax"), int(bool(normalize)), float(scaling), 16,
                    _ptr(workspace.sorted), _ptr(workspace.tile_expert), _ptr(workspace.counters),
                    _stream()), "router_topk (with grouping)")
                workspace.grouped = (ids.data_ptr(), tokens, top_k, experts, 16, max_tiles)
                return
        _check(_fn.get("moe", "se_router_topk")(
            _ptr(logits), logits.stride(0), _ptr(bias), _ptr(ids), _ptr(weights), tokens, experts,
            top_k, int(scoring == "softmax"), int(bool(normalize)), float(scaling), _stream()),
            "router_topk")

    def route(self, x, weight, bias, top_k: int, logits, ids, weights, scoring="sigmoid", normalize=True,
              scaling: float = 1.0, workspace=None):
        """The whole router: ``logits = x @ weight.T`` in float32, then ``router_topk`` on them.
        Two launches.  (One launch in which the block that finishes its logits last routes was
        measured and is not faster on this chip: making the logits visible across the chip's eight
        L2 caches, the count and the barriers cost about 4.5 us, more than a kernel's boundary.)"""
        self.router_logits(x, weight, logits)
        self.router_topk(logits, bias, top_k, ids, weights, scoring=scoring, normalize=normalize,
                         scaling=scaling, workspace=workspace)

    def moe_align(self, ids, experts: int, ws: MoeWorkspace, tile_rows: int = 16):
        _i32(ids, "ids")
        assignments = ids.numel()
        capacity, max_tiles = moe_tile_bounds(assignments, experts, tile_rows)
        _require(ws.sorted.numel() >= capacity and ws.tile_expert.numel() >= max_tiles, "workspace too small")
        if experts > 4096:
            raise KernelShapeError(f"moe_align: {experts} experts are above the kernel's limit 4096")
        _check(_fn.get("moe", "se_moe_align")(
            _ptr(ids), assignments, experts, tile_rows, _ptr(ws.sorted), _ptr(ws.tile_expert),
            _ptr(ws.counters), _stream()), "moe_align")
        return max_tiles

    def _grouped_tiles(self, ids, experts: int, ws: MoeWorkspace, tile_rows: int) -> int:
        """Group the assignments by expert, unless the router's launch has done just that."""
        grouped, ws.grouped = ws.grouped, None
        tokens, top_k = ids.shape
        if grouped is not None and grouped[:5] == (ids.data_ptr(), tokens, top_k, experts, tile_rows):
            return grouped[5]
        return self.moe_align(ids, experts, ws, tile_rows)

    # ------------------------------------------------------------------ expert tables in tiles
    @staticmethod
    def takes_tiled_expert_weights(dtype, hidden: int, inter: int) -> bool:
        """Whether the expert products of these sizes run on the matrix-core kernels, which read
        the tables in tiles (below)."""
        return dtype == torch.bfloat16 and hidden % 128 == 0 and inter % 128 == 0

    @staticmethod
    def tile_expert_weights(w: torch.Tensor) -> torch.Tensor:
        """A copy of ``w [E, N, K]`` in tiles of 16 rows x 32 k: tile ``(n // 16, k // 32)`` is 512
        consecutive elements in the order ``[(k % 32) // 8][n % 16][k % 8]``, which is the order of
        the lanes that hold it as a matrix-core operand (lane ``16 * piece + row`` holds 8 elements).
        A wavefront then loads a tile as one contiguous kilobyte instead of 64 bytes from each of 16
        rows; measured on MI355X the latter arrives at a third of the former's rate."""
        experts, n, k = w.shape
        _require(n % 16 == 0 and k % 32 == 0, "tiles need rows in steps of 16 and k in steps of 32")
        return w.view(experts, n // 16, 16, k // 32, 4, 8).permute(0, 1, 3, 4, 2, 5).contiguous().view(experts, n, k)

    def arrange_expert_weights(self, w13: torch.Tensor, w2: torch.Tensor) -> bool:
        """Put both tables into tiles, in place, if the kernels for these sizes read tiles; says
        whether it did.  A few experts at a time, so that no second copy of a table exists."""
        hidden, inter = w13.shape[2], w2.shape[2]
        if w13.dtype != w2.dtype or not self.takes_tiled_expert_weights(w13.dtype, hidden, inter):
            return False
        for w in (w13, w2):
            for first in range(0, w.shape[0], 8):
                w[first:first + 8].copy_(self.tile_expert_weights(w[first:first + 8]))
        return True

    ACTIVATIONS = {"silu": 0, "gelu_tanh": 1}      # what a gated feed-forward applies to its gate
    # The device's choice between the mid kernel (tiles of 96 rows) and the wide one (tiles of 128).  The mid kernel
    # reads an expert's table once per tile, at 6.3 TB/s; the wide one reads it once (5.3 TB/s), or is bound by its
    # arithmetic, about 0.8 PFLOP/s, which is the time of reading one table per 151 rows.  Mid is chosen if its
    # tiles, times 84 %, are at most the larger of the experts that got rows and the rows / 151.
    AUTO_TILE_ROWS = (96, 128)
    AUTO_READ_PERCENT = 84
    AUTO_HEAVY_ROWS = 151

    def _activation(self, name: str) -> int:
        if name not in self.ACTIVATIONS:
            raise ValueError(f"activation {name!r} is unknown ({', '.join(self.ACTIVATIONS)})")
        return self.ACTIVATIONS[name]

    def moe_experts(self, x, w13, w2, ids, weights, out, ws: MoeWorkspace, kernel=None, tile_rows=None,
                    column_blocks=None, tiled: bool = False, sum_slots: bool = True, activation: str = "silu"):
        """``out[t] = sum_k weights[t,k] * W2_e(act(W1_e x_t) * W3_e x_t)``, ``e = ids[t,k]``, ``act`` silu
        or the tanh form of gelu;
        ``w13 [E, 2I, h]`` holds gate rows then up rows, ``w2 [E, h, I]``.  ``tiled``: the tables
        have been through ``arrange_expert_weights``; row-major tables of sizes the matrix-core
        kernels take are put into tiles here, call by call (tests; the model arranges them once).
        ``sum_slots=False``: the sum over a token's slots is left to the caller; the slots' results
        ``[tokens * top_k, hidden]`` are returned (a view of the workspace, good until its next use) and
        ``out`` is not written.
        ``kernel`` ("stream", "tall", "direct"), ``tile_rows`` and ``column_blocks`` override the
        choice of the matrix-core kernel and its tile (tests and measurements)."""
        tokens, hidden = x.shape
        experts, two_i, _ = w13.shape
        inter = two_i // 2
        top_k = ids.shape[1]
        # The call of a decode step (tables in tiles, the router's launch has grouped the assignments, fewer than
        # three rows per expert: the streaming kernel on tiles of 16) in one expression; a call that fails a check,
        # and every other kind of call, takes the long way below, which names what is wrong.
        grouped = ws.grouped
        if (_SHORT_WAYS and tiled and kernel is None and tile_rows is None and column_blocks is None and grouped is not None
                and x.dtype == torch.bfloat16 and hidden % 128 == 0 and inter % 128 == 0
                and tokens * top_k < 3 * min(experts, tokens * top_k)
                and grouped[:5] == (ids.data_ptr(), tokens, top_k, experts, 16) and grouped[5] <= 65535
                and x.is_contiguous() and out.is_contiguous() and out.shape == x.shape
                and w13.shape == (experts, 2 * inter, hidden) and w2.shape == (experts, hidden, inter)
                and w13.is_contiguous() and w2.is_contiguous()
                and w13.dtype == x.dtype and w2.dtype == x.dtype and out.dtype == x.dtype
                and ids.dtype == torch.int32 and ids.is_contiguous() and ids.shape[0] == tokens and weights.shape == ids.shape
                and weights.dtype == torch.float32 and weights.is_contiguous()
                and ws.fits(tokens, top_k, experts, hidden, inter, x.dtype)):
            ws.grouped = None
            max_tiles, assignments = grouped[5], tokens * top_k
            act = self._activation(activation)
            blocks = 2 if max_tiles * (inter // 32) >= 2048 else 1
            takes = "hidden and intermediate sizes in multiples of 128"
            gg = _fn.get("moe_mfma", "se_grouped_gemm_mfma")
            sorted_, tile_expert, counters = _ptr(ws.sorted), _ptr(ws.tile_expert), _ptr(ws.counters)
            stream = _stream()
            _check(gg(_ptr(x), _ptr(w13), _ptr(ws.act), sorted_, tile_expert, counters, None, assignments, top_k, inter,
                      hidden, max_tiles, 0, 16, blocks, act, stream), "moe gate-up (stream)", takes)
            _check(gg(_ptr(ws.act), _ptr(w2), _ptr(ws.slot_out), sorted_, tile_expert, counters, _ptr(weights), assignments,
                      top_k, hidden, inter, max_tiles, 1, 16, blocks, act, stream), "moe down (stream)", takes)
            if not sum_slots:
                return ws.slot_out[:assignments]
            _check(_fn.get("moe", "se_moe_sum")(_ptr(ws.slot_out), _ptr(out), tokens, top_k, hidden, _code(x.dtype),
                                                stream), "moe_sum")
            return
        _require(x.is_contiguous() and out.is_contiguous() and out.shape == x.shape, "moe x/out")
        _require(w13.shape == (experts, 2 * inter, hidden) and w2.shape == (experts, hidden, inter)
                 and w13.is_contiguous() and w2.is_contiguous(), "expert weight shapes")
        _require(w13.dtype == x.dtype and w2.dtype == x.dtype and out.dtype == x.dtype, "moe dtypes")
        _require(ids.shape == (tokens, top_k) and weights.shape == (tokens, top_k)
                 and weights.dtype == torch.float32 and weights.is_contiguous(), "routing shapes")
        _require(ws.fits(tokens, top_k, experts, hidden, inter, x.dtype), "moe workspace does not fit")
        assignments = tokens * top_k
        code = _code(x.dtype)
        act = self._activation(activation)
        if self.takes_tiled_expert_weights(x.dtype, hidden, inter):
            if not tiled:
                w13, w2 = self.tile_expert_weights(w13), self.tile_expert_weights(w2)
            # matrix-core path, four kernels:
            #   "stream"  weights from memory straight into operands, tiles of 16 (32, 64) rows: an
            #             expert's table is read once per tile;
            #   "mid"     tiles of 64 or 96 rows: the output columns split over eight wavefronts that each stream
            #             their own weight rows into operands; the tile's rows shared through LDS;
            #   "direct"  64 or 128 rows x 256 weight rows, operands straight into LDS as contiguous
            #             kilobytes of the tiled tables, two blocks per CU;
            #   "tall"    64 x 128 tiles, operands through registers into LDS (sizes the two above do not take).
            # Which experts a step uses is known on the device only.  The host goes by the average rows per
            # expert: below three, "stream" (a decode batch of 64 keeps it; when the tokens of a step agree on a
            # few dozen experts it would read their tables once per 16 rows, and loses from 48 tokens on).  From
            # there on the device chooses between "mid" and "direct" ("auto", below).
            share = assignments / min(experts, assignments)
            direct_ok = inter % 128 == 0 and hidden % 256 == 0
            if kernel is None:
                if tile_rows is not None:
                    kernel = "stream" if tile_rows < 64 else ("direct" if tile_rows == 128 and direct_ok else "tall")
                else:
                    kernel = "stream" if share < 3 else ("auto" if direct_ok else "tall")
            if kernel not in ("stream", "tall", "direct", "mid", "auto"):
                raise ValueError(f"expert kernel {kernel!r} is unknown (stream, tall, direct, mid, auto)")
            if kernel in ("direct", "mid", "auto") and not direct_ok:
                raise KernelShapeError(f"the {kernel} expert kernel takes hidden sizes in steps of 256 and "
                                       "intermediate sizes in steps of 128")
            takes = "hidden and intermediate sizes in multiples of 128"
            if kernel == "auto":
                # the code of "mid" or of "direct", chosen where the spread of the rows over the experts is known: on
                # the device, by the kernel that groups the assignments; one launch holds both.
                # Measured at MiniMax-M2 sizes with the rows spread evenly: 64 rows per expert 1245 (mid) against
                # 1373 us (direct), 32 rows 1190 against 1290, 16 rows 1150 against 1250, 4 rows 1075 against 1164
                # (the tall kernel, which this replaces); at 128 rows per expert, and whenever the tokens of a prompt
                # agree on a few dozen experts, direct wins (an expert's table is then read once per 96 rows by mid).
                few_tile, many_tile = self.AUTO_TILE_ROWS
                max_tiles = max(moe_tile_bounds(assignments, experts, few_tile)[1],
                                moe_tile_bounds(assignments, experts, many_tile)[1])
                if max_tiles > 65535:
                    raise KernelShapeError("moe: too many tokens in one call; lower mlp_chunk_size")
                ws.grouped = None
                _check(_fn.get("moe", "se_moe_align_choice")(
                    _ptr(ids), assignments, experts, few_tile, many_tile, self.AUTO_READ_PERCENT, self.AUTO_HEAVY_ROWS,
                    _ptr(ws.sorted),
                    _ptr(ws.tile_expert), _ptr(ws.counters), _stream()), "moe_align (choice)")
                either = _fn.get("moe_mfma", "se_grouped_gemm_choice")
                _check(either(_ptr(x), _ptr(w13), _ptr(ws.act), _ptr(ws.sorted), _ptr(ws.tile_expert), _ptr(ws.counters),
                              None, assignments, top_k, inter, hidden, max_tiles, 0, act, _stream()), "moe gate-up (auto)", takes)
                _check(either(_ptr(ws.act), _ptr(w2), _ptr(ws.slot_out), _ptr(ws.sorted), _ptr(ws.tile_expert),
                              _ptr(ws.counters), _ptr(weights), assignments, top_k, hidden, inter, max_tiles, 1, act,
                              _stream()), "moe down (auto)", takes)
            else:
                if tile_rows is None:
                    tile_rows = {"stream": 16, "tall": 64, "direct": 128 if share >= 16 else 64, "mid": 96}[kernel]
                max_tiles = self._grouped_tiles(ids, experts, ws, tile_rows)
                if max_tiles > 65535:
                    raise KernelShapeError("moe: too many tokens in one call; lower mlp_chunk_size")
            if kernel == "stream":
                gg = _fn.get("moe_mfma", "se_grouped_gemm_mfma")
                if column_blocks is None:
                    column_blocks = 2 if max_tiles * (inter // 32) >= 2048 else 1
                _check(gg(_ptr(x), _ptr(w13), _ptr(ws.act), _ptr(ws.sorted), _ptr(ws.tile_expert),
                          _ptr(ws.counters), None, assignments, top_k, inter, hidden, max_tiles, 0, tile_rows,
                          column_blocks, act, _stream()), "moe gate-up (stream)", takes)
                _check(gg(_ptr(ws.act), _ptr(w2), _ptr(ws.slot_out), _ptr(ws.sorted), _ptr(ws.tile_expert),
                          _ptr(ws.counters), _ptr(weights), assignments, top_k, hidden, inter, max_tiles, 1,
                          tile_rows, column_blocks, act, _stream()), "moe down (stream)", takes)
            elif kernel != "auto":
                gt = _fn.get("moe_mfma", {"direct": "se_grouped_gemm_wide", "tall": "se_grouped_gemm_tall",
                                          "mid": "se_grouped_gemm_mid"}[kernel])
                _check(gt(_ptr(x), _ptr(w13), _ptr(ws.act), _ptr(ws.sorted), _ptr(ws.tile_expert),
                          _ptr(ws.counters), None, assignments, top_k, inter, hidden, max_tiles, 0, tile_rows,
                          act, _stream()), f"moe gate-up ({kernel})", takes)
                _check(gt(_ptr(ws.act), _ptr(w2), _ptr(ws.slot_out), _ptr(ws.sorted), _ptr(ws.tile_expert),
                          _ptr(ws.counters), _ptr(weights), assignments, top_k, hidden, inter, max_tiles, 1,
                          tile_rows, act, _stream()), f"moe down ({kernel})", takes)
        else:
            _require(not tiled, "the general expert kernel reads row-major tables")
            max_tiles = self._grouped_tiles(ids, experts, ws, 16)
            if max_tiles > 65535:
                raise KernelShapeError("moe: too many tokens in one call; lower mlp_chunk_size")
            gg = _fn.get("moe", "se_grouped_gemm_generic")
            _check(gg(_ptr(x), _ptr(w13), _ptr(ws.act), _ptr(ws.sorted), _ptr(ws.tile_expert),
                      _ptr(ws.counters), None, assignments, top_k, inter, hidden, max_tiles, 0, code,
                      act, _stream()), "moe gate-up")
            _check(gg(_ptr(ws.act), _ptr(w2), _ptr(ws.slot_out), _ptr(ws.sorted), _ptr(ws.tile_expert),
                      _ptr(ws.counters), _ptr(weights), assignments, top_k, hidden, inter, max_tiles, 1,
                      code, act, _stream()), "moe down")
        if not sum_slots:      # the caller sums: [tokens * top_k, hidden], a token's slots one after the other
            return ws.slot_out[:assignments]
        _check(_fn.get("moe", "se_moe_sum")(_ptr(ws.slot_out), _ptr(out), tokens, top_k, hidden, code,
                                            _stream()), "moe_sum")

    # Up to this many rows a dense product streams a weight matrix in rows once on MFMA.  Measured on MI355X
    # at 8192 x 3072 and 200064 x 3072: 8 rows 12.5 / 225 us against the library's 26 / 376; 32 rows 20 / 400
    # against 23 / 381; from 48 rows on the library wins (the kernel's activation loads then outweigh its
    # weight loads).  With a tiled copy of the matrix (``prepare_dense_weight``) the kernel's loads are
    # contiguous kilobytes that take the read-once hint: 200064 x 3072 at 8 rows 173 us (7.1 TB/s) against 196.
    # At 64 rows the library still wins (8192 x 3072: 23 against 30 us; the activation rows come from 16 rows
    # at 64 bytes each per load), so the limit is the same for both layouts.
    SKINNY_ROWS = 32
    TILED_SKINNY_ROWS = 32

    def prepare_dense_weight(self, weight: torch.Tensor):
        """A copy of ``weight [N, K]`` in the tiles the streaming kernel loads as contiguous kilobytes, for the
        products of steps with few rows (decode), or None if the kernel does not take the matrix.  The matrix
        in rows stays for the BLAS library, which takes the steps with many rows: a projection so held takes
        twice its bytes."""
        if (weight.dim() != 2 or weight.dtype != torch.bfloat16 or weight.shape[0] % 16 or weight.shape[1] % 128
                or not weight.is_contiguous()):
            return None
        return self.tile_expert_weights(weight[None])[0]

    def linear(self, x, weight, out, prepared=None):
        """``out = x @ weight.T``.  Few bfloat16 rows take the streaming matrix-core kernel (the BLAS
        library's choice for such shapes reads the weights at a fraction of memory speed), on ``prepared``
        (what ``prepare_dense_weight`` made of ``weight``) if it is given; everything else goes to the BLAS
        library."""
        rows, k = x.shape
        n = weight.shape[0]
        bf16 = torch.bfloat16
        if _SHORT_WAYS and prepared is not None:      # the call of a decode step: one expression, or the long way below
            if (rows <= self.TILED_SKINNY_ROWS and x.dtype == bf16 and prepared.dtype == bf16 and out.dtype == bf16
                    and weight.dtype == bf16 and k % 128 == 0 and n % 16 == 0 and prepared.shape == weight.shape
                    and weight.shape[1] == k and out.shape == (rows, n) and x.is_contiguous()
                    and prepared.is_contiguous() and weight.is_contiguous() and out.is_contiguous()):
                _check(_fn.get("moe_mfma", "se_skinny_gemm_mfma")(
                    _ptr(x), _ptr(prepared), _ptr(out), rows, n, k, 1, _stream()),
                    "skinny gemm", "K a multiple of 128, N a multiple of 16")
                return out
        limit = self.TILED_SKINNY_ROWS if prepared is not None else self.SKINNY_ROWS
        if (rows <= limit and x.dtype == bf16 and weight.dtype == bf16
                and k % 128 == 0 and n % 16 == 0 and x.is_contiguous() and weight.is_contiguous()
                and out.is_contiguous() and out.dtype == bf16):
            _require(weight.shape[1] == k and out.shape == (rows, n), "linear shapes")
            if prepared is not None:
                _require(prepared.shape == weight.shape and prepared.dtype == weight.dtype and prepared.is_contiguous(),
                         "linear: the prepared copy does not belong to this weight")
            _check(_fn.get("moe_mfma", "se_skinny_gemm_mfma")(
                _ptr(x), _ptr(weight if prepared is None else prepared), _ptr(out), rows, n, k,
                int(prepared is not None), _stream()), "skinny gemm", "K a multiple of 128, N a multiple of 16")
            return out
        return torch.mm(x, weight.t(), out=out)

    def silu_mul(self, x, out, activation: str = "silu"):
        """``out = act(x[:, :w]) * x[:, w:]``: the gated product of a dense feed-forward."""
        tokens, two_w = x.shape
        _require(x.is_contiguous() and out.is_contiguous() and out.shape == (tokens, two_w // 2)
                 and out.dtype == x.dtype, "silu_mul shapes")
        _check(_fn.get("moe", "se_silu_mul")(_ptr(x), _ptr(out), tokens, two_w // 2, _code(x.dtype),
                                             self._activation(activation), _stream()), "silu_mul")

    # ------------------------------------------------------------------ sampling
    def sample(self, logits, temperature, top_k, top_p, seeds, out):
        """One token per row of float ``logits``; ``temperature`` (float32), ``top_k`` (int32),
        ``top_p`` (float32) and ``seeds`` (int64, used as 64 raw bits) have one entry per row
        and may each be None (greedy / off / off / 0)."""
        rows, vocab = logits.shape
        _require(logits.dtype == torch.float32 and logits.stride(1) == 1, "logits must be float32")
        _i32(out, "out")
        _require(out.numel() == rows, "sample out length")
        for name, t, dt in (("temperature", temperature, torch.float32), ("top_k", top_k, torch.int32),
                            ("top_p", top_p, torch.float32), ("seeds", seeds, torch.int64)):
            if t is not None:
                _require(t.dtype == dt and t.numel() == rows and t.is_contiguous(), f"sample {name}")
        need = rows * (-(-vocab // 4096))
        if self._sample_partials is None or self._sample_partials[0].numel() < need:
            self._sample_partials = (torch.empty(need, dtype=torch.float32, device=logits.device),
                                     torch.empty(need, dtype=torch.int32, device=logits.device))
        if top_k is None and top_p is None:       # one arg-max per row, spread over many blocks
            _check(_fn.get("sampling", "se_sample_unfiltered")(
                _ptr(logits), logits.stride(0), rows, vocab, _ptr(temperature), _ptr(seeds),
                _ptr(self._sample_partials[0]), _ptr(self._sample_partials[1]), _ptr(out), _stream()),
                "sample")
            return
        # top-k / top-p: passes over the row that count and weigh its tokens by eight bits of their value at a time
        _require(temperature is not None, "sample: top_k / top_p need temperatures")
        filters = getattr(self, "_sample_filters", None)
        if filters is None or filters[0].numel() < need or filters[1].numel() < rows * 2048:
            filters = (torch.empty(need, dtype=torch.float32, device=logits.device),
                       torch.empty(rows * 2048, dtype=torch.int64, device=logits.device))
            self._sample_filters = filters
        _check(_fn.get("sampling", "se_sample")(
            _ptr(logits), logits.stride(0), rows, vocab, _ptr(temperature), _ptr(top_k), _ptr(top_p),
            _ptr(seeds), _ptr(self._sample_partials[0]), _ptr(self._sample_partials[1]), _ptr(filters[0]),
            _ptr(filters[1]), _ptr(out), _stream()), "sample")

    # ------------------------------------------------------------------ what the memory delivers
    PROBE_BLOCKS = 4096     # 16 blocks of 256 threads per CU, each thread with eight 16-byte loads in flight

    def stream_read(self, src: torch.Tensor, sink: torch.Tensor | None = None) -> torch.Tensor:
        """Read every byte of ``src`` once and nothing else: the kernel the weight-streaming kernels are
        priced against.  ``sink`` (int32, one word per block) takes the exclusive-or of what each block read."""
        _require(src.is_contiguous() and src.data_ptr() % 16 == 0 and (src.numel() * src.element_size()) % 16 == 0,
                 "stream_read: a contiguous tensor of a multiple of 16 bytes")
        if sink is None:
            sink = torch.empty(self.PROBE_BLOCKS, dtype=torch.int32, device=src.device)
        _i32(sink, "sink")
        _check(_fn.get("memory_probe", "se_stream_read")(_ptr(src), src.numel() * src.element_size(), _ptr(sink),
                                                         sink.numel(), _stream()), "stream_read")
        return sink

    def stream_copy(self, src: torch.Tensor, dst: torch.Tensor) -> torch.Tensor:
        _require(src.is_contiguous() and dst.is_contiguous() and src.dtype == dst.dtype and src.shape == dst.shape
                 and src.data_ptr() % 16 == 0 and dst.data_ptr() % 16 == 0
                 and (src.numel() * src.element_size()) % 16 == 0, "stream_copy: two contiguous tensors of one shape, 16-byte multiples")
        _check(_fn.get("memory_probe", "se_stream_copy")(_ptr(src), _ptr(dst), src.numel() * src.element_size(),
                                                         self.PROBE_BLOCKS, _stream()), "stream_copy")
        return dst

    def measure_memory(self, gib: float = 8.0, repeats: int = 5, device="cuda") -> dict:
        """Bytes per second of a kernel that only reads ``gib`` GiB (far beyond the caches) and of one that copies
        them (bytes read plus bytes written): the best of ``repeats`` runs each, after one untimed run."""
        words = int(gib * 2 ** 30) // 16
        src = torch.empty(words * 4, dtype=torch.int32, device=device).random_()
        sink = torch.empty(self.PROBE_BLOCKS, dtype=torch.int32, device=device)
        size = src.numel() * 4

        def best(run):
            run()
            rates = []
            for _ in range(repeats):
                first, last = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                first.record()
                run()
                last.record()
                last.synchronize()
                rates.append(first.elapsed_time(last) * 1e-3)
            return min(rates)

        read_s = best(lambda: self.stream_read(src, sink))
        dst = torch.empty_like(src)
        copy_s = best(lambda: self.stream_copy(src, dst))
        library_copy_s = best(lambda: dst.copy_(src))
        del src, dst
        return {"bytes": size, "read_GBps": round(size / read_s / 1e9, 1), "copy_GBps": round(2 * size / copy_s / 1e9, 1),
                "library_copy_GBps": round(2 * size / library_copy_s / 1e9, 1)}
