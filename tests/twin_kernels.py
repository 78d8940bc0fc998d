"""Plain tensor-library twins of the HIP kernels, with the kernels' interface and data layout.

Two uses, both in tests only: each kernel is checked against its twin on the GPU, and the
engine's host logic (cache, batches, scheduler, replay) is exercised on the CPU by handing it
this object instead of the HIP kernels.  Arithmetic is float32 with the kernels' rounding points
(``_r`` rounds through the storage dtype).
"""
from __future__ import annotations

import numpy as np
import torch

from sparseengine_amd.cache import layout


def _r(x: torch.Tensor, dtype: torch.dtype) -> torch.Tensor:
    return x.to(dtype).float()


class TwinWorkspace:
    def __init__(self, *args, **kwargs):
        pass

    def fits(self, *args) -> bool:
        return True


class TwinKernels:
    libraries = ()
    make_moe_workspace = TwinWorkspace

    # ------------------------------------------------------------------ embedding / norms
    def embedding(self, ids, table, out):
        out.copy_(table[ids.long()])        # a float table under bfloat16 activations is rounded here

    slot_sum_deferral_tokens = 64

    def rms_norm(self, x, weight, eps, out, residual=None, rows=None, write_residual=True, slots=1):
        z = x.float()
        if slots > 1:       # a token's slots, added in float in slot order and rounded to the storage type
            parts = z.view(-1, slots, z.shape[-1])
            acc = torch.zeros_like(parts[:, 0])
            for k in range(slots):
                acc = acc + parts[:, k]
            z = _r(acc, x.dtype)
        if residual is not None:
            z = z + residual.float()
        if rows is not None:
            z = z[rows.long()]
        elif residual is not None and write_residual:
            residual.copy_(z.to(residual.dtype))
        y = z * torch.rsqrt(z.square().mean(-1, keepdim=True) + eps) * weight.float()
        out.copy_(y.to(out.dtype))

    # ------------------------------------------------------------------ attention inputs
    def qk_norm_rope_store(self, qkv, positions, cos_sin, q_weight, k_weight, eps, heads, kv_heads,
                           head_dim, rotary_dim, cache=None, slots=None, page_size=0, pairing="neox",
                           per_head_norm=False):
        T = qkv.shape[0]
        dt = qkv.dtype
        qw, kw = heads * head_dim, kv_heads * head_dim
        q = qkv[:, :qw].float()
        k = qkv[:, qw:qw + kw].float()
        v = qkv[:, qw + kw:]
        if q_weight is not None:
            def flat(x, w):
                inv = torch.rsqrt(x.square().sum(-1, keepdim=True) / x.shape[-1] + eps)
                return _r(_r(x * inv, dt) * _r(w.float(), dt), dt)

            def per_head(x, w, n):       # one statistic per token and head; the product in float, rounded once
                x = x.view(T, n, head_dim)
                inv = torch.rsqrt(x.square().sum(-1, keepdim=True) / head_dim + eps)
                return _r(x * inv * w.float(), dt).reshape(T, n * head_dim)
            if per_head_norm:
                q, k = per_head(q, q_weight, heads), per_head(k, k_weight, kv_heads)
            else:
                q, k = flat(q, q_weight), flat(k, k_weight)
        if rotary_dim:
            half = rotary_dim // 2
            cs = cos_sin[positions.long()]
            cos, sin = cs[:, None, :half], cs[:, None, half:]

            def rot(x, n):
                x = x.view(T, n, head_dim)
                if pairing == "interleaved":     # neighbours (2 j, 2 j + 1) turn by angle j
                    x1, x2 = x[..., 0:rotary_dim:2], x[..., 1:rotary_dim:2]
                    turned = torch.stack((x1 * cos - x2 * sin, x2 * cos + x1 * sin), -1).reshape(T, n, rotary_dim)
                    return torch.cat((turned, x[..., rotary_dim:]), -1).reshape(T, -1)
                x1, x2 = x[..., :half], x[..., half:rotary_dim]
                return torch.cat((x1 * cos - x2 * sin, x2 * cos + x1 * sin, x[..., rotary_dim:]), -1).reshape(T, -1)
            q, k = rot(q, heads), rot(k, kv_heads)
        qkv[:, :qw] = q.to(dt)
        qkv[:, qw:qw + kw] = k.to(dt)
        if cache is not None:
            keep = slots >= 0
            s = slots[keep].long()
            page, off = s // page_size, s % page_size
            layout.write_keys(cache, page, off, qkv[keep, qw:qw + kw].view(-1, kv_heads, head_dim))
            layout.write_values(cache, page, off, v[keep].reshape(-1, kv_heads, head_dim))

    def paged_attention(self, q, cache, meta, out, scale, window=0):
        T, H, D = q.shape
        Hkv, ps = cache.shape[2], cache.shape[3]
        group = H // Hkv
        dt = q.dtype
        for t in range(T):
            pos = int(meta.positions[t])
            row = int(meta.token_row[t])
            first = max(0, pos - window + 1) if window else 0
            n = torch.arange(first, pos + 1, device=q.device)
            pages = meta.block_table[row, (n // ps)].long()
            keys = layout.read_keys(cache, pages, n % ps).float()      # [n, Hkv, D]
            vals = layout.read_values(cache, pages, n % ps).float()
            qt = q[t].float().view(Hkv, group, D)
            scores = torch.einsum("hgd,nhd->hgn", qt, keys) * scale
            m = scores.max(-1, keepdim=True).values
            p = torch.exp(scores - m)
            o = torch.einsum("hgn,nhd->hgd", _r(p, dt), vals) / p.sum(-1, keepdim=True)
            out[t] = o.reshape(-1).to(dt)

    # ------------------------------------------------------------------ mixture of experts
    def router_logits(self, x, weight, out):
        return torch.mm(x.float(), weight.t(), out=out)

    def router_topk(self, logits, bias, top_k, ids, weights, scoring="sigmoid", normalize=True, scaling=1.0,
                    workspace=None):
        s = torch.sigmoid(logits) if scoring == "sigmoid" else torch.softmax(logits, -1)
        sel = s + bias if bias is not None else s.clone()
        sel = torch.where(torch.isnan(sel), torch.full_like(sel, float("inf")), sel)
        T, E = sel.shape
        # the k largest, lowest index first among equals; then the reference's output order
        order = torch.argsort(sel, dim=-1, descending=True, stable=True)[:, :top_k]
        thr = sel.gather(1, order[:, -1:])
        chosen = torch.zeros_like(sel, dtype=torch.bool).scatter_(1, order, True)
        greater = chosen & (sel > thr)
        ties = chosen & ~greater
        idx = torch.arange(E, device=sel.device).expand(T, E)
        key = torch.where(greater, idx, torch.where(ties, idx + E, idx + 2 * E))
        out_ids = torch.argsort(key, dim=-1, stable=True)[:, :top_k]
        w = s.gather(1, out_ids)
        if normalize:
            w = w / w.sum(-1, keepdim=True)
        ids.copy_(out_ids.to(torch.int32))
        weights.copy_(w * scaling)

    def route(self, x, weight, bias, top_k, logits, ids, weights, scoring="sigmoid", normalize=True, scaling=1.0,
              workspace=None):
        self.router_logits(x, weight, logits)
        self.router_topk(logits, bias, top_k, ids, weights, scoring=scoring, normalize=normalize, scaling=scaling)

    @staticmethod
    def _act(gate, activation):
        if activation == "gelu_tanh":
            return torch.nn.functional.gelu(gate, approximate="tanh")
        assert activation == "silu"
        return gate * torch.sigmoid(gate)

    def moe_experts(self, x, w13, w2, ids, weights, out, ws=None, tiled=False, sum_slots=True, activation="silu"):
        dt = x.dtype
        T, h = x.shape
        E, two_i, _ = w13.shape
        I = two_i // 2
        K = ids.shape[1]
        slot_out = torch.zeros(T, K, h, dtype=torch.float32, device=x.device)
        xf = x.float()
        for e in range(E):
            tok, slot = torch.where(ids == e)
            if tok.numel() == 0:
                continue
            gu = xf[tok] @ w13[e].float().T
            gate, up = _r(gu[:, :I], dt), _r(gu[:, I:], dt)
            act = _r(_r(self._act(gate, activation), dt) * up, dt)
            y = (act @ w2[e].float().T) * weights[tok, slot, None]
            slot_out[tok, slot] = _r(y, dt)
        if not sum_slots:       # the caller adds the slots up: [tokens * top_k, hidden] in the storage type
            return slot_out.to(dt).view(T * K, h)
        out.copy_(slot_out.sum(1).to(dt))

    def silu_mul(self, x, out, activation="silu"):
        dt = x.dtype
        w = x.shape[1] // 2
        gate, up = x[:, :w].float(), x[:, w:].float()
        out.copy_((_r(self._act(gate, activation), dt) * up).to(dt))

    # ------------------------------------------------------------------ sampling
    @staticmethod
    def uniform(seed: int, vocab: int) -> np.ndarray:
        with np.errstate(over="ignore"):
            i = np.arange(1, vocab + 1, dtype=np.uint64)
            x = np.uint64(seed & (2**64 - 1)) + np.uint64(0x9E3779B97F4A7C15) * i
            x ^= x >> np.uint64(30)
            x *= np.uint64(0xBF58476D1CE4E5B9)
            x ^= x >> np.uint64(27)
            x *= np.uint64(0x94D049BB133111EB)
            x ^= x >> np.uint64(31)
        return ((x >> np.uint64(41)).astype(np.float32) + np.float32(0.5)) * np.float32(1.0 / 8388608.0)

    def sample(self, logits, temperature, top_k, top_p, seeds, out):
        rows, vocab = logits.shape
        for r in range(rows):
            row = logits[r].float().cpu()
            temp = float(temperature[r]) if temperature is not None else 0.0
            if not temp > 1e-10:
                out[r] = int(torch.argmax(row))
                continue
            l = row * np.float32(1.0 / np.float32(temp))
            keep = torch.ones(vocab, dtype=torch.bool)
            k = int(top_k[r]) if top_k is not None else 0
            if 0 < k < vocab:
                kth = torch.topk(l, k).values[-1]
                keep &= l >= kth
            p = float(top_p[r]) if top_p is not None else 1.0
            if p < 1.0:
                e = torch.where(keep, torch.exp(l - l.max()), torch.zeros_like(l))
                order = torch.argsort(l, descending=True, stable=True)
                sorted_e = e[order]
                # mass of strictly more probable tokens
                cum = torch.cumsum(sorted_e, 0) - sorted_e
                sl = l[order]
                first_of_value = torch.ones_like(sl, dtype=torch.bool)
                first_of_value[1:] = sl[1:] != sl[:-1]
                start = torch.cummax(torch.where(first_of_value, torch.arange(vocab), torch.zeros(vocab, dtype=torch.long)), 0).values
                strictly_more = cum[start]
                ok = strictly_more <= np.float32(p) * e.sum()
                keep_sorted = ok
                keep2 = torch.zeros(vocab, dtype=torch.bool)
                keep2[order] = keep_sorted
                keep &= keep2
            seed = int(seeds[r]) if seeds is not None else 0
            u = torch.from_numpy(self.uniform(seed, vocab))
            noisy = l - torch.log(-torch.log(u))
            noisy[~keep] = float("-inf")
            out[r] = int(torch.argmax(noisy))
