"""Sampling of one token per logits row.

Greedy rows take the arg-max; other rows are scaled by 1/temperature, cut to the top-k, then to
the nucleus of mass top_p among the survivors, and drawn from what is left (the reference's
order, layers/sampler.py:66-122).  The draw is the arg-max of logit + Gumbel noise, the same
distribution as the reference's ``probs / Exp(1)`` arg-max; the noise is a counter-based function
of (sampler seed, request seed, position), so a request's tokens do not depend on which other
requests share its batch.  Penalties (layers/sampler.py:11-64) are applied to the float logits
before the kernel; log-probabilities are ``log_softmax`` of the penalised float logits.
"""
from __future__ import annotations

import numpy as np
import torch

_MASK = (1 << 64) - 1


def mix64(x: int) -> int:
    """splitmix64 finaliser."""
    x = (x + 0x9E3779B97F4A7C15) & _MASK
    x = ((x ^ (x >> 30)) * 0xBF58476D1CE4E5B9) & _MASK
    x = ((x ^ (x >> 27)) * 0x94D049BB133111EB) & _MASK
    return x ^ (x >> 31)


def row_seed(sampler_seed: int, request_seed: int, position: int) -> int:
    """64 bits that identify one draw; returned as a signed value that fits an int64 tensor."""
    value = mix64(mix64(mix64(sampler_seed & _MASK) ^ (request_seed & _MASK)) ^ (position & _MASK))
    return value - (1 << 64) if value >= (1 << 63) else value


class Sampler:
    def __init__(self, kernels, device, sampler_seed: int = 0):
        self.kernels = kernels
        self.device = torch.device(device)
        self.sampler_seed = int(sampler_seed)

    def apply_penalties(self, logits: torch.Tensor, rows) -> torch.Tensor:
        """``rows``: per logits row (params, prompt ids, completion ids[, a dict that lives as long as the
        request]).  The distinct tokens of a prompt are worked out once per request and kept in that dict (a
        prompt of many thousand tokens would otherwise cost milliseconds of set building in every step).
        All rows are changed together, through flat positions ``row * vocab + token``: a dozen launches a
        step instead of a dozen a row.  A token named twice is still changed once."""
        if not any(row[0].presence_penalty != 0.0 or row[0].repetition_penalty != 1.0 for row in rows):
            return logits
        logits = logits.clone(memory_format=torch.contiguous_format)
        n, vocab = logits.shape
        flat = logits.view(-1)
        prompts, repeated, present = [], [], []
        for r, row in enumerate(rows):
            p, prompt, completion = row[:3]
            kept = row[3] if len(row) > 3 else None
            if p.repetition_penalty != 1.0:
                if prompt:
                    seen = kept.get("prompt_tokens") if kept is not None else None
                    if seen is None or seen.device != logits.device:
                        seen = torch.tensor(sorted(set(prompt)), dtype=torch.long, device=logits.device)
                        if kept is not None:
                            kept["prompt_tokens"] = seen
                    prompts.append(seen + r * vocab)
                repeated += [r * vocab + t for t in completion]
            if p.presence_penalty != 0.0:
                present += [r * vocab + t for t in completion]
        # one copy: the rows' two penalties, then the flat positions of the completions' tokens
        packed = np.empty(8 * n + 8 * (len(repeated) + len(present)), dtype=np.uint8)
        packed[:4 * n].view(np.float32)[:] = [row[0].repetition_penalty for row in rows]
        packed[4 * n:8 * n].view(np.float32)[:] = [row[0].presence_penalty for row in rows]
        packed[8 * n:].view(np.int64)[:] = repeated + present
        on_device = torch.from_numpy(packed).to(logits.device)
        repetition, presence = on_device[:4 * n].view(torch.float32), on_device[4 * n:8 * n].view(torch.float32)
        places = on_device[8 * n:].view(torch.int64)
        where = torch.cat(prompts + [places[:len(repeated)]]) if prompts else places[:len(repeated)]
        if where.numel():
            values, factor = flat[where], repetition[where // vocab]
            flat[where] = torch.where(values > 0, values / factor, values * factor)
        if present:
            where = places[len(repeated):]
            flat[where] = flat[where] - presence[where // vocab]
        return logits

    def sample(self, logits: torch.Tensor, rows, seeds_and_positions) -> list[int]:
        """``logits`` float32 ``[n, vocab]``; ``rows`` as in ``apply_penalties``;
        ``seeds_and_positions``: per row (request seed, index of the token being drawn)."""
        n = logits.shape[0]
        params = [row[0] for row in rows]
        out = torch.empty(n, dtype=torch.int32, device=logits.device)
        if all(p.greedy for p in params):
            self.kernels.sample(logits, None, None, None, None, out)
            return out.tolist()
        # the rows' settings go to the device in one copy: seeds (64 bits each), then temperatures, top_p, top_k
        packed = np.empty(n * 20, dtype=np.uint8)
        packed[:8 * n].view(np.int64)[:] = [row_seed(self.sampler_seed, s, pos) for s, pos in seeds_and_positions]
        packed[8 * n:12 * n].view(np.float32)[:] = [0.0 if p.greedy else p.temperature for p in params]
        packed[12 * n:16 * n].view(np.float32)[:] = [p.top_p for p in params]
        packed[16 * n:].view(np.int32)[:] = [p.top_k for p in params]
        on_device = torch.from_numpy(packed).to(logits.device)
        seeds = on_device[:8 * n].view(torch.int64)
        temperature = on_device[8 * n:12 * n].view(torch.float32)
        top_p = on_device[12 * n:16 * n].view(torch.float32) if any(p.top_p < 1.0 for p in params) else None
        top_k = on_device[16 * n:].view(torch.int32) if any(p.top_k for p in params) else None
        self.kernels.sample(logits, temperature, top_k, top_p, seeds, out)
        return out.tolist()

    @staticmethod
    def logprobs(logits: torch.Tensor, tokens: list[int], top: list[int | None]):
        """(log-probability of each chosen token, per row {token: logprob} of its top entries)."""
        if all(t is None for t in top):
            return [None] * len(tokens), [None] * len(tokens)
        logp = torch.log_softmax(logits, dim=-1)
        chosen = logp.gather(1, torch.tensor(tokens, device=logits.device)[:, None])
        most = max(k or 0 for k in top)
        if most:        # one top-k for all rows (a row's first k entries are its own top k), one copy to the host
            values, ids = torch.topk(logp, min(most, logp.shape[1]))
            chosen, values, ids = torch.cat((chosen, values), 1).tolist(), None, ids.tolist()
        else:
            chosen, ids = chosen.tolist(), None
        tops = []
        for r, k in enumerate(top):
            tops.append(None if k is None else dict(zip(ids[r][:k], chosen[r][1:1 + k])) if k else {})
        return [chosen[r][0] if k is not None else None for r, k in enumerate(top)], tops
