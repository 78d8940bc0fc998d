"""Trace generators of the replay tests and the bookkeeping to compare replays with each other.

Every generator returns trace records (the JSON objects ``bin/trace_run`` reads) that feed the same
requests in a different way: whole, whole minus a tail decoded one by one, in portions of changing
size, and mixed with other requests under a small page pool.
"""
from __future__ import annotations

import random

import numpy as np


def whole(requests: dict[str, list[int]]):
    """Each request alone, in one step, every position wanted."""
    return [{"step": i, "entries": [{"id": rid, "tokens": toks, "want": list(range(len(toks)))}], "end": [rid]}
            for i, (rid, toks) in enumerate(requests.items())]


def prefill_then_decode(requests, tail: int = 32):
    """All but the last ``tail`` tokens in one step, then the tail one token a step."""
    records, step = [], 0
    for rid, toks in requests.items():
        head = max(1, len(toks) - tail)
        records.append({"step": step, "entries": [{"id": rid, "tokens": toks[:head], "want": list(range(head))}], "end": []})
        step += 1
        for i in range(head, len(toks)):
            records.append({"step": step, "entries": [{"id": rid, "tokens": toks[i:i + 1], "want": [0]}],
                            "end": [rid] if i == len(toks) - 1 else []})
            step += 1
        if head == len(toks):
            records[-1]["end"] = [rid]
    return records


def changing_portions(requests, seed: int = 0, sizes=(7, 2, 16, 3, 2, 31, 1, 5, 64, 2, 9)):
    """One request at a time, cut into portions whose sizes cycle through ``sizes`` from a seeded start."""
    rng = random.Random(seed)
    records, step = [], 0
    for rid, toks in requests.items():
        k, i = rng.randrange(len(sizes)), 0
        while i < len(toks):
            n = min(sizes[k % len(sizes)], len(toks) - i)
            k += 1
            records.append({"step": step, "entries": [{"id": rid, "tokens": toks[i:i + n], "want": list(range(n))}],
                            "end": [rid] if i + n == len(toks) else []})
            i += n
            step += 1
    return records


def mixed(requests, seed: int = 0, max_live: int = 4, tail: int = 12, max_portion: int = 19):
    """Up to ``max_live`` requests at a time; a step holds portions of some prompts beside single
    (decoded) tokens of others; requests are sometimes left out of a step; a finished request
    makes room for the next.  Returns (records, peak of live tokens rounded up to 64 per request)."""
    rng = random.Random(seed)
    waiting = list(requests.items())
    live: dict[str, int] = {}          # id -> tokens fed so far
    records, step, peak = [], 0, 0
    while waiting or live:
        while waiting and len(live) < max_live:
            rid, _ = waiting.pop(0)
            live[rid] = 0
        entries, ended = [], []
        chosen = [rid for rid in live if rng.random() < 0.8] or [next(iter(live))]
        for rid in chosen:
            toks, fed = requests[rid], live[rid]
            in_tail = fed >= max(1, len(toks) - tail)
            n = 1 if in_tail else min(rng.randint(2, max_portion), max(1, len(toks) - tail) - fed)
            entries.append({"id": rid, "tokens": toks[fed:fed + n], "want": list(range(n))})
            live[rid] = fed + n
            if live[rid] == len(toks):
                ended.append(rid)
        peak = max(peak, sum(-(-max(v, 1) // 64) * 64 for v in live.values()))
        records.append({"step": step, "entries": entries, "end": ended})
        for rid in ended:
            del live[rid]
        step += 1
    return records, peak


def gather(records, logits_of_step: dict[int, np.ndarray]) -> dict[str, np.ndarray]:
    """Reassemble per request the logits rows in position order from the per-step arrays."""
    rows: dict[str, list] = {}
    for rec in records:
        arr = logits_of_step.get(rec["step"])
        cursor = 0
        for e in rec["entries"]:
            for _ in e.get("want", []):
                rows.setdefault(e["id"], []).append(arr[cursor])
                cursor += 1
        assert arr is None or cursor == arr.shape[0]
    return {rid: np.stack(r) for rid, r in rows.items()}
