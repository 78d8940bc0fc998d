"""The batch of one step as the parts see it.

A step is a list of items ``(row, tokens, want)``: a request's next tokens (a portion of its
prompt, or one decoded token) and the places among them whose logits are asked for.  The builder
reserves cache room for all items at once, packs every integer the kernels need into one host
buffer and sends it with a single copy.  Nothing here is global: the ``ForwardBatch`` object is
passed down to the parts (the reference passes a module-level context, utils/context.py:26-41,
and builds prefill and decode batches apart, engine/cache_manager/standard.py:2065-2206).
"""
from __future__ import annotations

from dataclasses import dataclass, field

import numpy as np
import torch

from ..cache.manager import CacheManager
from ..kernels.attention_work import DeviceAttentionWork, build_attention_work
from ..parts.base import StepScratch


@dataclass
class StepItem:
    row: int
    tokens: list[int]
    want: list[int] = field(default_factory=list)     # indices into ``tokens``


@dataclass
class GroupMeta:
    """Per cache group: where every token of the step lives and how to find its request's pages."""
    block_table: torch.Tensor      # int32 [items, pages]: compact table of the step's requests
    token_row: torch.Tensor        # int32 [T] index of the token's item = row of block_table
    positions: torch.Tensor        # int32 [T]
    slots: torch.Tensor            # int32 [T] page * page_size + offset of the token's own key
    page_size: int
    block_table_host: np.ndarray = None   # block_table on the host (for checks before a launch)
    # host copies for kernels that build a work list
    item_q_start: np.ndarray = None
    item_q_len: np.ndarray = None
    item_ctx_len: np.ndarray = None
    item_meta: torch.Tensor = None     # int32 [3, items] on the device: q_start, q_len, ctx_len
    max_ctx_len: int = 0
    max_q_len: int = 0
    # (query heads per kv head, window) -> (units, num_units, tasks, num_tasks, partial slots) of
    # the matrix-core attention kernel, prepared with the rest of the step's integers
    work: dict = field(default_factory=dict)


class ForwardBatch:
    def __init__(self, kernels, cache: CacheManager, dtype: torch.dtype, device, scratch: StepScratch):
        self.kernels = kernels
        self.cache = cache
        self.dtype = dtype
        self.device = device
        self.scratch = scratch
        self.num_tokens = 0
        self.num_items = 0
        self.token_ids = None          # int32 [T]
        self.positions = None          # int32 [T]
        self.token_item = None         # int32 [T]
        self.item_rows = None          # int32 [items]: the cache row (state slot) of every item
        self.item_rows_host = None
        # where every item's tokens lie in the step and how long its request is with them: host
        # copies (int32 numpy [items]) and one device tensor [3, items] = q_start, q_len, ctx_len.
        # They belong to the step, not to a cache group: a mixer that keeps state only reads them too.
        self.item_q_start = None
        self.item_q_len = None
        self.item_ctx_len = None
        self.item_meta = None
        self.schedule_position = 0     # the schedule position whose layer is running
        self.method = None             # the sparse method's runtime (config/method_registry.py)
        self.want_index = None         # int32 [wanted] token indices whose logits are returned
        self.groups: dict[int, GroupMeta] = {}
        self.taps: dict | None = None
        self.check_tables = False      # check every block-table entry a launch will read (a debug option)

    # views the mixers use ---------------------------------------------------------------
    def kv_view(self, position: int):
        """(layer tensor, GroupMeta) of the schedule position that owns the cache."""
        return self.cache.kv_layer(position), self.groups[self.cache.group_of_position[position]]

    def state_view(self, position: int) -> dict[str, torch.Tensor]:
        """name -> [rows, ...] state tensors of the position; index them with ``item_rows``."""
        return self.cache.state[position]

    def check_block_table(self, meta, window: int, num_pages: int, where: str = "") -> None:
        check_block_table(meta, window, num_pages, where)

    def buffer(self, key: str, shape, dtype=None) -> torch.Tensor:
        """A reusable scratch tensor whose leading dims are cut to ``shape``."""
        return self.scratch.view(key, shape if type(shape) is tuple else tuple(shape), dtype or self.dtype, self.device)


class BlockTableError(RuntimeError):
    pass


def check_block_table(meta, window: int, num_pages: int, where: str = "") -> None:
    """Before an attention launch: every block-table entry that the launch will read names a page of the
    pool.  Item ``i`` holds ``ctx_len[i]`` tokens of which the last ``q_len[i]`` are this step's queries; its
    first query sees the keys from ``max(0, position - window + 1)`` on (``window`` 0: all), so the entries
    from that key's page to the last key's page are read and must lie in ``[0, num_pages)``; entries before
    them may be -1 (pages a window has given back) and are not read.  A kernel that follows a bad entry
    reads outside the cache tensor, which the device may or may not answer with a memory fault.
    (The reference checks its slot tables the same way under a debug flag, layers/attention_backend.py:155-215.)"""
    table = getattr(meta, "block_table_host", None)
    if table is None:
        table = meta.block_table.cpu().numpy()
    q_len, ctx_len, page = np.asarray(meta.item_q_len), np.asarray(meta.item_ctx_len), int(meta.page_size)
    first_query = ctx_len - q_len
    low_key = np.maximum(0, first_query - window + 1) if window else np.zeros_like(ctx_len)
    if (q_len <= 0).any() or (first_query < 0).any():
        raise BlockTableError(f"{where}: an item with {q_len.tolist()} queries of {ctx_len.tolist()} tokens")
    first_page, until_page = low_key // page, -(-ctx_len // page)
    if int(until_page.max()) > table.shape[1]:
        raise BlockTableError(f"{where}: the block table has {table.shape[1]} columns, an item needs {int(until_page.max())}")
    column = np.arange(table.shape[1])[None, :]
    read = (column >= first_page[:, None]) & (column < until_page[:, None])
    bad = read & ((table < 0) | (table >= num_pages))
    if bad.any():
        item, col = (int(v[0]) for v in np.nonzero(bad))
        raise BlockTableError(
            f"{where}: item {item} (tokens {int(ctx_len[item])}, queries {int(q_len[item])}, window {window or 'none'}) "
            f"would read block-table entry {col} = {int(table[item, col])}; the pool has pages 0..{num_pages - 1}")


class BatchBuilder:
    """Turns step items into a ``ForwardBatch``: cache reservation + one packed host-to-device copy."""

    def __init__(self, kernels, cache: CacheManager, dtype, device, vocab_size: int,
                 attention_shapes: dict | None = None):
        """``attention_shapes``: cache group index -> set of (query heads per kv head, window) whose
        attention work lists are to be prepared with every batch."""
        self.kernels, self.cache, self.dtype, self.device = kernels, cache, dtype, torch.device(device)
        self.vocab_size = vocab_size
        self.attention_shapes = attention_shapes or {}
        self.scratch = StepScratch()
        self._host = None
        self._dev = None
        self._copied = None            # event after the last host-to-device copy

    def _buffers(self, n: int):
        if self._host is None or self._host.numel() < n:
            size = max(n, 4096) * 2
            pin = self.device.type == "cuda"
            self._host = torch.empty(size, dtype=torch.int32, pin_memory=pin)
            self._dev = torch.empty(size, dtype=torch.int32, device=self.device)
        return self._host, self._dev

    def build(self, items: list[StepItem]) -> ForwardBatch:
        if not items:
            raise ValueError("a step needs at least one item")
        cache = self.cache
        lengths = [len(it.tokens) for it in items]
        T, B = sum(lengths), len(items)
        if T == B and min(lengths) == 1:
            # a step of single tokens (decoding): the same checks and the same arrays without a loop over the items;
            # what the host spends here is time the device waits between two steps
            rows = np.asarray([it.row for it in items], dtype=np.int32)
            token_ids = np.asarray([it.tokens[0] for it in items], dtype=np.int64)
            if token_ids.min() < 0 or token_ids.max() >= self.vocab_size:
                bad = token_ids[(token_ids < 0) | (token_ids >= self.vocab_size)]
                raise ValueError(f"token id {int(bad[0])} is outside the vocabulary [0, {self.vocab_size})")
            token_ids = token_ids.astype(np.int32)
            for it in items:
                if it.want and any(w != 0 for w in it.want):
                    raise ValueError("a wanted place lies outside the item's tokens")
            positions = cache.row_len[rows].astype(np.int32)
            allocation = cache.append([(it.row, 1) for it in items])   # all or nothing
            q_start = token_item = np.arange(B, dtype=np.int32)
            q_len = np.ones(B, dtype=np.int32)
            ctx_len = positions + 1
            want = np.asarray([i for i, it in enumerate(items) for _ in it.want], dtype=np.int32)
        else:
            for it in items:
                if not it.tokens:
                    raise ValueError("an item without tokens")
                bad = [t for t in it.tokens if not 0 <= t < self.vocab_size]
                if bad:
                    raise ValueError(f"token id {bad[0]} is outside the vocabulary [0, {self.vocab_size})")
                if any(not 0 <= w < len(it.tokens) for w in it.want):
                    raise ValueError("a wanted place lies outside the item's tokens")
            starts = [int(cache.row_len[it.row]) for it in items]
            allocation = cache.append([(it.row, n) for it, n in zip(items, lengths)])   # all or nothing
            q_start = np.zeros(B, dtype=np.int32)
            q_start[1:] = np.cumsum(lengths[:-1])
            q_len = np.asarray(lengths, dtype=np.int32)
            ctx_len = np.asarray([s + n for s, n in zip(starts, lengths)], dtype=np.int32)
            token_ids = np.concatenate([np.asarray(it.tokens, dtype=np.int32) for it in items])
            positions = np.concatenate([np.arange(s, s + n, dtype=np.int32) for s, n in zip(starts, lengths)])
            token_item = np.repeat(np.arange(B, dtype=np.int32), lengths)
            want = np.asarray([q_start[i] + w for i, it in enumerate(items) for w in it.want], dtype=np.int32)
            rows = np.asarray([it.row for it in items], dtype=np.int32)

        tables = {}
        for group in cache.groups:
            width = max(1, -(-int(ctx_len.max()) // group.page_size))
            tables[group.index] = np.ascontiguousarray(group.table[rows, :width])

        item_meta_host = np.stack([q_start, q_len, ctx_len]).astype(np.int32)      # one part: [3, items]
        parts = [token_ids, positions, token_item, rows, item_meta_host.reshape(-1), want]
        for group in cache.groups:
            parts += [allocation.slots[group.index], tables[group.index].reshape(-1)]
        works = []
        if self.attention_shapes:
            for group in cache.groups:
                for ratio, window in sorted(self.attention_shapes.get(group.index, ())):
                    work = build_attention_work(q_len, ctx_len, ratio, group.request.kv_heads, window,
                                                head_dim=group.request.head_dim)
                    works.append((group.index, (ratio, window), work, len(parts)))
                    parts += [work.units.reshape(-1), work.tasks.reshape(-1), work.block_units.reshape(-1)]
        # every part starts on a 16-byte boundary: kernels read records of four ints at once
        total = sum(-(-p.size // 4) * 4 for p in parts)
        if self._copied is not None:
            self._copied.synchronize()  # the last step's copy has left the pinned buffer
        host, dev = self._buffers(total)
        host_np = host.numpy()
        offsets, cursor = [], 0
        for p in parts:
            host_np[cursor:cursor + p.size] = p.reshape(-1)
            offsets.append(cursor)
            cursor += -(-p.size // 4) * 4
        dev[:total].copy_(host[:total], non_blocking=True)
        if self.device.type == "cuda":
            self._copied = torch.cuda.Event()
            self._copied.record()

        def view(i, shape=None):
            v = dev[offsets[i]:offsets[i] + parts[i].size]
            return v if shape is None else v.view(shape)

        fb = ForwardBatch(self.kernels, cache, self.dtype, self.device, self.scratch)
        fb.num_tokens, fb.num_items = T, B
        fb.token_ids, fb.positions, fb.token_item = view(0), view(1), view(2)
        fb.item_rows, fb.item_rows_host = view(3), rows
        fb.want_index = view(5)
        item_meta = view(4, (3, B))
        fb.item_q_start, fb.item_q_len, fb.item_ctx_len, fb.item_meta = q_start, q_len, ctx_len, item_meta
        for gi, group in enumerate(cache.groups):
            fb.groups[group.index] = GroupMeta(
                block_table=view(6 + 2 * gi + 1, tables[group.index].shape),
                block_table_host=tables[group.index],
                token_row=fb.token_item, positions=fb.positions, slots=view(6 + 2 * gi),
                page_size=group.page_size, item_q_start=q_start, item_q_len=q_len,
                item_ctx_len=ctx_len, item_meta=item_meta, max_ctx_len=int(ctx_len.max()),
                max_q_len=int(q_len.max()))
        for group_index, key, work, at in works:
            fb.groups[group_index].work[key] = DeviceAttentionWork(
                view(at, work.units.shape), work.units.shape[0], view(at + 1, work.tasks.shape),
                work.tasks.shape[0], work.num_slots, view(at + 2, work.block_units.shape),
                work.block_units.shape[0], work.tiles_per_block)
        return fb
