"""The cache manager: paged keys and values with a block table per request, grouped by need,
and, beside them, slots of fixed size for per-request state.

A live request holds one *row* from admission to release.  For every *group* of cache-keeping
schedule positions with the same geometry (kv heads, head size, window) the row has a list of
pages; a page id addresses the same page in every layer tensor of its group.  Groups have pools
of their own.  Pages return to their pool when the request ends, or, in a windowed group, as soon
as every query still to come lies more than ``window`` tokens past the page's last key.  State
tensors are indexed by the same row id and zeroed on admission.

The reference keeps one token per slot (engine/cache_manager/standard.py:127-137,1752-1789) and
frees a request's slots at once on finish, preemption, abort or failure (:1951-1999); pages,
groups and window release are this engine's own design.
"""
from __future__ import annotations

from collections import deque
from dataclasses import dataclass, field

import numpy as np
import torch

from ..parts.base import PagedKVRequest, StateRequest
from .page_pool import OutOfPages, PageOwnershipError, PagePool


class OutOfRows(RuntimeError):
    pass


@dataclass
class KVGroup:
    """Schedule positions that share page geometry, a pool and a block table."""
    index: int
    request: PagedKVRequest
    positions: list[int]
    page_size: int
    pool: PagePool
    table: np.ndarray                      # [rows, max_pages] int32, -1 where no page is held
    first_live: np.ndarray                 # [rows] index of the first page still held
    layers: dict[int, torch.Tensor] = field(default_factory=dict)   # position -> [pages, 2, Hkv, ps, D]

    @property
    def window(self):
        return self.request.window

    def bytes_per_page(self, itemsize: int) -> int:
        r = self.request
        return len(self.positions) * 2 * r.kv_heads * self.page_size * r.head_dim * itemsize


@dataclass
class StepAllocation:
    """What an ``append`` decided: for every group the slot of every new token, in item order."""
    slots: dict[int, np.ndarray]           # group index -> int32 [tokens]


class CacheManager:
    def __init__(self, requests: dict[int, object], *, max_rows: int, max_model_len: int,
                 page_size: int, num_pages: int | dict | None = None, num_tokens: int | None = None,
                 dtype: torch.dtype, device, allocate_tensors: bool = True):
        """``requests``: schedule position -> PagedKVRequest | StateRequest (positions that read
        another position's cache are not listed).  ``page_size``: tokens per page of the groups whose
        request names none.  The pools' sizes: ``num_tokens`` (every group gets the pages that hold so
        many tokens) or ``num_pages`` (an int for all groups or {group index: pages})."""
        if page_size <= 0 or max_rows <= 0 or max_model_len <= 0:
            raise ValueError("page_size, max_rows and max_model_len must be positive")
        self.page_size = int(page_size)          # the default; a group's own is ``group.page_size``
        self.max_rows = int(max_rows)
        self.max_model_len = int(max_model_len)
        self.dtype, self.device = dtype, device

        by_geometry: dict[PagedKVRequest, list[int]] = {}
        self.state_positions: dict[int, StateRequest] = {}
        for position, req in sorted(requests.items()):
            if isinstance(req, PagedKVRequest):
                by_geometry.setdefault(req, []).append(position)
            elif isinstance(req, StateRequest):
                self.state_positions[position] = req
            elif req is not None:
                raise TypeError(f"position {position}: unknown cache request {req!r}")
        self.groups: list[KVGroup] = []
        self.group_of_position: dict[int, int] = {}
        for index, (req, positions) in enumerate(by_geometry.items()):
            ps = int(req.page_size or self.page_size)
            if ps <= 0 or ps % 8:
                raise ValueError(f"a cache page holds a multiple of 8 tokens (it keeps its elements in groups of "
                                 f"eight, cache/layout.py), got {ps}")
            if num_tokens is not None:
                pages = max(1, -(-int(num_tokens) // ps))      # a last page may be partly beyond the count
            else:
                pages = num_pages[index] if isinstance(num_pages, dict) else num_pages
            if pages is None:
                raise ValueError("num_pages or num_tokens must be given")
            group = KVGroup(index, req, positions, ps, PagePool(int(pages)),
                            np.full((self.max_rows, -(-self.max_model_len // ps)), -1, dtype=np.int32),
                            np.zeros(self.max_rows, dtype=np.int64))
            if allocate_tensors:
                for position in positions:
                    group.layers[position] = torch.zeros(
                        int(pages), 2, req.kv_heads, ps, req.head_dim, dtype=dtype, device=device)
            self.groups.append(group)
            for position in positions:
                self.group_of_position[position] = index

        self.state: dict[int, dict[str, torch.Tensor]] = {}
        for position, req in self.state_positions.items():
            self.state[position] = {
                name: torch.zeros((self.max_rows, *shape), dtype=dt or dtype, device=device)
                for name, shape, dt in req.tensors} if allocate_tensors else {}

        self._no_window = all(group.window is None for group in self.groups)
        self.row_len = np.zeros(self.max_rows, dtype=np.int64)
        self.row_owner: list[object | None] = [None] * self.max_rows
        self._free_rows = deque(range(self.max_rows))
        self._row_of: dict[object, int] = {}

    # ------------------------------------------------------------------ rows
    @property
    def num_free_rows(self) -> int:
        return len(self._free_rows)

    def has_row(self, request_id) -> bool:
        return request_id in self._row_of

    def row_of(self, request_id) -> int:
        return self._row_of[request_id]

    def admit(self, request_id) -> int:
        """Give the request a row (an empty block table and zeroed state)."""
        if request_id in self._row_of:
            raise ValueError(f"request {request_id!r} already holds row {self._row_of[request_id]}")
        if not self._free_rows:
            raise OutOfRows(f"all {self.max_rows} rows are taken")
        row = self._free_rows.popleft()
        self._row_of[request_id] = row
        self.row_owner[row] = request_id
        self.row_len[row] = 0
        for group in self.groups:
            group.first_live[row] = 0
        for tensors in self.state.values():
            for t in tensors.values():
                t[row].zero_()
        return row

    def free(self, request_id) -> None:
        """Give back every page of the request and its row."""
        if request_id not in self._row_of:
            raise PageOwnershipError(f"request {request_id!r} holds no row (freed twice?)")
        row = self._row_of.pop(request_id)
        for group in self.groups:
            held = group.table[row]
            pages = held[held >= 0].tolist()
            group.pool.release(pages, row)
            group.table[row, :] = -1
            group.first_live[row] = 0
        self.row_len[row] = 0
        self.row_owner[row] = None
        self._free_rows.append(row)

    # ------------------------------------------------------------------ capacity questions
    def _plan(self, group: KVGroup, row: int, new_tokens: int, length: int | None = None):
        """(pages to release first, pages to allocate) for appending ``new_tokens`` to the row."""
        ps = group.page_size
        length = int(self.row_len[row]) if length is None else length
        have_until = -(-length // ps)                       # pages [first_live, have_until) are held
        need_until = -(-(length + new_tokens) // ps)
        release_until = int(group.first_live[row])
        if group.window is not None:
            # the earliest query of this step sits at `length` and reads keys >= length - window + 1
            release_until = max(release_until, min(have_until, max(0, length - group.window + 1) // ps))
        return release_until, need_until - have_until

    def pages_needed(self, row: int, new_tokens: int) -> dict[int, int]:
        """Net pages every group's pool must still have free for this append."""
        out = {}
        for group in self.groups:
            release_until, alloc = self._plan(group, row, new_tokens)
            out[group.index] = alloc - (release_until - int(group.first_live[row]))
        return out

    def pages_for_tokens(self, tokens: int) -> dict[int, int]:
        """Pages of every group that a request of ``tokens`` tokens takes from an empty row."""
        return {g.index: -(-int(tokens) // g.page_size) for g in self.groups}

    def free_pages(self) -> dict[int, int]:
        return {g.index: g.pool.free_count for g in self.groups}

    def can_append(self, items) -> bool:
        """Whether ``append(items)`` would succeed; ``items`` = [(row, new_tokens)]."""
        need = {g.index: 0 for g in self.groups}
        for row, n in items:
            for gi, pages in self.pages_needed(row, n).items():
                need[gi] += pages
        free = self.free_pages()
        return all(need[gi] <= free[gi] for gi in need) and all(
            self.row_len[row] + n <= self.max_model_len for row, n in items)

    # ------------------------------------------------------------------ the append of a step
    def append(self, items) -> StepAllocation:
        """Reserve room for ``new_tokens`` more tokens of every listed row, all or nothing.

        Windowed groups first give back the pages no query of this step can reach.  Returns the
        slot (page * page_size + offset) of every new token per group."""
        rows = [row for row, _ in items]
        if len(set(rows)) != len(rows):
            raise ValueError("a row appears twice in one step")
        if self._no_window and all(n == 1 for _, n in items):
            return self._append_one_token_each(rows)
        for row, n in items:
            if self.row_owner[row] is None:
                raise PageOwnershipError(f"row {row} is not held by a request")
            if n <= 0:
                raise ValueError("an item must bring at least one token")
            if self.row_len[row] + n > self.max_model_len:
                raise ValueError(f"row {row}: {self.row_len[row]} + {n} tokens exceed max_model_len "
                                 f"{self.max_model_len}")
        if not self.can_append(items):
            raise OutOfPages(f"step of {sum(n for _, n in items)} tokens does not fit: free pages "
                             f"{self.free_pages()}")
        slots = {g.index: np.empty(sum(n for _, n in items), dtype=np.int32) for g in self.groups}
        for group in self.groups:
            ps = group.page_size
            # every release of the step comes before its first allocation: the check above
            # counted the pages that this step itself gives back
            for row, n in items:
                release_until, _ = self._plan(group, row, n)
                first = int(group.first_live[row])
                if release_until > first:
                    group.pool.release(group.table[row, first:release_until].tolist(), row)
                    group.table[row, first:release_until] = -1
                    group.first_live[row] = release_until
            cursor = 0
            for row, n in items:
                length = int(self.row_len[row])
                _, alloc = self._plan(group, row, n)
                if alloc:
                    have_until = -(-length // ps)
                    group.table[row, have_until:have_until + alloc] = group.pool.allocate(alloc, row)
                token_pos = np.arange(length, length + n)
                pages = group.table[row, token_pos // ps]
                slots[group.index][cursor:cursor + n] = pages * ps + token_pos % ps
                cursor += n
        for row, n in items:
            self.row_len[row] += n
        return StepAllocation(slots)

    def _append_one_token_each(self, rows: list[int]) -> StepAllocation:
        """``append`` for a step of single tokens where no group has a window (a decode step, whose time on the
        host is time the device waits): nothing is given back, and a row takes a new page exactly when its length
        is a multiple of the page size.  The same checks in the same order, the same pages in the same order."""
        limit = self.max_model_len
        for row in rows:
            if self.row_owner[row] is None:
                raise PageOwnershipError(f"row {row} is not held by a request")
            if self.row_len[row] + 1 > limit:
                raise ValueError(f"row {row}: {self.row_len[row]} + 1 tokens exceed max_model_len {limit}")
        index = np.asarray(rows, dtype=np.int64)
        lengths = self.row_len[index]
        fresh = []                               # per group: which items start a new page
        for group in self.groups:
            starts_page = np.nonzero(lengths % group.page_size == 0)[0]
            if starts_page.size > group.pool.free_count:
                raise OutOfPages(f"step of {len(rows)} tokens does not fit: free pages {self.free_pages()}")
            fresh.append(starts_page)
        slots = {}
        for group, starts_page in zip(self.groups, fresh):
            ps = group.page_size
            page_index = lengths // ps
            for i in starts_page.tolist():
                group.table[rows[i], page_index[i]] = group.pool.allocate(1, rows[i])[0]
            slots[group.index] = (group.table[index, page_index] * ps + lengths % ps).astype(np.int32)
        self.row_len[index] += 1
        return StepAllocation(slots)

    def truncate(self, row: int, length: int) -> None:
        """Forget the tokens beyond ``length`` (undo of an append whose step failed)."""
        if length > self.row_len[row]:
            raise ValueError("truncate cannot lengthen a row")
        for group in self.groups:
            ps = group.page_size
            keep_until = -(-length // ps)
            have_until = -(-int(self.row_len[row]) // ps)
            first = max(int(group.first_live[row]), keep_until)
            if have_until > first:
                group.pool.release(group.table[row, first:have_until].tolist(), row)
                group.table[row, first:have_until] = -1
        self.row_len[row] = length

    # ------------------------------------------------------------------ views for the step
    def kv_layer(self, position: int) -> torch.Tensor:
        return self.groups[self.group_of_position[position]].layers[position]

    def block_table_rows(self, group_index: int, rows, width: int | None = None) -> np.ndarray:
        table = self.groups[group_index].table
        return table[rows] if width is None else table[rows, :width]

    # ------------------------------------------------------------------ invariants
    def check_invariants(self) -> None:
        held_rows = set(self._row_of.values())
        if len(held_rows) != len(self._row_of) or held_rows & set(self._free_rows):
            raise PageOwnershipError("a row is held twice or is both held and free")
        if len(held_rows) + len(self._free_rows) != self.max_rows:
            raise PageOwnershipError("a row was lost")
        for group in self.groups:
            ps = group.page_size
            group.pool.check()
            seen: dict[int, int] = {}
            for row in range(self.max_rows):
                held = group.table[row]
                live = np.nonzero(held >= 0)[0]
                if row not in held_rows:
                    if live.size:
                        raise PageOwnershipError(f"free row {row} still lists pages")
                    continue
                first, until = int(group.first_live[row]), -(-int(self.row_len[row]) // ps)
                if live.tolist() != list(range(first, until)):
                    raise PageOwnershipError(
                        f"row {row} of group {group.index}: pages at {live.tolist()}, expected "
                        f"{first}..{until - 1} for length {int(self.row_len[row])}")
                for page in held[live].tolist():
                    if page in seen:
                        raise PageOwnershipError(f"page {page} is held by rows {seen[page]} and {row}")
                    if group.pool.owner(page) != row:
                        raise PageOwnershipError(f"page {page} in row {row}'s table is owned by "
                                                 f"{group.pool.owner(page)}")
                    seen[page] = row
            if len(seen) + group.pool.free_count != group.pool.num_pages:
                raise PageOwnershipError(f"group {group.index}: {len(seen)} held + "
                                         f"{group.pool.free_count} free != {group.pool.num_pages}")
