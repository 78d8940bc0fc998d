"""Work list of the matrix-core attention kernels (host side, numpy).

For one step and one (query heads per kv head) ratio: the rows of every item are cut into tiles
of 16.  A step with enough tiles to fill the chip (prompt portions) goes to the kernel that shares
keys and values through shared memory: a unit is a run of ``TILES_PER_BLOCK`` tiles of one item.
A step with few tiles (decoding) goes to the kernel with one wavefront per unit: every tile's keys
are cut into equal ranges (multiples of 32 keys) and a merge task per tile combines them.
"""
from __future__ import annotations

import ctypes
from dataclasses import dataclass

import numpy as np

UNIT_FIELDS = 8      # item, row_tile, key_begin, key_end, partial_slot (-1: none), q_start, q_len, ctx_len
TASK_FIELDS = 6      # item, row_tile, first_slot, num_splits, q_start, q_len
# a block's record: item, first_tile, key_begin, key_end, partial_slot of its first tile (-1: none), q_start,
# q_len, ctx_len, slots between two of its tiles (= key ranges per tile), 3 unused
BLOCK_UNIT_FIELDS = 12
# Measured on MI355X (48:8 heads of 128, pages of 64): one wavefront per SIMD is the sweet spot.
# 8 requests x 2048 keys take 20 us in 16 ranges of 128 keys against 24 us in 32 of 64; 64 requests
# x 2060 keys 102 us in 2 ranges (1024 wavefronts) against 146 us unsplit and 118 us in 4 ranges;
# 64 x 8192 keys 360 us (6.0 TB/s) against 550 us unsplit; 4 x 131072 keys 361 us (5.9 TB/s).
TARGET_WAVES = 1024    # wavefronts wanted in flight (256 CUs x 4 SIMDs)
MIN_SPLIT_KEYS = 128   # keys of a range; 64 when ranges of 128 would leave most of the chip idle (one request)
MAX_SPLITS = 256       # what the merge kernel's shared memory holds
TILES_PER_BLOCK = 8    # row tiles of one block of the shared-memory kernel
TILED_MAX_HEAD_DIM = 128
# Blocks, measured the same way (one request, causal flops): a portion of 512 tokens at context 16384 takes
# 322 us in 3 ranges (576 blocks: one round of the chip's 512 places and an eighth of another) and 249 us in 8
# ranges of 2048 keys (three rounds); at context 32768 594 against 443 us, a portion of 2048 at context 8192
# 419 against 393 us.  Ranges under about a thousand keys lose it again to their own start-up and to the merge
# (512 tokens at context 4096: 93 us in 3 or 4 ranges, 99 us in 8), and the rows of a whole prompt see more and
# more keys, so equal ranges leave most of its blocks with half-empty ones (2048 tokens: 75 us whole, 105 us in
# two ranges; 2048 at context 4096: 177 against 218 us): an item's keys are cut up only if the keys before its
# portion are at least three times the portion.
TARGET_BLOCKS = 1536   # blocks wanted in flight (three rounds of two per CU); fewer: their keys are split
MIN_BLOCK_KEYS = 2048
PREFIX_PER_PORTION = 3


@dataclass
class AttentionWork:
    """Both lists may be non-empty: a step's prompt portions go to the block kernel, its single
    tokens (whose few rows would leave a block mostly idle over a whole context) to the other."""
    units: np.ndarray        # int32 [num_units, UNIT_FIELDS]: (tile, key range) for one wavefront each
    tasks: np.ndarray        # int32 [num_tasks, TASK_FIELDS]: merges of split tiles
    num_slots: int           # partial results the units write
    block_units: np.ndarray  # int32 [num_block_units, UNIT_FIELDS]: runs of TILES_PER_BLOCK tiles for a block
    tiles_per_block: int = TILES_PER_BLOCK


@dataclass
class DeviceAttentionWork:
    """An ``AttentionWork`` whose lists lie in device memory (int32 tensors)."""
    units: object
    num_units: int
    tasks: object
    num_tasks: int
    num_slots: int
    block_units: object
    num_block_units: int
    tiles_per_block: int


_native = None      # the compiled builder (csrc/host_work.hip)


def _native_library():
    """The compiled builder; like every other library of the kernels it is built at first use and
    a failure to build or load it is an error (``KernelLibraryError``), not a quiet change of path."""
    global _native
    if _native is None:
        from . import library
        lib = library.load("host_work")
        i64p, i32p = ctypes.POINTER(ctypes.c_int64), ctypes.POINTER(ctypes.c_int32)
        lib.se_attention_work_plan.argtypes = [i64p, i64p, ctypes.c_int, ctypes.c_int, ctypes.c_int,
                                               ctypes.c_int, ctypes.c_int, i64p, i64p, i64p]
        lib.se_attention_work_fill.argtypes = [i64p, i64p, ctypes.c_int, ctypes.c_int, ctypes.c_int, i64p,
                                               i64p, i32p, i32p, i32p]
        _native = lib
    return _native


_BAD_LENGTHS = "attention work: every item needs at least one new token and no more new tokens than its context holds"


def build_attention_work(q_len, ctx_len, group: int, kv_heads: int, window: int = 0,
                         target_waves: int = TARGET_WAVES, head_dim: int = 0) -> AttentionWork:
    """The work lists of one step, from the compiled builder; ``build_attention_work_numpy`` states
    the rules and gives the same lists (the tests compare the two), about twenty times slower."""
    lib = _native_library()
    q = np.ascontiguousarray(q_len, dtype=np.int64)
    c = np.ascontiguousarray(ctx_len, dtype=np.int64)
    rules = np.asarray([target_waves, MIN_SPLIT_KEYS, MAX_SPLITS, TILES_PER_BLOCK, TILED_MAX_HEAD_DIM,
                        TARGET_BLOCKS, MIN_BLOCK_KEYS, PREFIX_PER_PORTION], dtype=np.int64)
    plan = np.empty((q.size, 6), dtype=np.int64)
    counts = np.empty(4, dtype=np.int64)
    i64p, i32p = ctypes.POINTER(ctypes.c_int64), ctypes.POINTER(ctypes.c_int32)
    as64 = lambda a: a.ctypes.data_as(i64p)
    status = lib.se_attention_work_plan(as64(q), as64(c), q.size, group, kv_heads, int(window or 0), int(head_dim or 0),
                                        as64(rules), as64(plan), as64(counts))
    if status == -2:
        raise ValueError(_BAD_LENGTHS)
    if status != 0:
        raise ValueError("attention work: bad arguments")
    units = np.empty((int(counts[0]), UNIT_FIELDS), dtype=np.int32)
    tasks = np.empty((int(counts[1]), TASK_FIELDS), dtype=np.int32)
    blocks = np.empty((int(counts[2]), BLOCK_UNIT_FIELDS), dtype=np.int32)
    lib.se_attention_work_fill(as64(q), as64(c), q.size, group, int(window or 0), as64(rules), as64(plan),
                               units.ctypes.data_as(i32p), tasks.ctypes.data_as(i32p), blocks.ctypes.data_as(i32p))
    return AttentionWork(units, tasks, int(counts[3]), blocks)


def build_attention_work_numpy(q_len, ctx_len, group: int, kv_heads: int, window: int = 0,
                               target_waves: int = TARGET_WAVES, head_dim: int = 0) -> AttentionWork:
    """``head_dim``: 0 keeps every item on the one-wavefront kernel (callers that do not know it).

    Items with at least half a block of tiles (prompt portions) go to the block kernel, the others
    keep one wavefront per tile.  In both classes the keys are cut into ranges when the class alone
    would not fill the chip; the number of ranges of an item follows its context, so that a long
    context beside short ones does not become the one long-running unit."""
    q_len = np.asarray(q_len, dtype=np.int64)
    ctx_len = np.asarray(ctx_len, dtype=np.int64)
    if ((q_len < 1) | (q_len > ctx_len)).any():
        raise ValueError(_BAD_LENGTHS)
    q_start = np.concatenate(([0], np.cumsum(q_len)[:-1]))      # items' tokens lie one after the other
    tiles = (q_len * group + 15) // 16
    reach = np.minimum(ctx_len, window + q_len) if window else ctx_len      # keys an item's tiles can read
    in_blocks = np.zeros(len(tiles), dtype=bool)
    if head_dim and head_dim % 32 == 0 and head_dim <= TILED_MAX_HEAD_DIM:
        in_blocks = tiles >= TILES_PER_BLOCK // 2

    def keys_per_unit(units_per_item, wanted: int, least: int) -> int:
        """Keys of a range so that all ranges together number about ``wanted``."""
        in_flight = int(units_per_item.sum()) * kv_heads
        if in_flight >= wanted:
            return 1 << 30
        if int((units_per_item * (reach // least)).sum()) * kv_heads < wanted // 2:
            least = max(32, least // 2)
        share = -(-int((units_per_item * reach).sum()) * kv_heads // wanted)
        return max(least, -(-share // 32) * 32)

    nblocks = np.where(in_blocks, -(-tiles // TILES_PER_BLOCK), 0)
    alone = np.where(in_blocks, 0, tiles)
    # blocks of an item whose portion is most of what it reads (a whole prompt) are never cut: they take
    # their places among the blocks wanted as they are
    cut = in_blocks & (reach - q_len >= PREFIX_PER_PORTION * q_len)
    whole = int(np.where(cut, 0, nblocks).sum()) * kv_heads
    block_keys = keys_per_unit(np.where(cut, nblocks, 0), TARGET_BLOCKS - whole, MIN_BLOCK_KEYS) if TARGET_BLOCKS > whole else 1 << 30
    keys = np.where(in_blocks, np.where(cut, block_keys, 1 << 30), keys_per_unit(alone, target_waves, MIN_SPLIT_KEYS))
    # equal ranges (multiples of 32 keys) over [first_key, ctx) of every item
    first_key = np.maximum(0, ctx_len - reach) // 32 * 32
    span = ctx_len - first_key
    splits = np.clip(-(-reach // keys), 1, MAX_SPLITS)
    chunk = -(-(-(-span // splits)) // 32) * 32
    splits = np.where(splits > 1, -(-span // np.maximum(chunk, 1)), 1)
    chunk = np.where(splits > 1, chunk, span)
    # partial slots: tile t, range s of an item -> base + t * splits + s, for items with several ranges
    slots_of = np.where(splits > 1, tiles * splits, 0)
    base = np.cumsum(slots_of) - slots_of
    num_slots = int(slots_of.sum())

    def expand(rows_per_item, fields: int, tiles_per_row: int):
        """One record per (row, range) of every item: rows are tiles or runs of tiles."""
        if not rows_per_item.any():
            return np.zeros((0, fields), dtype=np.int32), None
        count = rows_per_item * splits
        item = np.repeat(np.arange(len(tiles)), count)
        j = np.arange(int(count.sum())) - np.repeat(np.cumsum(count) - count, count)
        row, s = j // splits[item], j % splits[item]
        out = np.zeros((item.size, fields), dtype=np.int32)
        out[:, 0], out[:, 1] = item, row * tiles_per_row
        begin = first_key[item] + s * chunk[item]
        out[:, 2], out[:, 3] = begin, np.minimum(begin + chunk[item], ctx_len[item])
        out[:, 4] = np.where(splits[item] > 1, base[item] + row * tiles_per_row * splits[item] + s, -1)
        out[:, 5], out[:, 6], out[:, 7] = q_start[item], q_len[item], ctx_len[item]
        return out, item

    units, _ = expand(alone, UNIT_FIELDS, 1)
    blocks, block_item = expand(nblocks, BLOCK_UNIT_FIELDS, TILES_PER_BLOCK)
    if block_item is not None:
        blocks[:, 8] = splits[block_item]
    tasks = np.zeros((0, TASK_FIELDS), dtype=np.int32)
    if num_slots:
        merged = np.nonzero(splits > 1)[0]
        count = tiles[merged]
        item = np.repeat(merged, count)
        tile = np.arange(int(count.sum())) - np.repeat(np.cumsum(count) - count, count)
        tasks = np.zeros((item.size, TASK_FIELDS), dtype=np.int32)
        tasks[:, 0], tasks[:, 1], tasks[:, 2] = item, tile, base[item] + tile * splits[item]
        tasks[:, 3], tasks[:, 4], tasks[:, 5] = splits[item], q_start[item], q_len[item]

    if len(blocks):
        # longest first: a block's work grows with the position of its rows, and the blocks that are
        # started last decide when the kernel ends
        pos0 = ctx_len - q_len
        last_key = pos0[blocks[:, 0]] + ((blocks[:, 1].astype(np.int64) + TILES_PER_BLOCK) * 16 - 1) // group
        end = np.minimum(np.minimum(last_key + 1, ctx_len[blocks[:, 0]]), blocks[:, 3])
        begin = blocks[:, 2].astype(np.int64)
        if window:
            begin = np.maximum(begin, pos0[blocks[:, 0]] + (blocks[:, 1].astype(np.int64) * 16) // group - window + 1)
        blocks = blocks[np.argsort(-np.maximum(end - begin, 0), kind="stable")]
    return AttentionWork(units, tasks, num_slots, blocks)
