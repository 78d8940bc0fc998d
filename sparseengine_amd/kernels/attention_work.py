"""Work list of the matrix-core attention kernels (host side, numpy).

For one step and one (query heads per kv head) ratio: the rows of every item are cut into tiles
of 16.  A step with enough tiles to fill the chip (prompt portions) goes to the kernel that shares
keys and values through shared memory: a unit is a run of ``TILES_PER_BLOCK`` tiles of one item.
A step with few tiles (decoding) goes to the kernel with one wavefront per unit: every tile's keys
are cut into equal ranges (multiples of 32 keys) and a merge task per tile combines them.
"""
from __future__ import annotations

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
TARGET_BLOCKS = 512    # blocks wanted in flight (two per CU); fewer: their keys are split
MIN_BLOCK_KEYS = 512


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


def _record(rows: int, fields: int, item, tile, begin, end, slot, q_start, q_len, ctx) -> np.ndarray:
    block = np.zeros((rows, fields), dtype=np.int32)
    for column, value in enumerate((item, tile, begin, end, slot, q_start, q_len, ctx)):
        block[:, column] = value
    return block


def _ranges(first_key: int, ctx: int, splits: int):
    """``splits`` equal key ranges (multiples of 32 keys) over [first_key, ctx): begins, ends."""
    chunk = -(-(-(-(ctx - first_key) // splits)) // 32) * 32
    splits = -(-(ctx - first_key) // chunk)
    begins = first_key + np.arange(splits, dtype=np.int32) * chunk
    return begins, np.minimum(begins + chunk, ctx)


def build_attention_work(q_len, ctx_len, group: int, kv_heads: int, window: int = 0,
                         target_waves: int = TARGET_WAVES, head_dim: int = 0) -> AttentionWork:
    """``head_dim``: 0 keeps every item on the one-wavefront kernel (callers that do not know it).

    Items with at least half a block of tiles (prompt portions) go to the block kernel, the others
    keep one wavefront per tile.  In both classes the keys are cut into ranges when the class alone
    would not fill the chip; the number of ranges of an item follows its context, so that a long
    context beside short ones does not become the one long-running unit."""
    q_len = np.asarray(q_len, dtype=np.int64)
    ctx_len = np.asarray(ctx_len, dtype=np.int64)
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

    units, tasks, block_units, slot = [], [], [], 0
    nblocks = np.where(in_blocks, -(-tiles // TILES_PER_BLOCK), 0)
    alone = np.where(in_blocks, 0, tiles)
    block_keys = keys_per_unit(nblocks, TARGET_BLOCKS, MIN_BLOCK_KEYS)
    wave_keys = keys_per_unit(alone, target_waves, MIN_SPLIT_KEYS)
    for item in range(len(tiles)):
        n_tiles, ctx, ql, qs = int(tiles[item]), int(ctx_len[item]), int(q_len[item]), int(q_start[item])
        keys = block_keys if in_blocks[item] else wave_keys
        splits = max(1, min(-(-int(reach[item]) // keys), MAX_SPLITS))
        first_key = max(0, ctx - int(reach[item])) // 32 * 32
        begins, ends = _ranges(first_key, ctx, splits) if splits > 1 else (np.zeros(1, np.int32), np.full(1, ctx))
        splits = len(begins)
        tile_ids = np.arange(n_tiles, dtype=np.int32)
        if in_blocks[item]:
            first = np.arange(0, n_tiles, TILES_PER_BLOCK, dtype=np.int32)
            block = np.zeros((first.size, splits, BLOCK_UNIT_FIELDS), dtype=np.int32)
            block[:, :, 0], block[:, :, 1] = item, first[:, None]
            block[:, :, 2], block[:, :, 3] = begins[None, :], ends[None, :]
            block[:, :, 4] = -1 if splits == 1 else slot + first[:, None] * splits + np.arange(splits)[None, :]
            block[:, :, 5], block[:, :, 6], block[:, :, 7], block[:, :, 8] = qs, ql, ctx, splits
            block_units.append(block.reshape(-1, BLOCK_UNIT_FIELDS))
        elif splits == 1:
            units.append(_record(n_tiles, UNIT_FIELDS, item, tile_ids, 0, ctx, -1, qs, ql, ctx))
        else:
            block = np.zeros((n_tiles, splits, UNIT_FIELDS), dtype=np.int32)
            block[:, :, 0], block[:, :, 1] = item, tile_ids[:, None]
            block[:, :, 2], block[:, :, 3] = begins[None, :], ends[None, :]
            block[:, :, 4] = slot + tile_ids[:, None] * splits + np.arange(splits)[None, :]
            block[:, :, 5], block[:, :, 6], block[:, :, 7] = qs, ql, ctx
            units.append(block.reshape(-1, UNIT_FIELDS))
        if splits > 1:
            task = np.zeros((n_tiles, TASK_FIELDS), dtype=np.int32)
            task[:, 0], task[:, 1], task[:, 3] = item, tile_ids, splits
            task[:, 2] = slot + tile_ids * splits
            task[:, 4], task[:, 5] = qs, ql
            tasks.append(task)
            slot += n_tiles * splits

    blocks = np.concatenate(block_units) if block_units else np.zeros((0, BLOCK_UNIT_FIELDS), np.int32)
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
    return AttentionWork(np.concatenate(units) if units else np.zeros((0, UNIT_FIELDS), np.int32),
                         np.concatenate(tasks) if tasks else np.zeros((0, TASK_FIELDS), np.int32), slot, blocks)
