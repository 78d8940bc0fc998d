"""Work list of the matrix-core attention kernel (host side, numpy).

For one step and one (query heads per kv head) ratio: the rows of every item are cut into tiles
of 16; when the step has too few tiles to fill the chip, every tile's keys are cut into equal
ranges (multiples of 32 keys) and a merge task per tile combines them.
"""
from __future__ import annotations

from dataclasses import dataclass

import numpy as np

UNIT_FIELDS = 6      # item, row_tile, key_begin, key_end, partial_slot (-1: none), unused
TASK_FIELDS = 4      # item, row_tile, first_slot, num_splits
TARGET_WAVES = 2048  # wavefronts wanted in flight (256 CUs x 4 SIMDs x 2)
MIN_SPLIT_KEYS = 64
MAX_SPLITS = 256      # what the merge kernel's shared memory holds


@dataclass
class AttentionWork:
    units: np.ndarray        # int32 [num_units, UNIT_FIELDS]
    tasks: np.ndarray        # int32 [num_tasks, TASK_FIELDS]
    num_slots: int


def build_attention_work(q_len, ctx_len, group: int, kv_heads: int, window: int = 0,
                         target_waves: int = TARGET_WAVES) -> AttentionWork:
    q_len = np.asarray(q_len, dtype=np.int64)
    ctx_len = np.asarray(ctx_len, dtype=np.int64)
    tiles = (q_len * group + 15) // 16
    waves = int(tiles.sum()) * kv_heads
    want = 1 if waves >= target_waves else -(-target_waves // max(waves, 1))
    units, tasks, slot = [], [], 0
    for item, (n_tiles, ctx) in enumerate(zip(tiles.tolist(), ctx_len.tolist())):
        reach = min(ctx, window + int(q_len[item])) if window else ctx     # keys a tile can read
        splits = max(1, min(want, reach // MIN_SPLIT_KEYS, MAX_SPLITS))
        tile_ids = np.arange(n_tiles, dtype=np.int32)
        if splits == 1:
            block = np.zeros((n_tiles, UNIT_FIELDS), dtype=np.int32)
            block[:, 0], block[:, 1], block[:, 2], block[:, 3], block[:, 4] = item, tile_ids, 0, ctx, -1
            units.append(block)
            continue
        first_key = max(0, ctx - reach) // 32 * 32
        chunk = -(-(-(-(ctx - first_key) // splits)) // 32) * 32
        splits = -(-(ctx - first_key) // chunk)
        begins = first_key + np.arange(splits, dtype=np.int32) * chunk
        block = np.zeros((n_tiles, splits, UNIT_FIELDS), dtype=np.int32)
        block[:, :, 0] = item
        block[:, :, 1] = tile_ids[:, None]
        block[:, :, 2] = begins[None, :]
        block[:, :, 3] = np.minimum(begins + chunk, ctx)[None, :]
        block[:, :, 4] = slot + np.arange(n_tiles * splits, dtype=np.int32).reshape(n_tiles, splits)
        units.append(block.reshape(-1, UNIT_FIELDS))
        task = np.zeros((n_tiles, TASK_FIELDS), dtype=np.int32)
        task[:, 0], task[:, 1], task[:, 3] = item, tile_ids, splits
        task[:, 2] = slot + tile_ids * splits
        tasks.append(task)
        slot += n_tiles * splits
    return AttentionWork(np.concatenate(units) if units else np.zeros((0, UNIT_FIELDS), np.int32),
                         np.concatenate(tasks) if tasks else np.zeros((0, TASK_FIELDS), np.int32), slot)
