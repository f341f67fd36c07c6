"""CPU oracle for the segment metadata — TEST INFRASTRUCTURE, not product code.

Integer restatements (pure Python / numpy) of the three index layouts the reference derives
from the per-token slot vector.  Only tests/, __graft_entry__.smoke() and bench.py's
cpu_baseline leg may import this module.

Pinned by the reference's own vectors (tests/test_oracle_golden.py, tests/golden/meta.json):
  engine_layout        — tests/unit/test_lora_runtime.py:66-90 ([0,0,-1,0] -> [0,1,3],[0],[3],[0,3])
  kernel_meta_layout   — tests/unit/test_lora_layers.py:251-270 ([0,-1,1] -> [1,0,2],[1,1,1],
                         [0,1,2,3],[-1,0,1], 3 active) and tests/unit/test_triton_ops_cpu.py:36-142
                         (all -1 / empty -> reset state, captured-count rounding)
  graph_layout         — tests/unit/test_lora_cuda.py:412-417 (ids [-1,0], counts [0,1],
                         offsets [0,0,1]) and tests/unit/test_model_runner_extended.py:1024-1257
and cross-checked against each other and against a brute-force stable sort on random vectors.
No function here is "parity unpinned".
"""

from __future__ import annotations

import bisect

import numpy as np


def engine_layout(token_to_slot: list[int]):
    """(sorted_idx, active_slot_ids, num_tokens_per_slot, slot_start_offsets) with slot -1 left
    out, slots ascending and tokens ascending inside a slot — the engine-path builder
    (reference nanovllm_voxcpm/engine/lora_manager.py:77-91) and, on tensors, the torch builder
    (reference nanovllm_voxcpm/utils/context.py:77-116)."""
    by_slot: dict[int, list[int]] = {}
    for token, slot in enumerate(token_to_slot):
        if slot >= 0:
            by_slot.setdefault(slot, []).append(token)
    active = sorted(by_slot)
    counts = [len(by_slot[s]) for s in active]
    sorted_idx = [t for s in active for t in by_slot[s]]
    offsets = [0]
    for c in counts:
        offsets.append(offsets[-1] + c)
    return sorted_idx, active, counts, offsets


def kernel_meta_layout(token_to_slot: list[int], max_loras: int, captured_lora_counts: list[int] | None = None):
    """Buffers of LoRAKernelMeta.prepare_tensors
    (reference nanovllm_voxcpm/lora_ops/triton_ops/lora_kernel_metadata.py:39-68): a stable sort
    of *all* tokens by slot id (so slot -1 comes first), unique ids with counts, running totals
    written at [1 : 1 + n]; unused entries keep the reset values (id -1, count 0, start 0).

    Returns dict(sorted_idx, active_lora_ids, num_tokens_per_lora, lora_token_start_loc,
    no_lora_flag, num_active_loras).  When every token is -1 (or there are none) the reference
    returns right after the reset, so ``sorted_idx`` is None (buffer left as it was)."""
    ids = [-1] * (max_loras + 1)
    counts = [0] * (max_loras + 1)
    starts = [0] * (max_loras + 2)
    if all(s == -1 for s in token_to_slot):
        return dict(
            sorted_idx=None, active_lora_ids=ids, num_tokens_per_lora=counts, lora_token_start_loc=starts,
            no_lora_flag=True, num_active_loras=0,
        )
    arr = np.asarray(token_to_slot, dtype=np.int64)
    order = np.argsort(arr, kind="stable")
    uniq, cnt = np.unique(arr, return_counts=True)
    n = len(uniq)
    ids[:n] = [int(v) for v in uniq]
    counts[:n] = [int(v) for v in cnt]
    starts[1 : 1 + n] = [int(v) for v in np.cumsum(cnt)]
    num_active = n
    captured = sorted(captured_lora_counts) if captured_lora_counts else []
    if captured and num_active > 0:
        i = bisect.bisect_left(captured, num_active)
        if i < len(captured):
            num_active = captured[i]
    return dict(
        sorted_idx=[int(v) for v in order], active_lora_ids=ids, num_tokens_per_lora=counts,
        lora_token_start_loc=starts, no_lora_flag=False, num_active_loras=num_active,
    )


def graph_layout(token_to_slot: list[int] | None, no_lora_flag: bool, max_rows: int, max_lora_buckets: int,
                 previous_sorted: list[int] | None = None):
    """State of the fixed-address graph buffers after the runner refreshed them for a batch
    (reference nanovllm_voxcpm/engine/model_runner.py:719-797): buckets are dense by slot id with
    bucket 0 standing for slot -1 (its count stays 0), offsets are [0, running totals], the slot
    vector is padded with -1 and only the first (number of LoRA tokens) entries of the sorted
    index buffer are rewritten."""
    sorted_buf = list(previous_sorted) if previous_sorted is not None else list(range(max_rows))
    ids = list(range(-1, max_lora_buckets - 1))
    counts = [0] * max_lora_buckets
    offsets = [0] * (max_lora_buckets + 1)
    if no_lora_flag or token_to_slot is None:
        return dict(token_to_slot=[-1] * max_rows, token_indices_sorted_by_slot=sorted_buf, active_slot_ids=ids,
                    num_tokens_per_slot=counts, slot_start_offsets=offsets)
    padded = list(token_to_slot) + [-1] * (max_rows - len(token_to_slot))
    sorted_idx, active, per_slot, _ = engine_layout(list(token_to_slot))
    sorted_buf[: len(sorted_idx)] = sorted_idx
    for slot, c in zip(active, per_slot):
        counts[slot + 1] = c
    run = 0
    for b in range(max_lora_buckets):
        run += counts[b]
        offsets[b + 1] = run
    return dict(token_to_slot=padded, token_indices_sorted_by_slot=sorted_buf, active_slot_ids=ids,
                num_tokens_per_slot=counts, slot_start_offsets=offsets)


def big_tile_capacity(num_tokens: int, max_slots: int, big: int = 64) -> int:
    """Places in the plan's list of big tiles: at most ``most`` = num_tokens // big + min(max_slots,
    num_tokens) tiles exist; an eighth of them, the smallest ``root`` with 8 root^2 >= most, and two
    more fit every one of the eight blocks; rounded up to a multiple of 32."""
    most = num_tokens // big + min(max_slots, num_tokens)
    root = 1
    while 8 * root * root < most:
        root += 1
    return (most + 8 * (root + 2) + 31) & ~31


def big_tile_places(long_big: list[tuple[int, int, int]], num_tokens: int, max_slots: int, big: int = 64) -> list[int]:
    """Places of the big tiles (``long_big`` of plan_tiles, in slot order) in the plan's list of big
    tiles.  The list is cut into eight equal blocks, one per XCD.  The tiles are cut into runs of
    consecutive tiles, and run i goes to block i % 8, behind the runs the block already holds.
    Run length: the tiles split into 8 k runs, k the smallest for which a run is no longer than
    the average number of tiles (rounded down) of a slot that has any."""
    n = len(long_big)
    if n == 0:
        return []
    blk = big_tile_capacity(num_tokens, max_slots, big) // 8
    avg = n // len({slot for slot, _, _ in long_big})
    k = -(-n // (8 * avg))
    run = -(-n // (8 * k))
    places = []
    for t in range(n):
        i = t // run
        places.append((i % 8) * blk + (i // 8) * run + t % run)
    return places


def plan_tiles(token_to_slot: list[int], max_slots: int, threshold: int = 16, small: int = 16, big: int = 64):
    """Work lists the apply kernels walk, derived from the engine layout: for every slot in
    ascending order its segment is cut into tiles (slot, first position in sorted_idx, count).
    Returns (short_small, long_small, long_big): small tiles of segments shorter than
    ``threshold``, small tiles of the other segments, and big tiles of the other segments.
    Slot ids >= max_slots count as -1.  (No reference counterpart: the reference launches a
    grid over (slot bucket x row tile) and lets empty programs exit.)"""
    cleaned = [s if 0 <= s < max_slots else -1 for s in token_to_slot]
    _, active, counts, offsets = engine_layout(cleaned)
    short_small, long_small, long_big = [], [], []
    for slot, c, off in zip(active, counts, offsets):
        target = short_small if c < threshold else long_small
        for j in range(0, c, small):
            target.append((slot, off + j, min(small, c - j)))
        if c >= threshold:
            for j in range(0, c, big):
                long_big.append((slot, off + j, min(big, c - j)))
    return short_small, long_small, long_big


def plan_tiles_by_slot(token_to_slot: list[int], max_slots: int, small: int = 16):
    """The same small tiles listed by slot: ``first[s]`` = (count, first position in sorted_idx) of
    the first tile of slot id ``s`` for every s in [0, max_slots) (count 0 and the slot's position
    in the running totals for a slot without tokens), and ``further`` = (slot, first position,
    count) of every tile behind a slot's first one, slots ascending.  Slot ids >= max_slots count
    as -1.  (No reference counterpart, like plan_tiles.)"""
    cleaned = [s if 0 <= s < max_slots else -1 for s in token_to_slot]
    _, active, counts, offsets = engine_layout(cleaned)
    per_slot = dict(zip(active, zip(counts, offsets)))
    first, further, run = [], [], 0
    for s in range(max_slots):
        c, off = per_slot.get(s, (0, run))
        first.append((min(c, small), off))
        for j in range(small, c, small):
            further.append((s, off + j, min(small, c - j)))
        run = off + c
    return first, further
