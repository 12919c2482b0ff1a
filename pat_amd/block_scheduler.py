"""Legacy (v0) flat schedulers of the `prefix_attn` API: `pack_prefix_blocks`,
`pack_without_prefix`, `schedule`, `schedule_naive`
(prefix_attn/block_scheduler.py in the flashserve/PAT tree).

They predate the prefix-tree scheduler and are not on the decode path: neither the
reference's test, its kernel benchmark nor its vLLM backend calls them. They pack
level by level instead of building a tree: in every round the unfinished sequences are
grouped by their current block id into runs of neighbouring sequences; a lone sequence
takes all of its remaining blocks as one work item, a run is cut into items of at most
k sequences over the longest block run they all share.

`schedule` (sort-free entry: it lexsorts the block table itself and returns the
permutation) and `schedule_naive` return a `KernelInfo`; the two `pack_*` functions
return a flat record with the fields their docstrings in the reference list.
"""
from __future__ import annotations

from types import SimpleNamespace
from typing import Dict, List, Optional, Sequence, Tuple

import numpy as np
import torch

from .data_class import KernelInfo, SeqGroup
from .utils import make_ndarray_with_pad

__all__ = ["pack_prefix_blocks", "pack_without_prefix", "schedule", "schedule_naive"]


def _flat_pack(seq_lens: Sequence[int], rows: Sequence[Sequence[int]], block_size: int, k: int):
    """Round-based packing shared by `pack_prefix_blocks` and `schedule`
    (block_scheduler.py:64-138 / 404-480). Returns (items, split counts) where an item is
    (sequence ids, blocks, kv tokens, rank)."""
    n = len(rows)
    at = [0] * n                      # next unpacked block of every sequence
    splits = [0] * n
    items: List[Tuple[List[int], List[int], int, int]] = []

    while any(at[i] < len(rows[i]) for i in range(n)):
        # runs of neighbouring unfinished sequences per current block id, in first-seen order
        runs_of: Dict[int, List[List[int]]] = {}
        for i in range(n):
            if at[i] >= len(rows[i]):
                continue
            runs = runs_of.setdefault(rows[i][at[i]], [[]])
            if not runs[-1] or runs[-1][-1] + 1 == i:
                runs[-1].append(i)
            else:
                runs.append([i])
        for runs in runs_of.values():
            for run in runs:
                if len(run) == 1:
                    s = run[0]
                    rest = list(rows[s][at[s]:])
                    items.append(([s], rest, seq_lens[s] - at[s] * block_size, splits[s]))
                    at[s] = len(rows[s])
                    splits[s] += 1
                    continue
                for lo in range(0, len(run), k):
                    group = run[lo:lo + k]
                    shared: List[int] = []
                    ran_out = False
                    while True:
                        if any(at[p] >= len(rows[p]) for p in group):
                            ran_out = True
                            break
                        cur = rows[group[0]][at[group[0]]]
                        if any(rows[p][at[p]] != cur for p in group):
                            break
                        shared.append(cur)
                        for p in group:
                            at[p] += 1
                    if not shared:
                        continue
                    head = group[0]
                    if ran_out:   # the first sequence of the group ends inside the shared run
                        kv = block_size * (len(shared) - 1) + seq_lens[head] - (len(rows[head]) - 1) * block_size
                    else:
                        kv = block_size * len(shared)
                    items.append((list(group), shared, kv, splits[head]))
                    for p in group:
                        splits[p] += 1
    return items, splits


def pack_prefix_blocks(seq_group: SeqGroup, block_size: int, k: int = 64):
    """Packs a SORTED SeqGroup level by level. Returns a flat record whose `q_table` holds the
    first sequence of every item (items cover `num_seqs_per_CTA` neighbouring sequences)."""
    assert seq_group.is_sorted, "SeqGroup must be sorted"
    assert k <= 64, "max number of sequences in a CTA should be less than 64"
    rows = [s.block_ids for s in seq_group.sequences]
    lens = [s.seqlen for s in seq_group.sequences]
    items, splits = _flat_pack(lens, rows, block_size, k)
    n = len(rows)
    return SimpleNamespace(
        q_table=[seqs[0] for seqs, _, _, _ in items],
        block_table=[blocks for _, blocks, _, _ in items],
        num_seqs_per_CTA=[len(seqs) for seqs, _, _, _ in items],
        num_split_per_seq=list(splits),
        CTA_rank=[rank for _, _, _, rank in items],
        kv_in_CTA=[kv for _, _, kv, _ in items],
        max_split_per_seq=max(splits),
        max_seqs_in_CTA=max([len(seqs) for seqs, _, _, _ in items], default=1),
        max_blocks_in_CTA=max([len(blocks) for _, blocks, _, _ in items], default=0),
        sort_index=np.arange(n),
        reverse_index=np.arange(n),
    )


def pack_without_prefix(seq_group: SeqGroup, block_size: int):
    """One work item per sequence over its whole block list, no sharing
    (block_scheduler.py:155-202). Returns a flat record with the documented fields."""
    n = len(seq_group)
    return SimpleNamespace(
        q_table=list(range(n)),
        block_table=seq_group.get_block_ids(),
        num_seqs_per_CTA=[1] * n,
        num_split_per_seq=[1] * n,
        CTA_rank=[0] * n,
        kv_in_CTA=[s.seqlen for s in seq_group.sequences],
        max_split_per_seq=1,
        max_seqs_in_CTA=1,
        max_blocks_in_CTA=seq_group.max_num_blocks,
    )


def schedule(seq_lens: List[int], block_table: List[List[int]], block_size: int, k: int,
             qkv_tile_types: Optional[List[List[int]]], h_q_kv_ratio: int = 1) -> KernelInfo:
    """Sort-free flat scheduler (block_scheduler.py:348-505): lexsorts the zero-padded block table,
    packs in sorted order and files every item under the first tile type whose tile_q holds its
    rows. Sequence ids in the plan are positions in the SORTED batch; `sort_index` /
    `reverse_index` map between the two orders."""
    tiles = qkv_tile_types if qkv_tile_types is not None else [[64, 128, 4]]
    padded = make_ndarray_with_pad(block_table, 0, np.int32)
    order = np.lexsort(padded[:, ::-1].T)
    lens = [seq_lens[i] for i in order]
    rows = [padded[i][:(seq_lens[i] + block_size - 1) // block_size].tolist() for i in order]
    items, splits = _flat_pack(lens, rows, block_size, k)

    info = KernelInfo(max_split_per_seq=max(splits),
                      max_seqs_in_CTA=max([len(s) for s, _, _, _ in items if len(s) > 1], default=1),
                      max_blocks_in_CTA=max([len(b) for _, b, _, _ in items], default=0),
                      num_split_per_seq=list(splits),
                      reverse_index=np.argsort(order).tolist(),
                      sort_index=order.tolist())
    per_tile: List[List[Tuple[List[int], List[int], int, int]]] = [[] for _ in tiles]
    for item in items:
        for slot, (tile_q, _, _) in enumerate(tiles):
            if len(item[0]) * h_q_kv_ratio <= tile_q:
                per_tile[slot].append(item)
                break
    for tile, members in zip(tiles, per_tile):
        if not members:
            continue
        info.q_tables.append([s for s, _, _, _ in members])
        info.block_tables.append([b for _, b, _, _ in members])
        info.num_seqs_per_CTAs.append([len(s) for s, _, _, _ in members])
        info.CTA_ranks.append([r for _, _, _, r in members])
        info.kv_in_CTAs.append([kv for _, _, kv, _ in members])
        info.MNWs.append(tile)
    return info


def schedule_naive(seq_lens: List[int], block_table: List[List[int]], device: torch.device) -> KernelInfo:
    """One work item per sequence in the given order, already as int32 tensors on `device`
    (block_scheduler.py:508-553)."""
    assert isinstance(seq_lens, list)
    assert isinstance(block_table, list)
    padded = make_ndarray_with_pad(block_table, 0, np.int32)
    n = len(seq_lens)
    ident = torch.arange(n, dtype=torch.int64, device=device)
    ones = torch.ones(n, dtype=torch.int32, device=device)
    return KernelInfo(
        q_tables=[torch.arange(n, dtype=torch.int32, device=device)],
        block_tables=[torch.from_numpy(padded).to(device)],
        num_seqs_per_CTAs=[ones.clone()],
        num_split_per_seq=ones.clone(),
        CTA_ranks=[torch.zeros(n, dtype=torch.int32, device=device)],
        kv_in_CTAs=[torch.tensor(seq_lens, dtype=torch.int32, device=device)],
        MNWs=[[64, 128, 4]],
        max_split_per_seq=1,
        max_seqs_in_CTA=1,
        max_blocks_in_CTA=max(len(row) for row in padded),
        reverse_index=ident.clone(),
        sort_index=ident,
    )
