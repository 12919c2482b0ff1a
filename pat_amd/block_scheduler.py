"""Legacy (v0) flat schedulers of the `prefix_attn` API: `pack_prefix_blocks`,
`pack_without_prefix`, `schedule`, `schedule_naive`
(prefix_attn/block_scheduler.py in the flashserve/PAT tree).

They predate the prefix-tree scheduler and are not on the decode path: neither the
reference's test, its kernel benchmark nor its vLLM backend calls them. The names are
kept importable; `pack_without_prefix` is implemented because the prefix-oblivious
baseline plan is exactly its output. The other three raise until they are built.
"""
from __future__ import annotations

from types import SimpleNamespace
from typing import List

from .data_class import SeqGroup

__all__ = ["pack_prefix_blocks", "pack_without_prefix", "schedule", "schedule_naive"]


def pack_without_prefix(seq_group: SeqGroup, block_size: int):
    """One work item per sequence over its whole block list, no sharing
    (block_scheduler.py:155-202). Returns a namespace with the documented fields."""
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


def _not_built(name: str):
    raise NotImplementedError(
        f"prefix_attn.{name} is the superseded v0 scheduler; use PrefixTree.pack_schedule")


def pack_prefix_blocks(seq_group: SeqGroup, block_size: int, k: int = 64):
    _not_built("pack_prefix_blocks")


def schedule(*args, **kwargs):
    _not_built("schedule")


def schedule_naive(*args, **kwargs):
    _not_built("schedule_naive")
