"""Plan and batch containers of the `prefix_attn` Python API.

Same public names, fields and behaviour as prefix_attn/data_class.py of the
flashserve/PAT tree (PackedBox :101-171, KernelInfo :173-254, Sequence/SeqGroup
:22-98, create_seq_group :257-264); the implementation is this project's own.
"""
from __future__ import annotations

import random
from dataclasses import dataclass, field
from typing import Any, Iterable, List, Optional, Sequence as Seq

import torch

__all__ = ["PackedBox", "KernelInfo", "Sequence", "SeqGroup", "create_seq_group",
           "make_tensor_merge_split"]


def _pad_to_matrix(rows: Seq[Seq[int]], device, fill: int = 0) -> torch.Tensor:
    """Ragged int rows -> int32 [len(rows), widest] on `device`, right-padded with `fill`.

    One host staging tensor and one copy per table (the reference issues a
    `torch.tensor(..., device=...)` per table as well, data_class.py:228-253)."""
    width = max(len(r) for r in rows)
    host = torch.full((len(rows), width), fill, dtype=torch.int32)
    for i, r in enumerate(rows):
        if len(r):
            host[i, :len(r)] = torch.as_tensor(r, dtype=torch.int32)
    return host.to(device)


def _vector(values: Seq[int], device) -> torch.Tensor:
    return torch.tensor(list(values), dtype=torch.int32, device=device)


def make_tensor_merge_split(x: List[list], device, dtype: torch.dtype = torch.int32, pad=0,
                            pin_memory: bool = True):
    """Ragged lists -> one padded device tensor, returned as per-row views (data_class.py:8-19)."""
    lens = [len(r) for r in x]
    width = max(lens)
    host = torch.full((len(x), width), pad, dtype=dtype, pin_memory=pin_memory and torch.cuda.is_available())
    for i, r in enumerate(x):
        if lens[i]:
            host[i, :lens[i]] = torch.as_tensor(r, dtype=dtype)
    merged = host.to(device)
    return (merged[i][:lens[i]] for i in range(len(x)))


class Sequence:
    """One request: its physical block ids and its length in tokens."""

    def __init__(self, block_size: int, seqlen: int = 0):
        self.block_ids: List[int] = []
        self.block_size = block_size
        self.seqlen = seqlen

    def append_blocks(self, blocks: List[int], tokens: Optional[int] = None) -> None:
        """Appends blocks; the length grows by `tokens`, or by whole blocks when omitted."""
        self.block_ids.extend(blocks)
        self.seqlen += len(blocks) * self.block_size if tokens is None else tokens


class SeqGroup:
    """A decode batch. `SeqGroup(bs, lo, hi, n)` draws n lengths uniformly in [lo, hi]."""

    def __init__(self, block_size: int, min_seqlen: int = 0, max_seqlen: int = 0, num_seqs: int = 0):
        self.sequences = [Sequence(block_size, random.randint(min_seqlen, max_seqlen))
                          for _ in range(num_seqs)]
        self.is_sorted = False

    def __len__(self) -> int:
        return len(self.sequences)

    def __str__(self) -> str:
        rows = [f"\n[{', '.join(str(b) for b in s.block_ids)}], seqlen={s.seqlen}" for s in self.sequences]
        return f"SeqGroup: {', '.join(rows)}"

    @property
    def seqlens(self) -> List[int]:
        return [s.seqlen for s in self.sequences]

    @property
    def max_seqlen(self) -> int:
        return max(s.seqlen for s in self.sequences)

    @property
    def max_num_blocks(self) -> int:
        return max(len(s.block_ids) for s in self.sequences)

    def set_common_prefix_blocks(self, prefix_blocks: List[int]) -> None:
        """Gives every sequence long enough to hold it the same leading blocks (length unchanged)."""
        need = len(prefix_blocks)
        for s in self.sequences:
            if s.seqlen >= s.block_size * need:
                s.append_blocks(prefix_blocks, 0)

    def add_random_prefix_blocks(self, random_blocks: List[List[int]]) -> None:
        for s in self.sequences:
            s.append_blocks(random_blocks[random.randint(0, len(random_blocks) - 1)])
        self.is_sorted = False

    def get_padded_block_ids(self, padding_value: int = -1) -> List[List[int]]:
        width = self.max_num_blocks
        return [s.block_ids + [padding_value] * (width - len(s.block_ids)) for s in self.sequences]

    def get_block_ids(self) -> List[List[int]]:
        return [list(s.block_ids) for s in self.sequences]

    def sort(self, reverse: bool = False) -> None:
        self.sequences.sort(key=lambda s: s.block_ids, reverse=reverse)
        self.is_sorted = True


@dataclass
class PackedBox:
    """Work items of one kernel launch: per item a query table, a block table, the
    number of sequences, its rank among the sequence's partial results and its KV
    length in tokens."""
    q_table: Any = field(default_factory=list)
    block_table: Any = field(default_factory=list)
    num_seqs_per_CTA: Any = field(default_factory=list)
    CTA_rank: Any = field(default_factory=list)
    kv_in_CTA: Any = field(default_factory=list)

    def __str__(self) -> str:
        return ("PackedBox("
                f"\n\tq_table={self.q_table},"
                f"\n\tblock_table={self.block_table},"
                f"\n\tnum_seqs_per_CTA={self.num_seqs_per_CTA},"
                f"\n\tCTA_rank={self.CTA_rank},"
                f"\n\tkv_in_CTA={self.kv_in_CTA},"
                "\n)")

    def __lt__(self, other: "PackedBox") -> bool:
        return self.kv_in_CTA > other.kv_in_CTA

    def sort_by_kv_desc(self) -> None:
        """Orders the items by KV length, longest first."""
        order = sorted(range(len(self.kv_in_CTA)), key=self.kv_in_CTA.__getitem__, reverse=True)
        for name in ("q_table", "block_table", "num_seqs_per_CTA", "CTA_rank", "kv_in_CTA"):
            col = getattr(self, name)
            setattr(self, name, [col[i] for i in order])

    def to_tensor(self, device) -> None:
        if not isinstance(self.num_seqs_per_CTA, torch.Tensor):
            self.num_seqs_per_CTA = _vector(self.num_seqs_per_CTA, device)
            self.CTA_rank = _vector(self.CTA_rank, device)
            self.kv_in_CTA = _vector(self.kv_in_CTA, device)
        if not isinstance(self.q_table, torch.Tensor):
            self.q_table = _pad_to_matrix(self.q_table, device)
        if not isinstance(self.block_table, torch.Tensor):
            self.block_table = _pad_to_matrix(self.block_table, device)


@dataclass
class KernelInfo:
    """The plan of one decode step: per tile bucket the packed items, plus what all
    buckets share. Lists until `to_tensor(device)` turns them into int32 tensors
    (ragged tables right-padded with 0)."""
    q_tables: Any = field(default_factory=list)
    block_tables: Any = field(default_factory=list)
    num_seqs_per_CTAs: Any = field(default_factory=list)
    CTA_ranks: Any = field(default_factory=list)
    kv_in_CTAs: Any = field(default_factory=list)
    MNWs: List[List[int]] = field(default_factory=list)

    num_split_per_seq: Any = field(default_factory=list)
    max_split_per_seq: int = 0
    max_seqs_in_CTA: int = 0
    max_blocks_in_CTA: int = 0
    reverse_index: Any = None
    sort_index: Any = None
    # Not in the reference: per bucket, for every (box, sequence) the box's ordinal among the
    # boxes of that sequence. Passing it to prefix_attn_with_kvcache(..., slot_tables=...) files
    # partial results by this ordinal instead of by CTA_rank.
    slot_tables: Any = field(default_factory=list)

    def sort_for_launch(self) -> None:
        """Not in the reference: orders every bucket's items longest first (stable), on the list
        form, i.e. before `to_tensor`. The kernels start work items in table order, and the table
        form of `prefix_attn_with_kvcache` launches the tables as they are given; longest first
        keeps long items from starting last. The plan stays the same plan: rows of one bucket are
        independent work items."""
        per_box = [self.q_tables, self.block_tables, self.num_seqs_per_CTAs, self.CTA_ranks, self.kv_in_CTAs]
        if self.slot_tables:
            per_box.append(self.slot_tables)
        if any(isinstance(t, torch.Tensor) for col in per_box for t in col):
            raise ValueError("sort_for_launch() works on the list form: call it before to_tensor()")
        for b, kv in enumerate(self.kv_in_CTAs):
            order = sorted(range(len(kv)), key=kv.__getitem__, reverse=True)
            for col in per_box:
                col[b] = [col[b][i] for i in order]

    def to_tensor(self, device) -> None:
        def vectors(cols: Iterable) -> list:
            return [c if isinstance(c, torch.Tensor) else _vector(c, device) for c in cols]

        def matrices(tables: Iterable) -> list:
            return [t if isinstance(t, torch.Tensor) else _pad_to_matrix(t, device) for t in tables]

        if not isinstance(self.num_split_per_seq, torch.Tensor):
            self.num_split_per_seq = _vector(self.num_split_per_seq, device)
        for name in ("reverse_index", "sort_index"):
            v = getattr(self, name)
            if v is not None and not isinstance(v, torch.Tensor):
                setattr(self, name, _vector(v, device))
        if not isinstance(self.num_seqs_per_CTAs, torch.Tensor):
            self.num_seqs_per_CTAs = vectors(self.num_seqs_per_CTAs)
        if not isinstance(self.CTA_ranks, torch.Tensor):
            self.CTA_ranks = vectors(self.CTA_ranks)
        if not isinstance(self.kv_in_CTAs, torch.Tensor):
            self.kv_in_CTAs = vectors(self.kv_in_CTAs)
        if not all(isinstance(t, torch.Tensor) for t in self.q_tables):
            self.q_tables = matrices(self.q_tables)
        if not all(isinstance(t, torch.Tensor) for t in self.block_tables):
            self.block_tables = matrices(self.block_tables)
        if self.slot_tables and not all(isinstance(t, torch.Tensor) for t in self.slot_tables):
            self.slot_tables = matrices(self.slot_tables)


def create_seq_group(block_tables: List[List[int]], seq_lens: List[int], block_size: int) -> SeqGroup:
    """A SeqGroup holding exactly the given block-table rows and lengths."""
    group = SeqGroup(block_size=block_size, num_seqs=len(block_tables))
    for seq, row, n in zip(group.sequences, block_tables, seq_lens):
        seq.block_ids = row
        seq.seqlen = n
    return group
