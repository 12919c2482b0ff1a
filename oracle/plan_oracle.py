"""CPU restatement of the reference's Python prefix-tree scheduler.

TEST INFRASTRUCTURE ONLY. This module is the checker for plan parity: only tests,
the smoke check and the benchmark's CPU-baseline leg may import it. The product
(`pat_amd`) never does; it plans with the C++ scheduler in libpat_amd.

It restates, in plain Python over small dataclasses, the algorithm of
`prefix_attn/prefix_tree.py` in the flashserve/PAT tree (cited per function below),
including the incidental behaviours a bit-exact plan depends on: insertion order of
a node's children, the binary-search common-prefix probe, the float `ceil` of the
long-box cut, and the pop/append reordering of the balancer.

How it is pinned (tests/test_oracle_plan.py):
  * hand-traced known answers for the reference's own manual fixture
    (test/test.py:233-239) and for the 8-request shared-prefix batch,
  * closed forms for regular two/three-level trees and no-sharing batches,
  * structural invariants on random forests (every sequence's boxes tile its
    block-table row exactly once, ranks are 0..n-1, tile labels match),
  * golden plans written by the reference scheduler itself
    (tests/golden/plans_*.json, produced by tests/golden/make_plan_fixtures.py).
`pack_schedule(use_compute_model=True)` and `naive_schedule` are pinned by the
golden plans only.
"""
from __future__ import annotations

import math
from dataclasses import dataclass, field
from typing import Dict, List, Optional, Sequence, Tuple

DEFAULT_BUCKETS: List[List[int]] = [
    [64, 128, 4], [64, 64, 4], [64, 32, 4],
    [32, 128, 2], [32, 64, 2], [32, 32, 2], [32, 16, 2],
    [16, 128, 1], [16, 64, 1], [16, 32, 1], [16, 16, 1],
]


@dataclass
class Node:
    parent: int
    s: int                      # sequences through the node
    tokens: int                 # KV tokens held by the node
    seqs: List[int]
    blocks: List[int]
    kids: Dict[int, int] = field(default_factory=dict)   # first block id -> node id (ordered)


@dataclass
class Box:
    q_table: List[int]
    block_table: List[int]
    num_seqs: int
    kv: int
    rank: int


@dataclass
class PlanResult:
    MNWs: List[List[int]]
    q_tables: List[List[List[int]]]
    block_tables: List[List[List[int]]]
    num_seqs_per_CTAs: List[List[int]]
    CTA_ranks: List[List[int]]
    kv_in_CTAs: List[List[int]]
    num_split_per_seq: List[int]
    max_split_per_seq: int
    max_seqs_in_CTA: int
    max_blocks_in_CTA: int

    def as_dict(self) -> dict:
        return {k: getattr(self, k) for k in self.__dataclass_fields__}


def tile_label(rows: int, kv: int) -> Tuple[int, int, int]:
    """prefix_tree.py:462-482."""
    m, w = (64, 4) if rows > 32 else (32, 2) if rows > 16 else (16, 1)
    n = 16 if kv < 32 else 32 if kv < 64 else 64 if kv <= 128 else 128
    if m == 64:
        n = max(n, 32)
    return (m, n, w)


def _probe_common(a: Sequence[int], b: Sequence[int]) -> int:
    """prefix_tree.py:81-89 — index of the last common block by bisection."""
    lo, hi = -1, min(len(a), len(b))
    while hi - lo > 1:
        mid = (lo + hi) >> 1
        if a[mid] == b[mid]:
            lo = mid
        else:
            hi = mid
    return lo


# compute-model costs, prefix_tree.py:16-45
def _pad(tile, n):
    return tile - ((n - 1) % tile + 1)


def _waste(nq, nk, hratio):
    return _pad(64 if nq * hratio >= 64 else 16, nq) * nk * hratio


class PlanOracle:
    def __init__(self, block_size: int):
        self.bs = block_size
        self.nodes: List[Node] = [Node(-1, 1, 0, [], [])]
        self.split: List[int] = []

    # ---- tree -----------------------------------------------------------------
    def _new(self, parent, s, tokens, seqs, blocks) -> int:
        self.nodes.append(Node(parent, s, tokens, seqs, blocks))
        return len(self.nodes) - 1

    def insert(self, sid: int, seq_len: int, blocks: List[int]) -> None:
        """prefix_tree.py:95-144."""
        at, left = 0, len(blocks)
        while left:
            here = self.nodes[at]
            if blocks[0] not in here.kids:
                here.kids[blocks[0]] = self._new(at, 1, seq_len, [sid], blocks)
                return
            cid = here.kids[blocks[0]]
            child = self.nodes[cid]
            common = _probe_common(blocks, child.blocks) + 1
            if common == len(child.blocks):
                child.s += 1
                child.seqs.append(sid)
                at, left = cid, left - common
                seq_len -= common * self.bs
                blocks = blocks[common:]
                continue
            mid = self._new(at, child.s + 1, common * self.bs, list(child.seqs), child.blocks[:common])
            self.nodes[mid].kids[child.blocks[common]] = cid
            here.kids[child.blocks[0]] = mid
            child.parent = mid
            child.blocks = child.blocks[common:]
            child.tokens -= common * self.bs
            self.nodes[mid].seqs.append(sid)
            if common != left:
                leaf = self._new(mid, 1, min(left * self.bs, seq_len) - common * self.bs, [sid],
                                 blocks[common:])
                self.nodes[mid].kids[blocks[common]] = leaf
            return

    def build_radix_tree(self, seq_lens: List[int], block_table: List[List[int]]) -> None:
        """prefix_tree.py:146-149."""
        for i, row in enumerate(block_table):
            self.insert(i, seq_lens[i], list(row))
        self.split = [0] * len(block_table)

    # ---- packing --------------------------------------------------------------
    def _boxes_for(self, seqs: List[int], count: int, mm: int, inherited: List[int], node: Node,
                   out: List[Box]) -> None:
        """prefix_tree.py:277-286 / 307-316."""
        for s in range(0, count, mm):
            q = seqs[s:min(s + mm, count)]
            box = Box(q, inherited + node.blocks, min(mm, count - s),
                      self.bs * len(inherited) + node.tokens, self.split[q[0]])
            for x in q:
                self.split[x] += 1
            out.append(box)

    def _walk(self, nid: int, mm: int, hratio: int, model: bool, inherited: List[int],
              out: List[Box]) -> None:
        """prefix_tree.py:269-323 (model=False) and :325-381 (model=True)."""
        node = self.nodes[nid]
        if not node.kids:
            self._boxes_for(node.seqs, node.s, mm, inherited, node, out)
            return
        left = node.s
        kv_len = self.bs * len(inherited) + node.tokens
        stay, sink = [], []
        for cid in node.kids.values():
            c = self.nodes[cid]
            if model:
                cost_k = _waste(left, c.tokens, hratio) + _waste(c.s, kv_len, hratio) + 0.1 * c.s * hratio
                cost_q = _waste(left - c.s, kv_len, hratio) + _waste(c.s, kv_len + c.tokens, hratio)
                merge = cost_k > cost_q
            else:
                merge = left == c.s or (
                    math.ceil(left / mm) - math.ceil((left - c.s) / mm) - math.ceil(c.s / mm)
                ) * kv_len + 4 * c.s >= 0
            if merge:
                left -= c.s
                sink.append(cid)
            else:
                stay.append(cid)
        if left != 0:
            pooled: List[int] = []
            for cid in stay:
                pooled.extend(self.nodes[cid].seqs)
            self._boxes_for(pooled, left, mm, inherited, node, out)
        for cid in stay:
            self._walk(cid, mm, hratio, model, [], out)
        for cid in sink:
            self._walk(cid, mm, hratio, model, inherited + node.blocks, out)

    def _balance(self, boxes: List[Box], kv_heads: int) -> List[Box]:
        """prefix_tree.py:383-460."""
        if not boxes:
            return []
        long_blocks = sum(len(b.block_table) for b in boxes if b.kv > 256)
        long_boxes = sum(1 for b in boxes if b.kv > 256)
        if long_boxes:
            avg = long_blocks / long_boxes
            cut: List[Box] = []
            for b in boxes:
                n = len(b.block_table)
                if n > avg * 5:
                    pieces = math.ceil(n / avg)
                    size = math.ceil(n / pieces)
                    for i in range(pieces):
                        rank = b.rank if i == 0 else self.split[b.q_table[0]]
                        cut.append(Box(b.q_table, b.block_table[i * size:min((i + 1) * size, n)],
                                       b.num_seqs, min(b.kv - i * size * self.bs, size * self.bs), rank))
                        if i:
                            for x in b.q_table:
                                self.split[x] += 1
                else:
                    cut.append(b)
        else:
            cut = boxes
        want = 54 if kv_heads <= 4 else 27 if kv_heads <= 8 else 13 if kv_heads <= 16 \
            else 6 if kv_heads <= 32 else 4
        if len(cut) >= want:
            return cut
        while len(cut) < want and max(self.split) < 32:
            idx = max(range(len(cut)), key=lambda i: len(cut[i].block_table))
            b = cut.pop(idx)
            n = len(b.block_table)
            if n <= 8:
                cut.append(b)
                break
            half = math.ceil(n / 2)
            first = Box(b.q_table, b.block_table[:half], b.num_seqs, min(b.kv, half * self.bs), b.rank)
            second = Box(b.q_table, b.block_table[half:], b.num_seqs,
                         min(b.kv - half * self.bs, (n - half) * self.bs), self.split[b.q_table[0]])
            for x in b.q_table:
                self.split[x] += 1
            cut += [first, second]
        return cut

    def _emit(self, boxes: List[Box], buckets: List[List[int]], hratio: int, single: bool) -> PlanResult:
        """prefix_tree.py:574-614."""
        groups: Dict[Tuple[int, ...], List[Box]] = {tuple(b): [] for b in buckets}
        for b in boxes:
            key = tuple(buckets[0]) if single else tile_label(len(b.q_table) * hratio, b.kv)
            groups[key].append(b)
        res = PlanResult([], [], [], [], [], [], self.split, 0, 0, 0)
        for mnw in buckets:
            g = groups.get(tuple(mnw), [])
            if not g:
                continue
            res.MNWs.append(list(mnw))
            res.q_tables.append([b.q_table for b in g])
            res.block_tables.append([b.block_table for b in g])
            res.num_seqs_per_CTAs.append([b.num_seqs for b in g])
            res.CTA_ranks.append([b.rank for b in g])
            res.kv_in_CTAs.append([b.kv for b in g])
        res.max_split_per_seq = max(res.num_split_per_seq)
        res.max_seqs_in_CTA = max((len(b.q_table) for b in boxes), default=0)
        res.max_blocks_in_CTA = max((len(b.block_table) for b in boxes), default=0)
        return res

    def pack_schedule(self, MNWs: Optional[List[List[int]]] = None, HRatio: int = 1, kvHead: int = 8,
                      use_compute_model: bool = False) -> PlanResult:
        """prefix_tree.py:548-616."""
        buckets = MNWs if MNWs is not None else DEFAULT_BUCKETS
        mm = max(b[0] for b in buckets) // HRatio
        boxes: List[Box] = []
        for cid in self.nodes[0].kids.values():
            self._walk(cid, mm, HRatio, use_compute_model, [], boxes)
        boxes = self._balance(boxes, kvHead)
        return self._emit(boxes, buckets, HRatio, len(buckets) == 1)

    def naive_schedule(self, HRatio: int = 1) -> PlanResult:
        """prefix_tree.py:484-545."""
        mm = 64 // HRatio
        boxes: List[Box] = []

        def visit(nid: int) -> None:
            node = self.nodes[nid]
            self._boxes_for(node.seqs, node.s, mm, [], node, boxes)
            for cid in node.kids.values():
                visit(cid)

        for cid in self.nodes[0].kids.values():
            visit(cid)
        return self._emit(boxes, DEFAULT_BUCKETS, HRatio, False)


def plan(block_size: int, seq_lens: List[int], block_table: List[List[int]], MNWs=None, HRatio=1,
         kvHead=8, use_compute_model=False) -> dict:
    """One-shot helper: build + pack, returning plain lists (the KernelInfo fields)."""
    o = PlanOracle(block_size)
    o.build_radix_tree(seq_lens, block_table)
    return o.pack_schedule(MNWs, HRatio, kvHead, use_compute_model).as_dict()


def pad_rows(rows: List[List[int]]) -> List[List[int]]:
    """Zero padding of KernelInfo.to_tensor (prefix_attn/data_class.py:228-253)."""
    width = max(len(r) for r in rows)
    return [list(r) + [0] * (width - len(r)) for r in rows]
