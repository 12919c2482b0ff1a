"""Decode branch of the vLLM `PREFIX_ATTN` backend, without vLLM.

What plugin/vllm/attention/backends/prefix_attn.py of the flashserve/PAT tree does for the decode
tokens of a step, as two plain objects a backend (or a test with a stand-in for vLLM's
AttentionMetadata) can drive:

* `DecodePlan.from_metadata(meta)` is the `decode_metadata` property (:313-338): it drops the
  prefill rows of the step and starts an `AsyncTree` over the decode requests' lengths and the CPU
  copy of their block table, so the plan is built while the step's earlier work runs;
* `decode_attention(...)` is the tail of `PrefixAttentionImpl.forward` (:901-915): it splits
  vLLM's `[2, num_blocks, block_size, kv_heads, head_size]` cache, waits for the plan and calls
  `prefix_attn_with_kvcache` on `[B, 1, N, d]` views of the query and output.

* `DecodePlan.advance_step(block_tables_cpu)` is what multi-step decoding needs on top of the
  reference's `advance_step` (:377-448), which moves the lengths forward but leaves the tree as it
  was: every request grew by one token, so the work item that holds its tail gets one more token
  (and, at a page boundary, the next block id) in place on the device; the plan is rebuilt only
  when that is not possible (a tail shared by several requests, a block row that is full).

* `DecodePlan.from_previous(prev, meta, left, joined)` makes the next step's plan by editing the
  previous step's tree (requests that left, requests that joined, every row one step longer)
  instead of building a new tree; the result is the plan a fresh build gives.

`meta` only needs the attributes read here (`num_prefills`, `num_decode_tokens`, `seq_lens`,
`block_tables`, `block_tables_cpu`, `block_size`, `nheads`, `nheads_kv`,
`max_decode_query_len`); vLLM's own metadata class has them after the reference's overlay.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Any, List, Optional, Union

import numpy as np
import torch

from ._prefix_attn import PrefixTreeCPP, prefix_attn_with_kvcache
from .async_tree import AsyncTree

__all__ = ["DecodePlan", "decode_attention"]


@dataclass
class DecodePlan:
    """Per-step decode state shared by all attention layers of the step."""
    num_decode_tokens: int
    seq_lens: List[int]
    block_tables: Optional[torch.Tensor]       # device table of the decode requests
    tree: Union[AsyncTree, PrefixTreeCPP]
    max_decode_query_len: int = 1
    block_size: int = 16
    nheads: int = 1
    nheads_kv: int = 1
    replans: int = 0                           # times advance_step had to plan afresh
    _tails: Any = None                         # per request (bucket, box) of the item holding its tail
    _tail_kv: Any = None
    _launch_row: Any = None                    # per bucket: scheduler row -> (launch bucket, row)

    @classmethod
    def from_metadata(cls, meta: Any) -> Optional["DecodePlan"]:
        if meta.num_decode_tokens == 0:
            return None
        first = meta.num_prefills
        seq_lens = list(meta.seq_lens[first:])
        tables = None if meta.block_tables is None else meta.block_tables[first:]
        table_cpu = meta.block_tables_cpu[first:] if meta.block_tables_cpu.shape[0] != len(seq_lens) \
            else meta.block_tables_cpu
        device = tables.device if tables is not None else torch.device("cuda")
        tree = AsyncTree(block_size=meta.block_size, seq_lens=seq_lens, table=table_cpu, MNWs=None,
                         HRatio=meta.nheads // meta.nheads_kv, kvHead=meta.nheads_kv, device=device)
        return cls(num_decode_tokens=meta.num_decode_tokens, seq_lens=seq_lens, block_tables=tables, tree=tree,
                   max_decode_query_len=getattr(meta, "max_decode_query_len", 1), block_size=meta.block_size,
                   nheads=meta.nheads, nheads_kv=meta.nheads_kv)

    @classmethod
    def from_previous(cls, prev: "DecodePlan", meta: Any, left: List[int] = (), joined: int = 0) -> "DecodePlan":
        """The next step's plan made by editing the previous step's tree instead of building a new one
        (the reference builds one per step, `decode_metadata` :313-338). `left`: rows of the previous
        decode batch that are gone; the requests that stay keep their order and the `joined` new ones
        stand behind them in `meta` (vLLM appends to its running queue). Every remaining row's new
        length and block row come from `meta`. The tree and the plan are those a fresh build gives for
        this batch (`pat_tree_remove` / `pat_tree_append` / `pat_tree_grow`); rows that cannot be
        grown in place make the tree fall back to a fresh build by itself."""
        first = meta.num_prefills
        seq_lens = list(meta.seq_lens[first:])
        tables = None if meta.block_tables is None else meta.block_tables[first:]
        table_cpu = meta.block_tables_cpu[first:] if meta.block_tables_cpu.shape[0] != len(seq_lens) \
            else meta.block_tables_cpu
        tree = prev._ready_tree()
        for row in sorted(left, reverse=True):
            tree.remove_sequence(int(row))
        stay = len(seq_lens) - joined
        bs = meta.block_size
        for row in range(stay, len(seq_lens)):
            tree.append_sequence(int(seq_lens[row]), table_cpu[row, :-(-int(seq_lens[row]) // bs)].tolist())
        tree.advance(seq_lens, table_cpu)
        tree.pack_schedule(MNWs=None, HRatio=meta.nheads // meta.nheads_kv, kvHead=meta.nheads_kv)
        device = tables.device if tables is not None else prev._ready_tree().kernel_info.num_split_per_seq.device
        tree.kernel_info.to_gpu(device)
        return cls(num_decode_tokens=meta.num_decode_tokens, seq_lens=seq_lens, block_tables=tables, tree=tree,
                   max_decode_query_len=getattr(meta, "max_decode_query_len", 1), block_size=meta.block_size,
                   nheads=meta.nheads, nheads_kv=meta.nheads_kv)

    # ---- multi-step decoding ---------------------------------------------------------------
    def _ready_tree(self) -> PrefixTreeCPP:
        return self.tree.tree if isinstance(self.tree, AsyncTree) else self.tree

    def _find_tails(self, table_cpu: torch.Tensor):
        """For every request the (bucket, box) of the single-request item that ends with the
        request's last block, or -1 where the tail sits in an item shared with other requests."""
        info = self._ready_tree().kernel_info
        bs = self.block_size
        n = len(self.seq_lens)
        last_block = np.array([int(table_cpu[i, (self.seq_lens[i] - 1) // bs]) for i in range(n)])
        tails = np.full((n, 2), -1, dtype=np.int64)
        self._tail_kv = np.zeros(n, dtype=np.int64)      # host mirror of the tail items' token counts
        for b in range(len(info.MNWs)):
            nseq = info.num_seqs_per_CTAs[b].cpu().numpy()
            kv = info.kv_in_CTAs[b].cpu().numpy()
            qt = info.q_tables[b].cpu().numpy()
            bt = info.block_tables[b].cpu().numpy()
            for box in np.nonzero(nseq == 1)[0]:
                s = int(qt[box, 0])
                if kv[box] > 0 and bt[box, (kv[box] - 1) // bs] == last_block[s]:
                    tails[s] = (b, box)
                    self._tail_kv[s] = kv[box]
        return tails

    def _replan(self, table_cpu: torch.Tensor) -> None:
        device = self._ready_tree().kernel_info.num_split_per_seq.device
        self.tree = AsyncTree(block_size=self.block_size, seq_lens=list(self.seq_lens), table=table_cpu, MNWs=None,
                              HRatio=self.nheads // self.nheads_kv, kvHead=self.nheads_kv, device=device)
        self._tails = None
        self._launch_row = None
        self.replans += 1

    def advance_step(self, block_tables_cpu: torch.Tensor) -> bool:
        """Every decode request has grown by one token (`block_tables_cpu` already names the block
        that token went to). Returns True when the plan was updated in place, False when it was
        rebuilt."""
        bs = self.block_size
        table_cpu = block_tables_cpu[-len(self.seq_lens):] if block_tables_cpu.shape[0] != len(self.seq_lens) \
            else block_tables_cpu
        if self._tails is None:
            self._tails = self._find_tails(table_cpu)
        info = self._ready_tree().kernel_info
        old = list(self.seq_lens)
        self.seq_lens = [x + 1 for x in old]
        if (self._tails[:, 0] < 0).any():
            self._replan(table_cpu)
            return False
        new_blocks = {}                       # bucket -> ([box], [column], [block id])
        for s, n_old in enumerate(old):
            if n_old % bs:
                continue
            b, box = self._tails[s]
            col = -(-int(self._tail_kv[s]) // bs)           # blocks the item holds now
            boxes, cols, ids = new_blocks.setdefault(int(b), ([], [], []))
            boxes.append(int(box))
            cols.append(col)
            ids.append(int(table_cpu[s, n_old // bs]))
        # The tables the kernels read are launch copies (boxes in another order, a bucket perhaps
        # split in two with narrower block tables); the scheduler-order tables are kept in step so
        # that they go on describing the same plan. (table list, scheduler bucket) -> per table of
        # the list the rows of the given boxes.
        launch = info.launch_tables()
        targets = [(info.kv_in_CTAs, info.block_tables, lambda b, boxes: {b: (boxes, np.arange(len(boxes)))})]
        if launch["kv_in_CTAs"] is not info.kv_in_CTAs:
            if self._launch_row is None:
                self._launch_row = [tuple(t.numpy() for t in info.launch_position(b)) for b in range(len(info.MNWs))]

            def in_launch(b, boxes):
                lb, lr = self._launch_row[b]
                return {int(t): (lr[boxes[lb[boxes] == t]], np.nonzero(lb[boxes] == t)[0]) for t in np.unique(lb[boxes])}
            targets.append((launch["kv_in_CTAs"], launch["block_tables"], in_launch))
        # a block row that is full (in either copy) means a fresh plan
        for _, tables, place in targets:
            for b, (boxes, cols, _) in new_blocks.items():
                for t, (_, which) in place(b, np.asarray(boxes)).items():
                    if (np.asarray(cols)[which] >= tables[t].shape[1]).any():
                        self._replan(table_cpu)
                        return False
        # a small batch that is launched as one work item per request (KernelInfo.whole_sequence_tables):
        # those tables grow too; a request that outgrows its block row, or the form, means a fresh plan
        whole = info.whole_sequence_tables()
        if whole is not None:
            width = whole["block_tables"][0].shape[1]
            if any(n_old % bs == 0 and n_old // bs >= width for n_old in old) or max(self.seq_lens) > whole["longest_allowed"]:
                self._replan(table_cpu)
                return False
        self._tail_kv += 1
        device = info.num_split_per_seq.device
        if whole is not None:
            whole["kv_in_CTAs"][0].add_(1)
            crossed = [s for s, n_old in enumerate(old) if n_old % bs == 0]
            if crossed:
                flat = torch.as_tensor([s * width + old[s] // bs for s in crossed], device=device)
                ids = torch.as_tensor([int(table_cpu[s, old[s] // bs]) for s in crossed], dtype=torch.int32, device=device)
                whole["block_tables"][0].view(-1).index_copy_(0, flat, ids)
        for kvs, tables, place in targets:
            for b in range(len(info.MNWs)):
                grown = self._tails[self._tails[:, 0] == b, 1]
                if len(grown):
                    for t, (rows, _) in place(b, grown).items():
                        kvs[t].index_add_(0, torch.as_tensor(rows, device=device),
                                          torch.ones(len(rows), dtype=torch.int32, device=device))
                if b in new_blocks:
                    boxes, cols, ids = (np.asarray(x) for x in new_blocks[b])
                    for t, (rows, which) in place(b, boxes).items():
                        flat = rows * tables[t].shape[1] + cols[which]
                        tables[t].view(-1).index_copy_(0, torch.as_tensor(flat, device=device),
                                                       torch.as_tensor(ids[which], dtype=torch.int32, device=device))
        return True


def decode_attention(decode_query: torch.Tensor, kv_cache: torch.Tensor, plan: DecodePlan, softmax_scale: float,
                     decode_output: torch.Tensor) -> torch.Tensor:
    """decode_query / decode_output: [num_decode_tokens, num_heads, head_size];
    kv_cache: [2, num_blocks, block_size, num_kv_heads, head_size]. Writes and returns decode_output."""
    assert plan.max_decode_query_len <= 1, \
        "Speculative decoding with variable length queries is not supported yet."
    key_cache, value_cache = kv_cache[0], kv_cache[1]
    tree = plan.tree.tree if isinstance(plan.tree, AsyncTree) else plan.tree
    prefix_attn_with_kvcache(q=decode_query.unsqueeze(1), k_cache_paged=key_cache, v_cache_paged=value_cache,
                             tree=tree, softmax_scale=softmax_scale, out=decode_output.unsqueeze(1))
    return decode_output
