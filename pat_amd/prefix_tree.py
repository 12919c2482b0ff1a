"""`PrefixTree`: the Python-level scheduler API, backed by the C++ planner of libpat_amd.

Keeps the public surface of prefix_attn/prefix_tree.py in the flashserve/PAT tree
(`PrefixTree(block_size)`, `build_radix_tree`, `pack_schedule`, `naive_schedule`,
`getMNW`, the node arrays, `AsyncPrefixTreeScheduler`, `unpad`/`unpad_2d`) and
returns plans identical to it; the planning itself runs in native code through the
C ABI (include/pat_amd.h), so there is one scheduler in this package, not two.
"""
from __future__ import annotations

import ctypes as C
from concurrent.futures import Future
from threading import Thread
from typing import Dict, List, Optional, Sequence, Union

import numpy as np
import torch

from . import _lib
from .data_class import KernelInfo

__all__ = ["PrefixTree", "AsyncPrefixTreeScheduler", "unpad", "unpad_2d", "plan_to_kernel_info"]


def _as_i32(values) -> np.ndarray:
    return np.ascontiguousarray(np.asarray(values, dtype=np.int32).reshape(-1))


def _ptr(a: np.ndarray, ctype=C.c_int32):
    return a.ctypes.data_as(C.POINTER(ctype))


def _copy(ptr, n: int) -> List[int]:
    return np.ctypeslib.as_array(ptr, shape=(n,)).tolist() if n else []


def plan_to_kernel_info(view: _lib.PlanView) -> KernelInfo:
    """Copies a borrowed C plan into a KernelInfo of ragged Python lists."""
    ki = KernelInfo()
    for b in range(view.num_buckets):
        bk = view.buckets[b]
        n, ws, wb = bk.num_boxes, bk.max_seqs, bk.max_blocks
        q = np.ctypeslib.as_array(bk.q_table, shape=(n, ws)) if ws else np.zeros((n, 0), np.int32)
        t = np.ctypeslib.as_array(bk.block_table, shape=(n, wb)) if wb else np.zeros((n, 0), np.int32)
        ql, bl = _copy(bk.q_len, n), _copy(bk.block_len, n)
        ki.MNWs.append([bk.mnw[0], bk.mnw[1], bk.mnw[2]])
        ki.q_tables.append([q[i, :ql[i]].tolist() for i in range(n)])
        ki.block_tables.append([t[i, :bl[i]].tolist() for i in range(n)])
        ki.num_seqs_per_CTAs.append(_copy(bk.num_seqs, n))
        ki.CTA_ranks.append(_copy(bk.rank, n))
        ki.kv_in_CTAs.append(_copy(bk.kv, n))
        sl = np.ctypeslib.as_array(bk.q_slot, shape=(n, ws)) if ws else np.zeros((n, 0), np.int32)
        ki.slot_tables.append([sl[i, :ql[i]].tolist() for i in range(n)])
    ki.num_split_per_seq = _copy(view.num_split_per_seq, view.batch)
    ki.max_split_per_seq = view.max_split_per_seq
    ki.max_seqs_in_CTA = view.max_seqs_in_box
    ki.max_blocks_in_CTA = view.max_blocks_in_box
    return ki


class _NativeTree:
    """Owns one pat_tree handle."""

    def __init__(self, block_size: int):
        self._lib = _lib.load()
        handle = C.c_void_p()
        _lib.check(self._lib.pat_tree_create(int(block_size), C.byref(handle)))
        self._h = handle

    def __del__(self):
        h, self._h = getattr(self, "_h", None), None
        if h:
            self._lib.pat_tree_destroy(h)

    def build_rows(self, seq_lens: Sequence[int], rows: Sequence[Sequence[int]]) -> None:
        n = len(rows)
        if len(seq_lens) < n:
            raise IndexError("list index out of range")  # fewer lengths than block-table rows
        lens = _as_i32(list(seq_lens)[:n])
        offsets = np.zeros(n + 1, dtype=np.int64)
        if n:
            np.cumsum([len(r) for r in rows], out=offsets[1:])
        flat = _as_i32(np.concatenate([np.asarray(r, dtype=np.int32).reshape(-1) for r in rows])
                       if n and offsets[-1] else [])
        _lib.check(self._lib.pat_tree_build_rows(self._h, _ptr(lens), _ptr(flat),
                                                 _ptr(offsets, C.c_int64), n))

    def build_table(self, seq_lens: np.ndarray, table: np.ndarray) -> None:
        _lib.check(self._lib.pat_tree_build(self._h, _ptr(seq_lens), _ptr(table),
                                            int(table.shape[0]), int(table.shape[1])))

    def append(self, seq_len: int, blocks: Sequence[int]) -> None:
        b = _as_i32(list(blocks))
        _lib.check(self._lib.pat_tree_append(self._h, int(seq_len), _ptr(b), int(b.size)))

    def remove(self, seq: int) -> None:
        _lib.check(self._lib.pat_tree_remove(self._h, int(seq)))

    def grow(self, seq: int, new_len: int, more_blocks: Sequence[int]) -> None:
        b = _as_i32(list(more_blocks))
        _lib.check(self._lib.pat_tree_grow(self._h, int(seq), int(new_len), _ptr(b), int(b.size)))

    def num_seqs(self) -> int:
        return self._lib.pat_tree_num_seqs(self._h)

    def pack(self, MNWs, HRatio: int, kvHead: int, use_compute_model: bool, opts=None) -> None:
        if MNWs is None:
            arr, n = None, 0
        else:
            m = np.ascontiguousarray(np.asarray(MNWs, dtype=np.int32).reshape(-1, 3))
            if m.shape[0] == 0:
                raise ValueError("max() arg is an empty sequence")
            arr, n = _ptr(m), m.shape[0]
            self._keep = m
        _lib.check(self._lib.pat_tree_pack(self._h, arr, n, int(HRatio), int(kvHead),
                                           1 if use_compute_model else 0, opts))

    def naive(self, HRatio: int) -> None:
        _lib.check(self._lib.pat_tree_naive_schedule(self._h, int(HRatio)))

    def plan_view(self) -> _lib.PlanView:
        view = _lib.PlanView()
        _lib.check(self._lib.pat_tree_plan(self._h, C.byref(view)))
        return view

    def num_nodes(self) -> int:
        return self._lib.pat_tree_num_nodes(self._h)

    def node(self, i: int) -> _lib.NodeView:
        nv = _lib.NodeView()
        _lib.check(self._lib.pat_tree_node(self._h, i, C.byref(nv)))
        return nv


class PrefixTree:
    """Radix tree over the block-table rows of a decode batch + the packing scheduler.

    >>> tree = PrefixTree(block_size)
    >>> tree.build_radix_tree(seq_lens, block_table_rows)
    >>> info = tree.pack_schedule(MNWs=None, HRatio=h_q // h_kv, kvHead=h_kv)
    >>> info.to_tensor("cuda")
    """

    def __init__(self, block_size: int):
        self.block_size = block_size
        self._native = _NativeTree(block_size)
        self.split_per_seq: List[int] = []

    # -- construction -----------------------------------------------------------
    def build_radix_tree(self, seq_lens: List[int], block_table: List[List[int]]) -> None:
        """Inserts row i of `block_table` (used whole) with length seq_lens[i], in order."""
        self._native.build_rows(seq_lens, block_table)
        self.split_per_seq = [0] * len(block_table)

    # -- edits between decode steps (no counterpart in the reference, which builds a new tree per
    #    step: plugin/vllm/attention/backends/prefix_attn.py:330-338). After any of them the tree and
    #    the plans packed from it are those of a fresh build_radix_tree on the edited batch, provided
    #    every block two requests share is full for both. --------------------------------------------
    def append_sequence(self, seq_len: int, blocks: List[int]) -> int:
        """A request joins the batch behind the last row; returns its row."""
        self._native.append(seq_len, blocks)
        self.split_per_seq = [0] * self._native.num_seqs()
        return len(self.split_per_seq) - 1

    def remove_sequence(self, seq: int) -> None:
        """Row `seq` leaves the batch; the rows behind it move up by one."""
        self._native.remove(seq)
        self.split_per_seq = [0] * self._native.num_seqs()

    def grow_sequence(self, seq: int, new_len: int, more_blocks: Sequence[int] = ()) -> None:
        """Row `seq` now has new_len tokens and the blocks `more_blocks` behind its old ones. Raises
        ValueError (tree unchanged) when only a fresh build can know the new shape: the row grew inside a
        block it shares, or into blocks another row holds."""
        self._native.grow(seq, new_len, more_blocks)
        self.split_per_seq = [0] * self._native.num_seqs()

    # -- scheduling -------------------------------------------------------------
    def pack_schedule(self, MNWs: Optional[List[List[int]]] = None, HRatio: int = 1, kvHead: int = 8,
                      use_compute_model: bool = False) -> KernelInfo:
        self._native.pack(MNWs, HRatio, kvHead, use_compute_model)
        return self._finish()

    def naive_schedule(self, HRatio: int = 1) -> KernelInfo:
        self._native.naive(HRatio)
        return self._finish()

    def _finish(self) -> KernelInfo:
        ki = plan_to_kernel_info(self._native.plan_view())
        self.split_per_seq = ki.num_split_per_seq
        return ki

    def getMNW(self, m_val: int, kv_in_CTA: int):
        """Tile label (M, N, W) for a box of m_val rows over kv_in_CTA tokens."""
        m, w = (64, 4) if m_val > 32 else (32, 2) if m_val > 16 else (16, 1)
        n = 16 if kv_in_CTA < 32 else 32 if kv_in_CTA < 64 else 64 if kv_in_CTA <= 128 else 128
        return (m, max(n, 32) if m == 64 else n, w)

    # -- introspection (same names as the reference's parallel arrays) -----------
    @property
    def num_nodes(self) -> int:
        return self._native.num_nodes()

    @property
    def root(self) -> int:
        return 0

    def _nodes(self):
        return [self._native.node(i) for i in range(self.num_nodes)]

    @property
    def parents(self) -> List[int]:
        return [n.parent for n in self._nodes()]

    @property
    def s_values(self) -> List[int]:
        return [n.num_seqs for n in self._nodes()]

    @property
    def lens(self) -> List[int]:
        return [n.num_tokens for n in self._nodes()]

    @property
    def seq_indices(self) -> List[List[int]]:
        return [_copy(n.seq_ids, n.num_seq_ids) for n in self._nodes()]

    @property
    def block_ids(self) -> List[List[int]]:
        return [_copy(n.block_ids, n.num_blocks) for n in self._nodes()]

    @property
    def tree(self) -> Dict[int, Dict[int, int]]:
        """node id -> {first block id of child: child id}, children in insertion order."""
        out: Dict[int, Dict[int, int]] = {}
        nodes = self._nodes()
        for i, n in enumerate(nodes):
            kids = _copy(n.child_ids, n.num_children)
            out[i] = {nodes[c].block_ids[0]: c for c in kids}
        return out

    def print_tree(self) -> None:
        nodes, seqs, blocks = self._nodes(), self.seq_indices, self.block_ids

        def show(i: int, depth: int) -> None:
            n = nodes[i]
            print(" " * depth + f"Node {i}: S={n.num_seqs}, len={n.num_tokens}, seqs={seqs[i]}, blocks={blocks[i]}")
            for c in _copy(n.child_ids, n.num_children):
                show(c, depth + 2)

        show(0, 0)


def unpad(lst):
    """Drops trailing zeros of a padded row (keeps at least one entry)."""
    end = len(lst)
    while end > 1 and lst[end - 1] == 0:
        end -= 1
    return lst[:end]


def unpad_2d(table):
    return [unpad(row) for row in table]


class AsyncPrefixTreeScheduler(Thread):
    """Builds tree + plan + device tensors on a helper thread and resolves `future`
    with the KernelInfo (or the exception)."""

    def __init__(self, future: Future, block_tables: Union[List[List[int]], torch.Tensor],
                 seq_lens: List[int], num_decode_tokens: int, block_size: int, nheads: int,
                 nheads_kv: Optional[int], MNWs: Optional[List[List[int]]], device):
        super().__init__()
        self.future = future
        self.block_tables = block_tables
        self.seq_lens = seq_lens
        self.num_decode_tokens = num_decode_tokens
        self.block_size = block_size
        self.nheads = nheads
        self.nheads_kv = nheads_kv
        self.MNWs = MNWs
        self.device = device

    def run(self) -> None:
        try:
            rows = self.block_tables
            if isinstance(rows, torch.Tensor):
                rows = rows.cpu().tolist()
            tree = PrefixTree(self.block_size)
            tree.build_radix_tree(self.seq_lens, rows)
            ratio = self.nheads // self.nheads_kv if self.nheads_kv is not None else 64
            info = tree.pack_schedule(self.MNWs, ratio)
            info.to_tensor(device=self.device)
            self.future.set_result(info)
        except Exception as exc:  # surfaced by Future.result()
            self.future.set_exception(exc)
