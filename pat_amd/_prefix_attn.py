"""The extension-module surface of the reference (`prefix_attn._prefix_attn`), served by
libpat_amd through its C ABI.

Mirrors csrc/bindings.cpp of the flashserve/PAT tree:
  * `prefix_attn_with_kvcache` — table overload (:7-43, :76-95) and tree overload
    (:45-72, :148-157), told apart by the 4th argument;
  * `PrefixTreeCPP` (:100-146) with `build_radix_tree`, `pack_schedule`, `kernel_info`;
  * `KernelInfo.to_gpu(device)` (:97-98).
torch is used for what a binding needs from it: data pointers, strides, the current
HIP stream and scratch memory from the caching allocator. All computation happens in
the HIP kernels of libpat_amd; there is no PyTorch fallback path.
"""
from __future__ import annotations

import contextlib
import ctypes as C
from typing import List, Optional, Union

import numpy as np
import torch

from . import _lib
from .prefix_tree import _NativeTree

_current_device = getattr(torch._C, "_cuda_getDevice", torch.cuda.current_device)

__all__ = ["prefix_attn_with_kvcache", "PrefixTreeCPP", "KernelInfo", "paged_decode_baseline"]


def _check(cond: bool, msg: str) -> None:
    if not cond:
        raise RuntimeError(msg)


class KernelInfo:
    """Plan tensors of a `PrefixTreeCPP`: int32, on the CPU after `pack_schedule`, moved to
    the GPU by `to_gpu` (csrc/prefix_tree.h:7-39)."""

    def __init__(self) -> None:
        self.q_tables: List[torch.Tensor] = []
        self.block_tables: List[torch.Tensor] = []
        self.num_seqs_per_CTAs: List[torch.Tensor] = []
        self.CTA_ranks: List[torch.Tensor] = []
        self.kv_in_CTAs: List[torch.Tensor] = []
        # not in the reference: per (box, sequence) the box's ordinal among that sequence's
        # boxes; the kernels use it as a collision-free partial-result slot
        self.slot_tables: List[torch.Tensor] = []
        self.MNWs: List[List[int]] = []
        self.num_split_per_seq: torch.Tensor = torch.empty(0, dtype=torch.int32)
        self.max_split_per_seq = 0
        # not in the reference: boxes of this plan per sequence (what a launch by slot_tables merges;
        # num_split_per_seq keeps counting over repeated pack_schedule calls, as the reference's does)
        self.num_boxes_per_seq: torch.Tensor = torch.empty(0, dtype=torch.int32)
        self.max_boxes_per_seq = 0
        self.max_seqs_in_CTA = 0
        self.max_blocks_in_CTA = 0
        self._launch_cache: dict = {}
        # Launch copies of the per-bucket tables (what the kernels are given; the tables above keep
        # the scheduler's order): every bucket's boxes longest first, and a bucket whose few widest
        # boxes are more than twice as long as the rest split in two, so that the kernels do not
        # reserve workgroups for every box's KV up to the widest one's length. Workgroups start
        # in launch order and are dealt round-robin to the CUs, so longest-first gives every CU a
        # similar mix and keeps long boxes from starting last.
        self._launch_tables: Optional[dict] = None
        self._launch_order: List[torch.Tensor] = []   # per bucket: sorted position -> scheduler row
        # per bucket: (launch bucket, first sorted position, end) of each part it was split into
        self._launch_parts: List[List[tuple]] = []
        self._block_lens: List[np.ndarray] = []       # per bucket and box: block ids in its block_table row
        # the whole plan in one int32 buffer (pinned on the host when a GPU is there) of which every
        # tensor above and every launch copy is a view: one host-to-device copy moves the plan
        self._flat: Optional[torch.Tensor] = None
        self._flat_layout: Optional[_lib.FlatPlan] = None

    _PER_BOX = ("q_tables", "block_tables", "num_seqs_per_CTAs", "CTA_ranks", "kv_in_CTAs", "slot_tables")
    _MAX_LAUNCH_BUCKETS = 12      # what one launch of the C ABI takes
    _GROWTH_BLOCKS = 8

    def _sort_for_launch(self) -> None:
        """Builds the launch copies from the (host) plan tensors."""
        self._launch_order = [torch.argsort(kv, descending=True, stable=True) for kv in self.kv_in_CTAs]
        names = [name for name in self._PER_BOX if getattr(self, name)]
        tables = {name: [] for name in names}
        tables["MNWs"] = []
        self._launch_parts = []
        spare = self._MAX_LAUNCH_BUCKETS - len(self.MNWs)
        for b, order in enumerate(self._launch_order):
            kv = self.kv_in_CTAs[b][order].numpy()
            n = len(kv)
            cuts = [0, n]
            # a wide head: at most a quarter of the boxes, each more than twice as long as any other
            if spare > 0 and n >= 4 and b < len(self._block_lens):
                k = int((kv > kv[0] // 2).sum())
                if 0 < k <= n // 4:
                    cuts = [0, k, n]
                    spare -= 1
            parts = []
            for lo, hi in zip(cuts[:-1], cuts[1:]):
                rows = order[lo:hi]
                parts.append((len(tables["MNWs"]), lo, hi))
                tables["MNWs"].append(list(self.MNWs[b]))
                for name in names:
                    t = getattr(self, name)[b][rows]
                    if name == "block_tables" and lo > 0:
                        # the narrow part: as wide as its widest box, plus room for its boxes to
                        # grow by a few blocks in place between the steps of multi-step decoding
                        t = t[:, :max(1, int(self._block_lens[b][rows.numpy()].max()) + self._GROWTH_BLOCKS)]
                    tables[name].append(t.contiguous())
            self._launch_parts.append(parts)
        self._launch_tables = tables
        self._launch_cache.clear()

    def launch_tables(self) -> dict:
        """The per-bucket tables as the kernels get them (see `_launch_tables`), with the tile
        labels of the launch buckets under "MNWs"; the scheduler-order tables when no launch
        copies exist."""
        if self._launch_tables is not None:
            return self._launch_tables
        out = {name: getattr(self, name) for name in self._PER_BOX}
        out["MNWs"] = self.MNWs
        return out

    def launch_position(self, b: int):
        """For the boxes of scheduler bucket `b`, in scheduler order: (launch bucket, row in it) as two
        numpy arrays."""
        order = self._launch_order[b].cpu().numpy()
        pos = np.empty(len(order), dtype=np.int64)
        pos[order] = np.arange(len(order))
        bucket = np.empty(len(order), dtype=np.int64)
        row = np.empty(len(order), dtype=np.int64)
        for lb, lo, hi in self._launch_parts[b]:
            inside = (pos >= lo) & (pos < hi)
            bucket[inside] = lb
            row[inside] = pos[inside] - lo
        return bucket, row

    def to_gpu(self, device: Union[torch.device, str]) -> None:
        """Copies every plan tensor to `device` (asynchronously where the source is pinned)."""
        device = torch.device(device)
        if self._flat is not None:
            self._flat = self._flat.to(device, non_blocking=True)
            self._bind(self._flat)
            return

        def move(t: torch.Tensor) -> torch.Tensor:
            return t.to(device, non_blocking=True)

        self.q_tables = [move(t) for t in self.q_tables]
        self.block_tables = [move(t) for t in self.block_tables]
        self.num_seqs_per_CTAs = [move(t) for t in self.num_seqs_per_CTAs]
        self.CTA_ranks = [move(t) for t in self.CTA_ranks]
        self.kv_in_CTAs = [move(t) for t in self.kv_in_CTAs]
        self.slot_tables = [move(t) for t in self.slot_tables]
        self.num_split_per_seq = move(self.num_split_per_seq)
        self.num_boxes_per_seq = move(self.num_boxes_per_seq)
        if self._launch_tables is not None:
            self._launch_tables = {name: (ts if name in ("MNWs", "flags") else [move(t) for t in ts])
                                   for name, ts in self._launch_tables.items()}
            self._launch_order = [move(t) for t in self._launch_order]
        self._launch_cache.clear()

    @classmethod
    def _from_flat(cls, native) -> Optional["KernelInfo"]:
        """The plan of `native` (a `_NativeTree`) as views of one buffer the planner fills, launch
        copies included; None when the plan has more buckets than the flat form holds."""
        lib = _lib.load()
        layout = _lib.FlatPlan()
        if lib.pat_tree_flat_plan(native._h, C.byref(layout), None, 0) != 0:
            return None
        host = torch.empty(max(int(layout.total), 1), dtype=torch.int32, pin_memory=torch.cuda.is_available())
        _lib.check(lib.pat_tree_flat_plan(native._h, C.byref(layout), C.c_void_p(host.data_ptr()), host.numel()))
        ki = cls()
        ki._flat_layout = layout
        ki._flat = host
        ki.max_split_per_seq = layout.max_split_per_seq
        ki.max_boxes_per_seq = layout.max_boxes_per_seq
        ki.max_seqs_in_CTA = layout.max_seqs_in_box
        ki.max_blocks_in_CTA = layout.max_blocks_in_box
        ki._bind(host)
        return ki

    def _bind(self, flat: torch.Tensor) -> None:
        """(Re)creates every plan tensor as a view of `flat` (the buffer on the host or its copy on
        a device)."""
        lay = self._flat_layout

        def tables(f):
            n, ws, wb = f.num_boxes, f.max_seqs, f.max_blocks
            return {"q_tables": flat[f.q_table:f.q_table + n * ws].view(n, ws),
                    "slot_tables": flat[f.q_slot:f.q_slot + n * ws].view(n, ws),
                    "block_tables": flat[f.block_table:f.block_table + n * wb].view(n, wb),
                    "num_seqs_per_CTAs": flat[f.num_seqs:f.num_seqs + n],
                    "CTA_ranks": flat[f.rank:f.rank + n],
                    "kv_in_CTAs": flat[f.kv:f.kv + n]}

        self.num_split_per_seq = flat[lay.num_split_per_seq:lay.num_split_per_seq + lay.batch]
        self.num_boxes_per_seq = flat[lay.num_boxes_per_seq:lay.num_boxes_per_seq + lay.batch]
        for name in self._PER_BOX:
            setattr(self, name, [])
        self.MNWs, self._launch_order, self._launch_parts = [], [], []
        for b in range(lay.num_buckets):
            f = lay.buckets[b]
            self.MNWs.append([f.mnw[0], f.mnw[1], f.mnw[2]])
            for name, t in tables(f).items():
                getattr(self, name).append(t)
            self._launch_order.append(flat[lay.launch_order[b]:lay.launch_order[b] + f.num_boxes])
            self._launch_parts.append([])
        launch = {name: [] for name in self._PER_BOX}
        launch["MNWs"], launch["flags"] = [], []
        for i in range(lay.num_launch_buckets):
            f = lay.launch[i]
            launch["MNWs"].append([f.mnw[0], f.mnw[1], f.mnw[2]])
            launch["flags"].append(int(f.flags))
            for name, t in tables(f).items():
                launch[name].append(t)
            self._launch_parts[f.parent].append((i, f.first, f.first + f.num_boxes))
        self._launch_tables = launch
        self._launch_cache.clear()

    @classmethod
    def _from_view(cls, view: _lib.PlanView) -> "KernelInfo":
        ki = cls()
        for b in range(view.num_buckets):
            bk = view.buckets[b]
            n, ws, wb = bk.num_boxes, bk.max_seqs, bk.max_blocks

            def mat(ptr, w):
                a = np.ctypeslib.as_array(ptr, shape=(n, w)) if w else np.zeros((n, 0), np.int32)
                return torch.from_numpy(a.copy())

            def vec(ptr):
                return torch.from_numpy(np.ctypeslib.as_array(ptr, shape=(n,)).copy())

            ki.MNWs.append([bk.mnw[0], bk.mnw[1], bk.mnw[2]])
            ki.q_tables.append(mat(bk.q_table, ws))
            ki.block_tables.append(mat(bk.block_table, wb))
            ki.num_seqs_per_CTAs.append(vec(bk.num_seqs))
            ki.CTA_ranks.append(vec(bk.rank))
            ki.kv_in_CTAs.append(vec(bk.kv))
            ki.slot_tables.append(mat(bk.q_slot, ws))
            ki._block_lens.append(np.ctypeslib.as_array(bk.block_len, shape=(n,)).copy() if n else np.zeros(0, np.int32))
        ki.num_split_per_seq = torch.from_numpy(
            np.ctypeslib.as_array(view.num_split_per_seq, shape=(view.batch,)).copy())
        ki.num_boxes_per_seq = torch.from_numpy(
            np.ctypeslib.as_array(view.num_boxes_per_seq, shape=(view.batch,)).copy())
        ki.max_split_per_seq = view.max_split_per_seq
        ki.max_boxes_per_seq = view.max_boxes_per_seq
        ki.max_seqs_in_CTA = view.max_seqs_in_box
        ki.max_blocks_in_CTA = view.max_blocks_in_box
        ki._sort_for_launch()
        return ki


class PrefixTreeCPP:
    """Native radix tree + scheduler over a padded block table.

    `build_radix_tree(seq_lens, block_table)`: `seq_lens` is a list of ints or a CPU int32
    tensor, `block_table` a contiguous CPU int32 tensor [num_seqs, max_blocks]; row i uses
    its first ceil(seq_lens[i] / block_size) entries. `pack_schedule` stores the plan in
    `kernel_info`. Both release the GIL while the native code runs.
    """

    def __init__(self, block_size: int):
        self.block_size = int(block_size)
        self._native = _NativeTree(self.block_size)
        self.kernel_info = KernelInfo()

    def build_radix_tree(self, seq_lens: Union[List[int], torch.Tensor], block_table: torch.Tensor) -> None:
        _check(isinstance(block_table, torch.Tensor) and block_table.dim() == 2,
               "block_table must be a 2-D CPU Int32 Tensor")
        _check(block_table.device.type == "cpu" and block_table.dtype == torch.int32,
               "block_table must be a CPU Int32 Tensor")
        table = np.ascontiguousarray(block_table.numpy())
        if isinstance(seq_lens, torch.Tensor):
            _check(seq_lens.device.type == "cpu" and seq_lens.dtype == torch.int32,
                   "seq_lens must be a List[int] or a CPU Int32 Tensor")
            lens = np.ascontiguousarray(seq_lens.numpy().reshape(-1))
        elif isinstance(seq_lens, list):
            lens = np.asarray(seq_lens, dtype=np.int32)
        else:
            raise RuntimeError("seq_lens must be a List[int] or a CPU Int32 Tensor")
        _check(lens.shape[0] == table.shape[0], "Seq lens list mismatch")
        self._native.build_table(lens, table)

    def pack_schedule(self, MNWs: Optional[List[List[int]]] = None, HRatio: int = 1, kvHead: int = 8,
                      use_compute_model: bool = False) -> None:
        if MNWs is not None and len(MNWs) == 0:
            MNWs = None  # an empty list selects the default buckets (csrc/prefix_tree.h:189)
        self._native.pack(MNWs, HRatio, kvHead, use_compute_model)
        self.kernel_info = KernelInfo._from_flat(self._native) or KernelInfo._from_view(self._native.plan_view())


# --------------------------------------------------------------------------------------
#  forward
# --------------------------------------------------------------------------------------

def _strides3(t: torch.Tensor):
    return (C.c_int64 * 3)(t.stride(0), t.stride(1), t.stride(2))


class _Launch:
    """A prepared pat_fwd_args (+ the tensors it points into, kept alive)."""
    __slots__ = ("args", "buckets", "keep", "workspace", "need")


def _prepare(q, k, v, num_split, q_tables, block_tables, num_seqs, ranks, kvs, MNW, max_split,
             max_seqs, max_blocks, scale, out, lse, slot_tables=None, bucket_flags=None) -> _Launch:
    lib = _lib.load()
    # --- checks that need tensor metadata (csrc/api.h:131-181, :256-277) -----------------
    _check(q.dtype in (torch.float16, torch.bfloat16), "only support fp16 and bf16 data type")
    _check(k.dtype == q.dtype, "query and key must have the same dtype")
    _check(v.dtype == q.dtype, "query and value must have the same dtype")
    for name, t in (("q", q), ("kcache", k), ("vcache", v)):
        _check(t.is_cuda, f"{name} must be on CUDA")
    for t in (q, k, v):
        _check(t.dim() == 4 and t.stride(-1) == 1, "Input tensor must have contiguous last dimension")
    b, sq, h, d = q.shape
    nblk, page, hk, dk = k.shape
    _check(tuple(k.shape) == (nblk, page, hk, d), "kcache must have shape (num_blocks, page_block_size, n_heads_kv, head_size_og)")
    _check(tuple(v.shape) == (nblk, page, hk, d), "vcache must have shape (num_blocks, page_block_size, n_heads_kv, head_size_og)")
    _check(out.is_cuda and out.dtype == q.dtype and tuple(out.shape) == tuple(q.shape) and out.stride(-1) == 1,
           "out must be a CUDA tensor with q's shape and dtype and a contiguous last dimension")
    _check(num_split.is_cuda, "num_split_per_seq must be on CUDA")
    _check(num_split.dtype == torch.int32, "num_split_per_seq must have dtype torch.int32")
    _check(num_split.stride(-1) == 1, "num_split_per_seq must have contiguous last dimension")
    _check(tuple(num_split.shape) == (b,), "num_split_per_seq must have shape (batch_size)")
    nb = len(MNW)
    _check(all(len(x) == nb for x in (q_tables, block_tables, num_seqs, ranks, kvs)),
           "MNW and the per-bucket plan lists must have the same length")
    if slot_tables is not None and len(slot_tables) == 0:
        slot_tables = None
    _check(slot_tables is None or len(slot_tables) == nb, "slot_tables must have one entry per bucket")

    L = _Launch()
    L.buckets = (_lib.FwdBucket * max(nb, 1))()
    for i in range(nb):
        qt, bt, ns, rk, kv = q_tables[i], block_tables[i], num_seqs[i], ranks[i], kvs[i]
        ctas = qt.shape[0]
        for name, t in (("query_tables", qt), ("block_tables", bt), ("num_seqs_per_CTA", ns),
                        ("CTA_rank", rk), ("kv_in_CTA", kv)):
            _check(t.is_cuda, f"{name} must be on CUDA")
            _check(t.dtype == torch.int32, f"{name} must have dtype torch.int32")
            _check(t.numel() == 0 or t.stride(-1) == 1, f"{name} must have contiguous last dimension")
        _check(qt.dim() == 2 and bt.dim() == 2 and bt.shape[0] == ctas, "query_tables / block_tables must be (CTAs, width)")
        for name, t in (("num_seqs_per_CTA", ns), ("CTA_rank", rk), ("kv_in_CTA", kv)):
            _check(tuple(t.shape) == (ctas,), f"{name} must have shape (CTAs)")
        fb = L.buckets[i]
        fb.q_table, fb.block_table = qt.data_ptr(), bt.data_ptr()
        fb.num_seqs, fb.rank, fb.kv = ns.data_ptr(), rk.data_ptr(), kv.data_ptr()
        if slot_tables is not None:
            st = slot_tables[i]
            _check(st.is_cuda and st.dtype == torch.int32 and tuple(st.shape) == tuple(qt.shape)
                   and st.stride() == qt.stride(), "slot_tables must match query_tables (CUDA int32, same layout)")
            fb.q_slot = st.data_ptr()
        fb.q_table_stride = qt.stride(0) if ctas > 1 else max(qt.shape[1], 1)
        fb.block_table_stride = bt.stride(0) if ctas > 1 else max(bt.shape[1], 1)
        fb.num_boxes, fb.max_seqs, fb.max_blocks = ctas, qt.shape[1], bt.shape[1]
        fb.mnw[0], fb.mnw[1], fb.mnw[2] = int(MNW[i][0]), int(MNW[i][1]), int(MNW[i][2])
        fb.flags = int(bucket_flags[i]) if bucket_flags else 0

    a = _lib.FwdArgs()
    a.dtype = _lib.PAT_DTYPE_BF16 if q.dtype == torch.bfloat16 else _lib.PAT_DTYPE_F16
    a.batch, a.seqlen_q, a.heads, a.kv_heads = b, sq, h, hk
    a.head_dim, a.page_size, a.num_pages = d, page, nblk
    a.q, a.k, a.v, a.out = q.data_ptr(), k.data_ptr(), v.data_ptr(), out.data_ptr()
    a.q_stride, a.k_stride, a.v_stride, a.o_stride = _strides3(q), _strides3(k), _strides3(v), _strides3(out)
    a.num_split_per_seq = num_split.data_ptr()
    a.max_split_per_seq, a.max_seqs_in_box, a.max_blocks_in_box = int(max_split), int(max_seqs), int(max_blocks)
    a.softmax_scale = float(scale)
    a.num_buckets = nb
    a.buckets = C.cast(L.buckets, C.POINTER(_lib.FwdBucket))
    if lse is not None:
        _check(lse.is_cuda and lse.dtype == torch.float32 and lse.is_contiguous() and lse.numel() == b * h,
               "softmax_lse must be a contiguous CUDA float32 tensor with batch_size * n_heads elements")
        a.lse_out = lse.data_ptr()
    derived = None
    if slot_tables is None and int(max_split) > 1:
        # A plan without slot tables (the reference's call form): CTA_rank is not unique per sequence
        # on irregular forests, so the ordinals are derived from the q_tables on the device, once per
        # prepared launch (the cache keys hold the tables' version counters).
        sbytes = C.c_size_t(0)
        _lib.check(lib.pat_fwd_slots_bytes(C.byref(a), C.byref(sbytes)))
        derived = torch.empty(sbytes.value, dtype=torch.uint8, device=q.device)
        offsets = (C.c_int64 * max(nb, 1))()
        _lib.check(lib.pat_fwd_derive_slots(C.byref(a), C.c_void_p(derived.data_ptr()), sbytes.value, offsets,
                                            C.c_void_p(_raw_stream(q.device.index))))
        for i in range(nb):
            L.buckets[i].q_slot = derived.data_ptr() + 4 * offsets[i]
        a.num_split_per_seq = derived.data_ptr()
    need = C.c_size_t(0)
    _lib.check(lib.pat_fwd_workspace_bytes(C.byref(a), C.byref(need)))
    L.args, L.need = a, need.value
    # plan tensors stay referenced as long as the prepared launch does; q/k/v/out are the
    # caller's for the duration of the call only
    L.keep = (num_split, list(q_tables), list(block_tables), list(num_seqs), list(ranks), list(kvs),
              None if slot_tables is None else list(slot_tables), derived)
    L.workspace = None
    return L


def _raw_stream(index: int) -> int:
    """Handle of torch's current stream on device `index` (the short way when torch offers it)."""
    fast = getattr(torch._C, "_cuda_getCurrentRawStream", None)
    return fast(index) if fast is not None else torch.cuda.current_stream(index).cuda_stream


def _run(L: _Launch, device: torch.device) -> None:
    # scratch for the partial results, from torch's caching allocator on the current stream
    # (none for a single-slot launch, which writes `out` from its first kernel)
    if L.need:
        ws = torch.empty(L.need, dtype=torch.uint8, device=device)
        L.args.workspace = ws.data_ptr()
    else:
        L.args.workspace = None
    L.args.workspace_bytes = L.need
    rc = _lib.load().pat_fwd_launch(C.byref(L.args), C.c_void_p(_raw_stream(device.index)))
    if rc:
        _lib.check(rc)


_TABLE_LAUNCHES: dict = {}


def _table_key(q, k, v, out, lse, vals, slots, flags=None):
    """Identity of a table-form call: every tensor's address and layout plus the scalars. None when
    the arguments are not what a well-formed call passes (the full checks then raise)."""
    try:
        def ident(t):
            return (t.data_ptr(), tuple(t.shape), t.stride())
        def small(t):   # plan tensors: 1-D, or 2-D with contiguous rows (checked when the launch is built)
            return (t.data_ptr(), t.numel(), t.stride(0), t._version)
        lists = tuple(tuple(small(t) for t in vals[name]) for name in
                      ("query_tables", "block_tables", "num_seqs_per_CTAs", "CTA_ranks", "kv_in_CTAs"))
        return (ident(q), ident(k), ident(v), ident(out), q.dtype, None if lse is None else ident(lse),
                small(vals["num_split_per_seq"]), lists, tuple(tuple(m) for m in vals["MNW"]),
                int(vals["max_split_per_seq"]), int(vals["max_seqs_in_CTA"]), int(vals["max_blocks_in_CTA"]),
                float(vals["softmax_scale"]), None if not slots else tuple(small(t) for t in slots),
                None if not flags else tuple(int(f) for f in flags))
    except (AttributeError, TypeError, ValueError):
        return None


def prefix_attn_with_kvcache(q: torch.Tensor, k_cache_paged: torch.Tensor, v_cache_paged: torch.Tensor,
                             *rest, **kw) -> None:
    """Prefix-aware decode attention over a paged KV cache; writes `out` in place.

    Table form:  (q, k_cache_paged, v_cache_paged, num_split_per_seq, query_tables, block_tables,
                  num_seqs_per_CTAs, CTA_ranks, kv_in_CTAs, MNW, max_split_per_seq, max_seqs_in_CTA,
                  max_blocks_in_CTA, softmax_scale, out, timing_=None)
    Tree form:   (q, k_cache_paged, v_cache_paged, tree, softmax_scale, out)
    Both accept the extra keyword `softmax_lse` (float32 [batch, heads]) to receive the
    natural-log LSE, which the reference computes but does not return. The table form also
    accepts `slot_tables` (`KernelInfo.slot_tables`): with it, partial results are filed by each
    box's ordinal within its sequence instead of by CTA_rank, which stays correct on batches
    where the reference scheduler hands the same rank to two boxes of one sequence; and
    `bucket_flags` (one int per bucket, `PAT_BUCKET_EVEN` = 1 when no box of the bucket is shorter
    than 3/4 of its widest: a hint for the launch geometry, never needed for correctness).
    """
    lse = kw.pop("softmax_lse", None)
    slots = kw.pop("slot_tables", None)
    flags = kw.pop("bucket_flags", None)
    tree_names = ("tree", "softmax_scale", "out")
    table_names = ("num_split_per_seq", "query_tables", "block_tables", "num_seqs_per_CTAs", "CTA_ranks",
                   "kv_in_CTAs", "MNW", "max_split_per_seq", "max_seqs_in_CTA", "max_blocks_in_CTA",
                   "softmax_scale", "out", "timing_")
    is_tree = "tree" in kw or (len(rest) > 0 and isinstance(rest[0], PrefixTreeCPP))
    names = tree_names if is_tree else table_names
    if len(rest) > len(names):
        raise TypeError("prefix_attn_with_kvcache(): incompatible function arguments")
    vals = dict(zip(names, rest))
    for key, val in kw.items():
        if key not in names or key in vals:
            raise TypeError(f"prefix_attn_with_kvcache(): incompatible function arguments ({key})")
        vals[key] = val
    missing = [nm for nm in names if nm not in vals and nm != "timing_"]
    if missing:
        raise TypeError(f"prefix_attn_with_kvcache(): missing arguments {missing}")

    out = vals["out"]
    for name, t in (("q", q), ("kcache", k_cache_paged), ("vcache", v_cache_paged)):
        _check(isinstance(t, torch.Tensor) and t.is_cuda, f"{name} must be on CUDA")
    # the kernels launch on the current HIP device: switch only when q lives elsewhere
    index = q.device.index
    guard = torch.cuda.device(index) if index != _current_device() else contextlib.nullcontext()
    with guard:
        if is_tree:
            tree = vals["tree"]
            tree = getattr(tree, "tree", tree) if not isinstance(tree, PrefixTreeCPP) else tree
            info = tree.kernel_info
            key = (q.data_ptr(), k_cache_paged.data_ptr(), v_cache_paged.data_ptr(), out.data_ptr(),
                   tuple(q.shape), q.stride(), k_cache_paged.stride(), v_cache_paged.stride(), out.stride(),
                   q.dtype, float(vals["softmax_scale"]), None if lse is None else lse.data_ptr())
            L = info._launch_cache.get(key)
            if L is None:
                lt = info.launch_tables()
                # partial results are filed by slot_tables: the launch merges each sequence's boxes of
                # THIS plan (num_split_per_seq counts on over repeated pack_schedule calls)
                L = _prepare(q, k_cache_paged, v_cache_paged, info.num_boxes_per_seq, lt["q_tables"],
                             lt["block_tables"], lt["num_seqs_per_CTAs"], lt["CTA_ranks"], lt["kv_in_CTAs"],
                             lt["MNWs"], info.max_boxes_per_seq, info.max_seqs_in_CTA, info.max_blocks_in_CTA,
                             vals["softmax_scale"], out, lse, lt.get("slot_tables"), lt.get("flags"))
                if len(info._launch_cache) >= 256:
                    info._launch_cache.clear()
                info._launch_cache[key] = L
        else:
            # the prepared launch is kept per set of tensors: a decode step calls this once per layer
            # with the same plan, and building the argument block costs more than the kernels of a
            # small batch take. The key holds what the block was built from (addresses and
            # layouts); the tensors' contents are read by the kernels at every call.
            key = _table_key(q, k_cache_paged, v_cache_paged, out, lse, vals, slots, flags)
            L = _TABLE_LAUNCHES.get(key) if key is not None else None
            if L is None:
                L = _prepare(q, k_cache_paged, v_cache_paged, vals["num_split_per_seq"], vals["query_tables"],
                             vals["block_tables"], vals["num_seqs_per_CTAs"], vals["CTA_ranks"], vals["kv_in_CTAs"],
                             vals["MNW"], vals["max_split_per_seq"], vals["max_seqs_in_CTA"],
                             vals["max_blocks_in_CTA"], vals["softmax_scale"], out, lse, slots, flags)
                if key is not None:
                    if len(_TABLE_LAUNCHES) >= 64:
                        _TABLE_LAUNCHES.clear()
                    _TABLE_LAUNCHES[key] = L
        _run(L, q.device)


def paged_decode_baseline(q: torch.Tensor, k_cache_paged: torch.Tensor, v_cache_paged: torch.Tensor,
                          block_table: torch.Tensor, seq_lens: torch.Tensor, softmax_scale: float,
                          out: torch.Tensor, softmax_lse: Optional[torch.Tensor] = None,
                          even_lengths: bool = False) -> None:
    """Prefix-oblivious paged decode attention, the comparator of the benchmarks (not part of the
    reference's API): every request is one work item over its own row of `block_table` (device
    int32 `[batch, max_blocks]`), `seq_lens` (device int32 `[batch]`) tokens long; the same split
    and merge kernels run it. `even_lengths`: no request is shorter than 3/4 of the longest."""
    for name, t in (("q", q), ("kcache", k_cache_paged), ("vcache", v_cache_paged), ("block_table", block_table),
                    ("seq_lens", seq_lens)):
        _check(isinstance(t, torch.Tensor) and t.is_cuda, f"{name} must be on CUDA")
    _check(q.dtype in (torch.float16, torch.bfloat16) and k_cache_paged.dtype == q.dtype and v_cache_paged.dtype == q.dtype,
           "only support fp16 and bf16 data type")
    _check(q.dim() == 4 and k_cache_paged.dim() == 4 and v_cache_paged.dim() == 4, "q, kcache, vcache must be 4-D")
    _check(block_table.dtype == torch.int32 and block_table.dim() == 2 and block_table.stride(1) == 1,
           "block_table must be a 2-D int32 tensor with contiguous rows")
    _check(seq_lens.dtype == torch.int32 and seq_lens.dim() == 1 and seq_lens.is_contiguous(),
           "seq_lens must be a contiguous 1-D int32 tensor")
    b, sq, h, d = q.shape
    _check(sq == 1, "q must have shape (batch_size, 1, n_heads, head_size): decode only")
    _check(block_table.shape[0] == b and seq_lens.shape[0] == b, "block_table / seq_lens must have one row per request")
    _check(out.is_cuda and out.dtype == q.dtype and tuple(out.shape) == tuple(q.shape) and out.stride(-1) == 1,
           "out must be a CUDA tensor with q's shape and dtype and a contiguous last dimension")
    lib = _lib.load()
    a = _lib.BaselineArgs()
    a.dtype = _lib.PAT_DTYPE_BF16 if q.dtype == torch.bfloat16 else _lib.PAT_DTYPE_F16
    a.batch, a.heads, a.kv_heads, a.head_dim = b, h, k_cache_paged.shape[2], d
    a.page_size, a.num_pages, a.max_blocks = k_cache_paged.shape[1], k_cache_paged.shape[0], block_table.shape[1]
    a.q, a.k, a.v, a.out = q.data_ptr(), k_cache_paged.data_ptr(), v_cache_paged.data_ptr(), out.data_ptr()
    a.q_stride, a.k_stride, a.v_stride, a.o_stride = (_strides3(q), _strides3(k_cache_paged), _strides3(v_cache_paged),
                                                      _strides3(out))
    a.block_table, a.block_table_stride = block_table.data_ptr(), block_table.stride(0)
    a.seq_lens = seq_lens.data_ptr()
    a.softmax_scale = float(softmax_scale)
    a.flags = _lib.PAT_BUCKET_EVEN if even_lengths else 0
    if softmax_lse is not None:
        _check(softmax_lse.is_cuda and softmax_lse.dtype == torch.float32 and softmax_lse.is_contiguous()
               and softmax_lse.numel() == b * h, "softmax_lse must be a contiguous CUDA float32 tensor with batch_size * n_heads elements")
        a.lse_out = softmax_lse.data_ptr()
    need = C.c_size_t(0)
    _lib.check(lib.pat_paged_decode_baseline_workspace_bytes(C.byref(a), C.byref(need)))
    index = q.device.index
    guard = torch.cuda.device(index) if index != _current_device() else contextlib.nullcontext()
    with guard:
        ws = torch.empty(need.value, dtype=torch.uint8, device=q.device)
        a.workspace, a.workspace_bytes = ws.data_ptr(), need.value
        _lib.check(lib.pat_paged_decode_baseline_launch(C.byref(a), C.c_void_p(_raw_stream(index))))
