"""ctypes route to the forward entry points of libpat_amd, for code that drives the C ABI directly:
the raw C-ABI tests and the benchmarks' timed loops (`pat_fwd_launch` on a prepared argument
block, nothing else in the timed region).

The product binding is the compiled extension `pat_amd._prefix_attn`
(csrc/torch_ext/prefix_attn_ext.cc); this module builds the same `pat_fwd_args` from torch
tensors in Python so that a test can look inside it, change its workspace, or hand it to another
entry point (`pat_fwd_launch_static`, `pat_fwd_geometry_of`).
"""
from __future__ import annotations

import ctypes as C

import torch

from . import _lib

__all__ = ["prepare", "run"]


def _check(cond: bool, msg: str) -> None:
    if not cond:
        raise RuntimeError(msg)


def _strides3(t: torch.Tensor):
    return (C.c_int64 * 3)(t.stride(0), t.stride(1), t.stride(2))


class _Launch:
    """A prepared pat_fwd_args (+ the tensors it points into, kept alive)."""
    __slots__ = ("args", "buckets", "keep", "workspace", "need", "tuning", "tuned_us", "auto_us")


def prepare(q, k, v, num_split, q_tables, block_tables, num_seqs, ranks, kvs, MNW, max_split,
            max_seqs, max_blocks, scale, out, lse, slot_tables=None, bucket_flags=None, autotune=False, tuning=None,
            build_records=True) -> _Launch:
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
    L.tuning, L.tuned_us, L.auto_us = tuning, None, None
    if tuning is not None:          # a geometry measured earlier for this plan shape
        a.tuning = C.pointer(L.tuning)
    elif autotune:
        # measured choice of the launch geometry (pat_fwd_autotune): runs the launch a few times per
        # candidate on the current stream and synchronises it; `out` holds a valid result afterwards
        most = C.c_size_t(0)
        _lib.check(lib.pat_fwd_autotune_workspace_bytes(C.byref(a), C.byref(most)))
        scratch = torch.empty(max(most.value, 256), dtype=torch.uint8, device=q.device)
        a.workspace, a.workspace_bytes = scratch.data_ptr(), scratch.numel()
        L.tuning = _lib.FwdTuning()
        best_us, auto_us = C.c_float(0), C.c_float(0)
        evict = _evict_buffer(q.device)
        _lib.check(lib.pat_fwd_autotune(C.byref(a), C.c_void_p(_raw_stream(q.device.index)), 10,
                                        C.c_void_p(evict.data_ptr()), evict.numel(), C.byref(L.tuning),
                                        C.byref(best_us), C.byref(auto_us)))
        a.tuning = C.pointer(L.tuning)
        a.workspace, a.workspace_bytes = None, 0
        L.tuned_us, L.auto_us = best_us.value, auto_us.value
    records = None
    if build_records:
        # the launch records of this plan under the geometry just chosen: one small kernel now,
        # none in the launches
        rbytes, tag = C.c_size_t(0), C.c_uint64(0)
        _lib.check(lib.pat_fwd_records_bytes(C.byref(a), C.byref(rbytes)))
        records = torch.empty(rbytes.value, dtype=torch.uint8, device=q.device)
        _lib.check(lib.pat_fwd_build_records(C.byref(a), C.c_void_p(records.data_ptr()), rbytes.value, C.byref(tag),
                                             C.c_void_p(_raw_stream(q.device.index))))
        a.records, a.records_bytes, a.records_tag = records.data_ptr(), rbytes.value, tag.value
    need = C.c_size_t(0)
    _lib.check(lib.pat_fwd_workspace_bytes(C.byref(a), C.byref(need)))
    L.args, L.need = a, need.value
    # plan tensors stay referenced as long as the prepared launch does; q/k/v/out are the
    # caller's for the duration of the call only
    L.keep = (num_split, list(q_tables), list(block_tables), list(num_seqs), list(ranks), list(kvs),
              None if slot_tables is None else list(slot_tables), derived, records)
    L.workspace = None
    return L


_EVICT: dict = {}


def _evict_buffer(device: torch.device) -> torch.Tensor:
    """Per device: 320 MB that the tuning run reads between timed launches (larger than the 256 MB
    memory-side cache), allocated on first use and kept."""
    if device.index not in _EVICT:
        _EVICT[device.index] = torch.zeros(320 << 20, dtype=torch.uint8, device=device)
    return _EVICT[device.index]


def _raw_stream(index: int) -> int:
    """Handle of torch's current stream on device `index` (the short way when torch offers it)."""
    fast = getattr(torch._C, "_cuda_getCurrentRawStream", None)
    return fast(index) if fast is not None else torch.cuda.current_stream(index).cuda_stream


def run(L: _Launch, device: torch.device) -> None:
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


_prepare, _run = prepare, run
