"""ctypes binding of libpat_amd (declarations mirror include/pat_amd.h).

The library is built in-tree by `pat_amd.build` (hipcc, gfx950). There is no
fallback: if it is missing, importing anything that needs it raises.
"""
from __future__ import annotations

import ctypes as C
import os
from typing import Optional

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libpat_amd.so")

ABI_VERSION = 4

PAT_OK = 0
PAT_ERR_INVALID = -1
PAT_ERR_VALUE = -2
PAT_ERR_INDEX = -3
PAT_ERR_KEY = -4
PAT_ERR_HIP = -5
PAT_ERR_WORKSPACE = -6

PAT_DTYPE_F16 = 0
PAT_DTYPE_BF16 = 1

i32p = C.POINTER(C.c_int32)
i64p = C.POINTER(C.c_int64)


class SchedOpts(C.Structure):
    _fields_ = [("long_kv_tokens", C.c_int32), ("long_factor", C.c_int32),
                ("min_boxes", C.c_int32 * 5), ("stop_blocks", C.c_int32), ("max_split", C.c_int32)]


class NodeView(C.Structure):
    _fields_ = [("parent", C.c_int32), ("num_seqs", C.c_int32), ("num_tokens", C.c_int32),
                ("num_seq_ids", C.c_int32), ("num_blocks", C.c_int32), ("num_children", C.c_int32),
                ("seq_ids", i32p), ("block_ids", i32p), ("child_ids", i32p)]


class BucketView(C.Structure):
    _fields_ = [("mnw", C.c_int32 * 3), ("num_boxes", C.c_int32), ("max_seqs", C.c_int32),
                ("max_blocks", C.c_int32), ("q_table", i32p), ("block_table", i32p),
                ("q_len", i32p), ("block_len", i32p), ("num_seqs", i32p), ("rank", i32p),
                ("kv", i32p), ("q_slot", i32p)]


class PlanView(C.Structure):
    _fields_ = [("num_buckets", C.c_int32), ("batch", C.c_int32),
                ("buckets", C.POINTER(BucketView)), ("num_split_per_seq", i32p),
                ("max_split_per_seq", C.c_int32), ("max_seqs_in_box", C.c_int32),
                ("max_blocks_in_box", C.c_int32), ("num_boxes_per_seq", i32p),
                ("max_boxes_per_seq", C.c_int32)]


class FlatBucket(C.Structure):
    _fields_ = [("mnw", C.c_int32 * 3), ("num_boxes", C.c_int32), ("max_seqs", C.c_int32),
                ("max_blocks", C.c_int32), ("parent", C.c_int32), ("first", C.c_int32),
                ("flags", C.c_int32), ("pad_", C.c_int32), ("q_table", C.c_int64), ("q_slot", C.c_int64), ("block_table", C.c_int64),
                ("num_seqs", C.c_int64), ("rank", C.c_int64), ("kv", C.c_int64)]


MAX_FLAT_BUCKETS = 12


class FlatPlan(C.Structure):
    _fields_ = [("num_buckets", C.c_int32), ("num_launch_buckets", C.c_int32), ("batch", C.c_int32),
                ("max_split_per_seq", C.c_int32), ("max_seqs_in_box", C.c_int32),
                ("max_blocks_in_box", C.c_int32), ("total", C.c_int64), ("num_split_per_seq", C.c_int64),
                ("num_boxes_per_seq", C.c_int64), ("max_boxes_per_seq", C.c_int32), ("pad_", C.c_int32),
                ("launch_order", C.c_int64 * MAX_FLAT_BUCKETS), ("buckets", FlatBucket * MAX_FLAT_BUCKETS),
                ("launch", FlatBucket * MAX_FLAT_BUCKETS)]


class FwdBucket(C.Structure):
    _fields_ = [("q_table", C.c_void_p), ("block_table", C.c_void_p), ("num_seqs", C.c_void_p),
                ("rank", C.c_void_p), ("kv", C.c_void_p), ("q_slot", C.c_void_p),
                ("q_table_stride", C.c_int64), ("block_table_stride", C.c_int64),
                ("num_boxes", C.c_int32), ("max_seqs", C.c_int32), ("max_blocks", C.c_int32),
                ("mnw", C.c_int32 * 3), ("flags", C.c_int32)]


PAT_BUCKET_EVEN = 1


class BaselineArgs(C.Structure):
    _fields_ = [("dtype", C.c_int32), ("batch", C.c_int32), ("heads", C.c_int32), ("kv_heads", C.c_int32),
                ("head_dim", C.c_int32), ("page_size", C.c_int32), ("num_pages", C.c_int32),
                ("max_blocks", C.c_int32), ("q", C.c_void_p), ("k", C.c_void_p), ("v", C.c_void_p),
                ("out", C.c_void_p), ("q_stride", C.c_int64 * 3), ("k_stride", C.c_int64 * 3),
                ("v_stride", C.c_int64 * 3), ("o_stride", C.c_int64 * 3), ("block_table", C.c_void_p),
                ("block_table_stride", C.c_int64), ("seq_lens", C.c_void_p), ("softmax_scale", C.c_float),
                ("flags", C.c_int32), ("lse_out", C.c_void_p), ("workspace", C.c_void_p),
                ("workspace_bytes", C.c_size_t)]


class FwdTuning(C.Structure):
    _fields_ = [("chunk_tokens", C.c_int32), ("tall_chunk_tokens", C.c_int32),
                ("head_per_wave_tokens", C.c_int32), ("head_per_wave_long_tokens", C.c_int32),
                ("head_per_wave_long_wgs", C.c_int64), ("equalize_chunks", C.c_int32),
                ("direct_out", C.c_int32), ("tall_rows", C.c_int32), ("reserved", C.c_int32)]

    @classmethod
    def automatic(cls) -> "FwdTuning":
        return cls(0, 0, -1, 0, -1, -1, -1, 0, 0)


class FwdArgs(C.Structure):
    _fields_ = [("dtype", C.c_int32), ("batch", C.c_int32), ("seqlen_q", C.c_int32),
                ("heads", C.c_int32), ("kv_heads", C.c_int32), ("head_dim", C.c_int32),
                ("page_size", C.c_int32), ("num_pages", C.c_int32),
                ("q", C.c_void_p), ("k", C.c_void_p), ("v", C.c_void_p), ("out", C.c_void_p),
                ("lse_out", C.c_void_p),
                ("q_stride", C.c_int64 * 3), ("k_stride", C.c_int64 * 3),
                ("v_stride", C.c_int64 * 3), ("o_stride", C.c_int64 * 3),
                ("num_split_per_seq", C.c_void_p),
                ("max_split_per_seq", C.c_int32), ("max_seqs_in_box", C.c_int32),
                ("max_blocks_in_box", C.c_int32), ("softmax_scale", C.c_float),
                ("num_buckets", C.c_int32), ("buckets", C.POINTER(FwdBucket)),
                ("workspace", C.c_void_p), ("workspace_bytes", C.c_size_t),
                ("split_done_event", C.c_void_p), ("tuning", C.POINTER(FwdTuning)),
                ("records", C.c_void_p), ("records_bytes", C.c_size_t), ("records_tag", C.c_uint64)]


class FwdGeometry(C.Structure):
    _fields_ = [("chunk_tokens", C.c_int32), ("tall_chunk_tokens", C.c_int32),
                ("chunks_per_rank", C.c_int32), ("num_slots", C.c_int32),
                ("num_workgroups", C.c_int64), ("tall_rows", C.c_int32), ("reserved", C.c_int32)]


# Every symbol include/pat_amd.h declares: name -> (restype, argtypes)
SYMBOLS = {
    "pat_last_error": (C.c_char_p, []),
    "pat_abi_version": (C.c_int, []),
    "pat_tree_create": (C.c_int, [C.c_int32, C.POINTER(C.c_void_p)]),
    "pat_tree_destroy": (None, [C.c_void_p]),
    "pat_tree_build": (C.c_int, [C.c_void_p, i32p, i32p, C.c_int32, C.c_int32]),
    "pat_tree_build_rows": (C.c_int, [C.c_void_p, i32p, i32p, i64p, C.c_int32]),
    "pat_tree_pack": (C.c_int, [C.c_void_p, i32p, C.c_int32, C.c_int32, C.c_int32, C.c_int32,
                                C.POINTER(SchedOpts)]),
    "pat_tree_naive_schedule": (C.c_int, [C.c_void_p, C.c_int32]),
    "pat_tree_plan": (C.c_int, [C.c_void_p, C.POINTER(PlanView)]),
    "pat_tree_flat_plan": (C.c_int, [C.c_void_p, C.POINTER(FlatPlan), C.c_void_p, C.c_int64]),
    "pat_tree_num_nodes": (C.c_int, [C.c_void_p]),
    "pat_tree_append": (C.c_int, [C.c_void_p, C.c_int32, i32p, C.c_int32]),
    "pat_tree_remove": (C.c_int, [C.c_void_p, C.c_int32]),
    "pat_tree_grow": (C.c_int, [C.c_void_p, C.c_int32, C.c_int32, i32p, C.c_int32]),
    "pat_tree_num_seqs": (C.c_int, [C.c_void_p]),
    "pat_tree_node": (C.c_int, [C.c_void_p, C.c_int32, C.POINTER(NodeView)]),
    "pat_fwd_validate": (C.c_int, [C.POINTER(FwdArgs)]),
    "pat_fwd_workspace_bytes": (C.c_int, [C.POINTER(FwdArgs), C.POINTER(C.c_size_t)]),
    "pat_fwd_launch": (C.c_int, [C.POINTER(FwdArgs), C.c_void_p]),
    "pat_fwd_launch_static": (C.c_int, [C.POINTER(FwdArgs), C.c_void_p]),
    "pat_fwd_static_scratch_bytes": (C.c_size_t, []),
    "pat_fwd_slots_bytes": (C.c_int, [C.POINTER(FwdArgs), C.POINTER(C.c_size_t)]),
    "pat_fwd_derive_slots": (C.c_int, [C.POINTER(FwdArgs), C.c_void_p, C.c_size_t, i64p, C.c_void_p]),
    "pat_fwd_records_bytes": (C.c_int, [C.POINTER(FwdArgs), C.POINTER(C.c_size_t)]),
    "pat_fwd_records_tag": (C.c_int, [C.POINTER(FwdArgs), C.POINTER(C.c_uint64)]),
    "pat_fwd_build_records": (C.c_int, [C.POINTER(FwdArgs), C.c_void_p, C.c_size_t, C.POINTER(C.c_uint64), C.c_void_p]),
    "pat_fwd_autotune_workspace_bytes": (C.c_int, [C.POINTER(FwdArgs), C.POINTER(C.c_size_t)]),
    "pat_fwd_autotune": (C.c_int, [C.POINTER(FwdArgs), C.c_void_p, C.c_int32, C.c_void_p, C.c_size_t,
                                   C.POINTER(FwdTuning), C.POINTER(C.c_float), C.POINTER(C.c_float)]),
    "pat_fwd_set_tuning": (C.c_int, [C.POINTER(FwdTuning)]),
    "pat_fwd_get_tuning": (C.c_int, [C.POINTER(FwdTuning)]),
    "pat_paged_decode_baseline_workspace_bytes": (C.c_int, [C.POINTER(BaselineArgs), C.POINTER(C.c_size_t)]),
    "pat_paged_decode_baseline_launch": (C.c_int, [C.POINTER(BaselineArgs), C.c_void_p]),
    "pat_fwd_geometry_of": (C.c_int, [C.POINTER(FwdArgs), C.POINTER(FwdGeometry)]),
    "pat_selftest_device": (C.c_int, [C.c_void_p, C.POINTER(C.c_int32)]),
}

_lib: Optional[C.CDLL] = None


def load() -> C.CDLL:
    """Loads libpat_amd.so (once) and types its entry points. Raises if it is not built."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise ImportError(
            f"{LIB_PATH} is missing: build it with `python -m pat_amd.build` "
            "(hipcc, --offload-arch=gfx950). pat_amd has no CPU fallback.")
    # torch ships a HIP runtime of its own; loading it first lets the dynamic loader hand that same
    # runtime to this library (one runtime per process, whatever the import order of the caller)
    import torch  # noqa: F401
    lib = C.CDLL(LIB_PATH)
    for name, (res, args) in SYMBOLS.items():
        fn = getattr(lib, name)
        fn.restype = res
        fn.argtypes = args
    if lib.pat_abi_version() != ABI_VERSION:
        raise ImportError(f"{LIB_PATH}: ABI version {lib.pat_abi_version()} != {ABI_VERSION}, rebuild it")
    _lib = lib
    return lib


def last_error() -> str:
    return load().pat_last_error().decode("utf-8", "replace")


def check(code: int) -> None:
    """Turns a PAT_ERR_* code into the exception the reference API raises in that case."""
    if code == PAT_OK:
        return
    msg = last_error()
    if code == PAT_ERR_VALUE:
        if "by zero" in msg:
            raise ZeroDivisionError(msg)
        raise ValueError(msg)
    if code == PAT_ERR_INDEX:
        raise IndexError(msg)
    if code == PAT_ERR_KEY:
        raise KeyError(msg)
    raise RuntimeError(msg)
