"""pat_amd — prefix-aware decode attention over a paged KV cache for AMD MI355X.

Public API = the `prefix_attn` API of flashserve/PAT (prefix_attn/__init__.py:10-26),
implemented over libpat_amd (C ABI in include/pat_amd.h; HIP kernels for gfx950).
"""
# torch first: its libraries (and the HIP runtime under them) must be initialised before, and torn down
# after, the extension and libpat_amd that use them - loaded the other way round, the process ends
# in a crash inside the heap's clean-up when it exits
import torch  # noqa: F401
try:
    from ._prefix_attn import prefix_attn_with_kvcache, PrefixTreeCPP, paged_decode_baseline
except ImportError as exc:   # no fallback: the compiled binding and libpat_amd.so are the product
    raise ImportError(
        "pat_amd._prefix_attn (the compiled PyTorch-ROCm extension) or libpat_amd.so could not be loaded: "
        f"{exc}. Build both in-tree with `python -m pat_amd.build` (hipcc --offload-arch=gfx950, g++).") from exc
from .utils import generate_random_prefix_seqs, generate_random_kv_cache, generate_tree_seqs
from .data_class import PackedBox, Sequence, SeqGroup, KernelInfo
from .block_scheduler import pack_prefix_blocks, pack_without_prefix, schedule, schedule_naive
from .prefix_tree import PrefixTree
from .async_tree import AsyncTree

__all__ = [
    "prefix_attn_with_kvcache",
    "PrefixTree",
    "PrefixTreeCPP",
    "AsyncTree",
    "generate_random_prefix_seqs",
    "generate_random_kv_cache",
    "generate_tree_seqs",
    "pack_prefix_blocks",
    "pack_without_prefix",
    "schedule",
    "schedule_naive",
    "PackedBox",
    "Sequence",
    "SeqGroup",
    "KernelInfo",
]
