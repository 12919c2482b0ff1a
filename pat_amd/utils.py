"""Synthetic decode batches and paged KV caches (the harness side of the `prefix_attn`
API), plus the padding helpers the vLLM backend uses.

Public names and return conventions follow prefix_attn/utils.py of the flashserve/PAT
tree: `generate_random_kv_cache` (:10-46), `generate_tree_seqs` (:49-100),
`generate_random_prefix_seqs` (:105-164), `make_ndarray_with_pad` /
`make_tensor_with_pad` (:180-219).
"""
from __future__ import annotations

import math
import random
from typing import List, Optional, Tuple, TypeVar, Union

import numpy as np
import torch

from .data_class import SeqGroup

T = TypeVar("T")

TORCH_DTYPE_TO_NUMPY_DTYPE = {
    torch.float16: np.float16,
    torch.float32: np.float32,
    torch.float64: np.float64,
    torch.uint8: np.uint8,
    torch.int32: np.int32,
    torch.int64: np.int64,
}


def generate_random_kv_cache(seq_group: SeqGroup, num_blocks: int, block_size: int, nheads_kv: int,
                             head_dim: int, dtype: torch.dtype = torch.float16, device: str = "cuda",
                             seed: int = 0):
    """N(0,1) paged K/V plus their dense, per-request gathered form.

    Returns (seqlens[B] int32, k_cache[B, S, h_kv, d], v_cache[B, S, h_kv, d],
    kv_padding_mask[B, S] bool, block_table[B, max_blocks] int32 padded with 0,
    k_cache_paged[num_blocks, block_size, h_kv, d], v_cache_paged[...]) with
    S = max_blocks * block_size. K is drawn before V from `torch.random.manual_seed(seed)`.
    """
    torch.random.manual_seed(seed)
    shape = (num_blocks, block_size, nheads_kv, head_dim)
    k_paged = torch.randn(shape, dtype=dtype, device=device)
    v_paged = torch.randn(shape, dtype=dtype, device=device)
    table = torch.tensor(seq_group.get_padded_block_ids(padding_value=0), dtype=torch.int32, device=device)
    batch, width = table.shape
    gather = table.long()
    k_dense = k_paged[gather].reshape(batch, width * block_size, nheads_kv, head_dim)
    v_dense = v_paged[gather].reshape(batch, width * block_size, nheads_kv, head_dim)
    seqlens = torch.tensor(seq_group.seqlens, dtype=torch.int32, device=device)
    mask = torch.arange(width * block_size, device=device)[None, :] < seqlens[:, None]
    return seqlens, k_dense, v_dense, mask, table, k_paged, v_paged


def generate_tree_seqs(tree: str, block_size: int) -> Tuple[SeqGroup, int]:
    """Batch shaped like a prefix tree given as "n1,...,nk_l1,...,lk".

    Level i has n_i nodes of l_i tokens each (multiples of block_size); the batch size is
    n_k. Request i walks node `i // (batch // n_level)` on every level; block ids are
    handed out level by level; requests land in randomly shuffled batch slots.
    Returns (SeqGroup, total number of blocks).
    """
    counts_s, lens_s = tree.split("_")
    counts = [int(x) for x in counts_s.split(",")]
    lens = [int(x) for x in lens_s.split(",")]
    assert min(lens) >= block_size, "every level must hold at least one block"
    assert all(x % block_size == 0 for x in lens), "level lengths must be multiples of block_size"

    batch, total_len = counts[-1], sum(lens)
    group = SeqGroup(block_size, min_seqlen=total_len, max_seqlen=total_len, num_seqs=batch)

    next_block = 0
    level_nodes: List[List[List[int]]] = []
    for count, length in zip(counts, lens):
        per_node = length // block_size
        nodes = []
        for _ in range(count):
            nodes.append(list(range(next_block, next_block + per_node)))
            next_block += per_node
        level_nodes.append(nodes)

    slots = list(range(batch))
    random.shuffle(slots)
    for i in range(batch):
        row: List[int] = []
        for count, nodes in zip(counts, level_nodes):
            row.extend(nodes[i // (batch // count)])
        group.sequences[slots[i]].append_blocks(row, 0)
    return group, next_block


def generate_random_prefix_seqs(min_seqlen: int, max_seqlen: int, batch_size: int, num_prefix: int,
                                prefix_ratio: float, block_size: int, seed: int = 0) -> Tuple[SeqGroup, int]:
    """Batch whose requests share one common prefix of ceil(max_blocks * prefix_ratio) blocks
    (when long enough to hold it) followed by private blocks. Lengths are uniform in
    [min_seqlen, max_seqlen]. Returns (SeqGroup, total number of blocks)."""
    assert num_prefix <= batch_size
    random.seed(seed)
    max_blocks = math.ceil(max_seqlen / block_size)
    shared = math.ceil(max_blocks * prefix_ratio)
    group = SeqGroup(block_size, min_seqlen, max_seqlen, batch_size)

    prefix_ids = random.sample(range(0, shared), shared)
    group.set_common_prefix_blocks(prefix_ids)
    used = len(prefix_ids)
    for seq in group.sequences:
        has_prefix = seq.seqlen >= block_size * shared
        private_tokens = seq.seqlen - shared * block_size if has_prefix else seq.seqlen
        if private_tokens > 0:
            n = math.ceil(private_tokens / block_size)
            seq.append_blocks(random.sample(range(used, used + n), n), 0)
            used += n
    return group, used


def make_ndarray_with_pad(x: List[List[T]], pad: T, dtype, max_len: Optional[int] = None) -> np.ndarray:
    """Ragged rows -> dense [len(x), max_len] array, right-padded with `pad`."""
    if max_len is None:
        max_len = max(map(len, x), default=0)
    out = np.full((len(x), max_len), pad, dtype=dtype)
    for i, row in enumerate(x):
        assert len(row) <= max_len
        out[i, :len(row)] = row
    return out


def make_tensor_with_pad(x: List[list], pad: T, dtype: torch.dtype, max_len: Optional[int] = None,
                         device: Optional[Union[str, torch.device]] = None,
                         pin_memory: bool = False) -> torch.Tensor:
    """`make_ndarray_with_pad` as a torch tensor on `device` (optionally pinned)."""
    arr = make_ndarray_with_pad(x, pad, TORCH_DTYPE_TO_NUMPY_DTYPE[dtype], max_len=max_len)
    t = torch.from_numpy(arr).to(device)
    return t.pin_memory() if pin_memory else t
