"""Seeded synthetic decode batches for the benchmark configurations of this project.

Every workload is a `Workload`: block-table rows (physical ids are a seeded random
permutation, logical sharing = repeated ids), per-request lengths, head geometry and
dtype. Shared nodes are whole blocks (a partly filled page cannot be shared); leaves
may end inside a page.

  c1   8 requests, 256 shared + 32 private tokens, 8/8 heads, d 64
  c2   64 requests, 2048 shared + U[64,512] private, 32/8 heads, d 128, bf16   (headline)
  c3   128 requests, 1024 root, 8 x 512 mid (16 requests each), U[128,1024] leaves, fp16
  c4   256 requests, forest of 16 roots U[256,4096], depth <= 4, fan-out U{2,3,4},
       inner U[64,512], leaves U[32,256], 16/16 heads, d 64, fp16
  c5a  32 requests, 16384 shared + U[256,2048] private, 64/8 heads, d 128, bf16
  c5b  32 independent 4096-token requests (no sharing), 64/8 heads, d 128, bf16

A diagnostic beside them (not a benchmark configuration, not in NAMES):
  c5a-prefix  c5a's shared 16384-token prefix with 16-token private suffixes: a launch made of
              64-row boxes only, for profiling the tall-box path of the split kernel
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Dict, List, Optional, Tuple

import numpy as np
import torch

PAGE = 16


@dataclass
class Workload:
    name: str
    heads: int
    kv_heads: int
    head_dim: int
    dtype: torch.dtype
    page_size: int
    seq_lens: List[int]
    rows: List[List[int]]          # unpadded block-table rows
    num_blocks: int
    unique_tokens: int             # tokens over distinct tree nodes
    seed: int
    tree: dict = field(default_factory=dict)   # description of the drawn tree

    @property
    def batch(self) -> int:
        return len(self.rows)

    @property
    def total_tokens(self) -> int:
        return int(sum(self.seq_lens))

    def kv_bytes(self, tokens: int) -> int:
        """Bytes of K and V for `tokens` tokens over all kv heads."""
        return tokens * self.kv_heads * self.head_dim * 2 * torch.empty(0, dtype=self.dtype).element_size()

    @property
    def unique_kv_bytes(self) -> int:
        return self.kv_bytes(self.unique_tokens)

    def padded_table(self, pad: int = 0) -> torch.Tensor:
        width = max(len(r) for r in self.rows)
        t = torch.full((self.batch, width), pad, dtype=torch.int32)
        for i, r in enumerate(self.rows):
            t[i, :len(r)] = torch.tensor(r, dtype=torch.int32)
        return t

    def tensors(self, device, seed: Optional[int] = None, copies: int = 1):
        """q [B,1,H,d], k/v caches [copies][num_blocks, page, h_kv, d] ~ N(0,1), seeded."""
        gen = torch.Generator(device="cpu").manual_seed(self.seed if seed is None else seed)
        q = torch.randn(self.batch, 1, self.heads, self.head_dim, generator=gen).to(self.dtype).to(device)
        shape = (self.num_blocks, self.page_size, self.kv_heads, self.head_dim)
        ks, vs = [], []
        for _ in range(copies):
            ks.append(torch.randn(shape, generator=gen).to(self.dtype).to(device))
            vs.append(torch.randn(shape, generator=gen).to(self.dtype).to(device))
        if copies == 1:
            return q, ks[0], vs[0]
        return q, ks, vs


class _Alloc:
    """Hands out physical block ids from a seeded permutation of range(capacity)."""

    def __init__(self, rng: np.random.Generator, capacity: int):
        self.perm = rng.permutation(capacity).tolist()
        self.at = 0

    def take(self, n: int) -> List[int]:
        out = self.perm[self.at:self.at + n]
        assert len(out) == n, "block pool exhausted"
        self.at += n
        return out


def _blocks(tokens: int) -> int:
    return (tokens + PAGE - 1) // PAGE


def _round_page(tokens: int) -> int:
    return max(PAGE, int(round(tokens / PAGE)) * PAGE)


def _finish(name, heads, kv_heads, d, dtype, seed, lens, rows, alloc, unique, tree) -> Workload:
    return Workload(name, heads, kv_heads, d, dtype, PAGE, lens, rows, alloc.at, unique, seed, tree)


def shared_prefix(name: str, batch: int, prefix: int, lo: int, hi: int, heads: int, kv_heads: int, d: int,
                  dtype, seed: int) -> Workload:
    """One prefix shared by all requests + a private suffix of U[lo, hi] tokens each."""
    rng = np.random.default_rng(seed)
    suffix = rng.integers(lo, hi + 1, size=batch).tolist()
    alloc = _Alloc(rng, _blocks(prefix) + sum(_blocks(s) for s in suffix))
    pre = alloc.take(_blocks(prefix))
    rows = [pre + alloc.take(_blocks(s)) for s in suffix]
    lens = [prefix + s for s in suffix]
    return _finish(name, heads, kv_heads, d, dtype, seed, lens, rows, alloc, prefix + sum(suffix),
                   {"prefix": prefix, "suffix": suffix})


def independent(name: str, batch: int, length: int, heads: int, kv_heads: int, d: int, dtype, seed: int) -> Workload:
    rng = np.random.default_rng(seed)
    alloc = _Alloc(rng, batch * _blocks(length))
    rows = [alloc.take(_blocks(length)) for _ in range(batch)]
    return _finish(name, heads, kv_heads, d, dtype, seed, [length] * batch, rows, alloc, batch * length,
                   {"length": length})


def three_level(name: str, batch: int, root: int, mids: int, mid_len: int, lo: int, hi: int, heads: int,
                kv_heads: int, d: int, dtype, seed: int) -> Workload:
    rng = np.random.default_rng(seed)
    leaves = rng.integers(lo, hi + 1, size=batch).tolist()
    alloc = _Alloc(rng, _blocks(root) + mids * _blocks(mid_len) + sum(_blocks(x) for x in leaves))
    root_b = alloc.take(_blocks(root))
    mid_b = [alloc.take(_blocks(mid_len)) for _ in range(mids)]
    per = batch // mids
    rows = [root_b + mid_b[i // per] + alloc.take(_blocks(leaves[i])) for i in range(batch)]
    lens = [root + mid_len + x for x in leaves]
    return _finish(name, heads, kv_heads, d, dtype, seed, lens, rows, alloc,
                   root + mids * mid_len + sum(leaves), {"root": root, "mids": mids, "mid_len": mid_len,
                                                         "leaves": leaves})


def forest(name: str, batch: int, roots: int, heads: int, kv_heads: int, d: int, dtype, seed: int,
           root_range=(256, 4096), inner_range=(64, 512), leaf_range=(32, 256), max_depth: int = 4,
           fanout=(2, 3, 4)) -> Workload:
    """Irregular prefix forest with exactly `batch` leaves (= requests), spread evenly over the
    roots. A node at depth < max_depth with n > 1 leaves below it draws a fan-out in `fanout`
    (widened only when n could not fit otherwise) and splits n over its children at random."""
    rng = np.random.default_rng(seed)
    specs: List[dict] = []   # per request: list of (node tokens) along its path
    nodes_tokens = 0
    paths: List[List[Tuple[int, int]]] = []   # per request: [(node id, tokens)]
    node_tokens: Dict[int, int] = {}
    next_node = [0]

    def new_node(tokens: int) -> int:
        nid = next_node[0]
        next_node[0] += 1
        node_tokens[nid] = tokens
        return nid

    def grow(path: List[Tuple[int, int]], n: int, depth: int) -> None:
        # `path` ends at an internal node of depth `depth`; hang n leaves below it
        levels_left = max_depth - depth           # levels available below this node
        cap = max(fanout) ** (levels_left - 1) if levels_left >= 1 else 0   # leaves one child can hold
        k_min = max(2, -(-n // cap)) if n > 1 else 1
        k = int(rng.choice(fanout)) if n > 1 else 1
        k = min(max(k, k_min), n)
        # random composition of n into k parts, each in [1, cap]
        parts = [1] * k
        for _ in range(n - k):
            room = [i for i in range(k) if parts[i] < cap]
            parts[int(rng.choice(room))] += 1
        for part in parts:
            if part == 1:
                leaf = new_node(int(rng.integers(leaf_range[0], leaf_range[1] + 1)))
                paths.append(path + [(leaf, node_tokens[leaf])])
            else:
                inner = new_node(_round_page(int(rng.integers(inner_range[0], inner_range[1] + 1))))
                grow(path + [(inner, node_tokens[inner])], part, depth + 1)

    per_root = [batch // roots + (1 if i < batch % roots else 0) for i in range(roots)]
    for r in range(roots):
        root = new_node(_round_page(int(rng.integers(root_range[0], root_range[1] + 1))))
        grow([(root, node_tokens[root])], per_root[r], 1)
    assert len(paths) == batch

    alloc = _Alloc(rng, sum(_blocks(t) for t in node_tokens.values()))
    node_blocks = {nid: alloc.take(_blocks(t)) for nid, t in node_tokens.items()}
    order = rng.permutation(batch).tolist()      # requests arrive in shuffled order
    rows, lens = [], []
    for i in order:
        rows.append([b for nid, _ in paths[i] for b in node_blocks[nid]])
        lens.append(sum(t for _, t in paths[i]))
    tree = {"nodes": len(node_tokens), "max_path": max(len(p) for p in paths),
            "node_tokens": [node_tokens[i] for i in range(len(node_tokens))]}
    return _finish(name, heads, kv_heads, d, dtype, seed, lens, rows, alloc, sum(node_tokens.values()), tree)


def make(name: str, seed: int = 0) -> Workload:
    """Builds one of the named configurations (see module docstring)."""
    f16, bf16 = torch.float16, torch.bfloat16
    if name == "c1":
        return shared_prefix("c1", 8, 256, 32, 32, 8, 8, 64, f16, seed)
    if name == "c2":
        return shared_prefix("c2", 64, 2048, 64, 512, 32, 8, 128, bf16, seed)
    if name == "c3":
        return three_level("c3", 128, 1024, 8, 512, 128, 1024, 32, 8, 128, f16, seed)
    if name == "c4":
        return forest("c4", 256, 16, 16, 16, 64, f16, seed)
    if name == "c5a":
        return shared_prefix("c5a", 32, 16384, 256, 2048, 64, 8, 128, bf16, seed)
    if name == "c5b":
        return independent("c5b", 32, 4096, 64, 8, 128, bf16, seed)
    if name == "c5a-prefix":
        return shared_prefix("c5a-prefix", 32, 16384, 16, 16, 64, 8, 128, bf16, seed)
    raise KeyError(f"unknown workload {name!r}")


NAMES = ("c1", "c2", "c3", "c4", "c5a", "c5b")


def oblivious_plan(w: Workload, device) -> dict:
    """Plan of a prefix-oblivious paged decode: one work item per request over its whole block
    list (what `pack_without_prefix` describes), as the table-form arguments of
    `prefix_attn_with_kvcache`. The kernels split long items along KV by themselves."""
    group_rows = w.heads // w.kv_heads
    label = [16 if group_rows <= 16 else 32 if group_rows <= 32 else 64, 128, 1]
    b = w.batch
    ar = torch.arange(b, dtype=torch.int32)
    return dict(
        num_split_per_seq=torch.ones(b, dtype=torch.int32, device=device),
        query_tables=[ar.reshape(b, 1).to(device)],
        block_tables=[w.padded_table().to(device)],
        num_seqs_per_CTAs=[torch.ones(b, dtype=torch.int32, device=device)],
        CTA_ranks=[torch.zeros(b, dtype=torch.int32, device=device)],
        kv_in_CTAs=[torch.tensor(w.seq_lens, dtype=torch.int32, device=device)],
        MNW=[label],
        max_split_per_seq=1, max_seqs_in_CTA=1, max_blocks_in_CTA=max(len(r) for r in w.rows),
        # the hint the prefix-aware plan's launch copies carry (PAT_BUCKET_EVEN), where it serves
        # this plan too: requests of even length that share nothing (with shared pages the rule it
        # switches on makes this plan slower, c2: 64 -> 73 us, and the comparison should be against
        # the faster form)
        bucket_flags=[1 if 4 * min(w.seq_lens) >= 3 * max(w.seq_lens) and w.unique_tokens >= w.total_tokens else 0],
    )
