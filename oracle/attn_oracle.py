"""CPU restatement of the reference's PyTorch attention oracle, extended to paged KV.

TEST INFRASTRUCTURE ONLY. This is the checker for output parity and the timed CPU
baseline of the benchmark; only tests, the smoke check and the benchmark's CPU leg may
import it. The product path (`pat_amd`) never does.

What it restates (flashserve/PAT tree):
  * `attention_ref` of test/utils.py:7-58 — inputs upcast to fp32, kv heads repeated
    `h -> (h g)` for GQA (:36-37), scores = (q / sqrt(d)) . k (:39-40), key-padding
    positions set to -inf (:43-46), softmax over keys (:47), P.V (:54), output cast
    back to the input dtype (:58).
  * the dense gather of paged KV through the padded block table of
    prefix_attn/utils.py:31-44 (`k_cache_paged[block_table]`, mask = t < seqlen).
  * LSE = logsumexp of the scaled scores, natural log (csrc/softmax.h:169-188), which the
    reference computes on the GPU only; here it comes from torch.logsumexp.
  * the partial/merge algebra of the split kernels (csrc/pat_fwd_kernel.h:389-465):
    LSE = M + ln sum_i e^(LSE_i - M), out = sum_i e^(LSE_i - LSE) O_i.

GQA is evaluated per kv head on a [g, d] x [d, T] product instead of materialising the
repeated K/V (same arithmetic, no 8x copy).

How it is pinned (tests/test_oracle_attn.py): against
torch.nn.functional.scaled_dot_product_attention on the gathered dense KV, against a
float64 triple loop on tiny inputs, and by properties the mathematics fixes — uniform V
returns V, permuting physical block ids changes nothing, any KV split + merge equals
the unsplit result, LSE of identical keys is score + ln(T).
"""
from __future__ import annotations

import math
from typing import Dict, List, Optional, Sequence, Tuple

import torch


def attention_ref(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor,
                  key_padding_mask: Optional[torch.Tensor] = None,
                  scale: Optional[float] = None) -> Tuple[torch.Tensor, torch.Tensor]:
    """Dense reference. q [B, 1, H, d]; k, v [B, S, H_kv, d]; mask [B, S] (True = keep).

    Returns (out [B, 1, H, d] in q's dtype, lse [B, H] float32)."""
    b, sq, h, d = q.shape
    assert sq == 1
    hk = k.shape[2]
    g = h // hk
    # the reference divides by sqrt(d) (test/utils.py:39); an explicit scale multiplies
    qf = q.float() / math.sqrt(d) if scale is None else q.float() * scale
    qf = qf.reshape(b, hk, g, d)                                  # heads ordered (h_kv, g)
    kf, vf = k.float(), v.float()
    scores = torch.einsum("bhgd,bshd->bhgs", qf, kf)              # [B, H_kv, g, S]
    if key_padding_mask is not None:
        scores = scores.masked_fill(~key_padding_mask[:, None, None, :], float("-inf"))
    lse = torch.logsumexp(scores, dim=-1)                         # [B, H_kv, g]
    p = torch.softmax(scores, dim=-1)
    out = torch.einsum("bhgs,bshd->bhgd", p, vf)
    return out.reshape(b, 1, h, d).to(q.dtype), lse.reshape(b, h)


def gather_dense(paged: torch.Tensor, row: Sequence[int]) -> torch.Tensor:
    """[num_blocks, page, H_kv, d] + block ids -> [len(row) * page, H_kv, d]."""
    idx = torch.as_tensor(list(row), dtype=torch.long)
    blk = paged[idx]
    return blk.reshape(-1, paged.shape[2], paged.shape[3])


def paged_attention_ref(q: torch.Tensor, k_paged: torch.Tensor, v_paged: torch.Tensor,
                        rows: Sequence[Sequence[int]], seq_lens: Sequence[int],
                        scale: Optional[float] = None) -> Tuple[torch.Tensor, torch.Tensor]:
    """Reference over a paged cache, one request at a time (bounded memory).

    Returns (out [B, 1, H, d] in q's dtype, lse [B, H] float32)."""
    b, _, h, d = q.shape
    out = torch.empty_like(q)
    lse = torch.empty(b, h, dtype=torch.float32)
    for i in range(b):
        n = int(seq_lens[i])
        kd = gather_dense(k_paged, rows[i])[None]
        vd = gather_dense(v_paged, rows[i])[None]
        mask = (torch.arange(kd.shape[1]) < n)[None]
        o, l = attention_ref(q[i:i + 1], kd, vd, mask, scale)
        out[i], lse[i] = o[0], l[0]
    return out, lse


def partial_ref(q_rows: torch.Tensor, k_tok: torch.Tensor, v_tok: torch.Tensor, scale: float):
    """Attention of rows [R, d] over tokens [T, d] in fp32 -> (O [R, d] normalised, LSE [R])."""
    s = (q_rows.float() * scale) @ k_tok.float().T
    lse = torch.logsumexp(s, dim=-1)
    return torch.softmax(s, dim=-1) @ v_tok.float(), lse


def merge_ref(parts: List[Tuple[torch.Tensor, torch.Tensor]]):
    """LSE-weighted merge of partial results [(O_i [R, d], LSE_i [R])]."""
    lses = torch.stack([l for _, l in parts])                     # [n, R]
    total = torch.logsumexp(lses, dim=0)
    out = sum(torch.exp(l - total)[:, None] * o for o, l in parts)
    return out, total


def run_plan_ref(plan: Dict, q: torch.Tensor, k_paged: torch.Tensor, v_paged: torch.Tensor,
                 scale: Optional[float] = None) -> Tuple[torch.Tensor, torch.Tensor]:
    """Executes a scheduler plan (ragged KernelInfo lists) on the CPU: one partial per box and
    kv head, merged per sequence in CTA_rank order. Checks that every (sequence, rank) slot
    is produced exactly once. Returns (out [B, 1, H, d] in q's dtype, lse [B, H])."""
    b, _, h, d = q.shape
    hk, page = k_paged.shape[2], k_paged.shape[1]
    g = h // hk
    scale = 1.0 / math.sqrt(d) if scale is None else scale
    nsplit = list(plan["num_split_per_seq"])
    slots: List[List[Optional[Tuple[torch.Tensor, torch.Tensor]]]] = [[None] * n for n in nsplit]
    for q_tab, b_tab, n_seqs, ranks, kvs in zip(plan["q_tables"], plan["block_tables"],
                                                plan["num_seqs_per_CTAs"], plan["CTA_ranks"],
                                                plan["kv_in_CTAs"]):
        for seqs, blocks, n, rank, kv in zip(q_tab, b_tab, n_seqs, ranks, kvs):
            seqs = list(seqs)[:n]
            kd = gather_dense(k_paged, blocks)[:kv]               # [kv, H_kv, d]
            vd = gather_dense(v_paged, blocks)[:kv]
            rows = q[seqs, 0].reshape(len(seqs), hk, g, d)        # [n, H_kv, g, d]
            o = torch.empty(len(seqs), hk, g, d)
            l = torch.empty(len(seqs), hk, g)
            for head in range(hk):
                oo, ll = partial_ref(rows[:, head].reshape(-1, d), kd[:, head], vd[:, head], scale)
                o[:, head], l[:, head] = oo.reshape(len(seqs), g, d), ll.reshape(len(seqs), g)
            for j, s in enumerate(seqs):
                assert slots[s][rank] is None, f"sequence {s} rank {rank} produced twice"
                slots[s][rank] = (o[j].reshape(h, d), l[j].reshape(h))
    out = torch.empty_like(q)
    lse = torch.empty(b, h)
    for s in range(b):
        assert all(p is not None for p in slots[s]), f"sequence {s} is missing a partial"
        o, l = merge_ref(slots[s])
        out[s, 0], lse[s] = o.to(q.dtype), l
    return out, lse
