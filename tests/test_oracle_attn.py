"""Pins the attention oracle (oracle/attn_oracle.py) without the reference: a library routine,
a float64 brute force, and properties the mathematics fixes."""
import math

import pytest
import torch
import torch.nn.functional as F

from oracle import attn_oracle as ao
from oracle.plan_oracle import plan
from pat_amd import workloads


def _rand(shape, seed, dtype=torch.float32):
    g = torch.Generator().manual_seed(seed)
    return torch.randn(shape, generator=g).to(dtype)


@pytest.mark.parametrize("h,hk,d", [(8, 8, 64), (32, 8, 128), (16, 2, 64)])
def test_dense_matches_sdpa(h, hk, d):
    b, s = 3, 77
    q, k, v = _rand((b, 1, h, d), 1), _rand((b, s, hk, d), 2), _rand((b, s, hk, d), 3)
    lens = torch.tensor([77, 5, 40])
    mask = torch.arange(s)[None] < lens[:, None]
    out, _ = ao.attention_ref(q, k, v, mask)
    g = h // hk
    kk = k.repeat_interleave(g, dim=2).transpose(1, 2)       # [b, h, s, d], head order (h_kv g)
    vv = v.repeat_interleave(g, dim=2).transpose(1, 2)
    want = F.scaled_dot_product_attention(q.transpose(1, 2), kk, vv, attn_mask=mask[:, None, None, :])
    assert torch.allclose(out, want.transpose(1, 2), atol=2e-6, rtol=1e-5)


def test_dense_matches_float64_loops():
    b, h, hk, d, s = 2, 4, 2, 8, 11
    q, k, v = _rand((b, 1, h, d), 4), _rand((b, s, hk, d), 5), _rand((b, s, hk, d), 6)
    lens = [11, 6]
    mask = torch.arange(s)[None] < torch.tensor(lens)[:, None]
    out, lse = ao.attention_ref(q, k, v, mask)
    for bi in range(b):
        for hi in range(h):
            kv = hi // (h // hk)                              # query head hi uses kv head hi // g
            sc = [sum(float(q[bi, 0, hi, x]) * float(k[bi, t, kv, x]) for x in range(d)) / math.sqrt(d)
                  for t in range(lens[bi])]
            m = max(sc)
            z = sum(math.exp(x - m) for x in sc)
            assert abs(float(lse[bi, hi]) - (m + math.log(z))) < 1e-5
            for x in range(d):
                o = sum(math.exp(sc[t] - m) / z * float(v[bi, t, kv, x]) for t in range(lens[bi]))
                assert abs(float(out[bi, 0, hi, x]) - o) < 1e-5


def test_uniform_v_returns_v_and_lse_of_equal_keys():
    b, h, hk, d, s = 2, 8, 2, 64, 33
    q = _rand((b, 1, h, d), 7)
    k = _rand((b, 1, hk, d), 8).expand(b, s, hk, d).contiguous()      # all keys equal
    v = _rand((b, 1, hk, d), 9).expand(b, s, hk, d).contiguous()
    out, lse = ao.attention_ref(q, k, v, None)
    g = h // hk
    assert torch.allclose(out[:, 0], v[:, 0].repeat_interleave(g, dim=1), atol=1e-6)
    score = (q[:, 0].reshape(b, hk, g, d) / math.sqrt(d) * k[:, 0][:, :, None, :]).sum(-1).reshape(b, h)
    assert torch.allclose(lse, score + math.log(s), atol=1e-5)


def test_block_permutation_invariance_and_padding_ignored():
    w = workloads.make("c1", seed=5)
    q, k, v = w.tensors("cpu")
    q, k, v = q.float(), k.float(), v.float()
    out, lse = ao.paged_attention_ref(q, k, v, w.rows, w.seq_lens)
    perm = torch.randperm(w.num_blocks, generator=torch.Generator().manual_seed(0))
    inv = torch.empty_like(perm)
    inv[perm] = torch.arange(w.num_blocks)
    k2, v2 = k[perm], v[perm]                                  # block i moves to inv[i]
    rows2 = [[int(inv[x]) for x in r] for r in w.rows]
    out2, lse2 = ao.paged_attention_ref(q, k2, v2, rows2, w.seq_lens)
    assert torch.equal(out, out2) and torch.equal(lse, lse2)
    # tokens past seq_len must not matter
    k3 = k.clone()
    k3[w.rows[0][-1], 10:] = 1e4
    lens = list(w.seq_lens); lens[0] -= 6
    a, _ = ao.paged_attention_ref(q, k, v, w.rows, lens)
    b_, _ = ao.paged_attention_ref(q, k3, v, w.rows, lens)
    assert torch.equal(a[0], b_[0])


@pytest.mark.parametrize("cuts", [[5], [1, 2, 30], [16, 32, 48]])
def test_split_merge_equals_unsplit(cuts):
    r, d, t = 6, 64, 57
    q, k, v = _rand((r, d), 10), _rand((t, d), 11), _rand((t, d), 12)
    scale = 1 / math.sqrt(d)
    whole, lse = ao.partial_ref(q, k, v, scale)
    edges = [0] + cuts + [t]
    parts = [ao.partial_ref(q, k[a:b], v[a:b], scale) for a, b in zip(edges[:-1], edges[1:])]
    merged, lse_m = ao.merge_ref(parts)
    assert torch.allclose(merged, whole, atol=1e-6) and torch.allclose(lse_m, lse, atol=1e-6)


@pytest.mark.parametrize("name", ["c1", "c2"])
def test_plan_execution_equals_dense(name):
    # running the scheduler's plan box by box and merging by rank reproduces dense attention
    w = workloads.make(name, seed=1)
    q, k, v = w.tensors("cpu")
    q, k, v = q.float(), k.float(), v.float()
    p = plan(w.page_size, w.seq_lens, w.rows, None, w.heads // w.kv_heads, w.kv_heads)
    out_p, lse_p = ao.run_plan_ref(p, q, k, v)
    out_d, lse_d = ao.paged_attention_ref(q, k, v, w.rows, w.seq_lens)
    assert torch.allclose(out_p, out_d, atol=2e-5) and torch.allclose(lse_p, lse_d, atol=2e-5)
