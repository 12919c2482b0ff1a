"""The package keeps the reference's import surface (prefix_attn/__init__.py:10-26)."""
import torch

import pat_amd
import prefix_attn


def test_all_names_importable_from_both_packages():
    names = ["prefix_attn_with_kvcache", "PrefixTree", "PrefixTreeCPP", "AsyncTree", "generate_random_prefix_seqs",
             "generate_random_kv_cache", "generate_tree_seqs", "pack_prefix_blocks", "pack_without_prefix",
             "schedule", "schedule_naive", "PackedBox", "Sequence", "SeqGroup", "KernelInfo"]
    assert sorted(prefix_attn.__all__) == sorted(names)
    for n in names:
        assert getattr(prefix_attn, n) is getattr(pat_amd, n)
    from prefix_attn._prefix_attn import prefix_attn_with_kvcache, PrefixTreeCPP  # noqa: F401
    from prefix_attn.prefix_tree import PrefixTree, AsyncPrefixTreeScheduler, unpad_2d  # noqa: F401
    from prefix_attn.data_class import create_seq_group  # noqa: F401
    from prefix_attn.utils import make_tensor_with_pad  # noqa: F401


def test_generators_shapes():
    group, nblk = prefix_attn.generate_tree_seqs("1,2,4_64,256,32", 32)
    assert nblk == 2 + 2 * 8 + 4 * 1 and len(group) == 4 and group.seqlens == [352] * 4
    rows = group.get_block_ids()
    assert all(len(r) == 11 and r[:2] == [0, 1] for r in rows)
    seqlens, k, v, mask, table, kp, vp = prefix_attn.generate_random_kv_cache(group, nblk, 32, 2, 64, torch.float32, "cpu", 0)
    assert k.shape == (4, 352, 2, 64) and kp.shape == (nblk, 32, 2, 64) and table.dtype == torch.int32
    assert mask.all() and torch.equal(k[0, :32], kp[rows[0][0]])
    g2, n2 = prefix_attn.generate_random_prefix_seqs(100, 400, 6, 2, 0.5, 16, seed=1)
    assert len(g2) == 6 and all(len(s.block_ids) == -(-s.seqlen // 16) for s in g2.sequences)
    assert n2 == len({b for s in g2.sequences for b in s.block_ids})


def test_async_tree_on_cpu_device():
    from pat_amd import workloads
    w = workloads.make("c1")
    t = prefix_attn.AsyncTree(16, w.seq_lens, w.padded_table(), None, 1, 8, torch.device("cpu"))
    info = t.tree.kernel_info
    assert info.max_split_per_seq == 3 and info.MNWs == [[16, 64, 1], [16, 32, 1]]
    bad = prefix_attn.AsyncTree(16, [16], torch.zeros(2, 1, dtype=torch.int32), None, 1, 8, torch.device("cpu"))
    try:
        bad.tree
        raise AssertionError("expected the helper thread's error")
    except RuntimeError as e:
        assert "mismatch" in str(e)


def test_forward_refuses_cpu_tensors():
    from pat_amd import workloads
    w = workloads.make("c1")
    q, k, v = w.tensors("cpu")
    t = prefix_attn.PrefixTreeCPP(16)
    t.build_radix_tree(w.seq_lens, w.padded_table())
    t.pack_schedule(HRatio=1, kvHead=8)
    try:
        prefix_attn.prefix_attn_with_kvcache(q, k, v, t, 0.125, torch.empty_like(q))
        raise AssertionError("expected a device check to fail")
    except RuntimeError as e:
        assert "must be on CUDA" in str(e)


def test_python_plan_sort_for_launch_permutes_rows_only():
    from pat_amd import workloads
    w = workloads.make("c2")
    tree = prefix_attn.PrefixTree(w.page_size)
    tree.build_radix_tree(w.seq_lens, w.rows)
    ki = tree.pack_schedule(MNWs=None, HRatio=w.heads // w.kv_heads, kvHead=w.kv_heads, use_compute_model=False)
    before = [sorted(zip(map(tuple, ki.q_tables[b]), map(tuple, ki.block_tables[b]), ki.num_seqs_per_CTAs[b],
                         ki.CTA_ranks[b], ki.kv_in_CTAs[b])) for b in range(len(ki.MNWs))]
    ki.sort_for_launch()
    after = [sorted(zip(map(tuple, ki.q_tables[b]), map(tuple, ki.block_tables[b]), ki.num_seqs_per_CTAs[b],
                        ki.CTA_ranks[b], ki.kv_in_CTAs[b])) for b in range(len(ki.MNWs))]
    assert before == after                                       # the same items
    assert all(list(kv) == sorted(kv, reverse=True) for kv in ki.kv_in_CTAs)
    ki.to_tensor("cpu")
    try:
        ki.sort_for_launch()
        raise AssertionError("expected the tensor form to be refused")
    except ValueError as e:
        assert "before to_tensor" in str(e)
