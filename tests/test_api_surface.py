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


def test_extension_is_compiled_and_keeps_the_reference_signatures():
    # the reference's module is a compiled torch extension (csrc/bindings.cpp:74-158); so is this one
    from pat_amd import _prefix_attn as ext
    assert ext.__file__.endswith(".so")
    assert prefix_attn._prefix_attn is ext
    import re
    doc = " ".join(ext.prefix_attn_with_kvcache.__doc__.split())
    one, two = re.findall(r"\d\. prefix_attn_with_kvcache\((.*?)\) -> None", doc)
    names = lambda sig: re.findall(r"(?:^|, )(\*|\w+)(?=:|,)", sig)
    # argument names and order of csrc/bindings.cpp:76-95 and :148-157; keyword-only extras after "*"
    assert names(one) == ["q", "k_cache_paged", "v_cache_paged", "num_split_per_seq", "query_tables", "block_tables",
                          "num_seqs_per_CTAs", "CTA_ranks", "kv_in_CTAs", "MNW", "max_split_per_seq",
                          "max_seqs_in_CTA", "max_blocks_in_CTA", "softmax_scale", "out", "timing_", "*",
                          "softmax_lse", "slot_tables", "bucket_flags"]
    assert "timing_: object = None" in one
    assert names(two) == ["q", "k_cache_paged", "v_cache_paged", "tree", "softmax_scale", "out", "*", "softmax_lse"]
    t = ext.PrefixTreeCPP(block_size=16)
    assert t.block_size == 16 and t.kernel_info.MNWs == []
    sig = " ".join(ext.PrefixTreeCPP.pack_schedule.__doc__.split())
    assert re.search(r"MNWs: object = None, HRatio: [\w.]+ = 1, kvHead: [\w.]+ = 8, use_compute_model: bool = False", sig), sig


def test_extension_maps_planner_errors_to_python_exceptions():
    import pytest
    from pat_amd import PrefixTreeCPP
    t = PrefixTreeCPP(16)
    t.build_radix_tree([64, 64], torch.tensor([[0, 1, 2, 3], [0, 1, 4, 5]], dtype=torch.int32))
    with pytest.raises(KeyError):
        t.pack_schedule([[64, 128, 4], [16, 128, 1]], 1, 8)      # computed bucket not offered
    with pytest.raises(ZeroDivisionError):
        t.pack_schedule(None, 0, 8)
    empty = PrefixTreeCPP(16)
    empty.build_radix_tree([], torch.zeros(0, 1, dtype=torch.int32))
    with pytest.raises(ValueError):
        empty.pack_schedule(None, 1, 8)                          # max() of an empty batch
    t.pack_schedule([], 1, 8)                                     # an empty list selects the default buckets
    assert t.kernel_info.max_split_per_seq >= 1
    with pytest.raises(TypeError):
        prefix_attn.prefix_attn_with_kvcache(torch.zeros(1), torch.zeros(1), torch.zeros(1), "not a tree", 1.0,
                                             torch.zeros(1))


def test_planner_calls_release_the_gil():
    # build_radix_tree / pack_schedule run without the GIL (csrc/bindings.cpp:124,138): a Python
    # thread makes progress while another one plans a large batch
    import threading
    import time
    from pat_amd import PrefixTreeCPP
    n, width = 4096, 512
    table = torch.arange(n * width, dtype=torch.int32).view(n, width)
    table[:, :256] = torch.arange(256, dtype=torch.int32)          # a shared prefix
    lens = [width * 16] * n
    ticks, stop = [0], threading.Event()

    def spin():
        while not stop.is_set():
            ticks[0] += 1
            time.sleep(0)

    th = threading.Thread(target=spin)
    th.start()
    try:
        time.sleep(0.02)
        before, t0 = ticks[0], time.perf_counter()
        tree = PrefixTreeCPP(16)
        tree.build_radix_tree(lens, table)
        tree.pack_schedule(None, 4, 8)
        native_s, during = time.perf_counter() - t0, ticks[0] - before
    finally:
        stop.set()
        th.join()
    assert tree.kernel_info.num_split_per_seq.numel() == n
    # with the GIL held throughout, the other thread would get at most a few switches
    assert during > 20 or native_s < 0.005, (during, native_s)


def test_plan_tensors_keep_version_counters_under_inference_mode():
    """A plan packed under torch.inference_mode() is held in ordinary tensors: the binding tells
    in-place edits of a plan (DecodePlan.advance_step) by their version counters, which inference
    tensors do not have."""
    import torch
    from pat_amd import PrefixTreeCPP, workloads
    w = workloads.make("c1", seed=0)
    with torch.inference_mode():
        tree = PrefixTreeCPP(w.page_size)
        tree.build_radix_tree(w.seq_lens, w.padded_table())
        tree.pack_schedule(None, w.heads // w.kv_heads, w.kv_heads)
        flat = tree.kernel_info._flat
        assert flat is not None and not flat.is_inference()
        before = flat._version
        tree.kernel_info.kv_in_CTAs[0][0] += 1      # a view of the one buffer
        assert flat._version > before
    assert not tree.kernel_info.kv_in_CTAs[0].is_inference()


def _packed(spec: str, heads: int, kv_heads: int, page: int = 32):
    import random
    from pat_amd import PrefixTreeCPP, generate_tree_seqs
    random.seed(0)
    group, _ = generate_tree_seqs(spec, page)
    rows = group.get_block_ids()
    width = max(len(r) for r in rows)
    table = torch.zeros(len(rows), width, dtype=torch.int32)
    for i, r in enumerate(rows):
        table[i, :len(r)] = torch.tensor(r, dtype=torch.int32)
    tree = PrefixTreeCPP(page)
    tree.build_radix_tree(list(group.seqlens), table)
    tree.pack_schedule(None, heads // kv_heads, kv_heads)
    return tree.kernel_info, list(group.seqlens), rows


def test_one_work_item_per_request_where_sharing_saves_little():
    """The planner hands out the one-work-item-per-request tables (the launch the drop-in call then
    makes) for batches whose shared pages are cheaper to re-read from L2 than the plan's second kernel
    and partial rows are to pay, and for those only; sizes are of measured cases (plan / one item per
    request, us per call): 64 x (256 + 32) tokens at 64/8 heads 13.4 / 10.8, 8 x (1024 + 1024) at 32/8
    16.6 / 14.6, 128 x (256 + 32) at 16/2 13.0 / 7.9; 128 x (256 + 32) at 32/8 15.2 / 17.9,
    4 x (4096 + 32) at 32/8 13.3 / 15.3, 64 x (2048 + 32) at 32/8 15.8 / 25.4."""
    for spec, heads, kv_heads, expect in (("1,64_256,32", 64, 8, 2048), ("1,8_1024,1024", 32, 8, 2**31 - 1),
                                          ("1,128_256,32", 16, 2, 2**31 - 1), ("1,128_256,32", 32, 8, None),
                                          ("1,4_4096,32", 32, 8, None), ("1,64_1024,32", 32, 8, None),
                                          ("1,1024_2048,32", 64, 8, None)):
        info, lens, rows = _packed(spec, heads, kv_heads)
        whole = info.whole_sequence_tables()
        assert (whole is not None) == (expect is not None), spec
        if whole is None:
            continue
        assert whole["longest_allowed"] == expect, spec
        assert whole["max_split_per_seq"] == 1 and whole["MNWs"] == [[16, 128, 1]]
        assert whole["kv_in_CTAs"][0].tolist() == lens
        assert whole["q_tables"][0][:, 0].tolist() == list(range(len(lens)))
        assert whole["block_tables"][0].shape[1] == max(len(r) for r in rows)     # (the caller's table has no spare columns)
        for i, r in enumerate(rows):
            assert whole["block_tables"][0][i, :len(r)].tolist() == r
    # no request in two boxes: the plan has nothing to merge either, and is launched as it is
    info, _, _ = _packed("600_64", 32, 8)
    assert info.max_split_per_seq == 1 and info.whole_sequence_tables() is None


def test_launch_choice_can_be_forced(monkeypatch):
    """PAT_WHOLE_SEQUENCES, read when a plan is packed: 0 keeps every batch on the plan, 1 gives every batch
    the one-work-item-per-request tables."""
    monkeypatch.setenv("PAT_WHOLE_SEQUENCES", "0")
    info, _, _ = _packed("1,8_256,32", 8, 8)                 # a small batch: one item per request when left alone
    assert info.whole_sequence_tables() is None
    monkeypatch.setenv("PAT_WHOLE_SEQUENCES", "1")
    info, lens, _ = _packed("1,64_2048,256", 32, 8)          # heavy sharing: the plan when left alone
    whole = info.whole_sequence_tables()
    assert whole is not None and whole["kv_in_CTAs"][0].tolist() == lens
    monkeypatch.delenv("PAT_WHOLE_SEQUENCES")
    assert _packed("1,8_256,32", 8, 8)[0].whole_sequence_tables() is not None
    assert _packed("1,64_2048,256", 32, 8)[0].whole_sequence_tables() is None
