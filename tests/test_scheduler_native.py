"""The C++ scheduler of libpat_amd (through `PrefixTree` / `PrefixTreeCPP`) against the golden
plans of the reference scheduler and against the plan oracle on fresh random batches."""
import random

import pytest
import torch

from conftest import plan_fields, run_plan_case
from oracle.plan_oracle import PlanOracle, pad_rows
from pat_amd import PrefixTree, PrefixTreeCPP
from pat_amd import workloads


def _compare(case, got):
    if "raises" in case:
        assert got.get("raises") == case["raises"], case["name"]
    else:
        assert got.get("plans") == case["plans"], case["name"]


def test_golden_small(golden_small):
    for case in golden_small:
        _compare(case, run_plan_case(PrefixTree, case))


def test_golden_large(golden_large):
    for case in golden_large:
        _compare(case, run_plan_case(PrefixTree, case))


def test_golden_tree_arrays(golden_small):
    for case in golden_small:
        if "tree" not in case:
            continue
        t = PrefixTree(case["block_size"])
        t.build_radix_tree(list(case["seq_lens"]), [list(r) for r in case["rows"]])
        ref = case["tree"]
        assert t.parents == ref["parents"], case["name"]
        assert t.s_values == ref["s_values"], case["name"]
        assert t.lens == ref["lens"], case["name"]
        assert t.seq_indices == ref["seq_indices"], case["name"]
        assert t.block_ids == ref["block_ids"], case["name"]
        kids = t.tree
        assert [list(kids[i].values()) for i in range(t.num_nodes)] == ref["children"], case["name"]


def _random_batch(r: random.Random):
    bs = r.choice([16, 32, 64])
    rows, lens, nxt = [], [], 0
    for _ in range(r.choice([1, 4, 17, 60, 150])):
        row = []
        if rows and r.random() < 0.85:
            base = rows[r.randrange(len(rows))]
            row = list(base[:r.randint(0, len(base))])
        extra = r.randint(0 if row else 1, 25)
        row += list(range(nxt, nxt + extra)); nxt += extra
        rows.append(row)
        lens.append(max(1, len(row) * bs - r.randint(0, bs - 1)))
    return bs, lens, rows


@pytest.mark.parametrize("seed", range(60))
def test_matches_oracle_on_random_batches(seed):
    r = random.Random(7000 + seed)
    bs, lens, rows = _random_batch(r)
    hratio, kvh = r.choice([(1, 8), (2, 8), (4, 8), (8, 8), (1, 32), (8, 1), (4, 64)])
    model = seed % 4 == 1
    naive = seed % 9 == 5
    call = {"kind": "naive", "HRatio": hratio} if naive else \
        {"kind": "pack", "MNWs": None, "HRatio": hratio, "kvHead": kvh, "use_compute_model": model}
    case = {"block_size": bs, "seq_lens": lens, "rows": rows, "calls": [call] * (2 if seed % 11 == 0 else 1)}
    want, got = run_plan_case(PlanOracle, case), run_plan_case(PrefixTree, case)
    assert got.get("raises") == want.get("raises")
    assert got.get("plans") == want.get("plans")


@pytest.mark.parametrize("name", workloads.NAMES)
def test_padded_table_entry_point_matches_rows(name):
    # PrefixTreeCPP takes the zero-padded table + lengths; same plan as the ragged rows
    w = workloads.make(name, seed=3)
    hr = w.heads // w.kv_heads
    t = PrefixTree(w.page_size)
    t.build_radix_tree(w.seq_lens, w.rows)
    ki = t.pack_schedule(None, hr, w.kv_heads)
    c = PrefixTreeCPP(w.page_size)
    c.build_radix_tree(w.seq_lens, w.padded_table())
    c.pack_schedule(None, hr, w.kv_heads)
    info = c.kernel_info
    assert info.MNWs == ki.MNWs
    for i in range(len(ki.MNWs)):
        assert info.q_tables[i].tolist() == pad_rows(ki.q_tables[i])
        assert info.block_tables[i].tolist() == pad_rows(ki.block_tables[i])
        assert info.num_seqs_per_CTAs[i].tolist() == ki.num_seqs_per_CTAs[i]
        assert info.CTA_ranks[i].tolist() == ki.CTA_ranks[i]
        assert info.kv_in_CTAs[i].tolist() == ki.kv_in_CTAs[i]
        assert info.q_tables[i].dtype == torch.int32 and info.block_tables[i].dtype == torch.int32
    assert info.num_split_per_seq.tolist() == ki.num_split_per_seq
    assert (info.max_split_per_seq, info.max_seqs_in_CTA, info.max_blocks_in_CTA) == \
        (ki.max_split_per_seq, ki.max_seqs_in_CTA, ki.max_blocks_in_CTA)


def test_seq_lens_tensor_and_list_agree():
    w = workloads.make("c1")
    a, b = PrefixTreeCPP(16), PrefixTreeCPP(16)
    a.build_radix_tree(w.seq_lens, w.padded_table())
    b.build_radix_tree(torch.tensor(w.seq_lens, dtype=torch.int32), w.padded_table())
    a.pack_schedule(HRatio=1, kvHead=8)
    b.pack_schedule(HRatio=1, kvHead=8)
    assert [t.tolist() for t in a.kernel_info.block_tables] == [t.tolist() for t in b.kernel_info.block_tables]


def test_to_tensor_pads_with_zero():
    t = PrefixTree(16)
    t.build_radix_tree([33, 33, 33], [[0, 1, 5], [0, 2, 6], [3, 4, 7]])
    ki = t.pack_schedule(None, 4, 8)
    ki.to_tensor("cpu")
    assert ki.q_tables[1].tolist() == [[0, 1], [0, 0], [1, 0]]
    assert ki.block_tables[1].tolist() == [[0, 0], [1, 5], [2, 6]]
    assert ki.num_split_per_seq.dtype == torch.int32 and ki.kv_in_CTAs[0].tolist() == [33]


def test_error_mapping():
    t = PrefixTree(16)
    t.build_radix_tree([], [])
    with pytest.raises(ValueError):
        t.pack_schedule()                       # max() of an empty batch
    t = PrefixTree(16)
    t.build_radix_tree([64, 64], [[0, 1, 2, 3], [0, 1, 4, 5]])
    with pytest.raises(KeyError):
        t.pack_schedule([[64, 128, 4], [16, 128, 1]], 1, 8)   # computed bucket not offered
    with pytest.raises(ZeroDivisionError):
        t.pack_schedule(None, 0, 8)
    with pytest.raises(RuntimeError):
        PrefixTree(0)
    c = PrefixTreeCPP(16)
    with pytest.raises(RuntimeError, match="Seq lens list mismatch"):
        c.build_radix_tree([16], torch.zeros(2, 1, dtype=torch.int32))
    with pytest.raises(RuntimeError):
        c.build_radix_tree([64], torch.zeros(1, 2, dtype=torch.int32))   # needs 4 blocks, table has 2
    with pytest.raises(RuntimeError):
        c.build_radix_tree("nope", torch.zeros(1, 2, dtype=torch.int32))


@pytest.mark.parametrize("name", ["c1", "c2", "c3", "c4", "c5a"])
def test_flat_plan_equals_the_per_table_view(name):
    """The one-buffer form of the plan (pat_tree_flat_plan: scheduler-order tables + launch copies,
    sorted and split by the planner) against the per-table view with the launch copies built in
    Python: same tables, same launch order, same parts."""
    from pat_amd import PrefixTreeCPP, workloads
    from pat_amd._prefix_attn import KernelInfo
    w = workloads.make(name, seed=1)
    t = PrefixTreeCPP(w.page_size)
    t.build_radix_tree(w.seq_lens, w.padded_table())
    t.pack_schedule(None, w.heads // w.kv_heads, w.kv_heads)
    flat = t.kernel_info
    assert flat._flat is not None and flat._flat.dim() == 1
    view = KernelInfo._from_view(t._native.plan_view())
    assert flat.MNWs == view.MNWs and flat.max_split_per_seq == view.max_split_per_seq
    assert flat.max_seqs_in_CTA == view.max_seqs_in_CTA and flat.max_blocks_in_CTA == view.max_blocks_in_CTA
    assert torch.equal(flat.num_split_per_seq, view.num_split_per_seq)
    names = ("q_tables", "block_tables", "num_seqs_per_CTAs", "CTA_ranks", "kv_in_CTAs", "slot_tables")
    for key in names:
        assert all(torch.equal(a, b) for a, b in zip(getattr(flat, key), getattr(view, key))), key
    fl, vl = flat.launch_tables(), view.launch_tables()
    assert fl["MNWs"] == vl["MNWs"]
    for key in names:
        assert len(fl[key]) == len(vl[key]) and all(torch.equal(a, b) for a, b in zip(fl[key], vl[key])), key
    assert flat._launch_parts == view._launch_parts
    assert all(torch.equal(a.long(), b) for a, b in zip(flat._launch_order, view._launch_order))
    if name == "c4":
        assert max(len(p) for p in flat._launch_parts) == 2      # a bucket with a wide head
    # the device copy is one buffer too and its views line up
    flat.to_gpu("cpu")
    assert torch.equal(flat.launch_tables()["kv_in_CTAs"][0], vl["kv_in_CTAs"][0])


def test_flat_plan_marks_even_buckets():
    from pat_amd import PrefixTreeCPP, workloads
    flags = {}
    for name in ("c5b", "c3"):
        w = workloads.make(name, seed=0)
        t = PrefixTreeCPP(w.page_size)
        t.build_radix_tree(w.seq_lens, w.padded_table())
        t.pack_schedule(None, w.heads // w.kv_heads, w.kv_heads)
        lt = t.kernel_info.launch_tables()
        flags[name] = lt["flags"]
        for f, kv in zip(lt["flags"], lt["kv_in_CTAs"]):
            assert f == (1 if 4 * int(kv.min()) >= 3 * int(kv.max()) else 0)
    assert flags["c5b"] == [1]          # 32 requests of 4096 tokens
    assert flags["c3"][-1] == 0         # leaves of 128..1024 tokens


def test_repeated_pack_keeps_slots_and_box_counts_consistent():
    # the reference's split counters count on over repeated pack_schedule calls on one tree
    # (prefix_attn/prefix_tree.py:149 resets them only on a rebuild); the ordinals a launch files
    # partial results by, and the box counts it merges, describe the current plan alone
    w = workloads.make("c4", seed=0)
    t = PrefixTreeCPP(w.page_size)
    t.build_radix_tree(w.seq_lens, w.padded_table())
    seen = []
    for _ in range(2):
        t.pack_schedule(None, w.heads // w.kv_heads, w.kv_heads)
        ki = t.kernel_info
        top = torch.zeros(w.batch, dtype=torch.int64)
        count = torch.zeros(w.batch, dtype=torch.int64)
        for q, sl, n in zip(ki.q_tables, ki.slot_tables, ki.num_seqs_per_CTAs):
            for row in range(q.shape[0]):
                k = int(n[row])
                ids, ords = q[row, :k].long(), sl[row, :k].long()
                top[ids] = torch.maximum(top[ids], ords)
                count[ids] += 1
        assert torch.equal(top + 1, ki.num_boxes_per_seq.long())
        assert torch.equal(count, ki.num_boxes_per_seq.long())
        assert ki.max_boxes_per_seq == int(count.max())
        seen.append((ki.num_split_per_seq.clone(), ki.num_boxes_per_seq.clone()))
    assert torch.equal(seen[0][0], seen[0][1])            # first pack: the two counts agree
    assert torch.equal(seen[1][0], 2 * seen[0][0])        # second pack: the reference's counter doubled
    assert torch.equal(seen[1][1], seen[0][1])            # ... the plan's own count did not
