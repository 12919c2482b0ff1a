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
    sorted and split by the planner) against the ragged plan of the Python-level `PrefixTree` and a
    launch order derived here: same tables, same order, same parts."""
    import numpy as np
    from pat_amd import PrefixTreeCPP, workloads
    w = workloads.make(name, seed=1)
    t = PrefixTreeCPP(w.page_size)
    t.build_radix_tree(w.seq_lens, w.padded_table())
    t.pack_schedule(None, w.heads // w.kv_heads, w.kv_heads)
    flat = t.kernel_info
    assert flat._flat is not None and flat._flat.dim() == 1
    p = PrefixTree(w.page_size)
    p.build_radix_tree(w.seq_lens, w.rows)
    ref = p.pack_schedule(None, w.heads // w.kv_heads, w.kv_heads)
    assert flat.MNWs == ref.MNWs and flat.max_split_per_seq == ref.max_split_per_seq
    assert flat.max_seqs_in_CTA == ref.max_seqs_in_CTA and flat.max_blocks_in_CTA == ref.max_blocks_in_CTA
    assert flat.num_split_per_seq.tolist() == ref.num_split_per_seq
    assert flat.num_boxes_per_seq.tolist() == ref.num_split_per_seq     # first pack: the counts agree
    assert flat.max_boxes_per_seq == ref.max_split_per_seq

    def padded(rows, width):
        return [list(r) + [0] * (width - len(r)) for r in rows]

    for b in range(len(ref.MNWs)):
        assert flat.q_tables[b].tolist() == padded(ref.q_tables[b], flat.q_tables[b].shape[1])
        assert flat.slot_tables[b].tolist() == padded(ref.slot_tables[b], flat.q_tables[b].shape[1])
        assert flat.block_tables[b].tolist() == padded(ref.block_tables[b], flat.block_tables[b].shape[1])
        assert flat.num_seqs_per_CTAs[b].tolist() == ref.num_seqs_per_CTAs[b]
        assert flat.CTA_ranks[b].tolist() == ref.CTA_ranks[b]
        assert flat.kv_in_CTAs[b].tolist() == ref.kv_in_CTAs[b]
    # launch copies: boxes longest first (stable); a bucket whose wide head (at most a quarter of the
    # boxes, each more than twice as long as any other) is split off, the rest with a narrower table
    launch = flat.launch_tables()
    parts = flat._launch_parts
    at = 0
    for b in range(len(ref.MNWs)):
        kv = np.asarray(ref.kv_in_CTAs[b])
        order = np.argsort(-kv, kind="stable")
        assert flat._launch_order[b].tolist() == order.tolist()
        n = len(kv)
        k = int((kv[order] > kv[order][0] // 2).sum())
        cuts = [0, k, n] if (n >= 4 and 0 < k <= n // 4) else [0, n]
        assert [(lo, hi) for _, lo, hi in parts[b]] == list(zip(cuts[:-1], cuts[1:]))
        for lb, lo, hi in parts[b]:
            assert lb == at
            at += 1
            rows = torch.as_tensor(order[lo:hi].copy())
            assert launch["MNWs"][lb] == ref.MNWs[b]
            lw = launch["block_tables"][lb].shape[1]
            if lo > 0:
                longest = max(len(ref.block_tables[b][i]) for i in order[lo:hi])
                assert lw == min(flat.block_tables[b].shape[1], longest + 8)
            else:
                assert lw == flat.block_tables[b].shape[1]
            assert torch.equal(launch["block_tables"][lb], flat.block_tables[b][rows][:, :lw])
            for key, src in (("q_tables", flat.q_tables), ("slot_tables", flat.slot_tables),
                             ("num_seqs_per_CTAs", flat.num_seqs_per_CTAs), ("CTA_ranks", flat.CTA_ranks),
                             ("kv_in_CTAs", flat.kv_in_CTAs)):
                assert torch.equal(launch[key][lb], src[b][rows]), key
        pos_b, pos_r = flat.launch_position(b)
        for lb, lo, hi in parts[b]:
            assert pos_b[order[lo:hi]].tolist() == [lb] * (hi - lo)
            assert pos_r[order[lo:hi]].tolist() == list(range(hi - lo))
    assert at == len(launch["MNWs"])
    if name == "c4":
        assert max(len(p) for p in parts) == 2      # a bucket with a wide head
    # the device copy is one buffer too and its views line up
    before = [x.clone() for x in launch["kv_in_CTAs"]]
    flat.to_gpu("cpu")
    assert all(torch.equal(a, b) for a, b in zip(flat.launch_tables()["kv_in_CTAs"], before))


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
