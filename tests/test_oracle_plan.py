"""Pins the plan oracle (oracle/plan_oracle.py): hand-traced known answers, closed forms,
structural invariants and the golden plans written by the reference scheduler."""
import math
import random

import pytest

from conftest import plan_fields, run_plan_case
from oracle.plan_oracle import PlanOracle, plan, tile_label


def test_manual_fixture_hand_trace():
    # the reference's manual fixture (test/test.py:233-239), traced by hand through
    # prefix_tree.py: A(q[0,1] blk[0]) B(q[0] blk[1,5]) C(q[1] blk[2,6]) D(q[2] blk[3,4,7])
    p = plan(16, [33, 33, 33], [[0, 1, 5], [0, 2, 6], [3, 4, 7]], None, 4, 8)
    assert p["MNWs"] == [[16, 32, 1], [16, 16, 1]]
    assert p["q_tables"] == [[[2]], [[0, 1], [0], [1]]]
    assert p["block_tables"] == [[[3, 4, 7]], [[0], [1, 5], [2, 6]]]
    assert p["num_seqs_per_CTAs"] == [[1], [2, 1, 1]]
    assert p["CTA_ranks"] == [[0], [0, 1, 1]]
    assert p["kv_in_CTAs"] == [[33], [16, 17, 17]]
    assert p["num_split_per_seq"] == [2, 2, 1]
    assert (p["max_split_per_seq"], p["max_seqs_in_CTA"], p["max_blocks_in_CTA"]) == (2, 2, 3)


def test_shared_prefix_8_hand_trace():
    # 8 requests: 16 shared blocks P0..15 + 2 private; HRatio 1, 8 kv heads. The prefix box is
    # halved once by the balancer (9 boxes < 27) and the halves end up behind the leaves.
    P = list(range(16))
    rows = [P + [16 + 2 * i, 17 + 2 * i] for i in range(8)]
    p = plan(16, [288] * 8, rows, None, 1, 8)
    assert p["MNWs"] == [[16, 64, 1], [16, 32, 1]]
    assert p["q_tables"][0] == [list(range(8)), list(range(8))]
    assert p["block_tables"][0] == [P[8:], P[:8]]
    assert p["CTA_ranks"][0] == [2, 0] and p["kv_in_CTAs"][0] == [128, 128]
    assert p["q_tables"][1] == [[i] for i in range(8)]
    assert p["block_tables"][1] == [[16 + 2 * i, 17 + 2 * i] for i in range(8)]
    assert p["CTA_ranks"][1] == [1] * 8 and p["kv_in_CTAs"][1] == [32] * 8
    assert p["num_split_per_seq"] == [3] * 8 and p["max_split_per_seq"] == 3
    assert p["max_seqs_in_CTA"] == 8 and p["max_blocks_in_CTA"] == 8


@pytest.mark.parametrize("batch,hratio", [(64, 4), (32, 8), (128, 2)])
def test_two_level_closed_form(batch, hratio):
    # B requests under one long shared node, B a multiple of mm = 64 // hratio, enough boxes that
    # the balancer is idle: B/mm prefix boxes of rank 0, then one rank-1 leaf box per request.
    mm = 64 // hratio
    shared = list(range(128))
    rows = [shared + [128 + 4 * i + j for j in range(4)] for i in range(batch)]
    lens = [128 * 16 + 50 + (i % 14) for i in range(batch)]
    p = plan(16, lens, rows, None, hratio, 8)
    boxes = [(q, b, r, kv) for qs, bs, rs, kvs in zip(p["q_tables"], p["block_tables"], p["CTA_ranks"], p["kv_in_CTAs"])
             for q, b, r, kv in zip(qs, bs, rs, kvs)]
    prefix = [x for x in boxes if x[1] == shared]
    assert [x[0] for x in prefix] == [list(range(k * mm, (k + 1) * mm)) for k in range(batch // mm)]
    assert all(x[2] == 0 and x[3] == 2048 for x in prefix)
    leaves = [x for x in boxes if x[1] != shared]
    assert [x[0] for x in leaves] == [[i] for i in range(batch)]
    assert all(x[2] == 1 for x in leaves)
    assert [x[3] for x in leaves] == [l - 2048 for l in lens]
    assert p["num_split_per_seq"] == [2] * batch


def test_three_level_children_merge_when_full_tiles():
    # root + 8 mids with exactly mm = 16 requests each: every mid merges into the root's KV
    # (no tile is saved by splitting), so no box sits on the root alone.
    root, nxt = list(range(64)), 64
    rows, lens = [], []
    for m in range(8):
        mid = list(range(nxt, nxt + 32)); nxt += 32
        for _ in range(16):
            rows.append(root + mid + list(range(nxt, nxt + 10))); nxt += 10
            lens.append((64 + 32 + 10) * 16)
    p = plan(16, lens, rows, None, 4, 8)
    big = [(q, b) for qs, bs in zip(p["q_tables"], p["block_tables"]) for q, b in zip(qs, bs) if len(q) == 16]
    assert len(big) == 8
    for m, (q, b) in enumerate(big):
        assert q == list(range(16 * m, 16 * m + 16)) and b[:64] == root and len(b) == 96
    assert p["num_split_per_seq"] == [2] * 128


def test_no_sharing_one_box_per_request():
    rows = [list(range(256 * i, 256 * (i + 1))) for i in range(32)]
    p = plan(16, [4096] * 32, rows, None, 8, 8)
    assert p["MNWs"] == [[16, 128, 1]]
    assert p["q_tables"] == [[[i] for i in range(32)]]
    assert p["block_tables"] == [rows]
    assert p["CTA_ranks"] == [[0] * 32] and p["max_split_per_seq"] == 1


def test_tile_label_table():
    assert tile_label(64, 2048) == (64, 128, 4)
    assert tile_label(33, 16) == (64, 32, 4)      # M = 64 forces N >= 32
    assert tile_label(32, 31) == (32, 16, 2)
    assert tile_label(17, 63) == (32, 32, 2)
    assert tile_label(16, 128) == (16, 64, 1)     # 128 still maps to N = 64
    assert tile_label(4, 129) == (16, 128, 1)
    assert tile_label(1, 32) == (16, 32, 1)


def _check_invariants(block_size, lens, rows, p, hratio):
    """Every sequence's boxes tile its block-table row exactly once, there are num_split of them
    and their ranks stay below max_split. (Row order need not be rank order: the balancer gives
    the back half of a cut box the next free rank of the box's FIRST sequence. For the same
    reason ranks of one sequence can repeat when a cut box packs sequences with different
    numbers of earlier boxes, and can reach past that sequence's own num_split - hazards of the
    reference scheduler that a bit-exact plan keeps.)"""
    per_seq = {i: [] for i in range(len(rows))}
    for mnw, qs, bs, ns, rs, kvs in zip(p["MNWs"], p["q_tables"], p["block_tables"], p["num_seqs_per_CTAs"],
                                        p["CTA_ranks"], p["kv_in_CTAs"]):
        for q, b, n, r, kv in zip(qs, bs, ns, rs, kvs):
            assert n == len(q) and len(q) * hratio <= 64
            assert tuple(mnw) == tile_label(len(q) * hratio, kv)
            assert (len(b) - 1) * block_size < kv <= len(b) * block_size
            for s in q:
                per_seq[s].append((b, kv, r))
    for s, parts in per_seq.items():
        assert len(parts) == p["num_split_per_seq"][s]
        assert all(0 <= r < p["max_split_per_seq"] for _, _, r in parts)
        in_row_order = sorted(parts, key=lambda part: rows[s].index(part[0][0]))
        assert [x for b, _, _ in in_row_order for x in b] == rows[s]
        assert sum(kv for _, kv, _ in parts) == lens[s]


@pytest.mark.parametrize("seed", range(25))
def test_invariants_random_forests(seed):
    r = random.Random(seed)
    bs = r.choice([16, 32])
    rows, lens, nxt = [], [], 0
    for _ in range(r.choice([3, 10, 40, 90])):
        row = []
        if rows and r.random() < 0.85:
            base = rows[r.randrange(len(rows))]
            row = list(base[:r.randint(0, len(base) - 1)])     # never a whole earlier row
        extra = r.randint(1, 30)
        row += list(range(nxt, nxt + extra)); nxt += extra
        rows.append(row)
        lens.append(len(row) * bs - r.randint(0, bs - 1))
    hratio, kvh = r.choice([(1, 8), (4, 8), (8, 8), (2, 16)])
    p = plan(bs, lens, rows, None, hratio, kvh)
    _check_invariants(bs, lens, rows, p, hratio)


def test_golden_small(golden_small):
    for case in golden_small:
        got = run_plan_case(PlanOracle, case)
        if "raises" in case:
            assert got.get("raises") == case["raises"], case["name"]
        else:
            assert got["plans"] == case["plans"], case["name"]


def test_golden_large(golden_large):
    for case in golden_large:
        got = run_plan_case(PlanOracle, case)
        assert got.get("plans") == case["plans"], case["name"]


def test_golden_tree_structure(golden_small):
    for case in golden_small:
        if "tree" not in case:
            continue
        o = PlanOracle(case["block_size"])
        o.build_radix_tree(list(case["seq_lens"]), [list(r) for r in case["rows"]])
        t = case["tree"]
        assert [n.parent for n in o.nodes] == t["parents"], case["name"]
        assert [n.s for n in o.nodes] == t["s_values"], case["name"]
        assert [n.tokens for n in o.nodes] == t["lens"], case["name"]
        assert [n.seqs for n in o.nodes] == t["seq_indices"], case["name"]
        assert [n.blocks for n in o.nodes] == t["block_ids"], case["name"]
        assert [list(n.kids.values()) for n in o.nodes] == t["children"], case["name"]
