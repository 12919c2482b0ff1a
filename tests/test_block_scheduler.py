"""Legacy flat schedulers (pat_amd/block_scheduler.py) against what the reference fixes for them:

* `schedule`: plans the reference's own `prefix_attn.block_scheduler.schedule` produced
  (tests/golden/flat_plans.json.gz, written by tests/golden/make_flat_fixtures.py);
* `pack_prefix_blocks`: the worked example in its docstring (block_scheduler.py:18-42) and, on
  sorted batches, the `schedule` fixtures (the two share one sweep). The reference's function
  cannot produce vectors itself: it builds `PackedBox` with keyword arguments the dataclass does
  not have and raises TypeError on entry;
* `pack_without_prefix`: the worked example in its docstring (block_scheduler.py:162-189);
* `schedule_naive`: its closed form (one item per sequence, identity permutation).

Every `schedule` plan is also checked semantically: the items of a sequence hold exactly its row.
"""
import numpy as np
import pytest
import torch

from conftest import load_golden, plan_fields
from pat_amd import block_scheduler as bsched
from pat_amd.data_class import SeqGroup, Sequence


CASES = load_golden("flat_plans.json.gz")["cases"]


def covers(info, rows):
    """Every sequence's items together hold exactly the blocks of its row, each once (items of one
    sequence may sit in different tile buckets, so their order is not checked here)."""
    got = {i: [] for i in range(len(rows))}
    for qt, bt, ns in zip(info.q_tables, info.block_tables, info.num_seqs_per_CTAs):
        for seqs, blocks, n in zip(qt, bt, ns):
            assert len(seqs) == n
            for s in seqs:
                got[s].append(blocks)
    for s, parts in got.items():
        assert len(parts) == info.num_split_per_seq[s]
        assert sorted(b for blocks in parts for b in blocks) == sorted(rows[s])


@pytest.mark.parametrize("idx", range(len(CASES)))
def test_schedule_matches_reference_plans(idx):
    case = CASES[idx]
    info = bsched.schedule(list(case["seq_lens"]), [list(r) for r in case["rows"]], case["block_size"],
                           case["k"], case["tiles"], case["ratio"])
    want = case["plan"]
    got = plan_fields(info)
    for key in want:
        if key in ("reverse_index", "sort_index"):
            assert [int(x) for x in getattr(info, key)] == want[key], key
        else:
            assert got[key] == want[key], key
    order = want["sort_index"]
    covers(info, [case["rows"][i][:-(-case["seq_lens"][i] // case["block_size"])] for i in order])


def test_schedule_permutation_is_lexsort_of_padded_rows():
    rows = [[7, 8], [3, 4, 5], [3, 4], [7], [3, 9]]
    lens = [20, 40, 30, 5, 17]
    info = bsched.schedule(lens, rows, 16, 64, None)
    assert info.sort_index == [2, 1, 4, 3, 0]            # (3,4,0) (3,4,5) (3,9,0) (7,0,0) (7,8,0)
    assert [info.sort_index[i] for i in info.reverse_index] == list(range(5))
    assert info.MNWs == [[64, 128, 4]]


def letters(names):
    return [ord(c) for c in names]


def group_of(rows, b):
    group = SeqGroup(b)
    for r in rows:
        seq = Sequence(b)
        seq.append_blocks(letters(r))
        group.sequences.append(seq)
    return group


def test_pack_prefix_blocks_docstring_example():
    """block_scheduler.py:18-42. The listing there shows sequence 5 as two items [K, L, M] and [Z];
    the code it documents (and `schedule`, the same sweep, in the fixtures) hands a sequence that is
    alone on its current block ALL of its remaining blocks, so [K, L, M, Z] is one item and sequence 5
    has two partial results. Everything else is as listed."""
    b = 16
    rows = ["ABCDEFNOP", "ABCDEFQ", "ABCHIJRST", "ABCHIJU", "ABCHIJVWXY", "ABCKLMZ"]
    group = group_of(rows, b)
    group.is_sorted = True
    box = bsched.pack_prefix_blocks(group, b, k=64)
    assert box.q_table == [0, 0, 2, 5, 0, 1, 2, 3, 4]
    assert box.block_table == [letters(x) for x in ("ABC", "DEF", "HIJ", "KLMZ", "NOP", "Q", "RST", "U", "VWXY")]
    assert box.num_seqs_per_CTA == [6, 2, 3, 1, 1, 1, 1, 1, 1]
    assert box.num_split_per_seq == [3, 3, 3, 3, 3, 2]
    assert box.CTA_rank == [0, 1, 1, 1, 2, 2, 2, 2, 2]
    assert box.kv_in_CTA == [3 * b, 3 * b, 3 * b, 4 * b, 3 * b, b, 3 * b, b, 4 * b]
    assert box.max_split_per_seq == 3
    assert box.max_seqs_in_CTA == 6
    assert box.max_blocks_in_CTA == 4
    assert box.sort_index.tolist() == list(range(6)) and box.reverse_index.tolist() == list(range(6))


@pytest.mark.parametrize("idx", [i for i, c in enumerate(CASES) if len(c["plan"]["MNWs"]) == 1])
def test_pack_prefix_blocks_matches_reference_schedule_on_sorted_batches(idx):
    """On a batch already in lexsort order `pack_prefix_blocks` is the same sweep as `schedule`
    (block_scheduler.py:64-145 vs :401-481) with the first sequence in place of the sequence list."""
    case = CASES[idx]
    want = case["plan"]
    bs = case["block_size"]
    group = SeqGroup(bs)
    for i in want["sort_index"]:
        seq = Sequence(bs)
        n = case["seq_lens"][i]
        row = case["rows"][i][:-(-n // bs)]
        seq.append_blocks(row, n)
        group.sequences.append(seq)
    group.is_sorted = True
    box = bsched.pack_prefix_blocks(group, bs, case["k"])
    assert box.q_table == [q[0] for q in want["q_tables"][0]]
    assert box.block_table == want["block_tables"][0]
    assert box.num_seqs_per_CTA == want["num_seqs_per_CTAs"][0]
    assert box.CTA_rank == want["CTA_ranks"][0]
    assert box.kv_in_CTA == want["kv_in_CTAs"][0]
    assert box.num_split_per_seq == want["num_split_per_seq"]
    assert box.max_split_per_seq == want["max_split_per_seq"]
    assert box.max_blocks_in_CTA == want["max_blocks_in_CTA"]


def test_pack_prefix_blocks_requires_sorted_group():
    group = group_of(["A"], 16)
    group.is_sorted = False
    with pytest.raises(AssertionError):
        bsched.pack_prefix_blocks(group, 16)


def test_pack_without_prefix_docstring_example():
    b = 16
    rows = ["ABCDEFNOP", "ABCDEFQ", "ABCHIJRST", "ABCHIJU", "ABCHIJVWXY", "ABCKLMZ"]
    group = group_of(rows, b)
    box = bsched.pack_without_prefix(group, b)
    assert box.q_table == [0, 1, 2, 3, 4, 5]
    assert box.block_table == [letters(r) for r in rows]
    assert box.num_seqs_per_CTA == [1] * 6 and box.num_split_per_seq == [1] * 6 and box.CTA_rank == [0] * 6
    assert box.kv_in_CTA == [9 * b, 7 * b, 9 * b, 7 * b, 10 * b, 7 * b]
    assert (box.max_split_per_seq, box.max_seqs_in_CTA, box.max_blocks_in_CTA) == (1, 1, 10)


def test_schedule_naive_closed_form():
    rows = [[5, 6, 7], [9], [1, 2]]
    lens = [40, 3, 32]
    info = bsched.schedule_naive(lens, rows, torch.device("cpu"))
    assert info.MNWs == [[64, 128, 4]]
    assert info.q_tables[0].tolist() == [0, 1, 2] and info.q_tables[0].dtype == torch.int32
    assert info.block_tables[0].tolist() == [[5, 6, 7], [9, 0, 0], [1, 2, 0]]
    assert info.num_seqs_per_CTAs[0].tolist() == [1, 1, 1]
    assert info.num_split_per_seq.tolist() == [1, 1, 1]
    assert info.CTA_ranks[0].tolist() == [0, 0, 0]
    assert info.kv_in_CTAs[0].tolist() == lens
    assert (info.max_split_per_seq, info.max_seqs_in_CTA, info.max_blocks_in_CTA) == (1, 1, 3)
    assert info.sort_index.tolist() == [0, 1, 2] and info.reverse_index.tolist() == [0, 1, 2]
    with pytest.raises(AssertionError):
        bsched.schedule_naive(np.array(lens), rows, torch.device("cpu"))
