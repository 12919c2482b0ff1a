"""Edits of a built radix tree between decode steps (pat_tree_append / _remove / _grow) against a
fresh build of the edited batch: the tree itself (nodes, child order, sequence lists, token counts)
and the plans packed from it must be identical, through the ctypes face and through the extension.
The golden planner (the plan oracle) checks the fresh build's plan on the way."""
import random

import pytest
import torch

from oracle.plan_oracle import PlanOracle
from pat_amd import PrefixTree, PrefixTreeCPP
from conftest import plan_fields

PAGE = 16


def canonical(tree: PrefixTree):
    """The tree from its root: per node (sequences, tokens, sequence ids, blocks, children in order);
    node numbers, which depend on the history of a tree, do not appear."""
    nodes = tree._nodes()

    def walk(i):
        n = nodes[i]
        kids = [n.child_ids[k] for k in range(n.num_children)]
        return (n.num_seqs if i else None, n.num_tokens, tuple(n.seq_ids[k] for k in range(n.num_seq_ids)),
                tuple(n.block_ids[k] for k in range(n.num_blocks)), tuple(walk(c) for c in kids))

    return walk(0)


class Batch:
    """A decode batch over a paged cache with prefix sharing: requests share whole (full) blocks only."""

    def __init__(self, rng):
        self.rng, self.rows, self.lens, self.next_block = rng, [], [], 0

    def fresh(self, n):
        out = list(range(self.next_block, self.next_block + n))
        self.next_block += n
        return out

    def new_request(self):
        rng = self.rng
        shared = []
        if self.rows and rng.random() < 0.8:
            donor = rng.randrange(len(self.rows))
            full = self.lens[donor] // PAGE            # blocks of the donor that are full
            if full:
                shared = self.rows[donor][:rng.randint(1, full)]
        if shared and rng.random() < 0.15:
            own_tokens = 0                             # ends exactly where the shared blocks end
        else:
            own_tokens = rng.randint(1, 5 * PAGE)
        blocks = shared + self.fresh(-(-own_tokens // PAGE))
        return len(shared) * PAGE + own_tokens, blocks

    def table(self):
        width = max(len(r) for r in self.rows)
        t = torch.zeros(len(self.rows), width, dtype=torch.int32)
        for i, r in enumerate(self.rows):
            t[i, :len(r)] = torch.tensor(r, dtype=torch.int32)
        return t


def check_same(inc: PrefixTree, b: Batch, step, pack):
    ref = PrefixTree(PAGE)
    ref.build_radix_tree(list(b.lens), [list(r) for r in b.rows])
    assert canonical(inc) == canonical(ref), f"step {step}: trees differ"
    if pack:
        hratio, kv_heads = pack

        def plan_of(t):
            # (a request that ends on a node it shares leaves the reference's packer a box without
            # sequences on some trees: IndexError there, and here, for both trees alike)
            try:
                return plan_fields(t.pack_schedule(None, hratio, kv_heads))
            except IndexError as exc:
                return f"IndexError: {exc}"

        got, want = plan_of(inc), plan_of(ref)
        assert got == want, f"step {step}: plans differ"
        gold = PlanOracle(PAGE)
        gold.build_radix_tree(list(b.lens), [list(r) for r in b.rows])
        assert plan_of(gold) == want, f"step {step}: fresh plan differs from the golden planner's"


@pytest.mark.parametrize("seed", range(6))
def test_random_joins_leaves_and_growth_match_a_fresh_build(seed):
    rng = random.Random(seed)
    b = Batch(rng)
    for _ in range(rng.randint(1, 24)):
        n, blocks = b.new_request()
        b.lens.append(n)
        b.rows.append(blocks)
    inc = PrefixTree(PAGE)
    inc.build_radix_tree(list(b.lens), [list(r) for r in b.rows])
    heads = [(1, 8), (4, 8), (8, 8), (2, 4)]
    for step in range(120):
        op = rng.random()
        if op < 0.3 or len(b.rows) <= 1:
            n, blocks = b.new_request()
            row = inc.append_sequence(n, blocks)
            b.lens.append(n)
            b.rows.append(blocks)
            assert row == len(b.rows) - 1
        elif op < 0.55:
            i = rng.randrange(len(b.rows))
            inc.remove_sequence(i)
            del b.rows[i], b.lens[i]
        else:
            i = rng.randrange(len(b.rows))
            more_tokens = rng.choice([1, 1, 1, 2, PAGE, 3 * PAGE + 5])
            new_len = b.lens[i] + more_tokens
            more = b.fresh(-(-new_len // PAGE) - len(b.rows[i]))
            inc.grow_sequence(i, new_len, more)
            b.lens[i] = new_len
            b.rows[i] = b.rows[i] + more
        check_same(inc, b, step, heads[step % len(heads)] if step % 3 == 0 else None)


def test_a_decode_loop_on_the_headline_batch():
    """Every request of the headline batch grows a token per step, one leaves and one joins every
    fifth step: the edited tree's plan equals the fresh one at every step."""
    from pat_amd import workloads
    w = workloads.make("c2", seed=1)
    rows, lens = [list(r) for r in w.rows], list(w.seq_lens)
    nxt = w.num_blocks
    inc = PrefixTree(w.page_size)
    inc.build_radix_tree(list(lens), [list(r) for r in rows])
    prefix = 2048 // w.page_size
    b = Batch(random.Random(0))
    for step in range(1, 31):
        for i in range(len(rows)):
            more = []
            if lens[i] % w.page_size == 0:
                more = [nxt]
                nxt += 1
            lens[i] += 1
            rows[i] = rows[i] + more
            inc.grow_sequence(i, lens[i], more)
        if step % 5 == 0:
            i = (7 * step) % len(rows)
            inc.remove_sequence(i)
            del rows[i], lens[i]
            fresh = 64 + (37 * step) % 448
            blocks = rows[0][:prefix] + list(range(nxt, nxt + -(-fresh // w.page_size)))
            nxt += -(-fresh // w.page_size)
            inc.append_sequence(prefix * w.page_size + fresh, blocks)
            rows.append(blocks)
            lens.append(prefix * w.page_size + fresh)
        b.rows, b.lens = rows, lens
        check_same(inc, b, step, (w.heads // w.kv_heads, w.kv_heads))


def test_growth_only_a_fresh_build_can_place_is_refused():
    t = PrefixTree(PAGE)
    t.build_radix_tree([32, 48], [[1, 2], [1, 2, 3]])      # row 0 ends on the node it shares with row 1
    before = canonical(t)
    with pytest.raises(ValueError, match="another one holds"):
        t.grow_sequence(0, 40, [3])                        # into the block row 1 holds
    assert canonical(t) == before
    t2 = PrefixTree(PAGE)
    t2.build_radix_tree([20, 40], [[1, 2], [1, 2, 3]])     # row 0's last block is shared and not full
    with pytest.raises(ValueError, match="inside a block it shares"):
        t2.grow_sequence(0, 24, [])
    with pytest.raises(IndexError):
        t.remove_sequence(5)
    t.grow_sequence(0, 40, [9])                            # a block of its own: a new leaf, ahead of row 1's
    ref = PrefixTree(PAGE)
    ref.build_radix_tree([40, 48], [[1, 2, 9], [1, 2, 3]])
    assert canonical(t) == canonical(ref)


def test_extension_tree_edits_match_a_fresh_build():
    """The same through PrefixTreeCPP: plan tables, and the whole-sequence tables of a small batch
    (which are made from the extension's own copy of the batch), equal those of a fresh tree."""
    rng = random.Random(3)
    b = Batch(rng)
    for _ in range(6):
        n, blocks = b.new_request()
        b.lens.append(n)
        b.rows.append(blocks)
    inc = PrefixTreeCPP(PAGE)
    caller_table = b.table()
    kept = caller_table.clone()
    inc.build_radix_tree(list(b.lens), caller_table)
    for step in range(40):
        op = rng.random()
        if op < 0.3 or len(b.rows) <= 2:
            n, blocks = b.new_request()
            assert inc.append_sequence(n, blocks) == len(b.rows)
            b.lens.append(n)
            b.rows.append(blocks)
        elif op < 0.5:
            i = rng.randrange(len(b.rows))
            inc.remove_sequence(i)
            del b.rows[i], b.lens[i]
        else:
            i = rng.randrange(len(b.rows))
            new_len = b.lens[i] + rng.choice([1, 1, 2, PAGE + 3])
            more = b.fresh(-(-new_len // PAGE) - len(b.rows[i]))
            inc.grow_sequence(i, new_len, more)
            b.lens[i], b.rows[i] = new_len, b.rows[i] + more
        ref = PrefixTreeCPP(PAGE)
        ref.build_radix_tree(list(b.lens), b.table())
        inc.pack_schedule(None, 4, 8)
        ref.pack_schedule(None, 4, 8)
        gi, ri = inc.kernel_info, ref.kernel_info
        assert torch.equal(gi.num_split_per_seq, ri.num_split_per_seq), step
        assert [list(m) for m in gi.MNWs] == [list(m) for m in ri.MNWs], step
        for name in ("q_tables", "num_seqs_per_CTAs", "CTA_ranks", "kv_in_CTAs"):
            for x, y in zip(getattr(gi, name), getattr(ri, name)):
                assert torch.equal(x, y), (step, name)
        for x, y in zip(gi.block_tables, ri.block_tables):
            assert x.shape[0] == y.shape[0] and torch.equal(x[:, :min(x.shape[1], y.shape[1])], y[:, :min(x.shape[1], y.shape[1])]), step
        wi, wr = gi.whole_sequence_tables(), ri.whole_sequence_tables()
        assert (wi is None) == (wr is None), step
        if wi is not None:
            assert torch.equal(wi["kv_in_CTAs"][0], wr["kv_in_CTAs"][0]), step
            for r in range(len(b.rows)):
                nb = -(-b.lens[r] // PAGE)
                assert wi["block_tables"][0][r, :nb].tolist() == b.rows[r], (step, r)
    assert torch.equal(caller_table, kept), "the caller's block table was written to"


def test_extension_advance_grows_every_row_or_rebuilds():
    from pat_amd import workloads
    w = workloads.make("c3", seed=2)
    rows, lens = [list(r) for r in w.rows], list(w.seq_lens)
    nxt = w.num_blocks
    b = Batch(random.Random(0))
    inc = PrefixTreeCPP(w.page_size)
    b.rows, b.lens = rows, lens
    inc.build_radix_tree(list(lens), b.table())
    for step in range(20):
        for i in range(len(rows)):
            if lens[i] % w.page_size == 0:
                rows[i] = rows[i] + [nxt]
                nxt += 1
            lens[i] += 1
        assert inc.advance(list(lens), b.table()) is True
        ref = PrefixTreeCPP(w.page_size)
        ref.build_radix_tree(list(lens), b.table())
        inc.pack_schedule(None, w.heads // w.kv_heads, w.kv_heads)
        ref.pack_schedule(None, w.heads // w.kv_heads, w.kv_heads)
        for name in ("q_tables", "num_seqs_per_CTAs", "CTA_ranks", "kv_in_CTAs", "block_tables"):
            for x, y in zip(getattr(inc.kernel_info, name), getattr(ref.kernel_info, name)):
                assert torch.equal(x, y), (step, name)
    # a row that shrank cannot be grown: the call builds the tree afresh and says so
    lens[0] -= 1
    assert inc.advance(list(lens), b.table()) is False
    ref = PrefixTreeCPP(w.page_size)
    ref.build_radix_tree(list(lens), b.table())
    inc.pack_schedule(None, 4, 8)
    ref.pack_schedule(None, 4, 8)
    assert all(torch.equal(x, y) for x, y in zip(inc.kernel_info.kv_in_CTAs, ref.kernel_info.kv_in_CTAs))
