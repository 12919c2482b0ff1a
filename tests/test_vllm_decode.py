"""Decode branch of the vLLM backend (pat_amd/vllm_decode.py) driven by a stand-in for vLLM's
AttentionMetadata: plan construction on the CPU, attention through vLLM's cache layout on the GPU."""
import math
from types import SimpleNamespace

import pytest
import torch

from oracle import attn_oracle as ao
from pat_amd import PrefixTree, workloads
from pat_amd.vllm_decode import DecodePlan, decode_attention
from conftest import plan_fields


def fake_metadata(w, device, num_prefills=0):
    """What the backend's metadata holds for a step with `num_prefills` prompt rows ahead of the
    decode requests of workload w."""
    pad = torch.zeros(num_prefills, w.padded_table().shape[1], dtype=torch.int32)
    table_cpu = torch.cat([pad, w.padded_table()])
    return SimpleNamespace(num_prefills=num_prefills, num_decode_tokens=w.batch,
                           seq_lens=[7] * num_prefills + list(w.seq_lens),
                           block_tables=table_cpu.to(device), block_tables_cpu=table_cpu,
                           block_size=w.page_size, nheads=w.heads, nheads_kv=w.kv_heads, max_decode_query_len=1)


def test_decode_plan_drops_prefill_rows_and_matches_scheduler():
    w = workloads.make("c1", seed=3)
    plan = DecodePlan.from_metadata(fake_metadata(w, torch.device("cpu"), num_prefills=2))
    assert plan.num_decode_tokens == w.batch and plan.seq_lens == list(w.seq_lens)
    assert plan.block_tables.shape[0] == w.batch
    ref = PrefixTree(w.page_size)
    ref.build_radix_tree(w.seq_lens, w.rows)
    want = plan_fields(ref.pack_schedule(MNWs=None, HRatio=w.heads // w.kv_heads, kvHead=w.kv_heads))
    got = plan.tree.tree.kernel_info
    assert [list(m) for m in got.MNWs] == want["MNWs"]
    assert got.num_split_per_seq.tolist() == want["num_split_per_seq"]
    assert [t.tolist() for t in got.kv_in_CTAs] == want["kv_in_CTAs"]


def test_no_decode_tokens_no_plan():
    meta = SimpleNamespace(num_decode_tokens=0)
    assert DecodePlan.from_metadata(meta) is None


def test_variable_length_decode_queries_are_refused():
    w = workloads.make("c1", seed=3)
    plan = DecodePlan.from_metadata(fake_metadata(w, torch.device("cpu")))
    plan.max_decode_query_len = 2
    with pytest.raises(AssertionError, match="Speculative decoding"):
        decode_attention(torch.zeros(w.batch, w.heads, w.head_dim), torch.zeros(2, 1, 16, w.kv_heads, w.head_dim),
                         plan, 1.0, torch.zeros(w.batch, w.heads, w.head_dim))


@pytest.mark.gpu
@pytest.mark.parametrize("name", ["c1", "c2"])
def test_decode_attention_through_vllm_cache_layout(name):
    print(f"[case] vLLM decode branch {name}", flush=True)
    dev = torch.device("cuda:0")
    w = workloads.make(name, seed=4)
    q, k, v = w.tensors(dev)
    kv_cache = torch.stack([k, v])                       # [2, blocks, page, h_kv, d]
    plan = DecodePlan.from_metadata(fake_metadata(w, dev, num_prefills=1))
    query = q.squeeze(1).contiguous()                    # [B, N, d]
    output = torch.full_like(query, float("nan"))
    for _ in range(2):                                   # every layer of a step reuses the plan
        decode_attention(query, kv_cache, plan, 1.0 / math.sqrt(w.head_dim), output)
    torch.cuda.synchronize()
    ref, _ = ao.paged_attention_ref(q.cpu(), k.cpu(), v.cpu(), w.rows, w.seq_lens)
    err = (output.unsqueeze(1).float().cpu() - ref.float()).abs().max().item()
    tol = 2e-3 if w.dtype == torch.float16 else 1.6e-2
    print(f"[parity] vLLM decode {name}: max|out - ref| = {err:.3e} (tol {tol:.1e})", flush=True)
    assert err <= tol


@pytest.mark.gpu
def test_plan_built_on_the_helper_thread_serves_another_stream():
    # the helper thread uploads the plan on a stream of its own and returns when the copy is done:
    # a consumer that runs on a non-default stream right away must see the whole plan
    print("[case] vLLM decode branch on a side stream", flush=True)
    dev = torch.device("cuda:0")
    w = workloads.make("c2", seed=8)
    q, k, v = w.tensors(dev)
    kv_cache = torch.stack([k, v])
    query = q.squeeze(1).contiguous()
    output = torch.full_like(query, float("nan"))
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())        # the inputs were made on the current stream
    for _ in range(3):                                   # a fresh plan each time, used at once
        plan = DecodePlan.from_metadata(fake_metadata(w, dev))
        with torch.cuda.stream(side):
            decode_attention(query, kv_cache, plan, 1.0 / math.sqrt(w.head_dim), output)
    side.synchronize()
    ref, _ = ao.paged_attention_ref(q.cpu(), k.cpu(), v.cpu(), w.rows, w.seq_lens)
    err = (output.unsqueeze(1).float().cpu() - ref.float()).abs().max().item()
    print(f"[parity] side stream: max|out - ref| = {err:.3e}", flush=True)
    assert err <= 1.6e-2


def _grown(w, steps, spare_blocks):
    """Block table (CPU, padded) and lengths of workload w after `steps` more tokens per request; new
    blocks come from `spare_blocks` in request order."""
    rows = [list(r) for r in w.rows]
    lens = list(w.seq_lens)
    spare = iter(spare_blocks)
    for _ in range(steps):
        for i in range(len(rows)):
            if lens[i] % w.page_size == 0:
                rows[i].append(next(spare))
            lens[i] += 1
    return rows, lens


def _table(rows, width):
    t = torch.zeros(len(rows), width, dtype=torch.int32)
    for i, r in enumerate(rows):
        t[i, :len(r)] = torch.tensor(r, dtype=torch.int32)
    return t


def _few_long_many_short():
    """300 unrelated requests, 3 of 640 tokens and 297 of 130..240 (enough of them that the scheduler
    leaves the long ones whole): a bucket with a wide head, which the launch copies of the plan
    split in two."""
    lens = [640, 640, 624] + [130 + (37 * i) % 110 for i in range(296)] + [240]   # 240 = 15 pages: grows at step 1
    rows, nxt = [], 0
    for n in lens:
        nb = -(-n // 16)
        rows.append(list(range(nxt, nxt + nb)))
        nxt += nb
    return workloads.Workload("wide-head", 8, 8, 64, torch.float16, 16, lens, rows, nxt, sum(lens), 0)


def _little_sharing():
    """8 requests of 1023..1024 tokens over a 512-token shared prefix, 8/8 heads: longer than the
    small-batch form goes, and sharing saves too little for the plan's second kernel, so the batch is
    launched one work item per request (cut into pieces)."""
    shared = list(range(32))
    lens, rows, nxt = [], [], 32
    for i in range(8):
        n = 1024 - (i % 2)                    # even requests end on a page boundary: they grow at step 1
        nb = -(-n // 16)
        rows.append(shared + list(range(nxt, nxt + nb - 32)))
        nxt += nb - 32
        lens.append(n)
    return workloads.Workload("little-sharing", 8, 8, 64, torch.float16, 16, lens, rows, nxt, 512 + sum(n - 512 for n in lens), 0)


@pytest.mark.parametrize("case", ["c1", "wide-head", "little-sharing"])
def test_advance_step_keeps_the_plan_right_on_cpu(case):
    """After every in-place advance the plan, executed item by item by the oracle, gives dense
    attention over the grown requests (c1: 8 requests x 288 tokens, so step 1 crosses a page)."""
    w = {"c1": lambda: workloads.make("c1", seed=5), "wide-head": _few_long_many_short, "little-sharing": _little_sharing}[case]()
    steps = 20
    spare = list(range(w.num_blocks, w.num_blocks + 640))
    width = w.padded_table().shape[1] + 2
    meta = fake_metadata(w, torch.device("cpu"))
    meta.block_tables_cpu = _table(w.rows, width)
    meta.block_tables = meta.block_tables_cpu.clone()
    plan = DecodePlan.from_metadata(meta)
    gen = torch.Generator().manual_seed(1)
    q = torch.randn(w.batch, 1, w.heads, w.head_dim, generator=gen)
    k = torch.randn(w.num_blocks + 640, w.page_size, w.kv_heads, w.head_dim, generator=gen)
    v = torch.randn(w.num_blocks + 640, w.page_size, w.kv_heads, w.head_dim, generator=gen)
    in_place = 0
    for step in range(1, steps + 1):
        rows, lens = _grown(w, step, spare)
        in_place += plan.advance_step(_table(rows, width))
        assert plan.seq_lens == lens
        if step in (1, 2, 16, 17, 20):
            info = plan._ready_tree().kernel_info
            listed = {key: [t.tolist() for t in getattr(info, key)] for key in
                      ("q_tables", "block_tables", "num_seqs_per_CTAs", "CTA_ranks", "kv_in_CTAs")}
            listed["num_split_per_seq"] = info.num_split_per_seq.tolist()
            launch = info.launch_tables()       # the kernels' copies (longest box first) grew alike
            assert (max(len(p) for p in info._launch_parts) == 2) == (case == "wide-head")
            for b, order in enumerate(info._launch_order):
                for lb, lo, hi in info._launch_parts[b]:
                    lw = launch["block_tables"][lb].shape[1]
                    assert torch.equal(launch["kv_in_CTAs"][lb], info.kv_in_CTAs[b][order[lo:hi]])
                    assert torch.equal(launch["block_tables"][lb], info.block_tables[b][order[lo:hi]][:, :lw])
                    assert (launch["kv_in_CTAs"][lb][:-1] >= launch["kv_in_CTAs"][lb][1:] - step).all()
            whole = info.whole_sequence_tables()    # small batches are launched a work item per request
            assert (whole is not None) == (case in ("c1", "little-sharing"))
            if whole is not None:
                assert whole["kv_in_CTAs"][0].tolist() == lens and whole["q_tables"][0][:, 0].tolist() == list(range(w.batch))
                for i, r in enumerate(rows):
                    assert whole["block_tables"][0][i, :len(r)].tolist() == r
            if case == "little-sharing":
                # what is launched here are the one-item-per-request tables: those are executed (the plan of
                # such a batch, few requests cut into many boxes, can hold one rank twice for a request, as
                # the reference's does; the launch files its partial rows by box ordinal instead)
                listed = {"q_tables": [whole["q_tables"][0].tolist()], "block_tables": [whole["block_tables"][0].tolist()],
                          "num_seqs_per_CTAs": [whole["num_seqs_per_CTAs"][0].tolist()], "CTA_ranks": [whole["CTA_ranks"][0].tolist()],
                          "kv_in_CTAs": [whole["kv_in_CTAs"][0].tolist()], "num_split_per_seq": whole["num_split_per_seq"].tolist()}
            out, lse = ao.run_plan_ref(listed, q, k, v)
            ref, ref_lse = ao.paged_attention_ref(q, k, v, rows, lens)
            assert (out - ref).abs().max().item() < 1e-5, step
            assert (lse - ref_lse).abs().max().item() < 1e-5, step
    assert in_place + plan.replans == steps
    # a full block row may force a fresh plan now and then (more often where the scheduler has cut the
    # requests into many boxes with block rows of their own)
    assert in_place >= steps - (4 if case == "little-sharing" else 2)


@pytest.mark.gpu
@pytest.mark.parametrize("name", ["c2", "c1"])
def test_advance_step_on_gpu(name):
    # (c1: a batch small enough to be launched as one work item per request; those tables grow too)
    print(f"[case] vLLM multi-step advance {name}", flush=True)
    dev = torch.device("cuda:0")
    w = workloads.make(name, seed=6)
    steps = 18
    spare = list(range(w.num_blocks, w.num_blocks + 2 * w.batch))
    width = w.padded_table().shape[1] + 2
    meta = fake_metadata(w, dev)
    meta.block_tables_cpu = _table(w.rows, width)
    meta.block_tables = meta.block_tables_cpu.to(dev)
    plan = DecodePlan.from_metadata(meta)
    gen = torch.Generator().manual_seed(2)
    q = torch.randn(w.batch, 1, w.heads, w.head_dim, generator=gen).to(w.dtype)
    k = torch.randn(w.num_blocks + 2 * w.batch, w.page_size, w.kv_heads, w.head_dim, generator=gen).to(w.dtype)
    v = torch.randn(w.num_blocks + 2 * w.batch, w.page_size, w.kv_heads, w.head_dim, generator=gen).to(w.dtype)
    kv_cache = torch.stack([k, v]).to(dev)
    query = q.squeeze(1).to(dev)
    output = torch.empty_like(query)
    for step in range(1, steps + 1):
        rows, lens = _grown(w, step, spare)
        plan.advance_step(_table(rows, width))
        decode_attention(query, kv_cache, plan, 1.0 / math.sqrt(w.head_dim), output)
        if step in (1, 9, 18):
            torch.cuda.synchronize()
            ref, _ = ao.paged_attention_ref(q, k, v, rows, lens)
            err = (output.unsqueeze(1).float().cpu() - ref.float()).abs().max().item()
            print(f"[parity] advance step {step}: max|out - ref| = {err:.3e} (replans {plan.replans})", flush=True)
            assert err <= (1.6e-2 if w.dtype == torch.bfloat16 else 2e-3)


@pytest.mark.gpu
def test_fifty_replanned_decode_steps_with_requests_leaving_and_joining():
    """A serving loop on the headline batch: every step each request grows by a token, every fifth
    step one request finishes and a new one (same shared prefix, fresh suffix) takes its row, and
    the plan is built afresh from the step's metadata. Default settings make no tuning run at all;
    with tuning switched on the whole loop makes one per distinct plan shape it meets (a handful: the
    shape key rounds box counts and widths up to multiples of 8), never one per step.
    Parity against the dense reference on the step's own tables at several steps of both loops."""
    from pat_amd import _prefix_attn as ext
    print("[case] 50 re-planned decode steps of c2, requests leaving and joining", flush=True)
    dev = torch.device("cuda:0")
    w = workloads.make("c2", seed=8)
    steps, page = 50, w.page_size
    shared = min(len(r) for r in w.rows)
    prefix = None
    for depth in range(shared):                      # pages every request starts with
        if len({r[depth] for r in w.rows}) != 1:
            break
        prefix = depth + 1
    assert prefix and prefix * page >= 2048
    spare_blocks = 4 * w.batch + 12 * 40
    gen = torch.Generator().manual_seed(5)
    q = torch.randn(w.batch, 1, w.heads, w.head_dim, generator=gen).to(w.dtype)
    k = torch.randn(w.num_blocks + spare_blocks, page, w.kv_heads, w.head_dim, generator=gen).to(w.dtype)
    v = torch.randn(w.num_blocks + spare_blocks, page, w.kv_heads, w.head_dim, generator=gen).to(w.dtype)
    kv_cache = torch.stack([k, v]).to(dev)
    query = q.squeeze(1).to(dev)
    output = torch.empty_like(query)
    width = w.padded_table().shape[1] + 8

    def serve(tuning_on, incremental=False):
        rows, lens = [list(r) for r in w.rows], list(w.seq_lens)
        plan = None
        spare = iter(range(w.num_blocks, w.num_blocks + spare_blocks))
        ext.set_autotune(tuning_on)
        ext.clear_autotune_cache()
        before = ext.autotune_runs()
        worst = 0.0
        try:
            for step in range(1, steps + 1):
                for i in range(w.batch):                       # one more token each
                    if lens[i] % page == 0:
                        rows[i].append(next(spare))
                    lens[i] += 1
                left, joined = [], 0
                if step % 5 == 0:                              # one leaves, one joins
                    i = (7 * step) % w.batch
                    fresh = 64 + (37 * step) % 448
                    blocks = rows[i][:prefix] + [next(spare) for _ in range(-(-fresh // page))]
                    if incremental:                            # (behind the others, as vLLM queues it)
                        del rows[i], lens[i]
                        rows.append(blocks)
                        lens.append(prefix * page + fresh)
                        left, joined = [i], 1
                    else:                                      # (on the row that became free)
                        rows[i], lens[i] = blocks, prefix * page + fresh
                table = _table(rows, width)
                meta = SimpleNamespace(num_prefills=0, num_decode_tokens=w.batch, seq_lens=list(lens),
                                       block_tables=table.to(dev), block_tables_cpu=table, block_size=page,
                                       nheads=w.heads, nheads_kv=w.kv_heads, max_decode_query_len=1)
                if incremental and plan is not None:
                    plan = DecodePlan.from_previous(plan, meta, left, joined)
                else:
                    plan = DecodePlan.from_metadata(meta)
                decode_attention(query, kv_cache, plan, 1.0 / math.sqrt(w.head_dim), output)
                if step in (1, 5, 26, 50):
                    torch.cuda.synchronize()
                    ref, _ = ao.paged_attention_ref(q, k, v, rows, lens)
                    err = (output.unsqueeze(1).float().cpu() - ref.float()).abs().max().item()
                    worst = max(worst, err)
                    assert err <= 1.6e-2, (step, err)
            torch.cuda.synchronize()
        finally:
            ext.set_autotune(False)
        return ext.autotune_runs() - before, worst

    runs, worst = serve(False)
    print(f"[parity] default settings: {runs} tuning runs, max|out - ref| = {worst:.3e}", flush=True)
    runs_inc, worst_inc = serve(False, incremental=True)
    print(f"[parity] plans made by editing the previous step's tree: max|out - ref| = {worst_inc:.3e}", flush=True)
    assert runs_inc == 0
    assert runs == 0
    runs, worst = serve(True)
    print(f"[parity] tuning switched on: {runs} tuning runs over {steps} plans, max|out - ref| = {worst:.3e}", flush=True)
    assert runs <= 4


def test_next_step_plan_from_the_previous_tree_equals_a_fresh_one():
    """DecodePlan.from_previous edits the previous step's tree (rows gone, rows joined, every row a
    token longer): plan tables equal those of a plan built from the step's metadata alone."""
    w = workloads.make("c2", seed=8)
    page = w.page_size
    rows, lens, nxt = [list(r) for r in w.rows], list(w.seq_lens), w.num_blocks

    def meta_of():
        t = _table(rows, 180)
        return SimpleNamespace(num_prefills=0, num_decode_tokens=len(rows), seq_lens=list(lens), block_tables=t,
                               block_tables_cpu=t, block_size=page, nheads=w.heads, nheads_kv=w.kv_heads,
                               max_decode_query_len=1)

    plan = DecodePlan.from_metadata(meta_of())
    for step in range(1, 21):
        left, joined = [], 0
        for i in range(len(rows)):
            if lens[i] % page == 0:
                rows[i].append(nxt)
                nxt += 1
            lens[i] += 1
        if step % 5 == 0:
            i = (7 * step) % len(rows)
            left = [i]
            del rows[i], lens[i]
            fresh = 64 + (37 * step) % 448
            rows.append(rows[0][:2048 // page] + list(range(nxt, nxt + -(-fresh // page))))
            nxt += -(-fresh // page)
            lens.append(2048 + fresh)
            joined = 1
        meta = meta_of()
        plan = DecodePlan.from_previous(plan, meta, left, joined)
        fresh_plan = DecodePlan.from_metadata(meta)
        got, want = plan.tree.kernel_info, fresh_plan.tree.tree.kernel_info
        assert got.num_split_per_seq.tolist() == want.num_split_per_seq.tolist()
        for name in ("q_tables", "num_seqs_per_CTAs", "CTA_ranks", "kv_in_CTAs", "block_tables"):
            for x, y in zip(getattr(got, name), getattr(want, name)):
                assert torch.equal(x, y), (step, name)
