"""GPU parity: the HIP path (through the C ABI of libpat_amd) against the CPU attention oracle
on the same seeded inputs.

Tolerances: max-abs 2e-3 for fp16 and 1.6e-2 for bf16 outputs (fp32 accumulation on both
sides), LSE within 1e-4 relative.
"""
import math

import pytest
import torch

from oracle import attn_oracle as ao
from pat_amd import PrefixTree, PrefixTreeCPP, _prefix_attn, prefix_attn_with_kvcache, workloads

pytestmark = pytest.mark.gpu

TOL = {torch.float16: 2e-3, torch.bfloat16: 1.6e-2}
LSE_RTOL = 1e-4


def _device():
    assert torch.cuda.is_available(), "GPU tests need an AMD GPU"
    return torch.device("cuda:0")


def _oracle(w, q, k, v):
    return ao.paged_attention_ref(q.cpu(), k.cpu(), v.cpu(), w.rows, w.seq_lens)


def _assert_close(name, out, lse, ref_out, ref_lse, dtype):
    err = (out.float().cpu() - ref_out.float()).abs().max().item()
    lerr = ((lse.cpu() - ref_lse).abs() / ref_lse.abs().clamp_min(1.0)).max().item()
    # the strictly relative figure as well: it is larger than the gated one only where |LSE| < 1
    strict = ((lse.cpu() - ref_lse).abs() / ref_lse.abs().clamp_min(1e-30)).max().item()
    print(f"[parity] {name}: max|out - ref| = {err:.3e} (tol {TOL[dtype]:.1e}), LSE rel = {lerr:.3e} "
          f"(strictly relative {strict:.3e})", flush=True)
    assert err <= TOL[dtype], f"{name}: output error {err}"
    assert lerr <= LSE_RTOL, f"{name}: LSE error {lerr}"


def _run_tree(w, q, k, v, chunk_env=None):
    dev = q.device
    tree = PrefixTreeCPP(w.page_size)
    tree.build_radix_tree(w.seq_lens, w.padded_table())
    tree.pack_schedule(None, w.heads // w.kv_heads, w.kv_heads)
    tree.kernel_info.to_gpu(dev)
    out = torch.full_like(q, float("nan"))
    lse = torch.full((w.batch, w.heads), float("nan"), dtype=torch.float32, device=dev)
    prefix_attn_with_kvcache(q, k, v, tree, 1.0 / math.sqrt(w.head_dim), out, softmax_lse=lse)
    torch.cuda.synchronize()
    return out, lse


@pytest.mark.parametrize("name", workloads.NAMES)
def test_workload_tree_overload(name):
    print(f"[case] workload {name} tree overload", flush=True)
    dev = _device()
    w = workloads.make(name, seed=0)
    q, k, v = w.tensors(dev)
    out, lse = _run_tree(w, q, k, v)
    ref_out, ref_lse = _oracle(w, q, k, v)
    _assert_close(name, out, lse, ref_out, ref_lse, w.dtype)


@pytest.mark.parametrize("name,dtype", [("c1", torch.float16), ("c1", torch.bfloat16), ("c2", torch.float16),
                                        ("c4", torch.bfloat16)])
def test_workload_table_overload(name, dtype):
    # the benchmark's call form: Python PrefixTree + KernelInfo.to_tensor + positional tables
    print(f"[case] workload {name} table overload {dtype}", flush=True)
    dev = _device()
    w = workloads.make(name, seed=2)
    w.dtype = dtype
    q, k, v = w.tensors(dev)
    t = PrefixTree(w.page_size)
    t.build_radix_tree(w.seq_lens, w.rows)
    ki = t.pack_schedule(MNWs=None, HRatio=w.heads // w.kv_heads, kvHead=w.kv_heads, use_compute_model=False)
    ki.to_tensor(device=dev)
    out = torch.full_like(q, float("nan"))
    lse = torch.empty(w.batch, w.heads, dtype=torch.float32, device=dev)
    prefix_attn_with_kvcache(q, k, v, ki.num_split_per_seq, ki.q_tables, ki.block_tables, ki.num_seqs_per_CTAs,
                             ki.CTA_ranks, ki.kv_in_CTAs, ki.MNWs, ki.max_split_per_seq, ki.max_seqs_in_CTA,
                             ki.max_blocks_in_CTA, 1.0 / math.sqrt(w.head_dim), out, None, softmax_lse=lse,
                             slot_tables=ki.slot_tables if name == "c4" else None)
    torch.cuda.synchronize()
    ref_out, ref_lse = _oracle(w, q, k, v)
    _assert_close(f"{name}/{dtype}", out, lse, ref_out, ref_lse, dtype)


def _ragged_forest_workload(seed, heads, d, dtype):
    import random
    r = random.Random(seed)
    nxt = [0]

    def blocks(n):
        out = list(range(nxt[0], nxt[0] + n)); nxt[0] += n
        return out

    rows, lens = [], []
    for _ in range(5):                      # roots of very different lengths: the long-box cut fires
        root = blocks(r.choice([3, 30, 150, 260]))
        for _ in range(r.randint(1, 4)):
            mid = root + blocks(r.randint(1, 12))
            for _ in range(r.randint(1, 6)):
                row = mid + blocks(r.randint(1, 9))
                rows.append(row)
                lens.append(len(row) * 16 - r.randint(0, 15))
    perm = list(range(nxt[0])); r.shuffle(perm)
    rows = [[perm[x] for x in row] for row in rows]
    return workloads.Workload("ragged forest", heads[0], heads[1], d, dtype, 16, lens, rows, nxt[0], 0, seed)


@pytest.mark.parametrize("case", ["c4", "ragged"])
def test_reference_call_form_unchanged(case):
    # exactly benchmark/benchmark_kernel.py:247-265: Python PrefixTree, KernelInfo.to_tensor, sixteen
    # positional arguments, nothing else. On c4 at seed 0 the reference scheduler hands one CTA_rank
    # to two boxes of a sequence 11 times (and 5 ranks are >= that sequence's num_split): filing
    # partial results by rank would lose them, the binding derives collision-free slots itself.
    print(f"[case] reference call form, {case}", flush=True)
    dev = _device()
    w = workloads.make("c4", seed=0) if case == "c4" else _ragged_forest_workload(5, (16, 4), 128, torch.float16)
    q, k, v = w.tensors(dev)
    t = PrefixTree(w.page_size)
    t.build_radix_tree(w.seq_lens, w.rows)
    ki = t.pack_schedule(MNWs=None, HRatio=w.heads // w.kv_heads, kvHead=w.kv_heads, use_compute_model=False)
    if case == "c4":
        # the hazard is really there: some sequence sees one rank twice
        seen, twice = set(), 0
        for qt, rk in zip(ki.q_tables, ki.CTA_ranks):
            for row, rank in zip(qt, rk):
                for s in row:
                    twice += (s, rank) in seen
                    seen.add((s, rank))
        assert twice > 0
    ki.to_tensor(device=dev)
    out = torch.full_like(q, float("nan"))
    prefix_attn_with_kvcache(q, k, v, ki.num_split_per_seq, ki.q_tables, ki.block_tables, ki.num_seqs_per_CTAs,
                             ki.CTA_ranks, ki.kv_in_CTAs, ki.MNWs, ki.max_split_per_seq, ki.max_seqs_in_CTA,
                             ki.max_blocks_in_CTA, 1.0 / math.sqrt(w.head_dim), out, None)
    lse = torch.full((w.batch, w.heads), float("nan"), dtype=torch.float32, device=dev)
    out2 = torch.full_like(q, float("nan"))
    prefix_attn_with_kvcache(q, k, v, ki.num_split_per_seq, ki.q_tables, ki.block_tables, ki.num_seqs_per_CTAs,
                             ki.CTA_ranks, ki.kv_in_CTAs, ki.MNWs, ki.max_split_per_seq, ki.max_seqs_in_CTA,
                             ki.max_blocks_in_CTA, 1.0 / math.sqrt(w.head_dim), out2, None, softmax_lse=lse)
    torch.cuda.synchronize()
    ref_out, ref_lse = _oracle(w, q, k, v)
    assert torch.equal(out, out2)
    _assert_close(f"{case} reference call form", out, lse, ref_out, ref_lse, w.dtype)


def test_second_pack_schedule_on_one_tree():
    # the reference's per-sequence split counters count on over repeated pack_schedule calls; the
    # launch merges the boxes of the current plan, whatever the counters say
    print("[case] c3, pack_schedule twice on one tree", flush=True)
    dev = _device()
    w = workloads.make("c3", seed=1)
    q, k, v = w.tensors(dev)
    tree = PrefixTreeCPP(w.page_size)
    tree.build_radix_tree(w.seq_lens, w.padded_table())
    tree.pack_schedule(None, w.heads // w.kv_heads, w.kv_heads)
    first = tree.kernel_info.max_split_per_seq
    tree.pack_schedule(None, w.heads // w.kv_heads, w.kv_heads)
    assert tree.kernel_info.max_split_per_seq == 2 * first
    tree.kernel_info.to_gpu(dev)
    out = torch.full_like(q, float("nan"))
    lse = torch.full((w.batch, w.heads), float("nan"), dtype=torch.float32, device=dev)
    prefix_attn_with_kvcache(q, k, v, tree, 1.0 / math.sqrt(w.head_dim), out, softmax_lse=lse)
    torch.cuda.synchronize()
    ref_out, ref_lse = _oracle(w, q, k, v)
    _assert_close("c3 second pack", out, lse, ref_out, ref_lse, w.dtype)


@pytest.mark.parametrize("spec,heads,d,dtype", [("1,512_512,32", (32, 8), 64, torch.bfloat16),
                                                 ("1,4,256_32,512,32", (64, 8), 128, torch.bfloat16),
                                                 ("1,512_512,32", (32, 4), 128, torch.float16),
                                                 ("1,700_512,32", (24, 3), 64, torch.float16)])
def test_merge_of_many_rows(spec, heads, d, dtype):
    # 16384 rows (requests x query heads) or more with a few partial slots each: the merge kernel gives a
    # half-wave to every row there; both head_dims, both types, kv heads in and out of step with the 8
    # XCDs, a row count that leaves the last workgroup part idle
    print(f"[case] merge of many rows: {spec} heads {heads} d {d} {dtype}", flush=True)
    import random
    from pat_amd import generate_tree_seqs
    dev = _device()
    random.seed(3)
    group, nblk = generate_tree_seqs(spec, 32)
    w = workloads.Workload(spec, heads[0], heads[1], d, dtype, 32, group.seqlens, group.get_block_ids(), nblk, 0, 6)
    assert w.batch * w.heads >= 16384
    q, k, v = w.tensors(dev)
    tree = PrefixTreeCPP(w.page_size)
    tree.build_radix_tree(w.seq_lens, w.padded_table())
    tree.pack_schedule(None, w.heads // w.kv_heads, w.kv_heads)
    info = tree.kernel_info
    info.to_gpu(dev)
    assert info.whole_sequence_tables() is None and info.max_split_per_seq >= 2
    out = torch.full_like(q, float("nan"))
    lse = torch.full((w.batch, w.heads), float("nan"), dtype=torch.float32, device=dev)
    prefix_attn_with_kvcache(q, k, v, tree, 1.0 / math.sqrt(w.head_dim), out, softmax_lse=lse)
    torch.cuda.synchronize()
    assert info._launch_workspace_bytes[0] > 0          # partial rows: the merge kernel ran
    ref_out, ref_lse = _oracle(w, q, k, v)
    _assert_close("many rows " + spec, out, lse, ref_out, ref_lse, dtype)


def test_merge_of_more_than_256_slots(tuning):
    # five nested nodes -> every request sits in five boxes (naive_schedule: one box per node); with
    # 32-token chunks the 2048-token root reserves 64 slots per box: 320 slots per row, so the
    # merge kernel's loops past its 256 register-held slots run
    print("[case] merge of 320 slots per row", flush=True)
    import ctypes as C
    from pat_amd import _ctypes_launch, _lib
    dev = _device()
    nxt = [0]

    def blocks(n):
        out = list(range(nxt[0], nxt[0] + n)); nxt[0] += n
        return out

    root = blocks(128)
    rows, lens = [], []
    for i in range(16):
        if i % 8 == 0:
            a = blocks(4)
        if i % 4 == 0:
            b = blocks(4)
        if i % 2 == 0:
            c = blocks(2)
        row = root + a + b + c + blocks(2)
        rows.append(row)
        lens.append(len(row) * 16 - 15)
    w = workloads.Workload("nested", 8, 8, 64, torch.float16, 16, lens, rows, nxt[0], 0, 9)
    q, k, v = w.tensors(dev)
    t = PrefixTree(w.page_size)
    t.build_radix_tree(w.seq_lens, w.rows)
    ki = t.naive_schedule(1)
    assert ki.max_split_per_seq == 5
    ki.to_tensor(device=dev)
    tuning(chunk_tokens=32, tall_chunk_tokens=32)
    out = torch.full_like(q, float("nan"))
    lse = torch.full((w.batch, w.heads), float("nan"), dtype=torch.float32, device=dev)
    L = _ctypes_launch.prepare(q, k, v, ki.num_split_per_seq, ki.q_tables, ki.block_tables, ki.num_seqs_per_CTAs,
                              ki.CTA_ranks, ki.kv_in_CTAs, ki.MNWs, ki.max_split_per_seq, ki.max_seqs_in_CTA,
                              ki.max_blocks_in_CTA, 1.0 / math.sqrt(w.head_dim), out, lse)
    geo = _lib.FwdGeometry()
    assert _lib.load().pat_fwd_geometry_of(C.byref(L.args), C.byref(geo)) == 0
    assert geo.num_slots == 5 * 64
    _ctypes_launch.run(L, dev)
    torch.cuda.synchronize()
    ref_out, ref_lse = _oracle(w, q, k, v)
    _assert_close("320 slots", out, lse, ref_out, ref_lse, w.dtype)


@pytest.mark.parametrize("name", ["c5b", "c3"])
def test_table_overload_with_even_hint(name):
    # bucket_flags is a hint: on c5b (equal lengths) it is true and selects a kv head per wave on
    # long boxes, on c3 (ragged leaves) it is false; the result must not depend on it
    print(f"[case] workload {name} table overload with PAT_BUCKET_EVEN on every bucket", flush=True)
    from pat_amd._lib import PAT_BUCKET_EVEN
    dev = _device()
    w = workloads.make(name, seed=4)
    q, k, v = w.tensors(dev)
    t = PrefixTree(w.page_size)
    t.build_radix_tree(w.seq_lens, w.rows)
    ki = t.pack_schedule(MNWs=None, HRatio=w.heads // w.kv_heads, kvHead=w.kv_heads, use_compute_model=False)
    ki.to_tensor(device=dev)
    out = torch.full_like(q, float("nan"))
    lse = torch.empty(w.batch, w.heads, dtype=torch.float32, device=dev)
    prefix_attn_with_kvcache(q, k, v, ki.num_split_per_seq, ki.q_tables, ki.block_tables, ki.num_seqs_per_CTAs,
                             ki.CTA_ranks, ki.kv_in_CTAs, ki.MNWs, ki.max_split_per_seq, ki.max_seqs_in_CTA,
                             ki.max_blocks_in_CTA, 1.0 / math.sqrt(w.head_dim), out, None, softmax_lse=lse,
                             slot_tables=ki.slot_tables, bucket_flags=[PAT_BUCKET_EVEN] * len(ki.MNWs))
    torch.cuda.synchronize()
    ref_out, ref_lse = _oracle(w, q, k, v)
    _assert_close(f"{name}/even hint", out, lse, ref_out, ref_lse, w.dtype)


@pytest.mark.parametrize("case", ["combine", "head_per_wave", "tall_identical"])
def test_single_slot_launch_writes_out_directly(case, tuning):
    # every row has one partial slot (no sequence in two boxes, no box in two chunks): the split
    # kernel stores `out` itself, needs no workspace and no merge kernel follows
    # (csrc/api.h:230-238 does the same for max_split_per_seq == 1). All three epilogues. (Batches
    # of 27 boxes or more: below that the balancer halves boxes and every row has two slots.)
    print(f"[case] direct output, {case}", flush=True)
    from pat_amd import _ctypes_launch
    dev = _device()
    if case == "combine":          # few boxes of a few steps: 4 waves share a box, states combined in LDS
        w = workloads.independent("direct-a", 32, 300, 32, 8, 128, torch.bfloat16, 5)
    elif case == "head_per_wave":  # many one-step boxes: a kv head per wave
        w = workloads.independent("direct-b", 256, 100, 16, 8, 64, torch.float16, 6)
    else:                          # 32 groups of 8 requests with the same pages: boxes of 32 rows
        base = workloads.independent("direct-c", 32, 200, 32, 8, 128, torch.float16, 7)
        w = workloads.Workload("direct-c", 32, 8, 128, torch.float16, base.page_size, [200] * 256,
                               [list(base.rows[i // 8]) for i in range(256)], base.num_blocks, 32 * 200, 7)
    q, k, v = w.tensors(dev)
    tree = PrefixTreeCPP(w.page_size)
    tree.build_radix_tree(w.seq_lens, w.padded_table())
    tree.pack_schedule(None, w.heads // w.kv_heads, w.kv_heads)
    info = tree.kernel_info
    info.to_gpu(dev)
    assert info.max_split_per_seq == 1
    lt = info.launch_tables()

    def run(direct):
        tuning(direct_out=1 if direct else 0)
        out = torch.full_like(q, float("nan"))
        lse = torch.full((w.batch, w.heads), float("nan"), dtype=torch.float32, device=dev)
        L = _ctypes_launch.prepare(q, k, v, info.num_split_per_seq, lt["q_tables"], lt["block_tables"],
                                  lt["num_seqs_per_CTAs"], lt["CTA_ranks"], lt["kv_in_CTAs"], lt["MNWs"],
                                  info.max_split_per_seq, info.max_seqs_in_CTA, info.max_blocks_in_CTA,
                                  1.0 / math.sqrt(w.head_dim), out, lse, lt.get("slot_tables"), lt.get("flags"))
        assert (L.need == 0) == direct, f"direct {direct}: workspace {L.need} bytes"
        _ctypes_launch.run(L, dev)
        torch.cuda.synchronize()
        return out, lse

    out_d, lse_d = run(True)
    out_m, lse_m = run(False)
    ref_out, ref_lse = _oracle(w, q, k, v)
    _assert_close(f"direct/{case}", out_d, lse_d, ref_out, ref_lse, w.dtype)
    assert torch.equal(out_d, out_m), "direct store and merge kernel must agree bit for bit"
    assert torch.equal(lse_d, lse_m)


@pytest.mark.parametrize("pad", [8, 2])
def test_single_slot_launch_with_strided_out(pad):
    # `out` as a view with padded head rows: 8 extra elements keep 8-byte stores possible (direct
    # route), 2 do not (the launch falls back to partial slots + merge); same result either way
    print(f"[case] direct output into a strided view, head rows padded by {pad}", flush=True)
    from pat_amd import _ctypes_launch
    dev = _device()
    w = workloads.independent("direct-s", 48, 400, 32, 8, 128, torch.float16, 9)
    q, k, v = w.tensors(dev)
    tree = PrefixTreeCPP(w.page_size)
    tree.build_radix_tree(w.seq_lens, w.padded_table())
    tree.pack_schedule(None, w.heads // w.kv_heads, w.kv_heads)
    tree.kernel_info.to_gpu(dev)
    big = torch.full((w.batch, 1, w.heads, w.head_dim + pad), float("nan"), dtype=q.dtype, device=dev)
    out = big[..., :w.head_dim]
    lse = torch.empty(w.batch, w.heads, dtype=torch.float32, device=dev)
    prefix_attn_with_kvcache(q, k, v, tree, 1.0 / math.sqrt(w.head_dim), out, softmax_lse=lse)
    torch.cuda.synchronize()
    assert (tree.kernel_info._launch_workspace_bytes == [0]) == (pad == 8)
    assert torch.isnan(big[..., w.head_dim:]).all(), "the padding of the view must stay untouched"
    ref_out, ref_lse = _oracle(w, q, k, v)
    _assert_close(f"direct/strided{pad}", out, lse, ref_out, ref_lse, w.dtype)


@pytest.mark.parametrize("kind", ["naive", "compute_model", "sorted"])
def test_other_plans_of_the_python_scheduler(kind):
    # plans the kernels see less often: the per-node plan of naive_schedule (no merging, many small
    # items), the cost-model variant of pack_schedule, and a plan reordered by sort_for_launch
    print(f"[case] c3 {kind} plan, table form", flush=True)
    dev = _device()
    w = workloads.make("c3", seed=3)
    q, k, v = w.tensors(dev)
    t = PrefixTree(w.page_size)
    t.build_radix_tree(w.seq_lens, w.rows)
    hratio = w.heads // w.kv_heads
    if kind == "naive":
        ki = t.naive_schedule(hratio)
    else:
        ki = t.pack_schedule(MNWs=None, HRatio=hratio, kvHead=w.kv_heads, use_compute_model=(kind == "compute_model"))
    if kind == "sorted":
        ki.sort_for_launch()
    ki.to_tensor(device=dev)
    out = torch.full_like(q, float("nan"))
    lse = torch.empty(w.batch, w.heads, dtype=torch.float32, device=dev)
    prefix_attn_with_kvcache(q, k, v, ki.num_split_per_seq, ki.q_tables, ki.block_tables, ki.num_seqs_per_CTAs,
                             ki.CTA_ranks, ki.kv_in_CTAs, ki.MNWs, ki.max_split_per_seq, ki.max_seqs_in_CTA,
                             ki.max_blocks_in_CTA, 1.0 / math.sqrt(w.head_dim), out, None, softmax_lse=lse,
                             slot_tables=ki.slot_tables or None)
    torch.cuda.synchronize()
    ref_out, ref_lse = _oracle(w, q, k, v)
    _assert_close(f"c3 {kind}", out, lse, ref_out, ref_lse, w.dtype)


def test_manual_fixture_partial_pages():
    # the reference's manual fixture (test/test.py:233-239): 33-token requests, partly filled last pages
    print("[case] manual fixture", flush=True)
    dev = _device()
    w = workloads.Workload("manual", 32, 8, 128, torch.float16, 16, [33, 33, 33], [[0, 1, 5], [0, 2, 6], [3, 4, 7]],
                           13, 0, 0)
    q, k, v = w.tensors(dev)
    out, lse = _run_tree(w, q, k, v)
    ref_out, ref_lse = _oracle(w, q, k, v)
    _assert_close("manual", out, lse, ref_out, ref_lse, torch.float16)


@pytest.mark.parametrize("spec,heads", [("1,4,16_32,256,32", (64, 8)), ("1,8_640,32", (64, 8)),
                                        ("1,2,4,8,16,32,64_32,512,32,256,32,32,32", (64, 8)),
                                        ("4,16_4096,256", (32, 32)), ("1,10_4096,416", (16, 8)),
                                        # the rest of the reference's list, at its own 64/8 heads
                                        ("1,2,4,16,32,64,128,256,512_3072,1024,32,32,32,32,32,32,32", (64, 8)),
                                        ("1,2,4,16,32,64,256_4096,32,128,128,32,256,512", (64, 8)),
                                        ("1,2,4,16,32,64,128,256,512_3072,1024,512,256,128,32,256,512,32", (64, 8)),
                                        ("1,2,4,16,32,64,128,256,1024_512,32,128,128,32,256,512,32,32", (64, 8)),
                                        ("1,2,4,16,32,64,128,512_512,32,128,128,32,256,512,256", (64, 8)),
                                        ("1,2,4,16,32,64,128_512,32,128,128,32,256,512", (64, 8)),
                                        ("4_4096", (64, 8)), ("1,4,256_32,256,32", (64, 8)),
                                        ("1,16,32_2048,1024,256", (64, 8)), ("4,16_4096,256", (64, 8)),
                                        ("1,10_4096,416", (64, 8))])
def test_reference_tree_specs_page32(spec, heads):
    # tree batches of the reference's own test (test/test.py:174-187, all 14 of them): page 32, fp16, d 128
    print(f"[case] tree spec {spec} heads {heads}", flush=True)
    import random
    from pat_amd import generate_tree_seqs
    dev = _device()
    random.seed(11)
    group, nblk = generate_tree_seqs(spec, 32)
    w = workloads.Workload(spec, heads[0], heads[1], 128, torch.float16, 32, group.seqlens, group.get_block_ids(),
                           nblk, 0, 4)
    q, k, v = w.tensors(dev)
    out, lse = _run_tree(w, q, k, v)
    ref_out, ref_lse = _oracle(w, q, k, v)
    _assert_close(spec, out, lse, ref_out, ref_lse, torch.float16)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("d,heads", [(64, (8, 8)), (64, (16, 2)), (128, (8, 4)), (128, (16, 8))])
def test_ragged_random_forest(dtype, d, heads):
    print(f"[case] ragged forest d={d} heads={heads} {dtype}", flush=True)
    import random
    dev = _device()
    r = random.Random(d + heads[0])
    rows, lens, nxt = [], [], 0
    for _ in range(37):
        row = []
        if rows and r.random() < 0.8:
            base = rows[r.randrange(len(rows))]
            row = list(base[:r.randint(0, len(base) - 1)])
        extra = r.randint(1, 40)
        row += list(range(nxt, nxt + extra)); nxt += extra
        rows.append(row)
        lens.append(len(row) * 16 - r.randint(0, 15))
    perm = list(range(nxt)); r.shuffle(perm)
    rows = [[perm[x] for x in row] for row in rows]
    # on such forests the reference scheduler can hand one rank to two boxes of a request; the
    # tree form files partial results by box ordinal, so the result is right all the same
    w = workloads.Workload("forest", heads[0], heads[1], d, dtype, 16, lens, rows, nxt, 0, 9)
    q, k, v = w.tensors(dev)
    out, lse = _run_tree(w, q, k, v)
    ref_out, ref_lse = _oracle(w, q, k, v)
    _assert_close("forest", out, lse, ref_out, ref_lse, dtype)


@pytest.mark.parametrize("heads,k", [((8, 8), 64), ((32, 8), 16), ((16, 4), 5)])
def test_legacy_flat_schedule_plan(heads, k):
    # the v0 entry `schedule`: plans in lexsort order; q goes in sorted, the output comes back through
    # reverse_index (the reordering the reference's vLLM v0 backend did around the kernel)
    print(f"[case] legacy schedule() plan heads={heads} k={k}", flush=True)
    import random
    from pat_amd import schedule
    dev = _device()
    r = random.Random(k)
    rows, lens, nxt = [], [], 0
    for _ in range(45):
        row = []
        if rows and r.random() < 0.85:
            base = rows[r.randrange(len(rows))]
            row = list(base[:r.randint(0, len(base) - 1)])
        extra = r.randint(1, 24)
        row += list(range(nxt, nxt + extra)); nxt += extra
        rows.append(row)
        lens.append(len(row) * 16 - r.randint(0, 15))
    perm = list(range(1, nxt + 1)); r.shuffle(perm)          # page 0 is the table's padding value
    rows = [[perm[x] for x in row] for row in rows]
    w = workloads.Workload("flat", heads[0], heads[1], 128, torch.float16, 16, lens, rows, nxt + 1, 0, 5)
    q, k_cache, v_cache = w.tensors(dev)
    ki = schedule(lens, rows, 16, k, None, heads[0] // heads[1])
    ki.to_tensor(device=dev)
    order = ki.sort_index.long()
    out_sorted = torch.full_like(q, float("nan"))
    lse_sorted = torch.empty(w.batch, w.heads, dtype=torch.float32, device=dev)
    prefix_attn_with_kvcache(q[order].contiguous(), k_cache, v_cache, ki.num_split_per_seq, ki.q_tables,
                             ki.block_tables, ki.num_seqs_per_CTAs, ki.CTA_ranks, ki.kv_in_CTAs, ki.MNWs,
                             ki.max_split_per_seq, ki.max_seqs_in_CTA, ki.max_blocks_in_CTA,
                             1.0 / math.sqrt(w.head_dim), out_sorted, None, softmax_lse=lse_sorted)
    torch.cuda.synchronize()
    back = ki.reverse_index.long()
    ref_out, ref_lse = _oracle(w, q, k_cache, v_cache)
    _assert_close("legacy schedule", out_sorted[back], lse_sorted[back], ref_out, ref_lse, torch.float16)


@pytest.mark.parametrize("page,dtype,heads", [(48, torch.float16, (32, 8)), (64, torch.bfloat16, (32, 8)),
                                              (80, torch.float16, (16, 16)), (128, torch.bfloat16, (64, 8)),
                                              (16, torch.float16, (16, 2))])
def test_page_sizes_and_tiny_boxes(page, dtype, heads):
    # pages that are no power of two (the half -> page map divides by a reciprocal), shared nodes whose
    # length is no multiple of 32 (partial last step of a tall box), requests shorter than one MFMA tile
    print(f"[case] page {page} {dtype} heads={heads}", flush=True)
    import random
    dev = _device()
    r = random.Random(page)
    next_block = [0]

    def blocks(n):
        out = list(range(next_block[0], next_block[0] + n)); next_block[0] += n
        return out

    rows, lens = [], []
    root = blocks(3)                                   # 3 pages shared by everybody below
    for _ in range(20):
        mid = root + blocks(r.choice([1, 2, 5]))       # shared by 1..4 requests
        for _ in range(r.randint(1, 4)):
            own = r.randint(1, 3)
            row = mid + blocks(own)
            rows.append(row)
            lens.append((len(row) - 1) * page + r.randint(1, page))
    for n in (1, 2, 7, 15, 16, 17, 31, 33):            # tiny private requests
        rows.append(blocks(-(-n // page)))
        lens.append(n)
    perm = list(range(next_block[0])); r.shuffle(perm)
    rows = [[perm[x] for x in row] for row in rows]
    w = workloads.Workload("pages", heads[0], heads[1], 128, dtype, page, lens, rows, next_block[0], 0, page)
    q, k, v = w.tensors(dev)
    out, lse = _run_tree(w, q, k, v)
    ref_out, ref_lse = _oracle(w, q, k, v)
    _assert_close(f"page {page}", out, lse, ref_out, ref_lse, dtype)


def test_hip_graph_replay_matches_eager():
    # both kernels of a call captured into a HIP graph (what a serving loop does with a decode step):
    # every replay, with the program's own eager work between replays, must equal the eager result
    print("[case] HIP graph capture and replay, c2", flush=True)
    dev = _device()
    w = workloads.make("c2", seed=7)
    q, k, v = w.tensors(dev)
    tree = PrefixTreeCPP(w.page_size)
    tree.build_radix_tree(w.seq_lens, w.padded_table())
    tree.pack_schedule(None, w.heads // w.kv_heads, w.kv_heads)
    tree.kernel_info.to_gpu(dev)
    scale = 1.0 / math.sqrt(w.head_dim)
    q_static = q.clone()
    out_graph = torch.zeros_like(q)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        prefix_attn_with_kvcache(q_static, k, v, tree, scale, out_graph)      # warm-up outside the capture
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        prefix_attn_with_kvcache(q_static, k, v, tree, scale, out_graph)
    gen = torch.Generator(device="cpu").manual_seed(3)
    for trial in range(4):
        q_new = torch.randn(q.shape, generator=gen).to(w.dtype).to(dev)
        out_eager = torch.full_like(q, float("nan"))
        prefix_attn_with_kvcache(q_new, k, v, tree, scale, out_eager)
        torch.cuda.synchronize()
        q_static.copy_(q_new)
        out_graph.fill_(float("nan"))
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out_graph, out_eager), f"replay {trial} differs from the eager call"
    ref_out, _ = _oracle(w, q_static, k, v)
    assert (out_graph.float().cpu() - ref_out.float()).abs().max().item() <= TOL[w.dtype]


def test_device_selftest_reports_no_mismatch():
    # lane-swap reductions and the transposed LDS read behave as the split kernel assumes
    print("[case] device self-test", flush=True)
    import ctypes as C
    from pat_amd import _lib
    _device()
    failures = C.c_int32(-1)
    stream = torch.cuda.current_stream().cuda_stream
    _lib.check(_lib.load().pat_selftest_device(C.c_void_p(stream), C.byref(failures)))
    assert failures.value == 0


@pytest.mark.parametrize("heads,dtype", [((32, 8), torch.bfloat16), ((16, 16), torch.float16)])
def test_large_ragged_batch_all_launch_modes(heads, dtype, tuning):
    # a launch several times what fits on the device at once: short private tails (one kv head per
    # wave), mid-size shared nodes, a few long shared roots read by many 64-row boxes, boxes sorted
    # longest first for the launch
    print(f"[case] large ragged batch heads={heads} {dtype}", flush=True)
    import random
    dev = _device()
    r = random.Random(heads[0])
    next_block = [0]

    def blocks(n):
        out = list(range(next_block[0], next_block[0] + n)); next_block[0] += n
        return out

    rows, lens = [], []
    for _ in range(3):
        root = blocks(r.randint(40, 90))               # 640..1440 shared tokens
        for _ in range(r.randint(6, 10)):
            mid = root + blocks(r.randint(2, 20))
            for _ in range(r.randint(4, 24)):
                row = mid + blocks(r.randint(1, 14))
                rows.append(row)
                lens.append(len(row) * 16 - r.randint(0, 15))
    order = list(range(len(rows))); r.shuffle(order)
    rows, lens = [rows[i] for i in order], [lens[i] for i in order]
    perm = list(range(next_block[0])); r.shuffle(perm)
    rows = [[perm[x] for x in row] for row in rows]
    w = workloads.Workload("large", heads[0], heads[1], 128, dtype, 16, lens, rows, next_block[0], 0, 21)
    print(f"        {w.batch} requests, {next_block[0]} blocks", flush=True)
    q, k, v = w.tensors(dev)
    out, lse = _run_tree(w, q, k, v)
    ref_out, ref_lse = _oracle(w, q, k, v)
    _assert_close("large ragged", out, lse, ref_out, ref_lse, dtype)
    # the same batch with a kv head per wave on every bucket of <= 16-row boxes, long ones included
    # (the geometry a launch with thousands of such workgroups gets by itself)
    tuning(head_per_wave_long_wgs=0, head_per_wave_tokens=256)
    out, lse = _run_tree(w, q, k, v)
    _assert_close("large ragged, a kv head per wave", out, lse, ref_out, ref_lse, dtype)


@pytest.mark.parametrize("tall_rows", [16, 32])
@pytest.mark.parametrize("name", ["c2", "c3", "c5a", "forest64", "tails"])
def test_both_forms_of_the_tall_path(name, tall_rows, tuning):
    # boxes of 17..64 rows run on 32-row tiles (32x32x16 MFMAs, 64-token super-steps) or on a 16-row
    # tile per wave (16x16x32, 32-token steps); the launch picks one from its sizes, here each is forced
    print(f"[case] tall path on {tall_rows}-row tiles: {name}", flush=True)
    import ctypes as C
    from pat_amd import _ctypes_launch, _lib
    dev = _device()
    if name == "forest64":      # head_dim 64, fp16, ragged forest with 17..64-row boxes and partial last steps
        w = workloads.forest("forest64", 90, 3, 16, 4, 64, torch.float16, 11, root_range=(100, 1300),
                             inner_range=(16, 400), leaf_range=(1, 120))
    elif name == "tails":       # tall boxes whose length is no multiple of 64, 32 or 16 tokens, 17..40 rows
        w = workloads.shared_prefix("tails", 10, 16 * 37, 1, 9, 32, 8, 128, torch.bfloat16, 5)
    else:
        w = workloads.make(name, seed=2)
    tuning(tall_rows=tall_rows)
    q, k, v = w.tensors(dev)
    tree = PrefixTreeCPP(w.page_size)
    tree.build_radix_tree(w.seq_lens, w.padded_table())
    tree.pack_schedule(None, w.heads // w.kv_heads, w.kv_heads)
    info = tree.kernel_info
    info.to_gpu(dev)
    lt = info.launch_tables()
    L = _ctypes_launch.prepare(q, k, v, info.num_boxes_per_seq, lt["q_tables"], lt["block_tables"], lt["num_seqs_per_CTAs"],
                               lt["CTA_ranks"], lt["kv_in_CTAs"], lt["MNWs"], info.max_boxes_per_seq, info.max_seqs_in_CTA,
                               info.max_blocks_in_CTA, 1.0 / math.sqrt(w.head_dim), torch.empty_like(q), None,
                               lt["slot_tables"], lt.get("flags"))
    geo = _lib.FwdGeometry()
    assert _lib.load().pat_fwd_geometry_of(C.byref(L.args), C.byref(geo)) == 0 and geo.tall_rows == tall_rows
    assert any(m[0] > 16 for m in info.MNWs), "the case has no tall box"
    out, lse = _run_tree(w, q, k, v)
    ref_out, ref_lse = _oracle(w, q, k, v)
    _assert_close(f"{name}, {tall_rows}-row tiles", out, lse, ref_out, ref_lse, w.dtype)


def test_strided_views_and_output_in_place():
    # vLLM hands in views: q/out are slices of larger buffers, K and V live in one stacked tensor
    print("[case] strided views", flush=True)
    dev = _device()
    w = workloads.make("c1", seed=4)
    q, k, v = w.tensors(dev)
    kv = torch.stack([k, v])                      # [2, blocks, page, h, d]
    qbig = torch.zeros(w.batch + 3, w.heads, w.head_dim + 64, dtype=q.dtype, device=dev)
    qbig[3:, :, :w.head_dim] = q[:, 0]
    qv = qbig[3:, :, :w.head_dim].unsqueeze(1)
    obig = torch.zeros(w.batch + 5, w.heads, w.head_dim, dtype=q.dtype, device=dev)
    ov = obig[5:].unsqueeze(1)
    tree = PrefixTreeCPP(16)
    tree.build_radix_tree(w.seq_lens, w.padded_table())
    tree.pack_schedule(None, 1, 8)
    tree.kernel_info.to_gpu(dev)
    prefix_attn_with_kvcache(q=qv, k_cache_paged=kv[0], v_cache_paged=kv[1], tree=tree,
                             softmax_scale=0.125, out=ov)
    torch.cuda.synchronize()
    ref_out, _ = _oracle(w, q, k, v)
    assert (obig[5:].float().cpu() - ref_out[:, 0].float()).abs().max().item() <= 2e-3
    assert obig[:5].abs().max().item() == 0


def test_oblivious_plan_same_result_and_linearity():
    # size-independent properties at the headline size: (1) the prefix-oblivious plan gives the same
    # answer as the prefix-aware one; (2) attention is linear in V
    print("[case] c2 oblivious + linearity", flush=True)
    dev = _device()
    w = workloads.make("c2", seed=0)
    q, k, v = w.tensors(dev)
    out, lse = _run_tree(w, q, k, v)
    ob = workloads.oblivious_plan(w, dev)
    out2 = torch.empty_like(q)
    lse2 = torch.empty_like(lse)
    prefix_attn_with_kvcache(q, k, v, ob["num_split_per_seq"], ob["query_tables"], ob["block_tables"],
                             ob["num_seqs_per_CTAs"], ob["CTA_ranks"], ob["kv_in_CTAs"], ob["MNW"],
                             ob["max_split_per_seq"], ob["max_seqs_in_CTA"], ob["max_blocks_in_CTA"],
                             1.0 / math.sqrt(w.head_dim), out2, softmax_lse=lse2)
    torch.cuda.synchronize()
    assert (out.float() - out2.float()).abs().max().item() <= 1.6e-2
    assert ((lse - lse2).abs() / lse.abs().clamp_min(1)).max().item() <= 1e-4
    out3, _ = _run_tree(w, q, k, (v.float() * 2).to(v.dtype))
    assert (out3.float() - 2 * out.float()).abs().max().item() <= 3.2e-2


@pytest.mark.parametrize("scale", [-0.1, 0.0, 0.6, 1e-3])
def test_softmax_scale_sign_zero_and_spread(scale):
    # a negative scale, scale 0 (uniform attention), a large one (scores spread over +-80, so the
    # running maximum moves many times and most probabilities underflow) and a tiny one must all
    # match the oracle
    print(f"[case] c2-shaped batch, softmax_scale {scale}", flush=True)
    dev = _device()
    w = workloads.make("c2", seed=5)
    q, k, v = w.tensors(dev)
    tree = PrefixTreeCPP(w.page_size)
    tree.build_radix_tree(w.seq_lens, w.padded_table())
    tree.pack_schedule(None, w.heads // w.kv_heads, w.kv_heads)
    tree.kernel_info.to_gpu(dev)
    out = torch.full_like(q, float("nan"))
    lse = torch.full((w.batch, w.heads), float("nan"), dtype=torch.float32, device=dev)
    prefix_attn_with_kvcache(q, k, v, tree, scale, out, softmax_lse=lse)
    torch.cuda.synchronize()
    ref_out, ref_lse = ao.paged_attention_ref(q.cpu(), k.cpu(), v.cpu(), w.rows, w.seq_lens, scale)
    _assert_close(f"scale {scale}", out, lse, ref_out, ref_lse, w.dtype)


def test_reference_maximum_moves_with_sorted_keys():
    # keys ordered so that the scores of a request grow from page to page by large amounts (and
    # fall again where its pages go back in the pool): the accumulator is rescaled on most steps
    # of both the tall and the short path
    print("[case] sorted keys: growing maxima", flush=True)
    dev = _device()
    w = workloads.make("c2", seed=6)
    q, k, v = w.tensors(dev)
    q = torch.ones_like(q)
    ramp = torch.linspace(-3.0, 3.0, k.shape[0] * k.shape[1], device=dev).view(k.shape[0], k.shape[1], 1, 1)
    k = (ramp * torch.ones_like(k)).to(k.dtype)     # q.k = 128 * ramp, different per page and slot
    out, lse = _run_tree(w, q, k, v)
    ref_out, ref_lse = _oracle(w, q, k, v)
    _assert_close("sorted keys", out, lse, ref_out, ref_lse, w.dtype)


@pytest.mark.parametrize("name", ["c1", "c2", "c5b", "independent"])
def test_paged_decode_baseline_matches_oracle(name):
    # the prefix-oblivious comparator behind its own C-ABI entry point: block table + lengths in,
    # one work item per request, same kernels ("independent": 64 requests of 500 tokens, which the
    # launch serves with one slot per row and no merge kernel)
    from pat_amd import paged_decode_baseline
    print(f"[case] paged decode baseline {name}", flush=True)
    dev = _device()
    w = (workloads.independent("ind", 64, 500, 32, 8, 128, torch.bfloat16, 9) if name == "independent"
         else workloads.make(name, seed=9))
    q, k, v = w.tensors(dev)
    out = torch.full_like(q, float("nan"))
    lse = torch.full((w.batch, w.heads), float("nan"), dtype=torch.float32, device=dev)
    lens = torch.tensor(w.seq_lens, dtype=torch.int32, device=dev)
    paged_decode_baseline(q, k, v, w.padded_table().to(dev), lens, 1.0 / math.sqrt(w.head_dim), out,
                          softmax_lse=lse, even_lengths=(name == "c5b"))
    torch.cuda.synchronize()
    ref_out, ref_lse = _oracle(w, q, k, v)
    _assert_close(f"baseline {name}", out, lse, ref_out, ref_lse, w.dtype)


def test_validation_errors_on_gpu_tensors():
    dev = _device()
    w = workloads.make("c1")
    q, k, v = w.tensors(dev)
    tree = PrefixTreeCPP(16)
    tree.build_radix_tree(w.seq_lens, w.padded_table())
    tree.pack_schedule(None, 1, 8)
    out = torch.empty_like(q)
    with pytest.raises(RuntimeError, match="must be on CUDA"):
        prefix_attn_with_kvcache(q, k, v, tree, 0.125, out)          # plan still on the CPU
    tree.kernel_info.to_gpu(dev)
    with pytest.raises(RuntimeError, match="same dtype"):
        prefix_attn_with_kvcache(q, k.to(torch.bfloat16), v, tree, 0.125, out)
    with pytest.raises(RuntimeError, match="contiguous last dimension"):
        prefix_attn_with_kvcache(q.transpose(2, 3).contiguous().transpose(2, 3), k, v, tree, 0.125, out)
    with pytest.raises(RuntimeError, match="64 / 128"):
        prefix_attn_with_kvcache(q[..., :32].contiguous(), k[..., :32].contiguous(), v[..., :32].contiguous(), tree,
                                 0.125, out[..., :32].contiguous())


def test_randomized_workloads_fixed_seed(tuning):
    # 120 workloads drawn from a fixed seed: independent requests, one shared prefix, three-level trees
    # and irregular forests over 8 head configurations, both head dims and element types; small ones
    # (the oracle runs on the CPU). Batches without sharing of 27 requests or more take the
    # single-slot route, the rest every other route the launch geometry knows. The form of the tall
    # path is the launch's own choice in every third case and forced to 16 / 32 rows in the others.
    import numpy as np
    dev = _device()
    rng = np.random.default_rng(20240607)
    head_cfgs = [(8, 8), (16, 8), (32, 8), (64, 8), (16, 16), (32, 32), (8, 4), (16, 4)]
    done = 0
    while done < 120:
        h, hk = head_cfgs[rng.integers(len(head_cfgs))]
        d = int(rng.choice([64, 128]))
        dtype = [torch.float16, torch.bfloat16][rng.integers(2)]
        kind, seed = int(rng.integers(4)), int(rng.integers(1 << 30))
        if kind == 0:
            w = workloads.independent("rnd", int(rng.integers(1, 200)), int(rng.integers(1, 2600)), h, hk, d, dtype, seed)
        elif kind == 1:
            w = workloads.shared_prefix("rnd", int(rng.integers(2, 150)), int(rng.integers(1, 200)) * 16, 1,
                                        int(rng.integers(2, 700)), h, hk, d, dtype, seed)
        elif kind == 2:
            mids = int(rng.integers(1, 5))
            w = workloads.three_level("rnd", mids * int(rng.integers(2, 30)), int(rng.integers(1, 100)) * 16, mids,
                                      int(rng.integers(1, 40)) * 16, 1, int(rng.integers(2, 400)), h, hk, d, dtype, seed)
        else:
            w = workloads.forest("rnd", int(rng.integers(4, 100)), int(rng.integers(1, 5)), h, hk, d, dtype, seed,
                                 root_range=(64, 1500), inner_range=(16, 300), leaf_range=(1, 200))
        if w.kv_bytes(w.total_tokens) > 1.5e8:
            continue
        print(f"[case] random {done}: kind {kind} batch {w.batch} heads {h}/{hk} d {d} {dtype} seed {seed} tall form {(0, 16, 32)[done % 3]}", flush=True)
        tuning(tall_rows=(0, 16, 32)[done % 3])
        q, k, v = w.tensors(dev)
        out, lse = _run_tree(w, q, k, v)
        ref_out, ref_lse = _oracle(w, q, k, v)
        _assert_close(f"random {done}", out, lse, ref_out, ref_lse, dtype)
        done += 1


def test_autotuned_geometry_matches_oracle_and_is_remembered():
    # the measured choice of the launch geometry: whichever candidate wins, the result is the
    # oracle's; the C entry point reports a candidate that the launch accepts; the binding measures
    # once per plan shape and reuses the choice for other tensors of the same plan
    print("[case] autotune on c2: C entry point, then the drop-in call", flush=True)
    import ctypes as C
    from pat_amd import _ctypes_launch, _lib, _prefix_attn
    dev = _device()
    w = workloads.make("c2", seed=0)
    q, ks, vs = w.tensors(dev, copies=2)
    ref_out, ref_lse = _oracle(w, q, ks[0], vs[0])
    tree = PrefixTreeCPP(w.page_size)
    tree.build_radix_tree(w.seq_lens, w.padded_table())
    tree.pack_schedule(None, w.heads // w.kv_heads, w.kv_heads)
    info = tree.kernel_info
    info.to_gpu(dev)
    lt = info.launch_tables()
    out = torch.full_like(q, float("nan"))
    lse = torch.full((w.batch, w.heads), float("nan"), dtype=torch.float32, device=dev)
    L = _ctypes_launch.prepare(q, ks[0], vs[0], info.num_boxes_per_seq, lt["q_tables"], lt["block_tables"],
                               lt["num_seqs_per_CTAs"], lt["CTA_ranks"], lt["kv_in_CTAs"], lt["MNWs"],
                               info.max_boxes_per_seq, info.max_seqs_in_CTA, info.max_blocks_in_CTA,
                               1.0 / math.sqrt(w.head_dim), out, lse, lt["slot_tables"], lt.get("flags"), autotune=True)
    torch.cuda.synchronize()
    print(f"        tuning run: chosen {L.tuned_us:.1f} us, automatic {L.auto_us:.1f} us, overrides "
          f"{[getattr(L.tuning, f) for f, _ in _lib.FwdTuning._fields_]}", flush=True)
    assert 0 < L.tuned_us <= L.auto_us
    _assert_close("c2 after the tuning run", out, lse, ref_out, ref_lse, w.dtype)   # `out` is valid after tuning
    out.fill_(float("nan")); lse.fill_(float("nan"))
    _ctypes_launch.run(L, dev)
    torch.cuda.synchronize()
    _assert_close("c2 tuned launch", out, lse, ref_out, ref_lse, w.dtype)
    # the drop-in call: measured on first use, remembered for the second cache
    was = _prefix_attn.get_autotune()
    _prefix_attn.set_autotune(True)
    _prefix_attn.clear_autotune_cache()
    try:
        for i in range(2):
            out.fill_(float("nan")); lse.fill_(float("nan"))
            prefix_attn_with_kvcache(q, ks[i], vs[i], tree, 1.0 / math.sqrt(w.head_dim), out, softmax_lse=lse)
            torch.cuda.synchronize()
            if i == 0:
                _assert_close("c2 drop-in call, tuned", out, lse, ref_out, ref_lse, w.dtype)
        chosen = info._launch_tunings
        assert len(chosen) == 2 and chosen[0] == chosen[1] and len(chosen[0]) == 8
    finally:
        _prefix_attn.set_autotune(was)


@pytest.mark.parametrize("name", ["c2", "c4"])
def test_launch_records_prebuilt_or_built_by_the_launch(name):
    # The launch records of a plan (one per workgroup: rows, slots, pages) built once with
    # pat_fwd_build_records and handed to the launch, against a launch that builds them itself in its
    # workspace, against pat_fwd_launch_static doing the same in the built-in scratch: identical bits,
    # and the oracle's values. Records of another geometry are refused.
    print(f"[case] launch records, {name}: prebuilt / built by the launch / built in the static scratch", flush=True)
    import ctypes as C
    from pat_amd import _ctypes_launch, _lib
    lib = _lib.load()
    dev = _device()
    w = workloads.make(name, seed=0)
    q, k, v = w.tensors(dev)
    tree = PrefixTreeCPP(w.page_size)
    tree.build_radix_tree(w.seq_lens, w.padded_table())
    tree.pack_schedule(None, w.heads // w.kv_heads, w.kv_heads)
    info = tree.kernel_info
    info.to_gpu(dev)
    lt = info.launch_tables()
    stream = C.c_void_p(torch.cuda.current_stream(dev).cuda_stream)
    results = []
    for route in ("prebuilt", "by the launch", "static scratch"):
        out = torch.full_like(q, float("nan"))
        lse = torch.full((w.batch, w.heads), float("nan"), dtype=torch.float32, device=dev)
        L = _ctypes_launch.prepare(q, k, v, info.num_boxes_per_seq, lt["q_tables"], lt["block_tables"],
                                   lt["num_seqs_per_CTAs"], lt["CTA_ranks"], lt["kv_in_CTAs"], lt["MNWs"],
                                   info.max_boxes_per_seq, info.max_seqs_in_CTA, info.max_blocks_in_CTA,
                                   1.0 / math.sqrt(w.head_dim), out, lse, lt["slot_tables"], lt.get("flags"),
                                   build_records=route == "prebuilt")
        assert (L.args.records is not None) == (route == "prebuilt")
        if route == "static scratch":
            assert L.need <= lib.pat_fwd_static_scratch_bytes()
            L.args.workspace, L.args.workspace_bytes = None, 0
            rc = lib.pat_fwd_launch_static(C.byref(L.args), stream)
        else:
            ws = torch.empty(L.need, dtype=torch.uint8, device=dev)
            L.args.workspace, L.args.workspace_bytes = ws.data_ptr(), L.need
            rc = lib.pat_fwd_launch(C.byref(L.args), stream)
        assert rc == 0, _lib.last_error()
        torch.cuda.synchronize()
        results.append((route, L, out, lse))
    ref_out, ref_lse = _oracle(w, q, k, v)
    _assert_close(f"{name} prebuilt records", results[0][2], results[0][3], ref_out, ref_lse, w.dtype)
    for route, _, out, lse in results[1:]:
        assert torch.equal(out, results[0][2]) and torch.equal(lse, results[0][3]), route
    # the workspace of a launch that builds its own records is larger by exactly the records
    rbytes = C.c_size_t()
    assert lib.pat_fwd_records_bytes(C.byref(results[1][1].args), C.byref(rbytes)) == 0
    assert results[1][1].need == results[0][1].need + rbytes.value
    # records that belong to another geometry: refused, nothing enqueued
    L = results[0][1]
    L.args.records_tag ^= 1
    ws = torch.empty(max(L.need, 256), dtype=torch.uint8, device=dev)
    L.args.workspace, L.args.workspace_bytes = ws.data_ptr(), L.need
    assert lib.pat_fwd_launch(C.byref(L.args), stream) == _lib.PAT_ERR_INVALID
    assert "launch records" in _lib.last_error()


def test_process_that_imports_the_package_first_exits_cleanly():
    # `python -m pat_amd.bench_trees` imports the package before anything imported torch; the package
    # must bring torch (and the HIP runtime) up first, or the process crashes in the heap's clean-up
    # when it exits (after printing correct results). One small tree, in a child process.
    print("[case] python -m pat_amd.bench_trees in a child process: exit status", flush=True)
    import os
    import subprocess
    import sys
    _device()
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    res = subprocess.run([sys.executable, "-m", "pat_amd.bench_trees", "--trees", "1,256_256,32", "--heads", "32 8",
                          "--iters", "2", "--warmup", "1"], cwd=root, capture_output=True, text=True, timeout=110)
    print(res.stdout[-300:], flush=True)
    assert res.returncode == 0, f"exit status {res.returncode}: {res.stderr[-500:]}"
    assert "1,256_256,32" in res.stdout


def test_table_form_new_plan_at_recycled_addresses():
    # A serving loop drops a plan and builds the next one: same shapes, other contents, and the
    # allocator hands out the addresses just freed. What the binding remembers per plan (launch
    # records, derived slots) is looked up by address, so it must not outlive the plan's tensors.
    print("[case] table form, a new plan at the addresses of a dropped one", flush=True)
    dev = _device()

    def plan(w):
        t = PrefixTree(w.page_size)
        t.build_radix_tree(w.seq_lens, w.rows)
        ki = t.pack_schedule(MNWs=None, HRatio=w.heads // w.kv_heads, kvHead=w.kv_heads, use_compute_model=False)
        ki.to_tensor(device=dev)
        return ki

    def call(w, ki, q, k, v, out):
        prefix_attn_with_kvcache(q, k, v, ki.num_split_per_seq, ki.q_tables, ki.block_tables, ki.num_seqs_per_CTAs,
                                 ki.CTA_ranks, ki.kv_in_CTAs, ki.MNWs, ki.max_split_per_seq, ki.max_seqs_in_CTA,
                                 ki.max_blocks_in_CTA, 1.0 / math.sqrt(w.head_dim), out, None)

    wa, wb = workloads.make("c1", seed=0), workloads.make("c1", seed=1)
    assert wa.rows != wb.rows and [len(r) for r in wa.rows] == [len(r) for r in wb.rows]
    qa, ka, va = wa.tensors(dev)
    ki = plan(wa)
    addresses = [t.data_ptr() for t in ki.block_tables]
    out = torch.full_like(qa, float("nan"))
    call(wa, ki, qa, ka, va, out)
    # more launches of another plan than the binding remembers: the first plan's launch is forgotten
    wc = _ragged_forest_workload(3, (8, 4), 64, torch.float16)
    qc, kc, vc = wc.tensors(dev)
    kic = plan(wc)
    outs = [torch.empty_like(qc) for _ in range(70)]
    for o in outs:
        call(wc, kic, qc, kc, vc, o)
    torch.cuda.synchronize()
    del ki
    ki = plan(wb)
    print(f"[case] block tables of the new plan at the old addresses: {[t.data_ptr() for t in ki.block_tables] == addresses}", flush=True)
    qb, kb, vb = wb.tensors(dev)
    out = torch.full_like(qb, float("nan"))
    lse = None
    call(wb, ki, qb, kb, vb, out)
    torch.cuda.synchronize()
    ref_out, ref_lse = _oracle(wb, qb, kb, vb)
    err = (out.float().cpu() - ref_out.float()).abs().max().item()
    assert err <= TOL[wb.dtype], f"new plan at recycled addresses: output error {err}"


def test_launches_of_one_plan_from_two_streams():
    # What the binding builds per plan (launch records) is written by a kernel on the stream of the
    # first call; a call on another stream right behind it must be ordered after that kernel.
    print("[case] one plan, first call on one stream, second on another", flush=True)
    dev = _device()
    w = workloads.make("c3", seed=1)
    q, k, v = w.tensors(dev)
    tree = PrefixTreeCPP(w.page_size)
    tree.build_radix_tree(w.seq_lens, w.padded_table())
    tree.pack_schedule(None, w.heads // w.kv_heads, w.kv_heads)
    tree.kernel_info.to_gpu(dev)
    torch.cuda.synchronize()
    s1, s2 = torch.cuda.Stream(), torch.cuda.Stream()
    out1, out2 = torch.full_like(q, float("nan")), torch.full_like(q, float("nan"))
    lse1 = torch.full((w.batch, w.heads), float("nan"), dtype=torch.float32, device=dev)
    lse2 = lse1.clone()
    torch.cuda.synchronize()
    with torch.cuda.stream(s1):
        prefix_attn_with_kvcache(q, k, v, tree, 1.0 / math.sqrt(w.head_dim), out1, softmax_lse=lse1)
    with torch.cuda.stream(s2):
        prefix_attn_with_kvcache(q, k, v, tree, 1.0 / math.sqrt(w.head_dim), out2, softmax_lse=lse2)
    torch.cuda.synchronize()
    ref_out, ref_lse = _oracle(w, q, k, v)
    _assert_close("two streams, first", out1, lse1, ref_out, ref_lse, w.dtype)
    _assert_close("two streams, second", out2, lse2, ref_out, ref_lse, w.dtype)
    assert torch.equal(out1, out2)


def test_plans_built_under_inference_mode():
    # a plan packed, moved and used under torch.inference_mode(): the tree's own tensors keep their
    # version counters; a table-form plan of inference tensors (no counter) is served without
    # snapshots of its contents, so an in-place edit is seen by the next call
    print("[case] inference_mode: tree form and table form of inference tensors, c1", flush=True)
    dev = _device()
    w = workloads.make("c1", seed=3)
    q, k, v = w.tensors(dev)
    scale = 1.0 / math.sqrt(w.head_dim)
    ref_out, ref_lse = _oracle(w, q, k, v)
    with torch.inference_mode():
        tree = PrefixTreeCPP(w.page_size)
        tree.build_radix_tree(w.seq_lens, w.padded_table())
        tree.pack_schedule(None, w.heads // w.kv_heads, w.kv_heads)
        tree.kernel_info.to_gpu(dev)
        assert not tree.kernel_info._flat.is_inference()
        out = torch.full_like(q, float("nan"))
        lse = torch.full((w.batch, w.heads), float("nan"), dtype=torch.float32, device=dev)
        prefix_attn_with_kvcache(q, k, v, tree, scale, out, softmax_lse=lse)
        torch.cuda.synchronize()
        _assert_close("tree form under inference_mode", out, lse, ref_out, ref_lse, w.dtype)

        t = PrefixTree(w.page_size)
        t.build_radix_tree(w.seq_lens, w.rows)
        ki = t.pack_schedule(MNWs=None, HRatio=w.heads // w.kv_heads, kvHead=w.kv_heads, use_compute_model=False)
        ki.to_tensor(device=dev)
        assert ki.kv_in_CTAs[0].is_inference()

        def call(o, l):
            prefix_attn_with_kvcache(q, k, v, ki.num_split_per_seq, ki.q_tables, ki.block_tables, ki.num_seqs_per_CTAs,
                                     ki.CTA_ranks, ki.kv_in_CTAs, ki.MNWs, ki.max_split_per_seq, ki.max_seqs_in_CTA,
                                     ki.max_blocks_in_CTA, scale, o, softmax_lse=l)
        out.fill_(float("nan"))
        call(out, lse)
        torch.cuda.synchronize()
        _assert_close("table form of inference tensors", out, lse, ref_out, ref_lse, w.dtype)
        # every request loses its last token (an in-place edit torch does not count): the next call sees it
        lens = [n - 1 for n in w.seq_lens]
        for b in range(len(ki.kv_in_CTAs)):
            leaf = ki.num_seqs_per_CTAs[b] == 1
            ki.kv_in_CTAs[b] -= leaf.to(torch.int32)
        call(out, lse)
        torch.cuda.synchronize()
    ref2, ref2_lse = ao.paged_attention_ref(q.cpu(), k.cpu(), v.cpu(), w.rows, lens, scale)
    _assert_close("table form after an uncounted edit", out, lse, ref2, ref2_lse, w.dtype)


def test_graph_replay_reads_the_plan_tables_of_the_moment():
    # a captured call builds its launch records inside the graph: a replay after the plan tables
    # were rewritten (here by a captured copy_, which no version counter sees from the launch's side)
    # computes what an eager call on the same tables computes
    print("[case] HIP graph whose plan tables change between replays, c1-shaped", flush=True)
    dev = _device()
    w = workloads.make("c1", seed=4)
    q, k, v = w.tensors(dev)
    scale = 1.0 / math.sqrt(w.head_dim)
    t = PrefixTree(w.page_size)
    t.build_radix_tree(w.seq_lens, w.rows)
    ki = t.pack_schedule(MNWs=None, HRatio=w.heads // w.kv_heads, kvHead=w.kv_heads, use_compute_model=False)
    ki.to_tensor(device=dev)
    kv_full = [x.clone() for x in ki.kv_in_CTAs]
    kv_short = [x - (n == 1).to(torch.int32) * 5 for x, n in zip(ki.kv_in_CTAs, ki.num_seqs_per_CTAs)]   # leaves lose 5 tokens
    staged = [x.clone() for x in ki.kv_in_CTAs]
    out_graph = torch.zeros_like(q)

    def call(o):
        prefix_attn_with_kvcache(q, k, v, ki.num_split_per_seq, ki.q_tables, ki.block_tables, ki.num_seqs_per_CTAs,
                                 ki.CTA_ranks, ki.kv_in_CTAs, ki.MNWs, ki.max_split_per_seq, ki.max_seqs_in_CTA,
                                 ki.max_blocks_in_CTA, scale, o)

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        call(out_graph)                                                     # warm-up outside the capture
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        for dst, src in zip(ki.kv_in_CTAs, staged):
            dst.copy_(src)
        call(out_graph)
    for trial, (kvs, lens) in enumerate([(kv_short, [n - 5 for n in w.seq_lens]), (kv_full, list(w.seq_lens)),
                                         (kv_short, [n - 5 for n in w.seq_lens])]):
        for dst, src in zip(staged, kvs):
            dst.copy_(src)
        out_graph.fill_(float("nan"))
        graph.replay()
        torch.cuda.synchronize()
        ref_out, _ = ao.paged_attention_ref(q.cpu(), k.cpu(), v.cpu(), w.rows, lens, scale)
        err = (out_graph.float().cpu() - ref_out.float()).abs().max().item()
        print(f"[parity] replay {trial}: max|out - ref| = {err:.3e}", flush=True)
        assert err <= TOL[w.dtype], f"replay {trial}: {err}"
        out_eager = torch.full_like(q, float("nan"))
        # (an eager call works from a snapshot of the tables taken per version counter; the replay's
        # copy_ moved no counter, so the snapshots are dropped by hand)
        _prefix_attn.invalidate_plans()
        call(out_eager)                                                     # eager, same table contents
        torch.cuda.synchronize()
        assert torch.equal(out_eager, out_graph), f"replay {trial} differs from the eager call"


def test_first_call_under_capture_then_eager():
    # a launch whose very first call is captured (nothing but the capture's own pool has seen it)
    # and is then called eagerly before any replay: the eager call builds its own launch records
    print("[case] first call captured, then eager, c1", flush=True)
    dev = _device()
    w = workloads.make("c1", seed=5)
    q, k, v = w.tensors(dev)
    scale = 1.0 / math.sqrt(w.head_dim)
    warm = workloads.make("c1", seed=6)
    wq, wk, wv = warm.tensors(dev)
    wtree = PrefixTreeCPP(warm.page_size)
    wtree.build_radix_tree(warm.seq_lens, warm.padded_table())
    wtree.pack_schedule(None, warm.heads // warm.kv_heads, warm.kv_heads)
    wtree.kernel_info.to_gpu(dev)
    prefix_attn_with_kvcache(wq, wk, wv, wtree, scale, torch.empty_like(wq))   # the library itself is warm
    tree = PrefixTreeCPP(w.page_size)
    tree.build_radix_tree(w.seq_lens, w.padded_table())
    tree.pack_schedule(None, w.heads // w.kv_heads, w.kv_heads)
    tree.kernel_info.to_gpu(dev)
    torch.cuda.synchronize()
    out_graph = torch.zeros_like(q)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        prefix_attn_with_kvcache(q, k, v, tree, scale, out_graph)
    out = torch.full_like(q, float("nan"))
    lse = torch.full((w.batch, w.heads), float("nan"), dtype=torch.float32, device=dev)
    prefix_attn_with_kvcache(q, k, v, tree, scale, out, softmax_lse=lse)
    torch.cuda.synchronize()
    ref_out, ref_lse = _oracle(w, q, k, v)
    _assert_close("eager after a captured first call", out, lse, ref_out, ref_lse, w.dtype)
    graph.replay()
    torch.cuda.synchronize()
    assert (out_graph.float().cpu() - ref_out.float()).abs().max().item() <= TOL[w.dtype]


def test_small_batch_is_launched_as_whole_sequences():
    # 8 requests of 288 tokens: the tree form launches one work item per request - a single kernel
    # that writes `out` (no workspace, no merge) - and still equals the oracle; the plan tables stay
    # what the scheduler made
    print("[case] small batch (c1): one work item per request", flush=True)
    dev = _device()
    w = workloads.make("c1", seed=8)
    q, k, v = w.tensors(dev)
    tree = PrefixTreeCPP(w.page_size)
    tree.build_radix_tree(w.seq_lens, w.padded_table())
    tree.pack_schedule(None, w.heads // w.kv_heads, w.kv_heads)
    info = tree.kernel_info
    info.to_gpu(dev)
    whole = info.whole_sequence_tables()
    assert whole is not None and whole["max_split_per_seq"] == 1
    assert whole["kv_in_CTAs"][0].tolist() == list(w.seq_lens)
    assert info.max_split_per_seq >= 2            # the scheduler's plan: shared prefix boxes and a private one each
    out = torch.full_like(q, float("nan"))
    lse = torch.full((w.batch, w.heads), float("nan"), dtype=torch.float32, device=dev)
    prefix_attn_with_kvcache(q, k, v, tree, 1.0 / math.sqrt(w.head_dim), out, softmax_lse=lse)
    torch.cuda.synchronize()
    assert info._launch_workspace_bytes == [0]
    ref_out, ref_lse = _oracle(w, q, k, v)
    _assert_close("whole sequences", out, lse, ref_out, ref_lse, w.dtype)
    # a batch of the same shape with longer requests is launched as planned
    big = workloads.make("c2", seed=8)
    t2 = PrefixTreeCPP(big.page_size)
    t2.build_radix_tree(big.seq_lens, big.padded_table())
    t2.pack_schedule(None, big.heads // big.kv_heads, big.kv_heads)
    assert t2.kernel_info.whole_sequence_tables() is None


@pytest.mark.parametrize("route", ["0", "1"])
def test_request_without_tokens(route, monkeypatch):
    # a request of length 0 beside requests that share a prefix: its rows come out as zeros with LSE -inf
    # on both launches of the tree form (the plan, where it sits in no box and the merge kernel fills its
    # rows; one work item per request, where its item has no tokens), the others equal the oracle
    print(f"[case] a request without tokens, PAT_WHOLE_SEQUENCES={route}", flush=True)
    monkeypatch.setenv("PAT_WHOLE_SEQUENCES", route)
    dev = _device()
    shared = list(range(1, 9))
    rows = [[0]] + [shared + [9 + 2 * i, 10 + 2 * i] for i in range(6)]
    lens = [0] + [16 * 10 - 3 * i for i in range(6)]
    w = workloads.Workload("empty-request", 16, 4, 128, torch.float16, 16, lens, rows, 24, 0, 2)
    q, k, v = w.tensors(dev)
    tree = PrefixTreeCPP(w.page_size)
    tree.build_radix_tree(w.seq_lens, w.padded_table())
    tree.pack_schedule(None, w.heads // w.kv_heads, w.kv_heads)
    info = tree.kernel_info
    info.to_gpu(dev)
    assert (info.whole_sequence_tables() is not None) == (route == "1")
    assert info.num_split_per_seq.tolist()[0] == 0 and info.max_split_per_seq >= 2
    out = torch.full_like(q, float("nan"))
    lse = torch.full((w.batch, w.heads), float("nan"), dtype=torch.float32, device=dev)
    prefix_attn_with_kvcache(q, k, v, tree, 1.0 / math.sqrt(w.head_dim), out, softmax_lse=lse)
    torch.cuda.synchronize()
    assert (out[0] == 0).all() and (lse[0] == float("-inf")).all()
    ref_out, ref_lse = ao.paged_attention_ref(q[1:].cpu(), k.cpu(), v.cpu(), rows[1:], lens[1:])
    _assert_close("requests beside an empty one", out[1:], lse[1:], ref_out, ref_lse, w.dtype)


@pytest.mark.parametrize("spec,heads,kernels", [("1,8_1024,1024", (32, 8), 2), ("1,64_256,32", (64, 8), 1),
                                                ("1,128_256,32", (16, 2), 1), ("1,4,8_512,256,704", (32, 8), 2)])
def test_little_sharing_is_launched_as_whole_sequences(spec, heads, kernels):
    # batches whose sharing saves less than the plan's second kernel costs: the tree form launches one
    # work item per request - cut into pieces and merged when requests are long (a workspace then),
    # one kernel when they are short - and equals the oracle
    print(f"[case] little sharing: {spec} heads {heads}: one work item per request", flush=True)
    import random
    from pat_amd import generate_tree_seqs
    dev = _device()
    random.seed(5)
    group, nblk = generate_tree_seqs(spec, 32)
    w = workloads.Workload(spec, heads[0], heads[1], 128, torch.float16, 32, group.seqlens, group.get_block_ids(),
                           nblk, 0, 4)
    q, k, v = w.tensors(dev)
    tree = PrefixTreeCPP(w.page_size)
    tree.build_radix_tree(w.seq_lens, w.padded_table())
    tree.pack_schedule(None, w.heads // w.kv_heads, w.kv_heads)
    info = tree.kernel_info
    info.to_gpu(dev)
    whole = info.whole_sequence_tables()
    assert whole is not None and info.max_split_per_seq >= 2
    out = torch.full_like(q, float("nan"))
    lse = torch.full((w.batch, w.heads), float("nan"), dtype=torch.float32, device=dev)
    prefix_attn_with_kvcache(q, k, v, tree, 1.0 / math.sqrt(w.head_dim), out, softmax_lse=lse)
    torch.cuda.synchronize()
    assert (info._launch_workspace_bytes == [0]) == (kernels == 1)
    ref_out, ref_lse = _oracle(w, q, k, v)
    _assert_close("whole sequences " + spec, out, lse, ref_out, ref_lse, w.dtype)
