"""Kernel benchmark over the reference's tree sweep.

    python -m pat_amd.bench_trees [--trees all|<spec> ...] [--heads "32 8" ...] [--iters 100] [--json out.json]

The batches of benchmark/run_kernel_bench.sh:5-33 of the flashserve/PAT tree (20 prefix trees x 4 head
configurations, head_dim 128, fp16, 32-token pages, as benchmark/benchmark_kernel.py:624-700 sets
them up): for each, the prefix-aware plan and the prefix-oblivious plan (one work item per request)
run through the same two kernels, timed between HIP events around `--iters` back-to-back calls after
a warm-up, as the reference's `Timer` does (benchmark_kernel.py:31-52). Plans are built outside the
timed region. The KV cache is rotated over several copies so that no call is served from the
Infinity Cache. Prints one line per case and optionally writes them as JSON.
"""
from __future__ import annotations

import argparse
import ctypes as C
import json
import math
import random
import sys

import torch

TREES = [
    "1,10_4096,416", "1,256_256,32", "1,1024_2048,32", "1,2,64_1024,256,256", "1,4,256_32,256,32",
    "1,8,512_32,512,256", "1,8,512_32,2048,256", "1,8,512_512,512,256", "1,4,8,256_32,256,256,32",
    "1,4,16,512_1024,256,128,32", "1,4,16,64,256,1024_256,32,256,64,32,256",
    "1,16,32,64,128,1024_256,128,64,32,32,32", "1,16,32,64,256,1024_256,128,64,32,32,32",
    "1,8,16,32,64,128,1024_256,128,64,32,32,32,32", "1,8,16,32,64,256,1024_256,128,64,32,32,32,32",
    "2,8,16,256_256,256,32,32", "4,16,256,512_512,32,128,32", "8,16,32,256_512,512,256,32",
    "256_1024", "256_4096",
]
HEADS = ["32 32", "16 8", "32 8", "64 8"]
PAGE, HEAD_DIM = 32, 128


def unique_tokens(spec: str) -> int:
    counts, lens = (list(map(int, part.split(","))) for part in spec.split("_"))
    return sum(c * n for c, n in zip(counts, lens))


def run_case(spec: str, heads: int, kv_heads: int, iters: int, warmup: int, budget_bytes: int) -> dict:
    from . import PrefixTreeCPP, _ctypes_launch, _lib, generate_tree_seqs, workloads

    dev = torch.device("cuda:0")
    lib = _lib.load()
    random.seed(0)
    group, num_blocks = generate_tree_seqs(spec, PAGE)
    w = workloads.Workload(spec, heads, kv_heads, HEAD_DIM, torch.float16, PAGE, group.seqlens,
                           group.get_block_ids(), num_blocks, unique_tokens(spec), 0)
    cache_bytes = 2 * num_blocks * PAGE * kv_heads * HEAD_DIM * 2
    copies = max(1, min(8, budget_bytes // cache_bytes))
    gen = torch.Generator(device=dev).manual_seed(0)
    q = torch.randn(w.batch, 1, heads, HEAD_DIM, generator=gen, device=dev, dtype=torch.float16)
    shape = (num_blocks, PAGE, kv_heads, HEAD_DIM)
    ks = [torch.randn(shape, generator=gen, device=dev, dtype=torch.float16) for _ in range(copies)]
    vs = [torch.randn(shape, generator=gen, device=dev, dtype=torch.float16) for _ in range(copies)]
    out = torch.empty_like(q)
    scale = 1.0 / math.sqrt(HEAD_DIM)

    tree = PrefixTreeCPP(PAGE)
    tree.build_radix_tree(w.seq_lens, w.padded_table())
    tree.pack_schedule(None, heads // kv_heads, kv_heads)
    info = tree.kernel_info
    info.to_gpu(dev)
    lt = info.launch_tables()   # what prefix_attn_with_kvcache(tree=...) hands to the kernels
    aware = dict(num_split_per_seq=info.num_split_per_seq, query_tables=lt["q_tables"], block_tables=lt["block_tables"],
                 num_seqs_per_CTAs=lt["num_seqs_per_CTAs"], CTA_ranks=lt["CTA_ranks"], kv_in_CTAs=lt["kv_in_CTAs"],
                 MNW=lt["MNWs"], max_split_per_seq=info.max_split_per_seq, max_seqs_in_CTA=info.max_seqs_in_CTA,
                 max_blocks_in_CTA=info.max_blocks_in_CTA, bucket_flags=lt.get("flags"))
    aware_slots = lt["slot_tables"]
    whole = info.whole_sequence_tables()
    if whole is not None:
        # a small batch of short requests: the drop-in call launches one work item per request (one kernel)
        aware = dict(num_split_per_seq=whole["num_split_per_seq"], query_tables=whole["q_tables"],
                     block_tables=whole["block_tables"], num_seqs_per_CTAs=whole["num_seqs_per_CTAs"],
                     CTA_ranks=whole["CTA_ranks"], kv_in_CTAs=whole["kv_in_CTAs"], MNW=whole["MNWs"],
                     max_split_per_seq=whole["max_split_per_seq"], max_seqs_in_CTA=whole["max_seqs_in_CTA"],
                     max_blocks_in_CTA=whole["max_blocks_in_CTA"], bucket_flags=None)
        aware_slots = None
    oblivious = workloads.oblivious_plan(w, dev)

    def launches(plan, slots):
        made = [_ctypes_launch.prepare(q, ks[i], vs[i], plan["num_split_per_seq"], plan["query_tables"],
                                      plan["block_tables"], plan["num_seqs_per_CTAs"], plan["CTA_ranks"],
                                      plan["kv_in_CTAs"], plan["MNW"], plan["max_split_per_seq"],
                                      plan["max_seqs_in_CTA"], plan["max_blocks_in_CTA"], scale, out, None, slots,
                                      plan.get("bucket_flags"))
                for i in range(len(ks))]
        ws = torch.empty(made[0].need, dtype=torch.uint8, device=dev)
        for m in made:
            m.args.workspace, m.args.workspace_bytes = ws.data_ptr(), ws.numel()
        return made, ws

    stream = torch.cuda.current_stream().cuda_stream

    def timed(made) -> float:
        for i in range(warmup):
            _lib.check(lib.pat_fwd_launch(C.byref(made[i % len(made)].args), C.c_void_p(stream)))
        start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        start.record()
        for i in range(iters):
            lib.pat_fwd_launch(C.byref(made[i % len(made)].args), C.c_void_p(stream))
        stop.record()
        torch.cuda.synchronize()
        return start.elapsed_time(stop) / iters * 1e3

    made_a, keep_a = launches(aware, aware_slots)
    t_aware = timed(made_a)
    made_o, keep_o = launches(oblivious, None)
    t_obl = timed(made_o)
    unique_bytes = w.unique_kv_bytes
    geo = _lib.FwdGeometry()
    _lib.check(lib.pat_fwd_geometry_of(C.byref(made_a[0].args), C.byref(geo)))
    return {"workgroups": int(geo.num_workgroups), "tall_rows": int(geo.tall_rows), "whole_sequences": whole is not None, "tree": spec, "heads": heads, "kv_heads": kv_heads, "batch": w.batch, "unique_kv_mb": unique_bytes / 1e6,
            "total_kv_mb": w.kv_bytes(w.total_tokens) / 1e6, "pat_us": t_aware, "oblivious_us": t_obl,
            "speedup": t_obl / t_aware, "unique_kv_gbs": unique_bytes / t_aware / 1e3, "kv_copies": copies}


def main() -> None:
    ap = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    ap.add_argument("--trees", nargs="*", default=["all"])
    ap.add_argument("--heads", nargs="*", default=HEADS, help='"q_heads kv_heads" pairs')
    ap.add_argument("--iters", type=int, default=100)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--cache-budget-gib", type=float, default=8.0, help="memory for rotated KV copies per case")
    ap.add_argument("--json", default=None)
    a = ap.parse_args()
    if not torch.cuda.is_available():
        sys.exit("bench_trees needs an AMD GPU")
    trees = TREES if a.trees == ["all"] else a.trees
    rows = []
    print(f"{'tree':48s} {'heads':>6s} {'batch':>5s} {'uniq MB':>8s} {'PAT us':>9s} {'obliv us':>9s} {'x':>6s} {'uniq GB/s':>9s} {'wgs':>6s} {'tall':>4s}")
    for spec in trees:
        for pair in a.heads:
            hq, hkv = (int(x) for x in pair.split())
            r = run_case(spec, hq, hkv, a.iters, a.warmup, int(a.cache_budget_gib * 2**30))
            rows.append(r)
            print(f"{spec:48s} {hq:3d}/{hkv:<2d} {r['batch']:5d} {r['unique_kv_mb']:8.1f} {r['pat_us']:9.1f} "
                  f"{r['oblivious_us']:9.1f} {r['speedup']:6.2f} {r['unique_kv_gbs']:9.0f} {r['workgroups']:6d} {r['tall_rows']:4d}", flush=True)
            torch.cuda.empty_cache()
    if a.json:
        with open(a.json, "w") as f:
            json.dump(rows, f, indent=1)


if __name__ == "__main__":
    main()
