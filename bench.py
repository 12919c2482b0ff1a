#!/usr/bin/env python3
"""Benchmark of prefix-aware decode attention on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload c2]

A step is one call of the hot path (pat_fwd_launch through the C ABI of libpat_amd: split
kernel + merge kernel) on one decode batch of the named workload, with the plan already on
the device, under the launch geometry the library chooses from sizes alone (what the drop-in call
does by default). Synthetic, seeded N(0,1) inputs are resident in HBM before the timed region;
the KV cache is rotated over several copies whose total size exceeds the 256 MB Infinity Cache
so that consecutive steps cannot be served from it.

Prints ONE JSON line. `value` is unique-KV bytes / time per call (GB/s); `ms_per_step` is the
latency per call: W warm-up steps, then the K timed steps between two synchronisations, repeated
5 times; the median repetition is reported, `ms_per_step_spread` holds the fastest and slowest.
`roofline` covers the split kernel (HBM-bound): algorithmic bytes = unique KV bytes of the batch,
duration = mean split-kernel time from HIP events on the launch stream. `autotune` reports what
the optional measured choice of the geometry (pat_fwd_autotune, off by default in the product)
would give and what measuring costs; `records_build_us` the kernel that turns the plan tables into
launch records once per plan; `plan_build_ms_host` the host planner in steady state (tree + pack +
flat tables); `tree_next_step_ms_host` the next decode step's tree edited in place against built anew.
`cpu_baseline` times this repository's CPU restatement of the reference's PyTorch attention
on the host cores. `api_us_per_call` is the same loop through the drop-in call
`prefix_attn_with_kvcache(q, k, v, tree, scale, out)` of the compiled extension (workspace from
torch's allocator per call). The default run (workload c2) also measures the other five benchmark
workloads, more briefly, and lists them under `configs`.
"""
from __future__ import annotations

import argparse
import ctypes as C
import json
import math
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBPS = 8000.0          # MI355X HBM3E
INFINITY_CACHE_BYTES = 256 << 20


def measured_traffic_bytes(workload: str, seed: int, workgroups: int):
    """HBM bytes per split-kernel launch as rocprofv3 measured them (--pmc FETCH_SIZE + WRITE_SIZE, each
    scaled by the same counter's reading for a 1 GiB copy kernel), from the marker lines of the
    summaries under profiles/ (one per workload and launch geometry that was measured). None when
    there is no such measurement for this workload, seed and number of workgroups, or when the
    kernel sources have changed since it was taken."""
    import glob
    import hashlib
    import re
    h = hashlib.sha256()
    for rel in ("pat_amd/csrc/hip/pat_split.hip", "pat_amd/csrc/hip/fwd_params.hpp", "pat_amd/csrc/capi_fwd.hip"):
        h.update(open(os.path.join(ROOT, rel), "rb").read())
    for path in sorted(glob.glob(os.path.join(ROOT, "profiles", "pat_split_kernel_*.md"))):
        for m in re.finditer(r"bench-marker: workload=(\S+) seed=(\d+) workgroups=(\d+) traffic_bytes=(\d+) "
                             r"kernel_sources_sha256=([0-9a-f]+)", open(path).read()):
            if m.group(1) == workload and int(m.group(2)) == seed and int(m.group(3)) == workgroups and h.hexdigest() == m.group(5):
                return int(m.group(4))
    return None

WORKLOAD_TEXT = {
    "c1": "8 req, 256 shared + 32 private tokens, 8/8 heads, d64, fp16",
    "c2": "Llama-3-8B shape: batch 64, 2048-token shared prefix + U[64,512] suffix, 32/8 heads, d128, bf16, page 16",
    "c3": "batch 128, 1024 root + 8x512 mid + U[128,1024] leaves, 32/8 heads, d128, fp16",
    "c4": "batch 256, forest of 16 roots, depth<=4, 16/16 heads, d64, fp16",
    "c5a": "Llama-3-70B layer shape: batch 32, 16384 shared + U[256,2048], 64/8 heads, d128, bf16",
    "c5b": "batch 32 independent 4096-token contexts, 64/8 heads, d128, bf16",
    # diagnostic: a launch of 64-row boxes only (profiling the tall-box path)
    "c5a-prefix": "c5a's 16384-token shared prefix with 16-token suffixes, batch 32, 64/8 heads, d128, bf16",
}


class Hip:
    """hipEvent timing on a given stream, straight from the HIP runtime."""

    def __init__(self):
        self.lib = C.CDLL("libamdhip64.so")
        self.lib.hipEventCreate.argtypes = [C.POINTER(C.c_void_p)]
        self.lib.hipEventRecord.argtypes = [C.c_void_p, C.c_void_p]
        self.lib.hipEventElapsedTime.argtypes = [C.POINTER(C.c_float), C.c_void_p, C.c_void_p]
        self.lib.hipEventSynchronize.argtypes = [C.c_void_p]

    def event(self) -> C.c_void_p:
        e = C.c_void_p()
        assert self.lib.hipEventCreate(C.byref(e)) == 0
        return e

    def record(self, e, stream) -> None:
        assert self.lib.hipEventRecord(e, C.c_void_p(stream)) == 0

    def ms(self, a, b) -> float:
        out = C.c_float()
        assert self.lib.hipEventSynchronize(b) == 0
        assert self.lib.hipEventElapsedTime(C.byref(out), a, b) == 0
        return out.value


def measure(a, workload: str, steps: int, warmup: int, headline: bool) -> dict:
    """One workload: plan, timed C-ABI loop, per-kernel event times, the drop-in API loop, the
    prefix-oblivious comparator and (headline only) the CPU baseline."""
    import torch
    from pat_amd import PrefixTreeCPP, _ctypes_launch, _lib, prefix_attn_with_kvcache, workloads

    dev = torch.device("cuda:0")
    lib = _lib.load()
    hip = Hip()
    w = workloads.make(workload, seed=a.seed)
    cache_bytes = w.kv_bytes(w.num_blocks * w.page_size)
    copies = max(2, min(16, math.ceil(2.5 * INFINITY_CACHE_BYTES / cache_bytes)))
    q, ks, vs = w.tensors(dev, copies=copies)
    scale = 1.0 / math.sqrt(w.head_dim)

    batch_table = w.padded_table()     # (what a serving loop has at hand: the step's CPU block table)

    def plan():
        t0 = time.perf_counter()
        tree = PrefixTreeCPP(w.page_size)
        tree.build_radix_tree(w.seq_lens, batch_table)
        tree.pack_schedule(None, w.heads // w.kv_heads, w.kv_heads)
        return tree, (time.perf_counter() - t0) * 1e3

    def plan_next_step():
        # the tree of the next decode step (every request a token longer) made by editing this step's
        # tree (PrefixTreeCPP.advance) against building it anew; median of 5, milliseconds
        tree = PrefixTreeCPP(w.page_size)
        table = torch.cat([batch_table, torch.zeros(w.batch, 2, dtype=torch.int32)], dim=1)
        lens = list(w.seq_lens)
        tree.build_radix_tree(lens, table)
        spare, edit, build = w.num_blocks, [], []
        for _ in range(5):
            for i in range(w.batch):
                if lens[i] % w.page_size == 0:
                    table[i, lens[i] // w.page_size] = spare
                    spare += 1
                lens[i] += 1
            t0 = time.perf_counter()
            in_place = tree.advance(lens, table)
            edit.append((time.perf_counter() - t0) * 1e3)
            assert in_place
            fresh = PrefixTreeCPP(w.page_size)
            t0 = time.perf_counter()
            fresh.build_radix_tree(lens, table)
            build.append((time.perf_counter() - t0) * 1e3)
        return sorted(edit)[2], sorted(build)[2]

    _, plan_first_ms = plan()          # (the first call also pays for the pinned buffer pool)
    plan_runs = sorted(plan()[1] for _ in range(5))
    tree, _ = plan()
    plan_ms = plan_runs[len(plan_runs) // 2]
    info = tree.kernel_info
    info.to_gpu(dev)

    out = torch.empty_like(q)
    stream = torch.cuda.current_stream(dev).cuda_stream

    def prepare(plan_kw, slots, autotune):
        # `autotune`: one measured geometry per plan (pat_fwd_autotune), shared by the launches over the
        # rotated cache copies; otherwise the geometry the library derives from sizes.
        launches, tuning = [], None
        for i in range(copies):
            L = _ctypes_launch.prepare(q, ks[i], vs[i], plan_kw["num_split_per_seq"], plan_kw["query_tables"],
                                       plan_kw["block_tables"], plan_kw["num_seqs_per_CTAs"], plan_kw["CTA_ranks"],
                                       plan_kw["kv_in_CTAs"], plan_kw["MNW"], plan_kw["max_split_per_seq"],
                                       plan_kw["max_seqs_in_CTA"], plan_kw["max_blocks_in_CTA"], scale, out, None, slots,
                                       plan_kw.get("bucket_flags"), autotune=autotune and i == 0, tuning=tuning)
            tuning = L.tuning
            launches.append(L)
        ws = torch.empty(max(max(L.need for L in launches), 256), dtype=torch.uint8, device=dev)
        for L in launches:
            L.args.workspace, L.args.workspace_bytes = ws.data_ptr(), ws.numel()
        return launches, ws

    lt = info.launch_tables()   # what prefix_attn_with_kvcache(tree=...) hands to the kernels
    pat_kw = dict(num_split_per_seq=info.num_split_per_seq, query_tables=lt["q_tables"],
                  block_tables=lt["block_tables"], num_seqs_per_CTAs=lt["num_seqs_per_CTAs"],
                  CTA_ranks=lt["CTA_ranks"], kv_in_CTAs=lt["kv_in_CTAs"], MNW=lt["MNWs"],
                  max_split_per_seq=info.max_split_per_seq, max_seqs_in_CTA=info.max_seqs_in_CTA,
                  max_blocks_in_CTA=info.max_blocks_in_CTA, bucket_flags=lt.get("flags"))
    pat_slots = lt["slot_tables"]
    whole = info.whole_sequence_tables()
    if whole is not None:
        # a small batch of short requests: the drop-in call launches one work item per request (one kernel)
        pat_kw = dict(num_split_per_seq=whole["num_split_per_seq"], query_tables=whole["q_tables"],
                      block_tables=whole["block_tables"], num_seqs_per_CTAs=whole["num_seqs_per_CTAs"],
                      CTA_ranks=whole["CTA_ranks"], kv_in_CTAs=whole["kv_in_CTAs"], MNW=whole["MNWs"],
                      max_split_per_seq=whole["max_split_per_seq"], max_seqs_in_CTA=whole["max_seqs_in_CTA"],
                      max_blocks_in_CTA=whole["max_blocks_in_CTA"], bucket_flags=None)
        pat_slots = None
    pat_launches, pat_ws = prepare(pat_kw, pat_slots, False)

    def step(launches, i):
        rc = lib.pat_fwd_launch(C.byref(launches[i % copies].args), C.c_void_p(stream))
        if rc != 0:
            raise RuntimeError(_lib.last_error())

    def timed(launches, steps, warmup):
        # an idle GPU starts at low clocks: run untimed until 30 ms have passed (matters for the
        # workloads whose whole timed region is a few milliseconds), then the W warm-up steps
        spin = time.perf_counter()
        i = 0
        while time.perf_counter() - spin < 0.03:
            step(launches, i)
            i += 1
            if i % 64 == 0:
                torch.cuda.synchronize()
        for i in range(warmup):
            step(launches, i)
        torch.cuda.synchronize()
        t = time.perf_counter()
        for i in range(steps):
            step(launches, warmup + i)
        torch.cuda.synchronize()
        return (time.perf_counter() - t) * 1e3 / steps

    def timed_median(launches, steps, warmup, reps=5):
        runs = sorted(timed(launches, steps, warmup) for _ in range(reps))
        return runs[len(runs) // 2], runs[0], runs[-1]

    if a.kernel_loop_only:
        return {"ms_per_step": timed(pat_launches, steps, warmup), "steps": steps, "warmup": warmup}
    ms_per_step, ms_fastest, ms_slowest = timed_median(pat_launches, steps, warmup)

    # the record kernel of this plan (once per plan, outside the timed loop): HIP-event time of 5 builds
    rec_bytes = C.c_size_t(0)
    lib.pat_fwd_records_bytes(C.byref(pat_launches[0].args), C.byref(rec_bytes))
    rec_buf = torch.empty(max(rec_bytes.value, 256), dtype=torch.uint8, device=dev)
    rec_tag = C.c_uint64(0)
    rec_ev = [(hip.event(), hip.event()) for _ in range(5)]
    for e0, e1 in rec_ev:
        hip.record(e0, stream)
        rc = lib.pat_fwd_build_records(C.byref(pat_launches[0].args), C.c_void_p(rec_buf.data_ptr()), rec_bytes.value,
                                       C.byref(rec_tag), C.c_void_p(stream))
        assert rc == 0, _lib.last_error()
        hip.record(e1, stream)
    torch.cuda.synchronize()
    records_build_us = sorted(hip.ms(e0, e1) for e0, e1 in rec_ev)[2] * 1e3

    # per-kernel durations from HIP events on the launch stream (same step sequence)
    n_ev = min(steps, 100)
    ev = [(hip.event(), hip.event(), hip.event()) for _ in range(n_ev)]
    for i, (e0, e1, e2) in enumerate(ev):
        L = pat_launches[i % copies]
        L.args.split_done_event = e1
        hip.record(e0, stream)
        step(pat_launches, i)
        hip.record(e2, stream)
        L.args.split_done_event = None
    torch.cuda.synchronize()
    split_ms = sorted(hip.ms(e0, e1) for e0, e1, _ in ev)
    merge_ms = sorted(hip.ms(e1, e2) for _, e1, e2 in ev)
    call_ms = sorted(hip.ms(e0, e2) for e0, _, e2 in ev)
    mean = lambda xs: sum(xs) / len(xs)
    median = lambda xs: xs[len(xs) // 2]

    unique_bytes = w.unique_kv_bytes
    value = unique_bytes / (ms_per_step * 1e-3) / 1e9
    # An event record between two kernels costs the stream a pause of its own (1-3 us): the two
    # event intervals of a call add up to more than a free-running call. That surplus, shared equally
    # by the two intervals, is taken off to get the kernels' durations (rocprofv3's kernel trace of the
    # same loop agrees with the corrected figure, see profiles/).
    event_overhead_ms = max(0.0, (mean(split_ms) + mean(merge_ms) - ms_per_step) / 2)
    split_mean_ms = mean(split_ms) - event_overhead_ms
    achieved = unique_bytes / (split_mean_ms * 1e-3) / 1e9

    geo = _lib.FwdGeometry()
    lib.pat_fwd_geometry_of(C.byref(pat_launches[0].args), C.byref(geo))

    result = {
        "metric": "decode-attn us/call + unique-KV HBM GB/s (% of peak), Llama-3-8B shapes",
        "value": round(value, 2),
        "unit": "GB/s",
        "n_gpus": 1,
        "steps": steps,
        "warmup": warmup,
        "ms_per_step": round(ms_per_step, 6),
        "ms_per_step_spread": [round(ms_fastest, 6), round(ms_slowest, 6)],
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "bf16" if w.dtype == torch.bfloat16 else "f16",
        "data": "synthetic",
        "config": {"workload": f"{workload}: {WORKLOAD_TEXT[workload]}", "batch": w.batch,
                   "heads": w.heads, "kv_heads": w.kv_heads, "head_dim": w.head_dim, "page_size": w.page_size,
                   "seed": a.seed, "unique_kv_tokens": w.unique_tokens, "total_kv_tokens": w.total_tokens,
                   "kv_cache_copies_rotated": copies, "tree": w.tree},
        "us_per_call": round(ms_per_step * 1e3, 3),
        "pct_of_hbm_peak": round(100 * value / HBM_PEAK_GBPS, 2),
        "unique_kv_bytes": unique_bytes,
        "oblivious_kv_bytes": w.kv_bytes(w.total_tokens),
        # what the plan's work items read between them (L2 serves the re-reads of shared nodes)
        "plan_kv_bytes": w.kv_bytes(int(sum(int(kv.sum()) for kv in info.kv_in_CTAs))),
        "event_us": {"call_median": round(median(call_ms) * 1e3, 3), "split_mean": round(split_mean_ms * 1e3, 3),
                     "split_interval_mean": round(mean(split_ms) * 1e3, 3),
                     "merge_mean": round((mean(merge_ms) - event_overhead_ms) * 1e3, 3),
                     "merge_interval_mean": round(mean(merge_ms) * 1e3, 3),
                     "event_overhead_per_interval": round(event_overhead_ms * 1e3, 3)},
        "launched_as": "one work item per request" if whole is not None else "planned",
        "geometry": {"chunk_tokens": geo.chunk_tokens, "tall_chunk_tokens": geo.tall_chunk_tokens,
                     "chunks_per_rank": geo.chunks_per_rank, "workgroups": geo.num_workgroups},
        "plan_build_ms_host": round(plan_ms, 3),
        "plan_build_first_call_ms": round(plan_first_ms, 3),
        "tree_next_step_ms_host": dict(zip(("edited_in_place", "built_anew"), (round(x, 4) for x in plan_next_step()))),
        "records_build_us": round(records_build_us, 2),
        "autotune": None,
        "roofline": {"bound": "hbm", "kernel": "pat_split_kernel", "achieved": round(achieved, 2),
                     "peak": HBM_PEAK_GBPS, "unit": "GB/s", "frac": round(achieved / HBM_PEAK_GBPS, 4),
                     "traffic": None},
    }

    result["roofline"]["traffic"] = measured_traffic_bytes(workload, a.seed, int(geo.num_workgroups))

    if not a.no_autotune:
        # What the optional measured choice of the geometry would give (pat_fwd_autotune; off by default
        # in the product: it synchronises the stream and runs the launch some fifty times), and what the
        # measurement costs in wall time.
        torch.cuda.synchronize()
        t = time.perf_counter()
        tuned_launches, tuned_ws = prepare(pat_kw, pat_slots, True)
        torch.cuda.synchronize()
        tune_ms = (time.perf_counter() - t) * 1e3
        tuned_ms, _, _ = timed_median(tuned_launches, steps, warmup)
        L0 = tuned_launches[0]
        result["autotune"] = {
            "chosen": {f: getattr(L0.tuning, f) for f, _ in _lib.FwdTuning._fields_},
            "tuned_us_per_call": round(tuned_ms * 1e3, 3),
            "untuned_us_per_call": round(ms_per_step * 1e3, 3),
            "autotune_wall_ms": round(tune_ms, 2),
            "tuning_run_us": {"chosen": round(L0.tuned_us, 2), "automatic": round(L0.auto_us, 2)}}
        del tuned_launches, tuned_ws

    # the same steps through the drop-in call of the compiled extension (tree form): argument checks
    # and launch preparation are cached per (q, k, v, out), the workspace comes from torch's
    # caching allocator at every call
    def api_step(i):
        prefix_attn_with_kvcache(q, ks[i % copies], vs[i % copies], tree, scale, out)

    for i in range(max(warmup, copies)):
        api_step(i)
    torch.cuda.synchronize()
    t = time.perf_counter()
    for i in range(steps):
        api_step(i)
    torch.cuda.synchronize()
    result["api_us_per_call"] = round((time.perf_counter() - t) * 1e6 / steps, 3)

    if not a.no_oblivious:
        ob = workloads.oblivious_plan(w, dev)
        ob_kw = {k: ob[k] for k in pat_kw}
        ob_launches, ob_ws = prepare(ob_kw, None, False)
        ob_ms, _, _ = timed_median(ob_launches, steps, warmup, reps=3)
        result["oblivious_us_per_call"] = round(ob_ms * 1e3, 3)
        result["speedup_vs_oblivious"] = round(ob_ms / ms_per_step, 3)

    if headline and not a.no_cpu_baseline:
        from oracle import attn_oracle
        qc, kc, vc = q.cpu(), ks[0].cpu(), vs[0].cpu()
        cores = os.cpu_count() or 1
        cores = min(cores, int(os.environ.get("OMP_NUM_THREADS", cores)))
        torch.set_num_threads(cores)
        attn_oracle.paged_attention_ref(qc, kc, vc, w.rows, w.seq_lens, scale)    # warm-up
        runs, t_cpu = 0, 0.0
        while runs < 5 and t_cpu < 20.0:
            t = time.perf_counter()
            attn_oracle.paged_attention_ref(qc, kc, vc, w.rows, w.seq_lens, scale)
            t_cpu += time.perf_counter() - t
            runs += 1
        cpu_s = t_cpu / runs
        result["cpu_baseline"] = {"value": round(unique_bytes / cpu_s / 1e9, 4), "unit": "GB/s",
                                  "cores": torch.get_num_threads(), "kind": "port",
                                  "us_per_call": round(cpu_s * 1e6, 1),
                                  "sample": f"whole {workload} batch, fp32 PyTorch restatement of the reference's "
                                            f"attention_ref over gathered dense KV, mean of {runs} runs after 1 warm-up"}
    return result


def main() -> None:
    ap = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--workload", default="c2", choices=sorted(WORKLOAD_TEXT))
    ap.add_argument("--seed", type=int, default=0)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-oblivious", action="store_true")
    ap.add_argument("--no-autotune", action="store_true",
                    help="skip the side measurement of what pat_fwd_autotune would choose (the headline never uses it)")
    ap.add_argument("--no-configs", action="store_true",
                    help="do not measure the other benchmark workloads beside the named one")
    ap.add_argument("--kernel-loop-only", action="store_true",
                    help="run only warmup + timed steps (for rocprofv3 runs)")
    ap.add_argument("--calibrate-copy-mib", type=int, default=0,
                    help="instead of the benchmark, run a plain elementwise copy of this many MiB 5 times "
                         "(reads N, writes N bytes): the known-size kernel that scales rocprofv3's "
                         "FETCH_SIZE / WRITE_SIZE readings")
    a = ap.parse_args()
    if a.gpus != 1:
        print("bench.py: this build runs on ONE GPU (the path has no cross-GPU step); use --gpus 1",
              file=sys.stderr)
        sys.exit(2)

    import torch

    assert torch.cuda.is_available(), "bench.py needs an AMD GPU"
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    if a.calibrate_copy_mib > 0:
        n = a.calibrate_copy_mib << 20
        src = torch.ones(n // 4, dtype=torch.float32, device=dev)
        dst = torch.empty_like(src)
        for _ in range(5):
            torch.mul(src, 1.0, out=dst)        # one elementwise kernel: reads n bytes, writes n bytes
        torch.cuda.synchronize()
        print(json.dumps({"calibration_copy_bytes": n, "launches": 5}))
        return
    steps, warmup = a.steps, a.warmup
    result = measure(a, a.workload, steps, warmup, headline=True)
    if a.workload == "c2" and not a.no_configs and not a.kernel_loop_only:
        # the other benchmark workloads, measured the same way (fewer steps; CPU baseline for c2 only)
        result["configs"] = []
        for name in ("c1", "c3", "c4", "c5a", "c5b"):
            r = measure(a, name, max(20, min(steps, 100)), warmup, headline=False)
            result["configs"].append({
                "workload": r["config"]["workload"], "us_per_call": r["us_per_call"],
                "api_us_per_call": r["api_us_per_call"], "unique_kv_gbps": r["value"],
                "pct_of_hbm_peak": r["pct_of_hbm_peak"], "split_us": r["event_us"]["split_mean"],
                "merge_us": r["event_us"]["merge_mean"], "frac": r["roofline"]["frac"],
                "oblivious_us_per_call": r.get("oblivious_us_per_call"),
                "speedup_vs_oblivious": r.get("speedup_vs_oblivious"), "workgroups": r["geometry"]["workgroups"],
                "dtype": r["dtype"]})
    print(json.dumps(result))


if __name__ == "__main__":
    main()
