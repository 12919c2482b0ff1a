"""Writes tests/golden/plans_*.json.gz: inputs and plans produced by the reference's own
Python scheduler.

Run in the build container only (needs /root/reference, which never travels):

    python tests/golden/make_plan_fixtures.py

Why the reference is imported here: box *ordering* and rank assignment on irregular
forests, the float `ceil` chunking of the balancer on mixed-length batches, the
merge-vs-split decisions with a running sequence count, the compute-model variant and
`naive_schedule` are not fixed by any vector, closed form or invariant the reference
holds; only its scheduler can say what it emits there. Two pure-Python files are
loaded (prefix_attn/prefix_tree.py and prefix_attn/data_class.py) under a stub parent
package, because the package's __init__ needs its compiled CUDA extension.

The fixtures hold data only: block-table rows, lengths, call arguments, and the lists
the scheduler returned (or the name of the exception it raised).
"""
from __future__ import annotations

import gzip
import importlib.util
import json
import os
import random
import sys
import types

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
REF = "/root/reference/prefix_attn"
sys.path.insert(0, ROOT)


def load_reference():
    pkg = types.ModuleType("_ref_pa")
    pkg.__path__ = [REF]
    sys.modules["_ref_pa"] = pkg
    mods = {}
    for name in ("data_class", "prefix_tree"):
        spec = importlib.util.spec_from_file_location(f"_ref_pa.{name}", os.path.join(REF, f"{name}.py"))
        mod = importlib.util.module_from_spec(spec)
        sys.modules[f"_ref_pa.{name}"] = mod
        spec.loader.exec_module(mod)
        mods[name] = mod
    return mods["prefix_tree"].PrefixTree


def plan_dict(ki) -> dict:
    return {
        "MNWs": [list(m) for m in ki.MNWs],
        "q_tables": ki.q_tables,
        "block_tables": ki.block_tables,
        "num_seqs_per_CTAs": ki.num_seqs_per_CTAs,
        "CTA_ranks": ki.CTA_ranks,
        "kv_in_CTAs": ki.kv_in_CTAs,
        "num_split_per_seq": list(ki.num_split_per_seq),
        "max_split_per_seq": ki.max_split_per_seq,
        "max_seqs_in_CTA": ki.max_seqs_in_CTA,
        "max_blocks_in_CTA": ki.max_blocks_in_CTA,
    }


def tree_dict(t) -> dict:
    return {
        "parents": list(t.parents), "s_values": list(t.s_values), "lens": list(t.lens),
        "seq_indices": [list(x) for x in t.seq_indices], "block_ids": [list(x) for x in t.block_ids],
        "children": [list(t.tree[i].values()) if i in t.tree else [] for i in range(t.num_nodes)],
    }


def run_case(PrefixTree, case: dict, with_tree: bool) -> dict:
    out = dict(case)
    try:
        t = PrefixTree(case["block_size"])
        t.build_radix_tree(list(case["seq_lens"]), [list(r) for r in case["rows"]])
        if with_tree:
            out["tree"] = tree_dict(t)
        plans = []
        for call in case["calls"]:
            if call["kind"] == "naive":
                ki = t.naive_schedule(call["HRatio"])
            else:
                ki = t.pack_schedule(call["MNWs"], call["HRatio"], call["kvHead"], call["use_compute_model"])
            plans.append(json.loads(json.dumps(plan_dict(ki))))   # deep copy: lists alias tree state
        out["plans"] = plans
    except Exception as exc:  # the exception type is part of the observable behaviour
        out["raises"] = type(exc).__name__
    return out


def pack(hratio, kvhead, mnws=None, model=False):
    return {"kind": "pack", "MNWs": mnws, "HRatio": hratio, "kvHead": kvhead, "use_compute_model": model}


def tree_spec_rows(spec: str, bs: int, rng: random.Random):
    """Rows of the reference's "n1,..,nk_l1,..,lk" tree batches (prefix_attn/utils.py:49-100 shape)."""
    counts_s, lens_s = spec.split("_")
    counts = [int(x) for x in counts_s.split(",")]
    lens = [int(x) for x in lens_s.split(",")]
    batch = counts[-1]
    nxt, levels = 0, []
    for c, l in zip(counts, lens):
        nodes = []
        for _ in range(c):
            nodes.append(list(range(nxt, nxt + l // bs)))
            nxt += l // bs
        levels.append(nodes)
    slots = list(range(batch))
    rng.shuffle(slots)
    rows = [None] * batch
    for i in range(batch):
        row = []
        for c, nodes in zip(counts, levels):
            row.extend(nodes[i // (batch // c)])
        rows[slots[i]] = row
    return [sum(lens)] * batch, rows


def random_forest_rows(rng: random.Random, bs: int, batch: int, ragged: bool, allow_prefix_seqs: bool):
    """Random radix-like batches: sequences extend or branch off earlier ones."""
    rows, lens, nxt = [], [], 0
    for i in range(batch):
        if rows and rng.random() < 0.8:
            base = rows[rng.randrange(len(rows))]
            keep = rng.randint(0 if not allow_prefix_seqs else 1, len(base))
            row = list(base[:keep])
        else:
            row = []
        extra = rng.randint(0 if (allow_prefix_seqs and row) else 1, 12)
        row += list(range(nxt, nxt + extra))
        nxt += extra
        if not row:
            row = [nxt]
            nxt += 1
        rows.append(row)
        full = len(row) * bs
        lens.append(full - (rng.randint(0, bs - 1) if ragged else 0))
    return lens, rows


def main() -> None:
    PrefixTree = load_reference()
    from pat_amd import workloads

    small, large = [], []

    # reference's manual fixture (test/test.py:233-239) and its commented-out variants
    small.append({"name": "manual_33x3", "block_size": 16, "seq_lens": [33, 33, 33],
                  "rows": [[0, 1, 5], [0, 2, 6], [3, 4, 7]], "calls": [pack(4, 8)]})
    small.append({"name": "manual_8seq", "block_size": 16,
                  "seq_lens": [17, 36, 44, 44, 32, 36, 44, 44],
                  "rows": [[1, 2], [1, 2, 3], [4, 5, 6], [4, 5, 7], [4, 8], [1, 9, 10], [4, 5, 11], [4, 5, 12]],
                  "calls": [pack(4, 8)]})
    small.append({"name": "manual_padded", "block_size": 16, "seq_lens": [38, 38, 15, 15],
                  "rows": [[1, 2, 6], [1, 5, 8], [3, 0, 0], [7, 0, 0]], "calls": [pack(4, 8)]})

    # benchmark configurations of this project
    for name in workloads.NAMES:
        w = workloads.make(name, seed=0)
        hr = w.heads // w.kv_heads
        case = {"name": f"workload_{name}", "block_size": w.page_size, "seq_lens": w.seq_lens, "rows": w.rows,
                "calls": [pack(hr, w.kv_heads)]}
        (small if name == "c1" else large).append(case)
        if name in ("c1", "c2", "c4"):
            large.append({**case, "name": f"workload_{name}_model", "calls": [pack(hr, w.kv_heads, None, True)]})
            large.append({**case, "name": f"workload_{name}_naive", "calls": [{"kind": "naive", "HRatio": hr}]})
    for seed in (1, 2):
        for name in ("c2", "c4", "c5a"):
            w = workloads.make(name, seed=seed)
            large.append({"name": f"workload_{name}_seed{seed}", "block_size": w.page_size, "seq_lens": w.seq_lens,
                          "rows": w.rows, "calls": [pack(w.heads // w.kv_heads, w.kv_heads)]})

    # tree batches of the reference's unit test (test/test.py:174-187; block 32, 64/8 heads)
    rng = random.Random(1234)
    test_trees = ["4_4096", "4,16_4096,256", "1,8_640,32", "1,4,16_32,256,32", "1,2,4,8,16,32,64_32,512,32,256,32,32,32",
                  "1,4,256_32,256,32", "1,16,32_2048,1024,256", "1,10_4096,416",
                  "1,2,4,16,32,64,128_512,32,128,128,32,256,512"]
    for spec in test_trees:
        lens, rows = tree_spec_rows(spec, 32, rng)
        large.append({"name": f"testtree_{spec}", "block_size": 32, "seq_lens": lens, "rows": rows,
                      "calls": [pack(8, 8)]})
    # tree batches of the kernel benchmark (benchmark/run_kernel_bench.sh:5-33; block 32), 4 head configs
    bench_trees = ["1,256_256,32", "1,2,64_1024,256,256", "1,4,8,256_32,256,256,32", "2,8,16,256_256,256,32,32",
                   "8,16,32,256_512,512,256,32", "256_1024"]
    for spec in bench_trees:
        lens, rows = tree_spec_rows(spec, 32, rng)
        for hq, hkv in ((32, 32), (16, 8), (32, 8), (64, 8)):
            large.append({"name": f"benchtree_{spec}_h{hq}_{hkv}", "block_size": 32, "seq_lens": lens, "rows": rows,
                          "calls": [pack(hq // hkv, hkv)]})

    # random forests: ragged lengths, duplicates, sequences that are prefixes of others
    for i in range(40):
        r = random.Random(100 + i)
        bs = r.choice([16, 16, 32])
        batch = r.choice([1, 2, 3, 5, 8, 13, 24, 40, 70])
        lens, rows = random_forest_rows(r, bs, batch, ragged=True, allow_prefix_seqs=(i % 4 == 3))
        hr, kvh = r.choice([(1, 8), (4, 8), (8, 8), (1, 32), (2, 16), (4, 4), (8, 2)])
        calls = [pack(hr, kvh)]
        if i % 5 == 1:
            calls = [pack(hr, kvh, None, True)]
        if i % 5 == 2:
            calls = [{"kind": "naive", "HRatio": hr}]
        if i % 7 == 3:
            calls = [pack(hr, kvh), pack(hr, kvh)]      # split counters carry over between calls
        small.append({"name": f"forest_{i}", "block_size": bs, "seq_lens": lens, "rows": rows, "calls": calls})
    # long boxes in a mixed batch: exercises the float ceil of the balancer's first phase
    for i in range(12):
        r = random.Random(500 + i)
        bs = 16
        shared = list(range(0, r.randint(300, 900)))
        nxt = len(shared)
        rows, lens = [], []
        for _ in range(r.choice([4, 9, 20, 33])):
            extra = r.randint(1, 40)
            rows.append(shared + list(range(nxt, nxt + extra)))
            nxt += extra
            lens.append(len(rows[-1]) * bs - r.randint(0, bs - 1))
        for _ in range(r.randint(0, 6)):
            extra = r.randint(20, 200)
            rows.append(list(range(nxt, nxt + extra)))
            nxt += extra
            lens.append(extra * bs)
        hr, kvh = r.choice([(4, 8), (8, 8), (1, 16), (8, 4)])
        large.append({"name": f"longbox_{i}", "block_size": bs, "seq_lens": lens, "rows": rows, "calls": [pack(hr, kvh)]})

    # bucket lists given by the caller
    lens, rows = tree_spec_rows("1,4,16_32,256,32", 32, rng)
    small.append({"name": "single_bucket", "block_size": 32, "seq_lens": lens, "rows": rows,
                  "calls": [pack(4, 8, [[64, 128, 4]])]})
    small.append({"name": "missing_bucket", "block_size": 32, "seq_lens": lens, "rows": rows,
                  "calls": [pack(4, 8, [[64, 128, 4], [16, 128, 1]])]})
    small.append({"name": "hratio_too_large", "block_size": 32, "seq_lens": lens, "rows": rows,
                  "calls": [pack(8, 8, [[16, 64, 1], [16, 128, 1]])]})
    small.append({"name": "hratio_zero_mm", "block_size": 32, "seq_lens": lens, "rows": rows,
                  "calls": [pack(32, 8, [[16, 64, 1], [16, 128, 1]])]})
    small.append({"name": "empty_batch", "block_size": 16, "seq_lens": [], "rows": [], "calls": [pack(1, 8)]})
    small.append({"name": "identical_rows", "block_size": 16, "seq_lens": [40, 40, 40], "rows": [[5, 6, 7]] * 3,
                  "calls": [pack(1, 8)]})

    for fname, cases, with_tree in (("plans_small.json.gz", small, True), ("plans_large.json.gz", large, False)):
        done = [run_case(PrefixTree, c, with_tree) for c in cases]
        path = os.path.join(HERE, fname)
        with gzip.GzipFile(path, "wb", mtime=0) as f:
            f.write(json.dumps(done, separators=(",", ":")).encode())
        raised = sum(1 for c in done if "raises" in c)
        print(f"{fname}: {len(done)} cases ({raised} raising), {os.path.getsize(path) / 1024:.0f} KiB")


if __name__ == "__main__":
    main()
