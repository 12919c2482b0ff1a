"""Writes tests/golden/flat_plans.json.gz: inputs and plans produced by the reference's
legacy flat scheduler `prefix_attn.block_scheduler.schedule`.

Run in the build container only (needs /root/reference, which never travels):

    python tests/golden/make_flat_fixtures.py

Why the reference is imported here: the reference holds no test or vector for
`schedule`; the one worked example in its tree (the docstring of `pack_prefix_blocks`)
covers a single regular batch and none of the lexsort permutation, the run splitting on
unsorted neighbours, the k-chunking or the ends-inside-a-shared-run length rule. Four
pure-Python files are loaded (data_class, utils, prefix_tree, block_scheduler) under a
stub parent package, because the package's __init__ needs its compiled CUDA extension.

The fixtures hold data only: lengths, block-table rows, call arguments and the lists the
scheduler returned.
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
REF = "/root/reference/prefix_attn"


def load_reference():
    pkg = types.ModuleType("_ref_pa")
    pkg.__path__ = [REF]
    sys.modules["_ref_pa"] = pkg
    mods = {}
    for name in ("data_class", "utils", "prefix_tree", "block_scheduler"):
        spec = importlib.util.spec_from_file_location(f"_ref_pa.{name}", os.path.join(REF, f"{name}.py"))
        mod = importlib.util.module_from_spec(spec)
        sys.modules[f"_ref_pa.{name}"] = mod
        spec.loader.exec_module(mod)
        mods[name] = mod
    return mods["block_scheduler"].schedule


def batch(rng: random.Random, shape: str, bs: int):
    """(seq_lens, rows): shared-prefix batches in arrival (unsorted) order."""
    next_id = [1]

    def fresh(n):
        ids = list(range(next_id[0], next_id[0] + n))
        next_id[0] += n
        return ids

    rows, lens = [], []

    def emit(prefix, own_blocks):
        row = prefix + fresh(own_blocks)
        rows.append(row)
        lens.append((len(row) - 1) * bs + rng.randint(1, bs))

    if shape == "two_level":
        root = fresh(rng.randint(1, 6))
        for _ in range(rng.randint(2, 5)):
            mid = root + fresh(rng.randint(1, 4))
            for _ in range(rng.randint(1, 6)):
                emit(mid, rng.randint(0, 3))
    elif shape == "forest":
        for _ in range(rng.randint(2, 4)):
            root = fresh(rng.randint(1, 5))
            for _ in range(rng.randint(1, 7)):
                emit(root, rng.randint(0, 4))
    elif shape == "wide":
        root = fresh(rng.randint(1, 3))
        for _ in range(rng.randint(9, 40)):
            emit(root, rng.randint(0, 2))
    else:  # independent
        for _ in range(rng.randint(1, 8)):
            emit([], rng.randint(1, 6))
    rows = [r if r else fresh(1) for r in rows]
    lens = [max(n, 1) for n in lens]
    order = list(range(len(rows)))
    rng.shuffle(order)
    return [lens[i] for i in order], [rows[i] for i in order]


def main():
    schedule = load_reference()
    rng = random.Random(20240611)
    tiles_options = [None, [[64, 128, 4]], [[16, 128, 1], [32, 128, 2], [64, 128, 4]]]
    cases = []
    for shape in ("two_level", "forest", "wide", "independent"):
        for _ in range(8):
            bs = rng.choice([16, 32])
            lens, rows = batch(rng, shape, bs)
            tiles = rng.choice(tiles_options)
            ratio = rng.choice([1, 2, 4])
            k = rng.choice([4, 8, 16, 64])
            if tiles is not None:
                k = min(k, max(t[0] for t in tiles) // ratio)   # every item must fit some tile
            else:
                k = min(k, 64 // ratio)
            ki = schedule(list(lens), [list(r) for r in rows], bs, k,
                          None if tiles is None else [list(t) for t in tiles], ratio)
            cases.append({
                "shape": shape, "block_size": bs, "k": k, "tiles": tiles, "ratio": ratio,
                "seq_lens": lens, "rows": rows,
                "plan": {
                    "MNWs": [list(m) for m in ki.MNWs],
                    "q_tables": ki.q_tables, "block_tables": ki.block_tables,
                    "num_seqs_per_CTAs": ki.num_seqs_per_CTAs, "CTA_ranks": ki.CTA_ranks,
                    "kv_in_CTAs": ki.kv_in_CTAs, "num_split_per_seq": list(ki.num_split_per_seq),
                    "max_split_per_seq": int(ki.max_split_per_seq), "max_seqs_in_CTA": int(ki.max_seqs_in_CTA),
                    "max_blocks_in_CTA": int(ki.max_blocks_in_CTA),
                    "reverse_index": [int(x) for x in ki.reverse_index],
                    "sort_index": [int(x) for x in ki.sort_index],
                },
            })
    path = os.path.join(HERE, "flat_plans.json.gz")
    with gzip.GzipFile(path, "wb", mtime=0) as f:
        f.write(json.dumps({"cases": cases}, separators=(",", ":")).encode())
    print(f"{len(cases)} cases -> {path} ({os.path.getsize(path)} bytes)")


if __name__ == "__main__":
    main()
