"""The entry point that allocates nothing (pat_fwd_launch_static) against pat_fwd_launch, through
the C ABI: same kernels, the partial results in the library's built-in scratch array instead of a
caller's workspace. Two calls in a row, the second on a smaller batch (the scratch keeps the first
call's contents), bit-identical outputs required. Then the use it exists for: the call captured into
a HIP graph and replayed, every replay against an eager pat_fwd_launch."""
import ctypes as C
import math

import pytest
import torch

from pat_amd import PrefixTreeCPP, _ctypes_launch, _lib, workloads

pytestmark = pytest.mark.gpu


def _both_routes(name, w, dev):
    lib = _lib.load()
    q, k, v = w.tensors(dev)
    tree = PrefixTreeCPP(w.page_size)
    tree.build_radix_tree(w.seq_lens, w.padded_table())
    tree.pack_schedule(None, w.heads // w.kv_heads, w.kv_heads)
    info = tree.kernel_info
    info.to_gpu(dev)
    lt = info.launch_tables()
    results = []
    for static in (False, True):
        out = torch.full_like(q, float("nan"))
        lse = torch.full((w.batch, w.heads), float("nan"), dtype=torch.float32, device=dev)
        L = _ctypes_launch.prepare(q, k, v, info.num_boxes_per_seq, lt["q_tables"], lt["block_tables"],
                                  lt["num_seqs_per_CTAs"], lt["CTA_ranks"], lt["kv_in_CTAs"], lt["MNWs"],
                                  info.max_boxes_per_seq, info.max_seqs_in_CTA, info.max_blocks_in_CTA,
                                  1.0 / math.sqrt(w.head_dim), out, lse, lt["slot_tables"], lt.get("flags"))
        assert 0 < L.need <= lib.pat_fwd_static_scratch_bytes()
        stream = C.c_void_p(torch.cuda.current_stream(dev).cuda_stream)
        if static:
            L.args.workspace, L.args.workspace_bytes = None, 0
            rc = lib.pat_fwd_launch_static(C.byref(L.args), stream)
        else:
            ws = torch.empty(L.need, dtype=torch.uint8, device=dev)
            L.args.workspace, L.args.workspace_bytes = ws.data_ptr(), L.need
            rc = lib.pat_fwd_launch(C.byref(L.args), stream)
        assert rc == 0, _lib.last_error()
        torch.cuda.synchronize()
        results.append((out, lse))
    (out_a, lse_a), (out_b, lse_b) = results
    print(f"[no-alloc] {name}: workspace {L.need} bytes, outputs identical: {torch.equal(out_a, out_b)}", flush=True)
    assert not torch.isnan(out_b.float()).any() and not torch.isnan(lse_b).any()
    assert torch.equal(out_a, out_b) and torch.equal(lse_a, lse_b)


def test_static_scratch_entry_point_matches_workspace_entry_point():
    assert torch.cuda.is_available(), "GPU tests need an AMD GPU"
    dev = torch.device("cuda:0")
    print("[case] pat_fwd_launch_static vs pat_fwd_launch: c2, then the smaller c1", flush=True)
    _both_routes("c2", workloads.make("c2", seed=0), dev)
    _both_routes("c1", workloads.make("c1", seed=0), dev)   # smaller: stale partial results stay behind it


def test_static_scratch_entry_point_under_graph_capture():
    # what the entry point is for: a caller that captures the call into a HIP graph (no allocation
    # may happen there) and replays it; every replay against an eager pat_fwd_launch on the same inputs
    assert torch.cuda.is_available(), "GPU tests need an AMD GPU"
    dev = torch.device("cuda:0")
    print("[case] pat_fwd_launch_static captured into a HIP graph and replayed, c2", flush=True)
    lib = _lib.load()
    w = workloads.make("c2", seed=3)
    q, k, v = w.tensors(dev)
    tree = PrefixTreeCPP(w.page_size)
    tree.build_radix_tree(w.seq_lens, w.padded_table())
    tree.pack_schedule(None, w.heads // w.kv_heads, w.kv_heads)
    info = tree.kernel_info
    info.to_gpu(dev)
    lt = info.launch_tables()
    q_static = q.clone()
    out_graph = torch.zeros_like(q)
    out_eager = torch.zeros_like(q)

    def prepared(qq, oo):
        return _ctypes_launch.prepare(qq, k, v, info.num_boxes_per_seq, lt["q_tables"], lt["block_tables"],
                                      lt["num_seqs_per_CTAs"], lt["CTA_ranks"], lt["kv_in_CTAs"], lt["MNWs"],
                                      info.max_boxes_per_seq, info.max_seqs_in_CTA, info.max_blocks_in_CTA,
                                      1.0 / math.sqrt(w.head_dim), oo, None, lt["slot_tables"], lt.get("flags"))

    Lg, Le = prepared(q_static, out_graph), prepared(q_static, out_eager)
    Lg.args.workspace, Lg.args.workspace_bytes = None, 0
    ws = torch.empty(Le.need, dtype=torch.uint8, device=dev)
    Le.args.workspace, Le.args.workspace_bytes = ws.data_ptr(), Le.need
    # first call outside the capture (it looks up the scratch array's address once per device)
    assert lib.pat_fwd_launch_static(C.byref(Lg.args), C.c_void_p(torch.cuda.current_stream(dev).cuda_stream)) == 0, _lib.last_error()
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        rc = lib.pat_fwd_launch_static(C.byref(Lg.args), C.c_void_p(torch.cuda.current_stream(dev).cuda_stream))
    assert rc == 0, _lib.last_error()
    gen = torch.Generator(device="cpu").manual_seed(11)
    for trial in range(3):
        q_static.copy_(torch.randn(q.shape, generator=gen).to(w.dtype).to(dev))
        out_graph.fill_(float("nan"))
        out_eager.fill_(float("nan"))
        assert lib.pat_fwd_launch(C.byref(Le.args), C.c_void_p(torch.cuda.current_stream(dev).cuda_stream)) == 0, _lib.last_error()
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out_graph, out_eager), f"replay {trial} differs from the eager call"


def test_static_scratch_entry_point_without_prebuilt_records():
    # args.records == NULL: the split kernel decodes the plan tables per workgroup instead of reading
    # launch records; same results as the workspace entry point with records
    assert torch.cuda.is_available(), "GPU tests need an AMD GPU"
    dev = torch.device("cuda:0")
    print("[case] pat_fwd_launch_static with records == NULL vs pat_fwd_launch with records, c2 and c3", flush=True)
    lib = _lib.load()
    for name in ("c2", "c3"):
        w = workloads.make(name, seed=5)
        q, k, v = w.tensors(dev)
        tree = PrefixTreeCPP(w.page_size)
        tree.build_radix_tree(w.seq_lens, w.padded_table())
        tree.pack_schedule(None, w.heads // w.kv_heads, w.kv_heads)
        info = tree.kernel_info
        info.to_gpu(dev)
        lt = info.launch_tables()
        outs = []
        for static in (False, True):
            out = torch.full_like(q, float("nan"))
            lse = torch.full((w.batch, w.heads), float("nan"), dtype=torch.float32, device=dev)
            L = _ctypes_launch.prepare(q, k, v, info.num_boxes_per_seq, lt["q_tables"], lt["block_tables"],
                                      lt["num_seqs_per_CTAs"], lt["CTA_ranks"], lt["kv_in_CTAs"], lt["MNWs"],
                                      info.max_boxes_per_seq, info.max_seqs_in_CTA, info.max_blocks_in_CTA,
                                      1.0 / math.sqrt(w.head_dim), out, lse, lt["slot_tables"], lt.get("flags"),
                                      build_records=not static)
            assert (L.args.records is None or L.args.records == 0) == static
            stream = C.c_void_p(torch.cuda.current_stream(dev).cuda_stream)
            if static:
                if L.need > lib.pat_fwd_static_scratch_bytes():
                    pytest.skip(f"{name} needs {L.need} bytes of partial results")
                L.args.workspace, L.args.workspace_bytes = None, 0
                rc = lib.pat_fwd_launch_static(C.byref(L.args), stream)
            else:
                ws = torch.empty(L.need, dtype=torch.uint8, device=dev)
                L.args.workspace, L.args.workspace_bytes = ws.data_ptr(), L.need
                rc = lib.pat_fwd_launch(C.byref(L.args), stream)
            assert rc == 0, _lib.last_error()
            torch.cuda.synchronize()
            outs.append((out, lse))
        assert not torch.isnan(outs[1][0].float()).any()
        assert torch.equal(outs[0][0], outs[1][0]) and torch.equal(outs[0][1], outs[1][1]), name


_FIRST_CALL_CAPTURED = r"""
import ctypes as C, math, sys, torch
from pat_amd import PrefixTreeCPP, _ctypes_launch, _lib, workloads
dev = torch.device("cuda:0")
lib = _lib.load()
w = workloads.make("c1", seed=0)
q, k, v = w.tensors(dev)
tree = PrefixTreeCPP(w.page_size)
tree.build_radix_tree(w.seq_lens, w.padded_table())
tree.pack_schedule(None, w.heads // w.kv_heads, w.kv_heads)
info = tree.kernel_info
info.to_gpu(dev)
lt = info.launch_tables()
out = torch.zeros_like(q)
L = _ctypes_launch.prepare(q, k, v, info.num_boxes_per_seq, lt["q_tables"], lt["block_tables"], lt["num_seqs_per_CTAs"],
                           lt["CTA_ranks"], lt["kv_in_CTAs"], lt["MNWs"], info.max_boxes_per_seq, info.max_seqs_in_CTA,
                           info.max_blocks_in_CTA, 1.0 / math.sqrt(w.head_dim), out, None, lt["slot_tables"], lt.get("flags"))
L.args.workspace, L.args.workspace_bytes = None, 0
torch.cuda.synchronize()
graph = torch.cuda.CUDAGraph()
with torch.cuda.graph(graph):
    rc = lib.pat_fwd_launch_static(C.byref(L.args), C.c_void_p(torch.cuda.current_stream(dev).cuda_stream))
msg = _lib.last_error()
torch.cuda.synchronize()
# after one call outside a capture the same call captures
rc2 = lib.pat_fwd_launch_static(C.byref(L.args), C.c_void_p(torch.cuda.current_stream(dev).cuda_stream))
torch.cuda.synchronize()
graph2 = torch.cuda.CUDAGraph()
with torch.cuda.graph(graph2):
    rc3 = lib.pat_fwd_launch_static(C.byref(L.args), C.c_void_p(torch.cuda.current_stream(dev).cuda_stream))
eager = out.clone()
out.zero_()
graph2.replay()
torch.cuda.synchronize()
print("RC", rc, rc2, rc3, bool(torch.equal(eager, out)), "|", msg, flush=True)
"""


def test_static_scratch_first_call_under_capture_is_refused():
    # a fresh process whose first pat_fwd_launch_static on the device is made under stream capture:
    # a clear error and nothing enqueued; after one call outside a capture the same call captures
    import os
    import subprocess
    import sys
    assert torch.cuda.is_available(), "GPU tests need an AMD GPU"
    print("[case] pat_fwd_launch_static: first call on the device under capture, fresh process", flush=True)
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    r = subprocess.run([sys.executable, "-c", _FIRST_CALL_CAPTURED], cwd=root, capture_output=True, text=True, timeout=300)
    assert r.returncode == 0, r.stdout + r.stderr
    line = [ln for ln in r.stdout.splitlines() if ln.startswith("RC ")][-1]
    rc, rc2, rc3, same = line.split("|")[0].split()[1:5]
    assert int(rc) != 0 and "capture" in line.split("|", 1)[1], line
    assert int(rc2) == 0 and int(rc3) == 0 and same == "True", line
