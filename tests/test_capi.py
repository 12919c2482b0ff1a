"""libpat_amd loads, exports every symbol include/pat_amd.h declares, and its GPU-free entry
points (argument validation, launch geometry, workspace size) behave. No kernel is launched."""
import ctypes as C
import os
import re

import pytest

from pat_amd import _lib

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared_functions():
    text = open(os.path.join(ROOT, "include", "pat_amd.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(pat_[a-z_0-9]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    lib = _lib.load()
    names = _declared_functions()
    assert len(names) >= 15
    for name in names:
        assert hasattr(lib, name), f"libpat_amd.so does not export {name}"
    assert sorted(_lib.SYMBOLS) == names       # the ctypes table covers the header, no more, no less
    assert lib.pat_abi_version() == 4


def _args(**over):
    """A well-formed pat_fwd_args with fake (never dereferenced) device addresses."""
    fake = 0x10000
    b = (_lib.FwdBucket * 2)()
    for i, (m, boxes, seqs, blocks) in enumerate([(64, 4, 16, 128), (16, 64, 1, 32)]):
        b[i].q_table = b[i].block_table = b[i].num_seqs = b[i].rank = b[i].kv = fake
        b[i].q_table_stride, b[i].block_table_stride = seqs, blocks
        b[i].num_boxes, b[i].max_seqs, b[i].max_blocks = boxes, seqs, blocks
        b[i].mnw[0], b[i].mnw[1], b[i].mnw[2] = m, 128, 4 if m == 64 else 1
    a = _lib.FwdArgs()
    a.dtype, a.batch, a.seqlen_q, a.heads, a.kv_heads = _lib.PAT_DTYPE_BF16, 64, 1, 32, 8
    a.head_dim, a.page_size, a.num_pages = 128, 16, 4096
    a.q = a.k = a.v = a.out = a.num_split_per_seq = fake
    a.q_stride = (C.c_int64 * 3)(4096, 4096, 128)
    a.k_stride = (C.c_int64 * 3)(16 * 8 * 128, 8 * 128, 128)
    a.v_stride = (C.c_int64 * 3)(16 * 8 * 128, 8 * 128, 128)
    a.o_stride = (C.c_int64 * 3)(4096, 4096, 128)
    a.max_split_per_seq, a.max_seqs_in_box, a.max_blocks_in_box = 2, 16, 128
    a.softmax_scale = 0.088
    a.num_buckets, a.buckets = 2, C.cast(b, C.POINTER(_lib.FwdBucket))
    a._keep = b
    for k, v in over.items():
        setattr(a, k, v)
    return a


def test_validate_accepts_headline_shape():
    lib = _lib.load()
    assert lib.pat_fwd_validate(C.byref(_args())) == 0


@pytest.mark.parametrize("field,value,needle", [
    ("dtype", 7, "only support fp16 and bf16"),
    ("max_split_per_seq", 33, "only supports up to 32 splits"),
    ("max_split_per_seq", 0, "no case that a seq has no block"),
    ("head_dim", 96, "head_size_og must be 64 / 128"),
    ("page_size", 24, "divisible by 16"),
    ("kv_heads", 5, "must divide number of heads"),
    ("kv_heads", 2, "hq/hkv = 1, 2, 4, 8"),
    ("batch", 0, "batch size must be positive"),
    ("seqlen_q", 2, "decode only"),
    ("q", 0, "non-null"),
    ("num_buckets", 13, "between 1 and 12"),
])
def test_validate_rejects(field, value, needle):
    lib = _lib.load()
    rc = lib.pat_fwd_validate(C.byref(_args(**{field: value})))
    assert rc == _lib.PAT_ERR_INVALID
    assert needle in _lib.last_error()
    with pytest.raises(RuntimeError):
        _lib.check(rc)


def test_validate_rejects_bad_bucket_and_strides():
    lib = _lib.load()
    a = _args()
    a.buckets[0].mnw[0] = 48
    assert lib.pat_fwd_validate(C.byref(a)) == _lib.PAT_ERR_INVALID and "tile_q" in _lib.last_error()
    a = _args()
    a.k_stride = (C.c_int64 * 3)(16 * 8 * 128 + 4, 8 * 128, 128)
    assert lib.pat_fwd_validate(C.byref(a)) == _lib.PAT_ERR_INVALID and "multiples of 8" in _lib.last_error()
    a = _args()
    a.v_stride = (C.c_int64 * 3)(1 << 30, 8 * 128, 128)          # blocks 2^30 elements apart
    assert lib.pat_fwd_validate(C.byref(a)) == _lib.PAT_ERR_INVALID and "2^30 elements apart" in _lib.last_error()
    a = _args()
    a.k_stride = (C.c_int64 * 3)(1 << 29, 1 << 25, 128)          # a 16-token block spanning 2^29 elements
    assert lib.pat_fwd_validate(C.byref(a)) == _lib.PAT_ERR_INVALID and "span less than 1 GiB" in _lib.last_error()
    a = _args()
    a.buckets[1].max_seqs = 32      # 32 sequences x 4 heads per kv head > 64 rows
    a.buckets[1].q_table_stride = 32
    assert lib.pat_fwd_validate(C.byref(a)) == _lib.PAT_ERR_INVALID and "64 rows" in _lib.last_error()
    a = _args()
    a.buckets[1].max_seqs = 8       # 8 sequences x 4 heads = 32 rows in a bucket labelled tile_q 16
    a.buckets[1].q_table_stride = 8
    assert lib.pat_fwd_validate(C.byref(a)) == _lib.PAT_ERR_INVALID and "than its bucket's tile_q" in _lib.last_error()
    a.buckets[1].mnw[0] = 32        # ... which a tile_q 32 bucket holds
    assert lib.pat_fwd_validate(C.byref(a)) == 0


def test_geometry_and_workspace_are_consistent():
    lib = _lib.load()
    a = _args()
    g = _lib.FwdGeometry()
    assert lib.pat_fwd_geometry_of(C.byref(a), C.byref(g)) == 0
    assert g.chunk_tokens % 32 == 0 and g.tall_chunk_tokens % 32 == 0
    # the whole launch is resident at two workgroups per CU: the tall boxes take the 32-row form and are cut
    # until there are about three tall workgroups per eight CUs: 3 pieces; the 64 boxes of up to 512 tokens
    # run a kv head per wave on 256-token pieces (2 per box, 2 head groups)
    assert g.tall_rows == 32
    per_box = [3, 2]
    assert -(-128 * 16 // g.tall_chunk_tokens) == per_box[0]
    assert g.chunks_per_rank == max(per_box)
    assert g.num_slots == g.chunks_per_rank * 2
    assert g.num_workgroups == 8 * 4 * per_box[0] + 64 * per_box[1] * (8 // 4)
    need = C.c_size_t()
    assert lib.pat_fwd_workspace_bytes(C.byref(a), C.byref(need)) == 0
    rows = 64 * 32 * g.num_slots
    assert need.value >= rows * 128 * 4 + rows * 4
    # launching without a workspace is refused before any GPU call
    a.workspace, a.workspace_bytes = 0, 0
    assert lib.pat_fwd_launch(C.byref(a), None) == _lib.PAT_ERR_WORKSPACE


def test_single_slot_launch_needs_no_workspace(tuning):
    # no sequence in two boxes (max_split_per_seq 1), every box one chunk, a box per CU and kv head:
    # the launch writes `out` from its first kernel (csrc/api.h:230-238) and, given the plan's
    # launch records, needs no scratch
    lib = _lib.load()
    fake = 0x10000

    def plan(boxes, blocks, **over):
        b = (_lib.FwdBucket * 1)()
        b[0].q_table = b[0].block_table = b[0].num_seqs = b[0].rank = b[0].kv = fake
        b[0].q_table_stride, b[0].block_table_stride = 1, blocks
        b[0].num_boxes, b[0].max_seqs, b[0].max_blocks = boxes, 1, blocks
        b[0].mnw[0], b[0].mnw[1], b[0].mnw[2] = 16, 128, 1
        kw = dict(batch=boxes, max_split_per_seq=1, max_seqs_in_box=1, max_blocks_in_box=blocks, num_buckets=1,
                  buckets=C.cast(b, C.POINTER(_lib.FwdBucket)), records=fake)
        kw.update(over)
        a = _args(**kw)
        a._keep = b
        g, need = _lib.FwdGeometry(), C.c_size_t()
        assert lib.pat_fwd_geometry_of(C.byref(a), C.byref(g)) == 0
        assert lib.pat_fwd_workspace_bytes(C.byref(a), C.byref(need)) == 0
        return g, need.value

    tuning()
    g, need = plan(64, 100)                       # 64 boxes of 1600 tokens, 8 kv heads: 512 workgroups
    assert (g.chunks_per_rank, g.num_slots, need) == (1, 1, 0)
    g, need = plan(64, 100, out=fake + 2)         # `out` not 8-byte aligned: the two-kernel route
    assert g.num_slots == 1 and need > 0
    g, need = plan(64, 100, max_split_per_seq=2)  # some sequence sits in two boxes
    assert need > 0
    g, need = plan(16, 100)                       # 128 workgroups: cutting the boxes fills the device
    assert g.chunks_per_rank > 1 and need > 0
    g, need = plan(64, 200)                       # 3200 tokens: longer than a chunk can be
    assert g.chunks_per_rank > 1 and need > 0
    tuning(direct_out=0)
    g, need = plan(64, 100)
    assert g.num_slots == 1 and need > 0
    # without prebuilt records the launch writes them into its workspace: one per workgroup
    tuning()
    g, need = plan(64, 100, records=0)
    rec = C.c_size_t()
    a = _args()
    assert need > 0 and need % 256 == 0 and need >= g.num_workgroups * 64


def test_record_buffer_sizes_and_errors_without_a_gpu():
    lib = _lib.load()
    a = _args()
    g, need, rec = _lib.FwdGeometry(), C.c_size_t(), C.c_size_t()
    assert lib.pat_fwd_geometry_of(C.byref(a), C.byref(g)) == 0
    assert lib.pat_fwd_records_bytes(C.byref(a), C.byref(rec)) == 0
    # a record: 32-byte header, sequence id and slot per sequence of the widest box (16), page ids of the
    # longest piece, rounded up to 64 bytes
    pages = max(g.chunk_tokens, g.tall_chunk_tokens) // 16
    assert rec.value >= g.num_workgroups * (32 + 2 * 16 * 4 + 4)
    assert rec.value <= 256 + g.num_workgroups * ((32 + 2 * 16 * 4 + pages * 4 + 63) // 64 * 64)
    # the launch's own workspace holds the partial results and, without prebuilt records, the records
    assert lib.pat_fwd_workspace_bytes(C.byref(a), C.byref(need)) == 0
    with_records = C.c_size_t()
    b = _args(records=0x20000)
    assert lib.pat_fwd_workspace_bytes(C.byref(b), C.byref(with_records)) == 0
    assert need.value == with_records.value + rec.value
    tag = C.c_uint64()
    assert lib.pat_fwd_build_records(C.byref(a), None, 0, C.byref(tag), None) == _lib.PAT_ERR_INVALID
    assert lib.pat_fwd_build_records(C.byref(a), C.c_void_p(0x10000), 16, C.byref(tag), None) == _lib.PAT_ERR_WORKSPACE
    assert lib.pat_fwd_build_records(C.byref(a), C.c_void_p(0x10010), rec.value, C.byref(tag), None) == _lib.PAT_ERR_WORKSPACE
    # records whose tag does not belong to this launch are refused before any GPU call
    b.workspace, b.workspace_bytes, b.records_bytes, b.records_tag = 0x100000, with_records.value, rec.value, 12345
    assert lib.pat_fwd_launch(C.byref(b), None) == _lib.PAT_ERR_INVALID and "launch records" in _lib.last_error()


def test_static_scratch_and_slot_buffer_sizes_without_a_gpu():
    lib = _lib.load()
    assert lib.pat_fwd_static_scratch_bytes() == 64 << 20
    a = _args()
    need = C.c_size_t()
    assert lib.pat_fwd_slots_bytes(C.byref(a), C.byref(need)) == 0
    # one count per sequence + one ordinal per q_table entry, each piece 256-byte aligned
    assert need.value == 256 + 256 + 256     # 64 counts, 4 x 16 and 64 x 1 entries
    offsets = (C.c_int64 * 2)()
    assert lib.pat_fwd_derive_slots(C.byref(a), None, 0, offsets, None) == _lib.PAT_ERR_INVALID
    assert lib.pat_fwd_derive_slots(C.byref(a), C.c_void_p(0x10000), 16, offsets, None) == _lib.PAT_ERR_WORKSPACE
    # a launch whose partial results exceed the built-in scratch is refused before any GPU call
    big = _args(batch=4096, max_split_per_seq=32)
    assert lib.pat_fwd_workspace_bytes(C.byref(big), C.byref(need)) == 0 and need.value > (64 << 20)
    assert lib.pat_fwd_launch_static(C.byref(big), None) == _lib.PAT_ERR_WORKSPACE
    assert "built-in scratch" in _lib.last_error()


def test_tuning_round_trip(tuning):
    lib = _lib.load()
    tuning(chunk_tokens=256, direct_out=0)
    t = _lib.FwdTuning()
    assert lib.pat_fwd_get_tuning(C.byref(t)) == 0
    assert (t.chunk_tokens, t.tall_chunk_tokens, t.head_per_wave_tokens, t.direct_out) == (256, 0, -1, 0)
    g = _lib.FwdGeometry()
    assert lib.pat_fwd_geometry_of(C.byref(_args()), C.byref(g)) == 0 and g.chunk_tokens == 256
    # the form of the tall path: chosen per launch unless set
    for rows in (32, 16):
        tuning(tall_rows=rows)
        assert lib.pat_fwd_geometry_of(C.byref(_args()), C.byref(g)) == 0 and g.tall_rows == rows
    tuning(tall_rows=16)
    assert lib.pat_fwd_geometry_of(C.byref(_args()), C.byref(g)) == 0
    assert -(-128 * 16 // g.tall_chunk_tokens) == 4      # the 16-row form: a tall workgroup per two CUs


def test_tree_handles_and_errors():
    lib = _lib.load()
    h = C.c_void_p()
    assert lib.pat_tree_create(0, C.byref(h)) == _lib.PAT_ERR_INVALID
    assert lib.pat_tree_create(16, C.byref(h)) == 0
    view = _lib.PlanView()
    assert lib.pat_tree_plan(h, C.byref(view)) == _lib.PAT_ERR_INVALID and "no plan" in _lib.last_error()
    assert lib.pat_tree_num_nodes(h) == 1
    nv = _lib.NodeView()
    assert lib.pat_tree_node(h, 5, C.byref(nv)) == _lib.PAT_ERR_INDEX
    lib.pat_tree_destroy(h)


def test_baseline_workspace_and_errors_without_a_gpu():
    lib = _lib.load()
    fake = 0x10000
    a = _lib.BaselineArgs()
    a.dtype, a.batch, a.heads, a.kv_heads, a.head_dim = _lib.PAT_DTYPE_F16, 32, 64, 8, 128
    a.page_size, a.num_pages, a.max_blocks = 16, 8192, 256
    a.q = a.k = a.v = a.out = a.block_table = a.seq_lens = fake
    a.q_stride = (C.c_int64 * 3)(8192, 8192, 128)
    a.o_stride = (C.c_int64 * 3)(8192, 8192, 128)
    a.k_stride = (C.c_int64 * 3)(16 * 8 * 128, 8 * 128, 128)
    a.v_stride = (C.c_int64 * 3)(16 * 8 * 128, 8 * 128, 128)
    a.block_table_stride, a.softmax_scale = 256, 0.088
    need = C.c_size_t()
    assert lib.pat_paged_decode_baseline_workspace_bytes(C.byref(a), C.byref(need)) == 0
    # partial rows of 4096-token requests (>= 2 chunks) plus the three per-request tables
    assert need.value >= 32 * 64 * 2 * (128 + 1) * 4 + 3 * 32 * 4
    assert lib.pat_paged_decode_baseline_launch(C.byref(a), None) == _lib.PAT_ERR_WORKSPACE
    a.max_blocks = 0
    assert lib.pat_paged_decode_baseline_workspace_bytes(C.byref(a), C.byref(need)) == _lib.PAT_ERR_INVALID
    assert "max_blocks" in _lib.last_error()
    a.max_blocks, a.kv_heads = 256, 5
    assert lib.pat_paged_decode_baseline_workspace_bytes(C.byref(a), C.byref(need)) == _lib.PAT_ERR_INVALID


def test_form_of_the_tall_path_follows_the_launch():
    """32-row tiles when the whole launch is resident at two workgroups per CU or its long tall boxes
    outweigh the short ones; the 16-row form (a third resident workgroup per CU) otherwise."""
    lib = _lib.load()
    g = _lib.FwdGeometry()

    def form(tall_boxes, tall_blocks, short_boxes, short_blocks, batch):
        a = _args(batch=batch)
        b = a._keep
        b[0].num_boxes, b[0].max_blocks, b[0].block_table_stride = tall_boxes, tall_blocks, tall_blocks
        b[1].num_boxes, b[1].max_blocks, b[1].block_table_stride = short_boxes, short_blocks, short_blocks
        a.max_blocks_in_box = max(tall_blocks, short_blocks)
        assert lib.pat_fwd_geometry_of(C.byref(a), C.byref(g)) == 0, _lib.last_error()
        return g.tall_rows, g.num_workgroups

    assert form(4, 128, 64, 32, 64)[0] == 32            # the headline batch: everything resident at once
    assert form(16, 64, 128, 64, 128)[0] == 16          # a 3-level tree: 1024-token leaves outweigh the tall boxes
    assert form(24, 171, 32, 128, 32)[0] == 32          # a 16k prefix in 2736-token tall boxes over 2048-token suffixes
    assert form(128, 8, 1024, 2, 1024)[0] == 16         # many short tall boxes over a thousand 32-token leaves
    assert form(0, 128, 512, 64, 512)[0] == 16          # no tall box at all
