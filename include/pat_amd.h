/*
 * pat_amd.h — C ABI of libpat_amd: prefix-aware decode attention over a paged KV
 * cache for AMD MI355X (gfx950).
 *
 * Everything here is plain C: integers, pointers and sizes. No torch / pybind types.
 * A binding (ctypes, pybind11, cgo ...) converts its tensors to raw pointers +
 * element strides and calls these entry points.
 *
 * Every function returns PAT_OK (0) or a negative PAT_ERR_* code; the message of
 * the last failure on the calling thread is returned by pat_last_error().
 *
 * Reference interfaces replaced (paths relative to the flashserve/PAT tree):
 *   scheduler        prefix_attn/prefix_tree.py:47-616  (class PrefixTree)
 *                    csrc/prefix_tree.h:63-324          (PrefixTreeCPP twin)
 *                    csrc/bindings.cpp:100-146          (its pybind surface)
 *   plan containers  prefix_attn/data_class.py:173-254  (KernelInfo / to_tensor)
 *   forward          csrc/api.h:110-295                 (pat_mha_fwd_kvcache)
 *                    csrc/bindings.cpp:7-72             (both Python overloads)
 *   kernels          csrc/pat_fwd_kernel.h:25-310       (split-KV forward)
 *                    csrc/pat_fwd_kernel.h:314-467      (gather / merge)
 *                    csrc/pat_fwd_launch_template.h:35-98 (dispatch)
 */
#ifndef PAT_AMD_H_
#define PAT_AMD_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define PAT_ABI_VERSION 4

/* ---- status codes ------------------------------------------------------- */
#define PAT_OK 0
#define PAT_ERR_INVALID (-1) /* bad argument; bindings raise RuntimeError          */
#define PAT_ERR_VALUE (-2)   /* where the Python scheduler raises ValueError        */
#define PAT_ERR_INDEX (-3)   /* where the Python scheduler raises IndexError        */
#define PAT_ERR_KEY (-4)     /* where the Python scheduler raises KeyError          */
#define PAT_ERR_HIP (-5)     /* a HIP runtime call failed                           */
#define PAT_ERR_WORKSPACE (-6) /* workspace missing or too small                    */

#define PAT_DTYPE_F16 0
#define PAT_DTYPE_BF16 1

/* Message of the last error raised on this thread ("" if none). Never NULL. */
const char* pat_last_error(void);
/* Returns PAT_ABI_VERSION of the loaded library. */
int pat_abi_version(void);

/* ======================================================================== *
 *  Scheduler: radix tree over block-table rows -> packed boxes -> buckets   *
 * ======================================================================== */

typedef struct pat_tree pat_tree; /* opaque */

/* Tuning constants of the load balancer. Passing NULL to pat_tree_pack keeps the
 * reference's values (prefix_attn/prefix_tree.py:390-437), which is what plan
 * parity is defined against. */
typedef struct pat_sched_opts {
  int32_t long_kv_tokens;      /* boxes with kv > this enter the average (256)        */
  int32_t long_factor;         /* a box is cut when blocks > factor * average (5)      */
  int32_t min_boxes[5];        /* target #boxes for kv_heads <=4,<=8,<=16,<=32,else    */
                               /* (54, 27, 13, 6, 4)                                   */
  int32_t stop_blocks;         /* halving stops at boxes of <= this many blocks (8)    */
  int32_t max_split;           /* halving stops once a sequence has this many (32)     */
} pat_sched_opts;

/* One node of the radix tree (for inspection / tests). Pointers alias tree storage
 * and stay valid until the tree is rebuilt or destroyed. */
typedef struct pat_node_view {
  int32_t parent;       /* -1 for the root                                   */
  int32_t num_seqs;     /* s_value: sequences passing through the node       */
  int32_t num_tokens;   /* tokens of KV held by the node                     */
  int32_t num_seq_ids;  /* length of seq_ids                                 */
  int32_t num_blocks;   /* length of block_ids                               */
  int32_t num_children; /* length of child_ids (insertion order)             */
  const int32_t* seq_ids;
  const int32_t* block_ids;
  const int32_t* child_ids;
} pat_node_view;

/* One tile bucket of a plan. Rows of q_table / block_table are padded with 0 to
 * the bucket's widest row, exactly as KernelInfo.to_tensor does
 * (prefix_attn/data_class.py:228-253). q_len / block_len keep the unpadded
 * lengths so a binding can also rebuild the ragged Python lists. */
typedef struct pat_bucket_view {
  int32_t mnw[3];       /* tile label [M, N, W] of the bucket                */
  int32_t num_boxes;    /* "CTAs" in the reference                            */
  int32_t max_seqs;     /* q_table row width                                  */
  int32_t max_blocks;   /* block_table row width                              */
  const int32_t* q_table;     /* [num_boxes, max_seqs]                        */
  const int32_t* block_table; /* [num_boxes, max_blocks]                      */
  const int32_t* q_len;       /* [num_boxes]                                  */
  const int32_t* block_len;   /* [num_boxes]                                  */
  const int32_t* num_seqs;    /* [num_boxes]  num_seqs_per_CTA                */
  const int32_t* rank;        /* [num_boxes]  CTA_rank                        */
  const int32_t* kv;          /* [num_boxes]  kv_in_CTA (tokens)              */
  /* Not part of the reference plan: for box b and its j-th sequence s, the number of
   * earlier boxes of the plan (bucket order, then box order) that contain s. Unlike
   * CTA_rank it is unique per (sequence, box) by construction, also on forests where
   * the reference hands one rank to two boxes of a sequence. Same shape/padding as
   * q_table. */
  const int32_t* q_slot;      /* [num_boxes, max_seqs]                        */
} pat_bucket_view;

typedef struct pat_plan_view {
  int32_t num_buckets;
  int32_t batch;                    /* length of num_split_per_seq            */
  const pat_bucket_view* buckets;   /* [num_buckets]                          */
  const int32_t* num_split_per_seq; /* [batch]                                */
  int32_t max_split_per_seq;
  int32_t max_seqs_in_box;          /* KernelInfo.max_seqs_in_CTA             */
  int32_t max_blocks_in_box;        /* KernelInfo.max_blocks_in_CTA           */
  /* Not part of the reference plan: the number of boxes of THIS plan that contain each
   * sequence (= 1 + the sequence's largest q_slot) and its maximum. num_split_per_seq is the
   * reference's counter, which keeps counting over repeated pack calls on one tree
   * (prefix_attn/prefix_tree.py:149 resets it only when the tree is rebuilt); a launch that
   * files partial results by q_slot merges num_boxes_per_seq of them. */
  const int32_t* num_boxes_per_seq; /* [batch]                                */
  int32_t max_boxes_per_seq;
} pat_plan_view;

/* PrefixTree(block_size)                     prefix_attn/prefix_tree.py:48-59 */
int pat_tree_create(int32_t block_size, pat_tree** out);
void pat_tree_destroy(pat_tree* tree);

/* PrefixTreeCPP.build_radix_tree(seq_lens, block_table)
 *                                  csrc/bindings.cpp:103-126, prefix_tree.h:84-99
 * table is a dense [num_seqs, max_blocks] matrix; row i contributes its first
 * ceil(seq_lens[i] / block_size) entries, the rest is padding. The table is copied:
 * the caller may free it as soon as the call returns. */
int pat_tree_build(pat_tree* tree, const int32_t* seq_lens, const int32_t* table,
                   int32_t num_seqs, int32_t max_blocks);

/* PrefixTree.build_radix_tree(seq_lens, block_table: List[List[int]])
 *                                             prefix_attn/prefix_tree.py:146-149
 * Ragged rows: row i is flat_blocks[row_offsets[i] .. row_offsets[i+1]) and is used
 * whole, whatever seq_lens[i] says (as the Python class does). */
int pat_tree_build_rows(pat_tree* tree, const int32_t* seq_lens,
                        const int32_t* flat_blocks, const int64_t* row_offsets,
                        int32_t num_seqs);

/* Edits of a built tree between decode steps. No counterpart in the reference, which builds a new
 * tree from the whole batch for every step (plugin/vllm/attention/backends/prefix_attn.py:330-338,
 * 377-448). Sequence ids are batch rows:
 *   pat_tree_append  adds a row behind the last one (its id = pat_tree_num_seqs before the call);
 *   pat_tree_remove  deletes row `seq`; the rows behind it move up by one;
 *   pat_tree_grow    lengthens row `seq` to new_len tokens; more_blocks are the blocks it gained.
 * After any of them the tree, and every plan packed from it, is what pat_tree_build_rows gives for
 * the edited batch (same nodes, child order, sequence lists, token counts; split counters of a
 * fresh tree), provided that every block two rows share is full for both - what a paged KV cache
 * with prefix sharing guarantees. pat_tree_grow returns PAT_ERR_VALUE and leaves the tree as it was
 * when only a fresh build can know the new shape (the row grew inside a shared block, or into blocks
 * another row holds): build the tree again then. */
int pat_tree_append(pat_tree* tree, int32_t seq_len, const int32_t* blocks, int32_t num_blocks);
int pat_tree_remove(pat_tree* tree, int32_t seq);
int pat_tree_grow(pat_tree* tree, int32_t seq, int32_t new_len, const int32_t* more_blocks,
                  int32_t num_more);
int pat_tree_num_seqs(const pat_tree* tree);

/* PrefixTree.pack_schedule(MNWs, HRatio, kvHead, use_compute_model)
 *                                             prefix_attn/prefix_tree.py:548-616
 * mnws: n_mnws triples [M, N, W] or NULL (n_mnws 0) for the default 11 buckets.
 * The resulting plan is stored in the tree; read it with pat_tree_plan. As in the
 * Python class, the per-sequence split counters are NOT reset between calls. */
int pat_tree_pack(pat_tree* tree, const int32_t* mnws, int32_t n_mnws, int32_t hratio,
                  int32_t kv_heads, int32_t use_compute_model,
                  const pat_sched_opts* opts);

/* PrefixTree.naive_schedule(HRatio)           prefix_attn/prefix_tree.py:484-545 */
int pat_tree_naive_schedule(pat_tree* tree, int32_t hratio);

/* ------------------------------------------------------------------------ *
 *  The plan as ONE buffer (one host-to-device copy per decode step)         *
 *  replaces KernelInfo.to_tensor's copy per table, data_class.py:209-254,   *
 *  and PrefixTreeCPP's tensor aliases, csrc/prefix_tree.h:27-38             *
 * ------------------------------------------------------------------------ */
#define PAT_MAX_FLAT_BUCKETS 12

/* One bucket inside the flat buffer: shapes plus the offset of every table, in int32
 * elements from the start of the buffer. Tables are dense row-major. */
typedef struct pat_flat_bucket {
  int32_t mnw[3];
  int32_t num_boxes;
  int32_t max_seqs;    /* columns of q_table and q_slot                                  */
  int32_t max_blocks;  /* columns of block_table                                         */
  int32_t parent;      /* launch buckets: plan bucket the boxes come from; else own index */
  int32_t first;       /* launch buckets: position of the first box in the parent's
                          launch order; plan buckets: 0                                   */
  int32_t flags;       /* PAT_BUCKET_* hints that hold for the bucket                    */
  int32_t pad_;
  int64_t q_table, q_slot, block_table, num_seqs, rank, kv;
} pat_flat_bucket;

/* Layout of the flat plan. `buckets` is the plan exactly as pat_tree_plan shows it (the
 * scheduler's order). `launch` holds the copies meant for pat_fwd_launch: every bucket's
 * boxes longest first (stable), and a bucket in which at most a quarter of the boxes are
 * more than twice as long as all others split in two (the wide head first), so that the
 * forward kernels do not reserve work for every box up to the widest one's length; the
 * second part's block_table is as wide as its widest row plus 8 spare columns (room for
 * in-place growth between decode steps). launch_order[b] is the offset of plan bucket b's
 * permutation: entry i = plan row of the box at launch position i. */
typedef struct pat_flat_plan {
  int32_t num_buckets;
  int32_t num_launch_buckets;
  int32_t batch;
  int32_t max_split_per_seq, max_seqs_in_box, max_blocks_in_box;
  int64_t total;               /* int32 elements the buffer needs                        */
  int64_t num_split_per_seq;   /* offset, [batch]                                        */
  int64_t num_boxes_per_seq;   /* offset, [batch]: see pat_plan_view.num_boxes_per_seq   */
  int32_t max_boxes_per_seq;
  int32_t pad_;
  int64_t launch_order[PAT_MAX_FLAT_BUCKETS];
  pat_flat_bucket buckets[PAT_MAX_FLAT_BUCKETS];
  pat_flat_bucket launch[PAT_MAX_FLAT_BUCKETS];
} pat_flat_plan;

/* Describes the flat form of the current plan in *layout and, when dst is not NULL, writes
 * it (capacity in int32 elements, at least layout->total). dst may be pinned host memory.
 * Fails with PAT_ERR_INVALID when the plan has more than PAT_MAX_FLAT_BUCKETS buckets. */
int pat_tree_flat_plan(const pat_tree* tree, pat_flat_plan* layout, int32_t* dst, int64_t capacity);

/* Borrow the plan built by the last pack / naive_schedule call. */
int pat_tree_plan(const pat_tree* tree, pat_plan_view* out);

/* Node slots of the tree (slots given up by pat_tree_remove included: their parent is -2). */
int pat_tree_num_nodes(const pat_tree* tree);
int pat_tree_node(const pat_tree* tree, int32_t node, pat_node_view* out);

/* ======================================================================== *
 *  Forward: split-KV kernels over the plan + LSE merge                      *
 * ======================================================================== */

/* Per-bucket plan tables, resident in device memory (int32). */
typedef struct pat_fwd_bucket {
  const int32_t* q_table;     /* [num_boxes, q_table_stride]                  */
  const int32_t* block_table; /* [num_boxes, block_table_stride]              */
  const int32_t* num_seqs;    /* [num_boxes]                                  */
  const int32_t* rank;        /* [num_boxes]                                  */
  const int32_t* kv;          /* [num_boxes]                                  */
  const int32_t* q_slot;      /* optional [num_boxes, q_table_stride] (see     */
                              /* pat_bucket_view.q_slot); NULL: use CTA_rank   */
  /* Filing by CTA_rank (q_slot NULL) is what the reference does and is right only where every
   * sequence's boxes carry the ranks 0 .. num_split_per_seq - 1, each once (regular trees). Where
   * the scheduler repeats or skips a rank within a sequence (irregular forests), one partial
   * result overwrites another or the merge reads a slot nobody wrote: pass the planner's q_slot
   * and num_boxes_per_seq, or derive both on the device with pat_fwd_derive_slots. */
  int64_t q_table_stride;     /* elements between rows                        */
  int64_t block_table_stride; /* elements between rows                        */
  int32_t num_boxes;
  int32_t max_seqs;           /* valid columns of q_table                     */
  int32_t max_blocks;         /* valid columns of block_table                 */
  int32_t mnw[3];
  int32_t flags;              /* PAT_BUCKET_* hints, 0 when nothing is known  */
} pat_fwd_bucket;

/* Hint: no box of the bucket is shorter than 3/4 of its widest box (the launcher cannot see
 * lengths, which live in device memory). Long even buckets get one kv head per wave sooner
 * (contiguous reads across heads; safe only when no workgroup outlasts the others by much).
 * A wrong hint costs time, never correctness. */
#define PAT_BUCKET_EVEN 1

/* Overrides of the launch geometry. pat_fwd_set_tuning sets them process-wide (a tuning and test
 * aid, not meant to change while launches are in flight on other threads); pat_fwd_args.tuning sets
 * them for one launch (what pat_fwd_autotune's result is for). 0 / -1 = automatic, as noted per field. The
 * initial values come from the environment variables PAT_CHUNK_TOKENS, PAT_TALL_CHUNK_TOKENS,
 * PAT_HEAD_PER_WAVE_TOKENS, PAT_HEAD_PER_WAVE_LONG_WGS, PAT_HEAD_PER_WAVE_LONG_TOKENS,
 * PAT_EQUALIZE_CHUNKS, PAT_DIRECT_OUT, read once; pat_fwd_set_tuning(NULL) reads them again. */
typedef struct pat_fwd_tuning {
  int32_t chunk_tokens;              /* KV tokens per workgroup, boxes <= 16 rows (0: automatic)   */
  int32_t tall_chunk_tokens;         /* same for boxes of 17..64 rows (0: automatic)                */
  int32_t head_per_wave_tokens;      /* widest box of a bucket that runs a kv head per wave         */
                                     /* (-1: automatic, 0: never)                                   */
  int32_t head_per_wave_long_tokens; /* chunk of long boxes run a kv head per wave (0: automatic)   */
  int64_t head_per_wave_long_wgs;    /* such workgroups a bucket needs for that (-1: automatic)     */
  int32_t equalize_chunks;           /* even chunks per box: -1 automatic, 0 never, 1 always        */
  int32_t direct_out;                /* single-slot launches write `out` from the split kernel:     */
                                     /* -1 / 1 when possible, 0 never                               */
  int32_t tall_rows;                 /* rows per wave on boxes of 17..64 rows: 32 (32x32x16 MFMA    */
                                     /* tiles, 2 workgroups per CU at head_dim 128), 16 (16x16x32,  */
                                     /* 3 per CU), 0: chosen per launch from its sizes              */
  int32_t reserved;                  /* 0                                                           */
} pat_fwd_tuning;
int pat_fwd_set_tuning(const pat_fwd_tuning* tuning);
int pat_fwd_get_tuning(pat_fwd_tuning* out);

/* Mirrors the arguments of pat_mha_fwd_kvcache (csrc/api.h:110-127).
 * Strides are in ELEMENTS (as csrc/api.h:43); the last dimension of q, k, v, out
 * must be contiguous. Unlike the reference, V may have strides of its own.
 * K/V: one block spans less than 2^29 elements (stride[1] * page_size) and blocks
 * are less than 2^30 elements apart (stride[0]). */
typedef struct pat_fwd_args {
  int32_t dtype;       /* PAT_DTYPE_F16 | PAT_DTYPE_BF16 (q, k, v, out)      */
  int32_t batch;       /* q.size(0)                                           */
  int32_t seqlen_q;    /* q.size(1); decode: 1                                */
  int32_t heads;       /* q.size(2)                                           */
  int32_t kv_heads;    /* k.size(2)                                           */
  int32_t head_dim;    /* 64 | 128                                            */
  int32_t page_size;   /* k.size(1), multiple of 16                           */
  int32_t num_pages;   /* k.size(0)                                           */
  const void* q;       /* [batch, 1, heads, head_dim]                         */
  const void* k;       /* [num_pages, page_size, kv_heads, head_dim]          */
  const void* v;
  void* out;           /* [batch, 1, heads, head_dim], written in place       */
  float* lse_out;      /* optional [batch, heads] natural-log LSE, or NULL    */
  int64_t q_stride[3]; /* batch, row, head                                    */
  int64_t k_stride[3]; /* page, slot, head                                    */
  int64_t v_stride[3];
  int64_t o_stride[3]; /* batch, row, head                                    */
  const int32_t* num_split_per_seq; /* device int32 [batch]                   */
  int32_t max_split_per_seq;
  int32_t max_seqs_in_box;
  int32_t max_blocks_in_box;
  float softmax_scale;
  int32_t num_buckets;
  const pat_fwd_bucket* buckets; /* host array [num_buckets]                  */
  void* workspace;               /* device scratch, 256-byte aligned          */
  size_t workspace_bytes;
  void* split_done_event;        /* optional hipEvent_t recorded on the stream between the   */
                                 /* split kernel and the merge kernel (timing aid), or NULL  */
  const pat_fwd_tuning* tuning;  /* optional launch-geometry overrides for this call (host    */
                                 /* memory, read during the call); NULL: the process-wide ones */
  const void* records;           /* optional launch records of this plan (pat_fwd_build_records), */
  size_t records_bytes;          /* device memory; NULL: the launch builds them in its workspace  */
  uint64_t records_tag;          /* what pat_fwd_build_records returned with them                 */
} pat_fwd_args;

/* Argument checks of csrc/api.h:129-181 that need no GPU (dtype enum, head_dim,
 * page size, GQA ratio, split limits, strides, bucket labels). Pointers are only
 * tested for NULL. Runs on a machine without a GPU. */
int pat_fwd_validate(const pat_fwd_args* args);

/* Bytes of device scratch pat_fwd_launch needs for these arguments: partial outputs +
 * partial LSE (the reference allocates the equivalent per call at csrc/api.h:217-229) and,
 * when args->records is NULL, the launch records of this call. Depends only on sizes,
 * pointers' alignment and strides, never on device data. With prebuilt records it is 0 when
 * every row has a single partial slot (max_split_per_seq 1 and no box longer than a chunk):
 * the launch then writes `out` from its first kernel, as the reference does for
 * max_split_per_seq 1 (csrc/api.h:230-238), and `workspace` may be NULL. */
int pat_fwd_workspace_bytes(const pat_fwd_args* args, size_t* bytes);

/* Launch records: one small record per workgroup of the launch (which rows, which partial
 * slots, which KV pages, how many tokens), laid out so that the split kernel starts its KV
 * loads after a single round trip to memory. A device kernel writes them from the plan tables
 * (values checked and clamped there once, not in every launch). They depend on the plan tables'
 * contents, on the sizes in `args` and on the launch geometry (tuning), not on q / k / v / out:
 * build them once per plan and pass them to every launch of it (each layer of a decode step);
 * rebuild after the plan tables were edited. pat_fwd_launch with args->records == NULL builds
 * them itself on every call, in its workspace (one more small kernel per call).
 * No counterpart in the reference, whose kernel decodes the plan tables in every thread block
 * (csrc/pat_fwd_kernel.h:40-75).
 * pat_fwd_records_bytes: size of the buffer; pat_fwd_build_records: enqueues the record kernel
 * on `hip_stream` (`buffer`: device memory, 256-byte aligned) and returns the tag to put in
 * args->records_tag; a launch whose geometry or tables differ from the tag's fails with
 * PAT_ERR_INVALID and enqueues nothing. pat_fwd_records_tag: the tag alone (host arithmetic): two
 * argument blocks with the same tag can share one set of records (the layers of a model: same
 * plan tables, different q / k / v / out). */
int pat_fwd_records_bytes(const pat_fwd_args* args, size_t* bytes);
int pat_fwd_records_tag(const pat_fwd_args* args, uint64_t* tag);
int pat_fwd_build_records(const pat_fwd_args* args, void* buffer, size_t buffer_bytes,
                          uint64_t* tag, void* hip_stream);

/* prefix_attn_with_kvcache(...)   csrc/bindings.cpp:7-72 -> csrc/api.h:110-295
 * Enqueues the split-KV kernel and (unless the workspace size is 0, see above) the merge
 * kernel on `hip_stream` (a hipStream_t; NULL = the null stream) of the current device and
 * returns without synchronising. Rows of `out` (and `lse_out`) whose sequence sits in no box of
 * the plan: the merge kernel writes 0 (LSE -inf) there; a single-slot launch, which has no merge
 * kernel, leaves them as they were (the scheduler's plans put every sequence in a box; only a
 * hand-made plan can leave one out). */
int pat_fwd_launch(const pat_fwd_args* args, void* hip_stream);

/* pat_fwd_launch for callers that cannot allocate device memory (code under HIP graph capture,
 * serving loops and harnesses that forbid hipMalloc). No counterpart in the reference, whose
 * forward allocates its partial buffers per call (csrc/api.h:217-229). Same arguments, kernels and
 * results as pat_fwd_launch; args->workspace / workspace_bytes are ignored: the partial results go
 * to an array built into the library (pat_fwd_static_scratch_bytes() bytes, 64 MiB, one copy per GPU,
 * held until the process ends). Calls no hipMalloc / hipFree. A launch that needs more partial-result
 * space than the array holds fails with PAT_ERR_WORKSPACE and enqueues nothing. Every call on a GPU
 * uses that GPU's one array: calls that overlap on one GPU (two streams, two threads) race; calls
 * on one stream are ordered and safe. Nothing in the array has to be cleared between calls: every
 * slot a call reads it writes first (slots filed as described at pat_fwd_bucket.q_slot).
 * The first call on each device looks up the array's device address (hipGetSymbolAddress, which may
 * load the code object) and therefore must not be made while `hip_stream` is capturing: it fails with
 * PAT_ERR_INVALID there and enqueues nothing. Make one call on the device before the capture; later
 * calls, captured or not, only enqueue kernels. */
int pat_fwd_launch_static(const pat_fwd_args* args, void* hip_stream);
size_t pat_fwd_static_scratch_bytes(void);

/* Partial-result slots for a plan that carries none (pat_fwd_bucket.q_slot == NULL), e.g. the
 * tensors of KernelInfo.to_tensor passed positionally as benchmark/benchmark_kernel.py:247-265
 * does. Filing partial results by CTA_rank, as the reference kernel does
 * (csrc/block_info.h:29-35), loses one wherever the reference scheduler hands the same rank to two
 * boxes of a sequence (irregular forests). pat_fwd_derive_slots runs one small kernel on
 * `hip_stream` that reads the q_tables / num_seqs of args->buckets and writes into `buffer`
 * (device memory, 256-byte aligned, pat_fwd_slots_bytes() bytes):
 *   int32 [batch]                      boxes of the plan that contain each sequence, at offset 0
 *   int32 [num_boxes, q_table_stride]  per bucket i, at element offset bucket_offsets[i] (host
 *                                      array [num_buckets], filled by the call): for every
 *                                      (box, sequence) the box's ordinal among that sequence's
 *                                      boxes, buckets in order, boxes in order
 * The caller then launches with buckets[i].q_slot = buffer + bucket_offsets[i] and
 * num_split_per_seq = buffer. The result depends on the plan's contents: derive again after the
 * q_tables change. */
int pat_fwd_slots_bytes(const pat_fwd_args* args, size_t* bytes);
int pat_fwd_derive_slots(const pat_fwd_args* args, void* buffer, size_t buffer_bytes,
                         int64_t* bucket_offsets, void* hip_stream);


/* Measured choice of the launch geometry (no counterpart in the reference, whose tile shapes are
 * fixed per bucket). The best chunking of a launch depends on how its workgroups share the CUs,
 * which sizes alone do not predict for mid-size launches; pat_fwd_autotune runs the launch `reps`
 * times (after 2 untimed runs) under each of a few candidate geometries - the automatic one first -
 * on `hip_stream`, times them with HIP events, and stores in *best the overrides of the fastest
 * (the automatic values unless a candidate beats them by 4 % and 1 us). Pass the result as
 * pat_fwd_args.tuning of later launches with the same plan shape. `out` holds a valid result
 * afterwards. args->workspace must hold pat_fwd_autotune_workspace_bytes() bytes (the largest
 * candidate's need). `evict` (optional): a device buffer at least as large as the memory-side cache
 * (256 MB on MI355X) that is read before every timed launch, outside its interval, so that each runs
 * against HBM, as the layers of a model, each with a KV cache of its own, do; with NULL the launches
 * are timed back to back and inputs that fit the cache look faster than they will be. The call
 * SYNCHRONISES the stream (not for use under graph capture) and creates and destroys two HIP
 * events. best_us / auto_us (optional) receive the time per launch of the chosen and of the
 * automatic geometry. */
int pat_fwd_autotune_workspace_bytes(const pat_fwd_args* args, size_t* bytes);
int pat_fwd_autotune(const pat_fwd_args* args, void* hip_stream, int32_t reps, const void* evict,
                     size_t evict_bytes, pat_fwd_tuning* best, float* best_us, float* auto_us);

/* Description of the launch geometry chosen for `args` (for benchmarks/tests). */
typedef struct pat_fwd_geometry {
  int32_t chunk_tokens;      /* KV tokens one workgroup streams (boxes <= 16 rows) */
  int32_t tall_chunk_tokens; /* same for boxes of 17..64 rows                      */
  int32_t chunks_per_rank;   /* partial slots reserved per box                     */
  int32_t num_slots;         /* max_split_per_seq * chunks_per_rank                */
  int64_t num_workgroups;    /* split-kernel workgroups                            */
  int32_t tall_rows;         /* form of the tall path: 32 or 16 rows per wave      */
  int32_t reserved;
} pat_fwd_geometry;
int pat_fwd_geometry_of(const pat_fwd_args* args, pat_fwd_geometry* out);

/* ------------------------------------------------------------------------ *
 *  Prefix-oblivious paged decode: the comparator of the benchmarks          *
 *  (benchmark/benchmark_kernel.py runs FlashAttention / FlashInfer decode   *
 *  beside PAT, :270-330; here the same two kernels run the plan that        *
 *  block_scheduler.pack_without_prefix describes, prefix_attn/              *
 *  block_scheduler.py:155-202: one work item per request over its own block *
 *  row, split along KV by the launch geometry)                              *
 * ------------------------------------------------------------------------ */
typedef struct pat_baseline_args {
  int32_t dtype, batch, heads, kv_heads, head_dim, page_size, num_pages;
  int32_t max_blocks;            /* columns of block_table in use                 */
  const void* q;                 /* [batch, 1, heads, head_dim]                   */
  const void* k;                 /* [num_pages, page_size, kv_heads, head_dim]    */
  const void* v;
  void* out;                     /* like q                                        */
  int64_t q_stride[3], k_stride[3], v_stride[3], o_stride[3];   /* as pat_fwd_args */
  const int32_t* block_table;    /* device [batch, block_table_stride]            */
  int64_t block_table_stride;
  const int32_t* seq_lens;       /* device [batch], tokens                        */
  float softmax_scale;
  int32_t flags;                 /* PAT_BUCKET_* hints for the one bucket         */
  float* lse_out;                /* optional device [batch, heads]                */
  void* workspace;               /* device, 256-byte aligned                      */
  size_t workspace_bytes;
} pat_baseline_args;

int pat_paged_decode_baseline_workspace_bytes(const pat_baseline_args* args, size_t* bytes);
/* Enqueues a small table-fill kernel, the split kernel and the merge kernel on the stream. */
int pat_paged_decode_baseline_launch(const pat_baseline_args* args, void* hip_stream);

/* Device self-test (no counterpart in the reference): runs a one-wave kernel on `hip_stream` that
 * checks the lane-swap reductions and the transposed LDS read against their definitions - the
 * instruction-level facts the split kernel is built on - and stores the number of mismatches in
 * *failures (0 = all hold). Allocates 4 bytes of device memory and synchronises the stream: a
 * diagnostic, not part of the decode path. */
int pat_selftest_device(void* hip_stream, int32_t* failures);

#ifdef __cplusplus
} /* extern "C" */
#endif
#endif /* PAT_AMD_H_ */
