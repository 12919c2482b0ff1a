// Kernel-argument structures shared by the host launcher and the gfx950 kernels.
#pragma once
#include <cstdint>

namespace pat {

constexpr int kMaxBuckets = 12;    // the reference dispatches 12 tile shapes (static_switch.h:3-66)
constexpr int kWaves = 4;          // waves per split-kernel workgroup
constexpr int kThreads = kWaves * 64;
constexpr int kStepTokens = 32;    // KV tokens one wave consumes per loop iteration
constexpr int kGridX = 1 << 20;     // workgroups per grid.x slice (grid.y counts slices)
constexpr int kMaxChunkPages = 128; // page ids of a chunk: two per lane of a wave

// One workgroup's work: a launch record, written once per plan by the record kernel
// (capi_fwd.hip) and read by the split kernel in a single round trip. In memory:
//   RecordHead | int32 seq[max_seqs] | int32 slot[max_seqs] | int32 page[max_pages]
// seq[j] / slot[j]: batch index of the box's j-th sequence and the partial-result slot its rows
// of this piece go to (-1 / -1: no such row); page[i]: physical KV block of the piece's i-th page,
// already clamped to the cache. Records are record_stride bytes apart (a multiple of 64).
struct RecordHead {
  int32_t tokens;      // KV tokens of this piece; 0: nothing to compute (the workgroup only marks slots empty)
  int32_t rows;        // rows of the box (sequences x heads per kv head), <= 16 x tiles
  int32_t mode;        // bits 0-7: 16-row tiles (1 = KV steps split over waves on wave-private tiles,
                       // 2/4 = one wave per tile on tiles shared through LDS); bit 8: a kv head per wave
  int32_t head;        // first kv head this workgroup serves
  int32_t fill_begin;  // slots slot[j] + fill_begin .. slot[j] + fill_end - 1 of every row stay empty:
  int32_t fill_end;    // this workgroup marks them (-inf)
  int32_t pad[2];
};
static_assert(sizeof(RecordHead) == 32, "RecordHead is read as two 16-byte pieces");
constexpr int kRecordModeHeadPerWave = 0x100;

struct SplitParams {
  const char* records;      // one per workgroup, in launch order
  int32_t record_stride;    // bytes
  int32_t record_max_seqs;  // seq[] / slot[] entries per record
  const void* q;
  const void* k;
  const void* v;
  float* o_part;     // [batch, heads, num_slots, head_dim] fp32, normalised partial outputs
  float* lse_part;   // [batch, heads, num_slots] fp32, natural-log LSE of each partial (-inf = empty)
  int64_t q_stride_b, q_stride_h;              // elements
  int64_t k_stride_page, k_stride_slot, k_stride_h;
  int64_t v_stride_page, v_stride_slot, v_stride_h;
  int32_t heads, group;     // group = heads / kv_heads
  int32_t page_size;
  int32_t num_slots;        // partial-result slots per (sequence, head)
  int32_t total_items;      // workgroups of the launch
  float scale_log2;         // softmax_scale * log2(e)
  uint32_t hpp_magic;       // ceil(2^32 / (page_size / 16)): h / (page_size / 16) == umulhi(h, hpp_magic) for h < 2^16; unused when page_size / 16 is a power of two
  // single-slot launches (every row has one partial slot; no merge kernel follows): the rows go
  // to `out`.
  void* out;         // [batch, 1, heads, head_dim] in the element type
  float* lse_out;    // optional [batch, heads] fp32
  int64_t o_stride_b, o_stride_h;              // elements
  int32_t direct;    // 1: such a launch
  int32_t tall_rows; // rows per wave on boxes of 17..64 rows: 32 (32x32x16 tiles) or 16 (host side: picks the kernel instance)
};

// One tile bucket as the record kernel sees it.
struct RecordBucket {
  const int32_t* q_table;
  const int32_t* block_table;
  const int32_t* num_seqs;
  const int32_t* rank;
  const int32_t* kv;
  const int32_t* q_slot; // optional [num_boxes, q_stride]: ordinal of the box among its sequence's boxes
  int32_t q_stride;      // elements between q_table (and q_slot) rows
  int32_t bt_stride;     // elements between block_table rows
  int32_t num_boxes;
  int32_t max_seqs;      // valid q_table columns
  int32_t max_blocks;    // valid block_table columns
  int32_t chunk_tokens;  // KV tokens per workgroup (multiple of 32 and of page_size)
  int32_t chunks;        // workgroups along the KV axis reserved per box
  int32_t item_begin;    // first workgroup of this bucket in the launch
  int32_t row_tiles;     // 16-row tiles per box: 1, 2 or 4
  int32_t heads_per_wg;  // 1, or kWaves: wave w serves kv head h0 + w alone
};

struct RecordParams {
  char* records;
  int32_t record_stride, record_max_seqs, record_max_pages;
  int32_t num_buckets, total_items, grid_items;   // grid_items: total_items rounded up to the split kernel's grid
  int32_t batch, kv_heads, group, page_size, num_pages;
  int32_t chunks_per_rank;  // slots reserved per box ordinal
  int32_t max_split;
  RecordBucket bucket[kMaxBuckets];
};

struct MergeParams {
  const float* o_part;
  const float* lse_part;
  const int32_t* num_split_per_seq;
  void* out;
  float* lse_out;           // may be null
  int64_t o_stride_b, o_stride_h;
  int32_t batch, heads, head_dim;
  int32_t chunks_per_rank, num_slots, max_split;
  int32_t kv_heads;
};

}  // namespace pat
