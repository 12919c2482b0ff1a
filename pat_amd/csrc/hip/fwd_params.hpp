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

// One tile bucket as the split kernel sees it.
struct BucketDev {
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
  int32_t item_begin;    // first workgroup of this bucket in the launch (workgroups = items x head groups)
  int32_t row_tiles;     // 16-row tiles per box: 1 = KV steps split over waves, 2/4 = one wave per tile
  int32_t heads_per_wg;  // 1, or kWaves for buckets of very short boxes: wave w serves kv head h0 + w alone
};

struct SplitParams {
  const void* q;
  const void* k;
  const void* v;
  float* o_part;     // [batch, heads, num_slots, head_dim] fp32, normalised partial outputs
  float* lse_part;   // [batch, heads, num_slots] fp32, natural-log LSE of each partial (-inf = empty)
  int64_t q_stride_b, q_stride_h;              // elements
  int64_t k_stride_page, k_stride_slot, k_stride_h;
  int64_t v_stride_page, v_stride_slot, v_stride_h;
  int32_t batch, heads, kv_heads, group;       // group = heads / kv_heads
  int32_t page_size, num_pages;
  int32_t chunks_per_rank;  // slots reserved per CTA_rank
  int32_t num_slots;        // max_split_per_seq * chunks_per_rank
  int32_t max_split;
  int32_t total_items;      // workgroups over all buckets: (box, chunk) items x head groups, head group fastest
  float scale_log2;         // softmax_scale * log2(e)
  int32_t num_buckets;
  uint32_t hpp_magic;       // ceil(2^32 / (page_size / 16)): h / (page_size / 16) == umulhi(h, hpp_magic) for h < 2^16; unused when page_size / 16 is a power of two
  int32_t item_begin[kMaxBuckets];  // copy of bucket[i].item_begin at fixed offsets (INT32_MAX past the end)
  BucketDev bucket[kMaxBuckets];
  // single-slot launches (every row has one partial slot; no merge kernel follows): the rows go
  // to `out`. Kept behind the fields every launch reads, whose offsets the bucket search relies on.
  void* out;         // [batch, 1, heads, head_dim] in the element type
  float* lse_out;    // optional [batch, heads] fp32
  int64_t o_stride_b, o_stride_h;              // elements
  int32_t direct;    // 1: such a launch
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
