// extern "C" surface of the scheduler (declared in include/pat_amd.h).
#include <algorithm>
#include <climits>
#include <cstdint>
#include <cstring>
#include <memory>
#include <new>
#include <string>
#include <vector>

#include "capi_error.hpp"
#include "pat_amd.h"
#include "sched/radix_plan.hpp"

struct pat_tree {
  int block_size;
  std::unique_ptr<pat::RadixPlanner> planner;
  std::vector<int32_t> child_scratch;
};

namespace pat {
thread_local std::string g_last_error;
int fail(int code, const std::string& msg) {
  g_last_error = msg;
  return code;
}
}  // namespace pat

namespace {
template <typename F>
int guarded(F&& f) {
  try {
    f();
    return PAT_OK;
  } catch (const pat::SchedError& e) {
    return pat::fail(e.code, e.msg);
  } catch (const std::bad_alloc&) {
    return pat::fail(PAT_ERR_INVALID, "out of host memory");
  } catch (const std::exception& e) {
    return pat::fail(PAT_ERR_INVALID, e.what());
  }
}
}  // namespace

extern "C" {

const char* pat_last_error(void) { return pat::g_last_error.c_str(); }
int pat_abi_version(void) { return PAT_ABI_VERSION; }

int pat_tree_create(int32_t block_size, pat_tree** out) {
  if (out == nullptr) return pat::fail(PAT_ERR_INVALID, "pat_tree_create: out is NULL");
  if (block_size <= 0) return pat::fail(PAT_ERR_INVALID, "block_size must be positive");
  return guarded([&] {
    auto* t = new pat_tree;
    t->block_size = block_size;
    t->planner.reset(new pat::RadixPlanner(block_size));
    *out = t;
  });
}

void pat_tree_destroy(pat_tree* tree) { delete tree; }

int pat_tree_build_rows(pat_tree* tree, const int32_t* seq_lens, const int32_t* flat_blocks,
                        const int64_t* row_offsets, int32_t num_seqs) {
  if (tree == nullptr) return pat::fail(PAT_ERR_INVALID, "tree is NULL");
  if (num_seqs < 0) return pat::fail(PAT_ERR_INVALID, "num_seqs must be >= 0");
  if (num_seqs > 0 && (seq_lens == nullptr || row_offsets == nullptr))
    return pat::fail(PAT_ERR_INVALID, "seq_lens / row_offsets is NULL");
  for (int i = 0; i < num_seqs; ++i)
    if (row_offsets[i + 1] < row_offsets[i])
      return pat::fail(PAT_ERR_INVALID, "row_offsets must be non-decreasing");
  if (num_seqs > 0 && row_offsets[num_seqs] > row_offsets[0] && flat_blocks == nullptr)
    return pat::fail(PAT_ERR_INVALID, "flat_blocks is NULL");
  return guarded([&] {
    // A tree is built once per batch; building again starts from an empty tree.
    tree->planner.reset(new pat::RadixPlanner(tree->block_size));
    tree->planner->build(seq_lens, flat_blocks, row_offsets, num_seqs);
  });
}

int pat_tree_build(pat_tree* tree, const int32_t* seq_lens, const int32_t* table,
                   int32_t num_seqs, int32_t max_blocks) {
  if (tree == nullptr) return pat::fail(PAT_ERR_INVALID, "tree is NULL");
  if (num_seqs < 0 || max_blocks < 0)
    return pat::fail(PAT_ERR_INVALID, "num_seqs / max_blocks must be >= 0");
  if (num_seqs > 0 && (seq_lens == nullptr || (table == nullptr && max_blocks > 0)))
    return pat::fail(PAT_ERR_INVALID, "seq_lens / block_table is NULL");
  const int bs = tree->block_size;
  std::vector<int64_t> offsets((size_t)num_seqs + 1, 0);
  std::vector<int32_t> flat;
  for (int i = 0; i < num_seqs; ++i) {
    if (seq_lens[i] < 0) return pat::fail(PAT_ERR_INVALID, "seq_lens must be >= 0");
    const int64_t used = ((int64_t)seq_lens[i] + bs - 1) / bs;
    if (used > max_blocks)
      return pat::fail(PAT_ERR_INVALID, "seq_lens[" + std::to_string(i) + "] needs " +
                                            std::to_string(used) + " blocks but block_table has " +
                                            std::to_string(max_blocks) + " columns");
    const int32_t* row = table + (int64_t)i * max_blocks;
    flat.insert(flat.end(), row, row + used);
    offsets[(size_t)i + 1] = (int64_t)flat.size();
  }
  return pat_tree_build_rows(tree, seq_lens, flat.data(), offsets.data(), num_seqs);
}

int pat_tree_append(pat_tree* tree, int32_t seq_len, const int32_t* blocks, int32_t num_blocks) {
  if (tree == nullptr) return pat::fail(PAT_ERR_INVALID, "tree is NULL");
  if (seq_len < 0 || num_blocks < 0) return pat::fail(PAT_ERR_INVALID, "seq_len / num_blocks must be >= 0");
  if (num_blocks > 0 && blocks == nullptr) return pat::fail(PAT_ERR_INVALID, "blocks is NULL");
  return guarded([&] { tree->planner->append(seq_len, blocks, num_blocks); });
}

int pat_tree_remove(pat_tree* tree, int32_t seq) {
  if (tree == nullptr) return pat::fail(PAT_ERR_INVALID, "tree is NULL");
  return guarded([&] { tree->planner->remove(seq); });
}

int pat_tree_grow(pat_tree* tree, int32_t seq, int32_t new_len, const int32_t* more_blocks, int32_t num_more) {
  if (tree == nullptr) return pat::fail(PAT_ERR_INVALID, "tree is NULL");
  if (num_more > 0 && more_blocks == nullptr) return pat::fail(PAT_ERR_INVALID, "more_blocks is NULL");
  return guarded([&] { tree->planner->grow(seq, new_len, more_blocks, num_more); });
}

int pat_tree_num_seqs(const pat_tree* tree) {
  if (tree == nullptr) return pat::fail(PAT_ERR_INVALID, "tree is NULL");
  return tree->planner->num_seqs();
}

int pat_tree_pack(pat_tree* tree, const int32_t* mnws, int32_t n_mnws, int32_t hratio,
                  int32_t kv_heads, int32_t use_compute_model, const pat_sched_opts* opts) {
  if (tree == nullptr) return pat::fail(PAT_ERR_INVALID, "tree is NULL");
  if (n_mnws > 0 && mnws == nullptr) return pat::fail(PAT_ERR_INVALID, "mnws is NULL");
  return guarded(
      [&] { tree->planner->pack(mnws, n_mnws, hratio, kv_heads, use_compute_model != 0, opts); });
}

int pat_tree_naive_schedule(pat_tree* tree, int32_t hratio) {
  if (tree == nullptr) return pat::fail(PAT_ERR_INVALID, "tree is NULL");
  return guarded([&] { tree->planner->naive(hratio); });
}

int pat_tree_plan(const pat_tree* tree, pat_plan_view* out) {
  if (tree == nullptr || out == nullptr) return pat::fail(PAT_ERR_INVALID, "tree / out is NULL");
  const pat::Plan& p = tree->planner->plan();
  if (!p.valid) return pat::fail(PAT_ERR_INVALID, "no plan: call pat_tree_pack first");
  out->num_buckets = (int32_t)p.views.size();
  out->batch = (int32_t)p.num_split_per_seq.size();
  out->buckets = p.views.data();
  out->num_split_per_seq = p.num_split_per_seq.data();
  out->max_split_per_seq = p.max_split;
  out->max_seqs_in_box = p.max_seqs_in_box;
  out->max_blocks_in_box = p.max_blocks_in_box;
  out->num_boxes_per_seq = p.num_boxes_per_seq.data();
  out->max_boxes_per_seq = p.max_boxes;
  return PAT_OK;
}

static int flat_plan_impl(const pat_tree* tree, pat_flat_plan* layout, int32_t* dst, int64_t capacity) {
  if (tree == nullptr || layout == nullptr) return pat::fail(PAT_ERR_INVALID, "tree / layout is NULL");
  const pat::Plan& p = tree->planner->plan();
  if (!p.valid) return pat::fail(PAT_ERR_INVALID, "no plan: call pat_tree_pack first");
  const int nb = (int)p.buckets.size();
  if (nb > PAT_MAX_FLAT_BUCKETS)
    return pat::fail(PAT_ERR_INVALID, "the flat plan holds at most 12 buckets");
  constexpr int kGrowthBlocks = 8;
  std::memset(layout, 0, sizeof(*layout));
  layout->num_buckets = nb;
  layout->batch = (int32_t)p.num_split_per_seq.size();
  layout->max_split_per_seq = p.max_split;
  layout->max_boxes_per_seq = p.max_boxes;
  layout->max_seqs_in_box = p.max_seqs_in_box;
  layout->max_blocks_in_box = p.max_blocks_in_box;

  // launch order and parts of every bucket
  struct Part { int parent, lo, hi, width; };
  std::vector<std::vector<int32_t>> order((size_t)nb);
  std::vector<Part> parts;
  int spare = PAT_MAX_FLAT_BUCKETS - nb;
  for (int b = 0; b < nb; ++b) {
    const pat::Bucket& bk = p.buckets[(size_t)b];
    const int n = (int)bk.kv.size();
    auto& ord = order[(size_t)b];
    ord.resize((size_t)n);
    for (int i = 0; i < n; ++i) ord[(size_t)i] = i;
    std::stable_sort(ord.begin(), ord.end(), [&](int32_t x, int32_t y) { return bk.kv[(size_t)x] > bk.kv[(size_t)y]; });
    int cut = 0;
    if (spare > 0 && n >= 4) {
      const int32_t widest = bk.kv[(size_t)ord[0]];
      int k = 0;
      while (k < n && bk.kv[(size_t)ord[(size_t)k]] > widest / 2) ++k;
      if (k > 0 && k <= n / 4) { cut = k; --spare; }
    }
    if (cut == 0) {
      parts.push_back({b, 0, n, bk.max_blocks});
    } else {
      parts.push_back({b, 0, cut, bk.max_blocks});
      int32_t longest = 1;
      for (int i = cut; i < n; ++i) longest = std::max(longest, bk.block_len[(size_t)ord[(size_t)i]]);
      parts.push_back({b, cut, n, std::min<int32_t>(bk.max_blocks, longest + kGrowthBlocks)});
    }
  }
  layout->num_launch_buckets = (int32_t)parts.size();

  // offsets
  int64_t at = 0;
  auto take = [&](int64_t n) { const int64_t o = at; at += n; return o; };
  layout->num_split_per_seq = take(layout->batch);
  layout->num_boxes_per_seq = take(layout->batch);
  auto place = [&](pat_flat_bucket& f, const pat::Bucket& bk, int rows, int width, int parent, int first) {
    std::memcpy(f.mnw, bk.mnw, sizeof(f.mnw));
    f.num_boxes = rows; f.max_seqs = bk.max_seqs; f.max_blocks = width; f.parent = parent; f.first = first;
    f.flags = 0;
    f.q_table = take((int64_t)rows * bk.max_seqs);
    f.q_slot = take((int64_t)rows * bk.max_seqs);
    f.block_table = take((int64_t)rows * width);
    f.num_seqs = take(rows); f.rank = take(rows); f.kv = take(rows);
  };
  for (int b = 0; b < nb; ++b) {
    const pat::Bucket& bk = p.buckets[(size_t)b];
    place(layout->buckets[b], bk, (int)bk.kv.size(), bk.max_blocks, b, 0);
    layout->launch_order[b] = take((int64_t)bk.kv.size());
  }
  for (size_t i = 0; i < parts.size(); ++i) {
    const Part& pt = parts[i];
    place(layout->launch[i], p.buckets[(size_t)pt.parent], pt.hi - pt.lo, pt.width, pt.parent, pt.lo);
  }
  // hints: a bucket is even when no box is shorter than 3/4 of its widest one
  auto even = [&](const pat::Bucket& bk, const int32_t* ord, int lo, int hi) {
    int32_t widest = 0, shortest = INT32_MAX;
    for (int i = lo; i < hi; ++i) {
      const int32_t t = bk.kv[(size_t)(ord ? ord[i] : i)];
      widest = std::max(widest, t); shortest = std::min(shortest, t);
    }
    return hi > lo && (int64_t)shortest * 4 >= (int64_t)widest * 3 ? PAT_BUCKET_EVEN : 0;
  };
  for (int b = 0; b < nb; ++b)
    layout->buckets[b].flags = even(p.buckets[(size_t)b], nullptr, 0, (int)p.buckets[(size_t)b].kv.size());
  for (size_t i = 0; i < parts.size(); ++i)
    layout->launch[i].flags = even(p.buckets[(size_t)parts[i].parent], order[(size_t)parts[i].parent].data(), parts[i].lo, parts[i].hi);
  layout->total = at;
  if (dst == nullptr) return PAT_OK;
  if (capacity < at) return pat::fail(PAT_ERR_INVALID, "flat plan: buffer too small");

  // contents
  std::copy(p.num_split_per_seq.begin(), p.num_split_per_seq.end(), dst + layout->num_split_per_seq);
  std::copy(p.num_boxes_per_seq.begin(), p.num_boxes_per_seq.end(), dst + layout->num_boxes_per_seq);
  auto rows_to = [&](int32_t* out, const std::vector<int32_t>& table, int src_width, int width,
                     const int32_t* ord, int lo, int hi) {
    for (int i = lo; i < hi; ++i) {
      const int32_t* row = table.data() + (size_t)(ord ? ord[i] : i) * (size_t)src_width;
      std::copy(row, row + width, out + (size_t)(i - lo) * (size_t)width);
    }
  };
  auto vec_to = [&](int32_t* out, const std::vector<int32_t>& v, const int32_t* ord, int lo, int hi) {
    for (int i = lo; i < hi; ++i) out[i - lo] = v[(size_t)(ord ? ord[i] : i)];
  };
  auto fill = [&](const pat_flat_bucket& f, const pat::Bucket& bk, const int32_t* ord, int lo, int hi) {
    rows_to(dst + f.q_table, bk.q_table, bk.max_seqs, bk.max_seqs, ord, lo, hi);
    rows_to(dst + f.q_slot, bk.q_slot, bk.max_seqs, bk.max_seqs, ord, lo, hi);
    rows_to(dst + f.block_table, bk.block_table, bk.max_blocks, f.max_blocks, ord, lo, hi);
    vec_to(dst + f.num_seqs, bk.num_seqs, ord, lo, hi);
    vec_to(dst + f.rank, bk.rank, ord, lo, hi);
    vec_to(dst + f.kv, bk.kv, ord, lo, hi);
  };
  for (int b = 0; b < nb; ++b) {
    const pat::Bucket& bk = p.buckets[(size_t)b];
    fill(layout->buckets[b], bk, nullptr, 0, (int)bk.kv.size());
    std::copy(order[(size_t)b].begin(), order[(size_t)b].end(), dst + layout->launch_order[b]);
  }
  for (size_t i = 0; i < parts.size(); ++i) {
    const Part& pt = parts[i];
    fill(layout->launch[i], p.buckets[(size_t)pt.parent], order[(size_t)pt.parent].data(), pt.lo, pt.hi);
  }
  return PAT_OK;
}

int pat_tree_flat_plan(const pat_tree* tree, pat_flat_plan* layout, int32_t* dst, int64_t capacity) {
  int rc = PAT_OK;
  const int thrown = guarded([&] { rc = flat_plan_impl(tree, layout, dst, capacity); });
  return thrown ? thrown : rc;
}

int pat_tree_num_nodes(const pat_tree* tree) {
  if (tree == nullptr) return pat::fail(PAT_ERR_INVALID, "tree is NULL");
  return (int)tree->planner->nodes().size();
}

int pat_tree_node(const pat_tree* tree, int32_t node, pat_node_view* out) {
  if (tree == nullptr || out == nullptr) return pat::fail(PAT_ERR_INVALID, "tree / out is NULL");
  const auto& nodes = tree->planner->nodes();
  if (node < 0 || (size_t)node >= nodes.size())
    return pat::fail(PAT_ERR_INDEX, "node index out of range");
  const pat::RadixNode& n = nodes[(size_t)node];
  out->parent = n.parent;
  out->num_seqs = n.num_seqs;
  out->num_tokens = n.num_tokens;
  out->num_seq_ids = (int32_t)n.seq_ids.size();
  out->num_blocks = (int32_t)n.blocks.size();
  out->num_children = (int32_t)n.child_ids.size();
  out->seq_ids = n.seq_ids.data();
  out->block_ids = n.blocks.data();
  out->child_ids = n.child_ids.data();
  return PAT_OK;
}

}  // extern "C"
