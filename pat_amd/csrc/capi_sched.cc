// extern "C" surface of the scheduler (declared in include/pat_amd.h).
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
  return PAT_OK;
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
