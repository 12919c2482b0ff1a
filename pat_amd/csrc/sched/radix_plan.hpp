// Host-side scheduler of libpat_amd: radix tree over block-table rows, the
// split/merge packing heuristic, the load balancer and tile bucketing.
//
// The plan it emits is defined to be bit-identical with the reference's *Python*
// scheduler (prefix_attn/prefix_tree.py), including its incidental behaviours
// (dict insertion order of children, pop/append reordering in the balancer, the
// float ceil in the long-box cut). Nothing here depends on torch or HIP.
#pragma once

#include <cstdint>
#include <string>
#include <unordered_map>
#include <vector>

#include "pat_amd.h"

namespace pat {

// Thrown for conditions where the Python scheduler raises; `code` is a PAT_ERR_*.
struct SchedError {
  int code;
  std::string msg;
};

struct RadixNode {
  int parent = -1;
  int num_seqs = 1;               // "s_value"
  int num_tokens = 0;             // "lens"
  std::vector<int32_t> seq_ids;   // sequences recorded on the node
  std::vector<int32_t> blocks;    // physical block ids held by the node
  // Children in first-insertion order, keyed by their first block id. Replacing
  // the child under an existing key keeps the key's position (Python dict rule).
  std::vector<int32_t> child_keys;
  std::vector<int32_t> child_ids;
  std::unordered_map<int32_t, int32_t> key_pos;

  int find(int32_t key) const {
    auto it = key_pos.find(key);
    return it == key_pos.end() ? -1 : child_ids[it->second];
  }
  void drop(int32_t key) {
    auto it = key_pos.find(key);
    if (it == key_pos.end()) return;
    const int32_t at = it->second;
    child_keys.erase(child_keys.begin() + at);
    child_ids.erase(child_ids.begin() + at);
    key_pos.clear();
    for (size_t i = 0; i < child_keys.size(); ++i) key_pos.emplace(child_keys[i], (int32_t)i);
  }
  void put(int32_t key, int32_t child) {
    auto it = key_pos.find(key);
    if (it == key_pos.end()) {
      key_pos.emplace(key, (int32_t)child_ids.size());
      child_keys.push_back(key);
      child_ids.push_back(child);
    } else {
      child_ids[it->second] = child;
    }
  }
};

// One packed work item: a group of sequences attending to one run of KV blocks.
struct Box {
  std::vector<int32_t> seqs;    // q_table
  std::vector<int32_t> blocks;  // block_table
  int num_seqs = 0;             // num_seqs_per_CTA
  int kv = 0;                   // kv_in_CTA (tokens)
  int rank = 0;                 // CTA_rank
};

struct Bucket {
  int32_t mnw[3];
  int32_t max_seqs = 0, max_blocks = 0;
  std::vector<int32_t> q_table, block_table;  // padded, row-major
  std::vector<int32_t> q_slot;                // padded like q_table
  std::vector<int32_t> q_len, block_len, num_seqs, rank, kv;
};

struct Plan {
  std::vector<Bucket> buckets;
  std::vector<pat_bucket_view> views;
  std::vector<int32_t> num_split_per_seq;
  std::vector<int32_t> num_boxes_per_seq;   // boxes of this plan that hold each sequence
  int max_boxes = 0;
  int max_split = 0, max_seqs_in_box = 0, max_blocks_in_box = 0;
  bool valid = false;
};

class RadixPlanner {
 public:
  explicit RadixPlanner(int block_size);

  // rows[i] = block ids of sequence i (used whole).
  void build(const int32_t* seq_lens, const int32_t* flat_blocks, const int64_t* row_offsets,
             int num_seqs);
  // Edits of a built tree between decode steps. Each leaves the tree as build() would make it from the
  // edited batch (same nodes, children order, sequence lists and token counts), with the split counters
  // of a fresh tree, provided that every block two sequences share is full for both (what a paged KV
  // cache with prefix sharing guarantees). Sequence ids are batch rows: append() adds row num_seqs(),
  // remove() deletes a row and moves the later ones up, grow() lengthens a row in place.
  void append(int seq_len, const int32_t* blocks, int n);
  void remove(int seq);
  void grow(int seq, int new_len, const int32_t* more_blocks, int n_more);
  int num_seqs() const { return (int)seq_len_.size(); }

  void pack(const int32_t* mnws, int n_mnws, int hratio, int kv_heads, bool compute_model,
            const pat_sched_opts* opts);
  void naive(int hratio);

  const std::vector<RadixNode>& nodes() const { return nodes_; }
  const Plan& plan() const { return plan_; }
  int block_size() const { return bs_; }

 private:
  int add_node(int parent, int num_seqs, int num_tokens, std::vector<int32_t> seq_ids,
               std::vector<int32_t> blocks);
  void insert(int seq, int seq_len, const int32_t* blocks, int n);
  void emit_boxes(std::vector<Box>& out, const std::vector<int32_t>& seqs, int count, int mm,
                  const std::vector<int32_t>& inherited, const RadixNode& node);
  void descend(std::vector<Box>& out, int node, int mm, int hratio, bool compute_model,
               const std::vector<int32_t>& inherited);
  void descend_naive(std::vector<Box>& out, int node, int mm);
  std::vector<Box> balance(std::vector<Box> boxes, int kv_heads, const pat_sched_opts& o);
  void bucketize(const std::vector<Box>& boxes, const std::vector<std::vector<int32_t>>& buckets,
                 int hratio, bool force_single);

  std::vector<int> path_of(int seq) const;   // nodes that hold `seq`, root's child first
  void release_node(int node);
  void sort_children(int node);

  int bs_;
  std::vector<RadixNode> nodes_;
  std::vector<int> free_nodes_;              // slots of nodes_ given up by remove()
  std::vector<int32_t> seq_len_;             // tokens of each sequence
  std::vector<int32_t> split_per_seq_;
  Plan plan_;
};

void tile_label(int rows, int kv_tokens, int32_t out[3]);

}  // namespace pat
