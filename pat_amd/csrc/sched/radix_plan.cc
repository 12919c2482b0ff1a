// Scheduler implementation. Each function names the part of the reference's Python
// scheduler whose observable behaviour it reproduces (paths relative to the
// flashserve/PAT tree).
#include "radix_plan.hpp"

#include <algorithm>
#include <cmath>
#include <map>

namespace pat {

namespace {

const int32_t kDefaultBuckets[11][3] = {
    {64, 128, 4}, {64, 64, 4}, {64, 32, 4},              //
    {32, 128, 2}, {32, 64, 2}, {32, 32, 2}, {32, 16, 2},  //
    {16, 128, 1}, {16, 64, 1}, {16, 32, 1}, {16, 16, 1}};

const pat_sched_opts kReferenceOpts = {256, 5, {54, 27, 13, 6, 4}, 8, 32};

inline int64_t ceil_div(int64_t a, int64_t b) { return (a + b - 1) / b; }

// Python's % for a positive modulus.
inline int64_t py_mod(int64_t a, int64_t m) {
  int64_t r = a % m;
  return r < 0 ? r + m : r;
}

// Cost model of the optional "compute model" heuristic
// (prefix_attn/prefix_tree.py:16-45). Integer parts stay exact; only the merge
// penalty is a double, as in Python.
inline int64_t pad_rows(int64_t tile, int64_t n) { return tile - (py_mod(n - 1, tile) + 1); }
inline int64_t matmul_waste(int64_t n_q, int64_t n_k, int64_t hratio) {
  const int64_t tile = (n_q * hratio >= 64) ? 64 : 16;
  return pad_rows(tile, n_q) * n_k * hratio;
}

// Longest common prefix of two block runs, found the way the reference finds it:
// a binary search that presumes "equal up to some point, different after"
// (prefix_attn/prefix_tree.py:81-89). Returns the number of common blocks.
inline int common_prefix_blocks(const int32_t* a, int na, const int32_t* b, int nb) {
  int lo = -1, hi = std::min(na, nb);
  while (hi - lo > 1) {
    const int mid = (lo + hi) >> 1;
    if (a[mid] == b[mid]) lo = mid; else hi = mid;
  }
  return lo + 1;
}

}  // namespace

// Tile label of a box (prefix_attn/prefix_tree.py:462-482): M/W from the row count,
// N from the KV length, with N >= 32 whenever M == 64.
void tile_label(int rows, int kv_tokens, int32_t out[3]) {
  int m = 16, w = 1;
  if (rows > 32) { m = 64; w = 4; }
  else if (rows > 16) { m = 32; w = 2; }
  int n;
  if (kv_tokens < 32) n = 16;
  else if (kv_tokens < 64) n = 32;
  else if (kv_tokens <= 128) n = 64;
  else n = 128;
  if (m == 64) n = std::max(32, n);
  out[0] = m; out[1] = n; out[2] = w;
}

RadixPlanner::RadixPlanner(int block_size) : bs_(block_size) {
  add_node(-1, 1, 0, {}, {});  // root (prefix_attn/prefix_tree.py:58)
}

int RadixPlanner::add_node(int parent, int num_seqs, int num_tokens, std::vector<int32_t> seq_ids,
                           std::vector<int32_t> blocks) {
  RadixNode n;
  n.parent = parent;
  n.num_seqs = num_seqs;
  n.num_tokens = num_tokens;
  n.seq_ids = std::move(seq_ids);
  n.blocks = std::move(blocks);
  if (!free_nodes_.empty()) {
    const int at = free_nodes_.back();
    free_nodes_.pop_back();
    nodes_[(size_t)at] = std::move(n);
    return at;
  }
  nodes_.push_back(std::move(n));
  return (int)nodes_.size() - 1;
}

// prefix_attn/prefix_tree.py:95-144
void RadixPlanner::insert(int seq, int seq_len, const int32_t* blocks, int n) {
  int at = 0;  // root
  int left = n;
  while (left > 0) {
    const int32_t key = blocks[0];
    const int child = nodes_[at].find(key);
    if (child < 0) {
      const int leaf = add_node(at, 1, seq_len, {seq}, std::vector<int32_t>(blocks, blocks + left));
      nodes_[at].put(key, leaf);
      return;
    }
    const int child_blocks = (int)nodes_[child].blocks.size();
    const int common = common_prefix_blocks(blocks, left, nodes_[child].blocks.data(), child_blocks);
    if (common == child_blocks) {
      // the whole edge matches: walk down
      nodes_[child].num_seqs += 1;
      nodes_[child].seq_ids.push_back(seq);
      at = child;
      left -= common;
      seq_len -= common * bs_;
      blocks += common;
      continue;
    }
    // the edge matches only partly: cut it at `common`
    std::vector<int32_t> head(nodes_[child].blocks.begin(), nodes_[child].blocks.begin() + common);
    std::vector<int32_t> tail(nodes_[child].blocks.begin() + common, nodes_[child].blocks.end());
    const int32_t first = nodes_[child].blocks[0];
    const int mid = add_node(at, nodes_[child].num_seqs + 1, common * bs_, nodes_[child].seq_ids,
                             std::move(head));
    nodes_[mid].put(tail[0], child);
    nodes_[at].put(first, mid);
    nodes_[child].parent = mid;
    nodes_[child].num_tokens -= common * bs_;
    nodes_[child].blocks = std::move(tail);
    nodes_[mid].seq_ids.push_back(seq);
    if (common == left) return;  // the sequence ends on the cut itself
    const int leaf_tokens = std::min(left * bs_, seq_len) - common * bs_;
    const int leaf = add_node(mid, 1, leaf_tokens, {seq},
                              std::vector<int32_t>(blocks + common, blocks + left));
    nodes_[mid].put(blocks[common], leaf);
    return;
  }
}

// prefix_attn/prefix_tree.py:146-149
void RadixPlanner::build(const int32_t* seq_lens, const int32_t* flat_blocks,
                         const int64_t* row_offsets, int num_seqs) {
  for (int i = 0; i < num_seqs; ++i) {
    const int64_t b = row_offsets[i], e = row_offsets[i + 1];
    insert(i, seq_lens[i], flat_blocks + b, (int)(e - b));
  }
  seq_len_.assign(seq_lens, seq_lens + num_seqs);
  split_per_seq_.assign((size_t)num_seqs, 0);
}

// ---- edits of a built tree ---------------------------------------------------------------------
// The reference builds a new tree for every decode step
// (plugin/vllm/attention/backends/prefix_attn.py:330-338); these keep one tree in step with the batch.
// What makes the result equal to a fresh build: build() inserts rows in order, so a node's sequence
// list is ascending, and the children of a node stand in the order of their smallest sequence id
// (a child is created by the first row that needs it, and a cut keeps the cut child's place).

std::vector<int> RadixPlanner::path_of(int seq) const {
  std::vector<int> path;
  int at = 0;
  for (;;) {
    int next = -1;
    for (int child : nodes_[(size_t)at].child_ids) {
      const auto& ids = nodes_[(size_t)child].seq_ids;
      if (std::binary_search(ids.begin(), ids.end(), (int32_t)seq)) { next = child; break; }
    }
    if (next < 0) return path;
    path.push_back(next);
    at = next;
  }
}

void RadixPlanner::release_node(int node) {
  nodes_[(size_t)node] = RadixNode();
  nodes_[(size_t)node].parent = -2;   // not part of the tree
  nodes_[(size_t)node].num_seqs = 0;
  free_nodes_.push_back(node);
}

void RadixPlanner::sort_children(int node) {
  RadixNode& n = nodes_[(size_t)node];
  std::vector<size_t> order(n.child_ids.size());
  for (size_t i = 0; i < order.size(); ++i) order[i] = i;
  std::stable_sort(order.begin(), order.end(), [&](size_t a, size_t b) {
    return nodes_[(size_t)n.child_ids[a]].seq_ids.front() < nodes_[(size_t)n.child_ids[b]].seq_ids.front();
  });
  std::vector<int32_t> keys, ids;
  for (size_t i : order) { keys.push_back(n.child_keys[i]); ids.push_back(n.child_ids[i]); }
  n.child_keys = std::move(keys);
  n.child_ids = std::move(ids);
  n.key_pos.clear();
  for (size_t i = 0; i < n.child_keys.size(); ++i) n.key_pos.emplace(n.child_keys[i], (int32_t)i);
}

void RadixPlanner::append(int seq_len, const int32_t* blocks, int n) {
  const int seq = num_seqs();
  insert(seq, seq_len, blocks, n);
  seq_len_.push_back(seq_len);
  split_per_seq_.assign(seq_len_.size(), 0);
}

void RadixPlanner::remove(int seq) {
  if (seq < 0 || seq >= num_seqs()) throw SchedError{PAT_ERR_INDEX, "sequence index out of range"};
  const std::vector<int> path = path_of(seq);
  for (int node : path) {
    auto& ids = nodes_[(size_t)node].seq_ids;
    ids.erase(std::lower_bound(ids.begin(), ids.end(), (int32_t)seq));
    nodes_[(size_t)node].num_seqs -= 1;
  }
  // rows after the removed one move up
  for (RadixNode& n : nodes_)
    for (int32_t& id : n.seq_ids)
      if (id > seq) id -= 1;
  // deepest first: nodes without sequences go, and a node left with a single child that takes all of
  // its sequences is that child's head again (the cut that made it is undone)
  for (size_t i = path.size(); i-- > 0;) {
    const int node = path[i];
    const int parent = nodes_[(size_t)node].parent;
    if (nodes_[(size_t)node].seq_ids.empty()) {
      // (a node without sequences has no children: each child's sequences are among its own)
      nodes_[(size_t)parent].drop(nodes_[(size_t)node].blocks.empty() ? 0 : nodes_[(size_t)node].blocks[0]);
      release_node(node);
      continue;
    }
    RadixNode& n = nodes_[(size_t)node];
    if (n.child_ids.size() == 1 && nodes_[(size_t)n.child_ids[0]].num_seqs == n.num_seqs) {
      const int child = n.child_ids[0];
      RadixNode& c = nodes_[(size_t)child];
      n.blocks.insert(n.blocks.end(), c.blocks.begin(), c.blocks.end());
      n.num_tokens += c.num_tokens;
      n.child_keys = std::move(c.child_keys);
      n.child_ids = std::move(c.child_ids);
      n.key_pos = std::move(c.key_pos);
      for (int grandchild : n.child_ids) nodes_[(size_t)grandchild].parent = node;
      release_node(child);
    }
  }
  // a child whose smallest sequence id was the removed one may have to move back among its siblings
  for (int node : path)
    if (nodes_[(size_t)node].parent != -2) sort_children(nodes_[(size_t)node].parent);
  sort_children(0);
  seq_len_.erase(seq_len_.begin() + seq);
  split_per_seq_.assign(seq_len_.size(), 0);
}

void RadixPlanner::grow(int seq, int new_len, const int32_t* more_blocks, int n_more) {
  if (seq < 0 || seq >= num_seqs()) throw SchedError{PAT_ERR_INDEX, "sequence index out of range"};
  const int old_len = seq_len_[(size_t)seq];
  if (new_len < old_len || n_more < 0) throw SchedError{PAT_ERR_VALUE, "a sequence can only grow"};
  const std::vector<int> path = path_of(seq);
  if (path.empty()) throw SchedError{PAT_ERR_VALUE, "the sequence has no blocks in the tree: build it again"};
  const int last = path.back();
  RadixNode& tail = nodes_[(size_t)last];
  if (tail.seq_ids.size() == 1 && tail.child_ids.empty()) {
    // its own leaf: more tokens, and the new blocks behind the old ones
    tail.blocks.insert(tail.blocks.end(), more_blocks, more_blocks + n_more);
    tail.num_tokens += new_len - old_len;
  } else {
    // the sequence ended on a node it shares: the new blocks become its own leaf under that node,
    // unless they continue into one of the node's children (then only a fresh build knows the shape)
    if (n_more == 0) {
      if (new_len != old_len)
        throw SchedError{PAT_ERR_VALUE, "a sequence grew inside a block it shares: build the tree again"};
    } else {
      if (tail.find(more_blocks[0]) >= 0)
        throw SchedError{PAT_ERR_VALUE, "a sequence grew into blocks another one holds: build the tree again"};
      int shared_tokens = 0;
      for (int node : path) shared_tokens += nodes_[(size_t)node].num_tokens;
      const int leaf = add_node(last, 1, new_len - shared_tokens, {(int32_t)seq},
                                std::vector<int32_t>(more_blocks, more_blocks + n_more));
      nodes_[(size_t)last].put(more_blocks[0], leaf);
      sort_children(last);
    }
  }
  seq_len_[(size_t)seq] = new_len;
  split_per_seq_.assign(seq_len_.size(), 0);
}

// Cuts `count` sequences (ids taken from `seqs`) into boxes of at most mm sequences
// over the KV run inherited + node.blocks, handing out the next free rank of each
// box's first sequence (prefix_attn/prefix_tree.py:277-286, 307-316).
void RadixPlanner::emit_boxes(std::vector<Box>& out, const std::vector<int32_t>& seqs, int count,
                              int mm, const std::vector<int32_t>& inherited,
                              const RadixNode& node) {
  if (mm == 0) throw SchedError{PAT_ERR_VALUE, "range() arg 3 must not be zero"};
  for (int s = 0; s < count; s += mm) {
    Box box;
    const int lo = std::min<int>(s, (int)seqs.size());
    const int hi = std::min<int>(std::min(s + mm, count), (int)seqs.size());
    box.seqs.assign(seqs.begin() + lo, seqs.begin() + std::max(lo, hi));
    box.blocks = inherited;
    box.blocks.insert(box.blocks.end(), node.blocks.begin(), node.blocks.end());
    box.num_seqs = std::min(mm, count - s);
    box.kv = bs_ * (int)inherited.size() + node.num_tokens;
    if (box.seqs.empty()) throw SchedError{PAT_ERR_INDEX, "list index out of range"};
    box.rank = split_per_seq_.at((size_t)box.seqs[0]);
    for (int32_t q : box.seqs) split_per_seq_.at((size_t)q) += 1;
    out.push_back(std::move(box));
  }
}

// prefix_attn/prefix_tree.py:269-323 (and :325-381 when compute_model is set)
void RadixPlanner::descend(std::vector<Box>& out, int node_id, int mm, int hratio,
                           bool compute_model, const std::vector<int32_t>& inherited) {
  const RadixNode& node = nodes_[node_id];
  if (node.child_ids.empty()) {
    emit_boxes(out, node.seq_ids, node.num_seqs, mm, inherited, node);
    return;
  }
  int remaining = node.num_seqs;  // sequences still served by this node's own boxes
  const int64_t kv_len = (int64_t)bs_ * (int64_t)inherited.size() + node.num_tokens;
  std::vector<int> keep_here, push_down;
  for (int child : node.child_ids) {
    const int sc = nodes_[child].num_seqs;
    bool merge;
    if (compute_model) {
      // Call sites prefix_tree.py:352-353: the "split K" cost receives this node's
      // KV length in the child-length slot and vice versa.
      const int64_t child_len = nodes_[child].num_tokens;
      const int64_t cost_k_int = matmul_waste(remaining, child_len, hratio) +
                                 matmul_waste(sc, kv_len, hratio);
      const double cost_k = (double)cost_k_int + (0.1 * (double)sc) * (double)hratio;
      const int64_t cost_q = matmul_waste(remaining - sc, kv_len, hratio) +
                             matmul_waste(sc, kv_len + child_len, hratio);
      merge = cost_k > (double)cost_q;
    } else {
      if (remaining == sc) {
        merge = true;
      } else {
        if (mm == 0) throw SchedError{PAT_ERR_VALUE, "division by zero"};
        const int64_t tiles_saved = ceil_div(remaining, mm) - ceil_div(remaining - sc, mm) -
                                    ceil_div(sc, mm);
        merge = tiles_saved * kv_len + 4 * (int64_t)sc >= 0;
      }
    }
    if (merge) { remaining -= sc; push_down.push_back(child); }
    else keep_here.push_back(child);
  }
  if (remaining != 0) {
    std::vector<int32_t> seqs;
    for (int child : keep_here)
      seqs.insert(seqs.end(), nodes_[child].seq_ids.begin(), nodes_[child].seq_ids.end());
    emit_boxes(out, seqs, remaining, mm, inherited, node);
  }
  const std::vector<int32_t> none;
  for (int child : keep_here) descend(out, child, mm, hratio, compute_model, none);
  if (!push_down.empty()) {
    std::vector<int32_t> carried = inherited;
    carried.insert(carried.end(), node.blocks.begin(), node.blocks.end());
    for (int child : push_down) descend(out, child, mm, hratio, compute_model, carried);
  }
}

// prefix_attn/prefix_tree.py:484-505
void RadixPlanner::descend_naive(std::vector<Box>& out, int node_id, int mm) {
  const std::vector<int32_t> none;
  emit_boxes(out, nodes_[node_id].seq_ids, nodes_[node_id].num_seqs, mm, none, nodes_[node_id]);
  for (size_t i = 0; i < nodes_[node_id].child_ids.size(); ++i)
    descend_naive(out, nodes_[node_id].child_ids[i], mm);
}

// prefix_attn/prefix_tree.py:383-460
std::vector<Box> RadixPlanner::balance(std::vector<Box> boxes, int kv_heads,
                                       const pat_sched_opts& o) {
  if (boxes.empty()) return boxes;

  // Phase 1: cut boxes much longer than the average long box.
  int64_t long_blocks = 0, long_boxes = 0;
  for (const Box& b : boxes)
    if (b.kv > o.long_kv_tokens) { long_blocks += (int64_t)b.blocks.size(); long_boxes += 1; }
  std::vector<Box> cut;
  if (long_boxes != 0) {
    const double avg = (double)long_blocks / (double)long_boxes;
    const double limit = avg * (double)o.long_factor;
    for (Box& b : boxes) {
      const int nblk = (int)b.blocks.size();
      if ((double)nblk > limit) {
        const int pieces = (int)std::ceil((double)nblk / avg);
        const int piece_blocks = (int)ceil_div(nblk, pieces);
        for (int i = 0; i < pieces; ++i) {
          Box p;
          p.seqs = b.seqs;
          const int lo = std::min(i * piece_blocks, nblk);
          const int hi = std::min((i + 1) * piece_blocks, nblk);
          if (hi > lo) p.blocks.assign(b.blocks.begin() + lo, b.blocks.begin() + hi);
          p.num_seqs = b.num_seqs;
          p.kv = std::min(b.kv - i * piece_blocks * bs_, piece_blocks * bs_);
          if (i == 0) {
            p.rank = b.rank;
          } else {
            if (p.seqs.empty()) throw SchedError{PAT_ERR_INDEX, "list index out of range"};
            p.rank = split_per_seq_.at((size_t)p.seqs[0]);
            for (int32_t q : p.seqs) split_per_seq_.at((size_t)q) += 1;
          }
          cut.push_back(std::move(p));
        }
      } else {
        cut.push_back(std::move(b));
      }
    }
  } else {
    cut = std::move(boxes);
  }

  // Phase 2: halve the longest box until there are enough boxes for the device.
  int want;
  if (kv_heads <= 4) want = o.min_boxes[0];
  else if (kv_heads <= 8) want = o.min_boxes[1];
  else if (kv_heads <= 16) want = o.min_boxes[2];
  else if (kv_heads <= 32) want = o.min_boxes[3];
  else want = o.min_boxes[4];
  if ((int)cut.size() >= want) return cut;

  auto most_splits = [&]() {
    if (split_per_seq_.empty()) throw SchedError{PAT_ERR_VALUE, "max() arg is an empty sequence"};
    return *std::max_element(split_per_seq_.begin(), split_per_seq_.end());
  };
  while ((int)cut.size() < want && most_splits() < o.max_split) {
    size_t longest = 0;
    for (size_t i = 1; i < cut.size(); ++i)
      if (cut[i].blocks.size() > cut[longest].blocks.size()) longest = i;  // first maximum
    Box b = std::move(cut[longest]);
    cut.erase(cut.begin() + (std::ptrdiff_t)longest);
    const int nblk = (int)b.blocks.size();
    if (nblk <= o.stop_blocks) { cut.push_back(std::move(b)); break; }
    const int half = (int)ceil_div(nblk, 2);
    Box front, back;
    front.seqs = b.seqs;
    front.blocks.assign(b.blocks.begin(), b.blocks.begin() + half);
    front.num_seqs = b.num_seqs;
    front.kv = std::min(b.kv, half * bs_);
    front.rank = b.rank;
    back.seqs = b.seqs;
    back.blocks.assign(b.blocks.begin() + half, b.blocks.end());
    back.num_seqs = b.num_seqs;
    if (back.seqs.empty()) throw SchedError{PAT_ERR_INDEX, "list index out of range"};
    back.rank = split_per_seq_.at((size_t)back.seqs[0]);
    back.kv = std::min(b.kv - half * bs_, (nblk - half) * bs_);
    for (int32_t q : front.seqs) split_per_seq_.at((size_t)q) += 1;
    cut.push_back(std::move(front));
    cut.push_back(std::move(back));
  }
  return cut;
}

// Grouping into tile buckets and padding (prefix_attn/prefix_tree.py:574-614,
// prefix_attn/data_class.py:228-253).
void RadixPlanner::bucketize(const std::vector<Box>& boxes,
                             const std::vector<std::vector<int32_t>>& buckets, int hratio,
                             bool force_single) {
  std::map<std::vector<int32_t>, std::vector<size_t>> grouped;
  for (const auto& b : buckets) grouped[b];
  if (force_single) {
    auto& g = grouped[buckets[0]];
    for (size_t i = 0; i < boxes.size(); ++i) g.push_back(i);
  } else {
    for (size_t i = 0; i < boxes.size(); ++i) {
      int32_t label[3];
      tile_label((int)boxes[i].seqs.size() * hratio, boxes[i].kv, label);
      auto it = grouped.find(std::vector<int32_t>(label, label + 3));
      if (it == grouped.end())
        throw SchedError{PAT_ERR_KEY, "(" + std::to_string(label[0]) + ", " +
                                          std::to_string(label[1]) + ", " +
                                          std::to_string(label[2]) + ")"};
      it->second.push_back(i);
    }
  }

  Plan plan;
  std::vector<int32_t> boxes_seen(split_per_seq_.size(), 0);  // per sequence, boxes emitted so far
  for (const auto& mnw : buckets) {
    const auto& members = grouped[mnw];
    if (members.empty()) continue;
    Bucket bk;
    bk.mnw[0] = mnw[0]; bk.mnw[1] = mnw[1]; bk.mnw[2] = mnw[2];
    for (size_t i : members) {
      bk.max_seqs = std::max<int32_t>(bk.max_seqs, (int32_t)boxes[i].seqs.size());
      bk.max_blocks = std::max<int32_t>(bk.max_blocks, (int32_t)boxes[i].blocks.size());
    }
    bk.q_table.assign(members.size() * (size_t)bk.max_seqs, 0);
    bk.block_table.assign(members.size() * (size_t)bk.max_blocks, 0);
    bk.q_slot.assign(members.size() * (size_t)bk.max_seqs, 0);
    for (size_t r = 0; r < members.size(); ++r) {
      const Box& b = boxes[members[r]];
      std::copy(b.seqs.begin(), b.seqs.end(), bk.q_table.begin() + (std::ptrdiff_t)(r * bk.max_seqs));
      std::copy(b.blocks.begin(), b.blocks.end(),
                bk.block_table.begin() + (std::ptrdiff_t)(r * bk.max_blocks));
      for (size_t j = 0; j < b.seqs.size(); ++j)
        bk.q_slot[r * (size_t)bk.max_seqs + j] = boxes_seen.at((size_t)b.seqs[j])++;
      bk.q_len.push_back((int32_t)b.seqs.size());
      bk.block_len.push_back((int32_t)b.blocks.size());
      bk.num_seqs.push_back(b.num_seqs);
      bk.rank.push_back(b.rank);
      bk.kv.push_back(b.kv);
    }
    plan.buckets.push_back(std::move(bk));
  }
  plan.num_split_per_seq = split_per_seq_;
  if (plan.num_split_per_seq.empty())
    throw SchedError{PAT_ERR_VALUE, "max() arg is an empty sequence"};
  plan.max_split = *std::max_element(plan.num_split_per_seq.begin(), plan.num_split_per_seq.end());
  plan.max_boxes = *std::max_element(boxes_seen.begin(), boxes_seen.end());
  plan.num_boxes_per_seq = std::move(boxes_seen);
  for (const Box& b : boxes) {
    plan.max_seqs_in_box = std::max(plan.max_seqs_in_box, (int)b.seqs.size());
    plan.max_blocks_in_box = std::max(plan.max_blocks_in_box, (int)b.blocks.size());
  }
  for (const Bucket& bk : plan.buckets) {
    pat_bucket_view v;
    v.mnw[0] = bk.mnw[0]; v.mnw[1] = bk.mnw[1]; v.mnw[2] = bk.mnw[2];
    v.num_boxes = (int32_t)bk.num_seqs.size();
    v.max_seqs = bk.max_seqs;
    v.max_blocks = bk.max_blocks;
    v.q_table = bk.q_table.data();
    v.block_table = bk.block_table.data();
    v.q_len = bk.q_len.data();
    v.block_len = bk.block_len.data();
    v.num_seqs = bk.num_seqs.data();
    v.rank = bk.rank.data();
    v.kv = bk.kv.data();
    v.q_slot = bk.q_slot.data();
    plan.views.push_back(v);
  }
  plan.valid = true;
  plan_ = std::move(plan);
  // plan_ owns new vectors after the move: refresh the borrowed pointers
  for (size_t i = 0; i < plan_.buckets.size(); ++i) {
    const Bucket& bk = plan_.buckets[i];
    pat_bucket_view& v = plan_.views[i];
    v.q_table = bk.q_table.data();
    v.block_table = bk.block_table.data();
    v.q_len = bk.q_len.data();
    v.block_len = bk.block_len.data();
    v.num_seqs = bk.num_seqs.data();
    v.rank = bk.rank.data();
    v.kv = bk.kv.data();
    v.q_slot = bk.q_slot.data();
  }
}

// prefix_attn/prefix_tree.py:548-616
void RadixPlanner::pack(const int32_t* mnws, int n_mnws, int hratio, int kv_heads,
                        bool compute_model, const pat_sched_opts* opts) {
  std::vector<std::vector<int32_t>> buckets;
  if (mnws == nullptr || n_mnws <= 0) {
    for (const auto& b : kDefaultBuckets) buckets.emplace_back(b, b + 3);
  } else {
    for (int i = 0; i < n_mnws; ++i) buckets.emplace_back(mnws + 3 * i, mnws + 3 * i + 3);
  }
  if (hratio == 0) throw SchedError{PAT_ERR_VALUE, "integer division or modulo by zero"};
  if (hratio < 0) throw SchedError{PAT_ERR_INVALID, "HRatio must be positive"};
  int max_m = buckets[0][0];
  for (const auto& b : buckets) max_m = std::max(max_m, b[0]);
  const int mm = max_m / hratio;

  std::vector<Box> boxes;
  const std::vector<int32_t> none;
  const std::vector<int32_t> top = nodes_[0].child_ids;  // copy: nodes_ is not modified below
  for (int child : top) descend(boxes, child, mm, hratio, compute_model, none);
  boxes = balance(std::move(boxes), kv_heads, opts ? *opts : kReferenceOpts);
  bucketize(boxes, buckets, hratio, buckets.size() == 1);
}

// prefix_attn/prefix_tree.py:507-545
void RadixPlanner::naive(int hratio) {
  std::vector<std::vector<int32_t>> buckets;
  for (const auto& b : kDefaultBuckets) buckets.emplace_back(b, b + 3);
  if (hratio == 0) throw SchedError{PAT_ERR_VALUE, "integer division or modulo by zero"};
  if (hratio < 0) throw SchedError{PAT_ERR_INVALID, "HRatio must be positive"};
  const int mm = 64 / hratio;
  std::vector<Box> boxes;
  const std::vector<int32_t> top = nodes_[0].child_ids;
  for (int child : top) descend_naive(boxes, child, mm);
  bucketize(boxes, buckets, hratio, false);
}

}  // namespace pat
