// The compiled PyTorch-ROCm extension `_prefix_attn`: the Python surface of the reference's
// extension module (csrc/bindings.cpp:74-158 of the flashserve/PAT tree) over the C ABI of
// libpat_amd (include/pat_amd.h). Host code only: no kernel lives here. torch supplies device
// pointers, strides, the current HIP stream and scratch memory from its caching allocator.
//
//   prefix_attn_with_kvcache   table overload (bindings.cpp:7-43, :76-95) and tree overload
//                              (:45-72, :148-157)
//   PrefixTreeCPP              build_radix_tree / pack_schedule with the GIL released
//                              (:100-146), kernel_info
//   KernelInfo                 plan tensors + to_gpu (:97-98; csrc/prefix_tree.h:7-39)
//   paged_decode_baseline      the prefix-oblivious comparator (not in the reference's API)
#include <torch/extension.h>

#include <c10/core/DeviceGuard.h>
#include <c10/core/InferenceMode.h>
#include <c10/hip/HIPStream.h>
#include <hip/hip_runtime_api.h>

#include <cstring>
#include <memory>
#include <atomic>
#include <mutex>
#include <optional>
#include <string>
#include <unordered_map>
#include <vector>

#include "pat_amd.h"

namespace py = pybind11;

namespace {

using TensorList = std::vector<at::Tensor>;

// ---- errors ---------------------------------------------------------------------------------
// PAT_ERR_* -> the exception the reference API raises in the same situation. Call with the GIL held.
void check(int code) {
  if (code == PAT_OK) return;
  const std::string msg = pat_last_error();
  switch (code) {
    case PAT_ERR_VALUE:
      if (msg.find("by zero") != std::string::npos) {
        PyErr_SetString(PyExc_ZeroDivisionError, msg.c_str());
        throw py::error_already_set();
      }
      throw py::value_error(msg);
    case PAT_ERR_INDEX: throw py::index_error(msg);
    case PAT_ERR_KEY: throw py::key_error(msg);
    default: throw std::runtime_error(msg);
  }
}

void require(bool cond, const char* msg) {
  if (!cond) throw std::runtime_error(msg);
}
void require(bool cond, const std::string& msg) {
  if (!cond) throw std::runtime_error(msg);
}

void* raw_stream(const c10::Device& dev) {
  return static_cast<void*>(c10::hip::getCurrentHIPStream(dev.index()).stream());
}

c10::Device to_device(const py::object& obj) {
  if (py::isinstance<py::str>(obj)) return c10::Device(obj.cast<std::string>());
  return obj.cast<c10::Device>();
}

struct RecordSet;

// ---- a prepared launch ------------------------------------------------------------------------
// pat_fwd_args plus everything it points into. Built once per set of tensors (a decode step calls
// the forward once per layer with the same plan), launched many times.
struct Prepared {
  pat_fwd_args args;
  std::vector<pat_fwd_bucket> buckets;
  TensorList keep;          // plan tensors (and derived slots) stay alive as long as the launch does
  std::shared_ptr<RecordSet> records;   // the plan's launch records (shared by every launch of the plan)
  int64_t plan_version = -1;   // version of the plan tables the records were built from
  size_t need = 0;          // workspace bytes with prebuilt records
  size_t need_inline = 0;   // workspace bytes when the launch builds its records itself (args.records NULL)
  bool derive_slots = false;   // the plan came without slot tables: ordinals derived on the device
  pat_fwd_tuning tuning;    // the measured geometry of this plan shape (args.tuning points here when set)
  Prepared() { std::memset(&args, 0, sizeof(args)); std::memset(&tuning, 0, sizeof(tuning)); }
};

// ---- measured launch geometry, remembered per plan shape ---------------------------------------
// pat_fwd_autotune times a launch under a few candidate geometries. One measurement serves every
// launch of the same shape: the layers of a model call the forward with the same plan and
// different caches, and consecutive decode steps differ by a token per request. The shape key
// holds the head geometry and, per bucket, the tile label and the box count and block-table width
// rounded up to multiples of 8.
std::mutex g_tune_mutex;
std::unordered_map<std::string, pat_fwd_tuning> g_tuned;
std::atomic<int64_t> g_tuning_runs{0};   // measurements made since the module was loaded
// Opt-in (PAT_AUTOTUNE=1 or set_autotune(True)): the measurement synchronises the stream and runs
// the launch some fifty times, which a serving loop must not meet unasked; the automatic geometry
// (sizes only) is the default.
bool g_autotune = [] {
  const char* e = std::getenv("PAT_AUTOTUNE");
  return e != nullptr && std::atoi(e) != 0;
}();

std::string shape_key(const pat_fwd_args& a) {
  std::string k;
  auto add = [&](int64_t v) { k.append(reinterpret_cast<const char*>(&v), sizeof(v)); };
  auto up8 = [](int64_t v) { return (v + 7) / 8 * 8; };
  add(a.dtype); add(a.head_dim); add(a.heads); add(a.kv_heads); add(a.page_size); add(up8(a.batch));
  add(a.max_split_per_seq); add(a.num_buckets);   // (not whether an LSE is asked for: one call's geometry serves both)
  for (int i = 0; i < a.num_buckets; ++i) {
    const pat_fwd_bucket& b = a.buckets[i];
    add(b.mnw[0]); add(up8(b.num_boxes)); add(b.max_seqs); add(up8(b.max_blocks)); add(b.flags); add(b.q_slot != nullptr);
  }
  return k;
}

// Sets L.args.tuning from the remembered measurement of this shape, measuring first when there is
// none (not while the stream is being captured into a graph: the measurement synchronises).
void tune(Prepared& L, const c10::Device& dev) {
  if (!g_autotune) return;
  const std::string key = shape_key(L.args);
  {
    std::lock_guard<std::mutex> lock(g_tune_mutex);
    auto it = g_tuned.find(key);
    if (it != g_tuned.end()) { L.tuning = it->second; L.args.tuning = &L.tuning; return; }
  }
  void* stream = static_cast<void*>(c10::hip::getCurrentHIPStream(dev.index()).stream());
  hipStreamCaptureStatus capture = hipStreamCaptureStatusNone;
  if (hipStreamIsCapturing(static_cast<hipStream_t>(stream), &capture) != hipSuccess || capture != hipStreamCaptureStatusNone)
    return;
  size_t most = 0;
  check(pat_fwd_autotune_workspace_bytes(&L.args, &most));
  at::Tensor ws = at::empty({(int64_t)std::max<size_t>(most, 256)}, at::TensorOptions().dtype(at::kByte).device(dev));
  L.args.workspace = ws.data_ptr(); L.args.workspace_bytes = (size_t)ws.numel();
  // 320 MB per device, read between the timed launches (more than the 256 MB memory-side cache holds):
  // allocated at the first measurement and kept
  // (held for the life of the process and never destroyed: a static destructor would release device
  // memory after the HIP runtime has shut down)
  static std::mutex evict_mutex;
  static auto& evict_buffers = *new std::unordered_map<int, at::Tensor>();
  at::Tensor evict;
  {
    std::lock_guard<std::mutex> lock(evict_mutex);
    auto it = evict_buffers.find(dev.index());
    if (it == evict_buffers.end())
      it = evict_buffers.emplace(dev.index(), at::zeros({(int64_t)320 << 20}, at::TensorOptions().dtype(at::kByte).device(dev))).first;
    evict = it->second;
  }
  pat_fwd_tuning best;
  g_tuning_runs.fetch_add(1);
  const int rc = pat_fwd_autotune(&L.args, stream, 8, evict.data_ptr(), (size_t)evict.numel(), &best, nullptr, nullptr);
  L.args.workspace = nullptr; L.args.workspace_bytes = 0;
  check(rc);
  L.tuning = best; L.args.tuning = &L.tuning;
  std::lock_guard<std::mutex> lock(g_tune_mutex);
  if (g_tuned.size() >= 4096) g_tuned.clear();
  g_tuned[key] = best;
}

// ---- launch records, shared by the launches of one plan -----------------------------------------
// The records depend on the plan tables and the launch geometry, not on q / k / v / out: the layers
// of a model (one prepared launch each) share one set. They are a SNAPSHOT of the tables, taken when
// a launch first needs them and again when torch's version counter of a plan tensor has moved
// (in-place edits through torch: DecodePlan.advance_step). Edits torch does not count are not seen:
//   * while the stream is being captured into a graph no snapshot is used: the launch builds its
//     records itself (args.records NULL), so the record kernel is part of the graph and every replay
//     reads the tables as they are then;
//   * a plan held in inference tensors (no version counter) is served the same way at every call;
//   * anything else (raw-pointer writes by another library): KernelInfo.invalidate() /
//     invalidate_plans() drop the snapshots.
// One set of records: the tensor, and an event recorded behind the kernel that wrote it. A launch
// on another stream than the one that built the records waits for that event (torch orders work
// per stream only, and this tensor is not the caller's to synchronise).
constexpr int64_t kUntracked = -2;   // plan version of tensors without a version counter

struct RecordSet {
  at::Tensor tensor;
  hipEvent_t ready = nullptr;
  void* stream = nullptr;       // the stream that built them
  bool seen_ready = false;
  RecordSet() = default;
  RecordSet(const RecordSet&) = delete;
  RecordSet& operator=(const RecordSet&) = delete;
  ~RecordSet() { if (ready != nullptr) (void)hipEventDestroy(ready); }
};

bool capturing(void* stream) {
  hipStreamCaptureStatus status = hipStreamCaptureStatusNone;
  return hipStreamIsCapturing(static_cast<hipStream_t>(stream), &status) != hipSuccess || status != hipStreamCaptureStatusNone;
}

struct RecordStore {
  int64_t version = -1;
  std::unordered_map<uint64_t, std::shared_ptr<RecordSet>> by_tag;
  // plans that came without slot tables: the ordinals derived on the device (pat_fwd_derive_slots)
  at::Tensor derived_slots;
  std::vector<int64_t> derived_offsets;
  int64_t derived_version = -1;   // plan version whose ordinals the buffer holds (-1: none that may be relied on)
  // a store looked up by the plan tensors' addresses holds those tensors: as long as it exists no
  // other plan can be allocated at the same addresses and find records that are not its own
  TensorList keep;
};

// Snapshot of the plan at `version` for this launch; never called while the stream is being captured.
void attach_records(Prepared& L, RecordStore& store, int64_t version, const c10::Device& dev) {
  if (store.version != version) { store.by_tag.clear(); store.version = version; }
  pat_fwd_args& a = L.args;
  a.records = nullptr;
  uint64_t tag = 0;
  check(pat_fwd_records_tag(&a, &tag));
  auto it = store.by_tag.find(tag);
  if (it == store.by_tag.end()) {
    size_t rbytes = 0;
    check(pat_fwd_records_bytes(&a, &rbytes));
    auto set = std::make_shared<RecordSet>();
    set->tensor = at::empty({(int64_t)rbytes}, at::TensorOptions().dtype(at::kByte).device(dev));
    set->stream = raw_stream(dev);
    uint64_t built = 0;
    // (the derived slots of a plan without slot tables were written on this stream just before: the
    // event covers them too)
    check(pat_fwd_build_records(&a, set->tensor.data_ptr(), rbytes, &built, set->stream));
    require(hipEventCreateWithFlags(&set->ready, hipEventDisableTiming) == hipSuccess, "hipEventCreateWithFlags failed");
    require(hipEventRecord(set->ready, static_cast<hipStream_t>(set->stream)) == hipSuccess, "hipEventRecord failed");
    if (store.by_tag.size() >= 16) store.by_tag.clear();
    it = store.by_tag.emplace(built, set).first;
    tag = built;
  }
  L.records = it->second;
  L.plan_version = version;
  a.records = L.records->tensor.data_ptr(); a.records_bytes = (size_t)L.records->tensor.numel(); a.records_tag = tag;
  check(pat_fwd_workspace_bytes(&a, &L.need));
}

void strides3(const at::Tensor& t, int64_t out[3]) {
  out[0] = t.stride(0); out[1] = t.stride(1); out[2] = t.stride(2);
}

struct PlanTables {
  const TensorList* q_tables;
  const TensorList* block_tables;
  const TensorList* num_seqs;
  const TensorList* ranks;
  const TensorList* kvs;
  const TensorList* slots;                       // may be null
  const std::vector<std::vector<int>>* mnw;
  const std::vector<int>* flags;                 // may be null
};

// Checks that need tensor metadata follow csrc/api.h:131-181, :256-277 of the reference.
std::shared_ptr<Prepared> prepare(const at::Tensor& q, const at::Tensor& k, const at::Tensor& v,
                                  const at::Tensor& num_split, const PlanTables& pt, int max_split, int max_seqs,
                                  int max_blocks, double scale, const at::Tensor& out,
                                  const std::optional<at::Tensor>& lse, RecordStore& store, int64_t plan_version) {
  require(q.scalar_type() == at::kHalf || q.scalar_type() == at::kBFloat16, "only support fp16 and bf16 data type");
  require(k.scalar_type() == q.scalar_type(), "query and key must have the same dtype");
  require(v.scalar_type() == q.scalar_type(), "query and value must have the same dtype");
  require(q.is_cuda(), "q must be on CUDA");
  require(k.is_cuda(), "kcache must be on CUDA");
  require(v.is_cuda(), "vcache must be on CUDA");
  for (const at::Tensor* t : {&q, &k, &v})
    require(t->dim() == 4 && t->stride(-1) == 1, "Input tensor must have contiguous last dimension");
  const int64_t b = q.size(0), sq = q.size(1), h = q.size(2), d = q.size(3);
  const int64_t nblk = k.size(0), page = k.size(1), hk = k.size(2);
  require(k.size(3) == d, "kcache must have shape (num_blocks, page_block_size, n_heads_kv, head_size_og)");
  require(v.sizes() == k.sizes(), "vcache must have shape (num_blocks, page_block_size, n_heads_kv, head_size_og)");
  require(out.is_cuda() && out.scalar_type() == q.scalar_type() && out.sizes() == q.sizes() && out.stride(-1) == 1,
          "out must be a CUDA tensor with q's shape and dtype and a contiguous last dimension");
  require(num_split.is_cuda(), "num_split_per_seq must be on CUDA");
  require(num_split.scalar_type() == at::kInt, "num_split_per_seq must have dtype torch.int32");
  require(num_split.dim() == 1 && num_split.size(0) == b, "num_split_per_seq must have shape (batch_size)");
  require(num_split.stride(-1) == 1, "num_split_per_seq must have contiguous last dimension");
  const size_t nb = pt.mnw->size();
  require(pt.q_tables->size() == nb && pt.block_tables->size() == nb && pt.num_seqs->size() == nb &&
              pt.ranks->size() == nb && pt.kvs->size() == nb,
          "MNW and the per-bucket plan lists must have the same length");
  const TensorList* slots = (pt.slots != nullptr && !pt.slots->empty()) ? pt.slots : nullptr;
  require(slots == nullptr || slots->size() == nb, "slot_tables must have one entry per bucket");
  require(pt.flags == nullptr || pt.flags->empty() || pt.flags->size() == nb, "bucket_flags must have one entry per bucket");

  auto L = std::make_shared<Prepared>();
  L->buckets.resize(std::max<size_t>(nb, 1));
  std::memset(L->buckets.data(), 0, L->buckets.size() * sizeof(pat_fwd_bucket));
  for (size_t i = 0; i < nb; ++i) {
    const at::Tensor &qt = (*pt.q_tables)[i], &bt = (*pt.block_tables)[i], &ns = (*pt.num_seqs)[i],
                     &rk = (*pt.ranks)[i], &kv = (*pt.kvs)[i];
    const std::pair<const char*, const at::Tensor*> named[] = {
        {"query_tables", &qt}, {"block_tables", &bt}, {"num_seqs_per_CTA", &ns}, {"CTA_rank", &rk}, {"kv_in_CTA", &kv}};
    for (const auto& nt : named) {
      require(nt.second->is_cuda(), std::string(nt.first) + " must be on CUDA");
      require(nt.second->scalar_type() == at::kInt, std::string(nt.first) + " must have dtype torch.int32");
      require(nt.second->numel() == 0 || nt.second->stride(-1) == 1,
              std::string(nt.first) + " must have contiguous last dimension");
    }
    require(qt.dim() == 2 && bt.dim() == 2 && bt.size(0) == qt.size(0), "query_tables / block_tables must be (CTAs, width)");
    const int64_t ctas = qt.size(0);
    for (int j = 2; j < 5; ++j)
      require(named[j].second->dim() == 1 && named[j].second->size(0) == ctas,
              std::string(named[j].first) + " must have shape (CTAs)");
    pat_fwd_bucket& fb = L->buckets[i];
    fb.q_table = qt.data_ptr<int32_t>(); fb.block_table = bt.data_ptr<int32_t>();
    fb.num_seqs = ns.data_ptr<int32_t>(); fb.rank = rk.data_ptr<int32_t>(); fb.kv = kv.data_ptr<int32_t>();
    if (slots != nullptr) {
      const at::Tensor& st = (*slots)[i];
      require(st.is_cuda() && st.scalar_type() == at::kInt && st.sizes() == qt.sizes() && st.strides() == qt.strides(),
              "slot_tables must match query_tables (CUDA int32, same layout)");
      fb.q_slot = st.data_ptr<int32_t>();
      L->keep.push_back(st);
    }
    fb.q_table_stride = ctas > 1 ? qt.stride(0) : std::max<int64_t>(qt.size(1), 1);
    fb.block_table_stride = ctas > 1 ? bt.stride(0) : std::max<int64_t>(bt.size(1), 1);
    fb.num_boxes = (int32_t)ctas; fb.max_seqs = (int32_t)qt.size(1); fb.max_blocks = (int32_t)bt.size(1);
    require((*pt.mnw)[i].size() == 3, "MNW entries must be [M, N, W]");
    for (int j = 0; j < 3; ++j) fb.mnw[j] = (*pt.mnw)[i][(size_t)j];
    fb.flags = (pt.flags != nullptr && !pt.flags->empty()) ? (*pt.flags)[i] : 0;
    for (const auto& nt : named) L->keep.push_back(*nt.second);
  }
  L->keep.push_back(num_split);

  pat_fwd_args& a = L->args;
  a.dtype = q.scalar_type() == at::kBFloat16 ? PAT_DTYPE_BF16 : PAT_DTYPE_F16;
  a.batch = (int32_t)b; a.seqlen_q = (int32_t)sq; a.heads = (int32_t)h; a.kv_heads = (int32_t)hk;
  a.head_dim = (int32_t)d; a.page_size = (int32_t)page; a.num_pages = (int32_t)nblk;
  a.q = q.data_ptr(); a.k = k.data_ptr(); a.v = v.data_ptr(); a.out = out.data_ptr();
  strides3(q, a.q_stride); strides3(k, a.k_stride); strides3(v, a.v_stride); strides3(out, a.o_stride);
  a.num_split_per_seq = num_split.data_ptr<int32_t>();
  a.max_split_per_seq = max_split; a.max_seqs_in_box = max_seqs; a.max_blocks_in_box = max_blocks;
  a.softmax_scale = (float)scale;
  a.num_buckets = (int32_t)nb;
  a.buckets = L->buckets.data();
  if (lse.has_value()) {
    require(lse->is_cuda() && lse->scalar_type() == at::kFloat && lse->is_contiguous() && lse->numel() == b * h,
            "softmax_lse must be a contiguous CUDA float32 tensor with batch_size * n_heads elements");
    a.lse_out = lse->data_ptr<float>();
  }
  if (slots == nullptr && max_split > 1) {
    // A plan without slot tables (the reference's call form): CTA_rank is not unique per sequence on
    // irregular forests, so the ordinals are derived from the q_tables on the device: once per plan
    // version here or in run(), at every call where no snapshot may be used.
    L->derive_slots = true;
    if (!store.derived_slots.defined()) {
      size_t sbytes = 0;
      check(pat_fwd_slots_bytes(&a, &sbytes));
      store.derived_slots = at::empty({(int64_t)sbytes}, at::TensorOptions().dtype(at::kByte).device(q.device()));
      store.derived_offsets.assign(std::max<size_t>(nb, 1), 0);
      store.derived_version = -1;
    }
    void* stream = raw_stream(q.device());
    const bool snapshot = plan_version != kUntracked && !capturing(stream);
    if (!snapshot || store.derived_version != plan_version) {
      // (also what fills derived_offsets, which is host arithmetic)
      check(pat_fwd_derive_slots(&a, store.derived_slots.data_ptr(), (size_t)store.derived_slots.numel(),
                                 store.derived_offsets.data(), stream));
      store.derived_version = snapshot ? plan_version : -1;
    }
    int32_t* base = static_cast<int32_t*>(store.derived_slots.data_ptr());
    for (size_t i = 0; i < nb; ++i) L->buckets[i].q_slot = base + store.derived_offsets[i];
    a.num_split_per_seq = base;
    L->keep.push_back(store.derived_slots);
  }
  tune(*L, q.device());
  a.records = nullptr; a.records_bytes = 0;
  check(pat_fwd_workspace_bytes(&a, &L->need_inline));
  return L;
}

void run(Prepared& L, RecordStore& store, int64_t version, const c10::Device& dev) {
  void* stream = raw_stream(dev);
  const bool snapshot = version != kUntracked && !capturing(stream);
  pat_fwd_args& a = L.args;
  if (L.derive_slots && (!snapshot || store.derived_version != version)) {
    std::vector<int64_t> offsets(store.derived_offsets.size(), 0);
    a.records = nullptr;
    check(pat_fwd_derive_slots(&a, store.derived_slots.data_ptr(), (size_t)store.derived_slots.numel(), offsets.data(), stream));
    store.derived_version = snapshot ? version : -1;
  }
  size_t need;
  if (snapshot) {
    if (!L.records || L.plan_version != version) attach_records(L, store, version, dev);
    a.records = L.records->tensor.data_ptr(); a.records_bytes = (size_t)L.records->tensor.numel();
    need = L.need;
    if (!L.records->seen_ready && stream != L.records->stream) {
      // another stream than the one that wrote the records: ordered behind that kernel
      if (hipEventQuery(L.records->ready) == hipSuccess) L.records->seen_ready = true;
      else require(hipStreamWaitEvent(static_cast<hipStream_t>(stream), L.records->ready, 0) == hipSuccess, "hipStreamWaitEvent failed");
    }
  } else {
    // no snapshot: the launch builds its records from the tables as they are when it runs
    a.records = nullptr; a.records_bytes = 0;
    need = L.need_inline;
  }
  at::Tensor ws;   // scratch for the partial results (and inline records); stream-ordered reuse
  if (need > 0) {
    ws = at::empty({(int64_t)need}, at::TensorOptions().dtype(at::kByte).device(dev));
    a.workspace = ws.data_ptr();
  } else {
    a.workspace = nullptr;
  }
  a.workspace_bytes = need;
  check(pat_fwd_launch(&a, stream));
}

// ---- cache keys -----------------------------------------------------------------------------------
struct Key {
  std::string bytes;
  template <typename T> void add(const T& v) { bytes.append(reinterpret_cast<const char*>(&v), sizeof(T)); }
  void tensor(const at::Tensor& t) {   // address + layout
    add(t.data_ptr()); add((int)t.scalar_type()); add((int64_t)t.dim());
    for (int64_t s : t.sizes()) add(s);
    for (int64_t s : t.strides()) add(s);
  }
  void plan_tensor(const at::Tensor& t) {   // ... and the version counter: in-place edits of a plan count
    tensor(t); add(t.is_inference() ? kUntracked : (int64_t)t._version());
  }
};

// ---- KernelInfo -----------------------------------------------------------------------------------
struct LaunchPart { int bucket, lo, hi; };

struct KernelInfo {
  TensorList q_tables, block_tables, num_seqs, ranks, kvs, slot_tables;
  std::vector<std::vector<int>> mnws;
  at::Tensor num_split_per_seq = at::empty({0}, at::kInt);
  at::Tensor num_boxes_per_seq = at::empty({0}, at::kInt);
  int max_split = 0, max_boxes = 0, max_seqs = 0, max_blocks = 0;
  // launch copies: every bucket's boxes longest first, a bucket with a wide head split in two
  bool has_launch = false;
  TensorList l_q_tables, l_block_tables, l_num_seqs, l_ranks, l_kvs, l_slot_tables;
  std::vector<std::vector<int>> l_mnws;
  std::vector<int> l_flags;
  TensorList launch_order;                          // per bucket: launch position -> scheduler row
  std::vector<std::vector<LaunchPart>> launch_parts;  // per bucket: its launch buckets
  // the whole plan in one int32 buffer (pinned on the host when a GPU is there)
  std::optional<at::Tensor> flat;
  pat_flat_plan layout;
  // Small batches of short requests (see whole_sequences_pay): what the tree form launches there is one
  // work item per request over its own block row - a single kernel that writes `out`, where the
  // prefix-aware plan needs a second one to merge two or three partial results per request. Its
  // tables sit behind the plan in the same buffer: [batch] request ids, ones, zeros, lengths, then
  // the block rows [batch, ws_width].
  bool whole_seqs = false;
  int64_t ws_offset = 0;
  int ws_batch = 0, ws_width = 0, ws_tile = 16, ws_longest_allowed = 0;
  TensorList ws_q_table, ws_block_table, ws_num_seqs, ws_rank, ws_kv;
  std::vector<std::vector<int>> ws_mnw;
  at::Tensor ws_num_split;
  std::unordered_map<std::string, std::shared_ptr<Prepared>> cache;
  RecordStore records;

  // Counts in-place edits of the plan tables: every table is a view of one buffer, whose version
  // counter torch advances with each of them (a plan held table by table: the counters' sum).
  // kUntracked when a table is an inference tensor (no counter). invalidate() moves it by hand.
  int64_t generation = 0;
  int64_t plan_version() const {
    const int64_t gen = generation << 32;
    if (flat.has_value()) return flat->is_inference() ? kUntracked : gen + (int64_t)flat->_version();
    if (num_split_per_seq.is_inference() || num_boxes_per_seq.is_inference()) return kUntracked;
    int64_t v = gen + (int64_t)num_split_per_seq._version() + (int64_t)num_boxes_per_seq._version();
    for (const TensorList* l : {&q_tables, &block_tables, &num_seqs, &ranks, &kvs, &slot_tables})
      for (const at::Tensor& t : *l) {
        if (t.is_inference()) return kUntracked;
        v += (int64_t)t._version();
      }
    return v;
  }
  void invalidate() { ++generation; }

  void clear_tables() {
    for (TensorList* l : {&q_tables, &block_tables, &num_seqs, &ranks, &kvs, &slot_tables, &l_q_tables,
                          &l_block_tables, &l_num_seqs, &l_ranks, &l_kvs, &l_slot_tables, &launch_order,
                          &ws_q_table, &ws_block_table, &ws_num_seqs, &ws_rank, &ws_kv})
      l->clear();
    ws_mnw.clear();
    mnws.clear(); l_mnws.clear(); l_flags.clear(); launch_parts.clear();
    cache.clear();
    records = RecordStore();
  }

  // (Re)creates every plan tensor as a view of `buf` (the host buffer or its copy on a device).
  void bind(const at::Tensor& buf) {
    clear_tables();
    const pat_flat_plan& lay = layout;
    auto vec = [&](int64_t off, int64_t n) { return buf.narrow(0, off, n); };
    auto mat = [&](int64_t off, int64_t n, int64_t w) { return buf.narrow(0, off, n * w).view({n, w}); };
    num_split_per_seq = vec(lay.num_split_per_seq, lay.batch);
    num_boxes_per_seq = vec(lay.num_boxes_per_seq, lay.batch);
    for (int b = 0; b < lay.num_buckets; ++b) {
      const pat_flat_bucket& f = lay.buckets[b];
      mnws.push_back({f.mnw[0], f.mnw[1], f.mnw[2]});
      q_tables.push_back(mat(f.q_table, f.num_boxes, f.max_seqs));
      slot_tables.push_back(mat(f.q_slot, f.num_boxes, f.max_seqs));
      block_tables.push_back(mat(f.block_table, f.num_boxes, f.max_blocks));
      num_seqs.push_back(vec(f.num_seqs, f.num_boxes));
      ranks.push_back(vec(f.rank, f.num_boxes));
      kvs.push_back(vec(f.kv, f.num_boxes));
      launch_order.push_back(vec(lay.launch_order[b], f.num_boxes));
      launch_parts.emplace_back();
    }
    for (int i = 0; i < lay.num_launch_buckets; ++i) {
      const pat_flat_bucket& f = lay.launch[i];
      l_mnws.push_back({f.mnw[0], f.mnw[1], f.mnw[2]});
      l_flags.push_back(f.flags);
      l_q_tables.push_back(mat(f.q_table, f.num_boxes, f.max_seqs));
      l_slot_tables.push_back(mat(f.q_slot, f.num_boxes, f.max_seqs));
      l_block_tables.push_back(mat(f.block_table, f.num_boxes, f.max_blocks));
      l_num_seqs.push_back(vec(f.num_seqs, f.num_boxes));
      l_ranks.push_back(vec(f.rank, f.num_boxes));
      l_kvs.push_back(vec(f.kv, f.num_boxes));
      launch_parts[(size_t)f.parent].push_back({i, f.first, f.first + f.num_boxes});
    }
    has_launch = true;
    if (whole_seqs) {
      const int64_t b = ws_batch;
      ws_q_table.push_back(mat(ws_offset, b, 1));
      ws_num_seqs.push_back(vec(ws_offset + b, b));
      ws_num_split = vec(ws_offset + b, b);          // (ones as well: every request is one work item)
      ws_rank.push_back(vec(ws_offset + 2 * b, b));
      ws_kv.push_back(vec(ws_offset + 3 * b, b));
      ws_block_table.push_back(mat(ws_offset + 4 * b, b, ws_width));
      ws_mnw.push_back({ws_tile, 128, 1});
    }
  }

  // Copies every plan tensor to `device`: one copy of the one buffer, asynchronous from pinned memory
  // (the reference moves each table by itself, csrc/prefix_tree.h:27-38).
  void to_gpu(const c10::Device& device) {
    // (plan tensors are ordinary tensors also when the caller is in inference mode: their version
    // counters are what tells a launch that DecodePlan.advance_step edited them)
    c10::InferenceMode plain(false);
    if (flat.has_value()) {
      flat = flat->to(device, /*non_blocking=*/true);
      bind(*flat);
      return;
    }
    auto move = [&](TensorList& l) { for (auto& t : l) t = t.to(device, true); };
    for (TensorList* l : {&q_tables, &block_tables, &num_seqs, &ranks, &kvs, &slot_tables}) move(*l);
    num_split_per_seq = num_split_per_seq.to(device, true);
    num_boxes_per_seq = num_boxes_per_seq.to(device, true);
    cache.clear();
    records = RecordStore();
  }

  py::dict launch_tables() const {
    py::dict d;
    const bool l = has_launch;
    d["q_tables"] = l ? l_q_tables : q_tables;
    d["slot_tables"] = l ? l_slot_tables : slot_tables;
    d["block_tables"] = l ? l_block_tables : block_tables;
    d["num_seqs_per_CTAs"] = l ? l_num_seqs : num_seqs;
    d["CTA_ranks"] = l ? l_ranks : ranks;
    d["kv_in_CTAs"] = l ? l_kvs : kvs;
    d["MNWs"] = l ? l_mnws : mnws;
    d["flags"] = l ? l_flags : std::vector<int>(mnws.size(), 0);
    return d;
  }

  // The tables of the one-work-item-per-request launch, or None when the plan is launched as planned.
  py::object whole_sequence_tables() const {
    if (!whole_seqs) return py::none();
    py::dict d;
    d["q_tables"] = ws_q_table; d["block_tables"] = ws_block_table; d["num_seqs_per_CTAs"] = ws_num_seqs;
    d["CTA_ranks"] = ws_rank; d["kv_in_CTAs"] = ws_kv; d["MNWs"] = ws_mnw;
    d["num_split_per_seq"] = ws_num_split; d["max_split_per_seq"] = 1; d["max_seqs_in_CTA"] = 1;
    d["max_blocks_in_CTA"] = ws_width;
    d["longest_allowed"] = ws_longest_allowed;   // a request that outgrows this takes the batch back to the tree's plan
    return d;
  }

  // For the boxes of scheduler bucket b, in scheduler order: (launch bucket, row in it).
  std::pair<at::Tensor, at::Tensor> launch_position(int b) const {
    require(b >= 0 && (size_t)b < launch_order.size(), "bucket index out of range");
    const at::Tensor order = launch_order[(size_t)b].to(at::kCPU).to(at::kLong).contiguous();
    const int64_t n = order.numel();
    at::Tensor bucket = at::empty({n}, at::kLong), row = at::empty({n}, at::kLong);
    const int64_t* o = order.data_ptr<int64_t>();
    int64_t* pb = bucket.data_ptr<int64_t>();
    int64_t* pr = row.data_ptr<int64_t>();
    for (const LaunchPart& p : launch_parts[(size_t)b])
      for (int64_t pos = p.lo; pos < p.hi; ++pos) { pb[o[pos]] = p.bucket; pr[o[pos]] = pos - p.lo; }
    return {bucket, row};
  }
};

at::Tensor host_i32(int64_t n, const int32_t* src) {
  at::Tensor t = at::empty({n}, at::kInt);
  if (n > 0) std::memcpy(t.data_ptr<int32_t>(), src, (size_t)n * sizeof(int32_t));
  return t;
}

// ---- PrefixTreeCPP ----------------------------------------------------------------------------------
struct TreeHandle {
  pat_tree* h = nullptr;
  ~TreeHandle() { if (h) pat_tree_destroy(h); }
};

// Is a batch better served by one work item per request than by its prefix-aware plan? Yes when the
// whole launch is a few microseconds of latency anyway: every request short enough for one workgroup
// to walk in a few steps per wave, everything resident at once, and so little KV in total that
// re-reading shared pages (from L2) costs less than the merge kernel's launch and round trips.
// Measured (us per call, plan / one item per request): 8 requests of 288 tokens 6.7 / 5.9; 32 x 192:
// 10.4 / 6.5; 64 x 192: 10.4 / 8.3; 32 x 384: 13.7 / 9.3; 16 x 512: 13.6 / 10.0; 8 x 768: 10.6-13.1 /
// 9.4-10.0; 8 x 1088: 11.2 / 11.1. Without query-head groups (a kv head per query head: no 17..64-row
// boxes in the plan) the plan keeps up sooner: 12 x 576: 8.1 / 9.3, so the bound is 384 tokens there.
int whole_sequence_limit(int hratio) { return hratio >= 2 ? 768 : 384; }
// Beyond those small batches, the same launch serves any batch whose sharing saves little: the plan
// reads every shared page once and pays for it with a second kernel, partial rows and the slower steps of
// its 17..64-row boxes; one work item per request reads a shared page once per request that holds it,
// from L2 after the first time. Both launches were timed on 1-level trees of 2..128 requests with
// 256..16384 shared and 32..1024 private tokens at 32/32, 16/2, 32/8 and 64/8 heads, and on the reference's
// tree sweep (benchmark/run_kernel_bench.sh:5-33); least squares with non-negative coefficients gives, in
// us per call with U = MB of K and V the tree's nodes hold, S = MB that sharing saves (the same counted
// once per request, minus U), rows = batch x query heads:
//     one item per request  6.5 + 1.9 [a second kernel: see below] + 0.165 U + 0.070 S
//     the plan              9.4 + 0.179 U + 0.002 S x (query heads per kv head) + 0.39 rows / 1000
//                           (+ 0.4 rows / 1000 for every box of a request beyond two: the partial rows of
//                           deeper trees, from 72 trees of 2-4 levels timed afterwards)
// (mean error 6 % and 10 %). One item per request is launched when its estimate is the lower one (with the
// plan's constant at 9.8: that decides more of the close cases right) and S is below 200 MB (the measured
// range of close calls; beyond it the plan won every case). Over the 356 measured cases the choice is
// within 3 % of the faster launch in 329 (always the plan: 274) and at worst 19 % slower (always the plan:
// 66 %); on the 72 deeper trees (not used for the fit) and the reference's sweep, 141 of 144 and 4.5 % at worst; e.g. plan / one item per request: 64 x (256 + 32) tokens at 64/8
// heads 13.4 / 10.8 us, 8 x (1024 + 1024) at 32/8 16.6 / 14.6, 128 x (256 + 32) at 16/2 13.0 / 7.9, against
// 128 x (256 + 32) at 32/8 15.2 / 17.9, 4 x (4096 + 32) 13.3 / 15.3. No tree of the reference's sweep changes.
// A request walked by one workgroup needs no second kernel: up to 512 tokens, or up to 2048 when the batch
// has a box per CU (requests x kv heads >= 256); the launch cuts longer ones into pieces and merges them.
constexpr double kWholeSavedMaxMB = 200.;
// Returns the longest request the one-item-per-request launch stays right for (0: launch the plan).
// unique_tokens: tokens held by the tree's nodes; max_split: the most boxes of the plan a request sits in.
int whole_sequences_pay(const std::vector<int32_t>& lens, int kv_heads, int page, int hratio, int64_t unique_tokens,
                        int max_split) {
  const bool shared = max_split > 1;
  if (lens.empty() || kv_heads <= 0 || page <= 0) return 0;
  int64_t total = 0, longest = 0;
  for (int32_t n : lens) { total += n; longest = std::max<int64_t>(longest, n); }
  if (longest <= 0) return 0;
  // PAT_WHOLE_SEQUENCES=0 / 1: always the plan / always one work item per request (measurements, tests)
  if (const char* e = std::getenv("PAT_WHOLE_SEQUENCES")) {
    if (e[0] == '0') return 0;
    if (e[0] == '1') return INT32_MAX;
  }
  const int64_t token_bytes = (int64_t)kv_heads * 128 * 2 * 2;   // (at head_dim 128; the planner does not know it)
  int small = 0;
  if (longest <= whole_sequence_limit(hratio) && (int64_t)lens.size() * kv_heads <= 512 && total * token_bytes <= (int64_t)64 << 20)
    small = whole_sequence_limit(hratio);
  if (!shared || unique_tokens <= 0 || unique_tokens > total) return small;   // nothing to merge in the plan either
  const double unique_mb = (double)(unique_tokens * token_bytes) / 1e6;
  const double saved_mb = (double)((total - unique_tokens) * token_bytes) / 1e6;
  if (saved_mb >= kWholeSavedMaxMB) return small;
  const double rows = (double)lens.size() * kv_heads * hratio;
  const double plan_us = 9.8 + 0.179 * unique_mb + 0.002 * saved_mb * hratio + (0.39 + 0.4 * std::max(0, max_split - 2)) * rows / 1000.;
  const double whole_us = 6.5 + 0.165 * unique_mb + 0.070 * saved_mb;
  if (whole_us + 1.9 < plan_us) return INT32_MAX;
  const int64_t one_kernel = (int64_t)lens.size() * kv_heads >= 256 ? 2048 : 512;
  return whole_us < plan_us && longest <= one_kernel ? std::max(small, (int)one_kernel) : small;
}

struct PrefixTreeCPP {
  int block_size;
  std::vector<int32_t> batch_lens;   // the batch as build_radix_tree got it
  at::Tensor batch_table;
  bool own_table = false;            // batch_table is a copy of ours (edits never write the caller's tensor)
  std::shared_ptr<TreeHandle> native = std::make_shared<TreeHandle>();
  std::shared_ptr<KernelInfo> info = std::make_shared<KernelInfo>();

  explicit PrefixTreeCPP(int bs) : block_size(bs) { check(pat_tree_create(bs, &native->h)); }

  void build_radix_tree(const py::object& seq_lens, const py::object& table_obj) {
    require(THPVariable_Check(table_obj.ptr()), "block_table must be a 2-D CPU Int32 Tensor");
    const at::Tensor table_in = table_obj.cast<at::Tensor>();
    require(table_in.dim() == 2, "block_table must be a 2-D CPU Int32 Tensor");
    require(table_in.device().is_cpu() && table_in.scalar_type() == at::kInt, "block_table must be a CPU Int32 Tensor");
    const at::Tensor table = table_in.contiguous();
    std::vector<int32_t> lens_vec;
    at::Tensor lens_t;
    const int32_t* lens = nullptr;
    int64_t n_lens = 0;
    if (THPVariable_Check(seq_lens.ptr())) {
      lens_t = seq_lens.cast<at::Tensor>();
      require(lens_t.device().is_cpu() && lens_t.scalar_type() == at::kInt,
              "seq_lens must be a List[int] or a CPU Int32 Tensor");
      lens_t = lens_t.reshape({-1}).contiguous();
      lens = lens_t.data_ptr<int32_t>(); n_lens = lens_t.numel();
    } else if (py::isinstance<py::list>(seq_lens)) {
      lens_vec = seq_lens.cast<std::vector<int32_t>>();
      lens = lens_vec.data(); n_lens = (int64_t)lens_vec.size();
    } else {
      throw std::runtime_error("seq_lens must be a List[int] or a CPU Int32 Tensor");
    }
    require(n_lens == table.size(0), "Seq lens list mismatch");
    batch_lens.assign(lens, lens + n_lens);
    batch_table = table;
    own_table = false;
    int rc;
    {
      py::gil_scoped_release release;   // the tree is built without the GIL (csrc/bindings.cpp:124)
      rc = pat_tree_build(native->h, lens, table.data_ptr<int32_t>(), (int32_t)table.size(0), (int32_t)table.size(1));
    }
    check(rc);
  }

  // ---- edits between decode steps (include/pat_amd.h: pat_tree_append / _remove / _grow) -----------
  // The batch copy (lengths and block rows: what the whole-sequence tables are made from) follows.
  void set_row(int64_t row, const std::vector<int32_t>& blocks, int64_t first) {
    const int64_t need = first + (int64_t)blocks.size();
    if (!batch_table.defined() || batch_table.size(1) < need) {
      const int64_t rows = batch_table.defined() ? batch_table.size(0) : 0;
      at::Tensor wider = at::zeros({rows, need + 8}, at::TensorOptions().dtype(at::kInt));
      if (rows > 0 && batch_table.size(1) > 0)
        wider.slice(1, 0, batch_table.size(1)).copy_(batch_table);
      batch_table = wider;
      own_table = true;
    }
    if (!own_table) { batch_table = batch_table.clone(); own_table = true; }
    int32_t* dst = batch_table.data_ptr<int32_t>() + row * batch_table.size(1) + first;
    for (size_t i = 0; i < blocks.size(); ++i) dst[i] = blocks[i];
  }

  int64_t append_sequence(int seq_len, const std::vector<int32_t>& blocks) {
    check(pat_tree_append(native->h, seq_len, blocks.data(), (int32_t)blocks.size()));
    const int64_t row = (int64_t)batch_lens.size();
    const int64_t width = std::max<int64_t>(batch_table.defined() ? batch_table.size(1) : 0, (int64_t)blocks.size());
    at::Tensor taller = at::zeros({row + 1, width}, at::TensorOptions().dtype(at::kInt));
    if (row > 0 && batch_table.defined() && batch_table.size(1) > 0)
      taller.slice(0, 0, row).slice(1, 0, batch_table.size(1)).copy_(batch_table);
    batch_table = taller;
    own_table = true;
    batch_lens.push_back(seq_len);
    set_row(row, blocks, 0);
    return row;
  }

  void remove_sequence(int seq) {
    check(pat_tree_remove(native->h, seq));
    const int64_t rows = (int64_t)batch_lens.size();
    batch_lens.erase(batch_lens.begin() + seq);
    if (batch_table.defined() && batch_table.size(0) == rows)
      batch_table = at::cat({batch_table.slice(0, 0, seq), batch_table.slice(0, seq + 1, rows)}, 0).contiguous();
    own_table = true;
  }

  void grow_sequence(int seq, int new_len, const std::vector<int32_t>& more_blocks) {
    require(seq >= 0 && (size_t)seq < batch_lens.size(), "sequence index out of range");
    check(pat_tree_grow(native->h, seq, new_len, more_blocks.data(), (int32_t)more_blocks.size()));
    const int64_t had = ((int64_t)batch_lens[(size_t)seq] + block_size - 1) / block_size;
    batch_lens[(size_t)seq] = new_len;
    if (!more_blocks.empty()) set_row(seq, more_blocks, had);
  }

  // One decode step later: same rows, each with its new length and the block row of the step's
  // metadata (rows grow by appending blocks). Grows every row in place; when a row cannot be grown
  // (see pat_tree_grow) the tree is built afresh from the arguments. Returns true when no rebuild
  // was needed. Either way the tree is that of build_radix_tree(seq_lens, block_table).
  bool advance(const std::vector<int32_t>& seq_lens, const at::Tensor& table_in) {
    require(table_in.dim() == 2 && table_in.device().is_cpu() && table_in.scalar_type() == at::kInt,
            "block_table must be a 2-D CPU Int32 Tensor");
    require((int64_t)seq_lens.size() == table_in.size(0), "Seq lens list mismatch");
    const at::Tensor table = table_in.contiguous();
    bool grown = seq_lens.size() == batch_lens.size();
    if (grown) {
      py::gil_scoped_release release;
      const int32_t* t = table.data_ptr<int32_t>();
      const int64_t w = table.size(1);
      for (size_t i = 0; i < seq_lens.size() && grown; ++i) {
        if (seq_lens[i] == batch_lens[i]) continue;
        const int64_t had = ((int64_t)batch_lens[i] + block_size - 1) / block_size;
        const int64_t need = ((int64_t)seq_lens[i] + block_size - 1) / block_size;
        if (seq_lens[i] < batch_lens[i] || need > w) { grown = false; break; }
        grown = pat_tree_grow(native->h, (int32_t)i, seq_lens[i], t + (int64_t)i * w + had, (int32_t)(need - had)) == PAT_OK;
      }
    }
    if (!grown) {
      int rc;
      {
        py::gil_scoped_release release;
        rc = pat_tree_build(native->h, seq_lens.data(), table.data_ptr<int32_t>(), (int32_t)table.size(0), (int32_t)table.size(1));
      }
      check(rc);
    }
    batch_lens = seq_lens;
    batch_table = table;
    own_table = false;
    return grown;
  }

  void pack_schedule(const py::object& mnws_obj, int hratio, int kv_head, bool use_compute_model) {
    std::vector<int32_t> mnws;
    bool given = false;
    if (!mnws_obj.is_none()) {
      const auto rows = mnws_obj.cast<std::vector<std::vector<int>>>();
      // an empty list selects the default buckets (csrc/prefix_tree.h:189)
      for (const auto& r : rows) {
        require(r.size() == 3, "MNWs entries must be [M, N, W]");
        mnws.insert(mnws.end(), r.begin(), r.end());
      }
      given = !rows.empty();
    }
    auto fresh = std::make_shared<KernelInfo>();
    int rc, rc_flat = PAT_OK;
    at::Tensor host;
    {
      py::gil_scoped_release release;   // planning runs without the GIL (csrc/bindings.cpp:138)
      rc = pat_tree_pack(native->h, given ? mnws.data() : nullptr, given ? (int32_t)(mnws.size() / 3) : 0, hratio,
                         kv_head, use_compute_model ? 1 : 0, nullptr);
      if (rc == PAT_OK) rc_flat = pat_tree_flat_plan(native->h, &fresh->layout, nullptr, 0);
    }
    check(rc);
    c10::InferenceMode plain(false);   // plan tensors keep their version counters (see KernelInfo::to_gpu)
    if (rc_flat == PAT_OK) {
      int64_t total = std::max<int64_t>(fresh->layout.total, 1);
      const int64_t nb = (int64_t)batch_lens.size();
      int ws_allowed = 0;
      if (hratio >= 1 && hratio <= 16 && fresh->layout.batch == nb && batch_table.defined() && batch_table.size(0) == nb) {
        int64_t unique = 0;
        const int n_nodes = pat_tree_num_nodes(native->h);
        for (int i = 0; i < n_nodes; ++i) {
          pat_node_view node;
          if (pat_tree_node(native->h, i, &node) == PAT_OK && node.parent >= -1) unique += node.num_tokens;
        }
        ws_allowed = whole_sequences_pay(batch_lens, kv_head, block_size, hratio, unique, fresh->layout.max_split_per_seq);
      }
      if (ws_allowed > 0) {
        int64_t longest = 0;
        for (int32_t n : batch_lens) longest = std::max<int64_t>(longest, n);
        fresh->whole_seqs = true;
        fresh->ws_batch = (int)nb;
        // (8 spare columns: room for in-place growth between decode steps)
        fresh->ws_width = (int)std::min<int64_t>(batch_table.size(1), (longest + block_size - 1) / block_size + 8);
        fresh->ws_tile = 16;
        fresh->ws_longest_allowed = ws_allowed;
        fresh->ws_offset = total;
        total += 4 * nb + nb * fresh->ws_width;
      }
      host = at::empty({total}, at::TensorOptions().dtype(at::kInt).pinned_memory(at::hasHIP() || at::hasCUDA()));
      {
        py::gil_scoped_release release;
        rc = pat_tree_flat_plan(native->h, &fresh->layout, host.data_ptr<int32_t>(), host.numel());
      }
      check(rc);
      if (fresh->whole_seqs) {
        const int64_t nb = fresh->ws_batch, w = fresh->ws_width;
        int32_t* d = host.data_ptr<int32_t>() + fresh->ws_offset;
        const int32_t* src = batch_table.data_ptr<int32_t>();
        const int64_t src_w = batch_table.size(1);
        for (int64_t i = 0; i < nb; ++i) {
          d[i] = (int32_t)i; d[nb + i] = 1; d[2 * nb + i] = 0; d[3 * nb + i] = batch_lens[(size_t)i];
          const int64_t used = ((int64_t)batch_lens[(size_t)i] + block_size - 1) / block_size;
          for (int64_t j = 0; j < w; ++j) d[4 * nb + i * w + j] = j < used ? src[i * src_w + j] : 0;
        }
      }
      fresh->flat = host;
      fresh->max_split = fresh->layout.max_split_per_seq;
      fresh->max_boxes = fresh->layout.max_boxes_per_seq;
      fresh->max_seqs = fresh->layout.max_seqs_in_box;
      fresh->max_blocks = fresh->layout.max_blocks_in_box;
      fresh->bind(host);
    } else {
      // more buckets than one launch takes: the plan can still be read, table by table
      pat_plan_view view;
      check(pat_tree_plan(native->h, &view));
      for (int b = 0; b < view.num_buckets; ++b) {
        const pat_bucket_view& bk = view.buckets[b];
        const int64_t n = bk.num_boxes;
        fresh->mnws.push_back({bk.mnw[0], bk.mnw[1], bk.mnw[2]});
        fresh->q_tables.push_back(host_i32(n * bk.max_seqs, bk.q_table).view({n, bk.max_seqs}));
        fresh->slot_tables.push_back(host_i32(n * bk.max_seqs, bk.q_slot).view({n, bk.max_seqs}));
        fresh->block_tables.push_back(host_i32(n * bk.max_blocks, bk.block_table).view({n, bk.max_blocks}));
        fresh->num_seqs.push_back(host_i32(n, bk.num_seqs));
        fresh->ranks.push_back(host_i32(n, bk.rank));
        fresh->kvs.push_back(host_i32(n, bk.kv));
      }
      fresh->num_split_per_seq = host_i32(view.batch, view.num_split_per_seq);
      fresh->num_boxes_per_seq = host_i32(view.batch, view.num_boxes_per_seq);
      fresh->max_split = view.max_split_per_seq; fresh->max_boxes = view.max_boxes_per_seq;
      fresh->max_seqs = view.max_seqs_in_box; fresh->max_blocks = view.max_blocks_in_box;
    }
    info = fresh;
  }
};

// ---- forward ------------------------------------------------------------------------------------------
std::mutex g_table_mutex;
// (both hold device tensors and live until the process ends, undestroyed: see the evict buffers)
auto& g_table_launches = *new std::unordered_map<std::string, std::shared_ptr<Prepared>>();
auto& g_table_records = *new std::unordered_map<std::string, std::shared_ptr<RecordStore>>();   // per plan (tables + versions)

struct DeviceScope {   // the kernels launch on the current HIP device: switch only when q lives elsewhere
  std::optional<c10::DeviceGuard> guard;
  explicit DeviceScope(const at::Tensor& q) {
    require(q.is_cuda(), "q must be on CUDA");
    guard.emplace(q.device());
  }
};

void fwd_tables(const at::Tensor& q, const at::Tensor& k, const at::Tensor& v, const at::Tensor& num_split,
                const TensorList& q_tables, const TensorList& block_tables, const TensorList& num_seqs,
                const TensorList& ranks, const TensorList& kvs, const std::vector<std::vector<int>>& mnw,
                int max_split, int max_seqs, int max_blocks, double scale, const at::Tensor& out,
                const py::object& /*timing_: accepted and ignored, the reference never reads it (csrc/api.h:288-290)*/,
                const std::optional<at::Tensor>& lse, const std::optional<TensorList>& slot_tables,
                const std::optional<std::vector<int>>& bucket_flags) {
  require(k.is_cuda(), "kcache must be on CUDA");
  require(v.is_cuda(), "vcache must be on CUDA");
  DeviceScope scope(q);
  // The prepared launch is kept per set of tensors: a decode step calls this once per layer with the
  // same plan. The key holds what the argument block was built from (addresses, layouts, version
  // counters of the plan tensors); the tensors' contents are read by the kernels at every call.
  Key plan_key;
  plan_key.plan_tensor(num_split);
  for (const TensorList* l : {&q_tables, &block_tables, &num_seqs, &ranks, &kvs}) {
    plan_key.add((int64_t)l->size());
    for (const at::Tensor& t : *l) plan_key.plan_tensor(t);
  }
  for (const auto& m : mnw) for (int x : m) plan_key.add(x);
  plan_key.add(max_split); plan_key.add(max_seqs); plan_key.add(max_blocks);
  plan_key.add(slot_tables.has_value());
  if (slot_tables.has_value()) for (const at::Tensor& t : *slot_tables) plan_key.plan_tensor(t);
  if (bucket_flags.has_value()) for (int f : *bucket_flags) plan_key.add(f);
  Key key;
  key.tensor(q); key.tensor(k); key.tensor(v); key.tensor(out);
  key.add(lse.has_value()); if (lse.has_value()) key.tensor(*lse);
  key.add(scale);
  key.bytes += plan_key.bytes;

  // (version counters are part of the key: an edited plan is another key; tensors without a counter
  // are served without snapshots)
  bool tracked = !num_split.is_inference();
  for (const TensorList* l : {&q_tables, &block_tables, &num_seqs, &ranks, &kvs})
    for (const at::Tensor& t : *l) tracked = tracked && !t.is_inference();
  if (slot_tables.has_value()) for (const at::Tensor& t : *slot_tables) tracked = tracked && !t.is_inference();
  const int64_t version = tracked ? 0 : kUntracked;

  std::shared_ptr<Prepared> L;
  std::shared_ptr<RecordStore> store;
  {
    std::lock_guard<std::mutex> lock(g_table_mutex);
    auto it = g_table_launches.find(key.bytes);
    if (it != g_table_launches.end()) {
      L = it->second;
      auto st = g_table_records.find(plan_key.bytes);
      if (st != g_table_records.end()) store = st->second; else L.reset();
    }
  }
  if (!L) {
    PlanTables pt{&q_tables, &block_tables, &num_seqs, &ranks, &kvs,
                  slot_tables.has_value() ? &*slot_tables : nullptr, &mnw,
                  bucket_flags.has_value() ? &*bucket_flags : nullptr};
    // the launch records belong to the plan (tables + their versions), not to q / k / v / out
    {
      std::lock_guard<std::mutex> lock(g_table_mutex);
      // (launches hold pointers into their plan's store: both maps are emptied together)
      if (g_table_records.size() >= 16 && g_table_records.find(plan_key.bytes) == g_table_records.end()) {
        g_table_records.clear();
        g_table_launches.clear();
      }
      auto& slot = g_table_records[plan_key.bytes];
      if (!slot) {
        slot = std::make_shared<RecordStore>();
        slot->keep.push_back(num_split);
        for (const TensorList* l : {&q_tables, &block_tables, &num_seqs, &ranks, &kvs})
          for (const at::Tensor& t : *l) slot->keep.push_back(t);
        if (slot_tables.has_value()) for (const at::Tensor& t : *slot_tables) slot->keep.push_back(t);
      }
      store = slot;
    }
    L = prepare(q, k, v, num_split, pt, max_split, max_seqs, max_blocks, scale, out, lse, *store, version);
    std::lock_guard<std::mutex> lock(g_table_mutex);
    if (g_table_launches.size() >= 64) g_table_launches.clear();
    g_table_launches[key.bytes] = L;
  }
  run(*L, *store, version, q.device());
}

void fwd_tree(const at::Tensor& q, const at::Tensor& k, const at::Tensor& v, PrefixTreeCPP& tree, double scale,
              const at::Tensor& out, const std::optional<at::Tensor>& lse) {
  require(k.is_cuda(), "kcache must be on CUDA");
  require(v.is_cuda(), "vcache must be on CUDA");
  DeviceScope scope(q);
  KernelInfo& info = *tree.info;
  Key key;
  key.tensor(q); key.tensor(k); key.tensor(v); key.tensor(out); key.add(scale);
  key.add(lse.has_value()); if (lse.has_value()) key.tensor(*lse);
  std::shared_ptr<Prepared> L;
  const int64_t version = info.plan_version();
  auto it = info.cache.find(key.bytes);
  if (it != info.cache.end()) {
    L = it->second;   // (run() takes a new snapshot when the plan tables were edited in place since)
  } else {
    const bool l = info.has_launch;
    const std::vector<int> no_flags;
    // partial results are filed by slot_tables: the launch merges each sequence's boxes of THIS plan
    // (num_split_per_seq counts on over repeated pack_schedule calls)
    PlanTables pt{l ? &info.l_q_tables : &info.q_tables, l ? &info.l_block_tables : &info.block_tables,
                  l ? &info.l_num_seqs : &info.num_seqs, l ? &info.l_ranks : &info.ranks, l ? &info.l_kvs : &info.kvs,
                  l ? &info.l_slot_tables : &info.slot_tables, l ? &info.l_mnws : &info.mnws,
                  l ? &info.l_flags : &no_flags};
    require(!pt.mnw->empty(), "the tree has no plan: call pack_schedule and kernel_info.to_gpu first");
    if (info.whole_seqs && !info.ws_q_table.empty()) {
      // a small batch of short requests: one work item per request, one kernel (see KernelInfo::whole_seqs)
      PlanTables ws{&info.ws_q_table, &info.ws_block_table, &info.ws_num_seqs, &info.ws_rank, &info.ws_kv, nullptr,
                    &info.ws_mnw, &no_flags};
      L = prepare(q, k, v, info.ws_num_split, ws, 1, 1, info.ws_width, scale, out, lse, info.records, version);
    } else {
      L = prepare(q, k, v, info.num_boxes_per_seq, pt, info.max_boxes, info.max_seqs, info.max_blocks, scale, out, lse,
                  info.records, version);
    }
    if (info.cache.size() >= 256) info.cache.clear();
    info.cache[key.bytes] = L;
  }
  run(*L, info.records, version, q.device());
}

void paged_decode_baseline(const at::Tensor& q, const at::Tensor& k, const at::Tensor& v, const at::Tensor& block_table,
                           const at::Tensor& seq_lens, double scale, const at::Tensor& out,
                           const std::optional<at::Tensor>& lse, bool even_lengths) {
  const std::pair<const char*, const at::Tensor*> named[] = {
      {"q", &q}, {"kcache", &k}, {"vcache", &v}, {"block_table", &block_table}, {"seq_lens", &seq_lens}};
  for (const auto& nt : named) require(nt.second->is_cuda(), std::string(nt.first) + " must be on CUDA");
  require((q.scalar_type() == at::kHalf || q.scalar_type() == at::kBFloat16) && k.scalar_type() == q.scalar_type() &&
              v.scalar_type() == q.scalar_type(), "only support fp16 and bf16 data type");
  require(q.dim() == 4 && k.dim() == 4 && v.dim() == 4, "q, kcache, vcache must be 4-D");
  require(block_table.scalar_type() == at::kInt && block_table.dim() == 2 && block_table.stride(1) == 1,
          "block_table must be a 2-D int32 tensor with contiguous rows");
  require(seq_lens.scalar_type() == at::kInt && seq_lens.dim() == 1 && seq_lens.is_contiguous(),
          "seq_lens must be a contiguous 1-D int32 tensor");
  const int64_t b = q.size(0), h = q.size(2), d = q.size(3);
  require(q.size(1) == 1, "q must have shape (batch_size, 1, n_heads, head_size): decode only");
  require(block_table.size(0) == b && seq_lens.size(0) == b, "block_table / seq_lens must have one row per request");
  require(out.is_cuda() && out.scalar_type() == q.scalar_type() && out.sizes() == q.sizes() && out.stride(-1) == 1,
          "out must be a CUDA tensor with q's shape and dtype and a contiguous last dimension");
  pat_baseline_args a;
  std::memset(&a, 0, sizeof(a));
  a.dtype = q.scalar_type() == at::kBFloat16 ? PAT_DTYPE_BF16 : PAT_DTYPE_F16;
  a.batch = (int32_t)b; a.heads = (int32_t)h; a.kv_heads = (int32_t)k.size(2); a.head_dim = (int32_t)d;
  a.page_size = (int32_t)k.size(1); a.num_pages = (int32_t)k.size(0); a.max_blocks = (int32_t)block_table.size(1);
  a.q = q.data_ptr(); a.k = k.data_ptr(); a.v = v.data_ptr(); a.out = out.data_ptr();
  strides3(q, a.q_stride); strides3(k, a.k_stride); strides3(v, a.v_stride); strides3(out, a.o_stride);
  a.block_table = block_table.data_ptr<int32_t>(); a.block_table_stride = block_table.stride(0);
  a.seq_lens = seq_lens.data_ptr<int32_t>();
  a.softmax_scale = (float)scale;
  a.flags = even_lengths ? PAT_BUCKET_EVEN : 0;
  if (lse.has_value()) {
    require(lse->is_cuda() && lse->scalar_type() == at::kFloat && lse->is_contiguous() && lse->numel() == b * h,
            "softmax_lse must be a contiguous CUDA float32 tensor with batch_size * n_heads elements");
    a.lse_out = lse->data_ptr<float>();
  }
  size_t need = 0;
  check(pat_paged_decode_baseline_workspace_bytes(&a, &need));
  DeviceScope scope(q);
  at::Tensor ws = at::empty({(int64_t)need}, at::TensorOptions().dtype(at::kByte).device(q.device()));
  a.workspace = ws.data_ptr(); a.workspace_bytes = need;
  check(pat_paged_decode_baseline_launch(&a, raw_stream(q.device())));
}

}  // namespace

PYBIND11_MODULE(_prefix_attn, m) {
  m.doc() = "prefix-aware decode attention over a paged KV cache for AMD MI355X (libpat_amd)";
  require(pat_abi_version() == PAT_ABI_VERSION, "libpat_amd.so and the _prefix_attn extension were built from different headers");

  py::class_<KernelInfo, std::shared_ptr<KernelInfo>>(m, "KernelInfo")
      .def(py::init<>())
      .def("to_gpu", [](KernelInfo& ki, const py::object& device) { ki.to_gpu(to_device(device)); }, py::arg("device"))
      .def_readonly("q_tables", &KernelInfo::q_tables)
      .def_readonly("block_tables", &KernelInfo::block_tables)
      .def_readonly("num_seqs_per_CTAs", &KernelInfo::num_seqs)
      .def_readonly("CTA_ranks", &KernelInfo::ranks)
      .def_readonly("kv_in_CTAs", &KernelInfo::kvs)
      // not in the reference: per (box, sequence) the box's ordinal among that sequence's boxes, the
      // collision-free partial-result slot; and the boxes of this plan per sequence
      .def_readonly("slot_tables", &KernelInfo::slot_tables)
      .def_readonly("num_boxes_per_seq", &KernelInfo::num_boxes_per_seq)
      .def_readonly("max_boxes_per_seq", &KernelInfo::max_boxes)
      .def_readonly("MNWs", &KernelInfo::mnws)
      .def_readonly("num_split_per_seq", &KernelInfo::num_split_per_seq)
      .def_readonly("max_split_per_seq", &KernelInfo::max_split)
      .def_readonly("max_seqs_in_CTA", &KernelInfo::max_seqs)
      .def_readonly("max_blocks_in_CTA", &KernelInfo::max_blocks)
      .def("invalidate", &KernelInfo::invalidate,
           "Drops what launches remember about the plan tables' contents (launch records, derived slots): call it "
           "after writing to the tables by means torch's version counters do not see.")
      .def("launch_tables", &KernelInfo::launch_tables,
           "The per-bucket tables as the kernels get them (boxes longest first, a bucket with a wide head split "
           "in two) with their tile labels under \"MNWs\" and hints under \"flags\".")
      .def("whole_sequence_tables", &KernelInfo::whole_sequence_tables,
           "Small batches of short requests are launched as one work item per request (a single kernel that "
           "writes `out`): the tables of that launch, with its num_split_per_seq / max_* values, or None when "
           "the plan is launched as planned.")
      .def("launch_position", &KernelInfo::launch_position, py::arg("bucket"),
           "For the boxes of a scheduler bucket, in scheduler order: (launch bucket, row in it) as two int64 tensors.")
      .def_property_readonly("_flat", [](const KernelInfo& ki) -> py::object {
        return ki.flat.has_value() ? py::cast(*ki.flat) : py::none();
      })
      .def_property_readonly("_launch_order", [](const KernelInfo& ki) { return ki.launch_order; })
      .def_property_readonly("_launch_parts", [](const KernelInfo& ki) {
        std::vector<std::vector<std::tuple<int, int, int>>> out;
        for (const auto& parts : ki.launch_parts) {
          out.emplace_back();
          for (const LaunchPart& p : parts) out.back().emplace_back(p.bucket, p.lo, p.hi);
        }
        return out;
      })
      .def_property_readonly("_launch_tunings", [](const KernelInfo& ki) {
        std::vector<std::vector<int64_t>> out;   // per cached launch: the overrides in struct order, {} = none
        for (const auto& kv : ki.cache) {
          const pat_fwd_tuning& t = kv.second->tuning;
          if (kv.second->args.tuning == nullptr) out.emplace_back();
          else out.push_back({t.chunk_tokens, t.tall_chunk_tokens, t.head_per_wave_tokens, t.head_per_wave_long_tokens,
                              t.head_per_wave_long_wgs, t.equalize_chunks, t.direct_out, t.tall_rows});
        }
        return out;
      })
      .def_property_readonly("_launch_workspace_bytes", [](const KernelInfo& ki) {
        std::vector<size_t> out;
        for (const auto& kv : ki.cache) out.push_back(kv.second->need);
        return out;
      });

  py::class_<PrefixTreeCPP>(m, "PrefixTreeCPP", py::dynamic_attr())
      .def(py::init<int>(), py::arg("block_size"))
      .def_readonly("block_size", &PrefixTreeCPP::block_size)
      .def("build_radix_tree", &PrefixTreeCPP::build_radix_tree, py::arg("seq_lens"), py::arg("block_table"))
      .def("append_sequence", &PrefixTreeCPP::append_sequence, py::arg("seq_len"), py::arg("blocks"),
           "A request joins the batch behind the last row; returns its row. The tree is then what "
           "build_radix_tree gives for the edited batch.")
      .def("remove_sequence", &PrefixTreeCPP::remove_sequence, py::arg("seq"),
           "Row `seq` leaves the batch; the rows behind it move up by one.")
      .def("grow_sequence", &PrefixTreeCPP::grow_sequence, py::arg("seq"), py::arg("new_len"),
           py::arg("more_blocks") = std::vector<int32_t>(),
           "Row `seq` now has new_len tokens and `more_blocks` behind its old blocks. Raises ValueError (tree "
           "unchanged) when only a fresh build can know the new shape.")
      .def("advance", &PrefixTreeCPP::advance, py::arg("seq_lens"), py::arg("block_table"),
           "One decode step later: the same rows with their new lengths and block rows. Grows the tree in place "
           "(False: it had to be built afresh); the result equals build_radix_tree(seq_lens, block_table).")
      .def("pack_schedule", &PrefixTreeCPP::pack_schedule, py::arg("MNWs") = py::none(), py::arg("HRatio") = 1,
           py::arg("kvHead") = 8, py::arg("use_compute_model") = false)
      .def_property_readonly("kernel_info", [](const PrefixTreeCPP& t) { return t.info; });

  m.def("prefix_attn_with_kvcache", &fwd_tables, py::arg("q"), py::arg("k_cache_paged"), py::arg("v_cache_paged"),
        py::arg("num_split_per_seq"), py::arg("query_tables"), py::arg("block_tables"), py::arg("num_seqs_per_CTAs"),
        py::arg("CTA_ranks"), py::arg("kv_in_CTAs"), py::arg("MNW"), py::arg("max_split_per_seq"),
        py::arg("max_seqs_in_CTA"), py::arg("max_blocks_in_CTA"), py::arg("softmax_scale"), py::arg("out"),
        py::arg("timing_") = py::none(), py::kw_only(), py::arg("softmax_lse") = py::none(),
        py::arg("slot_tables") = py::none(), py::arg("bucket_flags") = py::none(),
        "Table form. Extra keywords: softmax_lse (float32 [batch, heads]) receives the natural-log LSE; "
        "slot_tables (KernelInfo.slot_tables) files partial results by each box's ordinal within its sequence "
        "(derived on the device when absent); bucket_flags are launch-geometry hints.");
  m.def("prefix_attn_with_kvcache", &fwd_tree, py::arg("q"), py::arg("k_cache_paged"), py::arg("v_cache_paged"),
        py::arg("tree"), py::arg("softmax_scale"), py::arg("out"), py::kw_only(), py::arg("softmax_lse") = py::none(),
        "Tree form: the plan of a PrefixTreeCPP whose kernel_info is on the device.");
  m.def("invalidate_plans", [] {
          std::lock_guard<std::mutex> lock(g_table_mutex);
          g_table_launches.clear();
          g_table_records.clear();
        },
        "Table form: drops every remembered launch and plan snapshot (launch records, derived slots). For plan "
        "tables written by means torch's version counters do not see.");
  m.def("set_autotune", [](bool on) { g_autotune = on; }, py::arg("enabled"),
        "Measured choice of the launch geometry (pat_fwd_autotune) the first time a plan shape is launched: off "
        "unless switched on here or with PAT_AUTOTUNE=1. The measurement runs the launch some fifty times on the "
        "current stream and synchronises it, once per shape.");
  m.def("get_autotune", [] { return g_autotune; });
  m.def("autotune_runs", [] { return g_tuning_runs.load(); },
        "Number of geometry measurements made since the module was loaded (0 unless tuning was switched on).");
  m.def("clear_autotune_cache", [] { std::lock_guard<std::mutex> lock(g_tune_mutex); g_tuned.clear(); });
  m.def("paged_decode_baseline", &paged_decode_baseline, py::arg("q"), py::arg("k_cache_paged"),
        py::arg("v_cache_paged"), py::arg("block_table"), py::arg("seq_lens"), py::arg("softmax_scale"), py::arg("out"),
        py::arg("softmax_lse") = py::none(), py::arg("even_lengths") = false,
        "Prefix-oblivious paged decode attention through the same kernels: one work item per request.");
}
