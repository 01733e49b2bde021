#include "hip_ops.h"

#include <c10/hip/HIPStream.h>
#include <hip/hip_runtime_api.h>

#include <atomic>
#include <map>

#include "gs_hip.h"

namespace gs {
namespace hip {
namespace {

std::atomic<uint64_t> g_seed{7777};
std::atomic<int64_t> g_algo{GS_SAMPLE_AUTO};
constexpr int64_t kOneLaunchMaxColumns = int64_t(1) << 26;
std::atomic<bool> g_deferred{true};

void Check(int status, const char* what) {
  TORCH_CHECK(status == GS_OK, what, " failed (", status, "): ", gs_status_string(status));
}

void* Stream(const torch::Tensor& t) {
  return static_cast<void*>(c10::hip::getCurrentHIPStream(t.device().index()).stream());
}

// Device tensors only: the reference has no CPU path either and aborts with
// "Not implemented warning" (src/graph_ops.cc:27); here that is an exception.
void NeedDevice(const torch::Tensor& t, const char* name) {
  TORCH_CHECK(t.defined(), name, " is undefined");
  TORCH_CHECK(t.is_cuda(), "Not implemented warning: ", name, " must be a GPU tensor");
  TORCH_CHECK(t.is_contiguous(), name, " must be contiguous");
}

int IdBytes(const torch::Tensor& t, const char* name) {
  NeedDevice(t, name);
  if (t.scalar_type() == torch::kInt64) return 8;
  if (t.scalar_type() == torch::kInt32) return 4;
  TORCH_CHECK(false, name, " must be int64 (or int32), got ", t.scalar_type());
}

void NeedI64(const torch::Tensor& t, const char* name) {
  NeedDevice(t, name);
  TORCH_CHECK(t.scalar_type() == torch::kInt64, name, " must be int64, got ", t.scalar_type());
}

void NeedF32(const torch::Tensor& t, const char* name) {
  NeedDevice(t, name);
  TORCH_CHECK(t.scalar_type() == torch::kFloat32, name, " must be float32, got ", t.scalar_type());
}

const int64_t* OptI64(const torch::optional<torch::Tensor>& t, const char* name) {
  if (!t.has_value() || !t.value().defined()) return nullptr;
  NeedI64(t.value(), name);
  return t.value().data_ptr<int64_t>();
}

// optional node-id tensor of the width `idb`
const void* OptIds(const torch::optional<torch::Tensor>& t, int idb, const char* name) {
  if (!t.has_value() || !t.value().defined()) return nullptr;
  TORCH_CHECK(IdBytes(t.value(), name) == idb, name, " must have the dtype of the graph ids");
  return t.value().data_ptr();
}

// The edge array (or edge weights) of a graph for a sampling call.  A graph without edges has
// an empty tensor there, whose pointer is null, and the entry points refuse a null array as
// long as there are columns; no degree is above zero then, so nothing is read through the
// pointer, and the offsets' address stands in.
const void* EdgeArray(const torch::Tensor& edges, const torch::Tensor& indptr) {
  return edges.numel() > 0 ? edges.data_ptr() : indptr.data_ptr();
}

torch::Tensor Scratch(size_t bytes, const torch::Tensor& like) {
  return torch::empty({static_cast<int64_t>(bytes < 256 ? 256 : bytes)},
                      torch::dtype(torch::kUInt8).device(like.device()));
}

// ---- result mailboxes: totals arrive in pinned host memory, no stream sync ----
// A ring of kBoxes {total, ticket} pairs per (thread, device); call number t posts
// to slot t % kBoxes, so a total stays readable until kBoxes later calls have
// been issued.
constexpr int64_t kBoxes = 1024;
constexpr int64_t kLost = -3;     // the slot was reused before anyone read it
constexpr int64_t kBinsFull = -4; // posted by the binned batch relabel: repeat on hash regions
constexpr int64_t kTooWide = -2;  // posted by the narrow relabel: a key needs more than 32 bits
constexpr int64_t kGaveUp = -1;   // posted when a tile's bounded wait ran out

// 64-bit ids go on the one-word table slots of 32-bit ids (GS_NARROW_IDS) until this thread
// meets one that does not fit 32 bits; from then on it asks for the two-array slots.
thread_local bool t_narrow_ids = true;
int TableIds(int idb) { return idb == 8 && t_narrow_ids ? (8 | GS_NARROW_IDS) : idb; }

struct HostBoxes {
  torch::Tensor buf;  // kBoxes x {total, ticket}, pinned
  gs_mailbox* ring = nullptr;
  int64_t next = 1;
  gs_mailbox* slot(int64_t ticket) const { return ring + ticket % kBoxes; }
};

HostBoxes& Boxes(int device) {
  thread_local std::map<int, HostBoxes> boxes;
  HostBoxes& b = boxes[device];
  if (!b.ring) {
    b.buf = torch::zeros({kBoxes * 2}, torch::TensorOptions().dtype(torch::kInt64).pinned_memory(true));
    b.ring = reinterpret_cast<gs_mailbox*>(b.buf.data_ptr<int64_t>());
  }
  return b;
}

// Spins until the kernel has posted `ticket`; every few thousand polls it asks
// the stream whether it has drained or failed, so a kernel that never posts
// turns into an error (or kLost when a later call took the slot), not a hang.
int64_t WaitBox(const gs_mailbox* box, int64_t ticket, void* stream, const char* what) {
  hipStream_t st = static_cast<hipStream_t>(stream);
  for (uint64_t n = 1;; ++n) {
    const int64_t seen = __atomic_load_n(&box->ticket, __ATOMIC_ACQUIRE);
    if (seen == ticket) break;
    if (seen > ticket) return kLost;
    if ((n & 0xFFF) == 0) {
      const hipError_t q = hipStreamQuery(st);
      if (q == hipSuccess) {
        const int64_t again = __atomic_load_n(&box->ticket, __ATOMIC_ACQUIRE);
        if (again == ticket) break;
        if (again > ticket) return kLost;
        TORCH_CHECK(false, what, ": the stream drained without reporting a total");
      }
      TORCH_CHECK(q == hipErrorNotReady, what, ": ", hipGetErrorString(q));
    }
    __builtin_ia32_pause();
  }
  const int64_t total = __atomic_load_n(&box->total, __ATOMIC_RELAXED);
  // the slot may have been rewritten between the two loads
  if (__atomic_load_n(&box->ticket, __ATOMIC_ACQUIRE) != ticket) return kLost;
  return total;  // kGaveUp and kTooWide are the caller's to act on
}

// A tile gave up waiting for its predecessors: the error word it raised stays in the
// look-back state until that is zero-filled, and would fail every later launch on it.  Clears
// it behind the failed launch (an all-zero state is valid under any epoch) and reports.
[[noreturn]] void GaveUp(const torch::Tensor& state, void* stream, const char* what) {
  if (state.defined())
    (void)hipMemsetAsync(state.data_ptr(), 0, static_cast<size_t>(state.numel()),
                         static_cast<hipStream_t>(stream));
  TORCH_CHECK(false, what, ": a tile gave up waiting for its predecessors; the look-back state "
              "has been cleared and the call can be repeated");
}

// Look-back state of the one-launch sampler, one per (device, stream): zero-filled
// when it is (re)allocated and when the epoch counter wraps, never in between.
struct FusedStateBuf {
  torch::Tensor buf;
  uint32_t epoch = 0;
};

FusedStateBuf& FusedState(size_t bytes, const torch::Tensor& like, void* stream) {
  thread_local std::map<std::pair<int, void*>, FusedStateBuf> states;
  FusedStateBuf& s = states[{like.device().index(), stream}];
  if (!s.buf.defined() || static_cast<size_t>(s.buf.numel()) < bytes) {
    const int64_t n = static_cast<int64_t>(bytes < 65536 ? 65536 : bytes);
    s.buf = torch::zeros({n}, torch::dtype(torch::kUInt8).device(like.device()));
    s.epoch = 0;
  }
  if (s.epoch == 16383) {
    s.buf.zero_();
    s.epoch = 0;
  }
  ++s.epoch;
  return s;
}

// Hash table of the relabel that follows the sampler, one per (thread, device, stream, id
// width): prepared when it is (re)allocated or after a failed call, left empty by every
// call, so no call starts by clearing it.
struct RelabelTable {
  torch::Tensor buf;
  int64_t items = 0;   // number of mapping items it was sized for
  bool clean = false;  // false: has to be prepared before the next use
  // 64-bit ids on the one-word slots of 32-bit ids (gs_relabel_sampled_narrow) until a key
  // turns up that does not fit 32 bits
  bool narrow = true;
};

RelabelTable& RelabelTableFor(const torch::Tensor& like, void* stream, int idb, int64_t items) {
  thread_local std::map<std::tuple<int, void*, int>, RelabelTable> tables;
  RelabelTable& t = tables[{like.device().index(), stream, idb}];
  if (!t.buf.defined() || t.items < items) {
    int64_t want = 1 << 16;
    while (want < items) want <<= 1;
    t.buf = torch::empty({static_cast<int64_t>(gs_relabel_table_bytes(want, idb))},
                         torch::dtype(torch::kUInt8).device(like.device()));
    t.items = want;
    t.clean = false;
  }
  if (!t.clean) {
    Check(gs_relabel_table_init(t.buf.data_ptr(), t.buf.numel(), idb == 8 && t.narrow ? 4 : idb,
                                stream),
          "gs_relabel_table_init");
    t.clean = true;
  }
  return t;
}

torch::TensorOptions I64(const torch::Tensor& like) {
  return torch::dtype(torch::kInt64).device(like.device());
}

int OpCode(const std::string& op) {
  if (op == "add") return GS_OP_ADD;
  if (op == "sub") return GS_OP_SUB;
  if (op == "mul") return GS_OP_MUL;
  if (op == "div") return GS_OP_DIV;
  if (op == "copy_lhs") return GS_OP_COPY_LHS;
  if (op == "copy_rhs") return GS_OP_COPY_RHS;
  if (op == "dot") return GS_OP_DOT;
  TORCH_CHECK(false, "Unsupported SpMM/SDDMM binary operator: ", op);
}

}  // namespace

namespace {
// a thread that called SetThreadSeed counts its own seeds until it calls SetSeed
thread_local bool t_own_seed = false;
thread_local uint64_t t_seed = 0;
}  // namespace

void SetSeed(uint64_t seed) {
  g_seed.store(seed);
  t_own_seed = false;  // the caller is back on the shared counter
}
void SetThreadSeed(uint64_t seed) {
  t_own_seed = true;
  t_seed = seed;
}
uint64_t NextSeed() { return t_own_seed ? t_seed++ : g_seed.fetch_add(1); }
uint64_t PeekSeed() { return t_own_seed ? t_seed : g_seed.load(); }
void RewindSeeds(uint64_t n) {
  if (t_own_seed)
    t_seed -= n;
  else
    g_seed.fetch_sub(n);
}
namespace {
std::atomic<bool> g_batched_no_wait{true};
std::atomic<int64_t> g_no_wait_counts[2];
}  // namespace
std::vector<int64_t> BatchedNoWaitCounts() {
  return {g_no_wait_counts[0].load(), g_no_wait_counts[1].load()};
}
void CountBatchedNoWait(bool went_through) { g_no_wait_counts[went_through ? 0 : 1].fetch_add(1); }
void SetBatchedNoWait(bool on) { g_batched_no_wait.store(on); }
bool BatchedNoWait() { return g_batched_no_wait.load(); }

namespace {
std::atomic<bool> g_ordered_sums{false};
}
void SetOrderedSums(bool on) { g_ordered_sums.store(on); }
bool OrderedSums() { return g_ordered_sums.load(); }
void SetSampleAlgo(int64_t algo) {
  TORCH_CHECK(algo == GS_SAMPLE_AUTO || algo == GS_SAMPLE_RESERVOIR, "unknown sampling algorithm ", algo);
  g_algo.store(algo);
}

namespace {
// values[at] of a device int64 array, through a mailbox: a one-thread kernel behind the producer
// posts it and the host spins on pinned memory, instead of a copy to pageable memory and a
// stream synchronisation
int64_t ReadTotal(const torch::Tensor& values, int64_t at, void* stream, const char* what) {
  HostBoxes& boxes = Boxes(values.get_device());
  const int64_t ticket = boxes.next++;
  Check(gs_post_total(values.data_ptr<int64_t>() + at, boxes.slot(ticket), ticket, stream), what);
  const int64_t total = WaitBox(boxes.slot(ticket), ticket, stream, what);
  return total == kLost ? values[at].item<int64_t>() : total;
}
}  // namespace

Posted PostValueSets(const std::vector<torch::Tensor>& sets, torch::Tensor& pinned) {
  Posted posted;
  if (sets.empty()) return posted;
  const int64_t n = sets[0].numel();
  const int device = sets[0].get_device();
  std::vector<const int64_t*> at(sets.size());
  for (size_t s = 0; s < sets.size(); ++s) {
    NeedI64(sets[s], "values");
    TORCH_CHECK(sets[s].numel() == n && sets[s].get_device() == device,
                "PostValueSets: the arrays must have one length and one device");
    at[s] = sets[s].data_ptr<int64_t>();
  }
  TORCH_CHECK(pinned.is_pinned() && pinned.scalar_type() == torch::kInt64 && pinned.is_contiguous() &&
                  static_cast<int64_t>(sets.size()) * n <= pinned.numel(),
              "PostValueSets: the target must be pinned int64 memory with room for the values");
  HostBoxes& boxes = Boxes(device);
  posted.ring = boxes.buf;
  posted.stream = Stream(sets[0]);
  constexpr size_t kPerLaunch = 32;  // arrays one launch of the library takes
  for (size_t first = 0; first < sets.size(); first += kPerLaunch) {
    const size_t count = std::min(kPerLaunch, sets.size() - first);
    posted.ticket = boxes.next++;
    posted.slot = boxes.slot(posted.ticket);
    Check(gs_post_value_sets(at.data() + first, static_cast<int>(count), n,
                             pinned.data_ptr<int64_t>() + static_cast<int64_t>(first) * n,
                             boxes.slot(posted.ticket), posted.ticket, posted.stream),
          "gs_post_value_sets");
  }
  return posted;
}

void WaitPosted(const Posted& posted) {
  if (!posted.slot) return;
  // (the slot went to a later call: wait for the stream instead)
  if (WaitBox(static_cast<const gs_mailbox*>(posted.slot), posted.ticket, posted.stream,
              "gs_post_value_sets") == kLost)
    TORCH_CHECK(hipStreamSynchronize(static_cast<hipStream_t>(posted.stream)) == hipSuccess,
                "gs_post_value_sets: the stream failed");
}

SliceResult ColSlicing(const torch::Tensor& indptr, const torch::Tensor& indices,
                       const torch::Tensor& column_ids, bool with_coo, bool with_select,
                       const EdgeData* edge, torch::Tensor* data_out) {
  NeedI64(indptr, "indptr");
  const int idb = IdBytes(indices, "indices");
  TORCH_CHECK(IdBytes(column_ids, "column ids") == idb, "column ids and indices differ in dtype");
  const int64_t S = column_ids.numel();
  auto sub_indptr = torch::empty({S + 1}, I64(indptr));
  auto ws = Scratch(gs_slice_workspace_bytes(S), indptr);
  void* st = Stream(indptr);
  Check(gs_slice_count(indptr.data_ptr<int64_t>(), indptr.numel() - 1, column_ids.data_ptr(), idb, S,
                       sub_indptr.data_ptr<int64_t>(), ws.data_ptr(), ws.numel(), st),
        "gs_slice_count");
  const int64_t nnz = ReadTotal(sub_indptr, S, st, "gs_slice_count");
  auto sub_indices = torch::empty({nnz}, indices.options());
  torch::Tensor select_index;
  if (with_select) select_index = torch::empty({nnz}, I64(indptr));
  torch::Tensor coo_col;
  if (with_coo) coo_col = torch::empty({nnz}, indices.options());
  const bool with_data = edge != nullptr && data_out != nullptr;
  if (with_data) *data_out = torch::empty({nnz}, edge->data.options());
  Check(gs_slice_fill_data(
            indptr.data_ptr<int64_t>(), indptr.numel() - 1, indices.data_ptr(), column_ids.data_ptr(),
            idb, S, sub_indptr.data_ptr<int64_t>(), nnz, sub_indices.data_ptr(),
            with_select ? select_index.data_ptr<int64_t>() : nullptr,
            with_coo ? coo_col.data_ptr() : nullptr,
            with_data ? edge->data.data_ptr<float>() : nullptr,
            with_data && edge->e_ids.has_value() ? edge->e_ids.value().data_ptr<int64_t>() : nullptr,
            with_data ? data_out->data_ptr<float>() : nullptr, st),
        "gs_slice_fill");
  return {sub_indptr, coo_col, sub_indices, select_index};
}

namespace {

// shared by uniform and weighted sampling: offsets, upper-bound buffers, narrow
template <typename Fill>
SliceResult SampleInto(const torch::Tensor& indptr, const torch::Tensor& indices,
                       const torch::Tensor& column_ids, int64_t fanout, bool replace, bool with_coo,
                       size_t extra_ws, Fill fill) {
  NeedI64(indptr, "indptr");
  const int idb = IdBytes(indices, "indices");
  const bool fused = column_ids.defined();
  if (fused)
    TORCH_CHECK(IdBytes(column_ids, "column ids") == idb, "column ids and indices differ in dtype");
  TORCH_CHECK(fanout >= 0, "fanout must be non-negative");
  const int64_t S = fused ? column_ids.numel() : indptr.numel() - 1;
  auto sub_indptr = torch::empty({S + 1}, I64(indptr));
  const int64_t cap = S * fanout;
  auto sub_indices = torch::empty({cap}, indices.options());
  auto select_index = torch::empty({cap}, I64(indptr));
  torch::Tensor coo_col;
  if (with_coo) coo_col = torch::empty({cap}, indices.options());
  size_t bytes = gs_sample_workspace_bytes(S, fanout);
  if (extra_ws > bytes) bytes = extra_ws;
  auto ws = Scratch(bytes, indptr);
  void* st = Stream(indptr);
  const void* cols = fused ? column_ids.data_ptr() : nullptr;
  Check(gs_sample_count(indptr.data_ptr<int64_t>(), indptr.numel() - 1, cols, idb, S, fanout, replace ? 1 : 0,
                        sub_indptr.data_ptr<int64_t>(), ws.data_ptr(), ws.numel(), st),
        "gs_sample_count");
  fill(cols, idb, S, sub_indptr, sub_indices, select_index, coo_col, ws, st);
  const int64_t nnz = ReadTotal(sub_indptr, S, Stream(sub_indptr), "total");  // the only host read of the call
  if (with_coo) coo_col = coo_col.narrow(0, 0, nnz);
  return {sub_indptr, coo_col, sub_indices.narrow(0, 0, nnz), select_index.narrow(0, 0, nnz)};
}

}  // namespace

namespace {
inline size_t Pad256(size_t n) { return (n + 255) / 256 * 256; }

// `count` elements of `type` starting `byte_offset` bytes into the 1-d byte tensor `base`, as
// a tensor that shares its storage: what base.narrow(...).view(type) gives, made directly (two
// trips through the operator dispatcher per output are a tenth of a minibatch's host time)
torch::Tensor Window(const torch::Tensor& base, size_t byte_offset, int64_t count,
                     c10::ScalarType type) {
  const auto meta = c10::scalarTypeToTypeMeta(type);
  auto t = at::detail::make_tensor<c10::TensorImpl>(c10::Storage(base.storage()), base.key_set(),
                                                    meta);
  auto* impl = t.unsafeGetTensorImpl();
  const size_t at_byte = static_cast<size_t>(base.storage_offset()) * base.element_size() + byte_offset;
  TORCH_CHECK(at_byte % meta.itemsize() == 0, "Window: misaligned for the element type");
  TORCH_CHECK(count >= 0 && byte_offset + static_cast<size_t>(count) * meta.itemsize() <= base.nbytes(),
              "Window: ", count, " elements at byte ", byte_offset, " do not fit the buffer");
  impl->set_storage_offset(static_cast<int64_t>(at_byte / meta.itemsize()));
  impl->set_sizes_contiguous({count});
  return t;
}

// One allocation cut into 256-byte aligned pieces: the outputs and the scratch of a call that
// would otherwise ask the allocator five times.
struct Pieces {
  size_t bytes = 0;
  size_t Add(size_t n) {
    const size_t at = bytes;
    bytes += Pad256(n > 0 ? n : 1);
    return at;
  }
};
}  // namespace

torch::Tensor Slice1d(const torch::Tensor& t, int64_t first, int64_t count) {
  TORCH_CHECK(t.dim() == 1 && t.is_contiguous() && first >= 0 && count >= 0 &&
                  first + count <= t.numel(),
              "Slice1d: [", first, ", ", first + count, ") of a 1-d tensor of ", t.numel());
  auto v = at::detail::make_tensor<c10::TensorImpl>(c10::Storage(t.storage()), t.key_set(), t.dtype());
  auto* impl = v.unsafeGetTensorImpl();
  impl->set_storage_offset(t.storage_offset() + first);
  impl->set_sizes_contiguous({count});
  return v;
}

int64_t PendingSample::Wait() const {
  int64_t nnz = WaitBox(static_cast<const gs_mailbox*>(box), ticket, stream, "gs_sample_uniform_fused");
  if (nnz == kLost) nnz = sub_indptr[S].item<int64_t>();
  if (nnz < 0) GaveUp(state_owner, stream, "gs_sample_uniform_fused");
  return nnz;
}

void SetDeferredSampling(bool on) { g_deferred.store(on); }
bool DeferredSampling() { return g_deferred.load(); }

bool OneLaunchApplies(int64_t S, int64_t fanout, bool replace) {
  // One launch beats the count / fill pair at every size measured (4x at 45k columns, 2x at
  // 4M); the bound only keeps the status array of the chained scan (8 bytes per 256 columns)
  // to a couple of megabytes.
  return g_algo.load() == GS_SAMPLE_AUTO && S <= kOneLaunchMaxColumns &&
         (replace || fanout <= GS_FUSED_MAX_FANOUT);
}

bool EdgeData::Fits(const torch::Tensor& data, const torch::optional<torch::Tensor>& e_ids) {
  if (!data.defined() || !data.is_cuda() || data.dim() != 1 || !data.is_contiguous() ||
      data.scalar_type() != torch::kFloat32)
    return false;
  if (e_ids.has_value() && e_ids.value().defined()) {
    const torch::Tensor& e = e_ids.value();
    if (!e.is_cuda() || e.dim() != 1 || !e.is_contiguous() || e.scalar_type() != torch::kInt64)
      return false;
  }
  return true;
}

// One launch, no host read: the total is posted to a mailbox and collected by Wait().
std::shared_ptr<PendingSample> ColSamplingDeferred(const torch::Tensor& indptr,
                                                   const torch::Tensor& indices,
                                                   const torch::Tensor& column_ids, int64_t fanout,
                                                   bool replace, bool with_coo, bool with_select,
                                                   const EdgeData* edge) {
  NeedI64(indptr, "indptr");
  const int idb = IdBytes(indices, "indices");
  const bool fused = column_ids.defined();
  if (fused)
    TORCH_CHECK(IdBytes(column_ids, "column ids") == idb, "column ids and indices differ in dtype");
  TORCH_CHECK(fanout >= 0, "fanout must be non-negative");
  auto p = std::make_shared<PendingSample>();
  p->S = fused ? column_ids.numel() : indptr.numel() - 1;
  const int64_t cap = p->S * fanout;
  {
    Pieces at;
    const size_t o_ptr = at.Add(static_cast<size_t>(p->S + 1) * 8);
    const size_t o_idx = at.Add(static_cast<size_t>(cap) * idb);
    const size_t o_sel = with_select ? at.Add(static_cast<size_t>(cap) * 8) : 0;
    const size_t o_coo = with_coo ? at.Add(static_cast<size_t>(cap) * idb) : 0;
    const size_t o_data = edge ? at.Add(static_cast<size_t>(cap) * 4) : 0;
    auto buf = Scratch(at.bytes, indptr);
    p->sub_indptr = Window(buf, o_ptr, p->S + 1, torch::kInt64);
    p->indices = Window(buf, o_idx, cap, indices.scalar_type());
    if (with_select) p->select_index = Window(buf, o_sel, cap, torch::kInt64);
    if (with_coo) p->coo_col = Window(buf, o_coo, cap, indices.scalar_type());
    if (edge) p->data = Window(buf, o_data, cap, torch::kFloat32);
  }
  if (edge) TORCH_CHECK(EdgeData::Fits(edge->data, edge->e_ids), "edge data the sampler cannot read");
  p->stream = Stream(indptr);
  p->device = indptr.device().index();
  FusedStateBuf& state = FusedState(gs_sample_fused_state_bytes(p->S), indptr, p->stream);
  HostBoxes& boxes = Boxes(p->device);
  p->ticket = boxes.next++;
  p->box = boxes.slot(p->ticket);
  p->box_owner = boxes.buf;
  p->state_owner = state.buf;
  Check(gs_sample_uniform_fused_data(
            indptr.data_ptr<int64_t>(), indptr.numel() - 1, EdgeArray(indices, indptr),
            fused ? column_ids.data_ptr() : nullptr, idb, p->S, fanout, replace ? 1 : 0, NextSeed(),
            nullptr, nullptr, p->sub_indptr.data_ptr<int64_t>(), p->indices.data_ptr(),
            with_select ? p->select_index.data_ptr<int64_t>() : nullptr,
            with_coo ? p->coo_col.data_ptr() : nullptr, cap,
            edge ? static_cast<const float*>(EdgeArray(edge->data, indptr)) : nullptr,
            edge ? OptI64(edge->e_ids, "e_ids") : nullptr,
            edge ? p->data.data_ptr<float>() : nullptr, state.buf.data_ptr(), state.buf.numel(),
            state.epoch, boxes.slot(p->ticket), p->ticket, p->stream),
        "gs_sample_uniform_fused");
  return p;
}

namespace {

SliceResult ColSamplingOneLaunch(const torch::Tensor& indptr, const torch::Tensor& indices,
                                 const torch::Tensor& column_ids, int64_t fanout, bool replace,
                                 bool with_coo) {
  auto p = ColSamplingDeferred(indptr, indices, column_ids, fanout, replace, with_coo, true);
  const int64_t nnz = p->Wait();
  torch::Tensor coo_col;
  if (with_coo) coo_col = p->coo_col.narrow(0, 0, nnz);
  return {p->sub_indptr, coo_col, p->indices.narrow(0, 0, nnz), p->select_index.narrow(0, 0, nnz)};
}

}  // namespace

SliceResult ColSampling(const torch::Tensor& indptr, const torch::Tensor& indices,
                        const torch::Tensor& column_ids, int64_t fanout, bool replace,
                        bool with_coo) {
  TORCH_CHECK(fanout >= 0, "fanout must be non-negative");
  const int64_t S = column_ids.defined() ? column_ids.numel() : indptr.numel() - 1;
  if (OneLaunchApplies(S, fanout, replace))
    return ColSamplingOneLaunch(indptr, indices, column_ids, fanout, replace, with_coo);
  return SampleInto(
      indptr, indices, column_ids, fanout, replace, with_coo, 0,
      [&](const void* cols, int idb, int64_t S, torch::Tensor& sub_indptr, torch::Tensor& sub_indices,
          torch::Tensor& select_index, torch::Tensor& coo_col, torch::Tensor& ws, void* st) {
        Check(gs_sample_uniform_fill(indptr.data_ptr<int64_t>(), indptr.numel() - 1, EdgeArray(indices, indptr), cols, idb, S,
                                     fanout, replace ? 1 : 0, static_cast<int>(g_algo.load()),
                                     NextSeed(), nullptr, nullptr, sub_indptr.data_ptr<int64_t>(),
                                     sub_indices.data_ptr(), select_index.data_ptr<int64_t>(),
                                     with_coo ? coo_col.data_ptr() : nullptr, ws.data_ptr(),
                                     ws.numel(), st),
              "gs_sample_uniform_fill");
      });
}

SliceResult ColSamplingProbs(const torch::Tensor& indptr, const torch::Tensor& indices,
                             const torch::Tensor& probs, const torch::Tensor& column_ids,
                             int64_t fanout, bool replace, bool with_coo) {
  NeedF32(probs, "edge_probs");
  const int64_t S = column_ids.defined() ? column_ids.numel() : indptr.numel() - 1;
  if (replace) {
    // inverse-CDF picks; the prefix sums of every column live in a scratch laid out like
    // the edges themselves (the offsets of the input, or of the column slice)
    torch::Tensor cdf_ptr = indptr;
    int64_t cdf_len = indices.numel();
    if (column_ids.defined()) {
      NeedI64(indptr, "indptr");
      cdf_ptr = torch::empty({S + 1}, I64(indptr));
      auto sws = Scratch(gs_slice_workspace_bytes(S), indptr);
      Check(gs_slice_count(indptr.data_ptr<int64_t>(), indptr.numel() - 1, column_ids.data_ptr(),
                           IdBytes(column_ids, "column ids"), S, cdf_ptr.data_ptr<int64_t>(),
                           sws.data_ptr(), sws.numel(), Stream(indptr)),
            "gs_slice_count");
      cdf_len = ReadTotal(cdf_ptr, S, Stream(cdf_ptr), "total");
    }
    auto cdf = torch::empty({cdf_len > 0 ? cdf_len : 1}, probs.options());
    return SampleInto(
        indptr, indices, column_ids, fanout, true, with_coo, 0,
        [&](const void* cols, int idb, int64_t S_, torch::Tensor& sub_indptr,
            torch::Tensor& sub_indices, torch::Tensor& select_index, torch::Tensor& coo_col,
            torch::Tensor&, void* st) {
          Check(gs_sample_weighted_replace(
                    indptr.data_ptr<int64_t>(), indptr.numel() - 1, EdgeArray(indices, indptr),
                    static_cast<const float*>(EdgeArray(probs, indptr)), cols, idb, S_, fanout, NextSeed(), nullptr,
                    sub_indptr.data_ptr<int64_t>(), cdf_ptr.data_ptr<int64_t>(),
                    cdf.data_ptr<float>(), sub_indices.data_ptr(),
                    select_index.data_ptr<int64_t>(), with_coo ? coo_col.data_ptr() : nullptr, st),
                "gs_sample_weighted_replace");
        });
  }
  return SampleInto(
      indptr, indices, column_ids, fanout, false, with_coo,
      gs_sample_weighted_workspace_bytes(S, fanout),
      [&](const void* cols, int idb, int64_t S_, torch::Tensor& sub_indptr,
          torch::Tensor& sub_indices, torch::Tensor& select_index, torch::Tensor& coo_col,
          torch::Tensor& ws, void* st) {
        Check(gs_sample_weighted_fill(indptr.data_ptr<int64_t>(), indptr.numel() - 1, EdgeArray(indices, indptr),
                                      static_cast<const float*>(EdgeArray(probs, indptr)), cols, idb, S_, fanout, NextSeed(),
                                      nullptr, nullptr, sub_indptr.data_ptr<int64_t>(),
                                      sub_indices.data_ptr(), select_index.data_ptr<int64_t>(),
                                      with_coo ? coo_col.data_ptr() : nullptr, ws.data_ptr(),
                                      ws.numel(), st),
              "gs_sample_weighted_fill");
      });
}

std::tuple<torch::Tensor, torch::Tensor, torch::Tensor> SampleOneKeepDim(
    const torch::Tensor& indptr, const torch::Tensor& indices, const torch::Tensor& column_ids) {
  NeedI64(indptr, "indptr");
  const int idb = IdBytes(indices, "indices");
  TORCH_CHECK(IdBytes(column_ids, "column ids") == idb, "column ids and indices differ in dtype");
  const int64_t S = column_ids.numel();
  auto sub_indptr = torch::empty({S + 1}, I64(indptr));
  auto sub_indices = torch::empty({S}, indices.options());
  auto select_index = torch::empty({S}, I64(indptr));
  Check(gs_sample_one_keepdim(indptr.data_ptr<int64_t>(), indptr.numel() - 1, EdgeArray(indices, indptr), column_ids.data_ptr(),
                              idb, S, NextSeed(), nullptr, sub_indptr.data_ptr<int64_t>(),
                              sub_indices.data_ptr(), select_index.data_ptr<int64_t>(),
                              Stream(indptr)),
        "gs_sample_one_keepdim");
  return {sub_indptr, sub_indices, select_index};
}

std::tuple<torch::Tensor, std::vector<torch::Tensor>> Relabel(
    const std::vector<torch::Tensor>& mapping, const std::vector<torch::Tensor>& queries) {
  TORCH_CHECK(!mapping.empty() && mapping.size() <= GS_MAX_SPANS && queries.size() <= GS_MAX_SPANS,
              "relabel takes 1..", GS_MAX_SPANS, " mapping tensors and at most ", GS_MAX_SPANS,
              " tensors to relabel");
  const int idb = IdBytes(mapping[0], "mapping tensor");
  gs_span m[GS_MAX_SPANS], q[GS_MAX_SPANS];
  void* out_ptr[GS_MAX_SPANS];
  int64_t M = 0;
  for (size_t i = 0; i < mapping.size(); ++i) {
    TORCH_CHECK(IdBytes(mapping[i], "mapping tensor") == idb, "relabel tensors differ in dtype");
    m[i] = {mapping[i].data_ptr(), mapping[i].numel()};
    M += mapping[i].numel();
  }
  std::vector<torch::Tensor> outs;
  for (size_t i = 0; i < queries.size(); ++i) {
    TORCH_CHECK(IdBytes(queries[i], "tensor to relabel") == idb, "relabel tensors differ in dtype");
    q[i] = {queries[i].data_ptr(), queries[i].numel()};
    outs.push_back(torch::empty_like(queries[i]));
    out_ptr[i] = outs.back().data_ptr();
  }
  auto frontier = torch::empty({M}, mapping[0].options());
  auto num = torch::empty({1}, I64(mapping[0]));
  auto ws = Scratch(gs_unique_workspace_bytes(M), mapping[0]);
  void* st = Stream(mapping[0]);
  HostBoxes& boxes = Boxes(mapping[0].device().index());
  int64_t U = kTooWide;
  for (int attempt = 0; attempt < 2 && U == kTooWide; ++attempt) {
    const int64_t ticket = boxes.next++;
    Check(gs_unique_relabel_notify(m, static_cast<int>(mapping.size()), q, out_ptr,
                                   static_cast<int>(queries.size()), TableIds(idb),
                                   frontier.data_ptr(), num.data_ptr<int64_t>(), ws.data_ptr(),
                                   ws.numel(), nullptr, boxes.slot(ticket), ticket, st),
          "gs_unique_relabel");
    U = WaitBox(boxes.slot(ticket), ticket, st, "gs_unique_relabel");
    if (U == kLost) U = num.item<int64_t>();
    if (U == kTooWide) t_narrow_ids = false;
  }
  TORCH_CHECK(U >= 0, "gs_unique_relabel: a tile gave up waiting for its predecessors");
  return {frontier.narrow(0, 0, U), outs};
}

// Relabel of (column ids, sampled ids) while the sampler's total is still on the
// device: everything is sized for the sampler's capacity, the kernels read the
// true length from sub_indptr[S], and both totals are collected at the end.
std::tuple<torch::Tensor, torch::Tensor, int64_t, torch::Tensor> RelabelDeferred(
    const torch::Tensor& col_ids, const PendingSample& p) {
  const int idb = IdBytes(col_ids, "column ids");
  TORCH_CHECK(IdBytes(p.indices, "sampled ids") == idb, "relabel tensors differ in dtype");
  const int64_t cap = p.indices.numel();
  const int64_t S = col_ids.numel();
  const int64_t M = S + cap;
  Pieces at;
  const size_t o_renamed = at.Add(static_cast<size_t>(cap) * idb);
  const size_t o_frontier = at.Add(static_cast<size_t>(M) * idb);
  const size_t o_num = at.Add(8);
  const size_t o_offsets = at.Add(static_cast<size_t>(p.sub_indptr.numel()) * 8);
  const size_t ws_bytes = gs_relabel_sampled_workspace_bytes(M);
  const size_t o_ws = at.Add(ws_bytes);
  auto buf = Scratch(at.bytes, col_ids);
  const auto id_type = col_ids.scalar_type();
  auto renamed = Window(buf, o_renamed, cap, id_type);
  auto frontier = Window(buf, o_frontier, M, id_type);
  auto num = Window(buf, o_num, 1, torch::kInt64);
  auto offsets_copy = Window(buf, o_offsets, p.sub_indptr.numel(), torch::kInt64);
  auto ws = Window(buf, o_ws, static_cast<int64_t>(ws_bytes), torch::kUInt8);
  RelabelTable& table = RelabelTableFor(col_ids, p.stream, idb, M);
  FusedStateBuf& state = FusedState(gs_relabel_sampled_state_bytes(M), col_ids, p.stream);
  HostBoxes& boxes = Boxes(p.device);
  int64_t nnz = -1, U = kTooWide;
  for (int attempt = 0; attempt < 2 && U == kTooWide; ++attempt) {
    const int64_t ticket = boxes.next++;
    table.clean = false;  // until both totals have come back
    if (idb == 8 && table.narrow) {
      Check(gs_relabel_sampled_narrow(col_ids.data_ptr(), S, p.indices.data_ptr(), cap,
                                      p.sub_indptr.data_ptr<int64_t>() + p.S, table.buf.data_ptr(),
                                      table.buf.numel(), frontier.data_ptr(), renamed.data_ptr(),
                                      num.data_ptr<int64_t>(), offsets_copy.data_ptr<int64_t>(),
                                      ws.data_ptr(), ws.numel(), state.buf.data_ptr(),
                                      state.buf.numel(), state.epoch, boxes.slot(ticket), ticket,
                                      p.stream),
            "gs_relabel_sampled_narrow");
    } else {
      Check(gs_relabel_sampled(col_ids.data_ptr(), S, p.indices.data_ptr(), cap,
                               p.sub_indptr.data_ptr<int64_t>() + p.S, idb, table.buf.data_ptr(),
                               table.buf.numel(), frontier.data_ptr(), renamed.data_ptr(),
                               num.data_ptr<int64_t>(), offsets_copy.data_ptr<int64_t>(),
                               ws.data_ptr(), ws.numel(), state.buf.data_ptr(), state.buf.numel(),
                               state.epoch, boxes.slot(ticket), ticket, p.stream),
            "gs_relabel_sampled");
    }
    if (nnz < 0) nnz = p.Wait();
    U = WaitBox(boxes.slot(ticket), ticket, p.stream, "gs_relabel_sampled");
    if (U == kLost) U = num.item<int64_t>();
    if (U == kTooWide) {
      // an id beyond 32 bits: from now on this table takes the two-array slots
      TORCH_CHECK(idb == 8 && table.narrow, "gs_relabel_sampled: unexpected status");
      table.narrow = false;
      // the error word is sticky: clear the state on the stream the kernels run on
      TORCH_CHECK(hipMemsetAsync(state.buf.data_ptr(), 0, state.buf.numel(),
                                 static_cast<hipStream_t>(p.stream)) == hipSuccess,
                  "hipMemsetAsync failed");
      RelabelTableFor(col_ids, p.stream, idb, M);                               // prepares it again
      FusedState(gs_relabel_sampled_state_bytes(M), col_ids, p.stream);       // next epoch
    }
  }
  if (U < 0) GaveUp(state.buf, p.stream, "gs_relabel_sampled");  // (the table stays marked)
  table.clean = true;
  return {Window(buf, o_frontier, U, id_type), Window(buf, o_renamed, nnz, id_type), nnz,
          offsets_copy};
}


// ---- a whole minibatch queued with no host read -------------------------------------
namespace {

// 64-bit ids ride on the chain's one-word table slots until this thread meets one that
// does not fit 32 bits; from then on its minibatches go layer by layer.
thread_local bool t_chain_ids_fit = true;
// the chain's launches and tables are sized for the bounds S * prod(1 + fanout); beyond this
// many items per layer the layer-by-layer path, which sizes by what was sampled, is used
constexpr int64_t kChainMaxItems = int64_t(1) << 24;  // (8192 seeds x [15, 10, 5] is 8.65 M)

// the two tables a chain uses in turn (a layer's relabel empties the table of the layer
// before it), one pair per (thread, device, stream); a chain in flight holds on to its pair
struct ChainTables {
  torch::Tensor buf[2];
  int64_t items = 0;
  bool clean = false;
};

std::shared_ptr<ChainTables> ChainTablesFor(const torch::Tensor& like, void* stream,
                                            int64_t items) {
  thread_local std::map<std::pair<int, void*>, std::shared_ptr<ChainTables>> tables;
  std::shared_ptr<ChainTables>& t = tables[{like.device().index(), stream}];
  if (!t) t = std::make_shared<ChainTables>();
  if (!t->buf[0].defined() || t->items < items) {
    int64_t want = 1 << 16;
    while (want < items) want <<= 1;
    for (auto& b : t->buf)
      b = torch::empty({static_cast<int64_t>(gs_relabel_table_bytes(want, 4))},
                       torch::dtype(torch::kUInt8).device(like.device()));
    t->items = want;
    t->clean = false;
  }
  if (!t->clean) {
    for (auto& b : t->buf)
      Check(gs_relabel_table_init(b.data_ptr(), b.numel(), 4, stream), "gs_relabel_table_init");
    t->clean = true;
  }
  return t;
}

}  // namespace

void DebugRaiseLookbackError(const torch::Tensor& like) {
  FusedStateBuf& s = FusedState(65536, like, Stream(like));
  // the error word is the first word of the state (carve_lookback)
  s.buf.narrow(0, 0, 4).view(torch::kInt32).fill_(1);
}

SeedState SaveSeedState() { return {t_own_seed, t_seed}; }
void RestoreSeedState(const SeedState& s) {
  t_own_seed = s.own;
  t_seed = s.seed;
}

bool LayerChainApplies(int64_t num_seeds, const std::vector<int64_t>& fanouts, bool replace) {
  if (g_algo.load() != GS_SAMPLE_AUTO || !t_chain_ids_fit || fanouts.empty()) return false;
  int64_t bound = num_seeds;
  for (int64_t k : fanouts) {
    if (k < 0 || (!replace && k > GS_FUSED_MAX_FANOUT)) return false;
    if (bound > kChainMaxItems / (1 + k)) return false;
    bound *= 1 + k;
  }
  return true;
}

std::shared_ptr<PendingLayers> SampleLayersQueued(const torch::Tensor& indptr,
                                                  const torch::Tensor& indices,
                                                  const torch::Tensor& seeds,
                                                  const std::vector<int64_t>& fanouts,
                                                  bool replace, const EdgeData* edge) {
  NeedI64(indptr, "indptr");
  const int idb = IdBytes(indices, "indices");
  TORCH_CHECK(IdBytes(seeds, "seeds") == idb, "seeds and indices differ in dtype");
  if (edge) TORCH_CHECK(EdgeData::Fits(edge->data, edge->e_ids), "edge data the sampler cannot read");
  const float* edge_data = edge ? static_cast<const float*>(EdgeArray(edge->data, indptr)) : nullptr;
  const int64_t* edge_ids = edge ? OptI64(edge->e_ids, "e_ids") : nullptr;
  const int64_t L = static_cast<int64_t>(fanouts.size());
  TORCH_CHECK(LayerChainApplies(seeds.numel(), fanouts, replace),
              "SampleLayersQueued: this minibatch has to go layer by layer");
  auto p = std::make_shared<PendingLayers>();
  p->layers.resize(L);
  p->stream = Stream(indptr);
  p->device = indptr.device().index();
  p->num_seeds = seeds.numel();
  // bounds: S_0 = #seeds, capacity_l = S_l * fanout_l, S_{l+1} = S_l + capacity_l
  std::vector<int64_t> S(L + 1);
  S[0] = seeds.numel();
  for (int64_t l = 0; l < L; ++l) S[l + 1] = S[l] * (1 + fanouts[l]);
  // ONE allocation for the whole minibatch, made before the first launch: per layer the
  // three outputs at their bounds (offsets, renamed ids, frontier) and what no caller sees (the
  // sampled ids before renaming, the items' table slots, the two counts).  The output tensors
  // are cut out of it after the last launch, while the device is already at work.
  std::vector<size_t> off_ids(L), off_ws(L), ws_bytes(L), off_counts(L), off_offsets(L),
      off_renamed(L), off_frontier(L), off_data(L);
  size_t bytes = 0, state_bytes = 0;
  for (int64_t l = 0; l < L; ++l) {
    const size_t cap = static_cast<size_t>(S[l] * fanouts[l]);
    off_offsets[l] = bytes;
    bytes += Pad256(static_cast<size_t>(S[l] + 1) * 8);
    off_renamed[l] = bytes;
    bytes += Pad256(cap * idb);
    off_frontier[l] = bytes;
    bytes += Pad256((static_cast<size_t>(S[l]) + cap) * idb);
    off_ids[l] = bytes;
    bytes += Pad256(cap * idb);
    off_data[l] = bytes;
    if (edge) bytes += Pad256(cap * 4);
    ws_bytes[l] = gs_layer_workspace_bytes(S[l], fanouts[l]);
    off_ws[l] = bytes;
    bytes += Pad256(ws_bytes[l]);
    off_counts[l] = bytes;
    bytes += 256;
    state_bytes = std::max(state_bytes, std::max(gs_layer_sample_state_bytes(S[l]),
                                                 gs_layer_relabel_state_bytes(S[l], fanouts[l])));
  }
  p->scratch = Scratch(bytes, indptr);
  char* base = static_cast<char*>(p->scratch.data_ptr());
  auto tables = ChainTablesFor(indptr, p->stream, S[L]);
  p->tables = tables;
  HostBoxes& boxes = Boxes(p->device);
  p->box_owner = boxes.buf;
  p->ring = boxes.ring;
  const void* cols = seeds.data_ptr();
  const int64_t* S_dev = nullptr;
  for (int64_t l = 0; l < L; ++l) {
    PendingLayers::Layer& y = p->layers[l];
    const int64_t cap = S[l] * fanouts[l];
    int64_t* offsets = reinterpret_cast<int64_t*>(base + off_offsets[l]);
    void* frontier = base + off_frontier[l];
    int64_t* counts = reinterpret_cast<int64_t*>(base + off_counts[l]);
    void* table = tables->buf[l & 1].data_ptr();
    const size_t table_bytes = tables->buf[l & 1].numel();
    const uint64_t seed = NextSeed();
    if (l == 0) p->first_seed = seed;
    FusedStateBuf& st1 = FusedState(state_bytes, indptr, p->stream);
    if (l == 0) p->state_owner = st1.buf;
    y.ticket_edges = boxes.next++;
    Check(gs_layer_sample(indptr.data_ptr<int64_t>(), indptr.numel() - 1, EdgeArray(indices, indptr), cols,
                          idb, S[l], S_dev, fanouts[l], replace ? 1 : 0, seed, nullptr, nullptr,
                          offsets, base + off_ids[l], cap, counts, nullptr, edge_data, edge_ids,
                          edge ? reinterpret_cast<float*>(base + off_data[l]) : nullptr, table,
                          table_bytes, base + off_ws[l], ws_bytes[l], st1.buf.data_ptr(),
                          st1.buf.numel(), st1.epoch, boxes.slot(y.ticket_edges), y.ticket_edges,
                          p->stream),
          "gs_layer_sample");
    FusedStateBuf& st2 = FusedState(state_bytes, indptr, p->stream);
    y.ticket_unique = boxes.next++;
    const bool has_prev = l > 0;
    Check(gs_layer_relabel(
              idb, S[l], S_dev, cap, counts, offsets, table, table_bytes, base + off_ws[l],
              ws_bytes[l], frontier, base + off_renamed[l], counts + 1, nullptr, st2.buf.data_ptr(), st2.buf.numel(), st2.epoch,
              has_prev ? tables->buf[(l - 1) & 1].data_ptr() : nullptr,
              has_prev ? static_cast<size_t>(tables->buf[(l - 1) & 1].numel()) : 0,
              has_prev ? base + off_ws[l - 1] : nullptr, has_prev ? ws_bytes[l - 1] : 0,
              has_prev ? S[l - 1] : 0,
              l >= 2 ? reinterpret_cast<int64_t*>(base + off_counts[l - 2]) + 1 : nullptr,
              has_prev ? S[l - 1] * fanouts[l - 1] : 0,
              has_prev ? reinterpret_cast<int64_t*>(base + off_counts[l - 1]) : nullptr,
              boxes.slot(y.ticket_unique), y.ticket_unique, p->stream),
          "gs_layer_relabel");
    cols = frontier;
    S_dev = counts + 1;
  }
  // the last layer's table has no later relabel to empty it
  Check(gs_layer_table_sweep(
            tables->buf[(L - 1) & 1].data_ptr(), tables->buf[(L - 1) & 1].numel(),
            base + off_ws[L - 1], ws_bytes[L - 1], S[L - 1],
            L >= 2 ? reinterpret_cast<int64_t*>(base + off_counts[L - 2]) + 1 : nullptr,
            S[L - 1] * fanouts[L - 1], reinterpret_cast<int64_t*>(base + off_counts[L - 1]),
            p->stream),
        "gs_layer_table_sweep");
  p->id_type = indices.scalar_type();
  p->with_data = edge != nullptr;
  for (int64_t l = 0; l < L; ++l) {
    p->layers[l].off_data = off_data[l];
    p->layers[l].off_offsets = off_offsets[l];
    p->layers[l].off_renamed = off_renamed[l];
    p->layers[l].off_frontier = off_frontier[l];
  }
  return p;
}

std::vector<torch::Tensor> PendingLayers::Collect() {
  const gs_mailbox* boxes = static_cast<const gs_mailbox*>(ring);
  std::vector<torch::Tensor> out;
  out.reserve(4 * layers.size());
  int64_t S = num_seeds;
  int64_t worst = 0;
  std::vector<int64_t> E(layers.size()), U(layers.size());
  // the last count first: once it is here every earlier one is
  for (size_t l = layers.size(); l-- > 0;) {
    U[l] = WaitBox(boxes + layers[l].ticket_unique % kBoxes, layers[l].ticket_unique, stream,
                   "gs_layer_relabel");
    E[l] = WaitBox(boxes + layers[l].ticket_edges % kBoxes, layers[l].ticket_edges, stream,
                   "gs_layer_sample");
    TORCH_CHECK(U[l] != kLost && E[l] != kLost,
                "more minibatches in flight than the ring of result mailboxes holds");
    worst = std::min(worst, U[l]);
  }
  if (worst < 0) {
    // an id beyond 32 bits (-2) or a tile that gave up (-1): either way the tables hold
    // leftovers and the look-back state a raised error word
    auto t = std::static_pointer_cast<ChainTables>(tables);
    if (t) t->clean = false;
    if (worst == kTooWide) {
      if (state_owner.defined())
        (void)hipMemsetAsync(state_owner.data_ptr(), 0, static_cast<size_t>(state_owner.numel()),
                             static_cast<hipStream_t>(stream));
      t_chain_ids_fit = false;
      throw IdsTooWide();
    }
    GaveUp(state_owner, stream, "gs_layer_relabel");
  }
  for (size_t l = 0; l < layers.size(); ++l) {
    out.push_back(Window(scratch, layers[l].off_frontier, U[l], id_type));
    out.push_back(Window(scratch, layers[l].off_offsets, S + 1, c10::ScalarType::Long));
    out.push_back(Window(scratch, layers[l].off_renamed, E[l], id_type));
    if (with_data) out.push_back(Window(scratch, layers[l].off_data, E[l], c10::ScalarType::Float));
    S = U[l];
  }
  return out;
}

std::tuple<torch::Tensor, torch::Tensor, torch::Tensor> BatchCsrRelabel(
    const torch::Tensor& seeds, const torch::Tensor& seeds_ptr, const torch::Tensor& ids,
    const torch::Tensor& ids_ptr) {
  const int idb = IdBytes(seeds, "seeds");
  TORCH_CHECK(IdBytes(ids, "indices") == idb, "seeds and indices differ in dtype");
  NeedI64(seeds_ptr, "seeds_ptr");
  NeedI64(ids_ptr, "indices_ptr");
  TORCH_CHECK(seeds_ptr.numel() == ids_ptr.numel() && seeds_ptr.numel() >= 2,
              "seeds_ptr and indices_ptr must both hold num_batches + 1 offsets");
  const int64_t B = seeds_ptr.numel() - 1;
  const int64_t M = seeds.numel() + ids.numel();
  auto unique = torch::empty({M}, seeds.options());
  auto unique_ptr = torch::empty({B + 1}, I64(seeds));
  auto out_ids = torch::empty_like(ids);
  auto num = torch::empty({1}, I64(seeds));
  auto ws = Scratch(gs_batch_relabel_workspace_bytes(M), seeds);
  void* st = Stream(seeds);
  HostBoxes& boxes = Boxes(seeds.device().index());
  int64_t U = kTooWide;
  int path = 0;  // the library chooses between bins and hash regions
  for (int attempt = 0; attempt < 3 && (U == kTooWide || U == kBinsFull); ++attempt) {
    const int64_t ticket = boxes.next++;
    Check(gs_batch_csr_relabel(seeds.data_ptr(), seeds_ptr.data_ptr<int64_t>(), ids.data_ptr(),
                               ids_ptr.data_ptr<int64_t>(), B, seeds.numel(), ids.numel(),
                               TableIds(idb) | path, unique.data_ptr(),
                               unique_ptr.data_ptr<int64_t>(), out_ids.data_ptr(),
                               num.data_ptr<int64_t>(), ws.data_ptr(), ws.numel(),
                               boxes.slot(ticket), ticket, st),
          "gs_batch_csr_relabel");
    U = WaitBox(boxes.slot(ticket), ticket, st, "gs_batch_csr_relabel");
    if (U == kLost) U = num.item<int64_t>();
    if (U == kTooWide) t_narrow_ids = false;
    if (U == kBinsFull) path = GS_RELABEL_REGIONS;  // a class outgrew its LDS table
  }
  TORCH_CHECK(U >= 0, "gs_batch_csr_relabel: a tile gave up waiting for its predecessors");
  return {unique.narrow(0, 0, U), unique_ptr, out_ids};
}

std::tuple<torch::Tensor, torch::Tensor, torch::Tensor> BatchCsrRelabelQueued(
    const torch::Tensor& seeds, const torch::Tensor& seeds_ptr, const torch::Tensor& ids,
    const torch::Tensor& ids_ptr, int64_t* num_unique, const PendingSample* producer) {
  const int idb = IdBytes(seeds, "seeds");
  TORCH_CHECK(IdBytes(ids, "indices") == idb, "seeds and indices differ in dtype");
  NeedI64(seeds_ptr, "seeds_ptr");
  NeedI64(ids_ptr, "indices_ptr");
  TORCH_CHECK(seeds_ptr.numel() == ids_ptr.numel() && seeds_ptr.numel() >= 2,
              "seeds_ptr and indices_ptr must both hold num_batches + 1 offsets");
  const int64_t B = seeds_ptr.numel() - 1;
  const int64_t M = seeds.numel() + ids.numel();
  const int table_ids = TableIds(idb);
  // (below half a million items the relabel on hash regions, three launches, is the quicker one:
  // there the caller's wait for the edge count costs less than the bins' eight launches)
  if ((idb == 8 && !(table_ids & GS_NARROW_IDS)) || B > 511 || M < (int64_t(1) << 19) ||
      M >= (int64_t(1) << 30))
    return {torch::Tensor(), torch::Tensor(), torch::Tensor()};
  auto unique = torch::empty({M}, seeds.options());
  auto unique_ptr = torch::empty({B + 1}, I64(seeds));
  auto out_ids = torch::empty_like(ids);
  auto ws = Scratch(gs_batch_relabel_bins_workspace_bytes(M, B), seeds);
  void* st = Stream(seeds);
  auto num = torch::empty({1}, I64(seeds));
  HostBoxes& boxes = Boxes(seeds.device().index());
  const int64_t ticket = boxes.next++;
  Check(gs_batch_csr_relabel(seeds.data_ptr(), seeds_ptr.data_ptr<int64_t>(), ids.data_ptr(),
                             ids_ptr.data_ptr<int64_t>(), B, seeds.numel(), ids.numel(),
                             table_ids | GS_RELABEL_BINS, unique.data_ptr(),
                             unique_ptr.data_ptr<int64_t>(), out_ids.data_ptr(),
                             num.data_ptr<int64_t>(), ws.data_ptr(), ws.numel(),
                             boxes.slot(ticket), ticket, st),
        "gs_batch_csr_relabel");
  int64_t U = WaitBox(boxes.slot(ticket), ticket, st, "gs_batch_csr_relabel");
  if (U == kLost) U = num.item<int64_t>();
  if (U == kTooWide) t_narrow_ids = false;
  if (U == kGaveUp) {
    // either the sampler the ids come from failed (its last offset is negative and the relabel
    // left at once: Wait() reports it and clears the sampler's look-back state) or a tile of
    // the relabel's own scan gave up (its state lives in the workspace and is gone with it)
    if (producer) producer->Wait();
    TORCH_CHECK(false, "gs_batch_csr_relabel: a tile gave up waiting for its predecessors");
  }
  *num_unique = U;
  return {unique, unique_ptr, out_ids};
}

torch::Tensor IndptrSplit(const torch::Tensor& indptr, const torch::Tensor& offsets,
                          int64_t total, torch::Tensor* cuts) {
  NeedI64(indptr, "indptr");
  NeedI64(offsets, "offsets");
  auto out = torch::empty({total}, I64(indptr));
  if (cuts) *cuts = torch::empty({offsets.numel()}, I64(indptr));
  Check(gs_indptr_split_cuts(indptr.data_ptr<int64_t>(), offsets.data_ptr<int64_t>(),
                             offsets.numel() - 1, total, out.data_ptr<int64_t>(),
                             cuts ? cuts->data_ptr<int64_t>() : nullptr, Stream(indptr)),
        "gs_indptr_split");
  return out;
}

torch::Tensor Unique(const torch::Tensor& ids) { return std::get<0>(Relabel({ids}, {})); }

torch::Tensor RandomWalk(const torch::Tensor& seeds, int64_t length, const torch::Tensor& indptr,
                         const torch::Tensor& indices) {
  NeedI64(indptr, "indptr");
  const int idb = IdBytes(indices, "indices");
  TORCH_CHECK(IdBytes(seeds, "seeds") == idb, "seeds and indices differ in dtype");
  TORCH_CHECK(length >= 0, "walk_length must be non-negative");
  const int64_t n = seeds.numel();
  auto trace = torch::empty({n * (length + 1)}, seeds.options());
  Check(gs_random_walk(indptr.data_ptr<int64_t>(), indptr.numel() - 1, indices.data_ptr(), idb, seeds.data_ptr(), n,
                       length, NextSeed(), nullptr, trace.data_ptr(), Stream(seeds)),
        "gs_random_walk");
  return trace;
}

torch::Tensor MetapathWalk(const torch::Tensor& seeds, const torch::Tensor& metapath,
                           const torch::Tensor& indptr_table, const torch::Tensor& indices_table,
                           const torch::Tensor& num_nodes_table, int id_bytes) {
  NeedI64(num_nodes_table, "relation sizes");
  TORCH_CHECK(IdBytes(seeds, "seeds") == id_bytes, "seeds and relation graphs differ in dtype");
  NeedI64(metapath, "metapath");
  const int64_t n = seeds.numel();
  const int64_t L = metapath.numel();
  auto trace = torch::empty({n * (L + 1)}, seeds.options());
  Check(gs_metapath_walk(reinterpret_cast<const int64_t* const*>(indptr_table.data_ptr<int64_t>()),
                         reinterpret_cast<const void* const*>(indices_table.data_ptr<int64_t>()),
                         num_nodes_table.data_ptr<int64_t>(), id_bytes, metapath.data_ptr<int64_t>(), L, seeds.data_ptr(), n, NextSeed(),
                         nullptr, trace.data_ptr(), Stream(seeds)),
        "gs_metapath_walk");
  return trace;
}

void SddmmCoo(const std::string& op, const Bcast& b, const torch::Tensor& row,
              const torch::Tensor& col, const torch::optional<torch::Tensor>& e_ids,
              const torch::Tensor& lhs, const torch::Tensor& rhs, torch::Tensor out, int lhs_target,
              int rhs_target) {
  const int code = OpCode(op);
  const int idb = IdBytes(row, "coo row");
  TORCH_CHECK(IdBytes(col, "coo col") == idb, "coo row and col differ in dtype");
  NeedF32(out, "out");
  if (code != GS_OP_COPY_RHS) NeedF32(lhs, "lhs");
  if (code != GS_OP_COPY_LHS) NeedF32(rhs, "rhs");
  Check(gs_sddmm_coo(code, row.data_ptr(), col.data_ptr(), idb, OptI64(e_ids, "e_ids"),
                     row.numel(), lhs.defined() ? lhs.data_ptr<float>() : nullptr,
                     rhs.defined() ? rhs.data_ptr<float>() : nullptr, out.data_ptr<float>(),
                     lhs_target, rhs_target, b.lhs_len, b.rhs_len, b.out_len, b.reduce_size,
                     b.lhs_off.defined() ? b.lhs_off.data_ptr<int64_t>() : nullptr,
                     b.rhs_off.defined() ? b.rhs_off.data_ptr<int64_t>() : nullptr, Stream(row)),
        "gs_sddmm_coo");
}

void SddmmCsc(const std::string& op, const Bcast& b, const torch::Tensor& indptr,
              const torch::Tensor& indices, const torch::optional<torch::Tensor>& e_ids,
              const torch::optional<torch::Tensor>& nid_map, const torch::Tensor& lhs,
              const torch::Tensor& rhs, torch::Tensor out, int lhs_target, int rhs_target) {
  const int code = OpCode(op);
  NeedI64(indptr, "indptr");
  const int idb = IdBytes(indices, "indices");
  NeedF32(out, "out");
  if (code != GS_OP_COPY_RHS) NeedF32(lhs, "lhs");
  if (code != GS_OP_COPY_LHS) NeedF32(rhs, "rhs");
  Check(gs_sddmm_csc(code, indptr.data_ptr<int64_t>(), indices.data_ptr(), idb,
                     OptI64(e_ids, "e_ids"), OptIds(nid_map, idb, "valid ids"), indptr.numel() - 1,
                     indices.numel(), lhs.defined() ? lhs.data_ptr<float>() : nullptr,
                     rhs.defined() ? rhs.data_ptr<float>() : nullptr, out.data_ptr<float>(),
                     lhs_target, rhs_target, b.lhs_len, b.rhs_len, b.out_len, b.reduce_size,
                     b.lhs_off.defined() ? b.lhs_off.data_ptr<int64_t>() : nullptr,
                     b.rhs_off.defined() ? b.rhs_off.data_ptr<int64_t>() : nullptr, Stream(indptr)),
        "gs_sddmm_csc");
}

void SegmentSum(const torch::Tensor& indptr, const torch::optional<torch::Tensor>& e_ids,
                const torch::optional<torch::Tensor>& n_ids, const torch::Tensor& data,
                torch::Tensor out, int64_t powk) {
  NeedI64(indptr, "indptr");
  NeedF32(data, "data");
  NeedF32(out, "out");
  const int idb = n_ids.has_value() && n_ids.value().defined() ? IdBytes(n_ids.value(), "valid ids") : 8;
  const int64_t nseg = indptr.numel() - 1;
  const int64_t nnz = e_ids.has_value() && e_ids.value().defined() ? e_ids.value().numel() : data.numel();
  auto ws = Scratch(gs_segment_workspace_bytes(nseg, nnz), indptr);
  Check(gs_segment_sum(indptr.data_ptr<int64_t>(), OptI64(e_ids, "e_ids"),
                       OptIds(n_ids, idb, "valid ids"), idb, data.data_ptr<float>(), nseg, nnz, powk,
                       out.data_ptr<float>(), ws.data_ptr(), ws.numel(), Stream(indptr)),
        "gs_segment_sum");
}

void CooSum(const torch::Tensor& target, const torch::optional<torch::Tensor>& e_ids,
            const torch::Tensor& data, torch::Tensor out, int64_t powk) {
  const int idb = IdBytes(target, "coo target");
  NeedF32(data, "data");
  NeedF32(out, "out");
  auto ws = Scratch(gs_coo_sum_workspace_bytes(target.numel(), out.numel()), target);
  Check(gs_coo_sum_binned(target.data_ptr(), idb, OptI64(e_ids, "e_ids"), data.data_ptr<float>(),
                          target.numel(), powk, out.numel(), out.data_ptr<float>(), ws.data_ptr(),
                          ws.numel(), Stream(target)),
        "gs_coo_sum_binned");
}

void SegmentNormalize(const torch::Tensor& indptr, const torch::optional<torch::Tensor>& e_ids,
                      const torch::Tensor& data, torch::Tensor out) {
  NeedI64(indptr, "indptr");
  NeedF32(data, "data");
  NeedF32(out, "out");
  const int64_t nseg = indptr.numel() - 1;
  const int64_t nnz = e_ids.has_value() && e_ids.value().defined() ? e_ids.value().numel() : data.numel();
  auto ws = Scratch(gs_segment_workspace_bytes(nseg, nnz), indptr);
  Check(gs_segment_normalize(indptr.data_ptr<int64_t>(), OptI64(e_ids, "e_ids"),
                             data.data_ptr<float>(), nseg, nnz, out.data_ptr<float>(), ws.data_ptr(),
                             ws.numel(), Stream(indptr)),
        "gs_segment_normalize");
}

void EDivUSum(const torch::Tensor& row, const torch::Tensor& col, const torch::Tensor& data,
              const torch::Tensor& divisor, torch::Tensor out_data, torch::Tensor out_sum) {
  const int idb = IdBytes(row, "coo row");
  TORCH_CHECK(IdBytes(col, "coo col") == idb, "coo row and col differ in dtype");
  NeedF32(data, "data");
  NeedF32(divisor, "divisor");
  Check(gs_e_div_u_sum(row.data_ptr(), col.data_ptr(), idb, data.data_ptr<float>(),
                       divisor.data_ptr<float>(), row.numel(), out_data.data_ptr<float>(),
                       out_sum.data_ptr<float>(), Stream(row)),
        "gs_e_div_u_sum");
}

SliceResult RowSlicingCsc(const torch::Tensor& indptr, const torch::Tensor& indices,
                          const torch::Tensor& row_ids, bool with_coo) {
  NeedI64(indptr, "indptr");
  const int idb = IdBytes(indices, "indices");
  TORCH_CHECK(IdBytes(row_ids, "row ids") == idb, "row ids and indices differ in dtype");
  const int64_t ncols = indptr.numel() - 1, nnz = indices.numel(), nr = row_ids.numel();
  auto out_indptr = torch::empty({ncols + 1}, I64(indptr));
  auto ws = Scratch(gs_row_slice_workspace_bytes(nr, nnz, ncols), indptr);
  void* st = Stream(indptr);
  Check(gs_row_slice_csc_mark(indptr.data_ptr<int64_t>(), indices.data_ptr(), idb, ncols, nnz,
                              row_ids.data_ptr(), nr, out_indptr.data_ptr<int64_t>(), ws.data_ptr(),
                              ws.numel(), st),
        "gs_row_slice_csc_mark");
  const int64_t kept = ReadTotal(out_indptr, ncols, Stream(out_indptr), "total");
  auto out_indices = torch::empty({kept}, indices.options());
  auto select_index = torch::empty({kept}, I64(indptr));
  torch::Tensor coo_col;
  if (with_coo) coo_col = torch::empty({kept}, indices.options());
  if (kept > 0)
    Check(gs_row_slice_csc_compact(indptr.data_ptr<int64_t>(), ncols, nnz, idb,
                                   out_indices.data_ptr(), select_index.data_ptr<int64_t>(),
                                   with_coo ? coo_col.data_ptr() : nullptr, ws.data_ptr(),
                                   ws.numel(), st),
          "gs_row_slice_csc_compact");
  return {out_indptr, coo_col, out_indices, select_index};
}

std::tuple<torch::Tensor, torch::Tensor, torch::Tensor> RowSlicingCoo(
    const torch::Tensor& key, const torch::Tensor& other, const torch::Tensor& ids,
    const torch::Tensor* flag, bool* flag_value) {
  const int idb = IdBytes(key, "coo ids");
  TORCH_CHECK(IdBytes(other, "coo ids") == idb && IdBytes(ids, "node ids") == idb,
              "coo ids and node ids differ in dtype");
  const int64_t E = key.numel(), n = ids.numel();
  auto num = torch::empty({1}, I64(key));
  auto ws = Scratch(gs_row_slice_workspace_bytes(n, E, 0), key);
  void* st = Stream(key);
  Check(gs_row_slice_coo_mark(key.data_ptr(), idb, E, ids.data_ptr(), n, num.data_ptr<int64_t>(),
                              ws.data_ptr(), ws.numel(), st),
        "gs_row_slice_coo_mark");
  int64_t kept;
  if (flag) {
    auto both = torch::stack({num.reshape({}), flag->to(torch::kInt64).reshape({})}).cpu();
    kept = both.data_ptr<int64_t>()[0];
    *flag_value = both.data_ptr<int64_t>()[1] != 0;
    if (!*flag_value) return {torch::Tensor(), torch::Tensor(), torch::Tensor()};
  } else {
    kept = ReadTotal(num, 0, Stream(num), "total");
  }
  auto out_key = torch::empty({kept}, key.options());
  auto out_other = torch::empty({kept}, key.options());
  auto select_index = torch::empty({kept}, I64(key));
  if (kept > 0)
    Check(gs_row_slice_coo_compact(other.data_ptr(), idb, E, out_key.data_ptr(),
                                   out_other.data_ptr(), select_index.data_ptr<int64_t>(),
                                   ws.data_ptr(), ws.numel(), st),
          "gs_row_slice_coo_compact");
  return {out_key, out_other, select_index};
}

std::tuple<torch::Tensor, torch::Tensor, torch::Tensor, torch::Tensor> ColRowSlicing(
    const torch::Tensor& indptr, const torch::Tensor& indices, const torch::Tensor& column_ids,
    const torch::Tensor& row_ids, const torch::optional<torch::Tensor>& col_ptr,
    const torch::optional<torch::Tensor>& row_ptr, int64_t encoding_size) {
  NeedI64(indptr, "indptr");
  const int idb = IdBytes(indices, "indices");
  TORCH_CHECK(IdBytes(column_ids, "column ids") == idb && IdBytes(row_ids, "row ids") == idb,
              "column ids, row ids and indices differ in dtype");
  const int64_t S = column_ids.numel(), nr = row_ids.numel(), ncols = indptr.numel() - 1;
  const bool batched = col_ptr.has_value();
  TORCH_CHECK(batched == row_ptr.has_value(), "column and row batch offsets come together");
  int64_t B = 0;
  if (batched) {
    B = col_ptr.value().numel() - 1;
    TORCH_CHECK(row_ptr.value().numel() == B + 1, "column and row batch offsets differ in length");
    TORCH_CHECK(encoding_size > 0, "a batched slice needs a positive encoding size");
  }
  void* st = Stream(indptr);
  auto sub_indptr = torch::empty({S + 1}, I64(indptr));
  {
    auto ws = Scratch(gs_slice_workspace_bytes(S), indptr);
    Check(gs_slice_count(indptr.data_ptr<int64_t>(), ncols, column_ids.data_ptr(), idb, S,
                         sub_indptr.data_ptr<int64_t>(), ws.data_ptr(), ws.numel(), st),
          "gs_slice_count");
  }
  const int64_t D = ReadTotal(sub_indptr, S, Stream(sub_indptr), "total");
  auto out_indptr = torch::empty({S + 1}, I64(indptr));
  auto ws = Scratch(gs_col_row_slice_workspace_bytes(nr, D), indptr);
  Check(gs_col_row_slice_mark(indptr.data_ptr<int64_t>(), ncols, indices.data_ptr(), idb,
                              column_ids.data_ptr(), S, sub_indptr.data_ptr<int64_t>(), D,
                              row_ids.data_ptr(), nr, OptI64(col_ptr, "column batch offsets"),
                              OptI64(row_ptr, "row batch offsets"), B, encoding_size,
                              out_indptr.data_ptr<int64_t>(), ws.data_ptr(), ws.numel(), st),
        "gs_col_row_slice_mark");
  const int64_t kept = ReadTotal(out_indptr, S, Stream(out_indptr), "total");
  auto out_indices = torch::empty({kept}, indices.options());
  auto select_index = torch::empty({kept}, I64(indptr));
  auto parent_index = torch::empty({kept}, I64(indptr));
  if (kept > 0)
    Check(gs_col_row_slice_compact(D, idb, out_indices.data_ptr(), select_index.data_ptr<int64_t>(),
                                   parent_index.data_ptr<int64_t>(), ws.data_ptr(), ws.numel(), st),
          "gs_col_row_slice_compact");
  return {out_indptr, out_indices, select_index, parent_index};
}

SliceResult DcscColSlicing(const torch::Tensor& indptr, const torch::Tensor& indices,
                           const torch::Tensor& nid_map, const torch::Tensor& column_ids,
                           bool with_coo, bool with_select) {
  // position of every requested column among the stored ones; -1 (not stored) is outside
  // [0, num_cols) and therefore an empty column for the slice kernels
  return ColSlicing(indptr, indices, IndexSearch(nid_map, column_ids), with_coo, with_select);
}

torch::Tensor Dcsc2CooCols(const torch::Tensor& indptr, int64_t nnz, const torch::Tensor& ids) {
  NeedI64(indptr, "indptr");
  const int idb = IdBytes(ids, "valid ids");
  TORCH_CHECK(ids.numel() == indptr.numel() - 1, "one id per stored column expected");
  auto col = torch::empty({nnz}, ids.options());
  Check(gs_dcsc2coo(indptr.data_ptr<int64_t>(), indptr.numel() - 1, nnz, ids.data_ptr(),
                    col.data_ptr(), idb, Stream(indptr)),
        "gs_dcsc2coo");
  return col;
}

std::tuple<torch::Tensor, torch::Tensor> CscCompress(const torch::Tensor& indptr,
                                                     const torch::Tensor& ids_like) {
  NeedI64(indptr, "indptr");
  const int idb = IdBytes(ids_like, "indices");
  const int64_t n = indptr.numel() - 1;
  auto val_ids = torch::empty({n}, ids_like.options());
  auto out_indptr = torch::empty({n + 1}, I64(indptr));
  auto num = torch::empty({1}, I64(indptr));
  auto ws = Scratch(gs_csc_compress_workspace_bytes(n), indptr);
  Check(gs_csc_compress(indptr.data_ptr<int64_t>(), n, idb, val_ids.data_ptr(),
                        out_indptr.data_ptr<int64_t>(), num.data_ptr<int64_t>(), ws.data_ptr(),
                        ws.numel(), Stream(indptr)),
        "gs_csc_compress");
  const int64_t kept = ReadTotal(num, 0, Stream(num), "total");
  return {out_indptr.narrow(0, 0, kept + 1), val_ids.narrow(0, 0, kept)};
}

torch::Tensor Csc2CooCols(const torch::Tensor& indptr, int64_t nnz, const torch::Tensor& ids_like) {
  NeedI64(indptr, "indptr");
  const int idb = IdBytes(ids_like, "indices");
  auto col = torch::empty({nnz}, ids_like.options());
  Check(gs_csc2coo(indptr.data_ptr<int64_t>(), indptr.numel() - 1, nnz, col.data_ptr(), idb,
                   Stream(indptr)),
        "gs_csc2coo");
  return col;
}

std::tuple<torch::Tensor, torch::Tensor, torch::optional<torch::Tensor>> Coo2Csc(
    const torch::Tensor& key, const torch::Tensor& value, int64_t num_keys, bool sorted) {
  const int idb = IdBytes(key, "coo key");
  TORCH_CHECK(IdBytes(value, "coo value") == idb, "coo key and value differ in dtype");
  const int64_t E = key.numel();
  auto indptr = torch::empty({num_keys + 1}, I64(key));
  if (sorted) {
    Check(gs_coo2csc(key.data_ptr(), value.data_ptr(), idb, E, num_keys, 1,
                     indptr.data_ptr<int64_t>(), nullptr, nullptr, nullptr, 0, Stream(key)),
          "gs_coo2csc");
    return {indptr, value, torch::nullopt};
  }
  auto out_value = torch::empty({E}, value.options());
  auto perm = torch::empty({E}, I64(key));
  auto ws = Scratch(gs_coo2csc_workspace_bytes(E, num_keys), key);
  Check(gs_coo2csc(key.data_ptr(), value.data_ptr(), idb, E, num_keys, 0,
                   indptr.data_ptr<int64_t>(), out_value.data_ptr(), perm.data_ptr<int64_t>(),
                   ws.data_ptr(), ws.numel(), Stream(key)),
        "gs_coo2csc");
  return {indptr, out_value, perm};
}

std::tuple<torch::Tensor, torch::Tensor> SortValuesByKey(const torch::Tensor& key,
                                                         const torch::Tensor& value,
                                                         int64_t num_keys) {
  const int idb = IdBytes(key, "sort key");
  TORCH_CHECK(IdBytes(value, "sort value") == idb, "sort key and value differ in dtype");
  const int64_t E = key.numel();
  auto out_value = torch::empty({E}, value.options());
  auto perm = torch::empty({E}, I64(key));
  if (E == 0) return {out_value, perm};
  auto ws = Scratch(gs_coo2csc_workspace_bytes(E, num_keys), key);
  Check(gs_coo2csc(key.data_ptr(), value.data_ptr(), idb, E, num_keys, 0, nullptr,
                   out_value.data_ptr(), perm.data_ptr<int64_t>(), ws.data_ptr(), ws.numel(),
                   Stream(key)),
        "gs_coo2csc");
  return {out_value, perm};
}

bool SortedUnionFits(int64_t count, const torch::Tensor& ids_like) {
  return count >= 1 && count <= gs_sorted_union_max(IdBytes(ids_like, "ids"));
}

std::tuple<torch::Tensor, torch::Tensor> SortedUnion(const torch::Tensor& a, const torch::Tensor& b) {
  const int idb = IdBytes(a, "a");
  TORCH_CHECK(IdBytes(b, "b") == idb, "SortedUnion: the two id lists differ in dtype");
  TORCH_CHECK(a.is_contiguous() && b.is_contiguous(), "SortedUnion: id lists must be contiguous");
  auto out = torch::empty({a.numel() + b.numel()}, a.options());
  auto count = torch::empty({1}, I64(a));
  Check(gs_sorted_union(a.data_ptr(), a.numel(), b.data_ptr(), b.numel(), idb, out.data_ptr(),
                        count.data_ptr<int64_t>(), Stream(a)),
        "gs_sorted_union");
  return {out, count};
}

std::tuple<torch::Tensor, torch::Tensor, torch::Tensor> CooPickRows(
    const torch::Tensor& row, const torch::Tensor& col, const torch::Tensor& nodes,
    const torch::Tensor& count, int64_t max_nodes, int64_t* kept) {
  const int idb = IdBytes(row, "row");
  TORCH_CHECK(IdBytes(col, "col") == idb && IdBytes(nodes, "nodes") == idb,
              "CooPickRows: ids differ in dtype");
  NeedI64(count, "count");
  const int64_t E = row.numel();
  TORCH_CHECK(col.numel() == E && nodes.numel() >= max_nodes && count.numel() >= 1,
              "CooPickRows: sizes do not fit");
  auto key = torch::empty({E}, row.options());
  auto pos = torch::empty({E}, row.options());
  auto totals = torch::empty({2}, I64(row));
  auto ws = Scratch(gs_coo_pick_rows_workspace_bytes(E), row);
  HostBoxes& boxes = Boxes(row.get_device());
  const int64_t ticket = boxes.next++;
  Check(gs_coo_pick_rows(row.data_ptr(), col.data_ptr(), idb, E, nodes.data_ptr(),
                         count.data_ptr<int64_t>(), max_nodes, key.data_ptr(), pos.data_ptr(),
                         totals.data_ptr<int64_t>(), boxes.slot(ticket), ticket, ws.data_ptr(),
                         ws.numel(), Stream(row)),
        "gs_coo_pick_rows");
  if (kept) {
    *kept = WaitBox(boxes.slot(ticket), ticket, Stream(row), "gs_coo_pick_rows");
    if (*kept == kLost) *kept = totals[1].item<int64_t>();
  }
  return {key, pos, totals};
}

std::tuple<torch::Tensor, torch::Tensor, torch::Tensor> CooBlockValues(
    const torch::Tensor& kept_key, const torch::Tensor& kept_pos, int64_t max_nodes,
    const torch::Tensor& row, const torch::optional<torch::Tensor>& data,
    const torch::Tensor& divisor, int64_t num_cols) {
  const int idb = IdBytes(row, "row");
  TORCH_CHECK(IdBytes(kept_key, "keys") == idb && IdBytes(kept_pos, "positions") == idb,
              "CooBlockValues: ids differ in dtype");
  NeedF32(divisor, "divisor");
  const int64_t kept = kept_key.numel();
  TORCH_CHECK(kept_pos.numel() == kept, "CooBlockValues: one position per key");
  const float* values = nullptr;
  if (data.has_value()) {
    NeedF32(data.value(), "data");
    TORCH_CHECK(data.value().numel() == row.numel() && data.value().is_contiguous(),
                "CooBlockValues: one contiguous value per edge");
    values = data.value().data_ptr<float>();
  }
  auto out_row = torch::empty({kept}, row.options());
  auto out_value = torch::empty({kept}, divisor.options());
  auto out_indptr = torch::empty({num_cols + 1}, I64(row));
  auto ws = Scratch(gs_coo_block_values_workspace_bytes(kept), row);
  Check(gs_coo_block_values(kept_key.data_ptr(), kept_pos.data_ptr(), kept, max_nodes, row.data_ptr(),
                            idb, values, divisor.data_ptr<float>(), num_cols, out_row.data_ptr(),
                            out_value.data_ptr<float>(), out_indptr.data_ptr<int64_t>(),
                            ws.data_ptr(), ws.numel(), Stream(row)),
        "gs_coo_block_values");
  return {out_row, out_value, out_indptr};
}

std::tuple<torch::Tensor, torch::Tensor> ListSampling(const torch::Tensor& data, int64_t k,
                                                      bool replace) {
  const int idb = IdBytes(data, "data");
  const int64_t n = data.numel();
  if (n <= k && !replace) return {data, torch::arange(n, I64(data))};  // list_sampling.cu:29-32
  auto out_data = torch::empty({k}, data.options());
  auto out_index = torch::empty({k}, I64(data));
  auto ws = Scratch(gs_list_sample_workspace_bytes(n, k), data);
  Check(gs_list_sample_uniform(data.data_ptr(), idb, n, k, replace ? 1 : 0, NextSeed(), nullptr,
                               out_data.data_ptr(), out_index.data_ptr<int64_t>(), ws.data_ptr(),
                               ws.numel(), Stream(data)),
        "gs_list_sample_uniform");
  return {out_data, out_index};
}

std::tuple<torch::Tensor, torch::Tensor> ListSamplingProbs(const torch::Tensor& data,
                                                           const torch::Tensor& probs, int64_t k,
                                                           bool replace) {
  const int idb = IdBytes(data, "data");
  NeedF32(probs, "probs");
  const int64_t n = data.numel();
  TORCH_CHECK(probs.numel() == n, "data and probs differ in length");
  if (n <= k && !replace) return {data, torch::arange(n, I64(data))};  // list_sampling_probs.cu:20-23
  TORCH_CHECK(!replace,
              "weighted list sampling with replacement is not built (only the A-Res path without "
              "replacement is)");
  auto out_data = torch::empty({k}, data.options());
  auto out_index = torch::empty({k}, I64(data));
  auto ws = Scratch(gs_list_sample_workspace_bytes(n, k), data);
  Check(gs_list_sample_weighted(data.data_ptr(), idb, probs.data_ptr<float>(), n, k, NextSeed(),
                                nullptr, out_data.data_ptr(), out_index.data_ptr<int64_t>(),
                                ws.data_ptr(), ws.numel(), Stream(data)),
        "gs_list_sample_weighted");
  return {out_data, out_index};
}

// --------------------------------------------------------- super-batch helpers
namespace {
int64_t NumBatches(const torch::Tensor& ptr, const char* name) {
  NeedI64(ptr, name);
  TORCH_CHECK(ptr.numel() >= 2, name, " must hold num_batches + 1 offsets");
  return ptr.numel() - 1;
}
}  // namespace

torch::Tensor BatchEncode(const torch::Tensor& data, const torch::Tensor& ptr, int64_t enc) {
  const int idb = IdBytes(data, "data");
  const int64_t B = NumBatches(ptr, "data_ptr");
  auto out = torch::empty_like(data);
  Check(gs_batch_encode(data.data_ptr(), idb, data.numel(), ptr.data_ptr<int64_t>(), B, enc,
                        out.data_ptr(), Stream(data)),
        "gs_batch_encode");
  return out;
}

torch::Tensor BatchDecode(const torch::Tensor& in, int64_t enc) {
  const int idb = IdBytes(in, "data");
  auto out = torch::empty_like(in);
  Check(gs_batch_decode(in.data_ptr(), idb, in.numel(), enc, out.data_ptr(), nullptr, Stream(in)),
        "gs_batch_decode");
  return out;
}

std::tuple<torch::Tensor, torch::Tensor> BatchOffsets(const torch::Tensor& in, int64_t B,
                                                      int64_t enc) {
  const int idb = IdBytes(in, "data");
  auto ptr = torch::empty({B + 1}, I64(in));
  auto out = torch::empty_like(in);
  Check(gs_batch_offsets(in.data_ptr(), idb, in.numel(), B, enc, ptr.data_ptr<int64_t>(),
                         out.data_ptr(), Stream(in)),
        "gs_batch_offsets");
  return {ptr, out};
}

std::tuple<torch::Tensor, torch::Tensor, torch::Tensor> BatchConcat(
    const std::vector<torch::Tensor>& data, const std::vector<torch::Tensor>& offsets) {
  TORCH_CHECK(!data.empty() && data.size() == offsets.size(),
              "BatchConcat takes as many offset tensors as data tensors, at least one");
  TORCH_CHECK(data.size() <= GS_MAX_SEGMENTS, "BatchConcat: at most ", GS_MAX_SEGMENTS,
              " tensors, got ", data.size());
  const int idb = IdBytes(data[0], "data");
  const int64_t B = NumBatches(offsets[0], "offsets");
  std::vector<const void*> dp;
  std::vector<const int64_t*> pp;
  int64_t longest = 0;
  for (size_t s = 0; s < data.size(); ++s) {
    TORCH_CHECK(IdBytes(data[s], "data") == idb, "BatchConcat: data tensors differ in dtype");
    TORCH_CHECK(NumBatches(offsets[s], "offsets") == B, "BatchConcat: offsets differ in length");
    dp.push_back(data[s].data_ptr());
    pp.push_back(offsets[s].data_ptr<int64_t>());
    longest = std::max(longest, data[s].numel());
  }
  void* st = Stream(data[0]);
  auto total_ptr = torch::empty({B + 1}, I64(data[0]));
  Check(gs_batch_concat_offsets(pp.data(), static_cast<int>(pp.size()), B,
                                total_ptr.data_ptr<int64_t>(), st),
        "gs_batch_concat_offsets");
  int64_t total = 0;
  for (const auto& d : data) total += d.numel();  // = total_ptr[B] when the offsets cover the data
  auto out = torch::empty({total}, data[0].options());
  auto key = torch::empty({total}, data[0].options());
  Check(gs_batch_concat_fill(dp.data(), pp.data(), static_cast<int>(pp.size()), B, longest, idb,
                             total_ptr.data_ptr<int64_t>(), out.data_ptr(), key.data_ptr(), st),
        "gs_batch_concat_fill");
  return {out, key, total_ptr};
}

void BatchSplit(const torch::Tensor& data, const torch::Tensor& data_ptr,
                const torch::optional<torch::Tensor>& data_key,
                const std::vector<torch::Tensor>& outs, const std::vector<torch::Tensor>& out_ptrs) {
  TORCH_CHECK(!outs.empty() && outs.size() == out_ptrs.size(),
              "BatchSplit takes as many offset tensors as output tensors, at least one");
  TORCH_CHECK(outs.size() <= GS_MAX_SEGMENTS, "BatchSplit: at most ", GS_MAX_SEGMENTS,
              " tensors, got ", outs.size());
  const int idb = IdBytes(data, "data");
  const int64_t B = NumBatches(data_ptr, "data_ptr");
  std::vector<void*> dp;
  std::vector<const int64_t*> pp;
  for (size_t s = 0; s < outs.size(); ++s) {
    TORCH_CHECK(IdBytes(outs[s], "output") == idb, "BatchSplit: outputs differ in dtype from data");
    TORCH_CHECK(NumBatches(out_ptrs[s], "output offsets") == B,
                "BatchSplit: offsets differ in length");
    dp.push_back(outs[s].data_ptr());
    pp.push_back(out_ptrs[s].data_ptr<int64_t>());
  }
  const void* key = nullptr;
  if (data_key.has_value() && data_key.value().defined()) {
    TORCH_CHECK(IdBytes(data_key.value(), "data_key") == idb && data_key.value().numel() == data.numel(),
                "BatchSplit: data_key must match data");
    key = data_key.value().data_ptr();
  }
  Check(gs_batch_split(data.data_ptr(), data_ptr.data_ptr<int64_t>(), key, idb, data.numel(), B,
                       dp.data(), pp.data(), static_cast<int>(pp.size()), Stream(data)),
        "gs_batch_split");
}

std::tuple<torch::Tensor, torch::Tensor, torch::Tensor, torch::Tensor> BatchCooRelabel(
    const torch::Tensor& seeds, const torch::Tensor& seeds_ptr, const torch::Tensor& coo_col,
    const torch::Tensor& coo_row, const torch::Tensor& coo_ptr) {
  const int idb = IdBytes(seeds, "seeds");
  TORCH_CHECK(IdBytes(coo_row, "coo_row") == idb && IdBytes(coo_col, "coo_col") == idb,
              "seeds and edges differ in dtype");
  TORCH_CHECK(coo_row.numel() == coo_col.numel(), "coo_row and coo_col differ in length");
  const int64_t B = NumBatches(seeds_ptr, "seeds_ptr");
  TORCH_CHECK(NumBatches(coo_ptr, "coo_ptr") == B, "seeds_ptr and coo_ptr differ in length");
  const int64_t M = seeds.numel() + coo_row.numel();
  auto unique = torch::empty({M}, seeds.options());
  auto unique_ptr = torch::empty({B + 1}, I64(seeds));
  auto out_row = torch::empty_like(coo_row);
  auto out_col = torch::empty_like(coo_col);
  auto num = torch::empty({1}, I64(seeds));
  auto ws = Scratch(gs_batch_relabel_workspace_bytes(M), seeds);
  void* st = Stream(seeds);
  HostBoxes& boxes = Boxes(seeds.device().index());
  int64_t U = kTooWide;
  for (int attempt = 0; attempt < 2 && U == kTooWide; ++attempt) {
    const int64_t ticket = boxes.next++;
    Check(gs_batch_coo_relabel(seeds.data_ptr(), seeds_ptr.data_ptr<int64_t>(), coo_row.data_ptr(),
                               coo_col.data_ptr(), coo_ptr.data_ptr<int64_t>(), B, seeds.numel(),
                               coo_row.numel(), TableIds(idb), unique.data_ptr(),
                               unique_ptr.data_ptr<int64_t>(), out_row.data_ptr(),
                               out_col.data_ptr(), num.data_ptr<int64_t>(), ws.data_ptr(),
                               ws.numel(), boxes.slot(ticket), ticket, st),
          "gs_batch_coo_relabel");
    U = WaitBox(boxes.slot(ticket), ticket, st, "gs_batch_coo_relabel");
    if (U == kLost) U = num.item<int64_t>();
    if (U == kTooWide) t_narrow_ids = false;
  }
  TORCH_CHECK(U >= 0, "gs_batch_coo_relabel: a tile gave up waiting for its predecessors");
  return {unique.narrow(0, 0, U), unique_ptr, out_row, out_col};
}

std::tuple<torch::Tensor, torch::Tensor, torch::Tensor, torch::Tensor> CooFilter(
    const torch::Tensor& key, const torch::Tensor& row, const torch::Tensor& col,
    const torch::optional<torch::Tensor>& key_ptr, const torch::Tensor& ids,
    const torch::optional<torch::Tensor>& ids_ptr) {
  const int idb = IdBytes(key, "coo ids");
  TORCH_CHECK(IdBytes(row, "coo ids") == idb && IdBytes(col, "coo ids") == idb &&
                  IdBytes(ids, "node ids") == idb,
              "coo ids and node ids differ in dtype");
  const int64_t E = key.numel(), n = ids.numel();
  TORCH_CHECK(row.numel() == E && col.numel() == E, "coo_row and coo_col differ in length");
  TORCH_CHECK(key_ptr.has_value() == ids_ptr.has_value(), "batch offsets come in pairs");
  int64_t B = 0;
  if (key_ptr.has_value()) {
    B = NumBatches(key_ptr.value(), "batch_ptr");
    TORCH_CHECK(NumBatches(ids_ptr.value(), "neighbors_ptr") == B, "batch offsets differ in length");
  }
  auto num = torch::empty({1}, I64(key));
  auto ws = Scratch(gs_row_slice_workspace_bytes(n, E, 0), key);
  void* st = Stream(key);
  Check(gs_coo_filter_mark(key.data_ptr(), idb, E, OptI64(key_ptr, "batch_ptr"), ids.data_ptr(), n,
                           OptI64(ids_ptr, "neighbors_ptr"), B, num.data_ptr<int64_t>(),
                           ws.data_ptr(), ws.numel(), st),
        "gs_coo_filter_mark");
  const int64_t kept = ReadTotal(num, 0, Stream(num), "total");
  auto out_row = torch::empty({kept}, key.options());
  auto out_col = torch::empty({kept}, key.options());
  auto select_index = torch::empty({kept}, I64(key));
  torch::Tensor out_ptr;
  if (B > 0) out_ptr = torch::empty({B + 1}, I64(key));
  Check(gs_coo_filter_compact(row.data_ptr(), col.data_ptr(), idb, E, OptI64(key_ptr, "batch_ptr"),
                              B, out_row.data_ptr(), out_col.data_ptr(),
                              select_index.data_ptr<int64_t>(),
                              B > 0 ? out_ptr.data_ptr<int64_t>() : nullptr, ws.data_ptr(),
                              ws.numel(), st),
        "gs_coo_filter_compact");
  return {out_row, out_col, out_ptr, select_index};
}

torch::Tensor IndexSearch(const torch::Tensor& data, const torch::Tensor& keys) {
  const int idb = IdBytes(data, "data");
  TORCH_CHECK(IdBytes(keys, "keys") == idb, "data and keys differ in dtype");
  auto out = torch::empty_like(keys);
  auto ws = Scratch(gs_index_search_workspace_bytes(data.numel()), data);
  Check(gs_index_search(data.data_ptr(), data.numel(), keys.data_ptr(), keys.numel(), idb,
                        out.data_ptr(), ws.data_ptr(), ws.numel(), Stream(data)),
        "gs_index_search");
  return out;
}

}  // namespace hip
}  // namespace gs
