// torch::Tensor front end of the C ABI (include/gs_hip.h): allocates outputs
// and scratch with the torch allocator, passes raw device pointers and the
// current HIP stream, turns a negative status into a c10::Error.
//
// This is the only file of the host layer that knows about the C ABI; it plays
// the part of the reference's src/cuda/graph_ops.h / tensor_ops.h / sddmm.h.
#pragma once

#include <torch/torch.h>

#include <memory>
#include <string>
#include <tuple>
#include <vector>

namespace gs {
namespace hip {

// {sub_indptr, coo_col (undefined when !with_coo), sub_indices, select_index}
using SliceResult = std::tuple<torch::Tensor, torch::Tensor, torch::Tensor, torch::Tensor>;

// Seed of the next sampling / walk call; every call consumes one value
// (seed, seed+1, ...).  The reference hard-wires its seeds, so two calls with
// the same launch geometry repeat the same draws (src/cuda/sampling.cu:138).
void SetSeed(uint64_t seed);
// The same for the calling thread only, which from then on no longer draws from the
// shared counter (until it calls SetSeed): for several sampler threads whose draws must
// not depend on how they interleave.
void SetThreadSeed(uint64_t seed);
uint64_t NextSeed();
// the seed the next NextSeed() of the calling thread will hand out, and n seeds handed back
// (for a call that drew, found it cannot go on this way, and leaves the draw to another path)
uint64_t PeekSeed();
void RewindSeeds(uint64_t n);
// whether Graph::SampleLayersBatched may queue a layer's relabel behind its sampler without
// waiting for the edge count (default on)
void SetBatchedNoWait(bool on);
bool BatchedNoWait();
// {layers whose relabel was queued that way, layers that waited for the edge count}, since load
std::vector<int64_t> BatchedNoWaitCounts();
void CountBatchedNoWait(bool went_through);
// off (default): Graph::Sum along the rows (columns) of a graph held as a COO only adds edge
// by edge with float atomics, so a sum of three or more addends can differ in its last bit
// from run to run (as on the reference's COO path, src/cuda/graph_ops.cu:45-64).  on: such a
// sum goes through the sorted format and adds in edge order, the same bits every run.
void SetOrderedSums(bool on);
bool OrderedSums();
// 0: Floyd selection for deg > fanout (default), 1: the reference's Algorithm R.
void SetSampleAlgo(int64_t algo);

// with_select false: select_index comes back undefined (nothing to gather edge data for)
struct EdgeData;
// edge (with data_out): the slice carries the edges' data over in the same pass, into *data_out
SliceResult ColSlicing(const torch::Tensor& indptr, const torch::Tensor& indices,
                       const torch::Tensor& column_ids, bool with_coo, bool with_select = true,
                       const EdgeData* edge = nullptr, torch::Tensor* data_out = nullptr);
// column_ids undefined: every column of the CSC
SliceResult ColSampling(const torch::Tensor& indptr, const torch::Tensor& indices,
                        const torch::Tensor& column_ids, int64_t fanout, bool replace,
                        bool with_coo);
// The edge data of a graph for a sampler to carry over to its samples in the same launch
// (what the reference gathers afterwards, src/graph.cc:544-557): data[e_ids ? e_ids[q] : q]
// for a sample taken at position q of the CSC's indices.
struct EdgeData {
  torch::Tensor data;                    // fp32, one value per edge id
  torch::optional<torch::Tensor> e_ids;  // the CSC's edge-id map, when it has one
  // whether the sampler kernels can read it: one contiguous fp32 value per edge on the device
  static bool Fits(const torch::Tensor& data, const torch::optional<torch::Tensor>& e_ids);
};

// A one-launch sample whose total the host has not read yet.  The buffers have
// the capacity S * fanout; Wait() collects the total from its mailbox (no stream
// synchronisation), after which the caller narrows them.
struct PendingSample {
  torch::Tensor sub_indptr;    // [S + 1], final
  torch::Tensor indices;       // capacity
  torch::Tensor select_index;  // capacity; undefined when not requested
  torch::Tensor coo_col;       // capacity; undefined when not requested
  torch::Tensor data;          // capacity; the samples' edge data, undefined without any
  int64_t S = 0;
  int64_t ticket = 0;
  void* stream = nullptr;
  int device = 0;
  // where the kernel posts the total: a slot of the launching thread's ring of pinned
  // mailboxes, kept alive here so that any thread may wait on it
  const void* box = nullptr;
  torch::Tensor box_owner;
  // the look-back state the launch used: zero-filled again (on `stream`) when a tile of the
  // launch gave up, since the error word in it is sticky
  torch::Tensor state_owner;
  int64_t Wait() const;
};
// Whether the fused sampler may hand back a graph before its edge count has reached the
// host (default on).  Off: every call settles before it returns, as the reference does.
void SetDeferredSampling(bool on);
bool DeferredSampling();
// whether ColSampling would take the one-launch path for this call
bool OneLaunchApplies(int64_t S, int64_t fanout, bool replace);
std::shared_ptr<PendingSample> ColSamplingDeferred(const torch::Tensor& indptr,
                                                   const torch::Tensor& indices,
                                                   const torch::Tensor& column_ids, int64_t fanout,
                                                   bool replace, bool with_coo, bool with_select,
                                                   const EdgeData* edge = nullptr);
// {frontier, relabelled sampled ids, number of sampled ids, copy of the sampler's
// offsets}: unique / relabel of (column ids, sampled ids) queued behind the sampler without
// reading its total
std::tuple<torch::Tensor, torch::Tensor, int64_t, torch::Tensor> RelabelDeferred(
    const torch::Tensor& col_ids, const PendingSample& p);

// Every layer of a minibatch queued back to back with no host read in between (per layer
// gs_layer_sample + gs_layer_relabel: the frontier of one layer and its length feed the next
// on the device).  Collect() waits for the counts and narrows.  Same draws and same results
// as ColSamplingDeferred + RelabelDeferred layer by layer with the seeds NextSeed() hands out.
struct PendingLayers {
  struct Layer {
    // where the layer's outputs start in `scratch` (bytes); their lengths come with the counts
    size_t off_frontier = 0, off_offsets = 0, off_renamed = 0, off_data = 0;
    int64_t ticket_edges = 0, ticket_unique = 0;
  };
  std::vector<Layer> layers;
  // the minibatch's one allocation: every layer's outputs at their bounds, the sampled ids
  // before renaming, slot numbers, counts; the collected tensors are windows of it
  torch::Tensor scratch;
  c10::ScalarType id_type = c10::ScalarType::Long;
  torch::Tensor box_owner;  // the pinned ring the tickets go to
  const void* ring = nullptr;
  torch::Tensor state_owner;     // the look-back state of the launches
  std::shared_ptr<void> tables;  // the pair of hash tables the layers used in turn
  void* stream = nullptr;
  int device = 0;
  int64_t num_seeds = 0;
  uint64_t first_seed = 0;  // layer l drew with first_seed + l
  bool with_data = false;   // the graph has edge data: every layer also holds its samples' data
  // {frontier, offsets over the layer's seeds, sampled ids renamed[, edge data of the samples
  // when the graph has edge data]} per layer.  Throws
  // IdsTooWide when a 64-bit id does not fit the chain's one-word table slots (the caller
  // repeats the minibatch layer by layer), c10::Error when a tile gave up waiting.
  std::vector<torch::Tensor> Collect();
};
struct IdsTooWide : public std::exception {
  const char* what() const noexcept override { return "an id beyond 32 bits"; }
};
// whether SampleLayersQueued takes this minibatch (uniform sampling by the one-launch
// kernel, bounds within the chain's table limit, ids that have fitted 32 bits so far)
bool LayerChainApplies(int64_t num_seeds, const std::vector<int64_t>& fanouts, bool replace);
std::shared_ptr<PendingLayers> SampleLayersQueued(const torch::Tensor& indptr,
                                                  const torch::Tensor& indices,
                                                  const torch::Tensor& seeds,
                                                  const std::vector<int64_t>& fanouts,
                                                  bool replace, const EdgeData* edge = nullptr);
// Device int64 arrays of one length -> pinned host memory, back to back, by a small kernel on
// the current stream (one launch per 32 arrays), without a copy call of the runtime.
// WaitPosted() then waits (a mailbox) until the last of them has landed, and with it everything
// queued before it on the same stream; any thread may wait.
struct Posted {
  const void* slot = nullptr;  // the mailbox of the last launch; null: nothing was posted
  torch::Tensor ring;          // keeps the mailbox alive
  int64_t ticket = 0;
  void* stream = nullptr;
};
Posted PostValueSets(const std::vector<torch::Tensor>& sets, torch::Tensor& pinned);
void WaitPosted(const Posted& posted);
// t[first : first + count] of a contiguous 1-d tensor, sharing its storage: what narrow()
// gives, made without a trip through the operator dispatcher (a super-batch hands back a few
// hundred such views per call).
torch::Tensor Slice1d(const torch::Tensor& t, int64_t first, int64_t count);
// For tests of the recovery path: raises the sticky error word in the look-back state of the
// calling thread's current stream on `like`'s device, as a tile that gave up waiting would.
// The next one-launch sampler or relabel on that state reports failure (every kernel still
// runs to its end), after which the host layer clears the state.
void DebugRaiseLookbackError(const torch::Tensor& like);
// the calling thread's seed counter as SetThreadSeed / SetSeed left it, to put it back
struct SeedState {
  bool own;
  uint64_t seed;
};
SeedState SaveSeedState();
void RestoreSeedState(const SeedState& s);

SliceResult ColSamplingProbs(const torch::Tensor& indptr, const torch::Tensor& indices,
                             const torch::Tensor& probs, const torch::Tensor& column_ids,
                             int64_t fanout, bool replace, bool with_coo);
std::tuple<torch::Tensor, torch::Tensor, torch::Tensor> SampleOneKeepDim(
    const torch::Tensor& indptr, const torch::Tensor& indices, const torch::Tensor& column_ids);

torch::Tensor Unique(const torch::Tensor& ids);
std::tuple<torch::Tensor, std::vector<torch::Tensor>> Relabel(
    const std::vector<torch::Tensor>& mapping, const std::vector<torch::Tensor>& queries);

// {unique (batch frontiers back to back), unique_ptr, relabelled ids}: one relabel per batch
std::tuple<torch::Tensor, torch::Tensor, torch::Tensor> BatchCsrRelabel(
    const torch::Tensor& seeds, const torch::Tensor& seeds_ptr, const torch::Tensor& ids,
    const torch::Tensor& ids_ptr);
// BatchCsrRelabel queued behind a sampler whose edge count has not been read: `ids` is the
// sampler's buffer, of which the first ids_ptr[B] entries (a device value) count; launches and
// outputs are sized by the buffer.  {unique (room for all items), unique_ptr, renamed ids (room
// for all ids)}; *num_unique = the frontiers' total length, waited for here, or a status the
// caller answers by waiting for the edge count and calling BatchCsrRelabel: -2 an id too wide,
// -4 a bucket's table full.  `producer`: the sampler the ids come from; when the relabel reports
// that it left because that sampler failed, the sampler is waited for, which raises its error
// and clears its look-back state.  Undefined tensors and *num_unique untouched when the path through
// bins is not the one to take the call (ids that do not ride in 32 bits, more than 511 batches,
// fewer than 2^19 items by the buffers' sizes).
std::tuple<torch::Tensor, torch::Tensor, torch::Tensor> BatchCsrRelabelQueued(
    const torch::Tensor& seeds, const torch::Tensor& seeds_ptr, const torch::Tensor& ids,
    const torch::Tensor& ids_ptr, int64_t* num_unique, const PendingSample* producer = nullptr);
// the batches' offsets, re-based, back to back (host_offsets: the same offsets on the host)
// cuts (optional): receives indptr[offsets], where every batch's edges start, from the same launch
torch::Tensor IndptrSplit(const torch::Tensor& indptr, const torch::Tensor& offsets,
                          int64_t total, torch::Tensor* cuts = nullptr);

torch::Tensor RandomWalk(const torch::Tensor& seeds, int64_t length, const torch::Tensor& indptr,
                         const torch::Tensor& indices);
torch::Tensor MetapathWalk(const torch::Tensor& seeds, const torch::Tensor& metapath,
                           const torch::Tensor& indptr_table, const torch::Tensor& indices_table,
                           const torch::Tensor& num_nodes_table, int id_bytes);

struct Bcast {
  int64_t lhs_len, rhs_len, out_len, reduce_size;
  torch::Tensor lhs_off, rhs_off;  // undefined when no broadcast
};
void SddmmCoo(const std::string& op, const Bcast& b, const torch::Tensor& row,
              const torch::Tensor& col, const torch::optional<torch::Tensor>& e_ids,
              const torch::Tensor& lhs, const torch::Tensor& rhs, torch::Tensor out, int lhs_target,
              int rhs_target);
void SddmmCsc(const std::string& op, const Bcast& b, const torch::Tensor& indptr,
              const torch::Tensor& indices, const torch::optional<torch::Tensor>& e_ids,
              const torch::optional<torch::Tensor>& nid_map, const torch::Tensor& lhs,
              const torch::Tensor& rhs, torch::Tensor out, int lhs_target, int rhs_target);

void SegmentSum(const torch::Tensor& indptr, const torch::optional<torch::Tensor>& e_ids,
                const torch::optional<torch::Tensor>& n_ids, const torch::Tensor& data,
                torch::Tensor out, int64_t powk);
void CooSum(const torch::Tensor& target, const torch::optional<torch::Tensor>& e_ids,
            const torch::Tensor& data, torch::Tensor out, int64_t powk);
void SegmentNormalize(const torch::Tensor& indptr, const torch::optional<torch::Tensor>& e_ids,
                      const torch::Tensor& data, torch::Tensor out);
void EDivUSum(const torch::Tensor& row, const torch::Tensor& col, const torch::Tensor& data,
              const torch::Tensor& divisor, torch::Tensor out_data, torch::Tensor out_sum);

SliceResult RowSlicingCsc(const torch::Tensor& indptr, const torch::Tensor& indices,
                          const torch::Tensor& row_ids, bool with_coo);
// {relabelled key, other, select_index}.  `flag` (a device scalar of any integer / bool type,
// or null) is read back in the same transfer as the count of kept edges and lands in
// *flag_value: a caller's own device-side check at no extra host wait; when it reads false the
// compaction is skipped and the three tensors come back undefined.
std::tuple<torch::Tensor, torch::Tensor, torch::Tensor> RowSlicingCoo(
    const torch::Tensor& key, const torch::Tensor& other, const torch::Tensor& ids,
    const torch::Tensor* flag = nullptr, bool* flag_value = nullptr);

// Induced-subgraph slice (columns column_ids, rows in row_ids) without writing the column
// slice: {out_indptr, out_indices, select_index, parent_index}.  select_index counts
// positions in the virtual column slice (the reference's nonzero(mask)); parent_index is the
// position of the edge in `indices`.  With batch offsets: a column of batch b keeps the rows
// of batch b's ids and rows keep their global id.
std::tuple<torch::Tensor, torch::Tensor, torch::Tensor, torch::Tensor> ColRowSlicing(
    const torch::Tensor& indptr, const torch::Tensor& indices, const torch::Tensor& column_ids,
    const torch::Tensor& row_ids, const torch::optional<torch::Tensor>& col_ptr = torch::nullopt,
    const torch::optional<torch::Tensor>& row_ptr = torch::nullopt, int64_t encoding_size = 0);

// ---- doubly-compressed formats (only the non-empty columns are stored; ids name them)
// column slice of a DCSC: a requested column that is not stored is an empty column
SliceResult DcscColSlicing(const torch::Tensor& indptr, const torch::Tensor& indices,
                           const torch::Tensor& nid_map, const torch::Tensor& column_ids,
                           bool with_coo, bool with_select = true);
// col[e] = ids[stored column owning e]
torch::Tensor Dcsc2CooCols(const torch::Tensor& indptr, int64_t nnz, const torch::Tensor& ids);
// {offsets of the non-empty columns, their ids}
std::tuple<torch::Tensor, torch::Tensor> CscCompress(const torch::Tensor& indptr,
                                                     const torch::Tensor& ids_like);

// col[e] = column owning edge e, in the dtype of `ids_like`
torch::Tensor Csc2CooCols(const torch::Tensor& indptr, int64_t nnz, const torch::Tensor& ids_like);
// {indptr, values in key order, sort permutation (nullopt when already sorted)}
std::tuple<torch::Tensor, torch::Tensor, torch::optional<torch::Tensor>> Coo2Csc(
    const torch::Tensor& key, const torch::Tensor& value, int64_t num_keys, bool sorted);

// {`value` in the stable order of `key` (keys below num_keys), the permutation}: the
// library's radix sort alone, no offsets built
std::tuple<torch::Tensor, torch::Tensor> SortValuesByKey(const torch::Tensor& key,
                                                         const torch::Tensor& value,
                                                         int64_t num_keys);

// ---- the tail of a layer-wise sampler on a column slice held as a COO (gs_layerwise.hip)
// whether na + nb ids of this width fit the one-workgroup sort of SortedUnion
bool SortedUnionFits(int64_t count, const torch::Tensor& ids_like);
// {distinct values of a and b in increasing order (room for all; the first *count hold),
// count: device int64[1]}
std::tuple<torch::Tensor, torch::Tensor> SortedUnion(const torch::Tensor& a, const torch::Tensor& b);
// the edges of (row, col) whose row is among the first *count of nodes (SortedUnion's pair),
// in edge order: {key = col << bits(max_nodes) | place of the row in nodes, position of the
// edge; both with room for every edge, totals: device int64[2] = {*count, kept edges}}.
// kept (may be null): the host waits for the number of kept edges (a mailbox) and puts it there.
std::tuple<torch::Tensor, torch::Tensor, torch::Tensor> CooPickRows(
    const torch::Tensor& row, const torch::Tensor& col, const torch::Tensor& nodes,
    const torch::Tensor& count, int64_t max_nodes, int64_t* kept = nullptr);
// the block of the kept edges of a COO whose edges come by column (CooPickRows' pair, cut to
// the kept count; the same max_nodes): inside every column in the order of the rows,
// {their row ids, data / divisor[row] (data undefined: ones), offsets of the num_cols columns}
std::tuple<torch::Tensor, torch::Tensor, torch::Tensor> CooBlockValues(
    const torch::Tensor& kept_key, const torch::Tensor& kept_pos, int64_t max_nodes,
    const torch::Tensor& row, const torch::optional<torch::Tensor>& data,
    const torch::Tensor& divisor, int64_t num_cols);

std::tuple<torch::Tensor, torch::Tensor> ListSampling(const torch::Tensor& data, int64_t k,
                                                      bool replace);
std::tuple<torch::Tensor, torch::Tensor> ListSamplingProbs(const torch::Tensor& data,
                                                           const torch::Tensor& probs, int64_t k,
                                                           bool replace);

// ---- super-batch helpers (a batched array = flat array + int64 offsets [B+1])
torch::Tensor BatchEncode(const torch::Tensor& data, const torch::Tensor& ptr, int64_t enc);
torch::Tensor BatchDecode(const torch::Tensor& in, int64_t enc);
// {offsets [B+1], decoded ids} of an encoded array sorted by batch
std::tuple<torch::Tensor, torch::Tensor> BatchOffsets(const torch::Tensor& in, int64_t B,
                                                      int64_t enc);
// {concatenation batch by batch, batch of each item, its offsets}
std::tuple<torch::Tensor, torch::Tensor, torch::Tensor> BatchConcat(
    const std::vector<torch::Tensor>& data, const std::vector<torch::Tensor>& offsets);
// scatters `data` back into outs (the inverse of BatchConcat)
void BatchSplit(const torch::Tensor& data, const torch::Tensor& data_ptr,
                const torch::optional<torch::Tensor>& data_key,
                const std::vector<torch::Tensor>& outs, const std::vector<torch::Tensor>& out_ptrs);
// {unique, unique_ptr, relabelled row, relabelled col}
std::tuple<torch::Tensor, torch::Tensor, torch::Tensor, torch::Tensor> BatchCooRelabel(
    const torch::Tensor& seeds, const torch::Tensor& seeds_ptr, const torch::Tensor& coo_col,
    const torch::Tensor& coo_row, const torch::Tensor& coo_ptr);
// edges whose key is among ids (of the same batch, with offsets): {row, col, offsets of the
// result (undefined without batches), select_index}; ids are kept, not renamed
std::tuple<torch::Tensor, torch::Tensor, torch::Tensor, torch::Tensor> CooFilter(
    const torch::Tensor& key, const torch::Tensor& row, const torch::Tensor& col,
    const torch::optional<torch::Tensor>& key_ptr, const torch::Tensor& ids,
    const torch::optional<torch::Tensor>& ids_ptr);
// position of each key in data, -1 when absent
torch::Tensor IndexSearch(const torch::Tensor& data, const torch::Tensor& keys);

}  // namespace hip
}  // namespace gs
