// gs::Graph -- the sparse-matrix object behind torch.classes.gs_classes.Graph.
//
// Public API (names, signatures, return orders) follows the reference's
// src/graph.h:11-128 for everything on the sampling hot path: loading, format
// caches, slicing, uniform / weighted / fused sampling, induced-subgraph slicing,
// relabel, valid-node queries, walks, Sum / Normalize / Divide / EDivUSum and SDDMM,
// and the batched ("super-batch") methods.
//
// A Graph keeps up to three cached formats of one matrix (CSC, CSR, COO), the
// edge data, and the global ids of its local columns / rows.  Children share
// storage with their parents; CreateSparseFormat fills caches lazily, so a
// Graph must not be used from two threads at once (same as the reference).
#pragma once

#include <torch/custom_class.h>
#include <torch/script.h>

#include <memory>
#include <string>
#include <tuple>
#include <vector>

#include "graph_storage.h"

namespace gs {

namespace hip {
struct PendingSample;
struct PendingLayers;
}

class Graph;
// a minibatch queued by Graph::QueueSampleLayers (TORCH_LIBRARY class gs_classes.QueuedLayers)
struct QueuedLayers : public torch::CustomClassHolder {
  c10::intrusive_ptr<Graph> graph;
  torch::Tensor seeds;
  std::vector<int64_t> fanouts;
  bool replace = false;
  std::shared_ptr<hip::PendingLayers> pending;  // null: `ready` holds the result
  std::vector<torch::Tensor> ready;
  bool collected = false;
  std::vector<torch::Tensor> Collect();
};

// a super-batch queued by Graph::QueueSampleLayersBatched (TORCH_LIBRARY class
// gs_classes.QueuedSuperBatch): every layer is launched, the per-minibatch cuts are on their
// way to pinned memory; Collect() waits for them and hands out the per-minibatch views
struct QueuedSuperBatch : public torch::CustomClassHolder {
  struct Layer {
    torch::Tensor frontier, offsets, renamed, data;
    std::shared_ptr<hip::PendingSample> sample;  // (queued form: kept until the cuts are back)
  };
  std::vector<Layer> layers;
  std::vector<torch::Tensor> cut_sets;  // device arrays the post reads
  torch::Tensor cuts;                   // pinned: per layer [seed | edge | frontier cuts]
  std::shared_ptr<void> posted;         // hip::Posted; null: `ready` holds the result
  int64_t num_batches = 0;
  bool with_data = false;
  std::vector<std::vector<torch::Tensor>> ready;
  bool collected = false;
  std::vector<std::vector<torch::Tensor>> Collect();
};

class Graph : public torch::CustomClassHolder {
 public:
  explicit Graph(bool is_subgraph) : is_subgraph_(is_subgraph) {}
  Graph(bool is_subgraph, torch::optional<torch::Tensor> col_ids,
        torch::optional<torch::Tensor> row_ids, int64_t num_cols, int64_t num_rows)
      : is_subgraph_(is_subgraph),
        num_cols_(num_cols),
        num_rows_(num_rows),
        col_ids_(col_ids),
        row_ids_(row_ids) {}

  // ---- loading and raw accessors
  void LoadCSC(torch::Tensor indptr, torch::Tensor indices);
  void LoadCOO(torch::Tensor row, torch::Tensor col);
  void LoadCSR(torch::Tensor indptr, torch::Tensor indices);
  void LoadCSCWithColIds(torch::Tensor column_ids, torch::Tensor indptr, torch::Tensor indices);
  void SetMetaData(torch::optional<torch::Tensor> col_ids, torch::optional<torch::Tensor> row_ids,
                   int64_t num_cols, int64_t num_rows);
  void SetCSC(std::shared_ptr<CSC> csc) {
    Settle();
    csc_ = csc;
  }
  void SetCSR(std::shared_ptr<CSR> csr) {
    Settle();
    csr_ = csr;
  }
  void SetCOO(std::shared_ptr<COO> coo) {
    Settle();
    coo_ = coo;
  }
  void SetCOOByTensor(torch::Tensor row, torch::Tensor col, torch::optional<torch::Tensor> e_ids,
                      bool row_sorted, bool col_sorted);
  void SetData(torch::Tensor data) {
    Settle();
    data_ = data;
  }
  // ids of the stored columns / rows when the CSC / CSR is doubly compressed
  void SetValidCols(torch::Tensor val_cols) { val_col_ids_ = val_cols; }
  void SetValidRows(torch::Tensor val_rows) { val_row_ids_ = val_rows; }
  void SetNumEdges(int64_t num_edges) {
    Settle();
    num_edges_ = num_edges;
  }
  std::shared_ptr<CSC> GetCSC() {
    Settle();
    return csc_;
  }
  std::shared_ptr<CSR> GetCSR() {
    Settle();
    return csr_;
  }
  std::shared_ptr<COO> GetCOO() {
    Settle();
    return coo_;
  }
  std::vector<torch::Tensor> GetCSCTensor();
  std::vector<torch::Tensor> GetCOOTensor();
  // (indptr, indices, e_ids) of the row-compressed format as it is held (CSR or DCSR);
  // made from the others as a CSR when the graph has none
  std::vector<torch::Tensor> GetCSRTensor();
  // (indptr, indices, indices_ptr): the CSC of a super-batch whose columns are cut into
  // batches at seeds_ptr, with the matching cut of the edges (examples/graphsage/batching.py:68)
  std::tuple<torch::Tensor, torch::Tensor, torch::Tensor> GetBatchCSC(torch::Tensor seeds_ptr);
  torch::optional<torch::Tensor> GetData(std::string order = "default");
  int64_t GetNumRows() { return num_rows_; }
  int64_t GetNumCols() { return num_cols_; }
  int64_t GetNumEdges() {
    Settle();
    return num_edges_;
  }

  // ---- format caches
  void CSC2CSR();
  void CSR2CSC();
  void CSC2DCSR();
  void CSR2DCSC();
  void CreateSparseFormat(int64_t format);

  // ---- structure operators (axis 0: columns, axis 1: rows)
  c10::intrusive_ptr<Graph> Slicing(torch::Tensor n_ids, int64_t axis, int64_t on_format,
                                    int64_t output_format, bool relabel = false);
  c10::intrusive_ptr<Graph> Sampling(int64_t axis, int64_t fanout, bool replace, int64_t on_format,
                                     int64_t output_format);
  c10::intrusive_ptr<Graph> SamplingProbs(int64_t axis, torch::Tensor edge_probs, int64_t fanout,
                                          bool replace, int64_t on_format, int64_t output_format);
  c10::intrusive_ptr<Graph> ColumnwiseFusedSlicingAndSampling(torch::Tensor column_index,
                                                              int64_t fanout, bool replace);
  // Every layer of a GraphSAGE-style minibatch in one call: what the loop of the reference's
  // examples (examples/graphsage/batching.py:125-138) does layer by layer with
  // ColumnwiseFusedSlicingAndSampling + Relabel, next seeds = frontier.  Returns the flat list
  // [frontier, offsets, indices] x layers (elements 0, 3, 4 of Relabel()'s tuple), and on a
  // graph with edge data [frontier, offsets, indices, data] x layers, data being the sampled
  // edges' share of it (what GetData("default") of the layer's sample gives); layer l draws
  // with the l-th seed the calling thread hands out next, so the result equals the loop's.
  // On a graph without id maps all layers are queued with no host read in between and the
  // sizes are collected once at the end.
  std::vector<torch::Tensor> SampleLayers(torch::Tensor seeds, std::vector<int64_t> fanouts,
                                          bool replace);
  // SampleLayers where the whole minibatch can be queued on the device (a root graph without
  // id maps, sizes the layer chain takes, edge data -- if any -- one fp32 value per edge);
  // otherwise nothing is sampled, no seed is consumed and the list is empty, so that the
  // caller goes layer by layer itself.
  std::vector<torch::Tensor> SampleLayersIfQueued(torch::Tensor seeds,
                                                  std::vector<int64_t> fanouts, bool replace);
  // The first half of SampleLayers when the whole minibatch can be queued (else nullptr, and
  // no seed is consumed): the caller collects later, other minibatches may be queued
  // meanwhile.  A collect that throws hip::IdsTooWide is answered with SampleLayersLoop under
  // the seed the chain started from.
  std::shared_ptr<hip::PendingLayers> QueueLayers(const torch::Tensor& seeds,
                                                  const std::vector<int64_t>& fanouts,
                                                  bool replace);
  std::vector<torch::Tensor> SampleLayersLoop(torch::Tensor seeds,
                                              const std::vector<int64_t>& fanouts, bool replace);
  // SampleLayers in two halves for a caller that wants the next minibatch queued before it
  // collects this one (one thread, one stream: the stream then never waits for the host
  // between minibatches).  The seeds of the draws are taken here, in call order; collect()
  // gives what SampleLayers would have returned.  Where the minibatch cannot be queued it is
  // sampled at once and collect() hands the result over.
  c10::intrusive_ptr<QueuedLayers> QueueSampleLayers(torch::Tensor seeds,
                                                     std::vector<int64_t> fanouts, bool replace);
  // Many minibatches as ONE launch sequence per layer (a "super-batch", the flow of the
  // reference's examples/graphsage/batching.py:59-98: fused sampling over the concatenated
  // seeds, the batches' edge offsets, one relabel per minibatch done in one pass, the splits),
  // run inside this layer: no interpreter between the launches, two host waits per layer (the
  // edge count, the frontier length), the per-minibatch cuts read back once at the end.
  // Returns per seed set what SampleLayers returns; minibatch b draws as row range
  // [ptr[b], ptr[b+1]) of one sampler call per layer, so its samples differ from those of a
  // SampleLayers call on the same seeds, while every block is a valid sample of its seeds.
  std::vector<std::vector<torch::Tensor>> SampleLayersBatched(
      const std::vector<torch::Tensor>& seed_sets, const std::vector<int64_t>& fanouts,
      bool replace);
  // The same in two halves: the call returns once the last layer is launched (the waits for
  // the earlier layers' frontier lengths are inside it), Collect() of the result waits for the
  // cuts and makes the views.  A caller that queues super-batch i + 1 before it collects
  // super-batch i has the host's work before the first and after the last launch of a call
  // (concatenating the seeds, some hundred views and their Python wrappers) run while the
  // stream is busy with the last layer.
  c10::intrusive_ptr<QueuedSuperBatch> QueueSampleLayersBatched(
      const std::vector<torch::Tensor>& seed_sets, const std::vector<int64_t>& fanouts,
      bool replace);
  // One layer of a layer-wise (LADIES-style) sampler as ONE call, the operator chain of the
  // reference's examples/ladies/ladies_raw.py:10-25 on a root graph:
  //   U = this[:, seeds]; prob = U.sum(axis=1, powk=2);
  //   picked = list_sampling_with_probs(all rows, prob, fanout, replace=false);
  //   nodes = unique(cat(seeds, picked));
  //   block of U[nodes, :].divide(prob[nodes], axis=1).normalize(axis=0)
  // Returns {frontier, offsets of the seeds' columns, renamed row ends, values}: what
  // Relabel() and GetData("default") of that chain's result give, the values already in the
  // order of the block's edges (so there is no edge-id map).  The slice, the sum and the pick
  // are the same calls as in the chain; behind them the edges of U are tested against the
  // node set and only the kept ones are put in order, and the host waits twice more (kept
  // count, frontier length).  Takes the list-sampling seed the chain would take.  Empty (nothing
  // drawn, no seed consumed) where it does not apply: a graph with id maps, more than
  // gs_sorted_union_max seeds + picks, a slice or a block without edges.
  std::vector<torch::Tensor> LayerwiseBlockIfFused(torch::Tensor seeds, int64_t fanout);
  // induced subgraph: columns column_seeds, rows row_seeds (renamed to their position in
  // row_seeds), CSC only (reference src/graph.cc:116-141)
  c10::intrusive_ptr<Graph> FusedBidirSlicing(torch::Tensor column_seeds, torch::Tensor row_seeds);
  // one induced subgraph per batch, columns and rows cut at col_ptr / row_ptr; rows keep
  // their ids (reference src/graph.cc:143-171)
  c10::intrusive_ptr<Graph> BatchFusedBidirSlicing(torch::Tensor column_seeds, torch::Tensor col_ptr,
                                                   torch::Tensor row_seeds, torch::Tensor row_ptr);
  // ---- super-batch methods (reference src/graph.cc:312-391,987-1040)
  // Column slice of all batches at once (n_ids cut at nid_ptr): (graph, edge offsets of the
  // batches).  Without id maps the columns are named batch * num_rows + id; with
  // `encoding` so are the rows, and the graph counts num_rows * num_batches rows.
  std::tuple<c10::intrusive_ptr<Graph>, torch::Tensor> BatchSlicing(
      torch::Tensor n_ids, torch::Tensor nid_ptr, int64_t axis, int64_t on_format,
      int64_t output_format, bool relabel, bool encoding);
  // the CSC cut into graphs of split_size columns each (the last may be shorter)
  std::vector<c10::intrusive_ptr<Graph>> Split(int64_t split_size);
  // column and row ids taken modulo encoding_size
  void Decode(int64_t encoding_size);
  // (row, col) of the column-sorted COO
  std::tuple<torch::Tensor, torch::Tensor> GetBatchCOO();
  torch::Tensor RandomWalk(torch::Tensor seeds, int64_t walk_length);

  // ---- edge-data operators
  torch::Tensor Sum(int64_t axis, int64_t powk, int64_t on_format);
  c10::intrusive_ptr<Graph> Normalize(int64_t axis, int64_t on_format);
  c10::intrusive_ptr<Graph> Divide(torch::Tensor divisor, int64_t axis, int64_t on_format);
  std::tuple<c10::intrusive_ptr<Graph>, torch::Tensor> EDivUSum(torch::Tensor divisor);
  void SDDMM(const std::string& op, torch::Tensor lhs, torch::Tensor rhs, torch::Tensor out,
             int64_t lhs_target, int64_t rhs_target, int64_t on_format);

  // ---- node queries; a "valid" node is a requested column or a non-isolated row
  torch::Tensor AllValidNode();
  torch::Tensor GetRows();
  torch::Tensor GetCols();
  torch::Tensor GetValidRows();
  torch::Tensor GetValidCols();
  torch::Tensor GetCOORows(bool is_original);  // global ids when is_original, else local
  torch::Tensor GetCOOCols(bool is_original);
  // (frontier, #frontier, #columns, offsets-or-row, indices-or-col, e_ids, "csc" | "coo")
  std::tuple<torch::Tensor, int64_t, int64_t, torch::Tensor, torch::Tensor,
             torch::optional<torch::Tensor>, std::string>
  Relabel();
  std::vector<torch::Tensor> MetaData();
  std::vector<torch::Tensor> COOMetaData();
  std::vector<torch::Tensor> CSCMetaData();

 private:
  c10::intrusive_ptr<Graph> Child(torch::optional<torch::Tensor> col_ids,
                                  torch::optional<torch::Tensor> row_ids, int64_t num_cols,
                                  int64_t num_rows) const;
  c10::intrusive_ptr<Graph> SameShape(torch::Tensor data);
  torch::Tensor DataOrOnes();
  torch::TensorOptions IdOptions() const;
  void InheritData(Graph* child, const torch::optional<torch::Tensor>& e_ids,
                   const torch::Tensor& select_index) const;
  c10::intrusive_ptr<Graph> RowSliceOfCoo(const torch::Tensor& n_ids);
  c10::intrusive_ptr<Graph> SampleImpl(int64_t axis, const torch::Tensor* edge_probs,
                                       int64_t fanout, bool replace, int64_t on_format,
                                       int64_t output_format);

  // A graph made by the fused sampler may still be waiting for its edge count: the
  // sampled ids sit in a buffer of the capacity columns x fanout and the count is
  // on its way to a host mailbox.  Settle() collects it and installs the CSC; every
  // public method does that first, except Relabel(), which queues its kernels
  // behind the sampler with the count still on the device.
  void Settle();
  std::shared_ptr<hip::PendingSample> pending_;

  // Compressed form a slice computed on the way to a COO-only result: not a format of
  // the graph yet (getters and Relabel do not see it), just what CreateSparseFormat
  // installs instead of converting the COO back.
  std::shared_ptr<CSC> spare_csc_;
  std::shared_ptr<CSR> spare_csr_;

  // 0 .. num_rows - 1 of a graph without a row id list, made once (GetRows hands it to the
  // list samplers of every layer)
  torch::Tensor all_rows_;

  bool is_subgraph_ = false;
  int64_t num_cols_ = 0;
  int64_t num_rows_ = 0;
  int64_t num_edges_ = 0;
  std::shared_ptr<CSC> csc_;
  std::shared_ptr<CSR> csr_;
  std::shared_ptr<COO> coo_;
  torch::optional<torch::Tensor> data_;
  torch::optional<torch::Tensor> col_ids_;  // global id of each local column
  torch::optional<torch::Tensor> row_ids_;  // global id of each local row
  // set when csc_ / csr_ is doubly compressed: stored column (row) i is local column
  // (row) val_col_ids_[i]; columns (rows) without edges are not stored
  torch::optional<torch::Tensor> val_col_ids_;
  torch::optional<torch::Tensor> val_row_ids_;
};

}  // namespace gs
