#include "graph.h"
#include "range.h"

#include "bcast.h"
#include "graph_ops.h"
#include "hip_ops.h"
#include "tensor_ops.h"

namespace gs {

namespace {

// _DCSC / _DCSR are the CSC / CSR with only the non-empty columns / rows stored
bool IsCscLike(int64_t format) { return format == _CSC || format == _DCSC; }
bool IsCsrLike(int64_t format) { return format == _CSR || format == _DCSR; }

torch::Tensor Pick(const torch::optional<torch::Tensor>& ids, const torch::Tensor& local) {
  return ids.has_value() ? ids.value().index({local}) : local;
}

}  // namespace

// ------------------------------------------------------------------ loading
void Graph::LoadCSC(torch::Tensor indptr, torch::Tensor indices) {
  csc_ = std::make_shared<CSC>(CSC{indptr, indices, torch::nullopt});
  num_cols_ = num_rows_ = indptr.numel() - 1;
  num_edges_ = indices.numel();
}

void Graph::LoadCSR(torch::Tensor indptr, torch::Tensor indices) {
  csr_ = std::make_shared<CSR>(CSR{indptr, indices, torch::nullopt});
  num_cols_ = num_rows_ = indptr.numel() - 1;
  num_edges_ = indices.numel();
}

// node count = the larger number of distinct endpoints (reference src/graph.cc:25-35)
void Graph::LoadCOO(torch::Tensor row, torch::Tensor col) {
  coo_ = std::make_shared<COO>(COO{row, col, torch::nullopt, false, false});
  const int64_t nr = std::get<0>(torch::_unique(row)).numel();
  const int64_t nc = std::get<0>(torch::_unique(col)).numel();
  num_cols_ = num_rows_ = std::max(nr, nc);
  num_edges_ = row.numel();
}

void Graph::LoadCSCWithColIds(torch::Tensor column_ids, torch::Tensor indptr,
                              torch::Tensor indices) {
  TORCH_CHECK(column_ids.numel() == indptr.numel() - 1,
              "length of column_ids is not aligned with indptr");
  csc_ = std::make_shared<CSC>(CSC{indptr, indices, torch::nullopt});
  col_ids_ = column_ids;
  num_cols_ = column_ids.numel();
  num_rows_ = indices.numel() ? indices.max().item<int64_t>() + 1 : 0;
  num_edges_ = indices.numel();
}

void Graph::SetMetaData(torch::optional<torch::Tensor> col_ids,
                        torch::optional<torch::Tensor> row_ids, int64_t num_cols,
                        int64_t num_rows) {
  col_ids_ = col_ids;
  row_ids_ = row_ids;
  num_cols_ = num_cols;
  num_rows_ = num_rows;
}

void Graph::SetCOOByTensor(torch::Tensor row, torch::Tensor col,
                           torch::optional<torch::Tensor> e_ids, bool row_sorted, bool col_sorted) {
  coo_ = std::make_shared<COO>(COO{row, col, e_ids, row_sorted, col_sorted});
}

torch::TensorOptions Graph::IdOptions() const {
  if (csc_) return csc_->indices.options();
  if (csr_) return csr_->indices.options();
  TORCH_CHECK(coo_ != nullptr, "the graph holds no sparse format");
  return coo_->row.options();
}

torch::Tensor Graph::DataOrOnes() {
  Settle();
  if (data_.has_value()) return data_.value();
  return torch::ones({num_edges_}, IdOptions().dtype(torch::kFloat32));
}

// edge data in the order of a format ("col": CSC order, "row": CSR order)
torch::optional<torch::Tensor> Graph::GetData(std::string order) {
  Settle();
  torch::Tensor data = DataOrOnes();
  if (order == "col") {
    if (!csc_) CreateSparseFormat(_CSC);  // a doubly-compressed CSC orders the edges alike
    if (csc_->e_ids.has_value()) return data.index({csc_->e_ids.value()});
  } else if (order == "row") {
    if (!csr_) CreateSparseFormat(_CSR);
    if (csr_->e_ids.has_value()) return data.index({csr_->e_ids.value()});
  }
  return data;
}

// ------------------------------------------------------------ format caches
void Graph::CSC2CSR() {
  Settle();
  CreateSparseFormat(_COO);
  SetCSR(GraphCOO2CSC(coo_, num_rows_, false));
}

void Graph::CSR2CSC() {
  Settle();
  CreateSparseFormat(_COO);
  SetCSC(GraphCOO2CSC(coo_, num_cols_, true));
}

void Graph::CSC2DCSR() {
  Settle();
  CreateSparseFormat(_COO);
  std::shared_ptr<CSR> csr;
  torch::Tensor val;
  std::tie(csr, val) = GraphCOO2DCSC(coo_, num_rows_, false);
  val_row_ids_ = val;
  SetCSR(csr);
}

void Graph::CSR2DCSC() {
  Settle();
  CreateSparseFormat(_COO);
  std::shared_ptr<CSC> csc;
  torch::Tensor val;
  std::tie(csc, val) = GraphCOO2DCSC(coo_, num_cols_, true);
  val_col_ids_ = val;
  SetCSC(csc);
}

// reference src/graph.cc:585-644
void Graph::CreateSparseFormat(int64_t format) {
  Range range("gs::CreateSparseFormat");
  Settle();
  if (format == _COO) {
    if (coo_) return;
    if (csc_)
      SetCOO(val_col_ids_.has_value() ? GraphDCSC2COO(csc_, val_col_ids_.value(), true)
                                      : GraphCSC2COO(csc_, true));
    else
      SetCOO(val_row_ids_.has_value() ? GraphDCSC2COO(csr_, val_row_ids_.value(), false)
                                      : GraphCSC2COO(csr_, false));
  } else if (format == _DCSC) {
    if (csc_) {
      TORCH_CHECK(val_col_ids_.has_value(), "Require DCSC, get CSC instead");
      return;
    }
    CSR2DCSC();
  } else if (format == _DCSR) {
    if (csr_) {
      TORCH_CHECK(val_row_ids_.has_value(), "Require DCSR, get CSR instead");
      return;
    }
    CSC2DCSR();
  } else if (format == _CSC) {
    if (csc_) {
      TORCH_CHECK(!val_col_ids_.has_value(), "Require CSC, get DCSC instead");
      return;
    }
    if (spare_csc_)
      SetCSC(std::move(spare_csc_));
    else if (coo_)
      SetCSC(GraphCOO2CSC(coo_, num_cols_, true));
    else
      CSR2CSC();
  } else if (format == _CSR) {
    if (csr_) {
      TORCH_CHECK(!val_row_ids_.has_value(), "Require CSR, get DCSR instead");
      return;
    }
    if (spare_csr_)
      SetCSR(std::move(spare_csr_));
    else if (coo_)
      SetCSR(GraphCOO2CSC(coo_, num_rows_, false));
    else
      CSC2CSR();
  } else {
    TORCH_CHECK(false, "unknown sparse format flag ", format);
  }
}

std::vector<torch::Tensor> Graph::GetCSCTensor() {
  Settle();
  if (!csc_) CreateSparseFormat(_CSC);
  return {csc_->indptr, csc_->indices, csc_->e_ids.value_or(torch::Tensor())};
}

std::tuple<torch::Tensor, torch::Tensor, torch::Tensor> Graph::GetBatchCSC(
    torch::Tensor seeds_ptr) {
  Settle();
  CreateSparseFormat(_CSC);
  return {csc_->indptr, csc_->indices, csc_->indptr.index({seeds_ptr})};
}

std::vector<torch::Tensor> Graph::GetCSRTensor() {
  Settle();
  if (!csr_) CreateSparseFormat(_CSR);
  return {csr_->indptr, csr_->indices, csr_->e_ids.value_or(torch::Tensor())};
}

std::vector<torch::Tensor> Graph::GetCOOTensor() {
  Settle();
  CreateSparseFormat(_COO);
  TORCH_CHECK(coo_->col_sorted, "GetCOOTensor expects a column-sorted COO");
  return {coo_->row, coo_->col, coo_->e_ids.value_or(torch::Tensor())};
}

// ------------------------------------------------------------------ helpers
c10::intrusive_ptr<Graph> Graph::Child(torch::optional<torch::Tensor> col_ids,
                                       torch::optional<torch::Tensor> row_ids, int64_t num_cols,
                                       int64_t num_rows) const {
  return c10::make_intrusive<Graph>(true, col_ids, row_ids, num_cols, num_rows);
}

// edge data follows the edges: data[e_ids[select_index]] (reference src/graph.cc:295-308)
void Graph::InheritData(Graph* child, const torch::optional<torch::Tensor>& e_ids,
                        const torch::Tensor& select_index) const {
  if (!data_.has_value()) return;
  torch::Tensor where = e_ids.has_value() ? e_ids.value().index({select_index}) : select_index;
  child->SetData(data_.value().index({where}));
}

// a graph with the same structure (shared format caches) and new edge data
c10::intrusive_ptr<Graph> Graph::SameShape(torch::Tensor data) {
  Settle();
  auto g = c10::make_intrusive<Graph>(is_subgraph_, col_ids_, row_ids_, num_cols_, num_rows_);
  g->SetCSC(csc_);
  g->SetCSR(csr_);
  g->SetCOO(coo_);
  g->SetNumEdges(num_edges_);
  g->SetData(data);
  g->val_col_ids_ = val_col_ids_;
  g->val_row_ids_ = val_row_ids_;
  return g;
}

// ------------------------------------------------------------------ slicing
c10::intrusive_ptr<Graph> Graph::Slicing(torch::Tensor n_ids, int64_t axis, int64_t on_format,
                                         int64_t output_format, bool relabel) {
  Range range("gs::Slicing");
  Settle();
  TORCH_CHECK(axis == 0 || axis == 1, "axis must be 0 (columns) or 1 (rows)");
  if (axis == 1 && on_format == _CSR && output_format == _COO && !relabel) {
    auto sliced = RowSliceOfCoo(n_ids);
    if (sliced) return sliced;
  }
  CreateSparseFormat(on_format);
  const bool with_coo = output_format & _COO;
  torch::optional<torch::Tensor> new_val_cols, new_val_rows;

  torch::optional<torch::Tensor> col_ids = col_ids_, row_ids = row_ids_;
  int64_t num_cols = num_cols_, num_rows = num_rows_;
  if (axis == 0) {
    col_ids = Pick(col_ids_, n_ids);
    num_cols = n_ids.numel();
  } else {
    row_ids = Pick(row_ids_, n_ids);
    num_rows = n_ids.numel();
  }

  std::shared_ptr<CSC> out_csc, spare_csc;
  std::shared_ptr<CSR> out_csr, spare_csr;
  std::shared_ptr<COO> out_coo;
  torch::Tensor select_index;
  torch::Tensor carried;  // the slice's share of the edge data, when its own pass brought it
  torch::optional<torch::Tensor> e_ids;
  int64_t num_edges = 0;

  if (on_format == _COO) {
    std::tie(out_coo, select_index) = COOColSlicing(coo_, n_ids, axis);
    num_edges = out_coo->row.numel();
    e_ids = coo_->e_ids;
  } else {
    // CSC and CSR are the same storage with the roles of rows and columns
    // swapped: "along" is the axis the offsets run over.
    const bool on_csc = IsCscLike(on_format);
    TORCH_CHECK(on_csc || IsCsrLike(on_format), "unknown sparse format flag ", on_format);
    TORCH_CHECK(output_format != (on_csc ? _CSR : _CSC),
                "Error in Slicing, Not implementation [on_format = ", on_csc ? "CSC" : "CSR",
                ", output_format = ", on_csc ? "CSR" : "CSC", "]");
    std::shared_ptr<CSC> fmt = on_csc ? csc_ : csr_;
    const torch::optional<torch::Tensor>& stored = on_csc ? val_col_ids_ : val_row_ids_;
    const bool along = (axis == 0) == on_csc;
    std::shared_ptr<_TMP> tmp;
    if (along) {
      // the result has one (possibly empty) column per requested id, so it is never
      // doubly compressed, whatever the input was (reference src/graph.cc:213-217)
      if (stored.has_value())
        std::tie(tmp, select_index) =
            DCSCColSlicing(fmt, stored.value(), n_ids, with_coo, data_.has_value());
      else if (data_.has_value() && hip::EdgeData::Fits(data_.value(), fmt->e_ids)) {
        // the edges' data ride along in the slice's own pass: no select_index, no gather
        const hip::EdgeData edge{data_.value(), fmt->e_ids};
        std::tie(tmp, select_index) = CSCColSlicing(fmt, n_ids, with_coo, false, &edge, &carried);
      } else
        std::tie(tmp, select_index) = CSCColSlicing(fmt, n_ids, with_coo, data_.has_value());
      if (relabel) {
        // the other side is renumbered by first occurrence (reference src/graph.cc:219-227)
        torch::Tensor frontier;
        std::vector<torch::Tensor> renamed;
        std::tie(frontier, renamed) =
            BatchTensorRelabel({tmp->coo_in_indices}, {tmp->coo_in_indices});
        tmp->coo_in_indices = renamed[0];
        if (on_csc) {
          row_ids = frontier;
          num_rows = frontier.numel();
        } else {
          col_ids = frontier;
          num_cols = frontier.numel();
        }
      }
    } else {
      TORCH_CHECK(!relabel, "Not implemented warning");
      std::tie(tmp, select_index) = CSCRowSlicing(fmt, n_ids, with_coo);
      // the stored columns stay the same ones (reference src/graph.cc:231,254)
      (on_csc ? new_val_cols : new_val_rows) = stored;
      if (with_coo && stored.has_value())
        tmp->coo_in_indptr = stored.value().index({tmp->coo_in_indptr});
    }
    if (output_format & (on_csc ? (_CSC | _DCSC) : (_CSR | _DCSR))) {
      auto compressed =
          std::make_shared<CSC>(CSC{tmp->indptr, tmp->coo_in_indices, torch::nullopt});
      (on_csc ? out_csc : out_csr) = compressed;
    } else if (along && tmp->indptr.defined()) {
      // the slice produced the offsets anyway: keep them aside so that a later
      // CreateSparseFormat finds the compressed format without re-deriving it from the COO
      auto compressed =
          std::make_shared<CSC>(CSC{tmp->indptr, tmp->coo_in_indices, torch::nullopt});
      (on_csc ? spare_csc : spare_csr) = compressed;
    }
    if (with_coo) {
      out_coo = on_csc ? std::make_shared<COO>(COO{tmp->coo_in_indices, tmp->coo_in_indptr,
                                                   torch::nullopt, false, true})
                       : std::make_shared<COO>(COO{tmp->coo_in_indptr, tmp->coo_in_indices,
                                                   torch::nullopt, true, false});
    }
    num_edges = tmp->coo_in_indices.numel();
    e_ids = fmt->e_ids;
  }

  auto ret = Child(col_ids, row_ids, num_cols, num_rows);
  ret->SetNumEdges(num_edges);
  ret->SetCOO(out_coo);
  ret->SetCSC(out_csc);
  ret->SetCSR(out_csr);
  ret->spare_csc_ = spare_csc;
  ret->spare_csr_ = spare_csr;
  if (out_csc) ret->val_col_ids_ = new_val_cols;
  if (out_csr) ret->val_row_ids_ = new_val_rows;
  if (carried.defined())
    ret->SetData(carried);
  else
    InheritData(ret.get(), e_ids, select_index);
  return ret;
}

// Rows n_ids of a graph that is held as a COO only (a column slice, as `U[nodes, :]` of the
// layer-wise samplers meets it: python/gs/matrix_api/matrix.py:104-105), without the CSR the
// reference builds of the whole slice first (src/graph.cc:258-283, a sort of every edge): the
// edges are filtered by the id set, and only the kept ones are sorted by their new row.  The
// filter keeps the COO's order and the sort is stable, so the result holds the same edges in
// the same order as the CSR and its slice give.  Only for ids that are strictly increasing
// (distinct: a row asked for twice appears twice in the reference's result); returns null
// when it does not apply, and the caller goes the reference's way.
c10::intrusive_ptr<Graph> Graph::RowSliceOfCoo(const torch::Tensor& n_ids) {
  if (csr_ || spare_csr_ || !coo_ || val_row_ids_.has_value() || n_ids.numel() == 0 ||
      coo_->row.numel() == 0)
    return nullptr;
  torch::Tensor increasing;  // device flag, read together with the count of kept edges
  if (n_ids.numel() > 1)
    increasing = (n_ids.narrow(0, 1, n_ids.numel() - 1) > n_ids.narrow(0, 0, n_ids.numel() - 1)).all();
  torch::Tensor new_row, cols, select_index;
  bool distinct = true;
  std::tie(new_row, cols, select_index) =
      hip::RowSlicingCoo(coo_->row, coo_->col, n_ids, increasing.defined() ? &increasing : nullptr,
                         &distinct);
  if (!distinct) return nullptr;
  torch::Tensor indptr, sorted_cols;
  torch::optional<torch::Tensor> perm;
  std::tie(indptr, sorted_cols, perm) = hip::Coo2Csc(new_row, cols, n_ids.numel(), false);
  if (perm.has_value()) select_index = select_index.index({perm.value()});
  auto ret = Child(col_ids_, Pick(row_ids_, n_ids), num_cols_, n_ids.numel());
  ret->SetNumEdges(sorted_cols.numel());
  ret->SetCOO(std::make_shared<COO>(COO{hip::Csc2CooCols(indptr, sorted_cols.numel(), sorted_cols),
                                        sorted_cols, torch::nullopt, true, false}));
  ret->spare_csr_ = std::make_shared<CSR>(CSR{indptr, sorted_cols, torch::nullopt});
  InheritData(ret.get(), coo_->e_ids, select_index);
  return ret;
}

std::vector<torch::Tensor> Graph::LayerwiseBlockIfFused(torch::Tensor seeds, int64_t fanout) {
  Range range("gs::LayerwiseBlock");
  Settle();
  if (col_ids_.has_value() || row_ids_.has_value() || val_col_ids_.has_value() ||
      val_row_ids_.has_value() || !(csc_ || coo_ || csr_))
    return {};
  const int64_t S = seeds.numel();
  const int64_t picks = std::min<int64_t>(fanout, num_rows_);
  if (S == 0 || picks <= 0 || seeds.dim() != 1 || !seeds.is_contiguous() ||
      seeds.scalar_type() != IdOptions().dtype().toScalarType() ||
      !hip::SortedUnionFits(S + picks, seeds))
    return {};
  int key_bits = 0;  // of column << bits(S + picks) | place among the nodes
  while ((int64_t(1) << key_bits) < S + picks) ++key_bits;
  int col_bits = 0;
  while ((int64_t(1) << col_bits) < S) ++col_bits;
  if (key_bits + col_bits > (seeds.element_size() == 4 ? 30 : 62)) return {};

  auto U = Slicing(seeds, 0, _CSC, _COO, false);
  // (the edges of a column slice come by column, which the block's ordering relies on)
  if (!U->coo_ || U->num_edges_ == 0 || U->coo_->e_ids.has_value() || !U->coo_->col_sorted) return {};
  if (U->data_.has_value() &&
      (U->data_.value().scalar_type() != torch::kFloat32 || U->data_.value().dim() != 1))
    return {};
  const uint64_t seed_before = hip::PeekSeed();
  torch::Tensor prob = U->Sum(1, 2, _CSR);
  torch::Tensor picked = std::get<0>(hip::ListSamplingProbs(GetRows(), prob, fanout, false));
  torch::Tensor nodes, count, kept_key, kept_pos, totals;
  std::tie(nodes, count) = hip::SortedUnion(seeds, picked);
  int64_t kept = 0;  // (the host waits here)
  std::tie(kept_key, kept_pos, totals) =
      hip::CooPickRows(U->coo_->row, U->coo_->col, nodes, count, S + picks, &kept);
  if (kept == 0) {
    hip::RewindSeeds(hip::PeekSeed() - seed_before);  // the chain draws for itself
    return {};
  }
  torch::Tensor rows, values, indptr;
  std::tie(rows, values, indptr) = hip::CooBlockValues(
      hip::Slice1d(kept_key, 0, kept), hip::Slice1d(kept_pos, 0, kept), S + picks, U->coo_->row,
      U->data_.has_value() ? torch::optional<torch::Tensor>(U->data_.value().contiguous())
                           : torch::nullopt,
      prob, S);
  torch::Tensor normalized = torch::empty_like(values);
  hip::SegmentNormalize(indptr, torch::nullopt, values, normalized);
  torch::Tensor frontier;
  std::vector<torch::Tensor> renamed;
  std::tie(frontier, renamed) = BatchTensorRelabel({seeds, rows}, {rows});
  return {frontier, indptr, renamed[0], normalized};
}

// ----------------------------------------------------------------- sampling
c10::intrusive_ptr<Graph> Graph::SampleImpl(int64_t axis, const torch::Tensor* edge_probs,
                                            int64_t fanout, bool replace, int64_t on_format,
                                            int64_t output_format) {
  Range range("gs::Sampling");
  Settle();
  CreateSparseFormat(on_format);
  const bool on_csc = (axis == 0 && on_format == _CSC);
  const bool on_csr = (axis == 1 && on_format == _CSR);
  TORCH_CHECK(on_csc || on_csr, "No implementation!");  // reference src/graph.cc:456
  TORCH_CHECK(output_format != (on_csc ? _CSR : _CSC),
              "Error in Sampling, Not implementation [on_format = ", on_csc ? "CSC" : "CSR",
              ", output_format = ", on_csc ? "CSR" : "CSC", "]");
  const bool with_coo = output_format & _COO;
  std::shared_ptr<CSC> fmt = on_csc ? csc_ : csr_;
  std::shared_ptr<_TMP> tmp;
  torch::Tensor select_index;
  if (edge_probs)
    std::tie(tmp, select_index) = CSCColSamplingProbs(fmt, *edge_probs, fanout, replace, with_coo);
  else
    std::tie(tmp, select_index) = CSCColSampling(fmt, fanout, replace, with_coo);

  auto ret = Child(col_ids_, row_ids_, num_cols_, num_rows_);
  if (output_format & (on_csc ? _CSC : _CSR)) {
    auto compressed = std::make_shared<CSC>(CSC{tmp->indptr, tmp->coo_in_indices, torch::nullopt});
    if (on_csc) ret->SetCSC(compressed); else ret->SetCSR(compressed);
  }
  if (with_coo) {
    ret->SetCOO(on_csc ? std::make_shared<COO>(COO{tmp->coo_in_indices, tmp->coo_in_indptr,
                                                   torch::nullopt, false, true})
                       : std::make_shared<COO>(COO{tmp->coo_in_indptr, tmp->coo_in_indices,
                                                   torch::nullopt, true, false}));
  }
  ret->SetNumEdges(tmp->coo_in_indices.numel());
  InheritData(ret.get(), fmt->e_ids, select_index);
  return ret;
}

c10::intrusive_ptr<Graph> Graph::Sampling(int64_t axis, int64_t fanout, bool replace,
                                          int64_t on_format, int64_t output_format) {
  return SampleImpl(axis, nullptr, fanout, replace, on_format, output_format);
}

c10::intrusive_ptr<Graph> Graph::SamplingProbs(int64_t axis, torch::Tensor edge_probs,
                                               int64_t fanout, bool replace, int64_t on_format,
                                               int64_t output_format) {
  return SampleImpl(axis, &edge_probs, fanout, replace, on_format, output_format);
}

// slice + sample without materialising the slice; the result holds a CSC only
// and the kernel is given the LOCAL column index (reference src/graph.cc:531-559)
void Graph::Settle() {
  if (!pending_) return;
  std::shared_ptr<hip::PendingSample> p = std::move(pending_);
  pending_.reset();
  const int64_t nnz = p->Wait();
  auto csc = std::make_shared<CSC>();
  csc->indptr = p->sub_indptr;
  csc->indices = p->indices.narrow(0, 0, nnz);
  csc_ = csc;
  num_edges_ = nnz;
  if (p->data.defined()) data_ = p->data.narrow(0, 0, nnz);
}

c10::intrusive_ptr<Graph> Graph::ColumnwiseFusedSlicingAndSampling(torch::Tensor column_index,
                                                                   int64_t fanout, bool replace) {
  Range range("gs::FusedSlicingSampling");
  Settle();
  TORCH_CHECK(csc_ != nullptr, "fused slicing + sampling needs the CSC format");
  torch::Tensor col_ids = Pick(col_ids_, column_index);
  auto ret = Child(col_ids, row_ids_, col_ids.numel(), num_rows_);
  // Nothing on the host needs the edge count yet, so the child is handed back while the
  // sampler runs and settles when it is first used.  Edge data follows the samples inside the
  // sampler's launch (the gathers of src/graph.cc:544-557) when the kernels can read it.
  const bool data_fits = !data_.has_value() || hip::EdgeData::Fits(data_.value(), csc_->e_ids);
  if (hip::DeferredSampling() && data_fits && !(fanout == 1 && replace) &&
      hip::OneLaunchApplies(column_index.numel(), fanout, replace)) {
    if (data_.has_value()) {
      const hip::EdgeData edge{data_.value(), csc_->e_ids};
      ret->pending_ = hip::ColSamplingDeferred(csc_->indptr, csc_->indices, column_index, fanout,
                                               replace, false, false, &edge);
    } else {
      ret->pending_ = hip::ColSamplingDeferred(csc_->indptr, csc_->indices, column_index, fanout,
                                               replace, false, false);
    }
    return ret;
  }
  std::shared_ptr<CSC> sampled;
  torch::Tensor select_index;
  std::tie(sampled, select_index) = FusedCSCColSlicingAndSampling(csc_, column_index, fanout, replace);
  ret->SetCSC(sampled);
  ret->SetNumEdges(sampled->indices.numel());
  InheritData(ret.get(), csc_->e_ids, select_index);
  return ret;
}

std::shared_ptr<hip::PendingLayers> Graph::QueueLayers(const torch::Tensor& seeds,
                                                       const std::vector<int64_t>& fanouts,
                                                       bool replace) {
  Settle();
  TORCH_CHECK(csc_ != nullptr, "fused slicing + sampling needs the CSC format");
  // a root graph: local ids are the global ones; edge data, when there is any, must be what
  // the sampler kernels can carry over themselves
  if (col_ids_.has_value() || row_ids_.has_value() || val_col_ids_.has_value() ||
      !hip::DeferredSampling())
    return nullptr;
  if (data_.has_value() && !hip::EdgeData::Fits(data_.value(), csc_->e_ids)) return nullptr;
  for (int64_t k : fanouts)
    if (k == 1 && replace) return nullptr;  // (one slot per column, -1 for an empty one)
  if (!hip::LayerChainApplies(seeds.numel(), fanouts, replace)) return nullptr;
  if (data_.has_value()) {
    const hip::EdgeData edge{data_.value(), csc_->e_ids};
    return hip::SampleLayersQueued(csc_->indptr, csc_->indices, seeds, fanouts, replace, &edge);
  }
  return hip::SampleLayersQueued(csc_->indptr, csc_->indices, seeds, fanouts, replace);
}

std::vector<torch::Tensor> Graph::SampleLayersLoop(torch::Tensor seeds,
                                                   const std::vector<int64_t>& fanouts,
                                                   bool replace) {
  std::vector<torch::Tensor> out;
  out.reserve(4 * fanouts.size());
  for (int64_t k : fanouts) {
    auto sub = ColumnwiseFusedSlicingAndSampling(seeds, k, replace);
    auto r = sub->Relabel();
    out.push_back(std::get<0>(r));  // frontier: source ids of the block, seeds first
    out.push_back(std::get<3>(r));  // offsets over the destinations
    out.push_back(std::get<4>(r));  // source positions in the frontier
    // the samples' edge data, in the order of the sampled edges (the sample has no edge-id map)
    if (data_.has_value()) out.push_back(sub->GetData("default").value());
    seeds = std::get<0>(r);
  }
  return out;
}

std::vector<torch::Tensor> Graph::SampleLayersIfQueued(torch::Tensor seeds,
                                                        std::vector<int64_t> fanouts,
                                                        bool replace) {
  auto pending = QueueLayers(seeds, fanouts, replace);
  if (!pending) return {};
  try {
    return pending->Collect();
  } catch (const hip::IdsTooWide&) {
    // the same minibatch again, layer by layer, under the seeds the chain drew with
    const hip::SeedState saved = hip::SaveSeedState();
    hip::SetThreadSeed(pending->first_seed);
    auto out = SampleLayersLoop(seeds, fanouts, replace);
    hip::RestoreSeedState(saved);
    return out;
  }
}

c10::intrusive_ptr<QueuedLayers> Graph::QueueSampleLayers(torch::Tensor seeds,
                                                          std::vector<int64_t> fanouts,
                                                          bool replace) {
  Range range("gs::QueueSampleLayers");
  auto q = c10::make_intrusive<QueuedLayers>();
  q->graph = c10::intrusive_ptr<Graph>::reclaim_copy(this);
  q->seeds = seeds;
  q->fanouts = fanouts;
  q->replace = replace;
  q->pending = QueueLayers(seeds, fanouts, replace);
  if (!q->pending) q->ready = SampleLayersLoop(seeds, fanouts, replace);
  return q;
}

std::vector<torch::Tensor> QueuedLayers::Collect() {
  TORCH_CHECK(!collected, "this minibatch has been collected already");
  collected = true;
  if (!pending) return std::move(ready);
  try {
    auto out = pending->Collect();
    pending.reset();
    return out;
  } catch (const hip::IdsTooWide&) {
    // the same minibatch again, layer by layer, under the seeds the chain drew with
    const hip::SeedState saved = hip::SaveSeedState();
    hip::SetThreadSeed(pending->first_seed);
    auto out = graph->SampleLayersLoop(seeds, fanouts, replace);
    hip::RestoreSeedState(saved);
    pending.reset();
    return out;
  }
}

std::vector<torch::Tensor> Graph::SampleLayers(torch::Tensor seeds, std::vector<int64_t> fanouts,
                                               bool replace) {
  Range range("gs::SampleLayers");
  auto out = SampleLayersIfQueued(seeds, fanouts, replace);
  if (out.empty() && !fanouts.empty()) return SampleLayersLoop(seeds, fanouts, replace);
  return out;
}

std::vector<std::vector<torch::Tensor>> Graph::SampleLayersBatched(
    const std::vector<torch::Tensor>& seed_sets, const std::vector<int64_t>& fanouts,
    bool replace) {
  return QueueSampleLayersBatched(seed_sets, fanouts, replace)->Collect();
}

c10::intrusive_ptr<QueuedSuperBatch> Graph::QueueSampleLayersBatched(
    const std::vector<torch::Tensor>& seed_sets, const std::vector<int64_t>& fanouts,
    bool replace) {
  Range range("gs::SampleLayersBatched");
  Settle();
  TORCH_CHECK(csc_ != nullptr, "fused slicing + sampling needs the CSC format");
  const int64_t B = static_cast<int64_t>(seed_sets.size());
  const int64_t L = static_cast<int64_t>(fanouts.size());
  auto q = c10::make_intrusive<QueuedSuperBatch>();
  q->num_batches = B;
  q->ready.resize(B);
  if (B == 0 || L == 0) return q;
  // what the one launch sequence cannot take goes minibatch by minibatch
  bool one_sequence = !col_ids_.has_value() && !row_ids_.has_value() && !val_col_ids_.has_value() &&
                      hip::DeferredSampling() &&
                      (!data_.has_value() || hip::EdgeData::Fits(data_.value(), csc_->e_ids));
  int64_t bound = 0;
  for (const auto& s : seed_sets) {
    TORCH_CHECK(s.defined() && s.dim() == 1 && s.device() == csc_->indptr.device() &&
                    s.scalar_type() == csc_->indices.scalar_type(),
                "every seed set must be a 1-d tensor of the graph's id type on its device");
    bound += s.numel();
  }
  for (int64_t k : fanouts) {
    one_sequence = one_sequence && !(k == 1 && replace) && hip::OneLaunchApplies(bound, k, replace);
    bound *= 1 + k;
  }
  if (!one_sequence) {
    for (int64_t b = 0; b < B; ++b) q->ready[b] = SampleLayers(seed_sets[b], fanouts, replace);
    return q;
  }
  const bool with_data = data_.has_value();
  q->with_data = with_data;
  const hip::EdgeData edge{with_data ? data_.value() : torch::Tensor(), csc_->e_ids};
  auto pinned = torch::TensorOptions().dtype(torch::kInt64).pinned_memory(true);
  std::vector<int64_t> cut(B + 1, 0);
  for (int64_t b = 0; b < B; ++b) cut[b + 1] = cut[b] + seed_sets[b].numel();
  auto host_ptr = torch::empty({B + 1}, pinned);
  std::copy(cut.begin(), cut.end(), host_ptr.data_ptr<int64_t>());
  torch::Tensor ptr = host_ptr.to(csc_->indptr.device(), /*non_blocking=*/true);
  torch::Tensor seeds = torch::cat(seed_sets);
  q->layers.resize(L);
  // per layer [seed cuts | edge cuts | frontier cuts], B + 1 each: device arrays, all sent to
  // pinned memory by ONE launch behind the last layer (a launch per array after every layer
  // stood between a layer's relabel and the next layer's sampler)
  q->cut_sets.reserve(3 * L);
  for (int64_t l = 0; l < L; ++l) {
    QueuedSuperBatch::Layer& y = q->layers[l];
    const int64_t S = seeds.numel();
    auto p = hip::ColSamplingDeferred(csc_->indptr, csc_->indices, seeds, fanouts[l], replace, false,
                                      false, with_data ? &edge : nullptr);
    // queued behind the sampler while its edge count is on its way: where every minibatch's
    // edges start, and the offsets of every minibatch re-based to its own first edge
    torch::Tensor ids_ptr;
    y.offsets = hip::IndptrSplit(p->sub_indptr, ptr, S + B, &ids_ptr);
    // The relabel is queued behind the sampler with the edge count still on the device (it
    // reads its items' number from the offsets; launches and buffers take the sampler's
    // capacity, which a layer fills to nine tenths and more), so a layer has ONE host wait, for
    // the frontier's length, which sizes the next layer's launches.  Where that form does not
    // apply (ids beyond 32 bits, more than 511 minibatches) or reports a status (a bucket's
    // table full), the edge count is waited for and the relabel done with the exact sizes.
    torch::Tensor uni_ptr;
    int64_t U = -1;
    if (hip::BatchedNoWait())
      std::tie(y.frontier, uni_ptr, y.renamed) =
          hip::BatchCsrRelabelQueued(seeds, ptr, p->indices, ids_ptr, &U, p.get());
    hip::CountBatchedNoWait(U >= 0);
    if (U >= 0) {
      y.frontier = hip::Slice1d(y.frontier, 0, U);
      if (with_data) y.data = p->data;
      y.sample = p;
    } else {
      const int64_t nnz = p->Wait();
      torch::Tensor ids = hip::Slice1d(p->indices, 0, nnz);
      if (with_data) y.data = hip::Slice1d(p->data, 0, nnz);
      std::tie(y.frontier, uni_ptr, y.renamed) = hip::BatchCsrRelabel(seeds, ptr, ids, ids_ptr);
    }
    q->cut_sets.push_back(ptr);
    q->cut_sets.push_back(ids_ptr);
    q->cut_sets.push_back(uni_ptr);
    seeds = y.frontier;
    ptr = uni_ptr;
  }
  // the cuts of all layers go to pinned memory by a small kernel of the library (a copy call of
  // the runtime per array cost the host 30-60 us each, a third of the call)
  q->cuts = torch::empty({3 * L * (B + 1)}, pinned);
  q->posted = std::make_shared<hip::Posted>(hip::PostValueSets(q->cut_sets, q->cuts));
  return q;
}

std::vector<std::vector<torch::Tensor>> QueuedSuperBatch::Collect() {
  TORCH_CHECK(!collected, "this super-batch has been collected already");
  collected = true;
  if (!posted) return std::move(ready);
  // one wait for the cuts of all layers, then views
  hip::WaitPosted(*std::static_pointer_cast<hip::Posted>(posted));
  const int64_t B = num_batches;
  const int64_t L = static_cast<int64_t>(layers.size());
  std::vector<std::vector<torch::Tensor>> out(B);
  for (int64_t b = 0; b < B; ++b) out[b].reserve((with_data ? 4 : 3) * L);
  for (int64_t l = 0; l < L; ++l) {
    const Layer& y = layers[l];
    const int64_t* s_cut = cuts.data_ptr<int64_t>() + 3 * l * (B + 1);
    const int64_t* e_cut = s_cut + (B + 1);
    const int64_t* u_cut = e_cut + (B + 1);
    for (int64_t b = 0; b < B; ++b) {
      out[b].push_back(hip::Slice1d(y.frontier, u_cut[b], u_cut[b + 1] - u_cut[b]));
      out[b].push_back(hip::Slice1d(y.offsets, s_cut[b] + b, s_cut[b + 1] - s_cut[b] + 1));
      out[b].push_back(hip::Slice1d(y.renamed, e_cut[b], e_cut[b + 1] - e_cut[b]));
      if (with_data) out[b].push_back(hip::Slice1d(y.data, e_cut[b], e_cut[b + 1] - e_cut[b]));
    }
  }
  layers.clear();
  cut_sets.clear();
  posted.reset();
  return out;
}

// The reference hands the kernel the GLOBAL ids of the seeds (src/graph.cc:120-128), which
// only works on a graph without id maps, and gathers the parent's edge data with positions
// of the virtual column slice (:131-137).  Here the kernel gets the local seeds and edge
// data follows the position in the parent's indices.
c10::intrusive_ptr<Graph> Graph::FusedBidirSlicing(torch::Tensor column_seeds,
                                                   torch::Tensor row_seeds) {
  Range range("gs::FusedBidirSlicing");
  Settle();
  CreateSparseFormat(_CSC);
  auto ret = Child(Pick(col_ids_, column_seeds), Pick(row_ids_, row_seeds), column_seeds.numel(),
                   row_seeds.numel());
  std::shared_ptr<CSC> sliced;
  torch::Tensor select_index, parent_index;
  std::tie(sliced, select_index) =
      FusedCSCColRowSlicing(csc_, column_seeds, row_seeds, &parent_index);
  ret->SetCSC(sliced);
  ret->SetNumEdges(sliced->indices.numel());
  InheritData(ret.get(), csc_->e_ids, parent_index);
  return ret;
}

c10::intrusive_ptr<Graph> Graph::BatchFusedBidirSlicing(torch::Tensor column_seeds,
                                                        torch::Tensor col_ptr,
                                                        torch::Tensor row_seeds,
                                                        torch::Tensor row_ptr) {
  Settle();
  CreateSparseFormat(_CSC);
  auto ret = Child(Pick(col_ids_, column_seeds), row_ids_, column_seeds.numel(), num_rows_);
  auto sliced = std::make_shared<CSC>();
  torch::Tensor select_index, parent_index;
  std::tie(sliced->indptr, sliced->indices, select_index, parent_index) = hip::ColRowSlicing(
      csc_->indptr, csc_->indices, column_seeds, row_seeds, col_ptr, row_ptr, num_rows_);
  ret->SetCSC(sliced);
  ret->SetNumEdges(sliced->indices.numel());
  InheritData(ret.get(), csc_->e_ids, parent_index);
  return ret;
}

std::tuple<c10::intrusive_ptr<Graph>, torch::Tensor> Graph::BatchSlicing(
    torch::Tensor n_ids, torch::Tensor nid_ptr, int64_t axis, int64_t on_format,
    int64_t output_format, bool relabel, bool encoding) {
  Range range("gs::BatchSlicing");
  Settle();
  TORCH_CHECK(axis == 0, "batch slicing only suppurt column slicing now");  // src/graph.cc:335
  TORCH_CHECK(on_format == _CSC, "Not Implementatin Error");                // src/graph.cc:364
  CreateSparseFormat(_CSC);
  const bool with_coo = output_format & _COO;
  const int64_t num_batches = nid_ptr.numel() - 1;
  torch::optional<torch::Tensor> col_ids =
      col_ids_.has_value() ? col_ids_.value().index({n_ids})
                           : hip::BatchEncode(n_ids, nid_ptr, num_rows_);
  torch::optional<torch::Tensor> row_ids = row_ids_;
  int64_t num_rows = num_rows_ * num_batches;

  std::shared_ptr<_TMP> tmp;
  torch::Tensor select_index;
  std::tie(tmp, select_index) = CSCColSlicing(csc_, n_ids, with_coo, data_.has_value());
  torch::Tensor coo_offsets = tmp->indptr.index({nid_ptr});
  if (encoding) tmp->coo_in_indices = hip::BatchEncode(tmp->coo_in_indices, coo_offsets, num_rows_);
  if (relabel) {
    torch::Tensor frontier;
    std::vector<torch::Tensor> renamed;
    std::tie(frontier, renamed) = BatchTensorRelabel({tmp->coo_in_indices}, {tmp->coo_in_indices});
    tmp->coo_in_indices = renamed[0];
    row_ids = frontier;
    num_rows = frontier.numel();
  }
  auto ret = Child(col_ids, row_ids, n_ids.numel(), num_rows);
  if (output_format & _CSC)
    ret->SetCSC(std::make_shared<CSC>(CSC{tmp->indptr, tmp->coo_in_indices, torch::nullopt}));
  if (with_coo)
    ret->SetCOO(std::make_shared<COO>(
        COO{tmp->coo_in_indices, tmp->coo_in_indptr, torch::nullopt, false, true}));
  ret->SetNumEdges(tmp->coo_in_indices.numel());
  InheritData(ret.get(), csc_->e_ids, select_index);
  return {ret, coo_offsets};
}

std::vector<c10::intrusive_ptr<Graph>> Graph::Split(int64_t split_size) {
  Settle();
  TORCH_CHECK(split_size > 0, "split_size must be positive");
  CreateSparseFormat(_CSC);
  const int64_t n = csc_->indptr.numel() - 1;
  std::vector<int64_t> cuts;
  for (int64_t c = 0; c < n; c += split_size) cuts.push_back(c);
  cuts.push_back(n);
  if (n == 0) return {};
  auto offsets = torch::tensor(cuts, torch::dtype(torch::kInt64)).to(csc_->indptr.device());
  std::vector<torch::Tensor> ptrs = IndptrSplitByOffset(csc_->indptr, offsets);
  std::vector<torch::Tensor> idx = SplitByOffset(csc_->indices, csc_->indptr.index({offsets}));
  std::vector<torch::Tensor> eid, nid;
  if (csc_->e_ids.has_value())
    eid = SplitByOffset(csc_->e_ids.value(), csc_->indptr.index({offsets}));
  if (col_ids_.has_value()) nid = torch::split(col_ids_.value(), split_size);
  std::vector<torch::Tensor> data;
  if (data_.has_value() && !csc_->e_ids.has_value())
    data = SplitByOffset(data_.value(), csc_->indptr.index({offsets}));
  std::vector<c10::intrusive_ptr<Graph>> out;
  for (size_t i = 0; i < ptrs.size(); ++i) {
    auto g = Child(col_ids_.has_value() ? torch::optional<torch::Tensor>(nid[i]) : torch::nullopt,
                   row_ids_, ptrs[i].numel() - 1, num_rows_);
    g->SetCSC(std::make_shared<CSC>(
        CSC{ptrs[i], idx[i],
            csc_->e_ids.has_value() ? torch::optional<torch::Tensor>(eid[i]) : torch::nullopt}));
    g->SetNumEdges(idx[i].numel());
    // the reference drops the edge data here (src/graph.cc:997-1012); a piece keeps its
    // share of it: through the parent's e_ids when there are any, else cut like the edges
    if (data_.has_value()) g->SetData(csc_->e_ids.has_value() ? data_.value() : data[i]);
    out.push_back(g);
  }
  return out;
}

// The reference's guard is inverted (it aborts exactly when the ids are there,
// src/graph.cc:1036-1037); the intent, "needs both id maps", is what is checked here.
void Graph::Decode(int64_t encoding_size) {
  TORCH_CHECK(col_ids_.has_value() && row_ids_.has_value(),
              "Error: Decoding should have both row and column id");
  col_ids_ = hip::BatchDecode(col_ids_.value(), encoding_size);
  row_ids_ = hip::BatchDecode(row_ids_.value(), encoding_size);
}

std::tuple<torch::Tensor, torch::Tensor> Graph::GetBatchCOO() {
  Settle();
  CreateSparseFormat(_COO);
  return {coo_->row, coo_->col};
}

torch::Tensor Graph::RandomWalk(torch::Tensor seeds, int64_t walk_length) {
  Range range("gs::RandomWalk");
  Settle();
  TORCH_CHECK(csc_ != nullptr, "random walks need the CSC format");
  return FusedRandomWalk(csc_, seeds, walk_length);
}

// --------------------------------------------------------- edge-data operators
torch::Tensor Graph::Sum(int64_t axis, int64_t powk, int64_t on_format) {
  Range range("gs::Sum");
  Settle();
  // Sums along the rows (columns) of a graph held as a COO only are added up by edge, straight
  // off the COO, instead of sorting every edge into a CSR (CSC) first: the row probabilities
  // of a layer-wise sampler's column slice are 2.8 M edges over 2.45 M rows.  The same sums,
  // the order of the float additions aside (as on the reference's own COO path, which adds
  // with atomics, src/cuda/graph_ops.cu:45-64).
  // hip::SetOrderedSums(true) keeps the sorted route, whose sums are the same bits every run.
  if (!hip::OrderedSums() &&
      ((axis == 1 && on_format == _CSR && !csr_ && !spare_csr_ && coo_ && !val_row_ids_.has_value()) ||
       (axis == 0 && on_format == _CSC && !csc_ && !spare_csc_ && coo_ && !val_col_ids_.has_value())))
    on_format = _COO;
  CreateSparseFormat(on_format);
  torch::Tensor data = DataOrOnes();
  // one entry per column (axis 0) / row (axis 1) OF THIS GRAPH OBJECT, so a
  // column slice summed along axis 1 yields a vector over all original rows
  torch::Tensor out = torch::zeros({axis == 0 ? num_cols_ : num_rows_}, data.options());
  if (on_format == _COO)
    COOGraphSum(coo_, data, out, powk, 1 - axis);
  else if (axis == 0 && IsCscLike(on_format))
    CSCGraphSum(csc_, val_col_ids_, data, out, powk);
  else if (axis == 1 && IsCsrLike(on_format))
    CSCGraphSum(csr_, val_row_ids_, data, out, powk);
  else
    TORCH_CHECK(false, "axis should be 0 or 1? on_format and axis do not match?");
  return out;
}

c10::intrusive_ptr<Graph> Graph::Normalize(int64_t axis, int64_t on_format) {
  Range range("gs::Normalize");
  Settle();
  CreateSparseFormat(on_format);
  torch::Tensor data = DataOrOnes();
  torch::Tensor out = torch::empty_like(data);
  if (axis == 0 && IsCscLike(on_format))
    hip::SegmentNormalize(csc_->indptr, csc_->e_ids, data, out);
  else if (axis == 1 && IsCsrLike(on_format))
    hip::SegmentNormalize(csr_->indptr, csr_->e_ids, data, out);
  else
    TORCH_CHECK(false, "Not Implementation Error");
  return SameShape(out);
}

c10::intrusive_ptr<Graph> Graph::Divide(torch::Tensor divisor, int64_t axis, int64_t on_format) {
  Range range("gs::Divide");
  Settle();
  CreateSparseFormat(on_format);
  torch::Tensor data = DataOrOnes();
  torch::Tensor out = torch::zeros({num_edges_}, data.options());
  if (on_format == _COO)
    COOGraphDiv(coo_, data, divisor, out, 1 - axis);
  else if (axis == 0 && IsCscLike(on_format))
    CSCGraphDiv(csc_, val_col_ids_, data, divisor, out);
  else if (axis == 1 && IsCsrLike(on_format))
    CSCGraphDiv(csr_, val_row_ids_, data, divisor, out);
  return SameShape(out);
}

std::tuple<c10::intrusive_ptr<Graph>, torch::Tensor> Graph::EDivUSum(torch::Tensor divisor) {
  Range range("gs::EDivUSum");
  Settle();
  CreateSparseFormat(_COO);
  torch::Tensor data = DataOrOnes();
  torch::Tensor out = torch::zeros({num_edges_}, data.options());
  torch::Tensor sum = torch::zeros({num_cols_}, data.options());
  hip::EDivUSum(coo_->row, coo_->col, data, divisor, out, sum);
  return {SameShape(out), sum};
}

// targets: 0 = source (row id), 1 = edge, 2 = destination (column id); on the
// CSR the compressed axis is the row, so 0 and 2 swap (reference src/graph.cc:975-976)
void Graph::SDDMM(const std::string& op, torch::Tensor lhs, torch::Tensor rhs, torch::Tensor out,
                  int64_t lhs_target, int64_t rhs_target, int64_t on_format) {
  Range range("gs::SDDMM");
  Settle();
  CreateSparseFormat(on_format);
  const hip::Bcast b = ToDevice(CalcBcastOff(op, lhs, rhs), out);
  if (on_format == _COO) {
    hip::SddmmCoo(op, b, coo_->row, coo_->col, coo_->e_ids, lhs, rhs, out,
                  static_cast<int>(lhs_target), static_cast<int>(rhs_target));
  } else if (IsCsrLike(on_format)) {
    const int lt = lhs_target == 1 ? 1 : static_cast<int>(2 - lhs_target);
    const int rt = rhs_target == 1 ? 1 : static_cast<int>(2 - rhs_target);
    hip::SddmmCsc(op, b, csr_->indptr, csr_->indices, csr_->e_ids, val_row_ids_, lhs, rhs, out, lt,
                  rt);
  } else if (IsCscLike(on_format)) {
    hip::SddmmCsc(op, b, csc_->indptr, csc_->indices, csc_->e_ids, val_col_ids_, lhs, rhs, out,
                  static_cast<int>(lhs_target), static_cast<int>(rhs_target));
  } else {
    TORCH_CHECK(false, "SDDMM only supports CSR and COO formats");
  }
}

// ---------------------------------------------------------------- node queries
torch::Tensor Graph::AllValidNode() {
  Range range("gs::AllValidNode");
  Settle();
  TORCH_CHECK(col_ids_.has_value(), "For sampling, col_ids_ is necessary!");
  torch::Tensor rows;
  if (row_ids_.has_value()) {
    rows = row_ids_.value();
  } else if (csc_) {
    rows = csc_->indices;
  } else {
    CreateSparseFormat(_COO);
    rows = coo_->row;
  }
  return hip::Unique(torch::cat({col_ids_.value(), rows}));
}

std::tuple<torch::Tensor, int64_t, int64_t, torch::Tensor, torch::Tensor,
           torch::optional<torch::Tensor>, std::string>
Graph::Relabel() {
  Range range("gs::Relabel");
  TORCH_CHECK(col_ids_.has_value(), "For sampling, col_ids_ is necessary!");
  torch::Tensor col_ids = col_ids_.value();
  torch::Tensor frontier;
  std::vector<torch::Tensor> renamed;
  if (pending_ && !row_ids_.has_value()) {
    // straight behind the sampler: its edge count stays on the device until the end
    std::shared_ptr<hip::PendingSample> p = std::move(pending_);
    pending_.reset();
    torch::Tensor indptr_copy, relabeled;  // the copy stands in for indptr.clone()
    int64_t nnz;
    std::tie(frontier, relabeled, nnz, indptr_copy) = hip::RelabelDeferred(col_ids, *p);
    auto csc = std::make_shared<CSC>();
    csc->indptr = p->sub_indptr;
    csc->indices = p->indices.narrow(0, 0, nnz);
    csc_ = csc;
    num_edges_ = nnz;
    if (p->data.defined()) data_ = p->data.narrow(0, 0, nnz);
    return {frontier, frontier.numel(), col_ids.numel(), indptr_copy, relabeled, csc_->e_ids, "csc"};
  }
  Settle();
  if (csc_) {
    // seeds first: the frontier starts with the column ids (reference src/graph.cc:789-811);
    // of a doubly-compressed CSC only the stored columns count (:790-791)
    if (val_col_ids_.has_value()) col_ids = col_ids.index({val_col_ids_.value()});
    torch::Tensor rows = Pick(row_ids_, csc_->indices);
    std::tie(frontier, renamed) = BatchTensorRelabel({col_ids, rows}, {rows});
    return {frontier, frontier.numel(), col_ids.numel(), csc_->indptr.clone(), renamed[0],
            csc_->e_ids, "csc"};
  }
  TORCH_CHECK(csr_ || coo_, "Error in Relabel!");
  CreateSparseFormat(_COO);
  torch::Tensor coo_col = col_ids.index({coo_->col});
  torch::Tensor coo_row = Pick(row_ids_, coo_->row);
  std::tie(frontier, renamed) = BatchTensorRelabel({col_ids, coo_row}, {coo_col, coo_row});
  return {frontier, frontier.numel(), col_ids.numel(), renamed[1], renamed[0], coo_->e_ids, "coo"};
}

torch::Tensor Graph::GetRows() {
  if (row_ids_.has_value()) return row_ids_.value();
  if (!all_rows_.defined() || all_rows_.numel() != num_rows_ ||
      all_rows_.options().dtype() != IdOptions().dtype() ||
      all_rows_.device() != IdOptions().device())
    all_rows_ = torch::arange(num_rows_, IdOptions());
  return all_rows_;
}

torch::Tensor Graph::GetCols() {
  return col_ids_.has_value() ? col_ids_.value() : torch::arange(num_cols_, IdOptions());
}

torch::Tensor Graph::GetValidRows() {
  Settle();
  return Pick(row_ids_, val_row_ids_.has_value() ? val_row_ids_.value()
                                                 : std::get<0>(torch::_unique(GetCOORows(false))));
}

torch::Tensor Graph::GetValidCols() {
  Settle();
  return Pick(col_ids_, val_col_ids_.has_value() ? val_col_ids_.value()
                                                 : std::get<0>(torch::_unique(GetCOOCols(false))));
}

torch::Tensor Graph::GetCOORows(bool is_original) {
  Settle();
  torch::Tensor rows;
  if (coo_) {
    rows = coo_->row;
  } else if (csc_ && !csc_->e_ids.has_value()) {
    rows = csc_->indices;
  } else {
    TORCH_CHECK(csr_ && !csr_->e_ids.has_value(), "Error in GetCOORows!");
    CreateSparseFormat(_COO);
    rows = coo_->row;
  }
  return is_original ? Pick(row_ids_, rows) : rows;
}

torch::Tensor Graph::GetCOOCols(bool is_original) {
  Settle();
  torch::Tensor cols;
  if (coo_) {
    cols = coo_->col;
  } else if (csc_ && !csc_->e_ids.has_value()) {
    CreateSparseFormat(_COO);
    cols = coo_->col;
  } else {
    TORCH_CHECK(csr_ && !csr_->e_ids.has_value(), "Error in GetCOOCols!");
    cols = csr_->indices;
  }
  return is_original ? Pick(col_ids_, cols) : cols;
}

std::vector<torch::Tensor> Graph::MetaData() {
  Settle();
  torch::Tensor col_ids = col_ids_.value_or(torch::Tensor());
  torch::Tensor row_ids = row_ids_.value_or(torch::Tensor());
  if (csc_) return {col_ids, row_ids, DataOrOnes(), csc_->indptr, csc_->indices};
  if (csr_) return {col_ids, row_ids, DataOrOnes(), csr_->indptr, csr_->indices};
  TORCH_CHECK(coo_ != nullptr, "the graph holds no sparse format");
  return {coo_->row, coo_->col};
}

std::vector<torch::Tensor> Graph::COOMetaData() {
  Settle();
  if (!coo_) return {};
  return {col_ids_.value_or(torch::Tensor()), row_ids_.value_or(torch::Tensor()),
          data_.value_or(torch::Tensor()), coo_->row, coo_->col};
}

std::vector<torch::Tensor> Graph::CSCMetaData() {
  Settle();
  if (!csc_) return {};
  return {col_ids_.value_or(torch::Tensor()), row_ids_.value_or(torch::Tensor()),
          data_.value_or(torch::Tensor()), csc_->indptr, csc_->indices};
}

}  // namespace gs
