#include "graph_ops.h"

#include "bcast.h"
#include "hip_ops.h"

namespace gs {

namespace {
std::pair<std::shared_ptr<_TMP>, torch::Tensor> Wrap(hip::SliceResult r) {
  auto tmp = std::make_shared<_TMP>();
  tmp->indptr = std::get<0>(r);
  tmp->coo_in_indptr = std::get<1>(r);
  tmp->coo_in_indices = std::get<2>(r);
  return {tmp, std::get<3>(r)};
}
}  // namespace

std::pair<std::shared_ptr<_TMP>, torch::Tensor> CSCColSlicing(std::shared_ptr<CSC> csc,
                                                              torch::Tensor node_ids,
                                                              bool with_coo, bool with_select,
                                                              const hip::EdgeData* edge,
                                                              torch::Tensor* data_out) {
  return Wrap(hip::ColSlicing(csc->indptr, csc->indices, node_ids, with_coo, with_select, edge,
                              data_out));
}

std::pair<std::shared_ptr<_TMP>, torch::Tensor> CSCRowSlicing(std::shared_ptr<CSC> csc,
                                                              torch::Tensor node_ids,
                                                              bool with_coo) {
  return Wrap(hip::RowSlicingCsc(csc->indptr, csc->indices, node_ids, with_coo));
}

// axis 0 keeps edges whose COLUMN is in node_ids, axis 1 edges whose ROW is;
// the kept side is relabelled to the position in node_ids
// (reference src/graph_ops.cc:173-190).
std::pair<std::shared_ptr<COO>, torch::Tensor> COOColSlicing(std::shared_ptr<COO> coo,
                                                             torch::Tensor node_ids, int64_t axis) {
  auto out = std::make_shared<COO>();
  torch::Tensor select_index;
  if (axis == 1)
    std::tie(out->row, out->col, select_index) = hip::RowSlicingCoo(coo->row, coo->col, node_ids);
  else
    std::tie(out->col, out->row, select_index) = hip::RowSlicingCoo(coo->col, coo->row, node_ids);
  out->row_sorted = coo->row_sorted;
  out->col_sorted = coo->col_sorted;
  return {out, select_index};
}

std::pair<std::shared_ptr<_TMP>, torch::Tensor> CSCColSampling(std::shared_ptr<CSC> csc,
                                                               int64_t fanout, bool replace,
                                                               bool with_coo) {
  return Wrap(hip::ColSampling(csc->indptr, csc->indices, torch::Tensor(), fanout, replace, with_coo));
}

std::pair<std::shared_ptr<_TMP>, torch::Tensor> CSCColSamplingProbs(std::shared_ptr<CSC> csc,
                                                                    torch::Tensor edge_probs,
                                                                    int64_t fanout, bool replace,
                                                                    bool with_coo) {
  return Wrap(hip::ColSamplingProbs(csc->indptr, csc->indices, edge_probs, torch::Tensor(), fanout,
                                    replace, with_coo));
}

std::pair<std::shared_ptr<CSC>, torch::Tensor> FusedCSCColSlicingAndSampling(
    std::shared_ptr<CSC> csc, torch::Tensor node_ids, int64_t fanout, bool replace) {
  auto out = std::make_shared<CSC>();
  torch::Tensor select_index;
  if (fanout == 1 && replace) {
    // one slot per column, -1 for an empty one (reference src/graph_ops.cc:228-234)
    std::tie(out->indptr, out->indices, select_index) =
        hip::SampleOneKeepDim(csc->indptr, csc->indices, node_ids);
  } else {
    auto r = hip::ColSampling(csc->indptr, csc->indices, node_ids, fanout, replace, false);
    out->indptr = std::get<0>(r);
    out->indices = std::get<2>(r);
    select_index = std::get<3>(r);
  }
  return {out, select_index};
}

std::pair<std::shared_ptr<CSC>, torch::Tensor> FusedCSCColRowSlicing(
    std::shared_ptr<CSC> csc, torch::Tensor column_ids, torch::Tensor row_ids,
    torch::Tensor* parent_index) {
  auto out = std::make_shared<CSC>();
  torch::Tensor select_index, parent;
  std::tie(out->indptr, out->indices, select_index, parent) =
      hip::ColRowSlicing(csc->indptr, csc->indices, column_ids, row_ids);
  if (parent_index) *parent_index = parent;
  return {out, select_index};
}

torch::Tensor TensorUnique(torch::Tensor node_ids) { return hip::Unique(node_ids); }

std::tuple<torch::Tensor, std::vector<torch::Tensor>> BatchTensorRelabel(
    const std::vector<torch::Tensor>& mapping_tensors,
    const std::vector<torch::Tensor>& to_be_relabeled_tensors) {
  return hip::Relabel(mapping_tensors, to_be_relabeled_tensors);
}

void CSCGraphSum(std::shared_ptr<CSC> csc, torch::optional<torch::Tensor> n_ids, torch::Tensor data,
                 torch::Tensor out_data, int64_t powk) {
  hip::SegmentSum(csc->indptr, csc->e_ids, n_ids, data, out_data, powk);
}

void COOGraphSum(std::shared_ptr<COO> coo, torch::Tensor data, torch::Tensor out_data, int64_t powk,
                 int target_side) {
  hip::CooSum(target_side == 0 ? coo->row : coo->col, coo->e_ids, data, out_data, powk);
}

// data / divisor[segment]: SDDMM "div" with lhs = edge data, rhs = the segment
// side (reference src/graph_ops.cc:291-312).
void CSCGraphDiv(std::shared_ptr<CSC> csc, torch::optional<torch::Tensor> n_ids, torch::Tensor data,
                 torch::Tensor divisor, torch::Tensor out_data) {
  const auto bcast = CalcBcastOff("div", data, divisor);
  hip::SddmmCsc("div", ToDevice(bcast, data), csc->indptr, csc->indices, csc->e_ids, n_ids, data,
                divisor, out_data, 1, 2);
}

void COOGraphDiv(std::shared_ptr<COO> coo, torch::Tensor data, torch::Tensor divisor,
                 torch::Tensor out_data, int target_side) {
  const auto bcast = CalcBcastOff("div", data, divisor);
  hip::SddmmCoo("div", ToDevice(bcast, data), coo->row, coo->col, coo->e_ids, data, divisor,
                out_data, 1, target_side == 0 ? 0 : 2);
}

std::shared_ptr<COO> GraphCSC2COO(std::shared_ptr<CSC> csc, bool CSC2COO) {
  auto coo = std::make_shared<COO>();
  torch::Tensor expanded = hip::Csc2CooCols(csc->indptr, csc->indices.numel(), csc->indices);
  if (CSC2COO) {
    coo->row = csc->indices;
    coo->col = expanded;
    coo->col_sorted = true;
  } else {  // the input is a CSR: offsets run over rows
    coo->row = expanded;
    coo->col = csc->indices;
    coo->row_sorted = true;
  }
  coo->e_ids = csc->e_ids;
  return coo;
}

std::shared_ptr<CSC> GraphCOO2CSC(std::shared_ptr<COO> coo, int64_t num_items, bool COO2CSC) {
  auto csc = std::make_shared<CSC>();
  torch::optional<torch::Tensor> perm;
  if (COO2CSC)
    std::tie(csc->indptr, csc->indices, perm) = hip::Coo2Csc(coo->col, coo->row, num_items, coo->col_sorted);
  else
    std::tie(csc->indptr, csc->indices, perm) = hip::Coo2Csc(coo->row, coo->col, num_items, coo->row_sorted);
  // edge ids follow the sort (reference src/graph_ops.cc:46-54)
  if (coo->e_ids.has_value())
    csc->e_ids = perm.has_value() ? coo->e_ids.value().index({perm.value()}) : coo->e_ids.value();
  else
    csc->e_ids = perm;
  return csc;
}

// sort by the compressed side, then keep only the offsets of the non-empty columns
std::pair<std::shared_ptr<CSC>, torch::Tensor> GraphCOO2DCSC(std::shared_ptr<COO> coo,
                                                             int64_t num_items, bool COO2DCSC) {
  std::shared_ptr<CSC> full = GraphCOO2CSC(coo, num_items, COO2DCSC);
  torch::Tensor val_ids;
  std::tie(full->indptr, val_ids) = hip::CscCompress(full->indptr, full->indices);
  return {full, val_ids};
}

std::shared_ptr<COO> GraphDCSC2COO(std::shared_ptr<CSC> csc, torch::Tensor ids, bool DCSC2COO) {
  auto coo = std::make_shared<COO>();
  torch::Tensor expanded = hip::Dcsc2CooCols(csc->indptr, csc->indices.numel(), ids);
  if (DCSC2COO) {
    coo->row = csc->indices;
    coo->col = expanded;
    coo->col_sorted = true;
  } else {
    coo->row = expanded;
    coo->col = csc->indices;
    coo->row_sorted = true;
  }
  coo->e_ids = csc->e_ids;
  return coo;
}

std::pair<std::shared_ptr<_TMP>, torch::Tensor> DCSCColSlicing(std::shared_ptr<CSC> csc,
                                                               torch::Tensor nid_map,
                                                               torch::Tensor node_ids,
                                                               bool with_coo, bool with_select) {
  return Wrap(hip::DcscColSlicing(csc->indptr, csc->indices, nid_map, node_ids, with_coo,
                                  with_select));
}

torch::Tensor FusedRandomWalk(std::shared_ptr<CSC> csc, torch::Tensor seeds, int64_t walk_length) {
  // flat [walk_length+1][n] buffer handed out with shape [n, walk_length+1]
  // (reference src/cuda/fusion/random_walk.cu:67)
  return hip::RandomWalk(seeds, walk_length, csc->indptr, csc->indices).reshape({seeds.numel(), -1});
}

}  // namespace gs
