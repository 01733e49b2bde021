#include "tensor_ops.h"

#include <algorithm>

#include "hip_ops.h"

namespace gs {

std::tuple<torch::Tensor, torch::Tensor> ListSampling(torch::Tensor data, int64_t num_picks,
                                                      bool replace) {
  return hip::ListSampling(data, num_picks, replace);
}

std::tuple<torch::Tensor, torch::Tensor> ListSamplingProbs(torch::Tensor data, torch::Tensor probs,
                                                           int64_t num_picks, bool replace) {
  return hip::ListSamplingProbs(data, probs, num_picks, replace);
}

std::vector<torch::Tensor> SplitByOffset(torch::Tensor data, torch::Tensor offset) {
  auto host = offset.to(torch::kCPU).contiguous();
  const int64_t* p = host.data_ptr<int64_t>();
  std::vector<int64_t> sizes;
  for (int64_t i = 0; i + 1 < host.numel(); ++i) sizes.push_back(p[i + 1] - p[i]);
  return torch::split_with_sizes(data, sizes);
}

std::vector<torch::Tensor> IndptrSplitByOffset(torch::Tensor indptr, torch::Tensor offsets) {
  auto host = offsets.to(torch::kCPU).contiguous();
  const int64_t* p = host.data_ptr<int64_t>();
  const int64_t B = host.numel() - 1;
  TORCH_CHECK(B >= 0, "offsets must hold at least one entry");
  std::vector<int64_t> sizes;
  int64_t total = 0;
  for (int64_t i = 0; i < B; ++i) {
    sizes.push_back(p[i + 1] - p[i] + 1);
    total += sizes.back();
  }
  if (B == 0) return {};
  TORCH_CHECK(p[0] == 0, "the first batch must start at column 0");
  return torch::split_with_sizes(hip::IndptrSplit(indptr, offsets.contiguous(), total), sizes);
}

std::vector<torch::Tensor> IndptrSplitBySize(torch::Tensor indptr, int64_t size) {
  TORCH_CHECK(size > 0, "size must be positive");
  const int64_t B = (indptr.numel() - 1) / size;  // a ragged tail is dropped, as in the reference
  auto offsets = torch::arange(B + 1, indptr.options()) * size;
  if (B == 0) return {};
  return torch::split(hip::IndptrSplit(indptr, offsets, B * (size + 1)), size + 1);
}

std::tuple<torch::Tensor, torch::Tensor, torch::Tensor, torch::Tensor> BatchCSRRelabel(
    torch::Tensor seeds, torch::Tensor seeds_ptr, torch::Tensor indices, torch::Tensor indices_ptr) {
  auto r = hip::BatchCsrRelabel(seeds, seeds_ptr, indices, indices_ptr);
  return {std::get<0>(r), std::get<1>(r), std::get<2>(r), indices_ptr};
}

torch::Tensor BatchEncode(torch::Tensor data, torch::Tensor data_ptr, int64_t encoding_size) {
  return hip::BatchEncode(data, data_ptr, encoding_size);
}

torch::Tensor BatchDecode(torch::Tensor in_data, int64_t encoding_size) {
  return hip::BatchDecode(in_data, encoding_size);
}

std::tuple<torch::Tensor, torch::Tensor> GetBatchOffsets(torch::Tensor data, int64_t num_batches,
                                                         int64_t encoding_size) {
  return hip::BatchOffsets(data, num_batches, encoding_size);
}

std::tuple<torch::Tensor, torch::Tensor, torch::Tensor> BatchConcat(
    const std::vector<torch::Tensor>& data_tensors,
    const std::vector<torch::Tensor>& offset_tensors) {
  return hip::BatchConcat(data_tensors, offset_tensors);
}

std::tuple<std::vector<torch::Tensor>, std::vector<torch::Tensor>> BatchSplit(
    torch::Tensor data, torch::Tensor data_ptr, torch::Tensor data_key,
    const std::vector<torch::Tensor>& out_tensors,
    const std::vector<torch::Tensor>& out_ptr_tensors) {
  hip::BatchSplit(data, data_ptr, data_key, out_tensors, out_ptr_tensors);
  return {out_tensors, out_ptr_tensors};
}

namespace {
// batch number of every item of a batched array
torch::Tensor KeysOf(const torch::Tensor& ptr, int64_t n, const torch::Tensor& like) {
  return hip::Csc2CooCols(ptr, n, like);
}
}  // namespace

std::tuple<torch::Tensor, torch::Tensor, torch::Tensor> BatchUnique(torch::Tensor data,
                                                                    torch::Tensor data_ptr) {
  // a relabel with no ids to rename: the frontier of batch b is its distinct values
  auto none = torch::empty({0}, data.options());
  auto none_ptr = torch::zeros_like(data_ptr);
  auto r = hip::BatchCsrRelabel(data, data_ptr, none, none_ptr);
  const torch::Tensor& unique = std::get<0>(r);
  const torch::Tensor& unique_ptr = std::get<1>(r);
  return {unique, unique_ptr, KeysOf(unique_ptr, unique.numel(), unique)};
}

std::tuple<torch::Tensor, torch::Tensor, torch::Tensor> BatchUniqueByKey(torch::Tensor data,
                                                                         torch::Tensor data_ptr,
                                                                         torch::Tensor data_key) {
  TORCH_CHECK(data_key.numel() == data.numel(), "data_key must name the batch of every item");
  return BatchUnique(data, data_ptr);
}

// The reference sorts every batch and then drops equal neighbours over the WHOLE array
// (src/cuda/batch_unique.cu:214-227), so a value that ends one batch and starts the next
// is lost from the second; here every batch keeps its own distinct values.
std::tuple<torch::Tensor, torch::Tensor, torch::Tensor> BatchUnique2(torch::Tensor data,
                                                                     torch::Tensor data_ptr) {
  torch::Tensor unique, unique_ptr, unique_key;
  std::tie(unique, unique_ptr, unique_key) = BatchUnique(data, data_ptr);
  if (unique.numel() == 0) return {unique, unique_ptr, unique_key};
  // order inside the batches: the library's stable radix sort by value, then by batch
  const int64_t span = unique.max().item<int64_t>() + 1;
  const int64_t batches = unique_ptr.numel() - 1;
  torch::Tensor by_value, order;
  std::tie(by_value, order) = hip::SortValuesByKey(unique, unique, span);
  auto batch_of = unique_key.to(unique.scalar_type()).index({order});
  auto sorted = std::get<0>(hip::SortValuesByKey(batch_of, by_value, batches));
  return {sorted, unique_ptr, unique_key};
}

std::tuple<torch::Tensor, torch::Tensor, torch::Tensor> BatchUniqueByKey2(torch::Tensor data,
                                                                          torch::Tensor data_ptr,
                                                                          torch::Tensor data_key) {
  TORCH_CHECK(data_key.numel() == data.numel(), "data_key must name the batch of every item");
  return BatchUnique2(data, data_ptr);
}

std::tuple<torch::Tensor, torch::Tensor, torch::Tensor, torch::Tensor> BatchCSRRelabelByKey(
    torch::Tensor seeds, torch::Tensor seeds_ptr, torch::Tensor seeds_key, torch::Tensor indices,
    torch::Tensor indices_ptr, torch::Tensor indices_key) {
  TORCH_CHECK(seeds_key.numel() == seeds.numel() && indices_key.numel() == indices.numel(),
              "the key tensors must name the batch of every item");
  return BatchCSRRelabel(seeds, seeds_ptr, indices, indices_ptr);
}

std::tuple<torch::Tensor, torch::Tensor, torch::Tensor, torch::Tensor, torch::Tensor>
BatchCOORelabel(torch::Tensor seeds, torch::Tensor seeds_ptr, torch::Tensor coo_col,
                torch::Tensor coo_row, torch::Tensor coo_ptr) {
  auto r = hip::BatchCooRelabel(seeds, seeds_ptr, coo_col, coo_row, coo_ptr);
  return {std::get<0>(r), std::get<1>(r), std::get<2>(r), std::get<3>(r), coo_ptr};
}

std::tuple<torch::Tensor, torch::Tensor, torch::Tensor, torch::Tensor, torch::Tensor>
BatchCOORelabelByKey(torch::Tensor seeds, torch::Tensor seeds_ptr, torch::Tensor seeds_key,
                     torch::Tensor coo_col, torch::Tensor coo_row, torch::Tensor coo_ptr,
                     torch::Tensor coo_key) {
  TORCH_CHECK(seeds_key.numel() == seeds.numel() && coo_key.numel() == coo_row.numel(),
              "the key tensors must name the batch of every item");
  return BatchCOORelabel(seeds, seeds_ptr, coo_col, coo_row, coo_ptr);
}

std::tuple<torch::Tensor, torch::Tensor, torch::Tensor> BatchCOOSlicing(
    int64_t axis, torch::Tensor coo_row, torch::Tensor coo_col, torch::Tensor batch_ptr,
    torch::Tensor neighbors, torch::Tensor neighbors_ptr) {
  TORCH_CHECK(axis == 0 || axis == 1, "axis must be 0 (columns) or 1 (rows)");
  auto r = hip::CooFilter(axis == 0 ? coo_col : coo_row, coo_row, coo_col, batch_ptr, neighbors,
                          neighbors_ptr);
  return {std::get<0>(r), std::get<1>(r), std::get<2>(r)};
}

std::tuple<torch::Tensor, torch::Tensor> COORowSlicingGlobalId(torch::Tensor coo_row,
                                                               torch::Tensor coo_col,
                                                               torch::Tensor row_ids) {
  auto r = hip::CooFilter(coo_row, coo_row, coo_col, torch::nullopt, row_ids, torch::nullopt);
  return {std::get<0>(r), std::get<1>(r)};
}

// One A-Res pick per range, each with a seed of its own.  A range no longer than
// num_picks is taken whole, in order (as ListSamplingProbs does; the reference's batched
// form returns such a range in key order, list_sampling_probs.cu:160-176).
std::tuple<torch::Tensor, torch::Tensor> BatchListSamplingProbs(torch::Tensor probs,
                                                                int64_t num_picks, bool replace,
                                                                torch::Tensor range) {
  TORCH_CHECK(!replace, "Not implemented warning");  // list_sampling_probs.cu:122
  auto host = range.to(torch::kCPU).contiguous();
  const int64_t* p = host.data_ptr<int64_t>();
  const int64_t B = host.numel() - 1;
  TORCH_CHECK(B >= 0, "range must hold at least one offset");
  std::vector<int64_t> out_range(B + 1, 0);
  for (int64_t b = 0; b < B; ++b)
    out_range[b + 1] = out_range[b] + std::min<int64_t>(p[b + 1] - p[b], num_picks);
  auto i64 = torch::dtype(torch::kInt64).device(probs.device());
  auto out_idx = torch::empty({out_range[B]}, i64);
  for (int64_t b = 0; b < B; ++b) {
    const int64_t n = p[b + 1] - p[b];
    if (n == 0) continue;
    auto positions = torch::arange(p[b], p[b + 1], i64);
    auto picked = hip::ListSamplingProbs(positions, probs.narrow(0, p[b], n), num_picks, false);
    out_idx.narrow(0, out_range[b], out_range[b + 1] - out_range[b]).copy_(std::get<0>(picked));
  }
  return {out_idx, torch::tensor(out_range, torch::dtype(torch::kInt64)).to(probs.device())};
}

torch::Tensor IndexSearch(torch::Tensor origin_data, torch::Tensor keys) {
  return hip::IndexSearch(origin_data, keys);
}

}  // namespace gs
