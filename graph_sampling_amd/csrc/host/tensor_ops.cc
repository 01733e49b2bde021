#include "tensor_ops.h"

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

}  // namespace gs
