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

}  // namespace gs
