// Tensor-level operations (API of the reference's src/tensor_ops.h:18-31).
#pragma once

#include <torch/torch.h>

#include <tuple>
#include <vector>

namespace gs {

// Picks num_picks of the items: Algorithm R without replacement, modulo draws
// with replacement.  Returns (selected_data, selected_index).
std::tuple<torch::Tensor, torch::Tensor> ListSampling(torch::Tensor data, int64_t num_picks,
                                                      bool replace);

// A-Res weighted pick without replacement.
std::tuple<torch::Tensor, torch::Tensor> ListSamplingProbs(torch::Tensor data, torch::Tensor probs,
                                                           int64_t num_picks, bool replace);

// data split at the given offsets (offset[i]..offset[i+1])
std::vector<torch::Tensor> SplitByOffset(torch::Tensor data, torch::Tensor offset);

}  // namespace gs
