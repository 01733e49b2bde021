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

// Offsets of a batched CSC cut at the batches' column ranges, each piece re-based to
// start at 0 (reference src/cuda/batch_split.cu:70-94; BySize: equal ranges, :31-46).
std::vector<torch::Tensor> IndptrSplitByOffset(torch::Tensor indptr, torch::Tensor offsets);
std::vector<torch::Tensor> IndptrSplitBySize(torch::Tensor indptr, int64_t size);

// One relabel per batch (reference src/cuda/batch_relabel.cu:331):
// (unique_tensor, unique_tensor_ptr, relabelled indices, indices_ptr).
std::tuple<torch::Tensor, torch::Tensor, torch::Tensor, torch::Tensor> BatchCSRRelabel(
    torch::Tensor seeds, torch::Tensor seeds_ptr, torch::Tensor indices, torch::Tensor indices_ptr);

}  // namespace gs
