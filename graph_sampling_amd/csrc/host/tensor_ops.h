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

// ---- the rest of the super-batch family (reference src/cuda/tensor_ops.h:41-104).  The
// "ByKey" forms take the batch number of every item next to the offsets; the two say the
// same thing in every caller, and only the offsets are read here.

// data[i] + batch(i) * encoding_size (src/cuda/batch_coding.cu:74)
torch::Tensor BatchEncode(torch::Tensor data, torch::Tensor data_ptr, int64_t encoding_size);
// in[i] mod encoding_size (src/cuda/batch_coding.cu:96)
torch::Tensor BatchDecode(torch::Tensor in_data, int64_t encoding_size);
// (offsets of the batches, decoded data) of encoded data sorted by batch (:110)
std::tuple<torch::Tensor, torch::Tensor> GetBatchOffsets(torch::Tensor data, int64_t num_batches,
                                                         int64_t encoding_size);
// (total, key, total_ptr): batch b of the result = batch b of every input, one after the
// other (src/cuda/batch_concat.cu:117)
std::tuple<torch::Tensor, torch::Tensor, torch::Tensor> BatchConcat(
    const std::vector<torch::Tensor>& data_tensors, const std::vector<torch::Tensor>& offset_tensors);
// the inverse, written into out_tensors (src/cuda/batch_split2.cu:100)
std::tuple<std::vector<torch::Tensor>, std::vector<torch::Tensor>> BatchSplit(
    torch::Tensor data, torch::Tensor data_ptr, torch::Tensor data_key,
    const std::vector<torch::Tensor>& out_tensors, const std::vector<torch::Tensor>& out_ptr_tensors);
// (unique, unique_ptr, unique_key): distinct values of every batch in first-occurrence
// order (src/cuda/batch_unique.cu:203,188)
std::tuple<torch::Tensor, torch::Tensor, torch::Tensor> BatchUnique(torch::Tensor data,
                                                                    torch::Tensor data_ptr);
std::tuple<torch::Tensor, torch::Tensor, torch::Tensor> BatchUniqueByKey(torch::Tensor data,
                                                                         torch::Tensor data_ptr,
                                                                         torch::Tensor data_key);
// the same with every batch's values in ascending order (src/cuda/batch_unique.cu:263,268)
std::tuple<torch::Tensor, torch::Tensor, torch::Tensor> BatchUnique2(torch::Tensor data,
                                                                     torch::Tensor data_ptr);
std::tuple<torch::Tensor, torch::Tensor, torch::Tensor> BatchUniqueByKey2(torch::Tensor data,
                                                                          torch::Tensor data_ptr,
                                                                          torch::Tensor data_key);
std::tuple<torch::Tensor, torch::Tensor, torch::Tensor, torch::Tensor> BatchCSRRelabelByKey(
    torch::Tensor seeds, torch::Tensor seeds_ptr, torch::Tensor seeds_key, torch::Tensor indices,
    torch::Tensor indices_ptr, torch::Tensor indices_key);
// (unique, unique_ptr, relabelled row, relabelled col, coo_ptr) (src/cuda/batch_relabel.cu:482)
std::tuple<torch::Tensor, torch::Tensor, torch::Tensor, torch::Tensor, torch::Tensor>
BatchCOORelabel(torch::Tensor seeds, torch::Tensor seeds_ptr, torch::Tensor coo_col,
                torch::Tensor coo_row, torch::Tensor coo_ptr);
std::tuple<torch::Tensor, torch::Tensor, torch::Tensor, torch::Tensor, torch::Tensor>
BatchCOORelabelByKey(torch::Tensor seeds, torch::Tensor seeds_ptr, torch::Tensor seeds_key,
                     torch::Tensor coo_col, torch::Tensor coo_row, torch::Tensor coo_ptr,
                     torch::Tensor coo_key);
// (row, col, ptr): the edges of every batch whose column (axis 0) / row (axis 1) is among
// the batch's neighbours; ids are kept (src/cuda/batch_slicing.cu:232)
std::tuple<torch::Tensor, torch::Tensor, torch::Tensor> BatchCOOSlicing(
    int64_t axis, torch::Tensor coo_row, torch::Tensor coo_col, torch::Tensor batch_ptr,
    torch::Tensor neighbors, torch::Tensor neighbors_ptr);
// (row, col) of the edges whose row is among row_ids; ids are kept (:325)
std::tuple<torch::Tensor, torch::Tensor> COORowSlicingGlobalId(torch::Tensor coo_row,
                                                               torch::Tensor coo_col,
                                                               torch::Tensor row_ids);
// (positions into probs, offsets): A-Res pick of num_picks items from every range
// (src/cuda/list_sampling_probs.cu:112-183)
std::tuple<torch::Tensor, torch::Tensor> BatchListSamplingProbs(torch::Tensor probs,
                                                                int64_t num_picks, bool replace,
                                                                torch::Tensor range);
// position of every key in origin_data, -1 when absent (src/tensor_ops.cc:24-33)
torch::Tensor IndexSearch(torch::Tensor origin_data, torch::Tensor keys);

}  // namespace gs
