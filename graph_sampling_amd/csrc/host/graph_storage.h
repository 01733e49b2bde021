// Sparse-format containers and format flags of the Graph object.
// Same shapes and names as the reference's src/graph_storage.h:9-36 so that
// code written against gs::CSC / gs::COO / _CSC ... compiles unchanged.
#pragma once

#include <torch/torch.h>

namespace gs {

struct CSC {
  torch::Tensor indptr;
  torch::Tensor indices;
  torch::optional<torch::Tensor> e_ids;
};

using CSR = CSC;

struct COO {
  torch::Tensor row;
  torch::Tensor col;
  torch::optional<torch::Tensor> e_ids;
  bool row_sorted = false;
  bool col_sorted = false;
};

// Result of a slice / sample before it is wrapped into a format:
// offsets, the per-edge segment index (COO side of the offsets) and the ids.
struct _TMP {
  torch::Tensor indptr;
  torch::Tensor coo_in_indptr;
  torch::Tensor coo_in_indices;
};

constexpr int64_t _COO = 1;
constexpr int64_t _CSC = 2;
constexpr int64_t _CSR = 4;
constexpr int64_t _DCSC = 8;
constexpr int64_t _DCSR = 16;

}  // namespace gs
