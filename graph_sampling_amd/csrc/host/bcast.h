// Broadcast offsets for SDDMM operands (the BcastOff / CalcBcastOff API of the
// reference's src/bcast.h:13-57).
#pragma once

#include <torch/torch.h>

#include <string>
#include <vector>

#include "hip_ops.h"

namespace gs {

struct BcastOff {
  // lhs_offset[i] / rhs_offset[i]: which scalar of each operand feeds output
  // position i; empty when the operands need no broadcasting.
  std::vector<int64_t> lhs_offset, rhs_offset;
  bool use_bcast;
  // operand lengths per node/edge, output length, reduction length (dot)
  int64_t lhs_len, rhs_len, out_len, reduce_size;
};

BcastOff CalcBcastOff(const std::string& op, torch::Tensor lhs, torch::Tensor rhs);

// Uploads the offset vectors next to `like` for the kernels.
hip::Bcast ToDevice(const BcastOff& b, const torch::Tensor& like);

}  // namespace gs
