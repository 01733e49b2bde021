#include "bcast.h"

#include <algorithm>

namespace gs {

namespace {

// feature shape of an operand (everything after the node/edge axis), right-aligned to `rank`
// axes with leading ones
std::vector<int64_t> FeatureShape(const torch::Tensor& t, int64_t rank) {
  std::vector<int64_t> shape(static_cast<size_t>(rank), 1);
  const int64_t have = t.dim() - 1;
  for (int64_t d = 0; d < have; ++d) shape[rank - have + d] = t.size(1 + d);
  return shape;
}

int64_t Product(const std::vector<int64_t>& v) {
  int64_t n = 1;
  for (int64_t x : v) n *= x;
  return n;
}

}  // namespace

// Which scalar (for dot: which reduce_size-long vector) of each operand feeds output position
// i, under NumPy broadcasting of the feature shapes; the table the reference builds in
// src/bcast.cc:24-75.  Written per output position: i is taken apart into its coordinates
// (row-major, last axis fastest), and an operand's offset is the row-major index of the same
// coordinates in its own shape, with 0 on every axis it has only one entry of.
BcastOff CalcBcastOff(const std::string& op, torch::Tensor lhs, torch::Tensor rhs) {
  BcastOff b;
  const bool dot = op == "dot";
  const bool copy = op == "copy_lhs" || op == "copy_rhs";
  const int64_t rank = std::max(lhs.dim(), rhs.dim()) - 1;
  std::vector<int64_t> ls = FeatureShape(lhs, rank), rs = FeatureShape(rhs, rank);
  b.lhs_len = Product(ls);
  b.rhs_len = Product(rs);
  b.reduce_size = dot ? lhs.size(lhs.dim() - 1) : 1;
  b.use_bcast = !copy && (lhs.dim() != rhs.dim() || ls != rs);
  if (!b.use_bcast) {
    b.out_len = (op == "copy_rhs" ? b.rhs_len : b.lhs_len) / b.reduce_size;
    return b;
  }
  if (dot) {  // the reduced axis is not an output axis; offsets count whole vectors
    ls.pop_back();
    rs.pop_back();
  }
  std::vector<int64_t> os(ls.size());
  for (size_t d = 0; d < ls.size(); ++d) os[d] = std::max(ls[d], rs[d]);
  b.out_len = Product(os);
  b.lhs_offset.resize(static_cast<size_t>(b.out_len));
  b.rhs_offset.resize(static_cast<size_t>(b.out_len));
  for (int64_t i = 0; i < b.out_len; ++i) {
    int64_t rest = i, at_l = 0, at_r = 0, step_l = 1, step_r = 1;
    for (size_t d = os.size(); d-- > 0;) {
      const int64_t coord = rest % os[d];
      rest /= os[d];
      if (coord < ls[d]) at_l += coord * step_l;
      if (coord < rs[d]) at_r += coord * step_r;
      step_l *= ls[d];
      step_r *= rs[d];
    }
    b.lhs_offset[static_cast<size_t>(i)] = at_l;
    b.rhs_offset[static_cast<size_t>(i)] = at_r;
  }
  return b;
}

hip::Bcast ToDevice(const BcastOff& b, const torch::Tensor& like) {
  hip::Bcast d;
  d.lhs_len = b.lhs_len;
  d.rhs_len = b.rhs_len;
  d.out_len = b.out_len;
  d.reduce_size = b.reduce_size;
  if (b.use_bcast) {
    auto host = torch::dtype(torch::kInt64);
    d.lhs_off = torch::tensor(b.lhs_offset, host).to(like.device());
    d.rhs_off = torch::tensor(b.rhs_offset, host).to(like.device());
  }
  return d;
}

}  // namespace gs
