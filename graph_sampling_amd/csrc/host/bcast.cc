#include "bcast.h"

#include <algorithm>

namespace gs {

namespace {
int64_t FeatureLen(const torch::Tensor& t) {
  int64_t n = 1;
  for (int64_t d = 1; d < t.dim(); ++d) n *= t.size(d);
  return n;
}

// size of feature axis `back` counted from the last one (0 = last); axis 0 of
// the tensor is the node/edge axis and never broadcasts
int64_t AxisFromBack(const torch::Tensor& t, int64_t back) {
  const int64_t d = t.dim() - 1 - back;
  return d < 1 ? 1 : t.size(d);
}
}  // namespace

// Same offsets as the reference's src/bcast.cc:24-75 (NumPy broadcasting of the
// feature shapes, last axis fastest; `dot` keeps its reduction axis out).
BcastOff CalcBcastOff(const std::string& op, torch::Tensor lhs, torch::Tensor rhs) {
  BcastOff b;
  b.lhs_len = FeatureLen(lhs);
  b.rhs_len = FeatureLen(rhs);
  b.reduce_size = 1;
  const bool copy = (op == "copy_lhs" || op == "copy_rhs");
  bool differs = lhs.dim() != rhs.dim();
  for (int64_t d = 1; !differs && d < lhs.dim(); ++d) differs = lhs.size(d) != rhs.size(d);
  b.use_bcast = !copy && differs;
  const bool dot = (op == "dot");
  if (!b.use_bcast) {
    b.out_len = (op == "copy_rhs") ? b.rhs_len : b.lhs_len;
    if (dot) {
      b.reduce_size = lhs.size(lhs.dim() - 1);
      b.out_len /= b.reduce_size;
    }
    return b;
  }
  const int64_t naxes = std::max(lhs.dim(), rhs.dim()) - 1;
  int64_t first = 0;
  if (dot) {
    b.reduce_size = lhs.size(lhs.dim() - 1);
    first = 1;
  }
  b.lhs_offset.assign(1, 0);
  b.rhs_offset.assign(1, 0);
  int64_t out_len = 1, stride_l = 1, stride_r = 1;
  for (int64_t back = first; back < naxes; ++back) {
    const int64_t dl = AxisFromBack(lhs, back), dr = AxisFromBack(rhs, back);
    const int64_t extent = std::max(dl, dr);
    for (int64_t i = 1; i < extent; ++i) {
      for (int64_t k = 0; k < out_len; ++k) {
        b.lhs_offset.push_back(b.lhs_offset[k] + (i < dl ? i * stride_l : 0));
        b.rhs_offset.push_back(b.rhs_offset[k] + (i < dr ? i * stride_r : 0));
      }
    }
    out_len *= extent;
    stride_l *= dl;
    stride_r *= dr;
  }
  b.out_len = out_len;
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
