// Segment (SpMV-style) reductions over edge data on gfx950.
//
// Replaces impl::CSCSumCUDA, impl::COOSumCUDA, impl::CSCNormalizeCUDA
// (reference src/cuda/graph_ops.cu:92,122,184) and impl::fusion::COOEDivUSum
// (src/cuda/fusion/edge_map_reduce.cu:10).
//
// The reference gives every segment to one thread (graph_ops.cu:16-39), which
// stalls a whole wave on a power-law hub.  Here a wave owns 64 consecutive
// segments: every lane loads its own (start, end) with one coalesced read of
// the offsets, short segments (<= 32 edges) are summed by their lane in edge
// order (bit-identical to a sequential sum), and each long segment is then
// summed by the whole wave with stride-64 coalesced loads and a butterfly
// reduction.  The typical layer-wise-sampler call has millions of mostly empty
// segments (graph.cc:657: one per graph row), so the common case is exactly
// one coalesced pass over the offsets and one over the output.
#include "gs_common.hpp"

namespace gs {
namespace {

constexpr int kThreads = 256;
constexpr int64_t kLaneMaxLen = 32;

__device__ __forceinline__ float powk_f(float x, int powk) {
  if (powk == 1) return x;  // graph_ops.cu:30
  float p = x;
  for (int i = 1; i < powk; ++i) p *= x;
  return p;
}

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int d = kWave / 2; d > 0; d >>= 1) v += __shfl_xor(v, d, kWave);
  return v;
}

// NORMALIZE = false: out[nmap ? nmap[s] : s] = sum f(data[d])
// NORMALIZE = true : out[d] = data[d] / sum data[d],  d = emap ? emap[e] : e
template <bool NORMALIZE, typename IdT>
__global__ void __launch_bounds__(kThreads)
segment_kernel(const int64_t* __restrict__ indptr, const int64_t* __restrict__ emap,
               const IdT* __restrict__ nmap, const float* __restrict__ data, int64_t num_seg,
               int powk, float* __restrict__ out) {
  const int lane = threadIdx.x & (kWave - 1);
  const int64_t s = static_cast<int64_t>(blockIdx.x) * kThreads + threadIdx.x;
  int64_t begin = 0, end = 0;
  if (s < num_seg) {
    begin = indptr[s];
    end = indptr[s + 1];
  }
  const int64_t len = end - begin;
  float acc = 0.0f;
  if (len <= kLaneMaxLen) {
    for (int64_t e = begin; e < end; ++e) acc += powk_f(data[emap ? emap[e] : e], powk);
  }
  // long segments: one at a time, all 64 lanes
  unsigned long long pending = __ballot(len > kLaneMaxLen);
  while (pending) {
    const int src = __ffsll(static_cast<long long>(pending)) - 1;
    pending &= pending - 1;
    const int64_t b = __shfl(begin, src, kWave);
    const int64_t e_end = __shfl(end, src, kWave);
    float part = 0.0f;
    for (int64_t e = b + lane; e < e_end; e += kWave) part += powk_f(data[emap ? emap[e] : e], powk);
    part = wave_sum(part);
    if (lane == src) acc = part;
    if (NORMALIZE) {
      for (int64_t e = b + lane; e < e_end; e += kWave) {
        const int64_t d = emap ? emap[e] : e;
        out[d] = data[d] / part;
      }
    }
  }
  if (s >= num_seg) return;
  if (NORMALIZE) {
    if (len <= kLaneMaxLen) {
      for (int64_t e = begin; e < end; ++e) {
        const int64_t d = emap ? emap[e] : e;
        out[d] = data[d] / acc;
      }
    }
  } else {
    out[nmap ? static_cast<int64_t>(nmap[s]) : s] = acc;
  }
}

// out[target[e]] += f(data[emap ? emap[e] : e])   (graph_ops.cu:45-64)
template <typename IdT>
__global__ void __launch_bounds__(kThreads)
coo_sum_kernel(const IdT* __restrict__ target, const int64_t* __restrict__ emap,
               const float* __restrict__ data, int64_t E, int powk, float* __restrict__ out) {
  const int64_t e = static_cast<int64_t>(blockIdx.x) * kThreads + threadIdx.x;
  if (e >= E) return;
  atomicAdd(out + target[e], powk_f(data[emap ? emap[e] : e], powk));
}

// edge_map_reduce.cu:15-23
template <typename IdT>
__global__ void __launch_bounds__(kThreads)
e_div_u_sum_kernel(const IdT* __restrict__ row, const IdT* __restrict__ col,
                   const float* __restrict__ data, const float* __restrict__ divisor, int64_t E,
                   float* __restrict__ out_data, float* __restrict__ out_sum) {
  const int64_t e = static_cast<int64_t>(blockIdx.x) * kThreads + threadIdx.x;
  if (e >= E) return;
  const float v = data[e] / divisor[row[e]];
  out_data[e] = v;
  atomicAdd(out_sum + col[e], v);
}

}  // namespace
}  // namespace gs

using namespace gs;

extern "C" {

int gs_segment_sum(const int64_t* indptr, const int64_t* e_ids, const void* n_ids, int id_bytes,
                   const float* data, int64_t num_segments, int64_t powk, float* out,
                   void* stream) {
  GS_REQUIRE(num_segments >= 0 && powk >= 1, "gs_segment_sum: negative size or powk < 1");
  GS_REQUIRE(num_segments == 0 || (indptr && data && out), "gs_segment_sum: null pointer");
  GS_REQUIRE(!n_ids || valid_id_bytes(id_bytes), "gs_segment_sum: id_bytes must be 4 or 8, got %d",
             id_bytes);
  if (num_segments == 0) return GS_OK;
  const dim3 grid(blocks_for(num_segments, kThreads));
  hipStream_t st = static_cast<hipStream_t>(stream);
  if (n_ids && id_bytes == 4)
    hipLaunchKernelGGL((segment_kernel<false, int32_t>), grid, dim3(kThreads), 0, st, indptr, e_ids,
                       static_cast<const int32_t*>(n_ids), data, num_segments,
                       static_cast<int>(powk), out);
  else
    hipLaunchKernelGGL((segment_kernel<false, int64_t>), grid, dim3(kThreads), 0, st, indptr, e_ids,
                       static_cast<const int64_t*>(n_ids), data, num_segments,
                       static_cast<int>(powk), out);
  return check_launch("segment_sum");
}

int gs_coo_sum(const void* target, int id_bytes, const int64_t* e_ids, const float* data, int64_t E,
               int64_t powk, float* out, void* stream) {
  GS_REQUIRE(E >= 0 && powk >= 1, "gs_coo_sum: negative size or powk < 1");
  GS_REQUIRE(E == 0 || (target && data && out), "gs_coo_sum: null pointer");
  GS_REQUIRE(valid_id_bytes(id_bytes), "gs_coo_sum: id_bytes must be 4 or 8, got %d", id_bytes);
  if (E == 0) return GS_OK;
  const dim3 grid(blocks_for(E, kThreads));
  hipStream_t st = static_cast<hipStream_t>(stream);
  if (id_bytes == 8)
    hipLaunchKernelGGL(coo_sum_kernel<int64_t>, grid, dim3(kThreads), 0, st,
                       static_cast<const int64_t*>(target), e_ids, data, E, static_cast<int>(powk),
                       out);
  else
    hipLaunchKernelGGL(coo_sum_kernel<int32_t>, grid, dim3(kThreads), 0, st,
                       static_cast<const int32_t*>(target), e_ids, data, E, static_cast<int>(powk),
                       out);
  return check_launch("coo_sum");
}

int gs_segment_normalize(const int64_t* indptr, const int64_t* e_ids, const float* data,
                         int64_t num_segments, float* out, void* stream) {
  GS_REQUIRE(num_segments >= 0, "gs_segment_normalize: negative size");
  GS_REQUIRE(num_segments == 0 || (indptr && data && out), "gs_segment_normalize: null pointer");
  if (num_segments == 0) return GS_OK;
  hipLaunchKernelGGL((segment_kernel<true, int64_t>), dim3(blocks_for(num_segments, kThreads)),
                     dim3(kThreads), 0, static_cast<hipStream_t>(stream), indptr, e_ids,
                     static_cast<const int64_t*>(nullptr), data, num_segments, 1, out);
  return check_launch("segment_normalize");
}

int gs_e_div_u_sum(const void* row, const void* col, int id_bytes, const float* data,
                   const float* divisor, int64_t E, float* out_data, float* out_sum,
                   void* stream) {
  GS_REQUIRE(E >= 0, "gs_e_div_u_sum: negative size");
  GS_REQUIRE(E == 0 || (row && col && data && divisor && out_data && out_sum),
             "gs_e_div_u_sum: null pointer");
  GS_REQUIRE(valid_id_bytes(id_bytes), "gs_e_div_u_sum: id_bytes must be 4 or 8, got %d", id_bytes);
  if (E == 0) return GS_OK;
  const dim3 grid(blocks_for(E, kThreads));
  hipStream_t st = static_cast<hipStream_t>(stream);
  if (id_bytes == 8)
    hipLaunchKernelGGL(e_div_u_sum_kernel<int64_t>, grid, dim3(kThreads), 0, st,
                       static_cast<const int64_t*>(row), static_cast<const int64_t*>(col), data,
                       divisor, E, out_data, out_sum);
  else
    hipLaunchKernelGGL(e_div_u_sum_kernel<int32_t>, grid, dim3(kThreads), 0, st,
                       static_cast<const int32_t*>(row), static_cast<const int32_t*>(col), data,
                       divisor, E, out_data, out_sum);
  return check_launch("e_div_u_sum");
}

}  // extern "C"
