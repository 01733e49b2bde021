// Segment (SpMV-style) reductions over edge data on gfx950.
//
// Replaces impl::CSCSumCUDA, impl::COOSumCUDA, impl::CSCNormalizeCUDA
// (reference src/cuda/graph_ops.cu:92,122,184) and impl::fusion::COOEDivUSum
// (src/cuda/fusion/edge_map_reduce.cu:10).
//
// The reference gives every segment to one thread (graph_ops.cu:16-39), which
// stalls a whole wave on a power-law hub.  Two decompositions are used here:
//  * by segment, for segments of at most 16 edges: one lane per segment, summed
//    in edge order (bit-identical to a sequential sum).  The typical
//    layer-wise-sampler call has millions of mostly empty segments
//    (graph.cc:657: one per graph row): one coalesced pass over the offsets and
//    one over the output.
//  * by edge, for everything longer: a wave owns 1024 consecutive edges whatever
//    segments they belong to, 64 at a time with coalesced loads; a lane finds
//    the segment of its edge among the offsets the chunk spans, a segmented scan
//    over the lanes folds the edges of one segment, and a run that is still open
//    at the end of a step is carried into the next.  A segment that lies inside
//    the chunk is written at once; the pieces of a segment that crosses chunk
//    borders go to a carry array and are added up, in chunk order, by the chunk
//    that holds the segment's head.  A 300 000-edge hub is thus 290 chunks of
//    work for 290 waves, and the order of the additions is fixed by the layout
//    alone, so results repeat from run to run.
#include "gs_common.hpp"

namespace gs {
namespace {

constexpr int kThreads = 256;
constexpr int kWaves = kThreads / kWave;
constexpr int64_t kLaneMaxLen = 16;
constexpr int64_t kChunk = 1024;  // edges per wave in the by-edge pass

__device__ __forceinline__ float powk_f(float x, int powk) {
  if (powk == 1) return x;  // graph_ops.cu:30
  float p = x;
  for (int i = 1; i < powk; ++i) p *= x;
  return p;
}

// last g in [lo, hi] with indptr[g] <= e
__device__ __forceinline__ int64_t segment_of(const int64_t* __restrict__ indptr, int64_t lo,
                                              int64_t hi, int64_t e) {
  while (lo < hi) {
    const int64_t mid = (lo + hi + 1) >> 1;
    if (indptr[mid] <= e) lo = mid; else hi = mid - 1;
  }
  return lo;
}

// ---- by segment: the short ones.  NORMALIZE writes out[d] = data[d] / sum instead.
template <bool NORMALIZE, typename IdT>
__global__ void __launch_bounds__(kThreads)
short_segments_kernel(const int64_t* __restrict__ indptr, const int64_t* __restrict__ emap,
                      const IdT* __restrict__ nmap, const float* __restrict__ data,
                      int64_t num_seg, int powk, float* __restrict__ out,
                      unsigned int* __restrict__ any_long) {
  const int64_t s = static_cast<int64_t>(blockIdx.x) * kThreads + threadIdx.x;
  int64_t begin = 0, end = 0;
  if (s < num_seg) {
    begin = indptr[s];
    end = indptr[s + 1];
  }
  const int64_t len = end - begin;
  if (__ballot(len > kLaneMaxLen) && (threadIdx.x & (kWave - 1)) == 0) *any_long = 1u;
  if (s >= num_seg || len > kLaneMaxLen) return;
  float acc = 0.0f;
  for (int64_t e = begin; e < end; ++e) acc += powk_f(data[emap ? emap[e] : e], powk);
  if (NORMALIZE) {
    for (int64_t e = begin; e < end; ++e) {
      const int64_t d = emap ? emap[e] : e;
      out[d] = data[d] / acc;
    }
  } else {
    out[nmap ? static_cast<int64_t>(nmap[s]) : s] = acc;
  }
}

__global__ void clear_flag_kernel(unsigned int* flag) {
  if (threadIdx.x == 0) *flag = 0u;
}

// ---- by edge: the long ones.
// Which segment owns an edge is found without a search per edge: every segment that starts
// inside the chunk marks its first edge in an LDS array of one int per edge (empty segments
// share a position; the highest id wins, which is the one that owns the edge), and a running
// maximum over the edges then gives each its segment, relative to the segment of the chunk's
// first edge.
struct ChunkSpan {
  int64_t begin, end, g_lo;
};

__device__ __forceinline__ ChunkSpan mark_heads(const int64_t* __restrict__ indptr,
                                                int64_t num_seg, int64_t nnz, int64_t c, int lane,
                                                int* head) {
  ChunkSpan span;
  span.begin = c * kChunk;
  span.end = span.begin + kChunk < nnz ? span.begin + kChunk : nnz;
  int64_t edge_g = 0;
  if (lane < 2) edge_g = segment_of(indptr, 0, num_seg - 1, lane == 0 ? span.begin : span.end - 1);
  span.g_lo = __shfl(edge_g, 0, kWave);
  const int64_t g_hi = __shfl(edge_g, 1, kWave);
  for (int i = lane; i < kChunk; i += kWave) head[i] = 0;
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_wave_barrier();
  for (int64_t g = span.g_lo + 1 + lane; g <= g_hi; g += kWave)
    atomicMax(&head[indptr[g] - span.begin], static_cast<int>(g - span.g_lo));
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_wave_barrier();
  return span;
}

// segment (relative to g_lo) of the edge at offset `at` of the chunk; carried = the last
// lane's answer of the step before
__device__ __forceinline__ int owner_of(const int* head, int at, bool live, int carried, int lane) {
  int g = live ? head[at] : 0;
#pragma unroll
  for (int d = 1; d < kWave; d <<= 1) {
    const int y = __shfl_up(g, d, kWave);
    if (lane >= d && y > g) g = y;
  }
  return g > carried ? g : carried;
}

// sums is indexed by segment (nmap applied when given); carry holds two floats per chunk:
// [2c] the piece of a segment that began before chunk c, [2c+1] the piece of a segment that
// begins in chunk c and goes on after it.
template <typename IdT>
__global__ void __launch_bounds__(kThreads)
long_segments_kernel(const int64_t* __restrict__ indptr, const int64_t* __restrict__ emap,
                     const IdT* __restrict__ nmap, const float* __restrict__ data,
                     int64_t num_seg, int64_t nnz, int powk, float* __restrict__ sums,
                     float* __restrict__ carry, const unsigned int* __restrict__ any_long) {
  __shared__ int s_head[kWaves][kChunk];
  if (*any_long == 0u) return;
  if (indptr[num_seg] < nnz) nnz = indptr[num_seg];  // the caller's count is an upper bound
  const int lane = threadIdx.x & (kWave - 1);
  const int64_t c = static_cast<int64_t>(blockIdx.x) * kWaves + threadIdx.x / kWave;
  if (c * kChunk >= nnz) return;
  int* head = s_head[threadIdx.x / kWave];
  const ChunkSpan span = mark_heads(indptr, num_seg, nnz, c, lane, head);
  const int64_t begin = span.begin, end = span.end;
  int g_carried = 0;     // segment of the last edge of the step before
  bool open = false;     // that segment's run goes on into this step
  float acc_open = 0.0f;
  float v = begin + lane < end ? powk_f(data[emap ? emap[begin + lane] : begin + lane], powk) : 0.0f;
  for (int64_t base = begin; base < end; base += kWave) {
    const int64_t e = base + lane;
    const bool live = e < end;
    const int64_t en = e + kWave;
    const float v_next = en < end ? powk_f(data[emap ? emap[en] : en], powk) : 0.0f;
    const int g_any = owner_of(head, static_cast<int>(e - begin), live, g_carried, lane);
    const int g = live ? g_any : -1;
    float x = v;
#pragma unroll
    for (int d = 1; d < kWave; d <<= 1) {
      const float y = __shfl_up(x, d, kWave);
      const int gy = __shfl_up(g, d, kWave);
      if (lane >= d && gy == g) x += y;
    }
    const int g_next = __shfl_down(g, 1, kWave);
    const bool run_end = live && (lane == kWave - 1 || g_next != g);
    if (run_end && open && g == g_carried) x += acc_open;  // only the first run can match
    bool closed = false, is_long = false, began_here = false;
    if (run_end) {
      const int64_t seg_b = indptr[span.g_lo + g], seg_e = indptr[span.g_lo + g + 1];
      closed = e == seg_e - 1;
      is_long = seg_e - seg_b > kLaneMaxLen;
      began_here = seg_b >= begin;
      if (closed && is_long) {
        if (began_here) {
          const int64_t gg = span.g_lo + g;
          sums[nmap ? static_cast<int64_t>(nmap[gg]) : gg] = x;
        } else {
          carry[2 * c] = x;
        }
      }
    }
    // at most one run is cut by the end of the step: the last live lane's
    const unsigned long long cut = __ballot(run_end && !closed);
    g_carried = __shfl(g_any, kWave - 1, kWave);  // unused lanes repeat the last edge's
    open = cut != 0;
    if (open) {
      const int src = __ffsll(static_cast<long long>(cut)) - 1;
      acc_open = __shfl(x, src, kWave);
      if (base + kWave >= end) {  // cut by the end of the chunk: hand the piece on
        const int longs = __shfl(static_cast<int>(is_long), src, kWave);
        const int here = __shfl(static_cast<int>(began_here), src, kWave);
        if (longs && lane == 0) carry[here ? 2 * c + 1 : 2 * c] = acc_open;
      }
    }
    v = v_next;
  }
}

// one lane per chunk: a chunk that holds the head of a long segment going on after it adds
// up the pieces, in chunk order
template <typename IdT>
__global__ void __launch_bounds__(kThreads)
carry_kernel(const int64_t* __restrict__ indptr, const IdT* __restrict__ nmap, int64_t num_seg,
             int64_t nnz, const float* __restrict__ carry, float* __restrict__ sums,
             const unsigned int* __restrict__ any_long) {
  if (*any_long == 0u) return;
  if (indptr[num_seg] < nnz) nnz = indptr[num_seg];  // the caller's count is an upper bound
  const int64_t c = static_cast<int64_t>(blockIdx.x) * kThreads + threadIdx.x;
  const int64_t begin = c * kChunk;
  if (begin >= nnz) return;
  const int64_t end = begin + kChunk < nnz ? begin + kChunk : nnz;
  const int64_t g = segment_of(indptr, 0, num_seg - 1, end - 1);
  const int64_t seg_b = indptr[g], seg_e = indptr[g + 1];
  if (seg_e <= end || seg_b < begin || seg_e - seg_b <= kLaneMaxLen) return;
  float total = carry[2 * c + 1];
  for (int64_t k = c + 1; k * kChunk < seg_e; ++k) total += carry[2 * k];
  sums[nmap ? static_cast<int64_t>(nmap[g]) : g] = total;
}

// out[d] = data[d] / sums[segment of e] for the edges of long segments
__global__ void __launch_bounds__(kThreads)
long_divide_kernel(const int64_t* __restrict__ indptr, const int64_t* __restrict__ emap,
                   const float* __restrict__ data, int64_t num_seg, int64_t nnz,
                   const float* __restrict__ sums, float* __restrict__ out,
                   const unsigned int* __restrict__ any_long) {
  __shared__ int s_head[kWaves][kChunk];
  if (*any_long == 0u) return;
  if (indptr[num_seg] < nnz) nnz = indptr[num_seg];  // the caller's count is an upper bound
  const int lane = threadIdx.x & (kWave - 1);
  const int64_t c = static_cast<int64_t>(blockIdx.x) * kWaves + threadIdx.x / kWave;
  if (c * kChunk >= nnz) return;
  int* head = s_head[threadIdx.x / kWave];
  const ChunkSpan span = mark_heads(indptr, num_seg, nnz, c, lane, head);
  int g_carried = 0;
  for (int64_t base = span.begin; base < span.end; base += kWave) {
    const int64_t e = base + lane;
    const bool live = e < span.end;
    const int g = owner_of(head, static_cast<int>(e - span.begin), live, g_carried, lane);
    g_carried = __shfl(g, kWave - 1, kWave);
    if (live) {
      const int64_t gg = span.g_lo + g;
      if (indptr[gg + 1] - indptr[gg] > kLaneMaxLen) {
        const int64_t d = emap ? emap[e] : e;
        out[d] = data[d] / sums[gg];
      }
    }
  }
}

struct SegmentScratch {
  unsigned int* any_long;
  float* carry;
  float* sums;  // normalize only
  bool ok;
};

inline int64_t num_chunks(int64_t nnz) { return nnz <= 0 ? 1 : (nnz + kChunk - 1) / kChunk; }

SegmentScratch carve_segment(void* workspace, size_t bytes, int64_t nnz, int64_t num_seg,
                             bool with_sums) {
  Carver ws(workspace, bytes);
  SegmentScratch s;
  s.any_long = ws.take<unsigned int>(64);
  s.carry = ws.take<float>(2 * num_chunks(nnz));
  s.sums = with_sums ? ws.take<float>(num_seg > 0 ? num_seg : 1) : nullptr;
  s.ok = ws.ok;
  return s;
}

template <typename IdT>
int segment_sum_impl(const int64_t* indptr, const int64_t* emap, const void* nmap,
                     const float* data, int64_t num_seg, int64_t nnz, int powk, float* out,
                     const SegmentScratch& s, hipStream_t st) {
  const IdT* nm = static_cast<const IdT*>(nmap);
  hipLaunchKernelGGL(clear_flag_kernel, dim3(1), dim3(64), 0, st, s.any_long);
  hipLaunchKernelGGL((short_segments_kernel<false, IdT>), dim3(blocks_for(num_seg, kThreads)),
                     dim3(kThreads), 0, st, indptr, emap, nm, data, num_seg, powk, out, s.any_long);
  if (nnz > kLaneMaxLen) {
    const int64_t chunks = num_chunks(nnz);
    hipLaunchKernelGGL(long_segments_kernel<IdT>, dim3(blocks_for(chunks, kWaves)), dim3(kThreads),
                       0, st, indptr, emap, nm, data, num_seg, nnz, powk, out, s.carry, s.any_long);
    hipLaunchKernelGGL(carry_kernel<IdT>, dim3(blocks_for(chunks, kThreads)), dim3(kThreads), 0, st,
                       indptr, nm, num_seg, nnz, s.carry, out, s.any_long);
  }
  return check_launch("segment_sum");
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

size_t gs_segment_workspace_bytes(int64_t num_segments, int64_t nnz) {
  if (num_segments < 1) num_segments = 1;
  return padded(256) + padded(static_cast<size_t>(2 * num_chunks(nnz)) * 4) +
         padded(static_cast<size_t>(num_segments) * 4);
}

int gs_segment_sum(const int64_t* indptr, const int64_t* e_ids, const void* n_ids, int id_bytes,
                   const float* data, int64_t num_segments, int64_t nnz, int64_t powk, float* out,
                   void* workspace, size_t workspace_bytes, void* stream) {
  GS_REQUIRE(num_segments >= 0 && nnz >= 0 && powk >= 1,
             "gs_segment_sum: negative size or powk < 1");
  GS_REQUIRE(num_segments == 0 || (indptr && out && (nnz == 0 || data)),
             "gs_segment_sum: null pointer");
  GS_REQUIRE(!n_ids || valid_id_bytes(id_bytes), "gs_segment_sum: id_bytes must be 4 or 8, got %d",
             id_bytes);
  if (num_segments == 0) return GS_OK;
  SegmentScratch s = carve_segment(workspace, workspace_bytes, nnz, num_segments, false);
  if (!s.ok) {
    set_error_text("gs_segment_sum: workspace needs %zu bytes, 256-byte aligned",
                   gs_segment_workspace_bytes(num_segments, nnz));
    return GS_ERR_WORKSPACE;
  }
  hipStream_t st = static_cast<hipStream_t>(stream);
  return n_ids && id_bytes == 4
             ? segment_sum_impl<int32_t>(indptr, e_ids, n_ids, data, num_segments, nnz,
                                         static_cast<int>(powk), out, s, st)
             : segment_sum_impl<int64_t>(indptr, e_ids, n_ids, data, num_segments, nnz,
                                         static_cast<int>(powk), out, s, st);
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
                         int64_t num_segments, int64_t nnz, float* out, void* workspace,
                         size_t workspace_bytes, void* stream) {
  GS_REQUIRE(num_segments >= 0 && nnz >= 0, "gs_segment_normalize: negative size");
  GS_REQUIRE(num_segments == 0 || nnz == 0 || (indptr && data && out),
             "gs_segment_normalize: null pointer");
  if (num_segments == 0 || nnz == 0) return GS_OK;
  SegmentScratch s = carve_segment(workspace, workspace_bytes, nnz, num_segments, true);
  if (!s.ok) {
    set_error_text("gs_segment_normalize: workspace needs %zu bytes, 256-byte aligned",
                   gs_segment_workspace_bytes(num_segments, nnz));
    return GS_ERR_WORKSPACE;
  }
  hipStream_t st = static_cast<hipStream_t>(stream);
  const int64_t* no_map = nullptr;
  hipLaunchKernelGGL(clear_flag_kernel, dim3(1), dim3(64), 0, st, s.any_long);
  hipLaunchKernelGGL((short_segments_kernel<true, int64_t>), dim3(blocks_for(num_segments, kThreads)),
                     dim3(kThreads), 0, st, indptr, e_ids, no_map, data, num_segments, 1, out,
                     s.any_long);
  if (nnz > kLaneMaxLen) {
    const int64_t chunks = num_chunks(nnz);
    hipLaunchKernelGGL(long_segments_kernel<int64_t>, dim3(blocks_for(chunks, kWaves)),
                       dim3(kThreads), 0, st, indptr, e_ids, no_map, data, num_segments, nnz, 1,
                       s.sums, s.carry, s.any_long);
    hipLaunchKernelGGL(carry_kernel<int64_t>, dim3(blocks_for(chunks, kThreads)), dim3(kThreads), 0,
                       st, indptr, no_map, num_segments, nnz, s.carry, s.sums, s.any_long);
    hipLaunchKernelGGL(long_divide_kernel, dim3(blocks_for(chunks, kWaves)), dim3(kThreads), 0, st,
                       indptr, e_ids, data, num_segments, nnz, s.sums, out, s.any_long);
  }
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
