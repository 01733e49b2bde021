// Uniform random walks and metapath walks on gfx950, one lane per walker.
//
// Replaces impl::fusion::FusedRandomWalkCUDA (reference
// src/cuda/fusion/random_walk.cu:52) and FusedMetapathRandomWalkCUDA
// (src/cuda/fusion/metapath_random_walk.cu:49).
//
// The trace is step-major, [length+1][n] (random_walk.cu:21,32,42), which is
// also the coalesced layout for one lane per walker: at every step the 64 lanes
// of a wave store 64 consecutive ids.  The walker keeps its current node in a
// register (the reference re-reads it from the trace, random_walk.cu:32).  A
// step is two dependent random reads (the indptr pair, then one neighbour), so
// the kernel is bound by HBM/TLB latency and lives on occupancy: 256 threads
// per workgroup, no LDS, ~24 VGPRs.  One Philox block feeds four steps.
#include "gs_common.hpp"

namespace gs {
namespace {

constexpr int kThreads = 256;

// A node outside [0, num_nodes) has no neighbours (the walker dies there), so a
// stray seed can never turn into a wild read.
template <typename IdT>
__device__ __forceinline__ int64_t step_from(const int64_t* __restrict__ indptr,
                                             const IdT* __restrict__ indices, int64_t num_nodes,
                                             int64_t curr, uint32_t x) {
  if (static_cast<uint64_t>(curr) >= static_cast<uint64_t>(num_nodes)) return -1;
  const int64_t start = indptr[curr];
  const int64_t deg = indptr[curr + 1] - start;
  if (deg <= 0) return -1;
  return static_cast<int64_t>(indices[start + static_cast<int64_t>(x % static_cast<uint32_t>(deg))]);
}

template <typename IdT>
__global__ void __launch_bounds__(kThreads)
random_walk_kernel(const int64_t* __restrict__ indptr, const IdT* __restrict__ indices,
                   int64_t num_nodes, const IdT* __restrict__ seeds, int64_t n, int64_t length, uint64_t seed,
                   const uint32_t* __restrict__ replay, IdT* __restrict__ trace) {
  const int64_t w = static_cast<int64_t>(blockIdx.x) * kThreads + threadIdx.x;
  if (w >= n) return;
  int64_t curr = static_cast<int64_t>(seeds[w]);
  trace[w] = static_cast<IdT>(curr);
  U4 x;
  for (int64_t t = 0; t < length; ++t) {
    if (!replay && (t & 3) == 0)
      x = draw_block(seed, kTagWalk, static_cast<uint64_t>(w), static_cast<uint64_t>(t >> 2));
    int64_t pick = -1;
    if (curr >= 0) {
      const uint32_t xv = replay ? replay[t * n + w] : x.v[t & 3];
      pick = step_from(indptr, indices, num_nodes, curr, xv);
    }
    trace[(t + 1) * n + w] = static_cast<IdT>(pick);
    curr = pick;
  }
}

template <typename IdT>
__global__ void __launch_bounds__(kThreads)
metapath_walk_kernel(const int64_t* const* __restrict__ all_indptr,
                     const IdT* const* __restrict__ all_indices,
                     const int64_t* __restrict__ all_num_nodes,
                     const int64_t* __restrict__ metapath, int64_t length,
                     const IdT* __restrict__ seeds, int64_t n, uint64_t seed,
                     const uint32_t* __restrict__ replay, IdT* __restrict__ trace) {
  const int64_t w = static_cast<int64_t>(blockIdx.x) * kThreads + threadIdx.x;
  if (w >= n) return;
  int64_t curr = static_cast<int64_t>(seeds[w]);
  trace[w] = static_cast<IdT>(curr);
  U4 x;
  for (int64_t t = 0; t < length; ++t) {
    if (!replay && (t & 3) == 0)
      x = draw_block(seed, kTagWalk, static_cast<uint64_t>(w), static_cast<uint64_t>(t >> 2));
    int64_t pick = -1;
    if (curr >= 0) {
      const int64_t rel = metapath[t];  // uniform over the wave: scalar loads
      const uint32_t xv = replay ? replay[t * n + w] : x.v[t & 3];
      pick = step_from(all_indptr[rel], all_indices[rel], all_num_nodes[rel], curr, xv);
    }
    trace[(t + 1) * n + w] = static_cast<IdT>(pick);
    curr = pick;
  }
}

}  // namespace
}  // namespace gs

using namespace gs;

extern "C" {

int gs_random_walk(const int64_t* indptr, int64_t num_nodes, const void* indices, int id_bytes,
                   const void* seeds, int64_t n, int64_t length, uint64_t seed, const uint32_t* replay,
                   void* trace, void* stream) {
  GS_REQUIRE(n >= 0 && length >= 0 && num_nodes >= 0, "gs_random_walk: negative size");
  GS_REQUIRE(n == 0 || (indptr && seeds && trace), "gs_random_walk: null pointer");
  GS_REQUIRE(valid_id_bytes(id_bytes), "gs_random_walk: id_bytes must be 4 or 8, got %d", id_bytes);
  if (n == 0) return GS_OK;
  hipStream_t st = static_cast<hipStream_t>(stream);
  const dim3 grid(blocks_for(n, kThreads));
  ProfileScope prof("random_walk", st);
  if (id_bytes == 8)
    hipLaunchKernelGGL((random_walk_kernel<int64_t>), grid, dim3(kThreads), 0, st, indptr,
                       static_cast<const int64_t*>(indices), num_nodes,
                       static_cast<const int64_t*>(seeds), n, length, seed, replay,
                       static_cast<int64_t*>(trace));
  else
    hipLaunchKernelGGL((random_walk_kernel<int32_t>), grid, dim3(kThreads), 0, st, indptr,
                       static_cast<const int32_t*>(indices), num_nodes,
                       static_cast<const int32_t*>(seeds), n, length, seed, replay,
                       static_cast<int32_t*>(trace));
  return check_launch("random_walk");
}

int gs_metapath_walk(const int64_t* const* all_indptr, const void* const* all_indices,
                     const int64_t* all_num_nodes, int id_bytes, const int64_t* metapath, int64_t length, const void* seeds,
                     int64_t n, uint64_t seed, const uint32_t* replay, void* trace,
                     void* stream) {
  GS_REQUIRE(n >= 0 && length >= 0, "gs_metapath_walk: negative size");
  GS_REQUIRE(n == 0 || (seeds && trace), "gs_metapath_walk: null pointer");
  GS_REQUIRE(n == 0 || length == 0 || (all_indptr && all_indices && all_num_nodes && metapath),
             "gs_metapath_walk: null relation tables");
  GS_REQUIRE(valid_id_bytes(id_bytes), "gs_metapath_walk: id_bytes must be 4 or 8, got %d", id_bytes);
  if (n == 0) return GS_OK;
  hipStream_t st = static_cast<hipStream_t>(stream);
  const dim3 grid(blocks_for(n, kThreads));
  ProfileScope prof("metapath_walk", st);
  if (id_bytes == 8)
    hipLaunchKernelGGL((metapath_walk_kernel<int64_t>), grid, dim3(kThreads), 0, st, all_indptr,
                       reinterpret_cast<const int64_t* const*>(all_indices), all_num_nodes, metapath,
                       length,
                       static_cast<const int64_t*>(seeds), n, seed, replay,
                       static_cast<int64_t*>(trace));
  else
    hipLaunchKernelGGL((metapath_walk_kernel<int32_t>), grid, dim3(kThreads), 0, st, all_indptr,
                       reinterpret_cast<const int32_t* const*>(all_indices), all_num_nodes, metapath,
                       length,
                       static_cast<const int32_t*>(seeds), n, seed, replay,
                       static_cast<int32_t*>(trace));
  return check_launch("metapath_walk");
}

}  // extern "C"
