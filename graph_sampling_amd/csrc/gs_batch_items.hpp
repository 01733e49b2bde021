// The items of a batched ("super-batch") relabel, laid out virtually as
// [seeds_0, ids_0, seeds_1, ids_1, ...] (the order the reference's prefix array has,
// src/cuda/batch_relabel.cu:152,163): shared by the relabel on hash regions (gs_unique.hip)
// and the binned relabel (gs_binrelabel.hip).
#pragma once

#include "gs_common.hpp"

namespace gs {

constexpr int64_t kStagedBatches = 511;  // batch offsets a workgroup keeps in LDS (2 x 4 KB)

template <typename IdT>
struct BatchItems {
  const IdT* seeds;
  const int64_t* seeds_ptr;
  const IdT* ids;
  const int64_t* ids_ptr;
  int64_t B;
  __device__ __forceinline__ int64_t start(int64_t b) const { return seeds_ptr[b] + ids_ptr[b]; }
  // last b in [lo, hi] with start(b) <= i
  __device__ __forceinline__ int64_t batch_of(int64_t i, int64_t lo, int64_t hi) const {
    while (lo < hi) {
      const int64_t mid = (lo + hi + 1) >> 1;
      if (start(mid) <= i) lo = mid; else hi = mid - 1;
    }
    return lo;
  }
  // (one read through a chosen address, not one of two reads: a read that may or may not
  // happen makes every later one wait for all that is in flight)
  __device__ __forceinline__ const IdT* where_in(int64_t b, int64_t i) const {
    const int64_t off = i - start(b);
    const int64_t n_seeds = seeds_ptr[b + 1] - seeds_ptr[b];
    return off < n_seeds ? seeds + seeds_ptr[b] + off : ids + ids_ptr[b] + off - n_seeds;
  }
  __device__ __forceinline__ IdT get_in(int64_t b, int64_t i) const { return *where_in(b, i); }
  // The batch offsets copied into LDS (when there are at most kStagedBatches batches), and
  // this object re-pointed at the copy: the searches and the offset reads that stand between
  // a lane and its key then cost no trip to memory.  Every thread of the workgroup calls it.
  __device__ __forceinline__ void stage_offsets(int64_t* lds_seeds_ptr, int64_t* lds_ids_ptr) {
    if (B > kStagedBatches) return;
    for (int64_t b = threadIdx.x; b <= B; b += blockDim.x) {
      lds_seeds_ptr[b] = seeds_ptr[b];
      lds_ids_ptr[b] = ids_ptr[b];
    }
    __syncthreads();
    seeds_ptr = lds_seeds_ptr;
    ids_ptr = lds_ids_ptr;
  }
  // batches of the first and the last item of a workgroup's range, through LDS
  __device__ __forceinline__ void block_range(int64_t first, int64_t last, int64_t* lds2,
                                              int64_t* lo, int64_t* hi) const {
    if (threadIdx.x < 2) lds2[threadIdx.x] = batch_of(threadIdx.x == 0 ? first : last, 0, B - 1);
    __syncthreads();
    *lo = lds2[0];
    *hi = lds2[1];
  }
};

__device__ __forceinline__ uint32_t hash32(unsigned long long key) {
  return static_cast<uint32_t>((key * 0x9E3779B97F4A7C15ull) >> 32);
}

}  // namespace gs
