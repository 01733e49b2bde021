// Column slicing and uniform neighbour sampling for CSC graphs on gfx950.
//
// Replaces impl::CSCColSlicingCUDA (reference src/cuda/slicing.cu:170),
// impl::CSCColSamplingCUDA (src/cuda/sampling.cu:157) and
// impl::fusion::FusedCSCColSlicingSampling[OneKeepDim]CUDA
// (src/cuda/fusion/slice_sampling.cu:146,157).
//
// Layout of the work:
//  * offsets: one tiled exclusive scan whose input (degree or min(degree,k)) is
//    computed on the fly from indptr, so no intermediate degree array exists;
//  * slice fill: edge-balanced -- every workgroup owns 2048 consecutive OUTPUT
//    positions and finds their rows by binary search in an LDS copy of the
//    offsets, so a power-law hub row is spread over many workgroups and all
//    stores are fully coalesced;
//  * sampling, default algorithm (GS_SAMPLE_AUTO): Floyd's k-subset selection,
//    k draws per row however large the row is, 8/16/32/64 lanes per row with the
//    draws in parallel and the duplicate check as a cross-lane broadcast chain;
//  * sampling, GS_SAMPLE_RESERVOIR (the reference's Algorithm R, deg-k draws
//    per row): rows are binned by degree.  k < deg <= 1024 runs inside a 16-lane
//    group with the k slots in LDS (ds_max); larger rows keep their slots in
//    the output buffer and are cut into 4096-draw chunks; the chunks go through
//    a device queue so that a second kernel spreads them evenly over the chip,
//    and a last pass gathers the ids.
#include "gs_common.hpp"

#include <mutex>

#include "gs_table.hpp"

GS_STAMPS_DEFINE(sampling)

namespace gs {
namespace {

// ------------------------------------------------------------- functors ----
// A column id outside [0, num_cols) is treated as an empty column everywhere in
// this file, so that stray ids (e.g. the -1 a dead-end walk step hands back) can
// never turn into a wild read.
__device__ __forceinline__ bool valid_col(int64_t c, int64_t num_cols) {
  return static_cast<uint64_t>(c) < static_cast<uint64_t>(num_cols);
}

// (Read without a branch: an absent id list is read at a stride of zero from the offsets,
// an id outside the graph reads entry 0 twice, and the value is then not used.)
template <typename IdT>
struct ColIds {
  const IdT* from;
  int64_t step;
  bool given;
  __device__ __forceinline__ ColIds(const IdT* cols, const int64_t* indptr)
      : from(cols ? cols : reinterpret_cast<const IdT*>(indptr)), step(cols ? 1 : 0), given(cols) {}
  __device__ __forceinline__ int64_t operator()(int64_t r) const {
    const IdT c = from[r * step];
    return given ? static_cast<int64_t>(c) : r;
  }
};

__device__ __forceinline__ int64_t degree_of(const int64_t* indptr, int64_t c, int64_t num_cols) {
  const bool ok = valid_col(c, num_cols);
  const int64_t lo = indptr[ok ? c : 0], hi = indptr[ok ? c + 1 : 0];
  return ok ? hi - lo : 0;
}

template <typename IdT>
struct ColDegree {
  const int64_t* indptr;
  const IdT* cols;  // nullptr: identity
  int64_t num_cols;
  __device__ __forceinline__ int64_t where(int64_t r) const { return ColIds<IdT>(cols, indptr)(r); }
  __device__ __forceinline__ int64_t count(int64_t c) const { return degree_of(indptr, c, num_cols); }
  __device__ __forceinline__ int64_t operator()(int64_t r) const { return count(where(r)); }
};

template <typename IdT>
struct ColCount {
  const int64_t* indptr;
  const IdT* cols;
  int64_t num_cols;
  int64_t k;
  int replace;
  __device__ __forceinline__ int64_t where(int64_t r) const { return ColIds<IdT>(cols, indptr)(r); }
  __device__ __forceinline__ int64_t count(int64_t c) const {
    const int64_t deg = degree_of(indptr, c, num_cols);
    if (replace) return deg == 0 ? 0 : k;
    return deg < k ? deg : k;
  }
  __device__ __forceinline__ int64_t operator()(int64_t r) const { return count(where(r)); }
};

// first index i in [0, n) with a[i] > v (n if none)
template <typename P>
__device__ __forceinline__ int64_t upper_bound(P a, int64_t n, int64_t v) {
  int64_t lo = 0, hi = n;
  while (lo < hi) {
    int64_t mid = (lo + hi) >> 1;
    if (a[mid] <= v) lo = mid + 1; else hi = mid;
  }
  return lo;
}

// ----------------------------------------------------------- slice fill ----
constexpr int kFillThreads = 256;
constexpr int kFillItems = 8;
constexpr int kFillTile = kFillThreads * kFillItems;
constexpr int kFillStage = 1024;  // rows of offsets staged in LDS

__global__ void post_total_kernel(const int64_t* __restrict__ value, gs_mailbox* box,
                                  int64_t ticket) {
  post_mailbox(box, *value, ticket);
}

// values[0..n) to pinned host memory with system-scope stores, then the mailbox
__global__ void __launch_bounds__(256)
post_values_kernel(const int64_t* __restrict__ values, int64_t n, int64_t* out, gs_mailbox* box,
                   int64_t ticket) {
  for (int64_t i = threadIdx.x; i < n; i += 256)
    __hip_atomic_store(&out[i], values[i], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
  __threadfence_system();
  __syncthreads();
  if (threadIdx.x == 0) post_mailbox(box, n, ticket);
}

// several arrays of n values each, one after the other, by one workgroup
constexpr int kPostSetsMax = 32;
struct PostSets {
  const int64_t* set[kPostSetsMax];
};

__global__ void __launch_bounds__(256)
post_value_sets_kernel(PostSets sets, int num_sets, int64_t n, int64_t* out, gs_mailbox* box,
                       int64_t ticket) {
  for (int s = 0; s < num_sets; ++s) {
    const int64_t* __restrict__ values = sets.set[s];
    for (int64_t i = threadIdx.x; i < n; i += 256)
      __hip_atomic_store(&out[s * n + i], values[i], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
  }
  __threadfence_system();
  __syncthreads();
  if (threadIdx.x == 0) post_mailbox(box, static_cast<int64_t>(num_sets) * n, ticket);
}

template <typename IdT, bool WITH_COO, bool WITH_DATA>
__global__ void __launch_bounds__(kFillThreads)
slice_fill_kernel(const int64_t* __restrict__ indptr, const IdT* __restrict__ indices,
                  const IdT* __restrict__ cols, int64_t num_cols, int64_t S,
                  const int64_t* __restrict__ sub_indptr,
                  int64_t nnz, IdT* __restrict__ sub_indices, int64_t* __restrict__ select_index,
                  IdT* __restrict__ coo_col, const float* __restrict__ edge_data,
                  const int64_t* __restrict__ edge_ids, float* __restrict__ data_out) {
  __shared__ int64_t s_ptr[kFillStage + 1];
  __shared__ int64_t s_in[kFillStage];
  __shared__ int64_t s_rows[2];
  const int64_t p0 = static_cast<int64_t>(blockIdx.x) * kFillTile;
  const int64_t p1 = p0 + kFillTile < nnz ? p0 + kFillTile : nnz;
  block_row_range(sub_indptr, S, p0, p1 - 1, s_rows);
  const int64_t row_lo = s_rows[0];
  const int64_t nrows = s_rows[1] - row_lo + 1;
  const bool staged = nrows <= kFillStage;
  if (staged) {
    for (int64_t i = threadIdx.x; i <= nrows; i += kFillThreads) {
      s_ptr[i] = sub_indptr[row_lo + i];
      if (i < nrows) {
        int64_t c = cols ? static_cast<int64_t>(cols[row_lo + i]) : row_lo + i;
        s_in[i] = valid_col(c, num_cols) ? indptr[c] : 0;  // invalid: empty row, never used
      }
    }
  }
  __syncthreads();
  // where each of the thread's edges comes from, then all the reads, then all the stores: a
  // read issued behind a store waits for it, and eight edges one after the other would wait
  // eight times
  int64_t row[kFillItems], q[kFillItems];
#pragma unroll
  for (int k = 0; k < kFillItems; ++k) {
    int64_t p = p0 + k * kFillThreads + threadIdx.x;
    if (p >= p1) p = p1 - 1;  // (past the end: the last edge again, read but not stored)
    if (staged) {
      int64_t i = upper_bound(s_ptr, nrows + 1, p) - 1;
      row[k] = row_lo + i;
      q[k] = s_in[i] + (p - s_ptr[i]);
    } else {
      row[k] = row_lo + upper_bound(sub_indptr + row_lo, nrows + 1, p) - 1;
      int64_t c = cols ? static_cast<int64_t>(cols[row[k]]) : row[k];  // non-empty row => valid id
      q[k] = indptr[c] + (p - sub_indptr[row[k]]);
    }
  }
  IdT v[kFillItems];
#pragma unroll
  for (int k = 0; k < kFillItems; ++k) v[k] = indices[q[k]];
  // the edges' data along with them (what the reference gathers afterwards from
  // select_index, src/graph.cc:68-73): data[e_ids ? e_ids[q] : q]
  float w[kFillItems];
  if (WITH_DATA) {
    int64_t at[kFillItems];
#pragma unroll
    for (int k = 0; k < kFillItems; ++k) at[k] = q[k];
    if (edge_ids) {
#pragma unroll
      for (int k = 0; k < kFillItems; ++k) at[k] = edge_ids[q[k]];
    }
#pragma unroll
    for (int k = 0; k < kFillItems; ++k) w[k] = edge_data[at[k]];
  }
#pragma unroll
  for (int k = 0; k < kFillItems; ++k) {
    const int64_t p = p0 + k * kFillThreads + threadIdx.x;
    if (p < p1) {
      sub_indices[p] = v[k];
      if (select_index) select_index[p] = q[k];
      if (WITH_COO) coo_col[p] = static_cast<IdT>(row[k]);
      if (WITH_DATA) data_out[p] = w[k];
    }
  }
}

// ------------------------------------------------------------- sampling ----
constexpr int kSampleThreads = 256;
constexpr int kGroup = 16;                                   // lanes per row
constexpr int kGroupsPerBlock = kSampleThreads / kGroup;     // 16
constexpr int kRowsPerBlock = 64;
constexpr int kRounds = kRowsPerBlock / kGroupsPerBlock;     // 4
constexpr int64_t kGroupMaxDeg = 1024;  // larger rows take the chunked path
constexpr int kChunkIters = 4;
constexpr int64_t kChunkDraws = int64_t(kSampleThreads) * 4 * kChunkIters;  // 4096
constexpr int kHubGrid = 2048;           // workgroups draining the chunk queue
constexpr int kChunkBits = 20;           // chunk index bits of a queue entry
constexpr int64_t kQueueExtra = 1 << 20; // queue capacity = S + kQueueExtra chunks
constexpr int64_t kMaxLdsFanout = 768;  // 16 groups * 768 * 4 B = 48 KB

template <typename IdT>
struct SampleArgs {
  const int64_t* indptr;
  const IdT* indices;
  const IdT* cols;
  int64_t num_cols;
  int64_t S;
  int64_t k;
  uint64_t seed;
  const uint32_t* replay;
  const int64_t* replay_ptr;
  const int64_t* sub_indptr;
  IdT* sub_indices;
  int64_t* select_index;
  IdT* coo_col;
  long long* queue;                 // chunk queue entries (row << kChunkBits | chunk), -1 = void
  unsigned long long* queue_count;  // chunks reserved so far (may exceed queue_cap)
  int64_t queue_cap;
};

// Draws idx in [4*q_lo, 4*q_hi) of row r and applies Algorithm R to int64 slots
// in global memory.  `stride` threads cooperate, this one is number `tid`.
template <typename IdT>
__device__ __forceinline__ void reservoir_draws_global(const SampleArgs<IdT>& a, int64_t r,
                                                       int64_t deg, long long* slot,
                                                       int64_t q_lo, int64_t q_hi, int tid,
                                                       int stride) {
  const int64_t k = a.k;
  const uint32_t* rp = a.replay ? a.replay + a.replay_ptr[r] : nullptr;
  for (int64_t q = q_lo + tid; q < q_hi; q += stride) {
    U4 x;
    if (!rp) x = draw_block(a.seed, kTagUniform, static_cast<uint64_t>(r), static_cast<uint64_t>(q));
#pragma unroll
    for (int t = 0; t < 4; ++t) {
      const int64_t idx = q * 4 + t;
      if (idx >= k && idx < deg) {
        const uint32_t xv = rp ? rp[idx - k] : x.v[t];
        const uint32_t num = xv % static_cast<uint32_t>(idx + 1);
        if (static_cast<int64_t>(num) < k) atomicMax(&slot[num], static_cast<long long>(idx));
      }
    }
  }
}

template <typename IdT>
__device__ __forceinline__ void load_row(const SampleArgs<IdT>& a, int64_t r, int64_t* start,
                                         int64_t* deg, int64_t* out_start) {
  int64_t c = a.cols ? static_cast<int64_t>(a.cols[r]) : r;
  if (valid_col(c, a.num_cols)) {
    *start = a.indptr[c];
    *deg = a.indptr[c + 1] - *start;
  } else {
    *start = 0;
    *deg = 0;
  }
  *out_start = a.sub_indptr[r];
}

// Without replacement.  Rows with deg <= k are copied, rows up to kGroupMaxDeg
// run Algorithm R in LDS (when GROUP_TIER), larger rows only get their slots
// initialised (slot j = j, stored in select_index) for the chunked passes.
template <typename IdT, bool WITH_COO, bool GROUP_TIER>
__global__ void __launch_bounds__(kSampleThreads) sample_rows_kernel(SampleArgs<IdT> a) {
  extern __shared__ int32_t s_slots[];
  const int g = threadIdx.x / kGroup;
  const int lane = threadIdx.x % kGroup;
  const int64_t k = a.k;
  int32_t* slot = s_slots + (GROUP_TIER ? g * k : 0);
  for (int round = 0; round < kRounds; ++round) {
    const int64_t r = static_cast<int64_t>(blockIdx.x) * kRowsPerBlock + round * kGroupsPerBlock + g;
    int mode = 0;  // 1 copy, 2 reservoir in LDS, 3 chunked
    int64_t start = 0, deg = 0, out_start = 0;
    if (r < a.S) {
      load_row(a, r, &start, &deg, &out_start);
      mode = deg <= k ? 1 : ((GROUP_TIER && deg <= kGroupMaxDeg) ? 2 : 3);
    }
    if (GROUP_TIER) {
      if (mode == 2)
        for (int64_t j = lane; j < k; j += kGroup) slot[j] = static_cast<int32_t>(j);
      __syncthreads();
      if (mode == 2) {
        const uint32_t* rp = a.replay ? a.replay + a.replay_ptr[r] : nullptr;
        for (int64_t q = (k >> 2) + lane; q <= ((deg - 1) >> 2); q += kGroup) {
          U4 x;
          if (!rp) x = draw_block(a.seed, kTagUniform, static_cast<uint64_t>(r), static_cast<uint64_t>(q));
#pragma unroll
          for (int t = 0; t < 4; ++t) {
            const int64_t idx = q * 4 + t;
            if (idx >= k && idx < deg) {
              const uint32_t xv = rp ? rp[idx - k] : x.v[t];
              const uint32_t num = xv % static_cast<uint32_t>(idx + 1);
              if (static_cast<int64_t>(num) < k) atomicMax(&slot[num], static_cast<int32_t>(idx));
            }
          }
        }
      }
      __syncthreads();
    }
    if (mode == 1) {
      for (int64_t j = lane; j < deg; j += kGroup) {
        a.sub_indices[out_start + j] = a.indices[start + j];
        a.select_index[out_start + j] = start + j;
        if (WITH_COO) a.coo_col[out_start + j] = static_cast<IdT>(r);
      }
    } else if (mode == 2) {
      for (int64_t j = lane; j < k; j += kGroup) {
        const int64_t p = start + slot[j];
        a.sub_indices[out_start + j] = a.indices[p];
        a.select_index[out_start + j] = p;
        if (WITH_COO) a.coo_col[out_start + j] = static_cast<IdT>(r);
      }
    } else if (mode == 3) {
      // slots start as j; the draws are queued as 4096-draw chunks
      for (int64_t j = lane; j < k; j += kGroup) a.select_index[out_start + j] = j;
      const int64_t q_lo = k >> 2, q_hi = ((deg - 1) >> 2) + 1;
      const int64_t q_per_chunk = kChunkDraws / 4;
      const int64_t nchunks = (q_hi - q_lo + q_per_chunk - 1) / q_per_chunk;
      unsigned long long base = 0;
      if (lane == 0) base = atomicAdd(a.queue_count, static_cast<unsigned long long>(nchunks));
      base = __shfl(base, 0, kGroup);
      if (static_cast<int64_t>(base) + nchunks <= a.queue_cap) {
        for (int64_t c = lane; c < nchunks; c += kGroup)
          a.queue[base + c] = static_cast<long long>((r << kChunkBits) | c);
      } else {
        // queue full: void the reserved tail and draw here with this group
        for (int64_t c = static_cast<int64_t>(base) + lane;
             c < a.queue_cap && c < static_cast<int64_t>(base) + nchunks; c += kGroup)
          a.queue[c] = -1;
        __threadfence();
        reservoir_draws_global(a, r, deg, reinterpret_cast<long long*>(a.select_index + out_start),
                               q_lo, q_hi, lane, kGroup);
      }
    }
    if (GROUP_TIER) __syncthreads();
  }
}

// Drains the chunk queue: one workgroup per 4096-draw chunk, grid-stride.
// Slots live in select_index (int64, initialised to j); global atomicMax is
// rare: a draw at position idx hits a slot with probability k/(idx+1).
template <typename IdT>
__global__ void __launch_bounds__(kSampleThreads) sample_hub_draw_kernel(SampleArgs<IdT> a) {
  const unsigned long long reserved = *a.queue_count;
  const int64_t n = reserved < static_cast<unsigned long long>(a.queue_cap)
                        ? static_cast<int64_t>(reserved)
                        : a.queue_cap;
  const int64_t q_per_chunk = kChunkDraws / 4;
  for (int64_t t = blockIdx.x; t < n; t += gridDim.x) {
    const long long e = a.queue[t];
    if (e < 0) continue;
    const int64_t r = e >> kChunkBits;
    const int64_t c = e & ((1 << kChunkBits) - 1);
    int64_t start, deg, out_start;
    load_row(a, r, &start, &deg, &out_start);
    const int64_t q_lo = (a.k >> 2) + c * q_per_chunk;
    int64_t q_hi = ((deg - 1) >> 2) + 1;
    if (q_lo + q_per_chunk < q_hi) q_hi = q_lo + q_per_chunk;
    reservoir_draws_global(a, r, deg, reinterpret_cast<long long*>(a.select_index + out_start),
                           q_lo, q_hi, threadIdx.x, kSampleThreads);
  }
}

static __global__ void zero_counter_kernel(unsigned long long* p) {
  if (threadIdx.x == 0) *p = 0;
}

// Turns the slots of chunked rows into (neighbour id, edge position).
template <typename IdT, bool WITH_COO>
__global__ void __launch_bounds__(kSampleThreads)
sample_hub_gather_kernel(SampleArgs<IdT> a, int64_t min_deg) {
  const int g = threadIdx.x / kGroup;
  const int lane = threadIdx.x % kGroup;
  const int64_t k = a.k;
  for (int round = 0; round < kRounds; ++round) {
    const int64_t r = static_cast<int64_t>(blockIdx.x) * kRowsPerBlock + round * kGroupsPerBlock + g;
    if (r >= a.S) continue;
    int64_t start, deg, out_start;
    load_row(a, r, &start, &deg, &out_start);
    if (!(deg > k && deg > min_deg)) continue;
    for (int64_t j = lane; j < k; j += kGroup) {
      const int64_t p = start + a.select_index[out_start + j];
      a.sub_indices[out_start + j] = a.indices[p];
      a.select_index[out_start + j] = p;
      if (WITH_COO) a.coo_col[out_start + j] = static_cast<IdT>(r);
    }
  }
}


// ------------------------------------------------------- Floyd selection ----
// G lanes (8/16/32/64, >= k) per row.  Lane i owns step i of Floyd's algorithm
// (Bentley & Floyd, CACM 30(9), 1987): j_i = deg-k+i, t_i = draw(r,i) % (j_i+1),
// and the chosen position is t_i unless an earlier step already chose it, in
// which case it is j_i.  All draws and moduli run in parallel; only the k-step
// "already chosen?" chain is sequential, and it is one cross-lane broadcast
// per step (lane m's choice is final once steps 0..m-1 have been broadcast).
// Lane i then writes output i, so a row's outputs are one contiguous run.
constexpr int kFloydThreads = 256;
constexpr int64_t kFloydMaxK = GS_FLOYD_MAX_FANOUT;

template <typename IdT, bool WITH_COO, int G>
__global__ void __launch_bounds__(kFloydThreads) sample_floyd_kernel(SampleArgs<IdT> a) {
  const int lane = threadIdx.x % G;
  const int64_t r = (static_cast<int64_t>(blockIdx.x) * kFloydThreads + threadIdx.x) / G;
  if (r >= a.S) return;
  const int k = static_cast<int>(a.k);
  int64_t start, deg, out_start;
  load_row(a, r, &start, &deg, &out_start);
  if (deg <= k) {
    if (lane < deg) {
      a.sub_indices[out_start + lane] = a.indices[start + lane];
      a.select_index[out_start + lane] = start + lane;
      if (WITH_COO) a.coo_col[out_start + lane] = static_cast<IdT>(r);
    }
    return;
  }
  uint32_t t = 0, j = 0;
  if (lane < k) {
    const uint32_t xv = a.replay ? a.replay[a.replay_ptr[r] + lane]
                                 : draw_one(a.seed, kTagUniform, static_cast<uint64_t>(r),
                                            static_cast<uint64_t>(lane));
    j = static_cast<uint32_t>(deg - k + lane);
    t = xv % (j + 1u);
  }
  bool taken = false;
  for (int m = 0; m < k - 1; ++m) {
    const uint32_t chosen_m = __shfl(taken ? j : t, m, G);
    if (lane > m && t == chosen_m) taken = true;
  }
  if (lane < k) {
    const int64_t q = start + (taken ? j : t);
    a.sub_indices[out_start + lane] = a.indices[q];
    a.select_index[out_start + lane] = q;
    if (WITH_COO) a.coo_col[out_start + lane] = static_cast<IdT>(r);
  }
}

// With replacement: slot j of row r = draw(r, j) % deg (sampling.cu:29-39).
template <typename IdT, bool WITH_COO>
__global__ void __launch_bounds__(kSampleThreads) sample_replace_kernel(SampleArgs<IdT> a) {
  const int g = threadIdx.x / kGroup;
  const int lane = threadIdx.x % kGroup;
  for (int round = 0; round < kRounds; ++round) {
    const int64_t r = static_cast<int64_t>(blockIdx.x) * kRowsPerBlock + round * kGroupsPerBlock + g;
    if (r >= a.S) continue;
    int64_t start, deg, out_start;
    load_row(a, r, &start, &deg, &out_start);
    const int64_t cnt = a.sub_indptr[r + 1] - out_start;
    const uint32_t* rp = a.replay ? a.replay + a.replay_ptr[r] : nullptr;
    for (int64_t q = lane; q * 4 < cnt; q += kGroup) {
      U4 x;
      if (!rp) x = draw_block(a.seed, kTagUniform, static_cast<uint64_t>(r), static_cast<uint64_t>(q));
#pragma unroll
      for (int t = 0; t < 4; ++t) {
        const int64_t j = q * 4 + t;
        if (j < cnt) {
          const uint32_t xv = rp ? rp[j] : x.v[t];
          const int64_t p = start + static_cast<int64_t>(xv % static_cast<uint32_t>(deg));
          a.sub_indices[out_start + j] = a.indices[p];
          a.select_index[out_start + j] = p;
          if (WITH_COO) a.coo_col[out_start + j] = static_cast<IdT>(r);
        }
      }
    }
  }
}

// One slot per column, -1 for an empty column (slice_sampling.cu:171-198).
template <typename IdT>
__global__ void __launch_bounds__(256)
sample_one_keepdim_kernel(const int64_t* __restrict__ indptr, const IdT* __restrict__ indices,
                          const IdT* __restrict__ cols, int64_t num_cols, int64_t S, uint64_t seed,
                          const uint32_t* __restrict__ replay, int64_t* __restrict__ sub_indptr,
                          IdT* __restrict__ sub_indices, int64_t* __restrict__ select_index) {
  const int64_t r = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (r > S) return;
  sub_indptr[r] = r;
  if (r == S) return;
  const int64_t c = static_cast<int64_t>(cols[r]);
  const bool ok = valid_col(c, num_cols);
  const int64_t start = ok ? indptr[c] : 0;
  const int64_t deg = ok ? indptr[c + 1] - start : 0;
  if (deg <= 0) {
    sub_indices[r] = static_cast<IdT>(-1);
    select_index[r] = -1;
  } else {
    const uint32_t x = replay ? replay[r] : draw_one(seed, kTagUniform, static_cast<uint64_t>(r), 0);
    const int64_t p = start + static_cast<int64_t>(x % static_cast<uint32_t>(deg));
    sub_indices[r] = indices[p];
    select_index[r] = p;
  }
}

// ----------------------------------------------------------- host glue -----
template <typename IdT>
int slice_count_impl(const int64_t* indptr, int64_t num_cols, const void* cols, int64_t S,
                     int64_t* sub_indptr, int64_t* tile_ws, hipStream_t stream) {
  ColDegree<IdT> f{indptr, static_cast<const IdT*>(cols), num_cols};
  return exclusive_scan(f, S, sub_indptr, tile_ws, stream);
}

template <typename IdT, bool WITH_COO, bool WITH_DATA>
void slice_fill_launch(const int64_t* indptr, int64_t num_cols, const void* indices,
                       const void* cols, int64_t S, const int64_t* sub_indptr, int64_t nnz,
                       void* sub_indices, int64_t* select_index, void* coo_col,
                       const float* edge_data, const int64_t* edge_ids, float* data_out,
                       hipStream_t stream) {
  const unsigned grid = static_cast<unsigned>((nnz + kFillTile - 1) / kFillTile);
  hipLaunchKernelGGL((slice_fill_kernel<IdT, WITH_COO, WITH_DATA>), dim3(grid), dim3(kFillThreads),
                     0, stream, indptr, static_cast<const IdT*>(indices),
                     static_cast<const IdT*>(cols), num_cols, S, sub_indptr, nnz,
                     static_cast<IdT*>(sub_indices), select_index, static_cast<IdT*>(coo_col),
                     edge_data, edge_ids, data_out);
}

template <typename IdT>
int slice_fill_impl(const int64_t* indptr, int64_t num_cols, const void* indices,
                    const void* cols, int64_t S, const int64_t* sub_indptr, int64_t nnz,
                    void* sub_indices, int64_t* select_index, void* coo_col,
                    const float* edge_data, const int64_t* edge_ids, float* data_out,
                    hipStream_t stream) {
  if (nnz == 0) return GS_OK;
  if (coo_col && data_out)
    slice_fill_launch<IdT, true, true>(indptr, num_cols, indices, cols, S, sub_indptr, nnz,
                                       sub_indices, select_index, coo_col, edge_data, edge_ids,
                                       data_out, stream);
  else if (coo_col)
    slice_fill_launch<IdT, true, false>(indptr, num_cols, indices, cols, S, sub_indptr, nnz,
                                        sub_indices, select_index, coo_col, edge_data, edge_ids,
                                        data_out, stream);
  else if (data_out)
    slice_fill_launch<IdT, false, true>(indptr, num_cols, indices, cols, S, sub_indptr, nnz,
                                        sub_indices, select_index, coo_col, edge_data, edge_ids,
                                        data_out, stream);
  else
    slice_fill_launch<IdT, false, false>(indptr, num_cols, indices, cols, S, sub_indptr, nnz,
                                         sub_indices, select_index, coo_col, edge_data, edge_ids,
                                         data_out, stream);
  return check_launch("slice_fill");
}

template <typename IdT>
int sample_count_impl(const int64_t* indptr, int64_t num_cols, const void* cols, int64_t S,
                      int64_t k, int replace, int64_t* sub_indptr, int64_t* tile_ws,
                      hipStream_t stream) {
  ColCount<IdT> f{indptr, static_cast<const IdT*>(cols), num_cols, k, replace};
  return exclusive_scan(f, S, sub_indptr, tile_ws, stream);
}

template <typename IdT, bool WITH_COO>
int sample_fill_impl(const SampleArgs<IdT>& a, int replace, int algo, hipStream_t stream) {
  if (a.S == 0) return GS_OK;
  const unsigned grid = static_cast<unsigned>((a.S + kRowsPerBlock - 1) / kRowsPerBlock);
  if (replace) {
    hipLaunchKernelGGL((sample_replace_kernel<IdT, WITH_COO>), dim3(grid), dim3(kSampleThreads), 0,
                       stream, a);
    return check_launch("sample_replace");
  }
  if (algo == GS_SAMPLE_AUTO && a.k <= kFloydMaxK) {
    ProfileScope prof("sample_floyd", stream);
    const int g = a.k <= 8 ? 8 : (a.k <= 16 ? 16 : (a.k <= 32 ? 32 : 64));
    const unsigned fgrid =
        static_cast<unsigned>((a.S * g + kFloydThreads - 1) / kFloydThreads);
    if (g == 8)
      hipLaunchKernelGGL((sample_floyd_kernel<IdT, WITH_COO, 8>), dim3(fgrid), dim3(kFloydThreads),
                         0, stream, a);
    else if (g == 16)
      hipLaunchKernelGGL((sample_floyd_kernel<IdT, WITH_COO, 16>), dim3(fgrid), dim3(kFloydThreads),
                         0, stream, a);
    else if (g == 32)
      hipLaunchKernelGGL((sample_floyd_kernel<IdT, WITH_COO, 32>), dim3(fgrid), dim3(kFloydThreads),
                         0, stream, a);
    else
      hipLaunchKernelGGL((sample_floyd_kernel<IdT, WITH_COO, 64>), dim3(fgrid), dim3(kFloydThreads),
                         0, stream, a);
    return check_launch("sample_floyd");
  }
  hipLaunchKernelGGL(zero_counter_kernel, dim3(1), dim3(64), 0, stream, a.queue_count);
  int64_t min_deg;
  if (a.k <= kMaxLdsFanout) {
    const size_t lds = static_cast<size_t>(kGroupsPerBlock) * a.k * sizeof(int32_t);
    hipLaunchKernelGGL((sample_rows_kernel<IdT, WITH_COO, true>), dim3(grid), dim3(kSampleThreads),
                       lds, stream, a);
    min_deg = kGroupMaxDeg;
  } else {
    hipLaunchKernelGGL((sample_rows_kernel<IdT, WITH_COO, false>), dim3(grid),
                       dim3(kSampleThreads), 0, stream, a);
    min_deg = 0;
  }
  hipLaunchKernelGGL((sample_hub_draw_kernel<IdT>), dim3(kHubGrid), dim3(kSampleThreads), 0,
                     stream, a);
  hipLaunchKernelGGL((sample_hub_gather_kernel<IdT, WITH_COO>), dim3(grid), dim3(kSampleThreads),
                     0, stream, a, min_deg);
  return check_launch("sample_rows");
}


// ------------------------------------------- one-launch slice + sample ----
// Counting, the scan of the counts and the fill in ONE kernel.  G lanes share a
// row (G = 1, 2, 4, 8 for a fanout up to 4, 8, 16, 32); a workgroup takes a tile of
// THREADS / G rows:
//  1. every lane of a row reads its column id and offsets (the lanes of a row ask for the
//     same addresses, which cost one request); the tile's counts are scanned and
//     the tile's sum is published for the look-back of the later tiles;
//  2. without replacement the row's lanes run Floyd's selection together: lane s
//     makes the Philox block of draws 4s..4s+3 and reduces them to their ranges
//     (the quarter-rate multiplies and the divisions, the bulk of the arithmetic,
//     spread over the lanes), then the "already chosen?" chain runs step by step
//     with one in-register lane move per step (quad_perm for G <= 4);
//  3. wave 0 walks back over the earlier tiles for the tile's output offset while
//     the other waves already gather;
//  4. lane s gathers and stores outputs 4s..4s+3 of its row: no search for the row
//     of an output, nothing parked in LDS.
// With replacement a lane makes 4 picks per round and a row takes as many rounds
// as its fanout needs.  The outputs must hold S * fanout entries; the true total
// lands in sub_indptr[S] (and in the host mailbox when one is given).  No
// workgroup does a read-modify-write on a shared address (see the look-back
// notes).  Launches of up to 2^17 lanes use 256-thread tiles (a minibatch layer of
// 1024 columns becomes 16 workgroups, not 4), larger ones 1024-thread tiles so that the
// chain of tiles stays short.
constexpr int kGroupThreadsSmall = 256;
constexpr int kGroupThreadsLarge = 1024;
constexpr int64_t kGroupSmallLanes = int64_t(1) << 17;
constexpr int kGroupMaxLanes = 8;

inline int group_lanes_for(int64_t fanout) {
  return fanout <= 4 ? 1 : (fanout <= 8 ? 2 : (fanout <= 16 ? 4 : 8));
}
// A linked launch is sized for a bound on the columns, of which the live ones are usually
// a fraction: it keeps the small tiles up to a larger bound (workgroups beyond the count
// leave at once and take no part in the look-back).
constexpr int64_t kGroupSmallLanesLinked = int64_t(1) << 21;
inline int group_tile_threads(int64_t S, int G, bool linked) {
  return S * G > (linked ? kGroupSmallLanesLinked : kGroupSmallLanes) ? kGroupThreadsLarge
                                                                      : kGroupThreadsSmall;
}
// tiles of the launch that samples S columns with G lanes each
inline int64_t group_tiles(int64_t S, int G, bool linked) {
  const int64_t rows = group_tile_threads(S, G, linked) / G;
  const int64_t tiles = (S + rows - 1) / rows;
  return tiles > 0 ? tiles : 1;
}
// most tiles any fanout can ask for
inline int64_t group_tiles_bound(int64_t S, bool linked) {
  const int64_t large = (S * kGroupMaxLanes + kGroupThreadsLarge - 1) / kGroupThreadsLarge;
  const int64_t small = (linked ? kGroupSmallLanesLinked : kGroupSmallLanes) / kGroupThreadsSmall;
  return (large > small ? large : small) + 1;
}

template <typename IdT>
struct FusedArgs {
  const int64_t* indptr;
  const IdT* indices;
  const IdT* cols;
  int64_t num_cols;
  int64_t S;
  int64_t k;
  uint64_t seed;
  const uint32_t* replay;
  const int64_t* replay_ptr;
  int64_t* sub_indptr;
  IdT* sub_indices;
  int64_t* select_index;
  IdT* coo_col;
  LookbackState lb;
  gs_mailbox* box;
  int64_t box_ticket;
  // LINKED kernels only (gs_layer_sample): the number of columns may live on the device (S is
  // then the bound the launch and the buffers are sized for), and every seed and every
  // sampled id is entered into the hash table of the relabel that follows: item r < S is
  // seed r, item S + e is output e; pos[item] = its slot; *num_edges = the total
  const int64_t* S_dev;
  PackedTable table;
  uint32_t* pos;
  int64_t* num_edges;
  // edge data that follows the samples (reference src/graph.cc:544-557): data_out[o] =
  // edge_data[edge_ids ? edge_ids[q] : q] for the output o taken at position q of `indices`;
  // data_out == nullptr: none
  const float* edge_data;
  const int64_t* edge_ids;
  float* data_out;
};

// Enters `key` as item `item` (one compare-and-swap in the common case); the slot goes to pos.
template <typename IdT>
__device__ __forceinline__ void linked_insert(const PackedTable& t, IdT key, int64_t item,
                                              uint32_t* __restrict__ pos, unsigned int* too_wide) {
  if (sizeof(IdT) == 8 && (static_cast<unsigned long long>(key) >> 32) != 0ull) {
    *too_wide = 2u;  // a 64-bit id that does not fit the one-word slots: reported as -2
    pos[item] = 0u;
    return;
  }
  pos[item] = t.template insert<false>(static_cast<long long>(key), static_cast<uint32_t>(item));
}

// the value lane `owner` of every G-lane group holds (owner is a constant after unrolling)
template <int G>
__device__ __forceinline__ uint32_t group_broadcast(uint32_t v, int owner) {
  if (G == 1) return v;
  const int x = static_cast<int>(v);
  if (G == 2) {  // pairs inside a quad: lanes (0,1) read lane owner, lanes (2,3) lane 2 + owner
    return static_cast<uint32_t>(owner == 0 ? __builtin_amdgcn_update_dpp(0, x, 0xA0, 0xF, 0xF, false)
                                            : __builtin_amdgcn_update_dpp(0, x, 0xF5, 0xF, 0xF, false));
  }
  if (G == 4) {
    switch (owner) {
      case 0: return static_cast<uint32_t>(__builtin_amdgcn_update_dpp(0, x, 0x00, 0xF, 0xF, false));
      case 1: return static_cast<uint32_t>(__builtin_amdgcn_update_dpp(0, x, 0x55, 0xF, 0xF, false));
      case 2: return static_cast<uint32_t>(__builtin_amdgcn_update_dpp(0, x, 0xAA, 0xF, 0xF, false));
      default: return static_cast<uint32_t>(__builtin_amdgcn_update_dpp(0, x, 0xFF, 0xF, 0xF, false));
    }
  }
  return static_cast<uint32_t>(__shfl(x, ((threadIdx.x & (kWave - 1)) & ~(G - 1)) | owner, kWave));
}

template <typename IdT, int G, bool REPLACE, int THREADS, bool LINKED>
__global__ void __launch_bounds__(THREADS) sample_group_kernel(FusedArgs<IdT> a) {
  constexpr int kRows = THREADS / G;
  constexpr int KMAX = 4 * G;
  __shared__ int64_t s_scan[THREADS / kWave + 1];
  __shared__ int64_t s_prefix;
  const unsigned int tile = blockIdx.x;
  unsigned int tiles = gridDim.x;
  const int sub = threadIdx.x & (G - 1);
  const int64_t my_row = static_cast<int64_t>(tile) * kRows + threadIdx.x / G;
  const int k = static_cast<int>(a.k);
  GS_STAMP_BEGIN();
  GS_STAMP(0);

  // ---- 1. the row's column and offsets
  // (with a device-side column count the reads below go by the bound, under which every
  // buffer is sized, and do not wait for the count; what lies beyond it is masked afterwards)
  int64_t start = 0, deg = 0, cnt = 0;
  int64_t c = -1;
  if (my_row < a.S) {
    c = a.cols ? static_cast<int64_t>(a.cols[my_row]) : my_row;
    if (valid_col(c, a.num_cols)) {
      start = a.indptr[c];
      deg = a.indptr[c + 1] - start;
    }
  }
  int64_t S = a.S;
  if (LINKED && a.S_dev) {
    const int64_t s_dev = *a.S_dev;
    S = s_dev < 0 ? 0 : (s_dev < a.S ? s_dev : a.S);
    const int64_t live = (S + kRows - 1) / kRows;
    tiles = static_cast<unsigned int>(live > 0 ? live : 1);
    if (tile >= tiles) return;  // the whole workgroup: nothing of it is below the count
    if (my_row >= S) deg = 0;
  }
  cnt = REPLACE ? (deg > 0 ? a.k : 0) : (deg < a.k ? deg : a.k);
  GS_STAMP(1);  // column id and offsets are here
  int64_t tile_total;
  const int64_t ex = block_exclusive_scan<THREADS>(sub == 0 ? cnt : 0, &tile_total, s_scan);
  const int64_t local = sub == 0 ? ex : ex - cnt;  // the row's first output, relative to the tile's
  if (threadIdx.x == 0) lookback_publish_sum(a.lb, tile, tile_total);
  GS_STAMP(2);  // counts scanned, tile sum published

  // ---- 2. Floyd's selection by the row's lanes: mine[u] = position of output 4*sub+u
  uint32_t mine[4] = {0u, 0u, 0u, 0u};
  if (!REPLACE && cnt > 0) {
    if (deg <= a.k) {
#pragma unroll
      for (int u = 0; u < 4; ++u) mine[u] = static_cast<uint32_t>(4 * sub + u);
    } else {
      const uint32_t lowest = static_cast<uint32_t>(deg - a.k);  // step i draws from [0, lowest + i]
      uint32_t t[4] = {0u, 0u, 0u, 0u};
      if (4 * sub < k) {
        U4 blk;
        if (a.replay) {
          const uint32_t* rp = a.replay + a.replay_ptr[my_row];
#pragma unroll
          for (int u = 0; u < 4; ++u) blk.v[u] = 4 * sub + u < k ? rp[4 * sub + u] : 0u;
        } else {
          blk = draw_block(a.seed, kTagUniform, static_cast<uint64_t>(my_row),
                           static_cast<uint64_t>(sub));
        }
#pragma unroll
        for (int u = 0; u < 4; ++u) t[u] = blk.v[u] % (lowest + static_cast<uint32_t>(4 * sub + u) + 1u);
      }
      uint32_t chosen[KMAX];
#pragma unroll
      for (int i = 0; i < KMAX; ++i) {
        if (i < k) {
          const uint32_t ti = t[i & 3];  // the owner's lane holds the step's draw
          bool taken = false;
#pragma unroll
          for (int m = 0; m < i; ++m) taken |= chosen[m] == ti;
          const uint32_t c = group_broadcast<G>(taken ? lowest + static_cast<uint32_t>(i) : ti, i >> 2);
          chosen[i] = c;
          if (sub == (i >> 2)) mine[i & 3] = c;
        }
      }
    }
  }
  GS_STAMP(3);  // selection done
  if (threadIdx.x < kWave) {
    const int64_t before = lookback_exclusive_prefix(a.lb, tile, tile_total);
    if (threadIdx.x == 0) s_prefix = before;
  }
  GS_STAMP(4);  // look-back done

  // ---- 3. gather: outputs 4*sub .. 4*sub+3 of the row (round 0)
  const IdT* __restrict__ indices = a.indices;
  const uint32_t* rp_replace = REPLACE && a.replay && cnt > 0 ? a.replay + a.replay_ptr[my_row] : nullptr;
  int64_t q[4];
  IdT v[4];
#pragma unroll
  for (int u = 0; u < 4; ++u) q[u] = -1;
  if (cnt > 0) {
    if (REPLACE) {
      U4 blk;
      if (rp_replace) {
#pragma unroll
        for (int u = 0; u < 4; ++u) blk.v[u] = 4 * sub + u < k ? rp_replace[4 * sub + u] : 0u;
      } else {
        blk = draw_block(a.seed, kTagUniform, static_cast<uint64_t>(my_row),
                         static_cast<uint64_t>(sub));
      }
#pragma unroll
      for (int u = 0; u < 4; ++u) mine[u] = blk.v[u] % static_cast<uint32_t>(deg);
    }
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      if (4 * sub + u < cnt) {
        q[u] = start + mine[u];
        v[u] = indices[q[u]];
      }
    }
  }
  // the edge data of the same four picks, asked for while the ids are on their way
  float w[4] = {0.f, 0.f, 0.f, 0.f};
  if (a.data_out && cnt > 0) {
    int64_t at_data[4];
#pragma unroll
    for (int u = 0; u < 4; ++u) at_data[u] = q[u];
    if (a.edge_ids) {
#pragma unroll
      for (int u = 0; u < 4; ++u)
        if (q[u] >= 0) at_data[u] = a.edge_ids[q[u]];
    }
#pragma unroll
    for (int u = 0; u < 4; ++u)
      if (q[u] >= 0) w[u] = a.edge_data[at_data[u]];
  }
  __syncthreads();
  const int64_t out0 = s_prefix;
  GS_STAMP(5);  // the tile's offset is known to every wave, the first gathers are back
  if (my_row < S && sub == 0) a.sub_indptr[my_row] = out0 + local;
  if (tile == tiles - 1 && threadIdx.x == 0) {
    int64_t total = out0 + tile_total;
    if (!LINKED && __hip_atomic_load(a.lb.error, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT))
      total = -1;  // (a linked launch leaves the verdict to the relabel behind it)
    a.sub_indptr[S] = total;
    if (LINKED) *a.num_edges = total;
    post_mailbox(a.box, total, a.box_ticket);
  }
  const int64_t row_out = out0 + local;
#pragma unroll
  for (int u = 0; u < 4; ++u) {
    if (q[u] >= 0) {
      const int64_t o = row_out + 4 * sub + u;
      a.sub_indices[o] = v[u];
      if (a.select_index) a.select_index[o] = q[u];
      if (a.coo_col) a.coo_col[o] = static_cast<IdT>(my_row);
      if (a.data_out) a.data_out[o] = w[u];
    }
  }
  if (LINKED) {
    // the compare-and-swaps of a lane (its four outputs; the row's first lane also enters the
    // seed) go out together; what they found is looked at after
    uint32_t p[4] = {0u, 0u, 0u, 0u}, seed_p = 0u;
    unsigned long long prev[4] = {0ull, 0ull, 0ull, 0ull}, seed_prev = 0ull;
    bool seed_live = sub == 0 && my_row < S;
    if (seed_live) {
      if (sizeof(IdT) == 8 && (static_cast<unsigned long long>(c) >> 32) != 0ull) {
        *a.lb.error = 2u;
        a.pos[my_row] = 0u;
        seed_live = false;
      } else {
        seed_p = a.table.home(c);
        seed_prev = a.table.probe(c, static_cast<uint32_t>(my_row), seed_p);
      }
    }
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      if (q[u] >= 0) {
        if (sizeof(IdT) == 8 && (static_cast<unsigned long long>(v[u]) >> 32) != 0ull) {
          *a.lb.error = 2u;
          a.pos[S + row_out + 4 * sub + u] = 0u;
          q[u] = -1;
        } else {
          p[u] = a.table.home(static_cast<long long>(v[u]));
          prev[u] = a.table.probe(static_cast<long long>(v[u]),
                                  static_cast<uint32_t>(S + row_out + 4 * sub + u), p[u]);
        }
      }
    }
    // What the five compare-and-swaps found is sorted out in rounds over all of them, not item
    // by item: the items that have their slot store it (and lower the index there where
    // theirs is smaller) one after the other with nothing to wait for in between; those that
    // met another key probe the next slot, all together, and come round again.  Item by item,
    // every item's store waited for the one before, because a loop that may issue another
    // compare-and-swap stood between them.
    long long key[5];
    uint32_t item[5], at[5];
    unsigned long long seen[5];
    unsigned int open = 0u;
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      key[u] = static_cast<long long>(v[u]);
      item[u] = static_cast<uint32_t>(S + row_out + 4 * sub + u);
      at[u] = p[u];
      seen[u] = prev[u];
      if (q[u] >= 0) open |= 1u << u;
    }
    key[4] = c;
    item[4] = static_cast<uint32_t>(my_row);
    at[4] = seed_p;
    seen[4] = seed_prev;
    if (seed_live) open |= 1u << 4;
    while (open) {
      // what every open probe found, before anything is stored: the first look waits for the
      // compare-and-swaps, and nothing below reads memory until the next round's probes
      unsigned int home = 0u, down = 0u;
#pragma unroll
      for (int u = 0; u < 5; ++u) {
        if (open >> u & 1u) {
          const unsigned int f = a.table.found(key[u], item[u], seen[u]);
          home |= (f & 1u) << u;
          down |= (f >> 1) << u;
        }
      }
#pragma unroll
      for (int u = 0; u < 5; ++u) {
        if (home >> u & 1u) {
          if (down >> u & 1u) a.table.lower(key[u], item[u], at[u]);
          a.pos[item[u]] = at[u];
        }
      }
      open &= ~home;
#pragma unroll
      for (int u = 0; u < 5; ++u) {
        if (open >> u & 1u) {
          at[u] = (at[u] + 1) & a.table.mask;
          seen[u] = a.table.probe(key[u], item[u], at[u]);
        }
      }
    }
  }
  if (REPLACE) {
    // further rounds of a fanout above 4 * G picks: 4 * G more outputs of the row each
    for (int j0 = KMAX; j0 < cnt; j0 += KMAX) {
      const int j = j0 + 4 * sub;
      U4 blk;
      if (rp_replace) {
#pragma unroll
        for (int u = 0; u < 4; ++u) blk.v[u] = j + u < cnt ? rp_replace[j + u] : 0u;
      } else {
        blk = draw_block(a.seed, kTagUniform, static_cast<uint64_t>(my_row),
                         static_cast<uint64_t>(j >> 2));
      }
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        if (j + u < cnt) {
          const int64_t p = start + blk.v[u] % static_cast<uint32_t>(deg);
          const int64_t o = row_out + j + u;
          const IdT got = indices[p];
          a.sub_indices[o] = got;
          if (a.select_index) a.select_index[o] = p;
          if (a.coo_col) a.coo_col[o] = static_cast<IdT>(my_row);
          if (a.data_out) a.data_out[o] = a.edge_data[a.edge_ids ? a.edge_ids[p] : p];
          if (LINKED) linked_insert<IdT>(a.table, got, S + o, a.pos, a.lb.error);
        }
      }
    }
  }
  GS_STAMP(6);  // stores done
  GS_STAMP_END(1, 7);
}

template <typename IdT, int G, bool REPLACE, bool LINKED>
int sample_group_launch(const FusedArgs<IdT>& a, hipStream_t stream) {
  const unsigned grid = static_cast<unsigned>(group_tiles(a.S, G, LINKED));
  if (group_tile_threads(a.S, G, LINKED) == kGroupThreadsLarge)
    hipLaunchKernelGGL((sample_group_kernel<IdT, G, REPLACE, kGroupThreadsLarge, LINKED>),
                       dim3(grid), dim3(kGroupThreadsLarge), 0, stream, a);
  else
    hipLaunchKernelGGL((sample_group_kernel<IdT, G, REPLACE, kGroupThreadsSmall, LINKED>),
                       dim3(grid), dim3(kGroupThreadsSmall), 0, stream, a);
  return check_launch("sample_fused");
}

template <typename IdT, bool REPLACE, bool LINKED>
int sample_fused_dispatch(const FusedArgs<IdT>& a, hipStream_t stream) {
  switch (group_lanes_for(a.k)) {
    case 1: return sample_group_launch<IdT, 1, REPLACE, LINKED>(a, stream);
    case 2: return sample_group_launch<IdT, 2, REPLACE, LINKED>(a, stream);
    case 4: return sample_group_launch<IdT, 4, REPLACE, LINKED>(a, stream);
    default: return sample_group_launch<IdT, 8, REPLACE, LINKED>(a, stream);
  }
}

// ---- the same launch for very many columns: one row per lane ----
// Above kRowLaneMinColumns the launch is no longer a chain of round trips but a stream, and
// what counts is how many independent gathers are in flight and how the stores coalesce:
// a lane owns a row for the count and for Floyd's selection (positions parked in LDS), then
// the tile's outputs are written edge-parallel -- lane e finds its row by a binary search in
// the LDS offsets, keeps 8 gathers in flight and stores fully coalesced.  (With G lanes per
// row most lanes of a low-degree row idle and every lane stores at a stride: 4.2 M columns,
// fanout 10, 398 us against 257 us.)  Same draws, same outputs.
#ifndef GS_ROW_LANE_MIN_COLUMNS
#define GS_ROW_LANE_MIN_COLUMNS (int64_t(1) << 18)
#endif
constexpr int64_t kRowLaneMinColumns = GS_ROW_LANE_MIN_COLUMNS;
constexpr int kFusedThreads = 256;
constexpr int kFusedRows = 256;
constexpr int kFusedBatch = 8;  // gathers a lane keeps in flight in the fill
constexpr int kPickStride = kFusedRows + 1;  // odd stride: conflict-free by row and by step

template <typename IdT, int KMAX, bool REPLACE>
__global__ void __launch_bounds__(kFusedThreads) sample_row_lane_kernel(FusedArgs<IdT> a) {
  extern __shared__ uint32_t s_pick[];  // [k][kPickStride], without replacement only
  __shared__ int64_t s_start[kFusedRows];
  __shared__ uint32_t s_deg[kFusedRows];
  __shared__ uint32_t s_rel[kFusedRows + 1];  // output offsets relative to the tile's first
  __shared__ int64_t s_scan[kFusedThreads / kWave + 1];
  __shared__ int64_t s_prefix;
  const unsigned int tile = blockIdx.x;
  const unsigned int tiles = gridDim.x;
  const int64_t row0 = static_cast<int64_t>(tile) * kFusedRows;
  const int k = static_cast<int>(a.k);
  const int64_t my_row = row0 + threadIdx.x;

  // ---- 1. one row per lane
  int64_t start = 0, deg = 0, cnt = 0;
  if (my_row < a.S) {
    const int64_t c = a.cols ? static_cast<int64_t>(a.cols[my_row]) : my_row;
    if (valid_col(c, a.num_cols)) {
      start = a.indptr[c];
      deg = a.indptr[c + 1] - start;
    }
    cnt = REPLACE ? (deg > 0 ? a.k : 0) : (deg < a.k ? deg : a.k);
  }
  int64_t tile_total;
  const int64_t local = block_exclusive_scan<kFusedThreads>(cnt, &tile_total, s_scan);
  if (threadIdx.x == 0) lookback_publish_sum(a.lb, tile, tile_total);
  s_start[threadIdx.x] = start;
  s_deg[threadIdx.x] = static_cast<uint32_t>(deg);
  s_rel[threadIdx.x] = static_cast<uint32_t>(local);
  if (threadIdx.x == 0) s_rel[kFusedRows] = static_cast<uint32_t>(tile_total);

  // ---- 2. Floyd's selection, one row per lane, positions to LDS
  if (!REPLACE && cnt > 0) {
    if (deg <= a.k) {
      for (int i = 0; i < static_cast<int>(deg); ++i) s_pick[i * kPickStride + threadIdx.x] = i;
    } else {
      const uint32_t* rp = a.replay ? a.replay + a.replay_ptr[my_row] : nullptr;
      uint32_t chosen[KMAX];
      U4 blk;
#pragma unroll
      for (int i = 0; i < KMAX; ++i) {
        if (i < k) {
          if ((i & 3) == 0 && !rp)
            blk = draw_block(a.seed, kTagUniform, static_cast<uint64_t>(my_row),
                             static_cast<uint64_t>(i >> 2));
          const uint32_t xv = rp ? rp[i] : blk.v[i & 3];
          const uint32_t j = static_cast<uint32_t>(deg - a.k + i);
          const uint32_t t = xv % (j + 1u);
          bool taken = false;
#pragma unroll
          for (int m = 0; m < i; ++m) taken |= chosen[m] == t;
          chosen[i] = taken ? j : t;
          s_pick[i * kPickStride + threadIdx.x] = chosen[i];
        }
      }
    }
  }
  if (threadIdx.x < kWave) {
    const int64_t before = lookback_exclusive_prefix(a.lb, tile, tile_total);
    if (threadIdx.x == 0) s_prefix = before;
  }
  __syncthreads();
  const int64_t out0 = s_prefix;
  if (my_row < a.S) a.sub_indptr[my_row] = out0 + local;
  if (tile == tiles - 1 && threadIdx.x == 0) {
    int64_t total = out0 + tile_total;
    if (__hip_atomic_load(a.lb.error, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT)) total = -1;
    a.sub_indptr[a.S] = total;
    post_mailbox(a.box, total, a.box_ticket);
  }

  // ---- 3. edge-parallel gather and store, kFusedBatch gathers in flight per lane
  const uint32_t n_out = static_cast<uint32_t>(tile_total);
  const IdT* __restrict__ indices = a.indices;
  for (uint32_t base = threadIdx.x; base < n_out; base += kFusedThreads * kFusedBatch) {
    int64_t q[kFusedBatch];
    int64_t r[kFusedBatch];
    IdT v[kFusedBatch];
#pragma unroll
    for (int u = 0; u < kFusedBatch; ++u) {
      const uint32_t e = base + u * kFusedThreads;
      q[u] = -1;
      if (e < n_out) {
        int lo = 0, hi = kFusedRows;  // last row with s_rel[row] <= e
        while (lo < hi) {
          const int mid = (lo + hi) >> 1;
          if (s_rel[mid] <= e) lo = mid + 1; else hi = mid;
        }
        const int row = lo - 1;
        const uint32_t j = e - s_rel[row];
        r[u] = row0 + row;
        uint32_t pick;
        if (REPLACE) {
          const uint32_t xv = a.replay ? a.replay[a.replay_ptr[r[u]] + j]
                                       : draw_one(a.seed, kTagUniform, static_cast<uint64_t>(r[u]),
                                                  static_cast<uint64_t>(j));
          pick = xv % s_deg[row];
        } else {
          pick = s_pick[j * kPickStride + row];
        }
        q[u] = s_start[row] + pick;
        v[u] = indices[q[u]];
      }
    }
    float w[kFusedBatch];
    if (a.data_out) {
      int64_t at_data[kFusedBatch];
#pragma unroll
      for (int u = 0; u < kFusedBatch; ++u) at_data[u] = q[u];
      if (a.edge_ids) {
#pragma unroll
        for (int u = 0; u < kFusedBatch; ++u)
          if (q[u] >= 0) at_data[u] = a.edge_ids[q[u]];
      }
#pragma unroll
      for (int u = 0; u < kFusedBatch; ++u) w[u] = q[u] >= 0 ? a.edge_data[at_data[u]] : 0.f;
    }
#pragma unroll
    for (int u = 0; u < kFusedBatch; ++u) {
      const uint32_t e = base + u * kFusedThreads;
      if (q[u] >= 0) {
        a.sub_indices[out0 + e] = v[u];
        if (a.select_index) a.select_index[out0 + e] = q[u];
        if (a.coo_col) a.coo_col[out0 + e] = static_cast<IdT>(r[u]);
        if (a.data_out) a.data_out[out0 + e] = w[u];
      }
    }
  }
}

template <typename IdT>
int sample_row_lane_launch(const FusedArgs<IdT>& a, bool replace, hipStream_t stream) {
  const unsigned grid = static_cast<unsigned>((a.S + kFusedRows - 1) / kFusedRows);
  if (replace) {
    hipLaunchKernelGGL((sample_row_lane_kernel<IdT, 1, true>), dim3(grid), dim3(kFusedThreads), 0,
                       stream, a);
    return check_launch("sample_fused");
  }
  const size_t lds = static_cast<size_t>(a.k) * kPickStride * sizeof(uint32_t);
  if (a.k <= 8)
    hipLaunchKernelGGL((sample_row_lane_kernel<IdT, 8, false>), dim3(grid), dim3(kFusedThreads),
                       lds, stream, a);
  else if (a.k <= 16)
    hipLaunchKernelGGL((sample_row_lane_kernel<IdT, 16, false>), dim3(grid), dim3(kFusedThreads),
                       lds, stream, a);
  else
    hipLaunchKernelGGL((sample_row_lane_kernel<IdT, 32, false>), dim3(grid), dim3(kFusedThreads),
                       lds, stream, a);
  return check_launch("sample_fused");
}

template <typename IdT>
int sample_fused_launch(const FusedArgs<IdT>& a, bool replace, bool linked, hipStream_t stream) {
  ProfileScope prof(linked ? "layer_sample" : "sample_fused", stream);
  if (!linked && a.S >= kRowLaneMinColumns) return sample_row_lane_launch<IdT>(a, replace, stream);
  if (linked)
    return replace ? sample_fused_dispatch<IdT, true, true>(a, stream)
                   : sample_fused_dispatch<IdT, false, true>(a, stream);
  return replace ? sample_fused_dispatch<IdT, true, false>(a, stream)
                 : sample_fused_dispatch<IdT, false, false>(a, stream);
}

static __global__ void post_zero_kernel(int64_t* sub_indptr, gs_mailbox* box, int64_t ticket) {
  if (threadIdx.x == 0) {
    sub_indptr[0] = 0;
    post_mailbox(box, 0, ticket);
  }
}

template <typename IdT>
int sample_fused_t(const int64_t* indptr, int64_t num_cols, const void* indices,
                   const void* column_ids, int64_t S, int64_t fanout, int replace, uint64_t seed,
                   const uint32_t* replay, const int64_t* replay_ptr, int64_t* sub_indptr,
                   void* sub_indices, int64_t* select_index, void* coo_col, LookbackState lb,
                   gs_mailbox* box, int64_t ticket, hipStream_t st, bool linked = false,
                   const int64_t* S_dev = nullptr, PackedTable table = PackedTable(),
                   uint32_t* pos = nullptr, int64_t* num_edges = nullptr,
                   const float* edge_data = nullptr, const int64_t* edge_ids = nullptr,
                   float* data_out = nullptr) {
  FusedArgs<IdT> a{indptr,
                   static_cast<const IdT*>(indices),
                   static_cast<const IdT*>(column_ids),
                   num_cols,
                   S,
                   fanout,
                   seed,
                   replay,
                   replay_ptr,
                   sub_indptr,
                   static_cast<IdT*>(sub_indices),
                   select_index,
                   static_cast<IdT*>(coo_col),
                   lb,
                   box,
                   ticket,
                   S_dev,
                   table,
                   pos,
                   num_edges,
                   edge_data,
                   edge_ids,
                   data_out};
  return sample_fused_launch<IdT>(a, replace != 0, linked, st);
}

}  // namespace
}  // namespace gs

using namespace gs;

template <typename IdT>
static int sample_uniform_fill_t(const int64_t* indptr, int64_t num_cols, const void* indices,
                                 const void* column_ids, int64_t S, int64_t fanout, int replace, uint64_t seed,
                                 const uint32_t* replay, const int64_t* replay_ptr,
                                 const int64_t* sub_indptr, void* sub_indices,
                                 int64_t* select_index, void* coo_col, long long* queue,
                                 unsigned long long* queue_count, int64_t queue_cap, int algo,
                                 hipStream_t st) {
  SampleArgs<IdT> a{indptr,
                    static_cast<const IdT*>(indices),
                    static_cast<const IdT*>(column_ids),
                    num_cols,
                    S,
                    fanout,
                    seed,
                    replay,
                    replay_ptr,
                    sub_indptr,
                    static_cast<IdT*>(sub_indices),
                    select_index,
                    static_cast<IdT*>(coo_col),
                    queue,
                    queue_count,
                    queue_cap};
  return coo_col ? sample_fill_impl<IdT, true>(a, replace, algo, st)
                 : sample_fill_impl<IdT, false>(a, replace, algo, st);
}

// ---- the same sampler for callers that cannot allocate ----
// Its look-back state (what gs_sample_uniform_fused takes as `state`) lives in a device
// array of this library instead of a caller's buffer: room for GS_FUSED_STATIC_MAX_COLUMNS
// columns.  In host code the array's name is only a stand-in; its device address is asked
// for once per device (hipGetSymbolAddress) and kept.
namespace gs {
namespace {
constexpr int64_t kStaticTiles = (GS_FUSED_STATIC_MAX_COLUMNS * kGroupMaxLanes) / kGroupThreadsLarge + 1;  // = group_tiles_bound of the maximum
constexpr size_t kStaticStateBytes = ((kStaticTiles * 8 + 255) / 256) * 256 + 256 + 256;
constexpr int kMaxDevices = 64;

struct StaticState {
  void* ptr = nullptr;  // device address of `scratch` on this device
  uint32_t epoch = 0;   // last epoch handed out; 0 = the array has to be zero-filled first
};
StaticState g_static_state[kMaxDevices];
std::mutex g_static_mu;

static __global__ void __launch_bounds__(256) zero_words_kernel(unsigned long long* p, size_t n) {
  const size_t i = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (i < n) p[i] = 0ull;
}
}  // namespace
}  // namespace gs

static __device__ __align__(256) unsigned char scratch[gs::kStaticStateBytes];

extern "C" {

size_t gs_slice_workspace_bytes(int64_t num_cols) { return scan_workspace_bytes(num_cols); }

int gs_slice_count(const int64_t* indptr, int64_t num_cols, const void* column_ids, int id_bytes,
                   int64_t S, int64_t* sub_indptr, void* workspace, size_t workspace_bytes,
                   void* stream) {
  GS_REQUIRE(indptr && sub_indptr && S >= 0 && num_cols >= 0,
             "gs_slice_count: null pointer or negative size");
  GS_REQUIRE(S == 0 || column_ids, "gs_slice_count: column_ids is null");
  GS_REQUIRE(valid_id_bytes(id_bytes), "gs_slice_count: id_bytes must be 4 or 8, got %d", id_bytes);
  Carver ws(workspace, workspace_bytes);
  int64_t* tiles = ws.take<int64_t>(scan_num_tiles(S) + 1);
  if (!ws.ok) {
    set_error_text("gs_slice_count: workspace needs %zu bytes, 256-byte aligned",
                   gs_slice_workspace_bytes(S));
    return GS_ERR_WORKSPACE;
  }
  hipStream_t st = static_cast<hipStream_t>(stream);
  return id_bytes == 8
             ? slice_count_impl<int64_t>(indptr, num_cols, column_ids, S, sub_indptr, tiles, st)
             : slice_count_impl<int32_t>(indptr, num_cols, column_ids, S, sub_indptr, tiles, st);
}

int gs_post_total(const int64_t* value, gs_mailbox* mailbox, int64_t ticket, void* stream) {
  GS_REQUIRE(value && mailbox, "gs_post_total: null pointer");
  hipLaunchKernelGGL(post_total_kernel, dim3(1), dim3(1), 0, static_cast<hipStream_t>(stream), value,
                     mailbox, ticket);
  return check_launch("post_total");
}

int gs_post_values(const int64_t* values, int64_t n, int64_t* host_out, gs_mailbox* mailbox,
                   int64_t ticket, void* stream) {
  GS_REQUIRE(n >= 0 && (n == 0 || (values && host_out)), "gs_post_values: null pointer or negative size");
  hipLaunchKernelGGL(post_values_kernel, dim3(1), dim3(256), 0, static_cast<hipStream_t>(stream),
                     values, n, host_out, mailbox, ticket);
  return check_launch("post_values");
}

int gs_post_value_sets(const int64_t* const* sets, int num_sets, int64_t n, int64_t* host_out,
                       gs_mailbox* mailbox, int64_t ticket, void* stream) {
  GS_REQUIRE(num_sets >= 0 && num_sets <= kPostSetsMax && n >= 0,
             "gs_post_value_sets: between 0 and %d arrays of a non-negative length", kPostSetsMax);
  GS_REQUIRE(num_sets == 0 || n == 0 || (sets && host_out), "gs_post_value_sets: null pointer");
  PostSets by_value = {};
  for (int s = 0; s < num_sets; ++s) {
    GS_REQUIRE(n == 0 || sets[s], "gs_post_value_sets: null array");
    by_value.set[s] = sets[s];
  }
  hipLaunchKernelGGL(post_value_sets_kernel, dim3(1), dim3(256), 0,
                     static_cast<hipStream_t>(stream), by_value, num_sets, n, host_out, mailbox,
                     ticket);
  return check_launch("post_values");
}

int gs_slice_fill(const int64_t* indptr, int64_t num_cols, const void* indices,
                  const void* column_ids, int id_bytes, int64_t S, const int64_t* sub_indptr,
                  int64_t nnz, void* sub_indices, int64_t* select_index, void* coo_col,
                  void* stream) {
  return gs_slice_fill_data(indptr, num_cols, indices, column_ids, id_bytes, S, sub_indptr, nnz,
                            sub_indices, select_index, coo_col, nullptr, nullptr, nullptr, stream);
}

int gs_slice_fill_data(const int64_t* indptr, int64_t num_cols, const void* indices,
                       const void* column_ids, int id_bytes, int64_t S, const int64_t* sub_indptr,
                       int64_t nnz, void* sub_indices, int64_t* select_index, void* coo_col,
                       const float* edge_data, const int64_t* edge_ids, float* data_out,
                       void* stream) {
  GS_REQUIRE(indptr && sub_indptr && S >= 0 && nnz >= 0 && num_cols >= 0,
             "gs_slice_fill: null pointer or negative size");
  GS_REQUIRE(nnz == 0 || (indices && column_ids && sub_indices),
             "gs_slice_fill: null buffer with nnz > 0");
  GS_REQUIRE(edge_data ? (data_out != nullptr || nnz == 0) : (!data_out && !edge_ids),
             "gs_slice_fill: edge_data, its output and the edge-id map go together");
  GS_REQUIRE(valid_id_bytes(id_bytes), "gs_slice_fill: id_bytes must be 4 or 8, got %d", id_bytes);
  hipStream_t st = static_cast<hipStream_t>(stream);
  if (!edge_data) data_out = nullptr;
  return id_bytes == 8 ? slice_fill_impl<int64_t>(indptr, num_cols, indices, column_ids, S,
                                                  sub_indptr, nnz, sub_indices, select_index,
                                                  coo_col, edge_data, edge_ids, data_out, st)
                       : slice_fill_impl<int32_t>(indptr, num_cols, indices, column_ids, S,
                                                  sub_indptr, nnz, sub_indices, select_index,
                                                  coo_col, edge_data, edge_ids, data_out, st);
}

size_t gs_sample_workspace_bytes(int64_t S, int64_t fanout) {
  (void)fanout;
  const int64_t s = S < 0 ? 0 : S;
  return scan_workspace_bytes(s) + padded(8) + padded(static_cast<size_t>(s + kQueueExtra) * 8);
}

int gs_sample_count(const int64_t* indptr, int64_t num_cols, const void* column_ids, int id_bytes,
                    int64_t S, int64_t fanout, int replace, int64_t* sub_indptr, void* workspace,
                    size_t workspace_bytes, void* stream) {
  GS_REQUIRE(indptr && sub_indptr && S >= 0 && fanout >= 0 && num_cols >= 0,
             "gs_sample_count: null pointer or negative size");
  GS_REQUIRE(column_ids || S <= num_cols, "gs_sample_count: S exceeds num_cols without column_ids");
  GS_REQUIRE(valid_id_bytes(id_bytes), "gs_sample_count: id_bytes must be 4 or 8, got %d", id_bytes);
  Carver ws(workspace, workspace_bytes);
  int64_t* tiles = ws.take<int64_t>(scan_num_tiles(S) + 1);
  if (!ws.ok) {
    set_error_text("gs_sample_count: workspace needs %zu bytes, 256-byte aligned",
                   gs_sample_workspace_bytes(S, fanout));
    return GS_ERR_WORKSPACE;
  }
  hipStream_t st = static_cast<hipStream_t>(stream);
  return id_bytes == 8
             ? sample_count_impl<int64_t>(indptr, num_cols, column_ids, S, fanout, replace,
                                          sub_indptr, tiles, st)
             : sample_count_impl<int32_t>(indptr, num_cols, column_ids, S, fanout, replace,
                                          sub_indptr, tiles, st);
}

int gs_sample_uniform_fill(const int64_t* indptr, int64_t num_cols, const void* indices,
                           const void* column_ids, int id_bytes, int64_t S, int64_t fanout,
                           int replace, int algo, uint64_t seed,
                           const uint32_t* replay, const int64_t* replay_ptr,
                           const int64_t* sub_indptr, void* sub_indices, int64_t* select_index,
                           void* coo_col, void* workspace, size_t workspace_bytes, void* stream) {
  GS_REQUIRE(indptr && sub_indptr && S >= 0 && fanout >= 0 && num_cols >= 0,
             "gs_sample_uniform_fill: null pointer or negative size");
  GS_REQUIRE(column_ids || S <= num_cols,
             "gs_sample_uniform_fill: S exceeds num_cols without column_ids");
  GS_REQUIRE(S == 0 || fanout == 0 || (indices && sub_indices && select_index),
             "gs_sample_uniform_fill: null buffer");
  GS_REQUIRE(valid_id_bytes(id_bytes), "gs_sample_uniform_fill: id_bytes must be 4 or 8, got %d",
             id_bytes);
  GS_REQUIRE((replay == nullptr) == (replay_ptr == nullptr),
             "gs_sample_uniform_fill: replay and replay_ptr must be given together");
  GS_REQUIRE(algo == GS_SAMPLE_AUTO || algo == GS_SAMPLE_RESERVOIR,
             "gs_sample_uniform_fill: unknown algo %d", algo);
  if (fanout == 0 || S == 0) return GS_OK;
  // same carving as gs_sample_count, so one workspace serves both calls
  Carver ws(workspace, workspace_bytes);
  ws.take<int64_t>(scan_num_tiles(S) + 1);
  unsigned long long* queue_count = ws.take<unsigned long long>(1);
  const int64_t queue_cap = S + kQueueExtra;
  long long* queue = ws.take<long long>(static_cast<size_t>(queue_cap));
  if (!ws.ok) {
    set_error_text("gs_sample_uniform_fill: workspace needs %zu bytes, 256-byte aligned",
                   gs_sample_workspace_bytes(S, fanout));
    return GS_ERR_WORKSPACE;
  }
  hipStream_t st = static_cast<hipStream_t>(stream);
  return id_bytes == 8
             ? sample_uniform_fill_t<int64_t>(indptr, num_cols, indices, column_ids, S, fanout, replace, seed,
                                              replay, replay_ptr, sub_indptr, sub_indices,
                                              select_index, coo_col, queue, queue_count,
                                              queue_cap, algo, st)
             : sample_uniform_fill_t<int32_t>(indptr, num_cols, indices, column_ids, S, fanout, replace, seed,
                                              replay, replay_ptr, sub_indptr, sub_indices,
                                              select_index, coo_col, queue, queue_count,
                                              queue_cap, algo, st);
}

size_t gs_sample_fused_state_bytes(int64_t S) {
  const int64_t s = S < 0 ? 0 : S;
  return lookback_state_bytes(group_tiles_bound(s, false));
}

int gs_sample_uniform_fused(const int64_t* indptr, int64_t num_cols, const void* indices,
                            const void* column_ids, int id_bytes, int64_t S, int64_t fanout,
                            int replace, uint64_t seed, const uint32_t* replay,
                            const int64_t* replay_ptr, int64_t* sub_indptr, void* sub_indices,
                            int64_t* select_index, void* coo_col, int64_t capacity,
                            void* state, size_t state_bytes, uint32_t epoch,
                            gs_mailbox* mailbox, int64_t mailbox_ticket, void* stream) {
  return gs_sample_uniform_fused_data(indptr, num_cols, indices, column_ids, id_bytes, S, fanout,
                                      replace, seed, replay, replay_ptr, sub_indptr, sub_indices,
                                      select_index, coo_col, capacity, nullptr, nullptr, nullptr,
                                      state, state_bytes, epoch, mailbox, mailbox_ticket, stream);
}

int gs_sample_uniform_fused_data(const int64_t* indptr, int64_t num_cols, const void* indices,
                                 const void* column_ids, int id_bytes, int64_t S, int64_t fanout,
                                 int replace, uint64_t seed, const uint32_t* replay,
                                 const int64_t* replay_ptr, int64_t* sub_indptr,
                                 void* sub_indices, int64_t* select_index, void* coo_col,
                                 int64_t capacity, const float* edge_data,
                                 const int64_t* edge_ids, float* data_out, void* state,
                                 size_t state_bytes, uint32_t epoch, gs_mailbox* mailbox,
                                 int64_t mailbox_ticket, void* stream) {
  GS_REQUIRE(edge_data ? (data_out != nullptr || S * fanout == 0) : (!data_out && !edge_ids),
             "gs_sample_uniform_fused_data: edge_data and data_out go together (edge_ids needs both)");
  GS_REQUIRE(indptr && sub_indptr && S >= 0 && fanout >= 0 && num_cols >= 0,
             "gs_sample_uniform_fused: null pointer or negative size");
  GS_REQUIRE(column_ids || S <= num_cols,
             "gs_sample_uniform_fused: S exceeds num_cols without column_ids");
  GS_REQUIRE(valid_id_bytes(id_bytes), "gs_sample_uniform_fused: id_bytes must be 4 or 8, got %d",
             id_bytes);
  GS_REQUIRE((replay == nullptr) == (replay_ptr == nullptr),
             "gs_sample_uniform_fused: replay and replay_ptr must be given together");
  if (!replace && fanout > GS_FUSED_MAX_FANOUT) {
    set_error_text("gs_sample_uniform_fused: fanout %lld without replacement exceeds %d; use "
                   "gs_sample_count + gs_sample_uniform_fill",
                   static_cast<long long>(fanout), GS_FUSED_MAX_FANOUT);
    return GS_ERR_UNSUPPORTED;
  }
  GS_REQUIRE(S == 0 || fanout == 0 || capacity >= S * fanout,
             "gs_sample_uniform_fused: outputs must hold S * fanout = %lld entries, capacity is %lld",
             static_cast<long long>(S * fanout), static_cast<long long>(capacity));
  GS_REQUIRE(S == 0 || fanout == 0 || (indices && sub_indices),
             "gs_sample_uniform_fused: null buffer");
  hipStream_t st = static_cast<hipStream_t>(stream);
  if (S == 0) {
    hipLaunchKernelGGL(post_zero_kernel, dim3(1), dim3(64), 0, st, sub_indptr, mailbox,
                       mailbox_ticket);
    return check_launch("sample_fused");
  }
  GS_REQUIRE(epoch >= 1 && epoch <= kLbMaxEpoch,
             "gs_sample_uniform_fused: epoch must be 1..%u, got %u", kLbMaxEpoch, epoch);
  GS_REQUIRE(S * fanout <= static_cast<int64_t>(kLbValue),
             "gs_sample_uniform_fused: S * fanout exceeds 2^48");
  Carver ws(state, state_bytes);
  // carved for the most tiles any fanout asks for, so that the size does not depend on it
  LookbackState lb = carve_lookback(ws, group_tiles_bound(S, false), epoch);
  if (!ws.ok) {
    set_error_text("gs_sample_uniform_fused: state needs %zu bytes, 256-byte aligned",
                   gs_sample_fused_state_bytes(S));
    return GS_ERR_WORKSPACE;
  }
  return id_bytes == 8
             ? sample_fused_t<int64_t>(indptr, num_cols, indices, column_ids, S, fanout, replace,
                                       seed, replay, replay_ptr, sub_indptr, sub_indices,
                                       select_index, coo_col, lb, mailbox, mailbox_ticket, st,
                                       false, nullptr, PackedTable(), nullptr, nullptr, edge_data,
                                       edge_ids, data_out)
             : sample_fused_t<int32_t>(indptr, num_cols, indices, column_ids, S, fanout, replace,
                                       seed, replay, replay_ptr, sub_indptr, sub_indices,
                                       select_index, coo_col, lb, mailbox, mailbox_ticket, st,
                                       false, nullptr, PackedTable(), nullptr, nullptr, edge_data,
                                       edge_ids, data_out);
}

size_t gs_layer_sample_state_bytes(int64_t S_bound) {
  return lookback_state_bytes(group_tiles_bound(S_bound < 0 ? 0 : S_bound, true));
}

int gs_layer_sample(const int64_t* indptr, int64_t num_cols, const void* indices,
                    const void* column_ids, int id_bytes, int64_t S_bound, const int64_t* S_dev,
                    int64_t fanout, int replace, uint64_t seed, const uint32_t* replay,
                    const int64_t* replay_ptr, int64_t* sub_indptr, void* sub_indices,
                    int64_t capacity, int64_t* num_edges, int64_t* select_index,
                    const float* edge_data, const int64_t* edge_ids, float* data_out, void* table,
                    size_t table_bytes, void* workspace, size_t workspace_bytes, void* state,
                    size_t state_bytes, uint32_t epoch, gs_mailbox* mailbox,
                    int64_t mailbox_ticket, void* stream) {
  GS_REQUIRE(edge_data ? (data_out != nullptr || capacity == 0) : (!data_out && !edge_ids),
             "gs_layer_sample: edge_data and data_out go together (edge_ids needs both)");
  GS_REQUIRE(indptr && sub_indptr && num_edges && table && workspace && state && S_bound >= 0 &&
                 fanout >= 0 && num_cols >= 0,
             "gs_layer_sample: null pointer or negative size");
  GS_REQUIRE(S_bound == 0 || column_ids, "gs_layer_sample: column_ids is null");
  GS_REQUIRE(valid_id_bytes(id_bytes), "gs_layer_sample: id_bytes must be 4 or 8, got %d", id_bytes);
  GS_REQUIRE((replay == nullptr) == (replay_ptr == nullptr),
             "gs_layer_sample: replay and replay_ptr must be given together");
  if (!replace && fanout > GS_FUSED_MAX_FANOUT) {
    set_error_text("gs_layer_sample: fanout %lld without replacement exceeds %d",
                   static_cast<long long>(fanout), GS_FUSED_MAX_FANOUT);
    return GS_ERR_UNSUPPORTED;
  }
  GS_REQUIRE(capacity >= S_bound * fanout,
             "gs_layer_sample: outputs must hold S_bound * fanout = %lld entries, capacity is %lld",
             static_cast<long long>(S_bound * fanout), static_cast<long long>(capacity));
  GS_REQUIRE(S_bound == 0 || fanout == 0 || (indices && sub_indices), "gs_layer_sample: null buffer");
  GS_REQUIRE(epoch >= 1 && epoch <= kLbMaxEpoch, "gs_layer_sample: epoch must be 1..%u, got %u",
             kLbMaxEpoch, epoch);
  const int64_t M_bound = S_bound + capacity;
  if (M_bound >= (int64_t(1) << 31)) {
    set_error_text("gs_layer_sample: %lld items exceed the supported 2^31",
                   static_cast<long long>(M_bound));
    return GS_ERR_UNSUPPORTED;
  }
  PackedTable t;
  if (!shape_linked_table<PackedTable>(table, table_bytes, M_bound, &t)) {
    set_error_text("gs_layer_sample: the table holds fewer than the %lld slots this call needs "
                   "(or is misaligned)",
                   static_cast<long long>(linked_table_capacity(M_bound)));
    return GS_ERR_WORKSPACE;
  }
  uint32_t* pos = nullptr;
  Carver ws(state, state_bytes);
  LookbackState lb = carve_lookback(ws, group_tiles_bound(S_bound, true), epoch);
  if (!carve_layer_workspace(workspace, workspace_bytes, M_bound, &pos) || !ws.ok) {
    set_error_text("gs_layer_sample: workspace needs %zu bytes and state %zu bytes, 256-byte aligned",
                   layer_workspace_bytes(M_bound), gs_layer_sample_state_bytes(S_bound));
    return GS_ERR_WORKSPACE;
  }
  hipStream_t st = static_cast<hipStream_t>(stream);
  return id_bytes == 8
             ? sample_fused_t<int64_t>(indptr, num_cols, indices, column_ids, S_bound, fanout,
                                       replace, seed, replay, replay_ptr, sub_indptr, sub_indices,
                                       select_index, nullptr, lb, mailbox, mailbox_ticket, st, true,
                                       S_dev, t, pos, num_edges, edge_data, edge_ids, data_out)
             : sample_fused_t<int32_t>(indptr, num_cols, indices, column_ids, S_bound, fanout,
                                       replace, seed, replay, replay_ptr, sub_indptr, sub_indices,
                                       select_index, nullptr, lb, mailbox, mailbox_ticket, st, true,
                                       S_dev, t, pos, num_edges, edge_data, edge_ids, data_out);
}

// device address of `scratch` on the current device, resolved once per device (not under
// stream capture: the lookup is a runtime call of its own)
// (stream_known: `stream` is the stream of a launch and is asked whether it is being captured;
// the calls that launch nothing leave every stream alone)
static int static_state_of_current_device(const char* who, bool stream_known, hipStream_t stream,
                                          bool* capturing, gs::StaticState** out) {
  int device = -1;
  if (hipGetDevice(&device) != hipSuccess || device < 0 || device >= kMaxDevices) {
    set_error_text("%s: no current device (or its number is above %d)", who, kMaxDevices - 1);
    return GS_ERR_LAUNCH;
  }
  hipStreamCaptureStatus cap = hipStreamCaptureStatusNone;
  if (stream_known && hipStreamIsCapturing(stream, &cap) != hipSuccess) {
    set_error_text("%s: hipStreamIsCapturing failed", who);
    return GS_ERR_LAUNCH;
  }
  *capturing = cap != hipStreamCaptureStatusNone;
  StaticState& st = g_static_state[device];
  if (!st.ptr) {
    if (*capturing) {
      set_error_text("%s: the first call on a device resolves the address of the library's "
                     "state array, which cannot be done while the stream is being captured; call "
                     "gs_sample_uniform_fused_static_init before the capture", who);
      return GS_ERR_UNSUPPORTED;
    }
    void* p = nullptr;
    const hipError_t e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
    if (e != hipSuccess || !p) {
      set_error_text("%s: hipGetSymbolAddress: %s", who, hipGetErrorString(e));
      return GS_ERR_LAUNCH;
    }
    st.ptr = p;
    st.epoch = 0;
  }
  *out = &st;
  return GS_OK;
}

int gs_sample_uniform_fused_static_init(void) {
  std::lock_guard<std::mutex> lock(g_static_mu);
  bool capturing = false;
  StaticState* st = nullptr;
  return static_state_of_current_device("gs_sample_uniform_fused_static_init", false, nullptr,
                                        &capturing, &st);
}

int gs_sample_uniform_fused_static_reset(void) {
  std::lock_guard<std::mutex> lock(g_static_mu);
  bool capturing = false;
  StaticState* st = nullptr;
  GS_RETURN_IF_ERROR(static_state_of_current_device("gs_sample_uniform_fused_static_reset", false,
                                                    nullptr, &capturing, &st));
  st->epoch = 0;  // the next call zero-fills the array (error word included) before it runs
  return GS_OK;
}

namespace gs {
namespace {
static __global__ void raise_error_word_kernel(unsigned int* error) { *error = 1u; }
}  // namespace
}  // namespace gs

int gs_sample_uniform_fused_static_debug_raise(void* stream) {
  std::lock_guard<std::mutex> lock(g_static_mu);
  bool capturing = false;
  StaticState* st = nullptr;
  GS_RETURN_IF_ERROR(static_state_of_current_device("gs_sample_uniform_fused_static_debug_raise",
                                                    true, static_cast<hipStream_t>(stream),
                                                    &capturing, &st));
  // the error word is the first word of a look-back state (carve_lookback)
  hipLaunchKernelGGL(raise_error_word_kernel, dim3(1), dim3(1), 0, static_cast<hipStream_t>(stream),
                     static_cast<unsigned int*>(st->ptr));
  return check_launch("gs_sample_uniform_fused_static_debug_raise");
}

int gs_sample_uniform_fused_static(const int64_t* indptr, int64_t num_cols, const void* indices,
                                   const void* column_ids, int id_bytes, int64_t S,
                                   int64_t fanout, int replace, uint64_t seed,
                                   const uint32_t* replay, const int64_t* replay_ptr,
                                   int64_t* sub_indptr, void* sub_indices,
                                   int64_t* select_index, void* coo_col, int64_t capacity,
                                   gs_mailbox* mailbox, int64_t mailbox_ticket, void* stream) {
  if (S > GS_FUSED_STATIC_MAX_COLUMNS) {
    set_error_text("gs_sample_uniform_fused_static: %lld columns exceed the %lld the library's "
                   "own state holds; use gs_sample_uniform_fused with a caller's state buffer",
                   static_cast<long long>(S), static_cast<long long>(GS_FUSED_STATIC_MAX_COLUMNS));
    return GS_ERR_UNSUPPORTED;
  }
  void* state = nullptr;
  uint32_t epoch = 0;
  {
    std::lock_guard<std::mutex> lock(g_static_mu);
    bool capturing = false;
    StaticState* st = nullptr;
    GS_RETURN_IF_ERROR(static_state_of_current_device("gs_sample_uniform_fused_static", true,
                                                      static_cast<hipStream_t>(stream), &capturing,
                                                      &st));
    // The epochs are counted here, on the host, and go into the launch as an argument.  A call
    // that is being recorded into a graph will run again, as often as the graph is replayed,
    // with that same argument: so a recorded call always starts from a zero-filled array under
    // epoch 1 (the fill kernel is recorded in front of it), which is right on every replay,
    // and leaves the count at "fill first" for whatever call comes next.  Otherwise the array
    // is filled on first use, when every epoch has been used, and after a reset.
    if (capturing || st->epoch == 0 || st->epoch >= kLbMaxEpoch) {
      const size_t words = kStaticStateBytes / 8;
      hipLaunchKernelGGL(zero_words_kernel, dim3(static_cast<unsigned>((words + 255) / 256)),
                         dim3(256), 0, static_cast<hipStream_t>(stream),
                         static_cast<unsigned long long*>(st->ptr), words);
      GS_RETURN_IF_ERROR(check_launch("gs_sample_uniform_fused_static (state fill)"));
      st->epoch = 0;
    }
    state = st->ptr;
    epoch = st->epoch + 1;
    st->epoch = capturing ? 0 : epoch;
  }
  return gs_sample_uniform_fused(indptr, num_cols, indices, column_ids, id_bytes, S, fanout,
                                 replace, seed, replay, replay_ptr, sub_indptr, sub_indices,
                                 select_index, coo_col, capacity, state, kStaticStateBytes, epoch,
                                 mailbox, mailbox_ticket, stream);
}

int gs_sample_one_keepdim(const int64_t* indptr, int64_t num_cols, const void* indices,
                          const void* column_ids, int id_bytes, int64_t S, uint64_t seed,
                          const uint32_t* replay,
                          int64_t* sub_indptr, void* sub_indices, int64_t* select_index,
                          void* stream) {
  GS_REQUIRE(indptr && sub_indptr && S >= 0 && num_cols >= 0,
             "gs_sample_one_keepdim: null pointer or negative size");
  GS_REQUIRE(S == 0 || (indices && column_ids && sub_indices && select_index),
             "gs_sample_one_keepdim: null buffer");
  GS_REQUIRE(valid_id_bytes(id_bytes), "gs_sample_one_keepdim: id_bytes must be 4 or 8, got %d",
             id_bytes);
  hipStream_t st = static_cast<hipStream_t>(stream);
  const unsigned grid = static_cast<unsigned>((S + 1 + 255) / 256);
  if (id_bytes == 8) {
    hipLaunchKernelGGL((sample_one_keepdim_kernel<int64_t>), dim3(grid), dim3(256), 0, st, indptr,
                       static_cast<const int64_t*>(indices), static_cast<const int64_t*>(column_ids),
                       num_cols, S, seed, replay, sub_indptr, static_cast<int64_t*>(sub_indices),
                       select_index);
  } else {
    hipLaunchKernelGGL((sample_one_keepdim_kernel<int32_t>), dim3(grid), dim3(256), 0, st, indptr,
                       static_cast<const int32_t*>(indices), static_cast<const int32_t*>(column_ids),
                       num_cols, S, seed, replay, sub_indptr, static_cast<int32_t*>(sub_indices),
                       select_index);
  }
  return check_launch("sample_one_keepdim");
}

}  // extern "C"

// ---- self-test of the bounded wait: the chained scan alone, one tile left out ----
namespace gs {
namespace {
__global__ void __launch_bounds__(kWave) lookback_selftest_kernel(LookbackState lb, int64_t tiles,
                                                                   int64_t missing,
                                                                   int64_t* total) {
  // workgroup b plays tile b, or b + 1 from the missing tile on: that tile's status word is
  // never written, so its first successor waits for it in vain
  const int64_t tile = missing >= 0 && static_cast<int64_t>(blockIdx.x) >= missing
                           ? static_cast<int64_t>(blockIdx.x) + 1
                           : static_cast<int64_t>(blockIdx.x);
  if (threadIdx.x == 0) lookback_publish_sum(lb, static_cast<unsigned int>(tile), 1);
  const int64_t before = lookback_exclusive_prefix(lb, static_cast<unsigned int>(tile), 1);
  if (tile == tiles - 1 && threadIdx.x == 0) {
    int64_t t = before + 1;
    if (__hip_atomic_load(lb.error, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT)) t = -1;
    *total = t;
  }
}
}  // namespace
}  // namespace gs

extern "C" int gs_selftest_lookback(void* state, size_t state_bytes, uint32_t epoch, int64_t tiles,
                                    int64_t missing_tile, int spin_limit, int64_t* total,
                                    void* stream) {
  using namespace gs;
  GS_REQUIRE(state && total && tiles >= 2 && tiles <= (int64_t(1) << 20),
             "gs_selftest_lookback: null pointer, or tiles outside 2..2^20");
  GS_REQUIRE(missing_tile >= -1 && missing_tile < tiles - 1,
             "gs_selftest_lookback: the missing tile must not be the last one");
  GS_REQUIRE(spin_limit >= 1 && spin_limit <= kLookbackSpinLimit,
             "gs_selftest_lookback: spin_limit must be in 1..%d", kLookbackSpinLimit);
  GS_REQUIRE(epoch >= 1 && epoch <= kLbMaxEpoch, "gs_selftest_lookback: epoch must be 1..%u",
             kLbMaxEpoch);
  Carver ws(state, state_bytes);
  LookbackState lb = carve_lookback(ws, tiles, epoch);
  if (!ws.ok) {
    set_error_text("gs_selftest_lookback: state needs %zu bytes, 256-byte aligned",
                   lookback_state_bytes(tiles));
    return GS_ERR_WORKSPACE;
  }
  lb.spin_limit = spin_limit;
  const unsigned grid = static_cast<unsigned>(missing_tile >= 0 ? tiles - 1 : tiles);
  hipLaunchKernelGGL(lookback_selftest_kernel, dim3(grid), dim3(kWave), 0,
                     static_cast<hipStream_t>(stream), lb, tiles, missing_tile, total);
  return check_launch("selftest_lookback");
}
