// List sampling on gfx950: pick k of n items, uniformly or by weight.
//
// Replaces impl::ListSamplingCUDA (reference src/cuda/list_sampling.cu:79) and
// impl::ListSamplingProbsCUDA (src/cuda/list_sampling_probs.cu:185).
//
// Uniform, without replacement: Algorithm R over positions exactly as the
// reference (list_sampling.cu:54-71): index[j] = j, then every idx in [k, n)
// draws num = draw(idx) % (idx+1) and raises index[num] to idx when num < k.
//
// Weighted (A-Res): the reference computes a key per item and then fully
// radix-sorts all n (key, index) pairs to keep the first k
// (list_sampling_probs.cu:76-86).  Here the k-th largest 64-bit composite
// (ordered key << 32 | ~position) is found by a six-level radix SELECT
// (11+11+10 bits of key, 11+11+10 bits of position): each level is one pass
// over the 4-byte keys with LDS-private histograms; the pick of a level (which
// bin holds the k-th item) is made at the head of the NEXT level's kernel, by every
// workgroup for itself from the finished histogram, so a level is one launch and
// not two.  Then exactly k survivors are gathered and only those k are sorted
// (bitonic, in LDS).  Algorithmic traffic is 4 B/item/level instead of 12 B/item per
// radix-sort pass over key+index pairs.
#include "gs_common.hpp"

namespace gs {
namespace {

constexpr int kThreads = 256;
constexpr int kBins = 2048;
constexpr int kLevels = 6;
constexpr int64_t kMaxWeightedPicks = 8192;  // bitonic sort of the survivors in 64 KB of LDS
__constant__ int c_shift[kLevels] = {53, 42, 32, 21, 10, 0};
__constant__ int c_width[kLevels] = {11, 11, 10, 11, 11, 10};

// ------------------------------------------------------------- uniform -----
template <typename IdT>
__global__ void __launch_bounds__(kThreads)
list_replace_kernel(const IdT* __restrict__ data, int64_t n, int64_t k, uint64_t seed,
                    const uint32_t* __restrict__ replay, IdT* __restrict__ out_data,
                    int64_t* __restrict__ out_index) {
  const int64_t j = static_cast<int64_t>(blockIdx.x) * kThreads + threadIdx.x;
  if (j >= k) return;
  const uint32_t x = replay ? replay[j] : draw_one(seed, kTagListUniform, 0, static_cast<uint64_t>(j));
  const int64_t id = static_cast<int64_t>(x % static_cast<uint32_t>(n));
  out_index[j] = id;
  out_data[j] = data[id];
}

__global__ void __launch_bounds__(kThreads) iota_kernel(int64_t* out, int64_t k) {
  const int64_t j = static_cast<int64_t>(blockIdx.x) * kThreads + threadIdx.x;
  if (j < k) out[j] = j;
}

__global__ void __launch_bounds__(kThreads)
list_reservoir_kernel(int64_t n, int64_t k, uint64_t seed, const uint32_t* __restrict__ replay,
                      int64_t* __restrict__ out_index) {
  const int64_t q = (k >> 2) + static_cast<int64_t>(blockIdx.x) * kThreads + threadIdx.x;
  if (q * 4 >= n) return;
  U4 x;
  if (!replay) x = draw_block(seed, kTagListUniform, 0, static_cast<uint64_t>(q));
#pragma unroll
  for (int t = 0; t < 4; ++t) {
    const int64_t idx = q * 4 + t;
    if (idx >= k && idx < n) {
      const uint32_t xv = replay ? replay[idx - k] : x.v[t];
      const uint32_t num = xv % static_cast<uint32_t>(idx + 1);
      if (static_cast<int64_t>(num) < k)
        atomicMax(reinterpret_cast<long long*>(out_index) + num, static_cast<long long>(idx));
    }
  }
}

template <typename IdT>
__global__ void __launch_bounds__(kThreads)
list_gather_kernel(const IdT* __restrict__ data, const int64_t* __restrict__ index, int64_t k,
                   IdT* __restrict__ out_data) {
  const int64_t j = static_cast<int64_t>(blockIdx.x) * kThreads + threadIdx.x;
  if (j < k) out_data[j] = data[index[j]];
}

// ------------------------------------------------------------ weighted -----
// state[L]: the selection after the picks of levels 0 .. L-1 (state[0]: nothing picked)
struct SelectState {
  unsigned long long prefix;     // digits chosen so far, in place
  unsigned long long remaining;  // how many of the matching items are still wanted
  unsigned long long gathered;   // survivor counter (state[0] only)
  unsigned long long done;       // every item under the prefix is wanted: lower digits do not matter
};

__device__ __forceinline__ unsigned long long list_composite(uint32_t okey, int64_t i) {
  return (static_cast<unsigned long long>(okey) << 32) | (0xFFFFFFFFu - static_cast<uint32_t>(i));
}

__global__ void __launch_bounds__(kThreads)
select_init_kernel(uint32_t* hist, SelectState* st, int64_t k) {
  for (int i = threadIdx.x; i < kLevels * kBins; i += kThreads) hist[i] = 0;
  if (threadIdx.x == 0) {
    st->prefix = 0;
    st->remaining = static_cast<unsigned long long>(k);
    st->gathered = 0;
    st->done = 0;
  }
}

// Level 0: keys (list_sampling_probs.cu:62-78) + histogram of their top 11 bits.
__global__ void __launch_bounds__(kThreads)
keys_hist_kernel(const float* __restrict__ probs, int64_t n, uint64_t seed,
                 const uint32_t* __restrict__ replay, uint32_t* __restrict__ okey,
                 uint32_t* __restrict__ hist) {
  __shared__ uint32_t s_hist[kBins];
  for (int i = threadIdx.x; i < kBins; i += kThreads) s_hist[i] = 0;
  __syncthreads();
  const int64_t nq = (n + 3) >> 2;
  for (int64_t q = static_cast<int64_t>(blockIdx.x) * kThreads + threadIdx.x; q < nq;
       q += static_cast<int64_t>(gridDim.x) * kThreads) {
    U4 x;
    if (!replay) x = draw_block(seed, kTagListWeighted, 0, static_cast<uint64_t>(q));
#pragma unroll
    for (int t = 0; t < 4; ++t) {
      const int64_t i = q * 4 + t;
      if (i < n) {
        const uint32_t xv = replay ? replay[i] : x.v[t];
        const uint32_t ok = float_to_ordered(ares_key(xv, probs[i]));
        okey[i] = ok;
        atomicAdd(&s_hist[ok >> 21], 1u);
      }
    }
  }
  __syncthreads();
  for (int i = threadIdx.x; i < kBins; i += kThreads)
    if (s_hist[i]) atomicAdd(&hist[i], s_hist[i]);
}

// The bin of `level` that holds the `remaining`-th largest item under the prefix, from the
// finished histogram of that level.  Called by every thread of a workgroup; every
// workgroup of a launch arrives at the same answer.
struct PickScratch {
  int64_t scan[kThreads / kWave + 1];
  SelectState out;
};

__device__ __forceinline__ SelectState pick_level(const uint32_t* __restrict__ hist, int level,
                                                  const SelectState& in, PickScratch* lds) {
  if (in.done) return in;
  const uint32_t* h = hist + level * kBins;
  constexpr int kPer = kBins / kThreads;  // 8 consecutive bins per thread
  int64_t mine = 0;
#pragma unroll
  for (int j = 0; j < kPer; ++j) mine += h[threadIdx.x * kPer + j];
  int64_t total;
  const int64_t below = block_exclusive_scan<kThreads>(mine, &total, lds->scan);
  if (threadIdx.x == 0) lds->out = in;
  __syncthreads();
  const unsigned long long want = in.remaining;
  unsigned long long above = static_cast<unsigned long long>(total - below - mine);  // bins of threads > t
  if (above < want && want <= above + static_cast<unsigned long long>(mine)) {
    for (int j = kPer - 1; j >= 0; --j) {
      const unsigned long long cnt = h[threadIdx.x * kPer + j];
      if (want <= above + cnt) {
        SelectState s = in;
        s.prefix |= static_cast<unsigned long long>(threadIdx.x * kPer + j) << c_shift[level];
        s.remaining = want - above;
        // all of the bin is wanted (typically a bin of one): with the lower digits left at zero
        // "composite >= prefix" already selects exactly the wanted items
        if (want - above == cnt) s.done = 1;
        lds->out = s;
        break;
      }
      above += cnt;
    }
  }
  __syncthreads();
  const SelectState r = lds->out;
  __syncthreads();
  return r;
}

// Levels 1..5: the pick of the level before, then the histogram of this level's digit over
// the items that match the prefix.  Workgroup 0 leaves the state after the pick in
// state[level] for the next launch.
__global__ void __launch_bounds__(kThreads)
level_hist_kernel(const uint32_t* __restrict__ okey, int64_t n, int level, SelectState* state,
                  uint32_t* __restrict__ hist) {
  __shared__ uint32_t s_hist[kBins];
  __shared__ PickScratch s_pick;
  const SelectState st = pick_level(hist, level - 1, state[level - 1], &s_pick);
  if (blockIdx.x == 0 && threadIdx.x == 0) {
    state[level].prefix = st.prefix;
    state[level].remaining = st.remaining;
    state[level].done = st.done;
  }
  if (st.done) return;  // a pick took its whole bin: nothing left to split
  for (int i = threadIdx.x; i < kBins; i += kThreads) s_hist[i] = 0;
  __syncthreads();
  const unsigned long long prefix = st.prefix;
  const int up = c_shift[level - 1];
  const int sh = c_shift[level];
  const uint32_t mask = (1u << c_width[level]) - 1u;
  for (int64_t i = static_cast<int64_t>(blockIdx.x) * kThreads + threadIdx.x; i < n;
       i += static_cast<int64_t>(gridDim.x) * kThreads) {
    const unsigned long long c = list_composite(okey[i], i);
    if ((c >> up) == (prefix >> up)) atomicAdd(&s_hist[static_cast<uint32_t>(c >> sh) & mask], 1u);
  }
  __syncthreads();
  uint32_t* h = hist + level * kBins;
  for (int i = threadIdx.x; i < kBins; i += kThreads)
    if (s_hist[i]) atomicAdd(&h[i], s_hist[i]);
}

// The pick of the last level, then the items at or above the k-th.
__global__ void __launch_bounds__(kThreads)
survivors_kernel(const uint32_t* __restrict__ okey, int64_t n, SelectState* state,
                 const uint32_t* __restrict__ hist, unsigned long long* __restrict__ cand,
                 int64_t k) {
  __shared__ PickScratch s_pick;
  const SelectState st = pick_level(hist, kLevels - 1, state[kLevels - 1], &s_pick);
  const unsigned long long kth = st.prefix;
  for (int64_t i = static_cast<int64_t>(blockIdx.x) * kThreads + threadIdx.x; i < n;
       i += static_cast<int64_t>(gridDim.x) * kThreads) {
    const unsigned long long c = list_composite(okey[i], i);
    if (c >= kth) {
      const unsigned long long slot = atomicAdd(&state[0].gathered, 1ull);
      if (static_cast<int64_t>(slot) < k) cand[slot] = c;
    }
  }
}

// One workgroup: bitonic sort (descending) of the k survivors, then emit.
template <typename IdT>
__global__ void __launch_bounds__(1024)
sort_emit_kernel(const unsigned long long* __restrict__ cand, int64_t k, int padded_k,
                 const IdT* __restrict__ data, IdT* __restrict__ out_data,
                 int64_t* __restrict__ out_index) {
  extern __shared__ unsigned long long s_c[];
  for (int i = threadIdx.x; i < padded_k; i += blockDim.x) s_c[i] = i < k ? cand[i] : 0ull;
  __syncthreads();
  for (int size = 2; size <= padded_k; size <<= 1) {
    for (int stride = size >> 1; stride > 0; stride >>= 1) {
      for (int t = threadIdx.x; t < padded_k / 2; t += blockDim.x) {
        const int lo = 2 * t - (t & (stride - 1));
        const int hi = lo + stride;
        const bool descending = ((lo & size) == 0);
        const unsigned long long a = s_c[lo], b = s_c[hi];
        if ((a < b) == descending) {
          s_c[lo] = b;
          s_c[hi] = a;
        }
      }
      __syncthreads();
    }
  }
  for (int j = threadIdx.x; j < k; j += blockDim.x) {
    const int64_t pos = 0xFFFFFFFFu - static_cast<uint32_t>(s_c[j]);
    out_index[j] = pos;
    out_data[j] = data[pos];
  }
}

struct WeightedScratch {
  uint32_t* okey;
  uint32_t* hist;
  SelectState* state;
  unsigned long long* cand;
  bool ok;
};

WeightedScratch carve_weighted(void* ws_ptr, size_t bytes, int64_t n, int64_t k) {
  Carver ws(ws_ptr, bytes);
  WeightedScratch s;
  s.okey = ws.take<uint32_t>(n > 0 ? n : 1);
  s.hist = ws.take<uint32_t>(kLevels * kBins);
  s.state = ws.take<SelectState>(kLevels);
  s.cand = ws.take<unsigned long long>(k > 0 ? k : 1);
  s.ok = ws.ok;
  return s;
}

template <typename IdT>
int list_uniform_impl(const void* data, int64_t n, int64_t k, int replace, uint64_t seed,
                      const uint32_t* replay, void* out_data, int64_t* out_index, hipStream_t st) {
  const IdT* d = static_cast<const IdT*>(data);
  IdT* od = static_cast<IdT*>(out_data);
  if (replace) {
    hipLaunchKernelGGL((list_replace_kernel<IdT>), dim3(blocks_for(k, kThreads)), dim3(kThreads), 0,
                       st, d, n, k, seed, replay, od, out_index);
    return check_launch("list_sample_uniform");
  }
  const int64_t m = n < k ? n : k;  // n <= k: identity (list_sampling.cu:29-32)
  hipLaunchKernelGGL(iota_kernel, dim3(blocks_for(m, kThreads)), dim3(kThreads), 0, st, out_index, m);
  if (n > k) {
    const int64_t nq = ((n - 1) >> 2) - (k >> 2) + 1;
    hipLaunchKernelGGL(list_reservoir_kernel, dim3(blocks_for(nq, kThreads)), dim3(kThreads), 0, st,
                       n, k, seed, replay, out_index);
  }
  hipLaunchKernelGGL((list_gather_kernel<IdT>), dim3(blocks_for(m, kThreads)), dim3(kThreads), 0, st,
                     d, out_index, m, od);
  return check_launch("list_sample_uniform");
}

template <typename IdT>
int list_weighted_impl(const void* data, const float* probs, int64_t n, int64_t k, uint64_t seed,
                       const uint32_t* replay, void* out_data, int64_t* out_index,
                       const WeightedScratch& s, hipStream_t st) {
  const int64_t tiles = (n + kThreads * 8 - 1) / (kThreads * 8);
  const unsigned grid = static_cast<unsigned>(tiles < 256 ? (tiles < 1 ? 1 : tiles) : 256);
  hipLaunchKernelGGL(select_init_kernel, dim3(1), dim3(kThreads), 0, st, s.hist, s.state, k);
  hipLaunchKernelGGL(keys_hist_kernel, dim3(grid), dim3(kThreads), 0, st, probs, n, seed, replay,
                     s.okey, s.hist);
  for (int level = 1; level < kLevels; ++level)
    hipLaunchKernelGGL(level_hist_kernel, dim3(grid), dim3(kThreads), 0, st, s.okey, n, level,
                       s.state, s.hist);
  hipLaunchKernelGGL(survivors_kernel, dim3(grid), dim3(kThreads), 0, st, s.okey, n, s.state, s.hist,
                     s.cand, k);
  int padded_k = 2;
  while (padded_k < k) padded_k <<= 1;
  hipLaunchKernelGGL((sort_emit_kernel<IdT>), dim3(1), dim3(1024),
                     static_cast<size_t>(padded_k) * 8, st, s.cand, k, padded_k,
                     static_cast<const IdT*>(data), static_cast<IdT*>(out_data), out_index);
  return check_launch("list_sample_weighted");
}

}  // namespace
}  // namespace gs

using namespace gs;

extern "C" {

size_t gs_list_sample_workspace_bytes(int64_t n, int64_t k) {
  if (n < 1) n = 1;
  if (k < 1) k = 1;
  return padded(static_cast<size_t>(n) * 4) + padded(kLevels * kBins * 4) +
         padded(kLevels * sizeof(SelectState)) + padded(static_cast<size_t>(k) * 8);
}

int gs_list_sample_uniform(const void* data, int id_bytes, int64_t n, int64_t k, int replace,
                           uint64_t seed, const uint32_t* replay, void* out_data,
                           int64_t* out_index, void* workspace, size_t workspace_bytes,
                           void* stream) {
  (void)workspace;
  (void)workspace_bytes;
  GS_REQUIRE(n >= 0 && k >= 0, "gs_list_sample_uniform: negative size");
  GS_REQUIRE(valid_id_bytes(id_bytes), "gs_list_sample_uniform: id_bytes must be 4 or 8, got %d",
             id_bytes);
  if (k == 0 || n == 0) return GS_OK;
  GS_REQUIRE(data && out_data && out_index, "gs_list_sample_uniform: null pointer");
  hipStream_t st = static_cast<hipStream_t>(stream);
  return id_bytes == 8
             ? list_uniform_impl<int64_t>(data, n, k, replace, seed, replay, out_data, out_index, st)
             : list_uniform_impl<int32_t>(data, n, k, replace, seed, replay, out_data, out_index, st);
}

int gs_list_sample_weighted(const void* data, int id_bytes, const float* probs, int64_t n,
                            int64_t k, uint64_t seed, const uint32_t* replay, void* out_data,
                            int64_t* out_index, void* workspace, size_t workspace_bytes,
                            void* stream) {
  GS_REQUIRE(n >= 0 && k >= 0, "gs_list_sample_weighted: negative size");
  GS_REQUIRE(valid_id_bytes(id_bytes), "gs_list_sample_weighted: id_bytes must be 4 or 8, got %d",
             id_bytes);
  if (k == 0 || n == 0) return GS_OK;
  GS_REQUIRE(data && probs && out_data && out_index, "gs_list_sample_weighted: null pointer");
  GS_REQUIRE(n > k, "gs_list_sample_weighted: n <= k is the identity and is left to the caller");
  if (k > kMaxWeightedPicks || n >= (int64_t(1) << 32)) {
    set_error_text("gs_list_sample_weighted: k = %lld above the supported %lld (or n >= 2^32)",
                   static_cast<long long>(k), static_cast<long long>(kMaxWeightedPicks));
    return GS_ERR_UNSUPPORTED;
  }
  WeightedScratch s = carve_weighted(workspace, workspace_bytes, n, k);
  if (!s.ok) {
    set_error_text("gs_list_sample_weighted: workspace needs %zu bytes, 256-byte aligned",
                   gs_list_sample_workspace_bytes(n, k));
    return GS_ERR_WORKSPACE;
  }
  hipStream_t st = static_cast<hipStream_t>(stream);
  return id_bytes == 8 ? list_weighted_impl<int64_t>(data, probs, n, k, seed, replay, out_data,
                                                     out_index, s, st)
                       : list_weighted_impl<int32_t>(data, probs, n, k, seed, replay, out_data,
                                                     out_index, s, st);
}

}  // extern "C"
