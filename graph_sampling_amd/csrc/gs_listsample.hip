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
// (list_sampling_probs.cu:76-86).  Here one histogram pass finds the narrow class
// of composites (ordered key << 32 | ~position) that holds the k-th largest, a
// second pass sets aside what lies above it and the class itself, and one
// workgroup sorts those few items (bitonic, in LDS): the weights are read once,
// the 4-byte keys written once and read once.
#include "gs_common.hpp"

namespace gs {
namespace {

constexpr int kThreads = 256;
constexpr int64_t kMaxWeightedPicks = 8192;

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
// The picks are the k largest 64-bit composites (ordered key << 32 | ~position): larger key
// first, among equal keys the smaller position.  Four launches:
//  1. clear the histogram and the two counters;
//  2. keys (list_sampling_probs.cu:62-78) and a histogram over 4096 classes in composite
//     order: classes 2048.. = the top 11 bits of the key; classes 0..2047 = the items without
//     a positive weight (their keys are all -inf, so that among them only the position
//     decides), 2048 runs of consecutive positions, earlier runs above later ones;
//     the workgroup that finishes last finds, from the complete histogram, the class that
//     holds the k-th composite;
//  3. items of the classes above it are wanted outright and go to `cand`, the items of that
//     class go to `ties`;
//  4. the place of a pick in the result is the number of candidates above it: counted for 64
//     candidates per workgroup against all of them, those below place k emitted.
// The class of the k-th composite is narrow by construction: a key class is a quarter octave
// of the key's magnitude, which holds under 0.4 k items around the k-th largest of distinct
// keys whatever the weights are, and a run of positions holds n / 2048 items.  A class of
// more than 8192 items only arises from keys that repeat thousands of times (replayed draws
// that are all alike); one workgroup of step 3 then radix-selects inside the class over all n
// keys: right, and slow.
constexpr int kKeyBins = 2048;
constexpr int kClasses = 2 * kKeyBins;
constexpr uint32_t kOrderedNegInf = 0x007FFFFFu;  // float_to_ordered(-inf): no key is below it
constexpr int kTieCap = 8192;
constexpr int kInnerLevels = 5;  // digits of the composite below the key's top 11 bits
__constant__ int c_shift[kInnerLevels + 1] = {53, 42, 32, 21, 10, 0};
__constant__ int c_width[kInnerLevels + 1] = {11, 11, 10, 11, 11, 10};

// cand and ties are kept as kLists lists each (a workgroup appends to list blockIdx % kLists):
// additions to ONE counter queue up at its address, 11 ns apiece
constexpr int kLists = 64;
struct SelectCounters {
  unsigned int above[kLists];  // entries of the cand lists (k slots each)
  unsigned int ties[kLists];   // entries of the ties lists (kTieCap slots each)
  unsigned int finished;     // workgroups of the key pass that have added their counts
  // the class that holds the k-th largest composite (left by the key pass's last workgroup):
  // `pick_above` items sit in the classes over it, pick_above < k <= pick_above + pick_count
  uint32_t pick_class;
  uint32_t pick_count;
  uint32_t pick_above;
};
constexpr int kPassThreads = 1024;  // of the two passes over all items

__device__ __forceinline__ unsigned long long list_composite(uint32_t okey, int64_t i) {
  return (static_cast<unsigned long long>(okey) << 32) | (0xFFFFFFFFu - static_cast<uint32_t>(i));
}

// run_shift: the smallest shift with (n - 1) >> shift < 2048
__device__ __forceinline__ uint32_t class_of(uint32_t okey, int64_t i, int run_shift) {
  return okey == kOrderedNegInf
             ? static_cast<uint32_t>(kKeyBins - 1) - static_cast<uint32_t>(i >> run_shift)
             : static_cast<uint32_t>(kKeyBins) + (okey >> 21);
}

__global__ void __launch_bounds__(kThreads)
select_init_kernel(uint32_t* hist, SelectCounters* st) {
  for (int i = threadIdx.x; i < kClasses; i += kThreads) hist[i] = 0;
  if (threadIdx.x < kLists) {
    st->above[threadIdx.x] = 0;
    st->ties[threadIdx.x] = 0;
  }
  if (threadIdx.x == 0) st->finished = 0;
}

// A wave's items without weight lie in one run of positions or two: one count for those that
// share the first such lane's class, one each for the rest and for the items with a key.
__device__ __forceinline__ void count_class(uint32_t* s_hist, uint32_t cls, bool weightless) {
  if (!weightless) {
    atomicAdd(&s_hist[cls], 1u);
    return;
  }
  const uint32_t lead = __builtin_amdgcn_readfirstlane(cls);
  const unsigned long long same = __ballot(cls == lead);
  if (cls != lead) {
    atomicAdd(&s_hist[cls], 1u);
  } else if ((same & ((1ull << (threadIdx.x & (kWave - 1))) - 1ull)) == 0ull) {
    atomicAdd(&s_hist[cls], static_cast<uint32_t>(__popcll(same)));
  }
}

struct ClassPick {
  uint32_t cls;
  uint32_t count;
  int64_t above;
};
template <int THREADS>
struct PickScratch {
  int64_t scan[THREADS / kWave + 1];
  ClassPick out;
};
template <int THREADS>
__device__ __forceinline__ ClassPick pick_class(const uint32_t* hist, int64_t k,
                                                PickScratch<THREADS>* lds);

__global__ void __launch_bounds__(kPassThreads)
keys_hist_kernel(const float* __restrict__ probs, int64_t n, int run_shift, int64_t k, uint64_t seed,
                 const uint32_t* __restrict__ replay, uint32_t* __restrict__ okey,
                 uint32_t* hist, SelectCounters* st) {
  constexpr int kThreads = kPassThreads;
  __shared__ uint32_t s_hist[kClasses];
  __shared__ PickScratch<kPassThreads> s_pick;
  __shared__ bool s_last;
  for (int i = threadIdx.x; i < kClasses; i += kThreads) s_hist[i] = 0;
  __syncthreads();
  const int64_t nq = (n + 3) >> 2;
  const bool wide = (reinterpret_cast<uintptr_t>(probs) & 15u) == 0;  // okey is always aligned
  for (int64_t q = static_cast<int64_t>(blockIdx.x) * kThreads + threadIdx.x; q < nq;
       q += static_cast<int64_t>(gridDim.x) * kThreads) {
    U4 x;
    if (!replay) x = draw_block(seed, kTagListWeighted, 0, static_cast<uint64_t>(q));
    const bool full = q * 4 + 3 < n;
    float w[4];
    if (full && wide) {
      const float4 v = reinterpret_cast<const float4*>(probs)[q];
      w[0] = v.x, w[1] = v.y, w[2] = v.z, w[3] = v.w;
    } else {
#pragma unroll
      for (int t = 0; t < 4; ++t) w[t] = q * 4 + t < n ? probs[q * 4 + t] : 0.0f;
    }
    uint32_t ok[4];
#pragma unroll
    for (int t = 0; t < 4; ++t) {
      const int64_t i = q * 4 + t;
      const uint32_t xv = replay ? (i < n ? replay[i] : 0u) : x.v[t];
      ok[t] = float_to_ordered(ares_key(xv, w[t]));
      if (i < n) count_class(s_hist, class_of(ok[t], i, run_shift), ok[t] == kOrderedNegInf);
    }
    if (full) {
      reinterpret_cast<uint4*>(okey)[q] = make_uint4(ok[0], ok[1], ok[2], ok[3]);
    } else {
#pragma unroll
      for (int t = 0; t < 4; ++t)
        if (q * 4 + t < n) okey[q * 4 + t] = ok[t];
    }
  }
  __syncthreads();
  for (int i = threadIdx.x; i < kClasses; i += kThreads)
    if (s_hist[i]) atomicAdd(&hist[i], s_hist[i]);
  // The workgroup that finishes last sees every count and makes the pick for the later
  // launches.  The additions are device-scope operations, done where every workgroup sees them
  // once they are acknowledged, so every thread waits for the acknowledgements of its OWN
  // additions (the vector-memory counter; a workgroup-scope release alone need not wait for
  // them) before the barrier that precedes the ticket.  A device-scope fence would do too, but
  // writes the L2's dirty lines back first -- all the keys just stored, 60 us of it at
  // 2.45 M items.  The pick reads the counts past the caches (device-scope loads).
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
  __syncthreads();
  if (threadIdx.x == 0) s_last = atomicAdd(&st->finished, 1u) == gridDim.x - 1;
  __syncthreads();
  if (!s_last) return;
  const ClassPick pick = pick_class<kPassThreads>(hist, k, &s_pick);
  if (threadIdx.x == 0) {
    st->pick_class = pick.cls;
    st->pick_count = pick.count;
    st->pick_above = static_cast<uint32_t>(pick.above);
  }
}

// The class that holds the k-th largest composite, from the finished histogram: `above` items
// sit in the classes over it (above < k <= above + count).  Called by every thread of a
// workgroup of THREADS.
template <int THREADS>
__device__ __forceinline__ ClassPick pick_class(const uint32_t* hist, int64_t k,
                                                PickScratch<THREADS>* lds) {
  constexpr int kPer = kClasses / THREADS;  // consecutive classes of a thread
  uint32_t h[kPer];
  int64_t mine = 0;
#pragma unroll
  for (int j = 0; j < kPer; ++j) {
    h[j] = __hip_atomic_load(&hist[threadIdx.x * kPer + j], __ATOMIC_RELAXED,
                             __HIP_MEMORY_SCOPE_AGENT);
    mine += h[j];
  }
  int64_t total;
  const int64_t below = block_exclusive_scan<THREADS>(mine, &total, lds->scan);
  int64_t above = total - below - mine;  // classes of the threads after this one
  if (above < k && k <= above + mine) {
#pragma unroll
    for (int j = kPer - 1; j >= 0; --j) {
      if (above < k && k <= above + h[j]) {
        lds->out.cls = threadIdx.x * kPer + j;
        lds->out.count = h[j];
        lds->out.above = above;
      }
      above += h[j];
    }
  }
  __syncthreads();
  const ClassPick r = lds->out;
  __syncthreads();
  return r;
}

// The `want` largest composites of class `pick.cls` into out[0 .. want), in no order, when the
// class is too large to sort: a radix select over the five digits below the key's top 11 bits,
// every level a pass over all n keys by this one workgroup.
struct SelectScratch {
  uint32_t hist[kKeyBins];
  int64_t scan[kPassThreads / kWave + 1];
  unsigned long long word[4];
};

__device__ void select_in_class(const uint32_t* __restrict__ okey, int64_t n, int run_shift,
                                const ClassPick& pick, int64_t want, unsigned long long* out,
                                SelectScratch* lds) {
  uint32_t* s_hist = lds->hist;
  unsigned long long* s_word = lds->word;
  // every item of the class shares the key's top 11 bits
  unsigned long long prefix =
      static_cast<unsigned long long>(pick.cls >= static_cast<uint32_t>(kKeyBins)
                                          ? pick.cls - kKeyBins
                                          : kOrderedNegInf >> 21)
      << c_shift[0];
  int64_t remaining = want;
  bool done = false;
  for (int level = 1; level <= kInnerLevels && !done; ++level) {
    for (int i = threadIdx.x; i < kKeyBins; i += kPassThreads) s_hist[i] = 0;
    __syncthreads();
    const int up = c_shift[level - 1], sh = c_shift[level];
    const uint32_t mask = (1u << c_width[level]) - 1u;
    for (int64_t i = threadIdx.x; i < n; i += kPassThreads) {
      const uint32_t ok = okey[i];
      const unsigned long long c = list_composite(ok, i);
      if (class_of(ok, i, run_shift) == pick.cls && (c >> up) == (prefix >> up))
        atomicAdd(&s_hist[static_cast<uint32_t>(c >> sh) & mask], 1u);
    }
    __syncthreads();
    // the digit that holds the remaining-th largest: two digits a thread, scanned from the top
    constexpr int kPer = kKeyBins / kPassThreads;
    int64_t mine = 0;
#pragma unroll
    for (int j = 0; j < kPer; ++j) mine += s_hist[threadIdx.x * kPer + j];
    int64_t total;
    const int64_t below = block_exclusive_scan<kPassThreads>(mine, &total, lds->scan);
    int64_t above = total - below - mine;
    if (above < remaining && remaining <= above + mine) {
      for (int j = kPer - 1; j >= 0; --j) {
        const int64_t cnt = s_hist[threadIdx.x * kPer + j];
        if (above < remaining && remaining <= above + cnt) {
          s_word[0] = prefix | (static_cast<unsigned long long>(threadIdx.x * kPer + j) << sh);
          s_word[1] = static_cast<unsigned long long>(remaining - above);
          // the whole digit is wanted: with the lower digits left at zero "composite >= prefix"
          // already selects exactly the wanted items
          s_word[2] = remaining - above == cnt ? 1ull : 0ull;
        }
        above += cnt;
      }
    }
    __syncthreads();
    prefix = s_word[0];
    remaining = static_cast<int64_t>(s_word[1]);
    done = s_word[2] != 0ull;
    __syncthreads();
  }
  if (threadIdx.x == 0) s_word[3] = 0ull;
  __syncthreads();
  for (int64_t i = threadIdx.x; i < n; i += kPassThreads) {
    const uint32_t ok = okey[i];
    const unsigned long long c = list_composite(ok, i);
    if (class_of(ok, i, run_shift) == pick.cls && c >= prefix) {
      const unsigned long long slot = atomicAdd(&s_word[3], 1ull);
      if (static_cast<int64_t>(slot) < want) out[slot] = c;
    }
  }
}

__global__ void __launch_bounds__(kPassThreads)
partition_kernel(const uint32_t* __restrict__ okey, int64_t n, int run_shift, int64_t k,
                 SelectCounters* st, unsigned long long* __restrict__ cand,
                 unsigned long long* __restrict__ ties) {
  constexpr int kThreads = kPassThreads;
  ClassPick pick;
  pick.cls = st->pick_class;
  pick.count = st->pick_count;
  const bool keep_ties = pick.count <= static_cast<uint32_t>(kTieCap);
  const int64_t list = blockIdx.x % kLists;
  const int64_t nq = (n + 3) >> 2;
  for (int64_t q = static_cast<int64_t>(blockIdx.x) * kThreads + threadIdx.x; q < nq;
       q += static_cast<int64_t>(gridDim.x) * kThreads) {
    uint32_t ok[4] = {0u, 0u, 0u, 0u};
    if (q * 4 + 3 < n) {
      const uint4 v = reinterpret_cast<const uint4*>(okey)[q];
      ok[0] = v.x, ok[1] = v.y, ok[2] = v.z, ok[3] = v.w;
    } else {
#pragma unroll
      for (int t = 0; t < 4; ++t)
        if (q * 4 + t < n) ok[t] = okey[q * 4 + t];
    }
#pragma unroll
    for (int t = 0; t < 4; ++t) {
      const int64_t i = q * 4 + t;
      if (i >= n) continue;
      const uint32_t cls = class_of(ok[t], i, run_shift);
      if (cls > pick.cls) {
        const unsigned int slot = atomicAdd(&st->above[list], 1u);
        if (static_cast<int64_t>(slot) < k) cand[list * k + slot] = list_composite(ok[t], i);
      } else if (cls == pick.cls && keep_ties) {
        const unsigned int slot = atomicAdd(&st->ties[list], 1u);
        if (slot < static_cast<unsigned int>(kTieCap))
          ties[static_cast<int64_t>(list) * kTieCap + slot] = list_composite(ok[t], i);
      }
    }
  }
  // a class too large for the lists: one workgroup cuts it down to the wanted entries, as
  // the first ties list (nothing else has been put there)
  if (!keep_ties && blockIdx.x == 0) {
    __shared__ SelectScratch s_select;
    pick.above = st->pick_above;
    const int64_t want = k - pick.above;
    select_in_class(okey, n, run_shift, pick, want, ties, &s_select);
    if (threadIdx.x == 0) st->ties[0] = static_cast<unsigned int>(want);
  }
}

// exclusive scan over the wave's lanes
__device__ __forceinline__ int wave_starts(int v) {
  const int lane = threadIdx.x & (kWave - 1);
  int incl = v;
#pragma unroll
  for (int d = 1; d < kWave; d <<= 1) {
    const int o = __shfl_up(incl, d, kWave);
    if (lane >= d) incl += o;
  }
  return incl - v;
}

// Entry i of the picks' candidates: the total_a entries of the kLists lists A come first, then
// the total_b entries of the lists B (0 for an i beyond both).  List l of a family lies at its
// base + l * stride; lane l of the wave holds the list's start (the exclusive scan of the
// lists' lengths), searched by shuffle: whole waves call this.
__device__ __forceinline__ unsigned long long list_entry(
    int i, const unsigned long long* __restrict__ a, int64_t stride_a, int start_a, int total_a,
    const unsigned long long* __restrict__ b, int64_t stride_b, int start_b, int total_b) {
  static_assert(kLists == kWave, "one lane per list");
  const bool in_a = i < total_a;
  const int j = in_a ? i : i - total_a;
  int lo = 0, hi = kLists;  // last list whose start is <= j
#pragma unroll
  for (int step = 0; step < 6; ++step) {
    const int mid = (lo + hi) >> 1;
    const int sa = __shfl(start_a, mid, kWave), sb = __shfl(start_b, mid, kWave);
    if ((in_a ? sa : sb) <= j) lo = mid; else hi = mid;
  }
  const int fa = __shfl(start_a, lo, kWave), fb = __shfl(start_b, lo, kWave);
  if (i >= total_a + total_b) return 0ull;
  return in_a ? a[lo * stride_a + (j - fa)] : b[lo * stride_b + (j - fb)];
}

// The picks in descending order of their composites, without a sort: the place of a candidate
// is the number of candidates above it (composites are distinct).  A workgroup places 64
// candidates, one per lane; all candidates pass through LDS in chunks, and each of its
// sixteen waves counts against a sixteenth of a chunk, every lane reading the same word at a
// time.  The candidates above the k-th composite's class are all picks; of the class, those
// that land in a place below k.
constexpr int kRankThreads = 1024;
constexpr int kRankWaves = kRankThreads / kWave;
constexpr int kRankChunk = 4096;

template <typename IdT>
__global__ void __launch_bounds__(kRankThreads)
rank_emit_kernel(int64_t k, const SelectCounters* __restrict__ st,
                 const unsigned long long* __restrict__ cand,
                 const unsigned long long* __restrict__ ties, const IdT* __restrict__ data,
                 IdT* __restrict__ out_data, int64_t* __restrict__ out_index) {
  __shared__ unsigned long long s_chunk[kRankChunk];
  __shared__ int s_place[kWave];
  const int lane = threadIdx.x & (kWave - 1);
  const int wave = threadIdx.x / kWave;
  const uint32_t in_class = st->pick_count;
  const int above = static_cast<int>(st->pick_above);
  const int len_ties = static_cast<int>(st->ties[lane]);
  const int len_cand = static_cast<int>(st->above[lane]);
  // a class too large for its lists was cut down to the wanted entries by the pass before
  const int count = in_class <= static_cast<uint32_t>(kTieCap) ? static_cast<int>(in_class)
                                                                : static_cast<int>(k) - above;
  const int total = above + count;
  if (static_cast<int>(blockIdx.x) * kWave >= total) return;
  const int e = blockIdx.x * kWave + lane;
  const int start_ties = wave_starts(len_ties), start_cand = wave_starts(len_cand);
  const unsigned long long mine =
      list_entry(e, cand, k, start_cand, above, ties, kTieCap, start_ties, count);
  if (threadIdx.x < kWave) s_place[threadIdx.x] = 0;
  int place = 0;
  for (int c0 = 0; c0 < total; c0 += kRankChunk) {
    const int len = total - c0 < kRankChunk ? total - c0 : kRankChunk;
    for (int r = 0; r < (len + kRankThreads - 1) / kRankThreads; ++r) {
      const int i = r * kRankThreads + threadIdx.x;
      const unsigned long long c =
          list_entry(c0 + i, cand, k, start_cand, above, ties, kTieCap, start_ties, count);
      if (i < len) s_chunk[i] = c;
    }
    __syncthreads();
    const int per = (len + kRankWaves - 1) / kRankWaves;
    const int j1 = (wave + 1) * per < len ? (wave + 1) * per : len;
#pragma unroll 8
    for (int j = wave * per; j < j1; ++j) place += s_chunk[j] > mine ? 1 : 0;
    __syncthreads();
  }
  atomicAdd(&s_place[lane], place);
  __syncthreads();
  if (wave == 0 && e < total && s_place[lane] < k) {
    const int64_t pos = 0xFFFFFFFFu - static_cast<uint32_t>(mine);
    out_index[s_place[lane]] = pos;
    out_data[s_place[lane]] = data[pos];
  }
}

struct WeightedScratch {
  uint32_t* okey;
  uint32_t* hist;
  SelectCounters* state;
  unsigned long long* cand;
  unsigned long long* ties;
  bool ok;
};

WeightedScratch carve_weighted(void* ws_ptr, size_t bytes, int64_t n, int64_t k) {
  Carver ws(ws_ptr, bytes);
  WeightedScratch s;
  s.okey = ws.take<uint32_t>(n > 0 ? n : 1);
  s.hist = ws.take<uint32_t>(kClasses);
  s.state = ws.take<SelectCounters>(1);
  s.cand = ws.take<unsigned long long>(static_cast<size_t>(kLists) * (k > 0 ? k : 1));
  s.ties = ws.take<unsigned long long>(static_cast<size_t>(kLists) * kTieCap);
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
  const int64_t tiles = (n + kPassThreads * 8 - 1) / (kPassThreads * 8);
  const unsigned grid = static_cast<unsigned>(tiles < 256 ? (tiles < 1 ? 1 : tiles) : 256);
  int run_shift = 0;
  while (((n - 1) >> run_shift) >= kKeyBins) ++run_shift;
  hipLaunchKernelGGL(select_init_kernel, dim3(1), dim3(kThreads), 0, st, s.hist, s.state);
  hipLaunchKernelGGL(keys_hist_kernel, dim3(grid), dim3(kPassThreads), 0, st, probs, n, run_shift,
                     k, seed, replay, s.okey, s.hist, s.state);
  hipLaunchKernelGGL(partition_kernel, dim3(grid), dim3(kPassThreads), 0, st, s.okey, n, run_shift,
                     k, s.state, s.cand, s.ties);
  hipLaunchKernelGGL((rank_emit_kernel<IdT>), dim3(blocks_for(k + kTieCap, kWave)),
                     dim3(kRankThreads), 0, st, k, s.state, s.cand, s.ties,
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
  return padded(static_cast<size_t>(n) * 4) + padded(kClasses * 4) +
         padded(sizeof(SelectCounters)) + padded(static_cast<size_t>(kLists) * k * 8) +
         padded(static_cast<size_t>(kLists) * kTieCap * 8);
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
