// Weighted neighbour sampling without replacement (A-Res) on gfx950.
//
// Replaces impl::CSCColSamplingProbsCUDA (reference
// src/cuda/sampling_probs.cu:268; kernel :25-110, which keeps a faiss
// WarpSelect heap per warp and is limited to fanout <= 32, :32).
//
// Every edge of a row with deg > k gets the key log2(u)/w (same order as the
// reference's u^(1/w), :71) and the k largest keys win, emitted in descending
// key order, ties by lower position.  Key and position travel as one 64-bit
// composite (ordered key << 32 | ~position): composites are distinct, so
// "largest k" is unambiguous and bit-reproducible.
//
// Selection is a wave-level top-k over at most 2048 candidates, 32 per lane, held in
// registers: the k-th largest of the 64 lanes' own maxima is a floor that at least k
// candidates reach, so everything below it is dropped at once; the few survivors
// (between k and 32 k, typically about 2 k) are packed into LDS with ballots and each
// one counts how many survivors beat it -- that count is its place in the output.  No
// per-lane sorted lists, no k rounds of wave-wide maxima.  Rows up to 2048 edges are
// one wave each.  Longer rows are cut into 2048-edge chunks that go through a device
// queue: one wave per chunk writes its local top-k composites, then one wave per
// long row merges them (per-lane sorted lists in LDS and k rounds of "largest head
// wins": the candidates of a hub's chunks can be many more than 2048).  That spreads a
// 10^5-edge hub over hundreds of waves instead of pinning one warp on it.
#include "gs_common.hpp"

namespace gs {
namespace {

constexpr int64_t kChunk = 2048;          // edges per wave task
constexpr int64_t kMaxFanout = 96;        // 64 lanes * 96 * 8 B = 48 KB of LDS per wave
constexpr int kQueueGrid = 1024;          // workgroups draining a queue
constexpr int64_t kQueueExtra = 1 << 19;  // chunk-queue capacity = S + kQueueExtra
constexpr int kQueueParts = 64;           // one lane per part where the parts are added up

template <typename IdT>
struct WArgs {
  const int64_t* indptr;
  const IdT* indices;
  const float* probs;
  const IdT* cols;
  int64_t num_cols;
  int64_t S;
  int k;
  uint64_t seed;
  const uint32_t* replay;
  const int64_t* replay_ptr;
  const int64_t* sub_indptr;
  IdT* sub_indices;
  int64_t* select_index;
  IdT* coo_col;
  // long rows
  // [1] long rows, [2 + q] chunks reserved in part q of the queue.  The queue is kept in
  // kQueueParts parts, each with a counter of its own (a workgroup reserves in part
  // blockIdx % kQueueParts): reservations at ONE counter queue up at its address, 11 ns
  // apiece, and 2000 rows above 256 edges among 45 k made that the rows kernel's last 20 us.
  unsigned long long* counters;
  long long* chunk_queue;        // row << 20 | chunk, -1 = void
  int64_t chunk_cap;             // slots of one part
  long long* long_rows;          // 3 entries per long row: row, first queue slot, #chunks
  unsigned long long* cand;      // chunk_cap * k composites
};

__device__ __forceinline__ unsigned long long composite(float key, uint32_t pos) {
  return (static_cast<unsigned long long>(float_to_ordered(key)) << 32) | (0xFFFFFFFFu - pos);
}
__device__ __forceinline__ uint32_t composite_pos(unsigned long long c) {
  return 0xFFFFFFFFu - static_cast<uint32_t>(c);
}

// insert c into this lane's descending list (at most k entries)
__device__ __forceinline__ void lane_insert(unsigned long long* list, int lane, int& cnt, int k,
                                            unsigned long long c) {
  if (cnt == k && c <= list[(k - 1) * kWave + lane]) return;
  int j = cnt < k ? cnt : k - 1;
  while (j > 0 && list[(j - 1) * kWave + lane] < c) {
    list[j * kWave + lane] = list[(j - 1) * kWave + lane];
    --j;
  }
  list[j * kWave + lane] = c;
  if (cnt < k) ++cnt;
}

__device__ __forceinline__ unsigned long long wave_max(unsigned long long v) {
#pragma unroll
  for (int d = kWave / 2; d > 0; d >>= 1) {
    const unsigned long long o = __shfl_xor(v, d, kWave);
    v = o > v ? o : v;
  }
  return v;
}

// k rounds of "largest list head wins"; emit(j, composite) is called by every
// lane with the same arguments (0 = fewer than j+1 candidates existed).
template <typename Emit>
__device__ __forceinline__ void wave_drain(const unsigned long long* list, int lane, int cnt, int k,
                                           Emit emit) {
  int head = 0;
  for (int j = 0; j < k; ++j) {
    const unsigned long long mine = head < cnt ? list[head * kWave + lane] : 0ull;
    const unsigned long long best = wave_max(mine);
    if (best != 0ull && mine == best) ++head;
    emit(j, best);
  }
}

template <typename IdT>
__device__ __forceinline__ unsigned long long edge_composite(const WArgs<IdT>& a, int64_t r,
                                                             int64_t start, const uint32_t* rp,
                                                             int64_t i, const U4& x) {
  const uint32_t xv = rp ? rp[i] : x.v[i & 3];
  return composite(ares_key(xv, a.probs[start + i]), static_cast<uint32_t>(i));
}

constexpr int kTrips = kChunk / (4 * kWave);  // a lane holds 4 consecutive edges per trip
constexpr int64_t kSmall = 4 * kWave;         // rows of one trip: selected where they are found

// composites of edges [lo, hi) of row r (lo a multiple of 2048, hi - lo <= TRIPS * 256):
// the lane's share, 0 where it has none.  A lane takes 4 consecutive edges (one Philox
// block) per trip.
template <int TRIPS, typename IdT>
__device__ __forceinline__ void load_items(const WArgs<IdT>& a, int64_t r, int64_t start,
                                           int64_t lo, int64_t hi, int lane,
                                           unsigned long long (&items)[TRIPS][4]) {
  const uint32_t* rp = a.replay ? a.replay + a.replay_ptr[r] : nullptr;
#pragma unroll
  for (int t = 0; t < TRIPS; ++t) {
    const int64_t q = (lo >> 2) + lane + t * kWave;
#pragma unroll
    for (int j = 0; j < 4; ++j) items[t][j] = 0ull;
    if (q * 4 < hi) {
      U4 x;
      if (!rp) x = draw_block(a.seed, kTagWeighted, static_cast<uint64_t>(r), static_cast<uint64_t>(q));
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const int64_t i = q * 4 + j;
        if (i < hi) items[t][j] = edge_composite(a, r, start, rp, i, x);
      }
    }
  }
}

__device__ __forceinline__ unsigned long long lane_value(unsigned long long v, int l) {
  const uint32_t lo = __builtin_amdgcn_readlane(static_cast<uint32_t>(v), l);
  const uint32_t hi = __builtin_amdgcn_readlane(static_cast<uint32_t>(v >> 32), l);
  return (static_cast<unsigned long long>(hi) << 32) | lo;
}

// The k largest of the wave's items, in descending order: emit(place, composite) is called
// once per winner by the lane that holds it in the end; returns how many there were
// (fewer than k when the wave holds fewer items).  `list` is the wave's k * 64 LDS words.
// Every lane of the wave calls this.
template <int TRIPS, typename Emit>
__device__ __forceinline__ int wave_topk(const unsigned long long (&items)[TRIPS][4],
                                         unsigned long long* list, int lane, int k, Emit emit) {
  unsigned long long mx = 0ull;
#pragma unroll
  for (int t = 0; t < TRIPS; ++t)
#pragma unroll
    for (int j = 0; j < 4; ++j) mx = items[t][j] > mx ? items[t][j] : mx;
  // floor: the k-th largest of the lanes' maxima (composites are distinct; lanes without
  // items hold 0 and never qualify).  At least k items reach it, so the winners do.
  int greater = 0;
#pragma unroll 8
  for (int l = 0; l < kWave; ++l) greater += lane_value(mx, l) > mx ? 1 : 0;
  const unsigned long long holder = __ballot(mx != 0ull && greater == k - 1);
  const unsigned long long floor_c = holder ? lane_value(mx, __ffsll(holder) - 1) : 0ull;
  // survivors, packed into LDS in (trip, item, lane) order
  const unsigned long long lower = (1ull << lane) - 1ull;
  int n = 0;
#pragma unroll
  for (int t = 0; t < TRIPS; ++t) {
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const bool keep = items[t][j] != 0ull && items[t][j] >= floor_c;
      const unsigned long long votes = __ballot(keep);
      if (keep) list[n + __popcll(votes & lower)] = items[t][j];
      n += __popcll(votes);
    }
  }
  // the wave's own stores must have landed before other lanes read them back
  __builtin_amdgcn_fence(__ATOMIC_SEQ_CST, "workgroup");
  for (int i = lane; i < n; i += kWave) {
    const unsigned long long mine = list[i];
    int place = 0;
    for (int x = 0; x < n; ++x) place += list[x] > mine ? 1 : 0;
    if (place < k) emit(place, mine);
  }
  // the list is free again only when every lane has finished reading it
  __builtin_amdgcn_fence(__ATOMIC_SEQ_CST, "workgroup");
  return n < k ? n : k;
}

// pick number j of row r is the edge the composite names; called by one lane
template <typename IdT, bool WITH_COO>
__device__ __forceinline__ void emit_final(const WArgs<IdT>& a, int64_t r, int64_t start,
                                           int64_t out_start, int j, unsigned long long c) {
  const int64_t q = start + composite_pos(c);
  a.sub_indices[out_start + j] = a.indices[q];
  a.select_index[out_start + j] = q;
  if (WITH_COO) a.coo_col[out_start + j] = static_cast<IdT>(r);
}

// One wave per row.  deg <= k: copy; deg <= 256: select here; longer: queue (rows up to
// 2048 edges as one chunk that the chunk pass finishes by itself).
template <typename IdT, bool WITH_COO>
__global__ void weighted_rows_kernel(WArgs<IdT> a) {
  extern __shared__ unsigned long long s_lists[];
  const int lane = threadIdx.x & (kWave - 1);
  const int wave = threadIdx.x / kWave;
  const int waves = blockDim.x / kWave;
  unsigned long long* list = s_lists + static_cast<size_t>(wave) * a.k * kWave;
  const int64_t r = static_cast<int64_t>(blockIdx.x) * waves + wave;
  if (r >= a.S) return;
  const int64_t c = a.cols ? static_cast<int64_t>(a.cols[r]) : r;
  // an id outside [0, num_cols) is an empty column
  if (static_cast<uint64_t>(c) >= static_cast<uint64_t>(a.num_cols)) return;
  const int64_t start = a.indptr[c];
  const int64_t deg = a.indptr[c + 1] - start;
  const int64_t out_start = a.sub_indptr[r];
  if (deg <= a.k) {
    for (int64_t j = lane; j < deg; j += kWave) {
      a.sub_indices[out_start + j] = a.indices[start + j];
      a.select_index[out_start + j] = start + j;
      if (WITH_COO) a.coo_col[out_start + j] = static_cast<IdT>(r);
    }
    return;
  }
  bool here = deg <= kSmall;
  if (!here) {
    const int64_t nchunks = (deg + kChunk - 1) / kChunk;
    const int64_t part = blockIdx.x & (kQueueParts - 1);
    const int64_t part0 = part * a.chunk_cap;
    unsigned long long base = 0;
    if (lane == 0)
      base = atomicAdd(&a.counters[2 + part], static_cast<unsigned long long>(nchunks));
    base = __shfl(base, 0, kWave);
    if (static_cast<int64_t>(base) + nchunks <= a.chunk_cap) {
      for (int64_t ch = lane; ch < nchunks; ch += kWave)
        a.chunk_queue[part0 + base + ch] = static_cast<long long>((r << 20) | ch);
      if (lane == 0 && nchunks > 1) {
        const unsigned long long slot = atomicAdd(&a.counters[1], 1ull);
        a.long_rows[slot * 3 + 0] = r;
        a.long_rows[slot * 3 + 1] = part0 + static_cast<long long>(base);
        a.long_rows[slot * 3 + 2] = nchunks;
      }
    } else {
      // this part of the queue is full: void the reserved tail and select the whole row with
      // this wave
      for (int64_t ch = static_cast<int64_t>(base) + lane;
           ch < a.chunk_cap && ch < static_cast<int64_t>(base) + nchunks; ch += kWave)
        a.chunk_queue[part0 + ch] = -1;
      here = true;
    }
  }
  if (here && deg <= kSmall) {
    unsigned long long items[1][4];
    load_items<1>(a, r, start, 0, deg, lane, items);
    wave_topk<1>(items, list, lane, a.k, [&](int j, unsigned long long c) {
      emit_final<IdT, WITH_COO>(a, r, start, out_start, j, c);
    });
  } else if (here) {
    // a row that found the queue full: this wave streams it whole
    int cnt = 0;
    for (int64_t i = lane; i < deg; i += kWave) {
      U4 x;
      const uint32_t* rp = a.replay ? a.replay + a.replay_ptr[r] : nullptr;
      if (!rp) x = draw_block(a.seed, kTagWeighted, static_cast<uint64_t>(r), static_cast<uint64_t>(i >> 2));
      lane_insert(list, lane, cnt, a.k, edge_composite(a, r, start, rp, i, x));
    }
    wave_drain(list, lane, cnt, a.k, [&](int j, unsigned long long best) {
      if (lane == (j & (kWave - 1)) && best != 0ull)
        emit_final<IdT, WITH_COO>(a, r, start, out_start, j, best);
    });
  }
}

// One wave per queued chunk: local top-k composites -> cand[slot * k + j]; the only chunk
// of a row is final and goes to the output.
template <typename IdT, bool WITH_COO>
__global__ void weighted_chunks_kernel(WArgs<IdT> a) {
  extern __shared__ unsigned long long s_lists[];
  const int lane = threadIdx.x & (kWave - 1);
  const int wave = threadIdx.x / kWave;
  const int waves = blockDim.x / kWave;
  unsigned long long* list = s_lists + static_cast<size_t>(wave) * a.k * kWave;
  // lane q: entries of part q, and how many lie in the parts before it
  static_assert(kQueueParts == kWave, "one lane per part of the queue");
  const unsigned long long reserved = a.counters[2 + lane];
  const int64_t mine = reserved < static_cast<unsigned long long>(a.chunk_cap)
                           ? static_cast<int64_t>(reserved)
                           : a.chunk_cap;
  int64_t incl = mine;
#pragma unroll
  for (int d = 1; d < kWave; d <<= 1) {
    const int64_t o = __shfl_up(incl, d, kWave);
    if (lane >= d) incl += o;
  }
  const int64_t before = incl - mine;
  const int64_t n = __shfl(incl, kWave - 1, kWave);
  for (int64_t v = static_cast<int64_t>(blockIdx.x) * waves + wave; v < n;
       v += static_cast<int64_t>(gridDim.x) * waves) {
    int lo_part = 0, hi_part = kQueueParts;  // the last part that starts at or before v
#pragma unroll
    for (int step = 0; step < 6; ++step) {
      const int mid = (lo_part + hi_part) >> 1;
      if (__shfl(before, mid, kWave) <= v) lo_part = mid; else hi_part = mid;
    }
    const int64_t t = static_cast<int64_t>(lo_part) * a.chunk_cap + (v - __shfl(before, lo_part, kWave));
    const long long e = a.chunk_queue[t];
    if (e < 0) continue;
    const int64_t r = e >> 20;
    const int64_t ch = e & ((1 << 20) - 1);
    const int64_t c = a.cols ? static_cast<int64_t>(a.cols[r]) : r;
    const int64_t start = a.indptr[c];
    const int64_t deg = a.indptr[c + 1] - start;
    const int64_t lo = ch * kChunk;
    const int64_t hi = lo + kChunk < deg ? lo + kChunk : deg;
    unsigned long long items[kTrips][4];
    load_items<kTrips>(a, r, start, lo, hi, lane, items);
    if (deg <= kChunk) {
      const int64_t out_start = a.sub_indptr[r];
      wave_topk<kTrips>(items, list, lane, a.k, [&](int j, unsigned long long c) {
        emit_final<IdT, WITH_COO>(a, r, start, out_start, j, c);
      });
      continue;
    }
    unsigned long long* out = a.cand + static_cast<size_t>(t) * a.k;
    const int found = wave_topk<kTrips>(items, list, lane, a.k,
                                        [&](int j, unsigned long long c) { out[j] = c; });
    for (int j = found + lane; j < a.k; j += kWave) out[j] = 0ull;  // fewer than k edges
  }
}

// One wave per long row: merge its chunks' candidates.
template <typename IdT, bool WITH_COO>
__global__ void weighted_merge_kernel(WArgs<IdT> a) {
  extern __shared__ unsigned long long s_lists[];
  const int lane = threadIdx.x & (kWave - 1);
  const int wave = threadIdx.x / kWave;
  const int waves = blockDim.x / kWave;
  unsigned long long* list = s_lists + static_cast<size_t>(wave) * a.k * kWave;
  const int64_t n = static_cast<int64_t>(a.counters[1]);
  for (int64_t t = static_cast<int64_t>(blockIdx.x) * waves + wave; t < n;
       t += static_cast<int64_t>(gridDim.x) * waves) {
    const int64_t r = a.long_rows[t * 3 + 0];
    const int64_t base = a.long_rows[t * 3 + 1];
    const int64_t m = a.long_rows[t * 3 + 2] * a.k;
    const int64_t c = a.cols ? static_cast<int64_t>(a.cols[r]) : r;
    const int64_t start = a.indptr[c];
    const int64_t out_start = a.sub_indptr[r];
    const unsigned long long* src = a.cand + static_cast<size_t>(base) * a.k;
    if (m <= kChunk) {
      // few enough candidates for the register-resident selection (0 = an empty slot)
      unsigned long long items[kTrips][4];
#pragma unroll
      for (int tr = 0; tr < kTrips; ++tr)
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          const int64_t i = (static_cast<int64_t>(tr) * 4 + j) * kWave + lane;
          items[tr][j] = i < m ? src[i] : 0ull;
        }
      wave_topk<kTrips>(items, list, lane, a.k, [&](int j, unsigned long long cmp) {
        emit_final<IdT, WITH_COO>(a, r, start, out_start, j, cmp);
      });
      continue;
    }
    int cnt = 0;
    for (int64_t i = lane; i < m; i += kWave) {
      const unsigned long long cmp = src[i];
      if (cmp != 0ull) lane_insert(list, lane, cnt, a.k, cmp);
    }
    wave_drain(list, lane, cnt, a.k, [&](int j, unsigned long long best) {
      if (lane == (j & (kWave - 1)) && best != 0ull)
        emit_final<IdT, WITH_COO>(a, r, start, out_start, j, best);
    });
  }
}

static __global__ void zero2_kernel(unsigned long long* p) {
  for (int i = threadIdx.x; i < 2 + kQueueParts; i += blockDim.x) p[i] = 0;
}

int waves_per_block(int64_t k) {
  // 48 KB of LDS per workgroup
  const int64_t per_wave = k * kWave * 8;
  int w = static_cast<int>((48 * 1024) / per_wave);
  return w >= 4 ? 4 : (w >= 2 ? 2 : 1);
}

template <typename IdT, bool WITH_COO>
int weighted_launch(const WArgs<IdT>& a, hipStream_t st) {
  const int waves = waves_per_block(a.k);
  const size_t lds = static_cast<size_t>(waves) * a.k * kWave * 8;
  const dim3 block(waves * kWave);
  hipLaunchKernelGGL(zero2_kernel, dim3(1), dim3(64), 0, st, a.counters);
  hipLaunchKernelGGL((weighted_rows_kernel<IdT, WITH_COO>),
                     dim3(static_cast<unsigned>((a.S + waves - 1) / waves)), block, lds, st, a);
  hipLaunchKernelGGL((weighted_chunks_kernel<IdT, WITH_COO>), dim3(kQueueGrid), block, lds, st, a);
  hipLaunchKernelGGL((weighted_merge_kernel<IdT, WITH_COO>), dim3(kQueueGrid), block, lds, st, a);
  return check_launch("sample_weighted");
}

template <typename IdT>
int weighted_impl(const int64_t* indptr, int64_t num_cols, const void* indices, const float* probs,
                  const void* cols, int64_t S, int64_t k, uint64_t seed, const uint32_t* replay,
                  const int64_t* replay_ptr, const int64_t* sub_indptr, void* sub_indices,
                  int64_t* select_index, void* coo_col, void* workspace, size_t workspace_bytes,
                  hipStream_t st) {
  Carver ws(workspace, workspace_bytes);
  WArgs<IdT> a;
  a.indptr = indptr;
  a.indices = static_cast<const IdT*>(indices);
  a.probs = probs;
  a.cols = static_cast<const IdT*>(cols);
  a.num_cols = num_cols;
  a.S = S;
  a.k = static_cast<int>(k);
  a.seed = seed;
  a.replay = replay;
  a.replay_ptr = replay_ptr;
  a.sub_indptr = sub_indptr;
  a.sub_indices = static_cast<IdT*>(sub_indices);
  a.select_index = select_index;
  a.coo_col = static_cast<IdT*>(coo_col);
  a.chunk_cap = (S + kQueueExtra) / kQueueParts;
  a.counters = ws.take<unsigned long long>(2 + kQueueParts);
  a.chunk_queue = ws.take<long long>(static_cast<size_t>(a.chunk_cap) * kQueueParts);
  a.long_rows = ws.take<long long>(static_cast<size_t>(S) * 3);
  a.cand = ws.take<unsigned long long>(static_cast<size_t>(a.chunk_cap) * kQueueParts * k);
  if (!ws.ok) {
    set_error_text("gs_sample_weighted_fill: workspace needs %zu bytes, 256-byte aligned",
                   gs_sample_weighted_workspace_bytes(S, k));
    return GS_ERR_WORKSPACE;
  }
  return coo_col ? weighted_launch<IdT, true>(a, st) : weighted_launch<IdT, false>(a, st);
}

// ------------------------------------------------ with replacement (inverse CDF) ----
// Replaces _CSRRowWiseSampleReplaceKernel (reference src/cuda/sampling_probs.cu:112-183).
// The prefix sums of max(prob, 0) over a column are built 64 edges at a time with a
// Kogge-Stone scan over the wave (x[i] += x[i-d], d = 1..32; the running total enters the
// next chunk through its first element, as in the reference's WarpScan loop :147-160) and
// kept in the caller's scratch; then every lane draws picks and searches them.  That chain
// is sequential, so a column is cut into blocks of 2048 edges: each block is scanned from
// zero by a wave of its own, the blocks' totals are added up in order, and entry i of block
// b stands for (sum of the totals before b) + (its value inside the block).  Columns up to
// 2048 edges are one block and one wave; a hub of 300 k edges is 146 waves instead of one
// wave walking 4640 chunks.  The order of the float additions is fixed by that scheme, so a
// host evaluation of the same steps gives the same bits.
constexpr int64_t kCdfBlock = 2048;
constexpr int kMaxBases = 2048;  // block sums of a column kept in LDS: columns up to 4 M edges

// prefix sums of max(prob, 0) over edges [lo, hi) of a column, from zero; returns their total
__device__ __forceinline__ float scan_block(const float* __restrict__ prob, int64_t lo, int64_t hi,
                                            float* __restrict__ out, int lane) {
  float carry = 0.0f;
  for (int64_t base = lo; base < hi; base += kWave) {
    float x = base + lane < hi ? prob[base + lane] : 0.0f;
    if (lane == 0) x += carry;
    x = x > 0.0f ? x : 0.0f;
#pragma unroll
    for (int d = 1; d < kWave; d <<= 1) {
      const float y = __shfl_up(x, d, kWave);
      if (lane >= d) x += y;
    }
    carry = __shfl(x, kWave - 1, kWave);
    if (base + lane < hi) out[base + lane] = x;
  }
  return carry;
}

// pick number j of row r: position `at` of the column that starts at `start`
template <typename IdT, bool WITH_COO>
__device__ __forceinline__ void emit_pick(const IdT* __restrict__ indices, int64_t start, int64_t at,
                                          int64_t r, int64_t slot, IdT* __restrict__ sub_indices,
                                          int64_t* __restrict__ select_index,
                                          IdT* __restrict__ coo_col) {
  sub_indices[slot] = indices[start + at];
  select_index[slot] = start + at;
  if (WITH_COO) coo_col[slot] = static_cast<IdT>(r);
}

__device__ __forceinline__ float pick_point(uint64_t seed, const uint32_t* __restrict__ replay,
                                            int64_t r, int64_t k, int64_t j, float total) {
  const uint32_t xd = replay ? replay[r * k + j]
                             : draw_one(seed, kTagWeighted, static_cast<uint64_t>(r),
                                        static_cast<uint64_t>(j));
  const float u = static_cast<float>((xd >> 8) + 1u) * 5.9604644775390625e-08f;
  return u * total;
}

// One wave per column of at most 2048 edges: scan, then picks.
template <typename IdT, bool WITH_COO>
__global__ void __launch_bounds__(256)
weighted_replace_kernel(const int64_t* __restrict__ indptr, int64_t num_cols,
                        const IdT* __restrict__ indices, const float* __restrict__ probs,
                        const IdT* __restrict__ cols, int64_t S, int64_t k, uint64_t seed,
                        const uint32_t* __restrict__ replay, const int64_t* __restrict__ sub_indptr,
                        const int64_t* __restrict__ cdf_ptr, float* __restrict__ cdf,
                        IdT* __restrict__ sub_indices, int64_t* __restrict__ select_index,
                        IdT* __restrict__ coo_col) {
  const int lane = threadIdx.x & (kWave - 1);
  const int64_t r = static_cast<int64_t>(blockIdx.x) * (blockDim.x / kWave) + threadIdx.x / kWave;
  if (r >= S) return;
  const int64_t c = cols ? static_cast<int64_t>(cols[r]) : r;
  if (c < 0 || c >= num_cols) return;
  const int64_t start = indptr[c];
  const int64_t deg = indptr[c + 1] - start;
  if (deg <= 0 || deg > kCdfBlock) return;  // longer columns: the two kernels below
  float* my_cdf = cdf + cdf_ptr[r];
  const float total = scan_block(probs + start, 0, deg, my_cdf, lane);
  // the wave's own stores must have landed before other lanes read them back
  __builtin_amdgcn_fence(__ATOMIC_SEQ_CST, "workgroup");
  const int64_t out_start = sub_indptr[r];
  for (int64_t j = lane; j < k; j += kWave) {
    const float rnd = pick_point(seed, replay, r, k, j, total);
    // first the block (here the only one) whose last entry exceeds rnd, then inside it: the
    // same steps as for the longer columns.  Prefix sums made by different addition trees
    // need not be monotone to the last bit, so the order of the probes is part of the result.
    int64_t lo = deg, hi = deg;
    if (total > rnd) lo = 0;
    while (lo < hi) {
      const int64_t mid = (lo + hi) >> 1;
      if (my_cdf[mid] <= rnd) lo = mid + 1; else hi = mid;
    }
    if (lo > deg - 1) lo = deg - 1;
    emit_pick<IdT, WITH_COO>(indices, start, lo, r, out_start + j, sub_indices, select_index, coo_col);
  }
}

// Blocks of the longer columns.  The scratch `cdf` is the columns' edges one after the
// other (cdf_ptr), so the work is found without a queue: a wave takes 2048 consecutive
// scratch positions, and at most two columns longer than that can touch them -- the one
// that holds the first position and the one that holds the last.  Of each, at most one
// block STARTS inside the wave's positions; that block is the wave's.
template <typename IdT>
__global__ void __launch_bounds__(256)
replace_blocks_kernel(const int64_t* __restrict__ indptr, const float* __restrict__ probs,
                      const IdT* __restrict__ cols, int64_t S, const int64_t* __restrict__ cdf_ptr,
                      float* __restrict__ cdf) {
  const int lane = threadIdx.x & (kWave - 1);
  const int64_t waves = static_cast<int64_t>(gridDim.x) * (blockDim.x / kWave);
  const int64_t D = cdf_ptr[S];
  for (int64_t g = static_cast<int64_t>(blockIdx.x) * (blockDim.x / kWave) + threadIdx.x / kWave;
       g * kCdfBlock < D; g += waves) {
    const int64_t t0 = g * kCdfBlock;
    const int64_t t1 = t0 + kCdfBlock < D ? t0 + kCdfBlock : D;
    int64_t owner[2];
#pragma unroll
    for (int side = 0; side < 2; ++side) {
      const int64_t at = side == 0 ? t0 : t1 - 1;
      int64_t lo = 0, hi = S + 1;  // first r with cdf_ptr[r] > at
      while (lo < hi) {
        const int64_t mid = (lo + hi) >> 1;
        if (cdf_ptr[mid] <= at) lo = mid + 1; else hi = mid;
      }
      owner[side] = lo - 1;
    }
#pragma unroll
    for (int side = 0; side < 2; ++side) {
      const int64_t r = owner[side];
      if (side == 1 && r == owner[0]) break;
      if (r < 0 || r >= S) continue;
      const int64_t region = cdf_ptr[r];
      const int64_t deg = cdf_ptr[r + 1] - region;
      if (deg <= kCdfBlock) continue;
      const int64_t from = (t0 > region ? t0 : region) - region;
      const int64_t p = (from + kCdfBlock - 1) / kCdfBlock * kCdfBlock;  // block start in the column
      if (region + p >= t1 || p >= deg) continue;
      const int64_t c = cols ? static_cast<int64_t>(cols[r]) : r;
      scan_block(probs + indptr[c], p, p + kCdfBlock < deg ? p + kCdfBlock : deg, cdf + region, lane);
    }
  }
}

// One wave per column longer than 2048 edges, after its blocks have been scanned: the
// blocks' totals are added up in order (LDS), then the picks search first the block, then
// inside it, comparing (sum before the block) + (value inside the block).
template <typename IdT, bool WITH_COO>
__global__ void __launch_bounds__(256)
replace_long_kernel(const int64_t* __restrict__ indptr, int64_t num_cols,
                    const IdT* __restrict__ indices, const IdT* __restrict__ cols, int64_t S,
                    int64_t k, uint64_t seed, const uint32_t* __restrict__ replay,
                    const int64_t* __restrict__ sub_indptr, const int64_t* __restrict__ cdf_ptr,
                    const float* __restrict__ cdf, IdT* __restrict__ sub_indices,
                    int64_t* __restrict__ select_index, IdT* __restrict__ coo_col) {
  __shared__ float s_base[256 / kWave][kMaxBases + 1];
  const int lane = threadIdx.x & (kWave - 1);
  const int wave = threadIdx.x / kWave;
  const int64_t r = static_cast<int64_t>(blockIdx.x) * (blockDim.x / kWave) + wave;
  if (r >= S) return;
  const int64_t c = cols ? static_cast<int64_t>(cols[r]) : r;
  if (c < 0 || c >= num_cols) return;
  const int64_t start = indptr[c];
  const int64_t deg = indptr[c + 1] - start;
  if (deg <= kCdfBlock) return;
  const float* my_cdf = cdf + cdf_ptr[r];
  const int64_t nblocks = (deg + kCdfBlock - 1) / kCdfBlock;
  const bool staged = nblocks <= kMaxBases;
  float* base = s_base[wave];  // base[b] = sum of the totals of blocks 0 .. b-1
  float total = 0.0f;
  if (staged) {
    for (int64_t b = lane; b < nblocks; b += kWave) {
      const int64_t end = (b + 1) * kCdfBlock < deg ? (b + 1) * kCdfBlock : deg;
      base[b + 1] = my_cdf[end - 1];
    }
    __builtin_amdgcn_fence(__ATOMIC_SEQ_CST, "workgroup");
    if (lane == 0) {
      float acc = 0.0f;
      base[0] = 0.0f;
      for (int64_t b = 0; b < nblocks; ++b) {
        acc = acc + base[b + 1];
        base[b + 1] = acc;
      }
      total = acc;
    }
    __builtin_amdgcn_fence(__ATOMIC_SEQ_CST, "workgroup");
  } else if (lane == 0) {
    for (int64_t b = 0; b < nblocks; ++b) {
      const int64_t end = (b + 1) * kCdfBlock < deg ? (b + 1) * kCdfBlock : deg;
      total = total + my_cdf[end - 1];
    }
  }
  total = __shfl(total, 0, kWave);
  const int64_t out_start = sub_indptr[r];
  for (int64_t j = lane; j < k; j += kWave) {
    const float rnd = pick_point(seed, replay, r, k, j, total);
    // first block whose last entry exceeds rnd, and the sum before it
    int64_t b = 0;
    float before = 0.0f;
    if (staged) {
      int64_t lo = 0, hi = nblocks;
      while (lo < hi) {
        const int64_t mid = (lo + hi) >> 1;
        if (base[mid + 1] <= rnd) lo = mid + 1; else hi = mid;
      }
      b = lo;
      before = b < nblocks ? base[b] : 0.0f;
    } else {
      for (; b < nblocks; ++b) {
        const int64_t end = (b + 1) * kCdfBlock < deg ? (b + 1) * kCdfBlock : deg;
        const float next = before + my_cdf[end - 1];
        if (next > rnd) break;
        before = next;
      }
    }
    int64_t at = deg - 1;
    if (b < nblocks) {
      int64_t lo = b * kCdfBlock;
      int64_t hi = lo + kCdfBlock < deg ? lo + kCdfBlock : deg;
      while (lo < hi) {
        const int64_t mid = (lo + hi) >> 1;
        if (before + my_cdf[mid] <= rnd) lo = mid + 1; else hi = mid;
      }
      at = lo > deg - 1 ? deg - 1 : lo;
    }
    emit_pick<IdT, WITH_COO>(indices, start, at, r, out_start + j, sub_indices, select_index, coo_col);
  }
}

template <typename IdT, bool WITH_COO>
int weighted_replace_launch(const int64_t* indptr, int64_t num_cols, const IdT* indices,
                            const float* probs, const IdT* cols, int64_t S, int64_t k, uint64_t seed,
                            const uint32_t* replay, const int64_t* sub_indptr, const int64_t* cdf_ptr,
                            float* cdf, IdT* sub_indices, int64_t* select_index, IdT* coo_col,
                            hipStream_t st) {
  const dim3 grid(static_cast<unsigned>((S + 3) / 4)), block(4 * kWave);
  hipLaunchKernelGGL((weighted_replace_kernel<IdT, WITH_COO>), grid, block, 0, st, indptr, num_cols,
                     indices, probs, cols, S, k, seed, replay, sub_indptr, cdf_ptr, cdf, sub_indices,
                     select_index, coo_col);
  hipLaunchKernelGGL((replace_blocks_kernel<IdT>), dim3(512), block, 0, st, indptr, probs, cols, S,
                     cdf_ptr, cdf);
  hipLaunchKernelGGL((replace_long_kernel<IdT, WITH_COO>), grid, block, 0, st, indptr, num_cols,
                     indices, cols, S, k, seed, replay, sub_indptr, cdf_ptr, cdf, sub_indices,
                     select_index, coo_col);
  return check_launch("sample_weighted_replace");
}

template <typename IdT>
int weighted_replace_impl(const int64_t* indptr, int64_t num_cols, const void* indices,
                          const float* probs, const void* cols, int64_t S, int64_t k, uint64_t seed,
                          const uint32_t* replay, const int64_t* sub_indptr, const int64_t* cdf_ptr,
                          float* cdf, void* sub_indices, int64_t* select_index, void* coo_col,
                          hipStream_t st) {
  const IdT* ind = static_cast<const IdT*>(indices);
  const IdT* cl = static_cast<const IdT*>(cols);
  IdT* si = static_cast<IdT*>(sub_indices);
  IdT* cc = static_cast<IdT*>(coo_col);
  return coo_col ? weighted_replace_launch<IdT, true>(indptr, num_cols, ind, probs, cl, S, k, seed,
                                                     replay, sub_indptr, cdf_ptr, cdf, si,
                                                     select_index, cc, st)
                 : weighted_replace_launch<IdT, false>(indptr, num_cols, ind, probs, cl, S, k, seed,
                                                      replay, sub_indptr, cdf_ptr, cdf, si,
                                                      select_index, cc, st);
}

}  // namespace
}  // namespace gs

using namespace gs;

extern "C" {

size_t gs_sample_weighted_workspace_bytes(int64_t S, int64_t fanout) {
  if (S < 0) S = 0;
  if (fanout < 1) fanout = 1;
  const size_t cap = static_cast<size_t>(S + kQueueExtra);
  return padded((2 + kQueueParts) * 8) + padded(cap * 8) + padded(static_cast<size_t>(S) * 24) +
         padded(cap * static_cast<size_t>(fanout) * 8);
}

int gs_sample_weighted_fill(const int64_t* indptr, int64_t num_cols, const void* indices,
                            const float* probs, const void* column_ids, int id_bytes, int64_t S,
                            int64_t fanout,
                            uint64_t seed, const uint32_t* replay, const int64_t* replay_ptr,
                            const int64_t* sub_indptr, void* sub_indices, int64_t* select_index,
                            void* coo_col, void* workspace, size_t workspace_bytes, void* stream) {
  GS_REQUIRE(indptr && sub_indptr && S >= 0 && fanout >= 0 && num_cols >= 0,
             "gs_sample_weighted_fill: null pointer or negative size");
  GS_REQUIRE(column_ids || S <= num_cols,
             "gs_sample_weighted_fill: S exceeds num_cols without column_ids");
  GS_REQUIRE(valid_id_bytes(id_bytes), "gs_sample_weighted_fill: id_bytes must be 4 or 8, got %d",
             id_bytes);
  GS_REQUIRE((replay == nullptr) == (replay_ptr == nullptr),
             "gs_sample_weighted_fill: replay and replay_ptr must be given together");
  if (S == 0 || fanout == 0) return GS_OK;
  GS_REQUIRE(indices && probs && sub_indices && select_index,
             "gs_sample_weighted_fill: null buffer");
  if (fanout > kMaxFanout) {
    set_error_text("gs_sample_weighted_fill: fanout %lld above the supported %lld "
                   "(the reference stops at 32)",
                   static_cast<long long>(fanout), static_cast<long long>(kMaxFanout));
    return GS_ERR_UNSUPPORTED;
  }
  hipStream_t st = static_cast<hipStream_t>(stream);
  return id_bytes == 8
             ? weighted_impl<int64_t>(indptr, num_cols, indices, probs, column_ids, S, fanout, seed, replay,
                                      replay_ptr, sub_indptr, sub_indices, select_index, coo_col,
                                      workspace, workspace_bytes, st)
             : weighted_impl<int32_t>(indptr, num_cols, indices, probs, column_ids, S, fanout, seed, replay,
                                      replay_ptr, sub_indptr, sub_indices, select_index, coo_col,
                                      workspace, workspace_bytes, st);
}

int gs_sample_weighted_replace(const int64_t* indptr, int64_t num_cols, const void* indices,
                               const float* probs, const void* column_ids, int id_bytes, int64_t S,
                               int64_t fanout, uint64_t seed, const uint32_t* replay,
                               const int64_t* sub_indptr, const int64_t* cdf_ptr, float* cdf,
                               void* sub_indices, int64_t* select_index, void* coo_col,
                               void* stream) {
  GS_REQUIRE(indptr && sub_indptr && cdf_ptr && S >= 0 && fanout >= 0 && num_cols >= 0,
             "gs_sample_weighted_replace: null pointer or negative size");
  GS_REQUIRE(column_ids || S <= num_cols,
             "gs_sample_weighted_replace: S exceeds num_cols without column_ids");
  GS_REQUIRE(valid_id_bytes(id_bytes),
             "gs_sample_weighted_replace: id_bytes must be 4 or 8, got %d", id_bytes);
  if (S == 0 || fanout == 0) return GS_OK;
  GS_REQUIRE(indices && probs && cdf && sub_indices && select_index,
             "gs_sample_weighted_replace: null buffer");
  hipStream_t st = static_cast<hipStream_t>(stream);
  return id_bytes == 8
             ? weighted_replace_impl<int64_t>(indptr, num_cols, indices, probs, column_ids, S,
                                              fanout, seed, replay, sub_indptr, cdf_ptr, cdf,
                                              sub_indices, select_index, coo_col, st)
             : weighted_replace_impl<int32_t>(indptr, num_cols, indices, probs, column_ids, S,
                                              fanout, seed, replay, sub_indptr, cdf_ptr, cdf,
                                              sub_indices, select_index, coo_col, st);
}

}  // extern "C"
