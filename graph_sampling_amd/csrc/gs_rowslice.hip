// Row slicing (keep the edges whose row id is in a given set) on gfx950.
//
// Replaces impl::CSCRowSlicingCUDA and impl::COORowSlicingCUDA (reference
// src/cuda/slicing.cu:528,768; node-set table NodeQueryHashmap :40-97).  Kept
// ids are relabelled to their position in `ids` (slicing.cu:477-480).
//
// Mark:    id-set table (capacity 2 * pow2 > n, as slicing.cu:468; Fibonacci
//          hashing instead of Hash64Shift) with a one-bit-per-hash filter in front of
//          it: most edges of a slice are not kept, and those leave after one read of a
//          bit array that stays in the caches instead of a chain of 8-byte slots.
//          What the pass leaves behind per edge is ONE BIT (kept or not) in 64-edge
//          words, the number of kept edges of the tile before each word, the count of
//          each 2048-edge tile, and the new ids of the kept edges packed to the front
//          of the tile's range of a scratch array.  An exclusive scan of the tile
//          counts (one entry per 2048 edges) gives every tile its place in the result.
//          For the CSC flavour the new offsets are kept_before(indptr[c]): no
//          per-column count pass, no warp reduction (slicing.cu:463-466), no
//          torch::nonzero.
// Compact: tiles without kept edges leave at once; the others copy their packed ids
//          and write edge positions (and owning columns, found like in the CSC -> COO
//          expansion) at tile base + rank from the bit words.
// The induced-subgraph slice and the batched membership filter below mark and compact the
// same way.
// When `ids` holds duplicates the reference keeps whichever store lands last
// (slicing.cu:56); here the largest position wins (atomicMax), deterministically.
#include "gs_common.hpp"

GS_STAMPS_DEFINE(rowslice)

namespace gs {
namespace {

constexpr int kThreads = 256;
constexpr int kItems = 8;
constexpr int kTile = kThreads * kItems;
constexpr int kStage = 1024;

struct IdSet {
  // slot p: key (-1 empty) at slots[2 p], value at slots[2 p + 1] -- one 16-byte read for a
  // lookup that finds its key in its home slot
  long long* slots;
  uint32_t mask;
  int shift;
  // bit (hash of key) is set for every key of the set: a clear bit proves absence
  uint32_t* filter;
  int filter_shift;
  // The filter folded down to at most kLdsFilterWords words (bit b of the filter is bit
  // b mod its size of this one): what a workgroup keeps in LDS.  The filter itself when that
  // is no larger.
  uint32_t* coarse;
  uint32_t coarse_mask;  // its number of bits - 1
  __device__ __forceinline__ uint32_t home(long long key) const {
    return static_cast<uint32_t>((static_cast<uint64_t>(key) * 0x9E3779B97F4A7C15ull) >> shift);
  }
  __device__ __forceinline__ uint32_t filter_bit(long long key) const {
    return static_cast<uint32_t>((static_cast<uint64_t>(key) * 0xD6E8FEB86659FD93ull) >>
                                 filter_shift);
  }
  __device__ __forceinline__ bool maybe(long long key) const {
    const uint32_t b = filter_bit(key);
    return (filter[b >> 5] >> (b & 31)) & 1u;
  }
  __device__ __forceinline__ void admit(long long key) const {
    const uint32_t b = filter_bit(key);
    atomicOr(&filter[b >> 5], 1u << (b & 31));
    if (coarse != filter) atomicOr(&coarse[(b & coarse_mask) >> 5], 1u << (b & 31));
  }
  // the same test against a copy of `coarse` in LDS
  __device__ __forceinline__ bool maybe_lds(const uint32_t* lds, long long key) const {
    const uint32_t b = filter_bit(key) & coarse_mask;
    return (lds[b >> 5] >> (b & 31)) & 1u;
  }
  __device__ __forceinline__ longlong2 slot(uint32_t p) const {
    return reinterpret_cast<const longlong2*>(slots)[p];
  }
  // value of `key` (-1: absent) given what its home slot holds; walks on in the rare case
  // that the slot belongs to another key
  __device__ __forceinline__ int64_t resolve(long long key, longlong2 kv) const {
    uint32_t p = home(key);
    while (kv.x != key && kv.x != -1) {
      p = (p + 1) & mask;
      kv = slot(p);
    }
    return kv.x == key ? kv.y : -1;
  }
  __device__ __forceinline__ int64_t query(long long key) const {
    return resolve(key, slot(home(key)));
  }
  // N lookups of a thread: the home slots of all of them are read together (a lookup written
  // as one loop after the other makes N round trips, since a wave nearly always has some lane
  // with a key to look up in each)
  template <int N>
  __device__ __forceinline__ void query_all(const long long (&key)[N], const bool (&want)[N],
                                            int64_t (&val)[N]) const {
    longlong2 kv[N];
#pragma unroll
    for (int k = 0; k < N; ++k)
      if (want[k]) kv[k] = slot(home(key[k]));
#pragma unroll
    for (int k = 0; k < N; ++k) val[k] = want[k] ? resolve(key[k], kv[k]) : -1;
  }
};

int64_t set_capacity(int64_t n) {
  int64_t cap = 1024;
  while (cap < 2 * n + 2) cap <<= 1;
  return cap;
}

// bits of the filter: 32 per id (3 % of the absent keys pass), between 1 KB and 1 MB
int64_t filter_bits(int64_t n) {
  int64_t bits = 8192;
  while (bits < 32 * n && bits < (int64_t(1) << 23)) bits <<= 1;
  return bits;
}

// A workgroup's copy of the folded filter: 128 KB of the 160 KB of LDS a compute unit has, so
// that one workgroup of 1024 lanes is resident per unit.  It pays where most keys are in no
// set: the index search (14 M keys against 256 k ids: 184 -> 98 us together with reading the
// home slots of a thread's eight keys at once), less so the mark pass of a row slice (whole
// graph, 200 k row ids: 0.84 -> 0.77 ms), and not the batched filter (0.10 -> 0.14 ms), which
// keeps the one-tile workgroups.
constexpr int kLdsFilterWords = 32768;
constexpr int kBigThreads = 1024;
#ifdef GS_PHASE_STAMPS
constexpr int64_t kLdsSearchMinKeys = int64_t(1) << 62;  // the marked kernels are the one-tile ones
#else
constexpr int64_t kLdsSearchMinKeys = int64_t(1) << 20;  // below: not worth 128 KB per workgroup
#endif

// clears the table and the filters; the grid covers the longer of them
__global__ void __launch_bounds__(kThreads)
set_init_kernel(IdSet t, int64_t cap, int64_t filter_words) {
  const int64_t i = static_cast<int64_t>(blockIdx.x) * kThreads + threadIdx.x;
  if (i < cap) {
    reinterpret_cast<longlong2*>(t.slots)[i] = make_longlong2(-1, -1);
  }
  if (i < filter_words) t.filter[i] = 0;
  if (t.coarse != t.filter && i < kLdsFilterWords) t.coarse[i] = 0;
}

// every thread of a workgroup of kBigThreads: the folded filter into LDS
__device__ __forceinline__ void load_filter(const IdSet& t, uint32_t* lds) {
  const int words = static_cast<int>((t.coarse_mask + 1u) >> 5);
  const uint4* src = reinterpret_cast<const uint4*>(t.coarse);
  for (int i = threadIdx.x; i < words / 4; i += kBigThreads)
    reinterpret_cast<uint4*>(lds)[i] = src[i];
  __syncthreads();
}

template <typename IdT>
__global__ void __launch_bounds__(kThreads)
set_insert_kernel(IdSet t, const IdT* __restrict__ ids, int64_t n) {
  const int64_t i = static_cast<int64_t>(blockIdx.x) * kThreads + threadIdx.x;
  if (i >= n) return;
  const long long key = static_cast<long long>(ids[i]);
  uint32_t p = t.home(key);
  while (true) {
    const unsigned long long prev =
        atomicCAS(reinterpret_cast<unsigned long long*>(&t.slots[2 * p]), ~0ull,
                  static_cast<unsigned long long>(key));
    if (prev == ~0ull || prev == static_cast<unsigned long long>(key)) break;
    p = (p + 1) & t.mask;
  }
  atomicMax(&t.slots[2 * p + 1], static_cast<long long>(i));
  t.admit(key);
}

template <typename P>
__device__ __forceinline__ int64_t upper_bound(P a, int64_t n, int64_t v) {
  int64_t lo = 0, hi = n;
  while (lo < hi) {
    int64_t mid = (lo + hi) >> 1;
    if (a[mid] <= v) lo = mid + 1; else hi = mid;
  }
  return lo;
}

// ------------------------------------------------------------ survivor marks ----
constexpr int kWords = kTile / kWave;  // 64-edge words of a tile

// What the mark pass leaves for the compaction: one bit per edge, the kept edges of the
// tile before each word, and (after the scan) the kept edges before each tile.
struct Marks {
  unsigned long long* mask;  // [n / 64 + 1]
  int32_t* word_rank;        // [n / 64 + 1]
  int64_t* tile_counts;      // [tiles]
  int64_t* tile_base;        // [tiles + 1], exclusive scan of tile_counts
  int64_t n;
  int64_t tiles;
  // kept edges among the first i, 0 <= i <= n
  __device__ __forceinline__ int64_t kept_before(int64_t i) const {
    if (i >= n) return tile_base[tiles];
    const int64_t w = i >> 6;
    const unsigned long long below = mask[w] & ((1ull << (i & 63)) - 1ull);
    return tile_base[i / kTile] + word_rank[w] + __popcll(below);
  }
};

struct LoadCounts {
  const int64_t* p;
  __device__ __forceinline__ int64_t operator()(int64_t i) const { return p[i]; }
};

// key of edge e for the id set; false: the edge cannot be kept
template <typename IdT>
struct PlainKey {
  const IdT* key;
  __device__ __forceinline__ int64_t tile_hint(int64_t, int64_t) const { return 0; }
  __device__ __forceinline__ bool operator()(int64_t e, int64_t, long long* out) const {
    *out = static_cast<long long>(key[e]);
    return true;
  }
};

constexpr int kBatchShift = 44;

// edge e belongs to the batch whose range of key_ptr holds it; set keys are id + (batch << 44)
template <typename IdT>
struct BatchedKey {
  const IdT* key;
  const int64_t* key_ptr;
  int64_t B;
  // the batch of the tile's first edge (-1: before the first batch), searched once per tile;
  // an edge of the tile then steps on from there, which is seldom a step at all
  __device__ __forceinline__ int64_t tile_hint(int64_t p0, int64_t E) const {
    if (p0 >= E) return B;
    int64_t lo = 0, hi = B + 1;  // first b with key_ptr[b] > p0
    while (lo < hi) {
      const int64_t mid = (lo + hi) >> 1;
      if (key_ptr[mid] <= p0) lo = mid + 1; else hi = mid;
    }
    return lo - 1;
  }
  __device__ __forceinline__ bool operator()(int64_t e, int64_t hint, long long* out) const {
    int64_t b = hint;
    while (b < B && key_ptr[b + 1] <= e) ++b;
    if (b < 0 || b >= B) return false;
    *out = static_cast<long long>(key[e]) + (static_cast<long long>(b) << kBatchShift);
    return true;
  }
};

// Tail of a mark pass.  The workgroup owns the 2048 positions from p0, position
// p0 + k * 256 + thread in round k, so that a wave's ballot in round k is the word of 64
// consecutive positions (word k * 4 + wave of the tile).  vals[k] >= 0: kept, and the
// value to pack to the front of the tile's range (with src[k] beside it when WITH_SRC).
// Every thread of the workgroup calls this; `tid` is the thread's number among the 256 that
// own tile `tile`.
template <typename IdT, bool WITH_VALUES, bool WITH_SRC>
__device__ __forceinline__ void publish_marks(const int64_t (&vals)[kItems],
                                              const int64_t (&src)[kItems], int64_t p0, int64_t n,
                                              const Marks& m, IdT* __restrict__ packed,
                                              int64_t* __restrict__ packed_src, int* s_pop,
                                              int* s_rank, int tid, int64_t tile) {
  const int lane = tid & (kWave - 1);
  const int wave = tid / kWave;
  unsigned long long bal[kItems];
#pragma unroll
  for (int k = 0; k < kItems; ++k) {
    bal[k] = __ballot(vals[k] >= 0);
    const int w = k * (kThreads / kWave) + wave;
    if (lane == 0) {
      s_pop[w] = __popcll(bal[k]);
      if (p0 + static_cast<int64_t>(w) * kWave < n) m.mask[(p0 >> 6) + w] = bal[k];
    }
  }
  __syncthreads();
  if (tid < kWave) {
    const int v = tid < kWords ? s_pop[tid] : 0;
    int incl = v;
#pragma unroll
    for (int d = 1; d < kWords; d <<= 1) {
      const int o = __shfl_up(incl, d, kWave);
      if (lane >= d) incl += o;
    }
    if (tid < kWords) {
      s_rank[tid] = incl - v;
      if (p0 + static_cast<int64_t>(tid) * kWave < n) m.word_rank[(p0 >> 6) + tid] = incl - v;
    }
    if (tid == kWords - 1 && tile < m.tiles) m.tile_counts[tile] = incl;
  }
  if (WITH_VALUES || WITH_SRC) {
    __syncthreads();
    const unsigned long long lower = (1ull << lane) - 1ull;
#pragma unroll
    for (int k = 0; k < kItems; ++k)
      if (vals[k] >= 0) {
        const int64_t at =
            p0 + s_rank[k * (kThreads / kWave) + wave] + __popcll(bal[k] & lower);
        if (WITH_VALUES) packed[at] = static_cast<IdT>(vals[k]);
        if (WITH_SRC) packed_src[at] = src[k];
      }
  }
}

// One tile of 2048 edges per workgroup.  The eight keys of a thread, their filter bits and
// their table probes are issued as three batches of independent loads.
template <typename IdT, typename KeyOf, bool WITH_VALUES>
__global__ void __launch_bounds__(kThreads)
mark_tiles_kernel(IdSet t, KeyOf key_of, int64_t E, Marks m, IdT* __restrict__ packed) {
  __shared__ int s_pop[kWords];
  __shared__ int s_rank[kWords];
  GS_STAMP_BEGIN();
  GS_STAMP(0);
  const int64_t p0 = static_cast<int64_t>(blockIdx.x) * kTile;
  const int64_t hint = key_of.tile_hint(p0, E);
  long long keys[kItems];
  bool pass[kItems];
#pragma unroll
  for (int k = 0; k < kItems; ++k) {
    const int64_t e = p0 + k * kThreads + threadIdx.x;
    keys[k] = -1;
    pass[k] = e < E && key_of(e, hint, &keys[k]);
  }
  GS_STAMP(1);  // keys are here
#pragma unroll
  for (int k = 0; k < kItems; ++k)
    if (pass[k]) pass[k] = t.maybe(keys[k]);
  GS_STAMP(2);  // filter bits are here
  int64_t vals[kItems];
  t.query_all<kItems>(keys, pass, vals);
  GS_STAMP(3);  // table lookups done
  publish_marks<IdT, WITH_VALUES, false>(vals, vals, p0, E, m, packed, nullptr, s_pop, s_rank,
                                         threadIdx.x, blockIdx.x);
  GS_STAMP(4);  // marks, ranks and packed ids stored
  GS_STAMP_END(9, 5);
}

// The same for many edges: workgroups of 1024 lanes that stay (four tiles at a time, then the
// next four, ...) and test the keys against the folded filter in LDS first.
template <typename IdT, typename KeyOf, bool WITH_VALUES>
__global__ void __launch_bounds__(kBigThreads)
mark_tiles_lds_kernel(IdSet t, KeyOf key_of, int64_t E, Marks m, IdT* __restrict__ packed) {
  constexpr int kSub = kBigThreads / kThreads;
  __shared__ uint32_t s_filter[kLdsFilterWords];
  __shared__ int s_pop[kSub][kWords];
  __shared__ int s_rank[kSub][kWords];
  load_filter(t, s_filter);
  const int sub = threadIdx.x / kThreads;
  const int tid = threadIdx.x % kThreads;
  const bool two_levels = t.coarse != t.filter;
  for (int64_t tile0 = static_cast<int64_t>(blockIdx.x) * kSub; tile0 < m.tiles;
       tile0 += static_cast<int64_t>(gridDim.x) * kSub) {
    const int64_t tile = tile0 + sub;
    const int64_t p0 = tile * kTile;
    const int64_t hint = key_of.tile_hint(p0, E);
    long long keys[kItems];
    bool pass[kItems];
#pragma unroll
    for (int k = 0; k < kItems; ++k) {
      const int64_t e = p0 + k * kThreads + tid;
      keys[k] = -1;
      pass[k] = e < E && key_of(e, hint, &keys[k]);
    }
#pragma unroll
    for (int k = 0; k < kItems; ++k)
      if (pass[k]) pass[k] = t.maybe_lds(s_filter, keys[k]);
    if (two_levels) {
#pragma unroll
      for (int k = 0; k < kItems; ++k)
        if (pass[k]) pass[k] = t.maybe(keys[k]);
    }
    int64_t vals[kItems];
    t.query_all<kItems>(keys, pass, vals);
    publish_marks<IdT, WITH_VALUES, false>(vals, vals, p0, E, m, packed, nullptr, s_pop[sub],
                                           s_rank[sub], tid, tile);
    __syncthreads();  // s_pop and s_rank are written again in the next round
  }
}

__global__ void __launch_bounds__(kThreads)
new_indptr_kernel(const int64_t* __restrict__ indptr, int64_t num_cols, Marks m,
                  int64_t* __restrict__ out_indptr) {
  const int64_t c = static_cast<int64_t>(blockIdx.x) * kThreads + threadIdx.x;
  if (c <= num_cols) out_indptr[c] = m.kept_before(indptr[c]);
}

__global__ void __launch_bounds__(kWave) copy_total_kernel(Marks m, int64_t* __restrict__ total) {
  if (threadIdx.x == 0 && blockIdx.x == 0) *total = m.tile_base[m.tiles];
}

// CSC compaction; a workgroup owns the 2048 input edges its mark workgroup owned.
template <bool WITH_COO, typename IdT>
__global__ void __launch_bounds__(kThreads)
csc_compact_kernel(const int64_t* __restrict__ indptr, int64_t num_cols, int64_t nnz, Marks m,
                   const IdT* __restrict__ packed, IdT* __restrict__ out_indices,
                   int64_t* __restrict__ select_index, IdT* __restrict__ coo_col) {
  __shared__ int64_t s_ptr[kStage + 1];
  __shared__ int64_t s_rows[2];
  const int64_t base = m.tile_base[blockIdx.x];
  const int64_t count = m.tile_base[blockIdx.x + 1] - base;
  if (count == 0) return;
  const int lane = threadIdx.x & (kWave - 1);
  const int wave = threadIdx.x / kWave;
  const int64_t p0 = static_cast<int64_t>(blockIdx.x) * kTile;
  const int64_t p1 = p0 + kTile < nnz ? p0 + kTile : nnz;
  // the tile's marks, ranks and packed ids are asked for before the search for its columns
  // (four dependent reads and a barrier), not behind it
  unsigned long long bits[kItems];
  int rank[kItems];
  IdT mine[kItems];
#pragma unroll
  for (int k = 0; k < kItems; ++k) {
    const int w = k * (kThreads / kWave) + wave;
    const bool in = p0 + static_cast<int64_t>(w) * kWave < p1;
    bits[k] = in ? m.mask[(p0 >> 6) + w] : 0ull;
    rank[k] = in ? m.word_rank[(p0 >> 6) + w] : 0;
    const int64_t r = threadIdx.x + static_cast<int64_t>(k) * kThreads;
    mine[k] = r < count ? packed[p0 + r] : IdT(0);
  }
  int64_t row_lo = 0, nrows = 0;
  bool staged = false;
  if (WITH_COO) {
    block_row_range(indptr, num_cols, p0, p1 - 1, s_rows);
    row_lo = s_rows[0];
    nrows = s_rows[1] - row_lo + 1;
    staged = nrows <= kStage;
    if (staged)
      for (int64_t i = threadIdx.x; i <= nrows; i += kThreads) s_ptr[i] = indptr[row_lo + i];
    __syncthreads();
  }
#pragma unroll
  for (int k = 0; k < kItems; ++k) {
    const int64_t r = threadIdx.x + static_cast<int64_t>(k) * kThreads;
    if (r < count) out_indices[base + r] = mine[k];
  }
  const unsigned long long lower = (1ull << lane) - 1ull;
#pragma unroll
  for (int k = 0; k < kItems; ++k) {
    const int w = k * (kThreads / kWave) + wave;
    const int64_t e = p0 + static_cast<int64_t>(w) * kWave + lane;
    if (!((bits[k] >> lane) & 1ull)) continue;
    const int64_t pos = base + rank[k] + __popcll(bits[k] & lower);
    select_index[pos] = e;
    if (WITH_COO)
      coo_col[pos] = static_cast<IdT>(row_lo + (staged ? upper_bound(s_ptr, nrows + 1, e)
                                                       : upper_bound(indptr + row_lo, nrows + 1, e)) - 1);
  }
}

// COO compaction and the membership filter's: KEY_OUT writes the packed new ids of the
// key side (row slice); otherwise both endpoints are copied as they are (filter).
template <bool KEY_OUT, typename IdT>
__global__ void __launch_bounds__(kThreads)
coo_compact_kernel(const IdT* __restrict__ key, const IdT* __restrict__ other, int64_t E, Marks m,
                   const IdT* __restrict__ packed, IdT* __restrict__ out_key,
                   IdT* __restrict__ out_other, int64_t* __restrict__ select_index) {
  const int64_t base = m.tile_base[blockIdx.x];
  const int64_t count = m.tile_base[blockIdx.x + 1] - base;
  if (count == 0 || !out_key || !out_other) return;
  const int lane = threadIdx.x & (kWave - 1);
  const int wave = threadIdx.x / kWave;
  const int64_t p0 = static_cast<int64_t>(blockIdx.x) * kTile;
  if (KEY_OUT)
    for (int64_t r = threadIdx.x; r < count; r += kThreads) out_key[base + r] = packed[p0 + r];
  const unsigned long long lower = (1ull << lane) - 1ull;
#pragma unroll
  for (int k = 0; k < kItems; ++k) {
    const int w = k * (kThreads / kWave) + wave;
    const int64_t e = p0 + static_cast<int64_t>(w) * kWave + lane;
    if (e - lane >= E) break;
    const unsigned long long bits = m.mask[(p0 >> 6) + w];
    if (!((bits >> lane) & 1ull)) continue;
    const int64_t pos = base + m.word_rank[(p0 >> 6) + w] + __popcll(bits & lower);
    if (!KEY_OUT) out_key[pos] = key[e];
    out_other[pos] = other[e];
    if (select_index) select_index[pos] = e;
  }
}

// ------------------------------------------- column slice + row slice in one go ----
// Induced-subgraph slicing: of the columns `cols`, keep the edges whose row is in the id
// set (reference src/cuda/fusion/column_row_slicing.cu:102-211; batched :225-355).  The
// column slice is never materialised: position p of the virtual sliced edge array is
// resolved to its column by binary search in the slice offsets (staged in LDS when the
// workgroup's 2048 positions span few columns) and to its position in the parent's
// indices from there; that parent position is kept for the compaction.
//
// Batched flavour (B > 0): columns and ids are cut into B batches at col_ptr / id_ptr; a
// column of batch b keeps the rows found in batch b's ids.  The table key is
// id + b * encoding_size and the value the id itself (rows keep their global id,
// column_row_slicing.cu:272), exactly as the reference composes it.
template <typename IdT>
__global__ void __launch_bounds__(kThreads)
set_insert_batched_kernel(IdSet t, const IdT* __restrict__ ids, int64_t n,
                          const int64_t* __restrict__ id_ptr, int64_t B, int64_t enc) {
  // the batch offsets in LDS when they fit: the search for an id's batch is seven dependent
  // reads, from memory seven trips before the first probe of the table (256 k ids in 64
  // batches: 62 us with the offsets read from memory)
  constexpr int kStagedOffsets = 1024;
  __shared__ int64_t s_ptr[kStagedOffsets];
  const bool staged = B + 1 <= kStagedOffsets;
  if (staged) {
    for (int j = threadIdx.x; j <= B; j += kThreads) s_ptr[j] = id_ptr[j];
    __syncthreads();
  }
  const int64_t i = static_cast<int64_t>(blockIdx.x) * kThreads + threadIdx.x;
  if (i >= n) return;
  const long long id = static_cast<long long>(ids[i]);
  const int64_t b = (staged ? upper_bound(s_ptr, B + 1, i) : upper_bound(id_ptr, B + 1, i)) - 1;
  if (b < 0 || b >= B) return;
  const long long key = id + b * enc;
  if (key == -1) return;
  uint32_t p = t.home(key);
  while (true) {
    const unsigned long long prev =
        atomicCAS(reinterpret_cast<unsigned long long*>(&t.slots[2 * p]), ~0ull,
                  static_cast<unsigned long long>(key));
    if (prev == ~0ull || prev == static_cast<unsigned long long>(key)) break;
    p = (p + 1) & t.mask;
  }
  atomicMax(&t.slots[2 * p + 1], id);
  t.admit(key);
}

template <typename IdT>
__global__ void __launch_bounds__(kThreads)
sliced_mark_kernel(IdSet t, const int64_t* __restrict__ indptr, const IdT* __restrict__ indices,
                   const IdT* __restrict__ cols, int64_t S, const int64_t* __restrict__ sub_indptr,
                   int64_t D, const int64_t* __restrict__ col_ptr, int64_t B, int64_t enc, Marks m,
                   IdT* __restrict__ packed, int64_t* __restrict__ packed_src) {
  __shared__ int64_t s_ptr[kStage + 1];
  __shared__ int64_t s_rows[2];
  __shared__ int s_pop[kWords];
  __shared__ int s_rank[kWords];
  const int64_t p0 = static_cast<int64_t>(blockIdx.x) * kTile;
  const int64_t p1 = p0 + kTile < D ? p0 + kTile : D;
  block_row_range(sub_indptr, S, p0, p1 - 1, s_rows);
  const int64_t row_lo = s_rows[0];
  const int64_t nrows = s_rows[1] - row_lo + 1;
  const bool staged = nrows <= kStage;
  if (staged)
    for (int64_t i = threadIdx.x; i <= nrows; i += kThreads) s_ptr[i] = sub_indptr[row_lo + i];
  __syncthreads();
  // The eight positions of a thread go through the same chain of reads (row of the position,
  // the row's column, the column's start, the edge's id): every link for all eight before the
  // next, so that eight reads are in flight at a time instead of one.
  long long keys[kItems], ids[kItems];
  int64_t src[kItems], row[kItems], off[kItems];
  bool pass[kItems];
#pragma unroll
  for (int k = 0; k < kItems; ++k) {
    const int64_t p = p0 + k * kThreads + threadIdx.x;
    keys[k] = ids[k] = -1;
    src[k] = row[k] = off[k] = 0;
    pass[k] = p < p1;
    if (!pass[k]) continue;
    const int64_t lr = (staged ? upper_bound(s_ptr, nrows + 1, p)
                               : upper_bound(sub_indptr + row_lo, nrows + 1, p)) - 1;
    row[k] = row_lo + lr;
    off[k] = p - (staged ? s_ptr[lr] : sub_indptr[row[k]]);
  }
  // a column that owns a position of the slice has passed the range check of the count
  int64_t col[kItems];
#pragma unroll
  for (int k = 0; k < kItems; ++k) col[k] = pass[k] ? static_cast<int64_t>(cols[row[k]]) : 0;
#pragma unroll
  for (int k = 0; k < kItems; ++k)
    if (pass[k]) src[k] = indptr[col[k]] + off[k];
#pragma unroll
  for (int k = 0; k < kItems; ++k)
    if (pass[k]) ids[k] = static_cast<long long>(indices[src[k]]);
#pragma unroll
  for (int k = 0; k < kItems; ++k) {
    if (!pass[k]) continue;
    if (B > 0) {
      const int64_t b = upper_bound(col_ptr, B + 1, row[k]) - 1;
      pass[k] = b >= 0 && b < B;
      keys[k] = ids[k] + b * enc;
    } else {
      keys[k] = ids[k];
    }
  }
#pragma unroll
  for (int k = 0; k < kItems; ++k)
    if (pass[k]) pass[k] = t.maybe(keys[k]);
  int64_t vals[kItems];
  t.query_all<kItems>(keys, pass, vals);
  if (B > 0) {
#pragma unroll
    for (int k = 0; k < kItems; ++k)
      if (vals[k] >= 0) vals[k] = ids[k];  // batched: rows keep their id
  }
  publish_marks<IdT, true, true>(vals, src, p0, D, m, packed, packed_src, s_pop, s_rank, threadIdx.x,
                                 blockIdx.x);
}

__global__ void __launch_bounds__(kThreads)
sliced_indptr_kernel(const int64_t* __restrict__ sub_indptr, int64_t S, Marks m,
                     int64_t* __restrict__ out_indptr) {
  const int64_t r = static_cast<int64_t>(blockIdx.x) * kThreads + threadIdx.x;
  if (r <= S) out_indptr[r] = m.kept_before(sub_indptr[r]);
}

template <typename IdT>
__global__ void __launch_bounds__(kThreads)
sliced_compact_kernel(int64_t D, Marks m, const IdT* __restrict__ packed,
                      const int64_t* __restrict__ packed_src, IdT* __restrict__ out_indices,
                      int64_t* __restrict__ select_index, int64_t* __restrict__ parent_index) {
  const int64_t base = m.tile_base[blockIdx.x];
  const int64_t count = m.tile_base[blockIdx.x + 1] - base;
  if (count == 0) return;
  const int lane = threadIdx.x & (kWave - 1);
  const int wave = threadIdx.x / kWave;
  const int64_t p0 = static_cast<int64_t>(blockIdx.x) * kTile;
  for (int64_t r = threadIdx.x; r < count; r += kThreads) {
    out_indices[base + r] = packed[p0 + r];
    if (parent_index) parent_index[base + r] = packed_src[p0 + r];
  }
  if (!select_index) return;
  const unsigned long long lower = (1ull << lane) - 1ull;
#pragma unroll
  for (int k = 0; k < kItems; ++k) {
    const int w = k * (kThreads / kWave) + wave;
    const int64_t p = p0 + static_cast<int64_t>(w) * kWave + lane;
    if (p - lane >= D) break;
    const unsigned long long bits = m.mask[(p0 >> 6) + w];
    if ((bits >> lane) & 1ull)
      select_index[base + m.word_rank[(p0 >> 6) + w] + __popcll(bits & lower)] = p;
  }
}

// ------------------------------------------------- batched membership filter ----
// Edge e belongs to the batch whose range of key_ptr holds e; it survives when key[e] is
// among the ids of the same batch.  Replaces the per-batch tables of
// impl::BatchCOOSlicingCUDA / BatchCOORowSlicingCUDA (reference src/cuda/batch_slicing.cu:
// 150-232, src/cuda/slicing.cu:659-770) by one table keyed with id + (batch << 44)
// (BatchedKey above); mark and compaction are the row slice's.
__global__ void __launch_bounds__(kThreads)
filter_batch_ptr_kernel(const int64_t* __restrict__ key_ptr, int64_t B, Marks m,
                        int64_t* __restrict__ out_ptr) {
  const int64_t b = static_cast<int64_t>(blockIdx.x) * kThreads + threadIdx.x;
  if (b <= B) out_ptr[b] = m.kept_before(key_ptr[b]);
}

// position of each key in `data` (-1 when absent): impl::IndexHashMapInsertCUDA +
// IndexHashMapSearchCUDA (reference src/cuda/index_search.cu:83-140)
template <typename IdT>
__global__ void __launch_bounds__(kThreads)
search_kernel(IdSet t, const IdT* __restrict__ keys, int64_t m, IdT* __restrict__ out) {
  const int64_t i = static_cast<int64_t>(blockIdx.x) * kThreads + threadIdx.x;
  if (i < m) out[i] = static_cast<IdT>(t.query(static_cast<long long>(keys[i])));
}

// The same for many keys: most of them are in no set, and the folded filter in LDS says so
// without a trip to memory.
template <typename IdT>
__global__ void __launch_bounds__(kBigThreads)
search_lds_kernel(IdSet t, const IdT* __restrict__ keys, int64_t m, IdT* __restrict__ out) {
  __shared__ uint32_t s_filter[kLdsFilterWords];
  load_filter(t, s_filter);
  const bool two_levels = t.coarse != t.filter;
  constexpr int kPer = 8;
  for (int64_t base = static_cast<int64_t>(blockIdx.x) * kBigThreads * kPer; base < m;
       base += static_cast<int64_t>(gridDim.x) * kBigThreads * kPer) {
    long long key[kPer];
    bool pass[kPer];
#pragma unroll
    for (int u = 0; u < kPer; ++u) {
      const int64_t i = base + u * kBigThreads + threadIdx.x;
      key[u] = i < m ? static_cast<long long>(keys[i]) : -1;
      pass[u] = i < m && t.maybe_lds(s_filter, key[u]);
    }
    if (two_levels) {
#pragma unroll
      for (int u = 0; u < kPer; ++u)
        if (pass[u]) pass[u] = t.maybe(key[u]);
    }
    int64_t val[kPer];
    t.query_all<kPer>(key, pass, val);
#pragma unroll
    for (int u = 0; u < kPer; ++u) {
      const int64_t i = base + u * kBigThreads + threadIdx.x;
      if (i < m) out[i] = static_cast<IdT>(val[u]);
    }
  }
}

// Workspace layout: [marks | (parent positions) | id-set keys | id-set values | filter].
// The marks (bit words, word ranks, tile counts and bases, scan tiles, packed new ids)
// and the parent positions depend on the edge count only, so the compact call finds them
// again without knowing how many ids the mark call was given.
void carve_set(Carver& ws, int64_t n_ids, IdSet* set, int64_t* cap, int64_t* filter_words) {
  *cap = set_capacity(n_ids);
  set->slots = ws.take<long long>(2 * *cap);
  set->mask = static_cast<uint32_t>(*cap - 1);
  int lg = 0;
  while ((int64_t(1) << lg) < *cap) ++lg;
  set->shift = 64 - lg;
  const int64_t bits = filter_bits(n_ids);
  *filter_words = bits / 32;
  set->filter = ws.take<uint32_t>(*filter_words);
  lg = 0;
  while ((int64_t(1) << lg) < bits) ++lg;
  set->filter_shift = 64 - lg;
  if (*filter_words > kLdsFilterWords) {
    set->coarse = ws.take<uint32_t>(kLdsFilterWords);
    set->coarse_mask = static_cast<uint32_t>(kLdsFilterWords) * 32u - 1u;
  } else {
    set->coarse = set->filter;
    set->coarse_mask = static_cast<uint32_t>(bits - 1);
  }
}

size_t set_bytes(int64_t n_ids) {
  const int64_t words = filter_bits(n_ids) / 32;
  return padded(set_capacity(n_ids) * 16) + padded(words * 4) +
         (words > kLdsFilterWords ? padded(kLdsFilterWords * 4) : 0);
}

struct MarkScratch {
  IdSet set;
  int64_t cap;
  int64_t filter_words;
  Marks m;
  int64_t* scan_tiles;
  void* packed;
  int64_t* packed_src;
  bool ok;
};

// tiles of an array of E positions; none when it is empty
int64_t mark_tiles(int64_t E) { return (E + kTile - 1) / kTile; }

size_t marks_bytes(int64_t E) {
  const int64_t words = E / kWave + 1;
  const int64_t tiles = mark_tiles(E);
  return padded(words * 8) + padded(words * 4) + padded((tiles + 1) * 8) + padded((tiles + 2) * 8) +
         scan_workspace_bytes(tiles) + padded((E > 0 ? E : 1) * 8);
}

MarkScratch carve_marks(void* workspace, size_t bytes, int64_t n_ids, int64_t E, bool with_set,
                        bool with_src = false) {
  MarkScratch s;
  Carver ws(workspace, bytes);
  const int64_t words = E / kWave + 1;
  s.m.n = E;
  s.m.tiles = mark_tiles(E);
  s.m.mask = ws.take<unsigned long long>(words);
  s.m.word_rank = ws.take<int32_t>(words);
  s.m.tile_counts = ws.take<int64_t>(s.m.tiles + 1);
  s.m.tile_base = ws.take<int64_t>(s.m.tiles + 2);
  s.scan_tiles = ws.take<int64_t>(scan_num_tiles(s.m.tiles) + 1);
  s.packed = ws.take<int64_t>(E > 0 ? E : 1);
  s.packed_src = with_src ? ws.take<int64_t>(E > 0 ? E : 1) : nullptr;
  s.cap = 0;
  s.filter_words = 0;
  if (with_set) carve_set(ws, n_ids, &s.set, &s.cap, &s.filter_words);
  s.ok = ws.ok;
  return s;
}

void init_set(const IdSet& set, int64_t cap, int64_t filter_words, hipStream_t st) {
  const int64_t n = cap > filter_words ? cap : filter_words;
  hipLaunchKernelGGL(set_init_kernel, dim3(blocks_for(n, kThreads)), dim3(kThreads), 0, st, set, cap,
                     filter_words);
}

// id set from `ids` (cut into B batches at ids_ptr when B > 0), marks of the E edge keys,
// scan of the tile counts
template <typename IdT>
int mark_common(const char* who, const void* key, int64_t E, const int64_t* key_ptr, const void* ids,
                int64_t n_ids, const int64_t* ids_ptr, int64_t B, bool with_values, MarkScratch& s,
                hipStream_t st) {
  init_set(s.set, s.cap, s.filter_words, st);
  if (n_ids > 0) {
    if (B > 0)
      hipLaunchKernelGGL(set_insert_batched_kernel<IdT>, dim3(blocks_for(n_ids, kThreads)),
                         dim3(kThreads), 0, st, s.set, static_cast<const IdT*>(ids), n_ids, ids_ptr, B,
                         int64_t(1) << kBatchShift);
    else
      hipLaunchKernelGGL(set_insert_kernel<IdT>, dim3(blocks_for(n_ids, kThreads)), dim3(kThreads), 0,
                         st, s.set, static_cast<const IdT*>(ids), n_ids);
  }
  if (E >= kLdsSearchMinKeys && B == 0) {
    // few workgroups that stay, one per compute unit and a second one waiting
    const int64_t groups = (s.m.tiles + kBigThreads / kThreads - 1) / (kBigThreads / kThreads);
    const dim3 grid(static_cast<unsigned>(groups < 512 ? groups : 512));
    IdT* packed = static_cast<IdT*>(s.packed);
    PlainKey<IdT> k{static_cast<const IdT*>(key)};
    if (with_values)
      hipLaunchKernelGGL((mark_tiles_lds_kernel<IdT, PlainKey<IdT>, true>), grid, dim3(kBigThreads),
                         0, st, s.set, k, E, s.m, packed);
    else
      hipLaunchKernelGGL((mark_tiles_lds_kernel<IdT, PlainKey<IdT>, false>), grid, dim3(kBigThreads),
                         0, st, s.set, k, E, s.m, packed);
  } else if (E > 0) {
    const dim3 grid(static_cast<unsigned>(s.m.tiles));
    IdT* packed = static_cast<IdT*>(s.packed);
    if (B > 0) {
      BatchedKey<IdT> k{static_cast<const IdT*>(key), key_ptr, B};
      hipLaunchKernelGGL((mark_tiles_kernel<IdT, BatchedKey<IdT>, false>), grid, dim3(kThreads), 0, st,
                         s.set, k, E, s.m, packed);
    } else {
      PlainKey<IdT> k{static_cast<const IdT*>(key)};
      if (with_values)
        hipLaunchKernelGGL((mark_tiles_kernel<IdT, PlainKey<IdT>, true>), grid, dim3(kThreads), 0, st,
                           s.set, k, E, s.m, packed);
      else
        hipLaunchKernelGGL((mark_tiles_kernel<IdT, PlainKey<IdT>, false>), grid, dim3(kThreads), 0, st,
                           s.set, k, E, s.m, packed);
    }
  }
  GS_RETURN_IF_ERROR(check_launch(who));
  LoadCounts f{s.m.tile_counts};
  return exclusive_scan(f, s.m.tiles, s.m.tile_base, s.scan_tiles, st);
}

}  // namespace
}  // namespace gs

using namespace gs;

extern "C" {

size_t gs_row_slice_workspace_bytes(int64_t num_row_ids, int64_t nnz, int64_t num_cols) {
  (void)num_cols;
  if (num_row_ids < 0) num_row_ids = 0;
  if (nnz < 0) nnz = 0;
  return set_bytes(num_row_ids) + marks_bytes(nnz);
}

int gs_row_slice_csc_mark(const int64_t* indptr, const void* indices, int id_bytes,
                          int64_t num_cols, int64_t nnz, const void* row_ids, int64_t num_row_ids,
                          int64_t* out_indptr, void* workspace, size_t workspace_bytes,
                          void* stream) {
  GS_REQUIRE(num_cols >= 0 && nnz >= 0 && num_row_ids >= 0, "gs_row_slice_csc_mark: negative size");
  GS_REQUIRE(indptr && out_indptr && (nnz == 0 || indices) && (num_row_ids == 0 || row_ids),
             "gs_row_slice_csc_mark: null pointer");
  GS_REQUIRE(valid_id_bytes(id_bytes), "gs_row_slice_csc_mark: id_bytes must be 4 or 8, got %d",
             id_bytes);
  MarkScratch s = carve_marks(workspace, workspace_bytes, num_row_ids, nnz, true);
  if (!s.ok) {
    set_error_text("gs_row_slice_csc_mark: workspace needs %zu bytes, 256-byte aligned",
                   gs_row_slice_workspace_bytes(num_row_ids, nnz, num_cols));
    return GS_ERR_WORKSPACE;
  }
  hipStream_t st = static_cast<hipStream_t>(stream);
  GS_RETURN_IF_ERROR(id_bytes == 8
                         ? mark_common<int64_t>("row_slice_csc_mark", indices, nnz, nullptr, row_ids,
                                                num_row_ids, nullptr, 0, true, s, st)
                         : mark_common<int32_t>("row_slice_csc_mark", indices, nnz, nullptr, row_ids,
                                                num_row_ids, nullptr, 0, true, s, st));
  hipLaunchKernelGGL(new_indptr_kernel, dim3(blocks_for(num_cols + 1, kThreads)), dim3(kThreads), 0,
                     st, indptr, num_cols, s.m, out_indptr);
  return check_launch("row_slice_csc_mark");
}

int gs_row_slice_csc_compact(const int64_t* indptr, int64_t num_cols, int64_t nnz, int id_bytes,
                             void* out_indices, int64_t* select_index, void* coo_col,
                             void* workspace, size_t workspace_bytes, void* stream) {
  GS_REQUIRE(num_cols >= 0 && nnz >= 0 && indptr, "gs_row_slice_csc_compact: bad argument");
  GS_REQUIRE(valid_id_bytes(id_bytes), "gs_row_slice_csc_compact: id_bytes must be 4 or 8, got %d",
             id_bytes);
  if (nnz == 0) return GS_OK;
  GS_REQUIRE(out_indices && select_index, "gs_row_slice_csc_compact: null output");
  MarkScratch s = carve_marks(workspace, workspace_bytes, 0, nnz, false);
  if (!s.ok) {
    set_error_text("gs_row_slice_csc_compact: pass the workspace given to gs_row_slice_csc_mark");
    return GS_ERR_WORKSPACE;
  }
  hipStream_t st = static_cast<hipStream_t>(stream);
  const dim3 grid(static_cast<unsigned>(s.m.tiles));
  if (id_bytes == 8) {
    int64_t* oi = static_cast<int64_t*>(out_indices);
    int64_t* cc = static_cast<int64_t*>(coo_col);
    const int64_t* pk = static_cast<const int64_t*>(s.packed);
    if (coo_col)
      hipLaunchKernelGGL((csc_compact_kernel<true, int64_t>), grid, dim3(kThreads), 0, st, indptr,
                         num_cols, nnz, s.m, pk, oi, select_index, cc);
    else
      hipLaunchKernelGGL((csc_compact_kernel<false, int64_t>), grid, dim3(kThreads), 0, st, indptr,
                         num_cols, nnz, s.m, pk, oi, select_index, cc);
  } else {
    int32_t* oi = static_cast<int32_t*>(out_indices);
    int32_t* cc = static_cast<int32_t*>(coo_col);
    const int32_t* pk = static_cast<const int32_t*>(s.packed);
    if (coo_col)
      hipLaunchKernelGGL((csc_compact_kernel<true, int32_t>), grid, dim3(kThreads), 0, st, indptr,
                         num_cols, nnz, s.m, pk, oi, select_index, cc);
    else
      hipLaunchKernelGGL((csc_compact_kernel<false, int32_t>), grid, dim3(kThreads), 0, st, indptr,
                         num_cols, nnz, s.m, pk, oi, select_index, cc);
  }
  return check_launch("row_slice_csc_compact");
}

int gs_row_slice_coo_mark(const void* key, int id_bytes, int64_t E, const void* ids,
                          int64_t num_ids, int64_t* num_kept, void* workspace,
                          size_t workspace_bytes, void* stream) {
  GS_REQUIRE(E >= 0 && num_ids >= 0 && num_kept, "gs_row_slice_coo_mark: bad argument");
  GS_REQUIRE((E == 0 || key) && (num_ids == 0 || ids), "gs_row_slice_coo_mark: null pointer");
  GS_REQUIRE(valid_id_bytes(id_bytes), "gs_row_slice_coo_mark: id_bytes must be 4 or 8, got %d",
             id_bytes);
  MarkScratch s = carve_marks(workspace, workspace_bytes, num_ids, E, true);
  if (!s.ok) {
    set_error_text("gs_row_slice_coo_mark: workspace needs %zu bytes, 256-byte aligned",
                   gs_row_slice_workspace_bytes(num_ids, E, 0));
    return GS_ERR_WORKSPACE;
  }
  hipStream_t st = static_cast<hipStream_t>(stream);
  GS_RETURN_IF_ERROR(id_bytes == 8 ? mark_common<int64_t>("row_slice_coo_mark", key, E, nullptr, ids,
                                                          num_ids, nullptr, 0, true, s, st)
                                   : mark_common<int32_t>("row_slice_coo_mark", key, E, nullptr, ids,
                                                          num_ids, nullptr, 0, true, s, st));
  hipLaunchKernelGGL(copy_total_kernel, dim3(1), dim3(kWave), 0, st, s.m, num_kept);
  return check_launch("row_slice_coo_mark");
}

int gs_row_slice_coo_compact(const void* other, int id_bytes, int64_t E, void* out_key,
                             void* out_other, int64_t* select_index, void* workspace,
                             size_t workspace_bytes, void* stream) {
  GS_REQUIRE(E >= 0, "gs_row_slice_coo_compact: negative size");
  GS_REQUIRE(valid_id_bytes(id_bytes), "gs_row_slice_coo_compact: id_bytes must be 4 or 8, got %d",
             id_bytes);
  if (E == 0) return GS_OK;
  GS_REQUIRE(other && out_key && out_other && select_index, "gs_row_slice_coo_compact: null pointer");
  MarkScratch s = carve_marks(workspace, workspace_bytes, 0, E, false);
  if (!s.ok) {
    set_error_text("gs_row_slice_coo_compact: pass the workspace given to gs_row_slice_coo_mark");
    return GS_ERR_WORKSPACE;
  }
  hipStream_t st = static_cast<hipStream_t>(stream);
  const dim3 grid(static_cast<unsigned>(s.m.tiles));
  if (id_bytes == 8)
    hipLaunchKernelGGL((coo_compact_kernel<true, int64_t>), grid, dim3(kThreads), 0, st,
                       static_cast<const int64_t*>(nullptr), static_cast<const int64_t*>(other), E,
                       s.m, static_cast<const int64_t*>(s.packed), static_cast<int64_t*>(out_key),
                       static_cast<int64_t*>(out_other), select_index);
  else
    hipLaunchKernelGGL((coo_compact_kernel<true, int32_t>), grid, dim3(kThreads), 0, st,
                       static_cast<const int32_t*>(nullptr), static_cast<const int32_t*>(other), E,
                       s.m, static_cast<const int32_t*>(s.packed), static_cast<int32_t*>(out_key),
                       static_cast<int32_t*>(out_other), select_index);
  return check_launch("row_slice_coo_compact");
}

size_t gs_col_row_slice_workspace_bytes(int64_t num_row_ids, int64_t D) {
  if (D < 0) D = 0;
  return gs_row_slice_workspace_bytes(num_row_ids, D, 0) + padded((D > 0 ? D : 1) * 8);
}

int gs_col_row_slice_mark(const int64_t* indptr, int64_t num_cols, const void* indices,
                          int id_bytes, const void* column_ids, int64_t S,
                          const int64_t* sub_indptr, int64_t D, const void* row_ids,
                          int64_t num_row_ids, const int64_t* col_batch_ptr,
                          const int64_t* row_batch_ptr, int64_t num_batches,
                          int64_t encoding_size, int64_t* out_indptr, void* workspace,
                          size_t workspace_bytes, void* stream) {
  (void)num_cols;
  GS_REQUIRE(S >= 0 && D >= 0 && num_row_ids >= 0 && num_batches >= 0,
             "gs_col_row_slice_mark: negative size");
  GS_REQUIRE(indptr && sub_indptr && out_indptr && (D == 0 || indices) && (S == 0 || column_ids) &&
                 (num_row_ids == 0 || row_ids),
             "gs_col_row_slice_mark: null pointer");
  GS_REQUIRE(num_batches == 0 || (col_batch_ptr && row_batch_ptr && encoding_size > 0),
             "gs_col_row_slice_mark: a batched call needs both batch offsets and an encoding size");
  GS_REQUIRE(valid_id_bytes(id_bytes), "gs_col_row_slice_mark: id_bytes must be 4 or 8, got %d",
             id_bytes);
  MarkScratch s = carve_marks(workspace, workspace_bytes, num_row_ids, D, true, true);
  if (!s.ok) {
    set_error_text("gs_col_row_slice_mark: workspace needs %zu bytes, 256-byte aligned",
                   gs_col_row_slice_workspace_bytes(num_row_ids, D));
    return GS_ERR_WORKSPACE;
  }
  hipStream_t st = static_cast<hipStream_t>(stream);
  init_set(s.set, s.cap, s.filter_words, st);
  auto run = [&](auto tag) {
    using IdT = decltype(tag);
    const IdT* ids = static_cast<const IdT*>(row_ids);
    if (num_row_ids > 0) {
      if (num_batches > 0)
        hipLaunchKernelGGL(set_insert_batched_kernel<IdT>, dim3(blocks_for(num_row_ids, kThreads)),
                           dim3(kThreads), 0, st, s.set, ids, num_row_ids, row_batch_ptr,
                           num_batches, encoding_size);
      else
        hipLaunchKernelGGL(set_insert_kernel<IdT>, dim3(blocks_for(num_row_ids, kThreads)),
                           dim3(kThreads), 0, st, s.set, ids, num_row_ids);
    }
    if (D > 0)
      hipLaunchKernelGGL(sliced_mark_kernel<IdT>, dim3(static_cast<unsigned>(s.m.tiles)),
                         dim3(kThreads), 0, st, s.set, indptr, static_cast<const IdT*>(indices),
                         static_cast<const IdT*>(column_ids), S, sub_indptr, D, col_batch_ptr,
                         num_batches, encoding_size, s.m, static_cast<IdT*>(s.packed), s.packed_src);
  };
  if (id_bytes == 8) run(int64_t{}); else run(int32_t{});
  GS_RETURN_IF_ERROR(check_launch("col_row_slice_mark"));
  LoadCounts f{s.m.tile_counts};
  GS_RETURN_IF_ERROR(exclusive_scan(f, s.m.tiles, s.m.tile_base, s.scan_tiles, st));
  hipLaunchKernelGGL(sliced_indptr_kernel, dim3(blocks_for(S + 1, kThreads)), dim3(kThreads), 0, st,
                     sub_indptr, S, s.m, out_indptr);
  return check_launch("col_row_slice_mark");
}

int gs_col_row_slice_compact(int64_t D, int id_bytes, void* out_indices, int64_t* select_index,
                             int64_t* parent_index, void* workspace, size_t workspace_bytes,
                             void* stream) {
  GS_REQUIRE(D >= 0, "gs_col_row_slice_compact: negative size");
  GS_REQUIRE(valid_id_bytes(id_bytes), "gs_col_row_slice_compact: id_bytes must be 4 or 8, got %d",
             id_bytes);
  if (D == 0) return GS_OK;
  GS_REQUIRE(out_indices, "gs_col_row_slice_compact: null output");
  MarkScratch s = carve_marks(workspace, workspace_bytes, 0, D, false, true);
  if (!s.ok) {
    set_error_text("gs_col_row_slice_compact: pass the workspace given to gs_col_row_slice_mark");
    return GS_ERR_WORKSPACE;
  }
  hipStream_t st = static_cast<hipStream_t>(stream);
  const dim3 grid(static_cast<unsigned>(s.m.tiles));
  if (id_bytes == 8)
    hipLaunchKernelGGL(sliced_compact_kernel<int64_t>, grid, dim3(kThreads), 0, st, D, s.m,
                       static_cast<const int64_t*>(s.packed), s.packed_src,
                       static_cast<int64_t*>(out_indices), select_index, parent_index);
  else
    hipLaunchKernelGGL(sliced_compact_kernel<int32_t>, grid, dim3(kThreads), 0, st, D, s.m,
                       static_cast<const int32_t*>(s.packed), s.packed_src,
                       static_cast<int32_t*>(out_indices), select_index, parent_index);
  return check_launch("col_row_slice_compact");
}

int gs_coo_filter_mark(const void* key, int id_bytes, int64_t E, const int64_t* key_batch_ptr,
                       const void* ids, int64_t num_ids, const int64_t* ids_batch_ptr,
                       int64_t num_batches, int64_t* num_kept, void* workspace,
                       size_t workspace_bytes, void* stream) {
  GS_REQUIRE(E >= 0 && num_ids >= 0 && num_batches >= 0 && num_kept,
             "gs_coo_filter_mark: bad argument");
  GS_REQUIRE((E == 0 || key) && (num_ids == 0 || ids), "gs_coo_filter_mark: null pointer");
  GS_REQUIRE(num_batches == 0 || (key_batch_ptr && ids_batch_ptr),
             "gs_coo_filter_mark: a batched call needs both batch offsets");
  GS_REQUIRE(num_batches < (int64_t(1) << (62 - kBatchShift)),
             "gs_coo_filter_mark: too many batches");
  GS_REQUIRE(valid_id_bytes(id_bytes), "gs_coo_filter_mark: id_bytes must be 4 or 8, got %d",
             id_bytes);
  MarkScratch s = carve_marks(workspace, workspace_bytes, num_ids, E, true);
  if (!s.ok) {
    set_error_text("gs_coo_filter_mark: workspace needs %zu bytes, 256-byte aligned",
                   gs_row_slice_workspace_bytes(num_ids, E, 0));
    return GS_ERR_WORKSPACE;
  }
  hipStream_t st = static_cast<hipStream_t>(stream);
  GS_RETURN_IF_ERROR(id_bytes == 8
                         ? mark_common<int64_t>("coo_filter_mark", key, E, key_batch_ptr, ids, num_ids,
                                                ids_batch_ptr, num_batches, false, s, st)
                         : mark_common<int32_t>("coo_filter_mark", key, E, key_batch_ptr, ids, num_ids,
                                                ids_batch_ptr, num_batches, false, s, st));
  hipLaunchKernelGGL(copy_total_kernel, dim3(1), dim3(kWave), 0, st, s.m, num_kept);
  return check_launch("coo_filter_mark");
}

int gs_coo_filter_compact(const void* row, const void* col, int id_bytes, int64_t E,
                          const int64_t* key_batch_ptr, int64_t num_batches, void* out_row,
                          void* out_col, int64_t* select_index, int64_t* out_batch_ptr,
                          void* workspace, size_t workspace_bytes, void* stream) {
  GS_REQUIRE(E >= 0 && num_batches >= 0, "gs_coo_filter_compact: negative size");
  GS_REQUIRE(valid_id_bytes(id_bytes), "gs_coo_filter_compact: id_bytes must be 4 or 8, got %d",
             id_bytes);
  GS_REQUIRE(!out_batch_ptr || (num_batches > 0 && key_batch_ptr),
             "gs_coo_filter_compact: batch offsets of the result need those of the input");
  MarkScratch s = carve_marks(workspace, workspace_bytes, 0, E, false);
  if (!s.ok) {
    set_error_text("gs_coo_filter_compact: pass the workspace given to gs_coo_filter_mark");
    return GS_ERR_WORKSPACE;
  }
  hipStream_t st = static_cast<hipStream_t>(stream);
  if (out_batch_ptr)
    hipLaunchKernelGGL(filter_batch_ptr_kernel, dim3(blocks_for(num_batches + 1, kThreads)),
                       dim3(kThreads), 0, st, key_batch_ptr, num_batches, s.m, out_batch_ptr);
  if (E > 0) {
    GS_REQUIRE(row && col, "gs_coo_filter_compact: null pointer");
    // no edge kept: the outputs are empty arrays and may be null (the kernel writes nothing)
    const dim3 grid(static_cast<unsigned>(s.m.tiles));
    if (id_bytes == 8)
      hipLaunchKernelGGL((coo_compact_kernel<false, int64_t>), grid, dim3(kThreads), 0, st,
                         static_cast<const int64_t*>(row), static_cast<const int64_t*>(col), E, s.m,
                         static_cast<const int64_t*>(nullptr), static_cast<int64_t*>(out_row),
                         static_cast<int64_t*>(out_col), select_index);
    else
      hipLaunchKernelGGL((coo_compact_kernel<false, int32_t>), grid, dim3(kThreads), 0, st,
                         static_cast<const int32_t*>(row), static_cast<const int32_t*>(col), E, s.m,
                         static_cast<const int32_t*>(nullptr), static_cast<int32_t*>(out_row),
                         static_cast<int32_t*>(out_col), select_index);
  }
  return check_launch("coo_filter_compact");
}

size_t gs_index_search_workspace_bytes(int64_t n) { return gs_row_slice_workspace_bytes(n, 0, 0); }

int gs_index_search(const void* data, int64_t n, const void* keys, int64_t m, int id_bytes,
                    void* out, void* workspace, size_t workspace_bytes, void* stream) {
  GS_REQUIRE(n >= 0 && m >= 0, "gs_index_search: negative size");
  GS_REQUIRE(valid_id_bytes(id_bytes), "gs_index_search: id_bytes must be 4 or 8, got %d", id_bytes);
  GS_REQUIRE((n == 0 || data) && (m == 0 || (keys && out)), "gs_index_search: null pointer");
  MarkScratch s = carve_marks(workspace, workspace_bytes, n, 0, true);
  if (!s.ok) {
    set_error_text("gs_index_search: workspace needs %zu bytes, 256-byte aligned",
                   gs_index_search_workspace_bytes(n));
    return GS_ERR_WORKSPACE;
  }
  hipStream_t st = static_cast<hipStream_t>(stream);
  init_set(s.set, s.cap, s.filter_words, st);
  auto run = [&](auto tag) {
    using IdT = decltype(tag);
    if (n > 0)
      hipLaunchKernelGGL(set_insert_kernel<IdT>, dim3(blocks_for(n, kThreads)), dim3(kThreads), 0,
                         st, s.set, static_cast<const IdT*>(data), n);
    if (m >= kLdsSearchMinKeys) {
      const int64_t groups = (m + kBigThreads * 8 - 1) / (kBigThreads * 8);
      hipLaunchKernelGGL(search_lds_kernel<IdT>, dim3(static_cast<unsigned>(groups < 512 ? groups : 512)),
                         dim3(kBigThreads), 0, st, s.set, static_cast<const IdT*>(keys), m,
                         static_cast<IdT*>(out));
    } else if (m > 0) {
      hipLaunchKernelGGL(search_kernel<IdT>, dim3(blocks_for(m, kThreads)), dim3(kThreads), 0, st,
                         s.set, static_cast<const IdT*>(keys), m, static_cast<IdT*>(out));
    }
  };
  if (id_bytes == 8) run(int64_t{}); else run(int32_t{});
  return check_launch("index_search");
}

}  // extern "C"
