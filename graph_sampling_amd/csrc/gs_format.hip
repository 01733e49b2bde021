// Sparse-format conversion on gfx950: CSC -> COO column expansion and
// COO -> CSC by a stable least-significant-digit radix sort.
//
// Replaces impl::CSC2COOCUDA and impl::COO2CSCCUDA (reference
// src/cuda/format_transform.cu:35,135; the reference leans on cub radix sort,
// whose stability pins the edge order, format_transform.cu:81-100).
//
//  * csc2coo: edge-balanced.  A workgroup owns 4096 consecutive edges; a first
//    launch over the columns has left the column of each tile's first edge in the
//    output, the offsets are read in order from there, the columns mark their first
//    edge in LDS and a running maximum turns the marks into column numbers (the
//    reference runs a full global binary search per edge, format_transform.cu:24-33).
//  * coo2csc: 8-bit digits, only ceil(log2(num_keys)/8) passes
//    (format_transform.cu:58-72 also sorts just the significant bits).  Each
//    pass is histogram -> scan -> stable scatter; the scatter ranks equal digits
//    inside a wave with 8 ballots (no LDS atomics, order preserved) and across
//    waves with a small LDS table.  What moves is one 64-bit word per edge, key
//    above and original position below, so a pass is 8 bytes in and 8 bytes out per
//    edge and the permutation falls out of the last pass.  indptr then comes from
//    one search per column in the sorted keys, confined to the keys of the
//    workgroup's 1024 columns (in LDS when they are few).
#include "gs_common.hpp"

namespace gs {
namespace {

constexpr int kThreads = 256;
constexpr int kItems = 8;
constexpr int kTile = kThreads * kItems;

template <typename P>
__device__ __forceinline__ int64_t upper_bound(P a, int64_t n, int64_t v) {
  int64_t lo = 0, hi = n;
  while (lo < hi) {
    int64_t mid = (lo + hi) >> 1;
    if (a[mid] <= v) lo = mid + 1; else hi = mid;
  }
  return lo;
}

constexpr int kCooItems = 16;
constexpr int kCooTile = kThreads * kCooItems;

// (A thread's sixteen marks lie side by side; one spare word after every sixteen keeps the
// threads of a wave on different LDS banks when each walks its own run.)
__device__ __forceinline__ int coo_slot(int i) { return i + (i >> 4); }

// First of two launches: every column with edges writes its number at the first position of
// each 4096-edge tile that begins inside it, so that the tile's workgroup finds the column
// of its first edge with one read instead of a search through the offsets.  The numbers go
// into the output itself (the tile overwrites its own first entry at the end).  A column
// that spans more than 64 tiles is written by its whole wave.
template <typename IdT>
__global__ void __launch_bounds__(kThreads)
coo_tile_heads_kernel(const int64_t* __restrict__ indptr, int64_t num_cols, IdT* __restrict__ col) {
  const int64_t c = static_cast<int64_t>(blockIdx.x) * kThreads + threadIdx.x;
  int64_t t0 = 0, t1 = -1;
  if (c < num_cols) {
    const int64_t s = indptr[c], e = indptr[c + 1];
    if (e > s) {
      t0 = (s + kCooTile - 1) / kCooTile;
      t1 = (e - 1) / kCooTile;
    }
  }
  const bool wide = t1 - t0 >= kWave;
  if (!wide)
    for (int64_t t = t0; t <= t1; ++t) col[t * kCooTile] = static_cast<IdT>(c);
  unsigned long long todo = __ballot(wide);
  const int lane = threadIdx.x & (kWave - 1);
  while (todo) {
    const int src = __ffsll(static_cast<long long>(todo)) - 1;
    todo &= todo - 1;
    const int64_t w0 = __shfl(t0, src, kWave), w1 = __shfl(t1, src, kWave);
    const int64_t wc = __shfl(c, src, kWave);
    for (int64_t t = w0 + lane; t <= w1; t += kWave) col[t * kCooTile] = static_cast<IdT>(wc);
  }
}

// A workgroup owns kCooTile consecutive edges.  The first entry of its output holds the last
// column that starts at or before the tile (left there by the launch above); from there the
// offsets are read in order, 256 at a time.  The columns that start inside the tile mark
// their first edge in LDS (of several empty columns at one position the highest wins, which
// is the owner), and a running maximum over the marks gives every edge its column: sixteen
// consecutive edges per thread, one maximum per thread across the workgroup.  No search.
// (DCSC: stored column c stands for node ids[c], format_transform.cu:48-60; a switch at
// compile time, because a load that may or may not happen before a store makes every store
// wait for everything in flight.)
template <typename IdT, bool DCSC>
__global__ void __launch_bounds__(kThreads)
csc2coo_kernel(const int64_t* __restrict__ indptr, int64_t num_cols, int64_t nnz,
               const IdT* __restrict__ ids, IdT* __restrict__ col) {
  __shared__ int s_mark[kCooTile + kCooTile / 16];
  __shared__ int s_wave[kThreads / kWave];
  __shared__ bool s_more;
  const int64_t p0 = static_cast<int64_t>(blockIdx.x) * kCooTile;
  const int64_t p1 = p0 + kCooTile < nnz ? p0 + kCooTile : nnz;
  const int64_t base = static_cast<int64_t>(col[p0]);  // holds edge p0
  for (int i = threadIdx.x; i < kCooTile + kCooTile / 16; i += kThreads) s_mark[i] = 0;
  const int64_t kNone = INT64_MAX;
  int64_t ahead = base + 1 + threadIdx.x <= num_cols ? indptr[base + 1 + threadIdx.x] : kNone;
  const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
  __syncthreads();
  // columns base + 1 ... that start before p1 start inside the tile (after p0: the last one
  // that starts at p0 is the base); the offsets are in order, so the last thread tells
  // whether the next 256 have to be looked at as well
  for (int64_t r = base + 1 + threadIdx.x;; r += kThreads) {
    const bool inside = ahead < p1;
    if (inside)
      atomicMax(&s_mark[coo_slot(static_cast<int>(ahead - p0))], static_cast<int>(r - base));
    if (threadIdx.x == kThreads - 1) s_more = inside;
    __syncthreads();
    if (!s_more) break;
    ahead = r + kThreads <= num_cols ? indptr[r + kThreads] : kNone;
    __syncthreads();  // (everyone has read the flag before it is written again)
  }
  const int at0 = threadIdx.x * (kCooItems + 1);
  int m[kCooItems];
  int run = 0;
#pragma unroll
  for (int k = 0; k < kCooItems; ++k) {
    const int v = s_mark[at0 + k];
    run = v > run ? v : run;
    m[k] = run;  // relative to what holds where the thread begins
  }
  // exclusive running maximum of the threads' last values
  int incl = run;
#pragma unroll
  for (int d = 1; d < kWave; d <<= 1) {
    const int y = __shfl_up(incl, d, kWave);
    if (lane >= d && y > incl) incl = y;
  }
  if (lane == kWave - 1) s_wave[wave] = incl;
  __syncthreads();
  int before = __shfl_up(incl, 1, kWave);
  if (lane == 0) before = 0;
  for (int w = 0; w < wave; ++w) before = s_wave[w] > before ? s_wave[w] : before;
  // column numbers (relative to base) go back into the marks' place, so that the stores
  // below are coalesced whatever the id width
#pragma unroll
  for (int k = 0; k < kCooItems; ++k) s_mark[at0 + k] = m[k] > before ? m[k] : before;
  __syncthreads();
  IdT out[kCooItems];
#pragma unroll
  for (int k = 0; k < kCooItems; ++k) {
    const int64_t c = base + s_mark[coo_slot(k * kThreads + threadIdx.x)];
    if (DCSC)
      out[k] = p0 + k * kThreads + threadIdx.x < p1 ? ids[c] : IdT(0);
    else
      out[k] = static_cast<IdT>(c);
  }
#pragma unroll
  for (int k = 0; k < kCooItems; ++k) {
    const int64_t p = p0 + k * kThreads + threadIdx.x;
    if (p < p1) col[p] = out[k];
  }
}

template <typename IdT, bool DCSC>
void launch_csc2coo(const int64_t* indptr, int64_t num_cols, int64_t nnz, const IdT* ids, IdT* col,
                    hipStream_t st) {
  hipLaunchKernelGGL((coo_tile_heads_kernel<IdT>), dim3(blocks_for(num_cols, kThreads)),
                     dim3(kThreads), 0, st, indptr, num_cols, col);
  hipLaunchKernelGGL((csc2coo_kernel<IdT, DCSC>), dim3(blocks_for(nnz, kCooTile)), dim3(kThreads),
                     0, st, indptr, num_cols, nnz, ids, col);
}

// CSC -> doubly-compressed CSC: the columns that own at least one edge, in order, and
// their offsets (what format_transform.cu:172-203 builds from the sorted COO).
struct NonEmptyColumn {
  const int64_t* indptr;
  __device__ __forceinline__ int64_t operator()(int64_t c) const {
    return indptr[c + 1] > indptr[c] ? 1 : 0;
  }
};

template <typename IdT>
__global__ void __launch_bounds__(kThreads)
compress_kernel(const int64_t* __restrict__ indptr, int64_t num_cols,
                const int64_t* __restrict__ prefix, IdT* __restrict__ val_ids,
                int64_t* __restrict__ out_indptr, int64_t* __restrict__ num_valid) {
  const int64_t c = static_cast<int64_t>(blockIdx.x) * kThreads + threadIdx.x;
  if (c > num_cols) return;
  if (c == num_cols) {
    const int64_t total = prefix[num_cols];
    out_indptr[total] = indptr[num_cols];
    *num_valid = total;
    return;
  }
  const int64_t begin = indptr[c];
  if (indptr[c + 1] > begin) {
    const int64_t w = prefix[c];
    val_ids[w] = static_cast<IdT>(c);
    out_indptr[w] = begin;
  }
}

// Sorted keys as the kernels below read them: an id array, or the sort's own words
// (key above the low idx_bits bits).
template <typename KeyT>
struct PlainKeys {
  const KeyT* key;
  __device__ __forceinline__ int64_t operator()(int64_t i) const {
    return static_cast<int64_t>(key[i]);
  }
};
struct WordKeys {
  const unsigned long long* word;
  int idx_bits;
  __device__ __forceinline__ int64_t operator()(int64_t i) const {
    return static_cast<int64_t>(word[i] >> idx_bits);
  }
};

template <typename Keys>
__device__ __forceinline__ int64_t first_not_below(const Keys& key, int64_t lo, int64_t hi,
                                                   int64_t c) {
  while (lo < hi) {
    const int64_t mid = (lo + hi) >> 1;
    if (key(mid) < c) lo = mid + 1; else hi = mid;
  }
  return lo;
}

// First position in [0, E) whose key is >= c, found by a whole wave: 64 probes split the
// range per step, so 2.7 M keys take four dependent loads instead of twenty-two.  Every
// lane of the wave calls this and gets the answer.
template <typename Keys>
__device__ __forceinline__ int64_t wave_first_not_below(const Keys& key, int64_t E, int64_t c) {
  const int lane = threadIdx.x & (kWave - 1);
  int64_t lo = 0, hi = E;
  while (lo < hi) {
    const int64_t step = (hi - lo + kWave - 1) / kWave;
    const int64_t at = lo + lane * step;
    const bool below = at < hi && key(at) < c;
    const int count = __popcll(__ballot(below));  // probes are sorted: the first `count` are below
    const int64_t new_lo = count > 0 ? lo + (count - 1) * step + 1 : lo;
    const int64_t end = lo + count * step;        // first probe that is not below, if there is one
    hi = (count < kWave && end < hi) ? end : hi;
    lo = new_lo;
  }
  return lo;
}

// indptr from sorted keys: indptr[c] = number of keys < c (format_transform.cu:123-156
// searches the whole key array once per column).  A workgroup owns 256 consecutive
// columns: two wave-wide searches bound the keys that belong to them, and the per-column
// searches run inside that range -- in LDS when it holds at most 4096 keys, which is every
// tile but those of hub columns.  A boundary-driven fill (every edge writes the offsets of
// the columns between it and its predecessor) was tried first and is worse at both ends:
// with few edges and millions of columns one lane fills a gap of a million offsets by
// itself, with many edges and few columns it reads every key to find a handful of
// boundaries.
constexpr int kPtrCols = kThreads;
constexpr int kPtrStage = 4096;

template <typename Keys>
__global__ void __launch_bounds__(kThreads)
indptr_from_sorted_kernel(Keys key, int64_t E, int64_t num_keys, int64_t* __restrict__ indptr) {
  __shared__ int64_t s_range[2];
  __shared__ int s_key[kPtrStage];
  const int64_t c0 = static_cast<int64_t>(blockIdx.x) * kPtrCols;
  const int64_t c1 = c0 + kPtrCols < num_keys + 1 ? c0 + kPtrCols : num_keys + 1;
  const int wave = threadIdx.x / kWave;
  if (wave < 2) {
    const int64_t at = wave_first_not_below(key, E, wave == 0 ? c0 : c1);
    if ((threadIdx.x & (kWave - 1)) == 0) s_range[wave] = at;
  }
  __syncthreads();
  const int64_t lo = s_range[0], hi = s_range[1];
  const int n = static_cast<int>(hi - lo <= kPtrStage ? hi - lo : -1);
  if (n >= 0) {
    for (int i = threadIdx.x; i < n; i += kThreads) s_key[i] = static_cast<int>(key(lo + i) - c0);
    __syncthreads();
  }
  const int64_t c = c0 + threadIdx.x;
  if (c >= c1) return;
  if (n >= 0) {
    const int want = static_cast<int>(c - c0);
    int a = 0, b = n;
    while (a < b) {
      const int mid = (a + b) >> 1;
      if (s_key[mid] < want) a = mid + 1; else b = mid;
    }
    indptr[c] = lo + a;
  } else {
    indptr[c] = first_not_below(key, lo, hi, c);
  }
}

// ------------------------------------------------------------ radix sort ----
// The sort moves ONE 64-bit word per edge: key above, position of the edge below
// (idx_bits = bits of the edge count).  Sorting the words is the stable sort of the keys,
// the low bits of the result are the permutation, and a pass reads and writes 8 bytes per
// edge instead of a widened key and a permutation entry each way.
constexpr int kRadixBits = 8;
constexpr int kRadix = 1 << kRadixBits;
constexpr int kWaves = kThreads / kWave;

__device__ __forceinline__ int digit_of(unsigned long long word, int shift) {
  return static_cast<int>((word >> shift) & (kRadix - 1));
}

// words of the first pass, made from the caller's keys on the fly
template <typename IdT>
struct FreshWords {
  const IdT* key;
  int idx_bits;
  __device__ __forceinline__ unsigned long long operator()(int64_t i) const {
    return (static_cast<unsigned long long>(key[i]) << idx_bits) |
           static_cast<unsigned long long>(i);
  }
};
struct StoredWords {
  const unsigned long long* word;
  __device__ __forceinline__ unsigned long long operator()(int64_t i) const { return word[i]; }
};

// A tile of the sort: 256 threads, 16 items each with 4-byte values, 8 with 8-byte values (the
// tile's words and values pass through LDS on their way out).
template <typename IdT>
struct SortTile {
  static constexpr int kPerThread = sizeof(IdT) == 4 ? 16 : 8;
  static constexpr int kSize = kThreads * kPerThread;
  static constexpr int kRounds = kSize / kWaves / kWave;  // rounds of 64 consecutive items per wave
};

// counts[d * num_blocks + b] = items of tile b with digit d
template <typename Src, int TILE>
__global__ void __launch_bounds__(kThreads)
radix_hist_kernel(Src src, int64_t E, int shift, int64_t num_blocks, int64_t* __restrict__ counts) {
  __shared__ int s_hist[kRadix];
  s_hist[threadIdx.x] = 0;
  __syncthreads();
  const int64_t base = static_cast<int64_t>(blockIdx.x) * TILE;
#pragma unroll
  for (int k = 0; k < TILE / kThreads; ++k) {
    const int64_t i = base + k * kThreads + threadIdx.x;
    if (i < E) atomicAdd(&s_hist[digit_of(src(i), shift)], 1);
  }
  __syncthreads();
  counts[static_cast<int64_t>(threadIdx.x) * num_blocks + blockIdx.x] = s_hist[threadIdx.x];
}

struct LoadI64 {
  const int64_t* p;
  __device__ __forceinline__ int64_t operator()(int64_t i) const { return p[i]; }
};

// where the last pass of the sort writes: the values in key order, the permutation, and
// the sorted keys themselves (for the offsets; null when nobody builds any)
template <typename IdT>
struct SortOutputs {
  IdT* value;
  int64_t* perm;
  IdT* key;
  int idx_bits;
};

// One pass of the sort over one tile, stable.  A wave owns a quarter of the tile, in index
// order, and visits it 64 consecutive items at a time: the rank of an item among the equal
// digits of its round comes from 8 ballots, the count of the wave's earlier rounds from a
// small LDS table only that wave touches (no workgroup barrier per round).  One barrier
// later the digits' totals are scanned, every item knows its place in the tile's sorted
// order and goes there in LDS together with its value; the tile then leaves in that
// order, so that the items of a digit are written as one run -- coalesced stores, where a
// scatter straight from registers wrote 8 bytes here and 8 bytes there.
// The value rides along with its word from the first pass on (read in input order then), so
// no pass gathers it by position; the LAST pass writes values, permutation and keys instead
// of words.
// SELF: `offsets` holds the tiles' raw counts and every workgroup adds up for itself where its
// runs start (a sort of few tiles: two launches less per pass than scanning the counts first).
constexpr int64_t kSelfScanTiles = 64;

template <typename IdT, typename Src, bool LAST, bool SELF>
__global__ void __launch_bounds__(kThreads)
radix_pass_kernel(Src src, const IdT* __restrict__ val_in, int64_t E, int shift,
                  int64_t num_blocks, const int64_t* __restrict__ offsets,
                  unsigned long long* __restrict__ out, IdT* __restrict__ val_out,
                  SortOutputs<IdT> last) {
  using T = SortTile<IdT>;
  __shared__ unsigned long long s_word[T::kSize];
  __shared__ int64_t s_base[kRadix];     // where the tile's run of a digit starts in memory
  __shared__ int s_cnt[kWaves][kRadix];  // per wave: count, then count of the earlier waves
  __shared__ int s_start[kRadix];        // where the run of a digit starts in the tile
  __shared__ int s_scan[kWaves];
  const int lane = threadIdx.x & (kWave - 1);
  const int wave = threadIdx.x / kWave;
  if (SELF) {
    // digit threadIdx.x: its items in all tiles, and in the tiles before this one
    __shared__ int64_t s_digits[kWaves];
    const int64_t* row = offsets + static_cast<int64_t>(threadIdx.x) * num_blocks;
    int64_t all = 0, before = 0;
    for (int64_t b = 0; b < num_blocks; ++b) {
      const int64_t c = row[b];
      all += c;
      before += b < static_cast<int64_t>(blockIdx.x) ? c : 0;
    }
    int64_t incl = all;
#pragma unroll
    for (int d = 1; d < kWave; d <<= 1) {
      const int64_t y = __shfl_up(incl, d, kWave);
      if (lane >= d) incl += y;
    }
    if (lane == kWave - 1) s_digits[wave] = incl;
    __syncthreads();
    int64_t lower = incl - all;  // items of the smaller digits
    for (int w = 0; w < wave; ++w) lower += s_digits[w];
    s_base[threadIdx.x] = lower + before;
  } else {
    s_base[threadIdx.x] = offsets[static_cast<int64_t>(threadIdx.x) * num_blocks + blockIdx.x];
  }
#pragma unroll
  for (int w = 0; w < kWaves; ++w) s_cnt[w][threadIdx.x] = 0;
  const int64_t base = static_cast<int64_t>(blockIdx.x) * T::kSize;
  const int64_t wave_base = base + static_cast<int64_t>(wave) * (T::kSize / kWaves);
  unsigned long long word[T::kRounds];
  IdT val[T::kRounds];
#pragma unroll
  for (int r = 0; r < T::kRounds; ++r) {
    const int64_t i = wave_base + r * kWave + lane;
    word[r] = i < E ? src(i) : ~0ull;
    val[r] = i < E ? val_in[i] : IdT(0);
  }
  __syncthreads();  // the tables are zero
  int place[T::kRounds];
#pragma unroll
  for (int r = 0; r < T::kRounds; ++r) {
    const bool live = wave_base + r * kWave + lane < E;
    const int d = digit_of(word[r], shift);
    unsigned long long peers = __ballot(live);
#pragma unroll
    for (int b = 0; b < kRadixBits; ++b) {
      const bool bit = (d >> b) & 1;
      const unsigned long long bal = __ballot(live && bit);
      peers &= bit ? bal : ~bal;
    }
    const int rank = __popcll(peers & ((1ull << lane) - 1ull));
    const int before = s_cnt[wave][d];  // the wave's earlier rounds (LDS operations of a wave keep their order)
    place[r] = before + rank;
    if (live && rank == 0) s_cnt[wave][d] = before + __popcll(peers);
  }
  __syncthreads();
  // digit threadIdx.x: counts of the waves -> counts of the earlier waves, total -> start
  int total = 0;
#pragma unroll
  for (int w = 0; w < kWaves; ++w) {
    const int c = s_cnt[w][threadIdx.x];
    s_cnt[w][threadIdx.x] = total;
    total += c;
  }
  int incl = total;
#pragma unroll
  for (int d = 1; d < kWave; d <<= 1) {
    const int y = __shfl_up(incl, d, kWave);
    if (lane >= d) incl += y;
  }
  if (lane == kWave - 1) s_scan[wave] = incl;
  __syncthreads();
  int start = incl - total;
  for (int w = 0; w < wave; ++w) start += s_scan[w];
  s_start[threadIdx.x] = start;
  __syncthreads();
  // (words first, then the values through the same LDS: half the footprint of staging both
  // at once, and twice the workgroups per compute unit)
#pragma unroll
  for (int r = 0; r < T::kRounds; ++r) {
    const int d = digit_of(word[r], shift);
    place[r] += s_start[d] + s_cnt[wave][d];
    if (wave_base + r * kWave + lane < E) s_word[place[r]] = word[r];
  }
  __syncthreads();
  const int n = static_cast<int>(E - base < T::kSize ? E - base : T::kSize);
  int64_t dst[T::kPerThread];
#pragma unroll
  for (int k = 0; k < T::kPerThread; ++k) {
    const int j = k * kThreads + threadIdx.x;
    dst[k] = -1;
    if (j < n) {
      const unsigned long long w = s_word[j];
      const int d = digit_of(w, shift);
      dst[k] = s_base[d] + (j - s_start[d]);
      if (LAST) {
        last.perm[dst[k]] = static_cast<int64_t>(w & ((1ull << last.idx_bits) - 1ull));
        if (last.key) last.key[dst[k]] = static_cast<IdT>(w >> last.idx_bits);
      } else {
        out[dst[k]] = w;
      }
    }
  }
  __syncthreads();
  IdT* s_val = reinterpret_cast<IdT*>(s_word);
#pragma unroll
  for (int r = 0; r < T::kRounds; ++r)
    if (wave_base + r * kWave + lane < E) s_val[place[r]] = val[r];
  __syncthreads();
  IdT* to = LAST ? last.value : val_out;
#pragma unroll
  for (int k = 0; k < T::kPerThread; ++k)
    if (dst[k] >= 0) to[dst[k]] = s_val[k * kThreads + threadIdx.x];
}

int bits_for(int64_t n) {  // smallest b with 2^b >= n
  int bits = 0;
  while ((int64_t(1) << bits) < n) ++bits;
  return bits;
}

int num_passes(int64_t num_keys) {
  return (bits_for(num_keys) + kRadixBits - 1) / kRadixBits;  // format_transform.cu:58-72
}

// Offsets of B consecutive column ranges, each re-based to start at 0 and laid
// out one after the other (batch b: offsets[b+1]-offsets[b]+1 entries starting
// at offsets[b] + b).  One output entry per lane, batch by binary search -- over a
// copy of the batch offsets in LDS when there are at most 1023 batches, so that only
// the two reads of indptr go to memory.
constexpr int kSplitStage = 1024;

__global__ void __launch_bounds__(kThreads)
indptr_split_kernel(const int64_t* __restrict__ indptr, const int64_t* __restrict__ offsets,
                    int64_t B, int64_t total, int64_t* __restrict__ out,
                    int64_t* __restrict__ cuts) {
  __shared__ int64_t s_off[kSplitStage];
  const bool staged = B <= kSplitStage;
  if (staged) {
    for (int64_t b = threadIdx.x; b < B; b += kThreads) s_off[b] = offsets[b];
    __syncthreads();
  }
  const int64_t* off = staged ? s_off : offsets;
  const int64_t q = static_cast<int64_t>(blockIdx.x) * kThreads + threadIdx.x;
  // where every batch's entries start (and the last one's end), for the caller's next cut
  if (cuts && q <= B) cuts[q] = indptr[offsets[q]];
  if (q >= total) return;
  int64_t lo = 0, hi = B - 1;  // last b with offsets[b] + b <= q
  while (lo < hi) {
    const int64_t mid = (lo + hi + 1) >> 1;
    if (off[mid] + mid <= q) lo = mid; else hi = mid - 1;
  }
  const int64_t begin = off[lo];
  out[q] = indptr[begin + (q - begin - lo)] - indptr[begin];
}

template <typename IdT, typename Src>
void launch_pass(Src src, bool last, bool self, dim3 grid, hipStream_t st, const IdT* vin, int64_t E,
                 int shift, int64_t blocks, const int64_t* where, unsigned long long* wout,
                 IdT* vout, const SortOutputs<IdT>& outs) {
  auto go = [&](auto kernel) {
    hipLaunchKernelGGL(kernel, grid, dim3(kThreads), 0, st, src, vin, E, shift, blocks, where, wout,
                       vout, outs);
  };
  if (last && self) go(radix_pass_kernel<IdT, Src, true, true>);
  else if (last) go(radix_pass_kernel<IdT, Src, true, false>);
  else if (self) go(radix_pass_kernel<IdT, Src, false, true>);
  else go(radix_pass_kernel<IdT, Src, false, false>);
}

template <typename IdT>
int coo2csc_impl(const IdT* key, const IdT* value, int64_t E, int64_t num_keys, int sorted,
                 int64_t* indptr, IdT* out_value, int64_t* perm, void* workspace,
                 size_t workspace_bytes, hipStream_t st) {
  const dim3 ptr_grid(blocks_for(num_keys + 1, kPtrCols));
  if (E == 0 && !indptr) return GS_OK;
  if (sorted || E == 0) {
    PlainKeys<IdT> keys{key};
    hipLaunchKernelGGL((indptr_from_sorted_kernel<PlainKeys<IdT>>), ptr_grid, dim3(kThreads), 0, st,
                       keys, E, num_keys, indptr);
    return check_launch("coo2csc");
  }
  const int idx_bits = bits_for(E);
  int passes = num_passes(num_keys);
  if (passes == 0) passes = 1;  // one key: still produces perm = identity
  if (idx_bits + passes * kRadixBits > 64) {
    set_error_text("gs_coo2csc: %lld edges with keys below %lld do not fit the sort's 64-bit words",
                   static_cast<long long>(E), static_cast<long long>(num_keys));
    return GS_ERR_UNSUPPORTED;
  }
  using T = SortTile<IdT>;
  const int64_t blocks = blocks_for(E, T::kSize);
  const int64_t table = kRadix * blocks;
  Carver ws(workspace, workspace_bytes);
  unsigned long long* wbuf[2] = {ws.take<unsigned long long>(E), ws.take<unsigned long long>(E)};
  IdT* vbuf[2] = {ws.take<IdT>(E), ws.take<IdT>(E)};
  int64_t* counts = ws.take<int64_t>(table);
  int64_t* offsets = ws.take<int64_t>(table + 1);
  int64_t* tiles = ws.take<int64_t>(scan_num_tiles(table) + 1);
  if (!ws.ok) {
    set_error_text("gs_coo2csc: workspace needs %zu bytes, 256-byte aligned",
                   gs_coo2csc_workspace_bytes(E, num_keys));
    return GS_ERR_WORKSPACE;
  }
  // the sorted keys (for the offsets) land where the last pass would have put its words
  IdT* sorted_keys = indptr ? reinterpret_cast<IdT*>(wbuf[(passes - 1) & 1]) : nullptr;
  const SortOutputs<IdT> outs{out_value, perm, sorted_keys, idx_bits};
  const dim3 grid(static_cast<unsigned>(blocks));
  const unsigned long long* win = nullptr;  // null: the first pass reads the caller's keys
  const IdT* vin = value;
  for (int p = 0; p < passes; ++p) {
    unsigned long long* wout = wbuf[p & 1];
    IdT* vout = vbuf[p & 1];
    const int shift = idx_bits + p * kRadixBits;
    const bool last = p == passes - 1;
    if (p == 0) {
      FreshWords<IdT> src{key, idx_bits};
      hipLaunchKernelGGL((radix_hist_kernel<FreshWords<IdT>, T::kSize>), grid, dim3(kThreads), 0, st,
                         src, E, shift, blocks, counts);
    } else {
      StoredWords src{win};
      hipLaunchKernelGGL((radix_hist_kernel<StoredWords, T::kSize>), grid, dim3(kThreads), 0, st, src,
                         E, shift, blocks, counts);
    }
    const bool self = blocks <= kSelfScanTiles;
    if (!self) {
      LoadI64 f{counts};
      GS_RETURN_IF_ERROR(exclusive_scan(f, table, offsets, tiles, st));
    }
    const int64_t* where = self ? counts : offsets;
    if (p == 0) {
      FreshWords<IdT> src{key, idx_bits};
      launch_pass<IdT>(src, last, self, grid, st, vin, E, shift, blocks, where, wout, vout, outs);
    } else {
      StoredWords src{win};
      launch_pass<IdT>(src, last, self, grid, st, vin, E, shift, blocks, where, wout, vout, outs);
    }
    win = wout;
    vin = vout;
  }
  if (indptr) {  // (null: the caller wants the sorted order only)
    PlainKeys<IdT> keys{sorted_keys};
    hipLaunchKernelGGL((indptr_from_sorted_kernel<PlainKeys<IdT>>), ptr_grid, dim3(kThreads), 0, st,
                       keys, E, num_keys, indptr);
  }
  return check_launch("coo2csc");
}

// ---------------------------------------------------- binned scatter-add ----
// out[target[e]] += data[e]^powk without an atomic to memory: one partition pass of the sort
// above brings the edges of every run of 2^bin_shift targets together (at most 256 runs),
// and a workgroup then adds a run's edges up in LDS and writes its sums with plain stores.
// Atomics to memory run at about ten per nanosecond on this part whatever the kernel does
// around them; edges that mostly hit different targets paid that price one by one.
constexpr int kBinThreads = 1024;
// A run with many edges (the hubs' run of a skewed graph holds a third of them) is shared by
// several workgroups, which then add their sums to memory with atomics: the additions to one
// LDS word queue up, and 16 k edges a workgroup measured fastest (2 M edges over 2.45 M
// targets: 0.32 ms with one workgroup a run, 0.14 at 64 k edges, 0.10 at 16 k or 8 k).
constexpr int kBinParts = 64;             // workgroups that may share one run of targets
constexpr int64_t kBinPartItems = 16384;  // edges a workgroup takes before a run is shared
constexpr int kBinMaxShift = 15;         // 2^15 sums = 128 KB of LDS

__global__ void __launch_bounds__(kBinThreads)
bin_sum_kernel(const unsigned long long* __restrict__ words, const int32_t* __restrict__ vals,
               const int64_t* __restrict__ offsets, int64_t num_blocks, int num_bins, int idx_bits,
               int bin_shift, int powk, int64_t num_targets, float* __restrict__ out) {
  extern __shared__ float s_sum[];
  // Which run, and which share of it, this workgroup takes: the launch has one workgroup per
  // share that can exist (a run of n edges has ceil(n / 16 k) of them, 64 at most), and every
  // workgroup works the numbering out for itself from the runs' sizes.  (A launch of 64
  // workgroups per run, most of which left at once, spent 30 of its 48 us handing 64 KB of LDS
  // to workgroups with nothing to do.)
  __shared__ int64_t s_scan[kBinThreads / kWave + 1];
  __shared__ int s_first[kRadix + 1];
  {
    int64_t mine = 0;
    if (threadIdx.x < num_bins) {
      const int64_t n = offsets[(threadIdx.x + 1) * num_blocks] - offsets[threadIdx.x * num_blocks];
      mine = (n + kBinPartItems - 1) / kBinPartItems;
      if (mine > kBinParts) mine = kBinParts;
    }
    int64_t total;
    const int64_t before = block_exclusive_scan<kBinThreads>(mine, &total, s_scan);
    if (threadIdx.x <= num_bins) s_first[threadIdx.x] = static_cast<int>(before);
    __syncthreads();
  }
  if (static_cast<int>(blockIdx.x) >= s_first[num_bins]) return;
  int bin = 0;
  for (int step = kRadix / 2; step > 0; step >>= 1)
    if (bin + step <= num_bins && s_first[bin + step] <= static_cast<int>(blockIdx.x)) bin += step;
  const int part = static_cast<int>(blockIdx.x) - s_first[bin];
  const int64_t lo = offsets[bin * num_blocks], hi = offsets[(bin + 1) * num_blocks];
  const int64_t n = hi - lo;
  int64_t parts = (n + kBinPartItems - 1) / kBinPartItems;
  if (parts > kBinParts) parts = kBinParts;
  const int width = 1 << bin_shift;
  for (int j = threadIdx.x; j < width; j += kBinThreads) s_sum[j] = 0.0f;
  __syncthreads();
  const int64_t per = (n + parts - 1) / parts;
  const int64_t begin = lo + part * per;
  const int64_t end = begin + per < hi ? begin + per : hi;
  const int64_t first = static_cast<int64_t>(bin) << bin_shift;
  // a thread's edges eight at a time, all reads (clamped to the part) before the first
  // addition: one edge at a time every addition waits for its own trip to memory
  constexpr int kBatch = 8;
  for (int64_t i0 = begin + threadIdx.x; i0 < end; i0 += kBinThreads * kBatch) {
    unsigned long long w[kBatch];
    int v[kBatch];
#pragma unroll
    for (int u = 0; u < kBatch; ++u) {
      const int64_t i = i0 + u * kBinThreads;
      w[u] = words[i < end ? i : end - 1];
    }
#pragma unroll
    for (int u = 0; u < kBatch; ++u) {
      const int64_t i = i0 + u * kBinThreads;
      v[u] = vals[i < end ? i : end - 1];
    }
#pragma unroll
    for (int u = 0; u < kBatch; ++u) {
      const int64_t t = static_cast<int64_t>(w[u] >> idx_bits) - first;
      // (a target beyond num_targets has no sum to go to: left out, as out has no room for it)
      if (i0 + u * kBinThreads < end && t >= 0 && t < width)
        atomicAdd(&s_sum[t], powk_f(__int_as_float(v[u]), powk));
    }
  }
  __syncthreads();
  if (parts > 1) {
    for (int j = threadIdx.x; j < width; j += kBinThreads) {
      const float x = s_sum[j];
      if (x != 0.0f && first + j < num_targets) unsafeAtomicAdd(out + first + j, x);
    }
    return;
  }
  // the run is this workgroup's alone: plain read, add, write -- a thread's sums eight at a
  // time, the reads (of a word that is always there where the sum is zero) before the writes
  for (int j0 = threadIdx.x; j0 < width; j0 += kBinThreads * kBatch) {
    float x[kBatch], was[kBatch];
#pragma unroll
    for (int u = 0; u < kBatch; ++u) {
      const int j = j0 + u * kBinThreads;
      x[u] = (j < width && first + j < num_targets) ? s_sum[j] : 0.0f;
    }
#pragma unroll
    for (int u = 0; u < kBatch; ++u) was[u] = out[x[u] != 0.0f ? first + j0 + u * kBinThreads : first];
#pragma unroll
    for (int u = 0; u < kBatch; ++u)
      if (x[u] != 0.0f) out[first + j0 + u * kBinThreads] = was[u] + x[u];
  }
}

// whether the binned path takes the call: 4-byte ids (the value rides along in an id-sized
// word), plain edge order, few enough targets for 256 runs of at most 2^15, enough edges
// for five launches to pay
inline bool bin_sum_applies(int id_bytes, const int64_t* e_ids, int64_t E, int64_t num_targets) {
  return id_bytes == 4 && !e_ids && E >= (int64_t(1) << 17) && num_targets > 0 &&
         num_targets <= (int64_t(kRadix) << kBinMaxShift) && E < (int64_t(1) << 31);
}

int bin_sum_impl(const int32_t* target, const float* data, int64_t E, int powk, int64_t num_targets,
                 float* out, void* workspace, size_t workspace_bytes, hipStream_t st) {
  using T = SortTile<int32_t>;
  const int64_t blocks = blocks_for(E, T::kSize);
  const int64_t table = kRadix * blocks;
  Carver ws(workspace, workspace_bytes);
  unsigned long long* words = ws.take<unsigned long long>(E);
  int32_t* vals = ws.take<int32_t>(E);
  int64_t* counts = ws.take<int64_t>(table);
  int64_t* offsets = ws.take<int64_t>(table + 1);
  int64_t* tiles = ws.take<int64_t>(scan_num_tiles(table) + 1);
  if (!ws.ok) {
    set_error_text("gs_coo_sum_binned: workspace needs %zu bytes, 256-byte aligned",
                   gs_coo_sum_workspace_bytes(E, num_targets));
    return GS_ERR_WORKSPACE;
  }
  const int idx_bits = bits_for(E);
  int bin_shift = bits_for(num_targets) - kRadixBits;
  if (bin_shift < 0) bin_shift = 0;
  const int shift = idx_bits + bin_shift;
  const dim3 grid(static_cast<unsigned>(blocks));
  FreshWords<int32_t> src{target, idx_bits};
  hipLaunchKernelGGL((radix_hist_kernel<FreshWords<int32_t>, T::kSize>), grid, dim3(kThreads), 0, st,
                     src, E, shift, blocks, counts);
  LoadI64 f{counts};
  GS_RETURN_IF_ERROR(exclusive_scan(f, table, offsets, tiles, st));
  const SortOutputs<int32_t> none{nullptr, nullptr, nullptr, idx_bits};
  launch_pass<int32_t>(src, false, false, grid, st, reinterpret_cast<const int32_t*>(data), E, shift,
                       blocks, offsets, words, vals, none);
  const int bins = static_cast<int>(((num_targets - 1) >> bin_shift) + 1);
  // (per call: the attribute belongs to the device the call runs on)
  const hipError_t lds_allowed = hipFuncSetAttribute(
      reinterpret_cast<const void*>(bin_sum_kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
      static_cast<int>(sizeof(float) << kBinMaxShift));
  if (lds_allowed != hipSuccess) {
    set_error_text("gs_coo_sum_binned: %s", hipGetErrorString(lds_allowed));
    return GS_ERR_LAUNCH;
  }
  const int64_t shares = E / kBinPartItems + bins;  // at most: sum of ceil(n / 16 k) over the runs
  hipLaunchKernelGGL(bin_sum_kernel, dim3(static_cast<unsigned>(shares)), dim3(kBinThreads),
                     sizeof(float) << bin_shift, st, words, vals, offsets, blocks, bins, idx_bits,
                     bin_shift, powk, num_targets, out);
  return check_launch("coo_sum_binned");
}

}  // namespace
}  // namespace gs

using namespace gs;

extern "C" {

int gs_csc2coo(const int64_t* indptr, int64_t num_cols, int64_t nnz, void* col, int id_bytes,
               void* stream) {
  GS_REQUIRE(num_cols >= 0 && nnz >= 0 && num_cols < (int64_t(1) << 31),
             "gs_csc2coo: negative size or more than 2^31 columns");
  GS_REQUIRE(nnz == 0 || (indptr && col), "gs_csc2coo: null pointer");
  GS_REQUIRE(valid_id_bytes(id_bytes), "gs_csc2coo: id_bytes must be 4 or 8, got %d", id_bytes);
  if (nnz == 0) return GS_OK;
  hipStream_t st = static_cast<hipStream_t>(stream);
  if (id_bytes == 8)
    launch_csc2coo<int64_t, false>(indptr, num_cols, nnz, nullptr, static_cast<int64_t*>(col), st);
  else
    launch_csc2coo<int32_t, false>(indptr, num_cols, nnz, nullptr, static_cast<int32_t*>(col), st);
  return check_launch("csc2coo");
}

int gs_dcsc2coo(const int64_t* indptr, int64_t num_cols, int64_t nnz, const void* ids, void* col,
                int id_bytes, void* stream) {
  GS_REQUIRE(num_cols >= 0 && nnz >= 0 && num_cols < (int64_t(1) << 31),
             "gs_dcsc2coo: negative size or more than 2^31 columns");
  GS_REQUIRE(nnz == 0 || (indptr && col && ids), "gs_dcsc2coo: null pointer");
  GS_REQUIRE(valid_id_bytes(id_bytes), "gs_dcsc2coo: id_bytes must be 4 or 8, got %d", id_bytes);
  if (nnz == 0) return GS_OK;
  hipStream_t st = static_cast<hipStream_t>(stream);
  if (id_bytes == 8)
    launch_csc2coo<int64_t, true>(indptr, num_cols, nnz, static_cast<const int64_t*>(ids),
                              static_cast<int64_t*>(col), st);
  else
    launch_csc2coo<int32_t, true>(indptr, num_cols, nnz, static_cast<const int32_t*>(ids),
                              static_cast<int32_t*>(col), st);
  return check_launch("dcsc2coo");
}

size_t gs_csc_compress_workspace_bytes(int64_t num_cols) {
  if (num_cols < 0) num_cols = 0;
  return padded(static_cast<size_t>(num_cols + 1) * 8) + scan_workspace_bytes(num_cols);
}

int gs_csc_compress(const int64_t* indptr, int64_t num_cols, int id_bytes, void* val_ids,
                    int64_t* out_indptr, int64_t* num_valid, void* workspace,
                    size_t workspace_bytes, void* stream) {
  GS_REQUIRE(num_cols >= 0 && indptr && out_indptr && num_valid && (num_cols == 0 || val_ids),
             "gs_csc_compress: bad argument");
  GS_REQUIRE(valid_id_bytes(id_bytes), "gs_csc_compress: id_bytes must be 4 or 8, got %d", id_bytes);
  Carver ws(workspace, workspace_bytes);
  int64_t* prefix = ws.take<int64_t>(num_cols + 1);
  int64_t* tiles = ws.take<int64_t>(scan_num_tiles(num_cols) + 1);
  if (!ws.ok) {
    set_error_text("gs_csc_compress: workspace needs %zu bytes, 256-byte aligned",
                   gs_csc_compress_workspace_bytes(num_cols));
    return GS_ERR_WORKSPACE;
  }
  hipStream_t st = static_cast<hipStream_t>(stream);
  NonEmptyColumn f{indptr};
  GS_RETURN_IF_ERROR(exclusive_scan(f, num_cols, prefix, tiles, st));
  const dim3 grid(blocks_for(num_cols + 1, kThreads));
  if (id_bytes == 8)
    hipLaunchKernelGGL(compress_kernel<int64_t>, grid, dim3(kThreads), 0, st, indptr, num_cols,
                       prefix, static_cast<int64_t*>(val_ids), out_indptr, num_valid);
  else
    hipLaunchKernelGGL(compress_kernel<int32_t>, grid, dim3(kThreads), 0, st, indptr, num_cols,
                       prefix, static_cast<int32_t*>(val_ids), out_indptr, num_valid);
  return check_launch("csc_compress");
}

size_t gs_coo2csc_workspace_bytes(int64_t E, int64_t num_keys) {
  (void)num_keys;
  if (E < 0) E = 0;
  // sized for the smaller tile (8-byte ids), which has the larger table
  const int64_t blocks = blocks_for(E, SortTile<int64_t>::kSize);
  const int64_t table = kRadix * blocks;
  const size_t n = static_cast<size_t>(E > 0 ? E : 1);
  return 2 * padded(n * 8) +  // the sort's words, ping-pong
         2 * padded(n * 8) +  // the values riding along, ping-pong
         padded(static_cast<size_t>(table) * 8) + padded(static_cast<size_t>(table + 1) * 8) +
         scan_workspace_bytes(table);
}

int gs_coo2csc(const void* key, const void* value, int id_bytes, int64_t E, int64_t num_keys,
               int sorted, int64_t* indptr, void* out_value, int64_t* perm, void* workspace,
               size_t workspace_bytes, void* stream) {
  GS_REQUIRE(E >= 0 && num_keys >= 0, "gs_coo2csc: negative size");
  GS_REQUIRE(indptr || !sorted, "gs_coo2csc: sorted keys and no indptr leave nothing to do");
  GS_REQUIRE(E == 0 || key, "gs_coo2csc: key is null");
  GS_REQUIRE(sorted || E == 0 || (value && out_value && perm),
             "gs_coo2csc: value/out_value/perm required when the keys are not sorted");
  GS_REQUIRE(valid_id_bytes(id_bytes), "gs_coo2csc: id_bytes must be 4 or 8, got %d", id_bytes);
  hipStream_t st = static_cast<hipStream_t>(stream);
  return id_bytes == 8
             ? coo2csc_impl<int64_t>(static_cast<const int64_t*>(key),
                                     static_cast<const int64_t*>(value), E, num_keys, sorted,
                                     indptr, static_cast<int64_t*>(out_value), perm, workspace,
                                     workspace_bytes, st)
             : coo2csc_impl<int32_t>(static_cast<const int32_t*>(key),
                                     static_cast<const int32_t*>(value), E, num_keys, sorted,
                                     indptr, static_cast<int32_t*>(out_value), perm, workspace,
                                     workspace_bytes, st);
}

int gs_indptr_split(const int64_t* indptr, const int64_t* offsets, int64_t num_batches,
                    int64_t total, int64_t* out, void* stream) {
  return gs_indptr_split_cuts(indptr, offsets, num_batches, total, out, nullptr, stream);
}

int gs_indptr_split_cuts(const int64_t* indptr, const int64_t* offsets, int64_t num_batches,
                         int64_t total, int64_t* out, int64_t* cuts, void* stream) {
  GS_REQUIRE(num_batches >= 0 && total >= 0, "gs_indptr_split: negative size");
  if (num_batches == 0 || (total == 0 && !cuts)) return GS_OK;
  GS_REQUIRE(indptr && offsets && (out || total == 0), "gs_indptr_split: null pointer");
  const int64_t lanes = cuts && num_batches + 1 > total ? num_batches + 1 : total;
  hipLaunchKernelGGL(indptr_split_kernel, dim3(blocks_for(lanes, kThreads)), dim3(kThreads), 0,
                     static_cast<hipStream_t>(stream), indptr, offsets, num_batches, total, out,
                     cuts);
  return check_launch("indptr_split");
}

size_t gs_coo_sum_workspace_bytes(int64_t E, int64_t num_targets) {
  if (E < 0) E = 0;
  if (!bin_sum_applies(4, nullptr, E, num_targets)) return 256;
  const int64_t blocks = blocks_for(E, SortTile<int32_t>::kSize);
  const int64_t table = kRadix * blocks;
  return padded(static_cast<size_t>(E) * 8) + padded(static_cast<size_t>(E) * 4) +
         padded(static_cast<size_t>(table) * 8) + padded(static_cast<size_t>(table + 1) * 8) +
         scan_workspace_bytes(table);
}

int gs_coo_sum_binned(const void* target, int id_bytes, const int64_t* e_ids, const float* data,
                      int64_t E, int64_t powk, int64_t num_targets, float* out, void* workspace,
                      size_t workspace_bytes, void* stream) {
  GS_REQUIRE(E >= 0 && powk >= 1 && num_targets >= 0,
             "gs_coo_sum_binned: negative size or powk < 1");
  GS_REQUIRE(E == 0 || (target && data && out), "gs_coo_sum_binned: null pointer");
  GS_REQUIRE(valid_id_bytes(id_bytes), "gs_coo_sum_binned: id_bytes must be 4 or 8, got %d",
             id_bytes);
  if (E == 0) return GS_OK;
  if (!bin_sum_applies(id_bytes, e_ids, E, num_targets))
    return coo_sum_bounded(target, id_bytes, e_ids, data, E, powk, num_targets, out, stream);
  return bin_sum_impl(static_cast<const int32_t*>(target), data, E, static_cast<int>(powk),
                      num_targets, out, workspace, workspace_bytes,
                      static_cast<hipStream_t>(stream));
}

}  // extern "C"
