// The tail of a layer-wise (LADIES / FastGCN style) sampler on a column slice held as a COO:
// the node set, the rows of the slice that belong to it, and the block's values in the order
// the reference's operator chain leaves them in
//   nodes = unique(cat(seeds, picked));  sub = U[nodes, :].divide(prob[nodes], axis=1)
//   (examples/ladies/ladies_raw.py:15-22: a CSR of all of U, src/graph.cc:258-283, its row
//   slice, a division by row, then a CSC of the result for normalize(axis=0) and the block,
//   src/graph.cc:585-644, 782-839)
// without the sorts of all of U: the edges are tested against the sorted node set (held in
// LDS), and only the kept ones are sorted, once, by (column, new row).
#include "gs_common.hpp"

namespace gs {
namespace {

// ---------------------------------------------------------------- node set ----
constexpr int kUnionThreads = 1024;

// out = the distinct values of a and b in increasing order (what torch.unique gives for ids,
// which are not negative), *count = how many: one workgroup, bitonic sort of 2^bits >= na + nb
// keys in LDS.
template <typename IdT>
__global__ void __launch_bounds__(kUnionThreads)
sorted_union_kernel(const IdT* __restrict__ a, int64_t na, const IdT* __restrict__ b, int64_t nb,
                    int slots, IdT* __restrict__ out, int64_t* __restrict__ count) {
  using KeyT = typename std::make_unsigned<IdT>::type;
  constexpr KeyT kNoKey = ~KeyT(0);  // sorts behind every id
  extern __shared__ unsigned long long s_raw[];
  KeyT* s_keys = reinterpret_cast<KeyT*>(s_raw);
  __shared__ int64_t s_scan[kUnionThreads / kWave + 1];
  for (int i = threadIdx.x; i < slots; i += kUnionThreads) {
    KeyT v = kNoKey;
    if (i < na)
      v = static_cast<KeyT>(a[i]);
    else if (i < na + nb)
      v = static_cast<KeyT>(b[i - na]);
    s_keys[i] = v;
  }
  __syncthreads();
  for (int k = 2; k <= slots; k <<= 1) {
    for (int j = k >> 1; j > 0; j >>= 1) {
      for (int t = threadIdx.x; t < slots / 2; t += kUnionThreads) {  // one pair a thread
        const int i = ((t & ~(j - 1)) << 1) | (t & (j - 1));
        const int other = i | j;
        const KeyT x = s_keys[i], y = s_keys[other];
        const bool ascending = (i & k) == 0;
        if ((x > y) == ascending) {
          s_keys[i] = y;
          s_keys[other] = x;
        }
      }
      __syncthreads();
    }
  }
  // a thread takes `per` consecutive keys, so that the distinct ones leave in order
  const int per = slots > kUnionThreads ? slots / kUnionThreads : 1;
  const int first = threadIdx.x * per;
  int64_t mine = 0;
  for (int u = 0; u < per; ++u) {
    const int i = first + u;
    if (i < slots && s_keys[i] != kNoKey && (i == 0 || s_keys[i] != s_keys[i - 1])) ++mine;
  }
  int64_t total;
  int64_t at = block_exclusive_scan<kUnionThreads>(mine, &total, s_scan);
  for (int u = 0; u < per; ++u) {
    const int i = first + u;
    if (i < slots && s_keys[i] != kNoKey && (i == 0 || s_keys[i] != s_keys[i - 1]))
      out[at++] = static_cast<IdT>(s_keys[i]);
  }
  if (threadIdx.x == 0) *count = total;
}

// ------------------------------------------------------------- row filter ----
constexpr int kPickThreads = 256;
constexpr int kPickItems = 16;
constexpr int kPickTile = kPickThreads * kPickItems;

// position of v in the sorted s_nodes[0..n), -1 when absent
template <typename IdT>
__device__ __forceinline__ int find_node(const IdT* s_nodes, int n, IdT v) {
  int lo = 0, hi = n;
  while (lo < hi) {
    const int mid = (lo + hi) >> 1;
    if (s_nodes[mid] < v)
      lo = mid + 1;
    else
      hi = mid;
  }
  return (lo < n && s_nodes[lo] == v) ? lo : -1;
}

// Pass one: place[e] = where the row of edge e stands among the nodes (a binary search of
// the node set in LDS), -1 when it is none of them; tile_counts[tile] = how many of the tile's
// edges are kept.  A thread takes 16 consecutive edges.  (An open-addressing table over the
// node set in LDS, built by every workgroup for itself, was no faster: 31 us against 31 us on
// 2.8 M edges and 1.5 k nodes, and 30 us against 19 us on 35 k edges.)
template <typename IdT>
__global__ void __launch_bounds__(kPickThreads)
pick_count_kernel(const IdT* __restrict__ row, int64_t E, const IdT* __restrict__ nodes,
                  const int64_t* __restrict__ num_nodes, int max_nodes,
                  int* __restrict__ place, int64_t* __restrict__ tile_counts) {
  extern __shared__ unsigned long long s_raw[];
  IdT* s_nodes = reinterpret_cast<IdT*>(s_raw);
  __shared__ int64_t s_scan[kPickThreads / kWave + 1];
  const int64_t n64 = *num_nodes;
  const int n = static_cast<int>(n64 < max_nodes ? n64 : max_nodes);
  for (int i = threadIdx.x; i < n; i += kPickThreads) s_nodes[i] = nodes[i];
  __syncthreads();
  const int64_t base = static_cast<int64_t>(blockIdx.x) * kPickTile + threadIdx.x * kPickItems;
  // all sixteen rows first (clamped, no condition in front of a read), then the searches
  IdT rows[kPickItems];
#pragma unroll
  for (int u = 0; u < kPickItems; ++u) rows[u] = row[base + u < E ? base + u : E - 1];
  int found[kPickItems];
  int64_t mine = 0;
#pragma unroll
  for (int u = 0; u < kPickItems; ++u) {
    found[u] = base + u < E ? find_node(s_nodes, n, rows[u]) : -1;
    mine += found[u] >= 0;
  }
#pragma unroll
  for (int u = 0; u < kPickItems; ++u)
    if (base + u < E) place[base + u] = found[u];
  int64_t total;
  block_exclusive_scan<kPickThreads>(mine, &total, s_scan);
  if (threadIdx.x == 0) tile_counts[blockIdx.x] = total;
}

// Pass two: the kept edges, in edge order, as key = column << node_bits | place and their
// position in the COO; the tile's first output place comes from the scan of the counts.
template <typename IdT>
__global__ void __launch_bounds__(kPickThreads)
pick_fill_kernel(const int* __restrict__ place, const IdT* __restrict__ col, int64_t E,
                 int node_bits, const int64_t* __restrict__ tile_offsets, int64_t num_tiles,
                 const int64_t* __restrict__ num_nodes, IdT* __restrict__ kept_key,
                 IdT* __restrict__ kept_pos, int64_t* __restrict__ totals, gs_mailbox* box,
                 int64_t ticket) {
  __shared__ int64_t s_scan[kPickThreads / kWave + 1];
  const int64_t base = static_cast<int64_t>(blockIdx.x) * kPickTile + threadIdx.x * kPickItems;
  int at[kPickItems];
  int64_t mine = 0;
#pragma unroll
  for (int u = 0; u < kPickItems; ++u) {
    at[u] = base + u < E ? place[base + u] : -1;
    mine += at[u] >= 0;
  }
  int64_t total;
  int64_t out = block_exclusive_scan<kPickThreads>(mine, &total, s_scan) + tile_offsets[blockIdx.x];
#pragma unroll
  for (int u = 0; u < kPickItems; ++u) {
    if (at[u] >= 0) {
      const int64_t e = base + u;
      kept_key[out] = static_cast<IdT>((static_cast<int64_t>(col[e]) << node_bits) | at[u]);
      kept_pos[out] = static_cast<IdT>(e);
      ++out;
    }
  }
  if (blockIdx.x == 0 && threadIdx.x == 0) {
    const int64_t kept = tile_offsets[num_tiles];
    totals[0] = *num_nodes;
    totals[1] = kept;
    post_mailbox(box, kept, ticket);
  }
}

struct LoadCounts {
  const int64_t* p;
  __device__ __forceinline__ int64_t operator()(int64_t i) const { return p[i]; }
};

// ------------------------------------------------------------ block values ----
// offsets of the columns from the kept edges' keys (which come by column): the thread of a
// column's first edge writes the offsets of that column and of the empty ones before it, the
// last edge's thread those of the columns behind
template <typename IdT>
__global__ void __launch_bounds__(256)
column_offsets_kernel(const IdT* __restrict__ kept_key, int64_t kept, int node_bits,
                      int64_t num_cols, int64_t* __restrict__ out_indptr,
                      unsigned int* __restrict__ num_long) {
  const int64_t i = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x;
  if (i == 0) *num_long = 0u;  // (the list of long columns is made by the next launch)
  if (kept == 0) {
    for (int64_t c = i; c <= num_cols; c += static_cast<int64_t>(gridDim.x) * 256) out_indptr[c] = 0;
    return;
  }
  if (i >= kept) return;
  const int64_t c = static_cast<int64_t>(kept_key[i]) >> node_bits;
  const int64_t before = i > 0 ? static_cast<int64_t>(kept_key[i - 1]) >> node_bits : -1;
  for (int64_t k = before + 1; k <= c && k <= num_cols; ++k) out_indptr[k] = i;
  if (i == kept - 1)
    for (int64_t k = c + 1; k <= num_cols; ++k) out_indptr[k] = kept;
}

// One workgroup per column puts the kept edges of its column in the order of (new row,
// position) -- the order of a stable sort of all kept edges by key, which for a few tens of
// thousands of edges is three radix passes of two launches each -- by a counting sort in LDS:
// a histogram over the 2^node_bits places, its scan, then the edges in their own order, 4096
// at a time: a wave walks them 64 at a time, a lane finds the lanes that hold the same place
// with one ballot per key bit and takes the bin's next free places in lane order; then all
// lanes write row id and value data / divisor[row] to where the edges go.  Work grows with the
// column's length, not its square: the hubs among a layer's seeds keep tens of thousands of
// edges (parallel edges included), most columns a few dozen.  FOUR_WAVES (up to 2048 places):
// each wave walks a quarter of the 4096 and counts per place in 16-bit counters of its own; an
// edge's place is the bin's start + the counts of the quarters before its own + its rank
// inside its quarter.
constexpr int kColumnStage = 4096;
constexpr int kColumnBatch = 4;
constexpr int kFourWavesBits = 11;
constexpr int kRankShift = 13;  // a key has at most 13 bits, a rank inside a quarter 12

constexpr int kShortColumn = 256;

// The columns with more than kShortColumn kept edges, listed for the workgroups that order them
// in LDS (a thread a column).
__global__ void __launch_bounds__(256)
long_columns_kernel(const int64_t* __restrict__ indptr, int64_t num_cols,
                    unsigned int* __restrict__ num_long, unsigned int* __restrict__ long_columns) {
  const int64_t c = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x;
  if (c < num_cols && indptr[c + 1] - indptr[c] > kShortColumn)
    long_columns[atomicAdd(num_long, 1u)] = static_cast<unsigned int>(c);
}

// The short columns (up to 256 kept edges: nearly all of them) by edge: a thread takes one kept
// edge, finds its column's range in the offsets, and counts the column's edges that come before
// its own by (key, position) -- the keys of a column lie side by side and the threads of a
// column read the same ones, out of the caches.  (A workgroup per column, long or short, cost
// 116 us for 82 k edges over 40 k columns: tens of thousands of workgroups with two edges each.)
template <typename IdT>
__device__ __forceinline__ void order_short_edge(int64_t i, const IdT* __restrict__ kept_key,
                                                 const IdT* __restrict__ kept_pos, int node_bits,
                                                 const int64_t* __restrict__ indptr,
                                                 const IdT* __restrict__ row,
                                                 const float* __restrict__ data,
                                                 const float* __restrict__ divisor,
                                                 IdT* __restrict__ out_row,
                                                 float* __restrict__ out_value) {
  const unsigned long long key = static_cast<unsigned long long>(kept_key[i]);
  const int64_t e = static_cast<int64_t>(kept_pos[i]);
  const int64_t column = static_cast<int64_t>(key >> node_bits);
  const int64_t lo = indptr[column], hi = indptr[column + 1];
  if (hi - lo > kShortColumn) return;  // (a long column: its own workgroup's)
  const IdT r = row[e];
  const float w = data ? data[e] : 1.0f;
  const float d = divisor[r];
  int64_t before = 0;
  for (int64_t j = lo; j < hi; ++j) {
    const unsigned long long y = static_cast<unsigned long long>(kept_key[j]);
    before += (y < key) || (y == key && j < i);  // (one column: the keys differ in the place only)
  }
  out_row[lo + before] = r;
  out_value[lo + before] = w / d;
}

template <typename IdT, bool FOUR_WAVES>
__global__ void __launch_bounds__(256)
order_columns_kernel(const IdT* __restrict__ kept_key, const IdT* __restrict__ kept_pos,
                     int node_bits, const int64_t* __restrict__ indptr,
                     const IdT* __restrict__ row, const float* __restrict__ data,
                     const float* __restrict__ divisor, IdT* __restrict__ out_row,
                     float* __restrict__ out_value, const unsigned int* __restrict__ num_long,
                     const unsigned int* __restrict__ long_columns, unsigned int long_blocks,
                     int64_t kept) {
  extern __shared__ unsigned long long s_raw[];
  __shared__ int64_t s_scan[256 / kWave + 1];
  // the launch's first long_blocks workgroups take a listed long column each, the others 256
  // kept edges of short columns: both kinds run side by side
  if (blockIdx.x >= long_blocks) {
    const int64_t i = static_cast<int64_t>(blockIdx.x - long_blocks) * 256 + threadIdx.x;
    if (i < kept)
      order_short_edge(i, kept_key, kept_pos, node_bits, indptr, row, data, divisor, out_row,
                       out_value);
    return;
  }
  if (blockIdx.x >= *num_long) return;
  const unsigned int column = long_columns[blockIdx.x];
  const int64_t lo = indptr[column], hi = indptr[column + 1];
  const int64_t len = hi - lo;
  const int places = 1 << node_bits;
  const unsigned int mask = static_cast<unsigned int>(places) - 1u;
  unsigned int* s_bin = reinterpret_cast<unsigned int*>(s_raw);
  unsigned int* s_key = s_bin + places;
  for (int j = threadIdx.x; j < places; j += 256) s_bin[j] = 0u;
  __syncthreads();
  // (here and below a thread's reads go out four at a time, clamped to the column, before the
  // first of them is used: one at a time each waits a whole trip to memory)
  for (int64_t j0 = threadIdx.x; j0 < len; j0 += 256 * kColumnBatch) {
    unsigned int k[kColumnBatch];
#pragma unroll
    for (int u = 0; u < kColumnBatch; ++u) {
      const int64_t j = j0 + u * 256;
      k[u] = static_cast<unsigned int>(kept_key[lo + (j < len ? j : len - 1)]) & mask;
    }
#pragma unroll
    for (int u = 0; u < kColumnBatch; ++u)
      if (j0 + u * 256 < len) atomicAdd(&s_bin[k[u]], 1u);
  }
  __syncthreads();
  {  // exclusive scan of the bins: a thread owns `per` consecutive ones
    const int per = places > 256 ? places / 256 : 1;
    const int first = threadIdx.x * per;
    int64_t mine = 0;
    for (int u = 0; u < per; ++u)
      if (first + u < places) mine += s_bin[first + u];
    int64_t total;
    int64_t at = block_exclusive_scan<256>(mine, &total, s_scan);
    for (int u = 0; u < per; ++u) {
      if (first + u < places) {
        const unsigned int n = s_bin[first + u];
        s_bin[first + u] = static_cast<unsigned int>(at);
        at += n;
      }
    }
  }
  __syncthreads();
  const int lane = threadIdx.x & (kWave - 1);
  // without data every value is one; the read then goes to a word that is always there
  const bool has_data = data != nullptr;
  const float* values = has_data ? data : divisor;
  for (int64_t base = 0; base < len; base += kColumnStage) {
    const int n = static_cast<int>(len - base < kColumnStage ? len - base : kColumnStage);
    for (int j0 = threadIdx.x; j0 < n; j0 += 256 * kColumnBatch) {
      unsigned int k[kColumnBatch];
#pragma unroll
      for (int u = 0; u < kColumnBatch; ++u) {
        const int j = j0 + u * 256;
        k[u] = static_cast<unsigned int>(kept_key[lo + base + (j < n ? j : n - 1)]) & mask;
      }
#pragma unroll
      for (int u = 0; u < kColumnBatch; ++u)
        if (j0 + u * 256 < n) s_key[j0 + u * 256] = k[u];
    }
    if (FOUR_WAVES) {
      unsigned int* zero = s_key + kColumnStage;  // the four waves' counters: 2 * places words
      for (int j = threadIdx.x; j < 2 * places; j += 256) zero[j] = 0u;
    }
    __syncthreads();
    if (FOUR_WAVES) {
      unsigned short* s_count = reinterpret_cast<unsigned short*>(s_key + kColumnStage);
      const int wave = threadIdx.x / kWave;
      const int quarter = ((n + 4 * kWave - 1) / (4 * kWave)) * kWave;
      const int q_hi = (wave + 1) * quarter < n ? (wave + 1) * quarter : n;
      unsigned short* mine = s_count + wave * places;
      for (int c = wave * quarter; c < q_hi; c += kWave) {
        const bool valid = c + lane < q_hi;
        const unsigned int k = valid ? s_key[c + lane] : 0u;
        unsigned long long peers = __ballot(valid);
        for (int b = 0; b < node_bits; ++b) {
          const bool bit = (k >> b) & 1u;
          const unsigned long long with_bit = __ballot(valid && bit);
          peers &= bit ? with_bit : ~with_bit;
        }
        if (valid) {
          const unsigned int ahead = __popcll(peers & ((1ull << lane) - 1ull));
          const unsigned int start = mine[k];
          s_key[c + lane] = k | ((start + ahead) << kRankShift);
          if (lane == 63 - __clzll(peers))
            mine[k] = static_cast<unsigned short>(start + __popcll(peers));
        }
      }
      __syncthreads();
      for (int j = threadIdx.x; j < n; j += 256) {
        const unsigned int v = s_key[j];
        const unsigned int k = v & ((1u << kRankShift) - 1u);
        unsigned int place = s_bin[k] + (v >> kRankShift);
        const int w = j / quarter;
        for (int before = 0; before < w; ++before) place += s_count[before * places + k];
        s_key[j] = place;
      }
      __syncthreads();
      for (int k = threadIdx.x; k < places; k += 256)
        s_bin[k] += static_cast<unsigned int>(s_count[k]) + s_count[places + k] +
                    s_count[2 * places + k] + s_count[3 * places + k];
    } else if (threadIdx.x < kWave) {
      for (int c = 0; c < n; c += kWave) {
        const bool valid = c + lane < n;
        const unsigned int k = valid ? s_key[c + lane] : 0u;
        unsigned long long peers = __ballot(valid);
        for (int b = 0; b < node_bits; ++b) {
          const bool bit = (k >> b) & 1u;
          const unsigned long long with_bit = __ballot(valid && bit);
          peers &= bit ? with_bit : ~with_bit;
        }
        if (valid) {
          const int ahead = __popcll(peers & ((1ull << lane) - 1ull));
          const unsigned int start = s_bin[k];
          s_key[c + lane] = start + static_cast<unsigned int>(ahead);  // the edge's place
          if (lane == 63 - __clzll(peers)) s_bin[k] = start + static_cast<unsigned int>(__popcll(peers));
        }
      }
    }
    __syncthreads();
    for (int j0 = threadIdx.x; j0 < n; j0 += 256 * kColumnBatch) {
      int64_t e[kColumnBatch];
      IdT r[kColumnBatch];
      float w[kColumnBatch], d[kColumnBatch];
#pragma unroll
      for (int u = 0; u < kColumnBatch; ++u) {
        const int j = j0 + u * 256;
        e[u] = static_cast<int64_t>(kept_pos[lo + base + (j < n ? j : n - 1)]);
      }
#pragma unroll
      for (int u = 0; u < kColumnBatch; ++u) r[u] = row[e[u]];
#pragma unroll
      for (int u = 0; u < kColumnBatch; ++u) {
        w[u] = values[has_data ? e[u] : 0];
        d[u] = divisor[r[u]];
      }
#pragma unroll
      for (int u = 0; u < kColumnBatch; ++u) {
        const int j = j0 + u * 256;
        if (j < n) {
          const int64_t dst = lo + s_key[j];
          out_row[dst] = r[u];
          out_value[dst] = (has_data ? w[u] : 1.0f) / d[u];
        }
      }
    }
    __syncthreads();
  }
}

template <typename IdT>
void order_columns_launch(int64_t num_cols, int64_t kept, int node_bits, hipStream_t st,
                          const void* kept_key, const void* kept_pos, const int64_t* indptr,
                          const void* row, const float* data, const float* divisor, void* out_row,
                          float* out_value, unsigned int* num_long, unsigned int* long_columns) {
  hipLaunchKernelGGL(long_columns_kernel, dim3(static_cast<unsigned>(blocks_for(num_cols, 256))),
                     dim3(256), 0, st, indptr, num_cols, num_long, long_columns);
  // at most kept / 257 columns are long
  const unsigned int long_blocks = static_cast<unsigned int>(kept / (kShortColumn + 1) + 1);
  const dim3 grid(long_blocks + static_cast<unsigned>(blocks_for(kept, 256)));
  const size_t places = size_t(1) << node_bits;
  if (node_bits <= kFourWavesBits)
    hipLaunchKernelGGL((order_columns_kernel<IdT, true>), grid, dim3(256),
                       (places + kColumnStage + 2 * places) * sizeof(unsigned int), st,
                       static_cast<const IdT*>(kept_key), static_cast<const IdT*>(kept_pos), node_bits,
                       indptr, static_cast<const IdT*>(row), data, divisor,
                       static_cast<IdT*>(out_row), out_value, num_long, long_columns, long_blocks,
                       kept);
  else
    hipLaunchKernelGGL((order_columns_kernel<IdT, false>), grid, dim3(256),
                       (places + kColumnStage) * sizeof(unsigned int), st,
                       static_cast<const IdT*>(kept_key), static_cast<const IdT*>(kept_pos), node_bits,
                       indptr, static_cast<const IdT*>(row), data, divisor,
                       static_cast<IdT*>(out_row), out_value, num_long, long_columns, long_blocks,
                       kept);
}

inline int bits_of(int64_t n) {  // smallest b with 2^b >= n
  int b = 0;
  while ((int64_t(1) << b) < n) ++b;
  return b;
}

template <typename IdT>
int sorted_union_t(const void* a, int64_t na, const void* b, int64_t nb, void* out, int64_t* count,
                   hipStream_t st) {
  int slots = 1 << bits_of(na + nb);
  if (slots < 2) slots = 2;
  const size_t keys = static_cast<size_t>(slots);
  hipLaunchKernelGGL(sorted_union_kernel<IdT>, dim3(1), dim3(kUnionThreads),
                     ((keys * sizeof(IdT) + 7) / 8) * 8, st,
                     static_cast<const IdT*>(a), na, static_cast<const IdT*>(b), nb, slots,
                     static_cast<IdT*>(out), count);
  return check_launch("sorted_union");
}

template <typename IdT>
int pick_rows_t(const void* row, const void* col, int64_t E, const void* nodes,
                const int64_t* num_nodes, int max_nodes, void* kept_key, void* kept_pos,
                int64_t* totals, gs_mailbox* box, int64_t ticket, void* workspace,
                size_t workspace_bytes, hipStream_t st) {
  const int64_t tiles = blocks_for(E, kPickTile);
  Carver ws(workspace, workspace_bytes);
  int64_t* counts = ws.take<int64_t>(tiles);
  int64_t* offsets = ws.take<int64_t>(tiles + 1);
  int64_t* scan_ws = ws.take<int64_t>(scan_num_tiles(tiles) + 1);
  int* place = ws.take<int>(E);
  if (!ws.ok) {
    set_error_text("gs_coo_pick_rows: workspace needs %zu bytes, 256-byte aligned",
                   gs_coo_pick_rows_workspace_bytes(E));
    return GS_ERR_WORKSPACE;
  }
  const int node_bits = bits_of(max_nodes);
  const size_t lds = ((static_cast<size_t>(max_nodes) * sizeof(IdT) + 7) / 8) * 8;
  const dim3 grid(static_cast<unsigned>(tiles));
  hipLaunchKernelGGL(pick_count_kernel<IdT>, grid, dim3(kPickThreads), lds, st,
                     static_cast<const IdT*>(row), E, static_cast<const IdT*>(nodes), num_nodes,
                     max_nodes, place, counts);
  LoadCounts f{counts};
  GS_RETURN_IF_ERROR(exclusive_scan(f, tiles, offsets, scan_ws, st));
  hipLaunchKernelGGL(pick_fill_kernel<IdT>, grid, dim3(kPickThreads), 0, st,
                     static_cast<const int*>(place), static_cast<const IdT*>(col), E, node_bits,
                     static_cast<const int64_t*>(offsets), tiles, num_nodes,
                     static_cast<IdT*>(kept_key), static_cast<IdT*>(kept_pos), totals, box, ticket);
  return check_launch("coo_pick_rows");
}

}  // namespace
}  // namespace gs

using namespace gs;

extern "C" {

int gs_sorted_union(const void* a, int64_t na, const void* b, int64_t nb, int id_bytes, void* out,
                    int64_t* count, void* stream) {
  GS_REQUIRE(na >= 0 && nb >= 0 && na + nb >= 1 && na + nb <= gs_sorted_union_max(id_bytes),
             "gs_sorted_union: %lld + %lld values, takes 1 to %lld",
             static_cast<long long>(na), static_cast<long long>(nb),
             static_cast<long long>(gs_sorted_union_max(id_bytes)));
  GS_REQUIRE((na == 0 || a) && (nb == 0 || b) && out && count, "gs_sorted_union: null pointer");
  GS_REQUIRE(valid_id_bytes(id_bytes), "gs_sorted_union: id_bytes must be 4 or 8, got %d", id_bytes);
  hipStream_t st = static_cast<hipStream_t>(stream);
  return id_bytes == 8 ? sorted_union_t<int64_t>(a, na, b, nb, out, count, st)
                       : sorted_union_t<int32_t>(a, na, b, nb, out, count, st);
}

int64_t gs_sorted_union_max(int id_bytes) { return id_bytes == 8 ? 4096 : 8192; }

size_t gs_coo_pick_rows_workspace_bytes(int64_t E) {
  const int64_t tiles = blocks_for(E, kPickTile);
  auto pad = [](size_t b) { return (b + 255u) & ~size_t(255); };
  return pad(tiles * 8) + pad((tiles + 1) * 8) + pad((scan_num_tiles(tiles) + 1) * 8) +
         pad(static_cast<size_t>(E < 1 ? 1 : E) * sizeof(int));
}

int gs_coo_pick_rows(const void* row, const void* col, int id_bytes, int64_t E, const void* nodes,
                     const int64_t* num_nodes, int64_t max_nodes, void* kept_key, void* kept_pos,
                     int64_t* totals, gs_mailbox* mailbox, int64_t ticket, void* workspace,
                     size_t workspace_bytes, void* stream) {
  GS_REQUIRE(valid_id_bytes(id_bytes), "gs_coo_pick_rows: id_bytes must be 4 or 8, got %d", id_bytes);
  GS_REQUIRE(E >= 1 && (id_bytes == 8 || E < (int64_t(1) << 31)),
             "gs_coo_pick_rows: %lld edges (at least one; below 2^31 with 4-byte ids)",
             static_cast<long long>(E));
  GS_REQUIRE(max_nodes >= 1 && max_nodes <= gs_sorted_union_max(id_bytes),
             "gs_coo_pick_rows: room for %lld nodes, takes 1 to %lld",
             static_cast<long long>(max_nodes), static_cast<long long>(gs_sorted_union_max(id_bytes)));
  GS_REQUIRE(row && col && nodes && num_nodes && kept_key && kept_pos && totals,
             "gs_coo_pick_rows: null pointer");
  hipStream_t st = static_cast<hipStream_t>(stream);
  const int n = static_cast<int>(max_nodes);
  return id_bytes == 8 ? pick_rows_t<int64_t>(row, col, E, nodes, num_nodes, n, kept_key, kept_pos,
                                              totals, mailbox, ticket, workspace, workspace_bytes, st)
                       : pick_rows_t<int32_t>(row, col, E, nodes, num_nodes, n, kept_key, kept_pos,
                                              totals, mailbox, ticket, workspace, workspace_bytes, st);
}

size_t gs_coo_block_values_workspace_bytes(int64_t kept) {
  if (kept < 0) kept = 0;
  return 256 + ((static_cast<size_t>(kept / (kShortColumn + 1) + 1) * sizeof(unsigned int) + 255u) &
                ~size_t(255));
}

int gs_coo_block_values(const void* kept_key, const void* kept_pos, int64_t kept, int64_t max_nodes,
                        const void* row, int id_bytes, const float* data, const float* divisor,
                        int64_t num_cols, void* out_row, float* out_value, int64_t* out_indptr,
                        void* workspace, size_t workspace_bytes, void* stream) {
  GS_REQUIRE(valid_id_bytes(id_bytes), "gs_coo_block_values: id_bytes must be 4 or 8, got %d",
             id_bytes);
  GS_REQUIRE(kept >= 0 && num_cols >= 0, "gs_coo_block_values: negative size");
  GS_REQUIRE(max_nodes >= 1 && max_nodes <= gs_sorted_union_max(id_bytes),
             "gs_coo_block_values: room for %lld nodes, takes 1 to %lld",
             static_cast<long long>(max_nodes), static_cast<long long>(gs_sorted_union_max(id_bytes)));
  GS_REQUIRE(out_indptr && (kept == 0 || (kept_key && kept_pos && row && divisor && out_row && out_value)),
             "gs_coo_block_values: null pointer");
  Carver ws(workspace, workspace_bytes);
  unsigned int* num_long = ws.take<unsigned int>(1);
  unsigned int* long_columns = ws.take<unsigned int>(static_cast<size_t>(kept / (kShortColumn + 1) + 1));
  if (!ws.ok) {
    set_error_text("gs_coo_block_values: workspace needs %zu bytes, 256-byte aligned",
                   gs_coo_block_values_workspace_bytes(kept));
    return GS_ERR_WORKSPACE;
  }
  hipStream_t st = static_cast<hipStream_t>(stream);
  const int node_bits = bits_of(max_nodes);
  const dim3 by_edge(static_cast<unsigned>(blocks_for(kept, 256)));
  if (id_bytes == 8) {
    hipLaunchKernelGGL(column_offsets_kernel<int64_t>, by_edge, dim3(256), 0, st,
                       static_cast<const int64_t*>(kept_key), kept, node_bits, num_cols, out_indptr,
                       num_long);
    if (kept > 0 && num_cols > 0)
      order_columns_launch<int64_t>(num_cols, kept, node_bits, st, kept_key, kept_pos, out_indptr, row,
                                    data, divisor, out_row, out_value, num_long, long_columns);
  } else {
    hipLaunchKernelGGL(column_offsets_kernel<int32_t>, by_edge, dim3(256), 0, st,
                       static_cast<const int32_t*>(kept_key), kept, node_bits, num_cols, out_indptr,
                       num_long);
    if (kept > 0 && num_cols > 0)
      order_columns_launch<int32_t>(num_cols, kept, node_bits, st, kept_key, kept_pos, out_indptr, row,
                                    data, divisor, out_row, out_value, num_long, long_columns);
  }
  return check_launch("coo_block_values");
}

}  // extern "C"
