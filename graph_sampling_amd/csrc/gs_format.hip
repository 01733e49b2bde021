// Sparse-format conversion on gfx950: CSC -> COO column expansion and
// COO -> CSC by a stable least-significant-digit radix sort.
//
// Replaces impl::CSC2COOCUDA and impl::COO2CSCCUDA (reference
// src/cuda/format_transform.cu:35,135; the reference leans on cub radix sort,
// whose stability pins the edge order, format_transform.cu:81-100).
//
//  * csc2coo: edge-balanced.  A workgroup owns 4096 consecutive edges, finds the
//    columns they span with two binary searches, lets those columns mark their
//    first edge in LDS and turns the marks into column numbers with a running
//    maximum (the reference runs a full global binary search per edge,
//    format_transform.cu:24-33).
//  * coo2csc: 8-bit digits, only ceil(log2(num_keys)/8) passes
//    (format_transform.cu:58-72 also sorts just the significant bits).  Each
//    pass is histogram -> scan -> stable scatter; the scatter ranks equal digits
//    inside a wave with 8 ballots (no LDS atomics, order preserved) and across
//    waves with a small LDS table.  indptr then comes from one binary search
//    per column in the sorted keys.
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

// A workgroup owns kCooTile consecutive edges.  The columns that start inside the tile mark
// their first edge in LDS (column-parallel, coalesced reads of the offsets; of several empty
// columns at one position the highest wins, which is the owner), and a running maximum
// over the marks gives every edge its column: sixteen consecutive edges per thread, one
// maximum per thread across the workgroup.  No search per edge.
template <typename IdT>
__global__ void __launch_bounds__(kThreads)
csc2coo_kernel(const int64_t* __restrict__ indptr, int64_t num_cols, int64_t nnz,
               const IdT* __restrict__ ids, IdT* __restrict__ col) {
  __shared__ int s_mark[kCooTile];
  __shared__ int64_t s_rows[2];
  __shared__ int s_wave[kThreads / kWave];
  const int64_t p0 = static_cast<int64_t>(blockIdx.x) * kCooTile;
  const int64_t p1 = p0 + kCooTile < nnz ? p0 + kCooTile : nnz;
  if (threadIdx.x < 2)
    s_rows[threadIdx.x] = upper_bound(indptr, num_cols + 1, threadIdx.x == 0 ? p0 : p1 - 1) - 1;
  for (int i = threadIdx.x; i < kCooTile; i += kThreads) s_mark[i] = 0;
  __syncthreads();
  const int64_t row_lo = s_rows[0], row_hi = s_rows[1];
  // columns row_lo + 1 .. row_hi start inside the tile (row_lo holds its first edge)
  for (int64_t r = row_lo + 1 + threadIdx.x; r <= row_hi; r += kThreads)
    atomicMax(&s_mark[indptr[r] - p0], static_cast<int>(r - row_lo));
  __syncthreads();
  const int at0 = threadIdx.x * kCooItems;
  int m[kCooItems];
  int run = 0;
#pragma unroll
  for (int k = 0; k < kCooItems; ++k) {
    const int v = s_mark[at0 + k];
    run = v > run ? v : run;
    m[k] = run;  // relative to what holds where the thread begins
  }
  // exclusive running maximum of the threads' last values
  const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
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
  // column numbers (relative to row_lo) go back into the marks' place, so that the stores
  // below are coalesced whatever the id width
  __syncthreads();
#pragma unroll
  for (int k = 0; k < kCooItems; ++k) s_mark[at0 + k] = m[k] > before ? m[k] : before;
  __syncthreads();
#pragma unroll
  for (int k = 0; k < kCooItems; ++k) {
    const int i = k * kThreads + threadIdx.x;
    const int64_t p = p0 + i;
    if (p < p1) {
      const int64_t c = row_lo + s_mark[i];
      // doubly-compressed: stored column c stands for node ids[c] (format_transform.cu:48-60)
      col[p] = ids ? ids[c] : static_cast<IdT>(c);
    }
  }
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

// indptr from sorted keys: indptr[c] = number of keys < c, one binary search per
// column (format_transform.cu:123-156 does the same).  A boundary-driven fill
// (every edge writes the offsets of the columns between it and its predecessor)
// was tried first and is worse at both ends: with few edges and millions of
// columns one lane fills a gap of a million offsets by itself, with many edges
// and few columns it reads every key to find a handful of boundaries.
template <typename KeyT>
__global__ void __launch_bounds__(kThreads)
indptr_from_sorted_kernel(const KeyT* __restrict__ key, int64_t E, int64_t num_keys,
                          int64_t* __restrict__ indptr) {
  const int64_t c = static_cast<int64_t>(blockIdx.x) * kThreads + threadIdx.x;
  if (c > num_keys) return;
  int64_t lo = 0, hi = E;  // first position whose key is >= c
  while (lo < hi) {
    const int64_t mid = (lo + hi) >> 1;
    if (static_cast<int64_t>(key[mid]) < c) lo = mid + 1; else hi = mid;
  }
  indptr[c] = lo;
}

// ------------------------------------------------------------ radix sort ----
constexpr int kRadixBits = 8;
constexpr int kRadix = 1 << kRadixBits;
constexpr int kWaves = kThreads / kWave;

__device__ __forceinline__ int digit_of(int64_t key, int shift) {
  return static_cast<int>((static_cast<uint64_t>(key) >> shift) & (kRadix - 1));
}

// counts[d * num_blocks + b] = items of tile b with digit d.  KeyT is the
// caller's id type in the first pass and int64 (the ping-pong buffers) after it.
template <typename KeyT>
__global__ void __launch_bounds__(kThreads)
radix_hist_kernel(const KeyT* __restrict__ keys, int64_t E, int shift, int64_t num_blocks,
                  int64_t* __restrict__ counts) {
  __shared__ int s_hist[kRadix];
  s_hist[threadIdx.x] = 0;
  __syncthreads();
  const int64_t base = static_cast<int64_t>(blockIdx.x) * kTile;
#pragma unroll
  for (int k = 0; k < kItems; ++k) {
    const int64_t i = base + k * kThreads + threadIdx.x;
    if (i < E) atomicAdd(&s_hist[digit_of(static_cast<int64_t>(keys[i]), shift)], 1);
  }
  __syncthreads();
  counts[static_cast<int64_t>(threadIdx.x) * num_blocks + blockIdx.x] = s_hist[threadIdx.x];
}

struct LoadI64 {
  const int64_t* p;
  __device__ __forceinline__ int64_t operator()(int64_t i) const { return p[i]; }
};

// Stable scatter of one tile.  Items are visited in index order, 256 per round;
// inside a round the rank of an item among equal digits is (earlier waves'
// count) + (lower lanes of its wave with the same digit).
template <typename KeyT>
__global__ void __launch_bounds__(kThreads)
radix_scatter_kernel(const KeyT* __restrict__ keys_in, const int64_t* __restrict__ perm_in,
                     int64_t E, int shift, int64_t num_blocks, const int64_t* __restrict__ offsets,
                     int64_t* __restrict__ keys_out, int64_t* __restrict__ perm_out) {
  __shared__ int64_t s_base[kRadix];
  __shared__ int s_cnt[kWaves][kRadix];
  const int lane = threadIdx.x & (kWave - 1);
  const int wave = threadIdx.x / kWave;
  s_base[threadIdx.x] = offsets[static_cast<int64_t>(threadIdx.x) * num_blocks + blockIdx.x];
  const int64_t base = static_cast<int64_t>(blockIdx.x) * kTile;
  for (int k = 0; k < kItems; ++k) {
#pragma unroll
    for (int w = 0; w < kWaves; ++w) s_cnt[w][threadIdx.x] = 0;
    __syncthreads();
    const int64_t i = base + k * kThreads + threadIdx.x;
    const bool live = i < E;
    int64_t key = 0;
    int d = 0;
    unsigned long long peers = __ballot(live);
    if (live) {
      key = static_cast<int64_t>(keys_in[i]);
      d = digit_of(key, shift);
    }
#pragma unroll
    for (int b = 0; b < kRadixBits; ++b) {
      const bool bit = (d >> b) & 1;
      const unsigned long long bal = __ballot(live && bit);
      peers &= bit ? bal : ~bal;
    }
    const int rank = __popcll(peers & ((1ull << lane) - 1ull));
    if (live && rank == 0) s_cnt[wave][d] = __popcll(peers);
    __syncthreads();
    if (live) {
      int64_t dst = s_base[d] + rank;
      for (int w = 0; w < wave; ++w) dst += s_cnt[w][d];
      keys_out[dst] = key;
      perm_out[dst] = perm_in ? perm_in[i] : i;
    }
    __syncthreads();
    int add = 0;
#pragma unroll
    for (int w = 0; w < kWaves; ++w) add += s_cnt[w][threadIdx.x];
    s_base[threadIdx.x] += add;
    __syncthreads();
  }
}

template <typename IdT>
__global__ void __launch_bounds__(kThreads)
gather_kernel(const IdT* __restrict__ value, const int64_t* __restrict__ perm, int64_t E,
              IdT* __restrict__ out) {
  const int64_t i = static_cast<int64_t>(blockIdx.x) * kThreads + threadIdx.x;
  if (i < E) out[i] = value[perm[i]];
}

int num_passes(int64_t num_keys) {
  int bits = 0;
  while ((int64_t(1) << bits) < num_keys) ++bits;  // format_transform.cu:58-72
  return (bits + kRadixBits - 1) / kRadixBits;
}

// Offsets of B consecutive column ranges, each re-based to start at 0 and laid
// out one after the other (batch b: offsets[b+1]-offsets[b]+1 entries starting
// at offsets[b] + b).  One output entry per lane, batch by binary search.
__global__ void __launch_bounds__(kThreads)
indptr_split_kernel(const int64_t* __restrict__ indptr, const int64_t* __restrict__ offsets,
                    int64_t B, int64_t total, int64_t* __restrict__ out) {
  const int64_t q = static_cast<int64_t>(blockIdx.x) * kThreads + threadIdx.x;
  if (q >= total) return;
  int64_t lo = 0, hi = B - 1;  // last b with offsets[b] + b <= q
  while (lo < hi) {
    const int64_t mid = (lo + hi + 1) >> 1;
    if (offsets[mid] + mid <= q) lo = mid; else hi = mid - 1;
  }
  const int64_t begin = offsets[lo];
  out[q] = indptr[begin + (q - begin - lo)] - indptr[begin];
}

template <typename IdT>
int coo2csc_impl(const IdT* key, const IdT* value, int64_t E, int64_t num_keys, int sorted,
                 int64_t* indptr, IdT* out_value, int64_t* perm, void* workspace,
                 size_t workspace_bytes, hipStream_t st) {
  if (sorted || E == 0) {
    hipLaunchKernelGGL((indptr_from_sorted_kernel<IdT>), dim3(blocks_for(num_keys + 1, kThreads)),
                       dim3(kThreads), 0, st, key, E, num_keys, indptr);
    return check_launch("coo2csc");
  }
  const int64_t blocks = blocks_for(E, kTile);
  const int64_t table = kRadix * blocks;
  Carver ws(workspace, workspace_bytes);
  int64_t* kbuf[2] = {ws.take<int64_t>(E), ws.take<int64_t>(E)};
  int64_t* pbuf = ws.take<int64_t>(E);
  int64_t* counts = ws.take<int64_t>(table);
  int64_t* offsets = ws.take<int64_t>(table + 1);
  int64_t* tiles = ws.take<int64_t>(scan_num_tiles(table) + 1);
  if (!ws.ok) {
    set_error_text("gs_coo2csc: workspace needs %zu bytes, 256-byte aligned",
                   gs_coo2csc_workspace_bytes(E, num_keys));
    return GS_ERR_WORKSPACE;
  }
  int passes = num_passes(num_keys);
  if (passes == 0) passes = 1;  // one key: still produces perm = identity
  const int64_t* kin = nullptr;  // null: the first pass reads the caller's keys
  const int64_t* pin = nullptr;
  // perm alternates between `perm` and pbuf so that the last pass lands in `perm`
  for (int p = 0; p < passes; ++p) {
    int64_t* kout = kbuf[p & 1];
    int64_t* pout = ((passes - 1 - p) & 1) ? pbuf : perm;
    if (p == 0)
      hipLaunchKernelGGL((radix_hist_kernel<IdT>), dim3(static_cast<unsigned>(blocks)),
                         dim3(kThreads), 0, st, key, E, 0, blocks, counts);
    else
      hipLaunchKernelGGL((radix_hist_kernel<int64_t>), dim3(static_cast<unsigned>(blocks)),
                         dim3(kThreads), 0, st, kin, E, p * kRadixBits, blocks, counts);
    LoadI64 f{counts};
    GS_RETURN_IF_ERROR(exclusive_scan(f, table, offsets, tiles, st));
    if (p == 0)
      hipLaunchKernelGGL((radix_scatter_kernel<IdT>), dim3(static_cast<unsigned>(blocks)),
                         dim3(kThreads), 0, st, key, pin, E, 0, blocks, offsets, kout, pout);
    else
      hipLaunchKernelGGL((radix_scatter_kernel<int64_t>), dim3(static_cast<unsigned>(blocks)),
                         dim3(kThreads), 0, st, kin, pin, E, p * kRadixBits, blocks, offsets, kout,
                         pout);
    kin = kout;
    pin = pout;
  }
  hipLaunchKernelGGL((gather_kernel<IdT>), dim3(blocks_for(E, kThreads)), dim3(kThreads), 0, st,
                     value, perm, E, out_value);
  hipLaunchKernelGGL((indptr_from_sorted_kernel<int64_t>), dim3(blocks_for(num_keys + 1, kThreads)),
                     dim3(kThreads), 0, st, kin, E, num_keys, indptr);
  return check_launch("coo2csc");
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
    hipLaunchKernelGGL((csc2coo_kernel<int64_t>), dim3(blocks_for(nnz, kCooTile)), dim3(kThreads), 0,
                       st, indptr, num_cols, nnz, static_cast<const int64_t*>(nullptr),
                       static_cast<int64_t*>(col));
  else
    hipLaunchKernelGGL((csc2coo_kernel<int32_t>), dim3(blocks_for(nnz, kCooTile)), dim3(kThreads), 0,
                       st, indptr, num_cols, nnz, static_cast<const int32_t*>(nullptr),
                       static_cast<int32_t*>(col));
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
    hipLaunchKernelGGL((csc2coo_kernel<int64_t>), dim3(blocks_for(nnz, kCooTile)), dim3(kThreads), 0,
                       st, indptr, num_cols, nnz, static_cast<const int64_t*>(ids),
                       static_cast<int64_t*>(col));
  else
    hipLaunchKernelGGL((csc2coo_kernel<int32_t>), dim3(blocks_for(nnz, kCooTile)), dim3(kThreads), 0,
                       st, indptr, num_cols, nnz, static_cast<const int32_t*>(ids),
                       static_cast<int32_t*>(col));
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
  const int64_t blocks = blocks_for(E, kTile);
  const int64_t table = kRadix * blocks;
  return 3 * padded(static_cast<size_t>(E > 0 ? E : 1) * 8) +  // keys ping-pong, perm pong
         padded(static_cast<size_t>(table) * 8) + padded(static_cast<size_t>(table + 1) * 8) +
         scan_workspace_bytes(table);
}

int gs_coo2csc(const void* key, const void* value, int id_bytes, int64_t E, int64_t num_keys,
               int sorted, int64_t* indptr, void* out_value, int64_t* perm, void* workspace,
               size_t workspace_bytes, void* stream) {
  GS_REQUIRE(E >= 0 && num_keys >= 0 && indptr, "gs_coo2csc: negative size or null indptr");
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
  GS_REQUIRE(num_batches >= 0 && total >= 0, "gs_indptr_split: negative size");
  if (num_batches == 0 || total == 0) return GS_OK;
  GS_REQUIRE(indptr && offsets && out, "gs_indptr_split: null pointer");
  hipLaunchKernelGGL(indptr_split_kernel, dim3(blocks_for(total, kThreads)), dim3(kThreads), 0,
                     static_cast<hipStream_t>(stream), indptr, offsets, num_batches, total, out);
  return check_launch("indptr_split");
}

}  // extern "C"
