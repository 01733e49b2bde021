// Row slicing (keep the edges whose row id is in a given set) on gfx950.
//
// Replaces impl::CSCRowSlicingCUDA and impl::COORowSlicingCUDA (reference
// src/cuda/slicing.cu:528,768; node-set table NodeQueryHashmap :40-97).  Kept
// ids are relabelled to their position in `ids` (slicing.cu:477-480).
//
// Mark:    id-set table (capacity 2 * pow2 > n, as slicing.cu:468; Fibonacci
//          hashing instead of Hash64Shift) -> val[e] = position or -1
//          -> prefix = exclusive scan of (val >= 0).  For the CSC flavour the
//          new offsets are simply prefix[indptr[c]]: no per-column count pass,
//          no warp reduction (slicing.cu:463-466), no torch::nonzero.
// Compact: survivors are written in edge order from (val, prefix); the owning
//          column of an edge is found like in the CSC -> COO expansion.
// When `ids` holds duplicates the reference keeps whichever store lands last
// (slicing.cu:56); here the largest position wins (atomicMax), deterministically.
#include "gs_common.hpp"

namespace gs {
namespace {

constexpr int kThreads = 256;
constexpr int kItems = 8;
constexpr int kTile = kThreads * kItems;
constexpr int kStage = 1024;

struct IdSet {
  long long* keys;  // -1 empty
  long long* vals;
  uint32_t mask;
  int shift;
  __device__ __forceinline__ uint32_t home(long long key) const {
    return static_cast<uint32_t>((static_cast<uint64_t>(key) * 0x9E3779B97F4A7C15ull) >> shift);
  }
  __device__ __forceinline__ int64_t query(long long key) const {
    uint32_t p = home(key);
    while (true) {
      const long long cur = keys[p];
      if (cur == key) return vals[p];
      if (cur == -1) return -1;
      p = (p + 1) & mask;
    }
  }
};

int64_t set_capacity(int64_t n) {
  int64_t cap = 1024;
  while (cap < 2 * n + 2) cap <<= 1;
  return cap;
}

__global__ void __launch_bounds__(kThreads) set_init_kernel(IdSet t, int64_t cap) {
  const int64_t i = static_cast<int64_t>(blockIdx.x) * kThreads + threadIdx.x;
  if (i < cap) {
    t.keys[i] = -1;
    t.vals[i] = -1;
  }
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
        atomicCAS(reinterpret_cast<unsigned long long*>(&t.keys[p]), ~0ull,
                  static_cast<unsigned long long>(key));
    if (prev == ~0ull || prev == static_cast<unsigned long long>(key)) break;
    p = (p + 1) & t.mask;
  }
  atomicMax(&t.vals[p], static_cast<long long>(i));
}

template <typename IdT>
__global__ void __launch_bounds__(kThreads)
mark_kernel(IdSet t, const IdT* __restrict__ key, int64_t E, int64_t* __restrict__ val) {
  const int64_t e = static_cast<int64_t>(blockIdx.x) * kThreads + threadIdx.x;
  if (e < E) val[e] = t.query(static_cast<long long>(key[e]));
}

struct Kept {
  const int64_t* val;
  __device__ __forceinline__ int64_t operator()(int64_t e) const { return val[e] >= 0 ? 1 : 0; }
};

__global__ void __launch_bounds__(kThreads)
new_indptr_kernel(const int64_t* __restrict__ indptr, int64_t num_cols,
                  const int64_t* __restrict__ prefix, int64_t* __restrict__ out_indptr) {
  const int64_t c = static_cast<int64_t>(blockIdx.x) * kThreads + threadIdx.x;
  if (c <= num_cols) out_indptr[c] = prefix[indptr[c]];
}

__global__ void __launch_bounds__(kThreads)
copy_total_kernel(const int64_t* __restrict__ prefix, int64_t E, int64_t* __restrict__ total) {
  if (threadIdx.x == 0 && blockIdx.x == 0) *total = prefix[E];
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

// CSC compaction; a workgroup owns 2048 consecutive input edges.
template <bool WITH_COO, typename IdT>
__global__ void __launch_bounds__(kThreads)
csc_compact_kernel(const int64_t* __restrict__ indptr, int64_t num_cols, int64_t nnz,
                   const int64_t* __restrict__ val, const int64_t* __restrict__ prefix,
                   IdT* __restrict__ out_indices, int64_t* __restrict__ select_index,
                   IdT* __restrict__ coo_col) {
  __shared__ int64_t s_ptr[kStage + 1];
  __shared__ int64_t s_rows[2];
  const int64_t p0 = static_cast<int64_t>(blockIdx.x) * kTile;
  const int64_t p1 = p0 + kTile < nnz ? p0 + kTile : nnz;
  int64_t row_lo = 0, nrows = 0;
  bool staged = false;
  if (WITH_COO) {
    if (threadIdx.x < 2)
      s_rows[threadIdx.x] = upper_bound(indptr, num_cols + 1, threadIdx.x == 0 ? p0 : p1 - 1) - 1;
    __syncthreads();
    row_lo = s_rows[0];
    nrows = s_rows[1] - row_lo + 1;
    staged = nrows <= kStage;
    if (staged)
      for (int64_t i = threadIdx.x; i <= nrows; i += kThreads) s_ptr[i] = indptr[row_lo + i];
    __syncthreads();
  }
#pragma unroll
  for (int k = 0; k < kItems; ++k) {
    const int64_t e = p0 + k * kThreads + threadIdx.x;
    if (e >= p1) break;
    const int64_t v = val[e];
    if (v < 0) continue;
    const int64_t w = prefix[e];
    out_indices[w] = static_cast<IdT>(v);
    select_index[w] = e;
    if (WITH_COO)
      coo_col[w] = static_cast<IdT>(row_lo + (staged ? upper_bound(s_ptr, nrows + 1, e)
                                                     : upper_bound(indptr + row_lo, nrows + 1, e)) - 1);
  }
}

template <typename IdT>
__global__ void __launch_bounds__(kThreads)
coo_compact_kernel(const IdT* __restrict__ other, int64_t E, const int64_t* __restrict__ val,
                   const int64_t* __restrict__ prefix, IdT* __restrict__ out_key,
                   IdT* __restrict__ out_other, int64_t* __restrict__ select_index) {
  const int64_t e = static_cast<int64_t>(blockIdx.x) * kThreads + threadIdx.x;
  if (e >= E) return;
  const int64_t v = val[e];
  if (v < 0) return;
  const int64_t w = prefix[e];
  out_key[w] = static_cast<IdT>(v);
  out_other[w] = other[e];
  select_index[w] = e;
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
  const int64_t i = static_cast<int64_t>(blockIdx.x) * kThreads + threadIdx.x;
  if (i >= n) return;
  const int64_t b = upper_bound(id_ptr, B + 1, i) - 1;
  if (b < 0 || b >= B) return;
  const long long id = static_cast<long long>(ids[i]);
  const long long key = id + b * enc;
  if (key == -1) return;
  uint32_t p = t.home(key);
  while (true) {
    const unsigned long long prev =
        atomicCAS(reinterpret_cast<unsigned long long*>(&t.keys[p]), ~0ull,
                  static_cast<unsigned long long>(key));
    if (prev == ~0ull || prev == static_cast<unsigned long long>(key)) break;
    p = (p + 1) & t.mask;
  }
  atomicMax(&t.vals[p], id);
}

template <typename IdT>
__global__ void __launch_bounds__(kThreads)
sliced_mark_kernel(IdSet t, const int64_t* __restrict__ indptr, const IdT* __restrict__ indices,
                   const IdT* __restrict__ cols, int64_t S, const int64_t* __restrict__ sub_indptr,
                   int64_t D, const int64_t* __restrict__ col_ptr, int64_t B, int64_t enc,
                   int64_t* __restrict__ val, int64_t* __restrict__ src) {
  __shared__ int64_t s_ptr[kStage + 1];
  __shared__ int64_t s_rows[2];
  const int64_t p0 = static_cast<int64_t>(blockIdx.x) * kTile;
  const int64_t p1 = p0 + kTile < D ? p0 + kTile : D;
  if (threadIdx.x < 2)
    s_rows[threadIdx.x] = upper_bound(sub_indptr, S + 1, threadIdx.x == 0 ? p0 : p1 - 1) - 1;
  __syncthreads();
  const int64_t row_lo = s_rows[0];
  const int64_t nrows = s_rows[1] - row_lo + 1;
  const bool staged = nrows <= kStage;
  if (staged)
    for (int64_t i = threadIdx.x; i <= nrows; i += kThreads) s_ptr[i] = sub_indptr[row_lo + i];
  __syncthreads();
#pragma unroll
  for (int k = 0; k < kItems; ++k) {
    const int64_t p = p0 + k * kThreads + threadIdx.x;
    if (p >= p1) break;
    const int64_t lr = (staged ? upper_bound(s_ptr, nrows + 1, p)
                               : upper_bound(sub_indptr + row_lo, nrows + 1, p)) - 1;
    const int64_t r = row_lo + lr;
    const int64_t first = staged ? s_ptr[lr] : sub_indptr[r];
    // a column that owns a position of the slice has passed the range check of the count
    const int64_t c = static_cast<int64_t>(cols[r]);
    const int64_t q = indptr[c] + (p - first);
    const long long id = static_cast<long long>(indices[q]);
    src[p] = q;
    if (B > 0) {
      const int64_t b = upper_bound(col_ptr, B + 1, r) - 1;
      val[p] = (b >= 0 && b < B && t.query(id + b * enc) >= 0) ? id : -1;
    } else {
      val[p] = t.query(id);
    }
  }
}

__global__ void __launch_bounds__(kThreads)
sliced_indptr_kernel(const int64_t* __restrict__ sub_indptr, int64_t S,
                     const int64_t* __restrict__ prefix, int64_t* __restrict__ out_indptr) {
  const int64_t r = static_cast<int64_t>(blockIdx.x) * kThreads + threadIdx.x;
  if (r <= S) out_indptr[r] = prefix[sub_indptr[r]];
}

template <typename IdT>
__global__ void __launch_bounds__(kThreads)
sliced_compact_kernel(int64_t D, const int64_t* __restrict__ val, const int64_t* __restrict__ prefix,
                      const int64_t* __restrict__ src, IdT* __restrict__ out_indices,
                      int64_t* __restrict__ select_index, int64_t* __restrict__ parent_index) {
  const int64_t p = static_cast<int64_t>(blockIdx.x) * kThreads + threadIdx.x;
  if (p >= D) return;
  const int64_t v = val[p];
  if (v < 0) return;
  const int64_t w = prefix[p];
  out_indices[w] = static_cast<IdT>(v);
  if (select_index) select_index[w] = p;
  if (parent_index) parent_index[w] = src[p];
}

// ------------------------------------------------- batched membership filter ----
// Edge e belongs to the batch whose range of key_ptr holds e; it survives when key[e] is
// among the ids of the same batch.  Replaces the per-batch tables of
// impl::BatchCOOSlicingCUDA / BatchCOORowSlicingCUDA (reference src/cuda/batch_slicing.cu:
// 150-232, src/cuda/slicing.cu:659-770) by one table keyed with id + (batch << 44).
constexpr int kBatchShift = 44;

template <typename IdT>
__global__ void __launch_bounds__(kThreads)
mark_batched_kernel(IdSet t, const IdT* __restrict__ key, int64_t E,
                    const int64_t* __restrict__ key_ptr, int64_t B, int64_t* __restrict__ val) {
  const int64_t e = static_cast<int64_t>(blockIdx.x) * kThreads + threadIdx.x;
  if (e >= E) return;
  const int64_t b = upper_bound(key_ptr, B + 1, e) - 1;
  val[e] = (b >= 0 && b < B)
               ? t.query(static_cast<long long>(key[e]) + (static_cast<long long>(b) << kBatchShift))
               : -1;
}

template <typename IdT>
__global__ void __launch_bounds__(kThreads)
filter_compact_kernel(const IdT* __restrict__ row, const IdT* __restrict__ col, int64_t E,
                      const int64_t* __restrict__ val, const int64_t* __restrict__ prefix,
                      IdT* __restrict__ out_row, IdT* __restrict__ out_col,
                      int64_t* __restrict__ select_index) {
  const int64_t e = static_cast<int64_t>(blockIdx.x) * kThreads + threadIdx.x;
  if (e >= E || val[e] < 0) return;
  const int64_t w = prefix[e];
  out_row[w] = row[e];
  out_col[w] = col[e];
  if (select_index) select_index[w] = e;
}

__global__ void __launch_bounds__(kThreads)
filter_batch_ptr_kernel(const int64_t* __restrict__ key_ptr, int64_t B,
                        const int64_t* __restrict__ prefix, int64_t* __restrict__ out_ptr) {
  const int64_t b = static_cast<int64_t>(blockIdx.x) * kThreads + threadIdx.x;
  if (b <= B) out_ptr[b] = prefix[key_ptr[b]];
}

// position of each key in `data` (-1 when absent): impl::IndexHashMapInsertCUDA +
// IndexHashMapSearchCUDA (reference src/cuda/index_search.cu:83-140)
template <typename IdT>
__global__ void __launch_bounds__(kThreads)
search_kernel(IdSet t, const IdT* __restrict__ keys, int64_t m, IdT* __restrict__ out) {
  const int64_t i = static_cast<int64_t>(blockIdx.x) * kThreads + threadIdx.x;
  if (i < m) out[i] = static_cast<IdT>(t.query(static_cast<long long>(keys[i])));
}

// Workspace layout: [val | prefix | scan tiles | (parent positions) | id-set].  All but
// the last depend on the edge count only, so the compact call finds them again without
// knowing how many ids the mark call was given.
struct Scratch {
  IdSet set;
  int64_t cap;
  int64_t* val;
  int64_t* prefix;
  int64_t* tiles;
  int64_t* src;
  bool ok;
};

Scratch carve(void* workspace, size_t bytes, int64_t n_ids, int64_t E, bool with_set,
              bool with_src = false) {
  Scratch s;
  Carver ws(workspace, bytes);
  s.val = ws.take<int64_t>(E > 0 ? E : 1);
  s.prefix = ws.take<int64_t>(E + 1);
  s.tiles = ws.take<int64_t>(scan_num_tiles(E) + 1);
  s.src = with_src ? ws.take<int64_t>(E > 0 ? E : 1) : nullptr;
  s.cap = 0;
  if (with_set) {
    s.cap = set_capacity(n_ids);
    s.set.keys = ws.take<long long>(s.cap);
    s.set.vals = ws.take<long long>(s.cap);
    s.set.mask = static_cast<uint32_t>(s.cap - 1);
    int lg = 0;
    while ((int64_t(1) << lg) < s.cap) ++lg;
    s.set.shift = 64 - lg;
  }
  s.ok = ws.ok;
  return s;
}

template <typename IdT>
int mark_common(const char* who, const void* key, int64_t E, const void* ids, int64_t n_ids,
                Scratch& s, hipStream_t st) {
  hipLaunchKernelGGL(set_init_kernel, dim3(blocks_for(s.cap, kThreads)), dim3(kThreads), 0, st,
                     s.set, s.cap);
  if (n_ids > 0)
    hipLaunchKernelGGL(set_insert_kernel<IdT>, dim3(blocks_for(n_ids, kThreads)), dim3(kThreads), 0,
                       st, s.set, static_cast<const IdT*>(ids), n_ids);
  if (E > 0)
    hipLaunchKernelGGL(mark_kernel<IdT>, dim3(blocks_for(E, kThreads)), dim3(kThreads), 0, st, s.set,
                       static_cast<const IdT*>(key), E, s.val);
  GS_RETURN_IF_ERROR(check_launch(who));
  Kept f{s.val};
  return exclusive_scan(f, E, s.prefix, s.tiles, st);
}

}  // namespace
}  // namespace gs

using namespace gs;

extern "C" {

size_t gs_row_slice_workspace_bytes(int64_t num_row_ids, int64_t nnz, int64_t num_cols) {
  (void)num_cols;
  if (num_row_ids < 0) num_row_ids = 0;
  if (nnz < 0) nnz = 0;
  const int64_t cap = set_capacity(num_row_ids);
  return 2 * padded(cap * 8) + padded((nnz > 0 ? nnz : 1) * 8) + padded((nnz + 1) * 8) +
         scan_workspace_bytes(nnz);
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
  Scratch s = carve(workspace, workspace_bytes, num_row_ids, nnz, true);
  if (!s.ok) {
    set_error_text("gs_row_slice_csc_mark: workspace needs %zu bytes, 256-byte aligned",
                   gs_row_slice_workspace_bytes(num_row_ids, nnz, num_cols));
    return GS_ERR_WORKSPACE;
  }
  hipStream_t st = static_cast<hipStream_t>(stream);
  GS_RETURN_IF_ERROR(id_bytes == 8 ? mark_common<int64_t>("row_slice_csc_mark", indices, nnz, row_ids,
                                                          num_row_ids, s, st)
                                   : mark_common<int32_t>("row_slice_csc_mark", indices, nnz, row_ids,
                                                          num_row_ids, s, st));
  hipLaunchKernelGGL(new_indptr_kernel, dim3(blocks_for(num_cols + 1, kThreads)), dim3(kThreads), 0,
                     st, indptr, num_cols, s.prefix, out_indptr);
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
  Scratch s = carve(workspace, workspace_bytes, 0, nnz, false);
  if (!s.ok) {
    set_error_text("gs_row_slice_csc_compact: pass the workspace given to gs_row_slice_csc_mark");
    return GS_ERR_WORKSPACE;
  }
  hipStream_t st = static_cast<hipStream_t>(stream);
  const dim3 grid(blocks_for(nnz, kTile));
  if (id_bytes == 8) {
    int64_t* oi = static_cast<int64_t*>(out_indices);
    int64_t* cc = static_cast<int64_t*>(coo_col);
    if (coo_col)
      hipLaunchKernelGGL((csc_compact_kernel<true, int64_t>), grid, dim3(kThreads), 0, st, indptr,
                         num_cols, nnz, s.val, s.prefix, oi, select_index, cc);
    else
      hipLaunchKernelGGL((csc_compact_kernel<false, int64_t>), grid, dim3(kThreads), 0, st, indptr,
                         num_cols, nnz, s.val, s.prefix, oi, select_index, cc);
  } else {
    int32_t* oi = static_cast<int32_t*>(out_indices);
    int32_t* cc = static_cast<int32_t*>(coo_col);
    if (coo_col)
      hipLaunchKernelGGL((csc_compact_kernel<true, int32_t>), grid, dim3(kThreads), 0, st, indptr,
                         num_cols, nnz, s.val, s.prefix, oi, select_index, cc);
    else
      hipLaunchKernelGGL((csc_compact_kernel<false, int32_t>), grid, dim3(kThreads), 0, st, indptr,
                         num_cols, nnz, s.val, s.prefix, oi, select_index, cc);
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
  Scratch s = carve(workspace, workspace_bytes, num_ids, E, true);
  if (!s.ok) {
    set_error_text("gs_row_slice_coo_mark: workspace needs %zu bytes, 256-byte aligned",
                   gs_row_slice_workspace_bytes(num_ids, E, 0));
    return GS_ERR_WORKSPACE;
  }
  hipStream_t st = static_cast<hipStream_t>(stream);
  GS_RETURN_IF_ERROR(id_bytes == 8
                         ? mark_common<int64_t>("row_slice_coo_mark", key, E, ids, num_ids, s, st)
                         : mark_common<int32_t>("row_slice_coo_mark", key, E, ids, num_ids, s, st));
  hipLaunchKernelGGL(copy_total_kernel, dim3(1), dim3(64), 0, st, s.prefix, E, num_kept);
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
  Scratch s = carve(workspace, workspace_bytes, 0, E, false);
  if (!s.ok) {
    set_error_text("gs_row_slice_coo_compact: pass the workspace given to gs_row_slice_coo_mark");
    return GS_ERR_WORKSPACE;
  }
  hipStream_t st = static_cast<hipStream_t>(stream);
  const dim3 grid(blocks_for(E, kThreads));
  if (id_bytes == 8)
    hipLaunchKernelGGL(coo_compact_kernel<int64_t>, grid, dim3(kThreads), 0, st,
                       static_cast<const int64_t*>(other), E, s.val, s.prefix,
                       static_cast<int64_t*>(out_key), static_cast<int64_t*>(out_other),
                       select_index);
  else
    hipLaunchKernelGGL(coo_compact_kernel<int32_t>, grid, dim3(kThreads), 0, st,
                       static_cast<const int32_t*>(other), E, s.val, s.prefix,
                       static_cast<int32_t*>(out_key), static_cast<int32_t*>(out_other),
                       select_index);
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
  Scratch s = carve(workspace, workspace_bytes, num_row_ids, D, true, true);
  if (!s.ok) {
    set_error_text("gs_col_row_slice_mark: workspace needs %zu bytes, 256-byte aligned",
                   gs_col_row_slice_workspace_bytes(num_row_ids, D));
    return GS_ERR_WORKSPACE;
  }
  hipStream_t st = static_cast<hipStream_t>(stream);
  hipLaunchKernelGGL(set_init_kernel, dim3(blocks_for(s.cap, kThreads)), dim3(kThreads), 0, st,
                     s.set, s.cap);
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
      hipLaunchKernelGGL(sliced_mark_kernel<IdT>, dim3(blocks_for(D, kTile)), dim3(kThreads), 0, st,
                         s.set, indptr, static_cast<const IdT*>(indices),
                         static_cast<const IdT*>(column_ids), S, sub_indptr, D, col_batch_ptr,
                         num_batches, encoding_size, s.val, s.src);
  };
  if (id_bytes == 8) run(int64_t{}); else run(int32_t{});
  GS_RETURN_IF_ERROR(check_launch("col_row_slice_mark"));
  Kept f{s.val};
  GS_RETURN_IF_ERROR(exclusive_scan(f, D, s.prefix, s.tiles, st));
  hipLaunchKernelGGL(sliced_indptr_kernel, dim3(blocks_for(S + 1, kThreads)), dim3(kThreads), 0, st,
                     sub_indptr, S, s.prefix, out_indptr);
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
  Scratch s = carve(workspace, workspace_bytes, 0, D, false, true);
  if (!s.ok) {
    set_error_text("gs_col_row_slice_compact: pass the workspace given to gs_col_row_slice_mark");
    return GS_ERR_WORKSPACE;
  }
  hipStream_t st = static_cast<hipStream_t>(stream);
  const dim3 grid(blocks_for(D, kThreads));
  if (id_bytes == 8)
    hipLaunchKernelGGL(sliced_compact_kernel<int64_t>, grid, dim3(kThreads), 0, st, D, s.val,
                       s.prefix, s.src, static_cast<int64_t*>(out_indices), select_index,
                       parent_index);
  else
    hipLaunchKernelGGL(sliced_compact_kernel<int32_t>, grid, dim3(kThreads), 0, st, D, s.val,
                       s.prefix, s.src, static_cast<int32_t*>(out_indices), select_index,
                       parent_index);
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
  if (num_batches == 0) {
    Scratch s0 = carve(workspace, workspace_bytes, num_ids, E, true);
    if (!s0.ok) {
      set_error_text("gs_coo_filter_mark: workspace needs %zu bytes, 256-byte aligned",
                     gs_row_slice_workspace_bytes(num_ids, E, 0));
      return GS_ERR_WORKSPACE;
    }
    hipStream_t st0 = static_cast<hipStream_t>(stream);
    GS_RETURN_IF_ERROR(id_bytes == 8 ? mark_common<int64_t>("coo_filter_mark", key, E, ids, num_ids,
                                                            s0, st0)
                                     : mark_common<int32_t>("coo_filter_mark", key, E, ids, num_ids,
                                                            s0, st0));
    hipLaunchKernelGGL(copy_total_kernel, dim3(1), dim3(64), 0, st0, s0.prefix, E, num_kept);
    return check_launch("coo_filter_mark");
  }
  Scratch s = carve(workspace, workspace_bytes, num_ids, E, true);
  if (!s.ok) {
    set_error_text("gs_coo_filter_mark: workspace needs %zu bytes, 256-byte aligned",
                   gs_row_slice_workspace_bytes(num_ids, E, 0));
    return GS_ERR_WORKSPACE;
  }
  hipStream_t st = static_cast<hipStream_t>(stream);
  hipLaunchKernelGGL(set_init_kernel, dim3(blocks_for(s.cap, kThreads)), dim3(kThreads), 0, st,
                     s.set, s.cap);
  auto run = [&](auto tag) {
    using IdT = decltype(tag);
    if (num_ids > 0)
      hipLaunchKernelGGL(set_insert_batched_kernel<IdT>, dim3(blocks_for(num_ids, kThreads)),
                         dim3(kThreads), 0, st, s.set, static_cast<const IdT*>(ids), num_ids,
                         ids_batch_ptr, num_batches, int64_t(1) << kBatchShift);
    if (E > 0)
      hipLaunchKernelGGL(mark_batched_kernel<IdT>, dim3(blocks_for(E, kThreads)), dim3(kThreads), 0,
                         st, s.set, static_cast<const IdT*>(key), E, key_batch_ptr, num_batches,
                         s.val);
  };
  if (id_bytes == 8) run(int64_t{}); else run(int32_t{});
  GS_RETURN_IF_ERROR(check_launch("coo_filter_mark"));
  Kept f{s.val};
  GS_RETURN_IF_ERROR(exclusive_scan(f, E, s.prefix, s.tiles, st));
  hipLaunchKernelGGL(copy_total_kernel, dim3(1), dim3(64), 0, st, s.prefix, E, num_kept);
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
  Scratch s = carve(workspace, workspace_bytes, 0, E, false);
  if (!s.ok) {
    set_error_text("gs_coo_filter_compact: pass the workspace given to gs_coo_filter_mark");
    return GS_ERR_WORKSPACE;
  }
  hipStream_t st = static_cast<hipStream_t>(stream);
  if (out_batch_ptr)
    hipLaunchKernelGGL(filter_batch_ptr_kernel, dim3(blocks_for(num_batches + 1, kThreads)),
                       dim3(kThreads), 0, st, key_batch_ptr, num_batches, s.prefix, out_batch_ptr);
  if (E > 0) {
    GS_REQUIRE(row && col && out_row && out_col, "gs_coo_filter_compact: null pointer");
    const dim3 grid(blocks_for(E, kThreads));
    if (id_bytes == 8)
      hipLaunchKernelGGL(filter_compact_kernel<int64_t>, grid, dim3(kThreads), 0, st,
                         static_cast<const int64_t*>(row), static_cast<const int64_t*>(col), E,
                         s.val, s.prefix, static_cast<int64_t*>(out_row),
                         static_cast<int64_t*>(out_col), select_index);
    else
      hipLaunchKernelGGL(filter_compact_kernel<int32_t>, grid, dim3(kThreads), 0, st,
                         static_cast<const int32_t*>(row), static_cast<const int32_t*>(col), E,
                         s.val, s.prefix, static_cast<int32_t*>(out_row),
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
  Scratch s = carve(workspace, workspace_bytes, n, 0, true);
  if (!s.ok) {
    set_error_text("gs_index_search: workspace needs %zu bytes, 256-byte aligned",
                   gs_index_search_workspace_bytes(n));
    return GS_ERR_WORKSPACE;
  }
  hipStream_t st = static_cast<hipStream_t>(stream);
  hipLaunchKernelGGL(set_init_kernel, dim3(blocks_for(s.cap, kThreads)), dim3(kThreads), 0, st,
                     s.set, s.cap);
  auto run = [&](auto tag) {
    using IdT = decltype(tag);
    if (n > 0)
      hipLaunchKernelGGL(set_insert_kernel<IdT>, dim3(blocks_for(n, kThreads)), dim3(kThreads), 0,
                         st, s.set, static_cast<const IdT*>(data), n);
    if (m > 0)
      hipLaunchKernelGGL(search_kernel<IdT>, dim3(blocks_for(m, kThreads)), dim3(kThreads), 0, st,
                         s.set, static_cast<const IdT*>(keys), m, static_cast<IdT*>(out));
  };
  if (id_bytes == 8) run(int64_t{}); else run(int32_t{});
  return check_launch("index_search");
}

}  // extern "C"
