// Unique / relabel on gfx950: an open-addressing hash table in HBM plus an
// ordered (first-occurrence) compaction.
//
// Replaces impl::TensorUniqueCUDA and impl::RelabelCUDA (reference
// src/cuda/unique_reindex.cu:174,179).  The reference's result order is "first
// occurrence in the concatenated mapping tensors" (unique_reindex.cu:106-144),
// independent of the table layout, so the table here is free to differ:
//  * capacity = power of two >= 2 * items (load <= 0.5; the reference runs at
//    0.5..1.0, unique_reindex.cu:74-78), Fibonacci hashing, linear probing
//    (the reference uses the identity hash, which clusters on consecutive ids);
//  * values are int32 and every item remembers its slot (4 B) so later passes
//    never probe again;
//  * the mapping tensors are read in place through a span table -- no
//    concatenated copy is materialised (the reference does torch::cat,
//    unique_reindex.cu:187-190);
//  * a query that aliases a mapping span is relabelled by slot gather.
#include "gs_common.hpp"

namespace gs {
namespace {

constexpr int kThreads = 256;

template <typename IdT>
struct Spans {
  const IdT* ptr[GS_MAX_SPANS];
  int64_t end[GS_MAX_SPANS];  // exclusive end offset of each span in the concatenation
  int n;
  __device__ __forceinline__ IdT get(int64_t i) const {
    int s = 0;
    int64_t begin = 0;
#pragma unroll
    for (int t = 0; t < GS_MAX_SPANS - 1; ++t) {
      if (t < n - 1 && i >= end[t]) {
        s = t + 1;
        begin = end[t];
      }
    }
    return ptr[s][i - begin];
  }
};

struct Table {
  long long* keys;  // -1 = empty
  int* vals;        // min index, later the rank
  uint32_t mask;
  int shift;  // 64 - log2(capacity)
  __device__ __forceinline__ uint32_t home(long long key) const {
    return static_cast<uint32_t>((static_cast<uint64_t>(key) * 0x9E3779B97F4A7C15ull) >> shift);
  }
};

__global__ void __launch_bounds__(kThreads) table_init_kernel(Table t, int64_t cap) {
  const int64_t i = static_cast<int64_t>(blockIdx.x) * kThreads + threadIdx.x;
  if (i < cap) {
    t.keys[i] = -1;
    t.vals[i] = 0x7fffffff;
  }
}

// insert (key -> min index) and remember the slot of every item
// (unique_reindex.cu:92-99, RelabelHashmap::Update :13-26)
template <typename IdT>
__global__ void __launch_bounds__(kThreads)
table_insert_kernel(Spans<IdT> x, int64_t M, Table t, int* __restrict__ pos) {
  const int64_t i = static_cast<int64_t>(blockIdx.x) * kThreads + threadIdx.x;
  if (i >= M) return;
  const long long key = static_cast<long long>(x.get(i));
  uint32_t p = t.home(key);
  while (true) {
    long long cur = __atomic_load_n(&t.keys[p], __ATOMIC_RELAXED);
    if (cur == key) break;
    if (cur == -1) {
      unsigned long long prev =
          atomicCAS(reinterpret_cast<unsigned long long*>(&t.keys[p]), ~0ull,
                    static_cast<unsigned long long>(key));
      if (prev == ~0ull || prev == static_cast<unsigned long long>(key)) break;
    }
    p = (p + 1) & t.mask;
  }
  atomicMin(&t.vals[p], static_cast<int>(i));
  pos[i] = static_cast<int>(p);
}

// 1 when item i is the first occurrence of its key (unique_reindex.cu:106-114)
struct IsFirst {
  const int* vals;
  const int* pos;
  __device__ __forceinline__ int64_t operator()(int64_t i) const {
    return vals[pos[i]] == static_cast<int>(i) ? 1 : 0;
  }
};

// frontier[rank] = key and slot value <- rank (unique_reindex.cu:127-144).  A
// first occurrence i has rank <= i, every later duplicate has index > i, so
// overwriting the slot while others still test `vals == my index` is safe.
template <typename IdT>
__global__ void __launch_bounds__(kThreads)
compact_kernel(Spans<IdT> x, int64_t M, Table t, const int* __restrict__ pos,
               const int64_t* __restrict__ prefix, IdT* __restrict__ frontier,
               int64_t* __restrict__ num_unique) {
  const int64_t i = static_cast<int64_t>(blockIdx.x) * kThreads + threadIdx.x;
  if (i == 0) *num_unique = prefix[M];
  if (i >= M) return;
  const int p = pos[i];
  if (t.vals[p] == static_cast<int>(i)) {
    const int64_t rank = prefix[i];
    frontier[rank] = x.get(i);
    t.vals[p] = static_cast<int>(rank);
  }
}

// out[i] = rank of q[i] (unique_reindex.cu:162-170); alias >= 0: q is the
// mapping span starting at concatenation offset `alias`, so reuse its slots.
template <typename IdT>
__global__ void __launch_bounds__(kThreads)
lookup_kernel(const IdT* __restrict__ q, int64_t n, Table t, const int* __restrict__ pos,
              int64_t alias, IdT* __restrict__ out) {
  const int64_t i = static_cast<int64_t>(blockIdx.x) * kThreads + threadIdx.x;
  if (i >= n) return;
  if (alias >= 0) {
    out[i] = static_cast<IdT>(t.vals[pos[alias + i]]);
    return;
  }
  const long long key = static_cast<long long>(q[i]);
  uint32_t p = t.home(key);
  int r = -1;
  while (true) {
    const long long cur = t.keys[p];
    if (cur == key) {
      r = t.vals[p];
      break;
    }
    if (cur == -1) break;
    p = (p + 1) & t.mask;
  }
  out[i] = static_cast<IdT>(r);
}

int64_t table_capacity(int64_t M) {
  int64_t cap = 1024;
  while (cap < 2 * M) cap <<= 1;
  return cap;
}

template <typename IdT>
int unique_relabel_impl(const gs_span* mapping, int n_mapping, const gs_span* query,
                        void* const* query_out, int n_query, void* frontier, int64_t* num_unique,
                        void* workspace, size_t workspace_bytes, hipStream_t stream) {
  Spans<IdT> x;
  int64_t M = 0;
  for (int s = 0; s < GS_MAX_SPANS; ++s) {
    x.ptr[s] = nullptr;
    x.end[s] = 0;
  }
  for (int s = 0; s < n_mapping; ++s) {
    x.ptr[s] = static_cast<const IdT*>(mapping[s].ptr);
    M += mapping[s].n;
    x.end[s] = M;
  }
  x.n = n_mapping;
  const int64_t cap = table_capacity(M);
  Carver ws(workspace, workspace_bytes);
  Table t;
  t.keys = ws.take<long long>(cap);
  t.vals = ws.take<int>(cap);
  int* pos = ws.take<int>(M > 0 ? M : 1);
  int64_t* prefix = ws.take<int64_t>(M + 1);
  int64_t* tiles = ws.take<int64_t>(scan_num_tiles(M) + 1);
  if (!ws.ok) {
    set_error_text("gs_unique_relabel: workspace needs %zu bytes, 256-byte aligned",
                   gs_unique_workspace_bytes(M));
    return GS_ERR_WORKSPACE;
  }
  t.mask = static_cast<uint32_t>(cap - 1);
  int lg = 0;
  while ((int64_t(1) << lg) < cap) ++lg;
  t.shift = 64 - lg;

  hipLaunchKernelGGL(table_init_kernel, dim3(blocks_for(cap, kThreads)), dim3(kThreads), 0, stream,
                     t, cap);
  if (M > 0)
    hipLaunchKernelGGL((table_insert_kernel<IdT>), dim3(blocks_for(M, kThreads)), dim3(kThreads), 0,
                       stream, x, M, t, pos);
  GS_RETURN_IF_ERROR(check_launch("unique insert"));
  IsFirst f{t.vals, pos};
  GS_RETURN_IF_ERROR(exclusive_scan(f, M, prefix, tiles, stream));
  hipLaunchKernelGGL((compact_kernel<IdT>), dim3(blocks_for(M, kThreads)), dim3(kThreads), 0, stream,
                     x, M, t, pos, prefix, static_cast<IdT*>(frontier), num_unique);
  for (int q = 0; q < n_query; ++q) {
    if (query[q].n == 0) continue;
    int64_t alias = -1, off = 0;
    for (int s = 0; s < n_mapping; ++s) {
      if (mapping[s].ptr == query[q].ptr && mapping[s].n == query[q].n) alias = off;
      off += mapping[s].n;
    }
    hipLaunchKernelGGL((lookup_kernel<IdT>), dim3(blocks_for(query[q].n, kThreads)), dim3(kThreads),
                       0, stream, static_cast<const IdT*>(query[q].ptr), query[q].n, t, pos, alias,
                       static_cast<IdT*>(query_out[q]));
  }
  return check_launch("unique_relabel");
}

}  // namespace
}  // namespace gs

using namespace gs;

extern "C" {

size_t gs_unique_workspace_bytes(int64_t M) {
  if (M < 0) M = 0;
  const int64_t cap = table_capacity(M);
  return padded(cap * 8) + padded(cap * 4) + padded((M > 0 ? M : 1) * 4) + padded((M + 1) * 8) +
         scan_workspace_bytes(M);
}

int gs_unique_relabel(const gs_span* mapping, int n_mapping, const gs_span* query,
                      void* const* query_out, int n_query, int id_bytes, void* frontier,
                      int64_t* num_unique, void* workspace, size_t workspace_bytes,
                      void* stream) {
  GS_REQUIRE(mapping && n_mapping >= 1 && n_mapping <= GS_MAX_SPANS,
             "gs_unique_relabel: 1..%d mapping spans required, got %d", GS_MAX_SPANS, n_mapping);
  GS_REQUIRE(n_query >= 0 && n_query <= GS_MAX_SPANS && (n_query == 0 || (query && query_out)),
             "gs_unique_relabel: 0..%d query spans required, got %d", GS_MAX_SPANS, n_query);
  GS_REQUIRE(valid_id_bytes(id_bytes), "gs_unique_relabel: id_bytes must be 4 or 8, got %d", id_bytes);
  GS_REQUIRE(num_unique, "gs_unique_relabel: num_unique is null");
  int64_t M = 0;
  for (int s = 0; s < n_mapping; ++s) {
    GS_REQUIRE(mapping[s].n >= 0 && (mapping[s].n == 0 || mapping[s].ptr),
               "gs_unique_relabel: mapping span %d is null or negative", s);
    M += mapping[s].n;
  }
  for (int q = 0; q < n_query; ++q)
    GS_REQUIRE(query[q].n >= 0 && (query[q].n == 0 || (query[q].ptr && query_out[q])),
               "gs_unique_relabel: query span %d is null or negative", q);
  GS_REQUIRE(M == 0 || frontier, "gs_unique_relabel: frontier is null");
  if (M >= (int64_t(1) << 30)) {
    set_error_text("gs_unique_relabel: %lld mapping items exceed the supported 2^30",
                   static_cast<long long>(M));
    return GS_ERR_UNSUPPORTED;
  }
  hipStream_t st = static_cast<hipStream_t>(stream);
  return id_bytes == 8 ? unique_relabel_impl<int64_t>(mapping, n_mapping, query, query_out, n_query,
                                                      frontier, num_unique, workspace,
                                                      workspace_bytes, st)
                       : unique_relabel_impl<int32_t>(mapping, n_mapping, query, query_out, n_query,
                                                      frontier, num_unique, workspace,
                                                      workspace_bytes, st);
}

}  // extern "C"
