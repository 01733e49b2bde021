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
//  * 32-bit ids use ONE 64-bit word per slot, (key << 32 | first index): an
//    insert is a single compare-and-swap in the common case, and a duplicate
//    lowers the index with a single atomicMin on the same word.  Device-scope
//    atomics are resolved memory-side on a multi-XCD part, so the number of
//    atomics per item, not bytes, is what this kernel is made of.  64-bit ids
//    keep separate key (int64) and index (int32) arrays;
//  * every item remembers its slot (4 B) so later passes never probe again;
//  * the mapping tensors are read in place through a span table -- no
//    concatenated copy is materialised (the reference does torch::cat,
//    unique_reindex.cu:187-190);
//  * the rank of a key is prefix[first index], so compaction and every relabel
//    lookup run in one final kernel; a query that aliases a mapping span is
//    relabelled by slot gather instead of probing.
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

__device__ __forceinline__ uint32_t fib_home(uint64_t key, int shift) {
  return static_cast<uint32_t>((key * 0x9E3779B97F4A7C15ull) >> shift);
}

// ---- slot layout for 32-bit ids: (key << 32 | first index), all ones = empty
struct PackedTable {
  unsigned long long* slots;
  uint32_t mask;
  int shift;
  static size_t bytes(int64_t cap) { return padded(cap * 8); }
  void carve(Carver& ws, int64_t cap) { slots = ws.take<unsigned long long>(cap); }
  __device__ __forceinline__ void clear(int64_t i) const { slots[i] = ~0ull; }
  // returns the slot of `key` after recording index i as a candidate first occurrence
  __device__ __forceinline__ uint32_t insert(long long key, uint32_t i) const {
    const unsigned long long hi = static_cast<unsigned long long>(static_cast<uint32_t>(key)) << 32;
    const unsigned long long word = hi | i;
    uint32_t p = fib_home(static_cast<uint32_t>(key), shift);
    while (true) {
      const unsigned long long prev = atomicCAS(&slots[p], ~0ull, word);
      if (prev == ~0ull) break;
      if ((prev >> 32) == (hi >> 32)) {
        if (static_cast<uint32_t>(prev) > i) atomicMin(&slots[p], word);
        break;
      }
      p = (p + 1) & mask;
    }
    return p;
  }
  __device__ __forceinline__ uint32_t first_index(uint32_t p) const {
    return static_cast<uint32_t>(slots[p]);
  }
  // first index of `key`, or -1 when absent (unique_reindex.cu:44-58)
  __device__ __forceinline__ int64_t find(long long key) const {
    const unsigned long long k32 = static_cast<uint32_t>(key);
    uint32_t p = fib_home(static_cast<uint32_t>(key), shift);
    while (true) {
      const unsigned long long s = slots[p];
      if (s == ~0ull) return -1;
      if ((s >> 32) == k32) return static_cast<uint32_t>(s);
      p = (p + 1) & mask;
    }
  }
};

// ---- slot layout for 64-bit ids: key array (-1 = empty) + first-index array
struct WideTable {
  long long* keys;
  int* vals;
  uint32_t mask;
  int shift;
  static size_t bytes(int64_t cap) { return padded(cap * 8) + padded(cap * 4); }
  void carve(Carver& ws, int64_t cap) {
    keys = ws.take<long long>(cap);
    vals = ws.take<int>(cap);
  }
  __device__ __forceinline__ void clear(int64_t i) const {
    keys[i] = -1;
    vals[i] = 0x7fffffff;
  }
  // (unique_reindex.cu:13-26 RelabelHashmap::Update)
  __device__ __forceinline__ uint32_t insert(long long key, uint32_t i) const {
    uint32_t p = fib_home(static_cast<uint64_t>(key), shift);
    while (true) {
      const unsigned long long prev =
          atomicCAS(reinterpret_cast<unsigned long long*>(&keys[p]), ~0ull,
                    static_cast<unsigned long long>(key));
      if (prev == ~0ull || prev == static_cast<unsigned long long>(key)) break;
      p = (p + 1) & mask;
    }
    // values only decrease, so a (possibly stale) read <= i proves the atomic unnecessary
    if (__atomic_load_n(&vals[p], __ATOMIC_RELAXED) > static_cast<int>(i))
      atomicMin(&vals[p], static_cast<int>(i));
    return p;
  }
  __device__ __forceinline__ uint32_t first_index(uint32_t p) const {
    return static_cast<uint32_t>(vals[p]);
  }
  __device__ __forceinline__ int64_t find(long long key) const {
    uint32_t p = fib_home(static_cast<uint64_t>(key), shift);
    while (true) {
      const long long cur = keys[p];
      if (cur == key) return vals[p];
      if (cur == -1) return -1;
      p = (p + 1) & mask;
    }
  }
};

template <typename IdT>
struct TableFor {
  using type = WideTable;
};
template <>
struct TableFor<int32_t> {
  using type = PackedTable;
};

template <typename T>
__global__ void __launch_bounds__(kThreads) table_init_kernel(T t, int64_t cap) {
  const int64_t i = static_cast<int64_t>(blockIdx.x) * kThreads + threadIdx.x;
  if (i < cap) t.clear(i);
}

// insert (key -> min index) and remember the slot of every item
// (unique_reindex.cu:92-99)
template <typename IdT, typename T>
__global__ void __launch_bounds__(kThreads)
table_insert_kernel(Spans<IdT> x, int64_t M, T t, uint32_t* __restrict__ pos) {
  const int64_t i = static_cast<int64_t>(blockIdx.x) * kThreads + threadIdx.x;
  if (i >= M) return;
  pos[i] = t.insert(static_cast<long long>(x.get(i)), static_cast<uint32_t>(i));
}

// 1 when item i is the first occurrence of its key (unique_reindex.cu:106-114)
template <typename T>
struct IsFirst {
  T t;
  const uint32_t* pos;
  __device__ __forceinline__ int64_t operator()(int64_t i) const {
    return t.first_index(pos[i]) == static_cast<uint32_t>(i) ? 1 : 0;
  }
};

struct Query {
  const void* in[GS_MAX_SPANS];
  void* out[GS_MAX_SPANS];
  int64_t end[GS_MAX_SPANS];    // exclusive end offset in the concatenation of queries
  int64_t alias[GS_MAX_SPANS];  // >= 0: the query is the mapping span starting there
  int n;
};

// Items [0, M): frontier[rank] = key for first occurrences
// (unique_reindex.cu:127-144).  Items [M, M+Q): relabel lookups
// (unique_reindex.cu:162-170), rank of a key = prefix[its first index].
template <typename IdT, typename T>
__global__ void __launch_bounds__(kThreads)
finish_kernel(Spans<IdT> x, int64_t M, T t, const uint32_t* __restrict__ pos,
              const int64_t* __restrict__ prefix, IdT* __restrict__ frontier,
              int64_t* __restrict__ num_unique, Query qs, int64_t Q) {
  const int64_t i = static_cast<int64_t>(blockIdx.x) * kThreads + threadIdx.x;
  if (i == 0) *num_unique = prefix[M];
  if (i < M) {
    if (t.first_index(pos[i]) == static_cast<uint32_t>(i)) frontier[prefix[i]] = x.get(i);
    return;
  }
  const int64_t j = i - M;
  if (j >= Q) return;
  int s = 0;
  int64_t begin = 0;
#pragma unroll
  for (int u = 0; u < GS_MAX_SPANS - 1; ++u) {
    if (u < qs.n - 1 && j >= qs.end[u]) {
      s = u + 1;
      begin = qs.end[u];
    }
  }
  const int64_t local = j - begin;
  int64_t first;
  if (qs.alias[s] >= 0) {
    first = t.first_index(pos[qs.alias[s] + local]);
  } else {
    first = t.find(static_cast<long long>(static_cast<const IdT*>(qs.in[s])[local]));
  }
  static_cast<IdT*>(qs.out[s])[local] = static_cast<IdT>(first < 0 ? -1 : prefix[first]);
}

int64_t table_capacity(int64_t M) {
  int64_t cap = 1024;
  while (cap < 2 * M) cap <<= 1;
  return cap;
}

template <typename IdT>
size_t workspace_bytes_for(int64_t M) {
  using T = typename TableFor<IdT>::type;
  const int64_t cap = table_capacity(M);
  return T::bytes(cap) + padded((M > 0 ? M : 1) * 4) + padded((M + 1) * 8) +
         scan_workspace_bytes(M);
}

template <typename IdT>
int unique_relabel_impl(const gs_span* mapping, int n_mapping, const gs_span* query,
                        void* const* query_out, int n_query, void* frontier, int64_t* num_unique,
                        void* workspace, size_t workspace_bytes, hipStream_t stream) {
  using T = typename TableFor<IdT>::type;
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
  T t;
  t.carve(ws, cap);
  uint32_t* pos = ws.take<uint32_t>(M > 0 ? M : 1);
  int64_t* prefix = ws.take<int64_t>(M + 1);
  int64_t* tiles = ws.take<int64_t>(scan_num_tiles(M) + 1);
  if (!ws.ok) {
    set_error_text("gs_unique_relabel: workspace needs %zu bytes, 256-byte aligned",
                   workspace_bytes_for<IdT>(M));
    return GS_ERR_WORKSPACE;
  }
  t.mask = static_cast<uint32_t>(cap - 1);
  int lg = 0;
  while ((int64_t(1) << lg) < cap) ++lg;
  t.shift = 64 - lg;

  Query qs;
  int64_t Q = 0;
  for (int q = 0; q < GS_MAX_SPANS; ++q) {
    qs.in[q] = nullptr;
    qs.out[q] = nullptr;
    qs.end[q] = 0;
    qs.alias[q] = -1;
  }
  for (int q = 0; q < n_query; ++q) {
    qs.in[q] = query[q].ptr;
    qs.out[q] = query_out[q];
    Q += query[q].n;
    qs.end[q] = Q;
    int64_t off = 0;
    for (int s = 0; s < n_mapping; ++s) {
      if (mapping[s].ptr == query[q].ptr && mapping[s].n == query[q].n) qs.alias[q] = off;
      off += mapping[s].n;
    }
  }
  qs.n = n_query;

  {
    ProfileScope prof("table_init", stream);
    hipLaunchKernelGGL((table_init_kernel<T>), dim3(blocks_for(cap, kThreads)), dim3(kThreads), 0,
                       stream, t, cap);
  }
  if (M > 0) {
    ProfileScope prof("table_insert", stream);
    hipLaunchKernelGGL((table_insert_kernel<IdT, T>), dim3(blocks_for(M, kThreads)), dim3(kThreads),
                       0, stream, x, M, t, pos);
  }
  GS_RETURN_IF_ERROR(check_launch("unique insert"));
  IsFirst<T> f{t, pos};
  GS_RETURN_IF_ERROR(exclusive_scan(f, M, prefix, tiles, stream));
  ProfileScope prof("unique_finish", stream);
  hipLaunchKernelGGL((finish_kernel<IdT, T>), dim3(blocks_for(M + Q, kThreads)), dim3(kThreads), 0,
                     stream, x, M, t, pos, prefix, static_cast<IdT*>(frontier), num_unique, qs, Q);
  return check_launch("unique_relabel");
}

}  // namespace
}  // namespace gs

using namespace gs;

extern "C" {

size_t gs_unique_workspace_bytes(int64_t M) {
  if (M < 0) M = 0;
  const size_t a = workspace_bytes_for<int64_t>(M);
  const size_t b = workspace_bytes_for<int32_t>(M);
  return a > b ? a : b;
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
