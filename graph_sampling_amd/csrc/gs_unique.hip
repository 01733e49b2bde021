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
//  * first-occurrence flags, their scan and the compaction run in ONE launch
//    (chained scan with look-back); the rank of a key is prefix[first index],
//    so every relabel lookup is two gathers in a last kernel, and a query that
//    aliases a mapping span is relabelled by slot gather instead of probing.
#include "gs_common.hpp"
#include "gs_batch_items.hpp"
#include <type_traits>

#include "gs_table.hpp"

GS_STAMPS_DEFINE(unique)

namespace gs {
namespace {

constexpr int kThreads = 256;

template <typename IdT>
struct Spans {
  const IdT* ptr[GS_MAX_SPANS];
  int64_t end[GS_MAX_SPANS];  // exclusive end offset of each span in the concatenation
  int n;
  // When last_len is set the last span's length lives on the device (a total an
  // earlier kernel on the stream produced and the host has not read yet):
  // items = fixed + max(*last_len, 0), and the host-side count is only a bound.
  const int64_t* last_len;
  int64_t fixed;
  __device__ __forceinline__ int64_t items(int64_t host_items) const {
    if (!last_len) return host_items;
    const int64_t n_last = *last_len;
    return fixed + (n_last > 0 ? n_last : 0);
  }
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

// empties the table and zeroes the look-back state of the compaction pass
template <typename T>
__global__ void __launch_bounds__(kThreads) table_init_kernel(T t, int64_t cap, LookbackState lb,
                                                              int64_t tiles) {
  const int64_t i = static_cast<int64_t>(blockIdx.x) * kThreads + threadIdx.x;
  if (i < cap) t.clear(i);
  if (i < tiles) lb.status[i] = 0ull;
  if (i == 0) *lb.error = 0u;
}

// insert (key -> min index) and remember the slot of every item
// (unique_reindex.cu:92-99)
// too_wide: set to 2 when T keeps 32 bits of a key and a key does not fit them (64-bit ids
// on the one-word slots); the compaction then reports -2 instead of a count
template <typename IdT, typename T, bool PEEK>
__global__ void __launch_bounds__(kThreads)
table_insert_kernel(Spans<IdT> x, int64_t M_bound, T t, uint32_t* __restrict__ pos,
                    unsigned int* __restrict__ too_wide) {
  const int64_t i = static_cast<int64_t>(blockIdx.x) * kThreads + threadIdx.x;
  if (i >= M_bound) return;
  GS_STAMP_BEGIN();
  GS_STAMP(0);
  // the key is read before the device-side length is known (the buffers hold M_bound items
  // whatever the length turns out to be): one round trip instead of two
  const IdT key = x.get(i);
  if (i >= x.items(M_bound)) return;
  GS_STAMP(1);  // key and length are here
  if (sizeof(IdT) == 8 && too_wide && (static_cast<unsigned long long>(key) >> 32) != 0ull) {
    *too_wide = 2u;
    pos[i] = 0u;
    return;
  }
  const uint32_t slot = t.template insert<PEEK>(static_cast<long long>(key), static_cast<uint32_t>(i));
  GS_STAMP(2);  // the slot is known
  pos[i] = slot;
  GS_STAMP(3);
  GS_STAMP_END(2, 4);
}

// The same for inputs where keys repeat a lot (the general relabel: edge ends of a block,
// node lists with hubs).  Thousands of occurrences of one key are thousands of atomics on
// one table word, and those queue up at the memory side (~11 ns each: 90 k edge ends over
// 1000 nodes took 58 us, 220 k copies of one key 1.2 ms).  Here the workgroup's 256 items
// first meet in a small LDS table; of the items that share a key only the one with the
// lowest index goes to the table in memory, and hands the slot it found to the others.
constexpr int kGroupSlots = 1024;
constexpr int kGroupProbes = 4;

template <typename IdT, typename T>
__global__ void __launch_bounds__(kThreads)
table_insert_grouped_kernel(Spans<IdT> x, int64_t M_bound, T t, uint32_t* __restrict__ pos,
                            unsigned int* __restrict__ too_wide) {
  __shared__ unsigned long long s_key[kGroupSlots];
  __shared__ unsigned int s_min[kGroupSlots];
  __shared__ unsigned int s_pos[kGroupSlots];
  for (int j = threadIdx.x; j < kGroupSlots; j += kThreads) {
    s_key[j] = ~0ull;
    s_min[j] = 0xFFFFFFFFu;
  }
  __syncthreads();
  const int64_t i = static_cast<int64_t>(blockIdx.x) * kThreads + threadIdx.x;
  bool live = i < x.items(M_bound);  // the last span's length may live on the device
  IdT key = IdT(0);
  if (live) {
    key = x.get(i);
    if (sizeof(IdT) == 8 && too_wide && (static_cast<unsigned long long>(key) >> 32) != 0ull) {
      *too_wide = 2u;
      pos[i] = 0u;
      live = false;
    }
  }
  const unsigned long long k64 = static_cast<unsigned long long>(static_cast<long long>(key));
  int slot = -1;  // the LDS slot of the item's key; none after a few probes: the item goes alone
  if (live && k64 != ~0ull) {
    unsigned int h = static_cast<unsigned int>((k64 * 0x9E3779B97F4A7C15ull) >> 40) & (kGroupSlots - 1);
    for (int probe = 0; probe < kGroupProbes; ++probe) {
      const unsigned long long seen = atomicCAS(&s_key[h], ~0ull, k64);
      if (seen == ~0ull || seen == k64) {
        slot = static_cast<int>(h);
        atomicMin(&s_min[h], static_cast<unsigned int>(i));
        break;
      }
      h = (h + 1) & (kGroupSlots - 1);
    }
  }
  __syncthreads();
  const bool leads = live && (slot < 0 || s_min[slot] == static_cast<unsigned int>(i));
  uint32_t p = 0u;
  if (leads) {
    p = t.template insert<true>(static_cast<long long>(key), static_cast<uint32_t>(i));
    if (slot >= 0) s_pos[slot] = p;
  }
  __syncthreads();
  if (live) pos[i] = leads ? p : s_pos[slot];
}

struct Query {
  const void* in[GS_MAX_SPANS];
  void* out[GS_MAX_SPANS];
  int64_t end[GS_MAX_SPANS];    // exclusive end offset in the concatenation of queries
  int64_t alias[GS_MAX_SPANS];  // >= 0: the query is the mapping span starting there
  int n;
};

// One launch for flags, their scan and the compaction: a tile of 2048 items,
// eight consecutive items per lane.  prefix[i] = number of first occurrences
// before item i (the rank of item i's key when i is a first occurrence),
// frontier[rank] = key (unique_reindex.cu:106-144).  The last tile knows the
// number of unique ids and reports it.
constexpr int kCompactItems = 8;
constexpr int kCompactTile = kThreads * kCompactItems;

template <typename IdT, typename T>
__global__ void __launch_bounds__(kThreads)
compact_kernel(Spans<IdT> x, int64_t M_bound, T t, const uint32_t* __restrict__ pos,
               int64_t* __restrict__ prefix, IdT* __restrict__ frontier,
               int64_t* __restrict__ num_unique, LookbackState lb, gs_mailbox* box,
               int64_t box_ticket, uint32_t* __restrict__ first_out) {
  __shared__ int64_t s_scan[kThreads / kWave + 1];
  __shared__ int64_t s_prefix;
  GS_STAMP_BEGIN();
  GS_STAMP(0);
  const int64_t M = x.items(M_bound);
  const unsigned int tile = blockIdx.x;
  const int64_t base = static_cast<int64_t>(tile) * kCompactTile +
                       static_cast<int64_t>(threadIdx.x) * kCompactItems;
  bool first[kCompactItems];
  int64_t mine = 0;
  // slot numbers, then the slots' words, then the stores: three batches, so that the eight
  // trips to the table are in flight together and none waits for a store before it
  // (no read carries a condition of its own -- the last entry again past the end: a read that
  // may or may not happen makes every later one wait for all that is in flight)
  uint32_t at[kCompactItems], fi[kCompactItems];
#pragma unroll
  for (int k = 0; k < kCompactItems; ++k) at[k] = 0u;
  if (M_bound > 0) {
#pragma unroll
    for (int k = 0; k < kCompactItems; ++k) at[k] = pos[base + k < M_bound ? base + k : M_bound - 1];
  }
  GS_STAMP(1);  // slot numbers (and the device-side length) are here
  // read under the host's bound, not the device-side length, so that the reads do not wait
  // for it; a slot number beyond the length is whatever the workspace held: masked
#pragma unroll
  for (int k = 0; k < kCompactItems; ++k) fi[k] = t.first_index(at[k] & t.mask);
#pragma unroll
  for (int k = 0; k < kCompactItems; ++k) {
    const int64_t i = base + k;
    first[k] = i < M && fi[k] == static_cast<uint32_t>(i);
    mine += first[k] ? 1 : 0;
  }
  // kept for the passes after this one: they need no second trip to the table (and the
  // last pass of gs_relabel_sampled must not read it any more: it empties it)
  if (first_out) {
#pragma unroll
    for (int k = 0; k < kCompactItems; ++k)
      if (base + k < M) first_out[base + k] = fi[k];
  }
  GS_STAMP(2);  // the slots' words are here
  int64_t tile_total;
  const int64_t local = block_exclusive_scan<kThreads>(mine, &tile_total, s_scan);
  if (threadIdx.x == 0) lookback_publish_sum(lb, tile, tile_total);
  GS_STAMP(3);  // flags scanned, tile sum published
  IdT key[kCompactItems];  // in flight while wave 0 walks back (every item's key, needed or not)
#pragma unroll
  for (int k = 0; k < kCompactItems; ++k) key[k] = IdT(0);
  if (M > 0) {
#pragma unroll
    for (int k = 0; k < kCompactItems; ++k) key[k] = x.get(base + k < M ? base + k : M - 1);
  }
  if (threadIdx.x < kWave) {
    const int64_t before = lookback_exclusive_prefix(lb, tile, tile_total);
    if (threadIdx.x == 0) s_prefix = before;
  }
  GS_STAMP(4);  // look-back done (and thread 0's keys)
  __syncthreads();
  GS_STAMP(5);
  int64_t run = s_prefix + local;
#pragma unroll
  for (int k = 0; k < kCompactItems; ++k) {
    const int64_t i = base + k;
    if (i < M) {
      prefix[i] = run;
      if (first[k]) frontier[run] = key[k];
    }
    run += first[k] ? 1 : 0;
  }
  if (tile == gridDim.x - 1 && threadIdx.x == 0) {
    int64_t total = s_prefix + tile_total;
    const unsigned int err = __hip_atomic_load(lb.error, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    if (err) total = err == 2u ? -2 : -1;  // 2: a key did not fit the one-word slots
    *num_unique = total;
    post_mailbox(box, total, box_ticket);
  }
  GS_STAMP(6);  // stores done
  GS_STAMP_END(3, 7);
}

// Relabel lookups (unique_reindex.cu:162-170): rank of a key = prefix[its first index].
template <typename IdT, typename T>
__global__ void __launch_bounds__(kThreads)
lookup_kernel(T t, const uint32_t* __restrict__ first_of, const int64_t* __restrict__ prefix,
              Query qs, int64_t Q_bound, const int64_t* __restrict__ q_len, int64_t M) {
  const int64_t j = static_cast<int64_t>(blockIdx.x) * kThreads + threadIdx.x;
  int64_t Q = Q_bound;
  if (q_len) {  // one query that aliases the device-sized last mapping span
    Q = *q_len;
    if (Q > Q_bound) Q = Q_bound;
  }
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
    // a query that is one of the mapping spans: the compaction has set its first indices aside
    first = first_of[qs.alias[s] + local];
  } else {
    const IdT key = static_cast<const IdT*>(qs.in[s])[local];
    const bool fits = sizeof(IdT) == 4 || !std::is_same<T, PackedTable>::value ||
                      (static_cast<unsigned long long>(key) >> 32) == 0ull;
    first = fits ? t.find(static_cast<long long>(key)) : -1;
  }
  // first >= M only when the insert pass gave up (an id too wide for the slots): the outputs
  // are void then, but no index may leave the arrays
  static_cast<IdT*>(qs.out[s])[local] =
      static_cast<IdT>(first < 0 || first >= M ? -1 : prefix[first]);
}

// Last pass of a relabel on a table that outlives the call (gs_relabel_sampled): item i >= S is
// sampled id number i - S, renamed to prefix[its first index]; every item then empties
// its slot, so the table is clean again for the next call without a clearing pass.  Nothing
// here reads the table: the first indices were set aside by the compaction.
template <typename IdT, typename T>
__global__ void __launch_bounds__(kThreads)
finish_linked_kernel(T t, const uint32_t* __restrict__ pos, const uint32_t* __restrict__ first,
                     const int64_t* __restrict__ prefix, int64_t S, int64_t M_bound,
                     const int64_t* __restrict__ sampled_len, IdT* __restrict__ out_ids,
                     int64_t* __restrict__ offsets_copy) {
  const int64_t i = static_cast<int64_t>(blockIdx.x) * kThreads + threadIdx.x;
  GS_STAMP_BEGIN();
  GS_STAMP(0);
  // the sampler's S + 1 offsets end at sampled_len: a second copy for the caller who hands
  // the relabelled block out beside the sampled graph (saves a device copy per call)
  if (offsets_copy && i <= S) offsets_copy[i] = (sampled_len - S)[i];
  // reads go by the host's bound so that they do not wait for the device-side length
  const uint32_t f = i < M_bound ? first[i] : 0u;
  GS_STAMP(1);  // first-occurrence index is here
  const int64_t rank = prefix[f < M_bound ? f : 0u];
  const uint32_t p = i < M_bound ? pos[i] : 0u;
  int64_t n = *sampled_len;
  if (n < 0) n = 0;
  int64_t M = S + n;
  if (M > M_bound) M = M_bound;
  GS_STAMP(2);  // rank, slot and length are here
  if (i >= M) return;
  if (i >= S) out_ids[i - S] = static_cast<IdT>(rank);
  t.clear(p);
  GS_STAMP(3);
  GS_STAMP_END(4, 4);
}

template <typename T>
__global__ void __launch_bounds__(kThreads) table_clear_kernel(T t, int64_t cap) {
  const int64_t i = static_cast<int64_t>(blockIdx.x) * kThreads + threadIdx.x;
  if (i < cap) t.clear(i);
}

inline int64_t compact_num_tiles(int64_t M) {
  return M <= 0 ? 1 : (M + kCompactTile - 1) / kCompactTile;
}

template <typename IdT>
size_t workspace_bytes_for(int64_t M) {
  using T = typename TableFor<IdT>::type;
  const int64_t cap = table_capacity(M);
  return T::bytes(cap) + 2 * padded((M > 0 ? M : 1) * 4) + padded((M + 1) * 8) +
         lookback_state_bytes(compact_num_tiles(M));
}

template <typename IdT, typename T>
int unique_relabel_impl(const gs_span* mapping, int n_mapping, const gs_span* query,
                        void* const* query_out, int n_query, void* frontier, int64_t* num_unique,
                        void* workspace, size_t workspace_bytes, const int64_t* last_span_len,
                        gs_mailbox* box, int64_t box_ticket, hipStream_t stream) {
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
  x.last_len = last_span_len;
  x.fixed = M - mapping[n_mapping - 1].n;
  const int64_t cap = table_capacity(M);
  Carver ws(workspace, workspace_bytes);
  T t;
  t.carve(ws, cap);
  uint32_t* pos = ws.take<uint32_t>(M > 0 ? M : 1);
  uint32_t* first = ws.take<uint32_t>(M > 0 ? M : 1);  // index of the first occurrence of item i's key
  int64_t* prefix = ws.take<int64_t>(M + 1);
  const int64_t tiles = compact_num_tiles(M);
  LookbackState lb = carve_lookback(ws, tiles, 1u);  // cleared by table_init on every call
  if (!ws.ok) {
    set_error_text("gs_unique_relabel: workspace needs %zu bytes, 256-byte aligned",
                   workspace_bytes_for<IdT>(M));
    return GS_ERR_WORKSPACE;
  }
  table_shape(t, cap);

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
    const int64_t n_init = cap > tiles ? cap : tiles;
    hipLaunchKernelGGL((table_init_kernel<T>), dim3(blocks_for(n_init, kThreads)), dim3(kThreads),
                       0, stream, t, cap, lb, tiles);
  }
  if (M > 0) {
    ProfileScope prof("table_insert", stream);
    constexpr bool kNarrow = sizeof(IdT) == 8 && std::is_same<T, PackedTable>::value;
    hipLaunchKernelGGL((table_insert_grouped_kernel<IdT, T>), dim3(blocks_for(M, kThreads)),
                       dim3(kThreads), 0, stream, x, M, t, pos,
                       kNarrow ? lb.error : static_cast<unsigned int*>(nullptr));
  }
  {
    ProfileScope prof("unique_compact", stream);
    hipLaunchKernelGGL((compact_kernel<IdT, T>), dim3(static_cast<unsigned>(tiles)), dim3(kThreads),
                       0, stream, x, M, t, pos, prefix, static_cast<IdT*>(frontier), num_unique, lb,
                       box, box_ticket, first);
  }
  if (Q > 0) {
    ProfileScope prof("unique_finish", stream);
    hipLaunchKernelGGL((lookup_kernel<IdT, T>), dim3(blocks_for(Q, kThreads)), dim3(kThreads), 0,
                       stream, t, first, prefix, qs, Q, last_span_len, M);
  }
  return check_launch("unique_relabel");
}


template <typename IdT, typename T>
int relabel_sampled_impl(const void* seed_keys, int64_t S, const void* sampled, int64_t capacity,
                         const int64_t* sampled_len, void* table, size_t table_bytes,
                         void* frontier, void* out_ids, int64_t* num_unique,
                         int64_t* offsets_copy, void* workspace,
                         size_t workspace_bytes, void* state, size_t state_bytes, uint32_t epoch,
                         gs_mailbox* box, int64_t box_ticket, hipStream_t stream) {
  const int64_t M = S + capacity;
  T t;
  if (!shape_linked_table<T>(table, table_bytes, M, &t)) {
    set_error_text("gs_relabel_sampled: the table holds fewer than the %lld slots this call "
                   "needs (or is misaligned)",
                   static_cast<long long>(linked_table_capacity(M)));
    return GS_ERR_WORKSPACE;
  }
  Carver ws(workspace, workspace_bytes);
  int64_t* prefix = ws.take<int64_t>(M + 1);
  uint32_t* first = ws.take<uint32_t>(M > 0 ? M : 1);
  uint32_t* pos = ws.take<uint32_t>(M > 0 ? M : 1);
  const int64_t tiles = compact_num_tiles(M);
  Carver sc(state, state_bytes);
  LookbackState lb = carve_lookback(sc, tiles, epoch);
  if (!ws.ok || !sc.ok) {
    set_error_text("gs_relabel_sampled: workspace needs %zu bytes and state %zu bytes, 256-byte aligned",
                   gs_relabel_sampled_workspace_bytes(M), gs_relabel_sampled_state_bytes(M));
    return GS_ERR_WORKSPACE;
  }
  Spans<IdT> x;
  for (int s = 0; s < GS_MAX_SPANS; ++s) {
    x.ptr[s] = nullptr;
    x.end[s] = 0;
  }
  x.ptr[0] = static_cast<const IdT*>(seed_keys);
  x.end[0] = S;
  x.ptr[1] = static_cast<const IdT*>(sampled);
  x.end[1] = M;
  x.n = 2;
  x.last_len = sampled_len;
  x.fixed = S;
  if (M > 0) {
    ProfileScope prof("table_insert", stream);
    // no peek here: sampled neighbours are mostly new keys, and the extra read costs the
    // GraphSAGE step 7 % (0.152 ms against 0.142)
    constexpr bool kNarrow = sizeof(IdT) == 8 && std::is_same<T, PackedTable>::value;
    hipLaunchKernelGGL((table_insert_kernel<IdT, T, false>), dim3(blocks_for(M, kThreads)),
                       dim3(kThreads), 0, stream, x, M, t, pos,
                       kNarrow ? lb.error : static_cast<unsigned int*>(nullptr));
  }
  {
    ProfileScope prof("unique_compact", stream);
    hipLaunchKernelGGL((compact_kernel<IdT, T>), dim3(static_cast<unsigned>(tiles)), dim3(kThreads),
                       0, stream, x, M, t, pos, prefix, static_cast<IdT*>(frontier), num_unique, lb,
                       box, box_ticket, first);
  }
  if (M > 0 || offsets_copy) {
    ProfileScope prof("unique_finish", stream);
    const int64_t threads = offsets_copy && S + 1 > M ? S + 1 : M;
    hipLaunchKernelGGL((finish_linked_kernel<IdT, T>), dim3(blocks_for(threads, kThreads)),
                       dim3(kThreads), 0, stream, t, pos, first, prefix, S, M, sampled_len,
                       static_cast<IdT*>(out_ids), offsets_copy);
  }
  return check_launch("relabel_sampled");
}

// ------------------------------------------- the relabel of gs_layer_relabel ----
// Second launch of a layer whose first (gs_layer_sample) has already entered every seed and
// every sampled id into the table: flags, their scan, the frontier AND the renaming of the
// sampled ids in one kernel.  The rank of a key is the rank of its first occurrence f, and
// f <= i for every item i that carries the key, so an item only ever needs results of its own
// or of EARLIER tiles -- the same dependence the look-back has:
//  * a tile stores, for each of its first occurrences, how far it stands from the tile's end
//    (12 bits per item, four items to a 64-bit word, the launch's epoch above them: a word
//    says by itself whether it is this launch's), then closes itself (inclusive prefix);
//  * rank(f) = inclusive prefix of f's tile - that distance: two reads in flight together for
//    an f of another tile, each polled until it is this launch's (bounded like the
//    look-back's waits), LDS for an f of the same tile.
// The key of an item is the upper half of its slot's word, so neither the seeds nor the
// sampled ids are read again.  The table is NOT emptied here (a later tile may still have to
// read a slot): the caller names it as `prev` in its next gs_layer_relabel on ANOTHER table,
// or sweeps it with gs_layer_table_sweep.
struct RankCounts {
  int64_t S_bound;
  const int64_t* S_dev;
  int64_t cap;
  const int64_t* E_dev;
  __device__ __forceinline__ void get(int64_t* S, int64_t* M) const {
    int64_t s = S_bound;
    if (S_dev) {
      s = *S_dev;
      s = s < 0 ? 0 : (s < S_bound ? s : S_bound);
    }
    int64_t e = *E_dev;
    e = e < 0 ? 0 : (e < cap ? e : cap);
    *S = s;
    *M = s + e;
  }
};

template <typename IdT>
struct RankArgs {
  PackedTable t;
  const uint32_t* pos;
  RankCounts n;
  unsigned long long* back;  // one 64-bit word per four items, in the look-back state
  IdT* frontier;
  IdT* out_ids;
  int64_t* num_unique;
  const int64_t* offsets;  // the sampler's offsets (S + 1 of them), copied to offsets_copy
  int64_t* offsets_copy;
  LookbackState lb;
  gs_mailbox* box;
  int64_t box_ticket;
  // the table of an earlier layer, emptied on the side
  PackedTable prev_t;
  const uint32_t* prev_pos;
  RankCounts prev_n;
};

// distances of a tile's first occurrences from its end: 1..2048, four to a word under the epoch
constexpr int kBackBits = 12;
constexpr unsigned long long kBackMask = (1ull << kBackBits) - 1;
constexpr int kBackEpochShift = 48;
static_assert(kCompactTile < (1 << kBackBits), "a distance must fit its field");

// the word of four items once its tile has stored it in this launch (0 after giving up, with
// the error raised)
__device__ __forceinline__ unsigned long long back_wait(const LookbackState& st,
                                                        const unsigned long long* back,
                                                        unsigned long long seen, uint32_t at) {
  int polls = 0;
  while (((seen >> kBackEpochShift) & kLbMaxEpoch) != st.epoch) {
    if (++polls > st.spin_limit) {
      lookback_raise(st);
      return 0ull;
    }
    if (polls > 16) __builtin_amdgcn_s_sleep(32);
    seen = lb_load(&back[at]);
  }
  return seen;
}

// workgroup `part` of `parts` empties its share of the slots a layer's items went to
__device__ __forceinline__ void sweep_slots(const PackedTable& t, const uint32_t* __restrict__ pos,
                                            const RankCounts& n, unsigned int part,
                                            unsigned int parts) {
  int64_t S, M;
  n.get(&S, &M);
  const int64_t g = static_cast<int64_t>(part) * kThreads + threadIdx.x;
  const int64_t stride = static_cast<int64_t>(parts) * kThreads;
  constexpr int kInFlight = 8;  // slot numbers a lane reads before it stores
  for (int64_t j = g; j < M; j += kInFlight * stride) {
    uint32_t slot[kInFlight];
#pragma unroll
    for (int u = 0; u < kInFlight; ++u) slot[u] = j + u * stride < M ? pos[j + u * stride] : 0u;
#pragma unroll
    for (int u = 0; u < kInFlight; ++u)
      if (j + u * stride < M) t.clear(slot[u] & t.mask);
  }
}

template <typename IdT>
__global__ void __launch_bounds__(kThreads) rank_linked_kernel(RankArgs<IdT> a) {
  __shared__ int64_t s_scan[kThreads / kWave + 1];
  __shared__ int64_t s_prefix;
  __shared__ unsigned short s_back[kCompactTile];
  GS_STAMP_BEGIN();
  GS_STAMP(0);
  const unsigned int tile = blockIdx.x;
  const int64_t M_bound = a.n.S_bound + a.n.cap;
  const int64_t base = static_cast<int64_t>(tile) * kCompactTile +
                       static_cast<int64_t>(threadIdx.x) * kCompactItems;
  // slot numbers go by the bound (the array is sized for it), so that they are on their way
  // together with the counts
  // (read without a branch, the last entry again past the end: a read that may or may not
  // happen makes every later one wait for all that is in flight)
  uint32_t at[kCompactItems];
#pragma unroll
  for (int k = 0; k < kCompactItems; ++k) at[k] = 0u;
  if (M_bound > 0) {
#pragma unroll
    for (int k = 0; k < kCompactItems; ++k)
      at[k] = a.pos[base + k < M_bound ? base + k : M_bound - 1];
  }
  int64_t S, M;
  a.n.get(&S, &M);
  const int64_t live = (M + kCompactTile - 1) / kCompactTile;
  const unsigned int tiles = static_cast<unsigned int>(live > 0 ? live : 1);
  // The launch is sized for the bound, so most of its workgroups usually have no items: those
  // empty the slots of the earlier layer while the others work.  Only when too few are idle
  // do the working ones share that job, at their ends.
  const unsigned int idle = gridDim.x - tiles;
  const bool idle_sweep = idle * 4u >= tiles;
  if (tile >= tiles) {
    if (a.prev_pos && idle_sweep)
      sweep_slots(a.prev_t, a.prev_pos, a.prev_n, tile - tiles, idle);
    return;
  }
  GS_STAMP(1);  // slot numbers and counts are here
  unsigned long long w[kCompactItems];
#pragma unroll
  for (int k = 0; k < kCompactItems; ++k) w[k] = a.t.slots[at[k] & a.t.mask];  // (any slot will do past M)
#pragma unroll
  for (int k = 0; k < kCompactItems; ++k)
    if (base + k >= M) w[k] = ~0ull;
  bool first[kCompactItems];
  int64_t mine = 0;
#pragma unroll
  for (int k = 0; k < kCompactItems; ++k) {
    first[k] = base + k < M && static_cast<uint32_t>(w[k]) == static_cast<uint32_t>(base + k);
    mine += first[k] ? 1 : 0;
  }
  GS_STAMP(2);  // the slots' words are here
  int64_t tile_total;
  const int64_t local = block_exclusive_scan<kThreads>(mine, &tile_total, s_scan);
  if (threadIdx.x == 0) lookback_publish_sum(a.lb, tile, tile_total, /*may_close=*/false);
  // distance of every first occurrence from the tile's end: to LDS for this tile's own
  // lookups, to memory (device-scope stores, four items a word) for those of later tiles
  {
    const unsigned long long tag = static_cast<unsigned long long>(a.lb.epoch) << kBackEpochShift;
    unsigned long long word[2] = {tag, tag};
    int64_t run = local;
#pragma unroll
    for (int k = 0; k < kCompactItems; ++k) {
      const unsigned int d = first[k] ? static_cast<unsigned int>(tile_total - run) : 0u;
      s_back[threadIdx.x * kCompactItems + k] = static_cast<unsigned short>(d);
      word[k >> 2] |= static_cast<unsigned long long>(d) << (kBackBits * (k & 3));
      run += first[k] ? 1 : 0;
    }
    if (base < M) lb_store(&a.back[base >> 2], word[0]);
    if (base + 4 < M) lb_store(&a.back[(base >> 2) + 1], word[1]);
  }
  GS_STAMP(3);  // flags scanned, sum published, distances stored
  if (threadIdx.x < kWave) {
    const int64_t before = lookback_exclusive_prefix(a.lb, tile, tile_total, /*publish=*/false);
    if (threadIdx.x == 0) s_prefix = before;
  }
  GS_STAMP(4);  // look-back done
  // every wave's distance stores have completed before the tile closes
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
  __syncthreads();
  const int64_t tile_excl = s_prefix;
  const int64_t tile_incl = tile_excl + tile_total;
  if (threadIdx.x == 0) lookback_publish_inclusive(a.lb, tile, tile_incl);
  GS_STAMP(5);
  // lookups of the sampled ids: both reads of every item first, the waits after
  unsigned long long bw[kCompactItems], st[kCompactItems];
#pragma unroll
  for (int k = 0; k < kCompactItems; ++k) {
    const int64_t i = base + k;
    const uint32_t f = static_cast<uint32_t>(w[k]);
    bw[k] = 0ull;
    st[k] = 0ull;
    if (i >= S && i < M && (f >> 11) != tile && f < i) {
      bw[k] = lb_load(&a.back[f >> 2]);
      st[k] = lb_load(&a.lb.status[f >> 11]);
    }
  }
  // every rank first (the reads, and the waits for tiles that have not closed yet), then all
  // the stores: a store between two items' reads would make the later read wait for it
  int64_t rank[kCompactItems];
#pragma unroll
  for (int k = 0; k < kCompactItems; ++k) {
    const int64_t i = base + k;
    rank[k] = -1;
    if (i >= S && i < M) {
      const uint32_t f = static_cast<uint32_t>(w[k]);
      if (f <= static_cast<uint32_t>(i)) {  // (anything else: the insert pass gave up on this id)
        if ((f >> 11) == tile) {
          rank[k] = tile_incl - s_back[f & (kCompactTile - 1)];
        } else {
          const int64_t incl = lookback_wait_inclusive(a.lb, st[k], f >> 11);
          const unsigned long long b = back_wait(a.lb, a.back, bw[k], f >> 2);
          rank[k] = incl - static_cast<int64_t>((b >> (kBackBits * (f & 3))) & kBackMask);
        }
      }
    }
  }
  {
    int64_t run = tile_excl + local;
#pragma unroll
    for (int k = 0; k < kCompactItems; ++k) {
      if (first[k]) a.frontier[run] = static_cast<IdT>(w[k] >> 32);
      run += first[k] ? 1 : 0;
    }
  }
#pragma unroll
  for (int k = 0; k < kCompactItems; ++k) {
    const int64_t i = base + k;
    if (i >= S && i < M) a.out_ids[i - S] = static_cast<IdT>(rank[k]);
  }
  if (a.offsets_copy) {
    const int64_t g = static_cast<int64_t>(tile) * kThreads + threadIdx.x;
    for (int64_t r = g; r <= S; r += static_cast<int64_t>(tiles) * kThreads)
      a.offsets_copy[r] = a.offsets[r];
  }
  if (tile == tiles - 1 && threadIdx.x == 0) {
    int64_t total = tile_incl;
    const unsigned int err = __hip_atomic_load(a.lb.error, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    if (err) total = err == 2u ? -2 : -1;  // 2: a key did not fit the one-word slots
    *a.num_unique = total;
    post_mailbox(a.box, total, a.box_ticket);
  }
  if (a.prev_pos && !idle_sweep) sweep_slots(a.prev_t, a.prev_pos, a.prev_n, tile, tiles);
  GS_STAMP(6);
  GS_STAMP_END(5, 7);
}

// empties the slots a layer used (the last layer of a minibatch has no later relabel to do it)
__global__ void __launch_bounds__(kThreads)
layer_sweep_kernel(PackedTable t, const uint32_t* __restrict__ pos, RankCounts n) {
  int64_t S, M;
  n.get(&S, &M);
  const int64_t j = static_cast<int64_t>(blockIdx.x) * kThreads + threadIdx.x;
  if (j < M) t.clear(pos[j] & t.mask);
}

// ------------------------------------------------ batched (super-batch) relabel ----
// B independent relabels in one pass: replaces impl::BatchCSRRelabelCUDA (reference
// src/cuda/batch_relabel.cu:331; kernels :90-232).  Batch b owns seeds
// [seeds_ptr[b], seeds_ptr[b+1]) and ids [indices_ptr[b], indices_ptr[b+1]); its
// frontier is the distinct values of (its seeds, then its ids) in first-occurrence
// order, the frontiers are concatenated by batch, and every id is renamed to its
// rank inside its own batch's frontier.
//
//  * The items are laid out virtually as [seeds_0, ids_0, seeds_1, ids_1, ...]
//    (the order the reference's prefix array has, batch_relabel.cu:152,163), so
//    one insert pass, one chained-scan compaction and one lookup pass serve all
//    batches.
//  * Like the reference, every batch hashes into a region of its own
//    (batch_relabel.cu:243-256), here twice its item count, carved out of one
//    array at 2 * start(b) with no size rounded to a power of two (the home slot
//    is a multiply-high of the hash by the region length).  Regions matter for
//    locality: consecutive items belong to the same batch, so the slots the chip
//    is hammering at any moment span a few megabytes instead of the whole table
//    (64 minibatches of layer 3: 270 MB), and the key needs no batch number, so
//    32-bit ids keep the one-word (key | first index) slot and its single CAS.
//  * A workgroup's items span one or two batches; it looks the range up once and
//    its lanes search inside it.
constexpr int64_t kRegionFactor = 2;

// one region per batch, slots (key << 32 | first index), all ones = empty
struct PackedRegions {
  unsigned long long* slots;
  static size_t bytes(int64_t cap) { return padded(cap * 8); }
  void carve(Carver& ws, int64_t cap) { slots = ws.take<unsigned long long>(cap); }
  __device__ __forceinline__ void clear(int64_t i) const { slots[i] = ~0ull; }
  __device__ __forceinline__ uint32_t insert(int64_t begin, int64_t len, long long key,
                                             uint32_t i) const {
    const unsigned long long hi = static_cast<unsigned long long>(static_cast<uint32_t>(key)) << 32;
    const unsigned long long word = hi | i;
    int64_t p = begin + static_cast<int64_t>((static_cast<unsigned long long>(hash32(
                                                  static_cast<uint32_t>(key))) *
                                              static_cast<unsigned long long>(len)) >>
                                             32);
    while (true) {
      // a look before the compare-and-swap: a slot that is taken needs none
      unsigned long long prev = __hip_atomic_load(&slots[p], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      if (prev == ~0ull) prev = atomicCAS(&slots[p], ~0ull, word);
      if (prev == ~0ull) break;
      if ((prev >> 32) == (hi >> 32)) {
        if (static_cast<uint32_t>(prev) > i) atomicMin(&slots[p], word);
        break;
      }
      if (++p == begin + len) p = begin;
    }
    return static_cast<uint32_t>(p);
  }
  __device__ __forceinline__ uint32_t first_index(uint32_t p) const {
    return static_cast<uint32_t>(slots[p]);
  }
  // slot of a key that may be absent (0xFFFFFFFF then); the region is never full
  __device__ __forceinline__ uint32_t find(int64_t begin, int64_t len, long long key) const {
    const unsigned long long hi = static_cast<uint32_t>(key);
    int64_t p = begin + static_cast<int64_t>((static_cast<unsigned long long>(hash32(
                                                  static_cast<uint32_t>(key))) *
                                              static_cast<unsigned long long>(len)) >>
                                             32);
    while (true) {
      const unsigned long long w = slots[p];
      if (w == ~0ull) return 0xFFFFFFFFu;
      if ((w >> 32) == hi) return static_cast<uint32_t>(p);
      if (++p == begin + len) p = begin;
    }
  }
};

// the same with 64-bit keys: key array (-1 = empty) + first-index array
struct WideRegions {
  long long* keys;
  int* vals;
  static size_t bytes(int64_t cap) { return padded(cap * 8) + padded(cap * 4); }
  void carve(Carver& ws, int64_t cap) {
    keys = ws.take<long long>(cap);
    vals = ws.take<int>(cap);
  }
  __device__ __forceinline__ void clear(int64_t i) const {
    keys[i] = -1;
    vals[i] = 0x7fffffff;
  }
  __device__ __forceinline__ uint32_t insert(int64_t begin, int64_t len, long long key,
                                             uint32_t i) const {
    int64_t p = begin + static_cast<int64_t>((static_cast<unsigned long long>(hash32(
                                                  static_cast<unsigned long long>(key))) *
                                              static_cast<unsigned long long>(len)) >>
                                             32);
    while (true) {
      const unsigned long long prev =
          atomicCAS(reinterpret_cast<unsigned long long*>(&keys[p]), ~0ull,
                    static_cast<unsigned long long>(key));
      if (prev == ~0ull || prev == static_cast<unsigned long long>(key)) break;
      if (++p == begin + len) p = begin;
    }
    if (__atomic_load_n(&vals[p], __ATOMIC_RELAXED) > static_cast<int>(i))
      atomicMin(&vals[p], static_cast<int>(i));
    return static_cast<uint32_t>(p);
  }
  __device__ __forceinline__ uint32_t first_index(uint32_t p) const {
    return static_cast<uint32_t>(vals[p]);
  }
  __device__ __forceinline__ uint32_t find(int64_t begin, int64_t len, long long key) const {
    int64_t p = begin + static_cast<int64_t>((static_cast<unsigned long long>(hash32(
                                                  static_cast<unsigned long long>(key))) *
                                              static_cast<unsigned long long>(len)) >>
                                             32);
    while (true) {
      const long long cur = keys[p];
      if (cur == -1) return 0xFFFFFFFFu;
      if (cur == key) return static_cast<uint32_t>(p);
      if (++p == begin + len) p = begin;
    }
  }
};

template <typename IdT>
struct RegionsFor {
  using type = WideRegions;
};
template <>
struct RegionsFor<int32_t> {
  using type = PackedRegions;
};

template <typename R>
__global__ void __launch_bounds__(kThreads) regions_init_kernel(R t, int64_t cap, LookbackState lb,
                                                                int64_t tiles) {
  const int64_t i = static_cast<int64_t>(blockIdx.x) * kThreads + threadIdx.x;
  if (i < cap) t.clear(i);
  if (i < tiles) lb.status[i] = 0ull;
  if (i == 0) *lb.error = 0u;
}

template <typename IdT, typename R>
__global__ void __launch_bounds__(kThreads)
batch_insert_kernel(BatchItems<IdT> x, int64_t M, R t, uint32_t* __restrict__ pos,
                    unsigned int* __restrict__ too_wide) {
  __shared__ int64_t s_range[2];
  __shared__ int64_t s_seeds_ptr[kStagedBatches + 1], s_ids_ptr[kStagedBatches + 1];
  x.stage_offsets(s_seeds_ptr, s_ids_ptr);
  const int64_t first = static_cast<int64_t>(blockIdx.x) * kThreads;
  const int64_t last = first + kThreads - 1 < M ? first + kThreads - 1 : M - 1;
  int64_t lo, hi;
  x.block_range(first, last, s_range, &lo, &hi);
  const int64_t i = first + threadIdx.x;
  if (i >= M) return;
  const int64_t b = x.batch_of(i, lo, hi);
  const int64_t begin = x.start(b);
  const IdT key = x.get_in(b, i);
  if (sizeof(IdT) == 8 && too_wide && (static_cast<unsigned long long>(key) >> 32) != 0ull) {
    *too_wide = 2u;  // 64-bit ids on one-word slots, and this one does not fit: reported as -2
    pos[i] = static_cast<uint32_t>(kRegionFactor * begin);
    return;
  }
  pos[i] = t.insert(kRegionFactor * begin, kRegionFactor * (x.start(b + 1) - begin),
                    static_cast<long long>(key), static_cast<uint32_t>(i));
}

// flags, chained scan and compaction over all batches at once (see compact_kernel)
template <typename IdT, typename R>
__global__ void __launch_bounds__(kThreads)
batch_compact_kernel(BatchItems<IdT> x, int64_t M, R t, uint32_t* __restrict__ pos,
                     int64_t* __restrict__ prefix, IdT* __restrict__ unique,
                     int64_t* __restrict__ num_unique, LookbackState lb, gs_mailbox* box,
                     int64_t box_ticket) {
  __shared__ int64_t s_scan[kThreads / kWave + 1];
  __shared__ int64_t s_prefix;
  __shared__ int64_t s_range[2];
  __shared__ int64_t s_seeds_ptr[kStagedBatches + 1], s_ids_ptr[kStagedBatches + 1];
  x.stage_offsets(s_seeds_ptr, s_ids_ptr);
  const unsigned int tile = blockIdx.x;
  const int64_t tile_first = static_cast<int64_t>(tile) * kCompactTile;
  const int64_t tile_last = tile_first + kCompactTile - 1 < M ? tile_first + kCompactTile - 1 : M - 1;
  int64_t lo = 0, hi = 0;
  if (M > 0) x.block_range(tile_first, tile_last, s_range, &lo, &hi);
  const int64_t base = tile_first + static_cast<int64_t>(threadIdx.x) * kCompactItems;
  bool first[kCompactItems];
  int64_t mine = 0;
  // The slots' words are read here once, eight trips in flight together: from now on pos[i]
  // is the index of the first occurrence of item i's key, and the lookups of the last pass
  // need no second trip to the table.
  // All reads carry no condition of their own (the last item again past the end; a read that
  // may or may not happen makes every later one wait for all that is in flight), and every
  // read of the thread's eight items stands before its first store.
  uint32_t at[kCompactItems], fi[kCompactItems];
  IdT key[kCompactItems];
#pragma unroll
  for (int k = 0; k < kCompactItems; ++k) at[k] = fi[k] = 0u;
  if (M > 0) {
    const IdT* from[kCompactItems];
#pragma unroll
    for (int k = 0; k < kCompactItems; ++k) {
      const int64_t i = base + k < M ? base + k : M - 1;
      at[k] = pos[i];
      from[k] = x.where_in(x.batch_of(i, lo, hi), i);
    }
#pragma unroll
    for (int k = 0; k < kCompactItems; ++k) {
      fi[k] = t.first_index(at[k]);
      key[k] = *from[k];  // in flight while wave 0 walks back
    }
  }
#pragma unroll
  for (int k = 0; k < kCompactItems; ++k) {
    const int64_t i = base + k;
    first[k] = i < M && fi[k] == static_cast<uint32_t>(i);
    mine += first[k] ? 1 : 0;
  }
  int64_t tile_total;
  const int64_t local = block_exclusive_scan<kThreads>(mine, &tile_total, s_scan);
  if (threadIdx.x == 0) lookback_publish_sum(lb, tile, tile_total);
#pragma unroll
  for (int k = 0; k < kCompactItems; ++k)
    if (base + k < M) pos[base + k] = fi[k];
  if (threadIdx.x < kWave) {
    const int64_t before = lookback_exclusive_prefix(lb, tile, tile_total);
    if (threadIdx.x == 0) s_prefix = before;
  }
  __syncthreads();
  int64_t run = s_prefix + local;
#pragma unroll
  for (int k = 0; k < kCompactItems; ++k) {
    const int64_t i = base + k;
    if (i < M) {
      prefix[i] = run;
      if (first[k]) unique[run] = key[k];
    }
    run += first[k] ? 1 : 0;
  }
  if (tile == gridDim.x - 1 && threadIdx.x == 0) {
    int64_t total = s_prefix + tile_total;
    const unsigned int err = __hip_atomic_load(lb.error, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    if (err) total = err == 2u ? -2 : -1;
    *num_unique = total;
    post_mailbox(box, total, box_ticket);
  }
}

// ids -> rank inside their batch's frontier; unique_ptr[b] = frontier offset of batch b
template <typename IdT, typename R>
__global__ void __launch_bounds__(kThreads)
batch_finish_kernel(BatchItems<IdT> x, int64_t num_ids, int64_t M, R t,
                    const uint32_t* __restrict__ pos, const int64_t* __restrict__ prefix,
                    const int64_t* __restrict__ num_unique, IdT* __restrict__ out_ids,
                    int64_t* __restrict__ unique_ptr, const IdT* __restrict__ extra,
                    IdT* __restrict__ out_extra) {
  __shared__ int64_t s_range[2];
  __shared__ int64_t s_seeds_ptr[kStagedBatches + 1], s_ids_ptr[kStagedBatches + 1];
  x.stage_offsets(s_seeds_ptr, s_ids_ptr);
  const int64_t first = static_cast<int64_t>(blockIdx.x) * kThreads;
  if (first < num_ids) {  // a workgroup of id lookups
    const int64_t last = first + kThreads - 1 < num_ids ? first + kThreads - 1 : num_ids - 1;
    if (threadIdx.x < 2) {
      const int64_t j = threadIdx.x == 0 ? first : last;
      int64_t lo = 0, hi = x.B - 1;  // last b with ids_ptr[b] <= j
      while (lo < hi) {
        const int64_t mid = (lo + hi + 1) >> 1;
        if (x.ids_ptr[mid] <= j) lo = mid; else hi = mid - 1;
      }
      s_range[threadIdx.x] = lo;
    }
    __syncthreads();
    const int64_t j = first + threadIdx.x;
    if (j >= num_ids) return;
    int64_t lo = s_range[0], hi = s_range[1];
    while (lo < hi) {
      const int64_t mid = (lo + hi + 1) >> 1;
      if (x.ids_ptr[mid] <= j) lo = mid; else hi = mid - 1;
    }
    const int64_t b = lo;
    const int64_t begin = x.start(b);
    const int64_t p = begin + (x.seeds_ptr[b + 1] - x.seeds_ptr[b]) + (j - x.ids_ptr[b]);
    // pos holds first-occurrence indices since the compaction.  An index beyond M only when
    // the insert pass gave up (an id too wide for the slots): the outputs are void then, but
    // no index may leave the arrays
    const uint32_t fi = pos[p];
    out_ids[j] = static_cast<IdT>(fi < M ? prefix[fi] - prefix[begin] : -1);
    if (extra) {
      // a second array cut like the ids (the other end of a COO edge): looked up, -1 if absent
      const bool fits = sizeof(IdT) == 4 || !std::is_same<R, PackedRegions>::value ||
                        (static_cast<unsigned long long>(extra[j]) >> 32) == 0ull;
      const uint32_t slot =
          fits ? t.find(kRegionFactor * begin, kRegionFactor * (x.start(b + 1) - begin),
                        static_cast<long long>(extra[j]))
               : 0xFFFFFFFFu;
      const uint32_t fe = slot == 0xFFFFFFFFu ? 0xFFFFFFFFu : t.first_index(slot);
      out_extra[j] = fe < M ? static_cast<IdT>(prefix[fe] - prefix[begin]) : IdT(-1);
    }
    return;
  }
  const int64_t b = first + threadIdx.x - (num_ids + kThreads - 1) / kThreads * kThreads;
  if (b <= x.B) unique_ptr[b] = x.start(b) < M ? prefix[x.start(b)] : *num_unique;
}

template <typename IdT>
size_t batch_workspace_bytes_for(int64_t M) {
  using R = typename RegionsFor<IdT>::type;
  return R::bytes(kRegionFactor * (M > 0 ? M : 1)) + padded((M > 0 ? M : 1) * 4) +
         padded((M + 1) * 8) + lookback_state_bytes(compact_num_tiles(M));
}

template <typename IdT, typename R>
int batch_relabel_impl(const void* seeds, const int64_t* seeds_ptr, const void* ids,
                       const int64_t* ids_ptr, int64_t B, int64_t num_seeds, int64_t num_ids,
                       void* unique, int64_t* unique_ptr, void* out_ids, int64_t* num_unique,
                       void* workspace, size_t workspace_bytes, gs_mailbox* box,
                       int64_t box_ticket, hipStream_t stream, const void* extra = nullptr,
                       void* out_extra = nullptr) {
  const int64_t M = num_seeds + num_ids;
  const int64_t cap = kRegionFactor * (M > 0 ? M : 1);
  Carver ws(workspace, workspace_bytes);
  R t;
  t.carve(ws, cap);
  uint32_t* pos = ws.take<uint32_t>(M > 0 ? M : 1);
  int64_t* prefix = ws.take<int64_t>(M + 1);
  const int64_t tiles = compact_num_tiles(M);
  LookbackState lb = carve_lookback(ws, tiles, 1u);
  if (!ws.ok) {
    set_error_text("gs_batch_csr_relabel: workspace needs %zu bytes, 256-byte aligned",
                   batch_workspace_bytes_for<IdT>(M));
    return GS_ERR_WORKSPACE;
  }
  BatchItems<IdT> x{static_cast<const IdT*>(seeds), seeds_ptr, static_cast<const IdT*>(ids), ids_ptr,
                    B};
  const int64_t n_init = cap > tiles ? cap : tiles;
  {
    ProfileScope prof("batch_init", stream);
    hipLaunchKernelGGL((regions_init_kernel<R>), dim3(blocks_for(n_init, kThreads)),
                       dim3(kThreads), 0, stream, t, cap, lb, tiles);
  }
  if (M > 0) {
    ProfileScope prof("batch_insert", stream);
    hipLaunchKernelGGL((batch_insert_kernel<IdT, R>), dim3(blocks_for(M, kThreads)), dim3(kThreads),
                       0, stream, x, M, t, pos,
                       sizeof(IdT) == 8 && std::is_same<R, PackedRegions>::value
                           ? lb.error
                           : static_cast<unsigned int*>(nullptr));
  }
  {
    ProfileScope prof("batch_compact", stream);
    hipLaunchKernelGGL((batch_compact_kernel<IdT, R>), dim3(static_cast<unsigned>(tiles)),
                       dim3(kThreads), 0, stream, x, M, t, pos, prefix, static_cast<IdT*>(unique),
                       num_unique, lb, box, box_ticket);
  }
  const int64_t id_blocks = (num_ids + kThreads - 1) / kThreads;
  const int64_t ptr_blocks = (B + 1 + kThreads - 1) / kThreads;
  ProfileScope prof("batch_finish", stream);
  hipLaunchKernelGGL((batch_finish_kernel<IdT, R>), dim3(static_cast<unsigned>(id_blocks + ptr_blocks)),
                     dim3(kThreads), 0, stream, x, num_ids, M, t, pos, prefix, num_unique,
                     static_cast<IdT*>(out_ids), unique_ptr, static_cast<const IdT*>(extra),
                     static_cast<IdT*>(out_extra));
  return check_launch("batch_csr_relabel");
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

int gs_unique_relabel_notify(const gs_span* mapping, int n_mapping, const gs_span* query,
                             void* const* query_out, int n_query, int id_bytes, void* frontier,
                             int64_t* num_unique, void* workspace, size_t workspace_bytes,
                             const int64_t* last_span_len, gs_mailbox* mailbox,
                             int64_t mailbox_ticket, void* stream) {
  GS_REQUIRE(mapping && n_mapping >= 1 && n_mapping <= GS_MAX_SPANS,
             "gs_unique_relabel: 1..%d mapping spans required, got %d", GS_MAX_SPANS, n_mapping);
  GS_REQUIRE(n_query >= 0 && n_query <= GS_MAX_SPANS && (n_query == 0 || (query && query_out)),
             "gs_unique_relabel: 0..%d query spans required, got %d", GS_MAX_SPANS, n_query);
  const bool narrow = (id_bytes & GS_NARROW_IDS) != 0;
  id_bytes &= ~GS_NARROW_IDS;
  GS_REQUIRE(valid_id_bytes(id_bytes) && (!narrow || id_bytes == 8),
             "gs_unique_relabel: id_bytes must be 4, 8 or 8 | GS_NARROW_IDS, got %d", id_bytes);
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
  if (last_span_len) {
    const gs_span& last = mapping[n_mapping - 1];
    GS_REQUIRE(n_query == 0 || (n_query == 1 && query[0].ptr == last.ptr && query[0].n == last.n),
               "gs_unique_relabel_notify: with a device-side length the only query allowed is "
               "the last mapping span itself");
  }
  hipStream_t st = static_cast<hipStream_t>(stream);
  if (id_bytes == 4)
    return unique_relabel_impl<int32_t, PackedTable>(mapping, n_mapping, query, query_out, n_query,
                                                     frontier, num_unique, workspace,
                                                     workspace_bytes, last_span_len, mailbox,
                                                     mailbox_ticket, st);
  return narrow ? unique_relabel_impl<int64_t, PackedTable>(mapping, n_mapping, query, query_out,
                                                            n_query, frontier, num_unique, workspace,
                                                            workspace_bytes, last_span_len, mailbox,
                                                            mailbox_ticket, st)
                : unique_relabel_impl<int64_t, WideTable>(mapping, n_mapping, query, query_out,
                                                          n_query, frontier, num_unique, workspace,
                                                          workspace_bytes, last_span_len, mailbox,
                                                          mailbox_ticket, st);
}

int gs_unique_relabel(const gs_span* mapping, int n_mapping, const gs_span* query,
                      void* const* query_out, int n_query, int id_bytes, void* frontier,
                      int64_t* num_unique, void* workspace, size_t workspace_bytes,
                      void* stream) {
  return gs_unique_relabel_notify(mapping, n_mapping, query, query_out, n_query, id_bytes, frontier,
                                  num_unique, workspace, workspace_bytes, nullptr, nullptr, 0,
                                  stream);
}

size_t gs_batch_relabel_workspace_bytes(int64_t num_items) {
  if (num_items < 0) num_items = 0;
  const size_t a = batch_workspace_bytes_for<int64_t>(num_items);
  const size_t b = batch_workspace_bytes_for<int32_t>(num_items);
  const size_t c = binned_relabel_workspace_bytes(num_items, kStagedBatches);
  return a > b ? (a > c ? a : c) : (b > c ? b : c);
}

size_t gs_batch_relabel_bins_workspace_bytes(int64_t num_items, int64_t num_batches) {
  return binned_relabel_workspace_bytes(num_items, num_batches);
}

int gs_batch_csr_relabel(const void* seeds, const int64_t* seeds_ptr, const void* ids,
                         const int64_t* ids_ptr, int64_t num_batches, int64_t num_seeds,
                         int64_t num_ids, int id_bytes, void* unique, int64_t* unique_ptr,
                         void* out_ids, int64_t* num_unique, void* workspace,
                         size_t workspace_bytes, gs_mailbox* mailbox, int64_t mailbox_ticket,
                         void* stream) {
  GS_REQUIRE(num_batches >= 1 && num_seeds >= 0 && num_ids >= 0,
             "gs_batch_csr_relabel: at least one batch and non-negative sizes required");
  GS_REQUIRE(seeds_ptr && ids_ptr && unique_ptr && num_unique, "gs_batch_csr_relabel: null pointer");
  GS_REQUIRE((num_seeds == 0 || seeds) && (num_ids == 0 || (ids && out_ids)) &&
                 (num_seeds + num_ids == 0 || unique),
             "gs_batch_csr_relabel: null buffer");
  const bool narrow = (id_bytes & GS_NARROW_IDS) != 0;
  const bool want_regions = (id_bytes & GS_RELABEL_REGIONS) != 0;
  const bool want_bins = (id_bytes & GS_RELABEL_BINS) != 0;
  id_bytes &= ~(GS_NARROW_IDS | GS_RELABEL_REGIONS | GS_RELABEL_BINS);
  GS_REQUIRE(valid_id_bytes(id_bytes) && (!narrow || id_bytes == 8),
             "gs_batch_csr_relabel: id_bytes must be 4, 8 or 8 | GS_NARROW_IDS, got %d", id_bytes);
  GS_REQUIRE(!(want_regions && want_bins),
             "gs_batch_csr_relabel: GS_RELABEL_REGIONS and GS_RELABEL_BINS exclude each other");
  if (num_seeds + num_ids >= (int64_t(1) << 30)) {
    set_error_text("gs_batch_csr_relabel: %lld items exceed the supported 2^30",
                   static_cast<long long>(num_seeds + num_ids));
    return GS_ERR_UNSUPPORTED;
  }
  hipStream_t st = static_cast<hipStream_t>(stream);
  // ids that ride in 32 bits go through the bins from about half a million items on
  const bool can_bin = (id_bytes == 4 || narrow) && num_seeds + num_ids > 0 &&
                       num_batches <= kStagedBatches;
  if (want_bins && !can_bin) {
    set_error_text("gs_batch_csr_relabel: GS_RELABEL_BINS needs ids that fit 32 bits, at least "
                   "one item and at most %lld batches", static_cast<long long>(kStagedBatches));
    return GS_ERR_UNSUPPORTED;
  }
  if (can_bin && !want_regions &&
      (want_bins || binned_relabel_applies(num_seeds + num_ids, num_batches)))
    return batch_relabel_binned(seeds, seeds_ptr, ids, ids_ptr, num_batches, num_seeds, num_ids,
                                id_bytes, unique, unique_ptr, out_ids, num_unique, workspace,
                                workspace_bytes, mailbox, mailbox_ticket, st);
  if (id_bytes == 4)
    return batch_relabel_impl<int32_t, PackedRegions>(
        seeds, seeds_ptr, ids, ids_ptr, num_batches, num_seeds, num_ids, unique, unique_ptr, out_ids,
        num_unique, workspace, workspace_bytes, mailbox, mailbox_ticket, st);
  return narrow ? batch_relabel_impl<int64_t, PackedRegions>(
                      seeds, seeds_ptr, ids, ids_ptr, num_batches, num_seeds, num_ids, unique,
                      unique_ptr, out_ids, num_unique, workspace, workspace_bytes, mailbox,
                      mailbox_ticket, st)
                : batch_relabel_impl<int64_t, WideRegions>(
                      seeds, seeds_ptr, ids, ids_ptr, num_batches, num_seeds, num_ids, unique,
                      unique_ptr, out_ids, num_unique, workspace, workspace_bytes, mailbox,
                      mailbox_ticket, st);
}

int gs_batch_coo_relabel(const void* seeds, const int64_t* seeds_ptr, const void* coo_row,
                         const void* coo_col, const int64_t* coo_ptr, int64_t num_batches,
                         int64_t num_seeds, int64_t num_edges, int id_bytes, void* unique,
                         int64_t* unique_ptr, void* out_row, void* out_col, int64_t* num_unique,
                         void* workspace, size_t workspace_bytes, gs_mailbox* mailbox,
                         int64_t mailbox_ticket, void* stream) {
  GS_REQUIRE(num_batches >= 1 && num_seeds >= 0 && num_edges >= 0,
             "gs_batch_coo_relabel: at least one batch and non-negative sizes required");
  GS_REQUIRE(seeds_ptr && coo_ptr && unique_ptr && num_unique, "gs_batch_coo_relabel: null pointer");
  GS_REQUIRE((num_seeds == 0 || seeds) &&
                 (num_edges == 0 || (coo_row && coo_col && out_row && out_col)) &&
                 (num_seeds + num_edges == 0 || unique),
             "gs_batch_coo_relabel: null buffer");
  const bool narrow = (id_bytes & GS_NARROW_IDS) != 0;
  id_bytes &= ~GS_NARROW_IDS;
  GS_REQUIRE(valid_id_bytes(id_bytes) && (!narrow || id_bytes == 8),
             "gs_batch_coo_relabel: id_bytes must be 4, 8 or 8 | GS_NARROW_IDS, got %d", id_bytes);
  if (num_seeds + num_edges >= (int64_t(1) << 30)) {
    set_error_text("gs_batch_coo_relabel: %lld items exceed the supported 2^30",
                   static_cast<long long>(num_seeds + num_edges));
    return GS_ERR_UNSUPPORTED;
  }
  hipStream_t st = static_cast<hipStream_t>(stream);
  if (id_bytes == 4)
    return batch_relabel_impl<int32_t, PackedRegions>(
        seeds, seeds_ptr, coo_row, coo_ptr, num_batches, num_seeds, num_edges, unique, unique_ptr,
        out_row, num_unique, workspace, workspace_bytes, mailbox, mailbox_ticket, st, coo_col,
        out_col);
  return narrow ? batch_relabel_impl<int64_t, PackedRegions>(
                      seeds, seeds_ptr, coo_row, coo_ptr, num_batches, num_seeds, num_edges, unique,
                      unique_ptr, out_row, num_unique, workspace, workspace_bytes, mailbox,
                      mailbox_ticket, st, coo_col, out_col)
                : batch_relabel_impl<int64_t, WideRegions>(
                      seeds, seeds_ptr, coo_row, coo_ptr, num_batches, num_seeds, num_edges, unique,
                      unique_ptr, out_row, num_unique, workspace, workspace_bytes, mailbox,
                      mailbox_ticket, st, coo_col, out_col);
}

size_t gs_relabel_table_bytes(int64_t max_items, int id_bytes) {
  if (max_items < 1) max_items = 1;
  const int64_t cap = linked_table_capacity(max_items);
  return id_bytes == 4 ? PackedTable::bytes(cap) : WideTable::bytes(cap);
}

int gs_relabel_table_init(void* table, size_t table_bytes, int id_bytes, void* stream) {
  GS_REQUIRE(table, "gs_relabel_table_init: null pointer");
  GS_REQUIRE(valid_id_bytes(id_bytes), "gs_relabel_table_init: id_bytes must be 4 or 8, got %d",
             id_bytes);
  hipStream_t st = static_cast<hipStream_t>(stream);
  if (id_bytes == 4) {
    const int64_t cap = linked_table_slots<PackedTable>(table_bytes);
    PackedTable t;
    GS_REQUIRE(cap > 0 && shape_linked_table<PackedTable>(table, table_bytes, cap / (2 * kLinkedFactor), &t),
               "gs_relabel_table_init: buffer too small or misaligned");
    hipLaunchKernelGGL(table_clear_kernel<PackedTable>, dim3(blocks_for(cap, kThreads)),
                       dim3(kThreads), 0, st, t, cap);
  } else {
    const int64_t cap = linked_table_slots<WideTable>(table_bytes);
    WideTable t;
    GS_REQUIRE(cap > 0 && shape_linked_table<WideTable>(table, table_bytes, cap / (2 * kLinkedFactor), &t),
               "gs_relabel_table_init: buffer too small or misaligned");
    hipLaunchKernelGGL(table_clear_kernel<WideTable>, dim3(blocks_for(cap, kThreads)),
                       dim3(kThreads), 0, st, t, cap);
  }
  return check_launch("relabel_table_init");
}

size_t gs_layer_workspace_bytes(int64_t S_bound, int64_t fanout) {
  if (S_bound < 0) S_bound = 0;
  if (fanout < 0) fanout = 0;
  return layer_workspace_bytes(S_bound + S_bound * fanout);
}

namespace {
// look-back status words, then the tiles' distance words (one per four items)
inline size_t layer_relabel_state_bytes(int64_t items) {
  return gs::lookback_state_bytes(gs::compact_num_tiles(items)) +
         gs::padded(static_cast<size_t>(items / 4 + 2) * 8);
}
}  // namespace

size_t gs_layer_relabel_state_bytes(int64_t S_bound, int64_t fanout) {
  if (S_bound < 0) S_bound = 0;
  if (fanout < 0) fanout = 0;
  return layer_relabel_state_bytes(S_bound + S_bound * fanout);
}

int gs_layer_relabel(int id_bytes, int64_t S_bound, const int64_t* S_dev, int64_t capacity,
                     const int64_t* num_edges, const int64_t* sub_indptr, void* table,
                     size_t table_bytes, void* workspace, size_t workspace_bytes, void* frontier,
                     void* out_ids, int64_t* num_unique, int64_t* offsets_copy, void* state,
                     size_t state_bytes, uint32_t epoch, void* prev_table, size_t prev_table_bytes,
                     const void* prev_workspace, size_t prev_workspace_bytes, int64_t prev_S_bound,
                     const int64_t* prev_S_dev, int64_t prev_capacity,
                     const int64_t* prev_num_edges, gs_mailbox* mailbox, int64_t mailbox_ticket,
                     void* stream) {
  GS_REQUIRE(S_bound >= 0 && capacity >= 0 && num_edges && table && workspace && num_unique && state,
             "gs_layer_relabel: null pointer or negative size");
  GS_REQUIRE(valid_id_bytes(id_bytes), "gs_layer_relabel: id_bytes must be 4 or 8, got %d", id_bytes);
  GS_REQUIRE((capacity == 0 || out_ids) && (S_bound + capacity == 0 || frontier),
             "gs_layer_relabel: null buffer");
  GS_REQUIRE(!offsets_copy || sub_indptr, "gs_layer_relabel: offsets_copy without sub_indptr");
  GS_REQUIRE(epoch >= 1 && epoch <= kLbMaxEpoch, "gs_layer_relabel: epoch must be in 1..%u",
             kLbMaxEpoch);
  const int64_t M_bound = S_bound + capacity;
  if (M_bound >= (int64_t(1) << 31)) {
    set_error_text("gs_layer_relabel: %lld items exceed the supported 2^31",
                   static_cast<long long>(M_bound));
    return GS_ERR_UNSUPPORTED;
  }
  PackedTable t, prev_t;
  prev_t.slots = nullptr;
  prev_t.mask = 0;
  prev_t.shift = 0;
  if (!shape_linked_table<PackedTable>(table, table_bytes, M_bound, &t)) {
    set_error_text("gs_layer_relabel: the table holds fewer than the %lld slots this call needs "
                   "(or is misaligned)",
                   static_cast<long long>(linked_table_capacity(M_bound)));
    return GS_ERR_WORKSPACE;
  }
  uint32_t* pos = nullptr;
  Carver sc(state, state_bytes);
  LookbackState lb = carve_lookback(sc, compact_num_tiles(M_bound), epoch);
  unsigned long long* back = sc.take<unsigned long long>(static_cast<size_t>(M_bound / 4 + 2));
  if (!carve_layer_workspace(workspace, workspace_bytes, M_bound, &pos) || !sc.ok) {
    set_error_text("gs_layer_relabel: workspace needs %zu bytes and state %zu bytes, 256-byte "
                   "aligned", layer_workspace_bytes(M_bound), layer_relabel_state_bytes(M_bound));
    return GS_ERR_WORKSPACE;
  }
  uint32_t* prev_pos = nullptr;
  const int64_t prev_bound = prev_S_bound + prev_capacity;
  if (prev_table) {
    GS_REQUIRE(prev_table != table, "gs_layer_relabel: the table to empty must be another table");
    GS_REQUIRE(prev_workspace && prev_num_edges && prev_S_bound >= 0 && prev_capacity >= 0,
               "gs_layer_relabel: the table to empty needs its layer's workspace and counts");
    if (!shape_linked_table<PackedTable>(prev_table, prev_table_bytes, prev_bound, &prev_t) ||
        !carve_layer_workspace(const_cast<void*>(prev_workspace), prev_workspace_bytes, prev_bound,
                               &prev_pos)) {
      set_error_text("gs_layer_relabel: the table to empty or its workspace is smaller than its "
                     "layer needed");
      return GS_ERR_WORKSPACE;
    }
  }
  hipStream_t st = static_cast<hipStream_t>(stream);
  const RankCounts n{S_bound, S_dev, capacity, num_edges};
  const RankCounts pn{prev_S_bound, prev_S_dev, prev_capacity, prev_num_edges};
  const dim3 grid(static_cast<unsigned>(compact_num_tiles(M_bound)));
  ProfileScope prof("layer_relabel", st);
  if (id_bytes == 8) {
    RankArgs<int64_t> a{t, pos, n, back, static_cast<int64_t*>(frontier),
                        static_cast<int64_t*>(out_ids), num_unique, sub_indptr, offsets_copy, lb,
                        mailbox, mailbox_ticket, prev_t, prev_pos, pn};
    hipLaunchKernelGGL((rank_linked_kernel<int64_t>), grid, dim3(kThreads), 0, st, a);
    return check_launch("layer_relabel");
  }
  RankArgs<int32_t> a{t, pos, n, back, static_cast<int32_t*>(frontier),
                      static_cast<int32_t*>(out_ids), num_unique, sub_indptr, offsets_copy, lb,
                      mailbox, mailbox_ticket, prev_t, prev_pos, pn};
  hipLaunchKernelGGL((rank_linked_kernel<int32_t>), grid, dim3(kThreads), 0, st, a);
  return check_launch("layer_relabel");
}

int gs_layer_table_sweep(void* table, size_t table_bytes, const void* workspace,
                         size_t workspace_bytes, int64_t S_bound, const int64_t* S_dev,
                         int64_t capacity, const int64_t* num_edges, void* stream) {
  GS_REQUIRE(table && workspace && num_edges && S_bound >= 0 && capacity >= 0,
             "gs_layer_table_sweep: null pointer or negative size");
  const int64_t M_bound = S_bound + capacity;
  PackedTable t;
  uint32_t* pos = nullptr;
  if (!shape_linked_table<PackedTable>(table, table_bytes, M_bound, &t) ||
      !carve_layer_workspace(const_cast<void*>(workspace), workspace_bytes, M_bound, &pos)) {
    set_error_text("gs_layer_table_sweep: the table or the workspace is smaller than the layer needed");
    return GS_ERR_WORKSPACE;
  }
  if (M_bound == 0) return GS_OK;
  const RankCounts n{S_bound, S_dev, capacity, num_edges};
  ProfileScope prof("layer_sweep", static_cast<hipStream_t>(stream));
  hipLaunchKernelGGL(layer_sweep_kernel, dim3(blocks_for(M_bound, kThreads)), dim3(kThreads), 0,
                     static_cast<hipStream_t>(stream), t, pos, n);
  return check_launch("layer_table_sweep");
}

size_t gs_relabel_sampled_workspace_bytes(int64_t num_items) {
  if (num_items < 1) num_items = 1;
  return padded(static_cast<size_t>(num_items + 1) * 8) +
         2 * padded(static_cast<size_t>(num_items) * 4);
}

size_t gs_relabel_sampled_state_bytes(int64_t num_items) {
  return lookback_state_bytes(compact_num_tiles(num_items));
}

int gs_relabel_sampled(const void* seed_keys, int64_t S, const void* sampled, int64_t capacity,
                       const int64_t* sampled_len, int id_bytes, void* table, size_t table_bytes,
                       void* frontier, void* out_ids, int64_t* num_unique,
                       int64_t* offsets_copy, void* workspace,
                       size_t workspace_bytes, void* state, size_t state_bytes, uint32_t epoch,
                       gs_mailbox* mailbox, int64_t mailbox_ticket, void* stream) {
  GS_REQUIRE(S >= 0 && capacity >= 0 && sampled_len && table && num_unique && state,
             "gs_relabel_sampled: null pointer or negative size");
  GS_REQUIRE((S == 0 || seed_keys) && (capacity == 0 || (sampled && out_ids)) &&
                 (S + capacity == 0 || frontier),
             "gs_relabel_sampled: null buffer");
  GS_REQUIRE(valid_id_bytes(id_bytes), "gs_relabel_sampled: id_bytes must be 4 or 8, got %d",
             id_bytes);
  GS_REQUIRE(epoch >= 1 && epoch <= kLbMaxEpoch, "gs_relabel_sampled: epoch must be in 1..%u",
             kLbMaxEpoch);
  if (S + capacity >= (int64_t(1) << 31)) {
    set_error_text("gs_relabel_sampled: %lld items exceed the supported 2^31",
                   static_cast<long long>(S + capacity));
    return GS_ERR_UNSUPPORTED;
  }
  hipStream_t st = static_cast<hipStream_t>(stream);
  return id_bytes == 8
             ? relabel_sampled_impl<int64_t, WideTable>(
                   seed_keys, S, sampled, capacity, sampled_len, table, table_bytes, frontier,
                   out_ids, num_unique, offsets_copy, workspace, workspace_bytes, state,
                   state_bytes, epoch, mailbox, mailbox_ticket, st)
             : relabel_sampled_impl<int32_t, PackedTable>(
                   seed_keys, S, sampled, capacity, sampled_len, table, table_bytes, frontier,
                   out_ids, num_unique, offsets_copy, workspace, workspace_bytes, state,
                   state_bytes, epoch, mailbox, mailbox_ticket, st);
}

int gs_relabel_sampled_narrow(const void* seed_keys, int64_t S, const void* sampled,
                              int64_t capacity, const int64_t* sampled_len, void* table,
                              size_t table_bytes, void* frontier, void* out_ids,
                              int64_t* num_unique, int64_t* offsets_copy, void* workspace,
                              size_t workspace_bytes, void* state, size_t state_bytes,
                              uint32_t epoch, gs_mailbox* mailbox, int64_t mailbox_ticket,
                              void* stream) {
  GS_REQUIRE(S >= 0 && capacity >= 0 && sampled_len && table && num_unique && state,
             "gs_relabel_sampled_narrow: null pointer or negative size");
  GS_REQUIRE((S == 0 || seed_keys) && (capacity == 0 || (sampled && out_ids)) &&
                 (S + capacity == 0 || frontier),
             "gs_relabel_sampled_narrow: null buffer");
  GS_REQUIRE(epoch >= 1 && epoch <= kLbMaxEpoch,
             "gs_relabel_sampled_narrow: epoch must be in 1..%u", kLbMaxEpoch);
  if (S + capacity >= (int64_t(1) << 31)) {
    set_error_text("gs_relabel_sampled_narrow: %lld items exceed the supported 2^31",
                   static_cast<long long>(S + capacity));
    return GS_ERR_UNSUPPORTED;
  }
  return relabel_sampled_impl<int64_t, PackedTable>(
      seed_keys, S, sampled, capacity, sampled_len, table, table_bytes, frontier, out_ids,
      num_unique, offsets_copy, workspace, workspace_bytes, state, state_bytes, epoch, mailbox,
      mailbox_ticket, static_cast<hipStream_t>(stream));
}

}  // extern "C"
