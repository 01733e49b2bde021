// Open-addressing hash tables of the unique / relabel kernels (first-occurrence index per
// key).
//
// capacity = power of two >= 2 * items, Fibonacci hashing, linear probing.  32-bit ids use
// ONE 64-bit word per slot, (key << 32 | first index): an insert is a single
// compare-and-swap in the common case and a duplicate lowers the index with a single
// atomicMin on the same word.  64-bit ids keep separate key (int64) and index (int32) arrays.
#pragma once

#include "gs_common.hpp"

namespace gs {

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
  // PEEK reads the slot first and leaves the compare-and-swap out when it is taken: worth a
  // load when keys repeat a lot (90 k edge ends over 1000 nodes queue up on the same words
  // otherwise), a loss when most keys are new.  A stale read is harmless: a slot only goes
  // from empty to a key, and its index only goes down.
  template <bool PEEK = false>
  __device__ __forceinline__ uint32_t insert(long long key, uint32_t i) const {
    uint32_t p = home(key);
    while (true) {
      unsigned long long prev = ~0ull;
      if (PEEK) prev = __hip_atomic_load(&slots[p], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      if (prev == ~0ull) prev = probe(key, i, p);
      if (landed(key, i, p, prev)) return p;
      p = (p + 1) & mask;
    }
  }
  // The insert in its two halves: probe issues the compare-and-swap on slot p and returns what the slot held; landed
  // acts on that: true when p is the key's slot (an index already there is lowered when
  // ours is smaller), false when the slot belongs to another key and p + 1 is next.
  __device__ __forceinline__ uint32_t home(long long key) const {
    return fib_home(static_cast<uint32_t>(key), shift);
  }
  __device__ __forceinline__ unsigned long long probe(long long key, uint32_t i, uint32_t p) const {
    const unsigned long long word =
        (static_cast<unsigned long long>(static_cast<uint32_t>(key)) << 32) | i;
    return atomicCAS(&slots[p], ~0ull, word);
  }
  __device__ __forceinline__ bool landed(long long key, uint32_t i, uint32_t p,
                                         unsigned long long prev) const {
    if (prev == ~0ull) return true;
    const unsigned long long hi = static_cast<unsigned long long>(static_cast<uint32_t>(key)) << 32;
    if ((prev >> 32) != (hi >> 32)) return false;
    if (static_cast<uint32_t>(prev) > i) atomicMin(&slots[p], hi | i);
    return true;
  }
  // `landed` in two steps for callers that sort out several probes at once: what a probe found
  // (no memory access: 0 = another key's slot, 1 = the key's slot, 3 = the key's slot and the
  // index there is to be lowered), and the lowering itself.
  __device__ __forceinline__ unsigned int found(long long key, uint32_t i,
                                                unsigned long long prev) const {
    if (prev == ~0ull) return 1u;
    if (static_cast<uint32_t>(prev >> 32) != static_cast<uint32_t>(key)) return 0u;
    return static_cast<uint32_t>(prev) > i ? 3u : 1u;
  }
  __device__ __forceinline__ void lower(long long key, uint32_t i, uint32_t p) const {
    atomicMin(&slots[p], (static_cast<unsigned long long>(static_cast<uint32_t>(key)) << 32) | i);
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
  template <bool PEEK = false>
  __device__ __forceinline__ uint32_t insert(long long key, uint32_t i) const {
    uint32_t p = home(key);
    while (true) {
      unsigned long long prev = ~0ull;
      if (PEEK)
        prev = __hip_atomic_load(reinterpret_cast<unsigned long long*>(&keys[p]), __ATOMIC_RELAXED,
                                 __HIP_MEMORY_SCOPE_AGENT);
      if (prev == ~0ull) prev = probe(key, i, p);
      if (landed(key, i, p, prev)) return p;
      p = (p + 1) & mask;
    }
  }
  __device__ __forceinline__ uint32_t home(long long key) const {
    return fib_home(static_cast<uint64_t>(key), shift);
  }
  __device__ __forceinline__ unsigned long long probe(long long key, uint32_t, uint32_t p) const {
    return atomicCAS(reinterpret_cast<unsigned long long*>(&keys[p]), ~0ull,
                     static_cast<unsigned long long>(key));
  }
  __device__ __forceinline__ bool landed(long long key, uint32_t i, uint32_t p,
                                         unsigned long long prev) const {
    if (prev != ~0ull && prev != static_cast<unsigned long long>(key)) return false;
    // values only decrease, so a (possibly stale) read <= i proves the atomic unnecessary
    if (__atomic_load_n(&vals[p], __ATOMIC_RELAXED) > static_cast<int>(i))
      atomicMin(&vals[p], static_cast<int>(i));
    return true;
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

inline int64_t table_capacity(int64_t M) {
  int64_t cap = 1024;
  while (cap < 2 * M) cap <<= 1;
  return cap;
}

// mask and hash shift of a table of `cap` slots (a power of two)
template <typename T>
inline void table_shape(T& t, int64_t cap) {
  t.mask = static_cast<uint32_t>(cap - 1);
  int lg = 0;
  while ((int64_t(1) << lg) < cap) ++lg;
  t.shift = 64 - lg;
}

// A table that outlives one call (gs_relabel_sampled) is emptied slot by slot by its last
// user, never as a whole, so its size costs nothing per call; it is kept four times
// sparser than a one-call table (load <= 1/8): fewer than one insert in ten walks past its
// home slot, and every such step is a round trip to memory that a whole wave waits for.
constexpr int64_t kLinkedFactor = 4;
inline int64_t linked_table_capacity(int64_t items) { return table_capacity(kLinkedFactor * items); }

// Laid out for the largest capacity the buffer can hold, used with the capacity the call
// needs.  False when it does not fit.
template <typename T>
inline bool shape_linked_table(void* buffer, size_t bytes, int64_t items, T* t) {
  int64_t cap_max = 1024;
  if (T::bytes(cap_max) > bytes) return false;
  while (T::bytes(cap_max * 2) <= bytes) cap_max <<= 1;
  const int64_t cap = linked_table_capacity(items);
  if (cap > cap_max) return false;
  Carver ws(buffer, bytes);
  t->carve(ws, cap_max);
  if (!ws.ok) return false;
  table_shape(*t, cap);
  return true;
}

// Workspace a layer's two launches share (gs_layer_sample, gs_layer_relabel): the slot of
// every item.
inline size_t layer_workspace_bytes(int64_t items) {
  if (items < 1) items = 1;
  return padded(static_cast<size_t>(items) * 4);
}
inline bool carve_layer_workspace(void* workspace, size_t bytes, int64_t items, uint32_t** pos) {
  if (items < 1) items = 1;
  Carver ws(workspace, bytes);
  *pos = ws.take<uint32_t>(static_cast<size_t>(items));
  return ws.ok;
}

template <typename T>
inline int64_t linked_table_slots(size_t bytes) {
  int64_t cap_max = 1024;
  if (T::bytes(cap_max) > bytes) return 0;
  while (T::bytes(cap_max * 2) <= bytes) cap_max <<= 1;
  return cap_max;
}

}  // namespace gs
