// Batched relabel without a memory-side atomic per item: bring the items of a batch together
// by hash class, find first occurrences per class in an LDS table, rank them by position.
//
// Same contract as the relabel on hash regions (gs_unique.hip: batch_relabel_impl; reference
// impl::BatchCSRRelabelCUDA, src/cuda/batch_relabel.cu:236-328): batch b owns seeds
// [seeds_ptr[b], seeds_ptr[b+1]) and ids [ids_ptr[b], ids_ptr[b+1]); its frontier is the
// distinct values of (its seeds, then its ids) in first-occurrence order; every id is renamed
// to its rank inside its own batch's frontier.
//
// The regions version pays one compare-and-swap on device memory per item, and those run at
// about 26 G/s on this machine whatever else happens.  Here the only atomics on memory are one
// counter addition per (4096-item tile, class):
//
//   plan      every batch is cut into P_b = 2^k classes of about 1-2 k items by the top bits
//             of its ids' hash; a class of a batch is a "bucket", numbered batch by batch
//   count     a workgroup counts its tile's items per bucket in LDS, adds the counts to memory
//   scan      bucket offsets
//   scatter   the same tile walk; every item's record (id << 32 | position) goes to its bucket.
//             The order inside a bucket is whatever the atomics make it: nothing below depends
//             on it, first occurrences are decided by the positions the records carry
//   flag      one workgroup per bucket: LDS table id -> smallest position; that position is
//             the id's first occurrence in the batch, and gets a byte in a flag array; every
//             record is rewritten to carry the first position of its id instead of the id
//   rank      chained scan over the flag bytes: per 64 positions a mask and the number of
//             first occurrences before them
//   rename    a plain pass over the records: the rank of a record's first position from mask
//             + count, the frontier written by rank, the ids renamed in place
//
// Buckets are handed to workgroups so that consecutive buckets -- one batch's -- run on the
// same XCD one after the other (workgroup w runs on XCD w % 8): the positions a batch's
// buckets store to (flags, renamed ids, frontier) are a megabyte or two that stays in that
// XCD's L2 until its lines are full.
//
// The ids may come from a sampler that is still running when the relabel is queued, and whose
// total is then read from the offsets on the device.  A sampler that failed leaves a negative
// last offset: every pass then leaves at once and the call reports -1, as a look-back of its
// own that gave up would.
//
// An LDS table that fills up (a bucket with more than its slots' worth of distinct ids: only
// a batch beyond ~16 M distinct ids can do that) raises an error word and the call reports
// -4: the caller repeats it on hash regions (GS_RELABEL_REGIONS).
#include "gs_common.hpp"
#include "gs_batch_items.hpp"

namespace gs {
namespace {

constexpr int kThreads = 256;
constexpr int kBucketItemsLog2 = 11;   // classes are sized for <= 2048 items on average
constexpr int kMaxClassesLog2 = 12;    // at most 4096 classes per batch
constexpr int kPartItems = 16;         // items of a thread in the count / scatter passes
constexpr int kPartTile = kThreads * kPartItems;
// LDS counters of a tile: the buckets of the batches it touches (two batches of 4096 classes
// at the most, and those wholly inside it, which have a class per 1024 items and two on top)
constexpr int kCounterCap = 2 * (1 << kMaxClassesLog2) + (kPartTile >> (kBucketItemsLog2 - 1)) +
                            2 * static_cast<int>(kStagedBatches) + 2;
constexpr int kSlots = 4096;           // LDS table of a bucket (8-byte slots)
constexpr int kFlagTile = kThreads * 64;  // positions of a workgroup in the rank pass
constexpr int kXcds = 8;
constexpr int kTrip = 8;  // records of a thread that are asked for together (a whole average bucket)

struct Plan {
  uint32_t* bucket_base;  // [B + 1]: first bucket of every batch; [B] = number of buckets
  uint32_t* classes_log2; // [B]
};

struct Bins {
  Plan plan;
  uint32_t* count;        // [buckets bound]: items per bucket
  uint32_t* fill;         // [buckets bound]: records placed so far
  int64_t* bucket_ptr;    // [buckets bound + 1]: first record of every bucket
  uint32_t* bucket_batch; // [buckets bound]: the batch of every bucket that holds records
  unsigned long long* records;  // [M]: id << 32 | position
  unsigned char* flags;   // [tiles * kFlagTile]: 1 at first occurrences
  uint4* ranks;           // per 64 positions: {flags as bits (x, y), first occurrences before them (z), 0}
  unsigned int* error;    // the look-back state's error word: 2 = id too wide, 3 = a table filled up
};

inline int64_t buckets_bound(int64_t M, int64_t B) { return (M >> (kBucketItemsLog2 - 1)) + 2 * B + 8; }
inline int64_t flag_tiles(int64_t M) { return M / kFlagTile + 1; }

// slot of an id in a bucket's table: other hash bits than the ones that chose the bucket
__device__ __forceinline__ uint32_t slot_of(uint32_t key) {
  return (key * 0x85EBCA6Bu) >> (32 - 12);
}
static_assert(kSlots == 1 << 12, "slot_of yields 12 bits");

__global__ void __launch_bounds__(kThreads)
bins_init_kernel(Bins s, int64_t flag_words16, int64_t buckets, LookbackState lb, int64_t tiles) {
  const int64_t i = static_cast<int64_t>(blockIdx.x) * kThreads + threadIdx.x;
  if (i < flag_words16) reinterpret_cast<uint4*>(s.flags)[i] = make_uint4(0u, 0u, 0u, 0u);
  if (i < buckets) {
    s.count[i] = 0u;
    s.fill[i] = 0u;
  }
  if (i < tiles) lb.status[i] = 0ull;
  if (i == 0) *lb.error = 0u;
}

// one workgroup: classes per batch and the numbering of the buckets
template <typename IdT>
__global__ void __launch_bounds__(512) bins_plan_kernel(BatchItems<IdT> x, Plan p) {
  __shared__ int64_t s_scan[512 / kWave + 1];
  const int64_t b = threadIdx.x;
  int64_t classes = 0;
  uint32_t lg = 0;
  if (b < x.B) {
    const int64_t m = x.ids_ptr[x.B] < 0 ? 0 : x.start(b + 1) - x.start(b);
    const int64_t want = (m + (int64_t(1) << kBucketItemsLog2) - 1) >> kBucketItemsLog2;
    while ((int64_t(1) << lg) < want && lg < kMaxClassesLog2) ++lg;
    classes = int64_t(1) << lg;
    p.classes_log2[b] = lg;
  }
  int64_t total;
  const int64_t before = block_exclusive_scan<512>(classes, &total, s_scan);
  if (b < x.B) p.bucket_base[b] = static_cast<uint32_t>(before);
  if (b == 0) p.bucket_base[x.B] = static_cast<uint32_t>(total);
}

// What the count and the scatter pass share: the tile's items, their batches and buckets.
template <typename IdT>
struct TileWalk {
  int64_t lo, hi;          // batches of the tile's first and last item
  uint32_t first_bucket;   // bucket_base[lo]
  uint32_t span;           // buckets of batches lo..hi, cut to the LDS counters
  // M comes in as the caller's count of items, which may be a bound: the offsets hold the
  // true one.  False: the tile lies beyond the items (the whole workgroup leaves).
  __device__ __forceinline__ bool open(BatchItems<IdT>& x, const Plan& p, int64_t& M,
                                       int64_t* s_seeds_ptr, int64_t* s_ids_ptr,
                                       uint32_t* s_base, uint32_t* s_lg, int64_t* s_range,
                                       uint32_t* s_cnt) {
    x.stage_offsets(s_seeds_ptr, s_ids_ptr);
    const int64_t held = x.seeds_ptr[x.B] + x.ids_ptr[x.B];
    if (held < M) M = held;
    if (x.ids_ptr[x.B] < 0) return false;  // the producer of the ids failed
    if (static_cast<int64_t>(blockIdx.x) * kPartTile >= M) return false;
    for (int64_t b = threadIdx.x; b <= x.B; b += kThreads) {
      s_base[b] = p.bucket_base[b];
      s_lg[b] = b < x.B ? p.classes_log2[b] : 0u;
    }
    const int64_t first = static_cast<int64_t>(blockIdx.x) * kPartTile;
    const int64_t last = first + kPartTile - 1 < M ? first + kPartTile - 1 : M - 1;
    x.block_range(first, last, s_range, &lo, &hi);  // (ends with a barrier: s_base is there)
    first_bucket = s_base[lo];
    const uint32_t all = s_base[hi + 1] - first_bucket;
    span = all < static_cast<uint32_t>(kCounterCap) ? all : static_cast<uint32_t>(kCounterCap);
    for (uint32_t c = threadIdx.x; c < span; c += kThreads) s_cnt[c] = 0u;
    __syncthreads();
    return true;
  }
};

// LDS of the two partition passes
struct PartShared {
  int64_t seeds_ptr[kStagedBatches + 1];
  int64_t ids_ptr[kStagedBatches + 1];
  uint32_t base[kStagedBatches + 1];
  uint32_t lg[kStagedBatches + 1];
  int64_t range[2];
  uint32_t cnt[kCounterCap];
};

// count (SCATTER false): items per bucket.  scatter: the same walk, then the tile's share of
// every bucket it touches is reserved with one addition and the records are placed.  (Tiles
// of several rounds of 4096 items -- fewer additions to memory, longer runs of records side
// by side -- were slower: 64 / 143 us against 55 / 105 us over 17 M items; workgroups that
// stay and loop are the slower shape on this machine.)
template <typename IdT, bool SCATTER>
__global__ void __launch_bounds__(kThreads)
bins_partition_kernel(BatchItems<IdT> x, int64_t M, Bins s) {
  __shared__ PartShared sh;
  TileWalk<IdT> w;
  if (!w.open(x, s.plan, M, sh.seeds_ptr, sh.ids_ptr, sh.base, sh.lg, sh.range, sh.cnt)) return;
  const int64_t tile_first = static_cast<int64_t>(blockIdx.x) * kPartTile;
  // where every item is: all reads of the thread's items stand together, none behind a
  // condition of its own (the last item again past the end)
  const IdT* from[kPartItems];
  uint32_t batch[kPartItems];
#pragma unroll
  for (int k = 0; k < kPartItems; ++k) {
    const int64_t i = tile_first + k * kThreads + threadIdx.x;
    const int64_t ic = i < M ? i : M - 1;
    const int64_t b = x.batch_of(ic, w.lo, w.hi);
    batch[k] = static_cast<uint32_t>(b);
    from[k] = x.where_in(b, ic);
  }
  IdT key[kPartItems];
#pragma unroll
  for (int k = 0; k < kPartItems; ++k) key[k] = *from[k];
  uint32_t bucket[kPartItems], rank[kPartItems];
  bool wide = false;
#pragma unroll
  for (int k = 0; k < kPartItems; ++k) {
    const int64_t i = tile_first + k * kThreads + threadIdx.x;
    const uint32_t lg = sh.lg[batch[k]];
    const uint32_t cls = lg ? hash32(static_cast<uint32_t>(key[k])) >> (32 - lg) : 0u;
    bucket[k] = sh.base[batch[k]] + cls;
    rank[k] = 0u;
    if (i < M) {
      if (sizeof(IdT) == 8 && (static_cast<unsigned long long>(key[k]) >> 32) != 0ull) wide = true;
      const uint32_t c = bucket[k] - w.first_bucket;
      if (c < w.span) {
        rank[k] = atomicAdd(&sh.cnt[c], 1u);
      } else if (SCATTER) {  // beyond the LDS counters: straight to memory
        rank[k] = static_cast<uint32_t>(s.bucket_ptr[bucket[k]]) + atomicAdd(&s.fill[bucket[k]], 1u);
        s.bucket_batch[bucket[k]] = batch[k];
      } else {
        atomicAdd(&s.count[bucket[k]], 1u);
      }
    }
  }
  if (wide) *s.error = 2u;  // 64-bit ids ride on 32-bit records: this one does not fit
  __syncthreads();
  for (uint32_t c = threadIdx.x; c < w.span; c += kThreads) {
    const uint32_t n = sh.cnt[c];
    if (!n) continue;
    const uint32_t bucket_c = w.first_bucket + c;
    if (SCATTER) {
      // the counter turns into the place of the tile's first record in the bucket
      sh.cnt[c] = static_cast<uint32_t>(s.bucket_ptr[bucket_c]) + atomicAdd(&s.fill[bucket_c], n);
      int64_t lo = w.lo, hi = w.hi;  // the batch the bucket belongs to, for the later passes
      while (lo < hi) {
        const int64_t mid = (lo + hi + 1) >> 1;
        if (sh.base[mid] <= bucket_c) lo = mid; else hi = mid - 1;
      }
      s.bucket_batch[bucket_c] = static_cast<uint32_t>(lo);
    } else {
      atomicAdd(&s.count[bucket_c], n);
    }
  }
  if (!SCATTER) return;
  __syncthreads();
#pragma unroll
  for (int k = 0; k < kPartItems; ++k) {
    const int64_t i = tile_first + k * kThreads + threadIdx.x;
    if (i < M) {
      const uint32_t c = bucket[k] - w.first_bucket;
      const uint32_t at = c < w.span ? sh.cnt[c] + rank[k] : rank[k];
      s.records[at] = (static_cast<unsigned long long>(static_cast<uint32_t>(key[k])) << 32) |
                      static_cast<unsigned long long>(static_cast<uint32_t>(i));
    }
  }
}

struct CountOf {
  const uint32_t* count;
  __device__ __forceinline__ int64_t operator()(int64_t i) const { return count[i]; }
};

// Bucket of workgroup w: XCD x = w % 8 takes the x-th eighth of the buckets, in order.
__device__ __forceinline__ int64_t bucket_of_workgroup(int64_t num_buckets) {
  const int64_t per = (num_buckets + kXcds - 1) / kXcds;
  const int64_t k = static_cast<int64_t>(blockIdx.x % kXcds) * per + blockIdx.x / kXcds;
  return blockIdx.x / kXcds < per && k < num_buckets ? k : -1;
}

// Enters the bucket's records into the LDS table: slot = id << 32 | smallest position.
// Raises the error word when the table is full.  The first trip's records are asked for
// before the table is cleared, so that the clearing hides under the trip.
__device__ __forceinline__ void table_fill(unsigned long long* __restrict__ tab,
                                           const unsigned long long* __restrict__ records,
                                           int64_t begin, int64_t end, unsigned int* error) {
  unsigned long long rec[kTrip];
#pragma unroll
  for (int u = 0; u < kTrip; ++u) {
    const int64_t r = begin + u * kThreads + threadIdx.x;
    rec[u] = records[r < end ? r : end - 1];
  }
  for (int c = threadIdx.x; c < kSlots; c += kThreads) tab[c] = ~0ull;
  __syncthreads();
  for (int64_t r0 = begin; r0 < end; r0 += kTrip * kThreads) {
#pragma unroll
    for (int u = 0; u < kTrip; ++u) {
      if (r0 + u * kThreads + threadIdx.x < end) {
        const uint32_t key = static_cast<uint32_t>(rec[u] >> 32);
        uint32_t p = slot_of(key);
        int probes = 0;
        while (true) {
          const unsigned long long prev = atomicCAS(&tab[p], ~0ull, rec[u]);
          if (prev == ~0ull) break;
          if (static_cast<uint32_t>(prev >> 32) == key) {
            if (prev > rec[u]) atomicMin(&tab[p], rec[u]);
            break;
          }
          p = (p + 1) & (kSlots - 1);
          if (++probes >= kSlots) {
            *error = 3u;
            break;
          }
        }
      }
    }
    if (r0 + kTrip * kThreads < end) {
#pragma unroll
      for (int u = 0; u < kTrip; ++u) {
        const int64_t r = r0 + (kTrip + u) * kThreads + threadIdx.x;
        rec[u] = records[r < end ? r : end - 1];
      }
    }
  }
  __syncthreads();
}

// One workgroup per bucket.  After the table is complete every record is rewritten in place
// for the last pass, which then needs no table: a first occurrence keeps its id and gets the
// top bit of its position set (and its byte in the flag array); any other record trades its
// id for the position of the id's first occurrence.
constexpr unsigned long long kFirstBit = 0x80000000ull;

__global__ void __launch_bounds__(kThreads) bins_flag_kernel(Bins s, int64_t B) {
  __shared__ unsigned long long tab[kSlots];
  const int64_t k = bucket_of_workgroup(s.plan.bucket_base[B]);
  if (k < 0) return;
  const int64_t begin = s.bucket_ptr[k], end = s.bucket_ptr[k + 1];
  if (begin == end) return;
  table_fill(tab, s.records, begin, end, s.error);
  for (int64_t r0 = begin; r0 < end; r0 += kTrip * kThreads) {
    unsigned long long rec[kTrip];
#pragma unroll
    for (int u = 0; u < kTrip; ++u) {
      const int64_t r = r0 + u * kThreads + threadIdx.x;
      rec[u] = s.records[r < end ? r : end - 1];
    }
    unsigned long long out[kTrip];
#pragma unroll
    for (int u = 0; u < kTrip; ++u) {
      out[u] = 0ull;
      // (a lane past the end holds a copy of the last record, which its owner may already have
      // rewritten: it must not look that up)
      if (r0 + u * kThreads + threadIdx.x < end) {
        const uint32_t key = static_cast<uint32_t>(rec[u] >> 32);
        uint32_t p = slot_of(key);
        int probes = 0;
        unsigned long long w = tab[p];
        while (static_cast<uint32_t>(w >> 32) != key && ++probes < kSlots) {
          p = (p + 1) & (kSlots - 1);
          w = tab[p];
        }
        out[u] = w == rec[u] ? rec[u] | kFirstBit
                             : (w << 32) | static_cast<unsigned long long>(static_cast<uint32_t>(rec[u]));
      }
    }
#pragma unroll
    for (int u = 0; u < kTrip; ++u) {
      const int64_t r = r0 + u * kThreads + threadIdx.x;
      if (r < end) {
        s.records[r] = out[u];
        if (out[u] & kFirstBit) s.flags[static_cast<uint32_t>(rec[u])] = 1;
      }
    }
  }
}

// 64 flag bytes of a thread -> one mask word; scan of the counts over all tiles
__global__ void __launch_bounds__(kThreads)
bins_rank_kernel(Bins s, int64_t M, int64_t B, const int64_t* __restrict__ seeds_ptr,
                 const int64_t* __restrict__ ids_ptr, int64_t* __restrict__ num_unique,
                 int64_t* __restrict__ unique_ptr, LookbackState lb, gs_mailbox* box,
                 int64_t box_ticket) {
  __shared__ int64_t s_scan[kThreads / kWave + 1];
  __shared__ int64_t s_prefix;
  __shared__ unsigned long long s_mask[kThreads];
  __shared__ uint32_t s_before[kThreads];
  const unsigned int tile = blockIdx.x;
  const int64_t word = static_cast<int64_t>(tile) * kThreads + threadIdx.x;
  const uint4* __restrict__ f = reinterpret_cast<const uint4*>(s.flags) + word * 4;
  uint4 q[4];
#pragma unroll
  for (int u = 0; u < 4; ++u) q[u] = f[u];
  unsigned long long m = 0ull;
#pragma unroll
  for (int u = 0; u < 4; ++u) {
    const uint32_t x[4] = {q[u].x, q[u].y, q[u].z, q[u].w};
#pragma unroll
    for (int v = 0; v < 4; ++v) {
      // four flag bytes (0 or 1 each) -> four bits, byte j at bit j
      const unsigned long long nib = ((x[v] & 0x01010101u) * 0x01020408u) >> 24 & 0xFu;
      m |= nib << (16 * u + 4 * v);
    }
  }
  const int64_t mine = __popcll(m);
  int64_t tile_total;
  const int64_t local = block_exclusive_scan<kThreads>(mine, &tile_total, s_scan);
  if (threadIdx.x == 0) lookback_publish_sum(lb, tile, tile_total);
  if (threadIdx.x < kWave) {
    const int64_t before = lookback_exclusive_prefix(lb, tile, tile_total);
    if (threadIdx.x == 0) s_prefix = before;
  }
  __syncthreads();
  const uint32_t before = static_cast<uint32_t>(s_prefix + local);
  s.ranks[word] = make_uint4(static_cast<uint32_t>(m), static_cast<uint32_t>(m >> 32), before, 0u);
  // frontier offsets: the rank at every batch's first position, by the thread that owns it
  s_mask[threadIdx.x] = m;
  s_before[threadIdx.x] = before;
  __syncthreads();
  const int64_t tile_first = static_cast<int64_t>(tile) * kFlagTile;
  for (int64_t b = threadIdx.x; b < B; b += kThreads) {
    const int64_t p = seeds_ptr[b] + ids_ptr[b] - tile_first;
    if (p >= 0 && p < kFlagTile)
      unique_ptr[b] = s_before[p >> 6] + __popcll(s_mask[p >> 6] & ((1ull << (p & 63)) - 1ull));
  }
  if (tile == gridDim.x - 1 && threadIdx.x == 0) {
    int64_t total = s_prefix + tile_total;
    const unsigned int err = __hip_atomic_load(lb.error, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    if (err) total = err == 2u ? -2 : (err == 3u ? -4 : -1);
    if (ids_ptr[B] < 0) total = -1;  // the producer of the ids failed: nothing was relabelled
    *num_unique = total;
    unique_ptr[B] = total;
    post_mailbox(box, total, box_ticket);
  }
}

// The last pass, over the records as they lie (bucket by bucket, which is batch by batch): a
// record knows the position of its id's first occurrence, whose rank is the count before its
// 64 positions plus the bits below it; first occurrences write the frontier, records of ids
// (not seeds) the renamed id.  Chunks of records go to workgroups like the buckets did, one
// batch after the other on one XCD.
constexpr int kRenameItems = 8;
constexpr int kRenameTile = kThreads * kRenameItems;

struct RenameShared {
  int64_t seeds_ptr[kStagedBatches + 1];
  int64_t ids_ptr[kStagedBatches + 1];
  int64_t range[2];
};

template <typename IdT>
__global__ void __launch_bounds__(kThreads)
bins_rename_kernel(BatchItems<IdT> x, int64_t M, Bins s, IdT* __restrict__ unique,
                   IdT* __restrict__ out_ids, const int64_t* __restrict__ unique_ptr) {
  __shared__ RenameShared sh;
  {  // (M may be a bound: the offsets hold the true count)
    const int64_t held = x.seeds_ptr[x.B] + x.ids_ptr[x.B];
    if (held < M) M = held;
    if (x.ids_ptr[x.B] < 0) return;  // the producer of the ids failed: no records were made
  }
  const int64_t chunks = (M + kRenameTile - 1) / kRenameTile;
  const int64_t per = (chunks + kXcds - 1) / kXcds;
  const int64_t chunk = static_cast<int64_t>(blockIdx.x % kXcds) * per + blockIdx.x / kXcds;
  if (blockIdx.x / kXcds >= per || chunk >= chunks) return;
  const int64_t first = chunk * kRenameTile;
  unsigned long long rec[kRenameItems];
#pragma unroll
  for (int u = 0; u < kRenameItems; ++u) {
    const int64_t r = first + u * kThreads + threadIdx.x;
    rec[u] = s.records[r < M ? r : M - 1];
  }
  x.stage_offsets(sh.seeds_ptr, sh.ids_ptr);
  // the entries of the first occurrences' positions: one 16-byte read each, all in flight
  uint4 e[kRenameItems];
  uint32_t pos[kRenameItems], at[kRenameItems];
#pragma unroll
  for (int u = 0; u < kRenameItems; ++u) {
    pos[u] = static_cast<uint32_t>(rec[u]) & ~static_cast<uint32_t>(kFirstBit);
    at[u] = (rec[u] & kFirstBit) ? pos[u] : static_cast<uint32_t>(rec[u] >> 32);
    e[u] = s.ranks[at[u] >> 6];
  }
  // records of a chunk belong to the batches of its first and last record and those between
  if (threadIdx.x < 2) {
    const int64_t r = threadIdx.x == 0 ? first : (first + kRenameTile - 1 < M ? first + kRenameTile - 1 : M - 1);
    const uint32_t p = static_cast<uint32_t>(s.records[r]) & ~static_cast<uint32_t>(kFirstBit);
    sh.range[threadIdx.x] = x.batch_of(p, 0, x.B - 1);
  }
  __syncthreads();
  const int64_t lo = sh.range[0], hi = sh.range[1];
#pragma unroll
  for (int u = 0; u < kRenameItems; ++u) {
    if (first + u * kThreads + threadIdx.x < M) {
      const unsigned long long m = static_cast<unsigned long long>(e[u].y) << 32 | e[u].x;
      const uint32_t rank = e[u].z + __popcll(m & ((1ull << (at[u] & 63u)) - 1ull));
      if (rec[u] & kFirstBit) unique[rank] = static_cast<IdT>(static_cast<uint32_t>(rec[u] >> 32));
      const int64_t b = x.batch_of(pos[u], lo, hi);
      const int64_t off = static_cast<int64_t>(pos[u]) - x.start(b);
      const int64_t n_seeds = x.seeds_ptr[b + 1] - x.seeds_ptr[b];
      if (off >= n_seeds)
        out_ids[x.ids_ptr[b] + off - n_seeds] =
            static_cast<IdT>(rank - static_cast<uint32_t>(unique_ptr[b]));
    }
  }
}

template <typename IdT>
int binned_impl(const void* seeds, const int64_t* seeds_ptr, const void* ids,
                const int64_t* ids_ptr, int64_t B, int64_t num_seeds, int64_t num_ids,
                void* unique, int64_t* unique_ptr, void* out_ids, int64_t* num_unique,
                void* workspace, size_t workspace_bytes, gs_mailbox* box, int64_t box_ticket,
                hipStream_t stream) {
  const int64_t M = num_seeds + num_ids;
  const int64_t nb = buckets_bound(M, B);
  const int64_t tiles = flag_tiles(M);
  Carver ws(workspace, workspace_bytes);
  Bins s;
  s.plan.bucket_base = ws.take<uint32_t>(B + 1);
  s.plan.classes_log2 = ws.take<uint32_t>(B);
  s.count = ws.take<uint32_t>(nb);
  s.fill = ws.take<uint32_t>(nb);
  s.bucket_ptr = ws.take<int64_t>(nb + 1);
  s.bucket_batch = ws.take<uint32_t>(nb);
  int64_t* scan_ws = ws.take<int64_t>(scan_num_tiles(nb) + 1);
  s.records = ws.take<unsigned long long>(M);
  s.flags = ws.take<unsigned char>(tiles * kFlagTile);
  s.ranks = ws.take<uint4>(tiles * kThreads);
  LookbackState lb = carve_lookback(ws, tiles, 1u);
  s.error = lb.error;
  if (!ws.ok) {
    set_error_text("gs_batch_csr_relabel: workspace needs %zu bytes, 256-byte aligned",
                   binned_relabel_workspace_bytes(M, B));
    return GS_ERR_WORKSPACE;
  }
  BatchItems<IdT> x{static_cast<const IdT*>(seeds), seeds_ptr, static_cast<const IdT*>(ids), ids_ptr,
                    B};
  const int64_t flag_words16 = tiles * kFlagTile / 16;
  int64_t n_init = flag_words16 > nb ? flag_words16 : nb;
  if (tiles > n_init) n_init = tiles;
  {
    ProfileScope prof("bins_init", stream);
    hipLaunchKernelGGL(bins_init_kernel, dim3(blocks_for(n_init, kThreads)), dim3(kThreads), 0,
                       stream, s, flag_words16, nb, lb, tiles);
    hipLaunchKernelGGL(bins_plan_kernel<IdT>, dim3(1), dim3(512), 0, stream, x, s.plan);
  }
  const unsigned part_grid = static_cast<unsigned>(blocks_for(M, kPartTile));
  {
    ProfileScope prof("bins_count", stream);
    hipLaunchKernelGGL((bins_partition_kernel<IdT, false>), dim3(part_grid), dim3(kThreads), 0,
                       stream, x, M, s);
  }
  GS_RETURN_IF_ERROR(exclusive_scan(CountOf{s.count}, nb, s.bucket_ptr, scan_ws, stream));
  {
    ProfileScope prof("bins_scatter", stream);
    hipLaunchKernelGGL((bins_partition_kernel<IdT, true>), dim3(part_grid), dim3(kThreads), 0,
                       stream, x, M, s);
  }
  // a workgroup per bucket (the bound: the number of buckets is on the device), rounded up so
  // that every XCD's share is whole
  const unsigned bucket_grid = static_cast<unsigned>((nb + kXcds - 1) / kXcds * kXcds);
  {
    ProfileScope prof("bins_flag", stream);
    hipLaunchKernelGGL(bins_flag_kernel, dim3(bucket_grid), dim3(kThreads), 0, stream, s, B);
  }
  {
    ProfileScope prof("bins_rank", stream);
    hipLaunchKernelGGL(bins_rank_kernel, dim3(static_cast<unsigned>(tiles)), dim3(kThreads), 0,
                       stream, s, M, B, seeds_ptr, ids_ptr, num_unique, unique_ptr, lb, box, box_ticket);
  }
  ProfileScope prof("bins_rename", stream);
  const int64_t chunks = (M + kRenameTile - 1) / kRenameTile;
  hipLaunchKernelGGL(bins_rename_kernel<IdT>,
                     dim3(static_cast<unsigned>((chunks + kXcds - 1) / kXcds * kXcds)), dim3(kThreads),
                     0, stream, x, M, s, static_cast<IdT*>(unique), static_cast<IdT*>(out_ids),
                     static_cast<const int64_t*>(unique_ptr));
  return check_launch("batch_csr_relabel (binned)");
}

}  // namespace

size_t binned_relabel_workspace_bytes(int64_t M, int64_t B) {
  if (M < 0) M = 0;
  if (B < 0) B = 0;
  const int64_t nb = buckets_bound(M, B);
  const int64_t tiles = flag_tiles(M);
  return padded((B + 1) * 4) + padded((B > 0 ? B : 1) * 4) + 3 * padded(nb * 4) +
         padded((nb + 1) * 8) + scan_workspace_bytes(nb) + padded((M > 0 ? M : 1) * 8) +
         padded(tiles * kFlagTile) + padded(tiles * kThreads * 16) + lookback_state_bytes(tiles);
}

bool binned_relabel_applies(int64_t M, int64_t B) {
  // below about half a million items the regions' three launches are quicker than eight;
  // positions ride in 32 bits; the batch offsets must fit the kernels' LDS copies
  return M >= (int64_t(1) << 19) && M < (int64_t(1) << 32) && B >= 1 &&
         B <= static_cast<int64_t>(kStagedBatches);
}

int batch_relabel_binned(const void* seeds, const int64_t* seeds_ptr, const void* ids,
                         const int64_t* ids_ptr, int64_t B, int64_t num_seeds, int64_t num_ids,
                         int id_bytes, void* unique, int64_t* unique_ptr, void* out_ids,
                         int64_t* num_unique, void* workspace, size_t workspace_bytes,
                         gs_mailbox* box, int64_t box_ticket, hipStream_t stream) {
  return id_bytes == 8
             ? binned_impl<int64_t>(seeds, seeds_ptr, ids, ids_ptr, B, num_seeds, num_ids, unique,
                                    unique_ptr, out_ids, num_unique, workspace, workspace_bytes,
                                    box, box_ticket, stream)
             : binned_impl<int32_t>(seeds, seeds_ptr, ids, ids_ptr, B, num_seeds, num_ids, unique,
                                    unique_ptr, out_ids, num_unique, workspace, workspace_bytes,
                                    box, box_ticket, stream);
}

}  // namespace gs
