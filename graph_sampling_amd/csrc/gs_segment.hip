// Segment (SpMV-style) reductions over edge data on gfx950.
//
// Replaces impl::CSCSumCUDA, impl::COOSumCUDA, impl::CSCNormalizeCUDA
// (reference src/cuda/graph_ops.cu:92,122,184) and impl::fusion::COOEDivUSum
// (src/cuda/fusion/edge_map_reduce.cu:10).
//
// The reference gives every segment to one thread (graph_ops.cu:16-39), which
// stalls a whole wave on a power-law hub.  Two decompositions are used here:
//  * by segment, for segments of at most 16 edges: one lane per segment, summed
//    in edge order (bit-identical to a sequential sum).  The typical
//    layer-wise-sampler call has millions of mostly empty segments
//    (graph.cc:657: one per graph row): one coalesced pass over the offsets and
//    one over the output.  The same pass enters every longer segment in the list
//    of the 1024-edge chunk its first edge falls in, and as the "incoming"
//    segment of every later chunk it reaches into.
//  * by edge, for the longer ones: a wave owns one chunk of 1024 consecutive
//    edges.  Its lanes pick up the chunk's segments (at most 61 can start in it,
//    plus the incoming one), mark where each starts and stops in an LDS array of
//    one int per edge, and a running "latest mark" over the edges then tells
//    every edge its owner without any search; a segmented scan folds 64 edges
//    per step, coalesced.  A segment that lies inside the chunk is written at
//    once; the pieces of a segment that crosses chunk borders go to a carry
//    array and are added up, in chunk order, by the chunk that holds its first
//    edge.  A 300 000-edge hub is 290 chunks of work for 290 waves, millions of
//    empty segments cost the by-edge pass nothing, and the order of the additions
//    is fixed by the layout alone, so results repeat from run to run.
#include <limits>
#include "gs_common.hpp"

namespace gs {
namespace {

constexpr int kThreads = 256;
constexpr int kWaves = kThreads / kWave;
constexpr int64_t kLaneMaxLen = 16;
constexpr int64_t kChunk = 1024;   // edges per wave in the by-edge pass
constexpr int kChunkList = 64;     // list slots per chunk: 1024 / 17 + 1 = 61 segments can start in one
constexpr int kIncomingLane = kWave - 1;

// Per-chunk bookkeeping of the by-edge pass, all in the caller's workspace.
struct Chunks {
  unsigned int* any_long;  // does any segment exceed kLaneMaxLen?
  unsigned int* count;     // [chunks] long segments starting in the chunk
  int* list;               // [chunks][kChunkList] their ids
  int* incoming;           // [chunks] long segment that starts earlier and reaches into the chunk, or -1
  int* outgoing;           // [chunks] long segment that starts here and goes on after the chunk, or -1
  float* carry;            // [chunks][2]: piece of the incoming segment, piece of the outgoing one
};

__global__ void __launch_bounds__(kThreads) clear_chunks_kernel(Chunks ck, int64_t chunks) {
  const int64_t c = static_cast<int64_t>(blockIdx.x) * kThreads + threadIdx.x;
  if (c == 0) *ck.any_long = 0u;
  if (c < chunks) {
    ck.count[c] = 0u;
    ck.incoming[c] = -1;
  }
}

// four floats side by side at any 4-byte boundary
struct __attribute__((packed, aligned(4))) Four {
  float a, b, c, d;
};

// ---- by segment: the short ones.  NORMALIZE writes out[d] = data[d] / sum instead.  EMAP:
// with an edge map (a compile-time switch: the two ways of reading hold different things in
// registers, and one kernel for both would run both at the occupancy of the larger).
template <bool NORMALIZE, bool EMAP, typename IdT>
__global__ void __launch_bounds__(kThreads)
short_segments_kernel(const int64_t* __restrict__ indptr, const int64_t* __restrict__ emap,
                      const IdT* __restrict__ nmap, const float* __restrict__ data,
                      int64_t num_seg, int64_t nnz, int powk, float* __restrict__ out, Chunks ck) {
  const int64_t s = static_cast<int64_t>(blockIdx.x) * kThreads + threadIdx.x;
  int64_t begin = 0, end = 0;
  if (s < num_seg) {
    begin = indptr[s];
    end = indptr[s + 1];
  }
  const int64_t len = end - begin;
  const int lane = threadIdx.x & (kWave - 1);
  const bool is_long = len > kLaneMaxLen;
  // the long segments of a wave enter their chunks' lists, one atomic per chunk touched
  unsigned long long todo = __ballot(is_long);
  if (todo && lane == 0) *ck.any_long = 1u;
  const int64_t c0 = begin / kChunk;
  while (todo) {
    const int64_t c = __shfl(c0, __ffsll(static_cast<long long>(todo)) - 1, kWave);
    const unsigned long long same = __ballot(is_long && c0 == c);
    const int leader = __ffsll(static_cast<long long>(same)) - 1;
    unsigned int base = 0;
    if (lane == leader) base = atomicAdd(ck.count + c, static_cast<unsigned int>(__popcll(same)));
    base = __shfl(base, leader, kWave);
    if (is_long && c0 == c)
      ck.list[c * kChunkList + base + __popcll(same & ((1ull << lane) - 1ull))] = static_cast<int>(s);
    todo &= ~same;
  }
  if (s >= num_seg) return;
  if (is_long) {
    const int64_t c1 = (end - 1) / kChunk;
    for (int64_t c = c0 + 1; c <= c1; ++c) ck.incoming[c] = static_cast<int>(s);
    return;
  }
  // at most kLaneMaxLen edges: a fixed number of predicated reads, all in flight together,
  // added up in edge order.  Without an edge map the lane's edges lie side by side and are
  // read four at a time (a lane's reads are scattered from its neighbours' either way: every
  // read instruction is a line access per lane, and this makes four of sixteen).
  float v[kLaneMaxLen];
  int64_t at[kLaneMaxLen];
  if (!EMAP) {
#pragma unroll
    for (int j = 0; j < kLaneMaxLen / 4; ++j) {
      const int64_t p = begin + 4 * j;
      Four q{0.0f, 0.0f, 0.0f, 0.0f};
      if (p + 3 < nnz && p < end) {
        q = *reinterpret_cast<const Four*>(data + p);
      } else {
        if (p < end) q.a = data[p];
        if (p + 1 < end) q.b = data[p + 1];
        if (p + 2 < end) q.c = data[p + 2];
      }
      v[4 * j] = q.a, v[4 * j + 1] = q.b, v[4 * j + 2] = q.c, v[4 * j + 3] = q.d;
#pragma unroll
      for (int u = 0; u < 4; ++u) at[4 * j + u] = p + u < end ? p + u : -1;
    }
  } else {
    // (predicated pair by pair: most segments here are far shorter than sixteen, and sweeps
    // of sixteen clamped reads cost more than the waits they save -- 52 against 36 us over
    // the 2.45 M mostly empty rows of a sliced graph)
#pragma unroll
    for (int k = 0; k < kLaneMaxLen; ++k) {
      at[k] = begin + k < end ? emap[begin + k] : -1;
      v[k] = at[k] >= 0 ? data[at[k]] : 0.0f;
    }
  }
  float acc = 0.0f;
#pragma unroll
  for (int k = 0; k < kLaneMaxLen; ++k)
    if (at[k] >= 0) acc += powk_f(v[k], powk);
  if (NORMALIZE) {
#pragma unroll
    for (int k = 0; k < kLaneMaxLen; ++k)
      if (at[k] >= 0) out[at[k]] = v[k] / acc;
  } else {
    out[nmap ? static_cast<int64_t>(nmap[s]) : s] = acc;
  }
}

// ---- by edge: the long ones.
// What a lane knows of the chunk's long segments: lane l < count holds the l-th of the list,
// the last lane the incoming one.
struct Owned {
  int g;           // segment, -1 = none
  int64_t b, e;    // its edge range
};

__device__ __forceinline__ Owned load_owned(const int64_t* __restrict__ indptr, const Chunks& ck,
                                            int64_t c, int lane) {
  Owned o;
  o.g = -1;
  o.b = o.e = 0;
  const int n = static_cast<int>(ck.count[c]);
  if (lane < n) o.g = ck.list[c * kChunkList + lane];
  if (lane == kIncomingLane) o.g = ck.incoming[c];
  if (o.g >= 0) {
    o.b = indptr[o.g];
    o.e = indptr[o.g + 1];
  }
  return o;
}

// mark[p] = lane + 2 where the lane's segment starts (or the chunk does, for the incoming
// one), 1 where a segment stops and no other starts, 0 elsewhere
__device__ __forceinline__ void write_marks(int* mark, const Owned& o, int64_t begin, int64_t end,
                                            int lane, bool skip = false) {
  for (int i = lane; i < kChunk; i += kWave) mark[i] = 0;
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_wave_barrier();
  if (o.g >= 0 && !skip) {
    atomicMax(&mark[(o.b > begin ? o.b : begin) - begin], lane + 2);
    if (o.e < end) atomicMax(&mark[o.e - begin], 1);
  }
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_wave_barrier();
}

// A step is 256 edges, four consecutive ones per lane (one 16-byte read of the marks, one of
// the data).  A long segment has at least 17 edges, so inside a lane's four at most one long
// run ends (at the lane's first mark) and at most one begins (at its last mark); what lies
// between belongs to short segments.  Lanes therefore exchange one value each: the cross-lane
// work per edge is a quarter of a lane-per-edge scan's.
constexpr int kLaneEdges = 4;
constexpr int kStep = kWave * kLaneEdges;

struct LaneMarks {
  int first_k, last_k;  // first and last marked edge among the lane's four, -1 = none
  int last_packed;      // (position + 1) << 8 | mark of the last one, 0 = none
};

__device__ __forceinline__ LaneMarks scan_lane_marks(const int (&m)[kLaneEdges], int at0) {
  LaneMarks lm;
  lm.first_k = lm.last_k = -1;
  lm.last_packed = 0;
#pragma unroll
  for (int k = 0; k < kLaneEdges; ++k) {
    if (m[k]) {
      if (lm.first_k < 0) lm.first_k = k;
      lm.last_k = k;
      lm.last_packed = (at0 + k + 1) << 8 | m[k];
    }
  }
  return lm;
}

// Value of the lane `CTRL` names (a data-parallel-primitive move inside the vector ALU, no
// trip through the LDS crossbar); lanes without a source, or outside ROWS, get `fill`.
// 0x111/0x112/0x114/0x118: the lane 1/2/4/8 below in the same row of 16; 0x142: lane 15 of
// the row below (rows 1 and 3 with ROWS = 0xa); 0x143: lane 31 (rows 2 and 3 with 0xc).
template <int CTRL, int ROWS>
__device__ __forceinline__ int lane_move(int fill, int v) {
  return __builtin_amdgcn_update_dpp(fill, v, CTRL, ROWS, 0xf, false);
}

// latest mark at or before the end of each lane (inclusive) given the lanes' own last marks;
// positions grow with the lane, so a maximum is "the latest".  Marks are >= 0.
__device__ __forceinline__ int latest_inclusive(int last_packed, int carried, int) {
  int p = last_packed;
  int y;
  y = lane_move<0x111, 0xf>(0, p); p = y > p ? y : p;
  y = lane_move<0x112, 0xf>(0, p); p = y > p ? y : p;
  y = lane_move<0x114, 0xf>(0, p); p = y > p ? y : p;
  y = lane_move<0x118, 0xf>(0, p); p = y > p ? y : p;
  y = lane_move<0x142, 0xa>(0, p); p = y > p ? y : p;
  y = lane_move<0x143, 0xc>(0, p); p = y > p ? y : p;
  return p > carried ? p : carried;
}

// inclusive sums of x over the lanes below that share the lane's key; keys do not decrease
// with the lane and are >= 0
__device__ __forceinline__ float keyed_inclusive_sum(float x, int key) {
#define GS_KEYED_STEP(CTRL, ROWS)                                                       \
  {                                                                                     \
    const int ky = lane_move<CTRL, ROWS>(-1, key);                                      \
    const float y = __builtin_bit_cast(float, lane_move<CTRL, ROWS>(0, __builtin_bit_cast(int, x))); \
    if (ky == key) x += y;                                                              \
  }
  GS_KEYED_STEP(0x111, 0xf)
  GS_KEYED_STEP(0x112, 0xf)
  GS_KEYED_STEP(0x114, 0xf)
  GS_KEYED_STEP(0x118, 0xf)
  GS_KEYED_STEP(0x142, 0xa)
  GS_KEYED_STEP(0x143, 0xc)
#undef GS_KEYED_STEP
  return x;
}

__device__ __forceinline__ int owner_of_mark(int packed) { return (packed & 0xFF) - 2; }

// sums is indexed by segment (nmap applied when given)
template <typename IdT>
__global__ void __launch_bounds__(kThreads)
long_segments_kernel(const int64_t* __restrict__ indptr, const int64_t* __restrict__ emap,
                     const IdT* __restrict__ nmap, const float* __restrict__ data,
                     int64_t num_seg, int64_t nnz, int powk, float* __restrict__ sums, Chunks ck) {
  __shared__ __attribute__((aligned(16))) int s_mark[kWaves][kChunk];
  if (*ck.any_long == 0u) return;
  if (indptr[num_seg] < nnz) nnz = indptr[num_seg];  // the caller's count is an upper bound
  const int lane = threadIdx.x & (kWave - 1);
  const int64_t c = static_cast<int64_t>(blockIdx.x) * kWaves + threadIdx.x / kWave;
  const int64_t begin = c * kChunk;
  if (begin >= nnz) return;
  const int64_t end = begin + kChunk < nnz ? begin + kChunk : nnz;
  int* mark = s_mark[threadIdx.x / kWave];
  const Owned own = load_owned(indptr, ck, c, lane);
  // no long segment touches the chunk (a chunk of a thousand one-edge rows): nothing to do
  if (__ballot(own.g >= 0) == 0ull) {
    if (lane == 0) ck.outgoing[c] = -1;
    return;
  }
  // The whole chunk lies inside the incoming segment (most chunks of a hub column do): one
  // sum, no marks, no scans.
  if (__shfl(own.g >= 0 ? own.e : int64_t(0), kIncomingLane, kWave) >= end) {
    float acc = 0.0f;
    if (!emap && end - begin == kChunk && (reinterpret_cast<uintptr_t>(data) & 15u) == 0) {
#pragma unroll
      for (int t = 0; t < kChunk / kStep; ++t) {
        const float4 v = *reinterpret_cast<const float4*>(data + begin + t * kStep + lane * kLaneEdges);
        acc += (powk_f(v.x, powk) + powk_f(v.y, powk)) + (powk_f(v.z, powk) + powk_f(v.w, powk));
      }
    } else if (end - begin == kChunk) {
      // the same additions in the same order through an edge map (or from unaligned data), so
      // that a sum does not depend on which of its layouts a graph holds
#pragma unroll
      for (int t = 0; t < kChunk / kStep; ++t) {
        const int64_t e = begin + t * kStep + lane * kLaneEdges;
        float v[kLaneEdges];
#pragma unroll
        for (int k = 0; k < kLaneEdges; ++k) v[k] = powk_f(data[emap ? emap[e + k] : e + k], powk);
        acc += (v[0] + v[1]) + (v[2] + v[3]);
      }
    } else {
      for (int64_t e = begin + lane; e < end; e += kWave)
        acc += powk_f(data[emap ? emap[e] : e], powk);
    }
#pragma unroll
    for (int d = kWave / 2; d > 0; d >>= 1) acc += __shfl_xor(acc, d, kWave);
    if (lane == 0) {
      ck.carry[2 * c] = acc;
      ck.outgoing[c] = -1;
    }
    return;
  }
  // An incoming segment of which fewer than four edges are left would start and stop inside
  // the first lane, the one case of a run that does not reach beyond a lane: it gets no marks
  // and lane 0 adds it up by itself.
  const int64_t in_left = __shfl(own.g >= 0 ? own.e - begin : int64_t(0), kIncomingLane, kWave);
  const int tiny = in_left < kLaneEdges ? static_cast<int>(in_left) : 0;
  // a full chunk of plain data: all four steps' reads are issued before the marks are made,
  // so that the scans below do not wait for memory step by step
  const bool ahead = !emap && end - begin == kChunk && (reinterpret_cast<uintptr_t>(data) & 15u) == 0;
  float4 early[kChunk / kStep];
  if (ahead) {
#pragma unroll
    for (int t = 0; t < kChunk / kStep; ++t)
      early[t] = *reinterpret_cast<const float4*>(data + begin + t * kStep + lane * kLaneEdges);
  }
  write_marks(mark, own, begin, end, lane, tiny > 0 && lane == kIncomingLane);
  int carried = 0;       // latest mark at the end of the step before
  bool open = false;     // that mark's segment is a long one: its run goes on
  float acc_open = 0.0f;
#pragma unroll
  for (int t = 0; t < kChunk / kStep; ++t) {
    const int64_t base = begin + t * kStep;
    if (base >= end) break;
    const int at0 = static_cast<int>(base - begin) + lane * kLaneEdges;
    const int64_t e0 = base + lane * kLaneEdges;
    int m[kLaneEdges];
    float v[kLaneEdges];
    {
      const int4 mm = *reinterpret_cast<const int4*>(mark + at0);
      m[0] = mm.x; m[1] = mm.y; m[2] = mm.z; m[3] = mm.w;
    }
    if (ahead) {
      v[0] = powk_f(early[t].x, powk);
      v[1] = powk_f(early[t].y, powk);
      v[2] = powk_f(early[t].z, powk);
      v[3] = powk_f(early[t].w, powk);
    } else {
#pragma unroll
      for (int k = 0; k < kLaneEdges; ++k) {
        const int64_t e = e0 + k;
        if (e >= end) m[k] = 0;
        v[k] = e < end ? powk_f(data[emap ? emap[e] : e], powk) : 0.0f;
      }
    }
    if (tiny > 0 && base == begin && lane == 0) {
      float piece = 0.0f;
#pragma unroll
      for (int k = 0; k < kLaneEdges - 1; ++k)
        if (k < tiny) piece += v[k];
      ck.carry[2 * c] = piece;
    }
    const LaneMarks lm = scan_lane_marks(m, at0);
    const bool has_mark = lm.first_k >= 0;
    float pre = 0.0f, post = 0.0f;  // edges before the first mark; from the last mark on
#pragma unroll
    for (int k = 0; k < kLaneEdges; ++k) {
      if (!has_mark || k < lm.first_k) pre += v[k];
      if (has_mark && k >= lm.last_k) post += v[k];
    }
    const int incl = latest_inclusive(lm.last_packed, carried, lane);
    // the mark in force where the lane begins: the lane below's (0x138: the whole wave
    // moved up by one lane), the step before's for lane 0
    const int in_packed = lane_move<0x138, 0xf>(carried, incl);
    const int in_owner = owner_of_mark(in_packed);
    // one value per lane: the start of a run where the lane holds a mark, else its four edges
    float x = has_mark ? (owner_of_mark(incl) >= 0 ? post : 0.0f) : (in_owner >= 0 ? pre : 0.0f);
    x = keyed_inclusive_sum(x, incl);
    // the incoming run's sum over the lanes before
    const float x_prev = __builtin_bit_cast(float, lane_move<0x138, 0xf>(0, __builtin_bit_cast(int, x)));
    const int src = in_owner >= 0 ? in_owner : 0;
    const int64_t in_b = __shfl(own.b, src, kWave);
    const int in_g = __shfl(own.g, src, kWave);
    if (has_mark && in_owner >= 0) {  // the incoming long run stops at this lane's first mark
      float total = x_prev + pre;
      if (open && in_packed == carried) total += acc_open;
      if (in_b >= begin)
        sums[nmap ? static_cast<int64_t>(nmap[in_g]) : in_g] = total;
      else
        ck.carry[2 * c] = total;
    }
    const int last = __builtin_amdgcn_readlane(incl, kWave - 1);
    const float x_last =
        __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, x), kWave - 1));
    const bool goes_on = owner_of_mark(last) >= 0;
    acc_open = goes_on ? x_last + (open && last == carried ? acc_open : 0.0f) : 0.0f;
    open = goes_on;
    carried = last;
  }
  // the run in force at the end of the chunk
  int out_g = -1;
  if (open) {
    const int owner = owner_of_mark(carried);
    const int64_t ob = __shfl(own.b, owner, kWave);
    const int64_t oe = __shfl(own.e, owner, kWave);
    const int og = __shfl(own.g, owner, kWave);
    if (lane == 0) {
      if (oe == end) {
        if (ob >= begin)
          sums[nmap ? static_cast<int64_t>(nmap[og]) : og] = acc_open;
        else
          ck.carry[2 * c] = acc_open;
      } else {
        ck.carry[ob >= begin ? 2 * c + 1 : 2 * c] = acc_open;
      }
    }
    if (oe != end && ob >= begin) out_g = og;
  }
  if (lane == 0) ck.outgoing[c] = out_g;
}

constexpr int64_t kCarryAlone = 16;  // pieces a single lane adds up by itself

// One lane per chunk: a chunk that holds the head of a long segment going on after it adds
// up the pieces, in chunk order.  A segment that goes on over more than 16 chunks (a hub
// column: hundreds) is added up by the whole wave instead of one lane walking the pieces.
template <typename IdT>
__global__ void __launch_bounds__(kThreads)
carry_kernel(const int64_t* __restrict__ indptr, const IdT* __restrict__ nmap, int64_t num_seg,
             int64_t nnz, float* __restrict__ sums, Chunks ck) {
  if (*ck.any_long == 0u) return;
  if (indptr[num_seg] < nnz) nnz = indptr[num_seg];
  const int lane = threadIdx.x & (kWave - 1);
  const int64_t c = static_cast<int64_t>(blockIdx.x) * kThreads + threadIdx.x;
  int g = -1;
  int64_t last = 0;  // last chunk the segment reaches
  if (c * kChunk < nnz) {
    g = ck.outgoing[c];
    if (g >= 0) last = (indptr[g + 1] - 1) / kChunk;
  }
  const bool wide = g >= 0 && last - c > kCarryAlone;
  if (g >= 0 && !wide) {
    float total = ck.carry[2 * c + 1];
    for (int64_t k = c + 1; k <= last; ++k) total += ck.carry[2 * k];
    sums[nmap ? static_cast<int64_t>(nmap[g]) : g] = total;
  }
  unsigned long long todo = __ballot(wide);
  while (todo) {
    const int l = __ffsll(static_cast<long long>(todo)) - 1;
    todo &= todo - 1;
    const int64_t from = __shfl(c, l, kWave) + 1;
    const int64_t to = __shfl(last, l, kWave);
    float part = 0.0f;
    for (int64_t k = from + lane; k <= to; k += kWave) part += ck.carry[2 * k];
#pragma unroll
    for (int d = kWave / 2; d > 0; d >>= 1) part += __shfl_xor(part, d, kWave);
    if (lane == l) sums[nmap ? static_cast<int64_t>(nmap[g]) : g] = ck.carry[2 * c + 1] + part;
  }
}

// The steps of a chunk in the divide pass.  AHEAD: a full chunk of plain, aligned data, whose
// four reads were issued before the marks were made; that variant contains no read at all, so
// its stores follow one another without waiting (in one body with the other variant every
// step waited for the store of the step before: a read that may happen makes the compiler
// wait for all that is in flight).
template <bool AHEAD>
__device__ __forceinline__ void divide_steps(const int* mark, const Owned& own, float own_sum,
                                             const float4 (&early)[kChunk / kStep],
                                             const int64_t* __restrict__ emap,
                                             const float* __restrict__ data, int64_t begin,
                                             int64_t end, int lane, float* __restrict__ out) {
  int carried = 0;
#pragma unroll
  for (int t = 0; t < kChunk / kStep; ++t) {
    const int64_t base = begin + t * kStep;
    if (!AHEAD && base >= end) break;
    const int at0 = static_cast<int>(base - begin) + lane * kLaneEdges;
    const int64_t e0 = base + lane * kLaneEdges;
    int m[kLaneEdges];
    {
      const int4 mm = *reinterpret_cast<const int4*>(mark + at0);
      m[0] = mm.x; m[1] = mm.y; m[2] = mm.z; m[3] = mm.w;
    }
    if (!AHEAD) {
#pragma unroll
      for (int k = 0; k < kLaneEdges; ++k)
        if (e0 + k >= end) m[k] = 0;
    }
    const LaneMarks lm = scan_lane_marks(m, at0);
    const int incl = latest_inclusive(lm.last_packed, carried, lane);
    int cur = lane_move<0x138, 0xf>(carried, incl);
    carried = __builtin_amdgcn_readlane(incl, kWave - 1);
    const float have[kLaneEdges] = {early[t].x, early[t].y, early[t].z, early[t].w};
    float res[kLaneEdges];
    bool mine[kLaneEdges];
#pragma unroll
    for (int k = 0; k < kLaneEdges; ++k) {
      if (m[k]) cur = (at0 + k + 1) << 8 | m[k];
      const int owner = owner_of_mark(cur);
      const float total = __shfl(own_sum, owner >= 0 ? owner : 0, kWave);
      const int64_t e = e0 + k;
      mine[k] = (AHEAD || e < end) && owner >= 0;
      res[k] = 0.0f;
      if (AHEAD) res[k] = have[k] / total;
      else if (mine[k]) res[k] = data[emap ? emap[e] : e] / total;
    }
    if (AHEAD && mine[0] && mine[1] && mine[2] && mine[3]) {
      *reinterpret_cast<float4*>(out + e0) = make_float4(res[0], res[1], res[2], res[3]);
    } else {
#pragma unroll
      for (int k = 0; k < kLaneEdges; ++k)
        if (mine[k]) out[!AHEAD && emap ? emap[e0 + k] : e0 + k] = res[k];
    }
  }
}

// out[d] = data[d] / sums[segment of e] for the edges of long segments
__global__ void __launch_bounds__(kThreads)
long_divide_kernel(const int64_t* __restrict__ indptr, const int64_t* __restrict__ emap,
                   const float* __restrict__ data, int64_t num_seg, int64_t nnz,
                   const float* __restrict__ sums, float* __restrict__ out, Chunks ck) {
  __shared__ __attribute__((aligned(16))) int s_mark[kWaves][kChunk];
  if (*ck.any_long == 0u) return;
  if (indptr[num_seg] < nnz) nnz = indptr[num_seg];
  const int lane = threadIdx.x & (kWave - 1);
  const int64_t c = static_cast<int64_t>(blockIdx.x) * kWaves + threadIdx.x / kWave;
  const int64_t begin = c * kChunk;
  if (begin >= nnz) return;
  const int64_t end = begin + kChunk < nnz ? begin + kChunk : nnz;
  int* mark = s_mark[threadIdx.x / kWave];
  const Owned own = load_owned(indptr, ck, c, lane);
  if (__ballot(own.g >= 0) == 0ull) return;  // no long segment touches the chunk
  const float own_sum = own.g >= 0 ? sums[own.g] : 0.0f;
  // a full chunk of plain data: all four steps' reads are issued together
  const bool ahead = !emap && end - begin == kChunk &&
                     ((reinterpret_cast<uintptr_t>(data) | reinterpret_cast<uintptr_t>(out)) & 15u) == 0;
  float4 early[kChunk / kStep];
#pragma unroll
  for (int t = 0; t < kChunk / kStep; ++t) early[t] = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
  // the whole chunk lies inside the incoming segment: one divisor, no marks
  if (__shfl(own.g >= 0 ? own.e : int64_t(0), kIncomingLane, kWave) >= end) {
    const float total = __shfl(own_sum, kIncomingLane, kWave);
    if (ahead) {
#pragma unroll
      for (int t = 0; t < kChunk / kStep; ++t)
        early[t] = *reinterpret_cast<const float4*>(data + begin + t * kStep + lane * kLaneEdges);
#pragma unroll
      for (int t = 0; t < kChunk / kStep; ++t)
        *reinterpret_cast<float4*>(out + begin + t * kStep + lane * kLaneEdges) =
            make_float4(early[t].x / total, early[t].y / total, early[t].z / total,
                        early[t].w / total);
      return;
    }
    for (int64_t e = begin + lane; e < end; e += kWave) {
      const int64_t d = emap ? emap[e] : e;
      out[d] = data[d] / total;
    }
    return;
  }
  if (ahead) {
#pragma unroll
    for (int t = 0; t < kChunk / kStep; ++t)
      early[t] = *reinterpret_cast<const float4*>(data + begin + t * kStep + lane * kLaneEdges);
  }
  write_marks(mark, own, begin, end, lane);
  if (ahead)
    divide_steps<true>(mark, own, own_sum, early, emap, data, begin, end, lane, out);
  else
    divide_steps<false>(mark, own, own_sum, early, emap, data, begin, end, lane, out);
}

inline int64_t num_chunks(int64_t nnz) { return nnz <= 0 ? 1 : (nnz + kChunk - 1) / kChunk; }

struct SegmentScratch {
  Chunks ck;
  float* sums;  // normalize only
  bool ok;
};

SegmentScratch carve_segment(void* workspace, size_t bytes, int64_t nnz, int64_t num_seg,
                             bool with_sums) {
  Carver ws(workspace, bytes);
  const int64_t chunks = num_chunks(nnz);
  SegmentScratch s;
  s.ck.any_long = ws.take<unsigned int>(64);
  s.ck.count = ws.take<unsigned int>(chunks);
  s.ck.list = ws.take<int>(chunks * kChunkList);
  s.ck.incoming = ws.take<int>(chunks);
  s.ck.outgoing = ws.take<int>(chunks);
  s.ck.carry = ws.take<float>(2 * chunks);
  s.sums = with_sums ? ws.take<float>(num_seg > 0 ? num_seg : 1) : nullptr;
  s.ok = ws.ok;
  return s;
}

size_t segment_workspace_bytes(int64_t num_seg, int64_t nnz) {
  const size_t chunks = static_cast<size_t>(num_chunks(nnz));
  return padded(256) + 3 * padded(chunks * 4) + padded(chunks * kChunkList * 4) +
         padded(chunks * 8) + padded(static_cast<size_t>(num_seg > 0 ? num_seg : 1) * 4);
}

template <typename IdT>
int segment_sum_impl(const int64_t* indptr, const int64_t* emap, const void* nmap,
                     const float* data, int64_t num_seg, int64_t nnz, int powk, float* out,
                     const SegmentScratch& s, hipStream_t st) {
  const IdT* nm = static_cast<const IdT*>(nmap);
  const int64_t chunks = num_chunks(nnz);
  hipLaunchKernelGGL(clear_chunks_kernel, dim3(blocks_for(chunks, kThreads)), dim3(kThreads), 0, st,
                     s.ck, chunks);
  if (emap)
    hipLaunchKernelGGL((short_segments_kernel<false, true, IdT>), dim3(blocks_for(num_seg, kThreads)),
                       dim3(kThreads), 0, st, indptr, emap, nm, data, num_seg, nnz, powk, out, s.ck);
  else
    hipLaunchKernelGGL((short_segments_kernel<false, false, IdT>), dim3(blocks_for(num_seg, kThreads)),
                       dim3(kThreads), 0, st, indptr, emap, nm, data, num_seg, nnz, powk, out, s.ck);
  if (nnz > kLaneMaxLen) {
    hipLaunchKernelGGL(long_segments_kernel<IdT>, dim3(blocks_for(chunks, kWaves)), dim3(kThreads),
                       0, st, indptr, emap, nm, data, num_seg, nnz, powk, out, s.ck);
    hipLaunchKernelGGL(carry_kernel<IdT>, dim3(blocks_for(chunks, kThreads)), dim3(kThreads), 0, st,
                       indptr, nm, num_seg, nnz, out, s.ck);
  }
  return check_launch("segment_sum");
}

// Sums by an arbitrary key (COO targets).  The reference adds every edge to its target with a
// global atomic (graph_ops.cu:45-64, edge_map_reduce.cu:15-23); on a power-law graph thousands
// of those hit the same address -- a hub row, or the one column a run of a column-sorted COO
// belongs to -- and queue up at the memory side (tens of ns each).  Here a workgroup first
// gathers its 2048 edges in an LDS table keyed by target (LDS atomics), then issues one global
// add per distinct target: a 300 000-edge hub costs 150 global adds instead of 300 000.  The
// adds are the hardware's fp32 adds, not the compare-and-swap loop a plain atomicAdd(float*)
// compiles to here.
constexpr int kAggEdges = 8;                   // edges per thread
constexpr int kAggTile = kThreads * kAggEdges;
constexpr int kAggSlots = 2 * kAggTile;        // LDS table: load <= 1/2

struct KeyedSums {
  long long key[kAggSlots];
  float sum[kAggSlots];
};

__device__ __forceinline__ void keyed_clear(KeyedSums& t) {
  for (int i = threadIdx.x; i < kAggSlots; i += kThreads) {
    t.key[i] = -1;
    t.sum[i] = 0.0f;
  }
  __syncthreads();
}

__device__ __forceinline__ void keyed_add(KeyedSums& t, long long key, float v) {
  unsigned int h = static_cast<unsigned int>((static_cast<unsigned long long>(key) *
                                              0x9E3779B97F4A7C15ull) >> 40) & (kAggSlots - 1);
  while (true) {
    const long long seen = static_cast<long long>(
        atomicCAS(reinterpret_cast<unsigned long long*>(&t.key[h]), ~0ull,
                  static_cast<unsigned long long>(key)));
    if (seen == -1 || seen == key) break;
    h = (h + 1) & (kAggSlots - 1);
  }
  unsafeAtomicAdd(&t.sum[h], v);
}

// (a key outside [0, bound) is left out)
__device__ __forceinline__ void keyed_flush(KeyedSums& t, float* __restrict__ out,
                                            long long bound = 0x7FFFFFFFFFFFFFFFll) {
  __syncthreads();
  for (int i = threadIdx.x; i < kAggSlots; i += kThreads)
    if (t.key[i] >= 0 && t.key[i] < bound) unsafeAtomicAdd(out + t.key[i], t.sum[i]);
}

// out[target[e]] += f(data[emap ? emap[e] : e])   (graph_ops.cu:45-64)
template <typename IdT>
__global__ void __launch_bounds__(kThreads)
coo_sum_kernel(const IdT* __restrict__ target, const int64_t* __restrict__ emap,
               const float* __restrict__ data, int64_t E, int powk, float* __restrict__ out,
               int64_t bound) {
  __shared__ KeyedSums table;
  keyed_clear(table);
  const int64_t base = static_cast<int64_t>(blockIdx.x) * kAggTile + threadIdx.x;
#pragma unroll
  for (int k = 0; k < kAggEdges; ++k) {
    const int64_t e = base + static_cast<int64_t>(k) * kThreads;
    if (e < E)
      keyed_add(table, static_cast<long long>(target[e]),
                powk_f(data[emap ? emap[e] : e], powk));
  }
  keyed_flush(table, out, bound);
}

// edge_map_reduce.cu:15-23
template <typename IdT>
__global__ void __launch_bounds__(kThreads)
e_div_u_sum_kernel(const IdT* __restrict__ row, const IdT* __restrict__ col,
                   const float* __restrict__ data, const float* __restrict__ divisor, int64_t E,
                   float* __restrict__ out_data, float* __restrict__ out_sum) {
  __shared__ KeyedSums table;
  keyed_clear(table);
  const int64_t base = static_cast<int64_t>(blockIdx.x) * kAggTile + threadIdx.x;
#pragma unroll
  for (int k = 0; k < kAggEdges; ++k) {
    const int64_t e = base + static_cast<int64_t>(k) * kThreads;
    if (e < E) {
      const float v = data[e] / divisor[row[e]];
      out_data[e] = v;
      keyed_add(table, static_cast<long long>(col[e]), v);
    }
  }
  keyed_flush(table, out_sum);
}

}  // namespace
}  // namespace gs

using namespace gs;

extern "C" {

size_t gs_segment_workspace_bytes(int64_t num_segments, int64_t nnz) {
  return segment_workspace_bytes(num_segments, nnz);
}

int gs_segment_sum(const int64_t* indptr, const int64_t* e_ids, const void* n_ids, int id_bytes,
                   const float* data, int64_t num_segments, int64_t nnz, int64_t powk, float* out,
                   void* workspace, size_t workspace_bytes, void* stream) {
  GS_REQUIRE(num_segments >= 0 && nnz >= 0 && powk >= 1,
             "gs_segment_sum: negative size or powk < 1");
  GS_REQUIRE(num_segments == 0 || (indptr && out && (nnz == 0 || data)),
             "gs_segment_sum: null pointer");
  GS_REQUIRE(!n_ids || valid_id_bytes(id_bytes), "gs_segment_sum: id_bytes must be 4 or 8, got %d",
             id_bytes);
  GS_REQUIRE(num_segments < (int64_t(1) << 31), "gs_segment_sum: more than 2^31 segments");
  if (num_segments == 0) return GS_OK;
  SegmentScratch s = carve_segment(workspace, workspace_bytes, nnz, num_segments, false);
  if (!s.ok) {
    set_error_text("gs_segment_sum: workspace needs %zu bytes, 256-byte aligned",
                   gs_segment_workspace_bytes(num_segments, nnz));
    return GS_ERR_WORKSPACE;
  }
  hipStream_t st = static_cast<hipStream_t>(stream);
  return n_ids && id_bytes == 4
             ? segment_sum_impl<int32_t>(indptr, e_ids, n_ids, data, num_segments, nnz,
                                         static_cast<int>(powk), out, s, st)
             : segment_sum_impl<int64_t>(indptr, e_ids, n_ids, data, num_segments, nnz,
                                         static_cast<int>(powk), out, s, st);
}

int gs_coo_sum(const void* target, int id_bytes, const int64_t* e_ids, const float* data, int64_t E,
               int64_t powk, float* out, void* stream) {
  return gs::coo_sum_bounded(target, id_bytes, e_ids, data, E, powk,
                             std::numeric_limits<int64_t>::max(), out, stream);
}

}  // extern "C"

// gs_coo_sum with targets outside [0, num_targets) left out (gs_coo_sum_binned's other path)
int gs::coo_sum_bounded(const void* target, int id_bytes, const int64_t* e_ids, const float* data,
                        int64_t E, int64_t powk, int64_t num_targets, float* out, void* stream) {
  GS_REQUIRE(E >= 0 && powk >= 1, "gs_coo_sum: negative size or powk < 1");
  GS_REQUIRE(E == 0 || (target && data && out), "gs_coo_sum: null pointer");
  GS_REQUIRE(valid_id_bytes(id_bytes), "gs_coo_sum: id_bytes must be 4 or 8, got %d", id_bytes);
  if (E == 0) return GS_OK;
  const dim3 grid(blocks_for(E, kAggTile));
  hipStream_t st = static_cast<hipStream_t>(stream);
  if (id_bytes == 8)
    hipLaunchKernelGGL(coo_sum_kernel<int64_t>, grid, dim3(kThreads), 0, st,
                       static_cast<const int64_t*>(target), e_ids, data, E, static_cast<int>(powk),
                       out, num_targets);
  else
    hipLaunchKernelGGL(coo_sum_kernel<int32_t>, grid, dim3(kThreads), 0, st,
                       static_cast<const int32_t*>(target), e_ids, data, E, static_cast<int>(powk),
                       out, num_targets);
  return check_launch("coo_sum");
}

extern "C" {


int gs_segment_normalize(const int64_t* indptr, const int64_t* e_ids, const float* data,
                         int64_t num_segments, int64_t nnz, float* out, void* workspace,
                         size_t workspace_bytes, void* stream) {
  GS_REQUIRE(num_segments >= 0 && nnz >= 0 && num_segments < (int64_t(1) << 31),
             "gs_segment_normalize: negative size or more than 2^31 segments");
  GS_REQUIRE(num_segments == 0 || nnz == 0 || (indptr && data && out),
             "gs_segment_normalize: null pointer");
  if (num_segments == 0 || nnz == 0) return GS_OK;
  SegmentScratch s = carve_segment(workspace, workspace_bytes, nnz, num_segments, true);
  if (!s.ok) {
    set_error_text("gs_segment_normalize: workspace needs %zu bytes, 256-byte aligned",
                   gs_segment_workspace_bytes(num_segments, nnz));
    return GS_ERR_WORKSPACE;
  }
  hipStream_t st = static_cast<hipStream_t>(stream);
  const int64_t* no_map = nullptr;
  const int64_t chunks = num_chunks(nnz);
  hipLaunchKernelGGL(clear_chunks_kernel, dim3(blocks_for(chunks, kThreads)), dim3(kThreads), 0, st,
                     s.ck, chunks);
  if (e_ids)
    hipLaunchKernelGGL((short_segments_kernel<true, true, int64_t>),
                       dim3(blocks_for(num_segments, kThreads)), dim3(kThreads), 0, st, indptr,
                       e_ids, no_map, data, num_segments, nnz, 1, out, s.ck);
  else
    hipLaunchKernelGGL((short_segments_kernel<true, false, int64_t>),
                       dim3(blocks_for(num_segments, kThreads)), dim3(kThreads), 0, st, indptr,
                       e_ids, no_map, data, num_segments, nnz, 1, out, s.ck);
  if (nnz > kLaneMaxLen) {
    hipLaunchKernelGGL(long_segments_kernel<int64_t>, dim3(blocks_for(chunks, kWaves)),
                       dim3(kThreads), 0, st, indptr, e_ids, no_map, data, num_segments, nnz, 1,
                       s.sums, s.ck);
    hipLaunchKernelGGL(carry_kernel<int64_t>, dim3(blocks_for(chunks, kThreads)), dim3(kThreads), 0,
                       st, indptr, no_map, num_segments, nnz, s.sums, s.ck);
    hipLaunchKernelGGL(long_divide_kernel, dim3(blocks_for(chunks, kWaves)), dim3(kThreads), 0, st,
                       indptr, e_ids, data, num_segments, nnz, s.sums, out, s.ck);
  }
  return check_launch("segment_normalize");
}

int gs_e_div_u_sum(const void* row, const void* col, int id_bytes, const float* data,
                   const float* divisor, int64_t E, float* out_data, float* out_sum,
                   void* stream) {
  GS_REQUIRE(E >= 0, "gs_e_div_u_sum: negative size");
  GS_REQUIRE(E == 0 || (row && col && data && divisor && out_data && out_sum),
             "gs_e_div_u_sum: null pointer");
  GS_REQUIRE(valid_id_bytes(id_bytes), "gs_e_div_u_sum: id_bytes must be 4 or 8, got %d", id_bytes);
  if (E == 0) return GS_OK;
  const dim3 grid(blocks_for(E, kAggTile));
  hipStream_t st = static_cast<hipStream_t>(stream);
  if (id_bytes == 8)
    hipLaunchKernelGGL(e_div_u_sum_kernel<int64_t>, grid, dim3(kThreads), 0, st,
                       static_cast<const int64_t*>(row), static_cast<const int64_t*>(col), data,
                       divisor, E, out_data, out_sum);
  else
    hipLaunchKernelGGL(e_div_u_sum_kernel<int32_t>, grid, dim3(kThreads), 0, st,
                       static_cast<const int32_t*>(row), static_cast<const int32_t*>(col), data,
                       divisor, E, out_data, out_sum);
  return check_launch("e_div_u_sum");
}

}  // extern "C"
