// Shared device/host helpers for the gfx950 kernels: status reporting, the
// Philox draw, wave-level primitives and a tiled exclusive scan.
#pragma once

#include <hip/hip_runtime.h>
#include <type_traits>
#include <utility>
#include <stdint.h>

#include "../../include/gs_hip.h"

namespace gs {

constexpr int kWave = 64;  // CDNA wavefront width

// ---------------------------------------------------------------- status ----
void set_error_text(const char* fmt, ...);

inline int check_launch(const char* what) {
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) {
    set_error_text("%s: %s", what, hipGetErrorString(e));
    return GS_ERR_LAUNCH;
  }
  return GS_OK;
}

#define GS_REQUIRE(cond, ...)            \
  do {                                   \
    if (!(cond)) {                       \
      ::gs::set_error_text(__VA_ARGS__); \
      return GS_ERR_INVALID_ARG;         \
    }                                    \
  } while (0)

#define GS_RETURN_IF_ERROR(expr) \
  do {                           \
    int _s = (expr);             \
    if (_s != GS_OK) return _s;  \
  } while (0)

inline bool valid_id_bytes(int b) { return b == 4 || b == 8; }

// ------------------------------------------------------------- profiling ----
// Optional per-kernel timing for benchmarks: when gs_profile_enable(name) names
// this launch site, the launch is bracketed by a hipEvent pair on its stream
// (see gs_profile_collect).  Off by default: one relaxed load per launch.
void profile_begin(const char* name, hipStream_t stream, int* slot);
void profile_end(hipStream_t stream, int slot);
struct ProfileScope {
  hipStream_t stream;
  int slot = -1;
  ProfileScope(const char* name, hipStream_t s) : stream(s) { profile_begin(name, s, &slot); }
  ~ProfileScope() {
    if (slot >= 0) profile_end(stream, slot);
  }
};

// ---------------------------------------------------------- phase stamps ----
// Only in builds with -DGS_PHASE_STAMPS (a measuring build, never the shipped library):
// thread 0 of every workgroup reads the 100 MHz wall clock at the marked places of a kernel,
// after waiting for its outstanding memory operations, and appends one record
// {kind, tile, tiles, stamps...} to a buffer the host registered per translation unit.
// Without the flag every macro below expands to nothing.
#ifdef GS_PHASE_STAMPS
constexpr int kStampSlots = 12;
constexpr int kStampRecordWords = 16;  // kind, tile, tiles, n, then the stamps
#define GS_STAMPS_DEFINE(tu)                                                            \
  namespace gs {                                                                        \
  static __device__ unsigned long long* g_stamp_buf;                                    \
  }                                                                                     \
  extern "C" int gs_debug_set_stamps_##tu(void* buf) {                                  \
    unsigned long long* p = static_cast<unsigned long long*>(buf);                      \
    return hipMemcpyToSymbol(HIP_SYMBOL(gs::g_stamp_buf), &p, sizeof(p)) == hipSuccess  \
               ? GS_OK                                                                  \
               : GS_ERR_LAUNCH;                                                         \
  }
#define GS_STAMP_BEGIN() unsigned long long _st[::gs::kStampSlots] = {}
#define GS_STAMP(k)                                                \
  do {                                                             \
    if (threadIdx.x == 0) {                                        \
      asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");  \
      _st[k] = wall_clock64();                                     \
    }                                                              \
  } while (0)
#define GS_STAMP_END(kind, n)                                                                 \
  do {                                                                                        \
    unsigned long long* _b = ::gs::g_stamp_buf;                                               \
    /* in large grids one workgroup in 16 (and the last) reports: the shared cursor is a */  \
    /* same-address atomic, and thousands of those would be what the stamps measure      */  \
    if (threadIdx.x == 0 && _b &&                                                             \
        (gridDim.x <= 256 || (blockIdx.x & 15u) == 0 || blockIdx.x == gridDim.x - 1)) {       \
      const unsigned long long _r = atomicAdd(&_b[0], 1ull);                                  \
      if (_r < _b[1]) {                                                                       \
        unsigned long long* _w = _b + ::gs::kStampRecordWords * (_r + 1);                     \
        _w[0] = (kind);                                                                       \
        _w[1] = blockIdx.x;                                                                   \
        _w[2] = gridDim.x;                                                                    \
        _w[3] = (n);                                                                          \
        for (int _k = 0; _k < ::gs::kStampSlots; ++_k) _w[4 + _k] = _st[_k];                  \
      }                                                                                       \
    }                                                                                         \
  } while (0)
#else
#define GS_STAMPS_DEFINE(tu)
#define GS_STAMP_BEGIN() do {} while (0)
#define GS_STAMP(k) do {} while (0)
#define GS_STAMP_END(kind, n) do {} while (0)
#endif

// Carves 256-byte aligned pieces out of the caller's workspace.
struct Carver {
  char* base;
  size_t cap;
  size_t off = 0;
  bool ok = true;
  Carver(void* p, size_t bytes) : base(static_cast<char*>(p)), cap(bytes) {
    if ((reinterpret_cast<uintptr_t>(p) & 255u) != 0) ok = false;
  }
  template <typename T>
  T* take(size_t count) {
    size_t bytes = (count * sizeof(T) + 255u) & ~size_t(255);
    if (!ok || off + bytes > cap) {
      ok = false;
      return nullptr;
    }
    T* r = reinterpret_cast<T*>(base + off);
    off += bytes;
    return r;
  }
};
inline size_t padded(size_t bytes) { return (bytes + 255u) & ~size_t(255); }

// ---------------------------------------------------------------- Philox ----
constexpr uint32_t kTagUniform = 1u;
constexpr uint32_t kTagWeighted = 2u;
constexpr uint32_t kTagWalk = 3u;
constexpr uint32_t kTagListUniform = 4u;
constexpr uint32_t kTagListWeighted = 5u;

struct U4 {
  uint32_t v[4];
};

// Philox4x32-10 (Salmon et al., SC'11).
__device__ __forceinline__ U4 philox4x32_10(uint32_t c0, uint32_t c1, uint32_t c2, uint32_t c3,
                                            uint32_t k0, uint32_t k1) {
#pragma unroll
  for (int round = 0; round < 10; ++round) {
    uint32_t hi0 = __umulhi(0xD2511F53u, c0);
    uint32_t lo0 = 0xD2511F53u * c0;
    uint32_t hi1 = __umulhi(0xCD9E8D57u, c2);
    uint32_t lo1 = 0xCD9E8D57u * c2;
    uint32_t n0 = hi1 ^ c1 ^ k0;
    uint32_t n2 = hi0 ^ c3 ^ k1;
    c0 = n0;
    c1 = lo1;
    c2 = n2;
    c3 = lo0;
    k0 += 0x9E3779B9u;
    k1 += 0xBB67AE85u;
  }
  U4 r;
  r.v[0] = c0;
  r.v[1] = c1;
  r.v[2] = c2;
  r.v[3] = c3;
  return r;
}

// The four draws for idx = 4q .. 4q+3 of `row`.
__device__ __forceinline__ U4 draw_block(uint64_t seed, uint32_t tag, uint64_t row, uint64_t q) {
  return philox4x32_10(static_cast<uint32_t>(q), static_cast<uint32_t>(row),
                       static_cast<uint32_t>(row >> 32),
                       tag | (static_cast<uint32_t>(q >> 32) << 8), static_cast<uint32_t>(seed),
                       static_cast<uint32_t>(seed >> 32));
}

__device__ __forceinline__ uint32_t draw_one(uint64_t seed, uint32_t tag, uint64_t row,
                                             uint64_t idx) {
  U4 b = draw_block(seed, tag, row, idx >> 2);
  return b.v[idx & 3];
}

// A-Res key log2(u)/w, u = ((x>>8)+1) * 2^-24.  Only correctly rounded binary32
// operations (explicit fmaf, IEEE division) so that a host evaluation of the
// same recipe gives the same bits; requires -ffp-contract=off.
__device__ __forceinline__ float log2_u24(uint32_t x) {
  uint32_t m = (x >> 8) + 1u;
  int e = 31 - __clz(static_cast<int>(m));
  float f = static_cast<float>(m) * __uint_as_float(static_cast<uint32_t>(127 - e) << 23);  // m * 2^-e, exact
  if (f > 1.41421356f) {
    f = f * 0.5f;
    e += 1;
  }
  float s = __fdiv_rn(f - 1.0f, f + 1.0f);
  float z = s * s;
  float p = __fmaf_rn(z, 0.11111111f, 0.14285715f);
  p = __fmaf_rn(z, p, 0.2f);
  p = __fmaf_rn(z, p, 0.33333334f);
  p = __fmaf_rn(z, p, 1.0f);
  float l = (s * 2.88539008f) * p;
  return l + static_cast<float>(e - 24);
}

__device__ __forceinline__ float ares_key(uint32_t x, float w) {
  if (!(w > 0.0f)) return -__builtin_inff();
  return __fdiv_rn(log2_u24(x), w);
}

// x^powk of the edge-data reductions (graph_ops.cu:30)
__device__ __forceinline__ float powk_f(float x, int powk) {
  if (powk == 1) return x;
  float p = x;
  for (int i = 1; i < powk; ++i) p *= x;
  return p;
}

// Order-preserving map float -> uint32 (larger float => larger uint).
__device__ __forceinline__ uint32_t float_to_ordered(float f) {
  uint32_t b = __float_as_uint(f);
  return (b & 0x80000000u) ? ~b : (b | 0x80000000u);
}

// ------------------------------------------------------------ id helpers ----
template <typename T>
__device__ __forceinline__ T ld(const T* p) {
  return *p;
}

inline int blocks_for(int64_t n, int per_block) {
  int64_t b = (n + per_block - 1) / per_block;
  return static_cast<int>(b < 1 ? 1 : b);
}

// ------------------------------------------------------- wave-wide search ----
// Number of leading elements of the sorted a[0..n) that are <= v (the first index whose
// element exceeds v), found by a whole wave: 64 probes split the range per step, so
// 2.45 M offsets take four dependent reads instead of twenty-two.  Every lane of the wave
// calls this and gets the answer.
__device__ __forceinline__ int64_t wave_upper_bound(const int64_t* __restrict__ a, int64_t n,
                                                    int64_t v) {
  const int lane = threadIdx.x & (kWave - 1);
  int64_t lo = 0, hi = n;
  while (lo < hi) {
    const int64_t step = (hi - lo + kWave - 1) / kWave;
    const int64_t at = lo + lane * step;
    const bool le = at < hi && a[at] <= v;
    const int count = __popcll(__ballot(le));  // probes are sorted: the first `count` are <= v
    const int64_t new_lo = count > 0 ? lo + (count - 1) * step + 1 : lo;
    const int64_t end = lo + count * step;     // first probe that exceeds v, if there is one
    hi = (count < kWave && end < hi) ? end : hi;
    lo = new_lo;
  }
  return lo;
}

// Rows (segments of the offsets ptr[0..n]) that hold positions p_first and p_last, into
// s_rows[0..1]: the first two waves of the workgroup search, every thread calls this and
// the values are there after the call (it ends with a workgroup barrier).
__device__ __forceinline__ void block_row_range(const int64_t* __restrict__ ptr, int64_t n,
                                                int64_t p_first, int64_t p_last,
                                                int64_t* s_rows) {
  const int wave = threadIdx.x / kWave;
  if (wave < 2) {
    const int64_t r = wave_upper_bound(ptr, n + 1, wave == 0 ? p_first : p_last) - 1;
    if ((threadIdx.x & (kWave - 1)) == 0) s_rows[wave] = r;
  }
  __syncthreads();
}

// ------------------------------------------------------------ block scan ----
// Exclusive scan of one int64 per thread over a block of kThreads threads
// (multiple of 64).  Returns the exclusive prefix; *total gets the block sum.
template <int kThreads>
__device__ __forceinline__ int64_t block_exclusive_scan(int64_t v, int64_t* total,
                                                        int64_t* lds /* kThreads/64 + 1 */) {
  const int lane = threadIdx.x & (kWave - 1);
  const int wave = threadIdx.x / kWave;
  int64_t incl = v;
#pragma unroll
  for (int d = 1; d < kWave; d <<= 1) {
    int64_t o = __shfl_up(incl, d, kWave);
    if (lane >= d) incl += o;
  }
  if (lane == kWave - 1) lds[wave] = incl;
  __syncthreads();
  constexpr int kWaves = kThreads / kWave;
  if (threadIdx.x == 0) {
    int64_t acc = 0;
#pragma unroll
    for (int w = 0; w < kWaves; ++w) {
      int64_t t = lds[w];
      lds[w] = acc;
      acc += t;
    }
    lds[kWaves] = acc;
  }
  __syncthreads();
  int64_t r = lds[wave] + incl - v;
  *total = lds[kWaves];
  __syncthreads();
  return r;
}

// ------------------------------------------------- device-wide scan (tiled) --
// out[i] = sum_{j<i} f(j) for i in [0, n]; out has n+1 entries.  Three phases:
// per-tile sums, a one-block scan of the tile sums, per-tile scan + offset.
// n <= kScanTile runs as a single launch.
constexpr int kScanThreads = 256;
constexpr int kScanItems = 8;
constexpr int kScanTile = kScanThreads * kScanItems;

inline int64_t scan_num_tiles(int64_t n) { return n <= 0 ? 1 : (n + kScanTile - 1) / kScanTile; }
inline size_t scan_workspace_bytes(int64_t n) { return padded((scan_num_tiles(n) + 1) * 8); }

// A scan functor is either `int64_t operator()(i)` or, when it chases a pointer, the pair
// `where(i)` (first read: which entry) and `count(entry)` (second read: its value).  The pair
// lets a thread issue the first reads of all its items, then all second reads, instead of
// walking two dependent reads per item one item after the other; neither may carry a
// condition of its own (a read that may or may not happen makes every later one wait for all
// that is in flight), so indices past the end are clamped and their values dropped.
template <typename F, typename = void>
struct scan_two_phase : std::false_type {};
template <typename F>
struct scan_two_phase<F, std::void_t<decltype(std::declval<const F&>().where(int64_t(0)))>>
    : std::true_type {};

// v[k] = f(at(k)) for at(k) < n, else 0; n > 0
template <typename F, int ITEMS, typename At>
__device__ __forceinline__ void scan_load(const F& f, int64_t n, At at, int64_t (&v)[ITEMS]) {
  if constexpr (scan_two_phase<F>::value) {
    decltype(f.where(int64_t(0))) key[ITEMS];
#pragma unroll
    for (int k = 0; k < ITEMS; ++k) key[k] = f.where(at(k) < n ? at(k) : n - 1);
#pragma unroll
    for (int k = 0; k < ITEMS; ++k) v[k] = f.count(key[k]);
  } else {
#pragma unroll
    for (int k = 0; k < ITEMS; ++k) v[k] = f(at(k) < n ? at(k) : n - 1);
  }
#pragma unroll
  for (int k = 0; k < ITEMS; ++k)
    if (at(k) >= n) v[k] = 0;
}

// Evaluates f once per item (f may chase pointers), parks the value in out[i]
// for the apply pass and reduces the tile.
template <typename F>
__global__ void __launch_bounds__(kScanThreads) scan_tile_sums_kernel(F f, int64_t n,
                                                                      int64_t* tile_sums,
                                                                      int64_t* out) {
  __shared__ int64_t lds[kScanThreads / kWave + 1];
  const int64_t base = static_cast<int64_t>(blockIdx.x) * kScanTile;
  auto at = [&](int k) { return base + k * kScanThreads + threadIdx.x; };
  int64_t v[kScanItems];
  int64_t acc = 0;
  if (n > 0) {
    scan_load(f, n, at, v);
#pragma unroll
    for (int k = 0; k < kScanItems; ++k) {
      if (at(k) < n) out[at(k)] = v[k];
      acc += v[k];
    }
  }
  int64_t total;
  block_exclusive_scan<kScanThreads>(acc, &total, lds);
  if (threadIdx.x == 0) tile_sums[blockIdx.x] = total;
}

// in-place exclusive scan of tile_sums[0..m) by one block; tile_sums[m] = total
static __global__ void __launch_bounds__(kScanThreads) scan_tile_offsets_kernel(int64_t* tile_sums,
                                                                         int64_t m) {
  __shared__ int64_t lds[kScanThreads / kWave + 1];
  int64_t carry = 0;
  for (int64_t base = 0; base < m; base += kScanThreads) {
    int64_t i = base + threadIdx.x;
    int64_t v = i < m ? tile_sums[i] : 0;
    int64_t total;
    int64_t ex = block_exclusive_scan<kScanThreads>(v, &total, lds);
    if (i < m) tile_sums[i] = carry + ex;
    carry += total;
  }
  if (threadIdx.x == 0) tile_sums[m] = carry;
}

// Thread t of the block owns items base + t*kScanItems .. +kScanItems-1 so the
// per-thread prefix is a running sum (blocked arrangement).  With `tiles` the
// item values are read back from out[] (parked there by scan_tile_sums_kernel),
// without it f is evaluated here.  SELF_PREFIX: `tiles` holds raw tile sums and
// the block adds up its predecessors itself, which saves the separate one-block
// offsets kernel when there are few tiles.
template <typename F, bool SELF_PREFIX>
__global__ void __launch_bounds__(kScanThreads) scan_apply_kernel(F f, int64_t n,
                                                                  const int64_t* tiles,
                                                                  int64_t* out) {
  __shared__ int64_t lds[kScanThreads / kWave + 1];
  int64_t tile_base = 0;
  if (tiles) {
    if (SELF_PREFIX) {
      int64_t part = 0;
      for (int64_t t = threadIdx.x; t < blockIdx.x; t += kScanThreads) part += tiles[t];
      block_exclusive_scan<kScanThreads>(part, &tile_base, lds);
    } else {
      tile_base = tiles[blockIdx.x];
    }
  }
  const int64_t base = static_cast<int64_t>(blockIdx.x) * kScanTile +
                       static_cast<int64_t>(threadIdx.x) * kScanItems;
  auto at = [&](int k) { return base + k; };
  int64_t v[kScanItems];
  int64_t acc = 0;
#pragma unroll
  for (int k = 0; k < kScanItems; ++k) v[k] = 0;
  if (n > 0) {
    if (tiles) {  // the values were parked in out by the sums pass
#pragma unroll
      for (int k = 0; k < kScanItems; ++k) v[k] = out[at(k) < n ? at(k) : n - 1];
#pragma unroll
      for (int k = 0; k < kScanItems; ++k)
        if (at(k) >= n) v[k] = 0;
    } else {
      scan_load(f, n, at, v);
    }
  }
#pragma unroll
  for (int k = 0; k < kScanItems; ++k) acc += v[k];
  int64_t total;
  int64_t ex = block_exclusive_scan<kScanThreads>(acc, &total, lds);
  int64_t run = ex + tile_base;
#pragma unroll
  for (int k = 0; k < kScanItems; ++k) {
    int64_t i = base + k;
    if (i < n) out[i] = run;
    run += v[k];
    if (i == n - 1) out[n] = run;
  }
  if (n == 0 && blockIdx.x == 0 && threadIdx.x == 0) out[0] = 0;
}

constexpr int64_t kScanSelfPrefixTiles = 4096;

// Enqueues the scan.  tile_ws: scan_workspace_bytes(n) bytes.
template <typename F>
inline int exclusive_scan(F f, int64_t n, int64_t* out, int64_t* tile_ws, hipStream_t stream) {
  const int64_t tiles = scan_num_tiles(n);
  if (tiles == 1) {
    hipLaunchKernelGGL((scan_apply_kernel<F, false>), dim3(1), dim3(kScanThreads), 0, stream, f, n,
                       static_cast<const int64_t*>(nullptr), out);
    return check_launch("scan_apply");
  }
  {
    ProfileScope prof("scan_tile_sums", stream);
    hipLaunchKernelGGL(scan_tile_sums_kernel<F>, dim3(static_cast<unsigned>(tiles)),
                       dim3(kScanThreads), 0, stream, f, n, tile_ws, out);
  }
  if (tiles <= kScanSelfPrefixTiles) {
    ProfileScope prof("scan_apply", stream);
    hipLaunchKernelGGL((scan_apply_kernel<F, true>), dim3(static_cast<unsigned>(tiles)),
                       dim3(kScanThreads), 0, stream, f, n, static_cast<const int64_t*>(tile_ws),
                       out);
    return check_launch("scan");
  }
  hipLaunchKernelGGL(scan_tile_offsets_kernel, dim3(1), dim3(kScanThreads), 0, stream, tile_ws,
                     tiles);
  hipLaunchKernelGGL((scan_apply_kernel<F, false>), dim3(static_cast<unsigned>(tiles)),
                     dim3(kScanThreads), 0, stream, f, n, static_cast<const int64_t*>(tile_ws),
                     out);
  return check_launch("scan");
}


// ------------------------------------------- single-pass scan (look-back) ----
// Chained-scan building blocks for kernels that count, scan and write in one
// launch.  Every tile (= workgroup, in blockIdx order) owns one 64-bit status
// word {flag:2 | epoch:14 | value:48}: flag 0 = nothing yet, 1 = the tile's own
// sum, 2 = the inclusive prefix up to and including the tile.  A word whose
// epoch is not the launch's epoch counts as "nothing yet", so the array needs no
// clearing between launches: it is zero-filled once and every launch passes an
// epoch (1..16383) that no earlier launch on the same array has used since.
// Nothing in the protocol is a same-address read-modify-write: on a multi-XCD
// part those serialise memory-side, and one per workgroup costs more than the
// rest of the kernel.
//
// A tile publishes its sum, then wave 0 walks back over its predecessors, 8
// windows of 64 per round trip, until it meets an inclusive prefix.  Workgroups
// are dispatched in blockIdx order, so the lowest unfinished tile is always
// resident and never waits on anyone: the walk cannot deadlock.  The wait is
// bounded all the same: after kLookbackSpinLimit polls the tile gives up,
// raises *error (sticky until the state is zero-filled again) and carries on
// with a zero, so every wave reaches the end of the kernel.
struct LookbackState {
  unsigned long long* status;  // one per tile
  unsigned int* error;
  unsigned int epoch;
  int spin_limit;  // polls of one status word before a tile gives up (kLookbackSpinLimit)
};

constexpr int kLbValueBits = 48;
constexpr unsigned long long kLbValue = (1ull << kLbValueBits) - 1;
constexpr unsigned int kLbMaxEpoch = (1u << 14) - 1;
constexpr int kLookbackSpinLimit = 1 << 20;
constexpr int kLookbackBurst = 8;  // windows of 64 predecessors requested together

inline size_t lookback_state_bytes(int64_t tiles) { return padded((tiles > 0 ? tiles : 1) * 8) + 256; }

inline LookbackState carve_lookback(Carver& ws, int64_t tiles, unsigned int epoch) {
  LookbackState st;
  st.error = ws.take<unsigned int>(64);  // first, so that it does not move with the tile count
  st.status = ws.take<unsigned long long>(tiles > 0 ? tiles : 1);
  st.epoch = epoch;
  st.spin_limit = kLookbackSpinLimit;
  return st;
}

__device__ __forceinline__ unsigned long long lb_word(unsigned int flag, unsigned int epoch,
                                                      int64_t value) {
  return (static_cast<unsigned long long>(flag) << 62) |
         (static_cast<unsigned long long>(epoch) << kLbValueBits) |
         (static_cast<unsigned long long>(value) & kLbValue);
}
// flag of a status word as seen by a launch with this epoch (0 when it is stale)
__device__ __forceinline__ unsigned int lb_flag(unsigned long long s, unsigned int epoch) {
  return ((s >> kLbValueBits) & kLbMaxEpoch) == epoch ? static_cast<unsigned int>(s >> 62) : 0u;
}
__device__ __forceinline__ unsigned long long lb_load(const unsigned long long* p) {
  return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ void lb_store(unsigned long long* p, unsigned long long v) {
  __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// A tile gives up: the error word is raised and made visible to the whole device before
// anything the tile publishes afterwards (the one place that pays for a device-scope fence).
__device__ __forceinline__ void lookback_raise(const LookbackState& st) {
  __hip_atomic_store(st.error, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "agent");
}

// Any one thread: makes the tile's own sum visible to its successors.  Call it as
// early as possible; whatever the tile does between this and the walk below
// gives its predecessors time to publish theirs.
// may_close = false: tile 0 too publishes its sum as a sum only (for callers that close their
// tiles themselves, later, with lookback_publish_inclusive).
__device__ __forceinline__ void lookback_publish_sum(const LookbackState& st, unsigned int tile,
                                                     int64_t total, bool may_close = true) {
  lb_store(&st.status[tile], lb_word(tile == 0 && may_close ? 2u : 1u, st.epoch, total));
}

// Any one thread: closes the tile (its inclusive prefix).  Only for callers that asked
// lookback_exclusive_prefix not to do it, because something else of the tile has to be
// complete first.
__device__ __forceinline__ void lookback_publish_inclusive(const LookbackState& st,
                                                           unsigned int tile, int64_t inclusive) {
  lb_store(&st.status[tile], lb_word(2u, st.epoch, inclusive));
}

// A closed tile's inclusive prefix, for readers other than the look-back itself: waits (with
// the same bound) until `tile` is closed.  Returns 0 after giving up, with *st.error raised.
__device__ __forceinline__ int64_t lookback_wait_inclusive(const LookbackState& st,
                                                           unsigned long long seen,
                                                           unsigned int tile) {
  int polls = 0;
  while (lb_flag(seen, st.epoch) != 2u) {
    if (++polls > st.spin_limit) {
      lookback_raise(st);
      return 0;
    }
    if (polls > 16) __builtin_amdgcn_s_sleep(32);
    seen = lb_load(&st.status[tile]);
  }
  return static_cast<int64_t>(seen & kLbValue);
}

// Call with all 64 lanes of wave 0, after lookback_publish_sum.  Returns the sum
// of all earlier tiles and (unless publish is false) publishes the tile's inclusive prefix.
__device__ __forceinline__ int64_t lookback_exclusive_prefix(const LookbackState& st,
                                                             unsigned int tile, int64_t total,
                                                             bool publish = true) {
  const int lane = threadIdx.x & (kWave - 1);
  if (tile == 0) return 0;
  const unsigned long long before_first = lb_word(2u, st.epoch, 0);  // "tile -1": inclusive 0
  int64_t running = 0;
  int64_t newest = static_cast<int64_t>(tile) - 1;  // lane l reads tile newest - l (- 64 per window)
  bool closed_seen = false;
  while (!closed_seen) {
    // a burst of windows is requested at once so that their latencies overlap
    unsigned long long s[kLookbackBurst];
#pragma unroll
    for (int w = 0; w < kLookbackBurst; ++w) {
      const int64_t j = newest - w * kWave - lane;
      s[w] = j >= 0 ? lb_load(&st.status[j]) : before_first;
    }
#pragma unroll
    for (int w = 0; w < kLookbackBurst; ++w) {
      if (!closed_seen) {
        const int64_t j = newest - w * kWave - lane;
        int polls = 0;
        while (lb_flag(s[w], st.epoch) == 0) {
          if (++polls > st.spin_limit) {
            lookback_raise(st);
            s[w] = before_first;
            break;
          }
          // a poll is itself a round trip to memory; back off only when the wait is long
          if (polls > 16) __builtin_amdgcn_s_sleep(32);
          s[w] = lb_load(&st.status[j]);
        }
        const unsigned long long closed = __ballot(lb_flag(s[w], st.epoch) == 2);
        const int first = closed ? __ffsll(static_cast<long long>(closed)) - 1 : kWave;
        int64_t v = lane <= first ? static_cast<int64_t>(s[w] & kLbValue) : 0;
#pragma unroll
        for (int d = kWave / 2; d > 0; d >>= 1) v += __shfl_xor(v, d, kWave);
        running += v;
        closed_seen = closed != 0;
      }
    }
    newest -= kLookbackBurst * kWave;
  }
  // (an error raised above was stored with device scope before this point)
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
  if (publish && lane == 0) lb_store(&st.status[tile], lb_word(2u, st.epoch, running + total));
  return running;
}

// ----------------------------------------------------------- host mailbox ----
// {total, ticket} in pinned host memory, written with system scope, total first.
__device__ __forceinline__ void post_mailbox(gs_mailbox* box, int64_t total, int64_t ticket) {
  if (!box) return;
  __hip_atomic_store(&box->total, total, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
  __hip_atomic_store(&box->ticket, ticket, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_SYSTEM);
}

// gs_coo_sum with a bound on the targets: one outside [0, num_targets) is left out
// (gs_segment.hip; gs_coo_sum_binned passes the calls it does not bin on to it)
int coo_sum_bounded(const void* target, int id_bytes, const int64_t* e_ids, const float* data,
                    int64_t E, int64_t powk, int64_t num_targets, float* out, void* stream);

// The batched relabel by hash classes and LDS tables (gs_binrelabel.hip): same outputs as
// the one on hash regions (gs_unique.hip), no memory-side atomic per item.  Ids must fit 32
// bits (id_bytes 8: the 64-bit ids are read and written as such).  *num_unique = -4 when a
// class held more distinct ids than its table: the call has to be repeated on hash regions.
size_t binned_relabel_workspace_bytes(int64_t M, int64_t B);
bool binned_relabel_applies(int64_t M, int64_t B);
int batch_relabel_binned(const void* seeds, const int64_t* seeds_ptr, const void* ids,
                         const int64_t* ids_ptr, int64_t B, int64_t num_seeds, int64_t num_ids,
                         int id_bytes, void* unique, int64_t* unique_ptr, void* out_ids,
                         int64_t* num_unique, void* workspace, size_t workspace_bytes,
                         gs_mailbox* box, int64_t box_ticket, hipStream_t stream);

}  // namespace gs
