// Generalised SDDMM on gfx950: out[eid, k] = op(lhs[sel_l, .], rhs[sel_r, .]).
//
// Replaces impl::SDDMMCOO / impl::SDDMMCSC (reference src/cuda/sddmm.cu:280,263;
// operators src/cuda/functor.h:11-136; target selection src/cuda/selector.h).
//
// None of this is a dense contraction: every edge gathers two feature rows at
// random, so the kernels are HBM/latency bound and use no MFMA.
//  * dot without broadcast (the layer-wise samplers' u_dot_v): a group of
//    16 lanes per edge reads both rows as float4 (one 256 B row of a 64-wide
//    feature = one fully coalesced request), multiplies, and reduces with a
//    4-step butterfly; 4 edges per wave.
//  * everything else: the reference's 2-D edge x feature decomposition
//    (sddmm.cu:197-209) with the operator and targets as template parameters.
//  * CSC flavour: the owning column of an edge comes from a binary search over
//    the offsets, done once per edge (the reference does it per edge too,
//    sddmm.cu:126-131).
#include "gs_common.hpp"

namespace gs {
namespace {

constexpr int kThreads = 256;

template <int OP>
__device__ __forceinline__ float apply_op(const float* l, const float* r, int64_t R) {
  if (OP == GS_OP_ADD) return l[0] + r[0];
  if (OP == GS_OP_SUB) return l[0] - r[0];
  if (OP == GS_OP_MUL) return l[0] * r[0];
  if (OP == GS_OP_DIV) return l[0] / r[0];
  if (OP == GS_OP_COPY_LHS) return l[0];
  if (OP == GS_OP_COPY_RHS) return r[0];
  float acc = 0.0f;  // functor.h:125-131
  for (int64_t i = 0; i < R; ++i) acc += l[i] * r[i];
  return acc;
}

__device__ __forceinline__ int64_t select3(int target, int64_t src, int64_t eid, int64_t dst) {
  return target == 0 ? src : (target == 1 ? eid : dst);
}

template <typename IdT>
struct SddmmArgs {
  const float* lhs;
  const float* rhs;
  float* out;
  const IdT* row;          // COO: row ids; CSC: indices
  const IdT* col;          // COO: col ids; CSC: nullptr
  const int64_t* indptr;   // CSC only
  const IdT* nid_map;      // CSC only, optional
  const int64_t* e_ids;    // optional
  int64_t num_cols;        // CSC only
  int64_t E;
  int64_t lhs_len, rhs_len, out_len, R;
  const int64_t* lhs_off;
  const int64_t* rhs_off;
  int lhs_target, rhs_target;
};

// last column c in [lo, hi] with indptr[c] <= e (the reference searches all columns for
// every edge, sddmm.cu:130; here a workgroup first narrows the range to the columns its
// own edges span, so the per-edge search is a few steps over offsets already in cache)
__device__ __forceinline__ int64_t column_of(const int64_t* __restrict__ indptr, int64_t lo,
                                             int64_t hi, int64_t e) {
  while (lo < hi) {
    const int64_t mid = (lo + hi + 1) >> 1;
    if (indptr[mid] <= e) lo = mid; else hi = mid - 1;
  }
  return lo;
}

// The same over all columns by a whole wave: 64 probes per round trip, so 2.45 M columns take
// 4 dependent reads instead of 21.
__device__ __forceinline__ int64_t wave_column_of(const int64_t* __restrict__ indptr,
                                                  int64_t num_cols, int64_t e, int lane) {
  int64_t lo = 0, hi = num_cols - 1;
  while (lo < hi) {
    const int64_t step = (hi - lo + kWave - 1) / kWave;
    const int64_t pos = lo + (lane + 1) * step;
    const bool ok = pos <= hi && indptr[pos] <= e;
    const int k = __popcll(__ballot(ok));  // the probes are ordered: ok is a run of leading lanes
    lo += k * step;
    hi = lo + step - 1 < hi ? lo + step - 1 : hi;
  }
  return lo;
}

// CSC only: columns of the workgroup's first and last edge into s_range[0..1], found by its
// first two waves; every thread of the (256-thread) workgroup must call it
constexpr int kStageCols = 1024;  // offsets of that many columns are kept in LDS

template <typename IdT>
__device__ __forceinline__ void block_column_range(const SddmmArgs<IdT>& a, int64_t e0, int64_t e1,
                                                   int64_t* s_range, int64_t* s_ptr) {
  if (!a.indptr) return;
  const int t = threadIdx.y * blockDim.x + threadIdx.x;
  const int wave = t / kWave;
  if (wave < 2) {
    const int64_t e = wave == 0 ? e0 : (e1 < a.E ? e1 : a.E - 1);
    const int64_t c = a.num_cols > 0 ? wave_column_of(a.indptr, a.num_cols, e, t % kWave) : 0;
    if (t % kWave == 0) s_range[wave] = c;
  }
  __syncthreads();
  const int64_t n = s_range[1] - s_range[0] + 1;
  if (n <= kStageCols) {
    for (int64_t i = t; i < n; i += kThreads) s_ptr[i] = a.indptr[s_range[0] + i];
    __syncthreads();
  }
}

// need_src / need_dst: whether an operand is taken at that end of the edge; an end nobody
// asks for is not looked up (the row ids of a CSC are a third of the bytes of a scalar
// operator over its edges)
template <typename IdT>
__device__ __forceinline__ void edge_endpoints(const SddmmArgs<IdT>& a, int64_t e,
                                               const int64_t* s_range, const int64_t* s_ptr,
                                               bool need_src, bool need_dst, int64_t* src,
                                               int64_t* dst, int64_t* eid) {
  *src = need_src ? static_cast<int64_t>(a.row[e]) : 0;
  *eid = a.e_ids ? a.e_ids[e] : e;
  if (!need_dst) {
    *dst = 0;
    return;
  }
  if (a.indptr) {
    const int64_t n = s_range[1] - s_range[0] + 1;
    const int64_t c = n <= kStageCols ? s_range[0] + column_of(s_ptr, 0, n - 1, e)
                                      : column_of(a.indptr, s_range[0], s_range[1], e);
    *dst = a.nid_map ? static_cast<int64_t>(a.nid_map[c]) : c;
  } else {
    *dst = static_cast<int64_t>(a.col[e]);
  }
}

// blockDim = (tx, 256/tx): tx walks the out_len positions of an edge, every thread row takes
// kEdgesPerRow edges (strided by the rows, so that a wave's accesses stay consecutive)
constexpr int kEdgesPerRow = 8;
template <int OP, typename IdT>
__global__ void __launch_bounds__(kThreads) sddmm_generic_kernel(SddmmArgs<IdT> a) {
  __shared__ int64_t s_range[2];
  __shared__ int64_t s_ptr[kStageCols];
  const int64_t per_block = static_cast<int64_t>(blockDim.y) * kEdgesPerRow;
  const int64_t e0 = static_cast<int64_t>(blockIdx.x) * per_block;
  const bool need_src = (OP != GS_OP_COPY_RHS && a.lhs_target == 0) ||
                        (OP != GS_OP_COPY_LHS && a.rhs_target == 0);
  const bool need_dst = (OP != GS_OP_COPY_RHS && a.lhs_target == 2) ||
                        (OP != GS_OP_COPY_LHS && a.rhs_target == 2);
  if (need_dst) block_column_range(a, e0, e0 + per_block - 1, s_range, s_ptr);
  // the ends of all eight edges first, so that their reads are in flight together
  int64_t src[kEdgesPerRow], dst[kEdgesPerRow], eid[kEdgesPerRow];
#pragma unroll
  for (int j = 0; j < kEdgesPerRow; ++j) {
    const int64_t e = e0 + static_cast<int64_t>(j) * blockDim.y + threadIdx.y;
    src[j] = dst[j] = 0;
    eid[j] = -1;
    if (e < a.E) edge_endpoints(a, e, s_range, s_ptr, need_src, need_dst, &src[j], &dst[j], &eid[j]);
  }
#pragma unroll
  for (int j = 0; j < kEdgesPerRow; ++j) {
    if (eid[j] < 0) continue;
    const float* l = (OP == GS_OP_COPY_RHS)
                         ? nullptr
                         : a.lhs + select3(a.lhs_target, src[j], eid[j], dst[j]) * a.lhs_len;
    const float* r = (OP == GS_OP_COPY_LHS)
                         ? nullptr
                         : a.rhs + select3(a.rhs_target, src[j], eid[j], dst[j]) * a.rhs_len;
    float* o = a.out + eid[j] * a.out_len;
    for (int64_t k = threadIdx.x; k < a.out_len; k += blockDim.x) {
      const int64_t la = a.lhs_off ? a.lhs_off[k] : k;
      const int64_t ra = a.rhs_off ? a.rhs_off[k] : k;
      o[k] = apply_op<OP>(l + la * a.R, r + ra * a.R, a.R);
    }
  }
}

// Scalar operands on a CSC (weight / per-column sum, weight * per-row factor ...): one value
// per edge in, one out.  The column of an edge is found as in the CSC -> COO expansion: a
// workgroup owns 4096 consecutive edges, the columns that start among them mark their first
// edge in LDS and a running maximum over the marks gives every edge its column -- no search
// per edge.  Then a pass with consecutive lanes on consecutive edges does the arithmetic.
constexpr int kScalarItems = 16;
constexpr int kScalarTile = kThreads * kScalarItems;

template <int OP, typename IdT>
__global__ void __launch_bounds__(kThreads) sddmm_scalar_csc_kernel(SddmmArgs<IdT> a) {
  __shared__ int s_mark[kScalarTile];
  __shared__ int64_t s_rows[2];
  __shared__ int s_wave[kThreads / kWave];
  const int64_t p0 = static_cast<int64_t>(blockIdx.x) * kScalarTile;
  const int64_t p1 = p0 + kScalarTile < a.E ? p0 + kScalarTile : a.E;
  for (int i = threadIdx.x; i < kScalarTile; i += kThreads) s_mark[i] = 0;
  block_row_range(a.indptr, a.num_cols, p0, p1 - 1, s_rows);
  const int64_t row_lo = s_rows[0], row_hi = s_rows[1];
  // columns row_lo + 1 .. row_hi start inside the tile (row_lo holds its first edge); of
  // several empty columns at one position the highest wins, which is the owner
  for (int64_t r = row_lo + 1 + threadIdx.x; r <= row_hi; r += kThreads)
    atomicMax(&s_mark[a.indptr[r] - p0], static_cast<int>(r - row_lo));
  __syncthreads();
  const int at0 = threadIdx.x * kScalarItems;
  int m[kScalarItems];
  int run = 0;
#pragma unroll
  for (int k = 0; k < kScalarItems; ++k) {
    const int v = s_mark[at0 + k];
    run = v > run ? v : run;
    m[k] = run;
  }
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
  __syncthreads();
#pragma unroll
  for (int k = 0; k < kScalarItems; ++k) s_mark[at0 + k] = m[k] > before ? m[k] : before;
  __syncthreads();
  const bool need_src = (OP != GS_OP_COPY_RHS && a.lhs_target == 0) ||
                        (OP != GS_OP_COPY_LHS && a.rhs_target == 0);
  // In three sweeps over the thread's sixteen edges -- where the operands are, the operands,
  // the results -- so that the reads of one edge do not wait for the store of the one before
  // (the output may overlap an operand: a read cannot be moved ahead of a store by itself).
  // The optional id maps are read without a branch (a branch before a read makes the read
  // wait for all before it): an absent map is read at a stride of zero from the offsets,
  // which are always there, and the value is then not used.
  const IdT* nid_from = a.nid_map ? a.nid_map : reinterpret_cast<const IdT*>(a.indptr);
  const int64_t* eid_from = a.e_ids ? a.e_ids : a.indptr;
  const IdT* src_from = need_src ? a.row : reinterpret_cast<const IdT*>(a.indptr);
  const int64_t nid_step = a.nid_map ? 1 : 0, eid_step = a.e_ids ? 1 : 0, src_step = need_src ? 1 : 0;
  constexpr int kHalf = kScalarItems / 2;  // (eight edges at a time keep the registers few)
#pragma unroll 1
  for (int k0 = 0; k0 < kScalarItems; k0 += kHalf) {
    int64_t at_l[kHalf], at_r[kHalf], at_o[kHalf];
    IdT nid_v[kHalf], src_v[kHalf];
#pragma unroll
    for (int k = 0; k < kHalf; ++k) {
      const int i = (k0 + k) * kThreads + threadIdx.x;
      const int64_t e = p0 + i < p1 ? p0 + i : p1 - 1;  // (past the end: the last edge again)
      at_l[k] = row_lo + s_mark[e - p0];
      nid_v[k] = nid_from[at_l[k] * nid_step];
      src_v[k] = src_from[e * src_step];
      at_o[k] = eid_from[e * eid_step];
    }
#pragma unroll
    for (int k = 0; k < kHalf; ++k) {
      const int i = (k0 + k) * kThreads + threadIdx.x;
      const int64_t e = p0 + i < p1 ? p0 + i : p1 - 1;
      const int64_t dst = a.nid_map ? static_cast<int64_t>(nid_v[k]) : at_l[k];
      const int64_t src = static_cast<int64_t>(src_v[k]);
      const int64_t eid = a.e_ids ? at_o[k] : e;
      at_l[k] = select3(a.lhs_target, src, eid, dst);
      at_r[k] = select3(a.rhs_target, src, eid, dst);
      at_o[k] = eid;
    }
    float lv[kHalf], rv[kHalf];
#pragma unroll
    for (int k = 0; k < kHalf; ++k) {
      lv[k] = (OP == GS_OP_COPY_RHS) ? 0.0f : a.lhs[at_l[k]];
      rv[k] = (OP == GS_OP_COPY_LHS) ? 0.0f : a.rhs[at_r[k]];
    }
#pragma unroll
    for (int k = 0; k < kHalf; ++k)
      if (p0 + (k0 + k) * kThreads + threadIdx.x < p1)
        a.out[at_o[k]] = apply_op<OP>(&lv[k], &rv[k], 1);
  }
}

template <int OP, typename IdT>
void launch_scalar_csc(const SddmmArgs<IdT>& a, hipStream_t st) {
  const unsigned grid = static_cast<unsigned>((a.E + kScalarTile - 1) / kScalarTile);
  hipLaunchKernelGGL((sddmm_scalar_csc_kernel<OP, IdT>), dim3(grid), dim3(kThreads), 0, st, a);
}

// Scalar operands where no column has to be found (a COO, or a CSC whose operands sit on the
// edge and on its row): eight edges per thread, strided by the workgroup, in three sweeps --
// the ends and the edge id, the operands, the results -- so that all reads of a sweep are in
// flight together and no read stands behind a store (the general kernel walks an edge at a
// time; one scalar per row over 124 M edges: 0.89 ms there).
constexpr int kFlatItems = 8;
constexpr int kFlatTile = kThreads * kFlatItems;

template <int OP, typename IdT>
__global__ void __launch_bounds__(kThreads) sddmm_scalar_flat_kernel(SddmmArgs<IdT> a) {
  const int64_t base = static_cast<int64_t>(blockIdx.x) * kFlatTile + threadIdx.x;
  const bool need_src = (OP != GS_OP_COPY_RHS && a.lhs_target == 0) ||
                        (OP != GS_OP_COPY_LHS && a.rhs_target == 0);
  const bool need_dst = (OP != GS_OP_COPY_RHS && a.lhs_target == 2) ||
                        (OP != GS_OP_COPY_LHS && a.rhs_target == 2);
  // an end nobody asks for is read at a stride of zero (the row ids are always there)
  const IdT* dst_from = need_dst ? a.col : a.row;
  const int64_t src_step = need_src ? 1 : 0, dst_step = need_dst ? 1 : 0;
  int64_t e[kFlatItems], eid[kFlatItems];
  IdT src[kFlatItems], dst[kFlatItems];
#pragma unroll
  for (int k = 0; k < kFlatItems; ++k) {
    e[k] = base + static_cast<int64_t>(k) * kThreads;
    if (e[k] >= a.E) e[k] = a.E - 1;  // (past the end: the last edge again, not stored)
    src[k] = a.row[e[k] * src_step];
    dst[k] = dst_from[e[k] * dst_step];
    eid[k] = e[k];
  }
  if (a.e_ids) {
#pragma unroll
    for (int k = 0; k < kFlatItems; ++k) eid[k] = a.e_ids[e[k]];
  }
  float lv[kFlatItems], rv[kFlatItems];
#pragma unroll
  for (int k = 0; k < kFlatItems; ++k) {
    const int64_t s = static_cast<int64_t>(src[k]), d = static_cast<int64_t>(dst[k]);
    lv[k] = (OP == GS_OP_COPY_RHS) ? 0.0f : a.lhs[select3(a.lhs_target, s, eid[k], d)];
    rv[k] = (OP == GS_OP_COPY_LHS) ? 0.0f : a.rhs[select3(a.rhs_target, s, eid[k], d)];
  }
#pragma unroll
  for (int k = 0; k < kFlatItems; ++k)
    if (base + static_cast<int64_t>(k) * kThreads < a.E) a.out[eid[k]] = apply_op<OP>(&lv[k], &rv[k], 1);
}

template <int OP, typename IdT>
void launch_scalar_flat(const SddmmArgs<IdT>& a, hipStream_t st) {
  const unsigned grid = static_cast<unsigned>((a.E + kFlatTile - 1) / kFlatTile);
  hipLaunchKernelGGL((sddmm_scalar_flat_kernel<OP, IdT>), dim3(grid), dim3(kThreads), 0, st, a);
}

// dot, no broadcast, out_len == 1, R % 4 == 0 and 16-byte aligned rows.
constexpr int kDotGroup = 16;
constexpr int kDotEdges = 4;  // edges per 16-lane group
template <typename IdT>
__global__ void __launch_bounds__(kThreads) sddmm_dot_rows_kernel(SddmmArgs<IdT> a) {
  __shared__ int64_t s_range[2];
  __shared__ int64_t s_ptr[kStageCols];
  const int lane = threadIdx.x % kDotGroup;
  constexpr int kGroups = kThreads / kDotGroup;
  const int64_t e0 = static_cast<int64_t>(blockIdx.x) * (kGroups * kDotEdges);
  block_column_range(a, e0, e0 + kGroups * kDotEdges - 1, s_range, s_ptr);
  for (int j = 0; j < kDotEdges; ++j) {
    const int64_t e = e0 + j * kGroups + threadIdx.x / kDotGroup;
    if (e >= a.E) return;
    int64_t src, dst, eid;
    edge_endpoints(a, e, s_range, s_ptr, true, true, &src, &dst, &eid);
    const float4* l =
        reinterpret_cast<const float4*>(a.lhs + select3(a.lhs_target, src, eid, dst) * a.lhs_len);
    const float4* r =
        reinterpret_cast<const float4*>(a.rhs + select3(a.rhs_target, src, eid, dst) * a.rhs_len);
    float acc = 0.0f;
    for (int64_t i = lane; i < a.R / 4; i += kDotGroup) {
      const float4 x = l[i];
      const float4 y = r[i];
      acc += x.x * y.x + x.y * y.y + x.z * y.z + x.w * y.w;
    }
#pragma unroll
    for (int d = kDotGroup / 2; d > 0; d >>= 1) acc += __shfl_xor(acc, d, kDotGroup);
    if (lane == 0) a.out[eid] = acc;
  }
}

template <int OP, typename IdT>
void launch_generic(const SddmmArgs<IdT>& a, hipStream_t st) {
  int tx = 1;
  while (tx < a.out_len && tx < kThreads) tx <<= 1;
  const int ty = kThreads / tx;
  const int64_t per_block = static_cast<int64_t>(ty) * kEdgesPerRow;
  const unsigned grid = static_cast<unsigned>((a.E + per_block - 1) / per_block);
  hipLaunchKernelGGL((sddmm_generic_kernel<OP, IdT>), dim3(grid), dim3(tx, ty), 0, st, a);
}

template <typename IdT>
int sddmm_dispatch(int op, const SddmmArgs<IdT>& a, hipStream_t st) {
  if (a.E == 0 || a.out_len == 0) return GS_OK;
  const bool aligned = (reinterpret_cast<uintptr_t>(a.lhs) % 16 == 0) &&
                       (reinterpret_cast<uintptr_t>(a.rhs) % 16 == 0) && a.lhs_len % 4 == 0 &&
                       a.rhs_len % 4 == 0;
  if (op == GS_OP_DOT && !a.lhs_off && !a.rhs_off && a.out_len == 1 && a.R % 4 == 0 && a.R >= 16 &&
      aligned) {
    const int64_t per_block = static_cast<int64_t>(kThreads / kDotGroup) * kDotEdges;
    const unsigned grid = static_cast<unsigned>((a.E + per_block - 1) / per_block);
    ProfileScope prof("sddmm_dot", st);
    hipLaunchKernelGGL(sddmm_dot_rows_kernel<IdT>, dim3(grid), dim3(kThreads), 0, st, a);
    return check_launch("sddmm_dot");
  }
  const bool to_dst = a.lhs_target == 2 || a.rhs_target == 2;
  if (a.indptr && to_dst && a.out_len == 1 && a.R == 1 && a.lhs_len == 1 && a.rhs_len == 1 &&
      !a.lhs_off && !a.rhs_off && a.num_cols < (int64_t(1) << 31)) {
    switch (op) {
      case GS_OP_ADD: launch_scalar_csc<GS_OP_ADD, IdT>(a, st); return check_launch("sddmm");
      case GS_OP_SUB: launch_scalar_csc<GS_OP_SUB, IdT>(a, st); return check_launch("sddmm");
      case GS_OP_MUL: launch_scalar_csc<GS_OP_MUL, IdT>(a, st); return check_launch("sddmm");
      case GS_OP_DIV: launch_scalar_csc<GS_OP_DIV, IdT>(a, st); return check_launch("sddmm");
      default: break;  // the copies and a one-element dot go the general way
    }
  }
  if ((!a.indptr || !to_dst) && a.row && (a.indptr || a.col) && a.out_len == 1 && a.R == 1 &&
      a.lhs_len == 1 && a.rhs_len == 1 && !a.lhs_off && !a.rhs_off) {
    switch (op) {
      case GS_OP_ADD: launch_scalar_flat<GS_OP_ADD, IdT>(a, st); return check_launch("sddmm");
      case GS_OP_SUB: launch_scalar_flat<GS_OP_SUB, IdT>(a, st); return check_launch("sddmm");
      case GS_OP_MUL: launch_scalar_flat<GS_OP_MUL, IdT>(a, st); return check_launch("sddmm");
      case GS_OP_DIV: launch_scalar_flat<GS_OP_DIV, IdT>(a, st); return check_launch("sddmm");
      default: break;  // the copies and a one-element dot go the general way
    }
  }
  switch (op) {
    case GS_OP_ADD: launch_generic<GS_OP_ADD, IdT>(a, st); break;
    case GS_OP_SUB: launch_generic<GS_OP_SUB, IdT>(a, st); break;
    case GS_OP_MUL: launch_generic<GS_OP_MUL, IdT>(a, st); break;
    case GS_OP_DIV: launch_generic<GS_OP_DIV, IdT>(a, st); break;
    case GS_OP_COPY_LHS: launch_generic<GS_OP_COPY_LHS, IdT>(a, st); break;
    case GS_OP_COPY_RHS: launch_generic<GS_OP_COPY_RHS, IdT>(a, st); break;
    case GS_OP_DOT: launch_generic<GS_OP_DOT, IdT>(a, st); break;
    default:
      set_error_text("Unsupported SpMM/SDDMM binary operator: %d", op);  // macro.h:30
      return GS_ERR_UNSUPPORTED;
  }
  return check_launch("sddmm");
}

int check_common(const char* who, int op, int64_t E, const float* lhs, const float* rhs, float* out,
                 int lhs_target, int rhs_target, int64_t lhs_len, int64_t rhs_len, int64_t out_len,
                 int64_t R) {
  GS_REQUIRE(E >= 0 && lhs_len >= 0 && rhs_len >= 0 && out_len >= 0 && R >= 1,
             "%s: negative size", who);
  GS_REQUIRE(lhs_target >= 0 && lhs_target <= 2 && rhs_target >= 0 && rhs_target <= 2,
             "%s: targets must be 0 (src), 1 (edge) or 2 (dst)", who);
  GS_REQUIRE(E == 0 || out, "%s: out is null", who);
  GS_REQUIRE(E == 0 || op == GS_OP_COPY_RHS || lhs, "%s: lhs is null", who);
  GS_REQUIRE(E == 0 || op == GS_OP_COPY_LHS || rhs, "%s: rhs is null", who);
  return GS_OK;
}

}  // namespace
}  // namespace gs

using namespace gs;

extern "C" {

int gs_sddmm_coo(int op, const void* row, const void* col, int id_bytes, const int64_t* e_ids,
                 int64_t E, const float* lhs, const float* rhs, float* out, int lhs_target,
                 int rhs_target, int64_t lhs_len, int64_t rhs_len, int64_t out_len,
                 int64_t reduce_size, const int64_t* lhs_off, const int64_t* rhs_off, void* stream) {
  GS_RETURN_IF_ERROR(check_common("gs_sddmm_coo", op, E, lhs, rhs, out, lhs_target, rhs_target,
                                  lhs_len, rhs_len, out_len, reduce_size));
  GS_REQUIRE(E == 0 || (row && col), "gs_sddmm_coo: null row/col");
  GS_REQUIRE(valid_id_bytes(id_bytes), "gs_sddmm_coo: id_bytes must be 4 or 8, got %d", id_bytes);
  hipStream_t st = static_cast<hipStream_t>(stream);
  if (id_bytes == 8) {
    SddmmArgs<int64_t> a{lhs, rhs, out, static_cast<const int64_t*>(row),
                         static_cast<const int64_t*>(col), nullptr, nullptr, e_ids, 0, E, lhs_len,
                         rhs_len, out_len, reduce_size, lhs_off, rhs_off, lhs_target, rhs_target};
    return sddmm_dispatch(op, a, st);
  }
  SddmmArgs<int32_t> a{lhs, rhs, out, static_cast<const int32_t*>(row),
                       static_cast<const int32_t*>(col), nullptr, nullptr, e_ids, 0, E, lhs_len,
                       rhs_len, out_len, reduce_size, lhs_off, rhs_off, lhs_target, rhs_target};
  return sddmm_dispatch(op, a, st);
}

int gs_sddmm_csc(int op, const int64_t* indptr, const void* indices, int id_bytes,
                 const int64_t* e_ids, const void* nid_map, int64_t num_cols, int64_t E,
                 const float* lhs, const float* rhs, float* out, int lhs_target, int rhs_target,
                 int64_t lhs_len, int64_t rhs_len, int64_t out_len, int64_t reduce_size,
                 const int64_t* lhs_off, const int64_t* rhs_off, void* stream) {
  GS_RETURN_IF_ERROR(check_common("gs_sddmm_csc", op, E, lhs, rhs, out, lhs_target, rhs_target,
                                  lhs_len, rhs_len, out_len, reduce_size));
  GS_REQUIRE(num_cols >= 0 && (E == 0 || (indptr && indices)), "gs_sddmm_csc: null indptr/indices");
  GS_REQUIRE(valid_id_bytes(id_bytes), "gs_sddmm_csc: id_bytes must be 4 or 8, got %d", id_bytes);
  hipStream_t st = static_cast<hipStream_t>(stream);
  if (id_bytes == 8) {
    SddmmArgs<int64_t> a{lhs, rhs, out, static_cast<const int64_t*>(indices), nullptr, indptr,
                         static_cast<const int64_t*>(nid_map), e_ids, num_cols, E, lhs_len, rhs_len,
                         out_len, reduce_size, lhs_off, rhs_off, lhs_target, rhs_target};
    return sddmm_dispatch(op, a, st);
  }
  SddmmArgs<int32_t> a{lhs, rhs, out, static_cast<const int32_t*>(indices), nullptr, indptr,
                       static_cast<const int32_t*>(nid_map), e_ids, num_cols, E, lhs_len, rhs_len,
                       out_len, reduce_size, lhs_off, rhs_off, lhs_target, rhs_target};
  return sddmm_dispatch(op, a, st);
}

}  // extern "C"
