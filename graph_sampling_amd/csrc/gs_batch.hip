// Super-batch plumbing on gfx950: the element-wise and gather/scatter helpers the
// reference uses to run many minibatches as one (examples/fastgcn/batching.py,
// examples/graphsage/batching.py).
//
//   encode / decode / offsets   src/cuda/batch_coding.cu:74-120
//   concat                      src/cuda/batch_concat.cu:13-119
//   split                       src/cuda/batch_split2.cu:12-100
//
// A "batched" array is one flat array plus int64 offsets [B+1] cutting it into B
// batches.  Everything here is one pass over the items, 2048 per workgroup: the items
// are read first, then the workgroup finds the batches of its first and last item
// once and its lanes search in between (the reads do not wait for the searches).
#include "gs_common.hpp"

namespace gs {
namespace {

constexpr int kThreads = 256;
constexpr int kItems = 8;
constexpr int kTile = kThreads * kItems;

// last b in [lo, hi] with ptr[b] <= i
__device__ __forceinline__ int64_t batch_of(const int64_t* __restrict__ ptr, int64_t i, int64_t lo,
                                            int64_t hi) {
  while (lo < hi) {
    const int64_t mid = (lo + hi + 1) >> 1;
    if (ptr[mid] <= i) lo = mid; else hi = mid - 1;
  }
  return lo;
}

// batch range of the items [first, last] of a workgroup, through LDS
__device__ __forceinline__ void block_batches(const int64_t* __restrict__ ptr, int64_t B,
                                              int64_t first, int64_t last, int64_t* lds2,
                                              int64_t* lo, int64_t* hi) {
  if (threadIdx.x < 2) lds2[threadIdx.x] = batch_of(ptr, threadIdx.x == 0 ? first : last, 0, B - 1);
  __syncthreads();
  *lo = lds2[0];
  *hi = lds2[1];
}

template <typename IdT>
__global__ void __launch_bounds__(kThreads)
encode_kernel(const IdT* __restrict__ data, int64_t n, const int64_t* __restrict__ ptr, int64_t B,
              int64_t enc, IdT* __restrict__ out) {
  __shared__ int64_t s_range[2];
  const int64_t first = static_cast<int64_t>(blockIdx.x) * kTile;
  const int64_t last = first + kTile - 1 < n ? first + kTile - 1 : n - 1;
  IdT v[kItems];
#pragma unroll
  for (int k = 0; k < kItems; ++k) {
    const int64_t i = first + k * kThreads + threadIdx.x;
    v[k] = i < n ? data[i] : IdT(0);
  }
  int64_t lo, hi;
  block_batches(ptr, B, first, last, s_range, &lo, &hi);
#pragma unroll
  for (int k = 0; k < kItems; ++k) {
    const int64_t i = first + k * kThreads + threadIdx.x;
    if (i < n) out[i] = static_cast<IdT>(static_cast<int64_t>(v[k]) + batch_of(ptr, i, lo, hi) * enc);
  }
}

template <typename IdT>
__global__ void __launch_bounds__(kThreads)
decode_kernel(const IdT* __restrict__ in, int64_t n, int64_t enc, IdT* __restrict__ out,
              IdT* __restrict__ batch) {
  const int64_t i = static_cast<int64_t>(blockIdx.x) * kThreads + threadIdx.x;
  if (i >= n) return;
  const int64_t v = static_cast<int64_t>(in[i]);
  const int64_t b = v / enc;
  if (out) out[i] = static_cast<IdT>(v - b * enc);
  if (batch) batch[i] = static_cast<IdT>(b);
}

// out_ptr[b + 1] = number of items whose batch (in[i] / enc) is <= b; `in` is sorted
// by batch (batch_coding.cu:113-119: upper bound over the decoded batch numbers)
template <typename IdT>
__global__ void __launch_bounds__(kThreads)
offsets_kernel(const IdT* __restrict__ in, int64_t n, int64_t enc, int64_t B,
               int64_t* __restrict__ out_ptr) {
  const int64_t b = static_cast<int64_t>(blockIdx.x) * kThreads + threadIdx.x;
  if (b == 0) out_ptr[0] = 0;
  if (b >= B) return;
  int64_t lo = 0, hi = n;
  while (lo < hi) {
    const int64_t mid = (lo + hi) >> 1;
    if (static_cast<int64_t>(in[mid]) / enc <= b) lo = mid + 1; else hi = mid;
  }
  out_ptr[b + 1] = lo;
}

struct Segments {
  const void* data[GS_MAX_SEGMENTS];
  const int64_t* ptr[GS_MAX_SEGMENTS];
  int n;
};

__global__ void __launch_bounds__(kThreads)
concat_offsets_kernel(Segments seg, int64_t B, int64_t* __restrict__ out_ptr) {
  const int64_t b = static_cast<int64_t>(blockIdx.x) * kThreads + threadIdx.x;
  if (b > B) return;
  int64_t sum = 0;
  for (int s = 0; s < seg.n; ++s) sum += seg.ptr[s][b];
  out_ptr[b] = sum;
}

// blockIdx.y = segment; item i of segment s, in batch b, goes to
// out_ptr[b] + (items of batch b in the segments before s) + (i - ptr_s[b])
template <typename IdT>
__global__ void __launch_bounds__(kThreads)
concat_fill_kernel(Segments seg, int64_t B, const int64_t* __restrict__ out_ptr,
                   IdT* __restrict__ out, IdT* __restrict__ key) {
  __shared__ int64_t s_range[2];
  const int s = blockIdx.y;
  const int64_t* ptr = seg.ptr[s];
  const int64_t n = ptr[B];
  const int64_t first = static_cast<int64_t>(blockIdx.x) * kTile;
  if (first >= n) return;
  const int64_t last = first + kTile - 1 < n ? first + kTile - 1 : n - 1;
  const IdT* in = static_cast<const IdT*>(seg.data[s]);
  IdT v[kItems];
#pragma unroll
  for (int k = 0; k < kItems; ++k) {
    const int64_t i = first + k * kThreads + threadIdx.x;
    v[k] = i < n ? in[i] : IdT(0);
  }
  int64_t lo, hi;
  block_batches(ptr, B, first, last, s_range, &lo, &hi);
#pragma unroll
  for (int k = 0; k < kItems; ++k) {
    const int64_t i = first + k * kThreads + threadIdx.x;
    if (i >= n) continue;
    const int64_t b = batch_of(ptr, i, lo, hi);
    int64_t before = 0;
    for (int t = 0; t < s; ++t) before += seg.ptr[t][b + 1] - seg.ptr[t][b];
    const int64_t w = out_ptr[b] + before + (i - ptr[b]);
    out[w] = v[k];
    if (key) key[w] = static_cast<IdT>(b);
  }
}

struct OutSegments {
  void* data[GS_MAX_SEGMENTS];
  const int64_t* ptr[GS_MAX_SEGMENTS];
  int n;
};

// the inverse: item `index` of batch b = key[index] (or found from data_ptr) goes back to
// the segment that holds its local position
template <typename IdT>
__global__ void __launch_bounds__(kThreads)
split_kernel(const IdT* __restrict__ data, const int64_t* __restrict__ data_ptr,
             const IdT* __restrict__ key, int64_t n, int64_t B, OutSegments seg) {
  __shared__ int64_t s_range[2];
  const int64_t first = static_cast<int64_t>(blockIdx.x) * kTile;
  const int64_t last = first + kTile - 1 < n ? first + kTile - 1 : n - 1;
  IdT v[kItems], kb[kItems];
#pragma unroll
  for (int k = 0; k < kItems; ++k) {
    const int64_t i = first + k * kThreads + threadIdx.x;
    v[k] = i < n ? data[i] : IdT(0);
    kb[k] = (key && i < n) ? key[i] : IdT(0);
  }
  int64_t lo = 0, hi = 0;
  if (!key) block_batches(data_ptr, B, first, last, s_range, &lo, &hi);
#pragma unroll
  for (int k = 0; k < kItems; ++k) {
    const int64_t i = first + k * kThreads + threadIdx.x;
    if (i >= n) continue;
    const int64_t b = key ? static_cast<int64_t>(kb[k]) : batch_of(data_ptr, i, lo, hi);
    if (b < 0 || b >= B) continue;
    int64_t local = i - data_ptr[b];
    for (int s = 0; s < seg.n; ++s) {
      const int64_t len = seg.ptr[s][b + 1] - seg.ptr[s][b];
      if (local < len) {
        static_cast<IdT*>(seg.data[s])[seg.ptr[s][b] + local] = v[k];
        break;
      }
      local -= len;
    }
  }
}

bool fits_id(int64_t B, int64_t enc, int id_bytes) {
  if (id_bytes == 8) return true;
  // the largest encoded value is below B * enc
  return enc > 0 && B <= (int64_t(1) << 31) / enc;
}

}  // namespace
}  // namespace gs

using namespace gs;

extern "C" {

int gs_batch_encode(const void* data, int id_bytes, int64_t n, const int64_t* ptr,
                    int64_t num_batches, int64_t encoding_size, void* out, void* stream) {
  GS_REQUIRE(n >= 0 && num_batches >= 1 && encoding_size > 0,
             "gs_batch_encode: sizes must be non-negative, with at least one batch");
  GS_REQUIRE(valid_id_bytes(id_bytes), "gs_batch_encode: id_bytes must be 4 or 8, got %d", id_bytes);
  GS_REQUIRE(fits_id(num_batches, encoding_size, id_bytes),
             "gs_batch_encode: %lld batches of encoding size %lld do not fit 32-bit ids",
             static_cast<long long>(num_batches), static_cast<long long>(encoding_size));
  if (n == 0) return GS_OK;
  GS_REQUIRE(data && ptr && out, "gs_batch_encode: null pointer");
  hipStream_t st = static_cast<hipStream_t>(stream);
  const dim3 grid(blocks_for(n, kTile));
  if (id_bytes == 8)
    hipLaunchKernelGGL(encode_kernel<int64_t>, grid, dim3(kThreads), 0, st,
                       static_cast<const int64_t*>(data), n, ptr, num_batches, encoding_size,
                       static_cast<int64_t*>(out));
  else
    hipLaunchKernelGGL(encode_kernel<int32_t>, grid, dim3(kThreads), 0, st,
                       static_cast<const int32_t*>(data), n, ptr, num_batches, encoding_size,
                       static_cast<int32_t*>(out));
  return check_launch("batch_encode");
}

int gs_batch_decode(const void* in, int id_bytes, int64_t n, int64_t encoding_size, void* out_data,
                    void* out_batch, void* stream) {
  GS_REQUIRE(n >= 0 && encoding_size > 0, "gs_batch_decode: bad size");
  GS_REQUIRE(valid_id_bytes(id_bytes), "gs_batch_decode: id_bytes must be 4 or 8, got %d", id_bytes);
  if (n == 0) return GS_OK;
  GS_REQUIRE(in && (out_data || out_batch), "gs_batch_decode: null pointer");
  hipStream_t st = static_cast<hipStream_t>(stream);
  const dim3 grid(blocks_for(n, kThreads));
  if (id_bytes == 8)
    hipLaunchKernelGGL(decode_kernel<int64_t>, grid, dim3(kThreads), 0, st,
                       static_cast<const int64_t*>(in), n, encoding_size,
                       static_cast<int64_t*>(out_data), static_cast<int64_t*>(out_batch));
  else
    hipLaunchKernelGGL(decode_kernel<int32_t>, grid, dim3(kThreads), 0, st,
                       static_cast<const int32_t*>(in), n, encoding_size,
                       static_cast<int32_t*>(out_data), static_cast<int32_t*>(out_batch));
  return check_launch("batch_decode");
}

int gs_batch_offsets(const void* in, int id_bytes, int64_t n, int64_t num_batches,
                     int64_t encoding_size, int64_t* out_ptr, void* out_data, void* stream) {
  GS_REQUIRE(n >= 0 && num_batches >= 0 && encoding_size > 0, "gs_batch_offsets: bad size");
  GS_REQUIRE(valid_id_bytes(id_bytes), "gs_batch_offsets: id_bytes must be 4 or 8, got %d", id_bytes);
  GS_REQUIRE(out_ptr && (n == 0 || in), "gs_batch_offsets: null pointer");
  hipStream_t st = static_cast<hipStream_t>(stream);
  const dim3 grid(blocks_for(num_batches > 0 ? num_batches : 1, kThreads));
  if (id_bytes == 8)
    hipLaunchKernelGGL(offsets_kernel<int64_t>, grid, dim3(kThreads), 0, st,
                       static_cast<const int64_t*>(in), n, encoding_size, num_batches, out_ptr);
  else
    hipLaunchKernelGGL(offsets_kernel<int32_t>, grid, dim3(kThreads), 0, st,
                       static_cast<const int32_t*>(in), n, encoding_size, num_batches, out_ptr);
  GS_RETURN_IF_ERROR(check_launch("batch_offsets"));
  if (out_data && n > 0) return gs_batch_decode(in, id_bytes, n, encoding_size, out_data, nullptr, stream);
  return GS_OK;
}

static int load_segments(const char* who, const void* const* data, const int64_t* const* ptrs,
                         int num_segments, Segments* seg) {
  GS_REQUIRE(num_segments >= 1 && num_segments <= GS_MAX_SEGMENTS,
             "%s: 1..%d segments supported, got %d", who, GS_MAX_SEGMENTS, num_segments);
  GS_REQUIRE(ptrs, "%s: null pointer", who);
  seg->n = num_segments;
  for (int s = 0; s < num_segments; ++s) {
    GS_REQUIRE(ptrs[s], "%s: segment %d has no offsets", who, s);
    seg->ptr[s] = ptrs[s];
    seg->data[s] = data ? data[s] : nullptr;
  }
  return GS_OK;
}

int gs_batch_concat_offsets(const int64_t* const* segment_ptrs_host, int num_segments,
                            int64_t num_batches, int64_t* out_ptr, void* stream) {
  GS_REQUIRE(num_batches >= 1 && out_ptr, "gs_batch_concat_offsets: bad argument");
  Segments seg;
  GS_RETURN_IF_ERROR(
      load_segments("gs_batch_concat_offsets", nullptr, segment_ptrs_host, num_segments, &seg));
  hipLaunchKernelGGL(concat_offsets_kernel, dim3(blocks_for(num_batches + 1, kThreads)),
                     dim3(kThreads), 0, static_cast<hipStream_t>(stream), seg, num_batches, out_ptr);
  return check_launch("batch_concat_offsets");
}

int gs_batch_concat_fill(const void* const* segment_data_host,
                         const int64_t* const* segment_ptrs_host, int num_segments,
                         int64_t num_batches, int64_t max_segment_len, int id_bytes,
                         const int64_t* out_ptr, void* out, void* out_key, void* stream) {
  GS_REQUIRE(num_batches >= 1 && max_segment_len >= 0 && out_ptr,
             "gs_batch_concat_fill: bad argument");
  GS_REQUIRE(valid_id_bytes(id_bytes), "gs_batch_concat_fill: id_bytes must be 4 or 8, got %d",
             id_bytes);
  GS_REQUIRE(segment_data_host, "gs_batch_concat_fill: null pointer");
  Segments seg;
  GS_RETURN_IF_ERROR(load_segments("gs_batch_concat_fill", segment_data_host, segment_ptrs_host,
                                   num_segments, &seg));
  if (max_segment_len == 0) return GS_OK;
  GS_REQUIRE(out, "gs_batch_concat_fill: null output");
  const dim3 grid(blocks_for(max_segment_len, kTile), num_segments);
  hipStream_t st = static_cast<hipStream_t>(stream);
  if (id_bytes == 8)
    hipLaunchKernelGGL(concat_fill_kernel<int64_t>, grid, dim3(kThreads), 0, st, seg, num_batches,
                       out_ptr, static_cast<int64_t*>(out), static_cast<int64_t*>(out_key));
  else
    hipLaunchKernelGGL(concat_fill_kernel<int32_t>, grid, dim3(kThreads), 0, st, seg, num_batches,
                       out_ptr, static_cast<int32_t*>(out), static_cast<int32_t*>(out_key));
  return check_launch("batch_concat_fill");
}

int gs_batch_split(const void* data, const int64_t* data_ptr, const void* data_key, int id_bytes,
                   int64_t n, int64_t num_batches, void* const* out_data_host,
                   const int64_t* const* out_ptrs_host, int num_segments, void* stream) {
  GS_REQUIRE(n >= 0 && num_batches >= 1, "gs_batch_split: bad size");
  GS_REQUIRE(valid_id_bytes(id_bytes), "gs_batch_split: id_bytes must be 4 or 8, got %d", id_bytes);
  GS_REQUIRE(num_segments >= 1 && num_segments <= GS_MAX_SEGMENTS,
             "gs_batch_split: 1..%d segments supported, got %d", GS_MAX_SEGMENTS, num_segments);
  GS_REQUIRE(data_ptr && out_data_host && out_ptrs_host, "gs_batch_split: null pointer");
  OutSegments seg;
  seg.n = num_segments;
  for (int s = 0; s < num_segments; ++s) {
    GS_REQUIRE(out_ptrs_host[s], "gs_batch_split: segment %d has no offsets", s);
    seg.data[s] = out_data_host[s];
    seg.ptr[s] = out_ptrs_host[s];
  }
  if (n == 0) return GS_OK;
  GS_REQUIRE(data, "gs_batch_split: null input");
  const dim3 grid(blocks_for(n, kTile));
  hipStream_t st = static_cast<hipStream_t>(stream);
  if (id_bytes == 8)
    hipLaunchKernelGGL(split_kernel<int64_t>, grid, dim3(kThreads), 0, st,
                       static_cast<const int64_t*>(data), data_ptr,
                       static_cast<const int64_t*>(data_key), n, num_batches, seg);
  else
    hipLaunchKernelGGL(split_kernel<int32_t>, grid, dim3(kThreads), 0, st,
                       static_cast<const int32_t*>(data), data_ptr,
                       static_cast<const int32_t*>(data_key), n, num_batches, seg);
  return check_launch("batch_split");
}

}  // extern "C"
