/*
 * gs_oracle.c -- CPU restatement of the czkkkkkk/graph_sampling hot path.
 *
 * TEST INFRASTRUCTURE ONLY.  This file is the parity checker for the HIP
 * kernels and the host-core baseline of the benchmark.  Nothing in the shipped
 * library may link, import or call it; only tests/, the smoke check and the
 * benchmark's cpu_baseline leg do.
 *
 * Every function restates one reference routine (file:line given at each
 * function, paths relative to the reference tree).  All ids are int64 and all
 * edge data float32, exactly the types the reference instantiates
 * (src/cuda/slicing.cu:176, src/cuda/sddmm.cu:267).
 *
 * Randomness.  The reference draws from cuRAND streams whose seeding depends
 * on the CUDA launch geometry (src/cuda/sampling.cu:51); no test of the
 * reference checks a sampled value, so those streams are "parity unpinned".
 * This restatement keeps the reference *algorithms* (Algorithm R reservoir,
 * A-Res top-k, modulo pick) -- plus, as a second selectable algorithm for
 * uniform sampling without replacement, Floyd's k-subset selection (see
 * gso_sample_uniform_fill) -- and defines the draw as a pure function
 *     draw(seed, tag, row, idx) = Philox4x32-10(key=seed, ctr=(idx/4,row,tag))[idx%4]
 * or, in replay mode, a lookup in a caller-supplied uint32 buffer.  Philox is
 * pinned by the Random123 known-answer vectors (tests/test_oracle_pins.py).
 *
 * Floating point.  A-Res keys are compared as log2(u)/w (monotone in the
 * reference's u^(1/w), src/cuda/sampling_probs.cu:71) through gso_log2_u24(),
 * which uses only correctly rounded IEEE-754 binary32 operations so that a
 * device implementation of the same recipe is bit-identical.  Build with
 * -ffp-contract=off.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>
#ifdef _OPENMP
#include <omp.h>
#endif

typedef int64_t i64;
typedef uint32_t u32;
typedef uint64_t u64;

#define GSO_TAG_UNIFORM 1u
#define GSO_TAG_WEIGHTED 2u
#define GSO_TAG_WALK 3u
#define GSO_TAG_LIST_UNIFORM 4u
#define GSO_TAG_LIST_WEIGHTED 5u

int gso_num_threads(void) {
#ifdef _OPENMP
  return omp_get_max_threads();
#else
  return 1;
#endif
}

void gso_set_num_threads(int n) {
#ifdef _OPENMP
  omp_set_num_threads(n);
#else
  (void)n;
#endif
}

/* ------------------------------------------------------------------------ */
/* Philox4x32-10 (Salmon et al., SC'11; Random123 philox.h).                 */
/* ------------------------------------------------------------------------ */
void gso_philox4x32_10(const u32 ctr[4], const u32 key[2], u32 out[4]) {
  u32 c0 = ctr[0], c1 = ctr[1], c2 = ctr[2], c3 = ctr[3];
  u32 k0 = key[0], k1 = key[1];
  for (int round = 0; round < 10; ++round) {
    u64 p0 = (u64)0xD2511F53u * c0;
    u64 p1 = (u64)0xCD9E8D57u * c2;
    u32 n0 = (u32)(p1 >> 32) ^ c1 ^ k0;
    u32 n1 = (u32)p1;
    u32 n2 = (u32)(p0 >> 32) ^ c3 ^ k1;
    u32 n3 = (u32)p0;
    c0 = n0; c1 = n1; c2 = n2; c3 = n3;
    k0 += 0x9E3779B9u;
    k1 += 0xBB67AE85u;
  }
  out[0] = c0; out[1] = c1; out[2] = c2; out[3] = c3;
}

/* The draw shared by every sampler of this build: one Philox block serves four
 * consecutive idx values of the same row. */
u32 gso_draw(u64 seed, u32 tag, u64 row, u64 idx) {
  u64 q = idx >> 2;
  u32 ctr[4] = {(u32)q, (u32)row, (u32)(row >> 32), tag | ((u32)(q >> 32) << 8)};
  u32 key[2] = {(u32)seed, (u32)(seed >> 32)};
  u32 out[4];
  gso_philox4x32_10(ctr, key, out);
  return out[idx & 3];
}

/* ------------------------------------------------------------------------ */
/* A-Res key: log2(u)/w with u = ((x>>8)+1) * 2^-24 in (0,1] (same range as   */
/* curand_uniform, src/cuda/sampling_probs.cu:71).                           */
/* ------------------------------------------------------------------------ */
float gso_log2_u24(u32 x) {
  u32 m = (x >> 8) + 1u; /* 1 .. 2^24 */
  int e = 31 - __builtin_clz(m);
  /* mantissa f = m / 2^e in [1,2): exact in binary32 */
  float f = (float)m * (1.0f / (float)(1u << e));
  if (f > 1.41421356f) {
    f = f * 0.5f;
    e += 1;
  }
  float s = (f - 1.0f) / (f + 1.0f);
  float z = s * s;
  /* 2*atanh(s)/ln2 = (2/ln2) * s * (1 + z/3 + z^2/5 + z^3/7 + z^4/9) */
  float p = fmaf(z, 0.11111111f, 0.14285715f);
  p = fmaf(z, p, 0.2f);
  p = fmaf(z, p, 0.33333334f);
  p = fmaf(z, p, 1.0f);
  float l = (s * 2.88539008f) * p;
  return l + (float)(e - 24);
}

float gso_ares_key(u32 x, float w) {
  if (!(w > 0.0f)) return -INFINITY; /* src/cuda/list_sampling_probs.cu:70-73 */
  return gso_log2_u24(x) / w;
}

/* ------------------------------------------------------------------------ */
/* Column slicing.  src/cuda/slicing.cu:101-168                              */
/* ------------------------------------------------------------------------ */
/* sub_indptr = exscan(deg(cols[r])), returns the total. (slicing.cu:133-147) */
/* A column id outside [0, num_cols) counts as an empty column in every routine
 * below (the reference reads indptr[id] unchecked; the build defines this so
 * that the -1 a dead-end step returns can be fed back in as a seed). */
static inline int col_ok(i64 c, i64 num_cols) { return c >= 0 && c < num_cols; }

i64 gso_slice_count(const i64* indptr, i64 num_cols, const i64* cols, i64 S, i64* sub_indptr) {
  i64 acc = 0;
  for (i64 r = 0; r < S; ++r) {
    sub_indptr[r] = acc;
    if (col_ok(cols[r], num_cols)) acc += indptr[cols[r] + 1] - indptr[cols[r]];
  }
  sub_indptr[S] = acc;
  return acc;
}

/* neighbour copy (slicing.cu:101-119); coo_col may be NULL (WITH_COO=false) */
void gso_slice_fill(const i64* indptr, const i64* indices, const i64* cols, i64 S,
                    const i64* sub_indptr, i64* sub_indices, i64* select_index,
                    i64* coo_col) {
#pragma omp parallel for schedule(dynamic, 64)
  for (i64 r = 0; r < S; ++r) {
    i64 out_start = sub_indptr[r];
    i64 n = sub_indptr[r + 1] - out_start;
    if (n == 0) continue;
    i64 in_start = indptr[cols[r]];
    for (i64 j = 0; j < n; ++j) {
      sub_indices[out_start + j] = indices[in_start + j];
      select_index[out_start + j] = in_start + j;
      if (coo_col) coo_col[out_start + j] = r;
    }
  }
}

/* ------------------------------------------------------------------------ */
/* Uniform column sampling.  src/cuda/sampling.cu:13-154 (cols == NULL: every */
/* column of the CSC) and src/cuda/fusion/slice_sampling.cu:14-143 (cols      */
/* given: fused slice + sample).                                             */
/* ------------------------------------------------------------------------ */
static inline i64 col_of(const i64* cols, i64 r) { return cols ? cols[r] : r; }

/* Selection algorithm for uniform sampling without replacement.
 * GSO_ALGO_RESERVOIR: Algorithm R on every row with deg > k, exactly the
 *   reference (sampling.cu:70-92); a row consumes deg-k draws.
 * GSO_ALGO_AUTO: rows with deg > k use Floyd's algorithm (Bentley & Floyd,
 *   CACM 30(9) 1987, "A sample of brilliance") when k <= GSO_FLOYD_MAX_K: k
 *   draws per row instead of deg-k, the same uniform distribution over
 *   k-subsets.  Larger k falls back to Algorithm R. */
#define GSO_ALGO_AUTO 0
#define GSO_ALGO_RESERVOIR 1
#define GSO_FLOYD_MAX_K 64

static inline int use_floyd(int algo, i64 k) { return algo == GSO_ALGO_AUTO && k <= GSO_FLOYD_MAX_K; }

/* sub_indptr = exscan(cnt), cnt = replace ? (deg ? k : 0) : min(deg,k)
 * (sampling.cu:107-119).  replay_ptr (optional, may be NULL) = exscan of the
 * number of draws each row consumes: replace ? cnt : (deg > k ? (Floyd ? k :
 * deg-k) : 0). */
i64 gso_sample_count(const i64* indptr, i64 num_cols, const i64* cols, i64 S, i64 k, int replace,
                     int algo, i64* sub_indptr, i64* replay_ptr) {
  i64 acc = 0, racc = 0;
  for (i64 r = 0; r < S; ++r) {
    i64 c = col_of(cols, r);
    i64 deg = col_ok(c, num_cols) ? indptr[c + 1] - indptr[c] : 0;
    i64 cnt = replace ? (deg == 0 ? 0 : k) : (deg < k ? deg : k);
    sub_indptr[r] = acc;
    acc += cnt;
    if (replay_ptr) {
      replay_ptr[r] = racc;
      racc += replace ? cnt : (deg > k ? (use_floyd(algo, k) ? k : deg - k) : 0);
    }
  }
  sub_indptr[S] = acc;
  if (replay_ptr) replay_ptr[S] = racc;
  return acc;
}

void gso_sample_uniform_fill(const i64* indptr, i64 num_cols, const i64* indices, const i64* cols,
                             i64 S, i64 k, int replace, int algo, u64 seed, const u32* replay,
                             const i64* replay_ptr, const i64* sub_indptr,
                             i64* sub_indices, i64* select_index, i64* coo_col) {
#pragma omp parallel
  {
    i64* slot = (i64*)malloc(sizeof(i64) * (size_t)(k > 0 ? k : 1));
#pragma omp for schedule(dynamic, 16)
    for (i64 r = 0; r < S; ++r) {
      i64 c = col_of(cols, r);
      if (!col_ok(c, num_cols)) continue;
      i64 in_start = indptr[c];
      i64 deg = indptr[c + 1] - in_start;
      i64 out_start = sub_indptr[r];
      i64 cnt = sub_indptr[r + 1] - out_start;
      const u32* rp = replay ? replay + replay_ptr[r] : NULL;
      if (replace) {
        /* sampling.cu:29-39: edge = rand % degree for each output slot */
        for (i64 j = 0; j < cnt; ++j) {
          u32 x = rp ? rp[j] : gso_draw(seed, GSO_TAG_UNIFORM, (u64)r, (u64)j);
          i64 q = in_start + (i64)(x % (u32)deg);
          sub_indices[out_start + j] = indices[q];
          select_index[out_start + j] = q;
          if (coo_col) coo_col[out_start + j] = r;
        }
      } else if (deg <= k) {
        /* sampling.cu:60-69: copy in order */
        for (i64 j = 0; j < deg; ++j) {
          sub_indices[out_start + j] = indices[in_start + j];
          select_index[out_start + j] = in_start + j;
          if (coo_col) coo_col[out_start + j] = r;
        }
      } else if (use_floyd(algo, k)) {
        /* Floyd: for step i (j = deg-k+i): t = draw % (j+1); take t unless it
         * is already taken, then take j.  Output in insertion order. */
        for (i64 i = 0; i < k; ++i) {
          i64 j = deg - k + i;
          u32 x = rp ? rp[i] : gso_draw(seed, GSO_TAG_UNIFORM, (u64)r, (u64)i);
          i64 t = (i64)(x % (u32)(j + 1));
          for (i64 m = 0; m < i; ++m)
            if (slot[m] == t) {
              t = j;
              break;
            }
          slot[i] = t;
        }
        for (i64 j = 0; j < k; ++j) {
          i64 q = in_start + slot[j];
          sub_indices[out_start + j] = indices[q];
          select_index[out_start + j] = q;
          if (coo_col) coo_col[out_start + j] = r;
        }
      } else {
        /* sampling.cu:70-92: Algorithm R; AtomicMax on the slot == the draw
         * with the largest idx that lands on the slot wins. */
        for (i64 j = 0; j < k; ++j) slot[j] = j;
        for (i64 idx = k; idx < deg; ++idx) {
          u32 x = rp ? rp[idx - k] : gso_draw(seed, GSO_TAG_UNIFORM, (u64)r, (u64)idx);
          u32 num = x % (u32)(idx + 1);
          if ((i64)num < k && slot[num] < idx) slot[num] = idx;
        }
        for (i64 j = 0; j < k; ++j) {
          i64 q = in_start + slot[j];
          sub_indices[out_start + j] = indices[q];
          select_index[out_start + j] = q;
          if (coo_col) coo_col[out_start + j] = r;
        }
      }
    }
    free(slot);
  }
}

/* fanout == 1 && replace through the fused entry: exactly one slot per column,
 * -1/-1 for an empty column.  src/cuda/fusion/slice_sampling.cu:157-200 */
void gso_sample_one_keepdim(const i64* indptr, i64 num_cols, const i64* indices, const i64* cols,
                            i64 S, u64 seed, const u32* replay, i64* sub_indptr,
                            i64* sub_indices, i64* select_index) {
  for (i64 r = 0; r <= S; ++r) sub_indptr[r] = r;
#pragma omp parallel for schedule(static)
  for (i64 r = 0; r < S; ++r) {
    i64 c = cols[r];
    i64 in_start = col_ok(c, num_cols) ? indptr[c] : 0;
    i64 deg = col_ok(c, num_cols) ? indptr[c + 1] - in_start : 0;
    if (deg == 0) {
      sub_indices[r] = -1;
      select_index[r] = -1;
    } else {
      u32 x = replay ? replay[r] : gso_draw(seed, GSO_TAG_UNIFORM, (u64)r, 0);
      i64 q = in_start + (i64)(x % (u32)deg);
      sub_indices[r] = indices[q];
      select_index[r] = q;
    }
  }
}

/* ------------------------------------------------------------------------ */
/* Weighted column sampling without replacement (A-Res).                     */
/* src/cuda/sampling_probs.cu:25-110.  probs is indexed by edge position of   */
/* the input CSC (:70).  Order: descending key, ties -> lower position.       */
/* Replay: one draw per edge of every row with deg > k (replay_ptr = exscan). */
/* ------------------------------------------------------------------------ */
typedef struct {
  float key;
  i64 pos;
} gso_kp;

static int kp_before(const gso_kp* a, const gso_kp* b) {
  if (a->key > b->key) return 1;
  if (a->key < b->key) return 0;
  return a->pos < b->pos;
}

static int kp_cmp(const void* a, const void* b) {
  const gso_kp* x = (const gso_kp*)a;
  const gso_kp* y = (const gso_kp*)b;
  if (kp_before(x, y)) return -1;
  if (kp_before(y, x)) return 1;
  return 0;
}

i64 gso_weighted_replay_count(const i64* indptr, i64 num_cols, const i64* cols, i64 S, i64 k,
                              i64* replay_ptr) {
  i64 acc = 0;
  for (i64 r = 0; r < S; ++r) {
    i64 c = col_of(cols, r);
    i64 deg = col_ok(c, num_cols) ? indptr[c + 1] - indptr[c] : 0;
    replay_ptr[r] = acc;
    acc += deg > k ? deg : 0;
  }
  replay_ptr[S] = acc;
  return acc;
}

void gso_sample_weighted_fill(const i64* indptr, i64 num_cols, const i64* indices,
                              const float* probs, const i64* cols, i64 S, i64 k, u64 seed, const u32* replay,
                              const i64* replay_ptr, const i64* sub_indptr,
                              i64* sub_indices, i64* select_index, i64* coo_col) {
#pragma omp parallel for schedule(dynamic, 16)
  for (i64 r = 0; r < S; ++r) {
    i64 c = col_of(cols, r);
    if (!col_ok(c, num_cols)) continue;
    i64 in_start = indptr[c];
    i64 deg = indptr[c + 1] - in_start;
    i64 out_start = sub_indptr[r];
    if (deg <= k) {
      for (i64 j = 0; j < deg; ++j) {
        sub_indices[out_start + j] = indices[in_start + j];
        select_index[out_start + j] = in_start + j;
        if (coo_col) coo_col[out_start + j] = r;
      }
      continue;
    }
    gso_kp* kp = (gso_kp*)malloc(sizeof(gso_kp) * (size_t)deg);
    const u32* rp = replay ? replay + replay_ptr[r] : NULL;
    for (i64 i = 0; i < deg; ++i) {
      u32 x = rp ? rp[i] : gso_draw(seed, GSO_TAG_WEIGHTED, (u64)r, (u64)i);
      kp[i].key = gso_ares_key(x, probs[in_start + i]);
      kp[i].pos = i;
    }
    qsort(kp, (size_t)deg, sizeof(gso_kp), kp_cmp);
    for (i64 j = 0; j < k; ++j) {
      i64 q = in_start + kp[j].pos;
      sub_indices[out_start + j] = indices[q];
      select_index[out_start + j] = q;
      if (coo_col) coo_col[out_start + j] = r;
    }
    free(kp);
  }
}

/* ------------------------------------------------------------------------ */
/* Weighted column sampling WITH replacement (inverse CDF).                   */
/* src/cuda/sampling_probs.cu:112-183.  cdf = inclusive prefix of             */
/* max(prob, 0) over the column's edges.  The reference scans warp-sized      */
/* chunks with cub::WarpScan and carries the running total into the first     */
/* element of the next chunk (:147-160); restated here with 64-wide chunks    */
/* and the scan written out as its Kogge-Stone steps (x[i] += x[i-d] for      */
/* d = 1, 2, .., 32), so that the float additions happen in one fixed order.  */
/* That chain is sequential along the column; so that a hub column is not one  */
/* chain of thousands of steps, a column is cut into blocks of 2048 edges:     */
/* every block is scanned from zero, the blocks' totals are added up in order, */
/* and entry i of block b is (sum of the totals before b) + (its value inside  */
/* the block).  Columns up to 2048 edges are one block: nothing changes there. */
/* Pick j of row r: u = ((draw >> 8) + 1) * 2^-24 in (0, 1], rand = u * total,*/
/* item = first position with cdf > rand, clamped to deg-1 (:164-171).        */
/* Replay: replay[r * k + j].  The concrete picks are parity unpinned         */
/* (no test of the reference calls SamplingProbs).                            */
/* ------------------------------------------------------------------------ */
static void cdf_chunks64(const float* prob, i64 deg, float* cdf) {
  float carry = 0.0f;
  for (i64 base = 0; base < deg; base += 64) {
    float x[64], y[64];
    for (int l = 0; l < 64; ++l) {
      float v = base + l < deg ? prob[base + l] : 0.0f;
      if (l == 0) v += carry;
      x[l] = v > 0.0f ? v : 0.0f;
    }
    for (int d = 1; d < 64; d <<= 1) {
      for (int l = 0; l < 64; ++l) y[l] = l >= d ? x[l] + x[l - d] : x[l];
      memcpy(x, y, sizeof(x));
    }
    carry = x[63];
    for (int l = 0; l < 64 && base + l < deg; ++l) cdf[base + l] = x[l];
  }
}

static void cdf_column(const float* prob, i64 deg, float* cdf) {
  float before = 0.0f;
  for (i64 lo = 0; lo < deg; lo += 2048) {
    i64 len = deg - lo < 2048 ? deg - lo : 2048;
    cdf_chunks64(prob + lo, len, cdf + lo);
    float block_total = cdf[lo + len - 1];
    if (lo > 0)
      for (i64 i = 0; i < len; ++i) cdf[lo + i] = before + cdf[lo + i];
    before = before + block_total;
  }
}

void gso_sample_weighted_replace(const i64* indptr, i64 num_cols, const i64* indices,
                                 const float* probs, const i64* cols, i64 S, i64 k, u64 seed,
                                 const u32* replay, const i64* sub_indptr, i64* sub_indices,
                                 i64* select_index, i64* coo_col) {
#pragma omp parallel for schedule(dynamic, 16)
  for (i64 r = 0; r < S; ++r) {
    i64 c = col_of(cols, r);
    if (!col_ok(c, num_cols)) continue;
    i64 in_start = indptr[c];
    i64 deg = indptr[c + 1] - in_start;
    if (deg <= 0) continue;
    i64 out_start = sub_indptr[r];
    float* cdf = (float*)malloc(sizeof(float) * (size_t)deg);
    cdf_column(probs + in_start, deg, cdf);
    const float total = cdf[deg - 1];
    for (i64 j = 0; j < k; ++j) {
      u32 x = replay ? replay[r * k + j] : gso_draw(seed, GSO_TAG_WEIGHTED, (u64)r, (u64)j);
      float u = (float)((x >> 8) + 1u) * 5.9604644775390625e-08f; /* 2^-24, exact */
      float rnd = u * total;
      /* first position with cdf > rnd: first the block whose last entry exceeds rnd,
       * then inside it.  Prefix sums made by different addition trees need not be
       * monotone to the last bit, so the probe sequence is part of the definition. */
      i64 nblocks = (deg + 2047) / 2048;
      i64 lo = 0, hi = nblocks;
      while (lo < hi) {
        i64 mid = (lo + hi) >> 1;
        i64 end = (mid + 1) * 2048 < deg ? (mid + 1) * 2048 : deg;
        if (cdf[end - 1] <= rnd) lo = mid + 1; else hi = mid;
      }
      if (lo < nblocks) {
        i64 b = lo;
        lo = b * 2048;
        hi = lo + 2048 < deg ? lo + 2048 : deg;
        while (lo < hi) {
          i64 mid = (lo + hi) >> 1;
          if (cdf[mid] <= rnd) lo = mid + 1; else hi = mid;
        }
      } else {
        lo = deg;
      }
      if (lo > deg - 1) lo = deg - 1;
      sub_indices[out_start + j] = indices[in_start + lo];
      select_index[out_start + j] = in_start + lo;
      if (coo_col) coo_col[out_start + j] = r;
    }
    free(cdf);
  }
}

/* ------------------------------------------------------------------------ */
/* List sampling.  src/cuda/list_sampling.cu:20-77 (uniform, Algorithm R over */
/* positions), src/cuda/list_sampling_probs.cu:11-91 (A-Res, keys sorted      */
/* descending, first k).  Returns the number of picks written.               */
/* ------------------------------------------------------------------------ */
i64 gso_list_sample_uniform(const i64* data, i64 n, i64 k, int replace, u64 seed,
                            const u32* replay, i64* out_data, i64* out_index) {
  if (n <= k && !replace) { /* list_sampling.cu:29-32 */
    for (i64 i = 0; i < n; ++i) {
      out_data[i] = data[i];
      out_index[i] = i;
    }
    return n;
  }
  if (replace) { /* :38-52 */
    for (i64 j = 0; j < k; ++j) {
      u32 x = replay ? replay[j] : gso_draw(seed, GSO_TAG_LIST_UNIFORM, 0, (u64)j);
      out_index[j] = (i64)(x % (u32)n);
      out_data[j] = data[out_index[j]];
    }
    return k;
  }
  for (i64 j = 0; j < k; ++j) out_index[j] = j; /* :54-71 */
  for (i64 idx = k; idx < n; ++idx) {
    u32 x = replay ? replay[idx - k] : gso_draw(seed, GSO_TAG_LIST_UNIFORM, 0, (u64)idx);
    u32 num = x % (u32)(idx + 1);
    if ((i64)num < k && out_index[num] < idx) out_index[num] = idx;
  }
  for (i64 j = 0; j < k; ++j) out_data[j] = data[out_index[j]];
  return k;
}

i64 gso_list_sample_weighted(const i64* data, const float* probs, i64 n, i64 k, u64 seed,
                             const u32* replay, i64* out_data, i64* out_index) {
  if (n <= k) { /* list_sampling_probs.cu:20-23 */
    for (i64 i = 0; i < n; ++i) {
      out_data[i] = data[i];
      out_index[i] = i;
    }
    return n;
  }
  gso_kp* kp = (gso_kp*)malloc(sizeof(gso_kp) * (size_t)n);
#pragma omp parallel for schedule(static)
  for (i64 i = 0; i < n; ++i) {
    u32 x = replay ? replay[i] : gso_draw(seed, GSO_TAG_LIST_WEIGHTED, 0, (u64)i);
    kp[i].key = gso_ares_key(x, probs[i]);
    kp[i].pos = i;
  }
  qsort(kp, (size_t)n, sizeof(gso_kp), kp_cmp);
  for (i64 j = 0; j < k; ++j) {
    out_index[j] = kp[j].pos;
    out_data[j] = data[kp[j].pos];
  }
  free(kp);
  return k;
}

/* ------------------------------------------------------------------------ */
/* Unique / relabel.  src/cuda/unique_reindex.cu:81-199.  The reference       */
/* output order is first occurrence (:106-144), independent of table layout.  */
/* ------------------------------------------------------------------------ */
static u64 mix64(u64 x) {
  x ^= x >> 33;
  x *= 0xff51afd7ed558ccdULL;
  x ^= x >> 33;
  x *= 0xc4ceb9fe1a85ec53ULL;
  x ^= x >> 33;
  return x;
}

typedef struct {
  i64* keys;
  i64* vals;
  u64 mask;
} gso_table;

static void table_init(gso_table* t, i64 n) {
  u64 cap = 16;
  while (cap < (u64)n * 2u) cap <<= 1;
  t->keys = (i64*)malloc(sizeof(i64) * cap);
  t->vals = (i64*)malloc(sizeof(i64) * cap);
  t->mask = cap - 1;
  for (u64 i = 0; i < cap; ++i) t->keys[i] = -1;
}

static void table_free(gso_table* t) {
  free(t->keys);
  free(t->vals);
}

/* returns the slot of key, inserting it with value v when absent */
static u64 table_upsert(gso_table* t, i64 key, i64 v, int* inserted) {
  u64 p = mix64((u64)key) & t->mask;
  while (1) {
    if (t->keys[p] == key) {
      *inserted = 0;
      return p;
    }
    if (t->keys[p] == -1) {
      t->keys[p] = key;
      t->vals[p] = v;
      *inserted = 1;
      return p;
    }
    p = (p + 1) & t->mask;
  }
}

static i64 table_find(const gso_table* t, i64 key) {
  u64 p = mix64((u64)key) & t->mask;
  while (1) {
    if (t->keys[p] == key) return t->vals[p];
    if (t->keys[p] == -1) return -1; /* unique_reindex.cu:52-54 */
    p = (p + 1) & t->mask;
  }
}

/* distinct values in first-occurrence order; returns their number */
i64 gso_unique(const i64* x, i64 n, i64* out) {
  gso_table t;
  table_init(&t, n);
  i64 u = 0;
  for (i64 i = 0; i < n; ++i) {
    int ins;
    table_upsert(&t, x[i], u, &ins);
    if (ins) out[u++] = x[i];
  }
  table_free(&t);
  return u;
}

/* frontier = unique(mapping); out[i] = rank of query[i] in frontier, -1 when
 * absent (unique_reindex.cu:154-199).  Returns |frontier|. */
i64 gso_relabel(const i64* mapping, i64 n_map, const i64* query, i64 n_query,
                i64* frontier, i64* out) {
  gso_table t;
  table_init(&t, n_map);
  i64 u = 0;
  for (i64 i = 0; i < n_map; ++i) {
    int ins;
    table_upsert(&t, mapping[i], u, &ins);
    if (ins) frontier[u++] = mapping[i];
  }
#pragma omp parallel for schedule(static)
  for (i64 i = 0; i < n_query; ++i) out[i] = table_find(&t, query[i]);
  table_free(&t);
  return u;
}

/* ------------------------------------------------------------------------ */
/* Random walks.  src/cuda/fusion/random_walk.cu:11-68,                      */
/* src/cuda/fusion/metapath_random_walk.cu:10-67.  trace memory is            */
/* [L+1][n] (step-major); -1 is absorbing; one draw per live step.           */
/* Replay buffer layout: [L][n].                                             */
/* ------------------------------------------------------------------------ */
void gso_random_walk(const i64* indptr, i64 num_nodes, const i64* indices, const i64* seeds, i64 n,
                     i64 L, u64 seed, const u32* replay, i64* trace) {
#pragma omp parallel for schedule(static)
  for (i64 w = 0; w < n; ++w) {
    i64 curr = seeds[w];
    trace[w] = curr;
    for (i64 t = 0; t < L; ++t) {
      i64 pick = -1;
      if (col_ok(curr, num_nodes)) {
        i64 start = indptr[curr];
        i64 deg = indptr[curr + 1] - start;
        if (deg > 0) {
          u32 x = replay ? replay[t * n + w] : gso_draw(seed, GSO_TAG_WALK, (u64)w, (u64)t);
          pick = indices[start + (i64)(x % (u32)deg)];
        }
      }
      trace[(t + 1) * n + w] = pick;
      curr = pick;
    }
  }
}

/* relation of step t is metapath[t]; (indptr, indices) tables per relation
 * (src/hetero_graph.cc:33-50, metapath_random_walk.cu:36-38). */
void gso_metapath_walk(const i64* const* all_indptr, const i64* const* all_indices,
                       const i64* all_num_nodes, const i64* metapath, i64 L, const i64* seeds, i64 n, u64 seed,
                       const u32* replay, i64* trace) {
#pragma omp parallel for schedule(static)
  for (i64 w = 0; w < n; ++w) {
    i64 curr = seeds[w];
    trace[w] = curr;
    for (i64 t = 0; t < L; ++t) {
      i64 pick = -1;
      if (col_ok(curr, all_num_nodes[metapath[t]])) {
        const i64* indptr = all_indptr[metapath[t]];
        const i64* indices = all_indices[metapath[t]];
        i64 start = indptr[curr];
        i64 deg = indptr[curr + 1] - start;
        if (deg > 0) {
          u32 x = replay ? replay[t * n + w] : gso_draw(seed, GSO_TAG_WALK, (u64)w, (u64)t);
          pick = indices[start + (i64)(x % (u32)deg)];
        }
      }
      trace[(t + 1) * n + w] = pick;
      curr = pick;
    }
  }
}

/* ------------------------------------------------------------------------ */
/* SDDMM.  src/cuda/sddmm.cu:21-154, src/cuda/functor.h:11-136,              */
/* src/cuda/selector.h:18-42, src/bcast.cc:24-75.                            */
/* op: 0 add 1 sub 2 mul 3 div 4 copy_lhs 5 copy_rhs 6 dot.                  */
/* target: 0 src(row id) 1 edge 2 dst(col id).                               */
/* lhs_off/rhs_off: broadcast offsets (NULL = identity).                     */
/* ------------------------------------------------------------------------ */
static inline float sddmm_op(int op, const float* l, const float* r, i64 R) {
  switch (op) {
    case 0: return l[0] + r[0];
    case 1: return l[0] - r[0];
    case 2: return l[0] * r[0];
    case 3: return l[0] / r[0];
    case 4: return l[0];
    case 5: return r[0];
    default: {
      float acc = 0.0f; /* functor.h:125-131 sequential order */
      for (i64 i = 0; i < R; ++i) acc += l[i] * r[i];
      return acc;
    }
  }
}

static inline i64 sel3(int target, i64 src, i64 eid, i64 dst) {
  return target == 0 ? src : (target == 1 ? eid : dst);
}

void gso_sddmm_coo(int op, const i64* row, const i64* col, const i64* e_ids, i64 E,
                   const float* lhs, const float* rhs, float* out, int lhs_target,
                   int rhs_target, i64 lhs_len, i64 rhs_len, i64 out_len, i64 R,
                   const i64* lhs_off, const i64* rhs_off) {
#pragma omp parallel for schedule(static)
  for (i64 e = 0; e < E; ++e) {
    i64 src = row[e], dst = col[e];
    i64 eid = e_ids ? e_ids[e] : e;
    const float* l = lhs ? lhs + sel3(lhs_target, src, eid, dst) * lhs_len : NULL;
    const float* r = rhs ? rhs + sel3(rhs_target, src, eid, dst) * rhs_len : NULL;
    for (i64 k = 0; k < out_len; ++k) {
      i64 la = lhs_off ? lhs_off[k] : k;
      i64 ra = rhs_off ? rhs_off[k] : k;
      out[eid * out_len + k] = sddmm_op(op, l ? l + la * R : NULL, r ? r + ra * R : NULL, R);
    }
  }
}

/* CSC flavour (sddmm.cu:118-154): src = indices[e], dst = column owning e
 * (optionally mapped through nid_map). */
void gso_sddmm_csc(int op, const i64* indptr, const i64* indices, const i64* e_ids,
                   const i64* nid_map, i64 num_cols, const float* lhs, const float* rhs,
                   float* out, int lhs_target, int rhs_target, i64 lhs_len, i64 rhs_len,
                   i64 out_len, i64 R, const i64* lhs_off, const i64* rhs_off) {
#pragma omp parallel for schedule(dynamic, 256)
  for (i64 c = 0; c < num_cols; ++c) {
    for (i64 e = indptr[c]; e < indptr[c + 1]; ++e) {
      i64 src = indices[e];
      i64 dst = nid_map ? nid_map[c] : c;
      i64 eid = e_ids ? e_ids[e] : e;
      const float* l = lhs ? lhs + sel3(lhs_target, src, eid, dst) * lhs_len : NULL;
      const float* r = rhs ? rhs + sel3(rhs_target, src, eid, dst) * rhs_len : NULL;
      for (i64 k = 0; k < out_len; ++k) {
        i64 la = lhs_off ? lhs_off[k] : k;
        i64 ra = rhs_off ? rhs_off[k] : k;
        out[eid * out_len + k] =
            sddmm_op(op, l ? l + la * R : NULL, r ? r + ra * R : NULL, R);
      }
    }
  }
}

/* ------------------------------------------------------------------------ */
/* Segment ops.  src/cuda/graph_ops.cu:16-188,                               */
/* src/cuda/fusion/edge_map_reduce.cu:10-25.                                 */
/* ------------------------------------------------------------------------ */
static inline float powk_f(float x, i64 powk) {
  if (powk == 1) return x; /* graph_ops.cu:30 */
  float p = x;
  for (i64 i = 1; i < powk; ++i) p *= x;
  return p;
}

/* out[nmap ? nmap[s] : s] = sum_{e in segment s, in order} f(data[emap?emap[e]:e]) */
void gso_segment_sum(const i64* indptr, const i64* e_ids, const i64* n_ids, const float* data,
                     i64 num_seg, i64 powk, float* out) {
#pragma omp parallel for schedule(dynamic, 256)
  for (i64 s = 0; s < num_seg; ++s) {
    float acc = 0.0f;
    for (i64 e = indptr[s]; e < indptr[s + 1]; ++e)
      acc += powk_f(data[e_ids ? e_ids[e] : e], powk);
    out[n_ids ? n_ids[s] : s] = acc;
  }
}

/* COO: out[target[e]] += f(data[emap?emap[e]:e]) (graph_ops.cu:45-64).  The
 * reference uses float atomics (order undefined); this restatement adds in
 * edge order. */
void gso_coo_sum(const i64* target, const i64* e_ids, const float* data, i64 E, i64 powk,
                 float* out) {
  for (i64 e = 0; e < E; ++e) out[target[e]] += powk_f(data[e_ids ? e_ids[e] : e], powk);
}

/* graph_ops.cu:132-158: out[d] = data[d] / sum_segment, d = emap ? emap[e] : e */
void gso_segment_normalize(const i64* indptr, const i64* e_ids, const float* data,
                           i64 num_seg, float* out) {
#pragma omp parallel for schedule(dynamic, 256)
  for (i64 s = 0; s < num_seg; ++s) {
    float acc = 0.0f;
    for (i64 e = indptr[s]; e < indptr[s + 1]; ++e) acc += data[e_ids ? e_ids[e] : e];
    for (i64 e = indptr[s]; e < indptr[s + 1]; ++e) {
      i64 d = e_ids ? e_ids[e] : e;
      out[d] = data[d] / acc;
    }
  }
}

/* edge_map_reduce.cu:15-23 */
void gso_e_div_u_sum(const i64* row, const i64* col, const float* data, const float* divisor,
                     i64 E, float* out_data, float* out_sum) {
  for (i64 e = 0; e < E; ++e) {
    out_data[e] = data[e] / divisor[row[e]];
    out_sum[col[e]] += out_data[e];
  }
}

/* ------------------------------------------------------------------------ */
/* Row slicing on CSC / on COO.  src/cuda/slicing.cu:417-539, :544-563,       */
/* :727-766.  Kept ids are relabeled to their position in row_ids.  When      */
/* row_ids holds duplicates the reference's table keeps an arbitrary one      */
/* (slicing.cu:56 plain store); this restatement keeps the last.             */
/* ------------------------------------------------------------------------ */
/* returns nnz kept.  out arrays are sized by the input nnz. */
i64 gso_row_slice_csc(const i64* indptr, const i64* indices, i64 num_cols, const i64* row_ids,
                      i64 n_rows, i64* out_indptr, i64* out_indices, i64* select_index,
                      i64* coo_col) {
  gso_table t;
  table_init(&t, n_rows);
  for (i64 i = 0; i < n_rows; ++i) {
    int ins;
    u64 p = table_upsert(&t, row_ids[i], i, &ins);
    t.vals[p] = i;
  }
  i64 w = 0;
  for (i64 c = 0; c < num_cols; ++c) {
    out_indptr[c] = w;
    for (i64 e = indptr[c]; e < indptr[c + 1]; ++e) {
      i64 v = table_find(&t, indices[e]);
      if (v != -1) {
        out_indices[w] = v;
        select_index[w] = e;
        if (coo_col) coo_col[w] = c;
        ++w;
      }
    }
  }
  out_indptr[num_cols] = w;
  table_free(&t);
  return w;
}

/* keep edges whose key[e] is in ids; key relabeled, other carried */
i64 gso_row_slice_coo(const i64* key, const i64* other, i64 E, const i64* ids, i64 n_ids,
                      i64* out_key, i64* out_other, i64* select_index) {
  gso_table t;
  table_init(&t, n_ids);
  for (i64 i = 0; i < n_ids; ++i) {
    int ins;
    u64 p = table_upsert(&t, ids[i], i, &ins);
    t.vals[p] = i;
  }
  i64 w = 0;
  for (i64 e = 0; e < E; ++e) {
    i64 v = table_find(&t, key[e]);
    if (v != -1) {
      out_key[w] = v;
      out_other[w] = other[e];
      select_index[w] = e;
      ++w;
    }
  }
  table_free(&t);
  return w;
}

/* ------------------------------------------------------------------------ */
/* Format conversion.  src/cuda/format_transform.cu:24-156,                   */
/* src/graph_ops.cc:13-60.                                                   */
/* ------------------------------------------------------------------------ */
/* CSC -> COO column vector: col[e] = owning column (format_transform.cu:24-46) */
void gso_csc2coo(const i64* indptr, i64 num_cols, i64* col) {
#pragma omp parallel for schedule(dynamic, 256)
  for (i64 c = 0; c < num_cols; ++c)
    for (i64 e = indptr[c]; e < indptr[c + 1]; ++e) col[e] = c;
}

/* COO -> CSC by *stable* sort on key (cub radix sort is stable,
 * format_transform.cu:81-100): perm = stable argsort(key); out_value =
 * value[perm]; indptr[c+1] = upper_bound(sorted key, c) (:123-156).
 * When sorted != 0 no reorder happens and perm is not written. */
void gso_coo2csc(const i64* key, const i64* value, i64 E, i64 num_keys, int sorted,
                 i64* indptr, i64* out_value, i64* perm) {
  for (i64 c = 0; c <= num_keys; ++c) indptr[c] = 0;
  for (i64 e = 0; e < E; ++e) indptr[key[e] + 1] += 1;
  for (i64 c = 0; c < num_keys; ++c) indptr[c + 1] += indptr[c];
  if (sorted) {
    for (i64 e = 0; e < E; ++e) out_value[e] = value[e];
    return;
  }
  i64* cursor = (i64*)malloc(sizeof(i64) * (size_t)(num_keys + 1));
  memcpy(cursor, indptr, sizeof(i64) * (size_t)(num_keys + 1));
  for (i64 e = 0; e < E; ++e) {
    i64 p = cursor[key[e]]++;
    out_value[p] = value[e];
    perm[p] = e;
  }
  free(cursor);
}
