/*
 * gs_hip.h -- C ABI of the MI355X (gfx950) graph-sampling kernels.
 *
 * This is the boundary a binding of czkkkkkk/graph_sampling links against in
 * place of its `gs::impl::*CUDA` functions (src/cuda/graph_ops.h:10-75,
 * src/cuda/tensor_ops.h:11-105, src/cuda/sddmm.h, the headers under src/cuda/fusion).  Each
 * entry point cites the reference routine it replaces.
 *
 * Conventions
 *  - Every pointer is a DEVICE pointer unless its name ends in `_host`.
 *  - Buffers are caller-owned; the library never allocates device memory.
 *    Scratch is passed as (workspace, workspace_bytes); the matching
 *    gs_*_workspace_bytes() gives the size.  Workspace must be 256-byte aligned.
 *  - `stream` is a hipStream_t passed as void* (NULL = the null stream).  Calls
 *    only enqueue work; they never synchronise.  Data-dependent result sizes
 *    are left in device memory (last element of an offsets array, or a device
 *    scalar) for the caller to read after its own synchronisation.
 *  - Offsets (indptr, sub_indptr, select_index, e_ids) are int64.  Node ids
 *    (indices, column ids, frontier, relabelled ids) are `id_bytes` wide: 8
 *    (int64, the reference's only instantiation, src/cuda/slicing.cu:176) or 4
 *    (int32 extension).
 *  - `num_cols` / `num_nodes` is the number of columns the offsets describe
 *    (indptr has num_cols + 1 entries).  A caller-supplied column id or walk
 *    seed outside [0, num_cols) is treated as an empty column / a dead walker;
 *    it is never dereferenced.  (The reference reads indptr[id] unchecked.)
 *  - Return value: GS_OK or a negative gs_status.  Nothing throws or aborts.
 *
 * Randomness.  draw(seed, tag, row, idx) =
 *     Philox4x32-10(key = seed, ctr = (idx/4, row_lo, row_hi, tag))[idx % 4].
 * When `replay` is non-NULL the draw is instead read from that uint32 buffer
 * (layout documented per entry point) so that two implementations fed the same
 * buffer return identical samples.
 */
#ifndef GS_HIP_H_
#define GS_HIP_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef enum gs_status {
  GS_OK = 0,
  GS_ERR_INVALID_ARG = -1,   /* null pointer, negative size, bad id_bytes ... */
  GS_ERR_WORKSPACE = -2,     /* workspace too small or misaligned */
  GS_ERR_UNSUPPORTED = -3,   /* combination not implemented (message says which) */
  GS_ERR_LAUNCH = -4         /* hipGetLastError() after a launch was not hipSuccess */
} gs_status;

/* Human-readable text for a status code; for GS_ERR_LAUNCH / GS_ERR_UNSUPPORTED
 * the text of the most recent failure on the calling thread. */
const char* gs_status_string(int status);

/* Library version (major*10000 + minor*100 + patch). */
int gs_version(void);

/* Result mailbox: 16 bytes of pinned, device-visible host memory (hipHostMalloc).
 * Entry points that take one let the kernel that produces a total (sampled edge
 * count, number of unique ids) also store {total, ticket} there with system
 * scope, total first.  The host may then spin on `ticket` instead of
 * synchronising the stream; work queued later on the same stream is still
 * ordered after the producing kernel.  NULL = no mailbox.  No counterpart in the
 * reference, which reads totals back with a blocking copy
 * (src/cuda/sampling.cu:124, src/cuda/unique_reindex.cu:120). */
typedef struct gs_mailbox {
  int64_t total;
  int64_t ticket;
} gs_mailbox;

/* Or-ed into id_bytes = 8 of gs_unique_relabel[_notify], gs_batch_csr_relabel and
 * gs_batch_coo_relabel: the 64-bit ids are promised to fit 32 bits (node ids of any graph below
 * 4.29 G nodes do), and the hash table uses the one-word slots of 32-bit ids -- one
 * compare-and-swap per insert instead of compare-and-swap, read and minimum.  Ids, frontier
 * and outputs stay 64-bit.  If a mapping id does not fit, *num_unique and the mailbox read -2
 * and nothing else written is valid: call again without the flag.  (The reference's API is
 * int64 throughout; this is how that costs no more than int32.) */
#define GS_NARROW_IDS 0x100

/* Or-ed into id_bytes of gs_batch_csr_relabel: which of its two implementations runs.  By
 * default ids that fit 32 bits (id_bytes 4, or 8 | GS_NARROW_IDS), from about half a million
 * items on and with at most 511 batches, are relabelled through bins (the items of a batch
 * are brought together by hash class and deduplicated in LDS: no atomic on memory per item);
 * everything else through one hash region per batch.  GS_RELABEL_REGIONS forces the second,
 * GS_RELABEL_BINS the first (refused with GS_ERR_UNSUPPORTED where it cannot run).  The bins
 * report *num_unique = -4 (mailbox too) when one class of one batch holds more distinct ids
 * than its LDS table (a single batch of more than ~16 M distinct ids): nothing else written is
 * valid then; call again with GS_RELABEL_REGIONS. */
#define GS_RELABEL_REGIONS 0x200
#define GS_RELABEL_BINS 0x400

/* Optional timing of one launch site, for benchmarks (no counterpart in the
 * reference).  gs_profile_enable("name") makes every later launch of that site
 * record a hipEvent pair on its stream (up to 4096 launches); NULL or ""
 * disables.  Sites: "sample_fused", "sample_floyd", "table_init", "table_insert",
 * "unique_compact", "unique_finish", "layer_sample", "layer_relabel", "layer_sweep",
 * "batch_init", "batch_insert", "batch_compact", "batch_finish", "bins_init", "bins_count",
 * "bins_scatter", "bins_flag", "bins_rank", "bins_rename", "scan_tile_sums",
 * "scan_apply", "random_walk", "metapath_walk", "sddmm_dot".  gs_profile_collect waits for the recorded
 * events, returns their summed duration and count (and, when per_launch_ms is
 * given, the first `cap` individual durations in launch order) and clears the
 * ring.  The events are created by the library and live until the process ends. */
int gs_profile_enable(const char* launch_site);
/* Time only every `every`-th launch of the enabled site (default 1 = all): an event
 * pair costs a few microseconds of queue time, which matters when the timed kernels
 * are themselves that short. */
int gs_profile_stride(int every);
int gs_profile_collect(double* total_ms, int64_t* launches, double* per_launch_ms, int64_t cap);

typedef enum gs_op {
  GS_OP_ADD = 0, GS_OP_SUB = 1, GS_OP_MUL = 2, GS_OP_DIV = 3,
  GS_OP_COPY_LHS = 4, GS_OP_COPY_RHS = 5, GS_OP_DOT = 6
} gs_op;

/* ------------------------------------------------------------------------- */
/* Column slicing: replaces impl::CSCColSlicingCUDA (src/cuda/slicing.cu:170). */
/* ------------------------------------------------------------------------- */
size_t gs_slice_workspace_bytes(int64_t num_cols);

/* sub_indptr[0..S] = exclusive scan of deg(column_ids[r]); total in sub_indptr[S]
 * (slicing.cu:133-147). */
int gs_slice_count(const int64_t* indptr, int64_t num_cols, const void* column_ids, int id_bytes,
                   int64_t S, int64_t* sub_indptr, void* workspace, size_t workspace_bytes,
                   void* stream);

/* Posts *value (a device int64, e.g. sub_indptr + S after gs_slice_count) to a mailbox from a
 * one-thread kernel queued on the stream: the host then spins on the mailbox instead of
 * copying the value back and synchronising the stream (the blocking read of
 * src/cuda/slicing.cu:147). */
int gs_post_total(const int64_t* value, gs_mailbox* mailbox, int64_t ticket, void* stream);
/* The same for an array: values[0..n) (device) are stored to host_out (pinned host memory, mapped
 * for the device) by one small kernel on the stream, and then {n, ticket} to the mailbox (may be
 * NULL): offsets a caller cuts its results by reach the host without a copy call. */
int gs_post_values(const int64_t* values, int64_t n, int64_t* host_out, gs_mailbox* mailbox,
                   int64_t ticket, void* stream);
/* Several arrays of the same length in one launch: sets is a HOST array of num_sets (at most 32)
 * device pointers, host_out receives sets[0][0..n), sets[1][0..n), ... one after the other, then
 * {num_sets * n, ticket} goes to the mailbox.  No counterpart in the reference (it reads
 * such offsets back one tensor at a time, examples/graphsage/batching.py:75-80). */
int gs_post_value_sets(const int64_t* const* sets, int num_sets, int64_t n, int64_t* host_out,
                       gs_mailbox* mailbox, int64_t ticket, void* stream);

/* Neighbour copy (slicing.cu:101-119).  nnz = sub_indptr[S] as read back by the
 * caller.  coo_col may be NULL (WITH_COO = false); select_index may be NULL when
 * the caller has no edge data to gather. */
int gs_slice_fill(const int64_t* indptr, int64_t num_cols, const void* indices,
                  const void* column_ids, int id_bytes, int64_t S, const int64_t* sub_indptr,
                  int64_t nnz, void* sub_indices, int64_t* select_index, void* coo_col,
                  void* stream);
/* gs_slice_fill that also carries the edges' data over in the same pass: data_out[p] =
 * edge_data[edge_ids ? edge_ids[q] : q] for the edge copied from position q of indices --
 * the gather the reference makes afterwards from select_index (src/graph.cc:68-73), which
 * the caller then need not ask for.  edge_data NULL (then edge_ids and data_out too):
 * gs_slice_fill. */
int gs_slice_fill_data(const int64_t* indptr, int64_t num_cols, const void* indices,
                       const void* column_ids, int id_bytes, int64_t S, const int64_t* sub_indptr,
                       int64_t nnz, void* sub_indices, int64_t* select_index, void* coo_col,
                       const float* edge_data, const int64_t* edge_ids, float* data_out,
                       void* stream);

/* ------------------------------------------------------------------------- */
/* Uniform neighbour sampling: replaces impl::CSCColSamplingCUDA              */
/* (src/cuda/sampling.cu:157; column_ids == NULL: every column 0..S-1 of the   */
/* CSC) and impl::fusion::FusedCSCColSlicingSamplingCUDA                      */
/* (src/cuda/fusion/slice_sampling.cu:146; column_ids given).                 */
/* ------------------------------------------------------------------------- */
size_t gs_sample_workspace_bytes(int64_t S, int64_t fanout);

/* Selection algorithm for uniform sampling WITHOUT replacement on rows with
 * deg > fanout.  Both give a uniformly distributed fanout-subset.
 *  GS_SAMPLE_RESERVOIR  the reference's Algorithm R (sampling.cu:70-92): slot j
 *      starts as j; for idx in [fanout, deg): num = draw(r, idx) % (idx+1), if
 *      num < fanout then slot[num] = max(slot[num], idx).  deg-fanout draws.
 *  GS_SAMPLE_AUTO       Floyd's selection when fanout <= GS_FLOYD_MAX_FANOUT
 *      (else Algorithm R): for step i in [0, fanout), j = deg-fanout+i,
 *      t = draw(r, i) % (j+1); position t is taken unless already taken, in
 *      which case j is.  fanout draws whatever the degree; output in step order. */
typedef enum gs_sample_algo { GS_SAMPLE_AUTO = 0, GS_SAMPLE_RESERVOIR = 1 } gs_sample_algo;
#define GS_FLOYD_MAX_FANOUT 64
/* largest fanout without replacement of the one-launch gs_sample_uniform_fused */
#define GS_FUSED_MAX_FANOUT 32

/* sub_indptr = exscan(cnt), cnt = replace ? (deg ? fanout : 0) : min(deg, fanout)
 * (sampling.cu:107-119). */
int gs_sample_count(const int64_t* indptr, int64_t num_cols, const void* column_ids, int id_bytes,
                    int64_t S, int64_t fanout, int replace, int64_t* sub_indptr, void* workspace,
                    size_t workspace_bytes, void* stream);

/* Fill for a sub_indptr made by gs_sample_count on the same stream.  Output
 * buffers need capacity S*fanout (an upper bound known without reading back).
 * Without replacement: deg <= fanout copies in order (sampling.cu:60-69), else
 * the algorithm `algo` selects; output is in slot / step order (unsorted).
 * With replacement: slot j = draw(r, j) % deg (sampling.cu:13-41).
 * replay / replay_ptr (both or neither): replay_ptr[S+1] offsets into replay;
 * a row with deg > fanout consumes deg-fanout draws (Algorithm R) or fanout
 * draws (Floyd), other rows none; with replacement every row consumes its
 * output count.  coo_col may be NULL. */
int gs_sample_uniform_fill(const int64_t* indptr, int64_t num_cols, const void* indices,
                           const void* column_ids, int id_bytes, int64_t S, int64_t fanout,
                           int replace, int algo, uint64_t seed,
                           const uint32_t* replay, const int64_t* replay_ptr,
                           const int64_t* sub_indptr, void* sub_indices, int64_t* select_index,
                           void* coo_col, void* workspace, size_t workspace_bytes, void* stream);

/* Column slice + uniform sample in ONE launch: count, offsets and fill together
 * (the same results as gs_sample_count + gs_sample_uniform_fill with
 * GS_SAMPLE_AUTO, bit for bit).  Replaces
 * impl::fusion::FusedCSCColSlicingSamplingCUDA (src/cuda/fusion/slice_sampling.cu:146)
 * and, with column_ids == NULL, impl::CSCColSamplingCUDA (src/cuda/sampling.cu:157),
 * without their mid-call host read.
 *   - without replacement fanout must be <= GS_FUSED_MAX_FANOUT (else
 *     GS_ERR_UNSUPPORTED: use the two-phase calls);
 *   - sub_indices / select_index / coo_col hold `capacity` >= S*fanout entries
 *     (select_index and coo_col may be NULL when the caller has no use for them);
 *     the true total is written to sub_indptr[S] (-1 if the kernel gave up
 *     waiting on another tile, which a healthy device never does) and to the
 *     mailbox when one is given;
 *   - state: gs_sample_fused_state_bytes(S) bytes, 256-byte aligned, zero-filled
 *     before its first use; epoch: 1..16383, different from the epoch of every
 *     earlier call on this buffer since it was last zero-filled (count up from
 *     1; zero-fill and start again after 16383).  Tiles mark their progress in
 *     `state` with the epoch, so nothing is cleared between calls.  Two calls
 *     running at the same time must not share a buffer. */
size_t gs_sample_fused_state_bytes(int64_t S);
int gs_sample_uniform_fused(const int64_t* indptr, int64_t num_cols, const void* indices,
                            const void* column_ids, int id_bytes, int64_t S, int64_t fanout,
                            int replace, uint64_t seed, const uint32_t* replay,
                            const int64_t* replay_ptr, int64_t* sub_indptr, void* sub_indices,
                            int64_t* select_index, void* coo_col, int64_t capacity,
                            void* state, size_t state_bytes, uint32_t epoch,
                            gs_mailbox* mailbox, int64_t mailbox_ticket, void* stream);

/* gs_sample_uniform_fused that also carries the graph's edge data over to the samples, in
 * the same launch: data_out[o] = edge_data[edge_ids ? edge_ids[q] : q] for the output o taken
 * at position q of `indices` (q is what select_index[o] receives).  Replaces the two torch
 * `index` gathers Graph::ColumnwiseFusedSlicingAndSampling makes after the sampler
 * (src/graph.cc:544-557: data_[e_ids[select_index]]).  edge_data: fp32, one value per edge id;
 * edge_ids: NULL, or the CSC's edge-id map (int64, one per position of `indices`); data_out:
 * `capacity` floats.  All three NULL: exactly gs_sample_uniform_fused. */
int gs_sample_uniform_fused_data(const int64_t* indptr, int64_t num_cols, const void* indices,
                                 const void* column_ids, int id_bytes, int64_t S, int64_t fanout,
                                 int replace, uint64_t seed, const uint32_t* replay,
                                 const int64_t* replay_ptr, int64_t* sub_indptr,
                                 void* sub_indices, int64_t* select_index, void* coo_col,
                                 int64_t capacity, const float* edge_data,
                                 const int64_t* edge_ids, float* data_out, void* state,
                                 size_t state_bytes, uint32_t epoch, gs_mailbox* mailbox,
                                 int64_t mailbox_ticket, void* stream);

/* gs_sample_uniform_fused for callers that cannot allocate (no counterpart in the
 * reference: it is for code under HIP graph capture, tight serving loops and harnesses
 * that forbid hipMalloc, which can bring outputs but no state buffer of the right age).
 * The look-back state lives in a device array of the library itself
 * (GS_FUSED_STATIC_MAX_COLUMNS columns, about 130 KB per device, held until the process
 * ends) and the library counts the epochs; the call allocates nothing, on the host side
 * of the device or on the device.  Same arguments, results and status codes as
 * gs_sample_uniform_fused otherwise; S above GS_FUSED_STATIC_MAX_COLUMNS is refused with
 * GS_ERR_UNSUPPORTED.  Runs on the current device.  Every call on a device shares that
 * device's array: calls that overlap in time on one device (two streams, two threads)
 * race; calls on one stream, or ordered by events, are fine.  Once per 16383 calls, at the
 * first call on a device and after a reset, a fill kernel on `stream` zeroes the array first.
 *
 * Under stream capture (hipStreamIsCapturing): the epoch is an argument of the launch, and a
 * recorded launch runs again on every replay, so a recorded call always consists of the fill
 * kernel followed by the sampler under epoch 1 -- two kernel nodes, right on every replay
 * whatever ran in between.  The address of the array is looked up at the first call on a
 * device, which must therefore come before the capture: call
 * gs_sample_uniform_fused_static_init() (idempotent, allocates nothing) on the device first;
 * a first call under capture is refused with GS_ERR_UNSUPPORTED.  A mailbox ticket recorded
 * into a graph is posted again on every replay.
 *
 * When a call reports a total of -1 (a tile's bounded wait ran out), the error word stays in
 * the library's array, which the caller cannot reach: call
 * gs_sample_uniform_fused_static_reset() and the next call starts from a zero-filled array.
 * gs_sample_uniform_fused_static_debug_raise(stream) raises that error word from the host
 * (test suites: every kernel still runs to its end). */
#define GS_FUSED_STATIC_MAX_COLUMNS ((int64_t)1 << 22)
int gs_sample_uniform_fused_static_init(void);
int gs_sample_uniform_fused_static_reset(void);
int gs_sample_uniform_fused_static_debug_raise(void* stream);
int gs_sample_uniform_fused_static(const int64_t* indptr, int64_t num_cols, const void* indices,
                                   const void* column_ids, int id_bytes, int64_t S,
                                   int64_t fanout, int replace, uint64_t seed,
                                   const uint32_t* replay, const int64_t* replay_ptr,
                                   int64_t* sub_indptr, void* sub_indices,
                                   int64_t* select_index, void* coo_col, int64_t capacity,
                                   gs_mailbox* mailbox, int64_t mailbox_ticket, void* stream);

/* Self-test of the one-launch kernels' bounded wait (no counterpart in the reference; for
 * test suites, not for the sampling path).  Runs the chained scan of gs_sample_uniform_fused
 * over `tiles` tiles that each contribute 1, on `state` under `epoch`, with tile
 * `missing_tile` left out of the launch (-1: none) and a tile giving up after `spin_limit`
 * polls of a predecessor's status word.  Every workgroup runs to its end whatever is
 * missing.  *total (device) receives `tiles` when every tile was there, -1 when a wait ran
 * out; the error word a give-up raises stays in `state` (every later one-launch call on it
 * reports -1) until the caller zero-fills it. */
int gs_selftest_lookback(void* state, size_t state_bytes, uint32_t epoch, int64_t tiles,
                         int64_t missing_tile, int spin_limit, int64_t* total, void* stream);

/* fanout == 1 with replacement through the fused entry: exactly one slot per
 * column, -1 in both outputs for an empty column; sub_indptr = 0..S.  Replaces
 * impl::fusion::FusedCSCColSlicingSamplingOneKeepDimCUDA
 * (src/cuda/fusion/slice_sampling.cu:157).  replay: one draw per column. */
int gs_sample_one_keepdim(const int64_t* indptr, int64_t num_cols, const void* indices,
                          const void* column_ids, int id_bytes, int64_t S, uint64_t seed,
                          const uint32_t* replay,
                          int64_t* sub_indptr, void* sub_indices, int64_t* select_index,
                          void* stream);

/* ------------------------------------------------------------------------- */
/* Weighted neighbour sampling without replacement (A-Res): replaces          */
/* impl::CSCColSamplingProbsCUDA (src/cuda/sampling_probs.cu:268).  Key of     */
/* edge i = log2(u_i)/w_i (monotone in the reference's u^(1/w)), w <= 0 ->     */
/* -inf; the fanout largest keys are emitted in descending key order, ties by  */
/* lower position.  probs is indexed by edge position of the input CSC.        */
/* sub_indptr comes from gs_sample_count(replace = 0).  replay_ptr: a row with */
/* deg > fanout consumes deg draws, any other row none.                        */
/* ------------------------------------------------------------------------- */
size_t gs_sample_weighted_workspace_bytes(int64_t S, int64_t fanout);

int gs_sample_weighted_fill(const int64_t* indptr, int64_t num_cols, const void* indices,
                            const float* probs, const void* column_ids, int id_bytes, int64_t S,
                            int64_t fanout,
                            uint64_t seed, const uint32_t* replay, const int64_t* replay_ptr,
                            const int64_t* sub_indptr, void* sub_indices, int64_t* select_index,
                            void* coo_col, void* workspace, size_t workspace_bytes, void* stream);

/* Weighted neighbour sampling WITH replacement (inverse CDF): replaces
 * _CSRRowWiseSampleReplaceKernel (src/cuda/sampling_probs.cu:112-183).  A column with
 * deg > 0 gets fanout picks.  cdf = inclusive prefix of max(probs, 0) over the column's
 * edges, built 64 edges at a time by a Kogge-Stone scan (x[i] += x[i-d], d = 1, 2, .., 32)
 * whose running total enters the next chunk through its first element.  A column longer
 * than 2048 edges is cut into blocks of 2048: every block is scanned from zero, the blocks'
 * totals are added up in order, and entry i of block b is (sum of the totals before b) +
 * (its value inside the block).  Pick j of row r: u = ((draw(r, j) >> 8) + 1) * 2^-24,
 * rand = u * cdf[deg-1], item = first position with cdf > rand (binary search for the
 * block whose last entry exceeds rand, then inside it), clamped to deg-1.  sub_indptr
 * comes from gs_sample_count(replace = 1).
 * cdf_ptr[S+1]: offsets of the columns' edges inside the scratch `cdf` (cdf_ptr[S] floats):
 * indptr itself when column_ids == NULL, else the sub_indptr of gs_slice_count.
 * replay: S * fanout draws, [r * fanout + j]. */
int gs_sample_weighted_replace(const int64_t* indptr, int64_t num_cols, const void* indices,
                               const float* probs, const void* column_ids, int id_bytes, int64_t S,
                               int64_t fanout, uint64_t seed, const uint32_t* replay,
                               const int64_t* sub_indptr, const int64_t* cdf_ptr, float* cdf,
                               void* sub_indices, int64_t* select_index, void* coo_col,
                               void* stream);

/* ------------------------------------------------------------------------- */
/* List sampling: replaces impl::ListSamplingCUDA (src/cuda/list_sampling.cu:79) */
/* and impl::ListSamplingProbsCUDA (src/cuda/list_sampling_probs.cu:185).       */
/* The caller handles n <= k without replacement (identity) itself.            */
/* out_index[k] int64, out_data[k] id_bytes wide.                              */
/* ------------------------------------------------------------------------- */
size_t gs_list_sample_workspace_bytes(int64_t n, int64_t k);

/* replay: k draws with replacement, n-k draws (idx = k..n-1) without. */
int gs_list_sample_uniform(const void* data, int id_bytes, int64_t n, int64_t k, int replace,
                           uint64_t seed, const uint32_t* replay, void* out_data,
                           int64_t* out_index, void* workspace, size_t workspace_bytes,
                           void* stream);

/* A-Res top-k over one list (without replacement); replay: n draws. */
int gs_list_sample_weighted(const void* data, int id_bytes, const float* probs, int64_t n,
                            int64_t k, uint64_t seed, const uint32_t* replay, void* out_data,
                            int64_t* out_index, void* workspace, size_t workspace_bytes,
                            void* stream);

/* ------------------------------------------------------------------------- */
/* Unique / relabel: replaces impl::TensorUniqueCUDA and impl::RelabelCUDA     */
/* (src/cuda/unique_reindex.cu:174,179).                                      */
/* ------------------------------------------------------------------------- */
typedef struct gs_span {
  const void* ptr; /* device pointer to ids (id_bytes wide) */
  int64_t n;       /* number of ids */
} gs_span;

#define GS_MAX_SPANS 4

size_t gs_unique_workspace_bytes(int64_t num_mapping_items);

/* frontier = distinct ids of concat(mapping[0..n_mapping)) in first-occurrence
 * order (unique_reindex.cu:106-144); *num_unique (device scalar) = its length.
 * For every query q: query_out[q][i] = rank of query[q].ptr[i] in frontier, -1
 * when absent (unique_reindex.cu:154-172).  n_query may be 0 (plain unique).
 * frontier needs capacity sum(mapping[].n).  Ids must not be -1. */
int gs_unique_relabel(const gs_span* mapping, int n_mapping, const gs_span* query,
                      void* const* query_out, int n_query, int id_bytes, void* frontier,
                      int64_t* num_unique, void* workspace, size_t workspace_bytes,
                      void* stream);

/* The same, for callers that keep the host out of the loop:
 *   - mailbox (NULL = none): the kernel that learns the number of unique ids also
 *     posts it there (see gs_mailbox).  *num_unique and the mailbox read -1 if the
 *     compaction gave up waiting on another tile.
 *   - last_span_len (NULL = none): device address of the true length of the LAST
 *     mapping span, for a span whose length an earlier kernel on the stream
 *     produced and the host has not read (the sampled ids of
 *     gs_sample_uniform_fused, length sub_indptr[S]).  mapping[n_mapping-1].n is
 *     then only its capacity; launches, table and frontier are sized for it and the
 *     kernels read the length themselves (a negative value counts as 0).  The only
 *     query allowed in this mode is that same span, cut to the same length. */
int gs_unique_relabel_notify(const gs_span* mapping, int n_mapping, const gs_span* query,
                             void* const* query_out, int n_query, int id_bytes, void* frontier,
                             int64_t* num_unique, void* workspace, size_t workspace_bytes,
                             const int64_t* last_span_len, gs_mailbox* mailbox,
                             int64_t mailbox_ticket, void* stream);

/* The relabel that follows a sampler, on a hash table that outlives the calls (no
 * counterpart in the reference, which allocates and fills a fresh table per call,
 * src/cuda/unique_reindex.cu:86-88).  Same result as gs_unique_relabel_notify with the
 * mapping (seed_keys[0..S), sampled[0..*sampled_len)) and `sampled` as the one query:
 * frontier (capacity S + capacity), out_ids (capacity), *num_unique and the mailbox.
 *   table: gs_relabel_table_bytes(max_items, id_bytes) bytes, 256-byte aligned, prepared
 *     once with gs_relabel_table_init; max_items >= S + capacity of every call.  The last
 *     kernel of a call empties exactly the slots the call used, so no call starts by
 *     clearing the table and its size costs nothing per call (it is kept at a load of at
 *     most 1/8).  A call that failed half-way (*num_unique == -1) leaves it undefined:
 *     prepare it again.  One call at a time per table.
 *   sampled_len: device address of the true number of sampled ids (sub_indptr + S of the
 *     sampler); `capacity` only bounds it.
 *   offsets_copy: NULL, or S + 1 slots that receive a copy of the sampler's offsets
 *     (sampled_len[-S .. 0]): Graph::Relabel returns `indptr.clone()` (src/graph.cc:807),
 *     and the copy made here costs no launch of its own.
 *   workspace: gs_relabel_sampled_workspace_bytes(S + capacity); state / epoch: as for
 *     gs_sample_uniform_fused, gs_relabel_sampled_state_bytes(S + capacity) bytes (the
 *     sampler's state buffer may be shared when large enough, with a fresh epoch). */
size_t gs_relabel_table_bytes(int64_t max_items, int id_bytes);
int gs_relabel_table_init(void* table, size_t table_bytes, int id_bytes, void* stream);
size_t gs_relabel_sampled_workspace_bytes(int64_t num_items);
size_t gs_relabel_sampled_state_bytes(int64_t num_items);
int gs_relabel_sampled(const void* seed_keys, int64_t S, const void* sampled, int64_t capacity,
                       const int64_t* sampled_len, int id_bytes, void* table, size_t table_bytes,
                       void* frontier, void* out_ids, int64_t* num_unique,
                       int64_t* offsets_copy, void* workspace,
                       size_t workspace_bytes, void* state, size_t state_bytes, uint32_t epoch,
                       gs_mailbox* mailbox, int64_t mailbox_ticket, void* stream);

/* gs_relabel_sampled for 64-bit ids whose values fit 32 bits (node ids of any graph below
 * 4.29 G nodes): the table is used with the one-word slots of 32-bit ids -- one
 * compare-and-swap per insert instead of compare-and-swap, read and minimum -- while ids,
 * frontier and out_ids stay 64-bit.  The table must have been prepared with
 * gs_relabel_table_init(..., id_bytes = 4) (a buffer sized by gs_relabel_table_bytes(..., 8)
 * is large enough for both layouts).  If a key does not fit, *num_unique and the mailbox read
 * -2, nothing else written is valid, and the error word of `state` stays set: zero `state`,
 * prepare the table again with id_bytes = 8 and call gs_relabel_sampled. */
int gs_relabel_sampled_narrow(const void* seed_keys, int64_t S, const void* sampled,
                              int64_t capacity, const int64_t* sampled_len, void* table,
                              size_t table_bytes, void* frontier, void* out_ids,
                              int64_t* num_unique, int64_t* offsets_copy, void* workspace,
                              size_t workspace_bytes, void* state, size_t state_bytes,
                              uint32_t epoch, gs_mailbox* mailbox, int64_t mailbox_ticket,
                              void* stream);

/* ------------------------------------------------------------------------- */
/* One GraphSAGE layer -- column slice + uniform sample, then relabel -- as TWO  */
/* launches that need no host read, so that a caller can queue all layers of a  */
/* minibatch back to back and wait once.  Replaces, for the loop of              */
/* examples/graphsage/batching.py:125-138, the pair                              */
/* impl::fusion::FusedCSCColSlicingSamplingCUDA (src/cuda/fusion/slice_sampling.cu:146) */
/* + impl::RelabelCUDA (src/cuda/unique_reindex.cu:179); results are those of    */
/* gs_sample_uniform_fused followed by gs_relabel_sampled, bit for bit.          */
/*                                                                               */
/* Sizes may live on the device: S_bound bounds the number of columns (launches  */
/* and buffers are sized for it), S_dev (NULL = S_bound is the number) is its    */
/* device address -- typically the num_unique of the previous layer, whose       */
/* frontier is this layer's column_ids.  A negative *S_dev counts as 0.          */
/*   table: gs_relabel_table_bytes(max S_bound + capacity, 4), prepared once with */
/*     gs_relabel_table_init(..., id_bytes = 4, ...): one-word slots.  64-bit ids */
/*     (id_bytes 8) must fit 32 bits; if one does not, *num_unique reads -2 (as   */
/*     gs_relabel_sampled_narrow).  gs_layer_sample fills it, gs_layer_relabel    */
/*     reads it and does NOT empty it: name it as `prev_table` (with that layer's */
/*     workspace and counts) in a later gs_layer_relabel on ANOTHER table, which  */
/*     empties it on the side, or call gs_layer_table_sweep.  Two tables used in  */
/*     turn keep every emptying off the critical path.                           */
/*   workspace: gs_layer_workspace_bytes(S_bound, fanout), shared by the layer's  */
/*     two calls and kept until the table has been emptied.                      */
/*   state / epoch: as for gs_sample_uniform_fused (zero-filled once, a fresh     */
/*     epoch per call); one buffer of max(gs_layer_sample_state_bytes,            */
/*     gs_layer_relabel_state_bytes) serves both calls and every layer, each call */
/*     with an epoch of its own: every word in it carries the epoch it was        */
/*     written under.                                                            */
/*   num_edges (device int64): written by gs_layer_sample (also at               */
/*     sub_indptr[S]), read by gs_layer_relabel.                                 */
/* ------------------------------------------------------------------------- */
size_t gs_layer_workspace_bytes(int64_t S_bound, int64_t fanout);
size_t gs_layer_sample_state_bytes(int64_t S_bound);
size_t gs_layer_relabel_state_bytes(int64_t S_bound, int64_t fanout);

/* First launch: the one-launch sampler (see gs_sample_uniform_fused: same draws, same
 * outputs; sub_indices holds `capacity` >= S_bound * fanout entries) which also enters
 * every seed (item r = seed r) and every sampled id (item S + e = output e) into `table`.
 * select_index (NULL, or `capacity` slots): position of every sample in `indices`.
 * edge_data / edge_ids / data_out (all NULL, or as for gs_sample_uniform_fused_data): the
 * edge data of the samples, data_[e_ids[select_index]] of src/graph.cc:544-557, written by
 * the lane that holds the position; output e of the layer keeps its place through
 * gs_layer_relabel, so data_out[e] belongs to out_ids[e]. */
int gs_layer_sample(const int64_t* indptr, int64_t num_cols, const void* indices,
                    const void* column_ids, int id_bytes, int64_t S_bound, const int64_t* S_dev,
                    int64_t fanout, int replace, uint64_t seed, const uint32_t* replay,
                    const int64_t* replay_ptr, int64_t* sub_indptr, void* sub_indices,
                    int64_t capacity, int64_t* num_edges, int64_t* select_index,
                    const float* edge_data, const int64_t* edge_ids, float* data_out, void* table,
                    size_t table_bytes, void* workspace, size_t workspace_bytes, void* state,
                    size_t state_bytes, uint32_t epoch, gs_mailbox* mailbox,
                    int64_t mailbox_ticket, void* stream);

/* Second launch: frontier (capacity S_bound + capacity; distinct ids of (seeds, sampled ids)
 * in first-occurrence order), *num_unique (device; -1 / -2 as gs_relabel_sampled_narrow),
 * out_ids[e] = rank of sampled id e, offsets_copy (NULL, or S + 1 slots that receive
 * sub_indptr[0..S]).  prev_*: NULL / 0, or the table, workspace and counts of an earlier
 * layer, whose slots are emptied here. */
int gs_layer_relabel(int id_bytes, int64_t S_bound, const int64_t* S_dev, int64_t capacity,
                     const int64_t* num_edges, const int64_t* sub_indptr, void* table,
                     size_t table_bytes, void* workspace, size_t workspace_bytes, void* frontier,
                     void* out_ids, int64_t* num_unique, int64_t* offsets_copy, void* state,
                     size_t state_bytes, uint32_t epoch, void* prev_table, size_t prev_table_bytes,
                     const void* prev_workspace, size_t prev_workspace_bytes, int64_t prev_S_bound,
                     const int64_t* prev_S_dev, int64_t prev_capacity,
                     const int64_t* prev_num_edges, gs_mailbox* mailbox, int64_t mailbox_ticket,
                     void* stream);

/* Empties the slots a layer filled (for the last layer of a run, which no later
 * gs_layer_relabel empties). */
int gs_layer_table_sweep(void* table, size_t table_bytes, const void* workspace,
                         size_t workspace_bytes, int64_t S_bound, const int64_t* S_dev,
                         int64_t capacity, const int64_t* num_edges, void* stream);

/* B relabels in one pass ("super-batch"): replaces impl::BatchCSRRelabelCUDA
 * (src/cuda/batch_relabel.cu:331).  Batch b owns seeds[seeds_ptr[b]..seeds_ptr[b+1])
 * and ids[ids_ptr[b]..ids_ptr[b+1]) (both *_ptr: device int64[num_batches+1]).
 * unique (capacity num_seeds+num_ids) = the batches' frontiers one after the other,
 * each the distinct values of (its seeds, then its ids) in first-occurrence order;
 * unique_ptr[num_batches+1] = their offsets; out_ids[j] = rank of ids[j] inside its own
 * batch's frontier; *num_unique (and the mailbox, when given) = total frontier length.
 * Ids must not be -1.  Workspace: gs_batch_relabel_workspace_bytes(num_seeds+num_ids). */
size_t gs_batch_relabel_workspace_bytes(int64_t num_items);
/* With GS_RELABEL_BINS, num_seeds and num_ids may be upper bounds (the sizes of the buffers):
 * the true counts are seeds_ptr[num_batches] and ids_ptr[num_batches] on the device, launches
 * and workspace (gs_batch_relabel_bins_workspace_bytes(bound, num_batches) suffices) are sized
 * by the bounds.  A caller can so queue a relabel behind a sampler whose edge count it has not
 * read.  A negative ids_ptr[num_batches] (the total a failed one-launch sampler leaves in its
 * offsets) makes every pass leave at once and *num_unique = -1. */
size_t gs_batch_relabel_bins_workspace_bytes(int64_t num_items, int64_t num_batches);
int gs_batch_csr_relabel(const void* seeds, const int64_t* seeds_ptr, const void* ids,
                         const int64_t* ids_ptr, int64_t num_batches, int64_t num_seeds,
                         int64_t num_ids, int id_bytes, void* unique, int64_t* unique_ptr,
                         void* out_ids, int64_t* num_unique, void* workspace,
                         size_t workspace_bytes, gs_mailbox* mailbox, int64_t mailbox_ticket,
                         void* stream);

/* The COO flavour: replaces impl::BatchCOORelabelCUDA (src/cuda/batch_relabel.cu:482).
 * Batch b owns seeds[seeds_ptr[b]..) and the edges [coo_ptr[b], coo_ptr[b+1]); its frontier
 * is the distinct values of (its seeds, then its coo_row) in first-occurrence order.
 * out_row[j] / out_col[j] = rank of coo_row[j] / coo_col[j] in the frontier of j's batch
 * (-1 for a column id that is not in it, batch_relabel.cu:352-374). */
int gs_batch_coo_relabel(const void* seeds, const int64_t* seeds_ptr, const void* coo_row,
                         const void* coo_col, const int64_t* coo_ptr, int64_t num_batches,
                         int64_t num_seeds, int64_t num_edges, int id_bytes, void* unique,
                         int64_t* unique_ptr, void* out_row, void* out_col, int64_t* num_unique,
                         void* workspace, size_t workspace_bytes, gs_mailbox* mailbox,
                         int64_t mailbox_ticket, void* stream);

/* ------------------------------------------------------------------------- */
/* Random walks: replace impl::fusion::FusedRandomWalkCUDA                    */
/* (src/cuda/fusion/random_walk.cu:52) and FusedMetapathRandomWalkCUDA         */
/* (src/cuda/fusion/metapath_random_walk.cu:49).  trace memory is              */
/* [length+1][n] (step-major); -1 is absorbing; one draw per live step;        */
/* replay layout [length][n].                                                  */
/* ------------------------------------------------------------------------- */
int gs_random_walk(const int64_t* indptr, int64_t num_nodes, const void* indices, int id_bytes,
                   const void* seeds, int64_t n, int64_t length, uint64_t seed, const uint32_t* replay,
                   void* trace, void* stream);

/* all_indptr / all_indices: device arrays of device pointers, one per relation
 * (src/hetero_graph.cc:33-50); all_num_nodes: device int64 array, the number of
 * columns of each relation; metapath: device int64[length] relation ids. */
int gs_metapath_walk(const int64_t* const* all_indptr, const void* const* all_indices,
                     const int64_t* all_num_nodes, int id_bytes, const int64_t* metapath,
                     int64_t length, const void* seeds, int64_t n, uint64_t seed,
                     const uint32_t* replay, void* trace, void* stream);

/* ------------------------------------------------------------------------- */
/* SDDMM: replaces impl::SDDMMCOO / impl::SDDMMCSC (src/cuda/sddmm.cu:280,263). */
/* out[eid, k] = op(lhs[sel_l, lhs_off[k]], rhs[sel_r, rhs_off[k]]) with         */
/* sel = src(0) / edge(1) / dst(2); dot reduces `reduce_size` trailing items.   */
/* lhs_off / rhs_off: device int64[out_len] broadcast offsets or NULL           */
/* (src/bcast.cc:24-75).  row / col / indices / nid_map are id_bytes wide.      */
/* ------------------------------------------------------------------------- */
int gs_sddmm_coo(int op, const void* row, const void* col, int id_bytes, const int64_t* e_ids,
                 int64_t E, const float* lhs, const float* rhs, float* out, int lhs_target,
                 int rhs_target, int64_t lhs_len, int64_t rhs_len, int64_t out_len,
                 int64_t reduce_size, const int64_t* lhs_off, const int64_t* rhs_off, void* stream);

/* CSC flavour: src = indices[e], dst = column owning e (through nid_map when
 * given, sddmm.cu:126-131). */
int gs_sddmm_csc(int op, const int64_t* indptr, const void* indices, int id_bytes,
                 const int64_t* e_ids, const void* nid_map, int64_t num_cols, int64_t E,
                 const float* lhs, const float* rhs, float* out, int lhs_target, int rhs_target,
                 int64_t lhs_len, int64_t rhs_len, int64_t out_len, int64_t reduce_size,
                 const int64_t* lhs_off, const int64_t* rhs_off, void* stream);

/* ------------------------------------------------------------------------- */
/* Segment ops: replace impl::CSCSumCUDA, COOSumCUDA, CSCNormalizeCUDA          */
/* (src/cuda/graph_ops.cu:92,122,184) and impl::fusion::COOEDivUSum             */
/* (src/cuda/fusion/edge_map_reduce.cu:10).  Node ids (n_ids, target, row, col) */
/* are id_bytes wide; e_ids are positions, always int64.                        */
/* ------------------------------------------------------------------------- */
/* workspace of gs_segment_sum / gs_segment_normalize; nnz = indptr[num_segments] */
size_t gs_segment_workspace_bytes(int64_t num_segments, int64_t nnz);

/* out[n_ids ? n_ids[s] : s] = sum over segment s of data[e_ids ? e_ids[e] : e]^powk.
 * Replaces impl::CSCSumCUDA (src/cuda/graph_ops.cu:92).  nnz: number of edges the offsets
 * cover (an upper bound will do).  A segment of at most 16 edges is summed in edge order; a
 * longer one by 1024-edge chunks of the edge array, four edges per lane, pieces across chunk
 * borders added in chunk order: a fixed order that depends on the layout only, but not the
 * sequential one. */
int gs_segment_sum(const int64_t* indptr, const int64_t* e_ids, const void* n_ids, int id_bytes,
                   const float* data, int64_t num_segments, int64_t nnz, int64_t powk, float* out,
                   void* workspace, size_t workspace_bytes, void* stream);

/* out[target[e]] += data[e_ids ? e_ids[e] : e]^powk  (out pre-zeroed by caller) */
int gs_coo_sum(const void* target, int id_bytes, const int64_t* e_ids, const float* data, int64_t E,
               int64_t powk, float* out, void* stream);

/* The same sums for callers that know how many targets there are (out has num_targets
 * entries; a target beyond is left out) and bring a workspace: with 4-byte ids, no e_ids,
 * at least 2^17 edges and at most 2^23 targets the edges are first brought together by runs
 * of targets (one partition pass of the sort behind gs_coo2csc) and then added up in LDS, a
 * run per workgroup, with no atomic to memory -- several times faster than gs_coo_sum when
 * most edges hit different targets.  Any other call is passed on to gs_coo_sum.  The order of
 * the additions is not fixed in either (impl::COOSumCUDA, src/cuda/graph_ops.cu:45-64, adds
 * with atomics too). */
size_t gs_coo_sum_workspace_bytes(int64_t E, int64_t num_targets);
int gs_coo_sum_binned(const void* target, int id_bytes, const int64_t* e_ids, const float* data,
                      int64_t E, int64_t powk, int64_t num_targets, float* out, void* workspace,
                      size_t workspace_bytes, void* stream);

/* out[d] = data[d] / sum of its segment, d = e_ids ? e_ids[e] : e */
int gs_segment_normalize(const int64_t* indptr, const int64_t* e_ids, const float* data,
                         int64_t num_segments, int64_t nnz, float* out, void* workspace,
                         size_t workspace_bytes, void* stream);

/* out_data[e] = data[e] / divisor[row[e]]; out_sum[col[e]] += out_data[e] */
int gs_e_div_u_sum(const void* row, const void* col, int id_bytes, const float* data,
                   const float* divisor, int64_t E, float* out_data, float* out_sum,
                   void* stream);

/* ------------------------------------------------------------------------- */
/* Row slicing: replaces impl::CSCRowSlicingCUDA and impl::COORowSlicingCUDA    */
/* (src/cuda/slicing.cu:528,768).  Kept ids are relabelled to their position    */
/* in row_ids.  Two phases: *_mark computes per-segment kept counts / a mask,   */
/* the caller reads the total, *_compact writes the survivors in order.  Ids    */
/* in and out are id_bytes wide; select_index is int64.                         */
/* ------------------------------------------------------------------------- */
size_t gs_row_slice_workspace_bytes(int64_t num_row_ids, int64_t nnz, int64_t num_cols);

/* out_indptr[0..num_cols] = exscan of kept edges per column; total in
 * out_indptr[num_cols]. */
int gs_row_slice_csc_mark(const int64_t* indptr, const void* indices, int id_bytes,
                          int64_t num_cols, int64_t nnz, const void* row_ids, int64_t num_row_ids,
                          int64_t* out_indptr, void* workspace, size_t workspace_bytes,
                          void* stream);

/* the workspace is the one the mark call filled */
int gs_row_slice_csc_compact(const int64_t* indptr, int64_t num_cols, int64_t nnz, int id_bytes,
                             void* out_indices, int64_t* select_index, void* coo_col,
                             void* workspace, size_t workspace_bytes, void* stream);

/* COO: keep edges whose key[e] is in ids.  *num_kept (device scalar). */
int gs_row_slice_coo_mark(const void* key, int id_bytes, int64_t E, const void* ids,
                          int64_t num_ids, int64_t* num_kept, void* workspace,
                          size_t workspace_bytes, void* stream);

int gs_row_slice_coo_compact(const void* other, int id_bytes, int64_t E, void* out_key,
                             void* out_other, int64_t* select_index, void* workspace,
                             size_t workspace_bytes, void* stream);

/* Column slice and row slice in one pass (induced subgraph): replaces
 * impl::fusion::CSCColRowSlicingCUDA and BatchCSCColRowSlicingCUDA
 * (src/cuda/fusion/column_row_slicing.cu:213,356).  Of the columns column_ids, keep the
 * edges whose row is in row_ids; the column slice itself is never written.
 *   sub_indptr, D: offsets and total of the plain column slice, from gs_slice_count.
 *   num_batches == 0: kept rows are renamed to their position in row_ids (:133-141).
 *   num_batches  > 0: columns and row ids are cut into batches at col_batch_ptr /
 *     row_batch_ptr (device int64[num_batches+1]); a column of batch b keeps the rows found
 *     in batch b's ids, under the key id + b*encoding_size, and rows keep their id (:272).
 * mark: out_indptr[S+1] = offsets of the result, total in out_indptr[S].
 * compact (same workspace): out_indices; select_index = position in the virtual column
 * slice (what the reference returns, :204-209); parent_index = position in the parent's
 * indices (what edge data has to be gathered with).  Either index array may be NULL. */
size_t gs_col_row_slice_workspace_bytes(int64_t num_row_ids, int64_t D);
int gs_col_row_slice_mark(const int64_t* indptr, int64_t num_cols, const void* indices,
                          int id_bytes, const void* column_ids, int64_t S,
                          const int64_t* sub_indptr, int64_t D, const void* row_ids,
                          int64_t num_row_ids, const int64_t* col_batch_ptr,
                          const int64_t* row_batch_ptr, int64_t num_batches,
                          int64_t encoding_size, int64_t* out_indptr, void* workspace,
                          size_t workspace_bytes, void* stream);
int gs_col_row_slice_compact(int64_t D, int id_bytes, void* out_indices, int64_t* select_index,
                             int64_t* parent_index, void* workspace, size_t workspace_bytes,
                             void* stream);

/* Membership filter of a COO that keeps global ids: replaces
 * impl::COORowSlicingGlobalIdCUDA, BatchCOOSlicingCUDA (src/cuda/batch_slicing.cu:325,232)
 * and BatchCOORowSlicingCUDA (src/cuda/slicing.cu:774).  Edge e survives when key[e] is
 * among `ids`; with num_batches > 0 the edges are cut into batches at key_batch_ptr and
 * the ids at ids_batch_ptr (device int64[num_batches+1]) and an edge is looked up among
 * the ids of its own batch (ids below 2^44).  mark: *num_kept (device scalar).  compact
 * (same workspace, gs_row_slice_workspace_bytes(num_ids, E, 0)): out_row / out_col = the
 * surviving edges in order, select_index (may be NULL) their positions, out_batch_ptr (may
 * be NULL) the batch offsets of the result.  When no edge survives the outputs are empty
 * and may be NULL. */
int gs_coo_filter_mark(const void* key, int id_bytes, int64_t E, const int64_t* key_batch_ptr,
                       const void* ids, int64_t num_ids, const int64_t* ids_batch_ptr,
                       int64_t num_batches, int64_t* num_kept, void* workspace,
                       size_t workspace_bytes, void* stream);
int gs_coo_filter_compact(const void* row, const void* col, int id_bytes, int64_t E,
                          const int64_t* key_batch_ptr, int64_t num_batches, void* out_row,
                          void* out_col, int64_t* select_index, int64_t* out_batch_ptr,
                          void* workspace, size_t workspace_bytes, void* stream);

/* out[i] = position of keys[i] in data, -1 when absent (the last position when data holds
 * a value twice): replaces impl::IndexHashMapInsertCUDA + IndexHashMapSearchCUDA
 * (src/cuda/index_search.cu:83,116; src/tensor_ops.cc:24-33).  out is id_bytes wide. */
size_t gs_index_search_workspace_bytes(int64_t n);
int gs_index_search(const void* data, int64_t n, const void* keys, int64_t m, int id_bytes,
                    void* out, void* workspace, size_t workspace_bytes, void* stream);

/* ------------------------------------------------------------------------- */
/* The rows of a column slice that a layer-wise sampler keeps, as the block's   */
/* values: what examples/ladies/ladies_raw.py:15-22 reaches through              */
/*   nodes = unique(cat(seeds, picked)); U[nodes, :].divide(prob[nodes], 1)      */
/* (a CSR of all of U, src/graph.cc:258-283 -> impl::CSCColSlicingCUDA,          */
/* src/cuda/graph_ops.cu division by row, then the CSC of the result,            */
/* src/graph.cc:585-644) without sorting the edges that are not kept.            */
/* ------------------------------------------------------------------------- */
/* out = the distinct values of a[na] and b[nb] in increasing order (torch.unique of their
 * concatenation, for ids >= 0), *count (device) = how many; out has room for na + nb.
 * 1 <= na + nb <= gs_sorted_union_max(id_bytes) (8192 / 4096 for 4- / 8-byte ids: one
 * workgroup sorts them in LDS). */
int64_t gs_sorted_union_max(int id_bytes);
int gs_sorted_union(const void* a, int64_t na, const void* b, int64_t nb, int id_bytes, void* out,
                    int64_t* count, void* stream);
/* Of the COO (row, col)[E], the edges whose row is among nodes[*num_nodes] (sorted, distinct,
 * at most max_nodes <= gs_sorted_union_max: the output of gs_sorted_union with its count
 * still on the device), in edge order: kept_key = col << bits | position of the row in
 * nodes, with bits = the smallest b that has 2^b >= max_nodes (the caller makes sure
 * num_cols << bits fits the id type), and kept_pos = the edge's position.  Both have room
 * for E entries.  totals (device int64[2]) = {*num_nodes, number of kept edges}; the number of
 * kept edges also goes to the mailbox (may be NULL). */
size_t gs_coo_pick_rows_workspace_bytes(int64_t E);
int gs_coo_pick_rows(const void* row, const void* col, int id_bytes, int64_t E, const void* nodes,
                     const int64_t* num_nodes, int64_t max_nodes, void* kept_key, void* kept_pos,
                     int64_t* totals, gs_mailbox* mailbox, int64_t ticket, void* workspace,
                     size_t workspace_bytes, void* stream);
/* The block of the kept edges (kept_key / kept_pos [kept] as gs_coo_pick_rows leaves them for a
 * COO whose edges come by column, with the same max_nodes): inside every column the edges are
 * put in the order of their rows (ties: of their positions) -- the order of a stable sort of
 * all kept edges by kept_key, done column by column -- and leave as out_row = their row
 * ids and out_value = data[pos] / divisor[row] (data NULL: ones; divisor is indexed by row id);
 * out_indptr[num_cols + 1] = the offsets of the columns.  Workspace (the list of the columns
 * with more than 256 kept edges): gs_coo_block_values_workspace_bytes(kept). */
size_t gs_coo_block_values_workspace_bytes(int64_t kept);
int gs_coo_block_values(const void* kept_key, const void* kept_pos, int64_t kept, int64_t max_nodes,
                        const void* row, int id_bytes, const float* data, const float* divisor,
                        int64_t num_cols, void* out_row, float* out_value, int64_t* out_indptr,
                        void* workspace, size_t workspace_bytes, void* stream);

/* ------------------------------------------------------------------------- */
/* Format conversion: replaces impl::CSC2COOCUDA and impl::COO2CSCCUDA          */
/* (src/cuda/format_transform.cu:35,135).                                      */
/* ------------------------------------------------------------------------- */
/* col[e] = column owning edge e (id_bytes wide) */
int gs_csc2coo(const int64_t* indptr, int64_t num_cols, int64_t nnz, void* col, int id_bytes,
               void* stream);

/* Doubly-compressed CSC (only the columns that own an edge are stored; ids[c] names stored
 * column c).  gs_dcsc2coo: col[e] = ids[column owning e], replaces impl::DCSC2COOCUDA
 * (src/cuda/format_transform.cu:48).  gs_csc_compress: CSC -> DCSC, the second half of
 * impl::COO2DCSCCUDA (src/cuda/format_transform.cu:172-203; the first half, the sort, is
 * gs_coo2csc): val_ids (capacity num_cols) = the non-empty columns in order, out_indptr
 * (capacity num_cols + 1) = their offsets, *num_valid (device scalar) = how many. */
int gs_dcsc2coo(const int64_t* indptr, int64_t num_cols, int64_t nnz, const void* ids, void* col,
                int id_bytes, void* stream);
size_t gs_csc_compress_workspace_bytes(int64_t num_cols);
int gs_csc_compress(const int64_t* indptr, int64_t num_cols, int id_bytes, void* val_ids,
                    int64_t* out_indptr, int64_t* num_valid, void* workspace,
                    size_t workspace_bytes, void* stream);

size_t gs_coo2csc_workspace_bytes(int64_t E, int64_t num_keys);

/* Stable counting sort of (key -> value), both id_bytes wide: indptr[num_keys+1],
 * out_value[E], perm[E] (int64; = stable argsort of key, the reference's
 * sort_index).  sorted != 0: only indptr is computed (out_value / perm
 * untouched, may be NULL).  indptr NULL (unsorted keys only): the sort alone, for keys with
 * no offsets to build (num_keys then only bounds the keys: the sort runs over its bits). */
int gs_coo2csc(const void* key, const void* value, int id_bytes, int64_t E, int64_t num_keys,
               int sorted, int64_t* indptr, void* out_value, int64_t* perm, void* workspace,
               size_t workspace_bytes, void* stream);

/* Offsets of a batched CSC cut into its batches: replaces
 * impl::SplitIndptrByOffsetCUDA / SplitIndptrBySizeCUDA (src/cuda/batch_split.cu:101,96).
 * offsets: device int64[num_batches+1], column ranges of the batches; out (length
 * total = offsets[num_batches] - offsets[0] + num_batches): batch b's
 * offsets[b+1]-offsets[b]+1 entries, re-based to start at 0, one batch after the other. */
int gs_indptr_split(const int64_t* indptr, const int64_t* offsets, int64_t num_batches,
                    int64_t total, int64_t* out, void* stream);
/* The same launch also leaves cuts[b] = indptr[offsets[b]], b = 0..num_batches (device int64,
 * may be NULL): where every batch's edges start, the third result of the GetBatchCSC call in
 * the reference's super-batch example (examples/graphsage/batching.py:67), without a separate
 * indexing launch. */
int gs_indptr_split_cuts(const int64_t* indptr, const int64_t* offsets, int64_t num_batches,
                         int64_t total, int64_t* out, int64_t* cuts, void* stream);

/* ------------------------------------------------------------------------- */
/* Super-batch plumbing.  A batched array is a flat array plus device int64     */
/* offsets [num_batches+1].                                                    */
/* ------------------------------------------------------------------------- */
/* out[i] = data[i] + batch(i) * encoding_size: replaces impl::BatchEncodeCUDA
 * (src/cuda/batch_coding.cu:74).  32-bit ids: num_batches * encoding_size must fit. */
int gs_batch_encode(const void* data, int id_bytes, int64_t n, const int64_t* ptr,
                    int64_t num_batches, int64_t encoding_size, void* out, void* stream);

/* out_data[i] = in[i] mod encoding_size, out_batch[i] = in[i] / encoding_size (either may be
 * NULL): replaces impl::BatchDecodeCUDA (src/cuda/batch_coding.cu:96). */
int gs_batch_decode(const void* in, int id_bytes, int64_t n, int64_t encoding_size, void* out_data,
                    void* out_batch, void* stream);

/* `in` encoded and sorted by batch: out_ptr[num_batches+1] = the batches' offsets, out_data
 * (may be NULL) the decoded ids: replaces impl::GetBatchOffsets (src/cuda/batch_coding.cu:110). */
int gs_batch_offsets(const void* in, int id_bytes, int64_t n, int64_t num_batches,
                     int64_t encoding_size, int64_t* out_ptr, void* out_data, void* stream);

/* Concatenation batch by batch: replaces impl::BatchConcatCUDA
 * (src/cuda/batch_concat.cu:117).  The *_host arguments are HOST arrays of num_segments
 * device pointers.  offsets: out_ptr[b] = sum over segments of their ptr[b] (total in
 * out_ptr[num_batches]).  fill: batch b of `out` = batch b of segment 0, then of segment
 * 1, ...; out_key[i] (may be NULL) = the batch of item i.  max_segment_len: the longest
 * segment (sizes the launch). */
#define GS_MAX_SEGMENTS 8
int gs_batch_concat_offsets(const int64_t* const* segment_ptrs_host, int num_segments,
                            int64_t num_batches, int64_t* out_ptr, void* stream);
int gs_batch_concat_fill(const void* const* segment_data_host,
                         const int64_t* const* segment_ptrs_host, int num_segments,
                         int64_t num_batches, int64_t max_segment_len, int id_bytes,
                         const int64_t* out_ptr, void* out, void* out_key, void* stream);

/* The inverse: replaces impl::BatchSplit2CUDA (src/cuda/batch_split2.cu:100).  Item i of
 * batch b (= data_key[i], or found from data_ptr when data_key is NULL) goes to the
 * segment whose share of batch b holds its local position, at out_ptrs[s][b] + ... */
int gs_batch_split(const void* data, const int64_t* data_ptr, const void* data_key, int id_bytes,
                   int64_t n, int64_t num_batches, void* const* out_data_host,
                   const int64_t* const* out_ptrs_host, int num_segments, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* GS_HIP_H_ */
