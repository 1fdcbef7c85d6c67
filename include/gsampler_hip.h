/*
 * gsampler_hip.h -- C ABI of the MI355X (gfx950) sampling kernels.
 *
 * Every entry point takes raw device pointers, element counts, a HIP stream
 * (passed as void*, it is a hipStream_t) and returns an int status
 * (GS_OK == 0).  No entry point allocates device memory: scratch space is a
 * caller-supplied workspace whose size the matching *_workspace_bytes()
 * function reports.  All ids, pointers-into-arrays and counts are int64,
 * all edge weights fp32, exactly as in the reference's tensors.
 *
 * Data-dependent output sizes use two phases: a *_count call fills a prefix
 * array on the device (its last element is the total), the caller reads that
 * total, allocates the outputs and calls *_fill.
 *
 * Random picks are a pure function of (seed, call_id, position of the column
 * / list element in its input array, draw index): Philox4x32-10 keyed by
 * seed + call_id * 0x9E3779B97F4A7C15 (mod 2^64), counter
 * (lo32(draw), hi32(draw), lo32(pos), hi32(pos)).  Launch geometry and
 * super-batching therefore never change a result.
 *
 * Each declaration cites the reference interface it stands in for
 * (paths relative to the gSampler source tree).
 */
#ifndef GSAMPLER_HIP_H_
#define GSAMPLER_HIP_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define GS_OK 0
#define GS_ERR_INVALID 1     /* bad argument (null pointer, negative size, ...) */
#define GS_ERR_HIP 2         /* a HIP runtime call failed; see gs_last_error() */
#define GS_ERR_WORKSPACE 3   /* workspace too small */
#define GS_ERR_UNSUPPORTED 4 /* valid request this build does not implement */

/* Sampling algorithm for uniform sampling without replacement. */
#define GS_ALGO_AUTO 0      /* Floyd when fanout <= 64, else reservoir */
#define GS_ALGO_RESERVOIR 1 /* the reference's Algorithm R in max-form */
#define GS_ALGO_FLOYD 2     /* Floyd's subset sampling, O(fanout) per column */

/* Sparse structure handed to the edge-wise operators. */
#define GS_FMT_COO 1        /* a = row[nnz], b = col[nnz] */
#define GS_FMT_COMPRESSED 2 /* a = indptr[num_major + 1], b = indices[nnz] */

/* Binary operators, reducers, operand targets and value types of the
 * edge-wise operators (names follow src/cuda/macro.h:7-33 of the reference). */
#define GS_OP_ADD 0
#define GS_OP_SUB 1
#define GS_OP_MUL 2
#define GS_OP_DIV 3
#define GS_OP_COPY_LHS 4
#define GS_OP_COPY_RHS 5
#define GS_OP_DOT 6
#define GS_REDUCE_SUM 0
#define GS_REDUCE_MAX 1
#define GS_REDUCE_MIN 2
#define GS_TARGET_U 0 /* source endpoint: row of a COO / indices of a compressed matrix */
#define GS_TARGET_E 1 /* the edge itself */
#define GS_TARGET_V 2 /* destination endpoint: column of a COO / owning segment */
#define GS_F32 0
#define GS_F64 1

typedef void* gs_stream_t;

/* Message of the last error raised on the calling thread ("" if none). */
const char* gs_last_error(void);
/* ABI revision; bumped whenever a signature changes. */
int gs_abi_version(void);

/* ------------------------------------------------------------------------
 * Per-kernel timing with HIP events on the launch stream (measurement aid; no
 * counterpart in the reference, which is profiled externally with Nsight).
 * While enabled every kernel launch is bracketed by two events; totals are
 * kept per kernel name.  gs_profile_count() waits for outstanding events.
 * ---------------------------------------------------------------------- */
void gs_profile_enable(int on);
void gs_profile_reset(void);
int gs_profile_count(void);
int gs_profile_get(int index, char* name, size_t name_bytes, long long* calls,
                   double* total_ms);

/* ------------------------------------------------------------------------
 * dst[0..n) = src[0..n).  dst may be pinned host memory that the device can
 * address: counts and batch pointer arrays that the host needs (to size the next
 * launch, to split results per batch) are sent this way, by a kernel in stream
 * order whose completion an event marks, instead of a memcpy call per array
 * (the reference reads them with blocking copies, e.g.
 * src/cuda/slicing.cu:146, src/cuda/batch/batch_split.cu:107-119).
 * ---------------------------------------------------------------------- */
int gs_copy_i64(const int64_t* src, int64_t n, int64_t* dst, gs_stream_t stream);

/* ------------------------------------------------------------------------
 * Exclusive prefix sum of n int64 values, in place allowed (in == out).
 * Stands in for cub_exclusiveSum, src/cuda/utils.h:18-28.
 * ---------------------------------------------------------------------- */
size_t gs_scan_workspace_bytes(int64_t n);
int gs_exclusive_scan_i64(const int64_t* in, int64_t* out, int64_t n,
                          void* workspace, size_t workspace_bytes,
                          gs_stream_t stream);

/* ------------------------------------------------------------------------
 * Per-column output count + prefix (count phase of slicing and sampling).
 *   column_ids == NULL : columns 0..num_items-1 of the CSC itself.
 *   fanout < 0         : whole column (slicing).
 *   replace            : count = degree == 0 ? 0 : fanout, else min(degree, fanout).
 * Column ids outside [0, num_cols) count as empty columns.
 * Writes sub_indptr[num_items + 1]; sub_indptr[num_items] is the edge total,
 * which the kernel that produces it also stores to *total_mirror when that is
 * given (a word of pinned host memory: the host then has the total as soon as
 * the stream reaches that point, without a copy of its own).
 * out_col_span (nullable, num_items words): where each requested column starts
 * in the matrix and how long it is, in one word (start in the low 40 bits, degree
 * in the 24 above; all ones when either does not fit).  The sampler fills below
 * take it as `col_span` and then read their columns' spans in a stream instead
 * of looking up every column's pointer pair a second time -- a 128-byte line of
 * `indptr` per column, a quarter of all lines a uniform fan-out-5 layer visits.
 * It is valid for the same indptr and column_ids only.
 * Stands in for the degree lambda + scan of
 *   src/cuda/slicing.cu:133-141, src/cuda/sampling.cu:112-124,
 *   src/cuda/fusion/slice_sampling.cu:111-124, src/cuda/sampling_probs.cu:201-216.
 * Workspace: gs_scan_workspace_bytes(num_items + 1).
 * ---------------------------------------------------------------------- */
int gs_csc_col_count(const int64_t* indptr, int64_t num_cols,
                     const int64_t* column_ids, int64_t num_items,
                     int64_t fanout, int replace, int64_t* sub_indptr,
                     int64_t* total_mirror, int64_t* out_col_span, void* workspace,
                     size_t workspace_bytes, gs_stream_t stream);

/* ------------------------------------------------------------------------
 * gs_csc_col_count for callers that cannot allocate device memory (code under
 * HIP graph capture, serving loops, harnesses that forbid hipMalloc): the same
 * result with the scan scratch in a fixed 512 KiB array inside the library
 * instead of a workspace, and no allocating call of any kind.  It has no
 * counterpart in the reference, whose scans allocate through the torch caching
 * allocator (src/cuda/utils.h:18-28).  At most 134 217 727 items; more is
 * rejected with GS_ERR_INVALID.  All calls on one GPU share that array: calls
 * that overlap in time on one GPU (different streams) race and must be
 * serialised by the caller.  The first call on a device looks up the array's
 * address (no allocation, but not capturable): make it before a capture.
 * ---------------------------------------------------------------------- */
int gs_csc_col_count_static(const int64_t* indptr, int64_t num_cols,
                            const int64_t* column_ids, int64_t num_items,
                            int64_t fanout, int replace, int64_t* sub_indptr,
                            gs_stream_t stream);

/* ------------------------------------------------------------------------
 * Column slicing A[:, column_ids] (fill phase).
 *   nnz = sub_indptr[num_items], as read back by the caller.
 *   out_coo_col   (nullable) : local column id of every output edge.
 *   out_indices              : global row id of every output edge.
 *   out_select               : position of the edge in `indices`.
 *   batch_ptr (nullable)     : [num_batches + 1] offsets into column_ids; with
 *     encode_stride > 0 the row id of an edge of batch b becomes
 *     id + b * encode_stride (src/cuda/batch/slicing.cu:25-27).
 * Stands in for OnIndptrSlicingCUDA (src/cuda/slicing.cu:169-181) and
 * BatchOnIndptrSlicingCUDA (src/cuda/batch/slicing.cu:100-120).
 * ---------------------------------------------------------------------- */
int gs_csc_col_slice_fill(const int64_t* indptr, int64_t num_cols,
                          const int64_t* indices, const int64_t* column_ids,
                          int64_t num_items, const int64_t* sub_indptr,
                          int64_t nnz, const int64_t* batch_ptr,
                          int64_t num_batches,
                          int64_t encode_stride, int64_t* out_coo_col,
                          int64_t* out_indices, int64_t* out_select,
                          gs_stream_t stream);

/* Edge data of a column slice: out_values[sub_indptr[i] + k] = values[indptr[c_i] + k]
 * for values of 4 or 8 bytes aligned with the parent's edges (c_i = column_ids[i],
 * or i when column_ids is NULL).  The same result as gathering values by the
 * edge positions that gs_csc_col_slice_fill wrote (data_index(edata, edge_index),
 * python/gs/matrix_api/matrix.py:19-23 behind the slice of :103) without reading
 * those positions back. */
int gs_csc_col_slice_values(const int64_t* indptr, const int64_t* column_ids,
                            int64_t num_items, const int64_t* sub_indptr, int64_t nnz,
                            const void* values, int64_t value_bytes, void* out_values,
                            gs_stream_t stream);

/* ------------------------------------------------------------------------
 * Uniform per-column sampling (fill phase), optionally fused with the column
 * slice (column_ids != NULL).  sub_indptr comes from gs_csc_col_count with
 * the same fanout / replace.  Columns with degree <= fanout are copied in
 * their original order (no replace).  `algo` is one of GS_ALGO_*.  `indices`
 * may be NULL, meaning "the edge position itself" (out_indices then repeats
 * out_select).  col_span (nullable) is what gs_csc_col_count left in
 * out_col_span for the same indptr and column_ids: with it neither of the two is
 * read (except for columns whose span did not fit a word); results are the same.
 * out_coo_col (nullable) receives the column of every edge: the
 * position i of its column among the call's columns or, when col_batch_ptr
 * (num_col_batches + 1 offsets that cut the call's columns into batches, nullable)
 * is given, i - col_batch_ptr[batch of i], the column's position inside its
 * batch.  That is the label the column gets in the batch's block whenever the
 * batch's seeds are distinct, so gs_unique_relabel / gs_unique_fill_relabel with
 * out_col_prefilled leave such labels as they are and only rewrite the batches
 * whose seeds repeat (the super-batched samplers of the reference relabel every
 * edge's column, src/cuda/batch/batch_relabel.cu:379-466).
 * Stands in for CSCColSamplingCUDA (src/cuda/sampling.cu:161-172) and
 * FusedCSCColSlicingSamplingCUDA (src/cuda/fusion/slice_sampling.cu:164-177).
 * ---------------------------------------------------------------------- */
int gs_csc_col_sample_uniform_fill(const int64_t* indptr, int64_t num_cols,
                                   const int64_t* indices,
                                   const int64_t* column_ids, int64_t num_items,
                                   int64_t fanout, int replace, int algo,
                                   uint64_t seed, uint64_t call_id,
                                   const int64_t* sub_indptr, const int64_t* col_span,
                                   int64_t* out_coo_col, int64_t* out_indices,
                                   int64_t* out_select,
                                   const int64_t* col_batch_ptr,
                                   int64_t num_col_batches, gs_stream_t stream);

/* The same with the row ids read from a 32-bit copy of `indices`
 * (indices32[e] == indices[e] for every edge, all ids < 2^31): identical
 * outputs (int64), half the bytes behind every random pick.  A matrix whose
 * row count allows it keeps such a copy beside the int64 array. */
int gs_csc_col_sample_uniform_fill_i32(const int64_t* indptr, int64_t num_cols,
                                       const int32_t* indices32,
                                       const int64_t* column_ids,
                                       int64_t num_items, int64_t fanout,
                                       int replace, int algo, uint64_t seed,
                                       uint64_t call_id,
                                       const int64_t* sub_indptr,
                                       const int64_t* col_span,
                                       int64_t* out_coo_col,
                                       int64_t* out_indices,
                                       int64_t* out_select,
                                       const int64_t* col_batch_ptr,
                                       int64_t num_col_batches,
                                       gs_stream_t stream);

/* ------------------------------------------------------------------------
 * Weighted per-column sampling (fill phase; counts come from
 * gs_csc_col_count).  probs[nnz] (fp32) is aligned with `indices`; indices may
 * be NULL, meaning "the edge position itself".
 *  without replacement (fanout <= 64): columns with degree <= fanout are copied
 *    whole and in order (zero weights included); otherwise the fanout edges
 *    with the smallest keys (-log2 u) / w, in ascending key order (ties: smaller
 *    edge offset; w <= 0: key +inf).  Stream: pos = column position, draw =
 *    edge offset.
 *  with replacement: integer CDF per column in cdf_scratch (uint64 per edge;
 *    column i uses cdf_scratch + cdf_offsets[i], or + indptr[column] when
 *    column_ids == NULL and cdf_offsets == NULL), pick j uses draw j.
 *  cdf != NULL (from gs_weight_cdf_build for the same indptr / indices / probs;
 *    probs may then be NULL, cdf_offsets / cdf_scratch are not used, and
 *    `indices` is only read when the CDF holds no row ids): every draw is
 *    a search in the column's entries of the CDF, O(fanout * log deg) per
 *    column instead of a pass over its weights.  Without replacement
 *    (fanout <= 64) this is successive weighted sampling: draw j takes a
 *    uniform point of the mass that is left and maps it past the intervals of
 *    the edges already taken, so a column costs exactly fanout searches.  The
 *    same distribution as the smallest-keys rule above, other picks; output in
 *    draw order; when fewer than fanout edges have positive (quantised)
 *    weight, zero-weight edges follow in index order.  Stream: pos = column
 *    position, draw = output slot.
 *  out_coo_col, col_batch_ptr, num_col_batches: as for the uniform sampler
 *    above (the column's position in the call, or inside its batch).
 *  col_span: as for the uniform sampler; read by the CDF form only.
 * Stands in for CSCColSamplingProbsCUDA (src/cuda/sampling_probs.cu:268-281).
 * ---------------------------------------------------------------------- */
/* Persistent packed CDF of a matrix's edge weights, the input of the fast
 * weighted sampler below: cdf[nnz + 1] 64-bit words.
 *   cdf[0]     = row_bits: how many low bits of an entry hold a row id (the
 *                bits that ids below num_rows need; 0 when indices == NULL or
 *                the ids need more than 32 bits: the sampler then reads the row
 *                ids from `indices`)
 *   cdf[e + 1] = share(e) << row_bits | indices[e]
 * share(e) = the part of the column's mass at or before edge e in units of
 * 2^-cb, cb = min(62, 64 - row_bits): floor(G(e) * 2^cb / T), with G the prefix
 * sums inside the column of the weights quantised to 31 bits against the
 * column's maximum (w <= 0 counts as 0) and T the column's total; 2^cb - 1 from
 * the last positive edge on; 0 throughout a column without positive weights.
 * Edge j of a column is drawn with probability (share(j) - share(j - 1)) /
 * (2^cb - 1).  Build it once per (matrix, weights): four passes over the edges.
 * No counterpart in the reference, whose sampler reads every weight of a
 * column on every call (src/cuda/sampling_probs.cu:25-110). */
size_t gs_weight_cdf_workspace_bytes(int64_t num_cols, int64_t nnz);
int gs_weight_cdf_build(const int64_t* indptr, int64_t num_cols,
                        const int64_t* indices, int64_t num_rows,
                        const float* probs, int64_t nnz, int64_t* cdf,
                        void* workspace, size_t workspace_bytes,
                        gs_stream_t stream);
int gs_csc_col_sample_weighted_fill(
    const int64_t* indptr, int64_t num_cols, const int64_t* indices,
    const float* probs, const int64_t* cdf, const int64_t* column_ids, int64_t num_items,
    int64_t fanout, int replace, uint64_t seed, uint64_t call_id,
    const int64_t* sub_indptr, const int64_t* col_span, const int64_t* cdf_offsets,
    void* cdf_scratch, int64_t* out_coo_col, int64_t* out_indices, int64_t* out_select,
    const int64_t* col_batch_ptr, int64_t num_col_batches, gs_stream_t stream);

/* Evaluates the key arithmetic on the device: out2[0] = -log2((r64>>12)+1)/2^52),
 * out2[1] = key of weight w at stream (seed, call_id, pos, draw).  Test hook. */
int gs_weighted_key_probe(uint64_t seed, uint64_t call_id, uint64_t pos,
                          uint64_t draw, float w, uint64_t r64, double* out2,
                          gs_stream_t stream);

/* ------------------------------------------------------------------------
 * Collective (list / layer-wise) sampling: picks positions of a list.
 *  gs_list_sample_uniform: K of n positions; n <= K without replacement gives
 *    0..n-1.  out_index holds min(K, n) (K with replacement) entries.
 *    ListSamplingCUDA, src/cuda/list_sampling.cu:70-73.
 *  gs_list_sample_weighted_{count,fill}: probs[n] fp32, optional
 *    range[num_segments + 1] (segments = mini-batches; NULL = one list).
 *    count writes out_range[num_segments + 1] (picks before each segment, last
 *    = total).  fill writes global positions: without replacement per segment
 *    the min(K, n_b) smallest keys in ascending key order (a segment with
 *    n_b <= K keeps its order); with replacement K picks through an integer
 *    CDF (stream pos = segment, draw = pick).  ListSamplingProbsCUDA
 *    (src/cuda/list_sampling_probs.cu:85-89), BatchListSamplingProbsCUDA
 *    (src/cuda/batch/list_sampling_probs.cu:102-107; the reference rejects
 *    replace there).
 * ---------------------------------------------------------------------- */
int gs_list_sample_uniform(int64_t n, int64_t num_picks, int replace, int algo,
                           uint64_t seed, uint64_t call_id, int64_t* out_index,
                           gs_stream_t stream);
size_t gs_list_sample_workspace_bytes(int64_t n, int64_t num_segments);
int gs_list_sample_weighted_count(const int64_t* range, int64_t n,
                                  int64_t num_segments, int64_t num_picks,
                                  int replace, int64_t* out_range,
                                  void* workspace, size_t workspace_bytes,
                                  gs_stream_t stream);
int gs_list_sample_weighted_fill(const float* probs, const int64_t* range,
                                 int64_t n, int64_t num_segments,
                                 int64_t num_picks, int replace, uint64_t seed,
                                 uint64_t call_id, const int64_t* out_range,
                                 int64_t total_picks, int64_t* out_index,
                                 void* workspace, size_t workspace_bytes,
                                 gs_stream_t stream);

/* ------------------------------------------------------------------------
 * Unique in first-occurrence order + relabel, for one batch or a super-batch.
 * For batch b the key sequence is
 *     seeds[seeds_ptr[b] : seeds_ptr[b+1]] ++ rows[rows_ptr[b] : rows_ptr[b+1]]
 * (seeds_ptr == rows_ptr == NULL means a single batch holding everything).
 *
 * count: finds the first occurrence of every key (state kept inside the
 *   workspace) and writes unique_ptr[num_batches + 1] (number of unique keys
 *   before each batch; the last element is the total U), and the same values
 *   to unique_ptr_mirror[num_batches + 1] when that is given (pinned host
 *   memory: the host then has the offsets without a copy of its own).
 * fill:  same arguments + the same workspace, untouched in between; writes
 *   out_unique[U].
 * relabel: after count, same workspace; out_row[num_rows_keys] = batch-local
 *   rank of every row key (nullable); out_col[num_rows_keys] = batch-local rank
 *   of seeds[c(e)] (nullable), c(e) being the position into `seeds` of edge e's
 *   column: edge_col[e], or -- for edges grouped by column, as a compressed
 *   matrix holds them -- the column c with col_indptr[c] <= e < col_indptr[c + 1]
 *   (col_indptr[num_seeds + 1], col_indptr[0] = 0; the coordinate form of such
 *   a matrix then need not exist: the reference expands it first,
 *   src/cuda/batch/batch_relabel.cu:480-498 takes coo_col).  Give one of the
 *   two, the other NULL.  May be called any number of times while the
 *   workspace is kept.  out_col_prefilled != 0 (with col_indptr): out_col already
 *   holds, for every edge, the place of its column inside its batch, as a sampler
 *   that was given col_batch_ptr writes it; those are the labels wherever the
 *   seeds of a batch are distinct, and only the edges of other batches are
 *   rewritten.
 * fill_relabel: fill and relabel in one launch (the two read the same state and
 *   write different outputs), for the caller that wants both at once, as
 *   BatchGraphRelabel does (src/cuda/batch/batch_relabel.cu:480-498 returns the
 *   frontier and both label arrays from one call).
 * Keys are any int64 values; one call takes at most 2^31 - 1 keys.  While all
 * keys of a call lie in [0, 2^32 - 2] a packed table entry holds the key itself;
 * when one does not (ids of a very large graph, ids encoded as id + batch *
 * num_rows, src/cuda/batch/slicing.cu:25-27), the kernels notice during the
 * partition pass and confirm every match of the 32-bit halves against the keys
 * themselves: same result, a few extra reads per repeated key.
 * Stands in for TensorUniqueCUDA / TensorRelabelCUDA
 * (src/cuda/unique_reindex.cu:174-199) and BatchCOORelabelCUDA
 * (src/cuda/batch/batch_relabel.cu:480-498).
 * ---------------------------------------------------------------------- */
size_t gs_unique_workspace_bytes(int64_t num_seeds, int64_t num_rows_keys,
                                 int64_t num_batches);
int gs_unique_count(const int64_t* seeds, const int64_t* seeds_ptr,
                    int64_t num_seeds, const int64_t* rows,
                    const int64_t* rows_ptr, int64_t num_rows_keys,
                    int64_t num_batches, int64_t* unique_ptr,
                    int64_t* unique_ptr_mirror, void* workspace,
                    size_t workspace_bytes, gs_stream_t stream);
int gs_unique_fill(const int64_t* seeds, const int64_t* seeds_ptr,
                   int64_t num_seeds, const int64_t* rows,
                   const int64_t* rows_ptr, int64_t num_rows_keys,
                   int64_t num_batches, const int64_t* unique_ptr,
                   int64_t* out_unique, void* workspace, size_t workspace_bytes,
                   gs_stream_t stream);
int gs_unique_relabel(const int64_t* seeds, const int64_t* seeds_ptr,
                      int64_t num_seeds, const int64_t* rows,
                      const int64_t* rows_ptr, int64_t num_rows_keys,
                      int64_t num_batches, const int64_t* edge_col,
                      const int64_t* col_indptr, int64_t* out_row, int64_t* out_col,
                      int out_col_prefilled, void* workspace, size_t workspace_bytes,
                      gs_stream_t stream);
int gs_unique_fill_relabel(const int64_t* seeds, const int64_t* seeds_ptr,
                           int64_t num_seeds, const int64_t* rows,
                           const int64_t* rows_ptr, int64_t num_rows_keys,
                           int64_t num_batches, const int64_t* unique_ptr,
                           int64_t* out_unique, const int64_t* edge_col,
                           const int64_t* col_indptr, int64_t* out_row, int64_t* out_col,
                           int out_col_prefilled, void* workspace, size_t workspace_bytes,
                           gs_stream_t stream);

/* ------------------------------------------------------------------------
 * out_first[r] = smallest position e with ids[e] == r, INT64_MAX when r does
 * not occur, for ids of a small dense range [0, num_ids) (ids outside it are
 * ignored).  The relabel step of a row-sliced matrix uses it: its rows are
 * positions in the list of picked rows, so first occurrences can be found per
 * picked row instead of per edge (no counterpart in the reference, which
 * hashes every edge, src/cuda/unique_reindex.cu:81-151).
 * ---------------------------------------------------------------------- */
int gs_first_position(const int64_t* ids, int64_t n, int64_t num_ids,
                      int64_t* out_first, gs_stream_t stream);

/* ------------------------------------------------------------------------
 * Frontier and labels for such a matrix in one launch.  Every edge of local
 * row l carries the key list_ids[l], so the unique of
 *     seeds ++ list_ids[row[e]] (e = 0, 1, ...)
 * in first-occurrence order -- what TensorUniqueCUDA / TensorRelabelCUDA
 * (src/cuda/unique_reindex.cu:174-199) compute over all edges -- is the unique
 * of seeds ++ (the listed ids in the order of first_pos, as gs_first_position
 * gives it; ids with first_pos == INT64_MAX are used by no edge and left out).
 *   out_frontier[num_seeds + num_ids]  the first out_count[0] entries are written
 *   out_count, out_count_mirror        nullable; device memory / pinned host memory
 *   out_list_label[num_ids]            label of list_ids[l] (0 for an unused id);
 *                                      the label of edge e's row is out_list_label[row[e]]
 *   out_seed_label[num_seeds]          label of seeds[c] (repeated seeds share one)
 * One work-group, all in LDS: num_seeds + num_ids <= GS_LIST_LABELS_MAX_KEYS,
 * more is refused with GS_ERR_INVALID (use gs_unique_count / gs_unique_relabel).
 * ---------------------------------------------------------------------- */
#define GS_LIST_LABELS_MAX_KEYS 2048
int gs_list_labels(const int64_t* seeds, int64_t num_seeds, const int64_t* list_ids,
                   const int64_t* first_pos, int64_t num_ids, int64_t* out_frontier,
                   int64_t* out_count, int64_t* out_count_mirror,
                   int64_t* out_list_label, int64_t* out_seed_label,
                   gs_stream_t stream);

/* ------------------------------------------------------------------------
 * Edge list -> compressed format, first half: stable sort of the edge
 * positions by their id on the axis to compress (`major`, ids in
 * [0, num_major)).  sorted_major receives the ids in order, perm the positions
 * (the e_ids of the new format); gs_sorted_to_indptr and two gathers by perm
 * finish the conversion.  COOSort / COO2CSCCUDA,
 * src/cuda/format_transform.cu:65-84,121-142.
 * Fewer than 2^32 edges with num_major <= 2^32 are sorted by the library's own
 * kernels: least significant digit first, 8 bits a pass over the bits that ids
 * below num_major need, 8 bytes per edge between the passes.  Tiles of a pass
 * learn the counts of the tiles before them from words those publish; a wait
 * for such a word is bounded, and a pass that reaches the bound goes on without
 * it (the outputs are then a permutation that is not fully sorted) and sets a
 * 32-bit flag in the workspace, at byte gs_coo_sort_flag_offset(nnz, num_major)
 * (-1: this call has no flag; rocPRIM's radix sort serves it).  The bound is
 * 65 536 polls of a word that another running work-group is about to write and
 * has never been reached; a caller that reads the flag after the call has
 * completed knows.
 * ---------------------------------------------------------------------- */
size_t gs_coo_sort_workspace_bytes(int64_t nnz, int64_t num_major);
int64_t gs_coo_sort_flag_offset(int64_t nnz, int64_t num_major);
int gs_coo_sort(const int64_t* major, int64_t nnz, int64_t num_major,
                int64_t* sorted_major, int64_t* perm, void* workspace,
                size_t workspace_bytes, gs_stream_t stream);

/* ------------------------------------------------------------------------
 * Row gather: out[i, :] = table[ids[i], :] for rows of `row_bytes` bytes of any
 * element type (node features of the sampled frontier, labels, edge data
 * behind an edge index).  `table` is device memory or pinned host memory that
 * the device can address; `ids` and `out` are device memory.  Replaces
 * IndexSelectCPUFromGPU (src/cuda/index_select_uvm.cu:9-50, pinned e_ids) and
 * the dgl.utils.gather_pinned_tensor_rows / data[index] calls of the callers
 * (python/gs/matrix_api/matrix.py:19-23,
 * examples/graphsage/graphsage_e2e.py:113-118).  An id outside [0, num_rows)
 * yields a row of zero bytes (the reference asserts on the device,
 * index_select_uvm.cu:16); when `bad_count` is not NULL it receives the number
 * of such ids.
 * ---------------------------------------------------------------------- */
int gs_gather_rows(const void* table, int64_t num_rows, int64_t row_bytes,
                   const int64_t* ids, int64_t n, void* out, int64_t* bad_count,
                   gs_stream_t stream);

/* ------------------------------------------------------------------------
 * Slicing across the compressed axis (row slicing of a CSC, A[picked, :]) and
 * coordinate-form slicing: keep the edges whose id in `ids[nnz]` belongs to
 * `picked[num_picked]`, relabel that id to its position in `picked` (smallest
 * position for a repeated id), keep the edge order.
 *  count: with indptr given writes out_indptr[num_major + 1] (all segments
 *    kept, out_indptr[num_major] = number of kept edges); out_total (nullable,
 *    device) receives the number of kept edges.
 *  fill:  same ids / workspace; out_minor[kept] = position in `picked`,
 *    out_select[kept] = edge position, out_major[kept] (nullable) =
 *    edge_major[e] if given else the segment of indptr holding e.
 * Ids are any int64 values (picked ids of 2^32 - 1 and above switch the
 * look-ups to confirming every match against the picked id, as in the unique
 * pass); at most 2^30 - 1 picked ids.  Stands in for OnIndicesSlicingCUDA
 * (src/cuda/slicing.cu:296-307) and COORowSlicingCUDA (src/cuda/slicing.cu:374-377).
 * ---------------------------------------------------------------------- */
size_t gs_minor_slice_workspace_bytes(int64_t nnz, int64_t num_picked);
int gs_minor_slice_count(const int64_t* ids, int64_t nnz, const int64_t* picked,
                         int64_t num_picked, const int64_t* indptr,
                         int64_t num_major, int64_t* out_indptr,
                         int64_t* out_total, void* workspace,
                         size_t workspace_bytes, gs_stream_t stream);
int gs_minor_slice_fill(const int64_t* ids, int64_t nnz, int64_t num_picked,
                        const int64_t* indptr, int64_t num_major,
                        const int64_t* edge_major, int64_t* out_major,
                        int64_t* out_minor, int64_t* out_select,
                        void* workspace, size_t workspace_bytes,
                        gs_stream_t stream);

/* ------------------------------------------------------------------------
 * Column slice and row slice in one: A[rows, cols] read straight from the
 * parent matrix, without writing the column slice A[:, cols] first.  Edge v of
 * that slice (sub_indptr = exclusive scan of the picked columns' degrees, e.g.
 * from gs_csc_col_count with fanout -1; slice_nnz = sub_indptr[num_cols_picked])
 * is tested like an edge of gs_minor_slice_*: kept when its row id is in
 * `rows`, relabelled to its position there, order kept.
 *  count: out_indptr[num_cols_picked + 1] and out_total (nullable, device).
 *    key_offset[num_cols_picked] (nullable) is added to the row ids of a column's
 *    edges before the test: the picked sets of the mini-batches of a super-batch
 *    are told apart as id + batch * stride on both sides.
 *    indices32 (nullable): the same row ids as `indices` in 32 bits; read instead
 *    of `indices` when given (half the bytes of the pass).
 *  fill: out_minor[kept] = position in `rows`, out_select[kept] = position of the
 *    edge in the PARENT's indices, out_major[kept] (nullable) = position of its
 *    column in `cols`.
 * Workspace: gs_minor_slice_workspace_bytes(slice_nnz, num_rows_picked), the
 * same buffer for both calls.  Stands in for CSCColRowSlicingCUDA and
 * BatchCSCColRowSlicingCUDA (src/cuda/fusion/column_row_slicing.cu:213-217,
 * 356-362; kernels :102-146, :220-264), whose select index addresses the
 * intermediate slice instead of the parent.
 * ---------------------------------------------------------------------- */
int gs_col_row_slice_count(const int64_t* indptr, const int64_t* indices,
                           const int32_t* indices32, const int64_t* cols,
                           const int64_t* key_offset, int64_t num_cols_picked,
                           const int64_t* sub_indptr, int64_t slice_nnz,
                           const int64_t* rows, int64_t num_rows_picked,
                           int64_t* out_indptr, int64_t* out_total, void* workspace,
                           size_t workspace_bytes, gs_stream_t stream);
int gs_col_row_slice_fill(const int64_t* indptr, const int64_t* indices, const int64_t* cols,
                          int64_t num_cols_picked, const int64_t* sub_indptr,
                          int64_t slice_nnz, int64_t num_rows_picked, int64_t* out_major,
                          int64_t* out_minor, int64_t* out_select, void* workspace,
                          size_t workspace_bytes, gs_stream_t stream);

/* ------------------------------------------------------------------------
 * Format conversion.
 *  gs_csc2coo: out_col[e] = column that owns edge position e
 *    (CSC2COOCUDA, src/cuda/format_transform.cu:24-46).
 *  gs_sorted_to_indptr: indptr[c] = #entries < c of a sorted id array, for
 *    c in [0, num_cols]; the COO -> CSC step after the sort by column
 *    (COO2CSCCUDA, src/cuda/format_transform.cu:109-142).  The sort itself is
 *    done by the caller.
 * ---------------------------------------------------------------------- */
int gs_csc2coo(const int64_t* indptr, int64_t num_cols, int64_t nnz,
               int64_t* out_col, gs_stream_t stream);
int gs_sorted_to_indptr(const int64_t* sorted_ids, int64_t nnz, int64_t num_cols,
                        int64_t* out_indptr, gs_stream_t stream);

/* ------------------------------------------------------------------------
 * Walks over CSC in-neighbours (a step moves from `curr` to one of the row ids
 * stored in column `curr`).  out_traces has (walk_length + 1) * num_seeds
 * entries in step-major order, out[step * num_seeds + walk]; step 0 is the
 * seed; -1 from a dead end onwards.
 *  gs_random_walk: uniform next hop.  FusedRandomWalkCUDA,
 *    src/cuda/fusion/random_walk.cu:49-70.
 *  gs_node2vec: second-order walk by rejection sampling with integer levels
 *    (return weight p, neighbour-of-previous weight q, otherwise 1); needs row
 *    ids sorted inside every column.  FusedNode2VecCUDA,
 *    src/cuda/fusion/node2vec.cu:139-162.
 *  gs_segment_sort_i64: sorts the ids of every segment (column).  key_bound:
 *    every key lies in [0, key_bound) (0 = not known).  For key_bound <= 2^32
 *    (the row ids of any matrix) the library's own kernels run: segments of up
 *    to 2048 ids are sorted in LDS in one read and one write, longer ones are
 *    first split by 11 bits of the ids at a time.  For a wider key_bound segment
 *    and key are radix-sorted as one word over the bits they use, and without
 *    one (or when the two do not fit 64 bits) a segmented radix sort over all 64
 *    bits runs (both rocPRIM).  keys_in and keys_out must not overlap.
 *    SortIndicesCUDA, src/cuda/sort_indices.cu:11-37.
 * ---------------------------------------------------------------------- */
int gs_random_walk(const int64_t* indptr, const int64_t* indices, int64_t num_cols,
                   const int64_t* seeds, int64_t num_seeds, int64_t walk_length,
                   uint64_t seed, uint64_t call_id, int64_t* out_traces,
                   gs_stream_t stream);
int gs_node2vec(const int64_t* indptr, const int64_t* indices, int64_t num_cols,
                const int64_t* seeds, int64_t num_seeds, int64_t walk_length,
                double p, double q, uint64_t seed, uint64_t call_id,
                int64_t* out_traces, gs_stream_t stream);
size_t gs_segment_sort_workspace_bytes(int64_t nnz, int64_t num_segments,
                                       int64_t key_bound);
int gs_segment_sort_i64(const int64_t* indptr, int64_t num_segments,
                        const int64_t* keys_in, int64_t* keys_out, int64_t nnz,
                        int64_t key_bound, void* workspace, size_t workspace_bytes,
                        gs_stream_t stream);

/* ------------------------------------------------------------------------
 * Super-batch bookkeeping.
 *  gs_decode_batch_ids: ids encoded as id + batch * stride -> out_batch =
 *    id / stride, out_orig = id - batch * stride (either output nullable).
 *    With gs_sorted_to_indptr over out_batch this is GetBatchOffsets,
 *    src/cuda/batch/encoding_decoding.cu:99-122.
 *  gs_split_indptr: batch b gets indptr[offset[b] .. offset[b+1]] rebased to
 *    start at 0, written at out[offset[b] + b ...]; out_len =
 *    offset[num_batches] - offset[0] + num_batches.  SplitIndptrByOffsetCUDA,
 *    src/cuda/batch/batch_split.cu:53-94.
 * ---------------------------------------------------------------------- */
int gs_decode_batch_ids(const int64_t* encoded, int64_t n, int64_t stride,
                        int64_t* out_orig, int64_t* out_batch,
                        gs_stream_t stream);
int gs_split_indptr(const int64_t* indptr, const int64_t* offset,
                    int64_t num_batches, int64_t out_len, int64_t* out,
                    gs_stream_t stream);
/* out_distinct[b] = 1 when the seeds of batch b are pairwise different, else 0,
 * read off the batch's frontier (unique keys in first-occurrence order, seeds
 * first, as gs_unique_fill writes it).  Tells whether the relabelled edges of a
 * batch are grouped by destination in seed order, i.e. whether the batch's
 * piece of gs_split_indptr is the block's compressed form.  No counterpart in
 * the reference, which hands DGL an edge list only
 * (python/gs/utils/to_dgl_block.py:19-23). */
int gs_batch_seeds_distinct(const int64_t* frontier, const int64_t* frontier_ptr,
                            const int64_t* seeds, const int64_t* seeds_ptr,
                            int64_t num_batches, int64_t* out_distinct,
                            gs_stream_t stream);

/* ------------------------------------------------------------------------
 * Edge-wise compute operators.  Common arguments: (format, a, b, num_major,
 * nnz) describe the structure; edge_map (nullable) maps an edge position to
 * the row of the edge-feature arrays (the e_ids of a converted format).
 * Feature arrays are row-major [n, len]; *_off (nullable) are broadcast offset
 * tables of out_len entries as computed by CalcBcastOff (src/bcast.cc:24-76).
 *
 * gs_sddmm: out[eid] = lhs[t_l] op rhs[t_r]            SDDMMCOO / SDDMMCSC,
 *   src/cuda/sddmm.cu:264-297.  fp32 or fp64.
 * gs_fused_u_op_v: two u-op-v SDDMMs in one sweep       FUSED_COO/CSC_U_OP_V,
 *   src/cuda/fusion/fused_coo_u_op_v.cu:109, fused_csc_u_op_v.cu:103.  Outputs
 *   are written through edge_map like gs_sddmm's (the reference's fused kernels
 *   write by edge position, which differs from its own SDDMM on a converted
 *   format).
 * gs_spmm: out[dst] = reduce(out[dst], op(u[src], e[eid])), fp32.  Outputs
 *   are accumulators: the caller zero-fills them (python/gs/ops/spmm.py:56).
 *   COO: u_target 0 reduces onto columns, 2 onto rows (atomics).  Compressed:
 *   reduces onto the segments of indptr; u_target is ignored.  num_out is the
 *   number of output rows.  workspace is optional (NULL / 0 is always valid):
 *   with gs_spmm_workspace_bytes(format, nnz, num_out) bytes a scalar COO sum
 *   accumulates per accelerator die and folds the copies at the end, which
 *   keeps its atomics inside one L2 each.
 *   SpMMCOO / SpMMCSC, src/cuda/spmm.cu:274-348.
 * gs_e_square_sum: out[dst] += sum e^2                  ESquareSumCSC/COO,
 *   src/cuda/fusion/fused_csc_e_square_sum.cu:110, fused_coo_e_square_sum.cu:13.
 * gs_e_div_u_sum: out[dst] += sum e / u[src]            EDivUSumCSC/COO,
 *   src/cuda/fusion/fused_csc_e_div_u_sum.cu:103, fused_coo_e_div_u_sum.cu:88.
 * ---------------------------------------------------------------------- */
int gs_sddmm(int format, const int64_t* a, const int64_t* b, int64_t num_major,
             int64_t nnz, const int64_t* edge_map, int op, int dtype,
             const void* lhs, const void* rhs, void* out, int lhs_target,
             int rhs_target, int64_t lhs_len, int64_t rhs_len, int64_t out_len,
             int64_t reduce_size, const int64_t* lhs_off, const int64_t* rhs_off,
             gs_stream_t stream);
int gs_fused_u_op_v(int format, const int64_t* a, const int64_t* b,
                    int64_t num_major, int64_t nnz, const int64_t* edge_map,
                    int op, int dtype,
                    const void* lhs1, const void* rhs1, void* out1,
                    const void* lhs2, const void* rhs2, void* out2,
                    int64_t lhs_len, int64_t rhs_len, int64_t out_len,
                    int64_t reduce_size, const int64_t* lhs_off,
                    const int64_t* rhs_off, gs_stream_t stream);
size_t gs_spmm_workspace_bytes(int format, int64_t nnz, int64_t num_out);
int gs_spmm(int format, const int64_t* a, const int64_t* b, int64_t num_major,
            int64_t nnz, const int64_t* edge_map, int op, int reduce,
            const float* ufeat, const float* efeat, float* out, int64_t* arg_u,
            int64_t* arg_e, int u_target, int64_t ufeat_len, int64_t efeat_len,
            int64_t out_len, const int64_t* u_off, const int64_t* e_off,
            int64_t num_out, void* workspace, size_t workspace_bytes,
            gs_stream_t stream);
int gs_e_square_sum(int format, const int64_t* a, const int64_t* b,
                    int64_t num_major, int64_t nnz, const int64_t* edge_map,
                    const float* efeat, float* out, int u_target,
                    int64_t feat_len, int64_t num_out, void* workspace,
                    size_t workspace_bytes, gs_stream_t stream);
/* out[row] += sum of e^2 over the edges of A[:, cols], read from the parent
 * matrix (the column slice is not written): cols / sub_indptr / slice_nnz as in
 * gs_col_row_slice_count (indices32 likewise), the value of the parent's edge p is efeat[edge_map[p]]
 * (efeat[p] when edge_map is NULL), out[num_out] an fp32 accumulator that the
 * caller zero-fills.  The workspace is optional
 * (NULL / 0 is valid, then every edge is an atomic add).  No counterpart in the
 * reference, which writes the slice and then runs ESquareSumCOO over it
 * (src/cuda/fusion/fused_coo_e_square_sum.cu:13-60). */
size_t gs_sliced_e_square_sum_workspace_bytes(int64_t slice_nnz, int64_t num_out);
int gs_sliced_e_square_sum(const int64_t* indptr, const int64_t* indices,
                           const int32_t* indices32, const int64_t* cols,
                           int64_t num_cols_picked, const int64_t* sub_indptr,
                           int64_t slice_nnz, const int64_t* edge_map, const float* efeat,
                           float* out, int64_t num_out, void* workspace,
                           size_t workspace_bytes, gs_stream_t stream);
int gs_e_div_u_sum(int format, const int64_t* a, const int64_t* b,
                   int64_t num_major, int64_t nnz, const int64_t* edge_map,
                   const float* ufeat, const float* efeat, float* out,
                   int u_target, int64_t feat_len, int64_t num_out,
                   void* workspace, size_t workspace_bytes, gs_stream_t stream);

/* ------------------------------------------------------------------------
 * Yardsticks (measurement helpers, no counterpart in the reference; no
 * operator calls them).
 *  gs_probe_stream_copy: dst[0..bytes) = src[0..bytes), 16 bytes per lane.
 *  gs_probe_line_gather: every lane reads 4 bytes from a 128-byte line of its
 *    own of `table`, chosen by a hash of its number and `salt` (ordered != 0:
 *    the same number of lines in address order); out needs num_picks / 4 + 1
 *    32-bit words.  How many scattered lines per second the GPU delivers.
 *  gs_probe_sample_uniform: one launch of the packed uniform sampler (int32
 *    row ids, without replacement, fanout <= 64) with parts switched off;
 *    variant is a sum of 1 (hash instead of Philox), 2 (no exchange among a
 *    column's lanes), 4 (column pointer not read: every column probe_degree
 *    long, outputs sized num_items * fanout), 8 (row ids not read), 16 (only
 *    the row id stored), 32 (nothing stored).  Built: 0, 1, 2, 4, 8, 24, 16,
 *    32, 40.  col_span (nullable) as for the sampler fills.
 * ---------------------------------------------------------------------- */
int gs_probe_stream_copy(const void* src, void* dst, int64_t bytes, gs_stream_t stream);
int gs_probe_line_gather(const void* table, int64_t table_bytes, int64_t num_picks,
                         uint64_t salt, int ordered, void* out, gs_stream_t stream);
int gs_probe_sample_uniform(
    const int64_t* indptr, int64_t num_cols, const int32_t* indices32,
    const int64_t* column_ids, int64_t num_items, int64_t fanout, int variant,
    int64_t probe_degree, uint64_t seed, uint64_t call_id, const int64_t* sub_indptr,
    const int64_t* col_span, int64_t* out_coo_col, int64_t* out_indices, int64_t* out_select,
    gs_stream_t stream);

#ifdef __cplusplus
}
#endif
#endif /* GSAMPLER_HIP_H_ */
