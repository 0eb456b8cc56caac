/*
 * C ABI of libfeatgraph_hip.so: FeatGraph's vanilla CSR SpMM and COO SDDMM
 * (and their multi-head forms) as hand-written HIP kernels for gfx950.
 *
 * These entry points take the place of the functions that the reference
 * obtains from tvm.build and then calls with positional device arrays:
 *   SpMM  : module/spmm.py:108-109 (build) and :159-160 (call), argument order
 *           (SrcFeat, indptr, indices, vals, Out);
 *   SDDMM : module/sddmm.py:89-90 (build) and :128 (call), argument order
 *           (SrcFeat, DstFeat, row, col, Out).
 *
 * Conventions
 *   - Every data pointer is DEVICE memory owned by the caller.  The library
 *     never copies user data between host and device and never allocates or
 *     frees a caller-visible buffer.  A plan owns only its private schedule
 *     arrays (row list, bounds, run records; sizes are given with each plan).
 *   - Index arrays are int32, values and features float32, row-major, dense.
 *   - Kernels are enqueued on `stream` (a hipStream_t passed as void*, NULL =
 *     the default stream) and the call returns without synchronising.  A plan
 *     belongs to the device that was current when it was created; running it
 *     with another device current returns FG_EINVAL.
 *   - Every output element is written by exactly one lane; results are
 *     deterministic and do not depend on launch shape or tile settings.
 *   - Return value: FG_OK or a negative FG_E* code; fg_last_error() then holds
 *     a message (thread-local).  No entry point aborts on bad arguments.
 *   - Index CONTENTS (column ids within range, monotone indptr) are the
 *     caller's contract, as they are for the reference's generated kernels;
 *     fg_spmm_plan_create checks indptr, fg_check_indices checks ids.
 */
#ifndef FEATGRAPH_HIP_H_
#define FEATGRAPH_HIP_H_

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define FG_API __attribute__((visibility("default")))

#define FG_OK 0
#define FG_EINVAL (-1)       /* bad argument (null pointer, negative size, shape mismatch) */
#define FG_EHIP (-2)         /* a HIP runtime call failed; message names it */
#define FG_ENOMEM (-3)       /* host or device allocation for a plan failed */
#define FG_EUNSUPPORTED (-4) /* argument combination outside what the kernels cover */

typedef struct fg_spmm_plan fg_spmm_plan;

/* Library version (major*100 + minor). */
FG_API int fg_version(void);

/* Message of the last failing call on this thread ("" when none). */
FG_API const char *fg_last_error(void);

/*
 * Degree-aware row schedule for one CSR adjacency matrix.  Replaces the
 * per-module preprocessing of SpMMbase.__init__ (module/spmm.py:58-69), which
 * in the reference only uploads the three CSR arrays.  Reads indptr once
 * (device to host), checks that it starts at 0, is non-decreasing and ends at
 * nnz, and stores on the device the row ids sorted by descending degree (ties
 * by ascending row id).  When the matrix is wide and dense enough for column
 * blocking to pay off and every row's column ids ascend, it also stores, per
 * block of about 20000 columns (equal widths), where that block starts inside every row (one device
 * pass over indices; (n_cols/20480 + 3) * n_rows int32), and for the default
 * kernel one 16-byte record {first nonzero, one past the last, row id} per row
 * and column-block pass, each pass sorted by descending run length (device
 * radix sorts; with blocks about (n_cols/20480) * 2 * n_rows records, else
 * n_rows).  The plan BORROWS indptr and indices: both must stay alive and
 * unchanged until fg_spmm_plan_destroy.
 */
FG_API int fg_spmm_plan_create(int64_t n_rows, int64_t n_cols, int64_t nnz, const int32_t *indptr,
                        const int32_t *indices, fg_spmm_plan **plan);
/*
 * The same with the caller's say on column blocking, the num_col_partitions of
 * VanillaSpMMx86 (module/spmm.py:198, util/adj_partitioning.py:42): 0 = as
 * fg_spmm_plan_create, 1 = no column blocks, P > 1 = P blocks of
 * ceil(n_cols / P) columns, used at every feature length (rows whose column ids
 * do not ascend still fall back to a single pass).  Never changes a result bit.
 */
FG_API int fg_spmm_plan_create_partitioned(int64_t n_rows, int64_t n_cols, int64_t nnz, const int32_t *indptr,
                                           const int32_t *indices, int32_t num_col_partitions, fg_spmm_plan **plan);
FG_API void fg_spmm_plan_destroy(fg_spmm_plan *plan);

/* Copies the plan's row order (n_rows int32) to HOST memory at row_order_host
 * and, when non-null, the largest row degree to *max_degree. */
FG_API int fg_spmm_plan_row_order(const fg_spmm_plan *plan, int32_t *row_order_host, int32_t *max_degree);

/*
 * Out[r, f] = sum over e in [indptr[r], indptr[r+1]) of vals[e] * feat[indices[e], f]
 * accumulated in float32, sequentially in CSR order from +0, one rounded
 * multiply and one rounded add per term: the loop nest of
 * vanilla_spmm_csr_x86 / _cuda (op/vanilla_spmm.py:46-56, :114-123).
 * feat is [n_cols, F], out is [n_rows, F]; rows without nonzeros become 0.
 * feat_tiles is the reference's num_feat_partitions (op/vanilla_spmm.py:41):
 * 0 lets the library choose the feature-tile width, P >= 1 asks for tiles of
 * about F/P floats.  It changes the launch shape only, never a result bit.
 */
FG_API int fg_spmm_csr_f32(const fg_spmm_plan *plan, const float *feat, const float *vals, float *out, int32_t F,
                    int32_t feat_tiles, void *stream);
/*
 * fg_spmm_csr_f32 over a feature matrix whose rows lie feat_pitch floats apart
 * (feat_pitch >= F, a multiple of 4; out keeps rows of F floats).  No
 * counterpart in the reference: a 256-byte piece of a row whose byte length is
 * not a multiple of the 128-byte cache line lies across three lines instead of
 * two, which costs gathers up to half as much again (100 floats against 128:
 * 4.7 against 3.4 ms on the 114.6M-nonzero graph); a caller that can afford a
 * copy of the features with rows padded to a multiple of 32 floats
 * (fg_pad_rows_f32) runs this entry point over the copy.  FG_EUNSUPPORTED when
 * the several-rows-per-wave kernel, the only one that takes a pitch, does not
 * take the call (then call fg_spmm_csr_f32 on the matrix itself).  Bit-identical
 * to fg_spmm_csr_f32.
 */
FG_API int fg_spmm_csr_pitched_f32(const fg_spmm_plan *plan, const float *feat, int32_t feat_pitch, const float *vals,
                                   float *out, int32_t F, void *stream);
/* out[i * pitch + k] = in[i * F + k] for i < n, k < F; the floats behind F in a row of out are left as they are
 * (the pitched entry points never use them).  in and out must not overlap. */
FG_API int fg_pad_rows_f32(int64_t n, int32_t F, int32_t pitch, const float *in, float *out, void *stream);

/*
 * fg_spmm_csr_f32 without a plan and without any allocation.  No counterpart in
 * the reference: it is for callers that cannot allocate device memory (code
 * under HIP graph capture, tight serving loops, harnesses that forbid
 * hipMalloc) and therefore cannot call fg_spmm_plan_create.  The row schedule
 * that a plan keeps in allocated memory (rows by descending degree and their
 * bounds) is rebuilt on the device at every call, by degree class, inside a
 * fixed 12 MiB array that is part of the library image, one copy per GPU;
 * the SpMM kernels of fg_spmm_csr_f32 then run over it.  Same result bits as
 * fg_spmm_csr_f32.  Limits: n_rows <= 1048576 (FG_EUNSUPPORTED beyond).  The
 * call enqueues kernels on `stream` and returns; it calls no hipMalloc /
 * hipFree, copies nothing and never synchronises.  Every call on a GPU uses
 * that GPU's one array: calls that overlap in time on the same GPU (two
 * streams, two threads) race on it and must be serialised by the caller.
 * The array's device address is looked up at the first call on each GPU, and
 * that lookup must not happen under stream capture: make one eager call per
 * GPU before recording the entry point into a HIP graph.  A first call that
 * finds `stream` capturing returns FG_EUNSUPPORTED and enqueues nothing.
 * indptr CONTENTS are the caller's contract (non-decreasing, 0 .. nnz); rows
 * whose bounds are out of range come out as zeros.
 */
FG_API int fg_spmm_csr_noalloc_f32(int64_t n_rows, int64_t n_cols, int64_t nnz, const int32_t *indptr,
                                   const int32_t *indices, const float *vals, const float *feat, float *out,
                                   int32_t F, void *stream);

/*
 * Generalised SpMM: the message and reduce slots of the reference's operator
 * template (op/vanilla_spmm.py:46-53: msgfunc forms adj_val * feat_val and
 * folds it with te.sum) opened to the other operators of "generalized SpMM"
 * (README.md:6).  The reference itself ships only (FG_MSG_MUL, FG_REDUCE_SUM).
 *   term(e, f) = msg(feat[indices[e], f], vals[e])
 *   Out[r, f]  = fold of the row's terms in CSR order
 * FG_REDUCE_SUM starts from +0; MAX / MIN fold as acc = (t > acc) ? t : acc;
 * MEAN is the sum divided by the row's degree (one rounded division).  Rows
 * without nonzeros give 0 under every reducer.  One rounded operation per
 * message and per fold step, so (MUL, SUM) equals fg_spmm_csr_f32 bit for bit.
 * vals may be null for FG_MSG_COPY_U.  Runs the kernel of fg_spmm_csr_f32 with
 * the message and the reducer in place of the multiply-add where that kernel
 * applies (feature lengths that are multiples of 4), a row-slot kernel
 * otherwise; one launch per column block of the plan (one launch over whole
 * rows when the plan has no blocks), MEAN one more for the division.  The
 * partial fold of a row is carried in `out` between launches, so `out` must
 * not be read by anything else on the stream until the last launch has finished.
 */
#define FG_MSG_MUL 0
#define FG_MSG_ADD 1
#define FG_MSG_SUB 2
#define FG_MSG_DIV 3
#define FG_MSG_COPY_U 4
#define FG_REDUCE_SUM 0
#define FG_REDUCE_MAX 1
#define FG_REDUCE_MIN 2
#define FG_REDUCE_MEAN 3
FG_API int fg_spmm_csr_general_f32(const fg_spmm_plan *plan, const float *feat, const float *vals, float *out,
                                   int32_t F, int32_t msg, int32_t reduce, void *stream);

/*
 * Multi-head generalised SpMM (no counterpart in the reference, whose
 * op/__init__.py:1-5 exports vanilla operators only; same message function as
 * op/vanilla_spmm.py:46-53 with a per-head weight):
 * Out[r, h, d] = sum over e in row r of w[e, h] * feat[indices[e], h, d].
 * feat [n_cols, H, D], w [nnz, H], out [n_rows, H, D].  H = 1 gives
 * fg_spmm_csr_f32 bit for bit.
 */
FG_API int fg_spmm_csr_mh_f32(const fg_spmm_plan *plan, const float *feat, const float *w, float *out, int32_t H,
                       int32_t D, int32_t feat_tiles, void *stream);

/*
 * The two above combined (no counterpart in the reference): the message and
 * reduce slots of op/vanilla_spmm.py:46-53 with a per-edge per-head value,
 *   term(e, h, d) = msg(feat[indices[e], h, d], w[e, h])
 *   Out[r, h, d]  = fold of the row's terms in CSR order,
 * msg / reduce as for fg_spmm_csr_general_f32 (same folds, same treatment of
 * rows without nonzeros, FG_REDUCE_MEAN divides by the row's degree).  feat
 * [n_cols, H, D], w [nnz, H] (may be null for FG_MSG_COPY_U), out
 * [n_rows, H, D].  (MUL, SUM) equals fg_spmm_csr_mh_f32 bit for bit and H = 1
 * equals fg_spmm_csr_general_f32.  One launch per column block of the plan,
 * the partial fold carried in `out`.
 */
FG_API int fg_spmm_csr_mh_general_f32(const fg_spmm_plan *plan, const float *feat, const float *w, float *out,
                                      int32_t H, int32_t D, int32_t msg, int32_t reduce, void *stream);

/*
 * Out[e] = sum_k src[col[e], k] * dst[row[e], k]   (op/vanilla_sddmm.py:43-47;
 * note src is indexed by COLUMN ids and dst by ROW ids, as the reference's
 * tests shape them: tests/test_module_sddmm.py:18-19).
 * src [n_cols, F], dst [n_rows, F], out [nnz].  Any nnz >= 0.
 */
FG_API int fg_sddmm_coo_f32(int64_t nnz, const int32_t *row, const int32_t *col, const float *src, const float *dst,
                     float *out, int32_t F, void *stream);

/*
 * Generalised SDDMM: the edge-function slot of op/vanilla_sddmm.py:43-47.
 * FG_EDGE_DOT is fg_sddmm_coo_f32 (out [nnz]); the other operators keep the
 * feature axis: Out[e, f] = src[col[e], f] op dst[row[e], f], out [nnz, F],
 * one rounded operation per element.
 */
#define FG_EDGE_DOT 0
#define FG_EDGE_ADD 1
#define FG_EDGE_SUB 2
#define FG_EDGE_MUL 3
#define FG_EDGE_DIV 4
FG_API int fg_sddmm_coo_general_f32(int64_t nnz, const int32_t *row, const int32_t *col, const float *src,
                                    const float *dst, float *out, int32_t F, int32_t edge_op, void *stream);

/*
 * Cache-blocking schedule for one COO edge list; takes the place that
 * SDDMMbase.__init__ gives to 2-D graph partitioning (module/sddmm.py:45-49).
 * When the matrix is wide and dense enough: for a list whose row ids ascend
 * and whose column ids ascend inside every row (COO derived from CSR) it
 * rebuilds the row pointer and stores where every block of columns starts
 * inside every row ((2 * n_cols/16384 + 3) * n_rows int32).  For a list in any
 * other order it sorts a copy of the list by (row, column) (one device radix
 * sort, stable), builds the same tables over the copy, and keeps the copy's
 * column ids, room for the results in that order and the routing that brings
 * them back to the caller's order in two steps that each permute inside blocks
 * of 32768 results ("sddmm.regroup" = 0: one gather instead): 16 bytes per
 * edge.  A call then runs the same kernel as for a sorted list and returns the
 * results, so they are always written in the caller's edge order (there is no
 * edge_mapping to apply) and equal the sorted list's bit for bit.  Because the results pass through memory that the plan
 * owns, two calls on ONE plan of an unsorted list must not overlap in time.
 * A list whose rows ascend while the columns inside a row do not gets the same
 * sorted copy (and may still be used with fg_sddmm_softmax_plan_f32, which
 * works on the caller's order).  Lists with ids outside the matrix and
 * "sddmm.sorted_copy" = 0 fall back to a copy re-ordered by column block and
 * destination row whose kernel scatters its results.
 * The plan BORROWS row and col, which must stay alive and unchanged until
 * fg_sddmm_plan_destroy.
 */
typedef struct fg_sddmm_plan fg_sddmm_plan;
FG_API int fg_sddmm_plan_create(int64_t nnz, int64_t n_rows, int64_t n_cols, const int32_t *row, const int32_t *col,
                                fg_sddmm_plan **plan);
/* The same with the caller's num_col_partitions (module/sddmm.py:169): 0 = library decides, 1 = no blocks,
 * P > 1 = P blocks of ceil(n_cols / P) columns. */
FG_API int fg_sddmm_plan_create_partitioned(int64_t nnz, int64_t n_rows, int64_t n_cols, const int32_t *row,
                                            const int32_t *col, int32_t num_col_partitions, fg_sddmm_plan **plan);
FG_API void fg_sddmm_plan_destroy(fg_sddmm_plan *plan);

/*
 * fg_sddmm_coo_mh_f32 on the plan's edge list.  With H = 1 and F >= 4 a blocked
 * plan runs one launch per feature tile of up to 128 floats (each tile adds its
 * partial dot product to Out, the reference's feature tiling:
 * op/vanilla_sddmm.py:49-60) over (row, column block) runs of a row-sorted
 * list -- the caller's own, or the plan's sorted copy of a list in any other
 * order -- with one Dst tile held in registers per run; with F a multiple of 4
 * and 16-byte aligned operands a plan built with sddmm.sorted_copy = 0 walks
 * its re-ordered list instead; otherwise this is the plain kernel.  All agree
 * within float32 rounding.
 */
FG_API int fg_sddmm_coo_plan_f32(const fg_sddmm_plan *plan, const float *src, const float *dst, float *out, int32_t H,
                                 int32_t D, void *stream);
/*
 * fg_sddmm_coo_plan_f32 (single head) over src and dst matrices whose rows lie
 * `pitch` floats apart (pitch >= F, a multiple of 4), for the same reason as
 * fg_spmm_csr_pitched_f32: rows that are not a multiple of the 128-byte cache
 * line cost the gathers up to a third as much again.  FG_EUNSUPPORTED when the
 * row-run kernel, the only one that takes a pitch, does not take the call.
 * The same result bits as fg_sddmm_coo_plan_f32.  No counterpart in the reference.
 */
FG_API int fg_sddmm_coo_plan_pitched_f32(const fg_sddmm_plan *plan, const float *src, const float *dst, int32_t pitch,
                                         float *out, int32_t F, void *stream);
FG_API int fg_sddmm_plan_describe(const fg_sddmm_plan *plan, int32_t H, int32_t D, char *buf, int64_t cap);

/*
 * fg_sddmm_coo_general_f32 on the plan's edge list (the edgefunc slot of
 * op/vanilla_sddmm.py:43-47 behind the plan that SDDMMbase.__init__ builds).
 * For a row-sorted list with column blocks the elementwise operators run over
 * the plan's (row, column block) runs, the Dst tile held in registers and the
 * Src gathers inside a band an L2 holds; other lists take the edge-parallel
 * kernel.  out [nnz, F] (FG_EDGE_DOT: [nnz]); every element is one rounded
 * operation, so both kernels give the same bits.
 */
FG_API int fg_sddmm_coo_general_plan_f32(const fg_sddmm_plan *plan, const float *src, const float *dst, float *out,
                                         int32_t F, int32_t edge_op, void *stream);

/*
 * Edge softmax (no counterpart in the reference; the step between the scores of
 * multi-head SDDMM and the weights of multi-head SpMM in a GAT-style layer).
 * The edge list is the CSR one: row r's edges are [indptr[r], indptr[r+1]).
 * out[e, h] = exp(scores[e, h] - max) / sum over the row's edges of
 * exp(scores[e', h] - max), max taken over the same edges, per head.  scores
 * and out are [nnz, H] and may be the same buffer.  A score of -inf is a masked
 * edge: weight 0 wherever it stands in the row; a row and head with nothing
 * but -inf gives NaN (0 / 0), as the textbook softmax does.
 * Accuracy: float32 throughout, with the device library's expf (documented to
 * 1 ulp).  A weight of this entry point is one expf and one division over a
 * sum of such terms: within rtol 1e-5 of the exact softmax of the float32
 * scores.  The fused entry points below (fg_sddmm_softmax_plan_f32,
 * fg_attention_csr_mh_f32) keep a running maximum and rescale their partial
 * sums by a further expf whenever it grows, and compute the scores in the same
 * kernel, whose float32 rounding enters the exponent: they are held to
 * rtol 5e-5 and 1e-4.
 */
FG_API int fg_edge_softmax_csr_f32(int64_t n_rows, const int32_t *indptr, const float *scores, float *out, int32_t H,
                                   void *stream);
/*
 * Backward of the edge softmax (no counterpart in the reference): with
 * `weights` the output of fg_edge_softmax_csr_f32 and `grad` the gradient that
 * arrives for it, both [nnz, H],
 *   out[e, h] = weights[e, h] * (grad[e, h] - sum over the row's edges e' of weights[e', h] * grad[e', h]),
 * the gradient for the scores.  out may be the same buffer as grad.
 */
FG_API int fg_edge_softmax_backward_csr_f32(int64_t n_rows, const int32_t *indptr, const float *weights,
                                            const float *grad, float *out, int32_t H, void *stream);
/*
 * Helpers of the multi-head backward (no counterpart in the reference).
 * fg_permute_rows_f32: out[i, :] = in[perm[i], :] for i in [0, n), rows of
 * `width` floats; carries per-edge weights from the order of a matrix's CSR
 * arrays to that of its transpose's.  perm entries must lie in [0, rows of
 * in); in and out must not overlap.  fg_add_f32: out[i] = a[i] + b[i] for
 * i in [0, n); out may be a or b.
 */
FG_API int fg_permute_rows_f32(int64_t n, int32_t width, const int32_t *perm, const float *in, float *out,
                               void *stream);
FG_API int fg_add_f32(int64_t n, const float *a, const float *b, float *out, void *stream);
/*
 * fg_sddmm_coo_mh_f32 followed by fg_edge_softmax_csr_f32, on the plan's edge
 * list, which must be row-sorted (FG_EUNSUPPORTED otherwise):
 * out[e, h] = softmax over the edges of row[e] of sum_d src[col[e], h, d] * dst[row[e], h, d].
 * When a vertex row (H * D floats) is one or two runs of 64 loads of 1, 2 or 4
 * floats and a head spans 4, 8 or 16 of a run's lanes (H = 8 with D in {8, 16,
 * 32, 64}; H = 4 with D in {16, 32, 64}; H = 16 with D in {4, 8, 16, 32}; ...)
 * one fused kernel computes a destination row's scores, keeps their running
 * maximum and sum, and normalises them in place, so the raw scores never
 * travel through a second kernel; other shapes run the two kernels one after
 * the other.  Float32
 * throughout; agrees with the float64 softmax of the float32 scores within
 * rtol 1e-5.
 */
FG_API int fg_sddmm_softmax_plan_f32(const fg_sddmm_plan *plan, const float *src, const float *dst, float *out,
                                     int32_t H, int32_t D, void *stream);

/* Multi-head SDDMM, edge softmax and multi-head SpMM as one operator (no
 * counterpart in the reference, which has the two ends as separate operators:
 * the multi-head scores of op/vanilla_sddmm.py:35-47 and the multi-head SpMM
 * of its benchmarks):
 *   out[r, h, :] = sum over the nonzeros e of row r of A[e, h] * value[indices[e], h, :],
 *   A[e, h] = softmax over the row's nonzeros of sum_d key[indices[e], h, d] * query[r, h, d].
 * key, value [n_cols, H, D]; query, out [n_rows, H, D]; rows without nonzeros
 * give zeros.  The scores and weights never exist in memory; when value == key
 * every neighbour row is gathered once for both uses.  Float32 throughout with a
 * running (max, sum) softmax: agrees with the three operators run one after the
 * other within rtol 1e-4 / atol 1e-5, not bit for bit (the weighted sum is
 * rescaled whenever the running maximum grows).  Shapes: those of the fused
 * score + softmax kernel (a head spans 4, 8 or 16 lanes of 1, 2 or 4 floats, a
 * vertex row is 64 or 128 such loads: H = 8 with D in {8, ..., 64}, H = 4 with
 * D in {16, 32, 64}, ...); FG_EUNSUPPORTED otherwise, and the caller runs
 * fg_sddmm_softmax_plan_f32 and fg_spmm_csr_mh_f32 instead. */
FG_API int fg_attention_csr_mh_f32(const fg_spmm_plan *plan, const float *key, const float *query, const float *value,
                                   float *out, int32_t H, int32_t D, void *stream);

/*
 * Multi-head SDDMM (no counterpart in the reference; the edge function of
 * op/vanilla_sddmm.py:47 per head): Out[e, h] = sum_d src[col[e], h, d] * dst[row[e], h, d].
 * src [n_cols, H, D], dst [n_rows, H, D], out [nnz, H].  H = 1 gives
 * fg_sddmm_coo_f32 bit for bit.
 */
FG_API int fg_sddmm_coo_mh_f32(int64_t nnz, const int32_t *row, const int32_t *col, const float *src, const float *dst,
                        float *out, int32_t H, int32_t D, void *stream);

/*
 * Debug aid: counts entries of idx[0..n) outside [0, bound) on the device and
 * writes the count to *n_bad (host).  Synchronises `stream`.
 */
FG_API int fg_check_indices(int64_t n, const int32_t *idx, int64_t bound, int64_t *n_bad, void *stream);

/*
 * ---- fg_probe_*: measurement aids, NOT part of the operator API ------------
 * The seven fg_probe_* entry points below exist for the benchmark only (bare
 * gather / store patterns that price what the memory system does); no module
 * class calls them, they have no counterpart in the reference, and they may
 * change or go away without notice.  A binding for the operators leaves them
 * out.
 *
 * The gather pattern of the
 * SpMM / SDDMM kernels with everything else left out.  Per feature tile of
 * `tile` floats (16, 32 or 64; F a multiple of it) it gathers about n_gathers
 * random rows of feat [n_rows, F] with 16-byte loads, tile/4 lanes per row,
 * sixteen gathers in flight per lane, one launch per band of band_rows
 * consecutive rows and per tile, bands in ascending order; no index or value
 * stream, no sums, no output (sink, one float, is never written for finite
 * features).  Its time is a floor for any kernel that moves the same rows
 * through the caches with the same blocking.  fg_probe_gather_count returns
 * the gathers per tile that such a call really issues (the request is rounded
 * to whole iterations of the grid), or -1 for arguments the probe rejects.
 * The matrix must span less than 4 GiB.
 */
FG_API int fg_probe_gather_f32(const float *feat, int64_t n_rows, int32_t F, int32_t tile, int32_t band_rows,
                               int64_t n_gathers, float *sink, void *stream);
FG_API int64_t fg_probe_gather_count(int64_t n_rows, int32_t tile, int32_t band_rows, int64_t n_gathers);
/*
 * The same for the multi-head operators, whose feature matrices are far beyond
 * any cache: about n_gathers whole rows of row_floats floats (128, 256, 512 or
 * 1024) from random places of feat [n_rows, row_floats], 16-byte loads, 64-bit
 * addressing, sixteen loads in flight per lane, one launch.  What it sustains
 * is the rate at which this part's HBM serves random row gathers.
 */
FG_API int fg_probe_gather_rows_f32(const float *feat, int64_t n_rows, int32_t row_floats, int64_t n_gathers,
                                    float *sink, void *stream);
FG_API int64_t fg_probe_gather_rows_count(int32_t row_floats, int64_t n_gathers);
/*
 * The same with result rows: after about every gathers_per_write gathered rows
 * (rounded to whole iterations of 16 / 8 / 4 rows for rows of up to 256 / 512 /
 * 1024 floats) a group of lanes also writes one whole row of out
 * [n_out_rows, row_floats], a random one.  An operator that gathers deg rows
 * and stores one per destination row moves this mix; on this part the stores
 * cost several times their share of the bytes, so the read-only probe is not a
 * floor such an operator can reach.  fg_probe_gather_write_rows_count gives the
 * gathers and the row writes that a call with these arguments issues.
 */
FG_API int fg_probe_gather_write_rows_f32(const float *feat, int64_t n_rows, int32_t row_floats, int64_t n_gathers,
                                          int32_t gathers_per_write, float *out, int64_t n_out_rows, float *sink,
                                          void *stream);
FG_API int fg_probe_gather_write_rows_count(int32_t row_floats, int64_t n_gathers, int32_t gathers_per_write,
                                            int64_t *gathers, int64_t *writes);
/*
 * The stores alone: about n_stores whole rows of out [n_out_rows, row_floats],
 * random ones, and nothing read.  Returns the number of rows stored (the
 * request rounded to whole rows per group of lanes), or -1 on a bad argument.
 * Together with the probes above it separates what the stores cost by
 * themselves from what they cost in between the gathers.
 */
FG_API int64_t fg_probe_store_rows_f32(float *out, int64_t n_out_rows, int32_t row_floats, int64_t n_stores,
                                       void *stream);
/*
 * Bare gathers of 64-float rows out of the first band_rows rows of feat (the
 * pattern of fg_probe_gather_f32 with a 64-float tile) with an index-like
 * stream of 8 bytes per gather read beside them from stream_buf, which holds
 * stream_dwords zero dwords of which the first window_dwords are used (powers
 * of two; the whole buffer: every piece comes from HBM, a small window: from
 * the Infinity Cache or L2).  mode 0: no stream; 1: every wave reads its own
 * piece with a vector load an iteration ahead; 2: one wave of every four reads
 * the pieces of all four and the other three gather; 3: as 1 through the
 * scalar cache.  Returns the gathers issued, or -1 on a bad argument.  It shows
 * what a stream of that size costs the gathers next to it, and by which path.
 */
FG_API int64_t fg_probe_gather_stream_f32(const float *feat, int32_t band_rows, int64_t n_gathers,
                                          const uint32_t *stream_buf, int64_t stream_dwords, int64_t window_dwords,
                                          int32_t mode, float *sink, void *stream);

/*
 * Launch-shape overrides for tuning and tests.  The store is process-global
 * and unsynchronised: a single-threaded hook, not to be called while another
 * thread is inside any entry point.  Some keys are read when a plan is created
 * and some at every launch (noted per key); a plan created under one setting
 * and launched under another stays correct, because every SpMM variant gives
 * identical bits and every SDDMM variant results within float32 rounding; only
 * the kernel choice changes.
 * Keys: "spmm.vec" (floats per lane: 1, 2, 4), "spmm.lpr" (lanes per row
 * slot: 8, 16, 32, 64), "spmm.unroll" (gathers in flight per lane: 4, 8, 16),
 * "spmm.sorted" (0/1: visit rows by descending degree or
 * in natural order), "spmm.blocked" (0/1: never / always run SpMM as one pass
 * per column block when the plan has blocks; read at plan creation and at
 * launch), "spmm.block_cols" (columns per block, read at plan creation),
 * "spmm.pipeline" (0/1: wave-per-row kernel that keeps three rows in flight),
 * "spmm.pipe_blocks" (its grid size), "spmm.buffer_loads" (0/1: gather through
 * a buffer resource with scalar row offsets; needs a feature matrix below 4 GiB),
 * "spmm.multi" (0/1: never / always use the several-rows-per-wave kernel where
 * it applies; by default it runs unless one of the shape keys above is set;
 * read at plan creation and at launch), "spmm.multi_blocks" (its grid size),
 * "spmm.multi_long" (run length from which a run gets a workgroup of its
 * own, default 1024; read at plan creation), "spmm.tile_interleave" (feature tiles
 * whose workgroups alternate inside one launch of that kernel: 1 or 2, default 2),
 * "spmm.general_multi" (0/1: whether fg_spmm_csr_general_f32 may use that
 * kernel; default 1), "spmm.relay" (0/1: whether the plan keeps, per pass layout of that kernel, a
 * copy of the column ids in the order the passes visit them; read at plan
 * creation; default 1),
 * "sddmm.blocked" (0/1: never / always build and use column blocks, read at
 * plan creation), "sddmm.block_cols" (columns per block, read at plan creation),
 * "sddmm.group" (lanes per dot product: 1..16),
 * "sddmm.batches" (64-edge batches per wave), "sddmm.fast" (0/1: unrolled
 * kernel for D in 16..512), "sddmm.buffer_loads" (0/1), "sddmm.rows" (0/1:
 * never / always use the row-run kernel when the plan has a row plan; read at
 * plan creation and at launch), "sddmm.rows_blocks" (its grid size),
 * "sddmm.rows_wide" (1: 64-float tiles only, 2: 128-float tiles over passes of
 * half the width for feature rows of 128 floats and more; by default 2 when a
 * (row, pass) run then still holds 8 edges on average),
 * "sddmm.sorted_copy" (0/1: whether a plan over a list that is not row-sorted
 * works on a sorted copy, read at plan creation; default 1), "sddmm.regroup"
 * (0/1: whether such a plan returns the results through two block-local
 * permutations or one gather, read at plan creation; default 1),
 * "sddmm.xcd" (0/1: whether the passes of the row-run kernel are pinned to the
 * part's eight dies -- workgroup x of a launch runs on die x % 8, so the
 * workgroups x % 8 == d take the passes d, d + 8, ... and each die's L2 keeps
 * the band of its own pass -- and whether the library's own blocks come in a
 * multiple of eight passes; read at plan creation and at launch; default 1;
 * same result bits either way),
 * "spmm.pad_rows" (0/1: whether VanillaSpMMhip and VanillaSDDMMhip, the Python modules, gather from
 * a copy of the features with rows padded to a multiple of 32 floats when the
 * feature length is beyond 64 floats and not one, fg_spmm_csr_pitched_f32 /
 * fg_sddmm_coo_plan_pitched_f32; the C entry points do
 * not read it; default 1),
 * "attention.blocks" (grid size of the fused attention kernel; by default one
 * vertex row per wave when a row is 1 KB or more, else 65536 workgroups that
 * walk the rows).  Value 0 restores the default of a size; for the 0/1 flags a
 * negative value does.
 * The spmm.* keys change the launch shape only; "sddmm.group" and
 * "sddmm.rows_wide" also change the shape of the summation tree, i.e. the last
 * bits of an SDDMM result.
 */
FG_API int fg_config_set(const char *key, int32_t value);
FG_API int fg_config_get(const char *key, int32_t *value);

/* Human-readable description of the launch the library would use for a
 * feature length (the counterpart of lower_to_ir, module/spmm.py:113-140).
 * Writes at most cap bytes including the terminator. */
FG_API int fg_spmm_describe(const fg_spmm_plan *plan, int32_t H, int32_t D, int32_t feat_tiles, char *buf, int64_t cap);
FG_API int fg_sddmm_describe(int64_t nnz, int32_t H, int32_t D, char *buf, int64_t cap);

#ifdef __cplusplus
}
#endif
#endif /* FEATGRAPH_HIP_H_ */
