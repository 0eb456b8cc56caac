// Shared declarations of libfeatgraph_hip.so: error reporting, tuning store,
// kernel argument blocks and the launchers that api.hip calls.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include <vector>

#include "../../include/featgraph_hip.h"

namespace fg {

// Records a message for fg_last_error() and returns `code`.
int fail(int code, const char *fmt, ...) __attribute__((format(printf, 2, 3)));

#define FG_HIP_TRY(expr)                                                                      \
  do {                                                                                        \
    hipError_t fg_err_ = (expr);                                                              \
    if (fg_err_ != hipSuccess) return ::fg::fail(FG_EHIP, "%s: %s", #expr, hipGetErrorString(fg_err_)); \
  } while (0)

// Launch-shape overrides (0 = library default).
struct Config {
  int spmm_vec = 0, spmm_lpr = 0, spmm_unroll = 0, spmm_sorted = -1;
  int spmm_blocked = -1, spmm_block_cols = 0, spmm_pipeline = -1, spmm_pipe_blocks = 0;
  int spmm_buffer_loads = -1;
  int spmm_multi = -1, spmm_multi_blocks = 0, spmm_multi_long = 0, spmm_tile_interleave = 0;
  int sddmm_group = 0, sddmm_batches = 0, sddmm_blocked = -1, sddmm_block_cols = 0;
  int sddmm_fast = -1, sddmm_buffer_loads = -1, sddmm_rows = -1, sddmm_rows_blocks = 0;
  int attention_blocks = 0, sddmm_rows_wide = 0, sddmm_sorted_copy = -1, sddmm_regroup = -1, spmm_relay = -1, spmm_general_multi = -1;
  int sddmm_xcd = -1, spmm_xcd = -1;
  int spmm_pad_rows = -1;
};
Config &config();

// Accelerator complex dies of the part, each with its own L2; workgroups of a launch go to them round-robin by
// their linear id (measured on MI355X: hardware XCC id == workgroup id % 8).
constexpr int kXcds = 8;
constexpr int kWaveSize = 64;
constexpr int kWavesPerBlock = 4;
constexpr int kBlockThreads = kWaveSize * kWavesPerBlock;

// One launch of the row-slot SpMM kernel.  A "slot" is a group of `lpr` lanes
// that owns one (row, feature tile) pair.
struct SpmmArgs {
  const int32_t *indptr;
  const int32_t *indices;
  const float *w;  // [nnz, H] edge weights (H == 1: the CSR values)
  const float *feat;
  float *out;
  const int32_t *row_order;  // rows by descending degree, or null for natural order
  int32_t n_rows;
  int32_t n_cols;
  int32_t F;  // floats per feature row (= H * D)
  int32_t H;
  int32_t D;
  int32_t n_tiles;
  int64_t n_slots;  // n_tiles * n_rows
  // Column-blocked passes: this launch covers only the nonzeros
  // [seg_lo[row], seg_hi[row]) of every row (one column block), for the tiles
  // tile_base .. tile_base + n_tiles - 1, and when `accumulate` is set it
  // continues the sums that an earlier pass left in `out`.
  const int32_t *seg_lo = nullptr;
  const int32_t *seg_hi = nullptr;
  int32_t tile_base = 0;
  int32_t accumulate = 0;
  // several-rows-per-wave kernel: one pass's records {first nonzero, one past the last, row id, 0}, n_rows of them
  const int4 *runs = nullptr;
  int32_t long_runs = 0;    // the first long_runs records are long runs: one workgroup each, in the first
  int32_t long_blocks = 0;  // long_blocks workgroups of the grid
  int32_t interleave_tiles = 1;  // this many tiles alternate workgroup by workgroup along grid.x; the rest along grid.y
  int32_t multi_tile = 0;        // floats per tile of the several-rows-per-wave kernel (16 / 32 / 64); 0: by feature length
  int32_t feat_pitch = 0;        // several-rows-per-wave kernel: floats from one feature row to the next; 0: F
  // records over a re-laid copy of the ids (MultiRuns::ids_p): `indices` is that copy, and a run's values start
  // at the CSR position in the record's fourth entry
  int32_t vals_by_csr = 0;
  // several-rows-per-wave kernel as the generalised operator: reduce = FG_REDUCE_SUM / MAX / MIN folds
  // msg(feature, value) (FG_MSG_*); reduce < 0 is the plain multiply-add
  int32_t reduce = -1;
  int32_t msg = 0;
};

struct SpmmShape {
  int vec, lpr, unroll;
  int pipeline = 0;       // wave-per-row kernel that keeps three rows in flight
  int pipe_blocks = 0;    // its grid size (workgroups per feature tile)
  int tile_width() const { return vec * lpr; }
};

SpmmShape spmm_choose_shape(const SpmmArgs &a, int feat_tiles);

int spmm_launch(const SpmmArgs &a, const SpmmShape &s, hipStream_t stream);

// Several-rows-per-wave kernel with 16-byte gathers (spmm_multi.hip): single head, feature length a multiple
// of 4, 16-byte aligned operands, rows and bounds from the plan.  Tiles are spmm_multi_tile(F) floats wide.
struct MultiRuns {
  int4 *rec = nullptr;  // [passes * n_rows], device, owned by the plan
  int32_t merge = 0;    // column blocks of the bounds table per pass
  int32_t passes = 0;
  int32_t *long_runs = nullptr;  // [passes], host, owned: how many of a pass's records are long runs
  // With several passes: the column ids laid out in the order the records are visited (pass after pass, inside a
  // pass by descending run length), every run starting on a multiple of four entries, so that a pass reads its
  // ids front to back instead of one short piece of the CSR array per run.  The records then hold
  // {first, last + 1 in this layout, row, first in the CSR arrays}.  Null: the records index the CSR arrays.
  int32_t *ids_p = nullptr;   // [relaid_n], device, owned
  int64_t relaid_n = 0;
};
// indices: the CSR column ids (for the re-laid copy; null builds none)
int multi_runs_build(const int32_t *seg, const int32_t *row_order, const int32_t *indices, int64_t nnz, int32_t n_rows,
                     int32_t n_blocks, int32_t merge, MultiRuns *out);
void multi_runs_free(MultiRuns *r);
int spmm_multi_tile(int32_t F);
bool spmm_multi_applies(const SpmmArgs &a);
bool spmm_multi_general_applies(const SpmmArgs &a);  // ... with a.reduce >= 0
int spmm_multi_launch(const SpmmArgs &a, hipStream_t stream);

// One launch of the edge-parallel SDDMM kernel over n_ve = nnz * H dot
// products of length D ("virtual edges": edge e, head h -> e * H + h).
struct SddmmArgs {
  const int32_t *row;
  const int32_t *col;
  const float *src;
  const float *dst;
  float *out;
  int64_t n_ve;
  int32_t H;
  int32_t D;
  int32_t stride;  // floats per vertex row (= H * D)
  int32_t batches;  // 64-dot batches per wave
  int64_t src_bytes = int64_t{1} << 40, dst_bytes = int64_t{1} << 40;  // extents of the two matrices
};

struct SddmmShape {
  int vec, group, batches;
};

SddmmShape sddmm_choose_shape(const SddmmArgs &a);
int sddmm_launch(const SddmmArgs &a, const SddmmShape &s, hipStream_t stream);

// Edge list of a COO matrix re-ordered by column block (sddmm_blocked.hip);
// device arrays owned by the SDDMM plan, all null when blocking is not used.
struct SddmmBlocks {
  int32_t *row_p = nullptr;  // [nnz] row ids in block-major order
  int32_t *col_p = nullptr;  // [nnz] column ids in block-major order
  int32_t *pos_p = nullptr;  // [nnz] position of each of these edges in the caller's list
  int32_t n_blocks = 0;
  int32_t block_cols = 0;
};

// Copy of a COO edge list sorted by (row, column) (sddmm_sorted.hip): lets the row-run kernel serve a list in
// any order.  Device arrays owned by the SDDMM plan, all null when there is no such copy.
struct SddmmSorted {
  int32_t *row_s = nullptr;    // [nnz] row ids in sorted order; freed once the row pointer is built
  int32_t *col_s = nullptr;    // [nnz] column ids in sorted order
  int32_t *where = nullptr;    // [nnz] place of the caller's edge e in the sorted list (null when `from` exists)
  float *results = nullptr;    // [nnz] the dot products in sorted order, between the kernel and the gather back
  // The gather back as two block-local permutations (null: one gather through `where`)
  uint16_t *a_local = nullptr;  // [nnz] place of sorted element i inside its block after step A
  int32_t *from = nullptr;      // [nnz] place after step A of the j-th element of the caller's blocks
  uint16_t *b_local = nullptr;  // [nnz] place of that element inside its block of the output
};
// Leaves *out empty (and returns FG_OK) for ids outside the matrix, sizes beyond int32 or when memory runs out.
int sddmm_sorted_build(int64_t nnz, int64_t n_rows, int64_t n_cols, const int32_t *row, const int32_t *col,
                       SddmmSorted *out);
void sddmm_sorted_free(SddmmSorted *s);
// out[e] = the result of the caller's edge e; s.results is left in another order
int sddmm_unsort_launch(const SddmmSorted &s, int64_t nnz, float *out, hipStream_t stream);

// num_col_partitions: 0 lets the library decide, 1 builds nothing, P > 1 builds P column blocks.
int sddmm_blocks_build(int64_t nnz, int64_t n_rows, int64_t n_cols, const int32_t *row, const int32_t *col,
                       int32_t num_col_partitions, SddmmBlocks *out);
void sddmm_blocks_free(SddmmBlocks *b);
// src / dst 16-byte aligned, F a multiple of 4; *_bytes: extents of the two matrices.
int sddmm_blocked_launch(const SddmmBlocks &b, int64_t nnz, const float *src, const float *dst, float *out, int32_t F,
                         int64_t src_bytes, int64_t dst_bytes, hipStream_t stream);
// One 64-float tile of every dot product of a (re-ordered) edge list: tile 0
// stores to out[pos[i]], later tiles add to it (sddmm.hip).
int sddmm_tile_launch(const int32_t *row_p, const int32_t *col_p, const int32_t *pos_p, int64_t nnz, const float *src,
                      const float *dst, float *out, int64_t src_bytes, int64_t dst_bytes, int32_t F, int tile,
                      hipStream_t stream);

// Row-run kernel over (column block, row) runs of a row-sorted edge list: one launch per tile, grid.y = column
// block.  A tile is sddmm_rows_tile(F, max_wide) floats: 16 / 32 / 64 for short rows, and max_wide (1 or 2)
// times 64 for longer ones.  seg / row_order are the bounds table and row list of a row plan built on the
// same matrix; a pass of a 64-float tile takes merge64 neighbouring blocks of the table, narrower tiles
// proportionally more, wider tiles proportionally fewer; merge64 = 0 means one block per pass for every tile
// (sddmm.hip).
int sddmm_rows_tile(int32_t F, int max_wide);
int sddmm_rows_launch(const int32_t *seg, const int32_t *row_order, int32_t n_rows, int32_t n_blocks, int32_t merge64,
                      int max_wide, const int32_t *col, const float *src, const float *dst, float *out,
                      int64_t src_bytes, int64_t dst_bytes, int32_t F, int32_t pitch, hipStream_t stream);
// The same schedule for the elementwise edge functions (op: FG_EDGE_ADD .. FG_EDGE_DIV), out [nnz, F].
int sddmm_rows_elementwise_launch(const int32_t *seg, const int32_t *row_order, int32_t n_rows, int32_t n_blocks,
                                  int32_t merge64, const int32_t *col, const float *src, const float *dst, float *out,
                                  int64_t src_bytes, int64_t dst_bytes, int32_t F, int op, hipStream_t stream);

// Generalised operators (general.hip): msg / reduce / op are the FG_MSG_* / FG_REDUCE_* / FG_EDGE_* codes.
int spmm_general_launch(const int32_t *row_order, const int32_t *seg, int32_t n_blocks, const int32_t *indices,
                        const float *vals, const float *feat, float *out, int32_t n_rows, int32_t F, int msg,
                        int reduce, hipStream_t stream);
// ... with H heads of D floats and per-edge per-head values vals [nnz, H]
int spmm_general_mh_launch(const int32_t *row_order, const int32_t *seg, int32_t n_blocks, const int32_t *indices,
                           const float *vals, const float *feat, float *out, int32_t n_rows, int32_t H, int32_t D,
                           int msg, int reduce, hipStream_t stream);
// out[r, :] /= degree of row r (rows without nonzeros stay 0): the last step of the mean over a sum
int spmm_mean_finish_launch(const int32_t *indptr, float *out, int32_t n_rows, int32_t F, hipStream_t stream);
int sddmm_elementwise_launch(const int32_t *row, const int32_t *col, const float *src, const float *dst, float *out,
                             int64_t nnz, int32_t F, int op, hipStream_t stream);

// Edge softmax over CSR rows, alone and fused into multi-head SDDMM (softmax.hip).
int edge_softmax_launch(const int32_t *indptr, const float *scores, float *out, int32_t n_rows, int32_t H,
                        hipStream_t stream);
bool sddmm_softmax_fused_applies(const float *src, const float *dst, int32_t H, int32_t D);
int sddmm_softmax_launch(const int32_t *row_order, const int32_t *indptr, const int32_t *indices, const float *src,
                         const float *dst, float *out, int32_t n_rows, int32_t H, int32_t D, hipStream_t stream);

// Pieces of the multi-head backward (backward.hip): gradient of the edge softmax, rows gathered through a
// permutation, elementwise sum.
int edge_softmax_backward_launch(const int32_t *indptr, const float *weights, const float *grad, float *out,
                                 int32_t n_rows, int32_t H, hipStream_t stream);
int permute_rows_launch(const int32_t *perm, const float *in, float *out, int64_t n, int32_t width, hipStream_t stream);
int add_launch(const float *a, const float *b, float *out, int64_t n, hipStream_t stream);
int pad_rows_launch(const float *in, float *out, int64_t n, int32_t F, int32_t pitch, hipStream_t stream);

// Multi-head SDDMM, edge softmax and multi-head SpMM as one kernel (attention.hip).
bool attention_fused_applies(const float *key, const float *query, const float *value, const float *out, int32_t H,
                             int32_t D);
int attention_launch(const int32_t *row_order, const int32_t *seg_lo, const int32_t *seg_hi, const int32_t *indices,
                     const float *key, const float *query, const float *value, float *out, int32_t n_rows, int32_t H,
                     int32_t D, hipStream_t stream);

inline bool aligned_to(const void *p, uintptr_t bytes) { return (reinterpret_cast<uintptr_t>(p) & (bytes - 1)) == 0; }

inline int pow2_ceil(int x) {
  int p = 1;
  while (p < x) p <<= 1;
  return p;
}

}  // namespace fg
