// C ABI of libfeatgraph_hip.so: argument validation, the SpMM row plan and
// the hand-off to the kernel launchers.  See include/featgraph_hip.h for the
// contract of every entry point.
#include <algorithm>
#include <cstdarg>
#include <cstdio>
#include <cstring>
#include <new>
#include <numeric>
#include <string>
#include <cstdlib>
#include <vector>

#include "common.hpp"

namespace fg {

namespace {
thread_local char g_error[512] = "";
Config g_config;
}  // namespace

int fail(int code, const char *fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_error, sizeof(g_error), fmt, ap);
  va_end(ap);
  return code;
}

Config &config() { return g_config; }

}  // namespace fg

struct fg_spmm_plan {
  int64_t n_rows, n_cols, nnz;
  const int32_t *indptr;   // borrowed, device
  const int32_t *indices;  // borrowed, device
  int32_t *row_order;      // owned, device: rows by descending degree
  int32_t max_degree;
  int device;
  // Row bounds in visiting order, optionally cut into column blocks:
  // seg[b * n_rows + i] is the position of the first nonzero of row row_order[i]
  // whose column id is >= b * block_cols, so block b of that row is
  // [seg[b][i], seg[b+1][i]) and the whole row is [seg[0][i], seg[n_blocks][i]).
  // n_blocks > 1 only when every row's column ids ascend.
  int32_t *seg;  // owned, device, (n_blocks + 1) * n_rows entries
  int32_t n_blocks;
  bool cols_unsorted = false;  // blocks were wanted but some row's column ids descend
  int32_t block_cols;
  // When the library sizes the blocks it may cut each block of the default width into `split` equal ones, so
  // that a kernel can take 1 .. split neighbouring blocks per pass; split_used is 1 when the caller sized them.
  int32_t split = 1, split_used = 1;
  // the library's own blocks come in a multiple of eight default-width passes (when there are seven or more), so
  // that passes pinned to the eight dies keep every die busy in every round
  bool xcd_round = false;
  int32_t requested_partitions;  // 0: library decides; 1: no column blocks; P > 1: P blocks, as the caller asked
  bool force_blocks;             // the caller's P > 1: use the blocks at every feature length
  // what the bounds table is built from: block width (0: default), blocks on / off / automatic (1 / 0 / -1),
  // and the nonzeros per (row, block) below which automatic mode keeps whole rows
  int32_t want_block_cols;
  int32_t default_block_cols;  // the library's own pass width for 64-float tiles when nobody sized the blocks
  int want_blocked;
  double min_per_segment;
  // Records of the several-rows-per-wave kernel: whole rows, and column-block passes for its tiles of 16, 32
  // and 64 floats (tables with the same blocks-per-pass share their records).
  fg::MultiRuns multi_whole;
  fg::MultiRuns multi_tile[3];
};

struct fg_sddmm_plan {
  int64_t nnz, n_rows, n_cols;
  const int32_t *row;  // borrowed, device
  const int32_t *col;  // borrowed, device
  bool force_blocks;   // the caller asked for column partitions: use them at every feature length
  int device = 0;      // the device that was current at creation
  fg::SddmmBlocks blocks;
  // Row-sorted lists (a COO list derived from CSR): the row pointer rebuilt from `row`, and a row plan over
  // it (visiting order + per-column-block bounds) for the row-run kernel.  Null otherwise.
  int32_t *indptr = nullptr;      // owned, device, n_rows + 1 entries
  fg_spmm_plan *rows = nullptr;   // owned
  // Any other list with valid ids: a copy sorted by (row, column), over which `indptr` and `rows` are then
  // built; the row-run kernel writes its results in that order and a gather returns them to the caller's.
  fg::SddmmSorted sorted;
  bool input_row_sorted = false;  // the caller's own list has ascending row ids (indptr then describes it too)
  const char *no_row_plan = nullptr;  // why the row pointer / row plan was not built, when it was skipped unchecked
};

static int row_plan_create(int64_t n_rows, int64_t n_cols, int64_t nnz, const int32_t *indptr, const int32_t *indices,
                           int32_t num_col_partitions, int32_t want_block_cols, int32_t default_block_cols,
                           int32_t split, int want_blocked, double min_per_segment, bool with_multi,
                           bool xcd_round, fg_spmm_plan **plan);

namespace {

__global__ void count_out_of_range_kernel(const int32_t *idx, int64_t n, int64_t bound, unsigned long long *n_bad) {
  const int64_t stride = static_cast<int64_t>(gridDim.x) * blockDim.x;
  unsigned long long bad = 0;
  for (int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x; i < n; i += stride) {
    const int64_t v = idx[i];
    bad += (v < 0 || v >= bound) ? 1u : 0u;
  }
  if (bad) atomicAdd(n_bad, bad);
}

// One wave per row: writes the bounds of every column block of row row_order[i]
// at position i, and raises *unsorted when two neighbouring column ids descend.
__global__ void build_segments_kernel(const int32_t *indptr, const int32_t *indices, const int32_t *row_order,
                                      int32_t n_rows, int32_t block_cols, int32_t n_blocks, int32_t *seg,
                                      int *unsorted) {
  const int i = blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
  const int lane = threadIdx.x & 63;
  if (i >= n_rows) return;
  const int row = row_order[i];
  const int start = indptr[row], end = indptr[row + 1];
  for (int e = start + lane; e <= end; e += 64) {  // e == end is the sentinel that closes the last blocks
    int bk = n_blocks, bp = -1;
    if (e < end) bk = min(max(indices[e] / block_cols, 0), n_blocks - 1);
    if (e > start) {
      bp = min(max(indices[e - 1] / block_cols, 0), n_blocks - 1);
      if (e < end && indices[e - 1] > indices[e]) atomicOr(unsorted, 1);
    }
    for (int b = bp + 1; b <= bk; ++b) seg[static_cast<int64_t>(b) * n_rows + i] = e;
  }
}

// Raises *bad when the row ids of an edge list descend somewhere or leave [0, n_rows).
__global__ void rows_sorted_kernel(const int32_t *row, int64_t nnz, int32_t n_rows, int *bad) {
  const int64_t stride = static_cast<int64_t>(gridDim.x) * blockDim.x;
  int b = 0;
  for (int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x; i < nnz; i += stride) {
    const int32_t r = row[i];
    b |= (r < 0 || r >= n_rows) ? 1 : 0;
    if (i + 1 < nnz) b |= row[i + 1] < r ? 1 : 0;
  }
  if (b) atomicOr(bad, 1);
}

// Row pointer of a row-sorted edge list: indptr[r] = number of edges whose row id is below r.
__global__ void indptr_from_rows_kernel(const int32_t *row, int64_t nnz, int32_t n_rows, int32_t *indptr) {
  const int64_t stride = static_cast<int64_t>(gridDim.x) * blockDim.x;
  for (int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x; i <= nnz; i += stride) {
    const int32_t prev = i > 0 ? row[i - 1] : -1;
    const int32_t cur = i < nnz ? row[i] : n_rows;
    for (int32_t r = prev + 1; r <= cur; ++r) indptr[r] = static_cast<int32_t>(i);
  }
}

// A plan's arrays live on the device that was current when it was built; launching with another device
// current would hand kernels on that device pointers into this one's memory.
int check_device(int plan_device) {
  int now = -1;
  FG_HIP_TRY(hipGetDevice(&now));
  if (now != plan_device)
    return fg::fail(FG_EINVAL, "the plan was built on device %d but device %d is current", plan_device, now);
  return FG_OK;
}

// Default pass widths, in columns, for tiles of 64 floats (narrower tiles take proportionally more columns, so the
// band of the feature matrix that a pass gathers from keeps its size).  One XCD's L2 is 4 MB = 16384 such rows.
// SDDMM is fastest with the band at that size; SpMM, which pays a read and a write of every row's partial sum
// per pass, with a band a quarter larger and correspondingly fewer passes (232,965-vertex graph, 64 floats:
// 12 passes of 19,414 columns 1.86 ms, 15 of 15,532 1.95 ms, 9 of 25,885 1.98 ms).
constexpr int32_t kSpmmBlockCols = 20480;
constexpr int32_t kSddmmBlockCols = 16384;
// The SDDMM row plan cuts each of those blocks in two: a pass of the row-run kernel takes both halves for a
// 64-float tile and one for a 128-float tile, so the band it gathers from stays 4 MB.
constexpr int32_t kSddmmSplit = 2;

int check_heads(int32_t H, int32_t D) {
  if (H < 1 || D < 1) return fg::fail(FG_EINVAL, "H = %d and D = %d must both be positive", H, D);
  if (static_cast<int64_t>(H) * D > (1 << 20))
    return fg::fail(FG_EUNSUPPORTED, "H*D = %lld exceeds 2^20 floats per vertex", (long long)H * D);
  return FG_OK;
}

int spmm_prepare(const fg_spmm_plan *plan, const float *feat, const float *w, float *out, int32_t H, int32_t D,
                 int32_t feat_tiles, fg::SpmmArgs *a, fg::SpmmShape *s) {
  if (!plan) return fg::fail(FG_EINVAL, "plan is null");
  if (int rc = check_heads(H, D)) return rc;
  if (int rc = check_device(plan->device)) return rc;
  if (feat_tiles < 0) return fg::fail(FG_EINVAL, "feat_tiles = %d is negative", feat_tiles);
  if (plan->n_rows > 0 && !out) return fg::fail(FG_EINVAL, "out is null");
  if (plan->nnz > 0 && (!feat || !w)) return fg::fail(FG_EINVAL, "feat or edge values are null");
  a->indptr = plan->indptr;
  a->indices = plan->indices;
  a->w = w;
  a->feat = feat;
  a->out = out;
  a->row_order = (fg::config().spmm_sorted == 0) ? nullptr : plan->row_order;
  if (a->row_order && plan->seg) {  // whole rows, in visiting order
    a->seg_lo = plan->seg;
    a->seg_hi = plan->seg + static_cast<int64_t>(plan->n_blocks) * plan->n_rows;
  }
  a->n_rows = static_cast<int32_t>(plan->n_rows);
  a->n_cols = static_cast<int32_t>(plan->n_cols);
  a->F = H * D;
  a->H = H;
  a->D = D;
  *s = fg::spmm_choose_shape(*a, feat_tiles);
  a->n_tiles = (a->F + s->tile_width() - 1) / s->tile_width();
  a->n_slots = static_cast<int64_t>(a->n_tiles) * a->n_rows;
  return FG_OK;
}

bool use_column_blocks(const fg_spmm_plan *plan, const fg::SpmmArgs &a, const fg::SpmmShape &s) {
  if (!plan->seg || plan->n_blocks < 2 || !a.row_order) return false;
  if (plan->force_blocks) return true;
  if (fg::config().spmm_blocked == 0) return false;
  if (fg::config().spmm_blocked > 0) return true;
  // worthwhile only while the whole gathered band does not fit an L2 anyway
  const int64_t band_bytes = static_cast<int64_t>(plan->n_cols) * std::min<int64_t>(s.tile_width(), a.F) * 4;
  if (a.F < 64) return false;  // short feature rows: the single pass is faster (measured at 32 floats)
  return band_bytes > (int64_t{6} << 20);
}

int multi_tile_index(int tile) { return tile == 16 ? 0 : tile == 32 ? 1 : 2; }

// Column blocks of the plan's table that one pass of the several-rows-per-wave kernel takes together, for
// tiles of `tile` floats: the band of the feature matrix that a pass gathers from (block width x tile bytes)
// should stay about one L2 (4 MB), so narrower tiles take wider blocks; blocks that the caller sized
// (partition count, spmm.block_cols) are used as they are.
int multi_merge(const fg_spmm_plan *plan, int tile) {
  if (plan->n_blocks < 2) return 1;
  if (plan->force_blocks || plan->want_block_cols > 0) return 1;
  return std::min(64 / tile, plan->n_blocks);  // the table's blocks are sized for 64-float tiles
}

int multi_build(fg_spmm_plan *p) {
  if (fg::config().spmm_multi == 0 || !p->seg || !p->row_order || p->n_rows == 0) return FG_OK;
  const int32_t n = static_cast<int32_t>(p->n_rows);
  if (int rc = fg::multi_runs_build(p->seg, p->row_order, p->indices, p->nnz, n, p->n_blocks, p->n_blocks, &p->multi_whole))
    return rc;
  if (p->n_blocks < 2) return FG_OK;
  const int tiles[3] = {16, 32, 64};
  for (int t = 0; t < 3; ++t) {
    const int merge = multi_merge(p, tiles[t]);
    if (merge >= p->n_blocks) continue;  // one pass: the whole-row records
    // 16 bytes per row and pass: with very many passes (a caller's large partition count on a thin matrix) the
    // records would dwarf the matrix itself; such plans keep the bounds table and the wave-per-row kernels
    const int64_t passes = (p->n_blocks + merge - 1) / merge;
    if (passes * p->n_rows * 16 > std::max<int64_t>(4 * p->nnz * 8, int64_t{256} << 20)) continue;
    bool shared = false;
    for (int u = 0; u < t && !shared; ++u)
      if (p->multi_tile[u].rec && p->multi_tile[u].merge == merge) {
        p->multi_tile[t] = p->multi_tile[u];
        shared = true;
      }
    if (!shared)
      if (int rc = fg::multi_runs_build(p->seg, p->row_order, p->indices, p->nnz, n, p->n_blocks, merge, &p->multi_tile[t]))
        return rc;
  }
  return FG_OK;
}

void multi_free(fg_spmm_plan *p) {
  for (int t = 0; t < 3; ++t) {
    for (int u = t + 1; u < 3; ++u)
      if (p->multi_tile[u].rec && p->multi_tile[u].rec == p->multi_tile[t].rec) p->multi_tile[u] = fg::MultiRuns();
    fg::multi_runs_free(&p->multi_tile[t]);
  }
  fg::multi_runs_free(&p->multi_whole);
}

// The records that a call uses: null when the kernel does not take the call.  The kernel is the default
// wherever it applies; an explicit launch shape (tuning keys, the caller's feature tiling) asks for the
// row-slot / wave-per-row kernels.
const fg::MultiRuns *multi_table(const fg_spmm_plan *plan, const fg::SpmmArgs &a, int32_t feat_tiles) {
  const fg::Config &c = fg::config();
  if (c.spmm_multi == 0 || !fg::spmm_multi_applies(a) || !plan->multi_whole.rec) return nullptr;
  if (c.spmm_multi < 0 && !(feat_tiles == 0 && c.spmm_vec == 0 && c.spmm_lpr == 0 && c.spmm_unroll == 0 &&
                            c.spmm_pipeline < 0 && c.spmm_sorted != 0))
    return nullptr;
  const int tile = fg::spmm_multi_tile(a.F);
  const fg::MultiRuns *blocked = &plan->multi_tile[multi_tile_index(tile)];
  if (plan->force_blocks && plan->n_blocks >= 2)  // the caller's blocks: the kernels that have them
    return blocked->rec && blocked->passes >= 2 ? blocked : nullptr;
  if (!blocked->rec || blocked->passes < 2) return &plan->multi_whole;
  if (c.spmm_blocked == 0) return &plan->multi_whole;
  const int64_t band_bytes = static_cast<int64_t>(plan->n_cols) * std::min<int>(tile, a.F) * 4;
  if (c.spmm_blocked < 0 && band_bytes <= (int64_t{6} << 20)) return &plan->multi_whole;  // fits an L2 anyway
  return blocked;
}

// Tiles whose workgroups alternate along grid.x.  Workgroups go to the XCDs round-robin, so with two tiles in
// turn half of the XCDs work on each and an L2 holds one tile's band; the two tiles read the same ids, values
// and records at about the same time.  Measured on the 232,965-vertex graph at 128 / 256 / 512 floats:
// 3.57 / 7.11 / 14.16 ms with pairs, 3.70 / 7.36 / 14.57 ms with tiles one after the other in one launch,
// 3.78 / 7.72 / 15.23 ms with one launch per tile and pass; four tiles in turn are slower again.
int multi_interleave(int n_tiles) {
  const int want = fg::config().spmm_tile_interleave;
  const int il = want > 0 ? want : 2;
  return (il > 1 && n_tiles % il == 0) ? il : 1;
}

// Feature rows of several 64-float tiles whose rest is 1 .. 32 floats: the rest runs as a tile of 16 or 32 floats
// (4 or 8 lanes per row, so 16 or 8 rows per wave) over the same records and passes, instead of a 64-float tile
// with most of its lanes idle (the 232,965-vertex graph at 65 / 72 / 96 floats: 4.1 / 3.4 / 3.4 ms with a 64-float
// rest tile).  0: no such rest.
int multi_tail_tile(int32_t F) {
  if (fg::spmm_multi_tile(F) != 64 || F < 64) return 0;
  const int rest = F % 64;
  return rest == 0 || rest > 32 ? 0 : rest <= 16 ? 16 : 32;
}

int multi_run(const fg_spmm_plan *plan, const fg::MultiRuns *runs, fg::SpmmArgs a, hipStream_t st) {
  if (runs->ids_p) {  // the records index the re-laid ids and say where each run's values start in the CSR array
    a.indices = runs->ids_p;
    a.vals_by_csr = 1;
  }
  const int tile = fg::spmm_multi_tile(a.F);
  const int n_tiles = (a.F + tile - 1) / tile;
  const int64_t n = plan->n_rows;
  auto long_split = [&](int pass) {
    a.long_runs = runs->long_runs[pass];
    a.long_blocks = std::min(a.long_runs, 2048);  // one workgroup per long run at a time
  };
  if (runs->passes == 1 && multi_tail_tile(a.F) == 0) {
    a.runs = runs->rec;
    long_split(0);
    a.tile_base = 0;
    a.n_tiles = n_tiles;
    a.accumulate = 0;
    return fg::spmm_multi_launch(a, st);
  }
  // one launch per pass, passes in ascending column order: launches on a stream run one after the other, so
  // every row's sum still grows in CSR order, carried from pass to pass in `out`.  A launch covers every feature
  // tile: workgroups are dispatched tile pair after tile pair, so the resident waves gather from one or two
  // tiles' bands at a time, a pair's tail overlaps the next pair's head, and there are n_tiles times fewer
  // launch boundaries than with a launch per (tile, pass).
  const int tail = multi_tail_tile(a.F);
  const int main_tiles = tail ? n_tiles - 1 : n_tiles;
  for (int b = 0; b < runs->passes; ++b) {
    a.runs = runs->rec + static_cast<int64_t>(b) * n;
    long_split(b);
    a.accumulate = b > 0;
    a.multi_tile = 0;
    a.tile_base = 0;
    a.n_tiles = main_tiles;
    a.interleave_tiles = multi_interleave(main_tiles);
    if (int rc = fg::spmm_multi_launch(a, st)) return rc;
    if (tail) {  // the same pass, the same records, fewer lanes per row
      a.multi_tile = tail;
      a.tile_base = main_tiles * (tile / tail);
      a.n_tiles = 1;
      a.interleave_tiles = 1;
      if (int rc = fg::spmm_multi_launch(a, st)) return rc;
    }
  }
  return FG_OK;
}

// n_rows / n_cols: matrix extents when known (a plan knows them), else 0.
int sddmm_prepare(int64_t nnz, const int32_t *row, const int32_t *col, const float *src, const float *dst,
                  float *out, int32_t H, int32_t D, fg::SddmmArgs *a, fg::SddmmShape *s, int64_t n_rows = 0,
                  int64_t n_cols = 0) {
  if (nnz < 0) return fg::fail(FG_EINVAL, "nnz = %lld is negative", (long long)nnz);
  if (int rc = check_heads(H, D)) return rc;
  if (nnz > 0 && (!row || !col || !src || !dst || !out)) return fg::fail(FG_EINVAL, "a data pointer is null");
  a->row = row;
  a->col = col;
  a->src = src;
  a->dst = dst;
  a->out = out;
  a->n_ve = nnz * H;
  a->H = H;
  a->D = D;
  a->stride = H * D;
  if (n_rows > 0) a->dst_bytes = n_rows * H * D * 4;
  if (n_cols > 0) a->src_bytes = n_cols * H * D * 4;
  *s = fg::sddmm_choose_shape(*a);
  a->batches = s->batches;
  return FG_OK;
}

// Builds the plan's bounds table.  Column blocks (n_blocks > 1) pay off when
// the band of the feature matrix that one block gathers from (block_cols rows
// of one 64-float tile, 4 MB by default) is about one XCD's L2 while the whole
// matrix does not, and when a row still has enough nonzeros per block to
// amortise re-reading its partial sum; otherwise the table holds whole rows.
int build_bounds(fg_spmm_plan *p) {
  if (p->n_rows == 0) return FG_OK;
  int64_t block_cols = p->want_block_cols > 0 ? p->want_block_cols : p->default_block_cols;
  const int P = p->requested_partitions;
  if (P > 1) block_cols = std::max<int64_t>(1, (p->n_cols + P - 1) / P);  // util/adj_partitioning.py:42
  int64_t n_blocks = p->n_cols > 0 ? (p->n_cols + block_cols - 1) / block_cols : 1;
  // whether blocks pay is judged at the default width, before any split
  const double per_segment =
      n_blocks > 0 ? static_cast<double>(p->nnz) / (static_cast<double>(p->n_rows) * n_blocks) : 0.0;
  // the library's own blocks: as many as the default width asks for (times the split), all of the same width
  p->split_used = 1;
  if (P <= 1 && p->want_block_cols <= 0 && n_blocks > 1) {
    if (p->xcd_round && n_blocks >= fg::kXcds - 1) n_blocks = (n_blocks + fg::kXcds - 1) / fg::kXcds * fg::kXcds;
    p->split_used = std::max(1, p->split);
    n_blocks *= p->split_used;
    block_cols = (p->n_cols + n_blocks - 1) / n_blocks;
  }
  if (P == 1 || n_blocks < 2 || p->nnz == 0)
    n_blocks = 1;
  else if (P == 0 && (p->want_blocked == 0 || (p->want_blocked < 0 && per_segment < p->min_per_segment)))
    n_blocks = 1;
  p->force_blocks = P > 1;
  int *flag = nullptr;
  FG_HIP_TRY(hipMalloc(&flag, sizeof(int)));
  for (;;) {
    if (n_blocks == 1) block_cols = 0x7fffffff, p->split_used = 1;
    int32_t *seg = nullptr;
    hipError_t err = hipMalloc(&seg, static_cast<size_t>(n_blocks + 1) * p->n_rows * sizeof(int32_t));
    if (err == hipErrorOutOfMemory && n_blocks > 1) {  // no room for the blocks: whole rows only
      (void)hipGetLastError();
      n_blocks = 1;
      continue;
    }
    int unsorted = 0;
    if (err == hipSuccess) err = hipMemset(flag, 0, sizeof(int));
    if (err == hipSuccess) {
      const int rows_per_block = 4;
      const unsigned grid = static_cast<unsigned>((p->n_rows + rows_per_block - 1) / rows_per_block);
      build_segments_kernel<<<dim3(grid), dim3(64 * rows_per_block)>>>(
          p->indptr, p->indices, p->row_order, static_cast<int32_t>(p->n_rows), static_cast<int32_t>(block_cols),
          static_cast<int32_t>(n_blocks), seg, flag);
      err = hipGetLastError();
    }
    if (err == hipSuccess) err = hipMemcpy(&unsorted, flag, sizeof(int), hipMemcpyDeviceToHost);
    if (err != hipSuccess) {
      if (seg) (void)hipFree(seg);
      (void)hipFree(flag);
      return fg::fail(err == hipErrorOutOfMemory ? FG_ENOMEM : FG_EHIP, "row bounds construction: %s",
                      hipGetErrorString(err));
    }
    if (unsorted && n_blocks > 1) {  // blocks would reorder the sums of such rows
      (void)hipFree(seg);
      n_blocks = 1;
      p->cols_unsorted = true;
      continue;
    }
    p->seg = seg;
    p->n_blocks = static_cast<int32_t>(n_blocks);
    p->block_cols = static_cast<int32_t>(block_cols);
    break;
  }
  (void)hipFree(flag);
  return FG_OK;
}

int *config_slot(const char *key) {
  fg::Config &c = fg::config();
  if (!key) return nullptr;
  if (!strcmp(key, "spmm.vec")) return &c.spmm_vec;
  if (!strcmp(key, "spmm.lpr")) return &c.spmm_lpr;
  if (!strcmp(key, "spmm.unroll")) return &c.spmm_unroll;
  if (!strcmp(key, "spmm.sorted")) return &c.spmm_sorted;
  if (!strcmp(key, "spmm.blocked")) return &c.spmm_blocked;
  if (!strcmp(key, "spmm.block_cols")) return &c.spmm_block_cols;
  if (!strcmp(key, "spmm.pipeline")) return &c.spmm_pipeline;
  if (!strcmp(key, "spmm.buffer_loads")) return &c.spmm_buffer_loads;
  if (!strcmp(key, "spmm.pipe_blocks")) return &c.spmm_pipe_blocks;
  if (!strcmp(key, "spmm.multi")) return &c.spmm_multi;
  if (!strcmp(key, "spmm.multi_blocks")) return &c.spmm_multi_blocks;
  if (!strcmp(key, "spmm.multi_long")) return &c.spmm_multi_long;
  if (!strcmp(key, "spmm.tile_interleave")) return &c.spmm_tile_interleave;
  if (!strcmp(key, "spmm.relay")) return &c.spmm_relay;
  if (!strcmp(key, "spmm.general_multi")) return &c.spmm_general_multi;
  if (!strcmp(key, "sddmm.group")) return &c.sddmm_group;
  if (!strcmp(key, "sddmm.batches")) return &c.sddmm_batches;
  if (!strcmp(key, "sddmm.blocked")) return &c.sddmm_blocked;
  if (!strcmp(key, "sddmm.block_cols")) return &c.sddmm_block_cols;
  if (!strcmp(key, "sddmm.fast")) return &c.sddmm_fast;
  if (!strcmp(key, "sddmm.buffer_loads")) return &c.sddmm_buffer_loads;
  if (!strcmp(key, "sddmm.rows")) return &c.sddmm_rows;
  if (!strcmp(key, "sddmm.rows_blocks")) return &c.sddmm_rows_blocks;
  if (!strcmp(key, "sddmm.rows_wide")) return &c.sddmm_rows_wide;
  if (!strcmp(key, "sddmm.sorted_copy")) return &c.sddmm_sorted_copy;
  if (!strcmp(key, "sddmm.regroup")) return &c.sddmm_regroup;
  if (!strcmp(key, "sddmm.xcd")) return &c.sddmm_xcd;
  if (!strcmp(key, "spmm.xcd")) return &c.spmm_xcd;
  if (!strcmp(key, "spmm.pad_rows")) return &c.spmm_pad_rows;
  if (!strcmp(key, "attention.blocks")) return &c.attention_blocks;
  return nullptr;
}

// FEATGRAPH_HIP_CONFIG="key=value,key=value" applies fg_config_set pairs when the
// library is loaded (handy under a profiler, where nothing else can reach in).
struct EnvConfig {
  EnvConfig() {
    const char *env = getenv("FEATGRAPH_HIP_CONFIG");
    if (!env) return;
    std::string text(env);
    size_t pos = 0;
    while (pos < text.size()) {
      size_t stop = text.find(',', pos);
      if (stop == std::string::npos) stop = text.size();
      const std::string item = text.substr(pos, stop - pos);
      const size_t eq = item.find('=');
      if (eq != std::string::npos) {
        if (fg_config_set(item.substr(0, eq).c_str(), atoi(item.c_str() + eq + 1)) != FG_OK)
          fprintf(stderr, "libfeatgraph_hip: ignoring FEATGRAPH_HIP_CONFIG item '%s'\n", item.c_str());
      }
      pos = stop + 1;
    }
  }
};

}  // namespace

extern "C" {

int fg_version(void) { return 100; }

const char *fg_last_error(void) { return fg::g_error; }

int fg_spmm_plan_create(int64_t n_rows, int64_t n_cols, int64_t nnz, const int32_t *indptr, const int32_t *indices,
                        fg_spmm_plan **plan) {
  return fg_spmm_plan_create_partitioned(n_rows, n_cols, nnz, indptr, indices, 0, plan);
}

int fg_spmm_plan_create_partitioned(int64_t n_rows, int64_t n_cols, int64_t nnz, const int32_t *indptr,
                                    const int32_t *indices, int32_t num_col_partitions, fg_spmm_plan **plan) {
  return row_plan_create(n_rows, n_cols, nnz, indptr, indices, num_col_partitions, fg::config().spmm_block_cols,
                         kSpmmBlockCols, 1, fg::config().spmm_blocked, 8.0, true, false, plan);
}

// want_block_cols / want_blocked / min_per_segment: see fg_spmm_plan; with_multi: also build the records of the
// several-rows-per-wave kernel.
static int row_plan_create(int64_t n_rows, int64_t n_cols, int64_t nnz, const int32_t *indptr, const int32_t *indices,
                           int32_t num_col_partitions, int32_t want_block_cols, int32_t default_block_cols,
                           int32_t split, int want_blocked, double min_per_segment, bool with_multi,
                           bool xcd_round, fg_spmm_plan **plan) {
  if (!plan) return fg::fail(FG_EINVAL, "plan output pointer is null");
  *plan = nullptr;
  if (num_col_partitions < 0)
    return fg::fail(FG_EINVAL, "num_col_partitions = %d is negative", num_col_partitions);
  if (n_rows < 0 || n_cols < 0 || nnz < 0)
    return fg::fail(FG_EINVAL, "negative size (n_rows=%lld n_cols=%lld nnz=%lld)", (long long)n_rows,
                    (long long)n_cols, (long long)nnz);
  if (n_rows >= 0x7fffffffLL || n_cols > 0x7fffffffLL || nnz > 0x7fffffffLL)
    return fg::fail(FG_EUNSUPPORTED, "sizes beyond int32 indexing are not supported");
  if (!indptr) return fg::fail(FG_EINVAL, "indptr is null");
  if (nnz > 0 && !indices) return fg::fail(FG_EINVAL, "indices is null");
  if (nnz > 0 && n_cols == 0) return fg::fail(FG_EINVAL, "nnz > 0 with n_cols = 0");

  std::vector<int32_t> host_indptr, order;
  try {
    host_indptr.resize(static_cast<size_t>(n_rows) + 1);
    order.resize(static_cast<size_t>(n_rows));
  } catch (const std::bad_alloc &) {
    return fg::fail(FG_ENOMEM, "host allocation for %lld rows failed", (long long)n_rows);
  }
  FG_HIP_TRY(hipMemcpy(host_indptr.data(), indptr, sizeof(int32_t) * (n_rows + 1), hipMemcpyDeviceToHost));
  if (host_indptr[0] != 0) return fg::fail(FG_EINVAL, "indptr[0] = %d, expected 0", host_indptr[0]);
  int32_t max_degree = 0;
  for (int64_t r = 0; r < n_rows; ++r) {
    const int64_t d = static_cast<int64_t>(host_indptr[r + 1]) - host_indptr[r];
    if (d < 0) return fg::fail(FG_EINVAL, "indptr decreases at row %lld", (long long)r);
    max_degree = std::max<int64_t>(max_degree, d);
  }
  if (host_indptr[n_rows] != nnz)
    return fg::fail(FG_EINVAL, "indptr[n_rows] = %d, expected nnz = %lld", host_indptr[n_rows], (long long)nnz);

  // Rows by descending degree; equal degrees keep ascending row ids, so the
  // list is a pure function of indptr.
  std::iota(order.begin(), order.end(), 0);
  const int32_t *ip = host_indptr.data();
  std::stable_sort(order.begin(), order.end(),
                   [ip](int32_t x, int32_t y) { return ip[x + 1] - ip[x] > ip[y + 1] - ip[y]; });

  fg_spmm_plan *p = new (std::nothrow) fg_spmm_plan();
  if (!p) return fg::fail(FG_ENOMEM, "plan allocation failed");
  p->n_rows = n_rows;
  p->n_cols = n_cols;
  p->nnz = nnz;
  p->indptr = indptr;
  p->indices = indices;
  p->row_order = nullptr;
  p->requested_partitions = num_col_partitions;
  p->force_blocks = false;
  p->want_block_cols = want_block_cols;
  p->default_block_cols = default_block_cols;
  p->split = split;
  p->xcd_round = xcd_round;
  p->want_blocked = want_blocked;
  p->min_per_segment = min_per_segment;
  p->max_degree = max_degree;
  p->device = 0;
  hipError_t err = hipGetDevice(&p->device);
  if (err == hipSuccess && n_rows > 0) err = hipMalloc(&p->row_order, sizeof(int32_t) * n_rows);
  if (err == hipSuccess && n_rows > 0)
    err = hipMemcpy(p->row_order, order.data(), sizeof(int32_t) * n_rows, hipMemcpyHostToDevice);
  if (err != hipSuccess) {
    if (p->row_order) (void)hipFree(p->row_order);
    delete p;
    return fg::fail(err == hipErrorOutOfMemory ? FG_ENOMEM : FG_EHIP, "plan upload: %s", hipGetErrorString(err));
  }
  p->seg = nullptr;
  p->n_blocks = 0;
  p->block_cols = 0;
  int rc = build_bounds(p);
  if (rc == FG_OK && with_multi) rc = multi_build(p);
  if (rc != FG_OK) {
    fg_spmm_plan_destroy(p);
    return rc;
  }
  *plan = p;
  return FG_OK;
}

void fg_spmm_plan_destroy(fg_spmm_plan *plan) {
  if (!plan) return;
  if (plan->row_order) (void)hipFree(plan->row_order);
  if (plan->seg) (void)hipFree(plan->seg);
  multi_free(plan);
  delete plan;
}

int fg_spmm_plan_row_order(const fg_spmm_plan *plan, int32_t *row_order_host, int32_t *max_degree) {
  if (!plan) return fg::fail(FG_EINVAL, "plan is null");
  if (max_degree) *max_degree = plan->max_degree;
  if (row_order_host && plan->n_rows > 0)
    FG_HIP_TRY(hipMemcpy(row_order_host, plan->row_order, sizeof(int32_t) * plan->n_rows, hipMemcpyDeviceToHost));
  return FG_OK;
}

int fg_spmm_csr_f32(const fg_spmm_plan *plan, const float *feat, const float *vals, float *out, int32_t F,
                    int32_t feat_tiles, void *stream) {
  return fg_spmm_csr_mh_f32(plan, feat, vals, out, 1, F, feat_tiles, stream);
}

int fg_spmm_csr_mh_f32(const fg_spmm_plan *plan, const float *feat, const float *w, float *out, int32_t H, int32_t D,
                       int32_t feat_tiles, void *stream) {
  fg::SpmmArgs a;
  fg::SpmmShape s;
  if (int rc = spmm_prepare(plan, feat, w, out, H, D, feat_tiles, &a, &s)) return rc;
  hipStream_t st = static_cast<hipStream_t>(stream);
  if (const fg::MultiRuns *runs = multi_table(plan, a, feat_tiles)) return multi_run(plan, runs, a, st);
  if (!use_column_blocks(plan, a, s)) return fg::spmm_launch(a, s, st);
  // One launch per (feature tile, column block), blocks in ascending column
  // order: launches on one stream run one after the other, so every row's sum
  // still grows in CSR order, carried from block to block in `out`.
  const int n_tiles = a.n_tiles;
  a.n_tiles = 1;
  a.n_slots = a.n_rows;
  for (int tile = 0; tile < n_tiles; ++tile) {
    a.tile_base = tile;
    for (int b = 0; b < plan->n_blocks; ++b) {
      a.seg_lo = plan->seg + static_cast<int64_t>(b) * plan->n_rows;
      a.seg_hi = a.seg_lo + plan->n_rows;
      a.accumulate = b > 0;
      if (int rc = fg::spmm_launch(a, s, st)) return rc;
    }
  }
  return FG_OK;
}

int fg_spmm_csr_pitched_f32(const fg_spmm_plan *plan, const float *feat, int32_t feat_pitch, const float *vals,
                            float *out, int32_t F, void *stream) {
  if (feat_pitch < F || feat_pitch % 4 != 0)
    return fg::fail(FG_EINVAL, "feat_pitch = %d must be a multiple of 4 and at least F = %d", feat_pitch, F);
  fg::SpmmArgs a;
  fg::SpmmShape s;
  if (int rc = spmm_prepare(plan, feat, vals, out, 1, F, 0, &a, &s)) return rc;
  const fg::MultiRuns *runs = multi_table(plan, a, 0);
  if (!runs) return fg::fail(FG_EUNSUPPORTED, "only the several-rows-per-wave kernel reads feature rows at a pitch of their own");
  a.feat_pitch = feat_pitch;
  return multi_run(plan, runs, a, static_cast<hipStream_t>(stream));
}

int fg_pad_rows_f32(int64_t n, int32_t F, int32_t pitch, const float *in, float *out, void *stream) {
  if (n < 0 || F < 1 || pitch < F) return fg::fail(FG_EINVAL, "need n >= 0 and 1 <= F <= pitch");
  if (n == 0) return FG_OK;
  if (!in || !out) return fg::fail(FG_EINVAL, "a data pointer is null");
  return fg::pad_rows_launch(in, out, n, F, pitch, static_cast<hipStream_t>(stream));
}

int fg_spmm_csr_general_f32(const fg_spmm_plan *plan, const float *feat, const float *vals, float *out, int32_t F,
                            int32_t msg, int32_t reduce, void *stream) {
  if (!plan) return fg::fail(FG_EINVAL, "plan is null");
  if (int rc = check_heads(1, F)) return rc;
  if (int rc = check_device(plan->device)) return rc;
  if (msg < FG_MSG_MUL || msg > FG_MSG_COPY_U) return fg::fail(FG_EINVAL, "msg = %d is not an FG_MSG_* code", msg);
  if (reduce < FG_REDUCE_SUM || reduce > FG_REDUCE_MEAN)
    return fg::fail(FG_EINVAL, "reduce = %d is not an FG_REDUCE_* code", reduce);
  if (plan->n_rows > 0 && !out) return fg::fail(FG_EINVAL, "out is null");
  if (plan->nnz > 0 && (!feat || (!vals && msg != FG_MSG_COPY_U)))
    return fg::fail(FG_EINVAL, "feat or edge values are null");
  if (plan->n_rows == 0) return FG_OK;
  hipStream_t st = static_cast<hipStream_t>(stream);
  // The several-rows-per-wave kernel takes the call where it would take the plain operator: same records, same
  // passes, the message and the reducer in place of the multiply-add; the mean is the sum followed by one
  // division per element.
  if (plan->nnz > 0 && fg::config().spmm_general_multi != 0) {
    fg::SpmmArgs a;
    fg::SpmmShape s;
    if (int rc = spmm_prepare(plan, feat, vals ? vals : feat, out, 1, F, 0, &a, &s)) return rc;
    a.reduce = reduce == FG_REDUCE_MEAN ? FG_REDUCE_SUM : reduce;
    a.msg = msg;
    const fg::MultiRuns *runs = multi_table(plan, a, 0);
    if (runs && fg::spmm_multi_general_applies(a)) {
      if (int rc = multi_run(plan, runs, a, st)) return rc;
      if (reduce == FG_REDUCE_MEAN)
        return fg::spmm_mean_finish_launch(plan->indptr, out, static_cast<int32_t>(plan->n_rows), F, st);
      return FG_OK;
    }
  }
  return fg::spmm_general_launch(plan->row_order, plan->seg, plan->n_blocks, plan->indices, vals, feat, out,
                                 static_cast<int32_t>(plan->n_rows), F, msg, reduce, st);
}

int fg_spmm_csr_mh_general_f32(const fg_spmm_plan *plan, const float *feat, const float *w, float *out, int32_t H,
                               int32_t D, int32_t msg, int32_t reduce, void *stream) {
  if (H == 1) return fg_spmm_csr_general_f32(plan, feat, w, out, D, msg, reduce, stream);
  if (!plan) return fg::fail(FG_EINVAL, "plan is null");
  if (int rc = check_heads(H, D)) return rc;
  if (int rc = check_device(plan->device)) return rc;
  if (msg < FG_MSG_MUL || msg > FG_MSG_COPY_U) return fg::fail(FG_EINVAL, "msg = %d is not an FG_MSG_* code", msg);
  if (reduce < FG_REDUCE_SUM || reduce > FG_REDUCE_MEAN)
    return fg::fail(FG_EINVAL, "reduce = %d is not an FG_REDUCE_* code", reduce);
  if (plan->n_rows > 0 && !out) return fg::fail(FG_EINVAL, "out is null");
  if (plan->nnz > 0 && (!feat || (!w && msg != FG_MSG_COPY_U)))
    return fg::fail(FG_EINVAL, "feat or edge weights are null");
  if (plan->n_rows == 0) return FG_OK;
  return fg::spmm_general_mh_launch(plan->row_order, plan->seg, plan->n_blocks, plan->indices, w, feat, out,
                                    static_cast<int32_t>(plan->n_rows), H, D, msg, reduce,
                                    static_cast<hipStream_t>(stream));
}

int fg_edge_softmax_backward_csr_f32(int64_t n_rows, const int32_t *indptr, const float *weights, const float *grad,
                                     float *out, int32_t H, void *stream) {
  if (n_rows < 0 || n_rows >= 0x7fffffffLL) return fg::fail(FG_EINVAL, "n_rows = %lld is out of range", (long long)n_rows);
  if (H < 1 || H > (1 << 20)) return fg::fail(FG_EINVAL, "H = %d is out of range", H);
  if (n_rows == 0) return FG_OK;
  if (!indptr || !weights || !grad || !out) return fg::fail(FG_EINVAL, "a data pointer is null");
  return fg::edge_softmax_backward_launch(indptr, weights, grad, out, static_cast<int32_t>(n_rows), H,
                                          static_cast<hipStream_t>(stream));
}

int fg_permute_rows_f32(int64_t n, int32_t width, const int32_t *perm, const float *in, float *out, void *stream) {
  if (n < 0) return fg::fail(FG_EINVAL, "n = %lld is negative", (long long)n);
  if (width < 1 || width > (1 << 20)) return fg::fail(FG_EINVAL, "width = %d is out of range", width);
  if (n == 0) return FG_OK;
  if (!perm || !in || !out) return fg::fail(FG_EINVAL, "a data pointer is null");
  return fg::permute_rows_launch(perm, in, out, n, width, static_cast<hipStream_t>(stream));
}

int fg_add_f32(int64_t n, const float *a, const float *b, float *out, void *stream) {
  if (n < 0) return fg::fail(FG_EINVAL, "n = %lld is negative", (long long)n);
  if (n == 0) return FG_OK;
  if (!a || !b || !out) return fg::fail(FG_EINVAL, "a data pointer is null");
  return fg::add_launch(a, b, out, n, static_cast<hipStream_t>(stream));
}

int fg_sddmm_coo_general_f32(int64_t nnz, const int32_t *row, const int32_t *col, const float *src, const float *dst,
                             float *out, int32_t F, int32_t edge_op, void *stream) {
  if (edge_op == FG_EDGE_DOT) return fg_sddmm_coo_f32(nnz, row, col, src, dst, out, F, stream);
  if (edge_op < FG_EDGE_DOT || edge_op > FG_EDGE_DIV)
    return fg::fail(FG_EINVAL, "edge_op = %d is not an FG_EDGE_* code", edge_op);
  if (nnz < 0) return fg::fail(FG_EINVAL, "nnz = %lld is negative", (long long)nnz);
  if (int rc = check_heads(1, F)) return rc;
  if (nnz > 0 && (!row || !col || !src || !dst || !out)) return fg::fail(FG_EINVAL, "a data pointer is null");
  return fg::sddmm_elementwise_launch(row, col, src, dst, out, nnz, F, edge_op, static_cast<hipStream_t>(stream));
}

int fg_sddmm_coo_f32(int64_t nnz, const int32_t *row, const int32_t *col, const float *src, const float *dst,
                     float *out, int32_t F, void *stream) {
  return fg_sddmm_coo_mh_f32(nnz, row, col, src, dst, out, 1, F, stream);
}

int fg_sddmm_coo_mh_f32(int64_t nnz, const int32_t *row, const int32_t *col, const float *src, const float *dst,
                        float *out, int32_t H, int32_t D, void *stream) {
  fg::SddmmArgs a;
  fg::SddmmShape s;
  if (int rc = sddmm_prepare(nnz, row, col, src, dst, out, H, D, &a, &s)) return rc;
  return fg::sddmm_launch(a, s, static_cast<hipStream_t>(stream));
}

// For a row-sorted edge list: rebuilds the row pointer and a row plan over (indptr, col) whose bounds table
// cuts every row into column blocks (only when each row's column ids ascend; otherwise whole rows).
// Leaves p->rows null for any other list.
static int build_row_runs(fg_sddmm_plan *p, int32_t num_col_partitions) {
  if (p->nnz == 0) return FG_OK;
  if (fg::config().sddmm_rows == 0) {
    p->no_row_plan = "the plan was created with sddmm.rows = 0, which skips the row pointer";
    return FG_OK;
  }
  if (p->n_rows >= 0x7fffffffLL || p->nnz > 0x7fffffffLL) {
    p->no_row_plan = "the row plan needs n_rows and nnz below 2^31";
    return FG_OK;
  }
  int *flag = nullptr;
  int bad = 0;
  FG_HIP_TRY(hipMalloc(&flag, sizeof(int)));
  hipError_t err = hipMemset(flag, 0, sizeof(int));
  const unsigned grid = static_cast<unsigned>(std::min<int64_t>((p->nnz + 255) / 256, 16384));
  if (err == hipSuccess) {
    rows_sorted_kernel<<<dim3(grid), dim3(256)>>>(p->row, p->nnz, static_cast<int32_t>(p->n_rows), flag);
    err = hipGetLastError();
  }
  if (err == hipSuccess) err = hipMemcpy(&bad, flag, sizeof(int), hipMemcpyDeviceToHost);
  (void)hipFree(flag);
  if (err != hipSuccess) return fg::fail(FG_EHIP, "row order check: %s", hipGetErrorString(err));
  const int32_t *rows_of = p->row, *cols_of = p->col;
  if (bad) {
    // not row-sorted (or ids outside the matrix, which the sort refuses): work on a sorted copy
    if (fg::config().sddmm_sorted_copy == 0 || fg::config().sddmm_blocked == 0) return FG_OK;
    if (int rc = fg::sddmm_sorted_build(p->nnz, p->n_rows, p->n_cols, p->row, p->col, &p->sorted)) return rc;
    if (!p->sorted.col_s) return FG_OK;
    rows_of = p->sorted.row_s;
    cols_of = p->sorted.col_s;
  }
  err = hipMalloc(&p->indptr, sizeof(int32_t) * (p->n_rows + 1));
  if (err != hipSuccess) {
    p->indptr = nullptr;
    return fg::fail(err == hipErrorOutOfMemory ? FG_ENOMEM : FG_EHIP, "row pointer: %s", hipGetErrorString(err));
  }
  indptr_from_rows_kernel<<<dim3(grid), dim3(256)>>>(rows_of, p->nnz, static_cast<int32_t>(p->n_rows), p->indptr);
  FG_HIP_TRY(hipGetLastError());
  FG_HIP_TRY(hipDeviceSynchronize());
  if (p->sorted.row_s) {
    (void)hipFree(p->sorted.row_s);
    p->sorted.row_s = nullptr;
  }
  // same block width as the re-ordered edge list (sddmm_blocked.hip); a run costs a wave a fixed amount of
  // work, so blocks need 8 edges per run on average (sparser lists keep whole rows and take the edge-list path)
  if (int rc = row_plan_create(p->n_rows, p->n_cols, p->nnz, p->indptr, cols_of, num_col_partitions,
                               fg::config().sddmm_block_cols, kSddmmBlockCols, kSddmmSplit, fg::config().sddmm_blocked,
                               8.0, false, fg::config().sddmm_xcd != 0, &p->rows))
    return rc;
  if (p->sorted.col_s && !(p->rows && p->rows->seg && p->rows->n_blocks >= 2)) {
    // too thin for column blocks: the sorted copy would buy nothing over the caller's list
    if (p->rows) fg_spmm_plan_destroy(p->rows);
    p->rows = nullptr;
    (void)hipFree(p->indptr);
    p->indptr = nullptr;
    fg::sddmm_sorted_free(&p->sorted);
  }
  p->input_row_sorted = !bad;
  if (!bad && p->rows && p->rows->cols_unsorted && fg::config().sddmm_sorted_copy != 0) {
    // Rows ascend but the columns inside some row do not, so the rows could not be cut into column blocks: a
    // copy sorted inside the rows can.  The row pointer is the same for both, and so is the visiting order.
    if (int rc = fg::sddmm_sorted_build(p->nnz, p->n_rows, p->n_cols, p->row, p->col, &p->sorted)) return rc;
    if (p->sorted.col_s) {
      (void)hipFree(p->sorted.row_s);
      p->sorted.row_s = nullptr;
      fg_spmm_plan *blocked = nullptr;
      if (int rc = row_plan_create(p->n_rows, p->n_cols, p->nnz, p->indptr, p->sorted.col_s, num_col_partitions,
                                   fg::config().sddmm_block_cols, kSddmmBlockCols, kSddmmSplit,
                                   fg::config().sddmm_blocked, 8.0, false, fg::config().sddmm_xcd != 0, &blocked))
        return rc;
      if (blocked && blocked->seg && blocked->n_blocks >= 2) {
        fg_spmm_plan_destroy(p->rows);
        p->rows = blocked;
      } else {
        if (blocked) fg_spmm_plan_destroy(blocked);
        fg::sddmm_sorted_free(&p->sorted);
      }
    }
  }
  return FG_OK;
}

int fg_sddmm_plan_create(int64_t nnz, int64_t n_rows, int64_t n_cols, const int32_t *row, const int32_t *col,
                         fg_sddmm_plan **plan) {
  return fg_sddmm_plan_create_partitioned(nnz, n_rows, n_cols, row, col, 0, plan);
}

int fg_sddmm_plan_create_partitioned(int64_t nnz, int64_t n_rows, int64_t n_cols, const int32_t *row,
                                     const int32_t *col, int32_t num_col_partitions, fg_sddmm_plan **plan) {
  if (!plan) return fg::fail(FG_EINVAL, "plan output pointer is null");
  *plan = nullptr;
  if (num_col_partitions < 0)
    return fg::fail(FG_EINVAL, "num_col_partitions = %d is negative", num_col_partitions);
  if (nnz < 0 || n_rows < 0 || n_cols < 0)
    return fg::fail(FG_EINVAL, "negative size (nnz=%lld n_rows=%lld n_cols=%lld)", (long long)nnz, (long long)n_rows,
                    (long long)n_cols);
  if (nnz > 0 && (!row || !col)) return fg::fail(FG_EINVAL, "row or col is null");
  if (nnz > 0 && (n_rows == 0 || n_cols == 0)) return fg::fail(FG_EINVAL, "edges in a matrix without rows or columns");
  fg_sddmm_plan *p = new (std::nothrow) fg_sddmm_plan();
  if (!p) return fg::fail(FG_ENOMEM, "plan allocation failed");
  p->nnz = nnz;
  p->n_rows = n_rows;
  p->n_cols = n_cols;
  p->row = row;
  p->col = col;
  p->force_blocks = num_col_partitions > 1;
  if (hipGetDevice(&p->device) != hipSuccess) {
    delete p;
    return fg::fail(FG_EHIP, "hipGetDevice failed");
  }
  if (int rc = build_row_runs(p, num_col_partitions)) {
    fg_sddmm_plan_destroy(p);
    return rc;
  }
  // the re-ordered edge list serves the lists that the row-run kernel cannot take
  const bool runs_blocked = p->rows && (p->rows->n_blocks >= 2 || num_col_partitions == 1);
  if (!runs_blocked || fg::config().sddmm_rows == 0) {
    if (int rc = fg::sddmm_blocks_build(nnz, n_rows, n_cols, row, col, num_col_partitions, &p->blocks)) {
      fg_sddmm_plan_destroy(p);
      return rc;
    }
  }
  *plan = p;
  return FG_OK;
}

void fg_sddmm_plan_destroy(fg_sddmm_plan *plan) {
  if (!plan) return;
  fg::sddmm_blocks_free(&plan->blocks);
  fg::sddmm_sorted_free(&plan->sorted);
  if (plan->rows) fg_spmm_plan_destroy(plan->rows);
  if (plan->indptr) (void)hipFree(plan->indptr);
  delete plan;
}

static bool sddmm_use_blocks(const fg_sddmm_plan *plan, const float *src, const float *dst, int32_t H, int32_t D) {
  // below 64 floats a tile would leave lanes idle and the plain kernel is as fast (measured at 32)
  if (!plan->force_blocks && (fg::config().sddmm_blocked == 0 || (fg::config().sddmm_blocked < 0 && D < 64))) return false;
  return plan->blocks.pos_p && H == 1 && D % 4 == 0 && fg::aligned_to(src, 16) &&
         fg::aligned_to(dst, 16);
}

// Column blocks of the table that one pass of the row-run kernel takes together for a 64-float tile: the band
// of Src that a pass gathers from (block width x tile bytes) should stay about one L2 (4 MB), so narrower
// tiles take more blocks and wider tiles fewer.  Blocks that the caller sized (partition count,
// sddmm.block_cols) are used as they are.
static int sddmm_rows_merge64(const fg_sddmm_plan *plan) {
  const fg_spmm_plan *r = plan->rows;
  if (plan->force_blocks || r->want_block_cols > 0 || r->n_blocks < 2) return 0;  // 0: one block per pass, always
  return r->split_used;
}

// Widest tile, in 64-float units (1 or 2), that the row-run kernel may use: the passes of a wider tile are
// narrower by the same factor, and a (row, pass) run should still hold 8 edges on average.
static int sddmm_rows_max_wide(const fg_sddmm_plan *plan) {
  const fg_spmm_plan *r = plan->rows;
  const int merge64 = sddmm_rows_merge64(plan);
  const int want = fg::config().sddmm_rows_wide;
  if (want > 0) return want >= 2 ? 2 : 1;  // asked for: also over blocks that the caller sized (their width stays)
  if (merge64 == 0 || merge64 % 2 != 0) return 1;
  const double per_block = static_cast<double>(plan->nnz) / (static_cast<double>(r->n_rows) * r->n_blocks);
  return per_block * (merge64 / 2) >= 8.0 ? 2 : 1;
}

static bool sddmm_use_row_runs(const fg_sddmm_plan *plan, const float *src, const float *dst, int32_t H, int32_t D) {
  const int mode = fg::config().sddmm_rows;
  if (!plan->rows || !plan->rows->seg || mode == 0) return false;
  // any feature length from four floats on: a lane's piece that the row's end cuts is moved back and masked
  if (H != 1 || D < 4 || !fg::aligned_to(src, 4) || !fg::aligned_to(dst, 4)) return false;
  if (mode > 0) return true;
  if (plan->rows->n_blocks < 2) return false;  // whole rows: the edge-list kernels take it
  if (plan->force_blocks) return true;
  if (fg::config().sddmm_blocked == 0) return false;
  return fg::config().sddmm_blocked > 0 || D >= 16;  // shorter rows leave most lanes of a 4-lane group idle
}

// the row-run kernel over feature rows that lie `pitch` floats apart
static int sddmm_row_runs(const fg_sddmm_plan *plan, const float *src, const float *dst, float *out, int32_t D,
                          int32_t pitch, void *stream) {
  if (int rc = check_heads(1, D)) return rc;
  if (!src || !dst || !out) return fg::fail(FG_EINVAL, "a data pointer is null");
  const fg_spmm_plan *r = plan->rows;
  const bool copy = plan->sorted.col_s != nullptr;
  if (int rc = fg::sddmm_rows_launch(r->seg, r->row_order, static_cast<int32_t>(r->n_rows), r->n_blocks,
                                     sddmm_rows_merge64(plan), sddmm_rows_max_wide(plan),
                                     copy ? plan->sorted.col_s : plan->col, src, dst, copy ? plan->sorted.results : out,
                                     plan->n_cols * int64_t{pitch} * 4, plan->n_rows * int64_t{pitch} * 4, D, pitch,
                                     static_cast<hipStream_t>(stream)))
    return rc;
  return copy ? fg::sddmm_unsort_launch(plan->sorted, plan->nnz, out, static_cast<hipStream_t>(stream)) : FG_OK;
}

int fg_sddmm_coo_plan_pitched_f32(const fg_sddmm_plan *plan, const float *src, const float *dst, int32_t pitch, float *out,
                                  int32_t F, void *stream) {
  if (!plan) return fg::fail(FG_EINVAL, "plan is null");
  if (pitch < F || pitch % 4 != 0)
    return fg::fail(FG_EINVAL, "pitch = %d must be a multiple of 4 and at least F = %d", pitch, F);
  if (plan->nnz > 0)
    if (int rc = check_device(plan->device)) return rc;
  if (!sddmm_use_row_runs(plan, src, dst, 1, F))
    return fg::fail(FG_EUNSUPPORTED, "only the row-run kernel reads feature rows at a pitch of their own");
  return sddmm_row_runs(plan, src, dst, out, F, pitch, stream);
}

int fg_sddmm_coo_plan_f32(const fg_sddmm_plan *plan, const float *src, const float *dst, float *out, int32_t H,
                          int32_t D, void *stream) {
  if (!plan) return fg::fail(FG_EINVAL, "plan is null");
  if (plan->nnz > 0)
    if (int rc = check_device(plan->device)) return rc;
  if (sddmm_use_row_runs(plan, src, dst, H, D)) return sddmm_row_runs(plan, src, dst, out, D, D, stream);
  if (!sddmm_use_blocks(plan, src, dst, H, D)) {
    fg::SddmmArgs a;
    fg::SddmmShape s;
    if (int rc = sddmm_prepare(plan->nnz, plan->row, plan->col, src, dst, out, H, D, &a, &s, plan->n_rows, plan->n_cols))
      return rc;
    return fg::sddmm_launch(a, s, static_cast<hipStream_t>(stream));
  }
  if (int rc = check_heads(H, D)) return rc;
  if (!src || !dst || !out) return fg::fail(FG_EINVAL, "a data pointer is null");
  return fg::sddmm_blocked_launch(plan->blocks, plan->nnz, src, dst, out, D, plan->n_cols * int64_t{D} * 4,
                                  plan->n_rows * int64_t{D} * 4, static_cast<hipStream_t>(stream));
}

int fg_sddmm_coo_general_plan_f32(const fg_sddmm_plan *plan, const float *src, const float *dst, float *out, int32_t F,
                                  int32_t edge_op, void *stream) {
  if (!plan) return fg::fail(FG_EINVAL, "plan is null");
  if (edge_op == FG_EDGE_DOT) return fg_sddmm_coo_plan_f32(plan, src, dst, out, 1, F, stream);
  if (edge_op < FG_EDGE_DOT || edge_op > FG_EDGE_DIV)
    return fg::fail(FG_EINVAL, "edge_op = %d is not an FG_EDGE_* code", edge_op);
  if (int rc = check_heads(1, F)) return rc;
  if (plan->nnz == 0) return FG_OK;
  if (int rc = check_device(plan->device)) return rc;
  if (!src || !dst || !out) return fg::fail(FG_EINVAL, "a data pointer is null");
  hipStream_t st = static_cast<hipStream_t>(stream);
  // the row-run schedule for the caller's own row-sorted list (a sorted copy would leave the [nnz, F] result in
  // the copy's order); everything else takes the edge-parallel kernel
  const fg_spmm_plan *r = plan->rows;
  if (r && r->seg && r->n_blocks >= 2 && !plan->sorted.col_s && fg::config().sddmm_rows != 0 && F % 4 == 0 &&
      fg::aligned_to(src, 16) && fg::aligned_to(dst, 16) && fg::aligned_to(out, 16))
    return fg::sddmm_rows_elementwise_launch(r->seg, r->row_order, static_cast<int32_t>(r->n_rows), r->n_blocks,
                                             std::max(1, sddmm_rows_merge64(plan)), plan->col, src, dst, out,
                                             plan->n_cols * int64_t{F} * 4, plan->n_rows * int64_t{F} * 4, F, edge_op, st);
  return fg::sddmm_elementwise_launch(plan->row, plan->col, src, dst, out, plan->nnz, F, edge_op, st);
}

int fg_edge_softmax_csr_f32(int64_t n_rows, const int32_t *indptr, const float *scores, float *out, int32_t H,
                            void *stream) {
  if (n_rows < 0 || n_rows >= 0x7fffffffLL) return fg::fail(FG_EINVAL, "n_rows = %lld is out of range", (long long)n_rows);
  if (H < 1 || H > (1 << 20)) return fg::fail(FG_EINVAL, "H = %d is out of range", H);
  if (n_rows == 0) return FG_OK;
  if (!indptr || !scores || !out) return fg::fail(FG_EINVAL, "a data pointer is null");
  return fg::edge_softmax_launch(indptr, scores, out, static_cast<int32_t>(n_rows), H, static_cast<hipStream_t>(stream));
}

int fg_sddmm_softmax_plan_f32(const fg_sddmm_plan *plan, const float *src, const float *dst, float *out, int32_t H,
                              int32_t D, void *stream) {
  if (!plan) return fg::fail(FG_EINVAL, "plan is null");
  if (int rc = check_heads(H, D)) return rc;
  if (plan->nnz == 0) return FG_OK;
  if (int rc = check_device(plan->device)) return rc;
  if (!src || !dst || !out) return fg::fail(FG_EINVAL, "a data pointer is null");
  if (plan->no_row_plan)  // the list's order was never looked at: do not blame it
    return fg::fail(FG_EUNSUPPORTED, "edge softmax needs the plan's row pointer: %s", plan->no_row_plan);
  if (!plan->indptr || !plan->rows || !plan->input_row_sorted)
    return fg::fail(FG_EUNSUPPORTED, "edge softmax needs a row-sorted edge list (each destination row's edges consecutive)");
  hipStream_t st = static_cast<hipStream_t>(stream);
  const int32_t n = static_cast<int32_t>(plan->n_rows);
  if (fg::sddmm_softmax_fused_applies(src, dst, H, D))
    return fg::sddmm_softmax_launch(plan->rows->row_order, plan->indptr, plan->col, src, dst, out, n, H, D, st);
  if (int rc = fg_sddmm_coo_plan_f32(plan, src, dst, out, H, D, stream)) return rc;
  return fg::edge_softmax_launch(plan->indptr, out, out, n, H, st);
}

int fg_attention_csr_mh_f32(const fg_spmm_plan *plan, const float *key, const float *query, const float *value,
                            float *out, int32_t H, int32_t D, void *stream) {
  if (!plan) return fg::fail(FG_EINVAL, "plan is null");
  if (int rc = check_heads(H, D)) return rc;
  if (plan->n_rows == 0) return FG_OK;
  if (int rc = check_device(plan->device)) return rc;
  if (!key || !query || !value || !out) return fg::fail(FG_EINVAL, "a data pointer is null");
  if (!fg::attention_fused_applies(key, query, value, out, H, D))
    return fg::fail(FG_EUNSUPPORTED,
                    "the fused attention kernel has no layout for H = %d, D = %d with these operand alignments: run "
                    "fg_sddmm_softmax_plan_f32 and fg_spmm_csr_mh_f32 one after the other",
                    H, D);
  const int32_t n = static_cast<int32_t>(plan->n_rows);
  return fg::attention_launch(plan->row_order, plan->seg, plan->seg + static_cast<int64_t>(plan->n_blocks) * n,
                              plan->indices, key, query, value, out, n, H, D, static_cast<hipStream_t>(stream));
}

int fg_sddmm_plan_describe(const fg_sddmm_plan *plan, int32_t H, int32_t D, char *buf, int64_t cap) {
  if (!plan) return fg::fail(FG_EINVAL, "plan is null");
  if (!buf || cap <= 0) return fg::fail(FG_EINVAL, "no room for the description");
  alignas(16) static float dummy[4];
  if (sddmm_use_row_runs(plan, dummy, dummy, H, D)) {
    // the first launch's tile (later launches of a long feature row may take a narrower rest)
    const int rows_tile = fg::sddmm_rows_tile(D, sddmm_rows_max_wide(plan));
    const int merge64 = sddmm_rows_merge64(plan);
    const int merge = merge64 == 0 ? 1 : rows_tile <= 64 ? merge64 * (64 / rows_tile) : std::max(1, merge64 / (rows_tile / 64));
    snprintf(buf, static_cast<size_t>(cap),
             "sddmm_coo nnz=%lld H=%d D=%d | kernel=row runs (%s), %d column blocks of %d, tile=%d "
             "floats x %d tiles (one launch each), floats/lane=%d lanes/dot=%d | grid=(blocks, column blocks) x %d "
             "threads each",
             (long long)plan->nnz, H, D,
             plan->sorted.col_s ? "copy of the edge list sorted by row and column, results gathered back to the caller's order"
                                : "row-sorted edge list",
             (plan->rows->n_blocks + merge - 1) / merge,
             static_cast<int>(std::min<int64_t>(int64_t{plan->rows->block_cols} * merge, 0x7fffffff)), rows_tile,
             (D + rows_tile - 1) / rows_tile, rows_tile <= 64 ? 4 : rows_tile / 16, std::min(rows_tile / 4, 16),
             fg::kBlockThreads);
    return FG_OK;
  }
  if (!sddmm_use_blocks(plan, dummy, dummy, H, D)) return fg_sddmm_describe(plan->nnz, H, D, buf, cap);
  const int64_t blocks = ((plan->nnz + 63) / 64 + fg::kWavesPerBlock - 1) / fg::kWavesPerBlock;
  snprintf(buf, static_cast<size_t>(cap),
           "sddmm_coo nnz=%lld H=%d D=%d | kernel=column-blocked edge list, %d column blocks of %d, tile=64 floats x "
           "%d tiles (one launch each), floats/lane=4 lanes/dot=16 | grid=%lld blocks x %d threads each",
           (long long)plan->nnz, H, D, plan->blocks.n_blocks, plan->blocks.block_cols, (D + 63) / 64,
           (long long)blocks, fg::kBlockThreads);
  return FG_OK;
}

int fg_check_indices(int64_t n, const int32_t *idx, int64_t bound, int64_t *n_bad, void *stream) {
  if (n < 0 || !n_bad) return fg::fail(FG_EINVAL, "negative length or null result pointer");
  *n_bad = 0;
  if (n == 0) return FG_OK;
  if (!idx) return fg::fail(FG_EINVAL, "idx is null");
  hipStream_t st = static_cast<hipStream_t>(stream);
  unsigned long long *counter = nullptr;
  FG_HIP_TRY(hipMalloc(&counter, sizeof(*counter)));
  unsigned long long host = 0;
  hipError_t err = hipMemcpyAsync(counter, &host, sizeof(host), hipMemcpyHostToDevice, st);
  if (err == hipSuccess) {
    const int blocks = static_cast<int>(std::min<int64_t>((n + 255) / 256, 4096));
    count_out_of_range_kernel<<<dim3(blocks), dim3(256), 0, st>>>(idx, n, bound, counter);
    err = hipGetLastError();
  }
  if (err == hipSuccess) err = hipMemcpyAsync(&host, counter, sizeof(host), hipMemcpyDeviceToHost, st);
  if (err == hipSuccess) err = hipStreamSynchronize(st);
  (void)hipFree(counter);
  if (err != hipSuccess) return fg::fail(FG_EHIP, "index check: %s", hipGetErrorString(err));
  *n_bad = static_cast<int64_t>(host);
  return FG_OK;
}

int fg_config_set(const char *key, int32_t value) {
  int *slot = config_slot(key);
  if (!slot) return fg::fail(FG_EINVAL, "unknown configuration key '%s'", key ? key : "(null)");
  const bool flag = slot == &fg::config().spmm_sorted ||
                    slot == &fg::config().spmm_blocked || slot == &fg::config().spmm_pipeline ||
                    slot == &fg::config().sddmm_blocked ||
                    slot == &fg::config().spmm_buffer_loads || slot == &fg::config().sddmm_fast ||
                    slot == &fg::config().sddmm_buffer_loads || slot == &fg::config().sddmm_rows ||
                    slot == &fg::config().spmm_multi || slot == &fg::config().sddmm_sorted_copy ||
                    slot == &fg::config().sddmm_regroup || slot == &fg::config().spmm_relay ||
                    slot == &fg::config().spmm_general_multi || slot == &fg::config().sddmm_xcd ||
                    slot == &fg::config().spmm_xcd || slot == &fg::config().spmm_pad_rows;
  // flags: 0 / 1 are explicit, anything negative restores the default;
  // sizes: 0 restores the default
  *slot = flag ? (value < 0 ? -1 : (value != 0)) : std::max(value, 0);
  return FG_OK;
}

int fg_config_get(const char *key, int32_t *value) {
  int *slot = config_slot(key);
  if (!slot || !value) return fg::fail(FG_EINVAL, "unknown configuration key or null result pointer");
  *value = *slot;
  return FG_OK;
}

int fg_spmm_describe(const fg_spmm_plan *plan, int32_t H, int32_t D, int32_t feat_tiles, char *buf, int64_t cap) {
  if (!buf || cap <= 0) return fg::fail(FG_EINVAL, "no room for the description");
  fg::SpmmArgs a;
  fg::SpmmShape s;
  // shape selection looks at pointer alignment only; describe the aligned case
  alignas(16) static float dummy[4];
  if (int rc = spmm_prepare(plan, dummy, dummy, dummy, H, D, feat_tiles, &a, &s)) return rc;
  if (const fg::MultiRuns *runs = multi_table(plan, a, feat_tiles)) {
    const int tile = fg::spmm_multi_tile(a.F);
    const int n_tiles = (a.F + tile - 1) / tile;
    const int n_passes = runs->passes, merge = runs->merge;
    const int tail = multi_tail_tile(a.F);
    const int main_tiles = tail ? n_tiles - 1 : n_tiles;
    char rest[96] = "";
    if (tail) snprintf(rest, sizeof(rest), ", the rest of the row as a tile of %d floats in a launch of its own", tail);
    char passes[288] = "1 launch";
    if (n_passes > 1)
      snprintf(passes, sizeof(passes), "%d launches (one per column block: %d column blocks of %d, each over %d tiles, %d in turn%s)",
               n_passes * (tail ? 2 : 1), n_passes,
               static_cast<int>(std::min<int64_t>(int64_t{plan->block_cols} * merge, 0x7fffffff)), main_tiles,
               multi_interleave(main_tiles), rest);
    else if (tail)
      snprintf(passes, sizeof(passes), "2 launches (%d tiles%s)", main_tiles, rest);
    snprintf(buf, static_cast<size_t>(cap),
             "spmm_csr rows=%lld cols=%lld nnz=%lld max_degree=%d H=%d D=%d | kernel=rows-per-wave(pipelined) "
             "floats/lane=4 lanes/row=%d rows/wave=%d tile=%d floats x %d tiles gathers-in-flight=%d "
             "rows=by-descending-degree | %s",
             (long long)plan->n_rows, (long long)plan->n_cols, (long long)plan->nnz, plan->max_degree, H, D, tile / 4,
             fg::kWaveSize / (tile / 4), tile, n_tiles, tile / 4, passes);
    return FG_OK;
  }
  const int rows_per_wave = fg::kWaveSize / s.lpr;
  const bool blocked = use_column_blocks(plan, a, s);
  const int64_t slots = blocked ? a.n_rows : a.n_slots;
  int64_t waves = (slots + rows_per_wave - 1) / rows_per_wave;
  if (s.pipeline)  // a fixed grid whose waves each walk several rows
    waves = std::min<int64_t>(waves, static_cast<int64_t>(s.pipe_blocks) * fg::kWavesPerBlock);
  char passes[96] = "1 launch";
  if (blocked)
    snprintf(passes, sizeof(passes), "%d launches (%d tiles x %d column blocks of %d)", a.n_tiles * plan->n_blocks,
             a.n_tiles, plan->n_blocks, plan->block_cols);
  snprintf(buf, static_cast<size_t>(cap),
           "spmm_csr rows=%lld cols=%lld nnz=%lld max_degree=%d H=%d D=%d | kernel=%s floats/lane=%d "
           "lanes/row-slot=%d tile=%d floats x %d tiles gathers-in-flight=%d rows=%s | %s, grid=%lld blocks x %d "
           "threads each",
           (long long)plan->n_rows, (long long)plan->n_cols, (long long)plan->nnz, plan->max_degree, H, D,
           s.pipeline ? "wave-per-row(pipelined)" : "row-slot", s.vec, s.lpr, s.tile_width(), a.n_tiles,
           s.unroll, a.row_order ? "by-descending-degree" : "natural", passes,
           (long long)((waves + fg::kWavesPerBlock - 1) / fg::kWavesPerBlock), fg::kBlockThreads);
  return FG_OK;
}

int fg_sddmm_describe(int64_t nnz, int32_t H, int32_t D, char *buf, int64_t cap) {
  if (!buf || cap <= 0) return fg::fail(FG_EINVAL, "no room for the description");
  fg::SddmmArgs a;
  fg::SddmmShape s;
  alignas(16) static float dummy[4];
  alignas(16) static int32_t idummy[4];
  if (int rc = sddmm_prepare(nnz, idummy, idummy, dummy, dummy, dummy, H, D, &a, &s)) return rc;
  const int64_t per_wave = static_cast<int64_t>(s.batches) * fg::kWaveSize;
  const int64_t waves = (a.n_ve + per_wave - 1) / per_wave;
  snprintf(buf, static_cast<size_t>(cap),
           "sddmm_coo nnz=%lld H=%d D=%d | floats/lane=%d lanes/dot=%d dots/wave-round=%d batches/wave=%d | "
           "grid=%lld blocks x %d threads",
           (long long)nnz, H, D, s.vec, s.group, fg::kWaveSize / s.group, s.batches,
           (long long)((waves + fg::kWavesPerBlock - 1) / fg::kWavesPerBlock), fg::kBlockThreads);
  return FG_OK;
}

}  // extern "C"

namespace {
const EnvConfig g_env_config;
}  // namespace
