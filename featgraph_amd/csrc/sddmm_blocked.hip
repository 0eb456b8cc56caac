// Column-blocked COO SDDMM for gfx950.
//
// The edge-parallel kernel of sddmm.hip gathers Src rows from all over the
// feature matrix, so nearly every gather misses the 4 MB L2 of its XCD (on the
// 232,965-vertex benchmark graph 28.6 GB per launch cross the L2 boundary at
// 64 floats, and the kernel sits on that boundary's ~7.6 TB/s).  Here the plan
// holds the edge list re-ordered by column block: first every edge whose column
// id is below block_cols, then the next block, and inside a block by destination
// row (a stable sort: equal keys keep the caller's order).  One launch walks
// that list front to back; workgroups
// are dispatched in list order, so at any moment the resident waves work on a
// short window of the list, i.e. on one column block, whose Src rows
// (block_cols x 64 floats = 4 MB per feature tile at the default 16384 columns)
// mostly stay in L2, and consecutive edges of a block share their Dst row, which L1
// serves.
//
// Long feature rows are processed in tiles of 64 floats, one launch per tile:
// tile t adds its 64-term partial dot product to Out[e] (the reference's x86
// feature tiling, op/vanilla_sddmm.py:49-60 and :68-72, which its CUDA schedules
// had to refuse for lack of a cross-block reduction; launches on one stream are
// ordered, so the running sums need no atomics).  Every Out[e] is written by one
// lane per tile, at the edge's original position: results are deterministic.
#include <rocprim/device/device_radix_sort.hpp>

#include "common.hpp"

namespace fg {
namespace {

constexpr int kTile = 64;  // floats per tile: 16 lanes x float4 per edge

// Sort key of an edge: its column block and, below it when row_bits > 0, its row id, so that inside a block the
// edges of one destination row sit together whatever order the caller listed them in.
__global__ void block_keys_kernel(const int32_t *row, const int32_t *col, int64_t nnz, int32_t block_cols,
                                  int32_t n_rows, int row_bits, uint32_t *keys, int32_t *ids) {
  const int64_t stride = static_cast<int64_t>(gridDim.x) * blockDim.x;
  for (int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x; i < nnz; i += stride) {
    uint32_t key = static_cast<uint32_t>(max(col[i], 0)) / static_cast<uint32_t>(block_cols);
    if (row_bits > 0) key = (key << row_bits) | static_cast<uint32_t>(min(max(row[i], 0), n_rows - 1));
    keys[i] = key;
    ids[i] = static_cast<int32_t>(i);
  }
}

__global__ void gather_edges_kernel(const int32_t *row, const int32_t *col, const int32_t *pos, int64_t nnz,
                                    int32_t *row_p, int32_t *col_p) {
  const int64_t stride = static_cast<int64_t>(gridDim.x) * blockDim.x;
  for (int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x; i < nnz; i += stride) {
    const int32_t e = pos[i];
    row_p[i] = row[e];
    col_p[i] = col[e];
  }
}

}  // namespace

void sddmm_blocks_free(SddmmBlocks *b) {
  if (b->row_p) (void)hipFree(b->row_p);
  if (b->col_p) (void)hipFree(b->col_p);
  if (b->pos_p) (void)hipFree(b->pos_p);
  *b = SddmmBlocks();
}

int sddmm_blocks_build(int64_t nnz, int64_t n_rows, int64_t n_cols, const int32_t *row, const int32_t *col,
                       int32_t num_col_partitions, SddmmBlocks *out) {
  *out = SddmmBlocks();
  const Config &cfg = config();
  if (num_col_partitions == 1 || nnz == 0 || n_rows == 0 || n_cols == 0 || nnz > 0x7fffffffLL) return FG_OK;
  if (num_col_partitions == 0 && cfg.sddmm_blocked == 0) return FG_OK;
  int64_t block_cols = cfg.sddmm_block_cols > 0 ? cfg.sddmm_block_cols : 16384;
  if (num_col_partitions > 1)  // the caller's count, block width as in util/adj_partitioning.py:98
    block_cols = std::max<int64_t>(1, (n_cols + num_col_partitions - 1) / num_col_partitions);
  const int64_t n_blocks = (n_cols + block_cols - 1) / block_cols;
  if (n_blocks < 2) return FG_OK;
  // on its own the library blocks only while a destination row still meets several of its edges inside one block
  if (num_col_partitions == 0 && cfg.sddmm_blocked < 0 &&
      static_cast<double>(nnz) / (static_cast<double>(n_rows) * n_blocks) < 4.0)
    return FG_OK;
  int bits = 1;
  while ((int64_t{1} << bits) < n_blocks) ++bits;
  // with room in a 32-bit key, order the edges of a block by destination row as well: consecutive edges then
  // share their Dst row (served by L1) also when the caller's list was in no particular order
  int row_bits = 1;
  while ((int64_t{1} << row_bits) < n_rows) ++row_bits;
  if (bits + row_bits > 32) row_bits = 0;
  bits += row_bits;

  uint32_t *keys = nullptr, *keys_sorted = nullptr;
  int32_t *ids = nullptr;
  void *tmp = nullptr;
  size_t tmp_bytes = 0;
  const size_t n = static_cast<size_t>(nnz);
  hipError_t err = hipMalloc(&keys, n * sizeof(uint32_t));
  if (err == hipSuccess) err = hipMalloc(&keys_sorted, n * sizeof(uint32_t));
  if (err == hipSuccess) err = hipMalloc(&ids, n * sizeof(int32_t));
  if (err == hipSuccess) err = hipMalloc(&out->pos_p, n * sizeof(int32_t));
  if (err == hipSuccess) err = hipMalloc(&out->row_p, n * sizeof(int32_t));
  if (err == hipSuccess) err = hipMalloc(&out->col_p, n * sizeof(int32_t));
  if (err == hipSuccess) {
    const int grid = static_cast<int>(std::min<int64_t>((nnz + 255) / 256, 65536));
    block_keys_kernel<<<dim3(grid), dim3(256)>>>(row, col, nnz, static_cast<int32_t>(block_cols),
                                                 static_cast<int32_t>(n_rows), row_bits, keys, ids);
    err = hipGetLastError();
  }
  if (err == hipSuccess)
    err = rocprim::radix_sort_pairs(nullptr, tmp_bytes, keys, keys_sorted, ids, out->pos_p,
                                             static_cast<unsigned>(nnz), 0, bits, nullptr);
  if (err == hipSuccess) err = hipMalloc(&tmp, tmp_bytes ? tmp_bytes : 1);
  if (err == hipSuccess)  // LSD radix sort: stable, so edges with equal keys keep the caller's order
    err = rocprim::radix_sort_pairs(tmp, tmp_bytes, keys, keys_sorted, ids, out->pos_p,
                                             static_cast<unsigned>(nnz), 0, bits, nullptr);
  if (err == hipSuccess) {
    const int grid = static_cast<int>(std::min<int64_t>((nnz + 255) / 256, 65536));
    gather_edges_kernel<<<dim3(grid), dim3(256)>>>(row, col, out->pos_p, nnz, out->row_p, out->col_p);
    err = hipGetLastError();
  }
  if (err == hipSuccess) err = hipDeviceSynchronize();
  if (keys) (void)hipFree(keys);
  if (keys_sorted) (void)hipFree(keys_sorted);
  if (ids) (void)hipFree(ids);
  if (tmp) (void)hipFree(tmp);
  if (err != hipSuccess) {
    sddmm_blocks_free(out);
    if (err == hipErrorOutOfMemory) {  // no room for the re-ordered list: the plain kernel still works
      (void)hipGetLastError();
      return FG_OK;
    }
    return fail(FG_EHIP, "SDDMM column-block construction: %s", hipGetErrorString(err));
  }
  out->n_blocks = static_cast<int32_t>(n_blocks);
  out->block_cols = static_cast<int32_t>(block_cols);
  return FG_OK;
}

int sddmm_blocked_launch(const SddmmBlocks &b, int64_t nnz, const float *src, const float *dst, float *out, int32_t F,
                         int64_t src_bytes, int64_t dst_bytes, hipStream_t stream) {
  const int n_tiles = (F + kTile - 1) / kTile;
  for (int t = 0; t < n_tiles; ++t)
    if (int rc = sddmm_tile_launch(b.row_p, b.col_p, b.pos_p, nnz, src, dst, out, src_bytes, dst_bytes, F, t, stream))
      return rc;
  return FG_OK;
}

}  // namespace fg
