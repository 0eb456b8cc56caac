// Column-blocked COO SDDMM for gfx950.
//
// The edge-parallel kernel of sddmm.hip gathers Src rows from all over the
// feature matrix, so nearly every gather misses the 4 MB L2 of its XCD (on the
// 232,965-vertex benchmark graph 28.6 GB per launch cross the L2 boundary at
// 64 floats, and the kernel sits on that boundary's ~7.6 TB/s).  Here the plan
// holds the edge list re-ordered by column block: first every edge whose column
// id is below block_cols, then the next block, and inside a block the caller's
// order (a stable sort).  One launch walks that list front to back; workgroups
// are dispatched in list order, so at any moment the resident waves work on a
// short window of the list, i.e. on one column block, whose Src rows
// (block_cols x 64 floats = 4 MB per feature tile at the default 16384 columns)
// mostly stay in L2.  If the
// caller's list is row-sorted, as a COO list derived from CSR is, consecutive
// edges of a block still share their Dst row, which L1 serves.
//
// Long feature rows are processed in tiles of 64 floats, one launch per tile:
// tile t adds its 64-term partial dot product to Out[e] (the reference's x86
// feature tiling, op/vanilla_sddmm.py:49-60 and :68-72, which its CUDA schedules
// had to refuse for lack of a cross-block reduction; launches on one stream are
// ordered, so the running sums need no atomics).  Every Out[e] is written by one
// lane per tile, at the edge's original position: results are deterministic.
#include <hipcub/hipcub.hpp>

#include "common.hpp"

namespace fg {
namespace {

constexpr int kTile = 64;  // floats per tile: 16 lanes x float4 per edge

template <int CTRL>
__device__ __forceinline__ float dpp_add(float x) {
  const int y = __builtin_amdgcn_update_dpp(0, __float_as_int(x), CTRL, 0xF, 0xF, false);
  return x + __int_as_float(y);
}

__global__ void block_keys_kernel(const int32_t *col, int64_t nnz, int32_t block_cols, uint32_t *keys, int32_t *ids) {
  const int64_t stride = static_cast<int64_t>(gridDim.x) * blockDim.x;
  for (int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x; i < nnz; i += stride) {
    keys[i] = static_cast<uint32_t>(max(col[i], 0)) / static_cast<uint32_t>(block_cols);
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

struct BlockedArgs {
  const int32_t *row_p;
  const int32_t *col_p;
  const int32_t *pos_p;
  const float *src;
  const float *dst;
  float *out;
  int64_t nnz;
  int32_t F;
  int32_t tile;
};

// 64 edges per wave; 16 lanes x float4 cover one 64-float tile of one edge, so
// four edges are in flight per round and 16 rounds finish the wave's 64 edges.
template <bool ACC>
__global__ __launch_bounds__(kBlockThreads) void sddmm_blocked_kernel(const BlockedArgs a) {
  const int lane = threadIdx.x & (kWaveSize - 1);
  const int gl = lane & 15;
  const int gbase = lane & ~15;
  const int64_t base = (static_cast<int64_t>(blockIdx.x) * kWavesPerBlock + (threadIdx.x >> 6)) * kWaveSize;
  if (base >= a.nnz) return;
  const int64_t i = base + lane;
  int my_row = 0, my_col = 0, my_pos = -1;
  if (i < a.nnz) {
    my_row = a.row_p[i];
    my_col = a.col_p[i];
    my_pos = a.pos_p[i];
  }
  float prev = 0.0f;
  if (ACC && my_pos >= 0) prev = a.out[my_pos];
  const int k = a.tile * kTile + gl * 4;
  const bool kok = k < a.F;
  const int64_t F = a.F;
  float res = 0.0f;
#pragma unroll 8
  for (int j = 0; j < 16; ++j) {
    const int from = gbase + j;
    const int r = __builtin_amdgcn_ds_bpermute(from << 2, my_row);
    const int c = __builtin_amdgcn_ds_bpermute(from << 2, my_col);
    float p = 0.0f;
    if (kok) {
      const float4 x = *reinterpret_cast<const float4 *>(a.src + static_cast<int64_t>(c) * F + k);
      const float4 y = *reinterpret_cast<const float4 *>(a.dst + static_cast<int64_t>(r) * F + k);
      p = __builtin_fmaf(x.x, y.x, p);
      p = __builtin_fmaf(x.y, y.y, p);
      p = __builtin_fmaf(x.z, y.z, p);
      p = __builtin_fmaf(x.w, y.w, p);
    }
    p = dpp_add<0xB1>(p);   // quad_perm [1,0,3,2]
    p = dpp_add<0x4E>(p);   // quad_perm [2,3,0,1]
    p = dpp_add<0x141>(p);  // row_half_mirror
    p = dpp_add<0x140>(p);  // row_mirror
    if (gl == j) res = p;
  }
  if (my_pos >= 0) a.out[my_pos] = ACC ? prev + res : res;
}

}  // namespace

void sddmm_blocks_free(SddmmBlocks *b) {
  if (b->row_p) (void)hipFree(b->row_p);
  if (b->col_p) (void)hipFree(b->col_p);
  if (b->pos_p) (void)hipFree(b->pos_p);
  *b = SddmmBlocks();
}

int sddmm_blocks_build(int64_t nnz, int64_t n_rows, int64_t n_cols, const int32_t *row, const int32_t *col,
                       SddmmBlocks *out) {
  *out = SddmmBlocks();
  const Config &cfg = config();
  if (cfg.sddmm_blocked == 0 || nnz == 0 || n_rows == 0 || nnz > 0x7fffffffLL) return FG_OK;
  const int64_t block_cols = cfg.sddmm_block_cols > 0 ? cfg.sddmm_block_cols : 16384;
  const int64_t n_blocks = (n_cols + block_cols - 1) / block_cols;
  if (n_blocks < 2) return FG_OK;
  // worthwhile while a destination row still meets several of its edges inside one block
  if (cfg.sddmm_blocked < 0 && static_cast<double>(nnz) / (static_cast<double>(n_rows) * n_blocks) < 4.0) return FG_OK;
  int bits = 1;
  while ((int64_t{1} << bits) < n_blocks) ++bits;

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
    block_keys_kernel<<<dim3(grid), dim3(256)>>>(col, nnz, static_cast<int32_t>(block_cols), keys, ids);
    err = hipGetLastError();
  }
  if (err == hipSuccess)
    err = hipcub::DeviceRadixSort::SortPairs(nullptr, tmp_bytes, keys, keys_sorted, ids, out->pos_p,
                                             static_cast<int>(nnz), 0, bits, nullptr);
  if (err == hipSuccess) err = hipMalloc(&tmp, tmp_bytes ? tmp_bytes : 1);
  if (err == hipSuccess)  // LSD radix sort: stable, so every block keeps the caller's edge order
    err = hipcub::DeviceRadixSort::SortPairs(tmp, tmp_bytes, keys, keys_sorted, ids, out->pos_p,
                                             static_cast<int>(nnz), 0, bits, nullptr);
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
                         hipStream_t stream) {
  BlockedArgs a;
  a.row_p = b.row_p;
  a.col_p = b.col_p;
  a.pos_p = b.pos_p;
  a.src = src;
  a.dst = dst;
  a.out = out;
  a.nnz = nnz;
  a.F = F;
  const int64_t waves = (nnz + kWaveSize - 1) / kWaveSize;
  const int64_t blocks = (waves + kWavesPerBlock - 1) / kWavesPerBlock;
  if (blocks > 0x7fffffffLL) return fail(FG_EUNSUPPORTED, "SDDMM launch needs %lld blocks", (long long)blocks);
  const int n_tiles = (F + kTile - 1) / kTile;
  for (int t = 0; t < n_tiles; ++t) {
    a.tile = t;
    if (t == 0)
      sddmm_blocked_kernel<false><<<dim3((unsigned)blocks), dim3(kBlockThreads), 0, stream>>>(a);
    else
      sddmm_blocked_kernel<true><<<dim3((unsigned)blocks), dim3(kBlockThreads), 0, stream>>>(a);
    FG_HIP_TRY(hipGetLastError());
  }
  return FG_OK;
}

}  // namespace fg
