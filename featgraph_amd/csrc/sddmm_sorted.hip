// SDDMM on an edge list in any order (gfx950): the plan's copy of the list sorted by (row, column), which lets
// the row-run kernel of sddmm.hip serve it, and the return of the results to the caller's order.
//
// fg_sddmm_plan_create sorts (row, column, position) once with a stable device radix sort.  A call then runs the
// row-run kernel over the copy -- the dot products land in sorted order in memory the plan owns -- and brings
// them back to the caller's positions: a fixed permutation of nnz floats, done as two permutations that each stay
// inside blocks of 32768 elements (below), or as one gather when that routing could not be built.
#include <rocprim/device/device_radix_sort.hpp>

#include "common.hpp"

namespace fg {
namespace {

// Sort key of an edge for the (row, column) order: row id above the column id.  Raises *bad for ids outside the
// matrix (such a list is left to the kernels that check nothing but gather nothing out of range either).
__global__ void row_col_keys_kernel(const int32_t *row, const int32_t *col, int64_t nnz, int32_t n_rows,
                                    int32_t n_cols, int col_bits, uint64_t *keys, int32_t *ids, int *bad) {
  const int64_t stride = static_cast<int64_t>(gridDim.x) * blockDim.x;
  int b = 0;
  for (int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x; i < nnz; i += stride) {
    const int32_t r = row[i], c = col[i];
    b |= (r < 0 || r >= n_rows || c < 0 || c >= n_cols) ? 1 : 0;
    keys[i] = (static_cast<uint64_t>(static_cast<uint32_t>(r)) << col_bits) | static_cast<uint32_t>(c);
    ids[i] = static_cast<int32_t>(i);
  }
  if (b) atomicOr(bad, 1);
}

// Splits the sorted keys back into ids and inverts the permutation: where[e] is the place of the caller's edge e
// in the sorted list.
__global__ void sorted_edges_kernel(const uint64_t *keys_sorted, const int32_t *pos, int64_t nnz, int col_bits,
                                    int32_t *row_s, int32_t *col_s, int32_t *where) {
  const int64_t stride = static_cast<int64_t>(gridDim.x) * blockDim.x;
  const uint64_t mask = (uint64_t{1} << col_bits) - 1;
  for (int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x; i < nnz; i += stride) {
    const uint64_t k = keys_sorted[i];
    row_s[i] = static_cast<int32_t>(k >> col_bits);
    col_s[i] = static_cast<int32_t>(k & mask);
    where[pos[i]] = static_cast<int32_t>(i);
  }
}

// out[e] = sorted[where[e]]: four edges per thread, stores coalesced, loads wherever the sort put the edges.
__global__ __launch_bounds__(256) void unsort_kernel(const float *sorted, const int32_t *where, float *out, int64_t nnz) {
  const int64_t stride = static_cast<int64_t>(gridDim.x) * blockDim.x * 4;
  for (int64_t i = (static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x) * 4; i < nnz; i += stride) {
    if (i + 3 < nnz && (reinterpret_cast<uintptr_t>(out + i) & 15) == 0) {
      const int4 w = *reinterpret_cast<const int4 *>(where + i);
      *reinterpret_cast<float4 *>(out + i) = make_float4(sorted[w.x], sorted[w.y], sorted[w.z], sorted[w.w]);
    } else {
      for (int64_t k = i; k < min(i + 4, nnz); ++k) out[k] = sorted[where[k]];
    }
  }
}

// ---- the gather back in two local steps -------------------------------------------------------------------
// out[e] = sorted[where[e]] reads 4 bytes from a random 128-byte line per edge.  The same permutation as two
// steps that each permute only inside a block of kRegroup elements, through LDS, with coalesced stores:
//   step A  block c of the sorted results is re-ordered, in place, by destination block:
//           staged[c*K + a_local[i]] = sorted[i]
//   step B  destination block b collects its elements, which lie in one short contiguous piece per source block
//           (from[j] walks them), and puts each at its place: out[b*K + b_local[j]] = staged[from[j]]
// so the only scattered accesses are step B's reads of pieces of K*K/nnz consecutive elements (9 on a list of
// 115M edges: 16M pieces instead of 115M single reads).
constexpr int kRegroup = 32768;        // elements per block: 128 KB of LDS
constexpr int kRegroupThreads = 1024;

__global__ void regroup_keys_kernel(const int32_t *pos, int64_t nnz, int block_bits, uint32_t *keys, int32_t *ids) {
  const int64_t stride = static_cast<int64_t>(gridDim.x) * blockDim.x;
  for (int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x; i < nnz; i += stride) {
    keys[i] = (static_cast<uint32_t>(i / kRegroup) << block_bits) | static_cast<uint32_t>(pos[i] / kRegroup);
    ids[i] = static_cast<int32_t>(i);
  }
}

// order_a[p]: which sorted element lands at place p of the staged array
__global__ void regroup_a_kernel(const int32_t *order_a, const int32_t *pos, int64_t nnz, uint16_t *a_local,
                                 uint32_t *keys_b, int32_t *ids_b, uint16_t *b_local_of_place) {
  const int64_t stride = static_cast<int64_t>(gridDim.x) * blockDim.x;
  for (int64_t p = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x; p < nnz; p += stride) {
    const int32_t i = order_a[p];
    const int32_t e = pos[i];
    a_local[i] = static_cast<uint16_t>(p % kRegroup);
    keys_b[p] = static_cast<uint32_t>(e / kRegroup);
    ids_b[p] = static_cast<int32_t>(p);
    b_local_of_place[p] = static_cast<uint16_t>(e % kRegroup);
  }
}

__global__ void regroup_b_kernel(const int32_t *from, const uint16_t *b_local_of_place, int64_t nnz, uint16_t *b_local) {
  const int64_t stride = static_cast<int64_t>(gridDim.x) * blockDim.x;
  for (int64_t j = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x; j < nnz; j += stride)
    b_local[j] = b_local_of_place[from[j]];
}

// One workgroup per block of kRegroup elements: lds[local[j]] = in[from ? from[j] : j], then the block is stored
// in order.  `local` is a permutation of the block's own places, so every LDS word is written once.
template <bool GATHER>
__global__ __launch_bounds__(kRegroupThreads) void regroup_kernel(const float *in, const int32_t *from,
                                                                  const uint16_t *local, float *out, int64_t nnz) {
  extern __shared__ float staged_block[];
  const int64_t base = static_cast<int64_t>(blockIdx.x) * kRegroup;
  const int count = static_cast<int>(min(static_cast<int64_t>(kRegroup), nnz - base));
  const int full = count & ~3;
  for (int t = threadIdx.x * 4; t < full; t += kRegroupThreads * 4) {  // base is a multiple of 4 elements
    const ushort4 l = *reinterpret_cast<const ushort4 *>(local + base + t);
    float4 v;
    if constexpr (GATHER) {
      const int4 f = *reinterpret_cast<const int4 *>(from + base + t);
      v = make_float4(in[f.x], in[f.y], in[f.z], in[f.w]);
    } else {
      v = *reinterpret_cast<const float4 *>(in + base + t);
    }
    staged_block[l.x] = v.x;
    staged_block[l.y] = v.y;
    staged_block[l.z] = v.z;
    staged_block[l.w] = v.w;
  }
  for (int t = full + threadIdx.x; t < count; t += kRegroupThreads)
    staged_block[local[base + t]] = in[GATHER ? static_cast<int64_t>(from[base + t]) : base + t];
  __syncthreads();
  if ((reinterpret_cast<uintptr_t>(out) & 15) == 0) {
    for (int t = threadIdx.x * 4; t < full; t += kRegroupThreads * 4)
      *reinterpret_cast<float4 *>(out + base + t) = *reinterpret_cast<const float4 *>(staged_block + t);
    for (int t = full + threadIdx.x; t < count; t += kRegroupThreads) out[base + t] = staged_block[t];
  } else {
    for (int t = threadIdx.x; t < count; t += kRegroupThreads) out[base + t] = staged_block[t];
  }
}

// Builds a_local / from / b_local from pos[i], the caller's place of sorted element i.
hipError_t regroup_build(const int32_t *pos, int64_t nnz, SddmmSorted *out) {
  const size_t n = static_cast<size_t>(nnz);
  const int64_t n_blocks = (nnz + kRegroup - 1) / kRegroup;
  int block_bits = 1;
  while ((int64_t{1} << block_bits) < n_blocks) ++block_bits;
  if (2 * block_bits > 32) return hipSuccess;  // beyond 2^31 edges anyway
  const int grid = static_cast<int>(std::min<int64_t>((nnz + 255) / 256, 65536));
  uint32_t *keys = nullptr, *keys_sorted = nullptr;
  int32_t *ids = nullptr, *order_a = nullptr;
  uint16_t *b_local_of_place = nullptr;
  void *tmp = nullptr;
  size_t tmp_a = 0, tmp_b = 0;
  hipError_t err = hipMalloc(&keys, n * sizeof(uint32_t));
  if (err == hipSuccess) err = hipMalloc(&keys_sorted, n * sizeof(uint32_t));
  if (err == hipSuccess) err = hipMalloc(&ids, n * sizeof(int32_t));
  if (err == hipSuccess) err = hipMalloc(&order_a, n * sizeof(int32_t));
  if (err == hipSuccess) err = hipMalloc(&b_local_of_place, n * sizeof(uint16_t));
  if (err == hipSuccess) err = hipMalloc(&out->a_local, n * sizeof(uint16_t));
  if (err == hipSuccess) err = hipMalloc(&out->b_local, n * sizeof(uint16_t));
  if (err == hipSuccess) err = hipMalloc(&out->from, n * sizeof(int32_t));
  if (err == hipSuccess)
    err = rocprim::radix_sort_pairs(nullptr, tmp_a, keys, keys_sorted, ids, order_a, static_cast<unsigned>(nnz), 0,
                                             2 * block_bits, nullptr);
  if (err == hipSuccess)
    err = rocprim::radix_sort_pairs(nullptr, tmp_b, keys, keys_sorted, ids, out->from, static_cast<unsigned>(nnz), 0,
                                             block_bits, nullptr);
  if (err == hipSuccess) err = hipMalloc(&tmp, std::max<size_t>(std::max(tmp_a, tmp_b), 1));
  if (err == hipSuccess) {
    regroup_keys_kernel<<<dim3(grid), dim3(256)>>>(pos, nnz, block_bits, keys, ids);
    err = hipGetLastError();
  }
  if (err == hipSuccess)  // source block above destination block; stable, so a piece keeps the sorted order
    err = rocprim::radix_sort_pairs(tmp, tmp_a, keys, keys_sorted, ids, order_a, static_cast<unsigned>(nnz), 0,
                                             2 * block_bits, nullptr);
  if (err == hipSuccess) {
    regroup_a_kernel<<<dim3(grid), dim3(256)>>>(order_a, pos, nnz, out->a_local, keys, ids, b_local_of_place);
    err = hipGetLastError();
  }
  if (err == hipSuccess)  // by destination block; stable, so a block's pieces come by ascending place
    err = rocprim::radix_sort_pairs(tmp, tmp_b, keys, keys_sorted, ids, out->from, static_cast<unsigned>(nnz), 0,
                                             block_bits, nullptr);
  if (err == hipSuccess) {
    regroup_b_kernel<<<dim3(grid), dim3(256)>>>(out->from, b_local_of_place, nnz, out->b_local);
    err = hipGetLastError();
  }
  if (err == hipSuccess) err = hipDeviceSynchronize();
  if (err == hipSuccess) {
    err = hipFuncSetAttribute(reinterpret_cast<const void *>(&regroup_kernel<false>),
                              hipFuncAttributeMaxDynamicSharedMemorySize, kRegroup * sizeof(float));
    if (err == hipSuccess)
      err = hipFuncSetAttribute(reinterpret_cast<const void *>(&regroup_kernel<true>),
                                hipFuncAttributeMaxDynamicSharedMemorySize, kRegroup * sizeof(float));
  }
  if (keys) (void)hipFree(keys);
  if (keys_sorted) (void)hipFree(keys_sorted);
  if (ids) (void)hipFree(ids);
  if (order_a) (void)hipFree(order_a);
  if (b_local_of_place) (void)hipFree(b_local_of_place);
  if (tmp) (void)hipFree(tmp);
  if (err != hipSuccess) {  // the one-step gather still works
    if (out->a_local) (void)hipFree(out->a_local);
    if (out->b_local) (void)hipFree(out->b_local);
    if (out->from) (void)hipFree(out->from);
    out->a_local = out->b_local = nullptr;
    out->from = nullptr;
  }
  return err;
}

}  // namespace

void sddmm_sorted_free(SddmmSorted *s) {
  if (s->a_local) (void)hipFree(s->a_local);
  if (s->b_local) (void)hipFree(s->b_local);
  if (s->from) (void)hipFree(s->from);
  if (s->row_s) (void)hipFree(s->row_s);
  if (s->col_s) (void)hipFree(s->col_s);
  if (s->where) (void)hipFree(s->where);
  if (s->results) (void)hipFree(s->results);
  *s = SddmmSorted();
}

int sddmm_sorted_build(int64_t nnz, int64_t n_rows, int64_t n_cols, const int32_t *row, const int32_t *col,
                       SddmmSorted *out) {
  *out = SddmmSorted();
  if (nnz == 0 || n_rows == 0 || n_cols == 0 || nnz > 0x7fffffffLL || n_rows >= 0x7fffffffLL || n_cols >= 0x7fffffffLL)
    return FG_OK;
  int col_bits = 1, row_bits = 1;
  while ((int64_t{1} << col_bits) < n_cols) ++col_bits;
  while ((int64_t{1} << row_bits) < n_rows) ++row_bits;

  uint64_t *keys = nullptr, *keys_sorted = nullptr;
  int32_t *ids = nullptr, *pos = nullptr;
  int *flag = nullptr;
  void *tmp = nullptr;
  size_t tmp_bytes = 0;
  int bad = 0;
  const size_t n = static_cast<size_t>(nnz);
  const int grid = static_cast<int>(std::min<int64_t>((nnz + 255) / 256, 65536));
  hipError_t err = hipMalloc(&keys, n * sizeof(uint64_t));
  if (err == hipSuccess) err = hipMalloc(&keys_sorted, n * sizeof(uint64_t));
  if (err == hipSuccess) err = hipMalloc(&ids, n * sizeof(int32_t));
  if (err == hipSuccess) err = hipMalloc(&pos, n * sizeof(int32_t));
  if (err == hipSuccess) err = hipMalloc(&flag, sizeof(int));
  if (err == hipSuccess) err = hipMalloc(&out->row_s, n * sizeof(int32_t));
  if (err == hipSuccess) err = hipMalloc(&out->col_s, n * sizeof(int32_t));
  if (err == hipSuccess) err = hipMalloc(&out->where, n * sizeof(int32_t));
  if (err == hipSuccess) err = hipMalloc(&out->results, n * sizeof(float));
  if (err == hipSuccess) err = hipMemset(flag, 0, sizeof(int));
  if (err == hipSuccess) {
    row_col_keys_kernel<<<dim3(grid), dim3(256)>>>(row, col, nnz, static_cast<int32_t>(n_rows),
                                                   static_cast<int32_t>(n_cols), col_bits, keys, ids, flag);
    err = hipGetLastError();
  }
  if (err == hipSuccess) err = hipMemcpy(&bad, flag, sizeof(int), hipMemcpyDeviceToHost);
  if (err == hipSuccess && !bad)
    err = rocprim::radix_sort_pairs(nullptr, tmp_bytes, keys, keys_sorted, ids, pos, static_cast<unsigned>(nnz), 0,
                                             row_bits + col_bits, nullptr);
  if (err == hipSuccess && !bad) err = hipMalloc(&tmp, tmp_bytes ? tmp_bytes : 1);
  if (err == hipSuccess && !bad)  // stable: edges listed twice keep the caller's order
    err = rocprim::radix_sort_pairs(tmp, tmp_bytes, keys, keys_sorted, ids, pos, static_cast<unsigned>(nnz), 0,
                                             row_bits + col_bits, nullptr);
  if (err == hipSuccess && !bad) {
    sorted_edges_kernel<<<dim3(grid), dim3(256)>>>(keys_sorted, pos, nnz, col_bits, out->row_s, out->col_s, out->where);
    err = hipGetLastError();
  }
  if (err == hipSuccess) err = hipDeviceSynchronize();
  if (keys) (void)hipFree(keys);
  if (keys_sorted) (void)hipFree(keys_sorted);
  if (ids) (void)hipFree(ids);
  if (tmp) (void)hipFree(tmp);
  if (err == hipSuccess && !bad && config().sddmm_regroup != 0) {
    // without the routing (no memory, no room for 128 KB of LDS per workgroup) the one-step gather serves
    if (regroup_build(pos, nnz, out) != hipSuccess) (void)hipGetLastError();
    if (out->from) {  // the one-step gather's index is not needed then
      (void)hipFree(out->where);
      out->where = nullptr;
    }
  }
  if (pos) (void)hipFree(pos);
  if (flag) (void)hipFree(flag);
  if (err != hipSuccess || bad) {
    sddmm_sorted_free(out);
    if (err == hipSuccess) return FG_OK;
    if (err == hipErrorOutOfMemory) {  // no room for the sorted copy: the other kernels still work
      (void)hipGetLastError();
      return FG_OK;
    }
    return fail(FG_EHIP, "SDDMM sorted edge list construction: %s", hipGetErrorString(err));
  }
  return FG_OK;
}

int sddmm_unsort_launch(const SddmmSorted &s, int64_t nnz, float *out, hipStream_t stream) {
  if (nnz == 0) return FG_OK;
  if (s.from) {
    const unsigned blocks = static_cast<unsigned>((nnz + kRegroup - 1) / kRegroup);
    const size_t lds = kRegroup * sizeof(float);
    // step A works in place: a workgroup has read its whole block before it stores the first element
    regroup_kernel<false><<<dim3(blocks), dim3(kRegroupThreads), lds, stream>>>(s.results, nullptr, s.a_local, s.results, nnz);
    FG_HIP_TRY(hipGetLastError());
    regroup_kernel<true><<<dim3(blocks), dim3(kRegroupThreads), lds, stream>>>(s.results, s.from, s.b_local, out, nnz);
    FG_HIP_TRY(hipGetLastError());
    return FG_OK;
  }
  const unsigned blocks = static_cast<unsigned>(std::min<int64_t>((nnz + 1023) / 1024, 1 << 20));
  unsort_kernel<<<dim3(blocks), dim3(256), 0, stream>>>(s.results, s.where, out, nnz);
  FG_HIP_TRY(hipGetLastError());
  return FG_OK;
}

}  // namespace fg
