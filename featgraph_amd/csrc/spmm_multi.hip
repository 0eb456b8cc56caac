// CSR SpMM, several rows per wave with 16-byte gathers (gfx950): the plan's run records, the re-laid column
// ids, and the launch of the kernel of spmm_multi_kernel.hpp for the plain operator; the generalised operator's
// instances live in spmm_multi_general_*.hip.
#include <rocprim/device/device_radix_sort.hpp>
#include <rocprim/device/device_scan.hpp>

#include "spmm_multi_kernel.hpp"

namespace fg {

// one per message, each in a file of its own
int spmm_multi_general_mul(const SpmmArgs &a, int64_t blocks, hipStream_t stream);
int spmm_multi_general_add(const SpmmArgs &a, int64_t blocks, hipStream_t stream);
int spmm_multi_general_sub(const SpmmArgs &a, int64_t blocks, hipStream_t stream);
int spmm_multi_general_div(const SpmmArgs &a, int64_t blocks, hipStream_t stream);
int spmm_multi_general_copy_u(const SpmmArgs &a, int64_t blocks, hipStream_t stream);

namespace {

// keys[i] = length of the run of visiting position i between two bounds rows; ids[i] = i
__global__ void run_keys_kernel(const int32_t *seg_lo, const int32_t *seg_hi, int32_t n, uint32_t *keys, int32_t *ids) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) {
    keys[i] = static_cast<uint32_t>(max(seg_hi[i] - seg_lo[i], 0));
    ids[i] = i;
  }
}

__global__ void count_long_runs_kernel(const uint32_t *keys, int32_t n, uint32_t threshold, int32_t *count) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  const bool is_long = i < n && keys[i] >= threshold;
  const unsigned long long votes = __ballot(is_long);
  if ((threadIdx.x & 63) == 0 && votes) atomicAdd(count, __popcll(votes));
}

__global__ void run_records_kernel(const int32_t *seg_lo, const int32_t *seg_hi, const int32_t *row_order,
                                   const int32_t *ids_sorted, int32_t n, int4 *rec) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) {
    const int pos = ids_sorted[i];
    rec[i] = make_int4(seg_lo[pos], seg_hi[pos], row_order[pos], 0);
  }
}

// Entries that a record's run takes in the re-laid arrays: its length rounded up to a multiple of four.
__global__ void padded_lengths_kernel(const int4 *rec, int64_t n, int32_t *len) {
  const int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (i < n) len[i] = (max(rec[i].y - rec[i].x, 0) + 3) & ~3;
}

// One wave per record: copies the run's column ids to its new place and rewrites the record as
// {first, last + 1 in the new layout, row, first in the CSR arrays}.
__global__ void relay_ids_kernel(int4 *rec, const int32_t *first_p, int64_t n, const int32_t *indices, int32_t *ids_p) {
  const int lane = threadIdx.x & (kWaveSize - 1);
  const int64_t waves = static_cast<int64_t>(gridDim.x) * (blockDim.x / kWaveSize);
  for (int64_t i = static_cast<int64_t>(blockIdx.x) * (blockDim.x / kWaveSize) + threadIdx.x / kWaveSize; i < n; i += waves) {
    const int4 r = rec[i];
    const int len = max(r.y - r.x, 0), to = first_p[i];
    for (int k = lane; k < len; k += kWaveSize) ids_p[to + k] = indices[r.x + k];
    if (lane == 0) rec[i] = make_int4(to, to + len, r.z, r.x);
  }
}

// The re-laid copy of the ids for a table of several passes.  Failure to allocate leaves the table as it is.
hipError_t relay_build(const int32_t *indices, int64_t nnz, int64_t n_rec, MultiRuns *out) {
  if (nnz + 3 * n_rec >= 0x7fffffffLL) return hipSuccess;
  int32_t *len = nullptr, *first_p = nullptr;
  void *tmp = nullptr;
  size_t tmp_bytes = 0;
  int32_t last[2] = {0, 0};
  hipError_t err = hipMalloc(&len, n_rec * sizeof(int32_t));
  if (err == hipSuccess) err = hipMalloc(&first_p, n_rec * sizeof(int32_t));
  if (err == hipSuccess)
    err = rocprim::exclusive_scan(nullptr, tmp_bytes, len, first_p, int32_t(0), static_cast<size_t>(n_rec), rocprim::plus<int32_t>(), nullptr);
  if (err == hipSuccess) err = hipMalloc(&tmp, tmp_bytes ? tmp_bytes : 1);
  const unsigned grid = static_cast<unsigned>((n_rec + 255) / 256);
  if (err == hipSuccess) {
    padded_lengths_kernel<<<dim3(grid), dim3(256)>>>(out->rec, n_rec, len);
    err = hipGetLastError();
  }
  if (err == hipSuccess)
    err = rocprim::exclusive_scan(tmp, tmp_bytes, len, first_p, int32_t(0), static_cast<size_t>(n_rec), rocprim::plus<int32_t>(), nullptr);
  if (err == hipSuccess) err = hipMemcpy(&last[0], first_p + n_rec - 1, sizeof(int32_t), hipMemcpyDeviceToHost);
  if (err == hipSuccess) err = hipMemcpy(&last[1], len + n_rec - 1, sizeof(int32_t), hipMemcpyDeviceToHost);
  const int64_t total = static_cast<int64_t>(last[0]) + last[1];
  int32_t *ids_p = nullptr;
  if (err == hipSuccess) err = hipMalloc(&ids_p, std::max<int64_t>(total, 1) * sizeof(int32_t));
  if (err == hipSuccess) err = hipMemset(ids_p, 0, std::max<int64_t>(total, 1) * sizeof(int32_t));  // padding: column 0
  if (err == hipSuccess) {
    const unsigned g2 = static_cast<unsigned>(std::min<int64_t>((n_rec + 3) / 4, 65536));
    relay_ids_kernel<<<dim3(g2), dim3(256)>>>(out->rec, first_p, n_rec, indices, ids_p);
    err = hipGetLastError();
  }
  if (err == hipSuccess) err = hipDeviceSynchronize();
  if (len) (void)hipFree(len);
  if (first_p) (void)hipFree(first_p);
  if (tmp) (void)hipFree(tmp);
  if (err != hipSuccess) {
    if (ids_p) (void)hipFree(ids_p);
    return err;  // the records are rewritten only by the last kernel: on failure before it they still index the CSR arrays
  }
  out->ids_p = ids_p;
  out->relaid_n = total;
  return hipSuccess;
}

}  // namespace

int spmm_multi_tile(int32_t F) { return F <= 16 ? 16 : F <= 32 ? 32 : 64; }

void multi_runs_free(MultiRuns *r) {
  if (r->rec) (void)hipFree(r->rec);
  if (r->ids_p) (void)hipFree(r->ids_p);
  delete[] r->long_runs;
  *r = MultiRuns();
}

// One record {first nonzero, one past the last, row id} per (pass, row): pass p covers the column blocks
// p * merge .. p * merge + merge - 1 of the bounds table, and inside a pass the rows come by descending run
// length (ties in the table's order), so the rows that share a wave finish together.
int multi_runs_build(const int32_t *seg, const int32_t *row_order, const int32_t *indices, int64_t nnz, int32_t n_rows,
                     int32_t n_blocks, int32_t merge, MultiRuns *out) {
  *out = MultiRuns();
  if (n_rows == 0 || n_blocks < 1) return FG_OK;
  merge = std::max(1, std::min(merge, n_blocks));
  const int passes = (n_blocks + merge - 1) / merge;
  const size_t n = static_cast<size_t>(n_rows);
  const uint32_t long_run = config().spmm_multi_long > 0 ? static_cast<uint32_t>(config().spmm_multi_long) : kLongRun;
  uint32_t *keys = nullptr, *keys_sorted = nullptr;
  int32_t *ids = nullptr, *ids_sorted = nullptr, *counts = nullptr;
  void *tmp = nullptr;
  size_t tmp_bytes = 0;
  out->long_runs = new (std::nothrow) int32_t[passes]();
  if (!out->long_runs) return fail(FG_ENOMEM, "host allocation for %d passes failed", passes);
  hipError_t err = hipMalloc(&out->rec, n * passes * sizeof(int4));
  if (err == hipSuccess) err = hipMalloc(&counts, passes * sizeof(int32_t));
  if (err == hipSuccess) err = hipMemset(counts, 0, passes * sizeof(int32_t));
  if (err == hipSuccess) err = hipMalloc(&keys, n * sizeof(uint32_t));
  if (err == hipSuccess) err = hipMalloc(&keys_sorted, n * sizeof(uint32_t));
  if (err == hipSuccess) err = hipMalloc(&ids, n * sizeof(int32_t));
  if (err == hipSuccess) err = hipMalloc(&ids_sorted, n * sizeof(int32_t));
  if (err == hipSuccess)
    err = rocprim::radix_sort_pairs_desc(nullptr, tmp_bytes, keys, keys_sorted, ids, ids_sorted,
                                                       static_cast<unsigned>(n_rows), 0, 32, nullptr);
  if (err == hipSuccess) err = hipMalloc(&tmp, tmp_bytes ? tmp_bytes : 1);
  const unsigned grid = static_cast<unsigned>((n_rows + 255) / 256);
  for (int p = 0; p < passes && err == hipSuccess; ++p) {
    const int32_t *lo = seg + static_cast<int64_t>(p) * merge * n_rows;
    const int32_t *hi = seg + static_cast<int64_t>(std::min((p + 1) * merge, n_blocks)) * n_rows;
    run_keys_kernel<<<dim3(grid), dim3(256)>>>(lo, hi, n_rows, keys, ids);
    count_long_runs_kernel<<<dim3(grid), dim3(256)>>>(keys, n_rows, long_run, counts + p);
    err = hipGetLastError();
    if (err == hipSuccess)  // LSD radix sort: stable
      err = rocprim::radix_sort_pairs_desc(tmp, tmp_bytes, keys, keys_sorted, ids, ids_sorted,
                                                         static_cast<unsigned>(n_rows), 0, 32, nullptr);
    if (err == hipSuccess) {
      run_records_kernel<<<dim3(grid), dim3(256)>>>(lo, hi, row_order, ids_sorted, n_rows, out->rec + p * n);
      err = hipGetLastError();
    }
  }
  if (err == hipSuccess) err = hipDeviceSynchronize();
  if (err == hipSuccess) err = hipMemcpy(out->long_runs, counts, passes * sizeof(int32_t), hipMemcpyDeviceToHost);
  if (keys) (void)hipFree(keys);
  if (keys_sorted) (void)hipFree(keys_sorted);
  if (ids) (void)hipFree(ids);
  if (ids_sorted) (void)hipFree(ids_sorted);
  if (counts) (void)hipFree(counts);
  if (tmp) (void)hipFree(tmp);
  if (err != hipSuccess) {
    multi_runs_free(out);
    if (err == hipErrorOutOfMemory) {  // no room for the records: the wave-per-row kernels still work
      (void)hipGetLastError();
      return FG_OK;
    }
    return fail(FG_EHIP, "SpMM run records: %s", hipGetErrorString(err));
  }
  out->merge = merge;
  out->passes = passes;
  if (passes >= 2 && indices && config().spmm_relay != 0) {
    const hipError_t e2 = relay_build(indices, nnz, static_cast<int64_t>(passes) * n_rows, out);
    if (e2 == hipErrorOutOfMemory) {
      (void)hipGetLastError();
    } else if (e2 != hipSuccess) {
      multi_runs_free(out);
      return fail(FG_EHIP, "SpMM re-laid column ids: %s", hipGetErrorString(e2));
    }
  }
  return FG_OK;
}

bool spmm_multi_applies(const SpmmArgs &a) {
  // Any feature length from four floats on (a lane that the row's end cuts takes the row's last four floats and
  // stores only its own); rows that are not 16-byte aligned are read with 4-byte aligned accesses.
  return a.H == 1 && a.F >= 4 && aligned_to(a.feat, 4) && aligned_to(a.out, 4);
}

bool spmm_multi_general_applies(const SpmmArgs &a) {
  return spmm_multi_applies(a);
}

// a.n_tiles tiles of spmm_multi_tile(a.F) floats starting at tile a.tile_base (grid.y); a.runs: one pass's records.
// a.reduce < 0: the plain operator; otherwise FG_REDUCE_SUM / MAX / MIN with the message a.msg.
int spmm_multi_launch(const SpmmArgs &a, hipStream_t stream) {
  if (a.n_rows == 0 || a.n_tiles == 0) return FG_OK;
  if (!spmm_multi_applies(a) || !a.runs)
    return fail(FG_EINVAL, "the several-rows-per-wave SpMM kernel does not take this call");
  const int64_t blocks = config().spmm_multi_blocks > 0 ? config().spmm_multi_blocks : 8192;
  if (a.long_runs < 0 || a.long_runs > a.n_rows || a.long_blocks < 0 || (a.long_runs > 0) != (a.long_blocks > 0))
    return fail(FG_EINVAL, "inconsistent long-run split (%d runs, %d workgroups)", a.long_runs, a.long_blocks);
  const int64_t pitch = a.feat_pitch ? a.feat_pitch : a.F;
  const bool buf = static_cast<int64_t>(a.n_cols) * pitch * 4 < (int64_t{1} << 32) && config().spmm_buffer_loads != 0;
  const bool u24 = a.n_cols <= (1 << 24) && pitch * 4 < (1 << 24);
  const int tile = a.multi_tile ? a.multi_tile : spmm_multi_tile(a.F);
  if (a.reduce >= 0) {
    if (!spmm_multi_general_applies(a))
      return fail(FG_EINVAL, "the generalised several-rows-per-wave kernel does not take this call");
    switch (a.msg) {
      case FG_MSG_MUL: return spmm_multi_general_mul(a, blocks, stream);
      case FG_MSG_ADD: return spmm_multi_general_add(a, blocks, stream);
      case FG_MSG_SUB: return spmm_multi_general_sub(a, blocks, stream);
      case FG_MSG_DIV: return spmm_multi_general_div(a, blocks, stream);
      case FG_MSG_COPY_U: return spmm_multi_general_copy_u(a, blocks, stream);
    }
    return fail(FG_EINVAL, "msg = %d is not an FG_MSG_* code", a.msg);
  }
  switch (tile) {
    case 16: return launch_multi<4, -1, FG_MSG_MUL>(a, blocks, buf, u24, stream);
    case 32: return launch_multi<8, -1, FG_MSG_MUL>(a, blocks, buf, u24, stream);
    default: return launch_multi<16, -1, FG_MSG_MUL>(a, blocks, buf, u24, stream);
  }
}

}  // namespace fg
