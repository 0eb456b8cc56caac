// "Column sweep" SpMM for gfx950: every wave of the launch is resident at once
// and all of them walk the column range of the adjacency matrix together, so
// that at any moment the whole chip gathers from one narrow band of feature
// rows that fits each XCD's 4 MB L2.
//
// The single-pass kernels (spmm.hip) let every wave walk its own row from the
// first column to the last; the waves are at unrelated columns, every XCD's
// L2 sees the whole feature band (59.6 MB per 64-float tile on the 232,965-
// vertex graph) and 86 % of the gathers miss it.  Here instead
//   - a wave owns R rows for the whole launch and keeps their R x 64 partial
//     sums in LDS (R <= 40: 16 waves per CU share the 160 KB);
//   - the plan stores, per wave, the nonzeros of its rows re-ordered
//     block-major: first everything in columns [0, block_cols), then the next
//     block, and inside a block row after row, each row's entries in CSR order.
//     The wave streams that list 64 entries at a time with coalesced loads;
//   - rows are dealt to waves in snake order over the degree-sorted row list,
//     so all waves hold about the same number of nonzeros, reach each column
//     block at about the same time, and leave it together.  Nothing
//     synchronises them: a wave that lags merely misses L2 more often.
// The rows of a matrix that do not fit one launch (rows > waves * R) are
// split into "generations", one launch each.
//
// Every output element is still produced by one lane adding its terms in CSR
// order (a row's entries keep their order in the list; the running sum moves
// between a register and LDS, both exact), with an unfused multiply and add,
// so results equal the single-pass kernels bit for bit.
#include <algorithm>
#include <functional>
#include <queue>
#include <utility>
#include <vector>

#include "common.hpp"

namespace fg {
namespace {

constexpr int kTile = 64;  // floats per lane row: one float per lane

// One wave per sweep wave: lays the wave's nonzeros out block-major.
// pos[gw * R + l] is the visiting position (index into the plan's bounds
// table) of the wave's l-th row, or -1.
__global__ void build_sweep_lists_kernel(const int32_t *seg, const int32_t *indices, const int32_t *pos,
                                         const int32_t *ptr, int32_t n_rows, int32_t n_blocks, int32_t R,
                                         int32_t n_sweep_waves, int32_t *sw_col, int32_t *sw_src, uint8_t *sw_lrow) {
  const int gw = blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
  const int lane = threadIdx.x & 63;
  if (gw >= n_sweep_waves) return;
  const int my_pos = lane < R ? pos[static_cast<int64_t>(gw) * R + lane] : -1;
  int64_t base = ptr[gw];
  for (int b = 0; b < n_blocks; ++b) {
    int lo = 0, len = 0;
    if (my_pos >= 0) {
      lo = seg[static_cast<int64_t>(b) * n_rows + my_pos];
      len = seg[static_cast<int64_t>(b + 1) * n_rows + my_pos] - lo;
    }
    int incl = len;  // inclusive prefix sum over the wave's rows
    for (int d = 1; d < 64; d <<= 1) {
      const int up = __shfl_up(incl, d);
      if (lane >= d) incl += up;
    }
    const int64_t at = base + incl - len;
    for (int k = 0; k < len; ++k) {
      sw_col[at + k] = indices[lo + k];
      sw_src[at + k] = lo + k;
      sw_lrow[at + k] = static_cast<uint8_t>(lane);
    }
    base += __shfl(incl, 63);
  }
}

struct SweepArgs {
  const int32_t *rows;  // [waves * R] of this generation
  const int32_t *ptr;   // [waves + 1] of this generation
  const int32_t *col;
  const int32_t *src;
  const uint8_t *lrow;
  const float *w;
  const float *feat;
  float *out;
  int32_t R, F, H, D, n_waves;
};

template <int U, bool MH>
__global__ __launch_bounds__(kBlockThreads) void spmm_sweep_kernel(const SweepArgs a) {
  extern __shared__ float lds[];
  const int lane = threadIdx.x & (kWaveSize - 1);
  const int wave_in_block = threadIdx.x >> 6;
  const int wave = __builtin_amdgcn_readfirstlane(static_cast<int>(blockIdx.x * kWavesPerBlock + wave_in_block));
  if (wave >= a.n_waves) return;
  float *const sums = lds + wave_in_block * a.R * kTile + lane;  // this wave's R x 64 partial sums, this lane's column
  const int f0 = static_cast<int>(blockIdx.y) * kTile + lane;
  const bool fok = f0 < a.F;
  const int head = (MH && fok) ? f0 / a.D : 0;
  const int64_t F = a.F;
  const float *fp = a.feat + f0;
  const float *wp = a.w + head;
  const int64_t w_stride = a.H;
  for (int l = 0; l < a.R; ++l) sums[l * kTile] = 0.0f;

  const int begin = __builtin_amdgcn_readfirstlane(a.ptr[wave]);
  const int end = __builtin_amdgcn_readfirstlane(a.ptr[wave + 1]);

  auto load_ids = [&](int base, int &col, int &src, int &lr) {
    col = src = lr = 0;
    if (base + lane < end) {
      col = a.col[base + lane];
      src = a.src[base + lane];
      lr = a.lrow[base + lane];
    }
  };
  auto load_val = [&](int base, int src, float &val) {
    val = 0.0f;
    if (!MH && base + lane < end) val = a.w[src];
  };

  int col0, src0, lr0, col1, src1, lr1;
  float val0, val1;
  load_ids(begin, col0, src0, lr0);
  load_ids(begin + kWaveSize, col1, src1, lr1);
  load_val(begin, src0, val0);

  int cur = __builtin_amdgcn_readfirstlane(lr0);  // row whose sum lives in `acc`
  float acc = 0.0f;

  for (int base = begin; base < end; base += kWaveSize) {
    const int n = min(kWaveSize, end - base);
    int col2, src2, lr2;
    load_val(base + kWaveSize, src1, val1);
    load_ids(base + 2 * kWaveSize, col2, src2, lr2);

    constexpr int NB = kWaveSize / U;
    float x[2][U];
    float v[2][U];
    auto issue = [&](int bt, int buf) {
#pragma unroll
      for (int u = 0; u < U; ++u) {
        const int j = bt * U + u;
        const bool on = j < n;  // wave-uniform
        const int c = __builtin_amdgcn_readlane(col0, j);
        x[buf][u] = (fok && on) ? fp[static_cast<int64_t>(c) * F] : 0.0f;
        if (MH) {
          const int s = __builtin_amdgcn_readlane(src0, j);
          v[buf][u] = on ? wp[static_cast<int64_t>(s) * w_stride] : 0.0f;
        } else {
          v[buf][u] = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(val0), j));
        }
      }
    };
    auto consume = [&](int bt, int buf) {
#pragma unroll
      for (int u = 0; u < U; ++u) {
        const int j = bt * U + u;
        if (j < n) {
          const int r = __builtin_amdgcn_readlane(lr0, j);
          if (r != cur) {  // wave-uniform: park the running sum, fetch the other row's
            sums[cur * kTile] = acc;
            acc = sums[r * kTile];
            cur = r;
          }
          acc = acc + v[buf][u] * x[buf][u];
        }
      }
    };
    issue(0, 0);
#pragma unroll
    for (int bt = 0; bt < NB; ++bt) {
      if (bt + 1 < NB && (bt + 1) * U < n) issue(bt + 1, (bt + 1) & 1);
      if (bt * U < n) consume(bt, bt & 1);
    }
    col0 = col1;
    src0 = src1;
    lr0 = lr1;
    val0 = val1;
    col1 = col2;
    src1 = src2;
    lr1 = lr2;
  }
  sums[cur * kTile] = acc;
  for (int l = 0; l < a.R; ++l) {
    const int row = a.rows[static_cast<int64_t>(wave) * a.R + l];  // wave-uniform
    if (row >= 0 && fok) a.out[static_cast<int64_t>(row) * F + f0] = sums[l * kTile];
  }
}

template <int U>
int launch(const SweepArgs &a, int n_tiles, size_t lds_bytes, hipStream_t stream) {
  const dim3 grid(static_cast<unsigned>((a.n_waves + kWavesPerBlock - 1) / kWavesPerBlock),
                  static_cast<unsigned>(n_tiles));
  if (a.H > 1)
    spmm_sweep_kernel<U, true><<<grid, dim3(kBlockThreads), lds_bytes, stream>>>(a);
  else
    spmm_sweep_kernel<U, false><<<grid, dim3(kBlockThreads), lds_bytes, stream>>>(a);
  FG_HIP_TRY(hipGetLastError());
  return FG_OK;
}

}  // namespace

void sweep_free(SweepPlan *sp) {
  if (sp->rows) (void)hipFree(sp->rows);
  if (sp->ptr) (void)hipFree(sp->ptr);
  if (sp->col) (void)hipFree(sp->col);
  if (sp->src) (void)hipFree(sp->src);
  if (sp->lrow) (void)hipFree(sp->lrow);
  *sp = SweepPlan();
}

int sweep_build(const std::vector<int32_t> &indptr, const std::vector<int32_t> &order, const int32_t *seg,
                int32_t n_blocks, const int32_t *indices, int64_t nnz, SweepPlan *sp) {
  *sp = SweepPlan();
  const Config &cfg = config();
  const int64_t n_rows = static_cast<int64_t>(order.size());
  if (n_rows == 0 || nnz == 0 || n_blocks < 2) return FG_OK;
  int device = 0, cus = 0, lds_per_cu = 0;
  FG_HIP_TRY(hipGetDevice(&device));
  FG_HIP_TRY(hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, device));
  FG_HIP_TRY(hipDeviceGetAttribute(&lds_per_cu, hipDeviceAttributeMaxSharedMemoryPerMultiprocessor, device));
  if (cus <= 0) return FG_OK;
  if (lds_per_cu <= 0) lds_per_cu = 64 * 1024;
  int waves_per_cu = cfg.spmm_sweep_waves_per_cu > 0 ? cfg.spmm_sweep_waves_per_cu : 16;
  waves_per_cu = std::max(kWavesPerBlock, (waves_per_cu / kWavesPerBlock) * kWavesPerBlock);
  const int blocks_per_cu = waves_per_cu / kWavesPerBlock;
  int r_max = (lds_per_cu / blocks_per_cu) / (kWavesPerBlock * kTile * 4);
  r_max = std::min(r_max, 64);
  if (r_max < 1) return FG_OK;
  const int64_t W = static_cast<int64_t>(cus) * waves_per_cu;
  const int64_t G = (n_rows + W * r_max - 1) / (W * r_max);
  const int R = static_cast<int>(std::min<int64_t>(r_max, (n_rows + G * W - 1) / (G * W) + 2));

  // Rows go to generations round-robin over the degree-sorted list (so every
  // generation sees the same degree mix) and, inside a generation, longest
  // first to the wave that holds the fewest nonzeros so far and still has a
  // free row: all waves of a launch end up with nearly the same list length.
  std::vector<int32_t> rows(static_cast<size_t>(G * W * R), -1), pos(static_cast<size_t>(G * W * R), -1);
  std::vector<int64_t> load(static_cast<size_t>(G * W), 0);
  {
    using Item = std::pair<int64_t, int32_t>;  // (nonzeros so far, wave), smallest first
    std::vector<int32_t> count(static_cast<size_t>(G * W), 0);
    for (int64_t g = 0; g < G; ++g) {
      std::priority_queue<Item, std::vector<Item>, std::greater<Item>> heap;
      for (int32_t w = 0; w < W; ++w) heap.push(Item(0, w));
      for (int64_t i = g; i < n_rows; i += G) {
        if (heap.empty()) return fail(FG_EINVAL, "sweep row assignment ran out of room");
        Item top = heap.top();
        heap.pop();
        const int64_t gw = g * W + top.second;
        const int32_t row = order[static_cast<size_t>(i)];
        const int32_t l = count[static_cast<size_t>(gw)]++;
        rows[static_cast<size_t>(gw * R + l)] = row;
        pos[static_cast<size_t>(gw * R + l)] = static_cast<int32_t>(i);
        top.first += indptr[row + 1] - indptr[row];
        load[static_cast<size_t>(gw)] = top.first;
        if (l + 1 < R) heap.push(top);
      }
    }
  }
  std::vector<int32_t> ptr(static_cast<size_t>(G * W + 1), 0);
  int64_t run = 0, max_load = 0;
  for (int64_t gw = 0; gw < G * W; ++gw) {
    ptr[static_cast<size_t>(gw)] = static_cast<int32_t>(run);
    run += load[static_cast<size_t>(gw)];
    max_load = std::max(max_load, load[static_cast<size_t>(gw)]);
  }
  ptr[static_cast<size_t>(G * W)] = static_cast<int32_t>(run);
  if (run != nnz) return fail(FG_EINVAL, "sweep lists cover %lld of %lld nonzeros", (long long)run, (long long)nnz);

  int32_t *d_pos = nullptr;
  hipError_t err = hipMalloc(&sp->rows, rows.size() * sizeof(int32_t));
  if (err == hipSuccess) err = hipMalloc(&sp->ptr, ptr.size() * sizeof(int32_t));
  if (err == hipSuccess) err = hipMalloc(&sp->col, static_cast<size_t>(nnz) * sizeof(int32_t));
  if (err == hipSuccess) err = hipMalloc(&sp->src, static_cast<size_t>(nnz) * sizeof(int32_t));
  if (err == hipSuccess) err = hipMalloc(&sp->lrow, static_cast<size_t>(nnz));
  if (err == hipSuccess) err = hipMalloc(&d_pos, pos.size() * sizeof(int32_t));
  if (err == hipSuccess) err = hipMemcpy(sp->rows, rows.data(), rows.size() * sizeof(int32_t), hipMemcpyHostToDevice);
  if (err == hipSuccess) err = hipMemcpy(sp->ptr, ptr.data(), ptr.size() * sizeof(int32_t), hipMemcpyHostToDevice);
  if (err == hipSuccess) err = hipMemcpy(d_pos, pos.data(), pos.size() * sizeof(int32_t), hipMemcpyHostToDevice);
  if (err == hipSuccess) {
    const int n_sweep_waves = static_cast<int>(G * W);
    const unsigned grid = static_cast<unsigned>((n_sweep_waves + kWavesPerBlock - 1) / kWavesPerBlock);
    build_sweep_lists_kernel<<<dim3(grid), dim3(kBlockThreads)>>>(seg, indices, d_pos, sp->ptr,
                                                                 static_cast<int32_t>(n_rows), n_blocks, R,
                                                                 n_sweep_waves, sp->col, sp->src, sp->lrow);
    err = hipGetLastError();
  }
  if (err == hipSuccess) err = hipDeviceSynchronize();
  if (d_pos) (void)hipFree(d_pos);
  if (err != hipSuccess) {
    sweep_free(sp);
    if (err == hipErrorOutOfMemory) {  // no room for the lists: the other kernels still work
      (void)hipGetLastError();
      return FG_OK;
    }
    return fail(FG_EHIP, "sweep list construction: %s", hipGetErrorString(err));
  }
  sp->generations = static_cast<int32_t>(G);
  sp->waves = static_cast<int32_t>(W);
  sp->rows_per_wave = R;
  sp->max_load = max_load;
  sp->mean_load = nnz / (G * W);
  return FG_OK;
}

int sweep_launch(const SweepPlan &sp, const SpmmArgs &a, int unroll, hipStream_t stream) {
  const int n_tiles = (a.F + kTile - 1) / kTile;
  const size_t lds_bytes = static_cast<size_t>(kWavesPerBlock) * sp.rows_per_wave * kTile * sizeof(float);
  for (int g = 0; g < sp.generations; ++g) {
    SweepArgs s;
    s.rows = sp.rows + static_cast<int64_t>(g) * sp.waves * sp.rows_per_wave;
    s.ptr = sp.ptr + static_cast<int64_t>(g) * sp.waves;
    s.col = sp.col;
    s.src = sp.src;
    s.lrow = sp.lrow;
    s.w = a.w;
    s.feat = a.feat;
    s.out = a.out;
    s.R = sp.rows_per_wave;
    s.F = a.F;
    s.H = a.H;
    s.D = a.D;
    s.n_waves = sp.waves;
    int rc;
    switch (unroll) {
      case 4: rc = launch<4>(s, n_tiles, lds_bytes, stream); break;
      case 8: rc = launch<8>(s, n_tiles, lds_bytes, stream); break;
      case 16: rc = launch<16>(s, n_tiles, lds_bytes, stream); break;
      case 64:
        if (a.H == 1) {
          const dim3 grid(static_cast<unsigned>((s.n_waves + kWavesPerBlock - 1) / kWavesPerBlock),
                          static_cast<unsigned>(n_tiles));
          spmm_sweep_kernel<64, false><<<grid, dim3(kBlockThreads), lds_bytes, stream>>>(s);
          rc = hipGetLastError() == hipSuccess ? FG_OK : fail(FG_EHIP, "sweep launch failed");
          break;
        }
        [[fallthrough]];
      default: rc = launch<32>(s, n_tiles, lds_bytes, stream); break;
    }
    if (rc) return rc;
  }
  return FG_OK;
}

}  // namespace fg
