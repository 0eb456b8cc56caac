// CSR SpMM for gfx950: Out[r,:] = sum_e w[e] * Feat[indices[e],:].
//
// Work decomposition.  The feature dimension is cut into tiles of
// TW = VEC * LPR floats.  A "slot" of LPR adjacent lanes owns one (row, tile)
// pair; every lane of the slot owns VEC adjacent output floats and walks the
// row's nonzeros from first to last, so each output element is the float32
// sum of its terms in CSR order starting from +0, with one rounded multiply
// and one rounded add per term (this file is compiled with -ffp-contract=off).
// That is the order and rounding of the reference's loop nest
// (op/vanilla_spmm.py:46-56 with the reorder at :73), so results do not depend
// on VEC, LPR, the unroll depth or the row schedule.
//
// Memory behaviour.  A gather of one neighbour row is LPR lanes * VEC floats
// of consecutive addresses (TW*4 bytes, 256 B..1 KB), i.e. whole cache lines.
// Column ids and values of a row are fetched LPR at a time with one coalesced
// load per slot and handed to the slot's lanes through cross-lane reads, so the
// index stream is read once per tile.  U independent gathers are issued before
// the U dependent adds, which is what hides the L2 / Infinity-Cache latency.
// Slots are numbered tile-major, so at any time the running waves gather from
// one TW-wide column band of the feature matrix (n_cols * TW * 4 bytes), which
// is the working set the Infinity Cache has to hold.
//
// Row schedule.  Rows are visited by descending degree (the plan's row list):
// the waves that start first take the hub rows, and the rows that share a wave
// (64 / LPR of them) have nearly equal lengths, so divergence inside a wave is
// small.
#include "common.hpp"

namespace fg {
namespace {

template <int VEC>
struct VecOf;
template <>
struct VecOf<1> {
  using type = float;
};
template <>
struct VecOf<2> {
  using type = float2;
};
template <>
struct VecOf<4> {
  using type = float4;
};

template <int VEC>
__device__ __forceinline__ typename VecOf<VEC>::type vzero();
template <>
__device__ __forceinline__ float vzero<1>() {
  return 0.0f;
}
template <>
__device__ __forceinline__ float2 vzero<2>() {
  return make_float2(0.0f, 0.0f);
}
template <>
__device__ __forceinline__ float4 vzero<4>() {
  return make_float4(0.0f, 0.0f, 0.0f, 0.0f);
}

// acc = acc + v * x, element by element, unfused.
__device__ __forceinline__ void axpy(float &acc, float v, float x) { acc = acc + v * x; }
__device__ __forceinline__ void axpy(float2 &acc, float v, float2 x) {
  acc.x = acc.x + v * x.x;
  acc.y = acc.y + v * x.y;
}
__device__ __forceinline__ void axpy(float4 &acc, float v, float4 x) {
  acc.x = acc.x + v * x.x;
  acc.y = acc.y + v * x.y;
  acc.z = acc.z + v * x.z;
  acc.w = acc.w + v * x.w;
}

// Value held by lane `src` of the calling lane's LPR-wide slot.
template <int LPR>
__device__ __forceinline__ int slot_read(int v, int src, int lane) {
  const int from = (lane & ~(LPR - 1)) | src;
  return __builtin_amdgcn_ds_bpermute(from << 2, v);
}

// General kernel: 64 / LPR slots per wave, per-lane gather addresses.
template <int VEC, int LPR, int U, bool MH>
__global__ __launch_bounds__(kBlockThreads) void spmm_slot_kernel(const SpmmArgs a) {
  using V = typename VecOf<VEC>::type;
  constexpr int RPW = kWaveSize / LPR;
  constexpr int TW = VEC * LPR;
  const int lane = threadIdx.x & (kWaveSize - 1);
  const int sl = lane & (LPR - 1);
  const int64_t slot =
      (static_cast<int64_t>(blockIdx.x) * kWavesPerBlock + (threadIdx.x >> 6)) * RPW + lane / LPR;
  if (slot >= a.n_slots) return;  // a slot leaves as a whole; cross-lane reads never leave the slot
  const int tile = static_cast<int>(slot / a.n_rows);
  const int i = static_cast<int>(slot - static_cast<int64_t>(tile) * a.n_rows);
  const int row = a.row_order ? a.row_order[i] : i;
  const int f0 = (a.tile_base + tile) * TW + sl * VEC;
  const bool fok = f0 < a.F;  // lanes past the end of a partial last tile only take part in the cross-lane reads
  const int head = (MH && fok) ? f0 / a.D : 0;
  const int64_t F = a.F;
  const float *fp = a.feat + (fok ? f0 : a.F - VEC);  // lanes past a partial tile re-read its last group and never store
  const float *wp = a.w + head;
  int e = a.seg_lo ? a.seg_lo[i] : a.indptr[row];
  const int end = a.seg_lo ? a.seg_hi[i] : a.indptr[row + 1];
  V acc = vzero<VEC>();
  float *const op = a.out + static_cast<int64_t>(row) * F + f0;
  if (a.accumulate) {
    if (e >= end) return;  // nothing of this row in this column block: the carried sum stays as it is
    if (fok) acc = *reinterpret_cast<const V *>(op);
  }
  for (; e < end; e += LPR) {
    const int n = min(LPR, end - e);
    int my_col = 0;
    float my_val = 0.0f;
    if (sl < n) {
      my_col = a.indices[e + sl];
      if (!MH) my_val = a.w[e + sl];
    }
    int j = 0;
    for (; j + U <= n; j += U) {
      V x[U];
      float v[U];
#pragma unroll
      for (int u = 0; u < U; ++u) {
        const int c = slot_read<LPR>(my_col, j + u, lane);
        x[u] = *reinterpret_cast<const V *>(fp + static_cast<int64_t>(c) * F);
        if (MH)
          v[u] = wp[static_cast<int64_t>(e + j + u) * a.H];
        else
          v[u] = __int_as_float(slot_read<LPR>(__float_as_int(my_val), j + u, lane));
      }
#pragma unroll
      for (int u = 0; u < U; ++u) axpy(acc, v[u], x[u]);
    }
    if (j < n) {  // fewer than U left: one masked batch, so these gathers overlap too
      V x[U];
      float v[U];
#pragma unroll
      for (int u = 0; u < U; ++u) {
        const int c = slot_read<LPR>(my_col, (j + u) & (LPR - 1), lane);
        const bool live = j + u < n;
        x[u] = live ? *reinterpret_cast<const V *>(fp + static_cast<int64_t>(c) * F) : vzero<VEC>();
        if (MH)
          v[u] = live ? wp[static_cast<int64_t>(e + j + u) * a.H] : 0.0f;
        else
          v[u] = __int_as_float(slot_read<LPR>(__float_as_int(my_val), (j + u) & (LPR - 1), lane));
      }
#pragma unroll
      for (int u = 0; u < U; ++u)
        if (j + u < n) axpy(acc, v[u], x[u]);
    }
  }
  if (fok) *reinterpret_cast<V *>(op) = acc;
}

// One neighbour row's VEC floats for this lane.  With BUF the feature matrix is
// addressed as a buffer resource: the load takes the lane's fixed byte offset in
// a vector register and the row's byte offset (column id * row bytes) in a
// scalar register, so a gather costs one scalar multiply and no vector
// arithmetic; it needs the whole matrix to span less than 4 GiB.  Otherwise the
// address is formed per lane in 64 bits.  Lanes past the end of a partial
// tile carry the offset of the row's last valid group and never store.
template <int VEC, bool BUF>
struct RowGather {
  using V = typename VecOf<VEC>::type;
  __amdgpu_buffer_rsrc_t rsrc;
  const char *base;
  int64_t row_bytes;
  uint32_t lane_off;

  __device__ __forceinline__ RowGather(const float *feat, int64_t n_rows, int64_t F, uint32_t lane_off_)
      : base(reinterpret_cast<const char *>(feat)), row_bytes(F * 4), lane_off(lane_off_) {
    // word 3 of the descriptor: 32-bit untyped data, as gfx9-family buffer loads expect
    rsrc = __builtin_amdgcn_make_buffer_rsrc(const_cast<float *>(feat), 0,
                                             BUF ? static_cast<int>(static_cast<uint32_t>(n_rows * F * 4)) : 0,
                                             0x00020000);
  }
  __device__ __forceinline__ V load(int col) const {  // col is wave-uniform
    if constexpr (BUF) {
      const int soff = col * static_cast<int>(row_bytes);
      if constexpr (VEC == 1)
        return __builtin_bit_cast(V, __builtin_amdgcn_raw_buffer_load_b32(rsrc, static_cast<int>(lane_off), soff, 0));
      else if constexpr (VEC == 2)
        return __builtin_bit_cast(V, __builtin_amdgcn_raw_buffer_load_b64(rsrc, static_cast<int>(lane_off), soff, 0));
      else
        return __builtin_bit_cast(V, __builtin_amdgcn_raw_buffer_load_b128(rsrc, static_cast<int>(lane_off), soff, 0));
    } else {
      return *reinterpret_cast<const V *>(base + static_cast<int64_t>(col) * row_bytes + lane_off);
    }
  }
};

// Gathers for the B nonzeros j .. j+B-1 of the current 64-id block (when !FULL
// only the first `live` of them exist), then the B dependent adds.  `between`
// runs after the gathers are issued and before their results are used: loads
// issued there stay in flight while the adds wait only for the (older) gathers.
template <int VEC, int B, bool MH, bool FULL, bool BUF, typename Between>
__device__ __forceinline__ void gather_batch(typename VecOf<VEC>::type &acc, const RowGather<VEC, BUF> &feat,
                                             int col_reg, float val_reg, const float *wp, int64_t w_stride,
                                             int64_t e0, int j, int live, Between between) {
  using V = typename VecOf<VEC>::type;
  V x[B];
  float v[B];
#pragma unroll
  for (int u = 0; u < B; ++u) {
    const bool on = FULL || u < live;  // wave-uniform
    const int c = __builtin_amdgcn_readlane(col_reg, (j + u) & (kWaveSize - 1));
    x[u] = on ? feat.load(c) : vzero<VEC>();
    if (MH)
      v[u] = on ? wp[(e0 + j + u) * w_stride] : 0.0f;
    else
      v[u] = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(val_reg), (j + u) & (kWaveSize - 1)));
  }
  between();
#pragma unroll
  for (int u = 0; u < B; ++u)
    if (FULL || u < live) axpy(acc, v[u], x[u]);
}

// Pipelined wave-per-row kernel.  A wave walks the rows wave, wave + W,
// wave + 2W, ... of the plan's row list (W = waves in the grid) and keeps three
// rows in flight: while it gathers for row k it has already asked for the first
// 64 column ids / values (and, in a column-blocked pass, the carried sum) of row
// k+1 and for the bounds of row k+2.  Short rows and short column-block
// segments therefore cost one memory round trip each instead of four in a row.
// blockIdx.y selects the feature tile.  Summation order per output element is
// unchanged: CSR order, one lane per element.
template <int VEC, int U, bool MH, bool BUF>
__global__ __launch_bounds__(kBlockThreads) void spmm_pipe_kernel(const SpmmArgs a) {
  using V = typename VecOf<VEC>::type;
  constexpr int TW = VEC * kWaveSize;
  const int lane = threadIdx.x & (kWaveSize - 1);
  const int n_waves = gridDim.x * kWavesPerBlock;
  const int n = a.n_rows;
  int item = __builtin_amdgcn_readfirstlane(static_cast<int>(blockIdx.x * kWavesPerBlock + (threadIdx.x >> 6)));
  const int f0 = (a.tile_base + static_cast<int>(blockIdx.y)) * TW + lane * VEC;
  const bool fok = f0 < a.F;
  const int head = (MH && fok) ? f0 / a.D : 0;
  const int64_t F = a.F;
  const RowGather<VEC, BUF> feat(a.feat, a.n_cols, F, static_cast<uint32_t>(fok ? f0 : a.F - VEC) * 4u);
  const float *wp = a.w + head;
  const int64_t w_stride = a.H;
  const bool carry = a.accumulate != 0;

  auto bounds = [&](int it, int &lo, int &hi, int &row) {
    lo = hi = row = 0;
    if (it < n) {
      lo = a.seg_lo[it];
      hi = a.seg_hi[it];
      row = a.row_order[it];
    }
  };
  auto first_block = [&](int lo, int hi, int row, int &col, float &val, V &acc) {
    col = 0;
    val = 0.0f;
    acc = vzero<VEC>();
    if (lane < hi - lo) {
      col = a.indices[lo + lane];
      if (!MH) val = a.w[lo + lane];
    }
    if (carry && hi > lo && fok) acc = *reinterpret_cast<const V *>(a.out + static_cast<int64_t>(row) * F + f0);
  };

  int lo_a, hi_a, row_a, col_a, lo_b, hi_b, row_b;
  float val_a;
  V acc_a;
  bounds(item, lo_a, hi_a, row_a);
  first_block(lo_a, hi_a, row_a, col_a, val_a, acc_a);
  bounds(item + n_waves, lo_b, hi_b, row_b);

  while (item < n) {
    int lo_c, hi_c, row_c, col_b = 0;
    float val_b = 0.0f;
    V acc_b = vzero<VEC>();
    bounds(item + 2 * n_waves, lo_c, hi_c, row_c);
    bool next_asked = false;
    auto ask_next = [&]() {  // first ids / values / carried sum of the next row, once, behind this row's first gathers
      if (!next_asked) first_block(lo_b, hi_b, row_b, col_b, val_b, acc_b);
      next_asked = true;
    };
    auto nothing = []() {};

    int e = lo_a;
    while (e < hi_a) {
      const int cnt = min(kWaveSize, hi_a - e);
      int col_n = 0;
      float val_n = 0.0f;
      auto ask_more = [&]() {  // the row's next 64 ids / values, behind this block's first gathers
        ask_next();
        const int more = hi_a - (e + kWaveSize);
        if (lane < more) {
          col_n = a.indices[e + kWaveSize + lane];
          if (!MH) val_n = a.w[e + kWaveSize + lane];
        }
      };
      int j = 0;
      bool asked = false;
      for (; j + U <= cnt; j += U) {
        if (!asked)
          gather_batch<VEC, U, MH, true, BUF>(acc_a, feat, col_a, val_a, wp, w_stride, e, j, U, ask_more);
        else
          gather_batch<VEC, U, MH, true, BUF>(acc_a, feat, col_a, val_a, wp, w_stride, e, j, U, nothing);
        asked = true;
      }
      const int left = cnt - j;
      if (left > 0) {
        if (left > 8 || U <= 8) {
          if (!asked)
            gather_batch<VEC, U, MH, false, BUF>(acc_a, feat, col_a, val_a, wp, w_stride, e, j, left, ask_more);
          else
            gather_batch<VEC, U, MH, false, BUF>(acc_a, feat, col_a, val_a, wp, w_stride, e, j, left, nothing);
        } else if (left > 4) {
          if (!asked)
            gather_batch<VEC, 8, MH, false, BUF>(acc_a, feat, col_a, val_a, wp, w_stride, e, j, left, ask_more);
          else
            gather_batch<VEC, 8, MH, false, BUF>(acc_a, feat, col_a, val_a, wp, w_stride, e, j, left, nothing);
        } else {
          if (!asked)
            gather_batch<VEC, 4, MH, false, BUF>(acc_a, feat, col_a, val_a, wp, w_stride, e, j, left, ask_more);
          else
            gather_batch<VEC, 4, MH, false, BUF>(acc_a, feat, col_a, val_a, wp, w_stride, e, j, left, nothing);
        }
      }
      e += kWaveSize;
      col_a = col_n;
      val_a = val_n;
    }
    ask_next();  // rows without nonzeros here never reached a gather
    if (fok && (hi_a > lo_a || !carry))
      *reinterpret_cast<V *>(a.out + static_cast<int64_t>(row_a) * F + f0) = acc_a;

    lo_a = lo_b;
    hi_a = hi_b;
    row_a = row_b;
    col_a = col_b;
    val_a = val_b;
    acc_a = acc_b;
    lo_b = lo_c;
    hi_b = hi_c;
    row_b = row_c;
    item += n_waves;
  }
}

template <int VEC, int LPR, int U>
int launch_slot(const SpmmArgs &a, hipStream_t stream) {
  constexpr int RPW = kWaveSize / LPR;
  const int64_t waves = (a.n_slots + RPW - 1) / RPW;
  const int64_t blocks = (waves + kWavesPerBlock - 1) / kWavesPerBlock;
  if (blocks > 0x7fffffffLL) return fail(FG_EUNSUPPORTED, "SpMM launch needs %lld blocks", (long long)blocks);
  if (a.H > 1)
    spmm_slot_kernel<VEC, LPR, U, true><<<dim3((unsigned)blocks), dim3(kBlockThreads), 0, stream>>>(a);
  else
    spmm_slot_kernel<VEC, LPR, U, false><<<dim3((unsigned)blocks), dim3(kBlockThreads), 0, stream>>>(a);
  FG_HIP_TRY(hipGetLastError());
  return FG_OK;
}

template <int VEC, int U>
int launch_pipe(const SpmmArgs &a, const SpmmShape &s, hipStream_t stream) {
  if (!a.seg_lo || !a.row_order) return fail(FG_EINVAL, "the pipelined kernel needs the plan's row list and bounds");
  // a fixed number of resident waves, each walking many rows
  int64_t blocks = static_cast<int64_t>(s.pipe_blocks);
  const int64_t needed = (static_cast<int64_t>(a.n_rows) + kWavesPerBlock - 1) / kWavesPerBlock;
  if (blocks > needed) blocks = needed;
  if (blocks < 1) blocks = 1;
  const dim3 grid(static_cast<unsigned>(blocks), static_cast<unsigned>(a.n_tiles));
  // buffer addressing needs the feature matrix to span less than 4 GiB
  const bool buf = static_cast<int64_t>(a.n_cols) * a.F * 4 < (int64_t{1} << 32) && config().spmm_buffer_loads != 0;
  if (a.H > 1) {
    if (buf)
      spmm_pipe_kernel<VEC, U, true, true><<<grid, dim3(kBlockThreads), 0, stream>>>(a);
    else
      spmm_pipe_kernel<VEC, U, true, false><<<grid, dim3(kBlockThreads), 0, stream>>>(a);
  } else {
    if (buf)
      spmm_pipe_kernel<VEC, U, false, true><<<grid, dim3(kBlockThreads), 0, stream>>>(a);
    else
      spmm_pipe_kernel<VEC, U, false, false><<<grid, dim3(kBlockThreads), 0, stream>>>(a);
  }
  FG_HIP_TRY(hipGetLastError());
  return FG_OK;
}

template <int VEC, int LPR>
int dispatch_unroll(const SpmmArgs &a, const SpmmShape &s, hipStream_t stream) {
  if (LPR == kWaveSize && s.pipeline) {
    switch (s.unroll) {
      case 4: return launch_pipe<VEC, 4>(a, s, stream);
      case 8: return launch_pipe<VEC, 8>(a, s, stream);
      case 16: return launch_pipe<VEC, 16>(a, s, stream);
      case 32: return launch_pipe<VEC, 32>(a, s, stream);
    }
  } else {
    switch (s.unroll) {
      case 4: return launch_slot<VEC, LPR, 4>(a, stream);
      case 8: return launch_slot<VEC, LPR, 8>(a, stream);
      case 16: return launch_slot<VEC, LPR, 16>(a, stream);
      case 32:
        if (LPR >= 32) return launch_slot<VEC, (LPR >= 32 ? LPR : 32), 32>(a, stream);
        break;
    }
  }
  return fail(FG_EINVAL, "spmm unroll %d is not one of 4, 8, 16, 32 (32 needs 32 or 64 lanes per slot)", s.unroll);
}

template <int VEC>
int dispatch_lpr(const SpmmArgs &a, const SpmmShape &s, hipStream_t stream) {
  switch (s.lpr) {
    case 8: return dispatch_unroll<VEC, 8>(a, s, stream);
    case 16: return dispatch_unroll<VEC, 16>(a, s, stream);
    case 32: return dispatch_unroll<VEC, 32>(a, s, stream);
    case 64: return dispatch_unroll<VEC, 64>(a, s, stream);
  }
  return fail(FG_EINVAL, "spmm lanes per row slot %d is not one of 8, 16, 32, 64", s.lpr);
}

}  // namespace

// Widest per-lane vector that the feature length, the head length and the
// base addresses allow.
static int spmm_max_vec(const SpmmArgs &a) {
  if (a.D % 4 == 0 && aligned_to(a.feat, 16) && aligned_to(a.out, 16)) return 4;
  if (a.D % 2 == 0 && aligned_to(a.feat, 8) && aligned_to(a.out, 8)) return 2;
  return 1;
}

SpmmShape spmm_choose_shape(const SpmmArgs &a, int feat_tiles) {
  const Config &cfg = config();
  SpmmShape s;
  const int max_vec = spmm_max_vec(a);
  // Tile width asked for.  By default 64 floats (one 256-byte gather per
  // neighbour and wave): on the 232,965-vertex benchmark graph narrow tiles beat
  // wide ones at every feature length, because each tile's column band of the
  // feature matrix is what has to stay cache-resident while it is gathered from.
  int want = a.F < 64 ? a.F : 64;
  // ... unless even a 64-float band of the feature matrix is far beyond the
  // 256 MB Infinity Cache (the 2.45M-vertex multi-head graph: 627 MB): then
  // every gather goes to HBM whatever the tiling, and wider tiles win by
  // reading the index and weight streams fewer times.
  const bool beyond_cache = static_cast<int64_t>(a.n_cols) * 256 > (int64_t{192} << 20);
  if (beyond_cache) want = a.F < 128 ? a.F : 128;
  if (feat_tiles >= 1) want = (a.F + feat_tiles - 1) / feat_tiles;
  int vec = 1;
  while (vec < max_vec && (want + vec - 1) / vec > kWaveSize) vec *= 2;
  // ... and there two rows per wave with 16-byte gathers measured best (2.45M-vertex graph, 8 heads of 64
  // floats: 23.5 ms against 25.6 ms for a wave per row with 8-byte gathers)
  const bool two_rows = beyond_cache && feat_tiles < 1 && want == 128 && max_vec == 4;
  if (two_rows) vec = 4;
  s.vec = (cfg.spmm_vec > 0 && cfg.spmm_vec <= max_vec) ? cfg.spmm_vec : vec;
  int lanes = pow2_ceil((want + s.vec - 1) / s.vec);
  if (lanes < 8) lanes = 8;
  // a wave per row with idle lanes (pipelined kernel) beats two rows per wave at 17..63 floats
  if (lanes > 16 && feat_tiles < 1 && !two_rows) lanes = kWaveSize;
  if (lanes > kWaveSize) lanes = kWaveSize;
  s.lpr = cfg.spmm_lpr > 0 ? cfg.spmm_lpr : lanes;
  s.unroll = cfg.spmm_unroll > 0 ? cfg.spmm_unroll : (two_rows ? 4 : s.lpr == 32 ? 32 : (s.lpr >= 16 ? 16 : 8));
  s.pipeline = cfg.spmm_pipeline >= 0 ? cfg.spmm_pipeline : 1;
  if (s.lpr != kWaveSize || !a.seg_lo || !a.row_order) s.pipeline = 0;
  s.pipe_blocks = cfg.spmm_pipe_blocks > 0 ? cfg.spmm_pipe_blocks : 16384;
  return s;
}

int spmm_launch(const SpmmArgs &a, const SpmmShape &s, hipStream_t stream) {
  if (a.n_slots == 0) return FG_OK;
  switch (s.vec) {
    case 1: return dispatch_lpr<1>(a, s, stream);
    case 2: return dispatch_lpr<2>(a, s, stream);
    case 4: return dispatch_lpr<4>(a, s, stream);
  }
  return fail(FG_EINVAL, "spmm floats per lane %d is not one of 1, 2, 4", s.vec);
}

}  // namespace fg
