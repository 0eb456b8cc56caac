// COO SDDMM for gfx950: Out[e,h] = sum_d Src[col[e],h,d] * Dst[row[e],h,d].
//
// The E*H dot products ("virtual edges" v = e*H + h, each of length D) are
// independent.  A wave takes 64 consecutive virtual edges at a time: it loads
// their row / column ids with one coalesced load each, then runs G rounds; in
// round j the wave's 64/G groups of G lanes each compute the dot product of
// virtual edge g*G + j, every lane multiplying VEC adjacent floats of the two
// gathered rows per step (G*VEC*4 contiguous bytes per group and step), then
// summing across the group with DPP row operations (no LDS traffic).  Lane
// g*G + j keeps that result, so after G rounds lane l holds the result of
// virtual edge l and the wave stores 64 consecutive floats at once.
//
// Every output has a single writer and a fixed summation tree, so results are
// deterministic and do not depend on the batch count; they do depend on G and
// VEC, which are fixed functions of D and of the pointer alignment.
#include <algorithm>

#include "common.hpp"

namespace fg {
namespace {

template <int CTRL>
__device__ __forceinline__ float dpp_add(float x) {
  const int y = __builtin_amdgcn_update_dpp(0, __float_as_int(x), CTRL, 0xF, 0xF, false);
  return x + __int_as_float(y);
}

// Sum over aligned groups of G lanes; every lane of the group gets the total.
// quad_perm [1,0,3,2] = 0xB1, [2,3,0,1] = 0x4E, row_half_mirror = 0x141,
// row_mirror = 0x140: after each step all lanes of the doubled group agree.
template <int G>
__device__ __forceinline__ float group_sum(float x) {
  if (G >= 2) x = dpp_add<0xB1>(x);
  if (G >= 4) x = dpp_add<0x4E>(x);
  if (G >= 8) x = dpp_add<0x141>(x);
  if (G >= 16) x = dpp_add<0x140>(x);
  return x;
}

template <int VEC>
__device__ __forceinline__ float dot_step(const float *pa, const float *pb, float acc);
template <>
__device__ __forceinline__ float dot_step<1>(const float *pa, const float *pb, float acc) {
  return __builtin_fmaf(*pa, *pb, acc);
}
template <>
__device__ __forceinline__ float dot_step<2>(const float *pa, const float *pb, float acc) {
  const float2 a = *reinterpret_cast<const float2 *>(pa), b = *reinterpret_cast<const float2 *>(pb);
  acc = __builtin_fmaf(a.x, b.x, acc);
  return __builtin_fmaf(a.y, b.y, acc);
}
template <>
__device__ __forceinline__ float dot_step<4>(const float *pa, const float *pb, float acc) {
  const float4 a = *reinterpret_cast<const float4 *>(pa), b = *reinterpret_cast<const float4 *>(pb);
  acc = __builtin_fmaf(a.x, b.x, acc);
  acc = __builtin_fmaf(a.y, b.y, acc);
  acc = __builtin_fmaf(a.z, b.z, acc);
  return __builtin_fmaf(a.w, b.w, acc);
}

template <int VEC, int G, bool MH>
__global__ __launch_bounds__(kBlockThreads) void sddmm_kernel(const SddmmArgs a) {
  const int lane = threadIdx.x & (kWaveSize - 1);
  const int gl = lane & (G - 1);
  const int gbase = lane & ~(G - 1);  // first lane of this lane's group = g*G
  const int64_t wave = static_cast<int64_t>(blockIdx.x) * kWavesPerBlock + (threadIdx.x >> 6);
  const int64_t stride = a.stride;
  const int D = a.D;
  for (int b = 0; b < a.batches; ++b) {
    const int64_t v_base = (wave * a.batches + b) * kWaveSize;
    if (v_base >= a.n_ve) return;  // wave-uniform
    const int64_t v = v_base + lane;
    int my_row = 0, my_col = 0;  // lanes past the end gather vertex 0 and drop the result
    if (v < a.n_ve) {
      const int64_t e = MH ? v / a.H : v;
      my_row = a.row[e];
      my_col = a.col[e];
    }
    float res = 0.0f;
#pragma unroll 4
    for (int j = 0; j < G; ++j) {
      const int from = gbase + j;
      const int r = __builtin_amdgcn_ds_bpermute(from << 2, my_row);
      const int c = __builtin_amdgcn_ds_bpermute(from << 2, my_col);
      int64_t off = gl * VEC;
      if (MH) off += static_cast<int64_t>((v_base + from) % a.H) * D;
      const float *pa = a.src + static_cast<int64_t>(c) * stride + off;
      const float *pb = a.dst + static_cast<int64_t>(r) * stride + off;
      float p = 0.0f;
      for (int k = gl * VEC; k < D; k += G * VEC) {
        p = dot_step<VEC>(pa, pb, p);
        pa += G * VEC;
        pb += G * VEC;
      }
      p = group_sum<G>(p);
      if (gl == j) res = p;
    }
    if (v < a.n_ve) a.out[v] = res;
  }
}


// ---------------------------------------------------------------------------
// Fast path: float4 lanes, dot length D = G*4*CH exactly (or one 64-float tile
// of a longer row), everything unrolled.  A wave takes 64 dot products; R
// rounds (64/G dot products each) are issued together, so 2*R*CH float4 gathers
// are in flight per lane before the first multiply, and no branch separates them.
// With BUF the two matrices are addressed as buffer resources with 32-bit
// per-lane byte offsets (one multiply-add per gather instead of 64-bit
// arithmetic); that needs each matrix to span less than 4 GiB.
struct FastArgs {
  const int32_t *row;   // per dot product (plain: edge list; blocked: re-ordered list)
  const int32_t *col;
  const int32_t *pos;   // blocked: where each result goes; plain: null
  const float *src;
  const float *dst;
  float *out;
  int64_t n_ve;         // dot products (edges * heads)
  int64_t src_bytes, dst_bytes;
  int32_t H, D, stride;  // stride: floats per vertex row
  int32_t first;         // first float of the row segment this launch covers (tile * 64)
  int32_t valid;         // floats of the segment that exist (64, or fewer in the last tile)
};

template <bool BUF>
struct VertexRows {
  __amdgpu_buffer_rsrc_t rsrc;
  const char *base;
  __device__ __forceinline__ VertexRows(const float *p, int64_t bytes) : base(reinterpret_cast<const char *>(p)) {
    rsrc = __builtin_amdgcn_make_buffer_rsrc(const_cast<float *>(p), 0,
                                             BUF ? static_cast<int>(static_cast<uint32_t>(bytes)) : 0, 0x00020000);
  }
  // float4 at byte offset vertex * row_bytes + off
  __device__ __forceinline__ float4 load(int vertex, uint32_t row_bytes, uint32_t off) const {
    if constexpr (BUF) {
      const uint32_t at = static_cast<uint32_t>(vertex) * row_bytes + off;
      return __builtin_bit_cast(float4, __builtin_amdgcn_raw_buffer_load_b128(rsrc, static_cast<int>(at), 0, 0));
    } else {
      // rows whose length is not a multiple of four floats start at 4-byte aligned addresses only
      struct alignas(4) Float4A {
        float x, y, z, w;
      };
      const Float4A q = *reinterpret_cast<const Float4A *>(base + static_cast<int64_t>(vertex) * row_bytes + off);
      return make_float4(q.x, q.y, q.z, q.w);
    }
  }
};

// MODE 0: plain (Out[v]), 1: blocked first tile (Out[pos] = sum), 2: blocked later tile (Out[pos] += sum)
template <int G, int CH, bool MH, int MODE, bool BUF>
__global__ __launch_bounds__(kBlockThreads) void sddmm_fast_kernel(const FastArgs a) {
  constexpr int R = (8 / CH) < G ? (8 / CH) : G;  // rounds per batch: up to 16 float4 gathers in flight per lane
  const int lane = threadIdx.x & (kWaveSize - 1);
  const int gl = lane & (G - 1);
  const int gbase = lane & ~(G - 1);
  const int64_t v_base = (static_cast<int64_t>(blockIdx.x) * kWavesPerBlock + (threadIdx.x >> 6)) * kWaveSize;
  if (v_base >= a.n_ve) return;  // wave-uniform
  const int64_t v = v_base + lane;
  int my_row = 0, my_col = 0;  // lanes past the end gather vertex 0 and drop the result
  int64_t my_pos = -1;
  if (v < a.n_ve) {
    const int64_t e = MH ? v / a.H : v;
    my_row = a.row[e];
    my_col = a.col[e];
    my_pos = MODE == 0 ? v : a.pos[v];
  }
  float prev = 0.0f;
  if (MODE == 2 && my_pos >= 0) prev = a.out[my_pos];
  const VertexRows<BUF> src(a.src, a.src_bytes), dst(a.dst, a.dst_bytes);
  const uint32_t row_bytes = static_cast<uint32_t>(a.stride) * 4u;
  // this lane's float4 inside the segment; lanes past a short last tile re-read its last float4 and add zero
  const bool kok = gl * 4 < a.valid;
  const uint32_t lane_bytes = static_cast<uint32_t>(a.first + (kok ? gl * 4 : a.valid - 4)) * 4u;
  float res = 0.0f;
#pragma unroll
  for (int jb = 0; jb < G; jb += R) {
    float4 x[R][CH], y[R][CH];
#pragma unroll
    for (int r = 0; r < R; ++r) {
      const int from = gbase + jb + r;
      const int rr = __builtin_amdgcn_ds_bpermute(from << 2, my_row);
      const int cc = __builtin_amdgcn_ds_bpermute(from << 2, my_col);
      uint32_t off = lane_bytes;
      if (MH) off += static_cast<uint32_t>((v_base + from) % a.H) * static_cast<uint32_t>(a.D) * 4u;
#pragma unroll
      for (int c = 0; c < CH; ++c) {
        x[r][c] = src.load(cc, row_bytes, off + c * G * 16);
        y[r][c] = dst.load(rr, row_bytes, off + c * G * 16);
      }
    }
#pragma unroll
    for (int r = 0; r < R; ++r) {
      float p = 0.0f;
#pragma unroll
      for (int c = 0; c < CH; ++c) {
        p = __builtin_fmaf(x[r][c].x, y[r][c].x, p);
        p = __builtin_fmaf(x[r][c].y, y[r][c].y, p);
        p = __builtin_fmaf(x[r][c].z, y[r][c].z, p);
        p = __builtin_fmaf(x[r][c].w, y[r][c].w, p);
      }
      p = kok ? p : 0.0f;
      p = group_sum<G>(p);
      if (gl == jb + r) res = p;
    }
  }
  if (my_pos >= 0) a.out[my_pos] = MODE == 2 ? prev + res : res;
}

template <int G, int CH, bool MH, int MODE>
int launch_fast_mode(const FastArgs &a, hipStream_t stream) {
  const int64_t waves = (a.n_ve + kWaveSize - 1) / kWaveSize;
  const int64_t blocks = (waves + kWavesPerBlock - 1) / kWavesPerBlock;
  if (blocks > 0x7fffffffLL) return fail(FG_EUNSUPPORTED, "SDDMM launch needs %lld blocks", (long long)blocks);
  const bool buf = a.src_bytes < (int64_t{1} << 32) && a.dst_bytes < (int64_t{1} << 32) && config().sddmm_buffer_loads != 0;
  if (buf)
    sddmm_fast_kernel<G, CH, MH, MODE, true><<<dim3((unsigned)blocks), dim3(kBlockThreads), 0, stream>>>(a);
  else
    sddmm_fast_kernel<G, CH, MH, MODE, false><<<dim3((unsigned)blocks), dim3(kBlockThreads), 0, stream>>>(a);
  FG_HIP_TRY(hipGetLastError());
  return FG_OK;
}


// ---------------------------------------------------------------------------
// Row-run kernel for a row-sorted edge list (a COO list derived from CSR) with
// column blocks.  A work item is one (column block, row) run of edges: they are
// consecutive in the caller's list and share their Dst row, so the wave loads
// that row's 64-float tile ONCE into registers (float4 per lane, the same in
// each of its four 16-lane groups) and each edge then costs a single gathered
// Src tile instead of two; the edge-list kernels above move 512 B per edge and
// tile through L1, which is what bounds them once the gathers hit L2.  Items
// are numbered block-major (blockIdx.y is the column block), so the resident
// waves gather from one column block of Src at a time, as in the re-ordered
// edge list, but results go straight to Out[e] with coalesced stores and no
// re-ordered copy of the list exists.  Group g takes the edges lo + 4*round + g;
// after at most 16 rounds a cross-lane move puts edge lo + l into lane l.
// Like the SpMM pipelined kernel a wave keeps three items in flight: gathers of
// item k, column ids / Dst tile / previous partial result of item k+1, bounds
// of item k+2.
struct RowsArgs {
  const int32_t *seg;        // [(n_blocks + 1) * n_rows] run bounds, rows in visiting order
  const int32_t *row_order;  // [n_rows]
  const int32_t *col;        // the caller's column ids
  const float *src;
  const float *dst;
  float *out;
  int64_t src_bytes, dst_bytes;
  int32_t n_rows, F;
  int32_t pitch;             // floats from one row of src / dst to the next (F unless the caller padded the rows)
  int32_t first, valid;      // the tile this launch covers
  int32_t n_blocks, merge;   // column blocks in the table; a pass covers `merge` neighbouring ones
  // Passes pinned to the dies: workgroup x of a launch runs on die x % 8, so the workgroups x % 8 == d take the
  // passes d, d + 8, ... (blockIdx.y counts those rounds) and every die's L2 keeps the band of ITS pass while the
  // die walks all rows, instead of all eight L2s holding copies of one band.  0: blockIdx.y is the pass.
  int32_t xcd_passes = 0;
};

// (pass, first item, item stride) of a workgroup's wave under either numbering.
__device__ __forceinline__ void rows_wave_place(const RowsArgs &a, int &pass, int &item, int &n_waves) {
  const int wave = static_cast<int>(threadIdx.x >> 6);
  if (a.xcd_passes) {
    pass = static_cast<int>(blockIdx.y) * kXcds + static_cast<int>(blockIdx.x % kXcds);
    item = static_cast<int>(blockIdx.x / kXcds) * kWavesPerBlock + wave;
    n_waves = static_cast<int>(gridDim.x / kXcds) * kWavesPerBlock;
  } else {
    pass = static_cast<int>(blockIdx.y);
    item = static_cast<int>(blockIdx.x) * kWavesPerBlock + wave;
    n_waves = static_cast<int>(gridDim.x) * kWavesPerBlock;
  }
}

// G: lanes per dot product; NT: 16-byte pieces per lane, 64 floats apart (a tile is 4 * G * NT floats; NT > 1
// needs G = 16); R: rounds whose gathers are issued together.  CUT: the tile's valid floats are not a multiple of
// four, so its end cuts some lane's piece: that lane reads the four floats that END at the tile's end instead
// (they may begin in the tile before; the feature row has at least four floats) and leaves the leading ones,
// which belong to its neighbour, out of its sum.
template <bool ACC, bool BUF, int R, int G, int NT, bool CUT>
__global__ __launch_bounds__(kBlockThreads) void sddmm_rows_kernel(const RowsArgs a) {
  static_assert(NT == 1 || G == 16, "a wide tile is made of whole 64-float pieces");
  constexpr int NG = kWaveSize / G;  // edges per round
  const int lane = threadIdx.x & (kWaveSize - 1);
  const int gl = lane & (G - 1);
  const int g = lane / G;
  const int n = a.n_rows;
  int pass, item, n_waves;
  rows_wave_place(a, pass, item, n_waves);
  item = __builtin_amdgcn_readfirstlane(item);
  if (pass * a.merge >= a.n_blocks) return;
  const int32_t *const seg_lo = a.seg + static_cast<int64_t>(pass) * a.merge * n;
  const int32_t *const seg_hi = a.seg + static_cast<int64_t>(min((pass + 1) * a.merge, a.n_blocks)) * n;
  const VertexRows<BUF> src(a.src, a.src_bytes), dst(a.dst, a.dst_bytes);
  const uint32_t row_bytes = static_cast<uint32_t>(a.pitch) * 4u;
  // piece k of this lane covers floats first + 64 k + 4 gl ..; lanes past the tile's end re-read its last
  // four floats and contribute zero
  bool kok[NT];
  int skip[NT];  // leading floats of the piece that are not this lane's (CUT)
  uint32_t lane_bytes[NT];
#pragma unroll
  for (int k = 0; k < NT; ++k) {
    const int start = k * 64 + gl * 4;
    kok[k] = start < a.valid;
    const int from = kok[k] ? min(start, a.valid - 4) : a.valid - 4;
    skip[k] = start - from;
    lane_bytes[k] = static_cast<uint32_t>(a.first + from) * 4u;
  }
  const int gather_from = G * (lane % NG) + lane / NG;  // lane holding the result of edge offset `lane`

  auto bounds = [&](int it, int &lo, int &hi, int &row) {
    lo = hi = row = 0;
    if (it < n) {
      lo = seg_lo[it];
      hi = seg_hi[it];
      row = a.row_order[it];
    }
  };
  auto first_block = [&](int lo, int hi, int row, int &col, float4(&y)[NT], float &prev) {
    col = 0;
    prev = 0.0f;
#pragma unroll
    for (int k = 0; k < NT; ++k) y[k] = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
    if (hi > lo) {
      if (lane < hi - lo) {
        col = a.col[lo + lane];
        if (ACC) prev = a.out[lo + lane];
      }
#pragma unroll
      for (int k = 0; k < NT; ++k) y[k] = dst.load(row, row_bytes, lane_bytes[k]);
    }
  };

  int lo_a, hi_a, row_a, col_a, lo_b, hi_b, row_b;
  float4 y_a[NT];
  float prev_a;
  bounds(item, lo_a, hi_a, row_a);
  first_block(lo_a, hi_a, row_a, col_a, y_a, prev_a);
  bounds(item + n_waves, lo_b, hi_b, row_b);

  while (item < n) {
    int lo_c, hi_c, row_c, col_b = 0;
    float4 y_b[NT];
#pragma unroll
    for (int k = 0; k < NT; ++k) y_b[k] = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
    float prev_b = 0.0f;
    bounds(item + 2 * n_waves, lo_c, hi_c, row_c);
    bool next_asked = false;
    auto ask_next = [&]() {
      if (!next_asked) first_block(lo_b, hi_b, row_b, col_b, y_b, prev_b);
      next_asked = true;
    };

    for (int e = lo_a; e < hi_a; e += kWaveSize) {
      const int cnt = min(kWaveSize, hi_a - e);
      int col_n = 0;
      float prev_n = 0.0f;
      const int rounds = (cnt + NG - 1) / NG;
      float res = 0.0f;
      // two batches of R rounds alternate: the gathers of one are in flight while the other is summed
      float4 xa[R][NT], xb[R][NT];
      auto issue = [&](int rb, float4(&x)[R][NT]) {
#pragma unroll
        for (int r = 0; r < R; ++r) {
          // edges past the run's end read column id 0 of an idle lane: a valid row, result never stored
          const int cc = __builtin_amdgcn_ds_bpermute(((NG * (rb + r) + g) & 63) << 2, col_a);
#pragma unroll
          for (int k = 0; k < NT; ++k) x[r][k] = src.load(cc, row_bytes, lane_bytes[k]);
        }
      };
      auto reduce = [&](int rb, const float4(&x)[R][NT]) {
#pragma unroll
        for (int r = 0; r < R; ++r) {
          float p = 0.0f;
#pragma unroll
          for (int k = 0; k < NT; ++k) {
            float q = 0.0f;
            if constexpr (CUT) {
              q = skip[k] > 0 ? q : __builtin_fmaf(x[r][k].x, y_a[k].x, q);
              q = skip[k] > 1 ? q : __builtin_fmaf(x[r][k].y, y_a[k].y, q);
              q = skip[k] > 2 ? q : __builtin_fmaf(x[r][k].z, y_a[k].z, q);
              q = __builtin_fmaf(x[r][k].w, y_a[k].w, q);
            } else {
              q = __builtin_fmaf(x[r][k].x, y_a[k].x, q);
              q = __builtin_fmaf(x[r][k].y, y_a[k].y, q);
              q = __builtin_fmaf(x[r][k].z, y_a[k].z, q);
              q = __builtin_fmaf(x[r][k].w, y_a[k].w, q);
            }
            p += kok[k] ? q : 0.0f;
          }
          p = group_sum<G>(p);
          if (gl == rb + r) res = p;
        }
      };
      issue(0, xa);
      {  // behind this run's first gathers: the next run's operands and this run's next 64 ids
        ask_next();
        const int more = hi_a - (e + kWaveSize);
        if (lane < more) {
          col_n = a.col[e + kWaveSize + lane];
          if (ACC) prev_n = a.out[e + kWaveSize + lane];
        }
      }
      for (int rb = 0; rb < rounds; rb += 2 * R) {
        const bool second = rb + R < rounds;
        if (second) issue(rb + R, xb);
        reduce(rb, xa);
        if (rb + 2 * R < rounds) issue(rb + 2 * R, xa);
        if (second) reduce(rb + R, xb);
      }
      const float mine = __int_as_float(__builtin_amdgcn_ds_bpermute(gather_from << 2, __float_as_int(res)));
      if (lane < cnt) a.out[e + lane] = ACC ? prev_a + mine : mine;
      col_a = col_n;
      prev_a = prev_n;
    }
    ask_next();

    lo_a = lo_b;
    hi_a = hi_b;
    row_a = row_b;
    col_a = col_b;
#pragma unroll
    for (int k = 0; k < NT; ++k) y_a[k] = y_b[k];
    prev_a = prev_b;
    lo_b = lo_c;
    hi_b = hi_c;
    row_b = row_c;
    item += n_waves;
  }
}

// The row-run schedule for the elementwise edge functions, Out[e, :] = Src[col[e], :] op Dst[row[e], :]: the same
// (column block, row) work items, the row's Dst tile in registers, one gathered Src tile per edge out of a band
// that an L2 holds -- and a 16-byte store per lane in place of the reduction, the edges of a round next to each
// other in Out.  The edge-parallel kernel of general.hip gathers both rows from all over the matrices; on the
// 114.6M-edge benchmark graph its Src gathers cross the L2 boundary once per edge, as much traffic again as the
// result itself.
template <int OP, bool BUF, int G>
__global__ __launch_bounds__(kBlockThreads) void sddmm_rows_elementwise_kernel(const RowsArgs a) {
  constexpr int NG = kWaveSize / G;  // edges per round
  constexpr int R = 4;               // rounds whose gathers are issued together; two such batches alternate
  const int lane = threadIdx.x & (kWaveSize - 1);
  const int gl = lane & (G - 1);
  const int g = lane / G;
  const int n = a.n_rows;
  int pass, item, n_waves;
  rows_wave_place(a, pass, item, n_waves);
  item = __builtin_amdgcn_readfirstlane(item);
  if (pass * a.merge >= a.n_blocks) return;
  const int32_t *const seg_lo = a.seg + static_cast<int64_t>(pass) * a.merge * n;
  const int32_t *const seg_hi = a.seg + static_cast<int64_t>(min((pass + 1) * a.merge, a.n_blocks)) * n;
  const VertexRows<BUF> src(a.src, a.src_bytes), dst(a.dst, a.dst_bytes);
  const uint32_t row_bytes = static_cast<uint32_t>(a.pitch) * 4u;
  const bool kok = gl * 4 < a.valid;  // lanes past the tile's end re-read its last four floats and store nothing
  const uint32_t lane_bytes = static_cast<uint32_t>(a.first + (kok ? gl * 4 : a.valid - 4)) * 4u;
  float *const out_lane = a.out + a.first + gl * 4;
  const int64_t F = a.F;

  auto bounds = [&](int it, int &lo, int &hi, int &row) {
    lo = hi = row = 0;
    if (it < n) {
      lo = seg_lo[it];
      hi = seg_hi[it];
      row = a.row_order[it];
    }
  };
  auto first_block = [&](int lo, int hi, int row, int &col, float4 &y) {
    col = 0;
    y = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
    if (hi > lo) {
      if (lane < hi - lo) col = a.col[lo + lane];
      y = dst.load(row, row_bytes, lane_bytes);
    }
  };

  int lo_a, hi_a, row_a, col_a, lo_b, hi_b, row_b;
  float4 y_a;
  bounds(item, lo_a, hi_a, row_a);
  first_block(lo_a, hi_a, row_a, col_a, y_a);
  bounds(item + n_waves, lo_b, hi_b, row_b);

  while (item < n) {
    int lo_c, hi_c, row_c, col_b = 0;
    float4 y_b = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
    bounds(item + 2 * n_waves, lo_c, hi_c, row_c);
    bool next_asked = false;
    auto ask_next = [&]() {
      if (!next_asked) first_block(lo_b, hi_b, row_b, col_b, y_b);
      next_asked = true;
    };

    for (int e = lo_a; e < hi_a; e += kWaveSize) {
      const int cnt = min(kWaveSize, hi_a - e);
      int col_n = 0;
      const int rounds = (cnt + NG - 1) / NG;
      float4 xa[R], xb[R];
      auto issue = [&](int rb, float4(&x)[R]) {
#pragma unroll
        for (int r = 0; r < R; ++r) {
          // edges past the run's end read column id 0 of an idle lane: a valid row, nothing stored
          const int cc = __builtin_amdgcn_ds_bpermute(((NG * (rb + r) + g) & 63) << 2, col_a);
          x[r] = src.load(cc, row_bytes, lane_bytes);
        }
      };
      auto store = [&](int rb, const float4(&x)[R]) {
#pragma unroll
        for (int r = 0; r < R; ++r) {
          const int idx = NG * (rb + r) + g;
          float4 v;
          if constexpr (OP == FG_EDGE_ADD) v = make_float4(x[r].x + y_a.x, x[r].y + y_a.y, x[r].z + y_a.z, x[r].w + y_a.w);
          if constexpr (OP == FG_EDGE_SUB) v = make_float4(x[r].x - y_a.x, x[r].y - y_a.y, x[r].z - y_a.z, x[r].w - y_a.w);
          if constexpr (OP == FG_EDGE_MUL) v = make_float4(x[r].x * y_a.x, x[r].y * y_a.y, x[r].z * y_a.z, x[r].w * y_a.w);
          if constexpr (OP == FG_EDGE_DIV) v = make_float4(x[r].x / y_a.x, x[r].y / y_a.y, x[r].z / y_a.z, x[r].w / y_a.w);
          if (idx < cnt && kok) *reinterpret_cast<float4 *>(out_lane + static_cast<int64_t>(e + idx) * F) = v;
        }
      };
      issue(0, xa);
      {  // behind this run's first gathers: the next run's operands and this run's next 64 ids
        ask_next();
        const int more = hi_a - (e + kWaveSize);
        if (lane < more) col_n = a.col[e + kWaveSize + lane];
      }
      for (int rb = 0; rb < rounds; rb += 2 * R) {
        const bool second = rb + R < rounds;
        if (second) issue(rb + R, xb);
        store(rb, xa);
        if (rb + 2 * R < rounds) issue(rb + 2 * R, xa);
        if (second) store(rb + R, xb);
      }
      col_a = col_n;
    }
    ask_next();

    lo_a = lo_b;
    hi_a = hi_b;
    row_a = row_b;
    col_a = col_b;
    y_a = y_b;
    lo_b = lo_c;
    hi_b = hi_c;
    row_b = row_c;
    item += n_waves;
  }
}

template <int VEC, int G>
int launch(const SddmmArgs &a, hipStream_t stream) {
  const int64_t per_wave = static_cast<int64_t>(a.batches) * kWaveSize;
  const int64_t waves = (a.n_ve + per_wave - 1) / per_wave;
  const int64_t blocks = (waves + kWavesPerBlock - 1) / kWavesPerBlock;
  if (blocks > 0x7fffffffLL) return fail(FG_EUNSUPPORTED, "SDDMM launch needs %lld blocks", (long long)blocks);
  if (a.H > 1)
    sddmm_kernel<VEC, G, true><<<dim3((unsigned)blocks), dim3(kBlockThreads), 0, stream>>>(a);
  else
    sddmm_kernel<VEC, G, false><<<dim3((unsigned)blocks), dim3(kBlockThreads), 0, stream>>>(a);
  FG_HIP_TRY(hipGetLastError());
  return FG_OK;
}

template <int VEC>
int dispatch_group(const SddmmArgs &a, const SddmmShape &s, hipStream_t stream) {
  switch (s.group) {
    case 1: return launch<VEC, 1>(a, stream);
    case 2: return launch<VEC, 2>(a, stream);
    case 4: return launch<VEC, 4>(a, stream);
    case 8: return launch<VEC, 8>(a, stream);
    case 16: return launch<VEC, 16>(a, stream);
  }
  return fail(FG_EINVAL, "sddmm lanes per dot product %d is not one of 1, 2, 4, 8, 16", s.group);
}

}  // namespace

SddmmShape sddmm_choose_shape(const SddmmArgs &a) {
  const Config &cfg = config();
  SddmmShape s;
  if (a.D % 4 == 0 && aligned_to(a.src, 16) && aligned_to(a.dst, 16))
    s.vec = 4;
  else if (a.D % 2 == 0 && aligned_to(a.src, 8) && aligned_to(a.dst, 8))
    s.vec = 2;
  else
    s.vec = 1;
  int g = pow2_ceil((a.D + s.vec - 1) / s.vec);
  if (g > 16) g = 16;
  s.group = cfg.sddmm_group > 0 ? cfg.sddmm_group : g;
  s.batches = cfg.sddmm_batches > 0 ? cfg.sddmm_batches : 4;
  return s;
}

// Fast variant for this (H, D), or 1 when there is none.
static int sddmm_launch_fast(const SddmmArgs &a, hipStream_t stream) {
  if (a.D % 4 != 0 || !aligned_to(a.src, 16) || !aligned_to(a.dst, 16) || config().sddmm_fast == 0) return 1;
  FastArgs f;
  f.row = a.row;
  f.col = a.col;
  f.pos = nullptr;
  f.src = a.src;
  f.dst = a.dst;
  f.out = a.out;
  f.n_ve = a.n_ve;
  f.src_bytes = a.src_bytes;
  f.dst_bytes = a.dst_bytes;
  f.H = a.H;
  f.D = a.D;
  f.stride = a.stride;
  f.first = 0;
  f.valid = a.D < 64 ? a.D : 64;
  const bool mh = a.H > 1;
  switch (a.D) {
    case 16: return mh ? launch_fast_mode<4, 1, true, 0>(f, stream) : launch_fast_mode<4, 1, false, 0>(f, stream);
    case 32: return mh ? launch_fast_mode<8, 1, true, 0>(f, stream) : launch_fast_mode<8, 1, false, 0>(f, stream);
    case 64: return mh ? launch_fast_mode<16, 1, true, 0>(f, stream) : launch_fast_mode<16, 1, false, 0>(f, stream);
    case 128: return mh ? launch_fast_mode<16, 2, true, 0>(f, stream) : launch_fast_mode<16, 2, false, 0>(f, stream);
    case 256: return mh ? launch_fast_mode<16, 4, true, 0>(f, stream) : launch_fast_mode<16, 4, false, 0>(f, stream);
    case 512: return mh ? launch_fast_mode<16, 8, true, 0>(f, stream) : launch_fast_mode<16, 8, false, 0>(f, stream);
  }
  return 1;
}

int sddmm_tile_launch(const int32_t *row_p, const int32_t *col_p, const int32_t *pos_p, int64_t nnz, const float *src,
                      const float *dst, float *out, int64_t src_bytes, int64_t dst_bytes, int32_t F, int tile,
                      hipStream_t stream) {
  FastArgs f;
  f.row = row_p;
  f.col = col_p;
  f.pos = pos_p;
  f.src = src;
  f.dst = dst;
  f.out = out;
  f.n_ve = nnz;
  f.src_bytes = src_bytes;
  f.dst_bytes = dst_bytes;
  f.H = 1;
  f.D = F;
  f.stride = F;
  f.first = tile * 64;
  f.valid = F - tile * 64 < 64 ? F - tile * 64 : 64;
  return tile == 0 ? launch_fast_mode<16, 1, false, 1>(f, stream) : launch_fast_mode<16, 1, false, 2>(f, stream);
}

template <int G, int NT, bool CUT>
static void rows_dispatch_cut(const RowsArgs &a, bool acc, bool buf, dim3 grid, hipStream_t stream) {
  constexpr int R = NT == 2 ? 1 : 2;  // rounds per batch: four 16-byte gathers in flight per lane, two batches
  if (!acc) {
    if (buf)
      sddmm_rows_kernel<false, true, R, G, NT, CUT><<<grid, dim3(kBlockThreads), 0, stream>>>(a);
    else
      sddmm_rows_kernel<false, false, R, G, NT, CUT><<<grid, dim3(kBlockThreads), 0, stream>>>(a);
  } else {
    if (buf)
      sddmm_rows_kernel<true, true, R, G, NT, CUT><<<grid, dim3(kBlockThreads), 0, stream>>>(a);
    else
      sddmm_rows_kernel<true, false, R, G, NT, CUT><<<grid, dim3(kBlockThreads), 0, stream>>>(a);
  }
}

template <int G, int NT>
static void rows_dispatch(const RowsArgs &a, bool acc, bool buf, dim3 grid, hipStream_t stream) {
  if (a.valid % 4 != 0)
    rows_dispatch_cut<G, NT, true>(a, acc, buf, grid, stream);
  else
    rows_dispatch_cut<G, NT, false>(a, acc, buf, grid, stream);
}

// Width of the (first) tile: the whole row when it is short (then fewer lanes share a dot product), else 64
// floats, or 128 when wide tiles are allowed and the row has that many left.  (256-float tiles over passes of
// a quarter of the width measured slower: 8.6 against 7.7 ms at 256 floats on the 114.6M-edge benchmark graph.)
int sddmm_rows_tile(int32_t F, int max_wide) {
  if (F <= 16) return 16;
  if (F <= 32) return 32;
  if (max_wide >= 2 && F > 96) return 128;  // 97 .. 127 floats: one partly filled wide tile beats two 64-float launches
  return 64;
}

// Grid of a row-run launch over `passes` passes with `blocks` workgroups each.  With eight passes or more the
// passes are pinned to the dies (RowsArgs::xcd_passes): grid.x = 8 * blocks, grid.y = rounds of eight passes;
// workgroups are dispatched x-fastest and 8 divides grid.x, so workgroup (x, y) runs on die x % 8.
static dim3 rows_grid(RowsArgs &a, int64_t blocks, int passes) {
  const int want = config().sddmm_xcd;
  a.xcd_passes = (want != 0 && passes >= kXcds) ? 1 : 0;
  if (a.xcd_passes)
    return dim3(static_cast<unsigned>(blocks * kXcds), static_cast<unsigned>((passes + kXcds - 1) / kXcds));
  return dim3(static_cast<unsigned>(blocks), static_cast<unsigned>(passes));
}

int sddmm_rows_launch(const int32_t *seg, const int32_t *row_order, int32_t n_rows, int32_t n_blocks, int32_t merge64,
                      int max_wide, const int32_t *col, const float *src, const float *dst, float *out,
                      int64_t src_bytes, int64_t dst_bytes, int32_t F, int32_t pitch, hipStream_t stream) {
  if (n_rows == 0) return FG_OK;
  RowsArgs a;
  a.pitch = pitch;
  a.seg = seg;
  a.row_order = row_order;
  a.col = col;
  a.src = src;
  a.dst = dst;
  a.out = out;
  a.src_bytes = src_bytes;
  a.dst_bytes = dst_bytes;
  a.n_rows = n_rows;
  a.F = F;
  int64_t blocks = config().sddmm_rows_blocks > 0 ? config().sddmm_rows_blocks : 16384;
  blocks = std::max<int64_t>(1, std::min<int64_t>(blocks, (n_rows + kWavesPerBlock - 1) / kWavesPerBlock));
  a.n_blocks = n_blocks;
  const bool buf = src_bytes < (int64_t{1} << 32) && dst_bytes < (int64_t{1} << 32) && config().sddmm_buffer_loads != 0;
  // One launch per tile; every launch after the first adds to the partial dot products that the one before
  // left in Out.  A long row is cut into the widest tiles allowed, its rest into narrower ones.
  for (int first = 0; first < F;) {
    const int tile = sddmm_rows_tile(F - first, max_wide);
    // the band a pass gathers from keeps its size: wider tiles take fewer of the table's blocks per pass
    // (merge64 = 0: the caller sized the blocks, one per pass whatever the tile)
    const int merge = std::max(1, std::min(tile <= 64 ? merge64 * (64 / tile) : merge64 / (tile / 64), n_blocks));
    a.merge = merge;
    a.first = first;
    a.valid = std::min(F - first, tile);
    const dim3 grid = rows_grid(a, blocks, (n_blocks + merge - 1) / merge);
    const bool acc = first > 0;
    if (tile == 16)
      rows_dispatch<4, 1>(a, acc, buf, grid, stream);
    else if (tile == 32)
      rows_dispatch<8, 1>(a, acc, buf, grid, stream);
    else if (tile == 64)
      rows_dispatch<16, 1>(a, acc, buf, grid, stream);
    else
      rows_dispatch<16, 2>(a, acc, buf, grid, stream);
    FG_HIP_TRY(hipGetLastError());
    first += a.valid;
  }
  return FG_OK;
}

template <int OP>
static void rows_elementwise_dispatch(const RowsArgs &a, int tile, bool buf, dim3 grid, hipStream_t stream) {
  if (tile == 16) {
    if (buf) sddmm_rows_elementwise_kernel<OP, true, 4><<<grid, dim3(kBlockThreads), 0, stream>>>(a);
    else sddmm_rows_elementwise_kernel<OP, false, 4><<<grid, dim3(kBlockThreads), 0, stream>>>(a);
  } else if (tile == 32) {
    if (buf) sddmm_rows_elementwise_kernel<OP, true, 8><<<grid, dim3(kBlockThreads), 0, stream>>>(a);
    else sddmm_rows_elementwise_kernel<OP, false, 8><<<grid, dim3(kBlockThreads), 0, stream>>>(a);
  } else {
    if (buf) sddmm_rows_elementwise_kernel<OP, true, 16><<<grid, dim3(kBlockThreads), 0, stream>>>(a);
    else sddmm_rows_elementwise_kernel<OP, false, 16><<<grid, dim3(kBlockThreads), 0, stream>>>(a);
  }
}

// Out [nnz, F]; same tables and pass widths as sddmm_rows_launch, one launch per tile of 16 / 32 / 64 floats,
// each writing its slice of every edge's row.  src / dst / out 16-byte aligned, F a multiple of 4.
int sddmm_rows_elementwise_launch(const int32_t *seg, const int32_t *row_order, int32_t n_rows, int32_t n_blocks,
                                  int32_t merge64, const int32_t *col, const float *src, const float *dst, float *out,
                                  int64_t src_bytes, int64_t dst_bytes, int32_t F, int op, hipStream_t stream) {
  if (n_rows == 0) return FG_OK;
  if (op < FG_EDGE_ADD || op > FG_EDGE_DIV) return fail(FG_EINVAL, "edge_op = %d is not an elementwise FG_EDGE_* code", op);
  RowsArgs a;
  a.pitch = F;
  a.seg = seg;
  a.row_order = row_order;
  a.col = col;
  a.src = src;
  a.dst = dst;
  a.out = out;
  a.src_bytes = src_bytes;
  a.dst_bytes = dst_bytes;
  a.n_rows = n_rows;
  a.F = F;
  int64_t blocks = config().sddmm_rows_blocks > 0 ? config().sddmm_rows_blocks : 16384;
  blocks = std::max<int64_t>(1, std::min<int64_t>(blocks, (n_rows + kWavesPerBlock - 1) / kWavesPerBlock));
  a.n_blocks = n_blocks;
  const bool buf = src_bytes < (int64_t{1} << 32) && dst_bytes < (int64_t{1} << 32) && config().sddmm_buffer_loads != 0;
  for (int first = 0; first < F;) {
    const int tile = sddmm_rows_tile(F - first, 1);
    a.merge = std::max(1, std::min(merge64 * (64 / tile), n_blocks));
    a.first = first;
    a.valid = std::min(F - first, tile);
    const dim3 grid = rows_grid(a, blocks, (n_blocks + a.merge - 1) / a.merge);
    switch (op) {
      case FG_EDGE_ADD: rows_elementwise_dispatch<FG_EDGE_ADD>(a, tile, buf, grid, stream); break;
      case FG_EDGE_SUB: rows_elementwise_dispatch<FG_EDGE_SUB>(a, tile, buf, grid, stream); break;
      case FG_EDGE_MUL: rows_elementwise_dispatch<FG_EDGE_MUL>(a, tile, buf, grid, stream); break;
      default: rows_elementwise_dispatch<FG_EDGE_DIV>(a, tile, buf, grid, stream); break;
    }
    FG_HIP_TRY(hipGetLastError());
    first += a.valid;
  }
  return FG_OK;
}

int sddmm_launch(const SddmmArgs &a, const SddmmShape &s, hipStream_t stream) {
  if (a.n_ve == 0) return FG_OK;
  if (config().sddmm_group == 0) {  // an explicit group size asks for the general kernel
    const int rc = sddmm_launch_fast(a, stream);
    if (rc != 1) return rc;
  }
  SddmmArgs b = a;
  b.batches = s.batches;
  switch (s.vec) {
    case 1: return dispatch_group<1>(b, s, stream);
    case 2: return dispatch_group<2>(b, s, stream);
    case 4: return dispatch_group<4>(b, s, stream);
  }
  return fail(FG_EINVAL, "sddmm floats per lane %d is not one of 1, 2, 4", s.vec);
}

}  // namespace fg
