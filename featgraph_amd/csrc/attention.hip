// Multi-head attention over a sparse graph in one kernel (gfx950): multi-head SDDMM, edge softmax and
// multi-head SpMM without the [nnz, H] scores or weights ever existing in memory.
//
//   out[r, h, :] = sum over the nonzeros e of row r of  A[e, h] * value[indices[e], h, :]
//   A[e, h]      = softmax over the row's nonzeros of   sum_d key[indices[e], h, d] * query[r, h, d]
//
// The reference has the two ends as separate operators (multi-head dot-product attention, the `feat_len = 1`
// footnote of op/vanilla_sddmm.py:35-47, and the multi-head SpMM its benchmarks describe) and nothing in
// between.  Run one after the other they gather every neighbour's row twice and write and re-read the edge
// weights; when `value` is `key` (attention over one set of vertex features) the fused kernel gathers each
// neighbour row once, which halves the traffic of the whole layer.
//
// One wave per destination row, rows in the plan's degree order.  The wave keeps the row's query in registers
// (layout: rowlayout.hpp), takes the neighbours in batches of CH, and keeps per head a running maximum m, the
// sum l of exp(score - m) and the weighted sum acc of value rows, all rescaled by exp(m_old - m_new) when a
// batch raises the maximum: each neighbour row is used for its score and for the weighted sum while it sits in
// registers.  Two batches alternate, so one batch's gathers are in flight while the other is consumed; the next
// row's ids are requested behind the current row's first gathers, and its first batch and its query behind the
// current row's last ones, so the wave never runs out of gathers between rows.  At the end out = acc / l.
#include <algorithm>
#include <cmath>

#include "common.hpp"
#include "rowlayout.hpp"

namespace fg {
namespace {

struct AttnArgs {
  const int32_t *row_order;  // rows by descending degree
  const int32_t *seg_lo;     // first nonzero of the i-th row in visiting order
  const int32_t *seg_hi;     // one past its last
  const int32_t *indices;
  const float *key;    // [n_cols, H, D], gathered by column id
  const float *query;  // [n_rows, H, D]
  const float *value;  // [n_cols, H, D]; equal to key when SHARED
  float *out;          // [n_rows, H, D]
  int32_t n_rows;
};

template <int LC, int VW, int NV, bool SHARED>
__global__ __launch_bounds__(kBlockThreads) void attention_kernel(const AttnArgs a) {
  constexpr int64_t ROW = int64_t{kWaveSize} * VW * NV;  // floats per vertex
  // neighbours per batch: two batches of gathers fit 64 registers (half of that each when values are separate)
  constexpr int CH0 = 32 / (NV * VW) > 8 ? 8 : 32 / (NV * VW);
  constexpr int CH = SHARED ? CH0 : CH0 / 2;
  static_assert(CH >= 2 && kWaveSize % (2 * CH) == 0, "two batches must not straddle a block of 64 ids");
  const int lane = threadIdx.x & (kWaveSize - 1);
  const unsigned lane_off = static_cast<unsigned>(lane) * VW;
  const int n_waves = gridDim.x * kWavesPerBlock;
  const int n = a.n_rows;
  int item = __builtin_amdgcn_readfirstlane(static_cast<int>(blockIdx.x * kWavesPerBlock + (threadIdx.x >> 6)));

  auto bounds = [&](int it, int &lo, int &hi, int &row) {
    lo = hi = row = 0;
    if (it < n) {
      lo = a.seg_lo[it];
      hi = a.seg_hi[it];
      row = a.row_order[it];
    }
  };
  auto first_ids = [&](int lo, int hi, int &col) {
    col = 0;
    if (lane < hi - lo) col = a.indices[lo + lane];
  };
  auto load_query = [&](int row, Floats<VW>(&y)[NV]) {
#pragma unroll
    for (int k = 0; k < NV; ++k)
      y[k] = load_floats<VW>(a.query + static_cast<int64_t>(row) * ROW + (lane_off + k * kWaveSize * VW));
  };

  int lo_a, hi_a, row_a, col_a, lo_b, hi_b, row_b;
  Floats<VW> y_a[NV];
  bounds(item, lo_a, hi_a, row_a);
  first_ids(lo_a, hi_a, col_a);
  load_query(__builtin_amdgcn_readfirstlane(row_a), y_a);  // row 0 when the wave has no row: valid memory
  bounds(item + n_waves, lo_b, hi_b, row_b);

  // Two batches of gathered rows alternate; A's first batch of a row is already in flight when the row's turn
  // comes (`primed`), requested behind the last batches of the row before it.
  Floats<VW> ka[CH][NV], kb[CH][NV];
  Floats<VW> va[SHARED ? 1 : CH][NV], vb[SHARED ? 1 : CH][NV];
  // Gathers of the neighbours t .. t + CH - 1 (t a multiple of CH) of a row of d nonzeros whose current block of
  // 64 column ids sits in `ids`.  A slot past the row's end repeats the row's last neighbour (a cache hit) and a
  // row without nonzeros reads vertex 0, so that every call issues the same number of loads: the compiler can
  // then count which loads a wait has to cover, and a batch's use does not wait for the batch issued after it.
  auto issue = [&](int ids, int t, int d, Floats<VW>(&xk)[CH][NV], Floats<VW>(&xv)[SHARED ? 1 : CH][NV]) {
#pragma unroll
    for (int u = 0; u < CH; ++u) {
      // the row's address is wave-uniform (scalar registers); the lane adds a 32-bit offset
      const int c = __builtin_amdgcn_readlane(ids, min(t + u, d - 1) & (kWaveSize - 1));
      const float *const krow = a.key + static_cast<int64_t>(c) * ROW;
      const float *const vrow = a.value + static_cast<int64_t>(c) * ROW;
#pragma unroll
      for (int k = 0; k < NV; ++k) {
        xk[u][k] = load_floats<VW>(krow + (lane_off + k * kWaveSize * VW));
        if (!SHARED) xv[u][k] = load_floats<VW>(vrow + (lane_off + k * kWaveSize * VW));
      }
    }
  };
  bool primed = false;

  while (item < n) {
    int lo_c, hi_c, row_c, col_b = 0;
    bounds(item + 2 * n_waves, lo_c, hi_c, row_c);
    lo_a = __builtin_amdgcn_readfirstlane(lo_a);
    const int deg = __builtin_amdgcn_readfirstlane(hi_a - lo_a);
    row_a = __builtin_amdgcn_readfirstlane(row_a);
    const int deg_b = __builtin_amdgcn_readfirstlane(hi_b - lo_b);  // 0 past the wave's last row

    float m[NV], l[NV];
    Floats<VW> acc[NV];
#pragma unroll
    for (int k = 0; k < NV; ++k) {
      m[k] = -__builtin_inff();
      l[k] = 0.0f;
#pragma unroll
      for (int q = 0; q < VW; ++q) acc[k].v[q] = 0.0f;
    }
    // ids of the block of 64 neighbours that the batches now read, and of the block after it
    int col_cur = col_a, col_nxt = 0;

    auto consume = [&](int t, const Floats<VW>(&xk)[CH][NV], const Floats<VW>(&xv)[SHARED ? 1 : CH][NV]) {
#pragma unroll
      for (int k = 0; k < NV; ++k) {
        float s[CH];
        float top = m[k];
#pragma unroll
        for (int u = 0; u < CH; ++u) {
          float p = 0.0f;
#pragma unroll
          for (int q = 0; q < VW; ++q) p = __builtin_fmaf(xk[u][k].v[q], y_a[k].v[q], p);
          p = group_sum<LC>(p);
          s[u] = t + u < deg ? p : -__builtin_inff();
          top = fmaxf(top, s[u]);
        }
        // the first neighbour of a batch always exists, so `top` is a score: exp(-inf - top) = 0 clears the
        // empty state and the neighbours past the row's end alike.  A score can itself be -inf (infinite
        // features): such a neighbour, like an empty state, weighs 0 rather than exp(-inf - -inf) = NaN
        const float keep = m[k] == -__builtin_inff() ? 0.0f : expf(m[k] - top);
        m[k] = top;
        l[k] *= keep;
#pragma unroll
        for (int q = 0; q < VW; ++q) acc[k].v[q] *= keep;
#pragma unroll
        for (int u = 0; u < CH; ++u) {
          const float w = s[u] == -__builtin_inff() ? 0.0f : expf(s[u] - top);
          l[k] += w;
#pragma unroll
          for (int q = 0; q < VW; ++q)
            acc[k].v[q] = __builtin_fmaf(w, SHARED ? xk[u][k].v[q] : xv[u][k].v[q], acc[k].v[q]);
        }
      }
    };

    if (deg > 0 && !primed) issue(col_cur, 0, deg, ka, va);
    primed = false;
    // behind this row's first gathers: the next row's ids and this row's second block of ids
    first_ids(lo_b, hi_b, col_b);
    if (deg > kWaveSize && lane < deg - kWaveSize) col_nxt = a.indices[lo_a + kWaveSize + lane];

    for (int t = 0; t < deg; t += 2 * CH) {
      // batches t and t + CH; behind them batch t + 2 CH, which may open the next block of ids, or, when this
      // row has no more, the first batch of the wave's next row
      issue(col_cur, t + CH, deg, kb, vb);
      consume(t, ka, va);
      const bool wraps = ((t + 2 * CH) & (kWaveSize - 1)) == 0;
      const bool more = t + 2 * CH < deg;
      issue(more ? (wraps ? col_nxt : col_cur) : col_b, more ? t + 2 * CH : 0, more ? deg : deg_b, ka, va);
      primed = !more && deg_b > 0;
      if (t + CH < deg) consume(t + CH, kb, vb);
      if (wraps) {
        col_cur = col_nxt;
        col_nxt = 0;
        const int ahead = t + 2 * CH + kWaveSize;  // first neighbour of the block after the one just opened
        if (ahead < deg && lane < deg - ahead) col_nxt = a.indices[lo_a + ahead + lane];
      }
    }

    float *const o = a.out + static_cast<int64_t>(row_a) * ROW + lane_off;
#pragma unroll
    for (int k = 0; k < NV; ++k) {
      Floats<VW> r;
      const float inv = deg > 0 ? 1.0f / l[k] : 0.0f;  // a row without nonzeros gives zeros, as SpMM does
#pragma unroll
      for (int q = 0; q < VW; ++q) r.v[q] = acc[k].v[q] * inv;
      store_floats<VW>(o + k * kWaveSize * VW, r);
    }

    lo_a = lo_b;
    hi_a = hi_b;
    row_a = row_b;
    col_a = col_b;
    // the next row's query, behind its first batch of gathers (row 0 past the wave's last row: valid memory)
    load_query(__builtin_amdgcn_readfirstlane(row_a), y_a);
    lo_b = lo_c;
    hi_b = hi_c;
    row_b = row_c;
    item += n_waves;
  }
}

template <int LC, int VW, int NV>
int launch_attention(const AttnArgs &a, hipStream_t stream) {
  // Rows of 1 KB and more: one row per wave (measured 2 - 4 % faster than waves that walk many rows: a wave
  // that ends after its stores never waits behind them); shorter rows: 65536 workgroups that walk the rows.
  const int64_t all = (static_cast<int64_t>(a.n_rows) + kWavesPerBlock - 1) / kWavesPerBlock;
  const int64_t want = config().attention_blocks > 0 ? config().attention_blocks
                       : kWaveSize * VW * NV >= 256  ? all
                                                     : (1 << 16);
  const int64_t blocks = std::max<int64_t>(1, std::min<int64_t>(all, want));
  const dim3 grid(static_cast<unsigned>(blocks)), block(kBlockThreads);
  if (a.key == a.value)
    attention_kernel<LC, VW, NV, true><<<grid, block, 0, stream>>>(a);
  else
    attention_kernel<LC, VW, NV, false><<<grid, block, 0, stream>>>(a);
  FG_HIP_TRY(hipGetLastError());
  return FG_OK;
}

}  // namespace

bool attention_fused_applies(const float *key, const float *query, const float *value, const float *out, int32_t H,
                             int32_t D) {
  int lc, vw, nv;
  if (H < 1 || D < 1 || !row_layout(H, D, &lc, &vw, &nv)) return false;
  return aligned_to(key, vw * 4) && aligned_to(query, vw * 4) && aligned_to(value, vw * 4) && aligned_to(out, vw * 4);
}

int attention_launch(const int32_t *row_order, const int32_t *seg_lo, const int32_t *seg_hi, const int32_t *indices,
                     const float *key, const float *query, const float *value, float *out, int32_t n_rows, int32_t H,
                     int32_t D, hipStream_t stream) {
  if (n_rows == 0) return FG_OK;
  AttnArgs a;
  a.row_order = row_order;
  a.seg_lo = seg_lo;
  a.seg_hi = seg_hi;
  a.indices = indices;
  a.key = key;
  a.query = query;
  a.value = value;
  a.out = out;
  a.n_rows = n_rows;
  int lc, vw, nv;
  if (!row_layout(H, D, &lc, &vw, &nv))
    return fail(FG_EUNSUPPORTED, "the fused attention kernel does not cover H = %d, D = %d", H, D);
#define FG_ATTN_CASE(LC, VW, NV) \
  if (lc == LC && vw == VW && nv == NV) return launch_attention<LC, VW, NV>(a, stream);
  FG_ATTN_CASE(4, 1, 1) FG_ATTN_CASE(4, 2, 1) FG_ATTN_CASE(4, 4, 1)
  FG_ATTN_CASE(8, 1, 1) FG_ATTN_CASE(8, 2, 1) FG_ATTN_CASE(8, 4, 1)
  FG_ATTN_CASE(16, 1, 1) FG_ATTN_CASE(16, 2, 1) FG_ATTN_CASE(16, 4, 1)
  FG_ATTN_CASE(4, 1, 2) FG_ATTN_CASE(4, 2, 2) FG_ATTN_CASE(4, 4, 2)
  FG_ATTN_CASE(8, 1, 2) FG_ATTN_CASE(8, 2, 2) FG_ATTN_CASE(8, 4, 2)
  FG_ATTN_CASE(16, 1, 2) FG_ATTN_CASE(16, 2, 2) FG_ATTN_CASE(16, 4, 2)
#undef FG_ATTN_CASE
  return fail(FG_EUNSUPPORTED, "the fused attention kernel does not cover H = %d, D = %d", H, D);
}

}  // namespace fg
