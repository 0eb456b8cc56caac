// Edge softmax, alone and fused into multi-head SDDMM (gfx950).
//
// In a GAT-style layer the attention scores S[e, h] of multi-head SDDMM are normalised over the edges of each
// destination row before multi-head SpMM consumes them:
//   A[e, h] = exp(S[e, h] - max_r,h) / sum over the row's edges e' of exp(S[e', h] - max_r,h).
// The reference has neither operator; the edge list is the CSR one (row-sorted), so a destination row's
// edges are consecutive and a wave can own a row.
//
// edge_softmax_kernel   one wave per row; the row's deg*H scores are 64 consecutive floats per step, lane l
//                       holding head l % H.  One pass keeps a running (max, sum of exponentials) per lane
//                       (the sum is rescaled whenever the max grows), a butterfly over the lanes of equal head
//                       merges them, a second pass writes the normalised values.
// sddmm_softmax_kernel  the same with the scores computed on the spot: the wave keeps its row's Dst features in
//                       registers (VEC floats per lane, LPH = 64/H lanes per head), gathers LPH neighbours per
//                       step, reduces each head's partial dot products inside its LPH lanes with DPP, and
//                       lane j of head h keeps neighbour j's score, so a step's LPH*H raw scores are 64
//                       consecutive floats of Out.  Rows of at most 64 edges keep their raw scores in registers
//                       and store each weight once; longer rows store the raw scores, and after the row's
//                       last step every lane re-reads the ones it wrote itself and normalises them in place.
//                       The raw scores never make the round trip through a separate kernel.
#include <algorithm>
#include <cmath>

#include "common.hpp"
#include "rowlayout.hpp"

namespace fg {
namespace {

// Running softmax state: m = largest score seen, l = sum of exp(score - m).
struct MaxSum {
  float m, l;
};

__device__ __forceinline__ void absorb(MaxSum &s, float x) {
  // a masked edge (score -inf) adds nothing, whichever position it has: without this a -inf that comes before
  // the row's first finite score would compute exp(-inf - -inf) = NaN
  if (x == -__builtin_inff()) return;
  if (x > s.m) {
    s.l = s.l * expf(s.m - x) + 1.0f;  // exp(-inf) = 0 covers the first score
    s.m = x;
  } else {
    s.l += expf(x - s.m);
  }
}

__device__ __forceinline__ MaxSum merge(const MaxSum &a, const MaxSum &b) {
  MaxSum r;
  r.m = fmaxf(a.m, b.m);
  // a side that has seen nothing has m = -inf and l = 0: its term must vanish, not become NaN
  const float la = a.l == 0.0f ? 0.0f : a.l * expf(a.m - r.m);
  const float lb = b.l == 0.0f ? 0.0f : b.l * expf(b.m - r.m);
  r.l = la + lb;
  return r;
}

// Merges the states of all lanes whose index agrees modulo `stride0` (a power of two below 64).
__device__ __forceinline__ MaxSum merge_lanes(MaxSum s, int stride0) {
  for (int d = stride0; d < kWaveSize; d <<= 1) {
    MaxSum o;
    o.m = __shfl_xor(s.m, d, kWaveSize);
    o.l = __shfl_xor(s.l, d, kWaveSize);
    s = merge(s, o);
  }
  return s;
}

// Second pass over a row's deg*H scores (consecutive floats starting at p): normalise in place / into q.
__device__ __forceinline__ void normalise_row(const float *p, float *q, int64_t count, int lane, float m, float l) {
  const float inv = 1.0f / l;
  for (int64_t t = lane; t < count; t += kWaveSize) q[t] = expf(p[t] - m) * inv;
}

// H divides 64.
__global__ __launch_bounds__(kBlockThreads) void edge_softmax_kernel(const int32_t *indptr, const float *scores,
                                                                     float *out, int32_t n_rows, int32_t H) {
  const int lane = threadIdx.x & (kWaveSize - 1);
  const int64_t n_waves = static_cast<int64_t>(gridDim.x) * kWavesPerBlock;
  for (int64_t r = static_cast<int64_t>(blockIdx.x) * kWavesPerBlock + (threadIdx.x >> 6); r < n_rows; r += n_waves) {
    const int64_t lo = indptr[r], hi = indptr[r + 1];
    if (hi <= lo) continue;
    const float *p = scores + lo * H;
    const int64_t count = (hi - lo) * H;
    MaxSum s = {-__builtin_inff(), 0.0f};
    for (int64_t t = lane; t < count; t += kWaveSize) absorb(s, p[t]);  // 64 % H == 0: t % H == lane % H
    s = merge_lanes(s, H);
    normalise_row(p, out + lo * H, count, lane, s.m, s.l);
  }
}

// Any H: lane j walks the edges lo + j, lo + j + 64, ... of the row, head by head.
__global__ __launch_bounds__(kBlockThreads) void edge_softmax_any_kernel(const int32_t *indptr, const float *scores,
                                                                         float *out, int32_t n_rows, int32_t H) {
  const int lane = threadIdx.x & (kWaveSize - 1);
  const int64_t n_waves = static_cast<int64_t>(gridDim.x) * kWavesPerBlock;
  for (int64_t r = static_cast<int64_t>(blockIdx.x) * kWavesPerBlock + (threadIdx.x >> 6); r < n_rows; r += n_waves) {
    const int64_t lo = indptr[r], hi = indptr[r + 1];
    for (int h = 0; h < H && hi > lo; ++h) {
      MaxSum s = {-__builtin_inff(), 0.0f};
      for (int64_t e = lo + lane; e < hi; e += kWaveSize) absorb(s, scores[e * H + h]);
      s = merge_lanes(s, 1);
      const float inv = 1.0f / s.l;
      for (int64_t e = lo + lane; e < hi; e += kWaveSize) out[e * H + h] = expf(scores[e * H + h] - s.m) * inv;
    }
  }
}

struct FusedArgs {
  const int32_t *row_order;  // rows by descending degree, or null for natural order
  const int32_t *indptr;
  const int32_t *indices;
  const float *src;  // [n_cols, H, D], gathered by column id
  const float *dst;  // [n_rows, H, D]
  float *out;        // [nnz, H]
  int32_t n_rows;
};

// Layout of a vertex row (H * D floats) over a wave: NV chunks of 64 * VW floats; in chunk k lane l holds the
// VW floats at k * 64 * VW + l * VW, so every load instruction of a gather covers consecutive addresses.  LC =
// D / VW adjacent lanes share a head inside a chunk, a chunk holds HC = 64 / LC heads, H = NV * HC.  A step takes
// EB = 64 / H neighbours; after the reduction over the LC lanes, lane jj of group g keeps, for chunk jj / EB and
// neighbour jj % EB, head (jj / EB) * HC + g: a step's 64 scores, 64 consecutive floats of Out.
template <int LC, int VW, int NV>
__global__ __launch_bounds__(kBlockThreads) void sddmm_softmax_kernel(const FusedArgs a) {
  constexpr int HC = kWaveSize / LC;
  constexpr int H = NV * HC;
  constexpr int EB = kWaveSize / H;
  constexpr int64_t ROW = int64_t{kWaveSize} * VW * NV;  // floats per vertex
  constexpr int CH = EB * NV * VW > 64 ? 64 / (NV * VW) : EB;  // neighbours whose gathers are in flight together
  static_assert(EB >= 1 && EB * NV == LC, "a step must fill the wave with scores");
  const int lane = threadIdx.x & (kWaveSize - 1);
  const int jj = lane & (LC - 1);
  const int g = lane / LC;
  const int my_edge = jj % EB;                 // which neighbour of a step this lane keeps
  const int my_chunk = jj / EB;                // ... and from which chunk
  const int my_head = my_chunk * HC + g;
  const int64_t n_waves = static_cast<int64_t>(gridDim.x) * kWavesPerBlock;
  for (int64_t i = static_cast<int64_t>(blockIdx.x) * kWavesPerBlock + (threadIdx.x >> 6); i < a.n_rows; i += n_waves) {
    const int r = __builtin_amdgcn_readfirstlane(a.row_order ? a.row_order[i] : static_cast<int>(i));
    const int lo = __builtin_amdgcn_readfirstlane(a.indptr[r]);
    const int hi = __builtin_amdgcn_readfirstlane(a.indptr[r + 1]);
    if (hi <= lo) continue;
    Floats<VW> y[NV];
#pragma unroll
    for (int k = 0; k < NV; ++k)
      y[k] = load_floats<VW>(a.dst + static_cast<int64_t>(r) * ROW + k * kWaveSize * VW + lane * VW);
    // this lane computes, stores, re-reads and normalises the scores (neighbour lo + my_edge + EB * step, head
    // my_head): the second pass only ever reads what the same lane wrote
    float *const mine_out = a.out + static_cast<int64_t>(lo) * H + static_cast<int64_t>(my_edge) * H + my_head;
    MaxSum s = {-__builtin_inff(), 0.0f};
    // one step: the scores of the EB neighbours whose column ids sit in lanes b .. b + EB - 1 of my_col; returns
    // this lane's.  (Issuing several steps' gathers together measured slower: more idle slots in short rows.)
    auto step = [&](int my_col, int b) {
      float mine = 0.0f;
      {
#pragma unroll
        for (int u0 = 0; u0 < EB; u0 += CH) {
          Floats<VW> x[CH][NV];
#pragma unroll
          for (int u = 0; u < CH; ++u) {
            // neighbours past the row's end gather vertex 0: valid memory, result dropped
            const int c = __builtin_amdgcn_readlane(my_col, (b + u0 + u) & (kWaveSize - 1));
#pragma unroll
            for (int k = 0; k < NV; ++k)
              x[u][k] = load_floats<VW>(a.src + static_cast<int64_t>(c) * ROW + k * kWaveSize * VW + lane * VW);
          }
#pragma unroll
          for (int u = 0; u < CH; ++u) {
#pragma unroll
            for (int k = 0; k < NV; ++k) {
              float p = 0.0f;
#pragma unroll
              for (int q = 0; q < VW; ++q) p = __builtin_fmaf(x[u][k].v[q], y[k].v[q], p);
              p = group_sum<LC>(p);
              if (my_edge == u0 + u && my_chunk == k) mine = p;
            }
          }
        }
      }
      return mine;
    };
    auto merge_head = [&]() {  // the lanes that hold one head: jj = my_chunk * EB + 0 .. EB - 1 of one group
      for (int d = 1; d < EB; d <<= 1) {
        MaxSum o;
        o.m = __shfl_xor(s.m, d, kWaveSize);
        o.l = __shfl_xor(s.l, d, kWaveSize);
        s = merge(s, o);
      }
    };
    const int deg = hi - lo;
    if (deg <= kWaveSize) {
      // short rows (most of a power-law graph): the raw scores stay in registers, one store per weight
      constexpr int STEPS = kWaveSize / EB;
      const int my_col = lane < deg ? a.indices[lo + lane] : 0;
      float mine[STEPS];
#pragma unroll
      for (int st = 0; st < STEPS; ++st) {
        mine[st] = 0.0f;
        if (st * EB < deg) {  // wave-uniform
          mine[st] = step(my_col, st * EB);
          if (st * EB + my_edge < deg) absorb(s, mine[st]);
        }
      }
      merge_head();
      const float inv = 1.0f / s.l;
#pragma unroll
      for (int st = 0; st < STEPS; ++st)
        if (st * EB + my_edge < deg) mine_out[static_cast<int64_t>(st * EB) * H] = expf(mine[st] - s.m) * inv;
      continue;
    }
    for (int e = lo; e < hi; e += kWaveSize) {
      const int cnt = min(kWaveSize, hi - e);  // wave-uniform
      const int my_col = lane < cnt ? a.indices[e + lane] : 0;
      for (int b = 0; b < cnt; b += EB) {
        const float mine = step(my_col, b);
        if (b + my_edge < cnt) {
          mine_out[static_cast<int64_t>(e - lo + b) * H] = mine;
          absorb(s, mine);
        }
      }
    }
    merge_head();
    const float inv = 1.0f / s.l;
    for (int t = my_edge; t < deg; t += EB) {
      float *p = mine_out + static_cast<int64_t>(t - my_edge) * H;
      *p = expf(*p - s.m) * inv;
    }
  }
}

template <int LC, int VW, int NV>
int launch_fused(const FusedArgs &a, hipStream_t stream) {
  const int64_t blocks = std::min<int64_t>((static_cast<int64_t>(a.n_rows) + kWavesPerBlock - 1) / kWavesPerBlock, 1 << 16);
  sddmm_softmax_kernel<LC, VW, NV><<<dim3(static_cast<unsigned>(blocks)), dim3(kBlockThreads), 0, stream>>>(a);
  FG_HIP_TRY(hipGetLastError());
  return FG_OK;
}

}  // namespace

int edge_softmax_launch(const int32_t *indptr, const float *scores, float *out, int32_t n_rows, int32_t H,
                        hipStream_t stream) {
  if (n_rows == 0) return FG_OK;
  const unsigned blocks = static_cast<unsigned>(
      std::min<int64_t>((static_cast<int64_t>(n_rows) + kWavesPerBlock - 1) / kWavesPerBlock, 1 << 16));
  if (H <= kWaveSize && kWaveSize % H == 0)
    edge_softmax_kernel<<<dim3(blocks), dim3(kBlockThreads), 0, stream>>>(indptr, scores, out, n_rows, H);
  else
    edge_softmax_any_kernel<<<dim3(blocks), dim3(kBlockThreads), 0, stream>>>(indptr, scores, out, n_rows, H);
  FG_HIP_TRY(hipGetLastError());
  return FG_OK;
}

// Whether the fused kernel covers this shape (see fused_layout) with operands aligned for its loads.
bool sddmm_softmax_fused_applies(const float *src, const float *dst, int32_t H, int32_t D) {
  int lc, vw, nv;
  if (H < 1 || D < 1 || !row_layout(H, D, &lc, &vw, &nv)) return false;
  return aligned_to(src, vw * 4) && aligned_to(dst, vw * 4);
}

int sddmm_softmax_launch(const int32_t *row_order, const int32_t *indptr, const int32_t *indices, const float *src,
                         const float *dst, float *out, int32_t n_rows, int32_t H, int32_t D, hipStream_t stream) {
  if (n_rows == 0) return FG_OK;
  FusedArgs a;
  a.row_order = row_order;
  a.indptr = indptr;
  a.indices = indices;
  a.src = src;
  a.dst = dst;
  a.out = out;
  a.n_rows = n_rows;
  int lc, vw, nv;
  if (!row_layout(H, D, &lc, &vw, &nv))
    return fail(FG_EUNSUPPORTED, "the fused score + softmax kernel does not cover H = %d, D = %d", H, D);
#define FG_FUSED_CASE(LC, VW, NV) \
  if (lc == LC && vw == VW && nv == NV) return launch_fused<LC, VW, NV>(a, stream);
  FG_FUSED_CASE(4, 1, 1) FG_FUSED_CASE(4, 2, 1) FG_FUSED_CASE(4, 4, 1)
  FG_FUSED_CASE(8, 1, 1) FG_FUSED_CASE(8, 2, 1) FG_FUSED_CASE(8, 4, 1)
  FG_FUSED_CASE(16, 1, 1) FG_FUSED_CASE(16, 2, 1) FG_FUSED_CASE(16, 4, 1)
  FG_FUSED_CASE(4, 1, 2) FG_FUSED_CASE(4, 2, 2) FG_FUSED_CASE(4, 4, 2)
  FG_FUSED_CASE(8, 1, 2) FG_FUSED_CASE(8, 2, 2) FG_FUSED_CASE(8, 4, 2)
  FG_FUSED_CASE(16, 1, 2) FG_FUSED_CASE(16, 2, 2) FG_FUSED_CASE(16, 4, 2)
#undef FG_FUSED_CASE
  return fail(FG_EUNSUPPORTED, "the fused score + softmax kernel does not cover H = %d, D = %d", H, D);
}

}  // namespace fg
