// Generalised SpMM and SDDMM: the message / reduce / edge-function slots of the reference's operator
// templates (op/vanilla_spmm.py:46-53 msgfunc + te.sum, op/vanilla_sddmm.py:43-47 edgefunc) opened to other
// operators.  The reference ships only (multiply, sum) and the dot product; README.md:6 names the general form.
//
//   SpMM   term(e, f) = msg(Feat[indices[e], f], vals[e])      msg: u*e, u+e, u-e, u/e, u
//          Out[r, f]  = fold of the row's terms in CSR order   reduce: sum (from +0), max, min,
//                                                              mean = sum / degree (one rounded division)
//          Rows without nonzeros give 0 under every reducer.  max / min fold as acc = (t > acc) ? t : acc, so
//          the result, the sign of a zero included, is fixed by the order.  One rounded operation per message
//          and per fold step (-ffp-contract=off), hence (u*e, sum) equals fg_spmm_csr_f32 bit for bit.
//   SDDMM  Out[e, f] = Src[col[e], f] op Dst[row[e], f]        op: +, -, *, /   (no reduction over f)
//
// The several-rows-per-wave kernel (spmm_multi_kernel.hpp) takes the generalised SpMM where it takes the plain
// one; the kernel here serves the other shapes.
// SpMM kernel: rows come in the plan's order (descending degree); a slot of LPR lanes owns one (row, tile)
// pair, every lane VEC adjacent floats; column ids and values are fetched LPR at a time with one coalesced
// load, a chunk ahead of their use, and handed out inside the slot with cross-lane reads; sixteen gathers are
// in flight per lane.  When the plan has column blocks the operator is one launch per block, each over the
// block's part of every row with the partial fold carried in Out, so a launch gathers from a band of the
// feature matrix that an L2 holds.
#include <algorithm>

#include "common.hpp"

namespace fg {
namespace {

template <int MSG>
__device__ __forceinline__ float message(float u, float e) {
  if constexpr (MSG == FG_MSG_MUL) return u * e;
  if constexpr (MSG == FG_MSG_ADD) return u + e;
  if constexpr (MSG == FG_MSG_SUB) return u - e;
  if constexpr (MSG == FG_MSG_DIV) return u / e;
  return u;
}

template <int RED>
__device__ __forceinline__ float fold(float acc, float t) {
  if constexpr (RED == FG_REDUCE_MAX) return (t > acc) ? t : acc;
  if constexpr (RED == FG_REDUCE_MIN) return (t < acc) ? t : acc;
  return acc + t;
}

struct GeneralArgs {
  const int32_t *row_order;  // rows by descending degree
  const int32_t *seg_lo;     // bounds, in that order, of the part of each row that this launch covers: the
  const int32_t *seg_hi;     // whole row, or its nonzeros inside one column block (a pass)
  const int32_t *row_lo;     // bounds of the whole rows
  const int32_t *row_hi;
  bool first_pass;           // the launch that writes the zeros of rows without nonzeros
  const int32_t *indices;
  const float *vals;
  const float *feat;
  float *out;
  int32_t n_rows, F, n_tiles;
  int32_t H = 1, D = 0;      // multi-head: vals is [nnz, H] and float f of a row belongs to head f / D
};

// MH: per-edge per-head values; a lane's VEC floats lie inside one head (D is a multiple of VEC), and the lane
// reads its head's value of every nonzero itself.
template <int VEC, int LPR, int MSG, int RED, bool MH>
__global__ __launch_bounds__(kBlockThreads) void spmm_general_kernel(const GeneralArgs a) {
  constexpr int RPW = kWaveSize / LPR;
  constexpr int TW = VEC * LPR;
  constexpr int U = 16;
  const int lane = threadIdx.x & (kWaveSize - 1);
  const int sl = lane & (LPR - 1);
  const int64_t slot = (static_cast<int64_t>(blockIdx.x) * kWavesPerBlock + (threadIdx.x >> 6)) * RPW + lane / LPR;
  if (slot >= static_cast<int64_t>(a.n_tiles) * a.n_rows) return;  // a slot leaves as a whole
  const int tile = static_cast<int>(slot / a.n_rows);
  const int i = static_cast<int>(slot - static_cast<int64_t>(tile) * a.n_rows);
  const int row = a.row_order[i];
  const int first = a.seg_lo[i], end = a.seg_hi[i];
  const int row_first = a.row_lo[i], row_end = a.row_hi[i];
  const int f0 = tile * TW + sl * VEC;
  const bool fok = f0 < a.F;  // lanes past a partial last tile only serve the cross-lane reads
  const int64_t F = a.F;
  const float *fp = a.feat + (fok ? f0 : a.F - VEC);
  float *op = a.out + static_cast<int64_t>(row) * F + f0;
  const int head = MH ? (fok ? f0 : a.F - VEC) / a.D : 0;
  const int64_t H = a.H;
  // A pass continues the fold where the pass before it stopped: the value it left in Out.  The pass that holds
  // the row's first nonzero starts afresh (sum: from +0; max / min: with the first message itself, as the
  // reference order of evaluation has it), and a pass without nonzeros of the row leaves Out alone.
  const bool starts = first == row_first;
  if (end <= first) {
    if (a.first_pass && row_end <= row_first && fok) {
      if constexpr (VEC == 4)
        *reinterpret_cast<float4 *>(op) = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
      else
        *op = 0.0f;
    }
    return;
  }
  float acc[VEC];
#pragma unroll
  for (int k = 0; k < VEC; ++k) acc[k] = 0.0f;
  if (!starts && fok) {
    if constexpr (VEC == 4) {
      const float4 q = *reinterpret_cast<const float4 *>(op);
      acc[0] = q.x, acc[1] = q.y, acc[2] = q.z, acc[3] = q.w;
    } else {
      acc[0] = *op;
    }
  }
  constexpr bool PICKS = RED == FG_REDUCE_MAX || RED == FG_REDUCE_MIN;
  // ids and values of the next LPR nonzeros are requested before the gathers of the current ones
  int next_col = 0;
  float next_val = 1.0f;
  if (sl < end - first) {
    next_col = a.indices[first + sl];
    if (!MH && MSG != FG_MSG_COPY_U) next_val = a.vals[first + sl];
  }
  for (int e = first; e < end; e += LPR) {
    const int n = min(LPR, end - e);
    const int my_col = next_col;
    const float my_val = next_val;
    next_col = 0;
    next_val = 1.0f;
    if (sl < end - (e + LPR)) {
      next_col = a.indices[e + LPR + sl];
      if (!MH && MSG != FG_MSG_COPY_U) next_val = a.vals[e + LPR + sl];
    }
    for (int j = 0; j < n; j += U) {
      float x[U][VEC];
      float v[U];
#pragma unroll
      for (int u = 0; u < U; ++u) {
        const int from = ((lane & ~(LPR - 1)) | ((j + u) & (LPR - 1))) << 2;
        const int c = __builtin_amdgcn_ds_bpermute(from, my_col);  // slots past n hold column 0: valid, unused
        if constexpr (MH) {
          v[u] = 1.0f;
          if (MSG != FG_MSG_COPY_U && j + u < n) v[u] = a.vals[static_cast<int64_t>(e + j + u) * H + head];
        } else {
          v[u] = __int_as_float(__builtin_amdgcn_ds_bpermute(from, __float_as_int(my_val)));
        }
        const float *p = fp + static_cast<int64_t>(c) * F;
        if constexpr (VEC == 4) {
          const float4 q = *reinterpret_cast<const float4 *>(p);
          x[u][0] = q.x, x[u][1] = q.y, x[u][2] = q.z, x[u][3] = q.w;
        } else {
          x[u][0] = *p;
        }
      }
#pragma unroll
      for (int u = 0; u < U; ++u)
        if (j + u < n) {
          const bool very_first = PICKS && u == 0 && starts && e == first && j == 0;
#pragma unroll
          for (int k = 0; k < VEC; ++k) {
            const float t = message<MSG>(x[u][k], v[u]);
            acc[k] = very_first ? t : fold<RED>(acc[k], t);
          }
        }
    }
  }
  if (!fok) return;
  if (RED == FG_REDUCE_MEAN && end == row_end) {
    const float count = static_cast<float>(row_end - row_first);
#pragma unroll
    for (int k = 0; k < VEC; ++k) acc[k] = acc[k] / count;
  }
  if constexpr (VEC == 4)
    *reinterpret_cast<float4 *>(op) = make_float4(acc[0], acc[1], acc[2], acc[3]);
  else
    *op = acc[0];
}

template <int VEC, int LPR, int MSG, int RED, bool MH>
int launch_general(const GeneralArgs &a, hipStream_t stream) {
  constexpr int RPW = kWaveSize / LPR;
  const int64_t slots = static_cast<int64_t>(a.n_tiles) * a.n_rows;
  const int64_t blocks = ((slots + RPW - 1) / RPW + kWavesPerBlock - 1) / kWavesPerBlock;
  if (blocks > 0x7fffffffLL) return fail(FG_EUNSUPPORTED, "generalised SpMM launch needs %lld blocks", (long long)blocks);
  spmm_general_kernel<VEC, LPR, MSG, RED, MH><<<dim3(static_cast<unsigned>(blocks)), dim3(kBlockThreads), 0, stream>>>(a);
  FG_HIP_TRY(hipGetLastError());
  return FG_OK;
}

template <int MSG, int RED>
int dispatch_shape(GeneralArgs a, bool vec4, hipStream_t stream) {
  a.n_tiles = (a.F + 63) / 64;  // both shapes cover 64 floats per slot
  if (a.H > 1) {
    if (vec4) return launch_general<4, 16, MSG, RED, true>(a, stream);
    return launch_general<1, 64, MSG, RED, true>(a, stream);
  }
  if (vec4) return launch_general<4, 16, MSG, RED, false>(a, stream);
  return launch_general<1, 64, MSG, RED, false>(a, stream);
}

template <int MSG>
int dispatch_reduce(const GeneralArgs &a, bool vec4, int reduce, hipStream_t stream) {
  switch (reduce) {
    case FG_REDUCE_SUM: return dispatch_shape<MSG, FG_REDUCE_SUM>(a, vec4, stream);
    case FG_REDUCE_MAX: return dispatch_shape<MSG, FG_REDUCE_MAX>(a, vec4, stream);
    case FG_REDUCE_MIN: return dispatch_shape<MSG, FG_REDUCE_MIN>(a, vec4, stream);
    case FG_REDUCE_MEAN: return dispatch_shape<MSG, FG_REDUCE_MEAN>(a, vec4, stream);
  }
  return fail(FG_EINVAL, "reduce = %d is not one of FG_REDUCE_SUM / MAX / MIN / MEAN", reduce);
}

// Thread per (edge, VEC adjacent floats): both operand rows are read with consecutive addresses across the
// threads of an edge, results are written coalesced.
template <int VEC, int OP>
__global__ __launch_bounds__(kBlockThreads) void sddmm_elementwise_kernel(const int32_t *row, const int32_t *col,
                                                                          const float *src, const float *dst,
                                                                          float *out, int64_t nnz, int32_t F) {
  const int64_t chunks = F / VEC;
  const int64_t total = nnz * chunks;
  const int64_t stride = static_cast<int64_t>(gridDim.x) * blockDim.x;
  for (int64_t t = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x; t < total; t += stride) {
    const int64_t e = t / chunks;
    const int64_t f = (t - e * chunks) * VEC;
    const float *pa = src + static_cast<int64_t>(col[e]) * F + f;
    const float *pb = dst + static_cast<int64_t>(row[e]) * F + f;
    float x[VEC], y[VEC], r[VEC];
    if constexpr (VEC == 4) {
      const float4 qa = *reinterpret_cast<const float4 *>(pa), qb = *reinterpret_cast<const float4 *>(pb);
      x[0] = qa.x, x[1] = qa.y, x[2] = qa.z, x[3] = qa.w;
      y[0] = qb.x, y[1] = qb.y, y[2] = qb.z, y[3] = qb.w;
    } else {
      x[0] = *pa;
      y[0] = *pb;
    }
#pragma unroll
    for (int k = 0; k < VEC; ++k) {
      if constexpr (OP == FG_EDGE_ADD) r[k] = x[k] + y[k];
      if constexpr (OP == FG_EDGE_SUB) r[k] = x[k] - y[k];
      if constexpr (OP == FG_EDGE_MUL) r[k] = x[k] * y[k];
      if constexpr (OP == FG_EDGE_DIV) r[k] = x[k] / y[k];
    }
    float *po = out + e * F + f;
    if constexpr (VEC == 4)
      *reinterpret_cast<float4 *>(po) = make_float4(r[0], r[1], r[2], r[3]);
    else
      *po = r[0];
  }
}

template <int OP>
int launch_elementwise(const int32_t *row, const int32_t *col, const float *src, const float *dst, float *out,
                       int64_t nnz, int32_t F, hipStream_t stream) {
  const bool vec4 = F % 4 == 0 && aligned_to(src, 16) && aligned_to(dst, 16) && aligned_to(out, 16);
  const int64_t total = nnz * (vec4 ? F / 4 : F);
  const unsigned blocks = static_cast<unsigned>(std::min<int64_t>((total + kBlockThreads - 1) / kBlockThreads, 1 << 20));
  if (vec4)
    sddmm_elementwise_kernel<4, OP><<<dim3(blocks), dim3(kBlockThreads), 0, stream>>>(row, col, src, dst, out, nnz, F);
  else
    sddmm_elementwise_kernel<1, OP><<<dim3(blocks), dim3(kBlockThreads), 0, stream>>>(row, col, src, dst, out, nnz, F);
  FG_HIP_TRY(hipGetLastError());
  return FG_OK;
}

}  // namespace

static int general_pass(GeneralArgs a, bool vec4, int msg, int reduce, hipStream_t stream) {
  switch (msg) {
    case FG_MSG_MUL: return dispatch_reduce<FG_MSG_MUL>(a, vec4, reduce, stream);
    case FG_MSG_ADD: return dispatch_reduce<FG_MSG_ADD>(a, vec4, reduce, stream);
    case FG_MSG_SUB: return dispatch_reduce<FG_MSG_SUB>(a, vec4, reduce, stream);
    case FG_MSG_DIV: return dispatch_reduce<FG_MSG_DIV>(a, vec4, reduce, stream);
    case FG_MSG_COPY_U: return dispatch_reduce<FG_MSG_COPY_U>(a, vec4, reduce, stream);
  }
  return fail(FG_EINVAL, "msg = %d is not one of FG_MSG_MUL / ADD / SUB / DIV / COPY_U", msg);
}

// seg: the plan's bounds table, (n_blocks + 1) * n_rows entries in visiting order.  With column blocks the rows
// are folded pass by pass in ascending column order, one launch per pass over all feature tiles, the partial
// results carried in `out` (launches on one stream are ordered, so every element still sees its terms in CSR
// order): the gathers of a pass then come from a band of the feature matrix that fits one L2.
int spmm_general_launch(const int32_t *row_order, const int32_t *seg, int32_t n_blocks, const int32_t *indices,
                        const float *vals, const float *feat, float *out, int32_t n_rows, int32_t F, int msg,
                        int reduce, hipStream_t stream) {
  return spmm_general_mh_launch(row_order, seg, n_blocks, indices, vals, feat, out, n_rows, 1, F, msg, reduce, stream);
}

// H heads of D floats: vals is [nnz, H]; H == 1 is the single-head operator.
int spmm_general_mh_launch(const int32_t *row_order, const int32_t *seg, int32_t n_blocks, const int32_t *indices,
                           const float *vals, const float *feat, float *out, int32_t n_rows, int32_t H, int32_t D,
                           int msg, int reduce, hipStream_t stream) {
  const int32_t F = H * D;
  if (n_rows == 0) return FG_OK;
  GeneralArgs a;
  a.row_order = row_order;
  a.row_lo = seg;
  a.row_hi = seg + static_cast<int64_t>(n_blocks) * n_rows;
  a.indices = indices;
  a.vals = vals;
  a.feat = feat;
  a.out = out;
  a.n_rows = n_rows;
  a.F = F;
  a.H = H;
  a.D = D;
  a.n_tiles = 1;
  // four floats per lane must lie inside one head
  const bool vec4 = D % 4 == 0 && aligned_to(feat, 16) && aligned_to(out, 16);
  const int passes = config().spmm_blocked == 0 ? 1 : std::max(1, n_blocks);
  for (int b = 0; b < passes; ++b) {
    a.seg_lo = passes == 1 ? a.row_lo : seg + static_cast<int64_t>(b) * n_rows;
    a.seg_hi = passes == 1 ? a.row_hi : seg + static_cast<int64_t>(b + 1) * n_rows;
    a.first_pass = b == 0;
    if (int rc = general_pass(a, vec4, msg, reduce, stream)) return rc;
  }
  return FG_OK;
}

namespace {
__global__ __launch_bounds__(kBlockThreads) void mean_finish_kernel(const int32_t *indptr, float *out, int64_t total, int32_t F) {
  const int64_t stride = static_cast<int64_t>(gridDim.x) * blockDim.x;
  for (int64_t t = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x; t < total; t += stride) {
    const int64_t r = t / F;
    const int32_t deg = indptr[r + 1] - indptr[r];
    if (deg > 0) out[t] = out[t] / static_cast<float>(deg);
  }
}
}  // namespace

int spmm_mean_finish_launch(const int32_t *indptr, float *out, int32_t n_rows, int32_t F, hipStream_t stream) {
  const int64_t total = static_cast<int64_t>(n_rows) * F;
  if (total == 0) return FG_OK;
  const unsigned blocks = static_cast<unsigned>(std::min<int64_t>((total + kBlockThreads - 1) / kBlockThreads, 1 << 16));
  mean_finish_kernel<<<dim3(blocks), dim3(kBlockThreads), 0, stream>>>(indptr, out, total, F);
  FG_HIP_TRY(hipGetLastError());
  return FG_OK;
}

int sddmm_elementwise_launch(const int32_t *row, const int32_t *col, const float *src, const float *dst, float *out,
                             int64_t nnz, int32_t F, int op, hipStream_t stream) {
  if (nnz == 0) return FG_OK;
  switch (op) {
    case FG_EDGE_ADD: return launch_elementwise<FG_EDGE_ADD>(row, col, src, dst, out, nnz, F, stream);
    case FG_EDGE_SUB: return launch_elementwise<FG_EDGE_SUB>(row, col, src, dst, out, nnz, F, stream);
    case FG_EDGE_MUL: return launch_elementwise<FG_EDGE_MUL>(row, col, src, dst, out, nnz, F, stream);
    case FG_EDGE_DIV: return launch_elementwise<FG_EDGE_DIV>(row, col, src, dst, out, nnz, F, stream);
  }
  return fail(FG_EINVAL, "edge_op = %d is not one of FG_EDGE_DOT / ADD / SUB / MUL / DIV", op);
}

}  // namespace fg
