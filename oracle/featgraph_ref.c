/*
 * TEST INFRASTRUCTURE, NOT PRODUCT CODE.
 *
 * CPU restatement of the FeatGraph reference's loop nests for vanilla CSR SpMM,
 * DDS SpMM and COO SDDMM, plus closed forms for the multi-head variants.  It is
 * the checker the HIP kernels are compared with, and the CPU baseline that the
 * benchmark times beside them.  Only the test-suite, the smoke check and the
 * benchmark's cpu_baseline leg may load it; the shipped package never does.
 *
 * Each function cites the reference lines it follows (paths relative to the
 * reference repository root).  The reference generates its native code through
 * TVM v0.7, which is not available to this build, so what is restated is the
 * loop nest that the tensor expressions and schedules define:
 *   - arithmetic is IEEE binary32, one multiply and one add per term, never
 *     fused (TVM's 'llvm' target without -mcpu has no FMA); build with
 *     -ffp-contract=off and without -ffast-math,
 *   - SpMM accumulates each output element sequentially in CSR order starting
 *     from +0 (te.sum over elem_idx); vectorisation is across the feature
 *     index only, which does not change any element's order,
 *   - SDDMM accumulates sequentially over k.  The order TVM's LLVM back end
 *     really uses for that reduction is not pinned by anything the reference
 *     holds (bit-level parity with TVM: parity unpinned); its own tests pin the
 *     result to the closed form within rtol=atol=1e-4.
 *
 * Pinned by tests/test_oracle.py: scipy's csr.dot and numpy gather-sum closed
 * forms (the reference's own checks, tests/test_module_spmm.py:29-30,
 * tests/test_module_sddmm.py:34-37), exact small-integer cases, fp64 brute
 * force, and the structural invariants listed there.
 */
#include <stdint.h>
#include <stdlib.h>
#include <string.h>
#ifdef _OPENMP
#include <omp.h>
#endif

#define FGREF_OK 0
#define FGREF_EINVAL -1
#define FGREF_ENOMEM -2

int fgref_version(void) { return 1; }

int fgref_num_threads(void) {
#ifdef _OPENMP
  return omp_get_max_threads();
#else
  return 1;
#endif
}

/* Stage A of both x86 SpMM variants and of the tiled SDDMM:
 * Reshaped[fo, nn, fi] = Feat[nn, fo*Fp + fi], rows in parallel.
 * op/vanilla_spmm.py:43-44 + :76, op/vanilla_sddmm.py:52-57. */
static void relayout_forward(const float *feat, float *resh, int64_t n, int64_t F, int64_t P, int par) {
  const int64_t Fp = F / P;
  for (int64_t fo = 0; fo < P; ++fo) {
#pragma omp parallel for schedule(static) if (par)
    for (int64_t nn = 0; nn < n; ++nn) {
      const float *s = feat + nn * F + fo * Fp;
      float *d = resh + (fo * n + nn) * Fp;
      for (int64_t fi = 0; fi < Fp; ++fi) d[fi] = s[fi];
    }
  }
}

/* Stage C: Out[nn, ff] = ReshapedOut[ff / Fp, nn, ff % Fp], rows in parallel.
 * op/vanilla_spmm.py:58-60 + :78. */
static void relayout_backward(const float *resh, float *out, int64_t n, int64_t F, int64_t P) {
  const int64_t Fp = F / P;
#pragma omp parallel for schedule(static)
  for (int64_t nn = 0; nn < n; ++nn)
    for (int64_t ff = 0; ff < F; ++ff) out[nn * F + ff] = resh[((ff / Fp) * n + nn) * Fp + (ff % Fp)];
}

/* vanilla_spmm_csr_x86 + schedule_vanilla_spmm_csr_x86
 * (op/vanilla_spmm.py:36-62 compute, :65-80 schedule).
 * Loop order after the reorder at :73: fo, row (parallel, :77), elem, fi.
 * `work` holds (n_src + n_dst) * F floats, or is NULL to allocate here. */
int fgref_spmm_csr_x86(int64_t n_dst, int64_t n_src, int64_t F, int64_t P, const int32_t *indptr,
                       const int32_t *indices, const float *vals, const float *src, float *out, float *work) {
  if (n_dst < 0 || n_src < 0 || F <= 0 || P <= 0 || F % P) return FGREF_EINVAL;
  float *own = NULL;
  if (!work) {
    own = (float *)malloc(sizeof(float) * (size_t)((n_src + n_dst) * F + 1));
    if (!own) return FGREF_ENOMEM;
    work = own;
  }
  float *rsf = work, *ro = work + n_src * F;
  const int64_t Fp = F / P;
  relayout_forward(src, rsf, n_src, F, P, 1);
  for (int64_t fo = 0; fo < P; ++fo) {
#pragma omp parallel for schedule(static)
    for (int64_t row = 0; row < n_dst; ++row) {
      float *acc = ro + (fo * n_dst + row) * Fp;
      for (int64_t fi = 0; fi < Fp; ++fi) acc[fi] = 0.0f;
      for (int64_t e = indptr[row]; e < indptr[row + 1]; ++e) {
        const float v = vals[e];
        const float *x = rsf + (fo * n_src + (int64_t)indices[e]) * Fp;
        for (int64_t fi = 0; fi < Fp; ++fi) acc[fi] = acc[fi] + v * x[fi];
      }
    }
  }
  relayout_backward(ro, out, n_dst, F, P);
  free(own);
  return FGREF_OK;
}

/* vanilla_spmm_dds_x86 + schedule_vanilla_spmm_dds_x86
 * (op/vanilla_spmm.py:188-224 compute, :227-246 schedule).
 * s1_pos has d1*(n_dst+1) entries; column ids in s1_idx are block-local and
 * are re-globalised with + p*ceil(n_src/d1) (:196, :208).  Per fo and per
 * source block p the partial sums Intermediate[p,row,:] are formed from +0
 * (:201-213) and then added into ReshapedOut in block order (:215-218, with
 * Intermediate computed at the reduce axis, :239). */
int fgref_spmm_dds_x86(int64_t n_dst, int64_t n_src, int64_t F, int64_t P, int64_t d1, const int32_t *s1_pos,
                       const int32_t *s1_idx, const float *vals, const float *src, float *out) {
  if (n_dst < 0 || n_src < 0 || F <= 0 || P <= 0 || F % P || d1 <= 0) return FGREF_EINVAL;
  const int64_t Fp = F / P, d2 = n_dst + 1, per = (n_src + d1 - 1) / d1;
  float *work = (float *)malloc(sizeof(float) * (size_t)((n_src + 2 * n_dst) * F + 1));
  if (!work) return FGREF_ENOMEM;
  float *rsf = work, *ro = work + n_src * F, *inter = ro + n_dst * F;
  relayout_forward(src, rsf, n_src, F, P, 1);
  for (int64_t fo = 0; fo < P; ++fo) {
    float *rof = ro + fo * n_dst * Fp;
    for (int64_t i = 0; i < n_dst * Fp; ++i) rof[i] = 0.0f;
    for (int64_t p = 0; p < d1; ++p) {
#pragma omp parallel for schedule(static)
      for (int64_t row = 0; row < n_dst; ++row) {
        float *acc = inter + row * Fp;
        for (int64_t fi = 0; fi < Fp; ++fi) acc[fi] = 0.0f;
        for (int64_t e = s1_pos[p * d2 + row]; e < s1_pos[p * d2 + row + 1]; ++e) {
          const float v = vals[e];
          const float *x = rsf + (fo * n_src + (int64_t)s1_idx[e] + p * per) * Fp;
          for (int64_t fi = 0; fi < Fp; ++fi) acc[fi] = acc[fi] + v * x[fi];
        }
      }
#pragma omp parallel for schedule(static)
      for (int64_t row = 0; row < n_dst; ++row)
        for (int64_t fi = 0; fi < Fp; ++fi) rof[row * Fp + fi] = rof[row * Fp + fi] + inter[row * Fp + fi];
    }
  }
  relayout_backward(ro, out, n_dst, F, P);
  free(work);
  return FGREF_OK;
}

/* vanilla_sddmm + schedule_vanilla_sddmm_x86 (op/vanilla_sddmm.py:37-63, :66-74).
 * Out[e] = sum_k Src[col[e],k] * Dst[row[e],k]; Src is indexed by COLUMN ids
 * and Dst by ROW ids (:47).  Serial: the schedule applies no parallel axis
 * (:66-74, TODO at :11).  With P > 1 both operands are first re-laid out
 * (:52-57) and the reduce axis is split with fo outermost (:71-72), so Out is
 * zeroed and then grows tile by tile; every element still adds its terms in
 * k order. */
int fgref_sddmm_x86(int64_t nnz, int64_t n_rows, int64_t n_cols, int64_t F, int64_t P, const int32_t *row,
                    const int32_t *col, const float *src, const float *dst, float *out) {
  if (nnz < 0 || F <= 0 || P <= 0 || F % P) return FGREF_EINVAL;
  if (P == 1) {
    for (int64_t e = 0; e < nnz; ++e) {
      const float *a = src + (int64_t)col[e] * F, *b = dst + (int64_t)row[e] * F;
      float acc = 0.0f;
      for (int64_t k = 0; k < F; ++k) acc = acc + a[k] * b[k];
      out[e] = acc;
    }
    return FGREF_OK;
  }
  const int64_t Fp = F / P;
  float *work = (float *)malloc(sizeof(float) * (size_t)((n_rows + n_cols) * F + 1));
  if (!work) return FGREF_ENOMEM;
  float *rs = work, *rd = work + n_cols * F;
  relayout_forward(src, rs, n_cols, F, P, 0);
  relayout_forward(dst, rd, n_rows, F, P, 0);
  for (int64_t e = 0; e < nnz; ++e) out[e] = 0.0f;
  for (int64_t fo = 0; fo < P; ++fo)
    for (int64_t e = 0; e < nnz; ++e) {
      const float *a = rs + (fo * n_cols + (int64_t)col[e]) * Fp, *b = rd + (fo * n_rows + (int64_t)row[e]) * Fp;
      float acc = out[e];
      for (int64_t fi = 0; fi < Fp; ++fi) acc = acc + a[fi] * b[fi];
      out[e] = acc;
    }
  free(work);
  return FGREF_OK;
}

/* Timing-only variant of the P == 1 SDDMM nest: the k reduction may be
 * re-associated into SIMD partial sums (what LLVM does to such a loop when
 * TVM enables fast-math), and `par` != 0 additionally spreads edges over all
 * cores, which the reference schedule does not do.  Not used as a checker. */
int fgref_sddmm_x86_fast(int64_t nnz, int64_t F, const int32_t *row, const int32_t *col, const float *src,
                         const float *dst, float *out, int par) {
  if (nnz < 0 || F <= 0) return FGREF_EINVAL;
#pragma omp parallel for schedule(static) if (par)
  for (int64_t e = 0; e < nnz; ++e) {
    const float *a = src + (int64_t)col[e] * F, *b = dst + (int64_t)row[e] * F;
    float acc = 0.0f;
#pragma omp simd reduction(+ : acc)
    for (int64_t k = 0; k < F; ++k) acc += a[k] * b[k];
    out[e] = acc;
  }
  return FGREF_OK;
}

/* The same two formulas with binary64 products and accumulation, for error
 * budgets: they tell reference rounding from kernel error. */
int fgref_spmm_csr_f64(int64_t n_dst, int64_t F, const int32_t *indptr, const int32_t *indices, const float *vals,
                       const float *src, double *out) {
  if (n_dst < 0 || F <= 0) return FGREF_EINVAL;
#pragma omp parallel for schedule(dynamic, 64)
  for (int64_t r = 0; r < n_dst; ++r) {
    double *acc = out + r * F;
    for (int64_t f = 0; f < F; ++f) acc[f] = 0.0;
    for (int64_t e = indptr[r]; e < indptr[r + 1]; ++e) {
      const double v = vals[e];
      const float *x = src + (int64_t)indices[e] * F;
      for (int64_t f = 0; f < F; ++f) acc[f] += v * (double)x[f];
    }
  }
  return FGREF_OK;
}

int fgref_sddmm_f64(int64_t nnz, int64_t F, const int32_t *row, const int32_t *col, const float *src,
                    const float *dst, double *out) {
  if (nnz < 0 || F <= 0) return FGREF_EINVAL;
#pragma omp parallel for schedule(static)
  for (int64_t e = 0; e < nnz; ++e) {
    const float *a = src + (int64_t)col[e] * F, *b = dst + (int64_t)row[e] * F;
    double acc = 0.0;
    for (int64_t k = 0; k < F; ++k) acc += (double)a[k] * (double)b[k];
    out[e] = acc;
  }
  return FGREF_OK;
}

/* Multi-head SDDMM.  The reference has no such operator (op/__init__.py:1-5
 * exports only vanilla_*); the definition is the vanilla edge function of
 * op/vanilla_sddmm.py:47 applied per head on [N,H,D] operands:
 * Out[e,h] = sum_d Src[col[e],h,d] * Dst[row[e],h,d], sequential in d. */
int fgref_sddmm_mh(int64_t nnz, int64_t H, int64_t D, const int32_t *row, const int32_t *col, const float *src,
                   const float *dst, float *out) {
  if (nnz < 0 || H <= 0 || D <= 0) return FGREF_EINVAL;
#pragma omp parallel for schedule(static)
  for (int64_t e = 0; e < nnz; ++e)
    for (int64_t h = 0; h < H; ++h) {
      const float *a = src + ((int64_t)col[e] * H + h) * D, *b = dst + ((int64_t)row[e] * H + h) * D;
      float acc = 0.0f;
      for (int64_t d = 0; d < D; ++d) acc = acc + a[d] * b[d];
      out[e * H + h] = acc;
    }
  return FGREF_OK;
}

/* Multi-head generalised SpMM (not in the reference either): the message
 * function of op/vanilla_spmm.py:46-53 with a per-edge per-head weight,
 * Out[r,h,d] = sum_{e in row r} W[e,h] * Src[indices[e],h,d], sequential in e. */
int fgref_spmm_mh(int64_t n_dst, int64_t H, int64_t D, const int32_t *indptr, const int32_t *indices,
                  const float *w, const float *src, float *out) {
  if (n_dst < 0 || H <= 0 || D <= 0) return FGREF_EINVAL;
  const int64_t F = H * D;
#pragma omp parallel for schedule(dynamic, 64)
  for (int64_t r = 0; r < n_dst; ++r) {
    float *acc = out + r * F;
    for (int64_t f = 0; f < F; ++f) acc[f] = 0.0f;
    for (int64_t e = indptr[r]; e < indptr[r + 1]; ++e) {
      const float *x = src + (int64_t)indices[e] * F;
      for (int64_t h = 0; h < H; ++h) {
        const float v = w[e * H + h];
        for (int64_t d = 0; d < D; ++d) acc[h * D + d] = acc[h * D + d] + v * x[h * D + d];
      }
    }
  }
  return FGREF_OK;
}

/* Generalised SpMM: the message and reduce slots of the reference's SpMM template
 * (op/vanilla_spmm.py:46-53: msgfunc builds adj_val * feat_val and folds it with
 * te.sum) opened to the operators that README.md:6 calls "generalized SpMM".
 * The reference ships only the (mul, sum) instance; the others are defined here:
 *   term(e, f) = msg(Src[indices[e], f], vals[e])   msg: 0 u*e, 1 u+e, 2 u-e, 3 u/e, 4 u
 *   Out[r, f]  = fold over e in CSR order           reduce: 0 sum (from +0), 1 max, 2 min,
 *                                                   3 mean = sum / degree (one rounded division)
 * max / min fold as acc = (t > acc) ? t : acc from the row's first term, so the
 * result (including the sign of a zero) is fixed by the order.  Rows without
 * nonzeros give 0 under every reducer.  (mul, sum) is fgref_spmm_csr_x86 bit for bit. */
static inline float fgref_msg(int msg, float u, float e) {
  switch (msg) {
    case 0: return u * e;
    case 1: return u + e;
    case 2: return u - e;
    case 3: return u / e;
    default: return u;
  }
}

int fgref_spmm_general(int64_t n_dst, int64_t F, const int32_t *indptr, const int32_t *indices, const float *vals,
                       const float *src, float *out, int msg, int reduce) {
  if (n_dst < 0 || F <= 0 || msg < 0 || msg > 4 || reduce < 0 || reduce > 3) return FGREF_EINVAL;
#pragma omp parallel for schedule(dynamic, 64)
  for (int64_t r = 0; r < n_dst; ++r) {
    float *acc = out + r * F;
    const int64_t lo = indptr[r], hi = indptr[r + 1];
    for (int64_t f = 0; f < F; ++f) acc[f] = 0.0f;
    for (int64_t e = lo; e < hi; ++e) {
      const float *x = src + (int64_t)indices[e] * F;
      const float v = msg == 4 ? 0.0f : vals[e];
      for (int64_t f = 0; f < F; ++f) {
        const float t = fgref_msg(msg, x[f], v);
        if (reduce == 0 || reduce == 3)
          acc[f] = acc[f] + t;
        else if (e == lo)
          acc[f] = t;
        else if (reduce == 1)
          acc[f] = (t > acc[f]) ? t : acc[f];
        else
          acc[f] = (t < acc[f]) ? t : acc[f];
      }
    }
    if (reduce == 3 && hi > lo) {
      const float n = (float)(hi - lo);
      for (int64_t f = 0; f < F; ++f) acc[f] = acc[f] / n;
    }
  }
  return FGREF_OK;
}

/* Generalised SDDMM with an elementwise edge function (the edgefunc slot of
 * op/vanilla_sddmm.py:43-47 without its reduction over k):
 * Out[e, f] = Src[col[e], f] op Dst[row[e], f], op: 1 add, 2 sub, 3 mul, 4 div.
 * (op 0, the dot product, is fgref_sddmm_x86.) */
int fgref_sddmm_general(int64_t nnz, int64_t F, const int32_t *row, const int32_t *col, const float *src,
                        const float *dst, float *out, int op) {
  if (nnz < 0 || F <= 0 || op < 1 || op > 4) return FGREF_EINVAL;
#pragma omp parallel for schedule(static)
  for (int64_t e = 0; e < nnz; ++e) {
    const float *a = src + (int64_t)col[e] * F, *b = dst + (int64_t)row[e] * F;
    float *o = out + e * F;
    for (int64_t f = 0; f < F; ++f)
      o[f] = op == 1 ? a[f] + b[f] : op == 2 ? a[f] - b[f] : op == 3 ? a[f] * b[f] : a[f] / b[f];
  }
  return FGREF_OK;
}

/* Edge softmax (not in the reference; it is the step between the attention
 * scores of multi-head SDDMM and the weights of multi-head SpMM in a GAT layer):
 * for every destination row r and head h, over the row's edges in CSR order,
 * Out[e, h] = exp(S[e, h] - max_r,h) / sum_e' exp(S[e', h] - max_r,h).
 * Computed in binary64 and rounded once, so it serves as the exact value that a
 * float32 kernel is held to within tolerance. */
#include <math.h>
int fgref_edge_softmax(int64_t n_dst, int64_t H, const int32_t *indptr, const float *scores, float *out) {
  if (n_dst < 0 || H <= 0) return FGREF_EINVAL;
#pragma omp parallel for schedule(dynamic, 64)
  for (int64_t r = 0; r < n_dst; ++r) {
    const int64_t lo = indptr[r], hi = indptr[r + 1];
    for (int64_t h = 0; h < H; ++h) {
      double m = -INFINITY, sum = 0.0;
      for (int64_t e = lo; e < hi; ++e) m = scores[e * H + h] > m ? scores[e * H + h] : m;
      for (int64_t e = lo; e < hi; ++e) sum += exp((double)scores[e * H + h] - m);
      for (int64_t e = lo; e < hi; ++e) out[e * H + h] = (float)(exp((double)scores[e * H + h] - m) / sum);
    }
  }
  return FGREF_OK;
}

/* Multi-head generalised SpMM (not in the reference): fgref_spmm_general with a
 * per-edge per-head weight, the message slot of op/vanilla_spmm.py:46-53 applied
 * head by head on [N,H,D] features:
 *   term(e, h, d) = msg(Src[indices[e], h, d], W[e, h]),  Out[r, h, d] = fold over e in CSR order.
 * Same folds as fgref_spmm_general (first term assigned for max / min, mean = sum / degree,
 * rows without nonzeros 0).  (mul, sum) is fgref_spmm_mh bit for bit; H = 1 is fgref_spmm_general. */
int fgref_spmm_mh_general(int64_t n_dst, int64_t H, int64_t D, const int32_t *indptr, const int32_t *indices,
                          const float *w, const float *src, float *out, int msg, int reduce) {
  if (n_dst < 0 || H <= 0 || D <= 0 || msg < 0 || msg > 4 || reduce < 0 || reduce > 3) return FGREF_EINVAL;
  const int64_t F = H * D;
#pragma omp parallel for schedule(dynamic, 64)
  for (int64_t r = 0; r < n_dst; ++r) {
    float *acc = out + r * F;
    const int64_t lo = indptr[r], hi = indptr[r + 1];
    for (int64_t f = 0; f < F; ++f) acc[f] = 0.0f;
    for (int64_t e = lo; e < hi; ++e) {
      const float *x = src + (int64_t)indices[e] * F;
      for (int64_t h = 0; h < H; ++h) {
        const float v = msg == 4 ? 0.0f : w[e * H + h];
        for (int64_t d = 0; d < D; ++d) {
          const int64_t f = h * D + d;
          const float t = fgref_msg(msg, x[f], v);
          if (reduce == 0 || reduce == 3)
            acc[f] = acc[f] + t;
          else if (e == lo)
            acc[f] = t;
          else if (reduce == 1)
            acc[f] = (t > acc[f]) ? t : acc[f];
          else
            acc[f] = (t < acc[f]) ? t : acc[f];
        }
      }
    }
    if (reduce == 3 && hi > lo) {
      const float n = (float)(hi - lo);
      for (int64_t f = 0; f < F; ++f) acc[f] = acc[f] / n;
    }
  }
  return FGREF_OK;
}

/* Backward of the edge softmax (not in the reference; the step between the
 * gradients of multi-head SpMM and multi-head SDDMM in a GAT layer).  With
 * A = softmax of the scores over a destination row's edges (per head) and G the
 * gradient that arrives for A, the gradient for the scores is
 *   dS[e, h] = A[e, h] * (G[e, h] - sum_{e' in the row} A[e', h] * G[e', h]).
 * Computed in binary64 from the float32 inputs and rounded once. */
int fgref_edge_softmax_backward(int64_t n_dst, int64_t H, const int32_t *indptr, const float *weights,
                                const float *grad, float *out) {
  if (n_dst < 0 || H <= 0) return FGREF_EINVAL;
#pragma omp parallel for schedule(dynamic, 64)
  for (int64_t r = 0; r < n_dst; ++r) {
    const int64_t lo = indptr[r], hi = indptr[r + 1];
    for (int64_t h = 0; h < H; ++h) {
      double dot = 0.0;
      for (int64_t e = lo; e < hi; ++e) dot += (double)weights[e * H + h] * (double)grad[e * H + h];
      for (int64_t e = lo; e < hi; ++e)
        out[e * H + h] = (float)((double)weights[e * H + h] * ((double)grad[e * H + h] - dot));
    }
  }
  return FGREF_OK;
}
