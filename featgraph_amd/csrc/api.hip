// C ABI of libfeatgraph_hip.so: argument validation, the SpMM row plan and
// the hand-off to the kernel launchers.  See include/featgraph_hip.h for the
// contract of every entry point.
#include <algorithm>
#include <cstdarg>
#include <cstdio>
#include <cstring>
#include <new>
#include <numeric>
#include <vector>

#include "common.hpp"

namespace fg {

namespace {
thread_local char g_error[512] = "";
Config g_config;
}  // namespace

int fail(int code, const char *fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_error, sizeof(g_error), fmt, ap);
  va_end(ap);
  return code;
}

Config &config() { return g_config; }

}  // namespace fg

struct fg_spmm_plan {
  int64_t n_rows, n_cols, nnz;
  const int32_t *indptr;   // borrowed, device
  const int32_t *indices;  // borrowed, device
  int32_t *row_order;      // owned, device: rows by descending degree
  int32_t max_degree;
  int device;
};

namespace {

__global__ void count_out_of_range_kernel(const int32_t *idx, int64_t n, int64_t bound, unsigned long long *n_bad) {
  const int64_t stride = static_cast<int64_t>(gridDim.x) * blockDim.x;
  unsigned long long bad = 0;
  for (int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x; i < n; i += stride) {
    const int64_t v = idx[i];
    bad += (v < 0 || v >= bound) ? 1u : 0u;
  }
  if (bad) atomicAdd(n_bad, bad);
}

int check_heads(int32_t H, int32_t D) {
  if (H < 1 || D < 1) return fg::fail(FG_EINVAL, "H = %d and D = %d must both be positive", H, D);
  if (static_cast<int64_t>(H) * D > (1 << 20))
    return fg::fail(FG_EUNSUPPORTED, "H*D = %lld exceeds 2^20 floats per vertex", (long long)H * D);
  return FG_OK;
}

int spmm_prepare(const fg_spmm_plan *plan, const float *feat, const float *w, float *out, int32_t H, int32_t D,
                 int32_t feat_tiles, fg::SpmmArgs *a, fg::SpmmShape *s) {
  if (!plan) return fg::fail(FG_EINVAL, "plan is null");
  if (int rc = check_heads(H, D)) return rc;
  if (feat_tiles < 0) return fg::fail(FG_EINVAL, "feat_tiles = %d is negative", feat_tiles);
  if (plan->n_rows > 0 && !out) return fg::fail(FG_EINVAL, "out is null");
  if (plan->nnz > 0 && (!feat || !w)) return fg::fail(FG_EINVAL, "feat or edge values are null");
  a->indptr = plan->indptr;
  a->indices = plan->indices;
  a->w = w;
  a->feat = feat;
  a->out = out;
  a->row_order = (fg::config().spmm_sorted == 0) ? nullptr : plan->row_order;
  a->n_rows = static_cast<int32_t>(plan->n_rows);
  a->F = H * D;
  a->H = H;
  a->D = D;
  *s = fg::spmm_choose_shape(*a, feat_tiles);
  a->n_tiles = (a->F + s->tile_width() - 1) / s->tile_width();
  a->n_slots = static_cast<int64_t>(a->n_tiles) * a->n_rows;
  return FG_OK;
}

int sddmm_prepare(int64_t nnz, const int32_t *row, const int32_t *col, const float *src, const float *dst,
                  float *out, int32_t H, int32_t D, fg::SddmmArgs *a, fg::SddmmShape *s) {
  if (nnz < 0) return fg::fail(FG_EINVAL, "nnz = %lld is negative", (long long)nnz);
  if (int rc = check_heads(H, D)) return rc;
  if (nnz > 0 && (!row || !col || !src || !dst || !out)) return fg::fail(FG_EINVAL, "a data pointer is null");
  a->row = row;
  a->col = col;
  a->src = src;
  a->dst = dst;
  a->out = out;
  a->n_ve = nnz * H;
  a->H = H;
  a->D = D;
  a->stride = H * D;
  *s = fg::sddmm_choose_shape(*a);
  a->batches = s->batches;
  return FG_OK;
}

int *config_slot(const char *key) {
  fg::Config &c = fg::config();
  if (!key) return nullptr;
  if (!strcmp(key, "spmm.vec")) return &c.spmm_vec;
  if (!strcmp(key, "spmm.lpr")) return &c.spmm_lpr;
  if (!strcmp(key, "spmm.unroll")) return &c.spmm_unroll;
  if (!strcmp(key, "spmm.scalar_path")) return &c.spmm_scalar_path;
  if (!strcmp(key, "spmm.sorted")) return &c.spmm_sorted;
  if (!strcmp(key, "sddmm.group")) return &c.sddmm_group;
  if (!strcmp(key, "sddmm.batches")) return &c.sddmm_batches;
  return nullptr;
}

}  // namespace

extern "C" {

int fg_version(void) { return 100; }

const char *fg_last_error(void) { return fg::g_error; }

int fg_spmm_plan_create(int64_t n_rows, int64_t n_cols, int64_t nnz, const int32_t *indptr, const int32_t *indices,
                        fg_spmm_plan **plan) {
  if (!plan) return fg::fail(FG_EINVAL, "plan output pointer is null");
  *plan = nullptr;
  if (n_rows < 0 || n_cols < 0 || nnz < 0)
    return fg::fail(FG_EINVAL, "negative size (n_rows=%lld n_cols=%lld nnz=%lld)", (long long)n_rows,
                    (long long)n_cols, (long long)nnz);
  if (n_rows >= 0x7fffffffLL || n_cols > 0x7fffffffLL || nnz > 0x7fffffffLL)
    return fg::fail(FG_EUNSUPPORTED, "sizes beyond int32 indexing are not supported");
  if (!indptr) return fg::fail(FG_EINVAL, "indptr is null");
  if (nnz > 0 && !indices) return fg::fail(FG_EINVAL, "indices is null");
  if (nnz > 0 && n_cols == 0) return fg::fail(FG_EINVAL, "nnz > 0 with n_cols = 0");

  std::vector<int32_t> host_indptr, order;
  try {
    host_indptr.resize(static_cast<size_t>(n_rows) + 1);
    order.resize(static_cast<size_t>(n_rows));
  } catch (const std::bad_alloc &) {
    return fg::fail(FG_ENOMEM, "host allocation for %lld rows failed", (long long)n_rows);
  }
  FG_HIP_TRY(hipMemcpy(host_indptr.data(), indptr, sizeof(int32_t) * (n_rows + 1), hipMemcpyDeviceToHost));
  if (host_indptr[0] != 0) return fg::fail(FG_EINVAL, "indptr[0] = %d, expected 0", host_indptr[0]);
  int32_t max_degree = 0;
  for (int64_t r = 0; r < n_rows; ++r) {
    const int64_t d = static_cast<int64_t>(host_indptr[r + 1]) - host_indptr[r];
    if (d < 0) return fg::fail(FG_EINVAL, "indptr decreases at row %lld", (long long)r);
    max_degree = std::max<int64_t>(max_degree, d);
  }
  if (host_indptr[n_rows] != nnz)
    return fg::fail(FG_EINVAL, "indptr[n_rows] = %d, expected nnz = %lld", host_indptr[n_rows], (long long)nnz);

  // Rows by descending degree; equal degrees keep ascending row ids, so the
  // list is a pure function of indptr.
  std::iota(order.begin(), order.end(), 0);
  const int32_t *ip = host_indptr.data();
  std::stable_sort(order.begin(), order.end(),
                   [ip](int32_t x, int32_t y) { return ip[x + 1] - ip[x] > ip[y + 1] - ip[y]; });

  fg_spmm_plan *p = new (std::nothrow) fg_spmm_plan();
  if (!p) return fg::fail(FG_ENOMEM, "plan allocation failed");
  p->n_rows = n_rows;
  p->n_cols = n_cols;
  p->nnz = nnz;
  p->indptr = indptr;
  p->indices = indices;
  p->row_order = nullptr;
  p->max_degree = max_degree;
  p->device = 0;
  hipError_t err = hipGetDevice(&p->device);
  if (err == hipSuccess && n_rows > 0) err = hipMalloc(&p->row_order, sizeof(int32_t) * n_rows);
  if (err == hipSuccess && n_rows > 0)
    err = hipMemcpy(p->row_order, order.data(), sizeof(int32_t) * n_rows, hipMemcpyHostToDevice);
  if (err != hipSuccess) {
    if (p->row_order) (void)hipFree(p->row_order);
    delete p;
    return fg::fail(err == hipErrorOutOfMemory ? FG_ENOMEM : FG_EHIP, "plan upload: %s", hipGetErrorString(err));
  }
  *plan = p;
  return FG_OK;
}

void fg_spmm_plan_destroy(fg_spmm_plan *plan) {
  if (!plan) return;
  if (plan->row_order) (void)hipFree(plan->row_order);
  delete plan;
}

int fg_spmm_plan_row_order(const fg_spmm_plan *plan, int32_t *row_order_host, int32_t *max_degree) {
  if (!plan) return fg::fail(FG_EINVAL, "plan is null");
  if (max_degree) *max_degree = plan->max_degree;
  if (row_order_host && plan->n_rows > 0)
    FG_HIP_TRY(hipMemcpy(row_order_host, plan->row_order, sizeof(int32_t) * plan->n_rows, hipMemcpyDeviceToHost));
  return FG_OK;
}

int fg_spmm_csr_f32(const fg_spmm_plan *plan, const float *feat, const float *vals, float *out, int32_t F,
                    int32_t feat_tiles, void *stream) {
  return fg_spmm_csr_mh_f32(plan, feat, vals, out, 1, F, feat_tiles, stream);
}

int fg_spmm_csr_mh_f32(const fg_spmm_plan *plan, const float *feat, const float *w, float *out, int32_t H, int32_t D,
                       int32_t feat_tiles, void *stream) {
  fg::SpmmArgs a;
  fg::SpmmShape s;
  if (int rc = spmm_prepare(plan, feat, w, out, H, D, feat_tiles, &a, &s)) return rc;
  return fg::spmm_launch(a, s, static_cast<hipStream_t>(stream));
}

int fg_sddmm_coo_f32(int64_t nnz, const int32_t *row, const int32_t *col, const float *src, const float *dst,
                     float *out, int32_t F, void *stream) {
  return fg_sddmm_coo_mh_f32(nnz, row, col, src, dst, out, 1, F, stream);
}

int fg_sddmm_coo_mh_f32(int64_t nnz, const int32_t *row, const int32_t *col, const float *src, const float *dst,
                        float *out, int32_t H, int32_t D, void *stream) {
  fg::SddmmArgs a;
  fg::SddmmShape s;
  if (int rc = sddmm_prepare(nnz, row, col, src, dst, out, H, D, &a, &s)) return rc;
  return fg::sddmm_launch(a, s, static_cast<hipStream_t>(stream));
}

int fg_check_indices(int64_t n, const int32_t *idx, int64_t bound, int64_t *n_bad, void *stream) {
  if (n < 0 || !n_bad) return fg::fail(FG_EINVAL, "negative length or null result pointer");
  *n_bad = 0;
  if (n == 0) return FG_OK;
  if (!idx) return fg::fail(FG_EINVAL, "idx is null");
  hipStream_t st = static_cast<hipStream_t>(stream);
  unsigned long long *counter = nullptr;
  FG_HIP_TRY(hipMalloc(&counter, sizeof(*counter)));
  unsigned long long host = 0;
  hipError_t err = hipMemcpyAsync(counter, &host, sizeof(host), hipMemcpyHostToDevice, st);
  if (err == hipSuccess) {
    const int blocks = static_cast<int>(std::min<int64_t>((n + 255) / 256, 4096));
    count_out_of_range_kernel<<<dim3(blocks), dim3(256), 0, st>>>(idx, n, bound, counter);
    err = hipGetLastError();
  }
  if (err == hipSuccess) err = hipMemcpyAsync(&host, counter, sizeof(host), hipMemcpyDeviceToHost, st);
  if (err == hipSuccess) err = hipStreamSynchronize(st);
  (void)hipFree(counter);
  if (err != hipSuccess) return fg::fail(FG_EHIP, "index check: %s", hipGetErrorString(err));
  *n_bad = static_cast<int64_t>(host);
  return FG_OK;
}

int fg_config_set(const char *key, int32_t value) {
  int *slot = config_slot(key);
  if (!slot) return fg::fail(FG_EINVAL, "unknown configuration key '%s'", key ? key : "(null)");
  const bool flag = slot == &fg::config().spmm_scalar_path || slot == &fg::config().spmm_sorted;
  // flags: 0 / 1 are explicit, anything negative restores the default;
  // sizes: 0 restores the default
  *slot = flag ? (value < 0 ? -1 : (value != 0)) : std::max(value, 0);
  return FG_OK;
}

int fg_config_get(const char *key, int32_t *value) {
  int *slot = config_slot(key);
  if (!slot || !value) return fg::fail(FG_EINVAL, "unknown configuration key or null result pointer");
  *value = *slot;
  return FG_OK;
}

int fg_spmm_describe(const fg_spmm_plan *plan, int32_t H, int32_t D, int32_t feat_tiles, char *buf, int64_t cap) {
  if (!buf || cap <= 0) return fg::fail(FG_EINVAL, "no room for the description");
  fg::SpmmArgs a;
  fg::SpmmShape s;
  // shape selection looks at pointer alignment only; describe the aligned case
  alignas(16) static float dummy[4];
  if (int rc = spmm_prepare(plan, dummy, dummy, dummy, H, D, feat_tiles, &a, &s)) return rc;
  const int rows_per_wave = fg::kWaveSize / s.lpr;
  const int64_t waves = (a.n_slots + rows_per_wave - 1) / rows_per_wave;
  snprintf(buf, static_cast<size_t>(cap),
           "spmm_csr rows=%lld cols=%lld nnz=%lld max_degree=%d H=%d D=%d | kernel=%s floats/lane=%d "
           "lanes/row-slot=%d tile=%d floats x %d tiles gathers-in-flight=%d rows=%s | grid=%lld blocks x %d threads",
           (long long)plan->n_rows, (long long)plan->n_cols, (long long)plan->nnz, plan->max_degree, H, D,
           s.scalar_path ? "wave-per-row(scalar ids)" : "row-slot", s.vec, s.lpr, s.tile_width(), a.n_tiles,
           s.unroll, a.row_order ? "by-descending-degree" : "natural",
           (long long)((waves + fg::kWavesPerBlock - 1) / fg::kWavesPerBlock), fg::kBlockThreads);
  return FG_OK;
}

int fg_sddmm_describe(int64_t nnz, int32_t H, int32_t D, char *buf, int64_t cap) {
  if (!buf || cap <= 0) return fg::fail(FG_EINVAL, "no room for the description");
  fg::SddmmArgs a;
  fg::SddmmShape s;
  alignas(16) static float dummy[4];
  alignas(16) static int32_t idummy[4];
  if (int rc = sddmm_prepare(nnz, idummy, idummy, dummy, dummy, dummy, H, D, &a, &s)) return rc;
  const int64_t per_wave = static_cast<int64_t>(s.batches) * fg::kWaveSize;
  const int64_t waves = (a.n_ve + per_wave - 1) / per_wave;
  snprintf(buf, static_cast<size_t>(cap),
           "sddmm_coo nnz=%lld H=%d D=%d | floats/lane=%d lanes/dot=%d dots/wave-round=%d batches/wave=%d | "
           "grid=%lld blocks x %d threads",
           (long long)nnz, H, D, s.vec, s.group, fg::kWaveSize / s.group, s.batches,
           (long long)((waves + fg::kWavesPerBlock - 1) / fg::kWavesPerBlock), fg::kBlockThreads);
  return FG_OK;
}

}  // extern "C"
