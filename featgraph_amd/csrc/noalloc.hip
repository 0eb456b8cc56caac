// fg_spmm_csr_noalloc_f32: CSR SpMM for callers that must not allocate.
//
// fg_spmm_csr_f32 runs over a plan whose row schedule (rows by descending
// degree and their bounds in that order) lives in device memory that
// fg_spmm_plan_create allocates.  This entry point builds the same kind of
// schedule on the device, per call, inside a fixed array that is part of the
// library image, and then launches the same wave-per-row kernels over it: no
// hipMalloc, no hipFree, no host copy, no synchronisation.
//
// The schedule is a counting sort of the rows by degree class
// (class = bit length of the degree, longest class first), so the waves that
// start first take the hub rows, as with a plan.  Positions inside a class come
// from atomic counters and may differ from call to call; results do not depend
// on the visiting order (each output element is one lane's sequential sum).
//
// The array is shared by every call on a GPU (each GPU has its own copy): two
// calls that overlap in time on one GPU race on it.
#include <mutex>

#include "common.hpp"

namespace {

constexpr int64_t kMaxRows = int64_t{1} << 20;  // rows the schedule array has room for
constexpr int kClasses = 33;                    // degree classes: bit lengths 0 .. 32
constexpr int kCounterInts = 128;               // [0, 33): class counts, [64, 97): class cursors

struct NoallocScratch {
  int32_t counters[kCounterInts];
  int32_t row_order[kMaxRows];
  int32_t seg_lo[kMaxRows];
  int32_t seg_hi[kMaxRows];
};

// Device memory beyond the caller's inputs and outputs: 12 MiB + 512 bytes per GPU, held until the process ends.
static __device__ __align__(256) unsigned char scratch[sizeof(NoallocScratch)];

constexpr int kMaxDevices = 64;
std::mutex g_mutex;
NoallocScratch *g_scratch[kMaxDevices] = {};  // device address of `scratch` on each GPU, looked up once per GPU

// The array's name is only a handle on the host; kernels and fills need its device address, which differs
// from GPU to GPU.  Called with the target device current.
int scratch_address(NoallocScratch **out, hipStream_t stream) {
  int device = -1;
  FG_HIP_TRY(hipGetDevice(&device));
  if (device < 0 || device >= kMaxDevices)
    return fg::fail(FG_EUNSUPPORTED, "device ordinal %d is outside the %d devices this entry point tracks", device,
                    kMaxDevices);
  std::lock_guard<std::mutex> lock(g_mutex);
  if (!g_scratch[device]) {
    // the lookup may load the library's code object on this GPU: not something to do while `stream` records a graph
    hipStreamCaptureStatus capturing = hipStreamCaptureStatusNone;
    if (hipStreamIsCapturing(stream, &capturing) != hipSuccess) (void)hipGetLastError();
    if (capturing != hipStreamCaptureStatusNone)
      return fg::fail(FG_EUNSUPPORTED,
                      "the first fg_spmm_csr_noalloc_f32 call on a GPU must not be under stream capture: call it "
                      "once eagerly on device %d before recording it", device);
    void *ptr = nullptr;
    FG_HIP_TRY(hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch)));
    if (!ptr) return fg::fail(FG_EHIP, "hipGetSymbolAddress returned a null address for the schedule array");
    g_scratch[device] = static_cast<NoallocScratch *>(ptr);
  }
  *out = g_scratch[device];
  return FG_OK;
}

__device__ __forceinline__ int degree_class(int32_t degree) { return 32 - __clz(max(degree, 0)); }

// The previous call's counts must not survive: a fill kernel rather than a memset, so that a caller may record
// the call into a HIP graph.
__global__ void clear_counters_kernel(int32_t *counters) {
  if (threadIdx.x < kCounterInts) counters[threadIdx.x] = 0;
}

// Rows per degree class, summed per workgroup in LDS first.
__global__ void count_classes_kernel(const int32_t *indptr, int32_t n_rows, int32_t *counters) {
  __shared__ int32_t local[kClasses];
  if (threadIdx.x < kClasses) local[threadIdx.x] = 0;
  __syncthreads();
  const int stride = gridDim.x * blockDim.x;
  for (int r = blockIdx.x * blockDim.x + threadIdx.x; r < n_rows; r += stride)
    atomicAdd(&local[degree_class(indptr[r + 1] - indptr[r])], 1);
  __syncthreads();
  if (threadIdx.x < kClasses && local[threadIdx.x]) atomicAdd(&counters[threadIdx.x], local[threadIdx.x]);
}

// cursors[c] = number of rows in the classes above c: the classes are laid out longest first.
__global__ void class_offsets_kernel(int32_t *counters) {
  if (threadIdx.x == 0 && blockIdx.x == 0) {
    int32_t at = 0;
    for (int c = kClasses - 1; c >= 0; --c) {
      counters[64 + c] = at;
      at += counters[c];
    }
  }
}

__global__ void place_rows_kernel(const int32_t *indptr, int32_t n_rows, int32_t nnz, NoallocScratch *s) {
  const int stride = gridDim.x * blockDim.x;
  for (int r = blockIdx.x * blockDim.x + threadIdx.x; r < n_rows; r += stride) {
    int32_t lo = indptr[r], hi = indptr[r + 1];
    const int c = degree_class(hi - lo);
    if (lo < 0 || hi > nnz || hi < lo) hi = lo = 0;  // a broken row pointer must not send a gather out of bounds
    const int pos = atomicAdd(&s->counters[64 + c], 1);
    s->row_order[pos] = r;
    s->seg_lo[pos] = lo;
    s->seg_hi[pos] = hi;
  }
}

}  // namespace

extern "C" int fg_spmm_csr_noalloc_f32(int64_t n_rows, int64_t n_cols, int64_t nnz, const int32_t *indptr,
                                       const int32_t *indices, const float *vals, const float *feat, float *out,
                                       int32_t F, void *stream) {
  if (n_rows < 0 || n_cols < 0 || nnz < 0)
    return fg::fail(FG_EINVAL, "negative size (n_rows=%lld n_cols=%lld nnz=%lld)", (long long)n_rows,
                    (long long)n_cols, (long long)nnz);
  if (n_rows > kMaxRows)
    return fg::fail(FG_EUNSUPPORTED,
                    "n_rows = %lld exceeds the %lld rows that the built-in schedule array holds; use a plan "
                    "(fg_spmm_plan_create + fg_spmm_csr_f32) for larger matrices",
                    (long long)n_rows, (long long)kMaxRows);
  if (n_cols > 0x7fffffffLL || nnz > 0x7fffffffLL)
    return fg::fail(FG_EUNSUPPORTED, "sizes beyond int32 indexing are not supported");
  if (F < 1) return fg::fail(FG_EINVAL, "F = %d must be positive", F);
  if (static_cast<int64_t>(F) > (1 << 20)) return fg::fail(FG_EUNSUPPORTED, "F = %d exceeds 2^20 floats per row", F);
  if (!indptr) return fg::fail(FG_EINVAL, "indptr is null");
  if (n_rows > 0 && !out) return fg::fail(FG_EINVAL, "out is null");
  if (nnz > 0 && (!indices || !vals || !feat)) return fg::fail(FG_EINVAL, "indices, vals or feat is null");
  if (nnz > 0 && n_cols == 0) return fg::fail(FG_EINVAL, "nnz > 0 with n_cols = 0");
  if (n_rows == 0) return FG_OK;

  NoallocScratch *s = nullptr;
  hipStream_t st = static_cast<hipStream_t>(stream);
  if (int rc = scratch_address(&s, st)) return rc;
  const int32_t n = static_cast<int32_t>(n_rows);
  const unsigned grid = static_cast<unsigned>(std::min<int64_t>((n_rows + 255) / 256, 2048));
  clear_counters_kernel<<<dim3(1), dim3(kCounterInts), 0, st>>>(s->counters);
  count_classes_kernel<<<dim3(grid), dim3(256), 0, st>>>(indptr, n, s->counters);
  class_offsets_kernel<<<dim3(1), dim3(64), 0, st>>>(s->counters);
  place_rows_kernel<<<dim3(grid), dim3(256), 0, st>>>(indptr, n, static_cast<int32_t>(nnz), s);
  FG_HIP_TRY(hipGetLastError());

  fg::SpmmArgs a;
  a.indptr = indptr;
  a.indices = indices;
  a.w = vals;
  a.feat = feat;
  a.out = out;
  a.row_order = s->row_order;
  a.seg_lo = s->seg_lo;
  a.seg_hi = s->seg_hi;
  a.n_rows = n;
  a.n_cols = static_cast<int32_t>(n_cols);
  a.F = F;
  a.H = 1;
  a.D = F;
  const fg::SpmmShape shape = fg::spmm_choose_shape(a, 0);
  a.n_tiles = (a.F + shape.tile_width() - 1) / shape.tile_width();
  a.n_slots = static_cast<int64_t>(a.n_tiles) * a.n_rows;
  return fg::spmm_launch(a, shape, st);
}
