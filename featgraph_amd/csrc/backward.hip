// Pieces that the backward of the multi-head operators needs beside the forward kernels themselves (the
// gradients of multi-head SpMM and SDDMM are again multi-head SpMM / SDDMM calls, over the matrix or its
// transpose):
//
//   edge softmax backward   dS[e, h] = A[e, h] * (G[e, h] - sum over the row's edges e' of A[e', h] * G[e', h])
//                           for the weights A of a row softmax and the gradient G that arrives for them.  One wave
//                           per destination row, as in the forward kernel (softmax.hip): a first sweep sums
//                           A * G per head (lanes of equal head merged by a butterfly), a second one writes dS.
//   row permutation         out[i, :] = in[perm[i], :] for rows of `width` floats: carries per-edge weights from
//                           the order of a matrix's CSR arrays to the order of its transpose's.
//   elementwise sum         out = a + b: joins the two contributions to the gradient of a vertex matrix that
//                           serves as key and as value.
#include <algorithm>

#include "common.hpp"

namespace fg {
namespace {

// Sum of x over all lanes whose index agrees modulo `stride0` (a power of two below 64).
__device__ __forceinline__ float sum_lanes(float x, int stride0) {
  for (int d = stride0; d < kWaveSize; d <<= 1) x += __shfl_xor(x, d, kWaveSize);
  return x;
}

// H divides 64: lane l sees head l % H of the row's consecutive (edge, head) pairs.
__global__ __launch_bounds__(kBlockThreads) void softmax_backward_kernel(const int32_t *indptr, const float *weights,
                                                                         const float *grad, float *out,
                                                                         int32_t n_rows, int32_t H) {
  const int lane = threadIdx.x & (kWaveSize - 1);
  const int64_t n_waves = static_cast<int64_t>(gridDim.x) * kWavesPerBlock;
  for (int64_t r = static_cast<int64_t>(blockIdx.x) * kWavesPerBlock + (threadIdx.x >> 6); r < n_rows; r += n_waves) {
    const int64_t lo = indptr[r], hi = indptr[r + 1];
    if (hi <= lo) continue;
    const float *a = weights + lo * H, *g = grad + lo * H;
    float *q = out + lo * H;
    const int64_t count = (hi - lo) * H;
    float dot = 0.0f;
    for (int64_t t = lane; t < count; t += kWaveSize) dot = __builtin_fmaf(a[t], g[t], dot);
    dot = sum_lanes(dot, H);
    for (int64_t t = lane; t < count; t += kWaveSize) q[t] = a[t] * (g[t] - dot);
  }
}

// Any H: lane j walks the edges lo + j, lo + j + 64, ... of the row, head by head.
__global__ __launch_bounds__(kBlockThreads) void softmax_backward_any_kernel(const int32_t *indptr,
                                                                             const float *weights, const float *grad,
                                                                             float *out, int32_t n_rows, int32_t H) {
  const int lane = threadIdx.x & (kWaveSize - 1);
  const int64_t n_waves = static_cast<int64_t>(gridDim.x) * kWavesPerBlock;
  for (int64_t r = static_cast<int64_t>(blockIdx.x) * kWavesPerBlock + (threadIdx.x >> 6); r < n_rows; r += n_waves) {
    const int64_t lo = indptr[r], hi = indptr[r + 1];
    for (int h = 0; h < H && hi > lo; ++h) {
      float dot = 0.0f;
      for (int64_t e = lo + lane; e < hi; e += kWaveSize) dot = __builtin_fmaf(weights[e * H + h], grad[e * H + h], dot);
      dot = sum_lanes(dot, 1);
      for (int64_t e = lo + lane; e < hi; e += kWaveSize) out[e * H + h] = weights[e * H + h] * (grad[e * H + h] - dot);
    }
  }
}

// One thread per float of the result: consecutive threads write consecutive floats and read the `width` floats
// of one source row together.
__global__ __launch_bounds__(kBlockThreads) void permute_rows_kernel(const int32_t *perm, const float *in, float *out,
                                                                     int64_t n, int32_t width) {
  const int64_t total = n * width;
  const int64_t stride = static_cast<int64_t>(gridDim.x) * blockDim.x;
  for (int64_t t = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x; t < total; t += stride) {
    const int64_t i = t / width;
    const int64_t k = t - i * width;
    out[t] = in[static_cast<int64_t>(perm[i]) * width + k];
  }
}

__global__ __launch_bounds__(kBlockThreads) void add_kernel(const float *a, const float *b, float *out, int64_t n) {
  const int64_t stride = static_cast<int64_t>(gridDim.x) * blockDim.x;
  for (int64_t t = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x; t < n; t += stride) out[t] = a[t] + b[t];
}

// out[i, 0 .. F-1] = in[i, 0 .. F-1] for rows of `pitch` floats in out (the floats behind F are left as they are)
__global__ __launch_bounds__(kBlockThreads) void pad_rows_kernel(const float *in, float *out, int64_t n, int32_t F, int32_t pitch) {
  const int64_t stride = static_cast<int64_t>(gridDim.x) * blockDim.x, total = n * F;
  for (int64_t t = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x; t < total; t += stride) {
    const int64_t row = t / F;
    out[row * pitch + (t - row * F)] = in[t];
  }
}

unsigned grid_for(int64_t threads) {
  return static_cast<unsigned>(std::max<int64_t>(1, std::min<int64_t>((threads + kBlockThreads - 1) / kBlockThreads, 1 << 16)));
}

}  // namespace

int edge_softmax_backward_launch(const int32_t *indptr, const float *weights, const float *grad, float *out,
                                 int32_t n_rows, int32_t H, hipStream_t stream) {
  if (n_rows == 0) return FG_OK;
  const unsigned blocks = grid_for(static_cast<int64_t>(n_rows) * kWaveSize);
  if (H <= kWaveSize && kWaveSize % H == 0)
    softmax_backward_kernel<<<dim3(blocks), dim3(kBlockThreads), 0, stream>>>(indptr, weights, grad, out, n_rows, H);
  else
    softmax_backward_any_kernel<<<dim3(blocks), dim3(kBlockThreads), 0, stream>>>(indptr, weights, grad, out, n_rows, H);
  FG_HIP_TRY(hipGetLastError());
  return FG_OK;
}

int permute_rows_launch(const int32_t *perm, const float *in, float *out, int64_t n, int32_t width, hipStream_t stream) {
  if (n == 0) return FG_OK;
  permute_rows_kernel<<<dim3(grid_for(n * width)), dim3(kBlockThreads), 0, stream>>>(perm, in, out, n, width);
  FG_HIP_TRY(hipGetLastError());
  return FG_OK;
}

int pad_rows_launch(const float *in, float *out, int64_t n, int32_t F, int32_t pitch, hipStream_t stream) {
  if (n == 0) return FG_OK;
  pad_rows_kernel<<<dim3(grid_for(n * F)), dim3(kBlockThreads), 0, stream>>>(in, out, n, F, pitch);
  FG_HIP_TRY(hipGetLastError());
  return FG_OK;
}

int add_launch(const float *a, const float *b, float *out, int64_t n, hipStream_t stream) {
  if (n == 0) return FG_OK;
  add_kernel<<<dim3(grid_for(n)), dim3(kBlockThreads), 0, stream>>>(a, b, out, n);
  FG_HIP_TRY(hipGetLastError());
  return FG_OK;
}

}  // namespace fg
