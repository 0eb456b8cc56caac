// Measurement aid: how fast the part serves the gather pattern of the SpMM / SDDMM kernels when nothing else
// is asked of it.
//
// fg_probe_gather_f32 issues n_gathers row gathers per feature tile with the kernels' own shape: a group of
// tile/4 lanes fetches one row's tile with 16-byte loads (a 64-float tile: four rows per wave instruction),
// sixteen gathers in flight per lane, the rows of one launch drawn from one band of `band_rows` consecutive
// rows, one launch per band and tile, bands in ascending order.  What it leaves out is everything a real
// operator adds: no index or value stream (row numbers come from a per-group random-number recurrence), no
// sums carried between launches, no ordered accumulation, no output.  The time it takes is therefore a floor
// for any kernel that moves the same rows through the same cache hierarchy with the same blocking, and
// bench.py reports operator time against it.
#include <algorithm>

#include "common.hpp"

namespace {

constexpr int kProbeBlocks = 4096;  // workgroups per launch

template <int G>
__global__ __launch_bounds__(fg::kBlockThreads) void probe_gather_kernel(const float *feat, uint32_t row_bytes,
                                                                         uint32_t tile_byte0, uint32_t band_lo,
                                                                         uint32_t band_rows, int iters,
                                                                         uint32_t bytes, float *sink) {
  constexpr int U = 16;
  const int lane = threadIdx.x & (fg::kWaveSize - 1);
  const int gl = lane & (G - 1), g = lane / G;
  const uint32_t wave = blockIdx.x * fg::kWavesPerBlock + (threadIdx.x >> 6);
  uint32_t s = wave * 2654435761u + static_cast<uint32_t>(g) * 40503u + band_lo * 97u + 12345u;
  float4 acc = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
  const __amdgpu_buffer_rsrc_t rsrc =
      __builtin_amdgcn_make_buffer_rsrc(const_cast<float *>(feat), 0, static_cast<int>(bytes), 0x00020000);
  for (int it = 0; it < iters; ++it) {
    float4 x[U];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      s = s * 1664525u + 1013904223u;
      const uint32_t r = band_lo + (s >> 8) % band_rows;
      const uint32_t off = r * row_bytes + tile_byte0 + static_cast<uint32_t>(gl) * 16u;
      x[u] = __builtin_bit_cast(float4, __builtin_amdgcn_raw_buffer_load_b128(rsrc, static_cast<int>(off), 0, 0));
    }
#pragma unroll
    for (int u = 0; u < U; ++u) {
      acc.x += x[u].x;
      acc.y += x[u].y;
      acc.z += x[u].z;
      acc.w += x[u].w;
    }
  }
  // keeps the loads alive; finite feature values never produce this sum
  if (acc.x + acc.y + acc.z + acc.w == __builtin_inff()) sink[0] = acc.x;
}

// Whole rows of `row_floats` floats (128, 256, or a multiple of 256) from anywhere in the matrix, addressed
// in 64 bits: the pattern of the multi-head operators, whose feature matrices are far larger than any cache.
// LPR lanes fetch one row with NV 16-byte loads each; 16 loads are in flight per lane.  With write_every > 0
// every group of LPR lanes also writes one whole row of `out` (a random one) after every write_every-th
// iteration, as an operator that produces one result row per so many gathered rows does.
template <int LPR, int NV>
__global__ __launch_bounds__(fg::kBlockThreads) void probe_rows_kernel(const float *feat, int64_t row_floats,
                                                                       uint32_t n_rows, int iters, float *sink,
                                                                       float *out, uint32_t out_rows,
                                                                       int write_every) {
  constexpr int U = 16 / NV;
  const int lane = threadIdx.x & (fg::kWaveSize - 1);
  const int gl = lane & (LPR - 1), g = lane / LPR;
  const uint32_t wave = blockIdx.x * fg::kWavesPerBlock + (threadIdx.x >> 6);
  uint32_t s = wave * 2654435761u + static_cast<uint32_t>(g) * 40503u + 12345u;
  float4 acc = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
  int until_write = write_every;
  for (int it = 0; it < iters; ++it) {
    float4 x[U][NV];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      s = s * 1664525u + 1013904223u;
      const uint32_t r = (s >> 4) % n_rows;
      const float *p = feat + static_cast<int64_t>(r) * row_floats + gl * 4;
#pragma unroll
      for (int k = 0; k < NV; ++k) x[u][k] = *reinterpret_cast<const float4 *>(p + k * 256);
    }
#pragma unroll
    for (int u = 0; u < U; ++u)
#pragma unroll
      for (int k = 0; k < NV; ++k) {
        acc.x += x[u][k].x;
        acc.y += x[u][k].y;
        acc.z += x[u][k].z;
        acc.w += x[u][k].w;
      }
    if (write_every > 0 && --until_write == 0) {
      until_write = write_every;
      const uint32_t r = (s >> 5) % out_rows;
      float *q = out + static_cast<int64_t>(r) * row_floats + gl * 4;
#pragma unroll
      for (int k = 0; k < NV; ++k) *reinterpret_cast<float4 *>(q + k * 256) = acc;
    }
  }
  if (acc.x + acc.y + acc.z + acc.w == __builtin_inff()) sink[0] = acc.x;
}

// Stores alone: every group of LPR lanes writes `rows_each` whole rows of `out`, random ones.
template <int LPR, int NV>
__global__ __launch_bounds__(fg::kBlockThreads) void probe_store_rows_kernel(float *out, int64_t row_floats,
                                                                             uint32_t out_rows, int rows_each) {
  const int lane = threadIdx.x & (fg::kWaveSize - 1);
  const int gl = lane & (LPR - 1), g = lane / LPR;
  const uint32_t wave = blockIdx.x * fg::kWavesPerBlock + (threadIdx.x >> 6);
  uint32_t s = wave * 2654435761u + static_cast<uint32_t>(g) * 40503u + 777u;
  const float4 v = make_float4(1.0f, 2.0f, 3.0f, static_cast<float>(lane));
  for (int it = 0; it < rows_each; ++it) {
    s = s * 1664525u + 1013904223u;
    float *q = out + static_cast<int64_t>((s >> 5) % out_rows) * row_floats + gl * 4;
#pragma unroll
    for (int k = 0; k < NV; ++k) *reinterpret_cast<float4 *>(q + k * 256) = v;
  }
}

// (lanes per row, loads per lane, rows per iteration of the grid) for a row length, or false.
bool rows_shape(int32_t row_floats, int *lpr, int *nv, int64_t *per_iter) {
  if (row_floats == 128)
    *lpr = 32, *nv = 1;
  else if (row_floats == 256)
    *lpr = 64, *nv = 1;
  else if (row_floats == 512)
    *lpr = 64, *nv = 2;
  else if (row_floats == 1024)
    *lpr = 64, *nv = 4;
  else
    return false;
  *per_iter = int64_t{kProbeBlocks} * fg::kWavesPerBlock * (fg::kWaveSize / *lpr) * (16 / *nv);
  return true;
}

// The gather pattern of probe_gather_kernel (64-float tiles, one 4 MB band) with an id / value-like stream beside
// it: 8 bytes per gathered row, read from `stream` at addresses no wave shares, wrapped into a window of
// window_dw dwords (the whole buffer: every piece comes from HBM; 64 MB: the Infinity Cache holds it; 256 KB: L2
// does).  MODE 1: every wave reads its own piece (512 bytes per sixteen gather instructions) with one vector load,
// requested an iteration ahead and mixed into the next iteration's row numbers, as an operator's ids are.
// MODE 2: the first wave of every workgroup reads the pieces of all four and gathers nothing; the other three
// gather a third more each.  MODE 3: as MODE 1 through the scalar cache (wave-uniform address).
template <int MODE>
__global__ __launch_bounds__(fg::kBlockThreads) void probe_gather_stream_kernel(const float *feat, uint32_t band_rows,
                                                                                const uint32_t *__restrict__ stream,
                                                                                uint32_t window_dw, int iters,
                                                                                uint32_t bytes, float *sink) {
  constexpr int U = 16;
  const int lane = threadIdx.x & (fg::kWaveSize - 1);
  const int gl = lane & 15, g = lane / 16;
  const uint32_t wave = __builtin_amdgcn_readfirstlane(blockIdx.x * fg::kWavesPerBlock + (threadIdx.x >> 6));
  uint32_t s = wave * 2654435761u + static_cast<uint32_t>(g) * 40503u + 12345u;
  float4 acc = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
  const __amdgpu_buffer_rsrc_t rsrc =
      __builtin_amdgcn_make_buffer_rsrc(const_cast<float *>(feat), 0, static_cast<int>(bytes), 0x00020000);
  const uint32_t mask = window_dw - 1;  // a power of two
  uint32_t id_now = 0, id_next = 0;
  if (MODE == 2) {
    if ((threadIdx.x >> 6) == 0) {
      uint32_t t = 0;
      for (int it = 0; it < iters * fg::kWavesPerBlock; it += 8) {
        uint2 v[8];
#pragma unroll
        for (int k = 0; k < 8; ++k) {
          const uint32_t at = ((blockIdx.x * static_cast<uint32_t>(fg::kWavesPerBlock * iters) + static_cast<uint32_t>(it + k)) * 128u) & mask;
          v[k] = *reinterpret_cast<const uint2 *>(stream + at + lane * 2);
        }
#pragma unroll
        for (int k = 0; k < 8; ++k) t += v[k].x + v[k].y;
      }
      if (t == 0x12345u) sink[1] = 1.0f;
      return;
    }
    iters = iters * 4 / 3;
  }
  for (int it = 0; it < iters; ++it) {
    const uint32_t at = ((wave * static_cast<uint32_t>(iters) + static_cast<uint32_t>(it)) * 128u) & mask;
    if (MODE == 1) {
      const uint2 v = *reinterpret_cast<const uint2 *>(stream + at + lane * 2);
      id_next = v.x + v.y;
    } else if (MODE == 3) {
      uint32_t t = 0;
#pragma unroll
      for (int k = 0; k < 128; ++k) t += stream[at + k];
      id_next = t;
    }
    float4 x[U];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      s = s * 1664525u + 1013904223u;
      const uint32_t r = ((s >> 8) + id_now) % band_rows;
      x[u] = __builtin_bit_cast(float4, __builtin_amdgcn_raw_buffer_load_b128(rsrc, static_cast<int>(r * 256u + gl * 16u), 0, 0));
    }
#pragma unroll
    for (int u = 0; u < U; ++u) {
      acc.x += x[u].x;
      acc.y += x[u].y;
      acc.z += x[u].z;
      acc.w += x[u].w;
    }
    id_now = id_next;
  }
  if (acc.x + acc.y + acc.z + acc.w == __builtin_inff()) sink[0] = acc.x;
}

}  // namespace

// Iterations of the grid and, with writes, iterations between a group's writes, for a request.
static int rows_iters(int64_t per_iter, int64_t n_gathers) {
  return static_cast<int>(std::max<int64_t>(1, (n_gathers + per_iter / 2) / per_iter));
}
static int rows_write_every(int nv, int32_t gathers_per_write) {
  const int u = 16 / nv;  // rows a group gathers per iteration
  return gathers_per_write <= 0 ? 0 : std::max(1, (gathers_per_write + u / 2) / u);
}

static int probe_rows_run(const float *feat, int64_t n_rows, int32_t row_floats, int64_t n_gathers,
                          int32_t gathers_per_write, float *out, int64_t n_out_rows, float *sink, void *stream) {
  if (!feat || !sink) return fg::fail(FG_EINVAL, "feat or sink is null");
  int lpr, nv;
  int64_t per_iter;
  if (!rows_shape(row_floats, &lpr, &nv, &per_iter))
    return fg::fail(FG_EINVAL, "row_floats = %d is not one of 128, 256, 512, 1024", row_floats);
  if (n_rows < 1 || n_rows > 0xffffffffLL || n_gathers < 0) return fg::fail(FG_EINVAL, "n_rows or n_gathers out of range");
  if (!fg::aligned_to(feat, 16)) return fg::fail(FG_EINVAL, "feat must be 16-byte aligned");
  const int we = rows_write_every(nv, gathers_per_write);
  if (we > 0 && (!out || n_out_rows < 1 || n_out_rows > 0xffffffffLL || !fg::aligned_to(out, 16)))
    return fg::fail(FG_EINVAL, "writes need a 16-byte aligned out with 1 .. 2^32 - 1 rows");
  hipStream_t st = static_cast<hipStream_t>(stream);
  const int iters = rows_iters(per_iter, n_gathers);
  const uint32_t n = static_cast<uint32_t>(n_rows), no = static_cast<uint32_t>(we > 0 ? n_out_rows : 1);
  const dim3 grid(kProbeBlocks), block(fg::kBlockThreads);
  if (row_floats == 128)
    probe_rows_kernel<32, 1><<<grid, block, 0, st>>>(feat, row_floats, n, iters, sink, out, no, we);
  else if (row_floats == 256)
    probe_rows_kernel<64, 1><<<grid, block, 0, st>>>(feat, row_floats, n, iters, sink, out, no, we);
  else if (row_floats == 512)
    probe_rows_kernel<64, 2><<<grid, block, 0, st>>>(feat, row_floats, n, iters, sink, out, no, we);
  else
    probe_rows_kernel<64, 4><<<grid, block, 0, st>>>(feat, row_floats, n, iters, sink, out, no, we);
  FG_HIP_TRY(hipGetLastError());
  return FG_OK;
}

extern "C" int fg_probe_gather_rows_f32(const float *feat, int64_t n_rows, int32_t row_floats, int64_t n_gathers,
                                        float *sink, void *stream) {
  return probe_rows_run(feat, n_rows, row_floats, n_gathers, 0, nullptr, 0, sink, stream);
}

extern "C" int64_t fg_probe_gather_rows_count(int32_t row_floats, int64_t n_gathers) {
  int lpr, nv;
  int64_t per_iter;
  if (!rows_shape(row_floats, &lpr, &nv, &per_iter) || n_gathers < 0) return -1;
  return rows_iters(per_iter, n_gathers) * per_iter;
}

extern "C" int fg_probe_gather_write_rows_f32(const float *feat, int64_t n_rows, int32_t row_floats,
                                              int64_t n_gathers, int32_t gathers_per_write, float *out,
                                              int64_t n_out_rows, float *sink, void *stream) {
  if (gathers_per_write < 1) return fg::fail(FG_EINVAL, "gathers_per_write = %d must be positive", gathers_per_write);
  return probe_rows_run(feat, n_rows, row_floats, n_gathers, gathers_per_write, out, n_out_rows, sink, stream);
}

extern "C" int fg_probe_gather_write_rows_count(int32_t row_floats, int64_t n_gathers, int32_t gathers_per_write,
                                                int64_t *gathers, int64_t *writes) {
  int lpr, nv;
  int64_t per_iter;
  if (!gathers || !writes) return fg::fail(FG_EINVAL, "a result pointer is null");
  if (!rows_shape(row_floats, &lpr, &nv, &per_iter) || n_gathers < 0 || gathers_per_write < 1)
    return fg::fail(FG_EINVAL, "row_floats, n_gathers or gathers_per_write out of range");
  const int iters = rows_iters(per_iter, n_gathers);
  const int64_t groups = int64_t{kProbeBlocks} * fg::kWavesPerBlock * (fg::kWaveSize / lpr);
  *gathers = iters * per_iter;
  *writes = groups * (iters / rows_write_every(nv, gathers_per_write));
  return FG_OK;
}

extern "C" int64_t fg_probe_store_rows_f32(float *out, int64_t n_out_rows, int32_t row_floats, int64_t n_stores,
                                           void *stream) {
  int lpr, nv;
  int64_t per_iter;
  if (!out || !rows_shape(row_floats, &lpr, &nv, &per_iter) || n_out_rows < 1 || n_out_rows > 0xffffffffLL ||
      n_stores < 0 || !fg::aligned_to(out, 16)) {
    fg::fail(FG_EINVAL, "out, row_floats (128, 256, 512 or 1024), n_out_rows or n_stores out of range");
    return -1;
  }
  const int64_t groups = int64_t{kProbeBlocks} * fg::kWavesPerBlock * (fg::kWaveSize / lpr);
  const int rows_each = static_cast<int>(std::max<int64_t>(1, (n_stores + groups / 2) / groups));
  const uint32_t no = static_cast<uint32_t>(n_out_rows);
  const dim3 grid(kProbeBlocks), block(fg::kBlockThreads);
  hipStream_t st = static_cast<hipStream_t>(stream);
  if (row_floats == 128)
    probe_store_rows_kernel<32, 1><<<grid, block, 0, st>>>(out, row_floats, no, rows_each);
  else if (row_floats == 256)
    probe_store_rows_kernel<64, 1><<<grid, block, 0, st>>>(out, row_floats, no, rows_each);
  else if (row_floats == 512)
    probe_store_rows_kernel<64, 2><<<grid, block, 0, st>>>(out, row_floats, no, rows_each);
  else
    probe_store_rows_kernel<64, 4><<<grid, block, 0, st>>>(out, row_floats, no, rows_each);
  if (hipGetLastError() != hipSuccess) {
    fg::fail(FG_EHIP, "probe launch failed");
    return -1;
  }
  return groups * rows_each;  // rows stored
}

extern "C" int fg_probe_gather_f32(const float *feat, int64_t n_rows, int32_t F, int32_t tile, int32_t band_rows,
                                   int64_t n_gathers, float *sink, void *stream) {
  if (!feat || !sink) return fg::fail(FG_EINVAL, "feat or sink is null");
  if (n_rows < 1 || F < 4 || F % 4 != 0) return fg::fail(FG_EINVAL, "need n_rows >= 1 and F a positive multiple of 4");
  if (tile != 16 && tile != 32 && tile != 64) return fg::fail(FG_EINVAL, "tile = %d is not one of 16, 32, 64", tile);
  if (F % tile != 0) return fg::fail(FG_EINVAL, "F = %d is not a multiple of the tile width %d", F, tile);
  if (band_rows < 1 || n_gathers < 0) return fg::fail(FG_EINVAL, "band_rows must be positive, n_gathers non-negative");
  if (n_rows * F * 4 >= (int64_t{1} << 32))
    return fg::fail(FG_EUNSUPPORTED, "the probe addresses the matrix with 32-bit offsets: below 4 GiB only");
  if (!fg::aligned_to(feat, 16)) return fg::fail(FG_EINVAL, "feat must be 16-byte aligned");
  hipStream_t st = static_cast<hipStream_t>(stream);
  const int G = tile / 4;
  const int64_t passes = (n_rows + band_rows - 1) / band_rows;
  const int blocks = kProbeBlocks;
  const int64_t per_iter = static_cast<int64_t>(blocks) * fg::kWavesPerBlock * (fg::kWaveSize / G) * 16;
  const int iters = static_cast<int>(std::max<int64_t>(1, (n_gathers / passes + per_iter / 2) / per_iter));
  const uint32_t bytes = static_cast<uint32_t>(n_rows * F * 4);
  for (int t = 0; t < F / tile; ++t) {
    for (int64_t p = 0; p < passes; ++p) {
      const uint32_t lo = static_cast<uint32_t>(p * band_rows);
      const uint32_t rows = static_cast<uint32_t>(std::min<int64_t>(band_rows, n_rows - p * band_rows));
      const uint32_t byte0 = static_cast<uint32_t>(t) * tile * 4u;
      if (G == 4)
        probe_gather_kernel<4><<<dim3(blocks), dim3(fg::kBlockThreads), 0, st>>>(feat, F * 4u, byte0, lo, rows, iters,
                                                                                bytes, sink);
      else if (G == 8)
        probe_gather_kernel<8><<<dim3(blocks), dim3(fg::kBlockThreads), 0, st>>>(feat, F * 4u, byte0, lo, rows, iters,
                                                                                bytes, sink);
      else
        probe_gather_kernel<16><<<dim3(blocks), dim3(fg::kBlockThreads), 0, st>>>(feat, F * 4u, byte0, lo, rows,
                                                                                 iters, bytes, sink);
    }
  }
  FG_HIP_TRY(hipGetLastError());
  return FG_OK;
}

// Gathers that one call of fg_probe_gather_f32 with these arguments issues per feature tile (the request is
// rounded to whole iterations of the launch grid).
extern "C" int64_t fg_probe_gather_count(int64_t n_rows, int32_t tile, int32_t band_rows, int64_t n_gathers) {
  if (n_rows < 1 || band_rows < 1 || (tile != 16 && tile != 32 && tile != 64) || n_gathers < 0) return -1;
  const int G = tile / 4;
  const int64_t passes = (n_rows + band_rows - 1) / band_rows;
  const int64_t per_iter = int64_t{kProbeBlocks} * fg::kWavesPerBlock * (fg::kWaveSize / G) * 16;
  const int64_t iters = std::max<int64_t>(1, (n_gathers / passes + per_iter / 2) / per_iter);
  return passes * iters * per_iter;
}

// n_gathers rows of 64 floats out of the first band_rows rows of feat, with 8 bytes per gather read from
// stream_buf beside them (mode and window as described at the kernel; mode 0: no stream).  stream_buf holds
// stream_dwords dwords of zeros, window_dwords of which are used; both are powers of two, window_dwords >= 65536.
// Returns the number of gathers issued (the request rounded to whole iterations of the grid), or -1.
extern "C" int64_t fg_probe_gather_stream_f32(const float *feat, int32_t band_rows, int64_t n_gathers,
                                              const uint32_t *stream_buf, int64_t stream_dwords, int64_t window_dwords,
                                              int32_t mode, float *sink, void *stream) {
  auto pow2 = [](int64_t v) { return v > 0 && (v & (v - 1)) == 0; };
  if (!feat || !sink || band_rows < 1 || band_rows > (1 << 23) || n_gathers < 0 || mode < 0 || mode > 3) {
    fg::fail(FG_EINVAL, "bad argument to the gather-and-stream probe");
    return -1;
  }
  if (mode != 0 && (!stream_buf || !pow2(stream_dwords) || !pow2(window_dwords) || window_dwords > stream_dwords ||
                    window_dwords < 65536 || stream_dwords > (int64_t{1} << 32) || !fg::aligned_to(stream_buf, 16))) {
    fg::fail(FG_EINVAL, "the stream buffer and its window are powers of two of dwords, the window at least 65536");
    return -1;
  }
  if (!fg::aligned_to(feat, 16)) {
    fg::fail(FG_EINVAL, "feat must be 16-byte aligned");
    return -1;
  }
  hipStream_t st = static_cast<hipStream_t>(stream);
  const int blocks = kProbeBlocks;
  const int64_t per_iter = static_cast<int64_t>(blocks) * fg::kWavesPerBlock * 4 * 16;
  int iters = static_cast<int>(std::max<int64_t>(1, (n_gathers + per_iter / 2) / per_iter));
  if (mode == 2) iters = (iters + 5) / 6 * 6;  // whole batches of eight pieces for the reading wave, 4/3 for the others
  const uint32_t bytes = static_cast<uint32_t>(band_rows) * 256u;
  const uint32_t window = static_cast<uint32_t>(mode ? window_dwords : 65536);
  const dim3 grid(blocks), block(fg::kBlockThreads);
  switch (mode) {
    case 0: probe_gather_stream_kernel<0><<<grid, block, 0, st>>>(feat, band_rows, stream_buf, window, iters, bytes, sink); break;
    case 1: probe_gather_stream_kernel<1><<<grid, block, 0, st>>>(feat, band_rows, stream_buf, window, iters, bytes, sink); break;
    case 2: probe_gather_stream_kernel<2><<<grid, block, 0, st>>>(feat, band_rows, stream_buf, window, iters, bytes, sink); break;
    default: probe_gather_stream_kernel<3><<<grid, block, 0, st>>>(feat, band_rows, stream_buf, window, iters, bytes, sink); break;
  }
  if (hipGetLastError() != hipSuccess) {
    fg::fail(FG_EHIP, "the gather-and-stream probe did not launch");
    return -1;
  }
  return static_cast<int64_t>(iters) * per_iter;
}
