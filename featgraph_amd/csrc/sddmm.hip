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

int sddmm_launch(const SddmmArgs &a, const SddmmShape &s, hipStream_t stream) {
  if (a.n_ve == 0) return FG_OK;
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
