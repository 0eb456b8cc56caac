// How the one-wave-per-destination-row multi-head kernels (softmax.hip, attention.hip) lay a vertex row of
// H * D floats over a wave, and the lane arithmetic that goes with it.
//
// A row is NV chunks of 64 * VW floats; in chunk k lane l holds the VW floats at k * 64 * VW + l * VW, so every
// load instruction of a gather covers consecutive addresses.  LC = D / VW adjacent lanes share a head inside a
// chunk, a chunk holds HC = 64 / LC heads, H = NV * HC.
#pragma once

#include "common.hpp"

namespace fg {

template <int VW>
struct Floats {
  float v[VW];
};

template <int VW>
__device__ __forceinline__ Floats<VW> load_floats(const float *p) {
  Floats<VW> r;
  if constexpr (VW == 1) {
    r.v[0] = *p;
  } else if constexpr (VW == 2) {
    const float2 q = *reinterpret_cast<const float2 *>(p);
    r.v[0] = q.x, r.v[1] = q.y;
  } else {
    const float4 q = *reinterpret_cast<const float4 *>(p);
    r.v[0] = q.x, r.v[1] = q.y, r.v[2] = q.z, r.v[3] = q.w;
  }
  return r;
}

template <int VW>
__device__ __forceinline__ void store_floats(float *p, const Floats<VW> &r) {
  if constexpr (VW == 1)
    *p = r.v[0];
  else if constexpr (VW == 2)
    *reinterpret_cast<float2 *>(p) = make_float2(r.v[0], r.v[1]);
  else
    *reinterpret_cast<float4 *>(p) = make_float4(r.v[0], r.v[1], r.v[2], r.v[3]);
}

template <int CTRL>
__device__ __forceinline__ float dpp_add(float x) {
  const int y = __builtin_amdgcn_update_dpp(0, __float_as_int(x), CTRL, 0xF, 0xF, false);
  return x + __int_as_float(y);
}

// Sum over aligned groups of G lanes (G <= 16); every lane of the group gets the total.
template <int G>
__device__ __forceinline__ float group_sum(float x) {
  if (G >= 2) x = dpp_add<0xB1>(x);    // quad_perm [1,0,3,2]
  if (G >= 4) x = dpp_add<0x4E>(x);    // quad_perm [2,3,0,1]
  if (G >= 8) x = dpp_add<0x141>(x);   // row_half_mirror
  if (G >= 16) x = dpp_add<0x140>(x);  // row_mirror
  return x;
}

// The layout for (H, D), or false when there is none: the widest load for which a head spans 4, 8 or 16 lanes
// of a chunk and the row is one or two chunks.
inline bool row_layout(int32_t H, int32_t D, int *lc, int *vw, int *nv) {
  for (int w = 4; w >= 1; w >>= 1) {
    if (D % w != 0) continue;
    const int c = D / w;
    if (c != 4 && c != 8 && c != 16) continue;
    const int hc = kWaveSize / c;
    if (H % hc != 0) continue;
    const int n = H / hc;
    if ((n != 1 && n != 2) || c % n != 0) continue;
    *lc = c, *vw = w, *nv = n;
    return true;
  }
  return false;
}

}  // namespace fg
