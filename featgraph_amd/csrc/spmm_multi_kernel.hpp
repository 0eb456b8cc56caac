// CSR SpMM, several rows per wave with 16-byte gathers (gfx950).
//
// A group of G adjacent lanes owns one row and one tile of 4*G floats of it
// (G = 16: 64 floats; 8: 32; 4: 16); a wave therefore works on 64/G rows at
// once and each of its gather instructions fetches 64/G neighbour rows, 16 bytes
// per lane.  Against the wave-per-row kernels (spmm.hip) that is a quarter of
// the memory instructions per nonzero and no scalar work per nonzero at all:
// the column id and value of the group's next nonzero reach its lanes through a
// cross-lane broadcast inside the group.  Every lane still walks its row's
// nonzeros from first to last with one rounded multiply and one rounded add per
// term (-ffp-contract=off), so every output element is the same float32 sum, bit
// for bit, as in the other kernels and in the reference's loop nest
// (op/vanilla_spmm.py:46-56).
//
// Work comes as records {first nonzero, one past the last, row, first nonzero
// in the CSR arrays}, one per row and column-block pass, which the plan sorts by
// descending run length inside each pass; the first two index either the CSR
// column ids or the plan's copy of them in the records' own order, and the
// values always sit at the CSR position.  The rows that share a wave then finish together (the wave runs
// until its longest row is done; shorter ones skip the adds, and their idle
// gathers re-read row 0 of the band and are dropped).  A lane holds the ids and
// values of four consecutive nonzeros, so one 16-byte load per lane brings 4*G
// nonzeros of every row of the wave.  Like the pipelined wave-per-row kernel a
// wave keeps three work items in flight: gathers of item k, first ids / values /
// carried sums of item k+1, record of item k+2; within an item the next batch
// of ids is asked for behind the current batch's first gathers (loads return in
// order, so the adds wait only for the gathers).  Runs of kLongRun nonzeros or
// more take the one-workgroup-per-run path below instead.
//
// RED / MSG turn the multiply-add into the generalised operator (README.md:6 of the reference): term =
// MSG(feature, value), folded with RED in the same order; a picking reducer (max / min) takes a row's first
// term as it is, which a run recognises by its CSR position being indptr[row].
//
// This file holds the kernel and its launcher as templates; spmm_multi.hip instantiates the plain operator and
// spmm_multi_general_*.hip the generalised one, one message per file (each instance is a large kernel, and the
// files compile side by side).
#pragma once

#include <algorithm>
#include <utility>

#include "common.hpp"

namespace fg {
namespace {

// Runs of at least this many nonzeros go to the one-workgroup-per-run path (spmm.multi_long overrides).  Measured on
// the 232,965-vertex graph at 16 / 32 / 64 floats: 512: 1.19 / 1.08 / 1.80 ms, 1024: 1.00 / 0.99 / 1.78, 2048: 1.14 / 1.33 / 2.10
// (below it the workgroups idle at their barriers too often, above it the chains of the several-rows path set the time).
constexpr uint32_t kLongRun = 1024;

template <int... Js, typename F>
__device__ __forceinline__ void static_for(std::integer_sequence<int, Js...>, F f) {
  (f(std::integral_constant<int, Js>{}), ...);
}

template <int CTRL>
__device__ __forceinline__ int dpp_mov(int x) {
  return __builtin_amdgcn_mov_dpp(x, CTRL, 0xf, 0xf, true);
}

// Value of lane J of the caller's G-lane group; hi_half: the group is the upper half of its row of 16 (G == 8).
template <int G, int J>
__device__ __forceinline__ int group_bcast(int x, bool hi_half) {
  if constexpr (G == 16) {
    (void)hi_half;
    return dpp_mov<0x150 + J>(x);  // lane J of each row of 16
  } else if constexpr (G == 8) {
    const int lo = dpp_mov<0x150 + J>(x), hi = dpp_mov<0x158 + J>(x);
    return hi_half ? hi : lo;
  } else {
    (void)hi_half;
    return dpp_mov<J * 0x55>(x);  // quad_perm [J, J, J, J]
  }
}

// Four adjacent floats at an address that is only known to be 4-byte aligned (feature rows whose length is not a
// multiple of four floats start anywhere): one 16-byte access where the address allows it.
struct alignas(4) Float4A {
  float x, y, z, w;
};
__device__ __forceinline__ float4 load4(const float *p) {
  const Float4A q = *reinterpret_cast<const Float4A *>(p);
  return make_float4(q.x, q.y, q.z, q.w);
}
__device__ __forceinline__ void store4(float *p, const float4 &v) {
  *reinterpret_cast<Float4A *>(p) = Float4A{v.x, v.y, v.z, v.w};
}
// The same without the first `skip` floats (1 .. 3), which belong to another lane.
__device__ __forceinline__ void store4_from(float *p, const float4 &v, int skip) {
  if (skip <= 1) p[1] = v.y;
  if (skip <= 2) p[2] = v.z;
  p[3] = v.w;
}

template <bool BUF, bool U24>
struct FeatRows {
  __amdgpu_buffer_rsrc_t rsrc;
  const char *base;
  int64_t row_bytes;
  __device__ __forceinline__ FeatRows(const float *feat, int64_t n_rows, int64_t F)
      : base(reinterpret_cast<const char *>(feat)), row_bytes(F * 4) {
    rsrc = __builtin_amdgcn_make_buffer_rsrc(const_cast<float *>(feat), 0,
                                             BUF ? static_cast<int>(static_cast<uint32_t>(n_rows * F * 4)) : 0,
                                             0x00020000);
  }
  __device__ __forceinline__ float4 load(int col, uint32_t lane_bytes) const {
    if constexpr (BUF) {
      uint32_t off;
      if constexpr (U24)  // column ids and the row pitch both below 2^24: one full-rate multiply-add
        off = __umul24(static_cast<uint32_t>(col), static_cast<uint32_t>(row_bytes)) + lane_bytes;
      else
        off = static_cast<uint32_t>(col) * static_cast<uint32_t>(row_bytes) + lane_bytes;
      return __builtin_bit_cast(float4, __builtin_amdgcn_raw_buffer_load_b128(rsrc, static_cast<int>(off), 0, 0));
    } else {
      return load4(reinterpret_cast<const float *>(base + static_cast<int64_t>(col) * row_bytes + lane_bytes));
    }
  }
};

__device__ __forceinline__ void axpy4(float4 &acc, float v, const float4 &x) {
  acc.x = acc.x + v * x.x;
  acc.y = acc.y + v * x.y;
  acc.z = acc.z + v * x.z;
  acc.w = acc.w + v * x.w;
}

// The generalised operator (RED >= 0): term = MSG(feature, value), folded with the reducer RED; RED < 0 is the
// plain multiply-add above.
template <int MSG>
__device__ __forceinline__ float message_of(float u, float e) {
  if constexpr (MSG == FG_MSG_MUL) return u * e;
  if constexpr (MSG == FG_MSG_ADD) return u + e;
  if constexpr (MSG == FG_MSG_SUB) return u - e;
  if constexpr (MSG == FG_MSG_DIV) return u / e;
  return u;
}

template <int RED>
__device__ __forceinline__ float fold_of(float acc, float t) {
  if constexpr (RED == FG_REDUCE_MAX) return (t > acc) ? t : acc;
  if constexpr (RED == FG_REDUCE_MIN) return (t < acc) ? t : acc;
  return acc + t;
}

// acc <- fold(acc, msg(x, v)) on four floats; `assign`: this is the row's first term and the reducer picks
// (max / min), so the term is taken as it is, a NaN included.
template <int RED, int MSG>
__device__ __forceinline__ void fold4(float4 &acc, float v, const float4 &x, bool assign) {
  if constexpr (RED < 0) {
    (void)assign;
    axpy4(acc, v, x);
  } else {
    const float4 t = make_float4(message_of<MSG>(x.x, v), message_of<MSG>(x.y, v), message_of<MSG>(x.z, v),
                                 message_of<MSG>(x.w, v));
    constexpr bool PICKS = RED == FG_REDUCE_MAX || RED == FG_REDUCE_MIN;
    if (PICKS && assign) {
      acc = t;
    } else {
      acc.x = fold_of<RED>(acc.x, t.x);
      acc.y = fold_of<RED>(acc.y, t.y);
      acc.z = fold_of<RED>(acc.z, t.z);
      acc.w = fold_of<RED>(acc.w, t.w);
    }
  }
}

// Column ids and values of four consecutive nonzeros, held by one lane.
struct Ids {
  int c[4];
  float v[4];
};
struct alignas(4) Int4U {
  int v[4];
};
struct alignas(4) Float4U {
  float v[4];
};

// Long runs.  A row's sum is a chain: its nonzeros are added one after the other, so a kernel that keeps k
// gathers of a row in flight cannot finish a run of L nonzeros sooner than L / k memory round trips, and on a
// power-law graph the longest rows then set the time of the whole launch (most visibly at short feature
// lengths, where everything else is quick: on the 232,965-vertex benchmark graph at 32 floats the rows beyond
// 8,192 nonzeros, 0.2 % of the matrix, cost a sixth of the time while one wave worked on each of their runs).
// Here a whole WORKGROUP works on ONE run.  Per step each of its four waves takes the next kLongRounds * 64/G
// consecutive nonzeros: its 64/G groups gather 64/G of them per round, so the gathers and the (rounded) products
// of four waves x kLongRounds rounds proceed at once, and only the adds stay ordered: the products go through LDS
// to the first 4*G lanes of the first wave, lane i of which owns float i of the tile and adds its terms one by
// one, the waves' regions in turn.  Same terms, same order, same roundings as everywhere else.
constexpr int kLongRounds = 8;  // rounds per wave and step

template <int G, bool BUF, bool U24, int RED, int MSG>
__device__ __forceinline__ void spmm_long_runs(const SpmmArgs &a, const FeatRows<BUF, U24> &feat, int first_run,
                                               int run_stride, int lane, int wave, uint32_t lane_bytes, float *lds,
                                               int tile) {
  constexpr int NG = kWaveSize / G;   // nonzeros per round
  constexpr int TW = 4 * G;           // floats per tile
  constexpr int R = kLongRounds;
  constexpr int RB = R * NG;          // nonzeros per wave and step
  constexpr int SB = kWavesPerBlock * RB;       // nonzeros per step
  constexpr int Q = (RB + kWaveSize - 1) / kWaveSize;  // ids per lane and step: lane l holds ids l, 64 + l, ...
  constexpr int REGION = R * 256;     // floats of LDS per wave: R rounds x 64 lanes x float4
  constexpr bool HAS_VALS = RED < 0 || MSG != FG_MSG_COPY_U;
  const int g = lane / G;
  const int64_t F = a.F;
  const bool carry = a.accumulate != 0;
  const int f1 = (a.tile_base + tile) * TW + lane;  // the float this lane sums
  const bool adder = wave == 0 && lane < TW && f1 < a.F;
  // the lane whose four floats the row's end cuts gathers the row's last four floats instead (see the kernel), so
  // the products of the floats from the last multiple of four on sit 4 - F % 4 slots further right
  const int slot = lane + ((a.F % 4 != 0 && f1 >= a.F - a.F % 4) ? 4 - a.F % 4 : 0);
  float *const mine = lds + wave * REGION;
  struct StepIds {
    int c[Q];
    float v[Q];
  };

  for (int it = first_run; it < a.long_runs; it += run_stride) {  // the same for all four waves
    const int4 rec = a.runs[it];
    const int lo = rec.x, len = rec.y - rec.x, row = rec.z;
    if (len <= 0) continue;
    const int vo = a.vals_by_csr ? rec.w - rec.x : 0;  // from a nonzero's place in the id array to its value's
    // a picking reducer takes the row's first term as it is instead of comparing it with a carried value
    bool starts = false;
    if constexpr (RED == FG_REDUCE_MAX || RED == FG_REDUCE_MIN) starts = (a.vals_by_csr ? rec.w : rec.x) == a.indptr[row];
    float acc = 0.0f;
    if (carry && adder && !starts) acc = a.out[static_cast<int64_t>(row) * F + f1];

    // this wave's nonzeros of step s: RB of them from `at(s)` on, as many as the run still has
    auto at = [&](int s) { return s * SB + wave * RB; };
    auto load_ids = [&](int s, StepIds &d) {
      const int e = lo + at(s), rem = len - at(s);
#pragma unroll
      for (int q = 0; q < Q; ++q) {
        d.c[q] = 0;  // past the run's end: id 0, a valid row to gather from, never added
        d.v[q] = 0.0f;
        if (kWaveSize * q + lane < min(rem, RB)) {
          d.c[q] = a.indices[e + kWaveSize * q + lane];
          if (HAS_VALS) d.v[q] = a.w[e + vo + kWaveSize * q + lane];
        }
      }
    };
    // round r of a step covers the wave's nonzeros NG*r .. NG*r + NG - 1, one per group
    auto issue = [&](float4(&x)[R], const StepIds &d, int cnt) {
      static_for(std::make_integer_sequence<int, R>{}, [&](auto r) {
        constexpr int j0 = NG * decltype(r)::value, q = j0 / kWaveSize, l0 = j0 % kWaveSize;
        if (j0 < cnt) x[r] = feat.load(__builtin_amdgcn_ds_bpermute((l0 + g) << 2, d.c[q]), lane_bytes);
      });
    };
    auto products = [&](const float4(&x)[R], const StepIds &d, int cnt) {
      static_for(std::make_integer_sequence<int, R>{}, [&](auto r) {
        constexpr int j0 = NG * decltype(r)::value, q = j0 / kWaveSize, l0 = j0 % kWaveSize;
        if (j0 < cnt) {
          const float v = __int_as_float(__builtin_amdgcn_ds_bpermute((l0 + g) << 2, __float_as_int(d.v[q])));
          // lane (g, gl) holds floats 4*gl .. 4*gl+3 of nonzero g: float index g*TW + 4*gl = 4*lane
          float4 t;
          if constexpr (RED < 0)
            t = make_float4(v * x[r].x, v * x[r].y, v * x[r].z, v * x[r].w);
          else
            t = make_float4(message_of<MSG>(x[r].x, v), message_of<MSG>(x[r].y, v), message_of<MSG>(x[r].z, v),
                            message_of<MSG>(x[r].w, v));
          *reinterpret_cast<float4 *>(mine + decltype(r)::value * 256 + 4 * lane) = t;
        }
      });
    };
    auto count = [&](int s) { return max(0, min(RB, len - at(s))); };

    const int n_steps = (len + SB - 1) / SB;
    float4 x[R];
    StepIds ids_cur, ids_nxt;
    load_ids(0, ids_cur);
    issue(x, ids_cur, count(0));
    load_ids(1, ids_nxt);
    // One step: this step's products go to LDS, the next step's gathers go out into the registers they leave,
    // the first wave adds the products in order, and the regions are free again.  Every wave passes both barriers.
    for (int s = 0; s < n_steps; ++s) {
      StepIds ids_after;
      load_ids(s + 2, ids_after);
      products(x, ids_cur, count(s));
      issue(x, ids_nxt, count(s + 1));
      __syncthreads();
      if (wave == 0 && lane < TW) {
        const int here = min(SB, len - s * SB);
#pragma unroll 8
        for (int t = 0; t < here; ++t) {
          const int w = t / RB, j = t % RB;
          const float term = lds[w * REGION + (j / NG) * 256 + (j % NG) * TW + slot];
          if constexpr (RED < 0)
            acc = acc + term;
          else if ((RED == FG_REDUCE_MAX || RED == FG_REDUCE_MIN) && starts && s == 0 && t == 0)
            acc = term;
          else
            acc = fold_of<RED>(acc, term);
        }
      }
      __syncthreads();
      ids_cur = ids_nxt;
      ids_nxt = ids_after;
    }
    if (adder) a.out[static_cast<int64_t>(row) * F + f1] = acc;
  }
}

template <int G, bool BUF, bool U24, int RED, int MSG>
__global__ __launch_bounds__(kBlockThreads) __attribute__((amdgpu_waves_per_eu(3))) void spmm_multi_kernel(const SpmmArgs a) {
  constexpr bool PICKS = RED == FG_REDUCE_MAX || RED == FG_REDUCE_MIN;
  constexpr int NG = kWaveSize / G;  // rows per wave
  constexpr int TW = 4 * G;          // floats per tile
  constexpr int B = 4 * G;           // nonzeros of a row per batch: lane l of its group holds ids 4l .. 4l+3
  constexpr int SC = 4;              // lanes' worth of ids whose gathers (4 each) are issued together
  const int lane = threadIdx.x & (kWaveSize - 1);
  const int gl = lane & (G - 1);
  const int g = lane / G;
  const bool hi_half = (lane & 8) != 0;
  // `il` tiles alternate workgroup by workgroup along x, the rest of the tiles lie along y: workgroups go to the
  // XCDs round-robin, so with il = 2 half of the XCDs work on each tile of a pair
  const int il = max(a.interleave_tiles, 1);
  const int tile = static_cast<int>(blockIdx.y) * il + static_cast<int>(blockIdx.x % il);
  const int bx = static_cast<int>(blockIdx.x / il);
  const int gx = static_cast<int>(gridDim.x / il);
  // A lane owns four adjacent floats.  Where the row ends inside them (feature lengths that are not a multiple of
  // four) the lane takes the row's LAST four floats instead: it repeats, bit for bit, what its neighbour computes
  // for the floats they share, and stores only its own (the shared ones may lie in the tile before, whose carried
  // sums another wave updates in the same launch).  Lanes wholly past the row only keep the wave's cross-lane
  // traffic going: they re-read the same last floats and store nothing.
  const int f0_nominal = (a.tile_base + tile) * TW + gl * 4;
  const bool fok = f0_nominal < a.F;
  const int f0 = min(f0_nominal, a.F - 4);
  const int shared = f0_nominal - f0;  // leading floats of the lane's four that are its neighbour's
  const int64_t F = a.F;
  const uint32_t lane_bytes = static_cast<uint32_t>(f0) * 4u;
  const FeatRows<BUF, U24> feat(a.feat, a.n_cols, a.feat_pitch ? a.feat_pitch : F);
  const bool carry = a.accumulate != 0;
  // the first workgroups take the long runs (the records come by descending length), one workgroup per run
  if (bx < a.long_blocks) {
    __shared__ float products[kWavesPerBlock * kLongRounds * 256];  // per wave: rounds x 64 lanes x float4
    spmm_long_runs<G, BUF, U24, RED, MSG>(a, feat, bx, a.long_blocks, lane, static_cast<int>(threadIdx.x >> 6),
                                          lane_bytes, products, tile);
    return;
  }
  const int n_waves = (gx - a.long_blocks) * kWavesPerBlock;
  const int n = a.n_rows;
  const int n_items = (n - a.long_runs + NG - 1) / NG;
  int item = __builtin_amdgcn_readfirstlane(
      static_cast<int>((bx - a.long_blocks) * kWavesPerBlock + (threadIdx.x >> 6)));

  const bool by_csr = a.vals_by_csr != 0;
  // vo: from a nonzero's place in the id array to its place in the value array
  auto bounds = [&](int it, int &lo, int &hi, int &row, int &vo) {
    lo = hi = vo = 0;
    row = -1;
    const int pos = a.long_runs + it * NG + g;
    if (it < n_items && pos < n) {
      const int4 r = a.runs[pos];
      lo = r.x;
      hi = r.y;
      row = r.z;
      if (by_csr) vo = r.w - r.x;
    }
  };
  // this lane's four ids / values of the batch that starts at nonzero e, of which the group has `rem` left;
  // slots past the end hold column id 0 (a valid row to gather from, never added)
  auto load_ids = [&](int e, int rem, int vo, Ids &d) {
    const int k0 = 4 * gl;
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      d.c[k] = 0;
      d.v[k] = 0.0f;
    }
    constexpr bool has_vals = RED < 0 || MSG != FG_MSG_COPY_U;  // a message that ignores the values may come without them
    if (k0 + 3 < rem) {
      const Int4U ci = *reinterpret_cast<const Int4U *>(a.indices + e + k0);
      Float4U vi = {{0.0f, 0.0f, 0.0f, 0.0f}};
      if (has_vals) vi = *reinterpret_cast<const Float4U *>(a.w + e + vo + k0);
#pragma unroll
      for (int k = 0; k < 4; ++k) {
        d.c[k] = ci.v[k];
        d.v[k] = vi.v[k];
      }
    } else {
#pragma unroll
      for (int k = 0; k < 4; ++k)
        if (k0 + k < rem) {
          d.c[k] = a.indices[e + k0 + k];
          if (has_vals) d.v[k] = a.w[e + vo + k0 + k];
        }
    }
  };
  // starts: the run begins its row (asked only by the picking reducers, which take the row's first term as it is
  // instead of comparing it with a carried value); lo + vo is the run's first place in the CSR arrays
  auto first_ids = [&](int lo, int hi, int row, int vo, bool &starts, Ids &d, float4 &acc) {
    load_ids(lo, hi - lo, vo, d);
    acc = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
    starts = false;
    if constexpr (PICKS)
      if (hi > lo) starts = lo + vo == a.indptr[row];
    if (carry && hi > lo && fok && !starts)
      acc = load4(a.out + static_cast<int64_t>(row) * F + f0);
  };

  int lo_a, hi_a, row_a, vo_a, lo_b, hi_b, row_b, vo_b;
  bool st_a, st_b = false;
  Ids ids_a;
  float4 acc_a;
  bounds(item, lo_a, hi_a, row_a, vo_a);
  first_ids(lo_a, hi_a, row_a, vo_a, st_a, ids_a, acc_a);
  bounds(item + n_waves, lo_b, hi_b, row_b, vo_b);

  while (item < n_items) {
    int lo_c, hi_c, row_c, vo_c, e = lo_a, rem = hi_a - lo_a;  // rem: nonzeros this group still has
    Ids ids_b;
    float4 acc_b;
    bounds(item + 2 * n_waves, lo_c, hi_c, row_c, vo_c);
    bool next_asked = false;

    while (__builtin_amdgcn_ballot_w64(rem > 0) != 0) {
      Ids ids_n;
      static_for(std::make_integer_sequence<int, G / SC>{}, [&](auto sc) {
        constexpr int l0 = decltype(sc)::value * SC;  // first id-holding lane of this step
        if (l0 == 0 || __builtin_amdgcn_ballot_w64(rem > 4 * l0) != 0) {
          float4 x[4 * SC];
          static_for(std::make_integer_sequence<int, SC>{}, [&](auto u) {
            constexpr int l = l0 + decltype(u)::value;
            if (decltype(u)::value == 0 || __builtin_amdgcn_ballot_w64(rem > 4 * l) != 0) {
#pragma unroll
              for (int k = 0; k < 4; ++k)
                x[4 * decltype(u)::value + k] = feat.load(group_bcast<G, l>(ids_a.c[k], hi_half), lane_bytes);
            }
          });
          if (l0 == 0) {  // behind the batch's first gathers: the next item's first ids (once), this item's next batch
            if (!next_asked) first_ids(lo_b, hi_b, row_b, vo_b, st_b, ids_b, acc_b);
            next_asked = true;
            load_ids(e + B, rem - B, vo_a, ids_n);
          }
          static_for(std::make_integer_sequence<int, SC>{}, [&](auto u) {
            constexpr int l = l0 + decltype(u)::value;
            if (__builtin_amdgcn_ballot_w64(rem >= 4 * l + 4) == ~0ull) {  // every group has these four nonzeros
#pragma unroll
              for (int k = 0; k < 4; ++k)
                fold4<RED, MSG>(acc_a, __int_as_float(group_bcast<G, l>(__float_as_int(ids_a.v[k]), hi_half)),
                           x[4 * decltype(u)::value + k], PICKS && l == 0 && k == 0 && st_a && e == lo_a);
            } else if (decltype(u)::value == 0 || __builtin_amdgcn_ballot_w64(rem > 4 * l) != 0) {
#pragma unroll
              for (int k = 0; k < 4; ++k) {
                const float v = __int_as_float(group_bcast<G, l>(__float_as_int(ids_a.v[k]), hi_half));
                if (4 * l + k < rem)
                  fold4<RED, MSG>(acc_a, v, x[4 * decltype(u)::value + k], PICKS && l == 0 && k == 0 && st_a && e == lo_a);
              }
            }
          });
        }
      });
      ids_a = ids_n;
      e += B;
      rem -= B;
    }
    if (!next_asked) first_ids(lo_b, hi_b, row_b, vo_b, st_b, ids_b, acc_b);  // no group had a nonzero here
    if (fok && row_a >= 0 && (hi_a > lo_a || !carry)) {
      float *const to = a.out + static_cast<int64_t>(row_a) * F + f0;
      if (shared == 0)
        store4(to, acc_a);
      else
        store4_from(to, acc_a, shared);
    }

    lo_a = lo_b;
    hi_a = hi_b;
    row_a = row_b;
    vo_a = vo_b;
    st_a = st_b;
    ids_a = ids_b;
    acc_a = acc_b;
    lo_b = lo_c;
    hi_b = hi_c;
    row_b = row_c;
    vo_b = vo_c;
    item += n_waves;
  }
}

template <int G, int RED, int MSG>
int launch_multi(const SpmmArgs &a, int64_t blocks, bool buf, bool u24, hipStream_t stream) {
  constexpr int NG = kWaveSize / G;
  const int64_t n_items = (static_cast<int64_t>(a.n_rows) - a.long_runs + NG - 1) / NG;
  blocks = std::max<int64_t>(1, std::min<int64_t>(blocks, (n_items + kWavesPerBlock - 1) / kWavesPerBlock));
  const int il = std::max(a.interleave_tiles, 1);
  if (a.n_tiles % il != 0) return fail(FG_EINVAL, "tile interleave %d does not divide %d tiles", il, a.n_tiles);
  const dim3 grid(static_cast<unsigned>((blocks + a.long_blocks) * il), static_cast<unsigned>(a.n_tiles / il));
  if constexpr (RED >= 0) {  // the generalised operator: buffer addressing with 24-bit offsets, or 64-bit addresses
    if (buf && u24)
      spmm_multi_kernel<G, true, true, RED, MSG><<<grid, dim3(kBlockThreads), 0, stream>>>(a);
    else
      spmm_multi_kernel<G, false, false, RED, MSG><<<grid, dim3(kBlockThreads), 0, stream>>>(a);
  } else if (buf && u24) {
    spmm_multi_kernel<G, true, true, RED, MSG><<<grid, dim3(kBlockThreads), 0, stream>>>(a);
  } else if (buf) {
    spmm_multi_kernel<G, true, false, RED, MSG><<<grid, dim3(kBlockThreads), 0, stream>>>(a);
  } else {
    spmm_multi_kernel<G, false, false, RED, MSG><<<grid, dim3(kBlockThreads), 0, stream>>>(a);
  }
  FG_HIP_TRY(hipGetLastError());
  return FG_OK;
}

// The generalised operator with message MSG and reducer RED, tile width by feature length as for the plain one.
template <int RED, int MSG>
int launch_multi_general_tile(const SpmmArgs &a, int64_t blocks, hipStream_t stream) {
  const int tile = a.multi_tile ? a.multi_tile : spmm_multi_tile(a.F);
  const int64_t pitch = a.feat_pitch ? a.feat_pitch : a.F;
  const bool buf = static_cast<int64_t>(a.n_cols) * pitch * 4 < (int64_t{1} << 32) && config().spmm_buffer_loads != 0;
  const bool u24 = a.n_cols <= (1 << 24) && pitch * 4 < (1 << 24);
  if (tile == 16) return launch_multi<4, RED, MSG>(a, blocks, buf, u24, stream);
  if (tile == 32) return launch_multi<8, RED, MSG>(a, blocks, buf, u24, stream);
  return launch_multi<16, RED, MSG>(a, blocks, buf, u24, stream);
}

template <int MSG>
int launch_multi_general(const SpmmArgs &a, int64_t blocks, hipStream_t stream) {
  switch (a.reduce) {
    case FG_REDUCE_SUM: return launch_multi_general_tile<FG_REDUCE_SUM, MSG>(a, blocks, stream);
    case FG_REDUCE_MAX: return launch_multi_general_tile<FG_REDUCE_MAX, MSG>(a, blocks, stream);
    case FG_REDUCE_MIN: return launch_multi_general_tile<FG_REDUCE_MIN, MSG>(a, blocks, stream);
  }
  return fail(FG_EINVAL, "reduce = %d has no several-rows-per-wave kernel", a.reduce);
}

}  // namespace
}  // namespace fg
