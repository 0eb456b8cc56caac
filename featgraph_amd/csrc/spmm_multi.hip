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
// Work comes as records {first nonzero, one past the last, row}, one per row
// and column-block pass, which the plan sorts by descending run length inside
// each pass: the rows that share a wave then finish together (the wave runs
// until its longest row is done; shorter ones skip the adds, and their idle
// gathers re-read row 0 of the band and are dropped).  A lane holds the ids and
// values of four consecutive nonzeros, so one 16-byte load per lane brings 4*G
// nonzeros of every row of the wave.  Like the pipelined wave-per-row kernel a
// wave keeps three work items in flight: gathers of item k, first ids / values /
// carried sums of item k+1, record of item k+2; within an item the next batch
// of ids is asked for behind the current batch's first gathers (loads return in
// order, so the adds wait only for the gathers).  Runs of kLongRun nonzeros or
// more take the one-wave-per-run path below instead.
#include <hipcub/hipcub.hpp>

#include <utility>

#include "common.hpp"

namespace fg {
namespace {

// Runs of at least this many nonzeros go to the one-wave-per-run path (spmm.multi_long overrides).
constexpr uint32_t kLongRun = 512;

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
      return *reinterpret_cast<const float4 *>(base + static_cast<int64_t>(col) * row_bytes + lane_bytes);
    }
  }
};

__device__ __forceinline__ void axpy4(float4 &acc, float v, const float4 &x) {
  acc.x = acc.x + v * x.x;
  acc.y = acc.y + v * x.y;
  acc.z = acc.z + v * x.z;
  acc.w = acc.w + v * x.w;
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
// lengths, where everything else is quick).  Here one wave works on ONE run: its 64/G groups take 64/G
// consecutive nonzeros per round, so the gathers and the (rounded) products of many nonzeros proceed at once,
// and only the adds stay ordered: the products go through LDS to the first 4*G lanes, lane i of which owns
// float i of the tile and adds its terms one by one.  Same terms, same order, same roundings as everywhere else.
constexpr int kLongRounds = 8;  // rounds per batch of the long-run path; two batches alternate

template <int G, bool BUF, bool U24>
__device__ __forceinline__ void spmm_long_runs(const SpmmArgs &a, const FeatRows<BUF, U24> &feat, int wave, int n_waves,
                                               int lane, uint32_t lane_bytes, float *lds, int tile) {
  constexpr int NG = kWaveSize / G;   // nonzeros per round
  constexpr int TW = 4 * G;           // floats per tile
  constexpr int R = kLongRounds;
  constexpr int BLK = 256;            // nonzeros per block of ids: lane l holds ids l, 64 + l, 128 + l, 192 + l
  constexpr int NB = BLK / NG / R;    // batches per block
  const int g = lane / G;
  const int64_t F = a.F;
  const bool carry = a.accumulate != 0;
  const int f1 = (a.tile_base + tile) * TW + lane;  // the float this lane sums
  const bool owner = lane < TW && f1 < a.F;

  int vo = 0;  // from a nonzero's place in the id array to its place in the value array
  auto load_ids = [&](int e, int rem, Ids &d) {
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      d.c[q] = 0;
      d.v[q] = 0.0f;
      if (64 * q + lane < rem) {
        d.c[q] = a.indices[e + 64 * q + lane];
        d.v[q] = a.w[e + vo + 64 * q + lane];
      }
    }
  };
  // round t of a block covers its nonzeros NG*t .. NG*t + NG - 1, one per group
  auto issue = [&](float4(&x)[R], auto b, const Ids &d, int cnt) {
    static_for(std::make_integer_sequence<int, R>{}, [&](auto r) {
      constexpr int t = decltype(b)::value * R + decltype(r)::value;
      constexpr int q = NG * t / 64, l0 = NG * t % 64;
      if (decltype(r)::value == 0 || NG * t < cnt) {
        const int c = __builtin_amdgcn_ds_bpermute((l0 + g) << 2, d.c[q]);  // past the run's end: id 0, never added
        x[r] = feat.load(c, lane_bytes);
      }
    });
  };
  auto consume = [&](const float4(&x)[R], auto b, const Ids &d, int cnt, float &acc) {
    static_for(std::make_integer_sequence<int, R>{}, [&](auto r) {
      constexpr int t = decltype(b)::value * R + decltype(r)::value;
      constexpr int q = NG * t / 64, l0 = NG * t % 64;
      if (NG * t < cnt) {
        const float v = __int_as_float(__builtin_amdgcn_ds_bpermute((l0 + g) << 2, __float_as_int(d.v[q])));
        // lane (g, gl) holds floats 4*gl .. 4*gl+3 of nonzero g: float index g*TW + 4*gl = 4*lane
        *reinterpret_cast<float4 *>(lds + decltype(r)::value * 256 + 4 * lane) =
            make_float4(v * x[r].x, v * x[r].y, v * x[r].z, v * x[r].w);
      }
    });
    // The products were stored with one lane mapping and are read back with another.  LDS serves a wave's
    // accesses in order; the fence and the barrier keep the compiler from moving the reads above the stores.
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    if (lane < TW) {
      static_for(std::make_integer_sequence<int, R>{}, [&](auto r) {
        constexpr int t = decltype(b)::value * R + decltype(r)::value;
#pragma unroll
        for (int h = 0; h < NG; ++h)
          if (NG * t + h < cnt) acc = acc + lds[decltype(r)::value * 256 + h * TW + lane];  // wave-uniform test
      });
    }
    // ... and the next batch's stores below these reads
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    __builtin_amdgcn_wave_barrier();
  };

  for (int it = wave; it < a.long_runs; it += n_waves) {
    const int4 rec = a.runs[it];
    const int lo = rec.x, hi = rec.y, row = rec.z;
    if (hi <= lo) continue;
    vo = a.vals_by_csr ? rec.w - rec.x : 0;
    float acc = 0.0f;
    float4 xa[R], xb[R];
    Ids ids_a;
    load_ids(lo, hi - lo, ids_a);
    if (carry && owner) acc = a.out[static_cast<int64_t>(row) * F + f1];
    issue(xa, std::integral_constant<int, 0>{}, ids_a, min(BLK, hi - lo));
    for (int e = lo; e < hi; e += BLK) {
      const int cnt = min(BLK, hi - e);
      const bool more = hi - e > BLK;
      Ids ids_n;
      load_ids(e + BLK, hi - e - BLK, ids_n);  // the next block's ids, behind this block's first gathers
      static_for(std::make_integer_sequence<int, NB>{}, [&](auto b) {
        constexpr int bi = decltype(b)::value;
        float4(&xc)[R] = (bi & 1) ? xb : xa;
        float4(&xn)[R] = (bi & 1) ? xa : xb;
        if constexpr (bi + 1 < NB) {
          if (NG * R * (bi + 1) < cnt) issue(xn, std::integral_constant<int, bi + 1>{}, ids_a, cnt);
        } else {
          if (more) issue(xn, std::integral_constant<int, 0>{}, ids_n, hi - e - BLK);  // NB is even: xn is xa again
        }
        if (NG * R * bi < cnt) consume(xc, b, ids_a, cnt, acc);
      });
      ids_a = ids_n;
    }
    if (owner) a.out[static_cast<int64_t>(row) * F + f1] = acc;
  }
}

template <int G, bool BUF, bool U24>
__global__ __launch_bounds__(kBlockThreads) void spmm_multi_kernel(const SpmmArgs a) {
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
  const int f0 = (a.tile_base + tile) * TW + gl * 4;
  const bool fok = f0 < a.F;  // F is a multiple of 4: a lane's four floats exist together
  const int64_t F = a.F;
  const uint32_t lane_bytes = static_cast<uint32_t>(fok ? f0 : a.F - 4) * 4u;
  const FeatRows<BUF, U24> feat(a.feat, a.n_cols, F);
  const bool carry = a.accumulate != 0;
  // the first workgroups take the long runs (the records come by descending length), one wave per run
  if (bx < a.long_blocks) {
    __shared__ float products[kWavesPerBlock][kLongRounds * 256];  // per wave: a batch of rounds x 64 lanes x float4
    spmm_long_runs<G>(a, feat, static_cast<int>(bx * kWavesPerBlock + (threadIdx.x >> 6)),
                      a.long_blocks * kWavesPerBlock, lane, lane_bytes, products[threadIdx.x >> 6], tile);
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
    if (k0 + 3 < rem) {
      const Int4U ci = *reinterpret_cast<const Int4U *>(a.indices + e + k0);
      const Float4U vi = *reinterpret_cast<const Float4U *>(a.w + e + vo + k0);
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
          d.v[k] = a.w[e + vo + k0 + k];
        }
    }
  };
  auto first_ids = [&](int lo, int hi, int row, int vo, Ids &d, float4 &acc) {
    load_ids(lo, hi - lo, vo, d);
    acc = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
    if (carry && hi > lo && fok) acc = *reinterpret_cast<const float4 *>(a.out + static_cast<int64_t>(row) * F + f0);
  };

  int lo_a, hi_a, row_a, vo_a, lo_b, hi_b, row_b, vo_b;
  Ids ids_a;
  float4 acc_a;
  bounds(item, lo_a, hi_a, row_a, vo_a);
  first_ids(lo_a, hi_a, row_a, vo_a, ids_a, acc_a);
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
            if (!next_asked) first_ids(lo_b, hi_b, row_b, vo_b, ids_b, acc_b);
            next_asked = true;
            load_ids(e + B, rem - B, vo_a, ids_n);
          }
          static_for(std::make_integer_sequence<int, SC>{}, [&](auto u) {
            constexpr int l = l0 + decltype(u)::value;
            if (__builtin_amdgcn_ballot_w64(rem >= 4 * l + 4) == ~0ull) {  // every group has these four nonzeros
#pragma unroll
              for (int k = 0; k < 4; ++k)
                axpy4(acc_a, __int_as_float(group_bcast<G, l>(__float_as_int(ids_a.v[k]), hi_half)),
                      x[4 * decltype(u)::value + k]);
            } else if (decltype(u)::value == 0 || __builtin_amdgcn_ballot_w64(rem > 4 * l) != 0) {
#pragma unroll
              for (int k = 0; k < 4; ++k) {
                const float v = __int_as_float(group_bcast<G, l>(__float_as_int(ids_a.v[k]), hi_half));
                if (4 * l + k < rem) axpy4(acc_a, v, x[4 * decltype(u)::value + k]);
              }
            }
          });
        }
      });
      ids_a = ids_n;
      e += B;
      rem -= B;
    }
    if (!next_asked) first_ids(lo_b, hi_b, row_b, vo_b, ids_b, acc_b);  // no group had a nonzero here
    if (fok && row_a >= 0 && (hi_a > lo_a || !carry))
      *reinterpret_cast<float4 *>(a.out + static_cast<int64_t>(row_a) * F + f0) = acc_a;

    lo_a = lo_b;
    hi_a = hi_b;
    row_a = row_b;
    vo_a = vo_b;
    ids_a = ids_b;
    acc_a = acc_b;
    lo_b = lo_c;
    hi_b = hi_c;
    row_b = row_c;
    vo_b = vo_c;
    item += n_waves;
  }
}

template <int G>
int launch_multi(const SpmmArgs &a, int64_t blocks, bool buf, bool u24, hipStream_t stream) {
  constexpr int NG = kWaveSize / G;
  const int64_t n_items = (static_cast<int64_t>(a.n_rows) - a.long_runs + NG - 1) / NG;
  blocks = std::max<int64_t>(1, std::min<int64_t>(blocks, (n_items + kWavesPerBlock - 1) / kWavesPerBlock));
  const int il = std::max(a.interleave_tiles, 1);
  if (a.n_tiles % il != 0) return fail(FG_EINVAL, "tile interleave %d does not divide %d tiles", il, a.n_tiles);
  const dim3 grid(static_cast<unsigned>((blocks + a.long_blocks) * il), static_cast<unsigned>(a.n_tiles / il));
  if (buf && u24)
    spmm_multi_kernel<G, true, true><<<grid, dim3(kBlockThreads), 0, stream>>>(a);
  else if (buf)
    spmm_multi_kernel<G, true, false><<<grid, dim3(kBlockThreads), 0, stream>>>(a);
  else
    spmm_multi_kernel<G, false, false><<<grid, dim3(kBlockThreads), 0, stream>>>(a);
  FG_HIP_TRY(hipGetLastError());
  return FG_OK;
}

// keys[i] = length of the run of visiting position i between two bounds rows; ids[i] = i
__global__ void run_keys_kernel(const int32_t *seg_lo, const int32_t *seg_hi, int32_t n, uint32_t *keys, int32_t *ids) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) {
    keys[i] = static_cast<uint32_t>(max(seg_hi[i] - seg_lo[i], 0));
    ids[i] = i;
  }
}

__global__ void count_long_runs_kernel(const uint32_t *keys, int32_t n, uint32_t threshold, int32_t *count) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  const bool is_long = i < n && keys[i] >= threshold;
  const unsigned long long votes = __ballot(is_long);
  if ((threadIdx.x & 63) == 0 && votes) atomicAdd(count, __popcll(votes));
}

__global__ void run_records_kernel(const int32_t *seg_lo, const int32_t *seg_hi, const int32_t *row_order,
                                   const int32_t *ids_sorted, int32_t n, int4 *rec) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) {
    const int pos = ids_sorted[i];
    rec[i] = make_int4(seg_lo[pos], seg_hi[pos], row_order[pos], 0);
  }
}

// Entries that a record's run takes in the re-laid arrays: its length rounded up to a multiple of four.
__global__ void padded_lengths_kernel(const int4 *rec, int64_t n, int32_t *len) {
  const int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (i < n) len[i] = (max(rec[i].y - rec[i].x, 0) + 3) & ~3;
}

// One wave per record: copies the run's column ids to its new place and rewrites the record as
// {first, last + 1 in the new layout, row, first in the CSR arrays}.
__global__ void relay_ids_kernel(int4 *rec, const int32_t *first_p, int64_t n, const int32_t *indices, int32_t *ids_p) {
  const int lane = threadIdx.x & (kWaveSize - 1);
  const int64_t waves = static_cast<int64_t>(gridDim.x) * (blockDim.x / kWaveSize);
  for (int64_t i = static_cast<int64_t>(blockIdx.x) * (blockDim.x / kWaveSize) + threadIdx.x / kWaveSize; i < n; i += waves) {
    const int4 r = rec[i];
    const int len = max(r.y - r.x, 0), to = first_p[i];
    for (int k = lane; k < len; k += kWaveSize) ids_p[to + k] = indices[r.x + k];
    if (lane == 0) rec[i] = make_int4(to, to + len, r.z, r.x);
  }
}

// The re-laid copy of the ids for a table of several passes.  Failure to allocate leaves the table as it is.
hipError_t relay_build(const int32_t *indices, int64_t nnz, int64_t n_rec, MultiRuns *out) {
  if (nnz + 3 * n_rec >= 0x7fffffffLL) return hipSuccess;
  int32_t *len = nullptr, *first_p = nullptr;
  void *tmp = nullptr;
  size_t tmp_bytes = 0;
  int32_t last[2] = {0, 0};
  hipError_t err = hipMalloc(&len, n_rec * sizeof(int32_t));
  if (err == hipSuccess) err = hipMalloc(&first_p, n_rec * sizeof(int32_t));
  if (err == hipSuccess)
    err = hipcub::DeviceScan::ExclusiveSum(nullptr, tmp_bytes, len, first_p, static_cast<int>(n_rec), nullptr);
  if (err == hipSuccess) err = hipMalloc(&tmp, tmp_bytes ? tmp_bytes : 1);
  const unsigned grid = static_cast<unsigned>((n_rec + 255) / 256);
  if (err == hipSuccess) {
    padded_lengths_kernel<<<dim3(grid), dim3(256)>>>(out->rec, n_rec, len);
    err = hipGetLastError();
  }
  if (err == hipSuccess)
    err = hipcub::DeviceScan::ExclusiveSum(tmp, tmp_bytes, len, first_p, static_cast<int>(n_rec), nullptr);
  if (err == hipSuccess) err = hipMemcpy(&last[0], first_p + n_rec - 1, sizeof(int32_t), hipMemcpyDeviceToHost);
  if (err == hipSuccess) err = hipMemcpy(&last[1], len + n_rec - 1, sizeof(int32_t), hipMemcpyDeviceToHost);
  const int64_t total = static_cast<int64_t>(last[0]) + last[1];
  int32_t *ids_p = nullptr;
  if (err == hipSuccess) err = hipMalloc(&ids_p, std::max<int64_t>(total, 1) * sizeof(int32_t));
  if (err == hipSuccess) err = hipMemset(ids_p, 0, std::max<int64_t>(total, 1) * sizeof(int32_t));  // padding: column 0
  if (err == hipSuccess) {
    const unsigned g2 = static_cast<unsigned>(std::min<int64_t>((n_rec + 3) / 4, 65536));
    relay_ids_kernel<<<dim3(g2), dim3(256)>>>(out->rec, first_p, n_rec, indices, ids_p);
    err = hipGetLastError();
  }
  if (err == hipSuccess) err = hipDeviceSynchronize();
  if (len) (void)hipFree(len);
  if (first_p) (void)hipFree(first_p);
  if (tmp) (void)hipFree(tmp);
  if (err != hipSuccess) {
    if (ids_p) (void)hipFree(ids_p);
    return err;  // the records are rewritten only by the last kernel: on failure before it they still index the CSR arrays
  }
  out->ids_p = ids_p;
  out->relaid_n = total;
  return hipSuccess;
}

}  // namespace

int spmm_multi_tile(int32_t F) { return F <= 16 ? 16 : F <= 32 ? 32 : 64; }

void multi_runs_free(MultiRuns *r) {
  if (r->rec) (void)hipFree(r->rec);
  if (r->ids_p) (void)hipFree(r->ids_p);
  delete[] r->long_runs;
  *r = MultiRuns();
}

// One record {first nonzero, one past the last, row id} per (pass, row): pass p covers the column blocks
// p * merge .. p * merge + merge - 1 of the bounds table, and inside a pass the rows come by descending run
// length (ties in the table's order), so the rows that share a wave finish together.
int multi_runs_build(const int32_t *seg, const int32_t *row_order, const int32_t *indices, int64_t nnz, int32_t n_rows,
                     int32_t n_blocks, int32_t merge, MultiRuns *out) {
  *out = MultiRuns();
  if (n_rows == 0 || n_blocks < 1) return FG_OK;
  merge = std::max(1, std::min(merge, n_blocks));
  const int passes = (n_blocks + merge - 1) / merge;
  const size_t n = static_cast<size_t>(n_rows);
  const uint32_t long_run = config().spmm_multi_long > 0 ? static_cast<uint32_t>(config().spmm_multi_long) : kLongRun;
  uint32_t *keys = nullptr, *keys_sorted = nullptr;
  int32_t *ids = nullptr, *ids_sorted = nullptr, *counts = nullptr;
  void *tmp = nullptr;
  size_t tmp_bytes = 0;
  out->long_runs = new (std::nothrow) int32_t[passes]();
  if (!out->long_runs) return fail(FG_ENOMEM, "host allocation for %d passes failed", passes);
  hipError_t err = hipMalloc(&out->rec, n * passes * sizeof(int4));
  if (err == hipSuccess) err = hipMalloc(&counts, passes * sizeof(int32_t));
  if (err == hipSuccess) err = hipMemset(counts, 0, passes * sizeof(int32_t));
  if (err == hipSuccess) err = hipMalloc(&keys, n * sizeof(uint32_t));
  if (err == hipSuccess) err = hipMalloc(&keys_sorted, n * sizeof(uint32_t));
  if (err == hipSuccess) err = hipMalloc(&ids, n * sizeof(int32_t));
  if (err == hipSuccess) err = hipMalloc(&ids_sorted, n * sizeof(int32_t));
  if (err == hipSuccess)
    err = hipcub::DeviceRadixSort::SortPairsDescending(nullptr, tmp_bytes, keys, keys_sorted, ids, ids_sorted,
                                                       static_cast<int>(n_rows), 0, 32, nullptr);
  if (err == hipSuccess) err = hipMalloc(&tmp, tmp_bytes ? tmp_bytes : 1);
  const unsigned grid = static_cast<unsigned>((n_rows + 255) / 256);
  for (int p = 0; p < passes && err == hipSuccess; ++p) {
    const int32_t *lo = seg + static_cast<int64_t>(p) * merge * n_rows;
    const int32_t *hi = seg + static_cast<int64_t>(std::min((p + 1) * merge, n_blocks)) * n_rows;
    run_keys_kernel<<<dim3(grid), dim3(256)>>>(lo, hi, n_rows, keys, ids);
    count_long_runs_kernel<<<dim3(grid), dim3(256)>>>(keys, n_rows, long_run, counts + p);
    err = hipGetLastError();
    if (err == hipSuccess)  // LSD radix sort: stable
      err = hipcub::DeviceRadixSort::SortPairsDescending(tmp, tmp_bytes, keys, keys_sorted, ids, ids_sorted,
                                                         static_cast<int>(n_rows), 0, 32, nullptr);
    if (err == hipSuccess) {
      run_records_kernel<<<dim3(grid), dim3(256)>>>(lo, hi, row_order, ids_sorted, n_rows, out->rec + p * n);
      err = hipGetLastError();
    }
  }
  if (err == hipSuccess) err = hipDeviceSynchronize();
  if (err == hipSuccess) err = hipMemcpy(out->long_runs, counts, passes * sizeof(int32_t), hipMemcpyDeviceToHost);
  if (keys) (void)hipFree(keys);
  if (keys_sorted) (void)hipFree(keys_sorted);
  if (ids) (void)hipFree(ids);
  if (ids_sorted) (void)hipFree(ids_sorted);
  if (counts) (void)hipFree(counts);
  if (tmp) (void)hipFree(tmp);
  if (err != hipSuccess) {
    multi_runs_free(out);
    if (err == hipErrorOutOfMemory) {  // no room for the records: the wave-per-row kernels still work
      (void)hipGetLastError();
      return FG_OK;
    }
    return fail(FG_EHIP, "SpMM run records: %s", hipGetErrorString(err));
  }
  out->merge = merge;
  out->passes = passes;
  if (passes >= 2 && indices && config().spmm_relay != 0) {
    const hipError_t e2 = relay_build(indices, nnz, static_cast<int64_t>(passes) * n_rows, out);
    if (e2 == hipErrorOutOfMemory) {
      (void)hipGetLastError();
    } else if (e2 != hipSuccess) {
      multi_runs_free(out);
      return fail(FG_EHIP, "SpMM re-laid column ids: %s", hipGetErrorString(e2));
    }
  }
  return FG_OK;
}

bool spmm_multi_applies(const SpmmArgs &a) {
  return a.H == 1 && a.F % 4 == 0 && a.F >= 4 && aligned_to(a.feat, 16) && aligned_to(a.out, 16);
}

// a.n_tiles tiles of spmm_multi_tile(a.F) floats starting at tile a.tile_base (grid.y); a.runs: one pass's records.
int spmm_multi_launch(const SpmmArgs &a, hipStream_t stream) {
  if (a.n_rows == 0 || a.n_tiles == 0) return FG_OK;
  if (!spmm_multi_applies(a) || !a.runs)
    return fail(FG_EINVAL, "the several-rows-per-wave SpMM kernel does not take this call");
  const int64_t blocks = config().spmm_multi_blocks > 0 ? config().spmm_multi_blocks : 8192;
  if (a.long_runs < 0 || a.long_runs > a.n_rows || a.long_blocks < 0 || (a.long_runs > 0) != (a.long_blocks > 0))
    return fail(FG_EINVAL, "inconsistent long-run split (%d runs, %d workgroups)", a.long_runs, a.long_blocks);
  const bool buf = static_cast<int64_t>(a.n_cols) * a.F * 4 < (int64_t{1} << 32) && config().spmm_buffer_loads != 0;
  const bool u24 = a.n_cols <= (1 << 24) && static_cast<int64_t>(a.F) * 4 < (1 << 24);
  switch (spmm_multi_tile(a.F)) {
    case 16: return launch_multi<4>(a, blocks, buf, u24, stream);
    case 32: return launch_multi<8>(a, blocks, buf, u24, stream);
    default: return launch_multi<16>(a, blocks, buf, u24, stream);
  }
}

}  // namespace fg
