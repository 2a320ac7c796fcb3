// Device-side helpers shared by the gfx950 kernels: the per-workgroup tile
// table (prefix sum of per-group tile counts kept in LDS) and dtype conversion.
#pragma once
#include <hip/hip_runtime.h>
#include "gmm_sched.h"

// Exclusive prefix sum of per-group tile counts into cum[0..G] (LDS), returns
// the total.  All NT threads of the workgroup must call it; it ends with a
// barrier.  For 3D x 3D there is no table: every group has the same grid.
template <int NT>
__device__ __forceinline__ int gmm_build_tile_table(const GmmParams& p, int bm, int bn, int32_t* cum) {
  const int tid = threadIdx.x;
  if (p.jag == GMM_JAG_NONE) return p.G * gmm_cdiv(p.M, bm) * gmm_cdiv(p.N, bn);

  const int extent = p.jag == GMM_JAG_M ? p.M : (p.jag == GMM_JAG_N ? p.N : p.K);
  for (int g = tid; g < GMM_MAX_GROUPS; g += NT) {
    int cnt = 0;
    if (g < p.G) {
      int lo, hi, tm, tn;
      gmm_group_range(p.offs, g, extent, lo, hi);
      gmm_group_grid(p.jag, lo, hi, p.M, p.N, bm, bn, p.align, tm, tn);
      cnt = tm * tn;
    }
    cum[g + 1] = cnt;
  }
  if (tid == 0) cum[0] = 0;
  __syncthreads();
  if (tid < 64) {
    // lane l owns entries 1 + 16 l .. 16 + 16 l
    constexpr int PER = GMM_MAX_GROUPS / 64;
    int v[PER];
    int run = 0;
#pragma unroll
    for (int i = 0; i < PER; ++i) { run += cum[1 + tid * PER + i]; v[i] = run; }
    int incl = run;
#pragma unroll
    for (int d = 1; d < 64; d <<= 1) {
      const int up = __shfl_up(incl, d, 64);
      if (tid >= d) incl += up;
    }
    const int before = incl - run;
#pragma unroll
    for (int i = 0; i < PER; ++i) cum[1 + tid * PER + i] = v[i] + before;
  }
  __syncthreads();
  return cum[p.G];
}

// Linear tile id -> tile, using the table above.
__device__ __forceinline__ GmmTile gmm_locate_tile(const GmmParams& p, const int32_t* cum, int t, int bm, int bn) {
  int g, local, lo = 0, hi = 0, tm, tn;
  if (p.jag == GMM_JAG_NONE) {
    tm = gmm_cdiv(p.M, bm);
    tn = gmm_cdiv(p.N, bn);
    g = t / (tm * tn);
    local = t - g * (tm * tn);
  } else {
    const int extent = p.jag == GMM_JAG_M ? p.M : (p.jag == GMM_JAG_N ? p.N : p.K);
    g = gmm_find_group(cum, p.G, t);
    local = t - cum[g];
    gmm_group_range(p.offs, g, extent, lo, hi);
    g = __builtin_amdgcn_readfirstlane(g);
    local = __builtin_amdgcn_readfirstlane(local);
    lo = __builtin_amdgcn_readfirstlane(lo);
    hi = __builtin_amdgcn_readfirstlane(hi);
    gmm_group_grid(p.jag, lo, hi, p.M, p.N, bm, bn, p.align, tm, tn);
  }
  int mt, nt;
  gmm_decode_in_group(local, tm, tn, mt, nt);
  return gmm_make_tile(p, g, lo, hi, mt, nt, bm, bn);
}

// ---- two-height tile list (gmm_sched.h): tables cum[0] (tall) and cum[1] (short), each G + 1 entries ---- //
template <int NT>
__device__ __forceinline__ void gmm_scan_table(int32_t* cum) {
  const int tid = threadIdx.x;
  if (tid < 64) {
    constexpr int PER = GMM_MAX_GROUPS / 64;
    int v[PER];
    int run = 0;
#pragma unroll
    for (int i = 0; i < PER; ++i) { run += cum[1 + tid * PER + i]; v[i] = run; }
    int incl = run;
#pragma unroll
    for (int d = 1; d < 64; d <<= 1) {
      const int up = __shfl_up(incl, d, 64);
      if (tid >= d) incl += up;
    }
    const int before = incl - run;
#pragma unroll
    for (int i = 0; i < PER; ++i) cum[1 + tid * PER + i] = v[i] + before;
  }
}

// Returns the total number of tiles; total_tall gets the number of tall ones (they come first in the launch
// order: the workgroups of all XCDs then work on tiles of one height in every round and stay in step, which
// keeps the operand panels they share in the Infinity Cache).
template <int NT>
__device__ __forceinline__ int gmm_build_tile_table2(const GmmParams& p, int bn, int32_t* cum_tall, int32_t* cum_short,
                                                     int& total_tall) {
  const int tid = threadIdx.x;
  if (p.jag == GMM_JAG_NONE) {
    const int tn = gmm_cdiv(p.N, bn);
    int n_tall, n_short, rem_rows;
    gmm_split_rows(p.M, p.tall, p.shrt, n_tall, n_short, rem_rows);
    total_tall = p.G * n_tall * tn;
    return total_tall + p.G * n_short * tn;
  }
  const int extent = p.jag == GMM_JAG_M ? p.M : (p.jag == GMM_JAG_N ? p.N : p.K);
  for (int g = tid; g < GMM_MAX_GROUPS; g += NT) {
    int ct = 0, cs = 0;
    if (g < p.G) {
      int lo, hi, n_tall, n_short, rem_rows;
      gmm_group_range(p.offs, g, extent, lo, hi);
      gmm_split_rows(gmm_group_rows(p.jag, lo, hi, p.M, p.align), p.tall, p.shrt, n_tall, n_short, rem_rows);
      const int tn = gmm_group_tile_cols(p.jag, lo, hi, p.N, p.align, bn);
      ct = n_tall * tn;
      cs = n_short * tn;
    }
    cum_tall[g + 1] = p.group_major ? ct + cs : ct;
    cum_short[g + 1] = p.group_major ? 0 : cs;
  }
  if (tid == 0) { cum_tall[0] = 0; cum_short[0] = 0; }
  __syncthreads();
  gmm_scan_table<NT>(cum_tall);
  gmm_scan_table<NT>(cum_short);
  __syncthreads();
  total_tall = cum_tall[p.G];
  return total_tall + cum_short[p.G];   // group-major order: everything is in the first table
}

// Tile id -> tile, per lane (ids differ between lanes).
__device__ __forceinline__ GmmTile gmm_locate_tile2(const GmmParams& p, const int32_t* cum_tall, const int32_t* cum_short,
                                                    int total_tall, int t, int bn) {
  int cls = t < total_tall ? 0 : 1;
  const int tc = cls ? t - total_tall : t;
  int g, local, lo = 0, hi = 0;
  if (p.group_major && p.jag != GMM_JAG_NONE) {
    // one table: a group's tall tiles, then its remainder tiles
    g = gmm_find_group(cum_tall, p.G, t);
    local = t - cum_tall[g];
    gmm_group_range(p.offs, g, p.jag == GMM_JAG_M ? p.M : (p.jag == GMM_JAG_N ? p.N : p.K), lo, hi);
    int n_tall, n_short, rem_rows;
    gmm_split_rows(gmm_group_rows(p.jag, lo, hi, p.M, p.align), p.tall, p.shrt, n_tall, n_short, rem_rows);
    const int tall_tiles = n_tall * gmm_group_tile_cols(p.jag, lo, hi, p.N, p.align, bn);
    cls = local < tall_tiles ? 0 : 1;
    if (cls) local -= tall_tiles;
  } else if (p.jag == GMM_JAG_NONE) {
    int n_tall, n_short, rem_rows;
    gmm_split_rows(p.M, p.tall, p.shrt, n_tall, n_short, rem_rows);
    const int per = (cls ? n_short : n_tall) * gmm_cdiv(p.N, bn);
    g = tc / per;
    local = tc - g * per;
  } else {
    const int32_t* cum = cls ? cum_short : cum_tall;
    g = gmm_find_group(cum, p.G, tc);
    local = tc - cum[g];
    gmm_group_range(p.offs, g, p.jag == GMM_JAG_M ? p.M : (p.jag == GMM_JAG_N ? p.N : p.K), lo, hi);
  }
  return gmm_make_tile2(p, g, lo, hi, cls, local, bn);
}

// Source row of product row m under a row gather; -1 if the index is outside the source matrix.
__device__ __forceinline__ int gmm_gather_row(const GmmParams& p, int m) {
  const int s = p.gather[m];
  return (s >= 0 && s < p.a_rows) ? s : -1;
}

// ---- element types -------------------------------------------------------- //
struct gmm_bf16 { uint16_t bits; };
struct gmm_f16 { _Float16 v; };

__device__ __forceinline__ float gmm_to_float(gmm_bf16 x) { return __uint_as_float(uint32_t(x.bits) << 16); }
__device__ __forceinline__ float gmm_to_float(gmm_f16 x) { return float(x.v); }
__device__ __forceinline__ float gmm_to_float(float x) { return x; }

// fp32 -> bf16 bits, round to nearest even, NaN stays NaN.
__device__ __forceinline__ uint16_t gmm_bf16_bits(float f) {
  uint32_t u = __float_as_uint(f);
  if ((u & 0x7fffffffu) > 0x7f800000u) return uint16_t((u >> 16) | 0x0040u);
  u += 0x7fffu + ((u >> 16) & 1u);
  return uint16_t(u >> 16);
}

template <typename T> __device__ __forceinline__ T gmm_from_float(float f);
template <> __device__ __forceinline__ gmm_bf16 gmm_from_float<gmm_bf16>(float f) { return gmm_bf16{gmm_bf16_bits(f)}; }
template <> __device__ __forceinline__ gmm_f16 gmm_from_float<gmm_f16>(float f) { return gmm_f16{_Float16(f)}; }
template <> __device__ __forceinline__ float gmm_from_float<float>(float f) { return f; }
