// Stride-generic grouped GEMM for gfx950: any row- or column-major operand,
// any alignment, bf16 / fp16 / fp32 inputs, fp32 accumulation (on the vector
// ALU for small problems, on the matrix cores with fp32 MFMAs otherwise),
// output in the input dtype or fp32.  It covers everything the MFMA
// kernels do not take (odd leading dimensions such as K = 33, N = 29, fp16 and
// fp32 operands) and serves as the on-device cross-check for them.
//
// One kernel handles the four variants; the tile list comes from gmm_sched.h.
// Computes what grouped_mm_bf16/kernels.py:197-245, 248-301, 304-419 and 475-521
// of the reference compute, but stores only elements that the tile's own group
// owns, in a single launch.
#include "gmm_device.h"
#include "gmm_launch.h"

namespace {

constexpr int GT = 64;   // output tile edge
constexpr int GK = 16;   // contraction step
constexpr int GNT = 256; // threads

template <typename InT, typename OutT>
__global__ void __launch_bounds__(GNT) gmm_generic_kernel(const GmmParams p) {
  __shared__ int32_t cum[GMM_MAX_GROUPS + 1];
  __shared__ float sa[GK][GT + 4];
  __shared__ float sb[GK][GT + 4];

  const int tid = threadIdx.x;
  const int total = gmm_build_tile_table<GNT>(p, GT, GT, cum);
  const InT* __restrict__ A = static_cast<const InT*>(p.a);
  const InT* __restrict__ B = static_cast<const InT*>(p.b);
  OutT* __restrict__ C = static_cast<OutT*>(p.c);

  const int tx = tid & 15, ty = tid >> 4;  // 16 x 16 threads, 4 x 4 outputs each

  for (int t = blockIdx.x; t < total; t += gridDim.x) {
    const GmmTile tile = gmm_locate_tile(p, cum, t, GT, GT);
    const InT* a = A + int64_t(tile.g) * p.a_sg;
    const InT* b = B + int64_t(tile.g) * p.b_sg;
    OutT* c = C + int64_t(tile.g) * p.c_sg;

    float acc[4][4] = {};
    for (int k0 = tile.k_lo; k0 < tile.k_hi; k0 += GK) {
      // A tile: GT rows x GK, B tile: GK x GT columns; 1024 elements each, 4 per thread
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int e = tid + i * GNT;
        {
          const int r = e / GK, kk = e % GK;
          const int m = tile.m0 + r, k = k0 + kk;
          float v = 0.f;
          if (m < p.M && k < tile.k_hi) {
            const int ms = p.gather ? gmm_gather_row(p, m) : m;   // a row index out of range reads as zeros
            if (ms >= 0) v = gmm_to_float(a[int64_t(ms) * p.a_sm + int64_t(k) * p.a_sk]);
          }
          sa[kk][r] = v;
        }
        {
          const int kk = e / GT, cidx = e % GT;
          const int n = tile.n0 + cidx, k = k0 + kk;
          float v = 0.f;
          if (n < p.N && k < tile.k_hi) v = gmm_to_float(b[int64_t(k) * p.b_sk + int64_t(n) * p.b_sn]);
          sb[kk][cidx] = v;
        }
      }
      __syncthreads();
#pragma unroll
      for (int kk = 0; kk < GK; ++kk) {
        float av[4], bv[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) av[i] = sa[kk][ty * 4 + i];
#pragma unroll
        for (int j = 0; j < 4; ++j) bv[j] = sb[kk][tx * 4 + j];
#pragma unroll
        for (int i = 0; i < 4; ++i)
#pragma unroll
          for (int j = 0; j < 4; ++j) acc[i][j] = __builtin_fmaf(av[i], bv[j], acc[i][j]);
      }
      __syncthreads();
    }

#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int m = tile.m0 + ty * 4 + i;
      if (m < tile.m_lo || m >= tile.m_hi) continue;
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const int n = tile.n0 + tx * 4 + j;
        if (n < tile.n_lo || n >= tile.n_hi) continue;
        c[int64_t(m) * p.c_sm + int64_t(n) * p.c_sn] = gmm_from_float<OutT>(acc[i][j]);
      }
    }
  }
}

// ---- the same contract on the matrix cores: 128 x 128 x 16 tiles, v_mfma_f32_32x32x2_f32 ------------------ //
// Operands are widened to fp32 on their way into LDS, so products are exact fp32 products of the inputs
// whatever their type, and the accumulation is fp32 (as in the kernel above; only the order of the sum
// differs).  Used when the problem has at least one full tile; small problems keep the 64 x 64 kernel.
constexpr int WT = 128;  // output tile edge
constexpr int WP = WT + 4;

typedef float gmm_f32x16 __attribute__((ext_vector_type(16)));

// Element e (0..2047) of a 128 x 16 operand tile for this thread, chosen so that consecutive threads walk
// the operand's contiguous dimension: returns (row or column in the tile, k in the chunk).
__device__ __forceinline__ void gmm_wide_coord(int e, bool k_contiguous, int& r, int& kk) {
  if (k_contiguous) { r = e >> 4; kk = e & 15; } else { kk = e >> 7; r = e & 127; }
}

template <typename InT, typename OutT>
__global__ void __launch_bounds__(GNT) gmm_wide_kernel(const GmmParams p) {
  __shared__ int32_t cum[GMM_MAX_GROUPS + 1];
  __shared__ float sa[2][GK][WP];
  __shared__ float sb[2][GK][WP];

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = wave & 1, wn = wave >> 1;
  const int total = gmm_build_tile_table<GNT>(p, WT, WT, cum);
  const InT* __restrict__ A = static_cast<const InT*>(p.a);
  const InT* __restrict__ B = static_cast<const InT*>(p.b);
  OutT* __restrict__ C = static_cast<OutT*>(p.c);
  const bool a_kc = p.a_sk == 1, b_kc = p.b_sk == 1;

  for (int t = blockIdx.x; t < total; t += gridDim.x) {
    const GmmTile tile = gmm_locate_tile(p, cum, t, WT, WT);
    const InT* a = A + int64_t(tile.g) * p.a_sg;
    const InT* b = B + int64_t(tile.g) * p.b_sg;
    OutT* c = C + int64_t(tile.g) * p.c_sg;

    gmm_f32x16 acc[2][2];
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
      for (int j = 0; j < 2; ++j) acc[i][j] = gmm_f32x16{0};

    float ra[8], rb[8];
    auto fetch = [&](int k0) {
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        int r, kk;
        gmm_wide_coord(tid + i * GNT, a_kc, r, kk);
        const int m = tile.m0 + r, k = k0 + kk;
        int ms = m < p.M ? m : -1;
        if (p.gather && ms >= 0) ms = gmm_gather_row(p, m);
        ra[i] = (ms >= 0 && k < tile.k_hi) ? gmm_to_float(a[int64_t(ms) * p.a_sm + int64_t(k) * p.a_sk]) : 0.f;
        gmm_wide_coord(tid + i * GNT, b_kc, r, kk);
        const int n = tile.n0 + r;
        const int kb = k0 + kk;
        rb[i] = (n < p.N && kb < tile.k_hi) ? gmm_to_float(b[int64_t(kb) * p.b_sk + int64_t(n) * p.b_sn]) : 0.f;
      }
    };
    auto stash = [&](int buf) {
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        int r, kk;
        gmm_wide_coord(tid + i * GNT, a_kc, r, kk);
        sa[buf][kk][r] = ra[i];
        gmm_wide_coord(tid + i * GNT, b_kc, r, kk);
        sb[buf][kk][r] = rb[i];
      }
    };

    int buf = 0;
    if (tile.k_lo < tile.k_hi) {
      fetch(tile.k_lo);
      stash(0);
    }
    __syncthreads();
    for (int k0 = tile.k_lo; k0 < tile.k_hi; k0 += GK) {
      const bool more = k0 + GK < tile.k_hi;
      if (more) fetch(k0 + GK);   // global loads of the next chunk fly under the MFMAs of this one
#pragma unroll
      for (int k2 = 0; k2 < GK; k2 += 2) {
        const int kr = k2 + (lane >> 5), col = lane & 31;
        const float a0 = sa[buf][kr][wm * 64 + col], a1 = sa[buf][kr][wm * 64 + 32 + col];
        const float b0 = sb[buf][kr][wn * 64 + col], b1 = sb[buf][kr][wn * 64 + 32 + col];
        acc[0][0] = __builtin_amdgcn_mfma_f32_32x32x2f32(a0, b0, acc[0][0], 0, 0, 0);
        acc[0][1] = __builtin_amdgcn_mfma_f32_32x32x2f32(a0, b1, acc[0][1], 0, 0, 0);
        acc[1][0] = __builtin_amdgcn_mfma_f32_32x32x2f32(a1, b0, acc[1][0], 0, 0, 0);
        acc[1][1] = __builtin_amdgcn_mfma_f32_32x32x2f32(a1, b1, acc[1][1], 0, 0, 0);
      }
      if (more) stash(buf ^ 1);
      __syncthreads();
      buf ^= 1;
    }

    // accumulator register 4 q + r of a 32 x 32 block: row 8 q + 4 (lane / 32) + r, column lane % 32
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
      for (int j = 0; j < 2; ++j) {
        const int n = tile.n0 + wn * 64 + j * 32 + (lane & 31);
        if (n < tile.n_lo || n >= tile.n_hi) continue;
#pragma unroll
        for (int x = 0; x < 16; ++x) {
          const int m = tile.m0 + wm * 64 + i * 32 + 8 * (x >> 2) + 4 * (lane >> 5) + (x & 3);
          if (m < tile.m_lo || m >= tile.m_hi) continue;
          c[int64_t(m) * p.c_sm + int64_t(n) * p.c_sn] = gmm_from_float<OutT>(acc[i][j][x]);
        }
      }
    __syncthreads();   // the next tile's first stash must not overtake this tile's last reads
  }
}

template <typename InT, typename OutT>
int launch_wide(const GmmParams& p, hipStream_t stream) {
  hipLaunchKernelGGL((gmm_wide_kernel<InT, OutT>), dim3(p.num_wg), dim3(GNT), 0, stream, p);
  return hipGetLastError() == hipSuccess ? 0 : 1;
}

template <typename InT, typename OutT>
int launch(const GmmParams& p, hipStream_t stream) {
  hipLaunchKernelGGL((gmm_generic_kernel<InT, OutT>), dim3(p.num_wg), dim3(GNT), 0, stream, p);
  return hipGetLastError() == hipSuccess ? 0 : 1;
}

}  // namespace

int gmm_launch_generic(GmmParams p, int in_dtype, int out_dtype, int num_cus, hipStream_t stream) {
  p.align = 1;
  p.xcd_remap = 0;
  // at least one full 128 x 128 tile and a contraction worth pipelining: the matrix-core kernel
  const bool wide = p.M >= WT && p.N >= WT && p.K >= 64;
  {
    const int edge = wide ? WT : GT;
    const int64_t bound = gmm_tile_bound(p.jag, p.G, p.M, p.N, edge, edge);
    const int64_t cap = int64_t(num_cus) * (wide ? 2 : 4);
    p.num_wg = int(bound < cap ? (bound < 1 ? 1 : bound) : cap);
  }
#define GMM_GENERIC_CASE(IN_CODE, OUT_CODE, IN_T, OUT_T) \
  if (in_dtype == IN_CODE && out_dtype == OUT_CODE) return wide ? launch_wide<IN_T, OUT_T>(p, stream) : launch<IN_T, OUT_T>(p, stream);
  GMM_GENERIC_CASE(GMM_DT_BF16, GMM_DT_BF16, gmm_bf16, gmm_bf16)
  GMM_GENERIC_CASE(GMM_DT_BF16, GMM_DT_F32, gmm_bf16, float)
  GMM_GENERIC_CASE(GMM_DT_F16, GMM_DT_F16, gmm_f16, gmm_f16)
  GMM_GENERIC_CASE(GMM_DT_F16, GMM_DT_F32, gmm_f16, float)
  GMM_GENERIC_CASE(GMM_DT_F32, GMM_DT_F32, float, float)
#undef GMM_GENERIC_CASE
  return -1;
}
