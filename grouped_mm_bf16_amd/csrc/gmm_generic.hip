// Stride-generic grouped GEMM for gfx950: any row- or column-major operand,
// any alignment, bf16 / fp16 / fp32 inputs, fp32 accumulation on the vector
// ALU, output in the input dtype or fp32.  It covers everything the MFMA
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
          if (m < p.M && k < tile.k_hi) v = gmm_to_float(a[int64_t(m) * p.a_sm + int64_t(k) * p.a_sk]);
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

template <typename InT, typename OutT>
int launch(const GmmParams& p, hipStream_t stream) {
  hipLaunchKernelGGL((gmm_generic_kernel<InT, OutT>), dim3(p.num_wg), dim3(GNT), 0, stream, p);
  return hipGetLastError() == hipSuccess ? 0 : 1;
}

}  // namespace

int gmm_launch_generic(GmmParams p, int in_dtype, int out_dtype, int num_cus, hipStream_t stream) {
  p.align = 1;
  p.xcd_remap = 0;
  {
    const int64_t bound = gmm_tile_bound(p.jag, p.G, p.M, p.N, 64, 64);
    p.num_wg = int(bound < int64_t(num_cus) * 4 ? (bound < 1 ? 1 : bound) : int64_t(num_cus) * 4);
  }
  if (in_dtype == GMM_DT_BF16 && out_dtype == GMM_DT_BF16) return launch<gmm_bf16, gmm_bf16>(p, stream);
  if (in_dtype == GMM_DT_BF16 && out_dtype == GMM_DT_F32) return launch<gmm_bf16, float>(p, stream);
  if (in_dtype == GMM_DT_F16 && out_dtype == GMM_DT_F16) return launch<gmm_f16, gmm_f16>(p, stream);
  if (in_dtype == GMM_DT_F16 && out_dtype == GMM_DT_F32) return launch<gmm_f16, float>(p, stream);
  if (in_dtype == GMM_DT_F32 && out_dtype == GMM_DT_F32) return launch<float, float>(p, stream);
  return -1;
}
