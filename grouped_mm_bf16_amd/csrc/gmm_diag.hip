// Diagnostics that put the measured throughput of the grouped kernels into context.
//
// gmm_diag_mfma_rate: a register-only loop of independent v_mfma_f32_32x32x16_bf16 (16 accumulator blocks
// per wave, 4 A and 4 B fragments, no memory traffic inside the loop).  Its rate is what the matrix pipe of
// the part sustains for the operand VALUES it is given: the clock follows the power of the multipliers, so
// random operands run slower than zeros.  The published peak assumes the maximum clock.
#include <hip/hip_runtime.h>
#include <stdint.h>
#include "../../include/grouped_mm_hip.h"

namespace {

typedef __bf16 diag_bf16x8 __attribute__((ext_vector_type(8)));
typedef float diag_f32x16 __attribute__((ext_vector_type(16)));

__global__ void __launch_bounds__(256) diag_mfma_kernel(const diag_bf16x8* __restrict__ frags, int nfrags, float* __restrict__ out,
                                                        int iters) {
  diag_bf16x8 a[4], b[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    a[i] = frags[(threadIdx.x * 8 + i) % nfrags];
    b[i] = frags[(threadIdx.x * 8 + 4 + i) % nfrags];
  }
  diag_f32x16 c[16];
#pragma unroll
  for (int i = 0; i < 16; ++i) c[i] = diag_f32x16{0};
  for (int it = 0; it < iters; ++it) {
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
      for (int j = 0; j < 4; ++j) c[i * 4 + j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[i], b[j], c[i * 4 + j], 0, 0, 0);
  }
  float r = 0;
#pragma unroll
  for (int i = 0; i < 16; ++i) r += c[i][i];
  out[blockIdx.x * 256 + threadIdx.x] = r;
}

}  // namespace

extern "C" int gmm_diag_mfma_rate(const void* frags, int64_t frag_bytes, void* out, int64_t out_bytes, int32_t waves_per_simd,
                                  int32_t iters, int32_t* blocks_out, void* stream) {
  if (!frags || !out || !blocks_out || frag_bytes < 16 || iters <= 0 || waves_per_simd < 1 || waves_per_simd > 2) return GMM_ERR_BAD_ARGUMENT;
  int dev = 0, cus = 0;
  if (hipGetDevice(&dev) != hipSuccess) return GMM_ERR_LAUNCH;
  if (hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus <= 0) return GMM_ERR_LAUNCH;
  const int blocks = cus * waves_per_simd;   // 4 waves per block: one or two waves on every SIMD
  *blocks_out = blocks;
  if (out_bytes < int64_t(blocks) * 256 * 4) return GMM_ERR_BAD_ARGUMENT;
  hipLaunchKernelGGL(diag_mfma_kernel, dim3(blocks), dim3(256), 0, static_cast<hipStream_t>(stream),
                     static_cast<const diag_bf16x8*>(frags), int(frag_bytes / 16), static_cast<float*>(out), iters);
  return hipGetLastError() == hipSuccess ? GMM_OK : GMM_ERR_LAUNCH;
}
