// Bench-only diagnostics, built into libgmm_diag.so (not part of the product library or its C ABI).
//
// gmm_diag_mfma_rate: a register-only loop of independent MFMAs (no memory traffic inside the loop), with the
// 128 x 128 accumulator block of a wave of the grouped kernels: shape 0 = v_mfma_f32_16x16x32_bf16 (64 blocks
// of 16 x 16, 8 A and 8 B fragments: the instruction the assembly tile uses), shape 1 =
// v_mfma_f32_32x32x16_bf16 (16 blocks of 32 x 32, 4 + 4 fragments).  Its rate is what the matrix pipe of the
// part sustains for the operand VALUES it is given: the clock follows the power drawn, so random operands run
// slower than zeros, and the 32 x 32 shape, which moves twice the accumulator data per FLOP, slower than the
// 16 x 16 one.  The published peak assumes the maximum clock.
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace {

typedef __bf16 diag_bf16x8 __attribute__((ext_vector_type(8)));
typedef float diag_f32x16 __attribute__((ext_vector_type(16)));
typedef float diag_f32x4 __attribute__((ext_vector_type(4)));

__global__ void __launch_bounds__(256) diag_mfma_32x32x16(const diag_bf16x8* __restrict__ frags, int nfrags,
                                                          float* __restrict__ out, int iters) {
  diag_bf16x8 a[4], b[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    a[i] = frags[(threadIdx.x * 16 + i) % nfrags];
    b[i] = frags[(threadIdx.x * 16 + 8 + i) % nfrags];
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
  for (int i = 0; i < 16; ++i) r += c[i][0] + c[i][15];
  out[blockIdx.x * 256 + threadIdx.x] = r;
}

// one iteration = 64 MFMAs of 16384 FLOP: twice the FLOPs of an iteration above (a k step of 32 instead of 16)
__global__ void __launch_bounds__(256) diag_mfma_16x16x32(const diag_bf16x8* __restrict__ frags, int nfrags,
                                                          float* __restrict__ out, int iters) {
  diag_bf16x8 a[8], b[8];
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    a[i] = frags[(threadIdx.x * 16 + i) % nfrags];
    b[i] = frags[(threadIdx.x * 16 + 8 + i) % nfrags];
  }
  diag_f32x4 c[64];
#pragma unroll
  for (int i = 0; i < 64; ++i) c[i] = diag_f32x4{0};
  for (int it = 0; it < iters; ++it) {
#pragma unroll
    for (int i = 0; i < 8; ++i)
#pragma unroll
      for (int j = 0; j < 8; ++j) c[i * 8 + j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[i], b[j], c[i * 8 + j], 0, 0, 0);
  }
  float r = 0;
#pragma unroll
  for (int i = 0; i < 64; ++i) r += c[i][0] + c[i][3];   // constant indices: a dynamic one would put c[] in scratch memory
  out[blockIdx.x * 256 + threadIdx.x] = r;
}

}  // namespace

// frags: device memory, frag_bytes >= 16, bf16 values of the caller's choice, 16 fragments of 8 values per
// thread (wrapping around): the first 8 feed the A operands, the last 8 the B operands.  `out` receives one
// float per thread (blocks * 256 floats); *blocks gets the number of 256-thread blocks launched (one or two
// waves on every SIMD), so that FLOP per launch = *blocks * 4 * iters * 1048576 for shape 0 and * 524288 for shape 1.  Returns 0, 1 (bad argument)
// or 2 (launch failed).
extern "C" int gmm_diag_mfma_rate(const void* frags, int64_t frag_bytes, void* out, int64_t out_bytes, int32_t waves_per_simd,
                                  int32_t iters, int32_t shape, int32_t* blocks_out, void* stream) {
  if (!frags || !out || !blocks_out || frag_bytes < 16 || iters <= 0 || waves_per_simd < 1 || waves_per_simd > 2) return 1;
  if (shape != 0 && shape != 1) return 1;
  int dev = 0, cus = 0;
  if (hipGetDevice(&dev) != hipSuccess) return 2;
  if (hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus <= 0) return 2;
  const int blocks = cus * waves_per_simd;   // 4 waves per block
  *blocks_out = blocks;
  if (out_bytes < int64_t(blocks) * 256 * 4) return 1;
  const auto kernel = shape == 0 ? diag_mfma_16x16x32 : diag_mfma_32x32x16;
  hipLaunchKernelGGL(kernel, dim3(blocks), dim3(256), 0, static_cast<hipStream_t>(stream),
                     static_cast<const diag_bf16x8*>(frags), int(frag_bytes / 16), static_cast<float*>(out), iters);
  return hipGetLastError() == hipSuccess ? 0 : 2;
}
