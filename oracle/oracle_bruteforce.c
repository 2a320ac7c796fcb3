/* Brute-force CPU restatement of grouped_mm: TEST INFRASTRUCTURE ONLY.
 *
 * Element-ownership form, one output element at a time with an fp64 sum.  It is
 * written differently from grouped_mm_oracle.py (which loops over groups and
 * calls a library matmul) on purpose, so that an indexing mistake in either one
 * shows up when tests/test_oracle.py compares them.
 *
 * Reference behaviour followed (paths relative to the reference tree):
 *   upper bound ............ grouped_mm_bf16/kernels.py:162-172
 *   2D x 3D row ownership .. grouped_mm_bf16/kernels.py:335-360, 392-419
 *   3D x 3D ................ grouped_mm_bf16/kernels.py:224-245
 *   2D x 2D K segment ...... grouped_mm_bf16/kernels.py:276-301 (zeros when empty)
 *   3D x 2D col ownership .. grouped_mm_bf16/kernels.py:502-521
 * Inputs are dense row-major fp32 arrays (the test converts bf16 -> fp32, which
 * is exact); outputs are fp64 so the caller rounds once.  Elements no group owns
 * are left untouched.
 */
#include <stdint.h>
#include <string.h>

int oracle_upper_bound(const int32_t *offs, int G, int idx) {
  int lo = 0, hi = G;
  while (lo < hi) {
    int mid = (lo + hi) / 2;
    if (idx < offs[mid]) hi = mid; else lo = mid + 1;
  }
  return lo;
}

/* fp32 -> bf16 bits, round to nearest even, NaN kept quiet. */
uint16_t oracle_f32_to_bf16_bits(float f) {
  uint32_t u;
  memcpy(&u, &f, 4);
  if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x0040u);
  u += 0x7fffu + ((u >> 16) & 1u);
  return (uint16_t)(u >> 16);
}

/* A [Mt,K], B [G,K,N], out [Mt,N] */
void oracle_2d3d(const float *a, const float *b, double *out, const int32_t *offs,
                 int G, int Mt, int N, int K) {
  for (int m = 0; m < Mt; ++m) {
    int g = oracle_upper_bound(offs, G, m);
    if (g >= G) continue;
    for (int n = 0; n < N; ++n) {
      double s = 0.0;
      for (int k = 0; k < K; ++k)
        s += (double)a[(size_t)m * K + k] * (double)b[((size_t)g * K + k) * N + n];
      out[(size_t)m * N + n] = s;
    }
  }
}

/* A [G,M,K], B [G,K,N], out [G,M,N] */
void oracle_3d3d(const float *a, const float *b, double *out, int G, int M, int N, int K) {
  for (int g = 0; g < G; ++g)
    for (int m = 0; m < M; ++m)
      for (int n = 0; n < N; ++n) {
        double s = 0.0;
        for (int k = 0; k < K; ++k)
          s += (double)a[((size_t)g * M + m) * K + k] * (double)b[((size_t)g * K + k) * N + n];
        out[((size_t)g * M + m) * N + n] = s;
      }
}

/* A [M,Kt], B [Kt,N], out [G,M,N]: each k contributes to the group that owns it */
void oracle_2d2d(const float *a, const float *b, double *out, const int32_t *offs,
                 int G, int M, int N, int Kt) {
  memset(out, 0, sizeof(double) * (size_t)G * M * N);
  for (int k = 0; k < Kt; ++k) {
    int g = oracle_upper_bound(offs, G, k);
    if (g >= G) continue;
    for (int m = 0; m < M; ++m)
      for (int n = 0; n < N; ++n)
        out[((size_t)g * M + m) * N + n] += (double)a[(size_t)m * Kt + k] * (double)b[(size_t)k * N + n];
  }
}

/* A [G,M,K], B [K,Nt], out [M,Nt] */
void oracle_3d2d(const float *a, const float *b, double *out, const int32_t *offs,
                 int G, int M, int Nt, int K) {
  for (int n = 0; n < Nt; ++n) {
    int g = oracle_upper_bound(offs, G, n);
    if (g >= G) continue;
    for (int m = 0; m < M; ++m) {
      double s = 0.0;
      for (int k = 0; k < K; ++k)
        s += (double)a[((size_t)g * M + m) * K + k] * (double)b[(size_t)k * Nt + n];
      out[(size_t)m * Nt + n] = s;
    }
  }
}
