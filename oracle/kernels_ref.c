/* CPU oracle for the two co-location kernels.  TEST INFRASTRUCTURE ONLY: the
 * shipped package never links or loads this file.
 *
 * The reference system has no device code; its compute/memory pair is library
 * ops (benchmarking/benchmark_suite/toy_models/conv_trainer.py:20-27,
 * bnorm_trainer.py:20-27).  What fixes these functions is therefore the
 * mathematics:
 *   triad: IEEE-754 fused multiply-add, one rounding per element, so the GPU
 *          result must be bit-identical (checked against fmaf here and, in the
 *          tests, against exact rational arithmetic on small cases);
 *   gemm:  the exact product of the bf16-rounded inputs, accumulated in double
 *          (error far below fp32's), against which the fp32-accumulating kernel
 *          is held to 1e-3 of the result's RMS.
 */
#include <math.h>
#include <stddef.h>
#include <stdint.h>
#include <string.h>

void oracle_triad_f32(float* a, const float* b, const float* c, float s, size_t n) {
  for (size_t i = 0; i < n; ++i) a[i] = fmaf(s, c[i], b[i]);
}

static float bf16_to_f32(uint16_t h) {
  uint32_t u = (uint32_t)h << 16;
  float f;
  memcpy(&f, &u, sizeof f);
  return f;
}

/* round-to-nearest-even fp32 -> bf16, NaN kept quiet */
uint16_t oracle_f32_to_bf16(float f) {
  uint32_t u;
  memcpy(&u, &f, sizeof u);
  if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x40u);
  u += 0x7fffu + ((u >> 16) & 1u);
  return (uint16_t)(u >> 16);
}

/* C[M,N] = A[M,K] * B[N,K]^T over bf16 bit patterns, double accumulation,
 * rows [row_begin, row_end) only (so big shapes can be sampled). */
void oracle_gemm_bf16_nt(const uint16_t* A, const uint16_t* B, double* C, int M,
                         int N, int K, int row_begin, int row_end) {
  (void)M;
  for (int i = row_begin; i < row_end; ++i)
    for (int j = 0; j < N; ++j) {
      double acc = 0.0;
      const uint16_t* a = A + (size_t)i * K;
      const uint16_t* b = B + (size_t)j * K;
      for (int k = 0; k < K; ++k) acc += (double)bf16_to_f32(a[k]) * (double)bf16_to_f32(b[k]);
      C[(size_t)(i - row_begin) * N + j] = acc;
    }
}
