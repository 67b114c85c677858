/* C ABI of liborion_kernels.so: the hand-written gfx950 co-location kernels.
 *
 * The reference system (eth-easl/orion) ships no device code; its co-location
 * experiments pair a compute-bound library op with a memory-bound one
 * (benchmarking/benchmark_suite/toy_models/conv_trainer.py:20-27,
 * benchmarking/benchmark_suite/toy_models/bnorm_trainer.py:20-27).  These two
 * entry points are that pair as explicit kernels.  All pointers are device
 * pointers; `stream` is a hipStream_t passed as void* (NULL = null stream).
 * Every call only enqueues work and returns; the caller synchronises.
 */
#ifndef ORION_KERNELS_H_
#define ORION_KERNELS_H_

#include <stddef.h>

#ifdef __cplusplus
extern "C" {
#endif

enum orion_status {
  ORION_OK = 0,
  ORION_ERR_ARG = 1,    /* null pointer or negative size */
  ORION_ERR_SHAPE = 2,  /* shape not a multiple of the kernel's tile */
  ORION_ERR_ALIGN = 3,  /* base pointer not 16-byte aligned */
  ORION_ERR_LAUNCH = 4  /* the HIP runtime rejected the launch */
};

/* a[i] = fmaf(s, c[i], b[i]) for i in [0, n): one fused multiply-add per
 * element, so results are bit-identical to C's fmaf on the host.
 * grid_blocks <= 0 selects the default launch (one 16-byte access per lane,
 * n / 256 workgroups of one 64-lane wavefront); a smaller positive value is
 * honoured with block-contiguous chunks of 256-lane workgroups.  ORION_ERR_SHAPE if n needs more than 2^31 - 1
 * workgroups.
 * Memory-bound stand-in for bnorm_trainer.py:20-27 of the reference. */
int orion_triad_f32(float* a, const float* b, const float* c, float s,
                    size_t n, int grid_blocks, void* stream);

/* C[M,N] = A[M,K] * B[N,K]^T.  A and B hold bf16 bit patterns (uint16_t),
 * both K-contiguous (row-major A, row-major B = the weight layout of a linear
 * layer).  Accumulation is fp32 on the matrix cores; C is fp32 when
 * out_is_f32 != 0, else bf16 rounded to nearest even.  Requires M % 256 == 0,
 * N % 256 == 0, K % 64 == 0 (ORION_ERR_SHAPE otherwise).
 * Compute-bound stand-in for conv_trainer.py:20-27 of the reference. */
int orion_gemm_bf16_nt(const void* A, const void* B, void* C, int M, int N,
                       int K, int out_is_f32, void* stream);

/* A non-blocking, default-priority stream limited to the first cu_count
 * compute units of the CU mask (hipExtStreamCreateWithCUMask; mask bit i lands
 * on XCD i % 8), or spanning the whole GPU when cu_count <= 0 or >= the CU
 * count.  The reference creates its streams inside the scheduler only
 * (src/scheduler/utils_sched.cpp:119-147); this pair exists for measuring the
 * kernels on masked streams without the scheduler. */
int orion_stream_create(int cu_count, void** stream_out);
int orion_stream_destroy(void* stream);

#ifdef __cplusplus
}
#endif
#endif /* ORION_KERNELS_H_ */
