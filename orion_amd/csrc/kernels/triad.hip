// Best-effort co-location kernel: fp32 streaming triad  a[i] = b[i] + s * c[i].
//
// HBM-bound: 12 algorithmic bytes per element (two 4-byte reads, one 4-byte
// write) against two flops.  Every lane moves 16 bytes per access
// (global_load_dwordx4 / global_store_dwordx4, non-temporal: nothing is reused),
// so a wavefront touches one fully coalesced 1 KiB segment per access.
//
// Default launch: one 16-byte access per lane and array and one wavefront per
// workgroup, i.e. n / 256 workgroups with no loop.  On MI355X this shape streams
// fastest -- the dispatcher keeps every CU's memory pipeline full with
// short-lived waves (measured over 3 x 1 GiB: 6.72 TB/s; 6.43 TB/s with four
// waves per workgroup, 6.4 with two accesses per lane, 4.6 for a 2048-workgroup
// grid-stride loop with four accesses in flight per lane).  A caller-chosen
// smaller grid walks block-contiguous chunks instead, so any number of compute
// units (a CU-masked stream may expose a fraction of the 256) drains it.
//
// The reference system has no device code of its own; this kernel stands in for
// the memory-bound half of its toy co-location pair
// (benchmarking/benchmark_suite/toy_models/bnorm_trainer.py:20-27).

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "kernels.h"

namespace {

constexpr int kTriadThreads = 256;  // chunked variant
constexpr int kOneShotThreads = 64; // one-shot variant: one wavefront per workgroup
// float4 accesses in flight per lane and per array in the chunked variant.
constexpr int kTriadUnroll = 4;

typedef float f32x4 __attribute__((ext_vector_type(4)));

__device__ __forceinline__ f32x4 triad4(f32x4 vb, f32x4 vc, float s) {
  f32x4 r;
  r.x = __builtin_fmaf(s, vc.x, vb.x);
  r.y = __builtin_fmaf(s, vc.y, vb.y);
  r.z = __builtin_fmaf(s, vc.z, vb.z);
  r.w = __builtin_fmaf(s, vc.w, vb.w);
  return r;
}

// Ragged tail (n not a multiple of 4): at most three scalar elements, done by
// the first lanes of workgroup 0.
__device__ __forceinline__ void triad_tail(float* a, const float* b, const float* c,
                                           float s, size_t n_vec4, size_t n) {
  if (blockIdx.x == 0) {
    const size_t tail = n_vec4 * 4 + threadIdx.x;
    if (tail < n) a[tail] = __builtin_fmaf(s, c[tail], b[tail]);
  }
}

__global__ __launch_bounds__(kOneShotThreads) void triad_f32_kernel(
    float* __restrict__ a, const float* __restrict__ b,
    const float* __restrict__ c, float s, size_t n_vec4, size_t n) {
  const size_t i = (size_t)blockIdx.x * kOneShotThreads + threadIdx.x;
  if (i < n_vec4) {
    const f32x4 vb = __builtin_nontemporal_load(reinterpret_cast<const f32x4*>(b) + i);
    const f32x4 vc = __builtin_nontemporal_load(reinterpret_cast<const f32x4*>(c) + i);
    __builtin_nontemporal_store(triad4(vb, vc, s), reinterpret_cast<f32x4*>(a) + i);
  }
  triad_tail(a, b, c, s, n_vec4, n);
}

// Caller-chosen grid: workgroup g owns the contiguous range
// [g * per_block, (g + 1) * per_block) of 16-byte elements.
__global__ __launch_bounds__(kTriadThreads) void triad_f32_chunked_kernel(
    float* __restrict__ a, const float* __restrict__ b,
    const float* __restrict__ c, float s, size_t n_vec4, size_t n) {
  const f32x4* __restrict__ b4 = reinterpret_cast<const f32x4*>(b);
  const f32x4* __restrict__ c4 = reinterpret_cast<const f32x4*>(c);
  f32x4* __restrict__ a4 = reinterpret_cast<f32x4*>(a);
  const size_t per_block = (n_vec4 + gridDim.x - 1) / gridDim.x;
  const size_t begin = (size_t)blockIdx.x * per_block;
  size_t end = begin + per_block;
  if (end > n_vec4) end = n_vec4;
  size_t i = begin + threadIdx.x;
  for (; i + (kTriadUnroll - 1) * kTriadThreads < end; i += kTriadUnroll * kTriadThreads) {
    f32x4 vb[kTriadUnroll], vc[kTriadUnroll];
#pragma unroll
    for (int u = 0; u < kTriadUnroll; ++u) {
      vb[u] = __builtin_nontemporal_load(&b4[i + u * kTriadThreads]);
      vc[u] = __builtin_nontemporal_load(&c4[i + u * kTriadThreads]);
    }
#pragma unroll
    for (int u = 0; u < kTriadUnroll; ++u)
      __builtin_nontemporal_store(triad4(vb[u], vc[u], s), &a4[i + u * kTriadThreads]);
  }
  for (; i < end; i += kTriadThreads) a4[i] = triad4(b4[i], c4[i], s);
  triad_tail(a, b, c, s, n_vec4, n);
}

}  // namespace

extern "C" int orion_triad_f32(float* a, const float* b, const float* c,
                               float s, size_t n, int grid_blocks,
                               void* stream) {
  if (n == 0) return ORION_OK;
  if (a == nullptr || b == nullptr || c == nullptr) return ORION_ERR_ARG;
  // 16-byte accesses need 16-byte aligned bases.
  if ((((uintptr_t)a | (uintptr_t)b | (uintptr_t)c) & 15u) != 0)
    return ORION_ERR_ALIGN;
  const size_t n_vec4 = n / 4;
  size_t one_shot = (n_vec4 + kOneShotThreads - 1) / kOneShotThreads;
  if (one_shot < 1) one_shot = 1;
  if (one_shot > 0x7fffffffu) return ORION_ERR_SHAPE;
  if (grid_blocks <= 0 || (size_t)grid_blocks >= one_shot) {
    hipLaunchKernelGGL(triad_f32_kernel, dim3((unsigned)one_shot), dim3(kOneShotThreads), 0,
                       (hipStream_t)stream, a, b, c, s, n_vec4, n);
  } else {
    hipLaunchKernelGGL(triad_f32_chunked_kernel, dim3((unsigned)grid_blocks),
                       dim3(kTriadThreads), 0, (hipStream_t)stream, a, b, c, s, n_vec4, n);
  }
  return hipGetLastError() == hipSuccess ? ORION_OK : ORION_ERR_LAUNCH;
}

// Stream helper for callers that hold no HIP binding of their own (the Python
// layer): a non-blocking stream spanning `cu_count` compute units (the first
// cu_count mask bits; bit i lands on XCD i % 8), or the whole GPU when
// cu_count <= 0 or covers every CU.  Default priority.
extern "C" int orion_stream_create(int cu_count, void** stream_out) {
  if (stream_out == nullptr) return ORION_ERR_ARG;
  int dev = 0, cus = 0;
  if (hipGetDevice(&dev) != hipSuccess ||
      hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess)
    return ORION_ERR_LAUNCH;
  hipStream_t s = nullptr;
  hipError_t err;
  if (cu_count <= 0 || cu_count >= cus) {
    err = hipStreamCreateWithFlags(&s, hipStreamNonBlocking);
  } else {
    uint32_t words[16] = {0};
    if (cus > 512) return ORION_ERR_ARG;
    for (int b = 0; b < cu_count; ++b) words[b / 32] |= 1u << (b % 32);
    err = hipExtStreamCreateWithCUMask(&s, (uint32_t)((cus + 31) / 32), words);
  }
  if (err != hipSuccess) return ORION_ERR_LAUNCH;
  *stream_out = (void*)s;
  return ORION_OK;
}

extern "C" int orion_stream_destroy(void* stream) {
  return hipStreamDestroy((hipStream_t)stream) == hipSuccess ? ORION_OK : ORION_ERR_LAUNCH;
}
