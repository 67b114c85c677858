// Best-effort co-location kernel: fp32 streaming triad  a[i] = b[i] + s * c[i].
//
// HBM-bound: 12 algorithmic bytes per element (two 4-byte reads, one 4-byte
// write) against two flops.  Every lane moves 16 bytes per access
// (global_load_dwordx4 / global_store_dwordx4), a wavefront therefore touches
// one fully coalesced 1 KiB segment per access, and each workgroup walks the
// arrays with a grid stride so that any number of compute units (a CU-masked
// stream may expose only a fraction of the 256) drains the same launch.
//
// The reference system has no device code of its own; this kernel stands in for
// the memory-bound half of its toy co-location pair
// (benchmarking/benchmark_suite/toy_models/bnorm_trainer.py:20-27).

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "kernels.h"

namespace {

constexpr int kTriadThreads = 256;
// float4 accesses in flight per lane and per array before the first use.
constexpr int kTriadUnroll = 4;

typedef float f32x4 __attribute__((ext_vector_type(4)));

__global__ __launch_bounds__(kTriadThreads) void triad_f32_kernel(
    float* __restrict__ a, const float* __restrict__ b,
    const float* __restrict__ c, float s, size_t n_vec4, size_t n) {
  const size_t tid = (size_t)blockIdx.x * kTriadThreads + threadIdx.x;
  const size_t nthreads = (size_t)gridDim.x * kTriadThreads;

  const f32x4* __restrict__ b4 = reinterpret_cast<const f32x4*>(b);
  const f32x4* __restrict__ c4 = reinterpret_cast<const f32x4*>(c);
  f32x4* __restrict__ a4 = reinterpret_cast<f32x4*>(a);

  size_t i = tid;
  // Main body: kTriadUnroll independent 16-byte loads per array are issued
  // before any of them is consumed, which keeps enough bytes in flight per CU
  // to cover HBM latency with few resident waves.
  for (; i + (kTriadUnroll - 1) * nthreads < n_vec4;
       i += kTriadUnroll * nthreads) {
    f32x4 vb[kTriadUnroll], vc[kTriadUnroll];
#pragma unroll
    for (int u = 0; u < kTriadUnroll; ++u) {
      vb[u] = __builtin_nontemporal_load(&b4[i + u * nthreads]);
      vc[u] = __builtin_nontemporal_load(&c4[i + u * nthreads]);
    }
#pragma unroll
    for (int u = 0; u < kTriadUnroll; ++u) {
      f32x4 r;
      r.x = __builtin_fmaf(s, vc[u].x, vb[u].x);
      r.y = __builtin_fmaf(s, vc[u].y, vb[u].y);
      r.z = __builtin_fmaf(s, vc[u].z, vb[u].z);
      r.w = __builtin_fmaf(s, vc[u].w, vb[u].w);
      __builtin_nontemporal_store(r, &a4[i + u * nthreads]);
    }
  }
  for (; i < n_vec4; i += nthreads) {
    f32x4 vb = b4[i], vc = c4[i], r;
    r.x = __builtin_fmaf(s, vc.x, vb.x);
    r.y = __builtin_fmaf(s, vc.y, vb.y);
    r.z = __builtin_fmaf(s, vc.z, vb.z);
    r.w = __builtin_fmaf(s, vc.w, vb.w);
    a4[i] = r;
  }
  // Ragged tail (n not a multiple of 4): at most three scalar elements.
  const size_t tail = n_vec4 * 4 + tid;
  if (tail < n) a[tail] = __builtin_fmaf(s, c[tail], b[tail]);
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
  if (grid_blocks <= 0) {
    // 8 workgroups per CU over 256 CUs: enough waves to hide HBM latency,
    // few enough that the grid-stride loop amortises launch and tail.
    grid_blocks = 256 * 8;
    size_t need = (n_vec4 + kTriadThreads - 1) / kTriadThreads;
    if (need < 1) need = 1;
    if ((size_t)grid_blocks > need) grid_blocks = (int)need;
  }
  hipLaunchKernelGGL(triad_f32_kernel, dim3((unsigned)grid_blocks),
                     dim3(kTriadThreads), 0, (hipStream_t)stream, a, b, c, s,
                     n_vec4, n);
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
