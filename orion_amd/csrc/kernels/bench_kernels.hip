// Native driver for the two co-location kernels, for profiler runs
// (rocprofv3 --kernel-trace / --pmc -- orion_amd/bench_kernels): it uses the
// system HIP runtime only, so a profiler sees exactly these kernels.
//
//   bench_kernels [--reps N] [--warmup N] [--gemm-n N] [--triad-elems N] [--triad-skew BYTES] [--mask CUS]
//                 [--pair 1]
//
// --pair 1 runs the two kernels at the same time instead: the GEMM on a stream
// over the whole GPU, the triad on a stream over --mask CUs, submissions
// interleaved so that neither queue runs dry (a pilot run finds how many triads
// one GEMM needs).  A kernel trace of that run gives each kernel's duration
// next to the other; hardware counters cannot, because the profiler serialises
// dispatches while it collects them.
//
// Per kernel it prints the average launch duration measured with HIP events on
// the stream the kernel runs on, and the achieved rate against its roofline.
// The GEMM holds the GPU at its power limit: after an idle period the clocks
// overshoot, dip, and settle within ~50 launches, so the timed launches follow
// --warmup untimed ones (default 100) and "burst" reports the first 20
// launches after the idle period separately.
// A plain 16-byte-per-lane copy kernel of known size runs as well: its
// FETCH_SIZE / WRITE_SIZE readings give the factor that scales the counters of
// the other kernels to bytes.
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include "orion_kernels.h"

#define CHECK(x)                                                              \
  do {                                                                        \
    hipError_t e_ = (x);                                                      \
    if (e_ != hipSuccess) {                                                   \
      fprintf(stderr, "%s:%d %s: %s\n", __FILE__, __LINE__, #x, hipGetErrorString(e_)); \
      exit(1);                                                                \
    }                                                                         \
  } while (0)

typedef float f32x4 __attribute__((ext_vector_type(4)));

// uniform(-1, 1) from a counter hash; fp32 or bf16 (upper half) output
__global__ void init_uniform(uint32_t* out, size_t n, uint32_t seed, int as_bf16_pairs) {
  size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  size_t stride = (size_t)gridDim.x * blockDim.x;
  for (; i < n; i += stride) {
    uint32_t x = (uint32_t)i * 2654435761u + seed;
    x ^= x >> 16; x *= 0x7feb352du; x ^= x >> 15; x *= 0x846ca68bu; x ^= x >> 16;
    float f = (float)(x >> 8) * (2.0f / 16777216.0f) - 1.0f;
    uint32_t bits = __builtin_bit_cast(uint32_t, f);
    if (as_bf16_pairs) {
      uint32_t y = x * 747796405u + 2891336453u;
      float g = (float)(y >> 8) * (2.0f / 16777216.0f) - 1.0f;
      out[i] = (bits >> 16) | (__builtin_bit_cast(uint32_t, g) & 0xffff0000u);
    } else {
      out[i] = bits;
    }
  }
}

__global__ __launch_bounds__(256) void copy_f32x4_kernel(f32x4* __restrict__ dst,
                                                         const f32x4* __restrict__ src,
                                                         size_t n_vec4) {
  size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
  size_t stride = (size_t)gridDim.x * 256;
  for (; i < n_vec4; i += stride) dst[i] = src[i];
}

static float time_ms(hipStream_t s, int reps, int warmup, void (*launch)(hipStream_t, void*), void* ctx) {
  hipEvent_t a, b;
  CHECK(hipEventCreate(&a));
  CHECK(hipEventCreate(&b));
  for (int i = 0; i < warmup; ++i) launch(s, ctx);
  CHECK(hipEventRecord(a, s));
  for (int i = 0; i < reps; ++i) launch(s, ctx);
  CHECK(hipEventRecord(b, s));
  CHECK(hipEventSynchronize(b));
  float ms = 0;
  CHECK(hipEventElapsedTime(&ms, a, b));
  CHECK(hipEventDestroy(a));
  CHECK(hipEventDestroy(b));
  return ms / reps;
}

struct GemmCtx { void *A, *B, *C; int n; };
struct TriadCtx { float *a, *b, *c; size_t n; };

static void launch_gemm(hipStream_t s, void* p) {
  GemmCtx* g = (GemmCtx*)p;
  if (orion_gemm_bf16_nt(g->A, g->B, g->C, g->n, g->n, g->n, 0, s) != ORION_OK) exit(2);
}
static void launch_triad(hipStream_t s, void* p) {
  TriadCtx* t = (TriadCtx*)p;
  if (orion_triad_f32(t->a, t->b, t->c, 1.7f, t->n, 0, s) != ORION_OK) exit(2);
}
static void launch_copy(hipStream_t s, void* p) {
  TriadCtx* t = (TriadCtx*)p;
  hipLaunchKernelGGL(copy_f32x4_kernel, dim3(2048), dim3(256), 0, s, (f32x4*)t->a,
                     (const f32x4*)t->b, t->n / 4);
}

// Both kernels at once; returns average ms per launch of each.
static void run_pair(hipStream_t sg, hipStream_t st, GemmCtx* g, TriadCtx* t, int n_gemm,
                     int n_triad, float* gemm_ms, float* triad_ms) {
  hipEvent_t e[4];
  for (auto& x : e) CHECK(hipEventCreate(&x));
  for (int i = 0; i < 3; ++i) launch_triad(st, t);  // the other stream is busy first
  CHECK(hipEventRecord(e[0], sg));
  CHECK(hipEventRecord(e[2], st));
  int done_t = 0;
  for (int i = 0; i < n_gemm; ++i) {
    launch_gemm(sg, g);
    const int want = (int)((long long)(i + 1) * n_triad / n_gemm);
    for (; done_t < want; ++done_t) launch_triad(st, t);
  }
  CHECK(hipEventRecord(e[1], sg));
  CHECK(hipEventRecord(e[3], st));
  CHECK(hipEventSynchronize(e[1]));
  CHECK(hipEventSynchronize(e[3]));
  CHECK(hipEventElapsedTime(gemm_ms, e[0], e[1]));
  CHECK(hipEventElapsedTime(triad_ms, e[2], e[3]));
  *gemm_ms /= n_gemm;
  *triad_ms /= (done_t > 0 ? done_t : 1);
  for (auto& x : e) CHECK(hipEventDestroy(x));
}

int main(int argc, char** argv) {
  int reps = 200, warmup = 100, gemm_n = 8192, mask = 0, pair = 0;
  size_t elems = (size_t)1 << 28, skew = 0;
  for (int i = 1; i + 1 < argc; i += 2) {
    if (!strcmp(argv[i], "--reps")) reps = atoi(argv[i + 1]);
    else if (!strcmp(argv[i], "--warmup")) warmup = atoi(argv[i + 1]);
    else if (!strcmp(argv[i], "--gemm-n")) gemm_n = atoi(argv[i + 1]);
    else if (!strcmp(argv[i], "--triad-elems")) elems = strtoull(argv[i + 1], nullptr, 10);
    else if (!strcmp(argv[i], "--mask")) mask = atoi(argv[i + 1]);
    else if (!strcmp(argv[i], "--triad-skew")) skew = strtoull(argv[i + 1], nullptr, 10);
    else if (!strcmp(argv[i], "--pair")) pair = atoi(argv[i + 1]);
  }
  hipStream_t full = nullptr, masked = nullptr;
  if (orion_stream_create(0, (void**)&full) != ORION_OK) return 3;
  if (orion_stream_create(mask, (void**)&masked) != ORION_OK) return 3;

  GemmCtx g;
  g.n = gemm_n;
  const size_t mat = (size_t)gemm_n * gemm_n;
  CHECK(hipMalloc(&g.A, mat * 2));
  CHECK(hipMalloc(&g.B, mat * 2));
  CHECK(hipMalloc(&g.C, mat * 2));
  hipLaunchKernelGGL(init_uniform, dim3(4096), dim3(256), 0, full, (uint32_t*)g.A, mat / 2, 1u, 1);
  hipLaunchKernelGGL(init_uniform, dim3(4096), dim3(256), 0, full, (uint32_t*)g.B, mat / 2, 2u, 1);
  TriadCtx t;
  t.n = elems;
  // --triad-skew S (a multiple of 16): c starts S bytes and a 2 S bytes further
  // into their allocations than b, so the three streams do not walk the memory
  // channels in lockstep
  if (skew % 16) return 4;
  CHECK(hipMalloc((void**)&t.a, elems * 4 + 2 * skew));
  CHECK(hipMalloc((void**)&t.b, elems * 4));
  CHECK(hipMalloc((void**)&t.c, elems * 4 + skew));
  t.a = (float*)((char*)t.a + 2 * skew);
  t.c = (float*)((char*)t.c + skew);
  hipLaunchKernelGGL(init_uniform, dim3(4096), dim3(256), 0, full, (uint32_t*)t.b, elems, 3u, 0);
  hipLaunchKernelGGL(init_uniform, dim3(4096), dim3(256), 0, full, (uint32_t*)t.c, elems, 4u, 0);
  CHECK(hipStreamSynchronize(full));

  const double flops = 2.0 * gemm_n * (double)gemm_n * gemm_n;
  if (pair) {
    float g_ms = 0, t_ms = 0;
    run_pair(full, masked, &g, &t, 30, 90, &g_ms, &t_ms);  // pilot; settles the clocks
    run_pair(full, masked, &g, &t, 30, (int)(30 * g_ms / t_ms) + 1, &g_ms, &t_ms);
    const int n_triad = (int)(reps * g_ms / t_ms) + 1;
    run_pair(full, masked, &g, &t, reps, n_triad, &g_ms, &t_ms);
    printf("{\"pair\": true, \"reps\": %d, \"triad_launches\": %d, \"cu_mask\": %d, "
           "\"gemm\": {\"n\": %d, \"ms\": %.5f, \"tflops\": %.2f, \"frac_of_2500\": %.4f}, "
           "\"triad\": {\"elems\": %zu, \"ms\": %.5f, \"gbs\": %.1f, \"frac_of_8000\": %.4f}}\n",
           reps, n_triad, mask, gemm_n, g_ms, flops / g_ms / 1e9, flops / g_ms / 1e9 / 2500.0,
           elems, t_ms, 12.0 * elems / t_ms / 1e6, 12.0 * elems / t_ms / 1e6 / 8000.0);
    return 0;
  }
  const float burst_ms = time_ms(full, 20, 0, launch_gemm, &g);
  const float gemm_ms = time_ms(full, reps, warmup, launch_gemm, &g);
  const float triad_ms = time_ms(masked, reps, 3, launch_triad, &t);
  const float copy_ms = time_ms(full, reps, 3, launch_copy, &t);
  printf("{\"reps\": %d, \"warmup\": %d, \"gemm\": {\"n\": %d, \"ms\": %.5f, \"tflops\": %.2f, "
         "\"frac_of_2500\": %.4f, \"burst_ms\": %.5f, \"burst_tflops\": %.2f}, "
         "\"triad\": {\"elems\": %zu, \"cu_mask\": %d, \"ms\": %.5f, \"gbs\": %.1f, \"frac_of_8000\": %.4f}, "
         "\"copy\": {\"bytes\": %zu, \"ms\": %.5f, \"gbs\": %.1f}}\n",
         reps, warmup, gemm_n, gemm_ms, flops / gemm_ms / 1e9, flops / gemm_ms / 1e9 / 2500.0,
         burst_ms, flops / burst_ms / 1e9, elems,
         mask, triad_ms, 12.0 * elems / triad_ms / 1e6, 12.0 * elems / triad_ms / 1e6 / 8000.0,
         elems * 8, copy_ms, 8.0 * elems / copy_ms / 1e6);
  return 0;
}
