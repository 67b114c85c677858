// A stand-in for the HIP runtime, for host-only tests of the capture and
// scheduler libraries (selected with ORION_HIP_LIBRARY).  TEST INFRASTRUCTURE.
//
// "Device" memory is host memory.  A launch runs its kernel -- a host function
// -- at once and marks its stream busy for a configurable time, so that events
// recorded after it complete later, like on a GPU.  Every call is appended to a
// log the tests read back.
#define __HIP_PLATFORM_AMD__ 1
#include <hip/hip_runtime_api.h>

#include <stdlib.h>
#include <string.h>
#include <time.h>

#include <atomic>
#include <mutex>
#include <vector>

int gettid_cached();

namespace {

int64_t now_ns() {
  timespec ts;
  clock_gettime(CLOCK_MONOTONIC, &ts);
  return (int64_t)ts.tv_sec * 1000000000ll + ts.tv_nsec;
}

struct FakeStream {
  int id;
  int cu_mask_bits;           // 0 = unmasked
  std::atomic<int64_t> busy_until{0};
};
struct FakeEvent {
  std::atomic<int64_t> done_at{0};
};

struct LogEntry {
  int kind;      // 0 launch, 1 copy, 2 fill, 3 malloc, 4 free, 5 event record,
                 // 6 stream wait event, 7 stream sync
  int stream_id;
  int tid;
  uint64_t a, b;
};

std::mutex g_mu;
std::vector<LogEntry> g_log;
std::vector<FakeStream*> g_streams;
std::atomic<int64_t> g_kernel_ns{20000};
std::atomic<int64_t> g_copy_ns{5000};
FakeStream g_null_stream{0, 0};

FakeStream* S(hipStream_t s) { return s ? (FakeStream*)s : &g_null_stream; }

void log_call(int kind, hipStream_t s, uint64_t a, uint64_t b) {
  std::lock_guard<std::mutex> l(g_mu);
  g_log.push_back({kind, S(s)->id, (int)gettid_cached(), a, b});
}

}  // namespace

#include <sys/syscall.h>
#include <unistd.h>
namespace {
int gettid_cached_impl() { return (int)syscall(SYS_gettid); }
}
int gettid_cached() { thread_local int t = gettid_cached_impl(); return t; }

namespace {
void occupy(hipStream_t s, int64_t ns) {
  FakeStream* st = S(s);
  int64_t now = now_ns();
  int64_t cur = st->busy_until.load();
  int64_t start = cur > now ? cur : now;
  st->busy_until.store(start + ns);
}
typedef void (*fake_kernel_t)(void** params);
}  // namespace

extern "C" {

// ---- control API for tests
void fakehip_reset(void) {
  std::lock_guard<std::mutex> l(g_mu);
  g_log.clear();
}
void fakehip_set_costs(long long kernel_ns, long long copy_ns) {
  g_kernel_ns = kernel_ns;
  g_copy_ns = copy_ns;
}
int fakehip_log_size(void) {
  std::lock_guard<std::mutex> l(g_mu);
  return (int)g_log.size();
}
int fakehip_log_get(int i, int* kind, int* stream_id, int* tid,
                    unsigned long long* a, unsigned long long* b) {
  std::lock_guard<std::mutex> l(g_mu);
  if (i < 0 || i >= (int)g_log.size()) return 1;
  *kind = g_log[i].kind; *stream_id = g_log[i].stream_id; *tid = g_log[i].tid;
  *a = g_log[i].a; *b = g_log[i].b;
  return 0;
}
int fakehip_stream_id(void* s) { return S((hipStream_t)s)->id; }
int fakehip_stream_mask_bits(int id) {
  std::lock_guard<std::mutex> l(g_mu);
  for (auto* s : g_streams) if (s->id == id) return s->cu_mask_bits;
  return -1;
}

// ---- built-in "kernels": host functions taking the launch's params array
// y[i] = a * x[i] + y[i];  params: float* y, float* x, float a, int n
void fake_kernel_saxpy(void** p) {
  float* y = *(float**)p[0];
  const float* x = *(const float**)p[1];
  const float a = *(float*)p[2];
  const int n = *(int*)p[3];
  for (int i = 0; i < n; ++i) y[i] = a * x[i] + y[i];
}
// y[i] = y[i] * y[i] + c;  params: float* y, float c, int n  (order-sensitive)
void fake_kernel_sqadd(void** p) {
  float* y = *(float**)p[0];
  const float c = *(float*)p[1];
  const int n = *(int*)p[2];
  for (int i = 0; i < n; ++i) y[i] = y[i] * y[i] + c;
}

// ---- the HIP subset
hipError_t hipLaunchKernel(const void* f, dim3 grid, dim3 block, void** args,
                           size_t, hipStream_t s) {
  log_call(0, s, (uint64_t)f, ((uint64_t)grid.x << 32) | block.x);
  ((fake_kernel_t)f)(args);
  occupy(s, g_kernel_ns);
  return hipSuccess;
}
hipError_t hipExtLaunchKernel(const void* f, dim3 grid, dim3 block, void** args,
                              size_t shmem, hipStream_t s, hipEvent_t, hipEvent_t, int) {
  return hipLaunchKernel(f, grid, block, args, shmem, s);
}
hipError_t hipLaunchCooperativeKernel(const void* f, dim3 grid, dim3 block,
                                      void** args, unsigned int shmem, hipStream_t s) {
  return hipLaunchKernel(f, grid, block, args, shmem, s);
}
hipError_t hipModuleLaunchKernel(hipFunction_t f, unsigned int gx, unsigned int,
                                 unsigned int, unsigned int bx, unsigned int,
                                 unsigned int, unsigned int, hipStream_t s,
                                 void** params, void**) {
  log_call(0, s, (uint64_t)f, ((uint64_t)gx << 32) | bx);
  ((fake_kernel_t)f)(params);
  occupy(s, g_kernel_ns);
  return hipSuccess;
}
hipError_t hipExtModuleLaunchKernel(hipFunction_t f, uint32_t gx, uint32_t gy,
                                    uint32_t gz, uint32_t bx, uint32_t by,
                                    uint32_t bz, size_t shmem, hipStream_t s,
                                    void** params, void** extra, hipEvent_t,
                                    hipEvent_t, uint32_t) {
  return hipModuleLaunchKernel(f, gx, gy, gz, bx, by, bz, (unsigned)shmem, s, params, extra);
}
hipError_t hipHccModuleLaunchKernel(hipFunction_t f, uint32_t gx, uint32_t gy,
                                    uint32_t gz, uint32_t bx, uint32_t by,
                                    uint32_t bz, size_t shmem, hipStream_t s,
                                    void** params, void** extra, hipEvent_t a,
                                    hipEvent_t b) {
  return hipExtModuleLaunchKernel(f, gx, gy, gz, bx, by, bz, shmem, s, params, extra, a, b, 0);
}
hipError_t hipModuleLaunchCooperativeKernel(hipFunction_t f, unsigned int gx,
                                            unsigned int gy, unsigned int gz,
                                            unsigned int bx, unsigned int by,
                                            unsigned int bz, unsigned int shmem,
                                            hipStream_t s, void** params) {
  return hipModuleLaunchKernel(f, gx, gy, gz, bx, by, bz, shmem, s, params, nullptr);
}
// A stand-in executable graph: up to eight host kernels run in order, logged as
// one launch (kind 0) like any other kernel.
struct FakeGraphExec {
  int n;
  fake_kernel_t fn[8];
  void** params[8];
};
hipError_t hipGraphLaunch(hipGraphExec_t exec, hipStream_t s) {
  FakeGraphExec* g = (FakeGraphExec*)exec;
  log_call(0, s, (uint64_t)exec, (uint64_t)g->n);
  for (int i = 0; i < g->n; ++i) g->fn[i](g->params[i]);
  occupy(s, g_kernel_ns * g->n);
  return hipSuccess;
}
hipError_t hipMalloc(void** p, size_t n) {
  *p = malloc(n ? n : 1);
  log_call(3, nullptr, (uint64_t)*p, n);
  return *p ? hipSuccess : hipErrorOutOfMemory;
}
hipError_t hipFree(void* p) {
  log_call(4, nullptr, (uint64_t)p, 0);
  free(p);
  return hipSuccess;
}
hipError_t hipMallocAsync(void** p, size_t n, hipStream_t s) {
  *p = malloc(n ? n : 1);
  log_call(3, s, (uint64_t)*p, n);
  return *p ? hipSuccess : hipErrorOutOfMemory;
}
hipError_t hipFreeAsync(void* p, hipStream_t s) {
  log_call(4, s, (uint64_t)p, 0);
  free(p);
  return hipSuccess;
}
hipError_t hipMemcpyAsync(void* d, const void* s_, size_t n, hipMemcpyKind, hipStream_t s) {
  log_call(1, s, (uint64_t)d, n);
  memcpy(d, s_, n);
  occupy(s, g_copy_ns);
  return hipSuccess;
}
hipError_t hipMemcpy(void* d, const void* s_, size_t n, hipMemcpyKind k) {
  return hipMemcpyAsync(d, s_, n, k, nullptr);
}
hipError_t hipMemcpyWithStream(void* d, const void* s_, size_t n, hipMemcpyKind k, hipStream_t s) {
  return hipMemcpyAsync(d, s_, n, k, s);
}
hipError_t hipMemcpy2DAsync(void* d, size_t dp, const void* s_, size_t sp, size_t w,
                            size_t h, hipMemcpyKind, hipStream_t s) {
  log_call(1, s, (uint64_t)d, w * h);
  for (size_t r = 0; r < h; ++r) memcpy((char*)d + r * dp, (const char*)s_ + r * sp, w);
  occupy(s, g_copy_ns);
  return hipSuccess;
}
hipError_t hipMemcpy2D(void* d, size_t dp, const void* s_, size_t sp, size_t w, size_t h,
                       hipMemcpyKind k) {
  return hipMemcpy2DAsync(d, dp, s_, sp, w, h, k, nullptr);
}
hipError_t hipMemsetAsync(void* d, int v, size_t n, hipStream_t s) {
  log_call(2, s, (uint64_t)d, n);
  memset(d, v, n);
  occupy(s, g_copy_ns);
  return hipSuccess;
}
hipError_t hipMemset(void* d, int v, size_t n) { return hipMemsetAsync(d, v, n, nullptr); }
hipError_t hipMemsetD32Async(hipDeviceptr_t d, int v, size_t n, hipStream_t s) {
  log_call(2, s, (uint64_t)d, n * 4);
  for (size_t i = 0; i < n; ++i) ((int*)d)[i] = v;
  occupy(s, g_copy_ns);
  return hipSuccess;
}
hipError_t hipMemsetD16Async(hipDeviceptr_t d, unsigned short v, size_t n, hipStream_t s) {
  log_call(2, s, (uint64_t)d, n * 2);
  for (size_t i = 0; i < n; ++i) ((unsigned short*)d)[i] = v;
  occupy(s, g_copy_ns);
  return hipSuccess;
}
hipError_t hipMemsetD8Async(hipDeviceptr_t d, unsigned char v, size_t n, hipStream_t s) {
  return hipMemsetAsync((void*)d, v, n, s);
}
hipError_t hipStreamSynchronize(hipStream_t s) {
  log_call(7, s, 0, 0);
  while (now_ns() < S(s)->busy_until.load()) {}
  return hipSuccess;
}
hipError_t hipStreamQuery(hipStream_t s) {
  return now_ns() >= S(s)->busy_until.load() ? hipSuccess : hipErrorNotReady;
}
hipError_t hipStreamWaitEvent(hipStream_t s, hipEvent_t e, unsigned int) {
  log_call(6, s, (uint64_t)e, 0);
  FakeStream* st = S(s);
  int64_t t = ((FakeEvent*)e)->done_at.load();
  if (t > st->busy_until.load()) st->busy_until.store(t);
  return hipSuccess;
}
static hipError_t new_stream(hipStream_t* out, int mask_bits) {
  FakeStream* st = new FakeStream();
  std::lock_guard<std::mutex> l(g_mu);
  st->id = (int)g_streams.size() + 1;
  st->cu_mask_bits = mask_bits;
  g_streams.push_back(st);
  *out = (hipStream_t)st;
  return hipSuccess;
}
hipError_t hipStreamCreateWithFlags(hipStream_t* out, unsigned int) { return new_stream(out, 0); }
hipError_t hipExtStreamCreateWithCUMask(hipStream_t* out, uint32_t words, const uint32_t* mask) {
  int bits = 0;
  for (uint32_t i = 0; i < words; ++i) bits += __builtin_popcount(mask[i]);
  return new_stream(out, bits);
}
hipError_t hipStreamDestroy(hipStream_t) { return hipSuccess; }  // ids stay valid for the log
hipError_t hipEventCreateWithFlags(hipEvent_t* e, unsigned) {
  *e = (hipEvent_t) new FakeEvent();
  return hipSuccess;
}
hipError_t hipEventDestroy(hipEvent_t e) { delete (FakeEvent*)e; return hipSuccess; }
hipError_t hipEventRecord(hipEvent_t e, hipStream_t s) {
  log_call(5, s, (uint64_t)e, 0);
  int64_t t = S(s)->busy_until.load();
  int64_t now = now_ns();
  ((FakeEvent*)e)->done_at.store(t > now ? t : now);
  return hipSuccess;
}
hipError_t hipEventQuery(hipEvent_t e) {
  return now_ns() >= ((FakeEvent*)e)->done_at.load() ? hipSuccess : hipErrorNotReady;
}
hipError_t hipEventSynchronize(hipEvent_t e) {
  while (now_ns() < ((FakeEvent*)e)->done_at.load()) {}
  return hipSuccess;
}
hipError_t hipEventElapsedTime(float* ms, hipEvent_t a, hipEvent_t b) {
  *ms = (float)(((FakeEvent*)b)->done_at.load() - ((FakeEvent*)a)->done_at.load()) / 1.0e6f;
  return hipSuccess;
}
hipError_t hipDeviceSynchronize(void) {
  std::vector<FakeStream*> all;
  { std::lock_guard<std::mutex> l(g_mu); all = g_streams; }
  for (auto* s : all) while (now_ns() < s->busy_until.load()) {}
  return hipSuccess;
}
hipError_t hipDeviceGetAttribute(int* v, hipDeviceAttribute_t a, int) {
  *v = a == hipDeviceAttributeMultiprocessorCount ? 256 : 0;
  return hipSuccess;
}
hipError_t hipSetDevice(int) { return hipSuccess; }
hipError_t hipGetDevice(int* d) { *d = 0; return hipSuccess; }
hipError_t hipGetLastError(void) { return hipSuccess; }
const char* hipGetErrorString(hipError_t) { return "fake hip error"; }
const char* hipKernelNameRef(const hipFunction_t) { return "fake_kernel"; }
const char* hipKernelNameRefByPtr(const void*, hipStream_t) { return "fake_kernel"; }

}  // extern "C"
