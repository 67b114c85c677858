// A stand-in for the HIP runtime, for host-only tests of the capture and
// scheduler libraries (selected with ORION_HIP_LIBRARY).  TEST INFRASTRUCTURE.
//
// "Device" memory is host memory.  Two modes:
//  * immediate (default): a launch runs its kernel -- a host function -- at once
//    and marks its stream busy for a configurable time, so that events recorded
//    after it complete later, like on a GPU;
//  * asynchronous (FAKEHIP_ASYNC=1): every stream is a queue; a launch copies its
//    arguments, as the real runtime does, and returns; one executor thread runs
//    the queued work later, each stream in order, the streams against each other
//    in an order it draws at random unless events say otherwise.  Work that the
//    library under test issues without the ordering it needs then computes wrong
//    results on the host, where it can be debugged, instead of faulting a GPU.
// Every call is appended to a log the tests read back.
#define __HIP_PLATFORM_AMD__ 1
#include <hip/hip_runtime_api.h>

#include <stdio.h>
#include <stdlib.h>
#include <string.h>
#include <time.h>

#include <atomic>
#include <condition_variable>
#include <deque>
#include <functional>
#include <memory>
#include <mutex>
#include <thread>
#include <vector>
#include "fakehip_kernels.h"

int gettid_cached();

namespace {

int64_t now_ns() {
  timespec ts;
  clock_gettime(CLOCK_MONOTONIC, &ts);
  return (int64_t)ts.tv_sec * 1000000000ll + ts.tv_nsec;
}

struct FakeEvent {
  std::atomic<int64_t> done_at{0};
  // asynchronous mode (under g_exec_mu): records are numbered; `completed` is
  // the number of the latest one the executor has reached
  uint64_t recorded = 0, completed = 0;
  int64_t completed_at = 0;
};
// One piece of queued work (asynchronous mode).
struct Op {
  enum Kind { RUN, RECORD, WAIT } kind;
  std::function<void()> run;
  FakeEvent* event;
  uint64_t number;     // RECORD: the record's number; WAIT: the one to wait for
  int64_t cost_ns;
};
struct FakeStream {
  int id = 0;
  int cu_mask_bits = 0;       // 0 = unmasked
  std::atomic<int64_t> busy_until{0};
  std::deque<Op> queue;       // asynchronous mode, under g_exec_mu
  bool running = false;
};

struct LogEntry {
  int kind;      // 0 launch, 1 copy, 2 fill, 3 malloc, 4 free, 5 event record,
                 // 6 stream wait event, 7 stream sync, 8 graph kernel node set,
                 // 9 host callback or stream memory operation
  int stream_id;
  int tid;
  uint64_t a, b;
};

std::mutex g_mu;
std::vector<LogEntry> g_log;
std::vector<FakeStream*> g_streams;
std::atomic<int64_t> g_kernel_ns{20000};
std::atomic<int64_t> g_copy_ns{5000};
FakeStream g_null_stream;

FakeStream* S(hipStream_t s) { return s ? (FakeStream*)s : &g_null_stream; }

// ---- asynchronous mode
const bool g_async = [] { const char* e = getenv("FAKEHIP_ASYNC"); return e && atoi(e) != 0; }();
// The executor thread outlives main(): what it uses is never destroyed.
std::mutex& g_exec_mu = *new std::mutex;
std::condition_variable& g_exec_cv = *new std::condition_variable;   // work queued, or completed
std::vector<FakeStream*>& g_exec_streams = *new std::vector<FakeStream*>;  // streams that had work
bool g_exec_started = false;
uint64_t g_exec_done = 0;

uint64_t next_random() {
  static uint64_t x = [] {
    const char* e = getenv("FAKEHIP_SEED");
    return e ? (uint64_t)atoll(e) * 2654435761u + 1 : (uint64_t)now_ns() | 1;
  }();
  x ^= x << 13; x ^= x >> 7; x ^= x << 17;
  return x;
}

// The executor: picks, at random, a stream whose first piece of work can run.
void executor() {
  std::unique_lock<std::mutex> lock(g_exec_mu);
  for (;;) {
    std::vector<FakeStream*> ready;
    bool progressed = false;
    for (FakeStream* st : g_exec_streams) {
      // markers cost nothing: take them as they come
      while (!st->queue.empty()) {
        Op& op = st->queue.front();
        if (op.kind == Op::RECORD) {
          if (op.number > op.event->completed) op.event->completed = op.number;
          op.event->completed_at = now_ns();
          op.event->done_at.store(op.event->completed_at);
          st->queue.pop_front();
          progressed = true;
        } else if (op.kind == Op::WAIT && op.event->completed >= op.number) {
          st->queue.pop_front();
          progressed = true;
        } else {
          break;
        }
      }
      if (!st->queue.empty() && st->queue.front().kind == Op::RUN) ready.push_back(st);
    }
    if (progressed) g_exec_cv.notify_all();
    if (ready.empty()) {
      if (!progressed) g_exec_cv.wait(lock);
      continue;
    }
    FakeStream* st = ready[next_random() % ready.size()];
    Op op = std::move(st->queue.front());
    st->queue.pop_front();
    st->running = true;
    lock.unlock();
    op.run();
    if (op.cost_ns > 0) {
      const int64_t until = now_ns() + op.cost_ns;
      while (now_ns() < until) {}
    }
    lock.lock();
    ++g_exec_done;
    st->running = false;
    g_exec_cv.notify_all();
  }
}

// FAKEHIP_DEBUG=1: what every queue holds, every two seconds (a hung test).
void reporter() {
  for (;;) {
    timespec two = {2, 0};
    nanosleep(&two, nullptr);
    std::lock_guard<std::mutex> lock(g_exec_mu);
    fprintf(stderr, "fakehip: %llu pieces of work run so far\n", (unsigned long long)g_exec_done);
    for (FakeStream* st : g_exec_streams) {
      if (st->queue.empty() && !st->running) continue;
      fprintf(stderr, "fakehip: stream %d: %zu queued%s", st->id, st->queue.size(),
              st->running ? ", running" : "");
      if (!st->queue.empty()) {
        const Op& op = st->queue.front();
        if (op.kind == Op::WAIT)
          fprintf(stderr, ", first waits for record %llu of event %p (at %llu of %llu)",
                  (unsigned long long)op.number, (void*)op.event,
                  (unsigned long long)op.event->completed, (unsigned long long)op.event->recorded);
        else
          fprintf(stderr, ", first is %s", op.kind == Op::RUN ? "work" : "a record");
      }
      fprintf(stderr, "\n");
    }
  }
}

void enqueue(hipStream_t s, Op op) {
  FakeStream* st = S(s);
  std::lock_guard<std::mutex> lock(g_exec_mu);
  if (!g_exec_started) {
    g_exec_started = true;
    std::thread(executor).detach();
    const char* dbg = getenv("FAKEHIP_DEBUG");
    if (dbg && atoi(dbg)) std::thread(reporter).detach();
  }
  bool known = false;
  for (FakeStream* k : g_exec_streams) known = known || k == st;
  if (!known) g_exec_streams.push_back(st);
  st->queue.push_back(std::move(op));
  g_exec_cv.notify_all();
}

void run_later(hipStream_t s, int64_t cost_ns, std::function<void()> fn) {
  enqueue(s, Op{Op::RUN, std::move(fn), nullptr, 0, cost_ns});
}

bool stream_idle_locked(FakeStream* st) { return st->queue.empty() && !st->running; }

void wait_stream_idle(hipStream_t s) {
  FakeStream* st = S(s);
  std::unique_lock<std::mutex> lock(g_exec_mu);
  g_exec_cv.wait(lock, [&] { return stream_idle_locked(st); });
}

void wait_device_idle() {
  std::unique_lock<std::mutex> lock(g_exec_mu);
  g_exec_cv.wait(lock, [&] {
    for (FakeStream* st : g_exec_streams) if (!stream_idle_locked(st)) return false;
    return true;
  });
}

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

// list.ptr[k][i] = list.ptr[k][i] * scale + list.bias for every tensor k of the
// list;  params: FakeTensorList list (by value, several KiB), float scale
void fake_kernel_multi(void** p) {
  const FakeTensorList* list = (const FakeTensorList*)p[0];
  const float scale = *(float*)p[1];
  for (int k = 0; k < list->count; ++k)
    for (int i = 0; i < list->n[k]; ++i) list->ptr[k][i] = list->ptr[k][i] * scale + list->bias;
}

// Argument sizes of the built-in kernels (what a real runtime reads from the
// code object): used to deep-copy a `void** args` list into a graph kernel node
// and to unpack a HIP_LAUNCH_PARAM_BUFFER_POINTER argument buffer.
static int fake_signature(const void* f, size_t sizes[4]) {
  if (f == (const void*)fake_kernel_saxpy) {
    sizes[0] = 8; sizes[1] = 8; sizes[2] = 4; sizes[3] = 4;
    return 4;
  }
  if (f == (const void*)fake_kernel_sqadd) {
    sizes[0] = 8; sizes[1] = 4; sizes[2] = 4;
    return 3;
  }
  if (f == (const void*)fake_kernel_multi) {
    sizes[0] = sizeof(FakeTensorList); sizes[1] = 4;
    return 2;
  }
  return -1;
}
// Where each argument of `f` sits in one argument buffer: every argument at its
// natural alignment (8 bytes for a structure).  Returns the buffer's size.
static size_t fake_offsets(const size_t sizes[4], int count, size_t offsets[4]) {
  size_t at = 0;
  for (int i = 0; i < count; ++i) {
    const size_t align = sizes[i] < 8 ? sizes[i] : 8;
    at = (at + align - 1) / align * align;
    offsets[i] = at;
    at += sizes[i];
  }
  return at;
}

// Largest block each built-in kernel may be launched with (__launch_bounds__).
static unsigned fake_launch_bounds(const void* f) {
  if (f == (const void*)fake_kernel_saxpy) return 256;
  if (f == (const void*)fake_kernel_sqadd) return 64;
  if (f == (const void*)fake_kernel_multi) return 512;
  return 1024;
}

// The calling thread's last error, as the runtime keeps it: set by a failing
// call, left alone by a successful one, read and reset by hipGetLastError.
static thread_local hipError_t tl_last_error = hipSuccess;
static hipError_t done(hipError_t e) {
  if (e != hipSuccess) tl_last_error = e;
  return e;
}

// Asynchronous mode: a launch's arguments are copied at the call, as the real
// runtime copies them into its argument buffer; the closure runs the kernel on
// the copies.
static std::function<void()> bind_kernel(const void* f, void** params) {
  size_t sizes[4];
  const int count = fake_signature(f, sizes);
  if (count < 0) return nullptr;
  size_t offsets[4];
  const size_t bytes = fake_offsets(sizes, count, offsets);
  // 8-byte units: the copies are read as pointers and structures
  auto store = std::make_shared<std::vector<uint64_t>>((bytes + 7) / 8);
  unsigned char* base = (unsigned char*)store->data();
  for (int i = 0; i < count; ++i) memcpy(base + offsets[i], params[i], sizes[i]);
  return [f, store, count, offsets_copy = std::vector<size_t>(offsets, offsets + count)] {
    void* p[4];
    for (int i = 0; i < count; ++i) p[i] = (unsigned char*)store->data() + offsets_copy[i];
    ((fake_kernel_t)f)(p);
  };
}
// Lays the arguments of `f` out over one argument buffer, every argument at its
// natural alignment.
static int unpack_buffer(const void* f, unsigned char* buffer, void* unpacked[4]) {
  size_t sizes[4], offsets[4];
  const int count = fake_signature(f, sizes);
  fake_offsets(sizes, count, offsets);
  for (int i = 0; i < count; ++i) unpacked[i] = buffer + offsets[i];
  return count;
}
static void record_later(hipEvent_t e, hipStream_t s) {
  FakeEvent* ev = (FakeEvent*)e;
  uint64_t number;
  {
    std::lock_guard<std::mutex> lock(g_exec_mu);
    number = ++ev->recorded;
  }
  enqueue(s, Op{Op::RECORD, nullptr, ev, number, 0});
}

// ---- graph kernel nodes: each owns a deep copy of its kernel's arguments
struct FakeGraph { int nodes; };
struct FakeKernelNode {
  hipKernelNodeParams params;
  void* slots[4];
  std::vector<uint64_t> storage;   // the node's own copy of the arguments
};
// `held`: the kernel the node holds when the call arrives (for a new node, the
// kernel it is being created for).  This stand-in is the pessimistic reading of
// what has been observed of the real runtime, which checks a node's new
// parameters against the launch bounds of the kernel the node *holds*
// (hipGraphKernelNodeSetParams on a node whose kernel has smaller bounds than
// the new block fails with hipErrorLaunchFailure): here the argument copy, too,
// follows the held kernel's argument list -- its count and sizes -- so a node
// that is given another kernel's parameters ends up with truncated or missing
// arguments, and a library that re-points nodes computes wrong results on the
// host.  Such calls are counted (fakehip_repointed_nodes).
std::atomic<long> g_repointed{0};
static hipError_t fake_node_set(FakeKernelNode* n, const hipKernelNodeParams* p,
                                const void* held) {
  size_t sizes[4], held_sizes[4];
  const int count = fake_signature(p->func, sizes);
  if (count < 0 || p->kernelParams == nullptr) return hipErrorInvalidDeviceFunction;
  if (p->blockDim.x * p->blockDim.y * p->blockDim.z > fake_launch_bounds(held))
    return hipErrorLaunchFailure;
  int copy_count = count;
  const size_t* copy_sizes = sizes;
  if (held != p->func) {
    g_repointed.fetch_add(1);
    copy_count = fake_signature(held, held_sizes);
    if (copy_count > count) copy_count = count;   // reads no further than the list given
    copy_sizes = held_sizes;
  }
  n->params = *p;
  size_t offsets[4];
  const size_t total = fake_offsets(sizes, count, offsets);
  n->storage.assign((total + 7) / 8, 0);
  unsigned char* base = (unsigned char*)n->storage.data();
  for (int i = 0; i < count; ++i) n->slots[i] = base + offsets[i];
  for (int i = 0; i < copy_count; ++i) {
    const size_t bytes = copy_sizes[i] < sizes[i] ? copy_sizes[i] : sizes[i];
    memcpy(n->slots[i], p->kernelParams[i], bytes);
  }
  n->params.kernelParams = n->slots;
  n->params.extra = nullptr;
  return hipSuccess;
}
long fakehip_repointed_nodes(void) { return g_repointed.load(); }
hipError_t hipGraphCreate(hipGraph_t* g, unsigned int) {
  *g = (hipGraph_t) new FakeGraph{0};
  return hipSuccess;
}
hipError_t hipGraphAddKernelNode(hipGraphNode_t* out, hipGraph_t g, const hipGraphNode_t*,
                                 size_t, const hipKernelNodeParams* p) {
  FakeKernelNode* n = new FakeKernelNode();
  hipError_t err = fake_node_set(n, p, p->func);
  if (err != hipSuccess) {
    delete n;
    return done(err);
  }
  ((FakeGraph*)g)->nodes += 1;
  *out = (hipGraphNode_t)n;
  log_call(8, nullptr, (uint64_t)p->func, 0);
  return hipSuccess;
}
hipError_t hipGraphKernelNodeSetParams(hipGraphNode_t node, const hipKernelNodeParams* p) {
  log_call(8, nullptr, (uint64_t)p->func, 1);
  return done(fake_node_set((FakeKernelNode*)node, p, ((FakeKernelNode*)node)->params.func));
}
hipError_t hipGraphKernelNodeGetParams(hipGraphNode_t node, hipKernelNodeParams* out) {
  *out = ((FakeKernelNode*)node)->params;
  return hipSuccess;
}
hipError_t hipGraphDestroyNode(hipGraphNode_t node) {
  delete (FakeKernelNode*)node;
  return hipSuccess;
}

// ---- the HIP subset
hipError_t hipLaunchKernel(const void* f, dim3 grid, dim3 block, void** args,
                           size_t, hipStream_t s) {
  if (block.x * block.y * block.z > fake_launch_bounds(f)) return done(hipErrorLaunchFailure);
  log_call(0, s, (uint64_t)f, ((uint64_t)grid.x << 32) | block.x);
  if (g_async) {
    if (auto fn = bind_kernel(f, args)) {
      run_later(s, g_kernel_ns, std::move(fn));
      return hipSuccess;
    }
  }
  ((fake_kernel_t)f)(args);
  occupy(s, g_kernel_ns);
  return hipSuccess;
}
hipError_t hipExtLaunchKernel(const void* f, dim3 grid, dim3 block, void** args,
                              size_t shmem, hipStream_t s, hipEvent_t start, hipEvent_t stop, int) {
  if (g_async && start) record_later(start, s);
  const hipError_t err = hipLaunchKernel(f, grid, block, args, shmem, s);
  if (g_async && stop) record_later(stop, s);
  return err;
}
hipError_t hipLaunchCooperativeKernel(const void* f, dim3 grid, dim3 block,
                                      void** args, unsigned int shmem, hipStream_t s) {
  return hipLaunchKernel(f, grid, block, args, shmem, s);
}
hipError_t hipModuleLaunchKernel(hipFunction_t f, unsigned int gx, unsigned int,
                                 unsigned int, unsigned int bx, unsigned int,
                                 unsigned int, unsigned int, hipStream_t s,
                                 void** params, void** extra) {
  log_call(0, s, (uint64_t)f, ((uint64_t)gx << 32) | bx);
  void* unpacked[4];
  if (params == nullptr && extra != nullptr) {
    // one argument buffer
    unsigned char* buffer = nullptr;
    const size_t* size = nullptr;
    for (int i = 0; extra[i] != HIP_LAUNCH_PARAM_END; i += 2) {
      if (extra[i] == HIP_LAUNCH_PARAM_BUFFER_POINTER) buffer = (unsigned char*)extra[i + 1];
      if (extra[i] == HIP_LAUNCH_PARAM_BUFFER_SIZE) size = (const size_t*)extra[i + 1];
    }
    size_t sizes[4];
    if (fake_signature((const void*)f, sizes) < 0 || buffer == nullptr) return hipErrorInvalidValue;
    if (g_async && size != nullptr) {
      auto copy = std::make_shared<std::vector<unsigned char>>(buffer, buffer + *size);
      run_later(s, g_kernel_ns, [f, copy] {
        void* p[4];
        unpack_buffer((const void*)f, copy->data(), p);
        ((fake_kernel_t)f)(p);
      });
      return hipSuccess;
    }
    unpack_buffer((const void*)f, buffer, unpacked);
    params = unpacked;
  }
  if (g_async) {
    if (auto fn = bind_kernel((const void*)f, params)) {
      run_later(s, g_kernel_ns, std::move(fn));
      return hipSuccess;
    }
  }
  ((fake_kernel_t)f)(params);
  occupy(s, g_kernel_ns);
  return hipSuccess;
}
hipError_t hipExtModuleLaunchKernel(hipFunction_t f, uint32_t gx, uint32_t gy,
                                    uint32_t gz, uint32_t bx, uint32_t by,
                                    uint32_t bz, size_t shmem, hipStream_t s,
                                    void** params, void** extra, hipEvent_t start,
                                    hipEvent_t stop, uint32_t) {
  if (g_async && start) record_later(start, s);
  const hipError_t err =
      hipModuleLaunchKernel(f, gx, gy, gz, bx, by, bz, (unsigned)shmem, s, params, extra);
  if (g_async && stop) record_later(stop, s);
  return err;
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
  if (g_async) {
    // a graph's kernels read the arguments the graph owns, when the graph runs
    run_later(s, g_kernel_ns * g->n, [g] { for (int i = 0; i < g->n; ++i) g->fn[i](g->params[i]); });
    return hipSuccess;
  }
  for (int i = 0; i < g->n; ++i) g->fn[i](g->params[i]);
  occupy(s, g_kernel_ns * g->n);
  return hipSuccess;
}
// Device memory: the size sits in a header in front of the block, so that a free
// can fill the block with 0xff first (float NaNs): work that still names freed
// memory then shows in the results even without a sanitizer.
constexpr size_t kBlockHeader = 64;
void* block_new(size_t n) {
  unsigned char* raw = (unsigned char*)malloc(kBlockHeader + (n ? n : 1));
  if (!raw) return nullptr;
  memcpy(raw, &n, sizeof n);
  return raw + kBlockHeader;
}
void block_delete(void* p) {
  if (!p) return;
  unsigned char* raw = (unsigned char*)p - kBlockHeader;
  size_t n;
  memcpy(&n, raw, sizeof n);
  memset(p, 0xff, n);
  free(raw);
}
hipError_t hipMalloc(void** p, size_t n) {
  *p = block_new(n);
  log_call(3, nullptr, (uint64_t)*p, n);
  return *p ? hipSuccess : hipErrorOutOfMemory;
}
hipError_t hipFree(void* p) {
  log_call(4, nullptr, (uint64_t)p, 0);
  if (g_async) wait_device_idle();   // the runtime waits for the device before it releases
  block_delete(p);
  return hipSuccess;
}
hipError_t hipMallocAsync(void** p, size_t n, hipStream_t s) {
  *p = block_new(n);
  log_call(3, s, (uint64_t)*p, n);
  return *p ? hipSuccess : hipErrorOutOfMemory;
}
hipError_t hipFreeAsync(void* p, hipStream_t s) {
  log_call(4, s, (uint64_t)p, 0);
  if (g_async) {
    run_later(s, 0, [p] { block_delete(p); });   // released in stream order
    return hipSuccess;
  }
  block_delete(p);
  return hipSuccess;
}
hipError_t hipMemcpyAsync(void* d, const void* s_, size_t n, hipMemcpyKind k, hipStream_t s) {
  log_call(1, s, (uint64_t)d, n);
  if (g_async) {
    if (k == hipMemcpyHostToDevice || k == hipMemcpyHostToHost) {
      // pageable host memory is staged before the call returns
      auto staged = std::make_shared<std::vector<unsigned char>>((const unsigned char*)s_,
                                                                 (const unsigned char*)s_ + n);
      run_later(s, g_copy_ns, [d, staged] { memcpy(d, staged->data(), staged->size()); });
    } else {
      run_later(s, g_copy_ns, [d, s_, n] { memcpy(d, s_, n); });
    }
    return hipSuccess;
  }
  memcpy(d, s_, n);
  occupy(s, g_copy_ns);
  return hipSuccess;
}
hipError_t hipMemcpy(void* d, const void* s_, size_t n, hipMemcpyKind k) {
  const hipError_t err = hipMemcpyAsync(d, s_, n, k, nullptr);
  if (g_async) wait_stream_idle(nullptr);
  return err;
}
hipError_t hipMemcpyWithStream(void* d, const void* s_, size_t n, hipMemcpyKind k, hipStream_t s) {
  const hipError_t err = hipMemcpyAsync(d, s_, n, k, s);
  if (g_async) wait_stream_idle(s);
  return err;
}
hipError_t hipMemcpy2DAsync(void* d, size_t dp, const void* s_, size_t sp, size_t w,
                            size_t h, hipMemcpyKind, hipStream_t s) {
  log_call(1, s, (uint64_t)d, w * h);
  auto copy = [d, dp, s_, sp, w, h] {
    for (size_t r = 0; r < h; ++r) memcpy((char*)d + r * dp, (const char*)s_ + r * sp, w);
  };
  if (g_async) {
    run_later(s, g_copy_ns, copy);
    return hipSuccess;
  }
  copy();
  occupy(s, g_copy_ns);
  return hipSuccess;
}
hipError_t hipMemcpy2D(void* d, size_t dp, const void* s_, size_t sp, size_t w, size_t h,
                       hipMemcpyKind k) {
  const hipError_t err = hipMemcpy2DAsync(d, dp, s_, sp, w, h, k, nullptr);
  if (g_async) wait_stream_idle(nullptr);
  return err;
}
hipError_t hipMemsetAsync(void* d, int v, size_t n, hipStream_t s) {
  log_call(2, s, (uint64_t)d, n);
  if (g_async) {
    run_later(s, g_copy_ns, [d, v, n] { memset(d, v, n); });
    return hipSuccess;
  }
  memset(d, v, n);
  occupy(s, g_copy_ns);
  return hipSuccess;
}
hipError_t hipMemset(void* d, int v, size_t n) {
  const hipError_t err = hipMemsetAsync(d, v, n, nullptr);
  if (g_async) wait_stream_idle(nullptr);
  return err;
}
hipError_t hipMemsetD32Async(hipDeviceptr_t d, int v, size_t n, hipStream_t s) {
  log_call(2, s, (uint64_t)d, n * 4);
  auto fill = [d, v, n] { for (size_t i = 0; i < n; ++i) ((int*)d)[i] = v; };
  if (g_async) {
    run_later(s, g_copy_ns, fill);
    return hipSuccess;
  }
  fill();
  occupy(s, g_copy_ns);
  return hipSuccess;
}
hipError_t hipMemsetD16Async(hipDeviceptr_t d, unsigned short v, size_t n, hipStream_t s) {
  log_call(2, s, (uint64_t)d, n * 2);
  auto fill = [d, v, n] { for (size_t i = 0; i < n; ++i) ((unsigned short*)d)[i] = v; };
  if (g_async) {
    run_later(s, g_copy_ns, fill);
    return hipSuccess;
  }
  fill();
  occupy(s, g_copy_ns);
  return hipSuccess;
}
hipError_t hipMemsetD8Async(hipDeviceptr_t d, unsigned char v, size_t n, hipStream_t s) {
  return hipMemsetAsync((void*)d, v, n, s);
}
// a host callback runs at once; a stream memory operation writes at once
hipError_t hipLaunchHostFunc(hipStream_t s, hipHostFn_t fn, void* user_data) {
  log_call(9, s, (uint64_t)fn, 0);
  if (g_async) {
    run_later(s, 0, [fn, user_data] { fn(user_data); });
    return hipSuccess;
  }
  fn(user_data);
  return hipSuccess;
}
hipError_t hipStreamWriteValue32(hipStream_t s, void* ptr, uint32_t value, unsigned int) {
  log_call(9, s, (uint64_t)ptr, value);
  if (g_async) {
    run_later(s, 0, [ptr, value] { *(volatile uint32_t*)ptr = value; });
    return hipSuccess;
  }
  *(volatile uint32_t*)ptr = value;
  return hipSuccess;
}
hipError_t hipStreamSynchronize(hipStream_t s) {
  log_call(7, s, 0, 0);
  if (g_async) {
    wait_stream_idle(s);
    return hipSuccess;
  }
  while (now_ns() < S(s)->busy_until.load()) {}
  return hipSuccess;
}
hipError_t hipStreamQuery(hipStream_t s) {
  if (g_async) {
    std::lock_guard<std::mutex> lock(g_exec_mu);
    return stream_idle_locked(S(s)) ? hipSuccess : hipErrorNotReady;
  }
  return now_ns() >= S(s)->busy_until.load() ? hipSuccess : hipErrorNotReady;
}
hipError_t hipStreamWaitEvent(hipStream_t s, hipEvent_t e, unsigned int) {
  log_call(6, s, (uint64_t)e, 0);
  if (g_async) {
    // waits for the record that is the event's latest at this call
    FakeEvent* ev = (FakeEvent*)e;
    uint64_t number;
    {
      std::lock_guard<std::mutex> lock(g_exec_mu);
      number = ev->recorded;
    }
    if (number != 0) enqueue(s, Op{Op::WAIT, nullptr, ev, number, 0});
    return hipSuccess;
  }
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
hipError_t hipEventDestroy(hipEvent_t e) {
  if (!g_async) delete (FakeEvent*)e;   // queued markers may still name it
  return hipSuccess;
}
hipError_t hipEventRecord(hipEvent_t e, hipStream_t s) {
  log_call(5, s, (uint64_t)e, 0);
  if (g_async) {
    record_later(e, s);
    return hipSuccess;
  }
  int64_t t = S(s)->busy_until.load();
  int64_t now = now_ns();
  ((FakeEvent*)e)->done_at.store(t > now ? t : now);
  return hipSuccess;
}
hipError_t hipEventQuery(hipEvent_t e) {
  if (g_async) {
    std::lock_guard<std::mutex> lock(g_exec_mu);
    return ((FakeEvent*)e)->completed >= ((FakeEvent*)e)->recorded ? hipSuccess : hipErrorNotReady;
  }
  return now_ns() >= ((FakeEvent*)e)->done_at.load() ? hipSuccess : hipErrorNotReady;
}
hipError_t hipEventSynchronize(hipEvent_t e) {
  if (g_async) {
    FakeEvent* ev = (FakeEvent*)e;
    std::unique_lock<std::mutex> lock(g_exec_mu);
    const uint64_t number = ev->recorded;
    g_exec_cv.wait(lock, [&] { return ev->completed >= number; });
    return hipSuccess;
  }
  while (now_ns() < ((FakeEvent*)e)->done_at.load()) {}
  return hipSuccess;
}
hipError_t hipEventElapsedTime(float* ms, hipEvent_t a, hipEvent_t b) {
  *ms = (float)(((FakeEvent*)b)->done_at.load() - ((FakeEvent*)a)->done_at.load()) / 1.0e6f;
  return hipSuccess;
}
hipError_t hipDeviceSynchronize(void) {
  if (g_async) {
    wait_device_idle();
    return hipSuccess;
  }
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
hipError_t hipGetLastError(void) {
  const hipError_t e = tl_last_error;
  tl_last_error = hipSuccess;
  return e;
}
hipError_t hipPeekAtLastError(void) { return tl_last_error; }
const char* hipGetErrorString(hipError_t) { return "fake hip error"; }
static const char* fake_name(const void* f) {
  if (f == (const void*)fake_kernel_saxpy) return "fake_kernel_saxpy";
  if (f == (const void*)fake_kernel_sqadd) return "fake_kernel_sqadd";
  if (f == (const void*)fake_kernel_multi) return "fake_kernel_multi";
  return "fake_kernel";
}
const char* hipKernelNameRef(const hipFunction_t f) { return fake_name((const void*)f); }
const char* hipKernelNameRefByPtr(const void* f, hipStream_t) { return fake_name(f); }

}  // extern "C"
