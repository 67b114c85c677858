// libinttemp.so: interposes the HIP runtime entry points through which kernels,
// copies, fills and allocations reach the GPU (PyTorch-ROCm, MIOpen, hipBLASLt,
// rocBLAS and aotriton all funnel into them), and turns each call of a client
// thread into a record handed to the scheduler.
//
// Reference: src/cuda_capture/intercept_temp.cpp (runtime interposers, block,
// stop), src/cuda_capture/utils_interc.cpp (get_idx, block).  The cuDNN/cuBLAS
// interposers of the reference (intercept_cudnn.cpp, intercept_cublas.cpp) have
// no separate counterpart: on ROCm those libraries launch through
// hipExtModuleLaunchKernel / hipLaunchKernel, which are interposed here, so
// library work is captured kernel by kernel.
#include "capture.h"
#include "tls_fresh.h"

#include <dlfcn.h>
#include <immintrin.h>
#include <sched.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>
#include <sys/syscall.h>
#include <time.h>
#include <unistd.h>

#include <mutex>
#include <vector>

using namespace orion;

namespace {

CaptureState g_state;

constexpr int kNotClient = -1;
constexpr int kUncached = -2;

// Thread-local state of this library uses the initial-exec model: one
// instruction per access, and never the dynamic loader's __tls_get_addr, whose
// slow path a thread can be stuck on (tls_fresh.h).  The library is loaded at
// program start (LD_PRELOAD), where that model always fits; loaded later, its few
// dozen bytes come out of the loader's static surplus.
#define ORION_TLS __attribute__((tls_model("initial-exec")))
thread_local uint32_t tl_epoch ORION_TLS = 0;
thread_local int tl_client ORION_TLS = kUncached;
// Set while a client thread runs a call the scheduler granted back to it, so
// the nested real call is not captured again.
thread_local int tl_bypass ORION_TLS = 0;

// ORION_CALL_TIMING=1: every thread adds up the time it spends inside the
// interposed launch and copy entry points (entry to return, the real call
// included), for orion_thread_time_in_calls_ns: lets a client loop split a
// request's submission time into "inside the runtime and this library" and
// "inside the framework".  Off: one predictable branch per call.
const bool g_call_timing = [] {
  const char* e = getenv("ORION_CALL_TIMING");
  return e && atoi(e) != 0;
}();
thread_local uint64_t tl_call_ns ORION_TLS = 0;
thread_local uint64_t tl_call_count ORION_TLS = 0;
thread_local int tl_call_depth ORION_TLS = 0;

struct CallTimer {
  timespec t0;
  bool on;
  CallTimer() : on(g_call_timing && tl_call_depth++ == 0) {
    if (on) clock_gettime(CLOCK_MONOTONIC, &t0);
  }
  ~CallTimer() {
    if (!g_call_timing) return;
    --tl_call_depth;
    if (!on) return;
    timespec t1;
    clock_gettime(CLOCK_MONOTONIC, &t1);
    tl_call_ns += (uint64_t)((t1.tv_sec - t0.tv_sec) * 1000000000ll + (t1.tv_nsec - t0.tv_nsec));
    ++tl_call_count;
  }
};

void flush_channel(ClientChannel& ch);   // defined with submit()
void run_postponed(bool everything);     // likewise
void postponed_fence();

inline dim3 to_dim3(const Dim3& d) { return dim3(d.x, d.y, d.z); }
inline Dim3 from_dim3(const dim3& d) { return Dim3{d.x, d.y, d.z}; }

inline void cpu_relax(unsigned& spins) {
  _mm_pause();
  if ((++spins & 0x3ff) == 0) sched_yield();
}

// Thread placement.  The reference pins client idx, and the scheduler as idx N,
// to CPU idx + 1 the first time it is identified (utils_interc.cpp:36-49).  Here
// that is an option (ORION_PIN_THREADS=1): measured on the 16-CPU hosts these
// GPUs come with, threads left to the kernel's placement run the high-priority
// request 0.05-0.07 ms faster at the median, alone and co-located, and whole
// runs that are slow from start to end (a fixed CPU that is busy with something
// else) turn up less often; the best-effort trainer gains 1 %.  When pinning is
// on, slot s is the (s + 1)-th CPU the process may run on, the first one staying
// with the interpreter's other threads; the masks in force before are put back
// when the capture is disarmed.  A CPU set too small for one CPU per slot leaves
// placement to the kernel as well.
struct Pinning {
  bool on = false;
  bool clients = true;        // false: only the scheduler thread is pinned
  int scheduler_slot = 0;
  int cpus[kMaxClients + 2];
  pid_t tid[kMaxClients + 1];
  cpu_set_t before[kMaxClients + 1];
};
Pinning g_pin;

// ORION_PIN_THREADS: 0 or unset none (default), 1 every client thread and the
// scheduler thread, "scheduler" the scheduler thread only, "top" all of them but
// counted down from the highest CPU the process may use instead of up from the
// second.
void pinning_reset(int slots) {
  for (pid_t& t : g_pin.tid) t = 0;
  const char* env = getenv("ORION_PIN_THREADS");
  g_pin.on = false;
  g_pin.clients = !(env && strcmp(env, "scheduler") == 0);
  g_pin.scheduler_slot = slots - 1;
  const bool from_top = env && strcmp(env, "top") == 0;
  if (!env || !*env || strcmp(env, "0") == 0) return;
  cpu_set_t allowed;
  if (sched_getaffinity(getpid(), sizeof allowed, &allowed) != 0) return;
  int n = 0;
  if (from_top) {
    // slot s -> cpus[s + 1]; one more CPU must remain for everybody else
    for (int c = CPU_SETSIZE - 1; c >= 0 && n < slots; --c)
      if (CPU_ISSET(c, &allowed)) g_pin.cpus[1 + n++] = c;
    g_pin.on = n == slots && CPU_COUNT(&allowed) > slots;
    return;
  }
  for (int c = 0; c < CPU_SETSIZE && n < slots + 1; ++c)
    if (CPU_ISSET(c, &allowed)) g_pin.cpus[n++] = c;
  g_pin.on = n == slots + 1;
}

void pin_caller(int slot, pid_t tid) {
  if (!g_pin.on || g_pin.tid[slot] == tid) return;
  if (!g_pin.clients && slot != g_pin.scheduler_slot) return;
  if (sched_getaffinity(0, sizeof(cpu_set_t), &g_pin.before[slot]) != 0) return;
  cpu_set_t one;
  CPU_ZERO(&one);
  CPU_SET(g_pin.cpus[slot + 1], &one);
  if (sched_setaffinity(0, sizeof one, &one) == 0) g_pin.tid[slot] = tid;
}

// Threads that are no client's own but issue work on a client's behalf (calls
// routed by the stream they name: a framework's autograd worker) are put on that
// client's CPU the first time they do, once per job (reference: the lazily
// registered backward threads of utils_interc.cpp:28-49 share their client's
// CPU); the client waits while such a thread works for it.
struct HelperPin {
  pid_t tid;
  int cpu;
  cpu_set_t before;
};
std::mutex g_helper_lock;
std::vector<HelperPin> g_helpers;
thread_local uint32_t tl_helper_epoch ORION_TLS = 0;

void pin_helper(int client) {
  if (!g_pin.on || !g_pin.clients) return;
  const uint32_t e = g_state.epoch.load(std::memory_order_acquire);
  if (tl_helper_epoch == e) return;      // placed (or tried) once per job
  tl_helper_epoch = e;
  HelperPin h;
  h.tid = (pid_t)syscall(SYS_gettid);
  h.cpu = g_pin.cpus[client + 1];
  if (sched_getaffinity(0, sizeof(cpu_set_t), &h.before) != 0) return;
  cpu_set_t one;
  CPU_ZERO(&one);
  CPU_SET(h.cpu, &one);
  if (sched_setaffinity(0, sizeof one, &one) != 0) return;
  std::lock_guard<std::mutex> hold(g_helper_lock);
  g_helpers.push_back(h);
}

void pinning_undo() {
  for (int s = 0; s <= kMaxClients; ++s) {
    if (g_pin.tid[s] == 0) continue;
    // a thread that has ended leaves ESRCH, which is fine
    (void)sched_setaffinity(g_pin.tid[s], sizeof(cpu_set_t), &g_pin.before[s]);
    g_pin.tid[s] = 0;
  }
  std::lock_guard<std::mutex> hold(g_helper_lock);
  for (const HelperPin& h : g_helpers)
    (void)sched_setaffinity(h.tid, sizeof(cpu_set_t), &h.before);
  g_helpers.clear();
}

int lookup_thread() {
  const pid_t tid = (pid_t)syscall(SYS_gettid);
  if (tid == g_state.scheduler_tid) return kNotClient;
  for (int i = 0; i < g_state.num_clients; ++i)
    if (g_state.client_tids[i] == tid) {
      pin_caller(i, tid);
      return i;
    }
  return kNotClient;
}

// Which client a call belongs to: the calling thread if it is a registered
// client thread, else the client that owns the stream the call names.
inline int client_for_call(hipStream_t stream) {
  if (!g_state.armed.load(std::memory_order_acquire)) return kNotClient;
  tls_fresh_touch();   // once per thread after each reload of the helper library
  if (tl_bypass) return kNotClient;
  const uint32_t e = g_state.epoch.load(std::memory_order_acquire);
  if (tl_epoch != e || tl_client == kUncached) {
    tl_client = lookup_thread();
    tl_epoch = e;
  }
  if (tl_client >= 0) return tl_client;
  if (stream == nullptr) return kNotClient;
  if ((pid_t)syscall(SYS_gettid) == g_state.scheduler_tid) return kNotClient;
  for (int i = 0; i < g_state.num_clients; ++i)
    for (auto& s : g_state.channels[i].own_streams)
      if (s.load(std::memory_order_relaxed) == stream) {
        pin_helper(i);
        return i;
      }
  return kNotClient;
}

// The stream the caller named in the intercepted call.
hipStream_t named_stream(const Record& r) {
  if (r.type <= RT_COOP_LAUNCH_KERNEL) return r.u.launch.stream;
  if (r.type <= RT_MODULE_COOP_LAUNCH) return r.u.module.stream;
  if (r.type <= RT_MEMCPY_2D_ASYNC) return r.u.copy.stream;
  if (r.type == RT_GRAPH_LAUNCH) return r.u.graph.stream;
  if (r.type == RT_MEMCPY_2D) return nullptr;
  if (r.type == RT_MALLOC_ASYNC) return r.u.malloc_.stream;
  if (r.type == RT_FREE_ASYNC) return r.u.free_.stream;
  if (r.type >= RT_MEMSET) return r.u.set.stream;
  return nullptr;
}

// Runs a record the scheduler granted back to its caller (blocking calls:
// allocation, free, synchronous copies and fills).  `stream` is the stream the
// scheduler assigned.
int execute_on_caller(Record& r, hipStream_t stream) {
  const HipApi* hip = orion_hip_api();
  hipError_t err = hipSuccess;
  ++tl_bypass;
  switch (r.type) {
    case RT_MALLOC:
      err = hip->hipMalloc(r.u.malloc_.ptr, r.u.malloc_.size);
      break;
    case RT_FREE:
      err = hip->hipFree(r.u.free_.ptr);
      break;
    case RT_MEMCPY:
    case RT_MEMCPY_WITH_STREAM:
      err = hip->hipMemcpyAsync(r.u.copy.dst, r.u.copy.src, r.u.copy.bytes,
                                r.u.copy.kind, stream);
      if (err == hipSuccess) err = hip->hipStreamSynchronize(stream);
      break;
    case RT_MEMSET:
      err = hip->hipMemsetAsync(r.u.set.dst, r.u.set.value, r.u.set.count, stream);
      if (err == hipSuccess) err = hip->hipStreamSynchronize(stream);
      break;
    case RT_MEMCPY_2D:
      err = hip->hipMemcpy2DAsync(r.u.copy.dst, r.u.copy.dpitch, r.u.copy.src, r.u.copy.spitch,
                                  r.u.copy.width, r.u.copy.height, r.u.copy.kind, stream);
      if (err == hipSuccess) err = hip->hipStreamSynchronize(stream);
      break;
    case RT_MALLOC_ASYNC:   // ordered after the client's earlier work, where it now runs
      err = hip->hipMallocAsync ? hip->hipMallocAsync(r.u.malloc_.ptr, r.u.malloc_.size, stream)
                                : hipErrorNotSupported;
      break;
    case RT_FREE_ASYNC:
      err = hip->hipFreeAsync ? hip->hipFreeAsync(r.u.free_.ptr, stream) : hipErrorNotSupported;
      break;
    default:
      err = hipErrorInvalidValue;
  }
  --tl_bypass;
  return (int)err;
}

}  // namespace

extern "C" {

CaptureState* orion_capture_state(void) { return &g_state; }

// Status a record carries when the scheduler hands a blocking call back to the
// thread that made it.
enum { ORION_GRANTED_TO_CALLER = orion::kRecordGranted };

bool orion_record_runs_on_caller(int type) {
  return type == RT_MALLOC || type == RT_FREE || type == RT_MEMCPY ||
         type == RT_MEMCPY_WITH_STREAM || type == RT_MEMSET || type == RT_MEMCPY_2D ||
         type == RT_MALLOC_ASYNC || type == RT_FREE_ASYNC;
}

// Issues a record's HIP call on `stream` (scheduler thread).  Returns the HIP
// status.  Records of the blocking kinds are not issued here: the scheduler
// grants them to the caller instead (see orion_record_runs_on_caller).
int orion_execute_record(const Record* rec, hipStream_t stream) {
  const HipApi* hip = orion_hip_api();
  const Record& r = *rec;
  hipError_t err;
  switch (r.type) {
    case RT_LAUNCH_KERNEL:
      err = hip->hipLaunchKernel(r.u.launch.func, to_dim3(r.u.launch.grid),
                                 to_dim3(r.u.launch.block), r.u.launch.args,
                                 r.u.launch.shmem, stream);
      break;
    case RT_EXT_LAUNCH_KERNEL:
      err = hip->hipExtLaunchKernel(r.u.launch.func, to_dim3(r.u.launch.grid),
                                    to_dim3(r.u.launch.block), r.u.launch.args,
                                    r.u.launch.shmem, stream, r.u.launch.start,
                                    r.u.launch.stop, r.u.launch.flags);
      break;
    case RT_COOP_LAUNCH_KERNEL:
      err = hip->hipLaunchCooperativeKernel(r.u.launch.func, to_dim3(r.u.launch.grid),
                                            to_dim3(r.u.launch.block), r.u.launch.args,
                                            (unsigned)r.u.launch.shmem, stream);
      break;
    case RT_MODULE_LAUNCH:
      err = hip->hipModuleLaunchKernel(r.u.module.f, r.u.module.gx, r.u.module.gy,
                                       r.u.module.gz, r.u.module.bx, r.u.module.by,
                                       r.u.module.bz, (unsigned)r.u.module.shmem,
                                       stream, r.u.module.params, r.u.module.extra);
      break;
    case RT_EXT_MODULE_LAUNCH:
      err = hip->hipExtModuleLaunchKernel(
          r.u.module.f, r.u.module.gx, r.u.module.gy, r.u.module.gz, r.u.module.bx,
          r.u.module.by, r.u.module.bz, r.u.module.shmem, stream, r.u.module.params,
          r.u.module.extra, r.u.module.start, r.u.module.stop, r.u.module.flags);
      break;
    case RT_MODULE_COOP_LAUNCH:
      err = hip->hipModuleLaunchCooperativeKernel(
          r.u.module.f, r.u.module.gx, r.u.module.gy, r.u.module.gz, r.u.module.bx,
          r.u.module.by, r.u.module.bz, (unsigned)r.u.module.shmem, stream,
          r.u.module.params);
      break;
    case RT_MEMCPY_ASYNC:
      err = hip->hipMemcpyAsync(r.u.copy.dst, r.u.copy.src, r.u.copy.bytes,
                                r.u.copy.kind, stream);
      break;
    case RT_MEMCPY_2D_ASYNC:
      err = hip->hipMemcpy2DAsync(r.u.copy.dst, r.u.copy.dpitch, r.u.copy.src,
                                  r.u.copy.spitch, r.u.copy.width, r.u.copy.height,
                                  r.u.copy.kind, stream);
      break;
    case RT_MEMSET_ASYNC:
      err = hip->hipMemsetAsync(r.u.set.dst, r.u.set.value, r.u.set.count, stream);
      break;
    case RT_MEMSET_D32_ASYNC:
      err = hip->hipMemsetD32Async((hipDeviceptr_t)r.u.set.dst, r.u.set.value,
                                   r.u.set.count, stream);
      break;
    case RT_MEMSET_D16_ASYNC:
      err = hip->hipMemsetD16Async((hipDeviceptr_t)r.u.set.dst,
                                   (unsigned short)r.u.set.value, r.u.set.count,
                                   stream);
      break;
    case RT_MEMSET_D8_ASYNC:
      err = hip->hipMemsetD8Async((hipDeviceptr_t)r.u.set.dst,
                                  (unsigned char)r.u.set.value, r.u.set.count,
                                  stream);
      break;
    case RT_GRAPH_LAUNCH:
      err = hip->hipGraphLaunch ? hip->hipGraphLaunch(r.u.graph.exec, stream)
                                : hipErrorNotSupported;
      break;
    default:
      // reference: "UNSUPPORTED OPERATION - ABORT", utils_sched.cpp:514-516
      fprintf(stderr, "orion: record type %d cannot be issued by the scheduler\n",
              r.type);
      abort();
  }
  return (int)err;
}

void orion_capture_arm(int num_clients, const int* client_tids, int scheduler_tid) {
  if (num_clients > kMaxClients) {
    fprintf(stderr, "orion: at most %d clients\n", kMaxClients);
    abort();
  }
  g_state.armed.store(0, std::memory_order_release);
  g_state.scheduler_polling.store(0, std::memory_order_release);
  run_postponed(true);   // the queue positions they wait for are about to be reset
  pinning_undo();
  pinning_reset(num_clients + 1);
  g_state.num_clients = num_clients;
  g_state.scheduler_tid = scheduler_tid;
  if ((pid_t)syscall(SYS_gettid) == scheduler_tid) pin_caller(num_clients, scheduler_tid);
  for (int i = 0; i < num_clients; ++i) {
    g_state.client_tids[i] = client_tids ? client_tids[i] : 0;
    ClientChannel& ch = g_state.channels[i];
    ch.tail.store(0);
    ch.head.store(0);
    ch.producer_lock.store(0);
    ch.flush_lock.store(0);
    ch.head_seen = 0;
    ch.deferred.store(0);
    ch.deferred_upto.store(0);
    ch.released_iters.store(0);
    ch.stop.store(0);
    ch.stop_ack.store(0);
    ch.last_stream.store(nullptr);
    ch.direct_stream.store(nullptr);
    ch.submitted.store(0);
    ch.block_calls.store(0);
    ch.may_run_ahead.store(0);
    // own_streams survive: a client may register its stream before setup runs
  }
  // Off unless asked for, and then only for the clients the scheduler clears
  // afterwards (orion_capture_allow_run_ahead): with a ResNet-50 trainer queueing
  // ahead beside a ResNet-50 inference client an MI355X has faulted, cause not
  // found, so no framework client is ever cleared (the hand-written kernel pair
  // runs with it, bit-exact).  On the host-only stand-in runtime the tests can
  // leave hipLaunchKernel synchronous (ORION_BE_RUN_AHEAD_HOLDERS=0), which takes
  // the graph kernel nodes out of the picture.
  const char* ahead = getenv("ORION_BE_RUN_AHEAD");
  const char* holders = orion_hip_api()->stand_in ? getenv("ORION_BE_RUN_AHEAD_HOLDERS") : nullptr;
  g_state.run_ahead.store(ahead && atoi(ahead) != 0 ? 1 : 0, std::memory_order_release);
  g_state.run_ahead_holders.store(holders && atoi(holders) == 0 ? 0 : 1, std::memory_order_release);
  g_state.epoch.fetch_add(1, std::memory_order_acq_rel);
  g_state.armed.store(1, std::memory_order_release);
}

void orion_capture_allow_run_ahead(int client, int allow) {
  if (client < 0 || client >= kMaxClients) return;
  g_state.channels[client].may_run_ahead.store(allow ? 1 : 0, std::memory_order_release);
}

void orion_capture_disarm(void) {
  const bool was_armed = g_state.armed.exchange(0, std::memory_order_acq_rel) != 0;
  g_state.epoch.fetch_add(1, std::memory_order_acq_rel);
  if (was_armed)
    for (int i = 0; i < g_state.num_clients; ++i) flush_channel(g_state.channels[i]);
  postponed_fence();   // nobody adds to the list once it has seen the capture disarmed
  run_postponed(true);
  pinning_undo();
}

void orion_capture_enter_loop(void) {
  for (int i = 0; i < g_state.num_clients; ++i) {
    ClientChannel& ch = g_state.channels[i];
    unsigned spins = 0;
    while (ch.flush_lock.exchange(1)) cpu_relax(spins);
    ch.flush_lock.store(0);
  }
}

// The CPU the capture pinned the calling thread to, or -1.
int orion_pinned_cpu(void) {
  const pid_t tid = (pid_t)syscall(SYS_gettid);
  for (int s = 0; s <= kMaxClients; ++s)
    if (g_pin.tid[s] == tid) return g_pin.cpus[s + 1];
  std::lock_guard<std::mutex> hold(g_helper_lock);
  for (const HelperPin& h : g_helpers)
    if (h.tid == tid) return h.cpu;
  return -1;
}

// Registers the calling thread as a thread of `client` (alternative to passing
// thread ids to setup; also used for helper threads a client spawns).
void orion_register_thread(int client) {
  if (client < 0 || client >= kMaxClients) return;
  tl_client = client;
  tl_epoch = g_state.epoch.load(std::memory_order_acquire);
}

// Declares that `stream` belongs to the calling client thread: calls that name
// it from unregistered threads (autograd workers) are routed to this client.
void orion_register_stream(void* stream) {
  int idx = tl_client;
  if (idx < 0) {
    const pid_t tid = (pid_t)syscall(SYS_gettid);
    for (int i = 0; i < g_state.num_clients; ++i)
      if (g_state.client_tids[i] == tid) idx = i;
  }
  if (idx < 0 || stream == nullptr) return;
  for (auto& s : g_state.channels[idx].own_streams) {
    hipStream_t cur = s.load();
    if (cur == (hipStream_t)stream) return;
    if (cur == nullptr) {
      s.store((hipStream_t)stream);
      return;
    }
  }
}

int orion_client_index(void) { return client_for_call(nullptr); }

// Records of `client` queued so far in this job, and how many of them were
// queued without their caller waiting for the dispatch.
unsigned long long orion_client_submitted(int client) {
  if (client < 0 || client >= kMaxClients) return 0;
  return g_state.channels[client].submitted.load(std::memory_order_relaxed);
}
unsigned long long orion_client_deferred(int client) {
  if (client < 0 || client >= kMaxClients) return 0;
  return g_state.channels[client].deferred.load(std::memory_order_relaxed);
}

// Time the calling thread has spent inside the interposed launch and copy entry
// points so far, and how many such calls it made (ORION_CALL_TIMING=1; zero
// otherwise).
unsigned long long orion_thread_time_in_calls_ns(void) { return tl_call_ns; }
unsigned long long orion_thread_calls(void) { return tl_call_count; }

// The client a call naming `stream` from the calling thread would be queued
// for, or a negative value when it would go straight to the runtime.
int orion_client_of_stream(void* stream) { return client_for_call((hipStream_t)stream); }

// While on, the calling thread's HIP calls go straight to the runtime: used by
// a client for work that must not count as part of an iteration (building the
// model, library auto-tuning runs whose kernel count is not reproducible).
void orion_thread_passthrough(int on) {
  tl_bypass = on ? 1 : 0;
  // the end of a client's un-captured warm-up: whatever it loaded lazily (solver
  // libraries, code objects) is in the process now
  if (!on && g_state.armed.load(std::memory_order_acquire)) tls_fresh_check();
}

// For the scheduler thread, once per completed iteration (the reloads are left
// to the client threads, which have time for them while they wait).
void orion_tls_fresh_touch(void) { tls_fresh_touch(); }

// The same cure for a thread that is not scheduled at all (a client on a plain
// stream calls it once per request): lets a measurement tell what the scheduling
// path costs from what the dynamic loader's slow path costs.
void orion_tls_fresh_check(void) { tls_fresh_check(); }

// -- control calls of the client loops (reference: intercept_temp.cpp:124-142)

// Returns once the scheduler has released iteration `it` of the calling client.
void block(int it) {
  const int idx = client_for_call(nullptr);
  if (idx < 0) return;  // not armed, or not a client: nothing to wait for
  ClientChannel& ch = g_state.channels[idx];
  ch.block_calls.store((int64_t)it + 1, std::memory_order_release);
  tls_fresh_check();    // while the GPU finishes the iteration
  unsigned spins = 0;
  while (ch.released_iters.load(std::memory_order_acquire) <= (int64_t)it) {
    if (!g_state.armed.load(std::memory_order_acquire)) return;
    cpu_relax(spins);
  }
  // a best-effort client between two iterations has time for the releases that
  // were postponed while records were queued ahead (each waits for the device)
  if (idx < g_state.num_clients - 1) run_postponed(false);
}

// Non-zero once the scheduler has asked the calling client to stop; the call
// acknowledges the request.  (The reference returns a C bool that its ctypes
// caller reads as int; an int is returned here.)
int stop(void) {
  const int idx = client_for_call(nullptr);
  if (idx < 0) return 0;
  tls_fresh_touch();
  ClientChannel& ch = g_state.channels[idx];
  const int res = ch.stop.load(std::memory_order_acquire);
  if (res) ch.stop_ack.store(1, std::memory_order_release);
  return res;
}

}  // extern "C"

namespace {

double stuck_limit_s() {
  static const double limit = [] {
    const char* e = getenv("ORION_STUCK_LIMIT_S");
    return e && atof(e) > 0 ? atof(e) : 20.0;
  }();
  return limit;
}

double monotonic_s() {
  timespec ts;
  clock_gettime(CLOCK_MONOTONIC, &ts);
  return (double)ts.tv_sec + 1e-9 * (double)ts.tv_nsec;
}

// Gives a record a deep copy of everything it points to, so that it can wait in
// the queue after the call that made it has returned.  Returns false when the
// record cannot be made self-contained (then the caller waits for its dispatch,
// as the reference's callers always do):
//  * hipLaunchKernel names its arguments through `void** args` without their
//    sizes.  The runtime knows them: a graph kernel node built from the same
//    parameters copies every argument, and hipGraphKernelNodeGetParams hands
//    back a parameter array that the node owns and that stays valid until the
//    node is given new parameters.  Each queue slot keeps one such node (in a
//    graph that is never launched) purely as the owner of the copy.
//  * module launches that pass their arguments as one buffer
//    (HIP_LAUNCH_PARAM_BUFFER_POINTER / _SIZE in `extra`: MIOpen, rocBLAS,
//    hipBLASLt) get the buffer copied into the slot.  Launches with a
//    `kernelParams` array, with timing events, or cooperative ones are left
//    alone.
//  * device-to-device copies and fills point to nothing on the host.
bool make_self_contained(ClientChannel& ch, uint32_t slot_index, Record& r) {
  SlotAux& aux = ch.aux[slot_index];
  switch (r.type) {
    case RT_LAUNCH_KERNEL: {
      const HipApi* hip = orion_hip_api();
      if (!g_state.run_ahead_holders.load(std::memory_order_relaxed)) return false;
      if (!hip->hipGraphCreate || !hip->hipGraphAddKernelNode ||
          !hip->hipGraphKernelNodeSetParams || !hip->hipGraphKernelNodeGetParams)
        return false;
      if (r.u.launch.args == nullptr) return false;
      if (ch.holder_graph == nullptr &&
          hip->hipGraphCreate(&ch.holder_graph, 0) != hipSuccess) {
        ch.holder_graph = nullptr;
        (void)hip->hipGetLastError();
        return false;
      }
      // What this function does on the caller's thread must leave the thread's
      // last-error slot as it was: the caller reads it right after the launch
      // (a framework's launch check), and the runtime keeps an error there
      // across later successful calls.  An error already waiting there is the
      // caller's to read: leave everything alone.
      if (hip->hipPeekAtLastError && hip->hipPeekAtLastError() != hipSuccess) return false;
      hipKernelNodeParams p = {};
      p.func = const_cast<void*>(r.u.launch.func);
      p.gridDim = to_dim3(r.u.launch.grid);
      p.blockDim = to_dim3(r.u.launch.block);
      p.sharedMemBytes = (unsigned int)r.u.launch.shmem;
      p.kernelParams = r.u.launch.args;
      // A node keeps the kernel it was created for: the runtime checks new
      // parameters against the launch bounds of the kernel the node *holds*
      // (hipErrorLaunchFailure when that one's are smaller than the new block),
      // so nothing it does with a node that changes kernels is relied on here.
      // Another kernel through this slot gets a fresh node.
      if (aux.holder && (aux.holder_func != r.u.launch.func ||
                         hip->hipGraphKernelNodeSetParams(aux.holder, &p) != hipSuccess)) {
        if (aux.holder_func == r.u.launch.func) (void)hip->hipGetLastError();
        if (hip->hipGraphDestroyNode) (void)hip->hipGraphDestroyNode(aux.holder);
        aux.holder = nullptr;
      }
      if (!aux.holder) {
        if (hip->hipGraphAddKernelNode(&aux.holder, ch.holder_graph, nullptr, 0, &p) != hipSuccess) {
          aux.holder = nullptr;
          (void)hip->hipGetLastError();   // the real launch will tell the caller what is wrong
          return false;
        }
        aux.holder_func = r.u.launch.func;
      }
      hipKernelNodeParams owned = {};
      if (hip->hipGraphKernelNodeGetParams(aux.holder, &owned) != hipSuccess ||
          owned.kernelParams == nullptr || owned.kernelParams == r.u.launch.args) {
        (void)hip->hipGetLastError();
        return false;
      }
      r.u.launch.args = owned.kernelParams;
      return true;
    }
    case RT_MODULE_LAUNCH:
    case RT_EXT_MODULE_LAUNCH: {
      if (r.u.module.params != nullptr || r.u.module.extra == nullptr) return false;
      if (r.u.module.start != nullptr || r.u.module.stop != nullptr) return false;
      const void* buffer = nullptr;
      const size_t* size = nullptr;
      void** e = r.u.module.extra;
      // exactly {POINTER, buffer, SIZE, &size, END}, in either order: anything
      // else (a longer list, a tag this code does not know) is left to the caller
      int i = 0;
      for (; i < 4 && e[i] != HIP_LAUNCH_PARAM_END; i += 2) {
        if (e[i] == HIP_LAUNCH_PARAM_BUFFER_POINTER && !buffer) buffer = e[i + 1];
        else if (e[i] == HIP_LAUNCH_PARAM_BUFFER_SIZE && !size) size = (const size_t*)e[i + 1];
        else return false;
      }
      if (e[i] != HIP_LAUNCH_PARAM_END) return false;
      if (!buffer || !size || *size == 0 || *size > kInlineKernarg) return false;
      memcpy(aux.kernarg, buffer, *size);
      aux.kernarg_size = *size;
      aux.extra[0] = HIP_LAUNCH_PARAM_BUFFER_POINTER;
      aux.extra[1] = aux.kernarg;
      aux.extra[2] = HIP_LAUNCH_PARAM_BUFFER_SIZE;
      aux.extra[3] = &aux.kernarg_size;
      aux.extra[4] = HIP_LAUNCH_PARAM_END;
      r.u.module.extra = aux.extra;
      return true;
    }
    case RT_MEMCPY_ASYNC:
    case RT_MEMCPY_2D_ASYNC:
      return r.u.copy.kind == hipMemcpyDeviceToDevice;
    case RT_MEMSET_ASYNC:
    case RT_MEMSET_D32_ASYNC:
    case RT_MEMSET_D16_ASYNC:
    case RT_MEMSET_D8_ASYNC:
      return true;
    default:
      return false;
  }
}

// While the scheduler is outside its loop (between two phases of a job, or gone
// for good), records that were queued without a waiting caller have nobody to
// issue them: whoever needs them issued (a caller that waits for the client's
// work or for the whole device, the thread that disarms, a producer that finds
// the capture disarmed) runs them here, in order.  Between two phases they go
// where the client's latest record went, so that they stay in order with it;
// once the capture is disarmed, to the streams their calls named, like every
// later call of the client.  Stops at a record whose caller waits for it (that
// caller runs it itself, see submit) and as soon as the scheduler is on its way
// back into its loop: it sets scheduler_polling first and then passes through
// flush_lock (orion_capture_enter_loop), so either this function sees the flag
// before it touches a record or the scheduler waits until this function is done.
void flush_channel(ClientChannel& ch) {
  unsigned spins = 0;
  while (ch.flush_lock.exchange(1)) cpu_relax(spins);
  for (;;) {
    const bool armed = g_state.armed.load() != 0;
    if (armed && g_state.scheduler_polling.load() != 0) break;
    const uint64_t head = ch.head.load(std::memory_order_acquire);
    if (head == ch.tail.load(std::memory_order_acquire)) break;
    Record* rec = &ch.slots[head & (kQueueSlots - 1)];
    if (rec->status == kRecordIssued && rec_class_of(rec->type) != REC_KERNEL) {
      // the notice of a call its caller has already made (not a kernel, which the
      // policy must count): nothing to run, and nobody should wait for it
      ch.head.store(head + 1, std::memory_order_release);
      continue;
    }
    if (rec->status != kRecordDeferred) break;
    // Between two phases of a job a kernel stays where it is: the policy counts
    // every kernel record against the client's profile rows, and one issued
    // here would be missing from that count.  The scheduler takes it when it is
    // back in its loop; copies and fills, which the policy does not count, go.
    if (armed && rec_class_of(rec->type) == REC_KERNEL) break;
    hipStream_t stream = armed ? ch.last_stream.load(std::memory_order_acquire) : nullptr;
    if (stream == nullptr) stream = named_stream(*rec);
    ++tl_bypass;
    const int st = orion_execute_record(rec, stream);
    --tl_bypass;
    if (st != (int)hipSuccess)
      fprintf(stderr, "orion: a queued call (type %d) failed with HIP error %d while the "
                      "scheduler was outside its loop\n", rec->type, st);
    ch.head.store(head + 1, std::memory_order_release);
  }
  ch.flush_lock.store(0);
}

// Waits until the scheduler (or, while it is outside its loop, this thread) has
// issued client idx's queue up to ticket `upto`.
void wait_issued_upto(ClientChannel& ch, uint64_t upto) {
  unsigned spins = 0;
  unsigned long waited = 0;
  double idle_since = 0.0;
  while (ch.head.load(std::memory_order_acquire) < upto) {
    if (!g_state.armed.load(std::memory_order_acquire) ||
        !g_state.scheduler_polling.load(std::memory_order_acquire))
      flush_channel(ch);
    if (ch.head.load(std::memory_order_acquire) >= upto) break;
    cpu_relax(spins);
    // a kernel queued while the scheduler is between two phases stays queued
    // (flush_channel leaves it to the policy); if the scheduler never comes
    // back for it, say so instead of spinning forever
    if ((++waited & 0xfffff) != 0) continue;
    if (g_state.scheduler_polling.load(std::memory_order_acquire)) {
      idle_since = 0.0;
      continue;
    }
    const double now = monotonic_s();
    if (idle_since == 0.0) idle_since = now;
    if (now - idle_since > stuck_limit_s()) {
      fprintf(stderr, "orion: a client has waited %.0f s for records it queued ahead while the "
                      "scheduler is not polling; its iteration probably holds more kernel "
                      "records than its profile's num_kernels\n", now - idle_since);
      abort();
    }
  }
}

// Returns once every record the client has queued so far has been issued: what
// a client-side wait, event record or query must see before it looks at a
// stream.
void wait_until_issued(int idx) {
  ClientChannel& ch = g_state.channels[idx];
  // a client that issues its own calls queues notices of calls already made
  if (ch.direct_stream.load(std::memory_order_acquire) != nullptr) return;
  wait_issued_upto(ch, ch.tail.load(std::memory_order_acquire));
}

// ---- releases while records are queued ahead
//
// hipFree waits for the device before it releases memory, and so does every
// program that frees memory other work may still use.  The runtime cannot wait
// for records that still sit in a queue here -- and the caller need not be the
// client that queued them: a framework's caching allocator hands a block back to
// its pool as soon as the last kernel using it has been *launched*, and any
// thread of the process (another client, an autograd worker) may then return the
// pool's blocks to the runtime (PyTorch does after every convolution algorithm
// search).  The call must not wait for those records either: when the scheduler
// issues a best-effort record depends on the high-priority client's progress,
// and the caller may be that client, or hold a lock that client needs (the
// allocator's).  So a release that arrives while any client has records queued
// ahead is postponed: it is noted with each queue's position and carried out by
// a later caller of one of these entry points (or when the capture is disarmed)
// once every queue has been issued past that position.  The caller gets
// hipSuccess at once; the memory stays reserved a little longer.
enum PostponedKind { kPostFree, kPostHostFree, kPostFreeHost, kPostModuleUnload };

struct Postponed {
  int kind;
  void* what;
  uint64_t upto[kMaxClients];
};

std::mutex g_postponed_lock;
std::vector<Postponed> g_postponed;
std::atomic<size_t> g_postponed_count{0};

void postponed_fence() { std::lock_guard<std::mutex> hold(g_postponed_lock); }

int release_now(int kind, void* what) {
  const HipApi* hip = orion_hip_api();
  switch (kind) {
    case kPostFree: return (int)hip->hipFree(what);
    case kPostHostFree: return (int)hip->hipHostFree(what);
    case kPostFreeHost: return (int)hip->hipFreeHost(what);
    default: return (int)hip->hipModuleUnload((hipModule_t)what);
  }
}

// Carries out the postponed releases whose queues have moved on (all of them
// with `everything`: nothing is queued any more).
void run_postponed(bool everything) {
  if (g_postponed_count.load(std::memory_order_acquire) == 0) return;
  std::vector<Postponed> ready;
  {
    std::lock_guard<std::mutex> hold(g_postponed_lock);
    size_t keep = 0;
    for (size_t k = 0; k < g_postponed.size(); ++k) {
      bool ok = true;
      for (int i = 0; ok && !everything && i < g_state.num_clients; ++i)
        ok = g_state.channels[i].head.load(std::memory_order_acquire) >= g_postponed[k].upto[i];
      if (ok) ready.push_back(g_postponed[k]);
      else g_postponed[keep++] = g_postponed[k];
    }
    g_postponed.resize(keep);
    g_postponed_count.store(keep, std::memory_order_release);
  }
  for (const Postponed& p : ready) {
    const int st = release_now(p.kind, p.what);
    if (st != (int)hipSuccess)
      fprintf(stderr, "orion: a postponed release (kind %d) failed with HIP error %d\n", p.kind, st);
  }
}

// True (and the release noted) if some client has records queued ahead that the
// scheduler has not issued yet; false if the caller can go ahead.
bool postpone_release(int kind, void* what) {
  if (!g_state.armed.load(std::memory_order_acquire) ||
      !g_state.run_ahead.load(std::memory_order_acquire) || tl_bypass)
    return false;
  // each release waits for the device: never on the high-priority client's thread
  if (tl_client != g_state.num_clients - 1) run_postponed(false);
  Postponed p;
  p.kind = kind;
  p.what = what;
  bool outstanding = false;
  for (int i = 0; i < g_state.num_clients; ++i) {
    ClientChannel& ch = g_state.channels[i];
    p.upto[i] = ch.deferred_upto.load(std::memory_order_acquire);
    if (ch.head.load(std::memory_order_acquire) < p.upto[i]) outstanding = true;
  }
  if (!outstanding) return false;
  {
    std::lock_guard<std::mutex> hold(g_postponed_lock);
    if (g_state.armed.load(std::memory_order_acquire)) {
      g_postponed.push_back(p);
      g_postponed_count.store(g_postponed.size(), std::memory_order_release);
      return true;
    }
  }
  // disarmed in the meantime: what is still queued is being run by whoever
  // disarmed, without a policy in the way, so waiting for it is safe
  for (int i = 0; i < g_state.num_clients; ++i) wait_issued_upto(g_state.channels[i], p.upto[i]);
  return false;
}

// Pushes `r` to client idx's queue and waits until the scheduler has taken it
// (reference: intercept_temp.cpp:404-416) -- unless the client is a best-effort
// one and the record can carry its arguments with it: then the call returns as
// soon as the record is queued, with hipSuccess (the reference returns success
// from every queued call); a failure of the real call then ends the job where
// the scheduler issues it.  Returns the HIP status of the call.
int submit(int idx, Record& r, bool wait) {
  ClientChannel& ch = g_state.channels[idx];
  unsigned spins = 0;
  while (ch.producer_lock.exchange(1, std::memory_order_acquire)) cpu_relax(spins);
  const uint64_t ticket = ch.tail.load(std::memory_order_relaxed);
  // room in the ring: the scheduler's head is looked at only when the value
  // seen last no longer proves it (its line lives in the scheduler's cache)
  while (ticket - ch.head_seen >= kQueueSlots) {
    ch.head_seen = ch.head.load(std::memory_order_acquire);
    if (ticket - ch.head_seen < kQueueSlots) break;
    // a full queue with the scheduler gone (a job that ended early): make room by
    // running what is queued, never by writing over it
    if (!g_state.armed.load(std::memory_order_acquire)) flush_channel(ch);
    cpu_relax(spins);
  }
  const uint32_t slot_index = (uint32_t)(ticket & (kQueueSlots - 1));
  Record* slot = &ch.slots[slot_index];
  r.status = 0;
  r.cell = nullptr;
  if (hipStream_t direct = ch.direct_stream.load(std::memory_order_acquire)) {
    // The scheduler lets this client issue its own calls: run the call here, on
    // the stream the scheduler named, under the producer lock so that the
    // notices reach the queue in issue order; nobody waits for the notice.  The
    // notice is the record's type and, for a kernel, what was launched (kept for
    // the scheduler's reports): the scheduler reads nothing else of a call that
    // has been made.
    int st;
    if (orion_record_runs_on_caller(r.type)) {
      st = execute_on_caller(r, direct);
    } else {
      ++tl_bypass;
      st = orion_execute_record(&r, direct);
      --tl_bypass;
    }
    if (ch.last_stream.load(std::memory_order_relaxed) != direct)
      ch.last_stream.store(direct, std::memory_order_release);
    slot->type = r.type;
    slot->status = kRecordIssued;
    slot->cell = nullptr;
    slot->u.launch.func = record_function(r);   // which kernel: for the scheduler's reports
    ch.tail.store(ticket + 1, std::memory_order_release);
    ch.submitted.store(ch.submitted.load(std::memory_order_relaxed) + 1, std::memory_order_relaxed);
    ch.producer_lock.store(0, std::memory_order_release);
    return st;
  }
  const bool deferred = wait && idx < g_state.num_clients - 1 &&
                        g_state.run_ahead.load(std::memory_order_relaxed) &&
                        ch.may_run_ahead.load(std::memory_order_relaxed) &&
                        make_self_contained(ch, slot_index, r);
  // The outcome of a record its caller waits for comes back through storage of
  // this call, never through the slot: once the scheduler has retired the record
  // the slot is free, and another thread of this client (an autograd worker, a
  // thread launching ahead) may already be writing ticket + kQueueSlots into it.
  WaitCell cell = {kRecordPending, nullptr};
  if (deferred) r.status = kRecordDeferred;
  else if (wait) r.cell = &cell;
  *slot = r;
  ch.tail.store(ticket + 1, std::memory_order_release);
  ch.submitted.store(ch.submitted.load(std::memory_order_relaxed) + 1, std::memory_order_relaxed);
  if (deferred) {
    ch.deferred.store(ch.deferred.load(std::memory_order_relaxed) + 1, std::memory_order_relaxed);
    ch.deferred_upto.store(ticket + 1, std::memory_order_release);
  }
  ch.producer_lock.store(0, std::memory_order_release);
  if (deferred) {
    // disarmed in the meantime: nobody will come for the record
    if (!g_state.armed.load(std::memory_order_acquire)) flush_channel(ch);
    return (int)hipSuccess;
  }
  if (!wait) return (int)hipSuccess;

  spins = 0;
  unsigned long waited = 0;
  double idle_since = 0.0;
  while (ch.head.load(std::memory_order_acquire) <= ticket) {
    // Clients submit only while the scheduler polls; between two calls of
    // schedule() they wait at a rendezvous.  A record that sits here for long
    // with the scheduler outside its loop can never be taken (the usual cause:
    // the iteration holds more kernel records than the client's profile names,
    // so the scheduler counted it complete and left): say so instead of
    // spinning forever, as the reference would (intercept_temp.cpp:404-416).
    if ((++waited & 0xfffff) == 0) {
      if (g_state.scheduler_polling.load(std::memory_order_acquire)) {
        idle_since = 0.0;
      } else {
        const double now = monotonic_s();
        if (idle_since == 0.0) idle_since = now;
        if (now - idle_since > stuck_limit_s()) {
          fprintf(stderr,
                  "orion: client %d has had a record (type %d) queued for %.0f s while the "
                  "scheduler is not polling; its iteration probably holds more kernel records "
                  "than its profile's num_kernels\n", idx, r.type, now - idle_since);
          abort();
        }
      }
    }
    if (!g_state.scheduler_polling.load(std::memory_order_acquire) &&
        g_state.armed.load(std::memory_order_acquire) && rec_class_of(r.type) != REC_KERNEL) {
      // Between two phases of a job nobody polls, and the scheduler thread will
      // not be back before this client has reached the rendezvous (a copy that
      // reads a result back after the last kernel of a warm-up iteration: the
      // reference's caller would spin forever, intercept_temp.cpp:404-416).  A
      // record the policy does not count is run here, in order, where the
      // client's latest record went -- under the flush lock, through which the
      // scheduler passes after raising scheduler_polling on its way back in, so
      // that exactly one of the two runs it.
      flush_channel(ch);   // records queued ahead of this one that nobody waits for
      unsigned lock_spins = 0;
      while (ch.flush_lock.exchange(1)) cpu_relax(lock_spins);
      const bool mine = !g_state.scheduler_polling.load() && g_state.armed.load() &&
                        ch.head.load(std::memory_order_acquire) == ticket;
      int st = 0;
      if (mine) {
        hipStream_t stream = ch.last_stream.load(std::memory_order_acquire);
        if (stream == nullptr) stream = named_stream(r);
        if (orion_record_runs_on_caller(r.type)) {
          st = execute_on_caller(r, stream);
        } else {
          ++tl_bypass;
          st = orion_execute_record(&r, stream);
          --tl_bypass;
        }
        ch.head.store(ticket + 1, std::memory_order_release);
      }
      ch.flush_lock.store(0);
      if (mine) return st;
    }
    if (!g_state.armed.load(std::memory_order_acquire)) {
      // The scheduler has left its loop for good.  Whatever it did not take is
      // run here, in order, on the stream the call named: first the records
      // queued ahead of this one that nobody waits for, then this one.  (The
      // slot still holds this record while head == ticket: nothing can be
      // written over a record that has not been retired.)
      flush_channel(ch);
      if (ch.head.load(std::memory_order_acquire) > ticket) break;
      if (ch.head.load(std::memory_order_acquire) < ticket) {
        cpu_relax(spins);   // another caller's record is ahead; it runs it itself
        continue;
      }
      int st;
      if (orion_record_runs_on_caller(r.type)) {
        st = execute_on_caller(r, named_stream(r));
      } else {
        ++tl_bypass;
        st = orion_execute_record(&r, named_stream(r));
        --tl_bypass;
      }
      ch.head.store(ticket + 1, std::memory_order_release);
      return st;
    }
    cpu_relax(spins);
  }
  // the scheduler wrote the cell before it moved head past the ticket
  if (cell.status == kRecordPending) {
    fprintf(stderr, "orion: client %d: record %llu (type %d) was retired without an outcome\n",
            idx, (unsigned long long)ticket, r.type);
    abort();
  }
  if (cell.status == ORION_GRANTED_TO_CALLER)
    return execute_on_caller(r, cell.sync_stream);
  return cell.status;
}

// Stream a client-side wait or event record is redirected to: where the
// client's latest record went.
inline hipStream_t redirected(int idx, hipStream_t given) {
  hipStream_t s = g_state.channels[idx].last_stream.load(std::memory_order_acquire);
  return s ? s : given;
}

}  // namespace

// ---------------------------------------------------------------------------
// Interposed HIP entry points.  Each one: find the client; not a client ->
// call the real function; else build the record, hand it over, return the
// status the scheduler (or the granted call) produced.
// ---------------------------------------------------------------------------
extern "C" {

hipError_t hipLaunchKernel(const void* f, dim3 grid, dim3 block, void** args,
                           size_t shmem, hipStream_t stream) {
  CallTimer timer;
  const int idx = client_for_call(stream);
  if (idx < 0) return orion_hip_api()->hipLaunchKernel(f, grid, block, args, shmem, stream);
  Record r;
  r.type = RT_LAUNCH_KERNEL;
  r.u.launch = {f, from_dim3(grid), from_dim3(block), args, shmem, stream, nullptr, nullptr, 0};
  return (hipError_t)submit(idx, r, true);
}

hipError_t hipExtLaunchKernel(const void* f, dim3 grid, dim3 block, void** args,
                              size_t shmem, hipStream_t stream, hipEvent_t start,
                              hipEvent_t stop_ev, int flags) {
  const int idx = client_for_call(stream);
  if (idx < 0)
    return orion_hip_api()->hipExtLaunchKernel(f, grid, block, args, shmem, stream,
                                               start, stop_ev, flags);
  Record r;
  r.type = RT_EXT_LAUNCH_KERNEL;
  r.u.launch = {f, from_dim3(grid), from_dim3(block), args, shmem, stream, start, stop_ev, flags};
  return (hipError_t)submit(idx, r, true);
}

hipError_t hipLaunchCooperativeKernel(const void* f, dim3 grid, dim3 block,
                                      void** args, unsigned int shmem,
                                      hipStream_t stream) {
  const int idx = client_for_call(stream);
  if (idx < 0)
    return orion_hip_api()->hipLaunchCooperativeKernel(f, grid, block, args, shmem, stream);
  Record r;
  r.type = RT_COOP_LAUNCH_KERNEL;
  r.u.launch = {f, from_dim3(grid), from_dim3(block), args, shmem, stream, nullptr, nullptr, 0};
  return (hipError_t)submit(idx, r, true);
}

hipError_t hipModuleLaunchKernel(hipFunction_t f, unsigned int gx, unsigned int gy,
                                 unsigned int gz, unsigned int bx, unsigned int by,
                                 unsigned int bz, unsigned int shmem,
                                 hipStream_t stream, void** params, void** extra) {
  CallTimer timer;
  const int idx = client_for_call(stream);
  if (idx < 0)
    return orion_hip_api()->hipModuleLaunchKernel(f, gx, gy, gz, bx, by, bz, shmem,
                                                  stream, params, extra);
  Record r;
  r.type = RT_MODULE_LAUNCH;
  r.u.module = {f, gx, gy, gz, bx, by, bz, shmem, stream, params, extra, nullptr, nullptr, 0};
  return (hipError_t)submit(idx, r, true);
}

hipError_t hipExtModuleLaunchKernel(hipFunction_t f, uint32_t gx, uint32_t gy,
                                    uint32_t gz, uint32_t bx, uint32_t by,
                                    uint32_t bz, size_t shmem, hipStream_t stream,
                                    void** params, void** extra, hipEvent_t start,
                                    hipEvent_t stop_ev, uint32_t flags) {
  CallTimer timer;
  const int idx = client_for_call(stream);
  if (idx < 0)
    return orion_hip_api()->hipExtModuleLaunchKernel(f, gx, gy, gz, bx, by, bz, shmem,
                                                     stream, params, extra, start,
                                                     stop_ev, flags);
  Record r;
  r.type = RT_EXT_MODULE_LAUNCH;
  r.u.module = {f, gx, gy, gz, bx, by, bz, shmem, stream, params, extra, start, stop_ev, flags};
  return (hipError_t)submit(idx, r, true);
}

hipError_t hipHccModuleLaunchKernel(hipFunction_t f, uint32_t gx, uint32_t gy,
                                    uint32_t gz, uint32_t bx, uint32_t by,
                                    uint32_t bz, size_t shmem, hipStream_t stream,
                                    void** params, void** extra, hipEvent_t start,
                                    hipEvent_t stop_ev) {
  return hipExtModuleLaunchKernel(f, gx, gy, gz, bx, by, bz, shmem, stream, params,
                                  extra, start, stop_ev, 0);
}

hipError_t hipModuleLaunchCooperativeKernel(hipFunction_t f, unsigned int gx,
                                            unsigned int gy, unsigned int gz,
                                            unsigned int bx, unsigned int by,
                                            unsigned int bz, unsigned int shmem,
                                            hipStream_t stream, void** params) {
  const int idx = client_for_call(stream);
  if (idx < 0)
    return orion_hip_api()->hipModuleLaunchCooperativeKernel(f, gx, gy, gz, bx, by, bz,
                                                             shmem, stream, params);
  Record r;
  r.type = RT_MODULE_COOP_LAUNCH;
  r.u.module = {f, gx, gy, gz, bx, by, bz, shmem, stream, params, nullptr, nullptr, nullptr, 0};
  return (hipError_t)submit(idx, r, true);
}

// A captured graph is one record: the policy places and admits it as a whole
// (its profile row carries the graph's duration), which is what a launch-bound
// inference client wants -- one hand-off and one launch per request.
hipError_t hipGraphLaunch(hipGraphExec_t exec, hipStream_t stream) {
  const int idx = client_for_call(stream);
  if (idx < 0) return orion_hip_api()->hipGraphLaunch(exec, stream);
  Record r;
  r.type = RT_GRAPH_LAUNCH;
  r.u.graph = {exec, stream};
  return (hipError_t)submit(idx, r, true);
}

hipError_t hipMalloc(void** ptr, size_t size) {
  const int idx = client_for_call(nullptr);
  if (idx < 0) return orion_hip_api()->hipMalloc(ptr, size);
  if (g_state.run_ahead.load(std::memory_order_acquire)) {
    // postponed releases wait for the device: not on the high-priority client
    if (idx < g_state.num_clients - 1) run_postponed(false);
    // An allocation is ordered against nothing, and its caller may hold a lock
    // the high-priority client needs (a caching allocator calls it under its
    // own): it must not wait behind records queued ahead, whose turn depends on
    // that client's progress.  With nothing queued it is a record like any
    // other, which every policy dispatches in the poll that sees it.
    ClientChannel& ch = g_state.channels[idx];
    if (ch.head.load(std::memory_order_acquire) < ch.deferred_upto.load(std::memory_order_acquire)) {
      hipError_t err = orion_hip_api()->hipMalloc(ptr, size);
      if (err == hipErrorOutOfMemory && g_postponed_count.load(std::memory_order_acquire) > 0) {
        // memory the caller believes free may still be held by postponed
        // releases: carry out the ones whose queues have moved on and try once
        // more (waiting for the others could wait for this very caller)
        (void)orion_hip_api()->hipGetLastError();
        run_postponed(false);
        err = orion_hip_api()->hipMalloc(ptr, size);
      }
      return err;
    }
  }
  Record r;
  r.type = RT_MALLOC;
  r.u.malloc_ = {ptr, size, nullptr};
  return (hipError_t)submit(idx, r, true);
}

// Stream-ordered allocation (an optional allocator backend of PyTorch, rocBLAS
// workspaces): ordered on the stream the client's work has been moved to.
hipError_t hipMallocAsync(void** ptr, size_t size, hipStream_t stream) {
  const int idx = client_for_call(stream);
  if (idx < 0 || !orion_hip_api()->hipMallocAsync)
    return orion_hip_api()->hipMallocAsync ? orion_hip_api()->hipMallocAsync(ptr, size, stream)
                                           : hipErrorNotSupported;
  Record r;
  r.type = RT_MALLOC_ASYNC;
  r.u.malloc_ = {ptr, size, stream};
  return (hipError_t)submit(idx, r, true);
}

hipError_t hipFreeAsync(void* ptr, hipStream_t stream) {
  const int idx = client_for_call(stream);
  if (idx < 0 || !orion_hip_api()->hipFreeAsync)
    return orion_hip_api()->hipFreeAsync ? orion_hip_api()->hipFreeAsync(ptr, stream)
                                         : hipErrorNotSupported;
  Record r;
  r.type = RT_FREE_ASYNC;
  r.u.free_ = {ptr, stream};
  return (hipError_t)submit(idx, r, true);
}

hipError_t hipFree(void* ptr) {
  // whoever calls: the memory may still be named by records queued ahead
  if (postpone_release(kPostFree, ptr)) return hipSuccess;
  const int idx = client_for_call(nullptr);
  if (idx < 0) return orion_hip_api()->hipFree(ptr);
  Record r;
  r.type = RT_FREE;
  r.u.free_ = {ptr, nullptr};
  return (hipError_t)submit(idx, r, true);
}

hipError_t hipMemcpy(void* dst, const void* src, size_t bytes, hipMemcpyKind kind) {
  const int idx = client_for_call(nullptr);
  if (idx < 0) return orion_hip_api()->hipMemcpy(dst, src, bytes, kind);
  Record r;
  r.type = RT_MEMCPY;
  r.u.copy = {dst, src, bytes, kind, nullptr, 0, 0, 0, 0};
  return (hipError_t)submit(idx, r, true);
}

hipError_t hipMemcpyAsync(void* dst, const void* src, size_t bytes,
                          hipMemcpyKind kind, hipStream_t stream) {
  CallTimer timer;
  const int idx = client_for_call(stream);
  if (idx < 0) return orion_hip_api()->hipMemcpyAsync(dst, src, bytes, kind, stream);
  Record r;
  r.type = RT_MEMCPY_ASYNC;
  r.u.copy = {dst, src, bytes, kind, stream, 0, 0, 0, 0};
  return (hipError_t)submit(idx, r, true);
}

hipError_t hipMemcpyWithStream(void* dst, const void* src, size_t bytes,
                               hipMemcpyKind kind, hipStream_t stream) {
  const int idx = client_for_call(stream);
  if (idx < 0) return orion_hip_api()->hipMemcpyWithStream(dst, src, bytes, kind, stream);
  Record r;
  r.type = RT_MEMCPY_WITH_STREAM;
  r.u.copy = {dst, src, bytes, kind, stream, 0, 0, 0, 0};
  return (hipError_t)submit(idx, r, true);
}

hipError_t hipMemcpy2DAsync(void* dst, size_t dpitch, const void* src, size_t spitch,
                            size_t width, size_t height, hipMemcpyKind kind,
                            hipStream_t stream) {
  const int idx = client_for_call(stream);
  if (idx < 0)
    return orion_hip_api()->hipMemcpy2DAsync(dst, dpitch, src, spitch, width, height,
                                             kind, stream);
  Record r;
  r.type = RT_MEMCPY_2D_ASYNC;
  r.u.copy = {dst, src, 0, kind, stream, dpitch, spitch, width, height};
  return (hipError_t)submit(idx, r, true);
}

hipError_t hipMemcpy2D(void* dst, size_t dpitch, const void* src, size_t spitch,
                       size_t width, size_t height, hipMemcpyKind kind) {
  const int idx = client_for_call(nullptr);
  if (idx < 0)
    return orion_hip_api()->hipMemcpy2D(dst, dpitch, src, spitch, width, height, kind);
  Record r;
  r.type = RT_MEMCPY_2D;
  r.u.copy = {dst, src, 0, kind, nullptr, dpitch, spitch, width, height};
  return (hipError_t)submit(idx, r, true);
}

hipError_t hipMemset(void* dst, int value, size_t bytes) {
  const int idx = client_for_call(nullptr);
  if (idx < 0) return orion_hip_api()->hipMemset(dst, value, bytes);
  Record r;
  r.type = RT_MEMSET;
  r.u.set = {dst, value, bytes, nullptr};
  return (hipError_t)submit(idx, r, true);
}

hipError_t hipMemsetAsync(void* dst, int value, size_t bytes, hipStream_t stream) {
  const int idx = client_for_call(stream);
  if (idx < 0) return orion_hip_api()->hipMemsetAsync(dst, value, bytes, stream);
  Record r;
  r.type = RT_MEMSET_ASYNC;
  r.u.set = {dst, value, bytes, stream};
  return (hipError_t)submit(idx, r, true);
}

hipError_t hipMemsetD32Async(hipDeviceptr_t dst, int value, size_t count,
                             hipStream_t stream) {
  const int idx = client_for_call(stream);
  if (idx < 0) return orion_hip_api()->hipMemsetD32Async(dst, value, count, stream);
  Record r;
  r.type = RT_MEMSET_D32_ASYNC;
  r.u.set = {(void*)dst, value, count, stream};
  return (hipError_t)submit(idx, r, true);
}

hipError_t hipMemsetD16Async(hipDeviceptr_t dst, unsigned short value, size_t count,
                             hipStream_t stream) {
  const int idx = client_for_call(stream);
  if (idx < 0) return orion_hip_api()->hipMemsetD16Async(dst, value, count, stream);
  Record r;
  r.type = RT_MEMSET_D16_ASYNC;
  r.u.set = {(void*)dst, (int)value, count, stream};
  return (hipError_t)submit(idx, r, true);
}

hipError_t hipMemsetD8Async(hipDeviceptr_t dst, unsigned char value, size_t count,
                            hipStream_t stream) {
  const int idx = client_for_call(stream);
  if (idx < 0) return orion_hip_api()->hipMemsetD8Async(dst, value, count, stream);
  Record r;
  r.type = RT_MEMSET_D8_ASYNC;
  r.u.set = {(void*)dst, (int)value, count, stream};
  return (hipError_t)submit(idx, r, true);
}

// -- waits and event records made by a client follow its work to the stream the
// scheduler put it on (the reference leaves them on the caller's idle stream),
// after every record the client has queued so far has been issued.

hipError_t hipStreamSynchronize(hipStream_t stream) {
  const HipApi* hip = orion_hip_api();
  const int idx = client_for_call(stream);
  if (idx < 0) return hip->hipStreamSynchronize(stream);
  wait_until_issued(idx);
  hipStream_t s = redirected(idx, stream);
  hipError_t err = hip->hipStreamSynchronize(s);
  if (err == hipSuccess && s != stream) err = hip->hipStreamSynchronize(stream);
  return err;
}

hipError_t hipStreamQuery(hipStream_t stream) {
  const HipApi* hip = orion_hip_api();
  const int idx = client_for_call(stream);
  if (idx < 0) return hip->hipStreamQuery(stream);
  {
    ClientChannel& ch = g_state.channels[idx];
    if (ch.direct_stream.load(std::memory_order_acquire) == nullptr &&
        ch.head.load(std::memory_order_acquire) < ch.tail.load(std::memory_order_acquire))
      return hipErrorNotReady;   // work still queued here has certainly not completed
  }
  return hip->hipStreamQuery(redirected(idx, stream));
}

hipError_t hipEventRecord(hipEvent_t event, hipStream_t stream) {
  const HipApi* hip = orion_hip_api();
  const int idx = client_for_call(stream);
  if (idx < 0) return hip->hipEventRecord(event, stream);
  wait_until_issued(idx);
  return hip->hipEventRecord(event, redirected(idx, stream));
}

hipError_t hipStreamWaitEvent(hipStream_t stream, hipEvent_t event, unsigned int flags) {
  const HipApi* hip = orion_hip_api();
  const int idx = client_for_call(stream);
  if (idx < 0) return hip->hipStreamWaitEvent(stream, event, flags);
  wait_until_issued(idx);
  return hip->hipStreamWaitEvent(redirected(idx, stream), event, flags);
}

// -- other calls that name a stream follow the client's work in the same way:
// host callbacks, stream memory operations and copies to and from device
// symbols (none has a counterpart in the reference, which leaves whatever it
// does not interpose on the caller's own idle stream, unordered against the
// work its scheduler moved elsewhere).  They are not records: the policy never
// sees them, like the waits and event records above.

hipError_t hipLaunchHostFunc(hipStream_t stream, hipHostFn_t fn, void* user_data) {
  const HipApi* hip = orion_hip_api();
  if (!hip->hipLaunchHostFunc) return hipErrorNotSupported;
  const int idx = client_for_call(stream);
  if (idx < 0) return hip->hipLaunchHostFunc(stream, fn, user_data);
  wait_until_issued(idx);
  return hip->hipLaunchHostFunc(redirected(idx, stream), fn, user_data);
}

hipError_t hipStreamWriteValue32(hipStream_t stream, void* ptr, uint32_t value,
                                 unsigned int flags) {
  const HipApi* hip = orion_hip_api();
  if (!hip->hipStreamWriteValue32) return hipErrorNotSupported;
  const int idx = client_for_call(stream);
  if (idx < 0) return hip->hipStreamWriteValue32(stream, ptr, value, flags);
  wait_until_issued(idx);
  return hip->hipStreamWriteValue32(redirected(idx, stream), ptr, value, flags);
}

hipError_t hipStreamWriteValue64(hipStream_t stream, void* ptr, uint64_t value,
                                 unsigned int flags) {
  const HipApi* hip = orion_hip_api();
  if (!hip->hipStreamWriteValue64) return hipErrorNotSupported;
  const int idx = client_for_call(stream);
  if (idx < 0) return hip->hipStreamWriteValue64(stream, ptr, value, flags);
  wait_until_issued(idx);
  return hip->hipStreamWriteValue64(redirected(idx, stream), ptr, value, flags);
}

hipError_t hipStreamWaitValue32(hipStream_t stream, void* ptr, uint32_t value,
                                unsigned int flags, uint32_t mask) {
  const HipApi* hip = orion_hip_api();
  if (!hip->hipStreamWaitValue32) return hipErrorNotSupported;
  const int idx = client_for_call(stream);
  if (idx < 0) return hip->hipStreamWaitValue32(stream, ptr, value, flags, mask);
  wait_until_issued(idx);
  return hip->hipStreamWaitValue32(redirected(idx, stream), ptr, value, flags, mask);
}

hipError_t hipStreamWaitValue64(hipStream_t stream, void* ptr, uint64_t value,
                                unsigned int flags, uint64_t mask) {
  const HipApi* hip = orion_hip_api();
  if (!hip->hipStreamWaitValue64) return hipErrorNotSupported;
  const int idx = client_for_call(stream);
  if (idx < 0) return hip->hipStreamWaitValue64(stream, ptr, value, flags, mask);
  wait_until_issued(idx);
  return hip->hipStreamWaitValue64(redirected(idx, stream), ptr, value, flags, mask);
}

hipError_t hipMemcpyToSymbolAsync(const void* symbol, const void* src, size_t bytes,
                                  size_t offset, hipMemcpyKind kind, hipStream_t stream) {
  const HipApi* hip = orion_hip_api();
  if (!hip->hipMemcpyToSymbolAsync) return hipErrorNotSupported;
  const int idx = client_for_call(stream);
  if (idx < 0) return hip->hipMemcpyToSymbolAsync(symbol, src, bytes, offset, kind, stream);
  wait_until_issued(idx);
  return hip->hipMemcpyToSymbolAsync(symbol, src, bytes, offset, kind, redirected(idx, stream));
}

hipError_t hipMemcpyFromSymbolAsync(void* dst, const void* symbol, size_t bytes, size_t offset,
                                    hipMemcpyKind kind, hipStream_t stream) {
  const HipApi* hip = orion_hip_api();
  if (!hip->hipMemcpyFromSymbolAsync) return hipErrorNotSupported;
  const int idx = client_for_call(stream);
  if (idx < 0) return hip->hipMemcpyFromSymbolAsync(dst, symbol, bytes, offset, kind, stream);
  wait_until_issued(idx);
  return hip->hipMemcpyFromSymbolAsync(dst, symbol, bytes, offset, kind, redirected(idx, stream));
}

// The blocking forms: after the client's earlier work, wherever it is.
hipError_t hipMemcpyToSymbol(const void* symbol, const void* src, size_t bytes, size_t offset,
                             hipMemcpyKind kind) {
  const HipApi* hip = orion_hip_api();
  if (!hip->hipMemcpyToSymbol) return hipErrorNotSupported;
  const int idx = client_for_call(nullptr);
  if (idx >= 0) {
    wait_until_issued(idx);
    if (hipStream_t s = redirected(idx, nullptr)) {
      hipError_t err = hip->hipStreamSynchronize(s);
      if (err != hipSuccess) return err;
    }
  }
  return hip->hipMemcpyToSymbol(symbol, src, bytes, offset, kind);
}

hipError_t hipMemcpyFromSymbol(void* dst, const void* symbol, size_t bytes, size_t offset,
                               hipMemcpyKind kind) {
  const HipApi* hip = orion_hip_api();
  if (!hip->hipMemcpyFromSymbol) return hipErrorNotSupported;
  const int idx = client_for_call(nullptr);
  if (idx >= 0) {
    wait_until_issued(idx);
    if (hipStream_t s = redirected(idx, nullptr)) {
      hipError_t err = hip->hipStreamSynchronize(s);
      if (err != hipSuccess) return err;
    }
  }
  return hip->hipMemcpyFromSymbol(dst, symbol, bytes, offset, kind);
}

// A client that waits for the whole device waits for its own queued records too.
hipError_t hipDeviceSynchronize(void) {
  const HipApi* hip = orion_hip_api();
  const int idx = client_for_call(nullptr);
  if (idx >= 0) wait_until_issued(idx);
  return hip->hipDeviceSynchronize();
}

// Releasing a code object or host memory that queued launches may still name:
// postponed like a hipFree while records are queued ahead (the runtime keeps
// what an issued launch needs alive by itself).
hipError_t hipModuleUnload(hipModule_t module) {
  const HipApi* hip = orion_hip_api();
  if (!hip->hipModuleUnload) return hipErrorNotSupported;
  if (postpone_release(kPostModuleUnload, (void*)module)) return hipSuccess;
  return hip->hipModuleUnload(module);
}

hipError_t hipHostFree(void* ptr) {
  const HipApi* hip = orion_hip_api();
  if (!hip->hipHostFree) return hipErrorNotSupported;
  if (postpone_release(kPostHostFree, ptr)) return hipSuccess;
  return hip->hipHostFree(ptr);
}

hipError_t hipFreeHost(void* ptr) {
  const HipApi* hip = orion_hip_api();
  if (!hip->hipFreeHost) return hipErrorNotSupported;
  if (postpone_release(kPostFreeHost, ptr)) return hipSuccess;
  return hip->hipFreeHost(ptr);
}

}  // extern "C"
