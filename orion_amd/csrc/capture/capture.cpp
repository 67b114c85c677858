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

#include <dlfcn.h>
#include <immintrin.h>
#include <sched.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>
#include <sys/syscall.h>
#include <time.h>
#include <unistd.h>

using namespace orion;

namespace {

CaptureState g_state;

constexpr int kNotClient = -1;
constexpr int kUncached = -2;

thread_local uint32_t tl_epoch = 0;
thread_local int tl_client = kUncached;
// Set while a client thread runs a call the scheduler granted back to it, so
// the nested real call is not captured again.
thread_local int tl_bypass = 0;

inline dim3 to_dim3(const Dim3& d) { return dim3(d.x, d.y, d.z); }
inline Dim3 from_dim3(const dim3& d) { return Dim3{d.x, d.y, d.z}; }

inline void cpu_relax(unsigned& spins) {
  _mm_pause();
  if ((++spins & 0x3ff) == 0) sched_yield();
}

// Thread placement (reference: utils_interc.cpp:36-49 pins client idx, and the
// scheduler as idx N, to CPU idx + 1 the first time it is identified).  Here
// slot s is the (s + 1)-th CPU the process may run on, the first one staying
// with the interpreter's other threads; the masks in force before are put back
// when the capture is disarmed.  ORION_PIN_THREADS=0 leaves placement to the
// kernel, as does a CPU set too small for one CPU per slot.
struct Pinning {
  bool on = false;
  int cpus[kMaxClients + 2];
  pid_t tid[kMaxClients + 1];
  cpu_set_t before[kMaxClients + 1];
};
Pinning g_pin;

void pinning_reset(int slots) {
  for (pid_t& t : g_pin.tid) t = 0;
  const char* env = getenv("ORION_PIN_THREADS");
  g_pin.on = false;
  if (env && atoi(env) == 0) return;
  cpu_set_t allowed;
  if (sched_getaffinity(getpid(), sizeof allowed, &allowed) != 0) return;
  int n = 0;
  for (int c = 0; c < CPU_SETSIZE && n < slots + 1; ++c)
    if (CPU_ISSET(c, &allowed)) g_pin.cpus[n++] = c;
  g_pin.on = n == slots + 1;
}

void pin_caller(int slot, pid_t tid) {
  if (!g_pin.on || g_pin.tid[slot] == tid) return;
  if (sched_getaffinity(0, sizeof(cpu_set_t), &g_pin.before[slot]) != 0) return;
  cpu_set_t one;
  CPU_ZERO(&one);
  CPU_SET(g_pin.cpus[slot + 1], &one);
  if (sched_setaffinity(0, sizeof one, &one) == 0) g_pin.tid[slot] = tid;
}

void pinning_undo() {
  for (int s = 0; s <= kMaxClients; ++s) {
    if (g_pin.tid[s] == 0) continue;
    // a thread that has ended leaves ESRCH, which is fine
    (void)sched_setaffinity(g_pin.tid[s], sizeof(cpu_set_t), &g_pin.before[s]);
    g_pin.tid[s] = 0;
  }
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
  if (!g_state.armed.load(std::memory_order_acquire) || tl_bypass) return kNotClient;
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
      if (s.load(std::memory_order_relaxed) == stream) return i;
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
    ch.released_iters.store(0);
    ch.stop.store(0);
    ch.stop_ack.store(0);
    ch.last_stream.store(nullptr);
    ch.direct_stream.store(nullptr);
    ch.submitted.store(0);
    ch.block_calls.store(0);
    // own_streams survive: a client may register its stream before setup runs
  }
  g_state.epoch.fetch_add(1, std::memory_order_acq_rel);
  g_state.armed.store(1, std::memory_order_release);
}

void orion_capture_disarm(void) {
  g_state.armed.store(0, std::memory_order_release);
  g_state.epoch.fetch_add(1, std::memory_order_acq_rel);
  pinning_undo();
}

// The CPU the capture pinned the calling thread to, or -1.
int orion_pinned_cpu(void) {
  const pid_t tid = (pid_t)syscall(SYS_gettid);
  for (int s = 0; s <= kMaxClients; ++s)
    if (g_pin.tid[s] == tid) return g_pin.cpus[s + 1];
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

// The client a call naming `stream` from the calling thread would be queued
// for, or a negative value when it would go straight to the runtime.
int orion_client_of_stream(void* stream) { return client_for_call((hipStream_t)stream); }

// While on, the calling thread's HIP calls go straight to the runtime: used by
// a client for work that must not count as part of an iteration (building the
// model, library auto-tuning runs whose kernel count is not reproducible).
void orion_thread_passthrough(int on) { tl_bypass = on ? 1 : 0; }

// -- control calls of the client loops (reference: intercept_temp.cpp:124-142)

// Returns once the scheduler has released iteration `it` of the calling client.
void block(int it) {
  const int idx = client_for_call(nullptr);
  if (idx < 0) return;  // not armed, or not a client: nothing to wait for
  ClientChannel& ch = g_state.channels[idx];
  ch.block_calls.store((int64_t)it + 1, std::memory_order_release);
  unsigned spins = 0;
  while (ch.released_iters.load(std::memory_order_acquire) <= (int64_t)it) {
    if (!g_state.armed.load(std::memory_order_acquire)) return;
    cpu_relax(spins);
  }
}

// Non-zero once the scheduler has asked the calling client to stop; the call
// acknowledges the request.  (The reference returns a C bool that its ctypes
// caller reads as int; an int is returned here.)
int stop(void) {
  const int idx = client_for_call(nullptr);
  if (idx < 0) return 0;
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

// Pushes `r` to client idx's queue and waits until the scheduler has taken it
// (or, for free(), only until it is queued: intercept_temp.cpp:214-236).
// Returns the HIP status of the call.
int submit(int idx, Record& r, bool wait) {
  ClientChannel& ch = g_state.channels[idx];
  unsigned spins = 0;
  while (ch.producer_lock.exchange(1, std::memory_order_acquire)) cpu_relax(spins);
  const uint64_t ticket = ch.tail.load(std::memory_order_relaxed);
  while (ticket - ch.head.load(std::memory_order_acquire) >= kQueueSlots) {
    if (!g_state.armed.load(std::memory_order_acquire)) break;
    cpu_relax(spins);
  }
  Record* slot = &ch.slots[ticket & (kQueueSlots - 1)];
  r.status = 0;
  r.sync_stream = nullptr;
  if (hipStream_t direct = ch.direct_stream.load(std::memory_order_acquire)) {
    // The scheduler lets this client issue its own calls: run the call here, on
    // the stream the scheduler named, under the producer lock so that the
    // notices reach the queue in issue order; nobody waits for the notice.
    int st;
    if (orion_record_runs_on_caller(r.type)) {
      st = execute_on_caller(r, direct);
    } else {
      ++tl_bypass;
      st = orion_execute_record(&r, direct);
      --tl_bypass;
    }
    ch.last_stream.store(direct, std::memory_order_release);
    r.status = kRecordIssued;
    *slot = r;
    ch.tail.store(ticket + 1, std::memory_order_release);
    ch.submitted.fetch_add(1, std::memory_order_relaxed);
    ch.producer_lock.store(0, std::memory_order_release);
    return st;
  }
  *slot = r;
  ch.tail.store(ticket + 1, std::memory_order_release);
  ch.submitted.fetch_add(1, std::memory_order_relaxed);
  ch.producer_lock.store(0, std::memory_order_release);
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
        timespec ts;
        clock_gettime(CLOCK_MONOTONIC, &ts);
        const double now = (double)ts.tv_sec + 1e-9 * (double)ts.tv_nsec;
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
    if (!g_state.armed.load(std::memory_order_acquire)) {
      // The scheduler has left its loop for good.  Whatever it did not take is
      // run here, in order, on the stream the call named.
      if (ch.head.load(std::memory_order_acquire) > ticket) break;
      int st;
      if (orion_record_runs_on_caller(slot->type)) {
        st = execute_on_caller(*slot, named_stream(*slot));
      } else {
        ++tl_bypass;
        st = orion_execute_record(slot, named_stream(*slot));
        --tl_bypass;
      }
      ch.head.store(ticket + 1, std::memory_order_release);
      return st;
    }
    cpu_relax(spins);
  }
  if (slot->status == ORION_GRANTED_TO_CALLER)
    return execute_on_caller(r, slot->sync_stream);
  return slot->status;
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
// scheduler put it on (the reference leaves them on the caller's idle stream).

hipError_t hipStreamSynchronize(hipStream_t stream) {
  const HipApi* hip = orion_hip_api();
  const int idx = client_for_call(stream);
  if (idx < 0) return hip->hipStreamSynchronize(stream);
  hipStream_t s = redirected(idx, stream);
  hipError_t err = hip->hipStreamSynchronize(s);
  if (err == hipSuccess && s != stream) err = hip->hipStreamSynchronize(stream);
  return err;
}

hipError_t hipStreamQuery(hipStream_t stream) {
  const HipApi* hip = orion_hip_api();
  const int idx = client_for_call(stream);
  if (idx < 0) return hip->hipStreamQuery(stream);
  return hip->hipStreamQuery(redirected(idx, stream));
}

hipError_t hipEventRecord(hipEvent_t event, hipStream_t stream) {
  const HipApi* hip = orion_hip_api();
  const int idx = client_for_call(stream);
  if (idx < 0) return hip->hipEventRecord(event, stream);
  return hip->hipEventRecord(event, redirected(idx, stream));
}

hipError_t hipStreamWaitEvent(hipStream_t stream, hipEvent_t event, unsigned int flags) {
  const HipApi* hip = orion_hip_api();
  const int idx = client_for_call(stream);
  if (idx < 0) return hip->hipStreamWaitEvent(stream, event, flags);
  return hip->hipStreamWaitEvent(redirected(idx, stream), event, flags);
}

}  // extern "C"
