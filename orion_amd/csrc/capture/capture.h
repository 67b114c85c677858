// Shared state of the interception layer (libinttemp.so).
//
// A client thread that calls an interposed HIP entry point does not execute it:
// it writes a Record into its client's hand-off queue.  In the reference the
// hand-off is synchronous (src/cuda_capture/intercept_temp.cpp:418-458 pushes,
// then block() spins until the queue is empty), which is also what keeps
// `void** args` -- pointers into the caller's frame -- alive until the launch.
// Here that is the default as well.  With ORION_BE_RUN_AHEAD=1 it holds only for
// the high-priority client, for every call whose result the caller needs, and
// for every client the scheduler has not cleared for it (see
// orion_capture_allow_run_ahead: only clients made of this library's own
// kernels are cleared; a framework model never is): a cleared best-effort
// client's kernel launches, device-to-device copies and fills are then queued
// with a deep copy of their arguments and the caller goes on at once (up to
// kQueueSlots records ahead), so that when the policy lets best-effort work in
// again after a pause the next records are already waiting instead of being
// produced one by one at the client's own pace.
//
// Differences from the reference, all inside this private contract:
//  * queues are single-producer/single-consumer rings with acquire/release
//    indices instead of std::queue + pthread_mutex
//    (src/cuda_capture/intercept_temp.cpp:8-19, utils_interc.cpp:53-64);
//  * client identity is cached per thread and can also be derived from the
//    stream a call names, so no thread id system call sits on the hot path and
//    autograd worker threads need no patched PyTorch
//    (src/cuda_capture/utils_interc.cpp:3-51);
//  * the real status of every call is handed back to the caller.
#pragma once

#include <atomic>
#include <cstddef>
#include <cstdint>

#include "../common/hip_api.h"
#include "../policy/policy.h"

namespace orion {

enum RecType : int32_t {
  RT_LAUNCH_KERNEL = 0,        // hipLaunchKernel
  RT_EXT_LAUNCH_KERNEL,        // hipExtLaunchKernel
  RT_COOP_LAUNCH_KERNEL,       // hipLaunchCooperativeKernel
  RT_MODULE_LAUNCH,            // hipModuleLaunchKernel
  RT_EXT_MODULE_LAUNCH,        // hipExtModuleLaunchKernel / hipHccModuleLaunchKernel
  RT_MODULE_COOP_LAUNCH,       // hipModuleLaunchCooperativeKernel
  RT_MEMCPY,                   // hipMemcpy
  RT_MEMCPY_ASYNC,             // hipMemcpyAsync
  RT_MEMCPY_WITH_STREAM,       // hipMemcpyWithStream
  RT_MEMCPY_2D_ASYNC,          // hipMemcpy2DAsync
  RT_MALLOC,                   // hipMalloc
  RT_FREE,                     // hipFree
  RT_MEMSET,                   // hipMemset
  RT_MEMSET_ASYNC,             // hipMemsetAsync
  RT_MEMSET_D32_ASYNC,         // hipMemsetD32Async
  RT_MEMSET_D16_ASYNC,         // hipMemsetD16Async
  RT_MEMSET_D8_ASYNC,          // hipMemsetD8Async
  RT_GRAPH_LAUNCH,             // hipGraphLaunch: a whole captured graph, one record
  RT_MEMCPY_2D,                // hipMemcpy2D (blocking)
  RT_MALLOC_ASYNC,             // hipMallocAsync
  RT_FREE_ASYNC,               // hipFreeAsync
  RT_COUNT
};

// Policy class of a record type (reference: which cases of schedule_kernel bump
// `seen`, src/scheduler/utils_sched.cpp:242-513).
inline int rec_class_of(int type) {
  if (type <= RT_MODULE_COOP_LAUNCH || type == RT_GRAPH_LAUNCH) return REC_KERNEL;
  if (type <= RT_MEMCPY_2D_ASYNC || type == RT_MEMCPY_2D) return REC_MEMCPY;
  if (type == RT_MALLOC || type == RT_MALLOC_ASYNC) return REC_MALLOC;
  if (type == RT_FREE || type == RT_FREE_ASYNC) return REC_FREE;
  return REC_MEMSET;
}

struct Dim3 {
  uint32_t x, y, z;
};

// By-value copy of the arguments of one intercepted call (reference:
// struct func_record, src/cuda_capture/intercept_temp.h:642-691).
// Where the scheduler leaves the outcome of a record whose caller waits for it:
// storage of the waiting call itself, not of the queue slot, which another
// thread of the same client may be writing its next record into by the time
// the waiter wakes up.
struct WaitCell {
  int32_t status;           // HIP status of the issued call, or kRecordGranted
  hipStream_t sync_stream;  // granted calls: the stream the scheduler assigned
};

struct Record {
  int32_t type;
  // caller -> scheduler: 0, kRecordIssued or kRecordDeferred
  int32_t status;
  // Non-null when the caller waits for the record: written by the scheduler
  // before it retires the record, read by the caller once the queue's head has
  // passed the record's ticket.
  WaitCell* cell;
  union {
    struct {
      const void* func;
      Dim3 grid, block;
      void** args;
      size_t shmem;
      hipStream_t stream;
      hipEvent_t start, stop;
      int flags;
    } launch;
    struct {
      hipFunction_t f;
      uint32_t gx, gy, gz, bx, by, bz;  // grid in blocks (module) or in work-items (ext)
      size_t shmem;
      hipStream_t stream;
      void** params;
      void** extra;
      hipEvent_t start, stop;
      uint32_t flags;
    } module;
    struct {
      void* dst;
      const void* src;
      size_t bytes;
      hipMemcpyKind kind;
      hipStream_t stream;
      size_t dpitch, spitch, width, height;
    } copy;
    struct {
      void** ptr;
      size_t size;
      hipStream_t stream;  // hipMallocAsync only
    } malloc_;
    struct {
      void* ptr;
      hipStream_t stream;  // hipFreeAsync only
    } free_;
    struct {
      void* dst;
      int value;
      size_t count;  // bytes, or elements for the D32/D16/D8 forms
      hipStream_t stream;
    } set;
    struct {
      hipGraphExec_t exec;
      hipStream_t stream;
    } graph;
  } u;
};

// What a kernel-class record launches: the host function, the module function
// or the executable graph.  Each is the first member of its struct, so a notice
// of a call already made (which carries nothing else) stores it through
// u.launch.func whatever the record's type.
inline const void* record_function(const Record& r) {
  if (r.type <= RT_COOP_LAUNCH_KERNEL) return r.u.launch.func;
  if (r.type <= RT_MODULE_COOP_LAUNCH) return (const void*)r.u.module.f;
  if (r.type == RT_GRAPH_LAUNCH) return (const void*)r.u.graph.exec;
  return nullptr;
}
static_assert(offsetof(Record, u.launch.func) == offsetof(Record, u.module.f) &&
              offsetof(Record, u.launch.func) == offsetof(Record, u.graph.exec),
              "the launched object must be the first member of every kernel record");

// Record::status values outside the HIP error range.
constexpr int32_t kRecordGranted = -1000;  // scheduler -> caller: run it yourself
constexpr int32_t kRecordIssued = -1001;   // caller -> scheduler: already issued
constexpr int32_t kRecordDeferred = -1002; // caller -> scheduler: nobody waits for the status
constexpr int32_t kRecordPending = -1003;  // a WaitCell nobody has written yet

constexpr int kMaxClients = 32;
constexpr uint32_t kQueueSlots = 64;  // power of two; how far a best-effort client runs ahead
// Largest kernel-argument buffer (HIP_LAUNCH_PARAM_BUFFER_POINTER form) a queued
// record carries with it; a launch with more waits for its dispatch instead.
constexpr size_t kInlineKernarg = 1024;

// What a queued record owns besides the Record itself: the deep copy of a
// module launch's argument buffer with the `extra` array that points to it, and
// (client thread only) the graph kernel node that owns the deep copy of a
// hipLaunchKernel argument list.
struct SlotAux {
  alignas(16) unsigned char kernarg[kInlineKernarg];
  size_t kernarg_size;
  void* extra[5];
  hipGraphNode_t holder;
  // the kernel `holder` was created for.  A node is only ever given new
  // parameters for that same kernel; a launch of another kernel through this
  // slot gets a fresh node.
  const void* holder_func;
};

// The members are grouped by who writes them, one cache line (or more) per
// writer: a launch-bound inference client issues a kernel every few microseconds
// and every line it shares with the polling scheduler thread costs it a round
// trip between two cores per call.
struct alignas(64) ClientChannel {
  Record slots[kQueueSlots];
  SlotAux aux[kQueueSlots];
  hipGraph_t holder_graph;   // owns the holder nodes; touched by the client's threads only

  // -- written by the producer and polled by the scheduler: nothing else here
  alignas(64) std::atomic<uint64_t> tail;

  // -- the producer's own: nobody else looks here on the hot path
  alignas(64) std::atomic<int> producer_lock;  // a client may submit from >1 thread
  uint64_t head_seen;                   // a past value of head (under producer_lock)
  std::atomic<uint64_t> submitted;      // records pushed, all types
  std::atomic<uint64_t> deferred;       // of those, queued without waiting for the dispatch
  // ticket + 1 of the latest record queued without a waiting caller: a release
  // that arrives before the scheduler has issued the queue up to here is
  // postponed (see postpone_release)
  std::atomic<uint64_t> deferred_upto;
  std::atomic<int64_t> block_calls;     // highest it+1 the client passed to block()
  // 1: this client's deferrable records may be queued without a waiting caller
  // (set by orion_capture_allow_run_ahead after every arm; 0 after arm)
  std::atomic<int> may_run_ahead;

  // -- written by the scheduler
  alignas(64) std::atomic<uint64_t> head;

  // -- control, written rarely
  // taken by whoever runs left-over queued records while the scheduler is
  // outside its loop (see flush_channel); the scheduler passes through it once
  // on its way back into the loop, after setting scheduler_polling
  alignas(64) std::atomic<int> flush_lock;
  // iteration hand-shake (reference: client_request_status / client_stop /
  // client_stop_ack, src/cuda_capture/intercept_temp.cpp:16-19)
  std::atomic<int64_t> released_iters;  // iterations released so far
  std::atomic<int> stop;
  std::atomic<int> stop_ack;
  // stream the client's most recent record went to; client-side waits and
  // event records are redirected there
  std::atomic<hipStream_t> last_stream;
  // streams the client itself names (its torch stream), for calls made on its
  // behalf by threads that are not registered (autograd workers)
  std::atomic<hipStream_t> own_streams[4];
  // Non-null while the scheduler lets this client issue its own calls: the
  // client executes each call on this stream at once and queues the record only
  // as a notice (status kRecordIssued), without waiting for it to be retired.
  // Used for a high-priority inference client, whose records the policy
  // dispatches unconditionally in the poll it sees them.
  std::atomic<hipStream_t> direct_stream;
};

struct CaptureState {
  std::atomic<int> armed;        // 0 = pass everything through
  // 1 (ORION_BE_RUN_AHEAD=1): best-effort clients (every client but the last)
  // that have been cleared for it (ClientChannel::may_run_ahead) queue
  // deferrable records without waiting.  Off by default, and while a profile is
  // captured (every kernel is timed where it is issued).
  std::atomic<int> run_ahead;
  // 0: hipLaunchKernel is never queued ahead.  Only the host-only tests on the
  // stand-in runtime can clear it (ORION_BE_RUN_AHEAD_HOLDERS=0 there).
  std::atomic<int> run_ahead_holders;
  std::atomic<uint32_t> epoch;   // bumped by every arm(): invalidates thread caches
  std::atomic<int> scheduler_polling;  // 1 while the scheduler thread is inside schedule()
  int num_clients;
  pid_t client_tids[kMaxClients];
  pid_t scheduler_tid;
  ClientChannel channels[kMaxClients];
};

}  // namespace orion

extern "C" {
// Private contract between libinttemp.so and scheduler_eval.so (reference: the
// globals scheduler_eval.cpp:572-658 reaches through dlsym).
orion::CaptureState* orion_capture_state(void);
// Starts routing the given client threads through their queues.
void orion_capture_arm(int num_clients, const int* client_tids, int scheduler_tid);
// Clears (or bars) client `client` for queueing records ahead of their dispatch
// under ORION_BE_RUN_AHEAD=1.  Every arm bars all clients again.  The scheduler
// clears only clients whose work is made of this library's own kernels.
void orion_capture_allow_run_ahead(int client, int allow);
// Stops routing (everything passes through again) and wakes every waiter.
void orion_capture_disarm(void);
// Called by the scheduler thread right after it has set scheduler_polling on its
// way into its loop: returns once nobody is running queued records on its behalf
// any more (see flush_channel).
void orion_capture_enter_loop(void);
// Keeps the calling thread's thread-local accesses on the dynamic loader's fast
// path (capture/tls_fresh.h); the scheduler thread calls it once per iteration.
void orion_tls_fresh_touch(void);
}
