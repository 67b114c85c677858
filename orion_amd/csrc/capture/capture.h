// Shared state of the interception layer (libinttemp.so).
//
// A client thread that calls an interposed HIP entry point does not execute it:
// it writes a Record into its client's hand-off queue and waits until the
// scheduler thread has taken it.  The hand-off is synchronous, like the
// reference's (src/cuda_capture/intercept_temp.cpp:418-458 pushes, then
// block() spins until the queue is empty), which is also what keeps
// `void** args` -- pointers into the caller's frame -- alive until the launch.
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
struct Record {
  int32_t type;
  // Written by the scheduler before it retires the record; read by the caller
  // after the hand-off completes.
  int32_t status;
  // Set by the scheduler for synchronous copies: the stream the copy was
  // enqueued on; the caller waits for it on its own thread.
  hipStream_t sync_stream;
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

// Record::status values outside the HIP error range.
constexpr int32_t kRecordGranted = -1000;  // scheduler -> caller: run it yourself
constexpr int32_t kRecordIssued = -1001;   // caller -> scheduler: already issued

constexpr int kMaxClients = 32;
constexpr uint32_t kQueueSlots = 8;   // power of two; occupancy is <= 2 in practice

struct alignas(64) ClientChannel {
  Record slots[kQueueSlots];
  alignas(64) std::atomic<uint64_t> tail;   // written by the producer
  alignas(64) std::atomic<uint64_t> head;   // written by the scheduler
  alignas(64) std::atomic<int> producer_lock;  // a client may submit from >1 thread
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
  std::atomic<uint64_t> submitted;      // records pushed, all types
  std::atomic<int64_t> block_calls;     // highest it+1 the client passed to block()
};

struct CaptureState {
  std::atomic<int> armed;        // 0 = pass everything through
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
// Stops routing (everything passes through again) and wakes every waiter.
void orion_capture_disarm(void);
}
