// Profile capture: runs ONE client alone, in submission order, on one stream
// spanning the whole GPU, and times every kernel it submits with a pair of HIP
// events passed to the launch itself (so the figure is the kernel's own
// execution time, not launch gaps).  The output is a per-record trace from
// which orion_amd/profiling builds the scheduler's profile CSV: one row per
// kernel-like record, in exactly the order and number the interception layer
// will see when the client later runs under the scheduler.
//
// Reference counterpart: the offline Nsight Compute / Nsight Systems runs of
// PROFILE.md:7-54 and profiling/postprocessing/process_ncu.py; there the row
// count has to be matched by hand against what the interposers capture.
#include <immintrin.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>
#include <sys/syscall.h>
#include <unistd.h>

#include <string>
#include <vector>

#include "../capture/capture.h"
#include "../common/kernel_name.h"

extern "C" {
int orion_execute_record(const orion::Record* rec, hipStream_t stream);
bool orion_record_runs_on_caller(int type);
}

namespace {

using namespace orion;
constexpr int kGrantedToCaller = orion::kRecordGranted;

struct Row {
  int iteration, index, type;
  std::string name;
  uint32_t gx, gy, gz, bx, by, bz;
  size_t shmem;
  int regs;
  size_t static_lds;
  hipEvent_t start, stop;
  float ns;
};

std::string short_name(const char* mangled) { return short_kernel_name(mangled); }

struct CaptureRun {
  const HipApi* hip = nullptr;
  hipStream_t stream = nullptr;
  std::vector<hipEvent_t> pool;
  size_t pool_at = 0;
  std::vector<Row> rows;        // current iteration
  int iteration = 0;
  FILE* out = nullptr;

  hipEvent_t event() {
    if (pool_at == pool.size()) {
      hipEvent_t e = nullptr;
      if (hip->hipEventCreateWithFlags(&e, 0 /* hipEventDefault: timing on */) != hipSuccess) {
        fprintf(stderr, "orion profile capture: hipEventCreateWithFlags failed\n");
        abort();
      }
      pool.push_back(e);
    }
    return pool[pool_at++];
  }
};

CaptureRun g_run;

void describe(const Record& r, Row* row, const HipApi* hip, hipStream_t stream) {
  row->type = r.type;
  row->regs = 0;
  row->static_lds = 0;
  if (r.type == RT_GRAPH_LAUNCH) {
    // a whole captured graph: no single grid; the profile writer gives it
    // every compute unit and an unknown class
    row->gx = row->gy = row->gz = row->bx = row->by = row->bz = 0;
    row->shmem = 0;
    row->name = "hipGraphLaunch";
    return;
  }
  if (r.type <= RT_COOP_LAUNCH_KERNEL) {
    row->gx = r.u.launch.grid.x; row->gy = r.u.launch.grid.y; row->gz = r.u.launch.grid.z;
    row->bx = r.u.launch.block.x; row->by = r.u.launch.block.y; row->bz = r.u.launch.block.z;
    row->shmem = r.u.launch.shmem;
    row->name = short_name(hip->hipKernelNameRefByPtr
                               ? hip->hipKernelNameRefByPtr(r.u.launch.func, stream) : nullptr);
    if (hip->hipFuncGetAttributes) {
      hipFuncAttributes attr;
      memset(&attr, 0, sizeof attr);
      if (hip->hipFuncGetAttributes(&attr, r.u.launch.func) == hipSuccess) {
        row->regs = attr.numRegs;
        row->static_lds = attr.sharedSizeBytes;
      }
    }
  } else {
    row->bx = r.u.module.bx; row->by = r.u.module.by; row->bz = r.u.module.bz;
    if (r.type == RT_EXT_MODULE_LAUNCH) {  // sizes are in work-items
      row->gx = r.u.module.gx / (row->bx ? row->bx : 1);
      row->gy = r.u.module.gy / (row->by ? row->by : 1);
      row->gz = r.u.module.gz / (row->bz ? row->bz : 1);
    } else {
      row->gx = r.u.module.gx; row->gy = r.u.module.gy; row->gz = r.u.module.gz;
    }
    row->shmem = r.u.module.shmem;
    row->name = short_name(hip->hipKernelNameRef ? hip->hipKernelNameRef(r.u.module.f) : nullptr);
    if (hip->hipFuncGetAttribute) {
      int v = 0;
      if (hip->hipFuncGetAttribute(&v, HIP_FUNC_ATTRIBUTE_NUM_REGS, r.u.module.f) == hipSuccess)
        row->regs = v;
      if (hip->hipFuncGetAttribute(&v, HIP_FUNC_ATTRIBUTE_SHARED_SIZE_BYTES, r.u.module.f) == hipSuccess)
        row->static_lds = (size_t)v;
    }
  }
}

// Launches a kernel-like record with timing events attached.
int launch_timed(const Record& r, hipStream_t stream, hipEvent_t start, hipEvent_t stop,
                 const HipApi* hip) {
  switch (r.type) {
    case RT_LAUNCH_KERNEL:
    case RT_EXT_LAUNCH_KERNEL:
      if (r.type == RT_EXT_LAUNCH_KERNEL && (r.u.launch.start || r.u.launch.stop)) break;
      return (int)hip->hipExtLaunchKernel(
          r.u.launch.func, dim3(r.u.launch.grid.x, r.u.launch.grid.y, r.u.launch.grid.z),
          dim3(r.u.launch.block.x, r.u.launch.block.y, r.u.launch.block.z), r.u.launch.args,
          r.u.launch.shmem, stream, start, stop, 0);
    case RT_MODULE_LAUNCH:
      return (int)hip->hipExtModuleLaunchKernel(
          r.u.module.f, r.u.module.gx * r.u.module.bx, r.u.module.gy * r.u.module.by,
          r.u.module.gz * r.u.module.bz, r.u.module.bx, r.u.module.by, r.u.module.bz,
          r.u.module.shmem, stream, r.u.module.params, r.u.module.extra, start, stop, 0);
    case RT_EXT_MODULE_LAUNCH:
      if (r.u.module.start || r.u.module.stop) break;  // the caller times it itself
      return (int)hip->hipExtModuleLaunchKernel(
          r.u.module.f, r.u.module.gx, r.u.module.gy, r.u.module.gz, r.u.module.bx,
          r.u.module.by, r.u.module.bz, r.u.module.shmem, stream, r.u.module.params,
          r.u.module.extra, start, stop, r.u.module.flags);
    default:
      break;
  }
  // cooperative launches and launches that carry the caller's own events:
  // bracket with recorded events instead
  (void)hip->hipEventRecord(start, stream);
  int st = orion_execute_record(&r, stream);
  (void)hip->hipEventRecord(stop, stream);
  return st;
}

void finish_iteration(CaptureRun& run) {
  (void)run.hip->hipStreamSynchronize(run.stream);
  for (Row& row : run.rows) {
    float ms = 0.0f;
    if (run.hip->hipEventElapsedTime(&ms, row.start, row.stop) != hipSuccess) ms = 0.0f;
    row.ns = ms * 1.0e6f;
    fprintf(run.out, "%d,%d,%d,%s,%u,%u,%u,%u,%u,%u,%zu,%d,%zu,%.0f\n", row.iteration,
            row.index, row.type, row.name.c_str(), row.gx, row.gy, row.gz, row.bx, row.by,
            row.bz, row.shmem, row.regs, row.static_lds, row.ns);
  }
  fflush(run.out);
  run.rows.clear();
  run.pool_at = 0;
}

}  // namespace

extern "C" {

// Starts a capture of the calling process's client thread `client_tid`; the
// trace is written to `trace_path` (CSV with a header line).
int orion_profile_begin(int client_tid, const char* trace_path) {
  CaptureRun& run = g_run;
  run.hip = orion_hip_api();
  run.out = fopen(trace_path, "w");
  if (!run.out) return 1;
  fprintf(run.out, "iteration,index,type,name,grid_x,grid_y,grid_z,block_x,block_y,block_z,"
                   "dyn_lds,regs,static_lds,duration_ns\n");
  if (!run.stream &&
      run.hip->hipStreamCreateWithFlags(&run.stream, hipStreamNonBlocking) != hipSuccess)
    return 2;
  run.iteration = 0;
  run.rows.clear();
  const int tid = client_tid;
  orion_capture_arm(1, &tid, (int)syscall(SYS_gettid));
  return 0;
}

// Serves the client until it has completed `until_iteration` iterations (an
// iteration ends when the client calls block()).  Call from the thread that
// called orion_profile_begin.
int orion_profile_run(int until_iteration) {
  CaptureRun& run = g_run;
  const HipApi* hip = run.hip;
  ClientChannel& ch = orion_capture_state()->channels[0];
  orion_capture_state()->scheduler_polling.store(1, std::memory_order_release);
  while (run.iteration < until_iteration) {
    const uint64_t head = ch.head.load(std::memory_order_relaxed);
    if (ch.tail.load(std::memory_order_acquire) == head) {
      if (ch.block_calls.load(std::memory_order_acquire) > run.iteration) {
        // the client has submitted the whole iteration and waits in block()
        finish_iteration(run);
        ch.released_iters.store((int64_t)run.iteration + 1, std::memory_order_release);
        ++run.iteration;
      } else {
        _mm_pause();
      }
      continue;
    }
    Record* rec = &ch.slots[head & (kQueueSlots - 1)];
    ch.last_stream.store(run.stream, std::memory_order_release);
    // the outcome goes to the waiting caller's own storage, before head moves
    WaitCell* cell = rec->cell;
    int status = (int)hipSuccess;
    if (orion_record_runs_on_caller(rec->type)) {
      if (cell) cell->sync_stream = run.stream;
      status = kGrantedToCaller;
    } else if (rec_class_of(rec->type) == REC_KERNEL) {
      Row row;
      row.iteration = run.iteration;
      row.index = (int)run.rows.size();
      describe(*rec, &row, hip, run.stream);
      row.start = run.event();
      row.stop = run.event();
      row.ns = 0;
      status = launch_timed(*rec, run.stream, row.start, row.stop, hip);
      run.rows.push_back(std::move(row));
    } else {
      status = orion_execute_record(rec, run.stream);
    }
    if (cell) cell->status = status;
    ch.head.store(head + 1, std::memory_order_release);
  }
  orion_capture_state()->scheduler_polling.store(0, std::memory_order_release);
  return 0;
}

int orion_profile_end(void) {
  CaptureRun& run = g_run;
  orion_capture_disarm();
  if (run.out) fclose(run.out);
  run.out = nullptr;
  return 0;
}

}  // extern "C"
