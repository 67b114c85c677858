// scheduler_eval.so: the scheduler behind the reference's C ABI
// (sched_init / setup / setup_change / schedule / reset,
// src/scheduler/scheduler_eval.cpp:489-676), rebuilt for MI355X.
//
// The poll loop itself is the pure policy core (policy/policy.cpp).  This file
// is its live PolicyHost: it peeks the hand-off queues of libinttemp.so, issues
// records on HIP streams, answers completion queries with HIP events, releases
// iterations and raises stops.
//
// MI355X specifics:
//  * the high-priority client owns one stream spanning all compute units; every
//    best-effort client owns one stream per CU-mask size
//    (hipExtStreamCreateWithCUMask; mask bit i lands on XCD i % 8, so a run of
//    low bits spreads evenly over the eight XCDs), and a best-effort kernel goes
//    to the smallest mask that holds its profiled CU need;
//  * all streams keep the default priority: streams of different priorities
//    are not used on this platform (the reference gives the high-priority
//    client cudaStreamCreateWithPriority(..., hp), utils_sched.cpp:119-147);
//  * when consecutive records of a client land on different streams an event
//    edge keeps them in program order;
//  * completion events are recorded when the policy first asks about them, not
//    after every record (the reference records one per dispatch,
//    utils_sched.cpp:520, out of a pool of 30000 per client, :149-157);
//  * calls that can block the host (allocation, free, synchronous copies and
//    fills) are granted back to the calling thread instead of being run on the
//    scheduler thread (the reference runs them inline, utils_sched.cpp:251-283).
#include <dlfcn.h>
#include <immintrin.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>
#include <sys/syscall.h>
#include <unistd.h>

#include <chrono>
#include <memory>
#include <string>
#include <vector>

#include "../capture/capture.h"
#include "../common/kernel_name.h"
#include "../policy/obslog.h"
#include "../policy/policy.h"
#include "orion_scheduler.h"

extern "C" {
int orion_execute_record(const orion::Record* rec, hipStream_t stream);
bool orion_record_runs_on_caller(int type);
}

namespace {

using namespace orion;
using Clock = std::chrono::steady_clock;

constexpr int kGrantedToCaller = orion::kRecordGranted;

[[noreturn]] void die(const std::string& what) {
  fprintf(stderr, "orion scheduler: %s\n", what.c_str());
  abort();
}

void check(hipError_t err, const char* what) {
  if (err != hipSuccess) {
    const HipApi* hip = orion_hip_api();
    die(std::string(what) + ": " +
        (hip->hipGetErrorString ? hip->hipGetErrorString(err) : "HIP error"));
  }
}

std::vector<int> parse_int_list(const char* text) {
  std::vector<int> out;
  if (!text) return out;
  const char* p = text;
  while (*p) {
    char* end = nullptr;
    long v = strtol(p, &end, 10);
    if (end == p) break;
    out.push_back((int)v);
    p = end;
    while (*p == ',' || *p == ' ') ++p;
  }
  return out;
}

class LiveHost : public PolicyHost {
 public:
  LiveHost(int n, int total_cus, const std::vector<int>& masks)
      : n_(n), total_cus_(total_cus), masks_(masks) {
    hip_ = orion_hip_api();
    cap_ = orion_capture_state();
    streams_.resize((size_t)n);
    last_event_.assign((size_t)n, nullptr);
    chain_event_.assign((size_t)n, nullptr);
    mark_event_.assign((size_t)n, nullptr);
    mark_slot_.assign((size_t)n, -1);
    last_recorded_.assign((size_t)n, true);
    last_slot_.assign((size_t)n, -1);
    last_kernel_stream_.assign((size_t)n, nullptr);
    client_stream_.assign((size_t)n, nullptr);
    used_streams_.resize((size_t)n);
    live_rows_.resize((size_t)n);
    cur_cu_slot_.assign((size_t)n, -1);
    start_pending_.assign((size_t)n, true);
    iter_start_.assign((size_t)n, Clock::now());
    first_start_.assign((size_t)n, Clock::time_point());
    dispatched_.assign((size_t)n, 0);
    durations_ms_.resize((size_t)n);
    create_streams();
  }

  ~LiveHost() override {
    for (auto& set : streams_)
      for (hipStream_t s : set)
        if (s) (void)hip_->hipStreamDestroy(s);
    for (hipEvent_t e : last_event_) if (e) (void)hip_->hipEventDestroy(e);
    for (hipEvent_t e : chain_event_) if (e) (void)hip_->hipEventDestroy(e);
    for (hipEvent_t e : mark_event_) if (e) (void)hip_->hipEventDestroy(e);
    if (update_event_) (void)hip_->hipEventDestroy(update_event_);
  }

  hipStream_t home_stream(int client) const {
    return streams_[(size_t)client].back();
  }
  void set_update_slot(int owner, int slot) {
    update_owner_ = owner;
    update_slot_ = slot;
    update_valid_ = false;
  }
  // Lets `client` issue its own calls on its widest stream (see
  // ClientChannel::direct_stream), or takes that permission back.
  void set_direct(int client, bool on) {
    hipStream_t s = on ? streams_[(size_t)client].back() : nullptr;
    cap_->channels[client].direct_stream.store(s, std::memory_order_release);
  }
  void begin_phase() {
    last_progress_ = Clock::now();
    for (int i = 0; i < n_; ++i) first_start_[(size_t)i] = Clock::time_point();
    phase_start_ = Clock::now();
  }
  const std::vector<std::vector<float>>& durations() const { return durations_ms_; }
  double seconds_since_first(int client) const {
    if (first_start_[(size_t)client] == Clock::time_point()) return 0.0;
    return std::chrono::duration<double>(Clock::now() - first_start_[(size_t)client]).count();
  }
  double seconds_in_phase() const {
    return std::chrono::duration<double>(Clock::now() - phase_start_).count();
  }
  uint64_t dispatched(int client) const { return dispatched_[(size_t)client]; }
  uint64_t stream_switches() const { return stream_switches_; }

  void set_policy(const Policy* p) { policy_ = p; }

  // ---- PolicyHost
  // One pause per poll while things happen; after a run of polls that changed
  // nothing (no record anywhere, or everything waiting for the GPU) a few more:
  // the loop then leaves the core's shared execution resources, and the
  // runtime's locks behind hipEventQuery, to the client threads, at the price of
  // a fraction of a microsecond before the next record is seen.
  void begin_poll() override {
    _mm_pause();
    if (idle_polls_ > 32)
      for (int i = 1; i < idle_pauses_; ++i) _mm_pause();
    if ((++polls_ & 0xfffff) == 0) watchdog();
  }

  void end_poll(bool effective) override { idle_polls_ = effective ? 0 : idle_polls_ + 1; }

  bool stop_ack(int client) override {
    return cap_->channels[client].stop_ack.load(std::memory_order_acquire) != 0;
  }

  int peek(int client) override {
    ClientChannel& ch = cap_->channels[client];
    const uint64_t head = ch.head.load(std::memory_order_relaxed);
    if (ch.tail.load(std::memory_order_acquire) == head) return REC_NONE;
    if (start_pending_[(size_t)client]) {
      // reference: client_starts[i], scheduler_eval.cpp:290-296
      iter_start_[(size_t)client] = Clock::now();
      start_pending_[(size_t)client] = false;
      if (first_start_[(size_t)client] == Clock::time_point())
        first_start_[(size_t)client] = iter_start_[(size_t)client];
    }
    return rec_class_of(ch.slots[head & (kQueueSlots - 1)].type);
  }

  bool event_done(int owner, int index) override {
    if (index == last_slot_[(size_t)owner]) {
      if (!last_recorded_[(size_t)owner]) {
        check(hip_->hipEventRecord(last_event_[(size_t)owner],
                                   last_kernel_stream_[(size_t)owner]),
              "hipEventRecord");
        last_recorded_[(size_t)owner] = true;
      }
      return hip_->hipEventQuery(last_event_[(size_t)owner]) == hipSuccess;
    }
    if (owner == update_owner_ && index == update_slot_ && update_valid_)
      return hip_->hipEventQuery(update_event_) == hipSuccess;
    if (index == mark_slot_[(size_t)owner])
      return hip_->hipEventQuery(mark_event_[(size_t)owner]) == hipSuccess;
    // An index the policy can only reach after the op completed long ago.
    return true;
  }

  // Class of the record waiting at the head of a client's queue (REC_NONE if
  // none), without the bookkeeping peek() does.
  int waiting_class(int client) const {
    ClientChannel& ch = cap_->channels[client];
    const uint64_t head = ch.head.load(std::memory_order_relaxed);
    if (ch.tail.load(std::memory_order_acquire) == head) return REC_NONE;
    return rec_class_of(ch.slots[head & (kQueueSlots - 1)].type);
  }

  int64_t iteration_us(int client) override {
    return std::chrono::duration_cast<std::chrono::microseconds>(
               Clock::now() - iter_start_[(size_t)client]).count();
  }

  void dispatch(const Dispatch& d) override {
    ClientChannel& ch = cap_->channels[d.client];
    const uint64_t head = ch.head.load(std::memory_order_relaxed);
    Record* rec = &ch.slots[head & (kQueueSlots - 1)];

    // A client ends every iteration with block(): when the policy starts
    // counting a new iteration for it (profile row 0) it must have called
    // block() for all the iterations already released.  If it has not, its
    // iteration holds more kernel records than its profile's num_kernels and
    // every later kernel would be matched with the wrong profile row (the
    // reference runs on silently, scheduler_eval.cpp:281-282, :409-420).
    if (d.rec_class == REC_KERNEL && d.op_index == 0 && policy_) {
      const long long done = policy_->cur_iters()[(size_t)d.client];
      const long long blocked = ch.block_calls.load(std::memory_order_acquire);
      if (blocked < done)
        die("client " + std::to_string(d.client) + " submits more kernel records per "
            "iteration than the " + std::to_string(policy_->num_kernels()[(size_t)d.client]) +
            " its profile names: " + std::to_string(done) + " iterations completed by count, "
            "block() called " + std::to_string(blocked) + " times" +
            where_it_differs(d.client, rec));
    }

    // Stream: the owner's stream set, at the slot the policy placed the kernel
    // in; records that are not kernels stay where the client's work is.
    auto& set = streams_[(size_t)d.owner];
    int slot = d.cu_slot;
    if (slot < 0) slot = cur_cu_slot_[(size_t)d.client];
    if (slot < 0 || slot >= (int)set.size()) slot = (int)set.size() - 1;
    hipStream_t stream = set[(size_t)slot];

    hipStream_t prev = client_stream_[(size_t)d.client];
    if (prev != nullptr && prev != stream) {
      // keep the client's records in program order across streams
      hipEvent_t e = chain_event_[(size_t)d.client];
      check(hip_->hipEventRecord(e, prev), "hipEventRecord(chain)");
      check(hip_->hipStreamWaitEvent(stream, e, 0), "hipStreamWaitEvent(chain)");
      ++stream_switches_;
    }
    client_stream_[(size_t)d.client] = stream;
    cur_cu_slot_[(size_t)d.client] = slot;
    // written only when it changes: the line also holds what the client reads on
    // every call (direct_stream), and a store here would take it away each time
    if (ch.last_stream.load(std::memory_order_relaxed) != stream)
      ch.last_stream.store(stream, std::memory_order_release);

    // The outcome goes to the waiting caller's own storage (Record::cell), and
    // must be there before head moves: from then on the slot is the client's
    // again, to write its next record into.
    WaitCell* cell = rec->cell;
    if (rec->status == orion::kRecordIssued) {
      // the client has issued this call itself, on the stream set_direct gave it
    } else if (orion_record_runs_on_caller(rec->type)) {
      if (!cell) die("a blocking call of client " + std::to_string(d.client) +
                     " was queued without a waiting caller");
      cell->sync_stream = stream;
      cell->status = kGrantedToCaller;
    } else {
      // A record queued without a waiting caller has told its caller "success"
      // already (as every queued call of the reference does); if the real call
      // fails now there is nobody to tell, so the job ends here.
      const int status = orion_execute_record(rec, stream);
      auto& used = used_streams_[(size_t)d.client];
      bool known = false;
      for (hipStream_t u : used) known = known || u == stream;
      if (!known) used.push_back(stream);
      if (cell) {
        cell->status = status;
      } else if (status != (int)hipSuccess) {
        die("a queued call of client " + std::to_string(d.client) + " (record type " +
            std::to_string(rec->type) + ", profile row " + std::to_string(d.op_index) +
            ") failed: " + (hip_->hipGetErrorString
                                ? hip_->hipGetErrorString((hipError_t)status)
                                : "HIP error"));
      }
    }
    if (d.rec_class == REC_KERNEL) {
      auto& rows = live_rows_[(size_t)d.client];
      if (d.op_index == 0) rows.clear();
      if ((size_t)d.op_index == rows.size()) rows.push_back({rec->type, record_function(*rec)});
      last_kernel_stream_[(size_t)d.owner] = stream;
      last_slot_[(size_t)d.owner] = d.event_slot;
      last_recorded_[(size_t)d.owner] = false;
      if (d.owner == update_owner_ && d.event_slot == update_slot_) {
        check(hip_->hipEventRecord(update_event_, stream), "hipEventRecord(update)");
        update_valid_ = true;
      }
    }
    ++dispatched_[(size_t)d.client];
    last_progress_ = Clock::now();
    // pop_from_queue: retiring the record releases the caller
    ch.head.store(head + 1, std::memory_order_release);
  }

  void iteration_done(int client, int iteration) override {
    ClientChannel& ch = cap_->channels[client];
    // The policy has just seen the iteration's last kernel complete: every
    // stream the client's records went to is idle, and this thread now waits
    // for each of them once, which costs nothing on the GPU and lets the runtime
    // release the commands it has kept for the stream.  Nobody else ever waits
    // for these streams (a client's own waits are answered from here: block()),
    // and the runtime, left alone, releases a stream's commands only when about
    // a thousand have piled up -- in the middle of a later iteration, inside
    // whichever launch hits the limit (measured on a ResNet-50 request of 371
    // launches issued by the client itself: every 8th of 3 requests took 0.6 ms
    // longer to submit, 35 us with an empty kernel).  Before the release, so
    // that the client cannot yet be adding work to the stream being waited for.
    for (hipStream_t s : used_streams_[(size_t)client]) (void)hip_->hipStreamSynchronize(s);
    used_streams_[(size_t)client].clear();
    if (hipStream_t direct = ch.direct_stream.load(std::memory_order_relaxed))
      (void)hip_->hipStreamSynchronize(direct);
    ch.released_iters.store((int64_t)iteration + 1, std::memory_order_release);
    orion_tls_fresh_touch();
    mark_slot_[(size_t)client] = -1;
    const float ms = (float)iteration_us(client) / 1000.0f;
    durations_ms_[(size_t)client].push_back(ms);
    start_pending_[(size_t)client] = true;
    last_progress_ = Clock::now();
    if (client == update_owner_) update_valid_ = false;
  }

  // Name of what a kernel-class record launches, as a profile's Name column
  // would hold it.
  std::string launched_name(int32_t type, const void* function) const {
    if (type == RT_GRAPH_LAUNCH) return "hipGraphLaunch";
    const char* raw = nullptr;
    if (type <= RT_COOP_LAUNCH_KERNEL) {
      if (hip_->hipKernelNameRefByPtr) raw = hip_->hipKernelNameRefByPtr(function, nullptr);
    } else if (hip_->hipKernelNameRef) {
      raw = hip_->hipKernelNameRef((hipFunction_t)function);
    }
    return short_kernel_name(raw);
  }

  // Where a client's iteration leaves its profile: the first row whose name
  // differs from the kernel the client launched there, with both names -- which
  // is what tells a changed convolution solver or an extra cast kernel apart
  // from a wrong num_kernels.  `extra`: a kernel record beyond the profile's
  // last row (the head of the client's queue), or null.
  std::string where_it_differs(int client, const Record* extra = nullptr) const {
    if (!policy_) return "";
    const auto& ops = policy_->ops(client);
    const auto& rows = live_rows_[(size_t)client];
    const int nk = policy_->num_kernels()[(size_t)client];
    char line[512];
    for (size_t i = 0; i < rows.size() && i < ops.size(); ++i) {
      const std::string live = launched_name(rows[i].type, rows[i].function);
      if (live != ops[i].name) {
        snprintf(line, sizeof line,
                 "\n  client %d: first difference at profile row %zu: the profile names '%s', "
                 "the client launched '%s'", client, i, ops[i].name.c_str(), live.c_str());
        return line;
      }
    }
    std::string out;
    snprintf(line, sizeof line, "\n  client %d: the %zu kernels launched so far in this iteration "
             "carry the names of profile rows 0..%zu", client, rows.size(),
             rows.empty() ? 0 : rows.size() - 1);
    out = rows.empty() ? "" : line;
    if (extra && rec_class_of(extra->type) == REC_KERNEL) {
      snprintf(line, sizeof line, "\n  client %d: after the profile's last row (%d rows) it "
               "launched '%s'", client, nk,
               launched_name(extra->type, record_function(*extra)).c_str());
      out += line;
    } else if ((int)rows.size() < nk && rows.size() < ops.size()) {
      snprintf(line, sizeof line, "\n  client %d: the profile's next row (%zu of %d) names '%s'",
               client, rows.size(), nk, ops[rows.size()].name.c_str());
      out += line;
    }
    return out;
  }

  // The record at the head of a client's queue, or null.
  const Record* head_record(int client) const {
    ClientChannel& ch = cap_->channels[client];
    const uint64_t head = ch.head.load(std::memory_order_relaxed);
    if (ch.tail.load(std::memory_order_acquire) == head) return nullptr;
    return &ch.slots[head & (kQueueSlots - 1)];
  }

  void set_stop(int client) override {
    cap_->channels[client].stop.store(1, std::memory_order_release);
  }

  // The policy will ask about this kernel after newer ones have gone out: an
  // event of its own, recorded now, behind the owner's latest kernel.
  void mark(int owner, int index) override {
    mark_slot_[(size_t)owner] = -1;
    if (index < 0 || index != last_slot_[(size_t)owner] ||
        last_kernel_stream_[(size_t)owner] == nullptr)
      return;   // nothing of the owner's is in flight under that index: "done"
    check(hip_->hipEventRecord(mark_event_[(size_t)owner], last_kernel_stream_[(size_t)owner]),
          "hipEventRecord(mark)");
    mark_slot_[(size_t)owner] = index;
  }

 private:
  // The reference spins forever when a client's kernel count disagrees with its
  // profile, or when a client dies mid-iteration (scheduler_eval.cpp:282, :389).
  // Here a scheduler that has neither dispatched nor completed anything for a
  // while, although a client waits in block() or holds a queued record, reports
  // what it sees and ends the process.
  void watchdog() {
    if (!policy_) return;
    const auto now = Clock::now();
    if (std::chrono::duration<double>(now - last_progress_).count() < stuck_limit_s_) return;
    bool someone_waits = false;
    std::string dump;
    for (int i = 0; i < n_; ++i) {
      ClientChannel& ch = cap_->channels[i];
      const long long blocked = ch.block_calls.load(std::memory_order_acquire);
      const long long released = ch.released_iters.load(std::memory_order_acquire);
      const unsigned long long queued = ch.tail.load(std::memory_order_acquire) -
                                        ch.head.load(std::memory_order_acquire);
      if (blocked > released || queued > 0) someone_waits = true;
      char line[256];
      snprintf(line, sizeof line,
               "\n  client %d: %d of %d kernel records seen this iteration, %llu queued, "
               "block() calls %lld, iterations released %lld, iterations done %d", i,
               policy_->seen()[(size_t)i], policy_->num_kernels()[(size_t)i], queued, blocked,
               released, policy_->cur_iters()[(size_t)i]);
      dump += line;
      if (blocked > released || queued > 0) dump += where_it_differs(i);
    }
    if (!someone_waits) {
      last_progress_ = now;
      return;
    }
    die("no dispatch and no completed iteration for " + std::to_string((int)stuck_limit_s_) +
        " s while clients wait; a client's kernel count probably differs from its profile's "
        "num_kernels, or a client died:" + dump);
  }

  void create_streams() {
    for (int c = 0; c < n_; ++c) {
      const bool is_hp = c == n_ - 1;
      check(hip_->hipEventCreateWithFlags(&last_event_[(size_t)c], hipEventDisableTiming),
            "hipEventCreateWithFlags");
      check(hip_->hipEventCreateWithFlags(&chain_event_[(size_t)c], hipEventDisableTiming),
            "hipEventCreateWithFlags");
      check(hip_->hipEventCreateWithFlags(&mark_event_[(size_t)c], hipEventDisableTiming),
            "hipEventCreateWithFlags");
      if (is_hp) {
        hipStream_t s = nullptr;
        check(hip_->hipStreamCreateWithFlags(&s, hipStreamNonBlocking),
              "hipStreamCreateWithFlags");
        streams_[(size_t)c].push_back(s);
        continue;
      }
      for (int m : masks_) {
        hipStream_t s = nullptr;
        if (m >= total_cus_ || !hip_->hipExtStreamCreateWithCUMask) {
          check(hip_->hipStreamCreateWithFlags(&s, hipStreamNonBlocking),
                "hipStreamCreateWithFlags");
        } else {
          // low m bits: m / 8 compute units on each of the eight XCDs
          std::vector<uint32_t> words((size_t)(total_cus_ + 31) / 32, 0u);
          for (int b = 0; b < m; ++b) words[(size_t)b / 32] |= 1u << (b % 32);
          check(hip_->hipExtStreamCreateWithCUMask(&s, (uint32_t)words.size(), words.data()),
                "hipExtStreamCreateWithCUMask");
        }
        streams_[(size_t)c].push_back(s);
      }
    }
    check(hip_->hipEventCreateWithFlags(&update_event_, hipEventDisableTiming),
          "hipEventCreateWithFlags");
  }

  int n_, total_cus_;
  std::vector<int> masks_;
  const Policy* policy_ = nullptr;
  uint64_t polls_ = 0;
  uint32_t idle_polls_ = 0;   // polls in a row that changed nothing
  const int idle_pauses_ = getenv("ORION_IDLE_PAUSES") && atoi(getenv("ORION_IDLE_PAUSES")) > 0
                               ? atoi(getenv("ORION_IDLE_PAUSES")) : 8;
  Clock::time_point last_progress_ = Clock::now();
  double stuck_limit_s_ = getenv("ORION_STUCK_LIMIT_S") ? atof(getenv("ORION_STUCK_LIMIT_S")) : 20.0;
  const HipApi* hip_;
  CaptureState* cap_;
  std::vector<std::vector<hipStream_t>> streams_;   // [client][cu slot]
  std::vector<hipEvent_t> last_event_, chain_event_, mark_event_;
  std::vector<int> mark_slot_;   // event index each mark event stands for, -1 = none
  std::vector<char> last_recorded_;
  std::vector<int> last_slot_;
  std::vector<hipStream_t> last_kernel_stream_, client_stream_;
  // streams this thread has issued records of the client's current iteration on
  std::vector<std::vector<hipStream_t>> used_streams_;
  // What the client launched at each profile row of its current iteration
  // (record type and the launched function): resolved to names only when a
  // count mismatch has to be reported.
  struct LiveRow { int32_t type; const void* function; };
  std::vector<std::vector<LiveRow>> live_rows_;
  std::vector<int> cur_cu_slot_;
  hipEvent_t update_event_ = nullptr;
  int update_owner_ = -1, update_slot_ = -1;
  bool update_valid_ = false;
  std::vector<char> start_pending_;
  std::vector<Clock::time_point> iter_start_, first_start_;
  Clock::time_point phase_start_;
  std::vector<uint64_t> dispatched_;
  uint64_t stream_switches_ = 0;
  std::vector<std::vector<float>> durations_ms_;
};

// All scheduler state is process-global: the reference's handle is an empty
// object whose pointer its ctypes caller truncates to 32 bits
// (scheduler_eval.cpp:6-46, scheduler_frontend.py:13), so the handle argument
// of every entry point is ignored here as well.
struct Global {
  std::unique_ptr<Policy> policy;
  std::unique_ptr<LiveHost> host;
  std::unique_ptr<Recorder> recorder;
  int n = 0;
  int total_cus = 0;
  std::vector<int> masks;
  std::vector<bool> is_train;
  std::string record_dir;
  bool verbose = true;
  bool hp_direct = true;  // ORION_HP_DIRECT=0: every client hands every call over
};
Global g;
int g_handle_token = 0;

void flush_recording() {
  if (!g.recorder || g.record_dir.empty()) return;
  const std::string obs = g.record_dir + "/observations.log";
  const std::string dec = g.record_dir + "/decisions.log";
  FILE* f = fopen(obs.c_str(), "a");
  if (f) { fwrite(g.recorder->observations().data(), 1, g.recorder->observations().size(), f); fclose(f); }
  f = fopen(dec.c_str(), "a");
  if (f) { fwrite(g.recorder->decisions().data(), 1, g.recorder->decisions().size(), f); fclose(f); }
  g.recorder->clear();
}

// What became of the best-effort clients' waiting records, poll by poll, over the
// whole job (Orion policy): printed, and written beside the recorded logs.
void write_admission_summary() {
  if (!g.policy) return;
  const auto& adm = g.policy->admission();
  std::string json = "{\"polls_with_a_record_waiting\": [";
  for (int i = 0; i < g.n; ++i) {
    const auto& a = adm[(size_t)i];
    char line[256];
    snprintf(line, sizeof line,
             "%s{\"client\": %d, \"admitted\": %llu, \"refused_cu_budget\": %llu, "
             "\"refused_same_class\": %llu, \"throttled\": %llu, \"admitted_oversized\": %llu}",
             i ? ", " : "", i,
             (unsigned long long)(a[ADM_ADMITTED] + a[ADM_OVERSIZED]),
             (unsigned long long)a[ADM_REFUSED_CUS], (unsigned long long)a[ADM_REFUSED_CLASS],
             (unsigned long long)a[ADM_THROTTLED], (unsigned long long)a[ADM_OVERSIZED]);
    json += line;
    if (g.verbose && i < g.n - 1)
      printf("Client %d: polls with a record waiting: %llu admitted (%llu of them oversized, "
             "alone on the smallest mask), %llu over the CU budget, "
             "%llu same class as the high-priority op, %llu throttled by the duration budget\n",
             i, (unsigned long long)(a[ADM_ADMITTED] + a[ADM_OVERSIZED]),
             (unsigned long long)a[ADM_OVERSIZED], (unsigned long long)a[ADM_REFUSED_CUS],
             (unsigned long long)a[ADM_REFUSED_CLASS], (unsigned long long)a[ADM_THROTTLED]);
  }
  json += "]}\n";
  if (!g.record_dir.empty()) {
    FILE* f = fopen((g.record_dir + "/admission.json").c_str(), "w");
    if (f) { fputs(json.c_str(), f); fclose(f); }
  }
}

}  // namespace

extern "C" {

void* sched_init(void) { return &g_handle_token; }

void setup(void* /*scheduler*/, int num_clients, int* tids, char** models,
           char** files, int* num_kernels, int* num_iters, bool* train, bool /*reef*/) {
  if (num_clients < 1 || num_clients > kMaxClients) die("client count out of range");
  const HipApi* hip = orion_hip_api();
  const pid_t mytid = (pid_t)syscall(SYS_gettid);

  // CUs of the device: what streams and CU masks are built from.
  int cus = 0;
  {
    int dev = 0;
    if (hip->hipGetDevice) (void)hip->hipGetDevice(&dev);
    check(hip->hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev),
          "hipDeviceGetAttribute(MultiprocessorCount)");
  }
  // The policy's max_sms (the reference hard-codes 80, its GPU's SM count,
  // scheduler_eval.cpp:9): the CU budget best-effort kernels may add up to while
  // a high-priority inference request is in flight.  The device's CU count
  // unless ORION_MAX_SMS names a smaller budget.
  int max_sms = cus;
  if (const char* e = getenv("ORION_MAX_SMS")) {
    if (atoi(e) > 0) max_sms = atoi(e);
  }
  g.total_cus = cus;
  g.masks = parse_int_list(getenv("ORION_BE_CU_MASKS"));
  if (g.masks.empty()) g.masks = {cus / 8, cus / 4, cus / 2, cus};
  for (size_t i = 0; i < g.masks.size(); ++i)
    if (g.masks[i] <= 0 || (i && g.masks[i] <= g.masks[i - 1]))
      die("ORION_BE_CU_MASKS must be an ascending list of positive CU counts");
  if (g.masks.back() < cus) g.masks.push_back(cus);
  if (const char* e = getenv("ORION_QUIET")) g.verbose = atoi(e) == 0;
  if (const char* e = getenv("ORION_HP_DIRECT")) g.hp_direct = atoi(e) != 0;

  std::vector<std::vector<OpInfo>> profiles((size_t)num_clients);
  std::vector<int> nk, ni;
  g.is_train.clear();
  for (int i = 0; i < num_clients; ++i) {
    std::string err;
    if (!parse_profile(files[i], &profiles[(size_t)i], &err)) die(err);
    if ((int)profiles[(size_t)i].size() < num_kernels[i])
      die(std::string(files[i]) + ": fewer rows than num_kernels");
    if (g.verbose)
      printf("KERNEL_INFO_FILE IS %s\n----------- SIZE: %zu\n", files[i],
             profiles[(size_t)i].size());
    nk.push_back(num_kernels[i]);
    ni.push_back(num_iters[i]);
    g.is_train.push_back(train[i]);
  }
  const bool as_written = getenv("ORION_SEQUENTIAL_AS_WRITTEN") &&
                          atoi(getenv("ORION_SEQUENTIAL_AS_WRITTEN")) != 0;
  g.n = num_clients;
  g.host.reset();  // streams of a previous job first
  // Placement option: keep a best-effort kernel that alone outlasts the duration
  // budget off the whole-GPU stream even while the high-priority client is idle.
  const bool confine_long = getenv("ORION_CONFINE_LONG_BE") &&
                            atoi(getenv("ORION_CONFINE_LONG_BE")) != 0;
  // Admission option: reserve the high-priority op's own CU need (see policy.h).
  const bool reserve_hp = getenv("ORION_RESERVE_HP_CUS") &&
                          atoi(getenv("ORION_RESERVE_HP_CUS")) != 0;
  // Admission option: let short best-effort kernels of the opposite class whose
  // CU need exceeds the device in alone, on the smallest mask (see policy.h).
  const bool admit_oversized = getenv("ORION_ADMIT_OVERSIZED") &&
                               atoi(getenv("ORION_ADMIT_OVERSIZED")) != 0;
  // Throttle option: let go at the half-way mark instead of waiting for every
  // best-effort stream to run empty (see policy.h).
  const bool sliding_throttle = getenv("ORION_SLIDING_THROTTLE") &&
                                atoi(getenv("ORION_SLIDING_THROTTLE")) != 0;
  g.policy.reset(new Policy(std::move(profiles), nk, ni, g.is_train, max_sms, g.masks,
                            !as_written, confine_long, reserve_hp, admit_oversized,
                            sliding_throttle));
  g.host.reset(new LiveHost(num_clients, cus, g.masks));
  g.host->set_policy(g.policy.get());
  g.recorder.reset();
  g.record_dir.clear();
  if (const char* dir = getenv("ORION_RECORD_DIR")) {
    if (*dir) {
      g.record_dir = dir;
      g.recorder.reset(new Recorder(g.host.get(), num_clients));
      g.recorder->header(max_sms, g.masks, confine_long, reserve_hp, admit_oversized,
                         sliding_throttle);
      for (int i = 0; i < num_clients; ++i)
        g.recorder->client(i, nk[(size_t)i], ni[(size_t)i], g.is_train[(size_t)i], files[i]);
      // start both logs afresh
      FILE* f = fopen((g.record_dir + "/observations.log").c_str(), "w");
      if (f) fclose(f);
      f = fopen((g.record_dir + "/decisions.log").c_str(), "w");
      if (f) fclose(f);
    }
  }
  orion_capture_arm(num_clients, tids, (int)mytid);
  // Queueing ahead of the dispatch (ORION_BE_RUN_AHEAD=1) is for clients made of
  // this library's own kernels only -- their launches are plain hipLaunchKernel
  // calls of one kernel each, and they run with it bit-exactly.  A framework
  // model as a best-effort client has faulted the GPU with it, cause not found,
  // so no other name is cleared; such a client keeps the synchronous hand-off
  // whatever the environment says.  (The host-only stand-in runtime launches
  // nothing on a GPU: there every client is cleared, which is what lets the
  // host tests drive that code.)
  const bool ahead = getenv("ORION_BE_RUN_AHEAD") && atoi(getenv("ORION_BE_RUN_AHEAD")) != 0;
  for (int i = 0; ahead && i < num_clients - 1; ++i) {
    const char* name = models ? models[i] : nullptr;
    const bool own_kernels = name && (strcmp(name, "gemm_bf16") == 0 || strcmp(name, "triad_f32") == 0);
    if (own_kernels || hip->stand_in) {
      orion_capture_allow_run_ahead(i, 1);
    } else if (g.verbose) {
      printf("orion: ORION_BE_RUN_AHEAD is ignored for client %d (%s): only gemm_bf16 and "
             "triad_f32 clients queue ahead of their dispatch\n", i, name ? name : "?");
    }
  }
}

void setup_change(void* /*scheduler*/, int client_id, char* file, int num_kernels) {
  if (!g.policy || client_id < 0 || client_id >= g.n) die("setup_change before setup");
  std::vector<OpInfo> ops;
  std::string err;
  if (!parse_profile(file, &ops, &err)) die(err);
  if ((int)ops.size() < num_kernels) die(std::string(file) + ": fewer rows than num_kernels");
  if (g.verbose) printf("KERNEL_INFO_FILE IS %s\n", file);
  g.policy->setup_change(client_id, std::move(ops), num_kernels);
  if (g.recorder) g.recorder->setup_change(client_id, num_kernels, file);
}

void* schedule(void* /*scheduler*/, int num_clients, bool profile_mode, int /*iter*/,
               bool warmup, int warmup_iters, bool reef, bool seq, int reef_depth,
               int hp_limit, int update_start) {
  if (!profile_mode) return nullptr;  // scheduler_eval.cpp:666
  if (!g.policy || num_clients != g.n) die("schedule before setup");
  ScheduleArgs a;
  a.warmup = warmup;
  a.warmup_iters = warmup_iters;
  a.algo = reef ? ALGO_REEF : (seq ? ALGO_SEQUENTIAL : ALGO_ORION);
  a.depth = reef_depth;
  a.hp_limit = hp_limit;
  a.update_start = update_start;
  const int hp = g.n - 1;
  if (g.is_train[(size_t)hp] && a.algo == ALGO_ORION)
    g.host->set_update_slot(hp, update_start - 1);
  else
    g.host->set_update_slot(-1, -1);
  // A high-priority inference client is dispatched unconditionally in the poll
  // that sees its record (scheduler_eval.cpp:311-321): the decision needs no
  // wait, so the client issues its calls itself and the queue carries notices.
  // Not under time slicing (the client must wait its turn) and not for a
  // training client (the update-phase event must follow one exact kernel).
  const bool direct = g.hp_direct && a.algo != ALGO_SEQUENTIAL && !g.is_train[(size_t)hp];
  g.host->set_direct(hp, direct);
  g.host->begin_phase();
  PolicyHost* host = g.host.get();
  if (g.recorder) {
    g.recorder->set_inner(g.host.get());
    g.recorder->begin_schedule(a);
    host = g.recorder.get();
  }
  orion_capture_state()->scheduler_polling.store(1);
  orion_capture_enter_loop();   // nobody runs queued records for this thread any more
  g.policy->schedule(*host, a);
  orion_capture_state()->scheduler_polling.store(0, std::memory_order_release);
  g.host->set_direct(hp, false);
  if (warmup) {
    // A warm-up phase ends with every client between two iterations, on its way
    // to the rendezvous with this thread.  A kernel still waiting in a queue
    // belongs to an iteration the policy has already counted as complete: the
    // client's iteration holds more kernel records than its profile names, and
    // it would wait for this thread forever while this thread waits for it.
    for (int i = 0; i < g.n; ++i)
      if (g.host->waiting_class(i) == REC_KERNEL)
        die("client " + std::to_string(i) + " submits more kernel records per iteration "
            "than the " + std::to_string(g.policy->num_kernels()[(size_t)i]) +
            " its profile names: one is still queued after the iteration was released" +
            g.host->where_it_differs(i, g.host->head_record(i)));
  }
  if (g.recorder) {
    g.recorder->end_schedule();
    flush_recording();
  }
  if (!warmup) {
    // scheduler_eval.cpp:455-462, :478-482
    if (g.verbose) {
      for (int i = 0; i < g.n; ++i)
        printf("Client %d, Total loop took %f sec, %d iterations, %llu records\n", i,
               g.host->seconds_since_first(i), g.policy->cur_iters()[(size_t)i],
               (unsigned long long)g.host->dispatched(i));
      printf("Total loop took %f sec (%llu cross-stream edges)\n",
             g.host->seconds_in_phase(), (unsigned long long)g.host->stream_switches());
      fflush(stdout);
    }
    write_admission_summary();
    // The measured run is over: whatever clients issue from now on is theirs.
    orion_capture_disarm();
  }
  return nullptr;
}

void* reset(void* /*scheduler*/, int /*num_clients*/) {
  // profile_reset (scheduler_eval.cpp:49-56) only clears per-iteration
  // counters that the policy core clears itself when an iteration completes.
  return nullptr;
}

void* orion_client_stream(int client) {
  if (!g.host || client < 0 || client >= g.n) return nullptr;
  return (void*)g.host->home_stream(client);
}

int orion_sched_num_cus(void) { return g.total_cus; }

int orion_sched_iteration_ms(int client, float* out, int cap) {
  if (!g.host || client < 0 || client >= g.n) return -1;
  const auto& d = g.host->durations()[(size_t)client];
  int k = (int)d.size() < cap ? (int)d.size() : cap;
  for (int i = 0; i < k; ++i) out[i] = d[(size_t)i];
  return (int)d.size();
}

void orion_sched_teardown(void) {
  orion_capture_disarm();
  g.recorder.reset();
  g.host.reset();
  g.policy.reset();
  g.n = 0;
}

}  // extern "C"
