// The dispatch policy of the scheduler as a pure state machine.
//
// Everything the policy observes (queue heads, event completion, stop
// acknowledgements, wall time) and everything it does (dispatch, release an
// iteration, raise a stop) goes through PolicyHost, so the same code runs
// against the live HIP runtime (scheduler/), against a recorded observation log
// (replay.cpp) and under test.  No HIP header is needed here.
//
// Restates, for gfx950, the policy of the reference scheduler:
//   src/scheduler/scheduler_eval.cpp:238-487  busy_wait_profile (Orion policy)
//   src/scheduler/scheduler_eval.cpp:93-165   schedule_reef
//   src/scheduler/scheduler_eval.cpp:167-236  schedule_sequential
//   src/scheduler/utils_sched.cpp:239-522     schedule_kernel bookkeeping
//   src/scheduler/scheduler_eval.cpp:498-540  profile parsing, setup_change
#pragma once

#include <array>
#include <cstdint>
#include <string>
#include <vector>

namespace orion {

// Record classes as the policy tells them apart.  Every library-op record is
// kernel-like (reference: enum func_type, cuda_capture/intercept_temp.h:642-660).
enum RecClass : int {
  REC_NONE = -1,
  REC_KERNEL = 0,
  REC_MEMCPY = 1,
  REC_MALLOC = 2,
  REC_FREE = 3,
  REC_MEMSET = 4,
};

inline bool is_mem_class(int c) { return c >= REC_MEMCPY && c <= REC_MEMSET; }
char rec_class_char(int c);           // 'k','c','m','f','s'
int rec_class_from_char(char ch);     // REC_NONE for '.', -2 for '-', -3 bad

enum Algo : int { ALGO_ORION = 0, ALGO_REEF = 1, ALGO_SEQUENTIAL = 2 };
const char* algo_name(int algo);
int algo_from_name(const std::string& name);  // -1 if unknown

// One profile row (reference: struct op_info, scheduler/utils_sched.h:90-98).
struct OpInfo {
  std::string name;
  int profile;     // 1 compute-bound, 0 memory-bound, -1 unknown
  int mem;
  int sm_used;     // compute units the op can occupy
  float duration;  // nanoseconds, fp32 like the reference
};

// Parses a profile CSV (header line, then Name,Profile,Memory_footprint,
// SM_usage,Duration).  Field conversion follows std::stoi / std::stof.
// Returns false and fills *err on an unreadable file or a malformed row.
bool parse_profile(const std::string& path, std::vector<OpInfo>* ops,
                   std::string* err);

// CU-mask placement of a best-effort kernel (no reference counterpart: the
// reference owns one stream per client).  `masks` are the sizes, ascending, of
// the CU-masked streams a best-effort client owns; the last one is the whole
// GPU.  While the high-priority client is idle a kernel may use the whole GPU.
// While it has a request in flight the kernel goes to the smallest mask that
// holds its profiled CU need, and never to the whole-GPU stream when a partial
// mask exists: the compute units outside the widest partial mask stay free for
// the high-priority client.  Records that are not kernels stay where the
// client's work is (-1).
int place_cu_slot(const std::vector<int>& masks, int rec_class, int sm_used,
                  int algo, bool hp_active, bool long_kernel);

struct Dispatch {
  int client;      // whose record
  int owner;       // whose stream / event array it goes to
  int rec_class;
  int op_index;    // profile row used (seen[client] before the dispatch)
  int event_slot;  // event_ids[owner] before the dispatch
  int cu_slot;     // CU-mask slot of the owner's stream set, -1 = unchanged
};

class PolicyHost {
 public:
  virtual ~PolicyHost() {}
  virtual void begin_poll() {}
  virtual void end_poll(bool /*effective*/) {}
  virtual bool stop_ack(int client) = 0;
  virtual int peek(int client) = 0;  // RecClass of the queue head or REC_NONE
  virtual bool event_done(int owner, int index) = 0;
  virtual int64_t iteration_us(int client) = 0;
  virtual void dispatch(const Dispatch& d) = 0;
  virtual void iteration_done(int client, int iteration) = 0;
  virtual void set_stop(int client) = 0;
  // Option sliding_throttle only: the policy will ask event_done(owner, index)
  // about this kernel later although newer ones will have been dispatched by
  // then; index is the owner's latest kernel at the time of the call.
  virtual void mark(int /*owner*/, int /*index*/) {}
};

// Per best-effort client, counted once per poll in which the client had a record
// waiting (Orion policy only): what became of it.  Bookkeeping beside the
// policy, not part of it -- no decision reads these.
enum Admission : int {
  ADM_ADMITTED = 0,       // dispatched
  ADM_REFUSED_CUS = 1,    // size + sm_used > the CU budget (scheduler_eval.cpp:339)
  ADM_REFUSED_CLASS = 2,  // fits, but has the running high-priority op's class (:340)
  ADM_THROTTLED = 3,      // admissible, but the duration budget is spent and the
                          // best-effort streams have not drained (:342-359)
  ADM_OVERSIZED = 4,      // admitted alone on the smallest mask although its CU
                          // need exceeds the budget (option admit_oversized)
  ADM_COUNT = 5
};

struct ScheduleArgs {
  bool warmup = false;
  int warmup_iters = 0;
  int algo = ALGO_ORION;
  int depth = 1;         // REEF queue depth, or Orion's best-effort budget (ns)
  int hp_limit = 1;      // tolerated high-priority training iteration (ms)
  int update_start = 1;  // first kernel of the optimizer-update phase
  int64_t max_polls = -1;  // >= 0: give up after that many polls (tests)
};

class Policy {
 public:
  // max_sms: compute units of the device (80 in the reference, 256 on MI355X).
  // sequential_fix: let the time-slicing policy dispatch when no other client
  // is mid-iteration; the reference text can never dispatch past warm-up.
  Policy(std::vector<std::vector<OpInfo>> profiles,
         std::vector<int> num_kernels, std::vector<int> num_iters,
         std::vector<bool> is_train, int max_sms,
         std::vector<int> cu_masks, bool sequential_fix,
         bool confine_long = false, bool reserve_hp = false,
         bool admit_oversized = false, bool sliding_throttle = false);

  void setup_change(int client, std::vector<OpInfo> ops, int num_kernels);

  // Runs the poll loop until every client has finished.  Returns the number
  // of polls, or -1 when max_polls ran out first.
  int64_t schedule(PolicyHost& host, const ScheduleArgs& args);

  int num_clients() const { return n_; }
  const std::vector<int>& cur_iters() const { return cur_iters_; }
  const std::vector<int>& seen() const { return seen_; }
  const std::vector<int>& num_kernels() const { return num_kernels_; }
  const std::vector<OpInfo>& ops(int client) const { return ops_[client]; }
  // polls per Admission outcome, per client (zero for the high-priority client)
  const std::vector<std::array<uint64_t, ADM_COUNT>>& admission() const { return admission_; }
  int sm_threshold() const { return sm_threshold_; }
  bool large_found() const { return large_found_; }
  long sum() const { return sum_; }

 private:
  void dispatch(PolicyHost& host, int client, int owner, int rec_class,
                bool smallest_mask = false);
  void reef(PolicyHost& host, const std::vector<int>& heads, int depth);
  int sequential(PolicyHost& host, const std::vector<int>& heads, int start);

  int n_;
  std::vector<std::vector<OpInfo>> ops_;
  std::vector<int> max_sms_clients_;
  std::vector<int> num_kernels_;
  std::vector<int> max_iters_;
  std::vector<bool> is_train_;
  int max_sms_;
  std::vector<int> cu_masks_;
  bool sequential_fix_;
  // Placement only: a best-effort kernel whose profiled duration alone exceeds
  // the duration budget is kept off the whole-GPU stream.
  bool confine_long_;
  // Admission option (not in the reference, whose rule never looks at the
  // high-priority op's own CU need, scheduler_eval.cpp:339): while a
  // high-priority inference request is in flight, best-effort kernels admitted
  // in one poll may add up to max_sms minus the CU need of the high-priority
  // op last dispatched.  A whole-GPU op -- a HIP-graph request -- then leaves
  // no room; short kernels with a small need leave nearly all of it.
  bool reserve_hp_;
  // Admission option (not in the reference).  The reference's CU clause
  // (size + sm_used <= max_sms, scheduler_eval.cpp:339-340) is written for a GPU
  // without compute-unit masks, where a kernel's profiled need is what it will
  // occupy; the need is not clipped to the device, so a kernel whose grid alone
  // exceeds the device can never be admitted while a high-priority inference
  // request is in flight and its whole client stands behind it.  On a CU-masked
  // stream the kernel occupies the mask, whatever its grid.  With the option
  // such a kernel is admitted while a request is in flight if it is the first
  // best-effort kernel admitted in the poll (size == 0: it is let in alone, and
  // its full need then closes the poll's budget), its class and the class of
  // the running high-priority op are both known and differ, and its profiled
  // duration is at most a quarter of the duration budget; it goes to the
  // smallest mask.  Everything else is the reference's rule.
  bool admit_oversized_;
  // Throttle option (not in the reference).  The reference stops admitting
  // best-effort kernels once the sum of their profiled durations exceeds the
  // budget and starts again only when EVERY best-effort stream has drained
  // (scheduler_eval.cpp:342-359, :366-368): the GPU's best-effort queue runs
  // empty every `budget` nanoseconds of work, and refills at the client's own
  // pace.  With the option the policy also remembers, when the sum first passes
  // half the budget, the latest kernel of every best-effort client (a mark) and
  // the sum at that point; while throttled it asks about the marks as well, and
  // once they have all completed it takes that part of the sum off and goes on
  // -- the outstanding work stays bounded by the budget, as in the reference,
  // but no longer has to fall to zero.
  bool sliding_throttle_;
  // survive between schedule() calls, like the reference's globals
  std::vector<int> seen_;
  std::vector<int> event_ids_;
  std::vector<int> cur_iters_;
  std::vector<bool> stops_;
  int penalty_ = 0;
  std::vector<std::array<uint64_t, ADM_COUNT>> admission_;
  // per-call state mirrored out for inspection
  int sm_threshold_ = 0;
  bool large_found_ = false;
  long sum_ = 0;
  int algo_ = ALGO_ORION;
  int be_budget_ = 0;  // Orion's best-effort duration budget of this call (ns)
  bool changed_ = false;
};

}  // namespace orion
