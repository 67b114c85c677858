// Observation and decision logs of a policy run.
//
// An observation log fixes a run: the job header plus, for every effective
// poll, the stop acknowledgements, queue heads, event-query answers and
// iteration times the policy consumed.  Polls that changed nothing are not
// logged; skipping them cannot change a decision because the policy rebuilds
// its per-poll state on every pass (reference:
// src/scheduler/scheduler_eval.cpp:277-302).
//
// Line formats (text, one record per line):
//   observation log
//     J <n> <max_sms> <cu mask sizes, comma separated> [L1] [R1] [O1] [T1]
//       (L1: long best-effort kernels are confined to a partial mask;
//        R1: the high-priority op's own CU need is reserved;
//        O1: short best-effort kernels of the opposite class whose CU need
//            exceeds the device are admitted alone on the smallest mask;
//        T1: the duration throttle lets go when the work outstanding at its
//            half-way mark has completed, not only when every stream is empty)
//     K <client> <num_kernels> <num_iters> <train 0|1> <profile path>
//     X <client> <num_kernels> <profile path>               setup_change
//     S <warmup 0|1> <warmup_iters> <algo> <depth> <hp_limit> <update_start>
//     P <acks hex> <heads> <event answers|-> <iteration us, comma sep.|->
//     E                                                     schedule returned
//   decision log
//     S, E, X <client>                                      structure
//     D <client> <owner> <class> <op_index> <event_slot> <cu_slot>
//     F <client> <iteration>                                iteration released
//     T <client>                                            stop raised
#pragma once

#include <string>
#include <vector>

#include "policy.h"

namespace orion {

// PolicyHost decorator: forwards to `inner` and writes both logs.
class Recorder : public PolicyHost {
 public:
  Recorder(PolicyHost* inner, int n) : inner_(inner), n_(n) {}
  void set_inner(PolicyHost* inner) { inner_ = inner; }
  // With marks, a line "P" precedes the decisions of every effective poll, so
  // the decision log lines up with the observation log's P lines one to one.
  void set_mark_polls(bool on) { mark_polls_ = on; }

  void header(int max_sms, const std::vector<int>& masks, bool confine_long = false,
              bool reserve_hp = false, bool admit_oversized = false,
              bool sliding_throttle = false);
  void client(int idx, int num_kernels, int num_iters, bool train,
              const std::string& profile_path);
  void setup_change(int client, int num_kernels, const std::string& path);
  void begin_schedule(const ScheduleArgs& a);
  void end_schedule();

  void begin_poll() override;
  void end_poll(bool effective) override;
  void mark(int owner, int index) override { inner_->mark(owner, index); }
  bool stop_ack(int client) override;
  int peek(int client) override;
  bool event_done(int owner, int index) override;
  int64_t iteration_us(int client) override;
  void dispatch(const Dispatch& d) override;
  void iteration_done(int client, int iteration) override;
  void set_stop(int client) override;

  const std::string& observations() const { return obs_; }
  const std::string& decisions() const { return dec_; }
  void clear() { obs_.clear(); dec_.clear(); }

 private:
  PolicyHost* inner_;
  int n_;
  bool mark_polls_ = false;
  std::string obs_, dec_;
  // current poll
  unsigned long long acks_ = 0;
  std::string heads_, events_, us_, poll_dec_;
};

// Replays an observation log through the native policy; returns false and
// fills *err when the log is malformed or the policy diverges from it.
bool replay_observations(const std::string& obs, bool sequential_fix,
                         std::string* decisions, std::string* err,
                         bool mark_polls = false);

}  // namespace orion
