#include "obslog.h"

#include <cstdarg>
#include <cstdio>
#include <cstdlib>
#include <deque>
#include <sstream>

namespace orion {

namespace {
void appendf(std::string* s, const char* fmt, ...) __attribute__((format(printf, 2, 3)));
void appendf(std::string* s, const char* fmt, ...) {
  char buf[512];
  va_list ap;
  va_start(ap, fmt);
  int n = vsnprintf(buf, sizeof buf, fmt, ap);
  va_end(ap);
  if (n > 0) s->append(buf, (size_t)(n < (int)sizeof buf ? n : (int)sizeof buf - 1));
}
}  // namespace

void Recorder::header(int max_sms, const std::vector<int>& masks, bool confine_long,
                      bool reserve_hp, bool admit_oversized, bool sliding_throttle) {
  appendf(&obs_, "J %d %d ", n_, max_sms);
  for (size_t i = 0; i < masks.size(); ++i)
    appendf(&obs_, i ? ",%d" : "%d", masks[i]);
  if (confine_long) obs_ += " L1";  // long best-effort kernels are confined
  if (reserve_hp) obs_ += " R1";    // the high-priority op's CU need is reserved
  if (admit_oversized) obs_ += " O1";  // oversized short kernels of the other class go in alone
  if (sliding_throttle) obs_ += " T1"; // the throttle lets go at its half-way mark
  obs_ += '\n';
}

void Recorder::client(int idx, int num_kernels, int num_iters, bool train,
                      const std::string& profile_path) {
  appendf(&obs_, "K %d %d %d %d ", idx, num_kernels, num_iters, train ? 1 : 0);
  obs_ += profile_path;
  obs_ += '\n';
}

void Recorder::setup_change(int client, int num_kernels,
                            const std::string& path) {
  appendf(&obs_, "X %d %d ", client, num_kernels);
  obs_ += path;
  obs_ += '\n';
  appendf(&dec_, "X %d\n", client);
}

void Recorder::begin_schedule(const ScheduleArgs& a) {
  appendf(&obs_, "S %d %d %s %d %d %d\n", a.warmup ? 1 : 0, a.warmup_iters,
          algo_name(a.algo), a.depth, a.hp_limit, a.update_start);
  dec_ += "S\n";
}

void Recorder::end_schedule() {
  obs_ += "E\n";
  dec_ += "E\n";
}

void Recorder::begin_poll() {
  inner_->begin_poll();
  acks_ = 0;
  for (int i = 0; i < n_; ++i)
    if (inner_->stop_ack(i)) acks_ |= 1ull << i;
  heads_.assign((size_t)n_, '-');
  events_.clear();
  us_.clear();
  poll_dec_.clear();
}

void Recorder::end_poll(bool effective) {
  if (effective) {
    appendf(&obs_, "P %llx ", acks_);
    obs_ += heads_;
    obs_ += ' ';
    obs_ += events_.empty() ? "-" : events_;
    obs_ += ' ';
    obs_ += us_.empty() ? "-" : us_;
    obs_ += '\n';
    if (mark_polls_) dec_ += "P\n";
    dec_ += poll_dec_;
  }
  inner_->end_poll(effective);
}

bool Recorder::stop_ack(int client) { return (acks_ >> client) & 1ull; }

int Recorder::peek(int client) {
  int c = inner_->peek(client);
  heads_[(size_t)client] = rec_class_char(c);
  return c;
}

bool Recorder::event_done(int owner, int index) {
  bool done = inner_->event_done(owner, index);
  events_ += done ? '1' : '0';
  return done;
}

int64_t Recorder::iteration_us(int client) {
  int64_t us = inner_->iteration_us(client);
  appendf(&us_, us_.empty() ? "%lld" : ",%lld", (long long)us);
  return us;
}

void Recorder::dispatch(const Dispatch& d) {
  appendf(&poll_dec_, "D %d %d %c %d %d %d\n", d.client, d.owner,
          rec_class_char(d.rec_class), d.op_index, d.event_slot, d.cu_slot);
  inner_->dispatch(d);
}

void Recorder::iteration_done(int client, int iteration) {
  appendf(&poll_dec_, "F %d %d\n", client, iteration);
  inner_->iteration_done(client, iteration);
}

void Recorder::set_stop(int client) {
  appendf(&poll_dec_, "T %d\n", client);
  inner_->set_stop(client);
}

// ---------------------------------------------------------------- replay

namespace {

struct LoggedPoll {
  unsigned long long acks;
  std::string heads;
  std::string events;
  std::vector<int64_t> us;
};

class ReplayHost : public PolicyHost {
 public:
  ReplayHost(const std::vector<LoggedPoll>* polls) : polls_(polls) {}
  bool failed() const { return !err_.empty(); }
  const std::string& error() const { return err_; }
  size_t polls_run() const { return at_; }

  void begin_poll() override {
    if (at_ >= polls_->size()) {
      fail("policy wants more polls than were logged");
      cur_ = &empty_;
    } else {
      cur_ = &(*polls_)[at_];
    }
    ++at_;
    ev_at_ = 0;
    us_at_ = 0;
  }
  void end_poll(bool effective) override {
    if (failed()) return;
    if (ev_at_ != cur_->events.size() || us_at_ != cur_->us.size())
      fail("logged observations left unread");
    else if (!effective)
      fail("logged poll changed nothing");
  }
  bool stop_ack(int client) override {
    // once diverged, report every client stopped so the loop winds down
    if (failed()) return true;
    return (cur_->acks >> client) & 1ull;
  }
  int peek(int client) override {
    if (failed()) return REC_NONE;
    int c = rec_class_from_char(cur_->heads[(size_t)client]);
    if (c == -2) { fail("client peeked but the log says it was not"); return REC_NONE; }
    if (c == -3) { fail("bad head character"); return REC_NONE; }
    return c;
  }
  bool event_done(int, int) override {
    if (failed()) return false;
    if (ev_at_ >= cur_->events.size()) { fail("unlogged event query"); return false; }
    return cur_->events[ev_at_++] == '1';
  }
  int64_t iteration_us(int) override {
    if (failed()) return 0;
    if (us_at_ >= cur_->us.size()) { fail("unlogged time read"); return 0; }
    return cur_->us[us_at_++];
  }
  void dispatch(const Dispatch&) override {}
  void iteration_done(int, int) override {}
  void set_stop(int) override {}

 private:
  void fail(const char* what) {
    if (!err_.empty()) return;
    std::ostringstream m;
    m << "poll " << (at_ ? at_ - 1 : 0) << ": " << what;
    err_ = m.str();
  }
  const std::vector<LoggedPoll>* polls_;
  const LoggedPoll* cur_ = nullptr;
  LoggedPoll empty_{0, "", "", {}};
  size_t at_ = 0, ev_at_ = 0, us_at_ = 0;
  std::string err_;
};

std::vector<std::string> split(const std::string& s, char sep, size_t max_parts) {
  std::vector<std::string> out;
  size_t at = 0;
  while (out.size() + 1 < max_parts) {
    size_t p = s.find(sep, at);
    if (p == std::string::npos) break;
    out.push_back(s.substr(at, p - at));
    at = p + 1;
  }
  out.push_back(s.substr(at));
  return out;
}

struct ClientDesc { int nk = 0, ni = 0; bool train = false; std::string path; bool set = false; };

}  // namespace

bool replay_observations(const std::string& obs, bool sequential_fix,
                         std::string* decisions, std::string* err, bool mark_polls) {
  std::vector<std::string> lines;
  {
    size_t at = 0;
    while (at < obs.size()) {
      size_t nl = obs.find('\n', at);
      if (nl == std::string::npos) nl = obs.size();
      lines.push_back(obs.substr(at, nl - at));
      at = nl + 1;
    }
  }
  auto bad = [&](size_t ln, const std::string& what) {
    if (err) {
      std::ostringstream m;
      m << "observation log line " << ln + 1 << ": " << what;
      *err = m.str();
    }
    return false;
  };

  int n = 0, max_sms = 0;
  bool confine_long = false, reserve_hp = false, admit_oversized = false;
  bool sliding_throttle = false;
  std::vector<int> masks;
  std::vector<ClientDesc> clients;
  Policy* policy = nullptr;
  std::vector<LoggedPoll> no_polls;
  ReplayHost idle(&no_polls);
  Recorder rec(&idle, 0);
  bool ok = true;

  for (size_t i = 0; ok && i < lines.size(); ++i) {
    const std::string& l = lines[i];
    if (l.empty()) continue;
    const char tag = l[0];
    if (tag == 'J') {
      auto p = split(l, ' ', 9);
      bool options_ok = p.size() >= 4 && p.size() <= 8;
      for (size_t k = 4; options_ok && k < p.size(); ++k) {
        if (p[k] == "L1") confine_long = true;
        else if (p[k] == "R1") reserve_hp = true;
        else if (p[k] == "O1") admit_oversized = true;
        else if (p[k] == "T1") sliding_throttle = true;
        else options_ok = false;
      }
      if (!options_ok) {
        ok = bad(i, "J needs 3 fields and optional L1 / R1 / O1 / T1");
        break;
      }
      n = atoi(p[1].c_str());
      max_sms = atoi(p[2].c_str());
      for (auto& m : split(p[3], ',', 1u << 20)) masks.push_back(atoi(m.c_str()));
      if (n < 1 || n > 64) { ok = bad(i, "client count out of range"); break; }
      clients.assign((size_t)n, ClientDesc());
      rec = Recorder(&idle, n);
      rec.set_mark_polls(mark_polls);
    } else if (tag == 'K') {
      auto p = split(l, ' ', 6);
      if (p.size() != 6) { ok = bad(i, "K needs 5 fields"); break; }
      int c = atoi(p[1].c_str());
      if (c < 0 || c >= n) { ok = bad(i, "client index out of range"); break; }
      clients[(size_t)c].nk = atoi(p[2].c_str());
      clients[(size_t)c].ni = atoi(p[3].c_str());
      clients[(size_t)c].train = atoi(p[4].c_str()) != 0;
      clients[(size_t)c].path = p[5];
      clients[(size_t)c].set = true;
    } else if (tag == 'X') {
      auto p = split(l, ' ', 4);
      if (p.size() != 4 || !policy) { ok = bad(i, "X before S or malformed"); break; }
      int c = atoi(p[1].c_str());
      if (c < 0 || c >= n) { ok = bad(i, "client index out of range"); break; }
      std::vector<OpInfo> ops;
      std::string perr;
      if (!parse_profile(p[3], &ops, &perr)) { ok = bad(i, perr); break; }
      policy->setup_change(c, std::move(ops), atoi(p[2].c_str()));
      rec.setup_change(c, atoi(p[2].c_str()), p[3]);
    } else if (tag == 'S') {
      auto p = split(l, ' ', 7);
      if (p.size() != 7 || n == 0) { ok = bad(i, "S needs 6 fields after J"); break; }
      if (!policy) {
        std::vector<std::vector<OpInfo>> profs((size_t)n);
        std::vector<int> nk, ni;
        std::vector<bool> tr;
        for (int c = 0; c < n && ok; ++c) {
          if (!clients[(size_t)c].set) { ok = bad(i, "missing K line"); break; }
          std::string perr;
          if (!parse_profile(clients[(size_t)c].path, &profs[(size_t)c], &perr)) {
            ok = bad(i, perr);
            break;
          }
          nk.push_back(clients[(size_t)c].nk);
          ni.push_back(clients[(size_t)c].ni);
          tr.push_back(clients[(size_t)c].train);
        }
        if (!ok) break;
        policy = new Policy(std::move(profs), nk, ni, tr, max_sms, masks,
                            sequential_fix, confine_long, reserve_hp, admit_oversized,
                            sliding_throttle);
      }
      ScheduleArgs a;
      a.warmup = atoi(p[1].c_str()) != 0;
      a.warmup_iters = atoi(p[2].c_str());
      a.algo = algo_from_name(p[3]);
      if (a.algo < 0) { ok = bad(i, "unknown algorithm"); break; }
      a.depth = atoi(p[4].c_str());
      a.hp_limit = atoi(p[5].c_str());
      a.update_start = atoi(p[6].c_str());
      std::vector<LoggedPoll> polls;
      size_t j = i + 1;
      for (; j < lines.size() && lines[j] != "E"; ++j) {
        auto q = split(lines[j], ' ', 5);
        if (q.size() != 5 || q[0] != "P" || (int)q[2].size() != n) {
          ok = bad(j, "expected a P line with one head per client");
          break;
        }
        LoggedPoll lp;
        lp.acks = strtoull(q[1].c_str(), nullptr, 16);
        lp.heads = q[2];
        if (q[3] != "-") lp.events = q[3];
        if (q[4] != "-")
          for (auto& u : split(q[4], ',', 1u << 20)) lp.us.push_back(atoll(u.c_str()));
        polls.push_back(std::move(lp));
      }
      if (!ok) break;
      if (j >= lines.size()) { ok = bad(i, "S without E"); break; }
      ReplayHost host(&polls);
      rec.set_inner(&host);
      rec.begin_schedule(a);
      a.max_polls = (int64_t)polls.size() + 1;
      policy->schedule(rec, a);
      rec.set_inner(&idle);
      if (host.failed()) { ok = bad(i, host.error()); break; }
      if (host.polls_run() != polls.size()) {
        ok = bad(i, "policy finished before the logged polls ran out");
        break;
      }
      rec.end_schedule();
      i = j;
    } else if (tag == 'E' || tag == 'P') {
      ok = bad(i, "stray line outside an S..E segment");
    } else if (tag != '#') {
      ok = bad(i, "unknown line tag");
    }
  }
  if (ok && decisions) *decisions = rec.decisions();
  delete policy;
  return ok;
}

}  // namespace orion
