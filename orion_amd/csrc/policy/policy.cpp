#include "policy.h"

#include <cerrno>
#include <climits>
#include <cstdlib>
#include <cstring>
#include <fstream>
#include <sstream>

namespace orion {

char rec_class_char(int c) {
  switch (c) {
    case REC_KERNEL: return 'k';
    case REC_MEMCPY: return 'c';
    case REC_MALLOC: return 'm';
    case REC_FREE: return 'f';
    case REC_MEMSET: return 's';
    default: return '.';
  }
}

int rec_class_from_char(char ch) {
  switch (ch) {
    case 'k': return REC_KERNEL;
    case 'c': return REC_MEMCPY;
    case 'm': return REC_MALLOC;
    case 'f': return REC_FREE;
    case 's': return REC_MEMSET;
    case '.': return REC_NONE;
    case '-': return -2;
    default: return -3;
  }
}

const char* algo_name(int algo) {
  switch (algo) {
    case ALGO_REEF: return "reef";
    case ALGO_SEQUENTIAL: return "sequential";
    default: return "orion";
  }
}

int algo_from_name(const std::string& name) {
  if (name == "orion") return ALGO_ORION;
  if (name == "reef") return ALGO_REEF;
  if (name == "sequential") return ALGO_SEQUENTIAL;
  return -1;
}

namespace {

// std::stoi / std::stof semantics without exceptions: leading white space,
// longest valid prefix, trailing characters ignored.
bool to_int(const std::string& s, int* out) {
  errno = 0;
  char* end = nullptr;
  long v = std::strtol(s.c_str(), &end, 10);
  if (end == s.c_str() || errno == ERANGE || v < INT_MIN || v > INT_MAX)
    return false;
  *out = (int)v;
  return true;
}

bool to_float(const std::string& s, float* out) {
  errno = 0;
  char* end = nullptr;
  float v = std::strtof(s.c_str(), &end);
  if (end == s.c_str()) return false;
  *out = v;
  return true;
}

}  // namespace

bool parse_profile(const std::string& path, std::vector<OpInfo>* ops,
                   std::string* err) {
  std::ifstream in(path);
  if (!in.is_open()) {
    if (err) *err = "cannot open profile " + path;
    return false;
  }
  std::string line;
  std::getline(in, line);  // header
  int row = 1;
  while (std::getline(in, line)) {
    ++row;
    std::vector<std::string> v;
    size_t at = 0;
    for (;;) {
      size_t comma = line.find(',', at);
      if (comma == std::string::npos) {
        v.push_back(line.substr(at));
        break;
      }
      v.push_back(line.substr(at, comma - at));
      at = comma + 1;
    }
    OpInfo info;
    if (v.size() < 5 || !to_int(v[1], &info.profile) ||
        !to_int(v[2], &info.mem) || !to_int(v[3], &info.sm_used) ||
        !to_float(v[4], &info.duration)) {
      if (err) {
        std::ostringstream m;
        m << path << ": row " << row << " is not Name,Profile,Memory_footprint,"
          << "SM_usage,Duration";
        *err = m.str();
      }
      return false;
    }
    info.name = v[0];
    ops->push_back(info);
  }
  return true;
}

int place_cu_slot(const std::vector<int>& masks, int rec_class, int sm_used,
                  int algo, bool hp_active, bool long_kernel) {
  if (rec_class != REC_KERNEL) return -1;
  const int last = (int)masks.size() - 1;
  if (algo != ALGO_ORION || last == 0) return last;
  if (!hp_active) return long_kernel ? last - 1 : last;
  for (int s = 0; s < last; ++s)
    if (sm_used <= masks[s]) return s;
  return last - 1;
}

static int max_sm_used(const std::vector<OpInfo>& ops) {
  int best = 0;
  for (const OpInfo& op : ops) best = op.sm_used > best ? op.sm_used : best;
  return best;
}

Policy::Policy(std::vector<std::vector<OpInfo>> profiles,
               std::vector<int> num_kernels, std::vector<int> num_iters,
               std::vector<bool> is_train, int max_sms,
               std::vector<int> cu_masks, bool sequential_fix, bool confine_long,
               bool reserve_hp, bool admit_oversized, bool sliding_throttle)
    : n_((int)profiles.size()),
      ops_(std::move(profiles)),
      num_kernels_(std::move(num_kernels)),
      max_iters_(std::move(num_iters)),
      is_train_(std::move(is_train)),
      max_sms_(max_sms),
      cu_masks_(std::move(cu_masks)),
      sequential_fix_(sequential_fix),
      confine_long_(confine_long),
      reserve_hp_(reserve_hp),
      admit_oversized_(admit_oversized),
      sliding_throttle_(sliding_throttle),
      seen_(n_, 0),
      event_ids_(n_, 0),
      cur_iters_(n_, 0),
      stops_(n_, false),
      admission_(n_, std::array<uint64_t, ADM_COUNT>{}) {
  if (cu_masks_.empty()) cu_masks_.push_back(max_sms_);
  for (int i = 0; i < n_; ++i) max_sms_clients_.push_back(max_sm_used(ops_[i]));
}

void Policy::setup_change(int client, std::vector<OpInfo> ops, int num_kernels) {
  ops_[client] = std::move(ops);
  max_sms_clients_[client] = max_sm_used(ops_[client]);
  num_kernels_[client] = num_kernels;
}

// schedule_kernel + pop_from_queue: kernel-like records advance the client's
// position in its profile and the owner's event index; memory records do not.
void Policy::dispatch(PolicyHost& host, int client, int owner, int rec_class,
                      bool smallest_mask) {
  Dispatch d;
  d.client = client;
  d.owner = owner;
  d.rec_class = rec_class;
  d.op_index = seen_[client];
  d.event_slot = event_ids_[owner];
  if (rec_class != REC_KERNEL) {
    d.cu_slot = -1;
  } else if (owner == n_ - 1) {
    d.cu_slot = 0;  // the high-priority stream spans the whole GPU
  } else if (smallest_mask) {
    d.cu_slot = 0;  // an oversized kernel let in beside a high-priority request
  } else {
    const OpInfo& op = ops_[client][d.op_index];
    d.cu_slot = place_cu_slot(cu_masks_, rec_class, op.sm_used, algo_,
                              seen_[n_ - 1] > 0,
                              confine_long_ && op.duration > (float)be_budget_);
  }
  host.dispatch(d);
  if (rec_class == REC_KERNEL) {
    event_ids_[owner] += 1;
    seen_[client] += 1;
  }
  changed_ = true;
}

void Policy::reef(PolicyHost& host, const std::vector<int>& heads, int depth) {
  if (n_ == 1) {
    if (heads[0] != REC_NONE) dispatch(host, 0, 0, heads[0]);
    return;
  }
  const int hp = n_ - 1;
  for (int i = 0; i < n_; ++i) {
    if (heads[i] == REC_NONE) continue;
    if (heads[i] == REC_MALLOC || cur_iters_[i] <= 10 ||
        cur_iters_[hp] >= max_iters_[hp]) {
      dispatch(host, i, i, heads[i]);
      return;
    }
  }
  if (heads[hp] != REC_NONE) {
    const int hp_idx = seen_[hp];
    dispatch(host, hp, hp, heads[hp]);
    const OpInfo& op1 = ops_[hp][hp_idx];
    for (int i = 0; i < hp; ++i) {
      if (heads[i] == REC_NONE) continue;
      const OpInfo& op0 = ops_[i][seen_[i]];
      if (op0.duration <= op1.duration && op0.sm_used >= op1.sm_used) {
        dispatch(host, i, i, heads[i]);
        return;
      }
    }
  } else {
    for (int i = 0; i < hp; ++i) {
      if (heads[i] != REC_NONE) {
        penalty_ += 1;
        changed_ = true;
      }
    }
    if (penalty_ >= depth) {
      for (int i = 0; i < hp; ++i)
        if (heads[i] != REC_NONE) dispatch(host, i, i, heads[i]);
      penalty_ = 0;
    }
  }
}

int Policy::sequential(PolicyHost& host, const std::vector<int>& heads,
                       int start) {
  if (n_ == 1) {
    if (heads[0] != REC_NONE) dispatch(host, 0, 0, heads[0]);
    return start;
  }
  const int hp = n_ - 1;
  if (heads[hp] != REC_NONE) {
    bool go = false;
    if (cur_iters_[hp] <= 10 || heads[hp] == REC_MALLOC) {
      go = true;
    } else {
      go = sequential_fix_;
      for (int i = 0; i < hp; ++i) {
        if (seen_[i] > 0) {
          go = false;
          break;
        }
      }
    }
    if (go) dispatch(host, hp, 0, heads[hp]);
  }
  const int end = start + n_;
  for (int t = start + 1; t < end; ++t) {
    const int i = t % (n_ - 1);
    if (heads[i] == REC_NONE) continue;
    bool go = false;
    if (cur_iters_[i] <= 10 || heads[i] == REC_MALLOC) {
      go = true;
    } else {
      go = sequential_fix_;
      for (int j = 0; j < n_; ++j) {
        if (i != j && seen_[j] > 0) {
          go = false;
          break;
        }
      }
    }
    if (go) {
      dispatch(host, i, 0, heads[i]);
      start = t;
      break;
    }
  }
  return start;
}

int64_t Policy::schedule(PolicyHost& host, const ScheduleArgs& args) {
  const int n = n_;
  const int hp = n - 1;
  const bool is_reef = args.algo == ALGO_REEF;
  const bool is_seq = args.algo == ALGO_SEQUENTIAL;
  algo_ = args.algo;
  be_budget_ = args.depth;
  std::vector<int> profiles(n, -1);
  bool large_found = false;
  long sum = 0;   // outstanding best-effort duration; long += float below
  long size = 0;  // CU need of the best-effort ops admitted in this poll
  int start = -1;
  int low_sms = 0;
  int high_sms = max_sms_clients_[0];
  int sm_threshold = max_sms_clients_[0] / 2;
  float hp_iter_duration = 0.0f;
  const float hp_limit_float = (float)args.hp_limit;
  int update_start = args.update_start;
  if (!is_train_[hp]) {
    sm_threshold = max_sms_;
    update_start = INT_MAX;
  }
  std::vector<int> heads(n);
  int64_t polls = 0;
  int hp_need = 0;  // CU need of the high-priority op last dispatched (reserve_hp_)
  // sliding_throttle_: per best-effort client the kernel that was its latest when
  // the sum passed half the budget (-1: none), and the sum at that moment
  std::vector<int> mark_index(n, -1);
  bool mark_valid = false;
  long mark_sum = 0;

  for (;;) {
    host.begin_poll();
    changed_ = false;
    size = 0;
    for (int i = 0; i < n; ++i) {
      heads[i] = REC_NONE;
      if (seen_[i] == num_kernels_[i]) continue;
      heads[i] = host.peek(i);
    }

    if (is_reef) {
      reef(host, heads, args.depth);
    } else if (is_seq) {
      start = sequential(host, heads, start);
    } else {
      if (heads[hp] != REC_NONE) {
        const int hp_profile = ops_[hp][seen_[hp]].profile;
        hp_need = ops_[hp][seen_[hp]].sm_used;
        dispatch(host, hp, hp, heads[hp]);
        profiles[hp] = hp_profile;
      }
      int room = sm_threshold;
      if (reserve_hp_ && !is_train_[hp]) {
        room = sm_threshold - (hp_need > 0 ? hp_need : 0);
        if (room < 0) room = 0;
      }
      const int end = start + n;
      for (int t = start + 1; t < end; ++t) {
        const int j = t % (n - 1);
        if (heads[j] == REC_NONE) continue;
        const OpInfo& op0 = ops_[j][seen_[j]];
        const int cls = heads[j];
        const bool mem_op = is_mem_class(cls);
        bool go = false;
        bool oversized = false;
        int outcome = ADM_REFUSED_CUS;
        if (n == 1 || seen_[hp] == 0 || mem_op) {
          go = true;
        } else if (cur_iters_[j] <= 10 || cur_iters_[hp] >= max_iters_[hp]) {
          go = true;
        } else if (seen_[hp] >= update_start && op0.sm_used <= sm_threshold &&
                   host.event_done(hp, update_start - 1)) {
          go = true;
        } else if (seen_[hp] > 0 && size + op0.sm_used <= room &&
                   (op0.profile == -1 || profiles[hp] == -1 ||
                    profiles[hp] != op0.profile)) {
          go = true;
        } else if (size + op0.sm_used <= room) {
          outcome = ADM_REFUSED_CLASS;
        } else if (admit_oversized_ && !is_train_[hp] && size == 0 &&
                   op0.sm_used > max_sms_ && op0.profile != -1 && profiles[hp] != -1 &&
                   profiles[hp] != op0.profile &&
                   op0.duration <= (float)(args.depth / 4)) {
          go = true;
          oversized = true;
        }
        if (go && large_found) {
          bool clear = true;
          for (int k = 0; k < n - 1; ++k) {
            if (event_ids_[k] >= 1 && !host.event_done(k, event_ids_[k] - 1)) {
              clear = false;
              break;
            }
          }
          if (clear) {
            large_found = false;
            sum = 0;
            changed_ = true;
            mark_valid = false;
          } else if (sliding_throttle_ && mark_valid) {
            bool half = true;
            for (int k = 0; k < n - 1; ++k) {
              if (mark_index[k] >= 0 && !host.event_done(k, mark_index[k])) {
                half = false;
                break;
              }
            }
            if (half) {
              // everything dispatched up to the marks has completed
              sum -= mark_sum;
              if (sum < 0) sum = 0;
              mark_valid = false;
              large_found = false;
              changed_ = true;
            } else {
              go = false;
              outcome = ADM_THROTTLED;
            }
          } else {
            go = false;
            outcome = ADM_THROTTLED;
          }
        }
        admission_[j][go ? (oversized ? ADM_OVERSIZED : ADM_ADMITTED) : outcome] += 1;
        if (go) {
          size += op0.sm_used;
          if (!mem_op) sum = (long)((float)sum + op0.duration);
          if (sum > args.depth && cur_iters_[hp] < max_iters_[hp])
            large_found = true;
          dispatch(host, j, j, cls, oversized);
          start = j;
          if (sliding_throttle_ && !mem_op && !mark_valid && sum > args.depth / 2) {
            for (int k = 0; k < n - 1; ++k) {
              mark_index[k] = event_ids_[k] - 1;
              if (mark_index[k] >= 0) host.mark(k, mark_index[k]);
            }
            mark_sum = sum;
            mark_valid = true;
          }
        }
      }
    }

    int finished = 0;
    for (int i = 0; i < n; ++i) {
      if (cur_iters_[i] == max_iters_[i] ||
          (args.warmup && cur_iters_[i] == args.warmup_iters) ||
          host.stop_ack(i)) {
        finished += 1;
      } else if (seen_[i] == num_kernels_[i]) {
        const int owner = is_seq ? 0 : i;
        bool ready = true;
        if (event_ids_[owner] >= 1 &&
            !host.event_done(owner, event_ids_[owner] - 1))
          ready = false;
        if (ready) {
          seen_[i] = 0;
          if (is_seq) event_ids_[0] = 0;
          event_ids_[i] = 0;
          mark_index[i] = -1;  // a completed iteration has nothing outstanding
          host.iteration_done(i, cur_iters_[i]);
          cur_iters_[i] += 1;
          changed_ = true;
          if (!is_reef && !is_seq && i == hp && is_train_[hp]) {
            // microseconds as float, divided by the double 1000.0, back to float
            float duration = (float)host.iteration_us(i);
            duration = (float)((double)duration / 1000.0);
            hp_iter_duration += duration;
            if (cur_iters_[i] % 10 == 0 && low_sms != sm_threshold) {
              const float avg = (float)((double)hp_iter_duration / 10.0);
              hp_iter_duration = 0.0f;
              if (avg > hp_limit_float) {
                high_sms = sm_threshold;
              } else {
                low_sms = sm_threshold;
              }
              sm_threshold = (low_sms + high_sms) / 2;
            }
          }
        }
        if (cur_iters_[i] == max_iters_[i] ||
            (args.warmup && cur_iters_[i] == args.warmup_iters) ||
            host.stop_ack(i)) {
          finished += 1;
          if (!args.warmup && i == n - 1) {
            for (int k = 0; k < n - 1; ++k) {
              if (!stops_[k]) changed_ = true;
              stops_[k] = true;
              host.set_stop(k);
            }
          }
        }
      }
    }

    sm_threshold_ = sm_threshold;
    large_found_ = large_found;
    sum_ = sum;
    host.end_poll(changed_ || finished == n);
    ++polls;
    if (finished == n) break;
    if (args.max_polls >= 0 && polls >= args.max_polls) return -1;
  }
  return polls;
}

}  // namespace orion
