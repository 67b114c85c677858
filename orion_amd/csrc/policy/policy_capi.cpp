// C ABI of liborion_policy.so: the policy core without any HIP dependency,
// for replaying observation logs and parsing profiles on a CPU-only host.
#include <cstdlib>
#include <cstring>
#include <string>

#include "obslog.h"
#include "orion_policy.h"
#include "policy.h"

namespace {
char* dup_string(const std::string& s) {
  char* p = (char*)malloc(s.size() + 1);
  if (p) memcpy(p, s.c_str(), s.size() + 1);
  return p;
}
}  // namespace

extern "C" {

static int replay(const char* observations, int sequential_fix, bool mark_polls,
                  char** decisions_out, char** error_out) {
  if (decisions_out) *decisions_out = nullptr;
  if (error_out) *error_out = nullptr;
  if (!observations) return 1;
  std::string dec, err;
  bool ok = orion::replay_observations(observations, sequential_fix != 0, &dec, &err,
                                       mark_polls);
  if (!ok) {
    if (error_out) *error_out = dup_string(err);
    return 2;
  }
  if (decisions_out) *decisions_out = dup_string(dec);
  return 0;
}

int orion_policy_replay(const char* observations, int sequential_fix,
                        char** decisions_out, char** error_out) {
  return replay(observations, sequential_fix, false, decisions_out, error_out);
}

int orion_policy_replay_by_poll(const char* observations, int sequential_fix,
                                char** decisions_out, char** error_out) {
  return replay(observations, sequential_fix, true, decisions_out, error_out);
}

void orion_policy_free(char* p) { free(p); }

int orion_profile_stats(const char* path, int* rows, int* max_sm_used,
                        double* duration_sum, char** error_out) {
  if (error_out) *error_out = nullptr;
  std::vector<orion::OpInfo> ops;
  std::string err;
  if (!path || !orion::parse_profile(path, &ops, &err)) {
    if (error_out) *error_out = dup_string(err);
    return 2;
  }
  int best = 0;
  double sum = 0.0;
  for (const auto& op : ops) {
    if (op.sm_used > best) best = op.sm_used;
    sum += (double)op.duration;
  }
  if (rows) *rows = (int)ops.size();
  if (max_sm_used) *max_sm_used = best;
  if (duration_sum) *duration_sum = sum;
  return 0;
}

int orion_profile_row(const char* path, int row, char* name, size_t name_cap,
                      int* profile, int* mem, int* sm_used, float* duration) {
  std::vector<orion::OpInfo> ops;
  std::string err;
  if (!path || !orion::parse_profile(path, &ops, &err)) return 2;
  if (row < 0 || row >= (int)ops.size()) return 1;
  const orion::OpInfo& op = ops[(size_t)row];
  if (name && name_cap) {
    strncpy(name, op.name.c_str(), name_cap - 1);
    name[name_cap - 1] = '\0';
  }
  if (profile) *profile = op.profile;
  if (mem) *mem = op.mem;
  if (sm_used) *sm_used = op.sm_used;
  if (duration) *duration = op.duration;
  return 0;
}

int orion_place_cu_slot(const int* masks, int n_masks, int rec_class,
                        int sm_used, int algo, int hp_active, int long_kernel) {
  std::vector<int> m(masks, masks + (n_masks > 0 ? n_masks : 0));
  if (m.empty()) return -1;
  return orion::place_cu_slot(m, rec_class, sm_used, algo, hp_active != 0,
                              long_kernel != 0);
}

}  // extern "C"
