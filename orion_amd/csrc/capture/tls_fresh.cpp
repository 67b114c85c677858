#include "tls_fresh.h"

#include <dlfcn.h>
#include <immintrin.h>
#include <link.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>
#include <time.h>

#include <mutex>
#include <string>

namespace orion {

std::atomic<uint32_t> g_tls_fresh_reloads{0};
__thread uint32_t tl_tls_fresh_seen __attribute__((tls_model("initial-exec"))) = 0;

namespace {

typedef unsigned long (*touch_fn)(void);

std::mutex g_reload_lock;
void* g_handle = nullptr;
std::atomic<touch_fn> g_touch{nullptr};
// threads inside (or about to enter) the loaded library: a reload waits for them
std::atomic<int> g_users{0};
std::atomic<unsigned long long> g_seen_adds{0}, g_seen_subs{0};
std::atomic<unsigned long long> g_touches{0};
std::atomic<int64_t> g_last_reload_ns{0};

int enabled() {
  static const int on = [] {
    const char* e = getenv("ORION_TLS_REFRESH");
    return e && strcmp(e, "0") == 0 ? 0 : 1;
  }();
  return on;
}

// liborion_tlsfresh.so lies beside this library (ORION_TLS_REFRESH_LIBRARY names
// another place: for programs that link these sources statically).
const std::string& helper_path() {
  static const std::string path = [] {
    if (const char* e = getenv("ORION_TLS_REFRESH_LIBRARY"))
      if (*e) return std::string(e);
    Dl_info info;
    std::string p;
    if (dladdr((void*)&tls_fresh_check, &info) && info.dli_fname) {
      p = info.dli_fname;
      const size_t cut = p.rfind('/');
      p = (cut == std::string::npos ? std::string(".") : p.substr(0, cut)) +
          "/liborion_tlsfresh.so";
    }
    return p;
  }();
  return path;
}

struct LoadCounts { unsigned long long adds, subs; };
int read_counts(struct dl_phdr_info* info, size_t, void* out) {
  ((LoadCounts*)out)->adds = info->dlpi_adds;
  ((LoadCounts*)out)->subs = info->dlpi_subs;
  return 1;   // the first object is enough: the counters are the process's
}

int64_t now_ns() {
  timespec ts;
  clock_gettime(CLOCK_MONOTONIC, &ts);
  return (int64_t)ts.tv_sec * 1000000000ll + ts.tv_nsec;
}

void reload_locked() {
  // nobody may be inside the old copy when it is unloaded
  g_touch.store(nullptr, std::memory_order_seq_cst);
  while (g_users.load(std::memory_order_seq_cst) != 0) _mm_pause();
  if (g_handle) dlclose(g_handle);
  g_handle = dlopen(helper_path().c_str(), RTLD_NOW | RTLD_LOCAL);
  touch_fn fn = g_handle ? (touch_fn)dlsym(g_handle, "orion_tls_touch") : nullptr;
  if (!fn) {
    static bool told = false;
    if (!told) {
      told = true;
      fprintf(stderr, "orion: %s cannot be loaded (%s); thread-local accesses of the clients "
                      "stay on the loader's slow path\n", helper_path().c_str(), dlerror());
    }
  }
  LoadCounts c{0, 0};
  dl_iterate_phdr(read_counts, &c);   // includes what this reload itself did
  g_seen_adds.store(c.adds, std::memory_order_relaxed);
  g_seen_subs.store(c.subs, std::memory_order_relaxed);
  g_last_reload_ns.store(now_ns(), std::memory_order_relaxed);
  g_touch.store(fn, std::memory_order_seq_cst);
  g_tls_fresh_reloads.fetch_add(1, std::memory_order_release);
}

}  // namespace

void tls_fresh_touch_slow() {
  if (!enabled()) {
    tl_tls_fresh_seen = g_tls_fresh_reloads.load(std::memory_order_relaxed);
    return;
  }
  const uint32_t count = g_tls_fresh_reloads.load(std::memory_order_acquire);
  g_users.fetch_add(1, std::memory_order_seq_cst);
  if (touch_fn fn = g_touch.load(std::memory_order_seq_cst)) {
    fn();
    g_touches.fetch_add(1, std::memory_order_relaxed);
  }
  g_users.fetch_sub(1, std::memory_order_release);
  // Also when there was nothing to call (a reload is under way, or the helper
  // library could not be loaded): the reload counter moves on when a reload
  // completes and brings the thread back here; until then it stays off the
  // shared counters above.
  tl_tls_fresh_seen = count;
}

void tls_fresh_check() {
  if (!enabled()) return;
  LoadCounts c{0, 0};
  dl_iterate_phdr(read_counts, &c);
  if (c.adds != g_seen_adds.load(std::memory_order_relaxed) ||
      c.subs != g_seen_subs.load(std::memory_order_relaxed)) {
    // a process that keeps loading libraries gets a reload every few
    // milliseconds, not one per call
    if (now_ns() - g_last_reload_ns.load(std::memory_order_relaxed) > 5000000ll) {
      std::unique_lock<std::mutex> hold(g_reload_lock, std::try_to_lock);
      if (hold.owns_lock()) reload_locked();
    }
  }
  tls_fresh_touch();
}

}  // namespace orion

extern "C" {

// How often the helper library has been reloaded and how many times a thread
// has called into a fresh copy (for tests and diagnostics).
void orion_tls_fresh_stats(unsigned long long* reloads, unsigned long long* touches) {
  if (reloads) *reloads = orion::g_tls_fresh_reloads.load(std::memory_order_relaxed);
  if (touches) *touches = orion::g_touches.load(std::memory_order_relaxed);
}

}  // extern "C"
