/* Host-only check that libinttemp.so takes a thread off the dynamic loader's
 * slow path for thread-local accesses.  TEST INFRASTRUCTURE.
 *
 * usage: tls_fresh_probe <libinttemp.so> <liba.so> <libb.so>
 * liba and libb each hold one thread-local counter behind touch_a / touch_b.
 * Prints, in ns per access of liba's counter: fresh (liba is the newest library
 * with thread-local storage), stale (libb loaded afterwards, never touched),
 * cured (after the capture library's check ran on this thread). */
#define _GNU_SOURCE
#include <dlfcn.h>
#include <stdio.h>
#include <stdlib.h>
#include <sys/syscall.h>
#include <time.h>
#include <unistd.h>

typedef long (*touch_t)(void);

static double now(void) {
  struct timespec t;
  clock_gettime(CLOCK_MONOTONIC, &t);
  return t.tv_sec + 1e-9 * t.tv_nsec;
}

static double ns_per_call(touch_t f) {
  double best = 1e30;
  for (int rep = 0; rep < 5; ++rep) {
    const long n = 4000000;
    long s = 0;
    const double t0 = now();
    for (long i = 0; i < n; ++i) s += f();
    const double dt = (now() - t0) / n * 1e9;
    if (s && dt < best) best = dt;
  }
  return best;
}

int main(int argc, char** argv) {
  if (argc < 4) return 2;
  void* cap = dlopen(argv[1], RTLD_NOW | RTLD_GLOBAL);
  if (!cap) { fprintf(stderr, "%s\n", dlerror()); return 3; }
  void (*arm)(int, const int*, int) = (void (*)(int, const int*, int))dlsym(cap, "orion_capture_arm");
  void (*disarm)(void) = (void (*)(void))dlsym(cap, "orion_capture_disarm");
  void (*passthrough)(int) = (void (*)(int))dlsym(cap, "orion_thread_passthrough");
  void (*stats)(unsigned long long*, unsigned long long*) =
      (void (*)(unsigned long long*, unsigned long long*))dlsym(cap, "orion_tls_fresh_stats");
  if (!arm || !disarm || !passthrough || !stats) return 4;

  void* ha = dlopen(argv[2], RTLD_NOW);
  if (!ha) { fprintf(stderr, "%s\n", dlerror()); return 3; }
  touch_t a = (touch_t)dlsym(ha, "touch_a");
  const double fresh = ns_per_call(a);
  void* hb = dlopen(argv[3], RTLD_NOW);   /* newer thread-local storage, never touched */
  if (!hb) { fprintf(stderr, "%s\n", dlerror()); return 3; }
  const double stale = ns_per_call(a);

  /* this thread as the only client of an armed capture; the end of its
   * un-captured phase is where the library checks */
  const int tid = (int)syscall(SYS_gettid);
  arm(1, &tid, 0);
  passthrough(1);
  passthrough(0);
  const double cured = ns_per_call(a);
  unsigned long long reloads = 0, touches = 0;
  stats(&reloads, &touches);
  disarm();
  printf("{\"fresh_ns\": %.3f, \"stale_ns\": %.3f, \"cured_ns\": %.3f, \"reloads\": %llu, "
         "\"touches\": %llu}\n", fresh, stale, cured, reloads, touches);
  return 0;
}
