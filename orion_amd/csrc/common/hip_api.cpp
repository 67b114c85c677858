#include "hip_api.h"

#include <dlfcn.h>
#include <link.h>
#include <pthread.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

namespace {

orion::HipApi g_api;
pthread_once_t g_once = PTHREAD_ONCE_INIT;

int find_loaded_runtime(struct dl_phdr_info* info, size_t, void* out) {
  const char* path = info->dlpi_name;
  if (!path || !*path) return 0;
  const char* base = strrchr(path, '/');
  base = base ? base + 1 : path;
  if (strncmp(base, "libamdhip64.so", 14) == 0) {
    *(const char**)out = path;
    return 1;
  }
  return 0;
}

void resolve() {
  void* handle = nullptr;
  const char* from = getenv("ORION_HIP_LIBRARY");
  static char chosen[4096];
  if (from && *from) {
    handle = dlopen(from, RTLD_NOW | RTLD_LOCAL);
    if (!handle) {
      fprintf(stderr, "orion: ORION_HIP_LIBRARY=%s: %s\n", from, dlerror());
      abort();
    }
  } else {
    const char* loaded = nullptr;
    dl_iterate_phdr(find_loaded_runtime, &loaded);
    if (loaded) {
      handle = dlopen(loaded, RTLD_NOW | RTLD_LOCAL | RTLD_NOLOAD);
      from = loaded;
    }
    if (!handle) {
      from = "libamdhip64.so.7";
      handle = dlopen(from, RTLD_NOW | RTLD_LOCAL);
    }
    if (!handle) {
      fprintf(stderr, "orion: no HIP runtime found (%s)\n", dlerror());
      abort();
    }
  }
  // the host-only stand-in is recognised by its own control call, not by how it
  // was named: a real runtime named through the variable is still a real runtime
  g_api.stand_in = dlsym(handle, "fakehip_set_costs") != nullptr;
  // ORION_STAND_IN_AS_DEVICE=1: a host test asks to be treated like a GPU
  // process (the variable can only take privileges away)
  if (const char* strict = getenv("ORION_STAND_IN_AS_DEVICE"))
    if (atoi(strict) != 0) g_api.stand_in = false;
  snprintf(chosen, sizeof chosen, "%s", from);
  g_api.library_path = chosen;
#define X(name, ret, params) g_api.name = (decltype(g_api.name))dlsym(handle, #name);
  ORION_HIP_FUNCTIONS(X)
#undef X
  if (!g_api.hipLaunchKernel || !g_api.hipMalloc || !g_api.hipStreamSynchronize) {
    fprintf(stderr, "orion: %s lacks core HIP entry points\n", from);
    abort();
  }
}

}  // namespace

extern "C" const orion::HipApi* orion_hip_api(void) {
  pthread_once(&g_once, resolve);
  return &g_api;
}
